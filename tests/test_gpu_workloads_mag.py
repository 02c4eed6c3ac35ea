"""The MAG240M-shaped configuration at the largest size this box serves: the node count is scaled
so that the 768-d fp16 feature table is as large as hipHostMalloc grants (the full table is 375 GB;
a box with 309 GB of RAM granted 68 GB: 44 M nodes, 19 M int8 rows cached), batches of 1024 seeds,
fan-out [25,15], int8 cache with the dequantisation inside the gather."""
import sys

import numpy as np
import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu
sys.path.insert(0, ROOT)


def test_mag240m_int8_at_the_largest_size_the_box_serves(lmi, oracle):
    import bench
    if bench.mem_available_gb() < 100:
        pytest.skip("needs a feature table of tens of GB in pinned host memory plus a host copy of the graph")
    w = dict(bench.WORKLOADS["mag240m-int8"])
    inputs = bench.build_inputs(lmi, w, 777, 0.0)
    srv = None
    try:
        assert inputs["feats"].nbytes > 40e9, "expected a table of tens of GB, got %.1f GB" % (inputs["feats"].nbytes / 1e9)
        srv, info = bench.build_server(lmi, w, inputs, 777, 16)
        for k, v in w.get("tune", {}).items():
            srv.tune(k, int(v))                      # the workload's own settings, as bench.py applies them
        stream = lmi.stream_create()
        feats = info["feats"].array
        indptr = lmi.to_host(info["d_indptr"], info["n_nodes"] + 1, np.int64)
        indices = lmi.to_host(info["d_indices"], info["n_edges"], np.int32)
        deg = np.diff(indptr)
        slot = srv.cache_dump(info["n_nodes"])
        assert int((slot >= 0).sum()) == info["cache_rows"] == int((80e9 * inputs["scale"]) // (768 + 4))
        thr = int(deg[slot >= 0].min())
        assert (deg[slot < 0] <= thr).all()
        B = w["batch"]
        # as bench.py issues them: groups of eight on sixteen pipes, the second queued behind the first
        # with nothing read in between
        counters = list(range(16))
        srv.run_group(list(range(8)), counters[:8], stream=stream)
        srv.run_group(list(range(8, 16)), counters[8:], stream=stream)
        got = [srv.fetch(pipe=k, stream=stream) for k in range(16)]
        srv.run_once(None, batch_counter=19, pipe=0, stream=stream)
        got.append(srv.fetch(pipe=0, stream=stream))
        counters.append(19)
        for c, g in zip(counters, got):
            o = oracle.sample_batch(indptr, indices, info["train"][c * B:(c + 1) * B], w["fanout"], 777 + c)
            assert list(g.node_counter) == list(o.node_counter) and list(g.edge_counter) == list(o.edge_counter)
            for name in ("ids", "agg_src_ids", "agg_src_off", "agg_dst_off"):
                assert np.array_equal(getattr(g, name), getattr(o, name)), name
            assert np.array_equal(g.cache_index, slot[o.ids])
            hit = g.cache_index >= 0
            assert hit.any() and (~hit).any()
            rows = feats[o.ids]
            assert g.features[~hit].tobytes() == rows[~hit].tobytes()
            # the codec works row by row: the oracle's codec on the host rows of the ids that hit is
            # what the cache holds for them
            q, sc = oracle.quantize_rows(rows[hit])
            assert g.features[hit].tobytes() == oracle.dequant_rows(q, sc, np.float16).tobytes()   # 0 ulp (1 allowed)
            x, y = rows[hit].astype(np.float32), g.features[hit].astype(np.float32)
            assert (np.abs(y - x) <= sc[:, None] * 0.5 + np.abs(y) * 2.0 ** -10 + 1e-7).all()
    finally:
        if srv:
            srv.close()
        bench.free_inputs(lmi, inputs)


def test_mag240m_node_count_with_narrow_rows(lmi, oracle):
    """Every node of the MAG240M-shaped graph (244 M nodes, 1.7 B edges: ids need 28 bits, three are
    left for the dedup table's epoch tag) and the full 103.6 M-row int8 cache, with the feature rows
    narrowed to 64 fp16 elements so that the table (31 GB) fits in the pinned memory a box grants."""
    import bench
    if bench.mem_available_gb() < 100:
        pytest.skip("needs 31 GB of pinned host memory plus a 9 GB host copy of the graph")
    w = dict(bench.WORKLOADS["mag240m-int8"])
    cache_rows = int(80e9 // (768 + 4))
    w["dim"] = 64
    w["cache"] = ("int8", float(cache_rows * (w["dim"] + 4)))
    inputs = bench.build_inputs(lmi, w, 778, 0.0)
    srv = None
    try:
        assert inputs["n_nodes"] == 244_160_499, "the 31 GB table was not granted whole"
        srv, info = bench.build_server(lmi, w, inputs, 778, 4)
        assert info["cache_rows"] == cache_rows
        stream = lmi.stream_create()
        feats = info["feats"].array
        indptr = lmi.to_host(info["d_indptr"], info["n_nodes"] + 1, np.int64)
        indices = lmi.to_host(info["d_indices"], info["n_edges"], np.int32)
        assert info["n_edges"] > 1.6e9 and int(indices.max()) >= 1 << 27
        slot = srv.cache_dump(info["n_nodes"])
        cached = slot >= 0
        assert int(cached.sum()) == cache_rows
        deg = np.diff(indptr)
        thr = int(deg[cached].min())
        assert (deg[~cached] <= thr).all()
        # ties at the threshold go to the smaller ids; slots number the cached nodes in id order
        tie = np.flatnonzero(deg == thr)
        n_in = int(cached[tie].sum())
        assert cached[tie[:n_in]].all() and not cached[tie[n_in:]].any()
        assert np.array_equal(slot[cached], np.arange(cache_rows, dtype=slot.dtype))
        del deg, tie
        B = w["batch"]
        # 20 batches on one pipe take the dedup table's epoch tag (3 bits here) once round
        for c in range(20):
            srv.run_once(None, batch_counter=c, pipe=0, stream=stream)
            if c not in (0, 7, 8, 19):
                continue
            g = srv.fetch(pipe=0, stream=stream)
            o = oracle.sample_batch(indptr, indices, info["train"][c * B:(c + 1) * B], w["fanout"], 778 + c)
            assert list(g.node_counter) == list(o.node_counter) and list(g.edge_counter) == list(o.edge_counter)
            for name in ("ids", "agg_src_ids", "agg_src_off", "agg_dst_off"):
                assert np.array_equal(getattr(g, name), getattr(o, name)), name
            assert int(o.ids.max()) >= 1 << 27
            assert np.array_equal(g.cache_index, slot[o.ids])
            hit = g.cache_index >= 0
            assert hit.any() and (~hit).any()
            rows = feats[o.ids]
            assert g.features[~hit].tobytes() == rows[~hit].tobytes()
            q, sc = oracle.quantize_rows(rows[hit])
            assert g.features[hit].tobytes() == oracle.dequant_rows(q, sc, np.float16).tobytes()
        srv.status()   # raises if any of the 20 batches left a fault on record
    finally:
        if srv:
            srv.close()
        bench.free_inputs(lmi, inputs)
