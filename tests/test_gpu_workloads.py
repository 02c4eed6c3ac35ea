"""The five target configurations (Cora-, products-, paper100m-, paper100m-LRU- and
MAG240M-shaped) as parity cases: the synthetic workload
builder of bench.py (graph generated on the GPU) at full size (cora, products,
paper100m in the groups bench.py issues) or at a stated fraction of the node count,
compared with the CPU oracle batch by batch."""
import os
import sys

import numpy as np
import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu
sys.path.insert(0, ROOT)


def build(lmi, name, scale):
    import bench
    w = dict(bench.WORKLOADS[name])
    if scale != 1.0:
        w["nodes"] = max(1000, int(w["nodes"] * scale))
        w["train"] = max(4 * w["batch"], int(w["train"] * scale))
        if w["cache"][0] in ("static", "lru", "int8"):
            w["cache"] = (w["cache"][0], w["cache"][1] * scale)
    srv, info = bench.build_workload(lmi, w, 4242, 2, 8.0)
    indptr = lmi.to_host(info["d_indptr"], info["n_nodes"] + 1, np.int64)
    indices = lmi.to_host(info["d_indices"], info["n_edges"], np.int32)
    return srv, info, w, indptr, indices


def check_batch(g, o):
    assert list(g.node_counter) == list(o.node_counter) and list(g.edge_counter) == list(o.edge_counter)
    for name in ("ids", "agg_src_ids", "agg_src_off", "agg_dst_off"):
        assert np.array_equal(getattr(g, name), getattr(o, name)), name
    for a, b in zip(g.blk_indptr, o.blk_indptr):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("name,scale", [("cora", 1.0), ("products", 1.0), ("paper100m", 0.02)])
def test_static_cache_workloads(lmi, oracle, name, scale):
    srv, info, w, indptr, indices = build(lmi, name, scale)
    stream = lmi.stream_create()
    feats = info["feats"].array
    try:
        slot_ref = oracle.static_cache_build(indptr, info["cache_rows"])
        assert np.array_equal(srv.cache_dump(info["n_nodes"]), slot_ref)
        B = w["batch"]
        for it in range(4):
            srv.run_once(None, batch_counter=it, rng_seed=900 + it, pipe=it % 2, stream=stream)
            g = srv.fetch(pipe=it % 2, stream=stream)
            o = oracle.sample_batch(indptr, indices, info["train"][it * B:(it + 1) * B], w["fanout"], 900 + it)
            check_batch(g, o)
            assert np.array_equal(g.cache_index, slot_ref[o.ids])
            assert g.features.tobytes() == feats[o.ids].tobytes()
            # size-independent properties: COO rows sorted = CSR, degree threshold of the hot set
            for k in range(g.hops):
                e0, e1 = g.edge_off[k], g.edge_off[k] + g.n_edges[k]
                assert np.array_equal(np.bincount(g.agg_dst_off[e0:e1], minlength=g.n_nodes[k]),
                                      np.diff(g.blk_indptr[k]))
            deg = np.diff(indptr)[g.ids]
            hit = g.cache_index >= 0
            if hit.any() and (~hit).any():
                assert deg[hit].min() >= deg[~hit].max()
    finally:
        srv.close()
        info["feats"].free()


def test_lru_workload_with_temporal_locality(lmi, oracle):
    """paper100m-shaped graph at 1/100 of the node count, 3 hops [15,10,5], LRU cache; 80 % of the
    seeds of a batch come from the frontiers of the previous 10 batches."""
    srv, info, w, indptr, indices = build(lmi, "paper100m-lru", 0.01)
    stream = lmi.stream_create()
    feats = info["feats"].array
    rb = feats.shape[1] * 4
    host_rows = feats.view(np.uint8).reshape(feats.shape[0], rb)
    ci = srv.cache_info()
    lru = oracle.Lru(int(ci.n_sets), int(ci.ways), rb)
    rng = np.random.default_rng(4)
    B, recent, hits = 512, [], 0
    try:
        for it in range(14):
            fresh = rng.choice(info["train"], B, replace=False)
            if recent:
                pool = np.unique(np.concatenate(recent[-10:]))
                k = min(int(0.8 * B), len(pool))
                seeds = np.concatenate([rng.choice(pool, k, replace=False), fresh[:B - k]])
            else:
                seeds = fresh
            seeds = np.array(list(dict.fromkeys(seeds.tolist())), np.int32)
            srv.run_once(seeds, rng_seed=70 + it, pipe=0, stream=stream)
            g = srv.fetch(pipe=0, stream=stream)
            o = oracle.sample_batch(indptr, indices, seeds, w["fanout"], 70 + it)
            check_batch(g, o)
            hit, fill, out = lru.access(o.ids, host_rows)
            assert np.array_equal(g.cache_index, hit)
            assert g.features.tobytes() == out.tobytes()
            recent.append(o.ids)
            hits += int((hit >= 0).sum())
        keys, use = srv.cache_dump(int(ci.capacity_rows), with_aux=True)
        okeys, ouse = lru.state()
        assert np.array_equal(keys, okeys) and np.array_equal(use, ouse)
        assert hits > 0
    finally:
        srv.close()
        info["feats"].free()


def test_int8_workload(lmi, oracle):
    """MAG240M-shaped: 768-d fp16 rows, int8 cache with per-row scale, fan-out [25,15], at 1/500 of
    the node count."""
    srv, info, w, indptr, indices = build(lmi, "mag240m-int8", 0.002)
    stream = lmi.stream_create()
    feats = info["feats"].array
    try:
        slot_ref = oracle.static_cache_build(indptr, info["cache_rows"])
        q, sc = oracle.quantize_rows(feats[np.flatnonzero(slot_ref >= 0)])
        B = w["batch"]
        for it in range(3):
            srv.run_once(None, batch_counter=it, rng_seed=30 + it, pipe=it % 2, stream=stream)
            g = srv.fetch(pipe=it % 2, stream=stream)
            o = oracle.sample_batch(indptr, indices, info["train"][it * B:(it + 1) * B], w["fanout"], 30 + it)
            check_batch(g, o)
            assert np.array_equal(g.cache_index, slot_ref[o.ids])
            ref = oracle.gather_rows_int8(o.ids, slot_ref[o.ids], q, sc, feats)
            assert g.features.tobytes() == ref.tobytes()     # 0 ulp (the specification allows 1)
            hit = g.cache_index >= 0
            assert hit.any() and (~hit).any()
            # the codec is lossy but bounded: |y - x| <= scale / 2 (+ fp16 rounding of y)
            x = feats[o.ids][hit].astype(np.float32)
            y = g.features[hit].astype(np.float32)
            bound = sc[slot_ref[o.ids][hit]][:, None] * 0.5 + np.abs(y) * 2.0 ** -10 + 1e-7
            assert (np.abs(y - x) <= bound).all()
    finally:
        srv.close()
        info["feats"].free()


@pytest.fixture(scope="module")
def paper100m_inputs(lmi):
    """The paper100m-shaped graph and feature table at their real size (111 M nodes, 1.6 B edges in
    HBM, 57 GB of rows in pinned host memory), built once for the tests below, with a host copy of
    the graph for the oracle."""
    import bench
    if bench.mem_available_gb() < 90:
        pytest.skip("needs about 75 GB of host memory for the feature table and a host copy of the graph")
    w = dict(bench.WORKLOADS["paper100m"])
    inputs = bench.build_inputs(lmi, w, 20260101, 0.0)
    if inputs["scale"] != 1.0:
        bench.free_inputs(lmi, inputs)
        pytest.skip("this box does not grant the full 57 GB feature table in pinned memory")
    inputs["indptr"] = lmi.to_host(inputs["d_indptr"], inputs["n_nodes"] + 1, np.int64)
    inputs["indices"] = lmi.to_host(inputs["d_indices"], inputs["n_edges"], np.int32)
    yield inputs
    bench.free_inputs(lmi, inputs)


def test_paper100m_hot_set_at_full_size(lmi, oracle, paper100m_inputs):
    """The 38 GB degree-ordered cache of the benchmark's own configuration, read back whole: the hot
    set is everything above the threshold degree plus the lowest ids among the ties, and a node's
    slot is its rank among the cached ids."""
    import bench
    w = dict(bench.WORKLOADS["paper100m"])
    srv, info = bench.build_server(lmi, w, paper100m_inputs, 20260101, 1)
    try:
        deg = np.diff(info["indptr"])
        slot = srv.cache_dump(info["n_nodes"])
        cached = slot >= 0
        thr = int(deg[cached].min())
        assert int(cached.sum()) == info["cache_rows"] and (deg[~cached] <= thr).all()
        ties = np.flatnonzero(deg == thr)
        n_ties_in = int(cached[ties].sum())
        assert cached[ties[:n_ties_in]].all() and not cached[ties[n_ties_in:]].any()
        assert np.array_equal(slot[cached], np.arange(info["cache_rows"], dtype=np.int32))   # slot = rank among cached ids
    finally:
        srv.close()


# (pipes, tuning, sizes of the groups issued back to back with nothing read in between): the last is what
# bench.py issues for the driver's `--steps 20` -- 7, 7, 6 on 16 pipes, batch i in pipe i % 16, so the
# third group takes over pipes of the first while the first group's host-link gather may still run
GROUPED = [(8, {}, [4]), (16, {"miss_blocks": 40}, [8, 8]), (16, {"miss_blocks": 48, "split_lookup": 2}, [7, 7, 6]),
           (16, {"miss_blocks": 48, "split_lookup": 2}, [8, 8, 8]),
           (16, {"miss_blocks": 40, "early_fork": 0}, [8, 8, 8])]


@pytest.mark.parametrize("pipes,tune,sizes", GROUPED,
                         ids=["4on8", "8+8on16", "7+7+6on16-split", "8+8+8on16-split", "8+8+8on16-latefork"])
def test_paper100m_at_full_size_in_groups(lmi, oracle, paper100m_inputs, pipes, tune, sizes):
    """The benchmark's own configuration at its real size (111 M nodes, 38 GB cache), issued exactly as
    bench.py's timed region issues it -- lmi_run_group, the same group sizes, pipes and tuning, every
    group queued before anything is read back: each batch still in a pipe afterwards bit for bit against
    the oracle, plus the properties that hold at any size."""
    import bench
    w = dict(bench.WORKLOADS["paper100m"])
    srv, info = bench.build_server(lmi, w, paper100m_inputs, 20260101, pipes)
    stream = lmi.stream_create()
    feats = info["feats"].array
    indptr, indices = info["indptr"], info["indices"]
    try:
        for k, v in tune.items():
            srv.tune(k, v)
        deg = np.diff(indptr)
        B, fanout = w["batch"], w["fanout"]
        first, holder = 3, {}                         # pipe -> batch counter of the batch it holds at the end
        i = first
        for n in sizes:
            ks = list(range(i, i + n))
            srv.run_group([(k - first) % pipes for k in ks], ks, stream=stream)
            holder.update({(k - first) % pipes: k for k in ks})
            i += n
        assert len(holder) == min(pipes, sum(sizes))
        got = {c: srv.fetch(pipe=p, stream=stream) for p, c in sorted(holder.items())}
        srv.status()
        # the same batch issued alone, later, on another pipe: a batch depends on nothing but its seeds and RNG seed
        c1 = sorted(got)[1]
        spare = (max(holder) + 1) % pipes             # every batch above is on the host by now
        srv.run_once(None, batch_counter=c1, pipe=spare, stream=stream)
        alone = srv.fetch(pipe=spare, stream=stream)
        check_batch(alone, got[c1])
        assert alone.features.tobytes() == got[c1].features.tobytes()
        for n_checked, (c, g) in enumerate(sorted(got.items())):
            seeds = info["train"][c * B:(c + 1) * B]
            o = oracle.sample_batch(indptr, indices, seeds, fanout, 20260101 + c)
            check_batch(g, o)
            assert g.features.tobytes() == feats[g.ids].tobytes()
            hit = g.cache_index >= 0
            assert deg[g.ids][hit].min() >= deg[g.ids][~hit].max()
            if n_checked >= 2:
                continue                              # the closed forms below on the first two batches
            assert np.array_equal(g.ids[:len(seeds)], seeds) and len(np.unique(g.ids)) == len(g.ids)
            n_prev = len(seeds)
            for h in range(g.hops):
                e0, e1 = g.edge_off[h], g.edge_off[h] + g.n_edges[h]
                src, dst = g.agg_src_ids[e0:e1], g.agg_dst_off[e0:e1]
                assert g.n_edges[h] == int(np.minimum(deg[g.ids[:n_prev]], fanout[h]).sum())
                assert np.array_equal(g.ids[g.agg_src_off[e0:e1]], src) and dst.max() < n_prev
                # new nodes are numbered by first appearance in edge order
                new = src[~np.isin(src, g.ids[:n_prev])]
                _, first_at = np.unique(new, return_index=True)
                assert np.array_equal(g.ids[n_prev:g.n_nodes[h + 1]], new[np.sort(first_at)])
                # a node of at most `fanout` neighbours contributes its whole row, in CSR order
                small = np.flatnonzero(deg[g.ids[:n_prev]] <= fanout[h])[:2000]
                rows = g.blk_indptr[h]
                for v in small:
                    assert np.array_equal(src[rows[v]:rows[v + 1]], indices[indptr[g.ids[v]]:indptr[g.ids[v] + 1]])
                # sampled edges exist in the graph (a sample of them), without repeats inside a row
                for e in np.linspace(0, len(src) - 1, 3000).astype(np.int64):
                    d = g.ids[dst[e]]
                    assert src[e] in indices[indptr[d]:indptr[d + 1]]
                n_prev = g.n_nodes[h + 1]
    finally:
        srv.close()


def test_paper100m_lru_at_full_size(lmi, oracle, paper100m_inputs):
    """The LRU configuration at its real shape: the full 111 M-node graph, batches of 4096 seeds,
    fan-out [15,10,5], a 20 GB 8-way LRU cache (39 M rows, 4.9 M sets), 80 % of a batch's seeds drawn
    from the frontiers of the previous 10 batches.  Every batch bit for bit against the oracle's
    sampler and its LRU model (policy only: the model keeps no 20 GB of rows); gathered rows against
    the host table; the final cache state slot by slot."""
    import bench
    w = dict(bench.WORKLOADS["paper100m-lru"])
    srv, info = bench.build_server(lmi, w, paper100m_inputs, 20260101, 2)
    stream = lmi.stream_create()
    feats = info["feats"].array
    indptr, indices = info["indptr"], info["indices"]
    ci = srv.cache_info()
    assert int(ci.ways) == 8 and int(ci.capacity_rows) == 20_000_000_000 // 512 // 8 * 8
    lru = oracle.Lru(int(ci.n_sets), int(ci.ways), 512)
    frac, depth = w["locality"]
    rng = np.random.default_rng(12)
    B, train, recent = w["batch"], info["train"], []
    hits = inserted = 0
    try:
        for it in range(12):
            n_loc = int(frac * B) if recent else 0
            parts = [train[rng.integers(0, len(train), B - n_loc)]]
            if n_loc:
                pool = np.concatenate(recent[-depth:])
                parts.insert(0, pool[rng.integers(0, len(pool), n_loc)])
            seeds = np.array(list(dict.fromkeys(np.concatenate(parts).tolist())), np.int32)   # distinct, order kept
            srv.run_once(seeds, rng_seed=500 + it, pipe=it % 2, stream=stream)
            g = srv.fetch(pipe=it % 2, stream=stream)
            o = oracle.sample_batch(indptr, indices, seeds, w["fanout"], 500 + it)
            check_batch(g, o)
            hit, fill, _ = lru.access(o.ids)
            assert np.array_equal(g.cache_index, hit), "hit/miss set of batch %d" % it
            assert g.features.tobytes() == feats[o.ids].tobytes()
            recent.append(o.ids)
            hits += int((hit >= 0).sum())
            inserted += int((fill >= 0).sum())
        keys, use = srv.cache_dump(int(ci.capacity_rows), with_aux=True)
        okeys, ouse = lru.state()
        assert np.array_equal(keys, okeys) and np.array_equal(use, ouse)
        assert hits > 100_000                               # the locality of the seed plan shows
        assert inserted > int((okeys >= 0).sum())           # some insertions evicted an earlier row
    finally:
        srv.close()
