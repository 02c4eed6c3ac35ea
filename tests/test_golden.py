"""The committed fixture tests/golden/spec_v1.npz (inputs + the outputs the oracle gave when
it was written, see tests/golden/make_golden.py) against the oracle as it is now (CPU) and
against the HIP path (GPU, without calling the oracle)."""
import os

import numpy as np
import pytest

from conftest import ROOT

G = np.load(os.path.join(ROOT, "tests", "golden", "spec_v1.npz"))
CASES = ["a", "b", "c"]


def batch_fields(b):
    return dict(ids=b.ids, src_ids=b.agg_src_ids, src=b.agg_src_off, dst=b.agg_dst_off, nc=b.node_counter,
                ec=b.edge_counter, indptr=np.concatenate(b.blk_indptr))


@pytest.mark.parametrize("tag", CASES)
def test_oracle_reproduces_the_golden_batches(oracle, tag):
    b = oracle.sample_batch(G["indptr"], G["indices"], G[tag + "_seeds"], list(G[tag + "_fanout"]), int(G[tag + "_rng"]))
    for k, v in batch_fields(b).items():
        np.testing.assert_array_equal(v, G[tag + "_" + k], err_msg=k)


def test_oracle_reproduces_the_golden_caches_and_codec(oracle):
    np.testing.assert_array_equal(oracle.static_cache_build(G["indptr"], int(G["static_cap"])), G["static_slots"])
    rows = G["feats"].view(np.uint8).reshape(len(G["feats"]), 64)
    lru = oracle.Lru(16, 4, 64)
    for k in range(3):
        b = oracle.sample_batch(G["indptr"], G["indices"], G["lru_seeds_%d" % k], [25, 10], 1236 + k)
        hit, fill, _ = lru.access(b.ids, rows)
        np.testing.assert_array_equal(hit, G["lru_hit_%d" % k])
        np.testing.assert_array_equal(fill, G["lru_fill_%d" % k])
    keys, use = lru.state()
    np.testing.assert_array_equal(keys, G["lru_keys"])
    np.testing.assert_array_equal(use, G["lru_use"])
    q, sc = oracle.quantize_rows(G["feats"][:64])
    assert q.tobytes() == G["q32"].tobytes() and sc.tobytes() == G["scale32"].tobytes()
    assert oracle.dequant_rows(q, sc, np.float32).tobytes() == G["deq32"].tobytes()
    q, sc = oracle.quantize_rows(G["feats"][:64].astype(np.float16))
    assert q.tobytes() == G["q16"].tobytes() and sc.tobytes() == G["scale16"].tobytes()
    assert oracle.dequant_rows(q, sc, np.float16).tobytes() == G["deq16"].tobytes()


def gpu_features(lmi, dtype=np.float32):
    hb = lmi.HostBuffer(G["feats"].shape, dtype)
    hb.array[...] = G["feats"].astype(dtype)
    return hb


@pytest.mark.gpu
@pytest.mark.parametrize("tag", CASES)
def test_gpu_reproduces_the_golden_batches(lmi, tag):
    fanout = [int(f) for f in G[tag + "_fanout"]]
    seeds = G[tag + "_seeds"]
    feats = gpu_features(lmi)
    srv = lmi.Server(len(seeds), fanout, 16)
    try:
        srv.load_graph(G["indptr"], G["indices"])
        srv.attach_features(feats)
        srv.build_static_cache(int(G["static_cap"]), lmi.TABLE_RANK)
        np.testing.assert_array_equal(srv.cache_dump(len(G["feats"])), G["static_slots"])
        srv.run_once(seeds, rng_seed=int(G[tag + "_rng"]))
        g = srv.fetch()
        for k, v in batch_fields(g).items():
            np.testing.assert_array_equal(v, G[tag + "_" + k], err_msg=k)
        np.testing.assert_array_equal(g.cache_index, G["static_slots"][G[tag + "_ids"]])
        assert g.features.tobytes() == G["feats"][G[tag + "_ids"]].tobytes()
    finally:
        srv.close()
        feats.free()


@pytest.mark.gpu
def test_gpu_reproduces_the_golden_lru_trace(lmi):
    feats = gpu_features(lmi)
    srv = lmi.Server(48, [25, 10], 16)
    try:
        srv.load_graph(G["indptr"], G["indices"])
        srv.attach_features(feats)
        srv.build_lru_cache(16, 4)
        for k in range(3):
            srv.run_once(G["lru_seeds_%d" % k], rng_seed=1236 + k)
            g = srv.fetch()
            np.testing.assert_array_equal(g.cache_index, G["lru_hit_%d" % k])
            assert g.features.tobytes() == G["feats"][g.ids].tobytes()
        keys, use = srv.cache_dump(64, with_aux=True)
        np.testing.assert_array_equal(keys, G["lru_keys"])
        np.testing.assert_array_equal(use, G["lru_use"])
    finally:
        srv.close()
        feats.free()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tag", [(np.float32, "32"), (np.float16, "16")])
def test_gpu_reproduces_the_golden_int8_rows(lmi, dtype, tag):
    """Rows 0..63 are the whole graph here: every node is cached, so a batch's rows come back
    as the golden dequantised rows of its ids."""
    n = 64
    indptr = np.arange(n + 1, dtype=np.int64)                 # a ring: node v -> v+1
    indices = ((np.arange(n) + 1) % n).astype(np.int32)
    hb = lmi.HostBuffer((n, 16), dtype)
    hb.array[...] = G["feats"][:n].astype(dtype)
    srv = lmi.Server(16, [1], 16, feat_dtype=lmi.F16 if dtype == np.float16 else lmi.F32)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(hb)
        srv.build_int8_cache(n, lmi.TABLE_DIRECT)
        seeds = np.arange(0, 32, 2, dtype=np.int32)
        srv.run_once(seeds, rng_seed=1)
        g = srv.fetch()
        assert (g.cache_index >= 0).all()
        # all degrees are equal, so slots follow ids
        assert g.features.tobytes() == G["deq" + tag][g.ids].tobytes()
    finally:
        srv.close()
        hb.free()
