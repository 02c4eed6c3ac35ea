"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on
the same seeded inputs.  Bit-exact for ids, edges, block CSRs, headers, hit/miss
sets and fp32/fp16 rows."""
import numpy as np
import pytest

from conftest import random_graph

pytestmark = pytest.mark.gpu


def assert_batch_equal(g, o):
    assert list(g.node_counter) == list(o.node_counter)
    assert list(g.edge_counter) == list(o.edge_counter)
    np.testing.assert_array_equal(g.ids, o.ids)
    np.testing.assert_array_equal(g.agg_src_ids, o.agg_src_ids)
    np.testing.assert_array_equal(g.agg_src_off, o.agg_src_off)
    np.testing.assert_array_equal(g.agg_dst_off, o.agg_dst_off)
    for k in range(g.hops):
        np.testing.assert_array_equal(g.blk_indptr[k], o.blk_indptr[k])


def make_features(lmi, rng, n, dim, dtype=np.float32):
    hb = lmi.HostBuffer((n, dim), dtype)
    hb.array[...] = rng.standard_normal((n, dim)).astype(dtype)
    return hb


@pytest.mark.parametrize("fanout,n_nodes,mean_deg,batch", [
    ([25, 10], 3000, 12, 64),
    ([3], 200, 4, 17),
    ([15, 10, 5], 5000, 20, 100),
    ([64, 2], 2000, 30, 50),
    ([1, 1, 1], 500, 3, 31),
    ([5, 33], 4000, 40, 128),
])
def test_sample_batch_parity(lmi, oracle, fanout, n_nodes, mean_deg, batch):
    rng = np.random.default_rng(hash((tuple(fanout), n_nodes)) & 0xFFFF)
    indptr, indices = random_graph(rng, n_nodes, mean_deg, hubs=5, hub_deg=700)
    feats = make_features(lmi, rng, n_nodes, 8)
    srv = lmi.Server(batch, fanout, 8, seed=77)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        for it in range(4):
            seeds = rng.choice(n_nodes, batch, replace=False).astype(np.int32)
            if it == 3:
                seeds = seeds[: batch // 2]  # short batch
            rs = 1000 + it
            srv.run_once(seeds, batch_counter=it, rng_seed=rs)
            g = srv.fetch()
            o = oracle.sample_batch(indptr, indices, seeds, fanout, rs)
            assert_batch_equal(g, o)
            np.testing.assert_array_equal(g.features, feats.array[o.ids])
            assert (g.cache_index == -1).all()
    finally:
        srv.close()
        feats.free()
