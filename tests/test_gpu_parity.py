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


@pytest.mark.parametrize("case", range(96))
def test_random_shapes_sweep(lmi, oracle, case):
    """Seeded sweep over shapes the fixed cases do not reach: one-node and two-node graphs,
    edgeless graphs, batches of one seed, repeated seeds, fan-outs 1..64 in any order, hubs with
    more than 2^16 neighbours; static, LRU, int8 or no cache; on a stream or not, two pipes."""
    rng = np.random.default_rng(1000 + case)
    hops = int(rng.integers(1, 4))
    fanout = [int(rng.choice([1, 2, 3, 5, 8, 16, 25, 33, 64])) for _ in range(hops)]
    n_nodes = int(rng.choice([1, 2, 50, 1000, 20000]))
    mean_deg = float(rng.choice([0, 1, 5, 40]))
    batch = int(rng.choice([1, 7, 64, 500]))
    hubs = int(rng.integers(0, 3)) if n_nodes >= 1000 else 0
    indptr, indices = random_graph(rng, n_nodes, mean_deg, hubs=hubs, hub_deg=int(rng.choice([300, 70000])),
                                   zero_frac=float(rng.choice([0.0, 0.3])))
    dim = int(rng.choice([4, 20, 128]))
    feats = make_features(lmi, rng, n_nodes, dim)
    host_rows = feats.array.view(np.uint8).reshape(n_nodes, dim * 4)
    srv = lmi.Server(batch, fanout, dim, pipes=2, seed=5)
    stream = lmi.stream_create() if case % 2 else None
    kind = ["static", "lru", "int8", "none"][case % 4]
    slot_ref = lru = q = sc = None
    try:
        if case % 3 == 0:
            srv.tune("use_graph", 1)
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        cap = int(rng.integers(1, n_nodes + 1))
        if kind == "static":
            srv.build_static_cache(cap, int(rng.integers(0, 3)))
            slot_ref = oracle.static_cache_build(indptr, cap)
        elif kind == "int8":
            srv.build_int8_cache(cap, int(rng.integers(0, 3)))
            slot_ref = oracle.static_cache_build(indptr, cap)
            q, sc = oracle.quantize_rows(feats.array[np.flatnonzero(slot_ref >= 0)])
        elif kind == "lru":
            n_sets, ways = int(rng.integers(1, 40)), int(rng.choice([1, 2, 8]))
            srv.build_lru_cache(n_sets, ways)
            lru = oracle.Lru(n_sets, ways, dim * 4)
        for it in range(3):
            seeds = rng.integers(0, n_nodes, int(rng.integers(1, batch + 1))).astype(np.int32)   # repeats allowed
            srv.run_once(seeds, rng_seed=50 + it, pipe=it % 2, stream=stream)
            g = srv.fetch(pipe=it % 2, stream=stream)
            o = oracle.sample_batch(indptr, indices, seeds, fanout, 50 + it)
            assert_batch_equal(g, o)
            if kind == "lru":
                hit, fill, out = lru.access(o.ids, host_rows)
                np.testing.assert_array_equal(g.cache_index, hit)
                assert g.features.tobytes() == out.tobytes()
            elif kind == "int8":
                np.testing.assert_array_equal(g.cache_index, slot_ref[o.ids])
                assert g.features.tobytes() == oracle.gather_rows_int8(o.ids, slot_ref[o.ids], q, sc, feats.array).tobytes()
            else:
                assert g.features.tobytes() == feats.array[o.ids].tobytes()
                if slot_ref is not None:
                    np.testing.assert_array_equal(g.cache_index, slot_ref[o.ids])
        if kind == "lru":
            keys, use = srv.cache_dump(lru.n_sets * lru.ways, with_aux=True)
            okeys, ouse = lru.state()
            np.testing.assert_array_equal(keys, okeys)
            np.testing.assert_array_equal(use, ouse)
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("fanout", [[25, 10], [64, 3], [5, 4, 3]])
def test_lds_staged_dedup_gives_the_same_batches(lmi, oracle, fanout):
    rng = np.random.default_rng(sum(fanout))
    n_nodes, batch = 2500, 120
    indptr, indices = random_graph(rng, n_nodes, 25, hubs=8, hub_deg=900)   # hubs: many duplicate neighbours per tile
    hot = rng.random(len(indices)) < 0.3
    indices[hot] = rng.integers(0, 20, int(hot.sum()))    # 30 % of all edges point at 20 hot nodes
    feats = make_features(lmi, rng, n_nodes, 8)
    srv = lmi.Server(batch, fanout, 8)
    stream = lmi.stream_create()
    try:
        srv.tune("lds_dedup", 1)
        srv.tune("use_graph", 1)
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        for it in range(4):
            seeds = rng.choice(n_nodes, batch, replace=False).astype(np.int32)
            st = stream if it % 2 else None          # graph replay and eager
            srv.run_once(seeds, rng_seed=40 + it, stream=st)
            assert_batch_equal(srv.fetch(stream=st), oracle.sample_batch(indptr, indices, seeds, fanout, 40 + it))
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("fused", [1, 0])
@pytest.mark.parametrize("batch,fanout", [(96, [25, 10]), (1800, [20, 5]), (700, [64, 2]), (300, [3, 4, 3])])
def test_count_and_sample_in_one_launch_or_two(lmi, oracle, batch, fanout, fused):
    """Both launch shapes of a hop (row counts + scan + sampling fused, or two launches), with
    small tiles (one node per lane group) and full 64-node tiles, against the oracle."""
    rng = np.random.default_rng(batch + fused)
    n_nodes = 6000
    indptr, indices = random_graph(rng, n_nodes, 18, zero_frac=0.1, hubs=6, hub_deg=700)
    feats = make_features(lmi, rng, n_nodes, 4)
    srv = lmi.Server(batch, fanout, 4)
    stream = lmi.stream_create()
    try:
        srv.tune("fuse_count", fused)
        srv.tune("use_graph", 1)
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        for it in range(3):
            seeds = rng.choice(n_nodes, batch if it < 2 else batch // 3, replace=False).astype(np.int32)
            st = stream if it % 2 else None          # graph replay and eager
            srv.run_once(seeds, rng_seed=7 + it, stream=st)
            assert_batch_equal(srv.fetch(stream=st), oracle.sample_batch(indptr, indices, seeds, fanout, 7 + it))
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("epochs", [0, 1, 3])
def test_dedup_table_epochs_wrap(lmi, oracle, epochs):
    """The dedup table is wiped only when its epoch tags run out; with the number of epochs
    capped at 0, 1 or 3 the wipe comes every batch, every 2nd or every 4th batch of a pipe, and
    entries left by earlier batches sit in the table in between."""
    rng = np.random.default_rng(90 + epochs)
    n_nodes, batch, fanout = 3000, 200, [12, 6]
    indptr, indices = random_graph(rng, n_nodes, 14, hubs=4, hub_deg=500)
    feats = make_features(lmi, rng, n_nodes, 4)
    srv = lmi.Server(batch, fanout, 4, pipes=2)
    stream = lmi.stream_create()
    try:
        srv.tune("table_epochs", epochs)
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        for it in range(14):
            # the same few seeds again and again: earlier batches leave exactly the keys the next one probes for
            seeds = rng.choice(400, batch, replace=False).astype(np.int32)
            srv.run_once(seeds, rng_seed=3 + it, pipe=it % 2, stream=stream if it % 3 else None)
            g = srv.fetch(pipe=it % 2, stream=stream if it % 3 else None)
            assert_batch_equal(g, oracle.sample_batch(indptr, indices, seeds, fanout, 3 + it))
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("cache", ["static", "int8", "none"])
@pytest.mark.parametrize("group,fanout", [(2, [25, 10]), (3, [6, 4, 3]), (4, [64, 2]), (8, [5])])
@pytest.mark.parametrize("split_lookup", [0, 2])
def test_groups_of_batches_share_their_launches(lmi, oracle, group, fanout, cache, split_lookup):
    """lmi_run_group: several mini-batches, each in its own pipe, go through the same kernel
    launches; every one of them must come out as if it had been run alone.  split_lookup: with two hops
    or more and a cache, the seeds and the first hop's nodes are looked up, and their misses fetched,
    before the later hops are sampled (no difference for one hop or without a cache)."""
    rng = np.random.default_rng(group * 10 + len(fanout))
    n_nodes, batch, dim = 5000, 150, 16
    indptr, indices = random_graph(rng, n_nodes, 15, hubs=5, hub_deg=600)
    feats = make_features(lmi, rng, n_nodes, dim)
    train = rng.permutation(n_nodes)[:4000].astype(np.int32)
    srv = lmi.Server(batch, fanout, dim, pipes=group, seed=9)
    stream = lmi.stream_create()
    slot_ref = q = sc = None
    try:
        if group == 3:
            srv.tune("protect_hits", 1)   # HBM gathers held back until earlier host-link gathers have drained
        if group == 4:
            srv.tune("group_miss", 0)     # one host-link gather launch per batch instead of one per group
        srv.tune("split_lookup", split_lookup)
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.load_idset(lmi.MODE_TRAIN, train)
        if cache == "static":
            srv.build_static_cache(1800, lmi.TABLE_RANK)
            slot_ref = oracle.static_cache_build(indptr, 1800)
        elif cache == "int8":
            srv.build_int8_cache(1800, lmi.TABLE_HASH)
            slot_ref = oracle.static_cache_build(indptr, 1800)
            q, sc = oracle.quantize_rows(feats.array[np.flatnonzero(slot_ref >= 0)])
        for rnd in range(3):
            pipes = list(range(group))
            if rnd == 1:   # caller seeds of different lengths, one batch short, one with a repeat
                seeds = [rng.choice(n_nodes, int(rng.integers(1, batch + 1)), replace=False).astype(np.int32)
                         for _ in pipes]
                seeds[0][-1] = seeds[0][0]
                srv.run_group(pipes, [0] * group, seeds=seeds, rng_seeds=[200 + k for k in pipes], stream=stream)
                want = [(seeds[k], 200 + k) for k in pipes]
            else:          # slices of the id set, default RNG seeds (server seed + batch counter)
                counters = [rnd * group + k for k in pipes]
                srv.run_group(pipes, counters, stream=stream if rnd else None)
                want = [(train[c * batch:(c + 1) * batch], 9 + c) for c in counters]
            for k in pipes:
                g = srv.fetch(pipe=k, stream=stream if rnd else None)
                o = oracle.sample_batch(indptr, indices, want[k][0], fanout, want[k][1])
                assert_batch_equal(g, o)
                if cache == "int8":
                    ref = oracle.gather_rows_int8(o.ids, slot_ref[o.ids], q, sc, feats.array)
                    assert g.features.tobytes() == ref.tobytes()
                else:
                    assert g.features.tobytes() == feats.array[o.ids].tobytes()
                if slot_ref is not None:
                    np.testing.assert_array_equal(g.cache_index, slot_ref[o.ids])
        # a group may not name a pipe twice, and the LRU cache takes one batch at a time
        with pytest.raises(lmi.LegionError):
            srv.run_group([0, 0], [0, 1])
        if group > 1:
            srv.build_lru_cache(32, 4)
            with pytest.raises(lmi.LegionError):
                srv.run_group([0, 1], [0, 1])
            srv.run_group([0], [0])
            g = srv.fetch(pipe=0)
            assert_batch_equal(g, oracle.sample_batch(indptr, indices, train[:batch], fanout, 9))
    finally:
        srv.close()
        feats.free()


def test_duplicate_seeds_and_isolated_nodes(lmi, oracle):
    rng = np.random.default_rng(5)
    indptr, indices = random_graph(rng, 300, 6, zero_frac=0.4)
    feats = make_features(lmi, rng, 300, 4)
    srv = lmi.Server(32, [4, 3], 4)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        seeds = rng.integers(0, 300, 32).astype(np.int32)
        seeds[5] = seeds[1]
        seeds[20] = seeds[1]
        srv.run_once(seeds, rng_seed=9)
        assert_batch_equal(srv.fetch(), oracle.sample_batch(indptr, indices, seeds, [4, 3], 9))
        # empty batch
        srv.run_once(np.zeros(0, np.int32), rng_seed=9)
        g = srv.fetch()
        assert g.n_nodes == [0, 0, 0] and g.n_edges == [0, 0]
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("cache", ["static", "int8", "lru", "none"])
def test_empty_and_one_seed_batches_between_full_ones(lmi, oracle, cache):
    """Ragged use: an empty batch, a batch of one isolated seed and a batch of one hub, alone and
    inside a group with full batches; the caches and the pipes carry on as if nothing had happened."""
    rng = np.random.default_rng(41)
    n_nodes, dim, fanout = 3000, 32, [6, 5]
    indptr, indices = random_graph(rng, n_nodes, 8, hubs=3, hub_deg=900, zero_frac=0.2)
    deg = np.diff(indptr)
    feats = make_features(lmi, rng, n_nodes, dim)
    srv = lmi.Server(64, fanout, dim, pipes=4)
    stream = lmi.stream_create()
    lru = oracle.Lru(64, 4, dim * 4)
    host_rows = feats.array.view(np.uint8).reshape(n_nodes, dim * 4)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        if cache == "static":
            srv.build_static_cache(800, lmi.TABLE_RANK)
            slot = oracle.static_cache_build(indptr, 800)
        elif cache == "int8":
            srv.build_int8_cache(800, lmi.TABLE_HASH)
            slot = oracle.static_cache_build(indptr, 800)
            q, sc = oracle.quantize_rows(feats.array[np.flatnonzero(slot >= 0)])
        elif cache == "lru":
            srv.build_lru_cache(64, 4)
        full = lambda: rng.choice(n_nodes, 64, replace=False).astype(np.int32)
        isolated = np.array([int(np.flatnonzero(deg == 0)[0])], np.int32)
        hub = np.array([int(np.argmax(deg))], np.int32)
        batches = [full(), np.zeros(0, np.int32), isolated, full(), hub, np.zeros(0, np.int32), full()]

        def check(g, seeds, rng_seed):
            o = oracle.sample_batch(indptr, indices, seeds, fanout, rng_seed)
            assert_batch_equal(g, o)
            if cache in ("static", "int8"):
                assert np.array_equal(g.cache_index, slot[o.ids])
            if cache == "int8":
                want = oracle.gather_rows_int8(o.ids, slot[o.ids], q, sc, feats.array)
            elif cache == "lru":
                hit, _, want = lru.access(o.ids, host_rows)
                assert np.array_equal(g.cache_index, hit)
            else:
                want = feats.array[o.ids]
            assert g.features.tobytes() == want.tobytes()
            if len(seeds) == 0:
                assert g.n_nodes == [0, 0, 0] and g.n_edges == [0, 0] and len(g.ids) == 0

        for t, seeds in enumerate(batches):          # one after the other
            srv.run_once(seeds, rng_seed=60 + t, pipe=t % 4, stream=stream)
            check(srv.fetch(pipe=t % 4, stream=stream), seeds, 60 + t)
        if cache != "lru":                           # and four at a time, the empty ones among them
            for first in (0, 3):
                group = batches[first:first + 4]
                srv.run_group([0, 1, 2, 3], [0] * 4, seeds=group, rng_seeds=[80 + first + k for k in range(4)], stream=stream)
                for k, seeds in enumerate(group):
                    check(srv.fetch(pipe=k, stream=stream), seeds, 80 + first + k)
        srv.status()
    finally:
        srv.close()
        feats.free()


def test_bad_seed_is_reported(lmi):
    rng = np.random.default_rng(6)
    indptr, indices = random_graph(rng, 100, 5)
    feats = make_features(lmi, rng, 100, 4)
    srv = lmi.Server(8, [3], 4)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.run_once(np.array([1, 2, 100, 3], np.int32), rng_seed=1)
        with pytest.raises(lmi.LegionError) as ei:
            srv.counters()
        assert ei.value.code == -5
        with pytest.raises(lmi.LegionError):
            srv.run_once(np.zeros(9, np.int32))  # more seeds than batch_size
    finally:
        srv.close()
        feats.free()


def test_a_bad_seed_stays_on_record_until_cleared(lmi, oracle):
    """The per-batch flag is wiped by the pipe's next batch; the server's own record is not: a
    caller that never reads a batch's counters (the runner loop, a benchmark) still learns of it,
    without touching the device."""
    rng = np.random.default_rng(16)
    indptr, indices = random_graph(rng, 400, 6)
    feats = make_features(lmi, rng, 400, 8)
    srv = lmi.Server(8, [3, 2], 8, pipes=2)
    stream = lmi.stream_create()
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.run_once(np.array([1, 2, 3], np.int32), rng_seed=1, stream=stream)
        srv.fetch(stream=stream)
        srv.status()                                         # nothing on record
        srv.batch_wait(stream=stream)
        srv.run_once(np.array([5, 400, -7, 9], np.int32), rng_seed=2, stream=stream)   # two ids outside [0, 400)
        lmi.check(lmi.lib().lmi_stream_sync(stream))
        good = np.array([7, 8, 9, 10], np.int32)
        srv.run_once(good, rng_seed=3, stream=stream)        # same pipe: wipes the per-batch flag
        g = srv.fetch(stream=stream)                         # ... so the counters no longer complain
        o = oracle.sample_batch(indptr, indices, good, [3, 2], 3)
        assert np.array_equal(g.ids, o.ids)
        with pytest.raises(lmi.LegionError) as ei:
            srv.status()
        assert ei.value.code == -5 and "seed id outside" in str(ei.value)
        with pytest.raises(lmi.LegionError) as ei:
            srv.batch_wait(stream=stream)                    # the same code where the runner joins a batch ...
        assert ei.value.code == -5
        srv.batch_wait(stream=stream)                        # ... once: the good batches after it wait in peace
        with pytest.raises(lmi.LegionError):
            srv.status()                                     # while the server's own record stays
        with pytest.raises(lmi.LegionError):
            srv.status(clear=True)                           # reports once more, then forgets
        srv.status()
        srv.batch_wait(stream=stream)
        srv.run_once(np.array([5, 401], np.int32), rng_seed=4, stream=stream)   # a new condition after the clear
        lmi.check(lmi.lib().lmi_stream_sync(stream))
        with pytest.raises(lmi.LegionError):
            srv.batch_wait(stream=stream)                    # is reported again, once
        srv.batch_wait(stream=stream)
        with pytest.raises(lmi.LegionError):
            srv.status(clear=True)
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("table", [0, 1, 2])
@pytest.mark.parametrize("dim,dtype", [(128, np.float32), (100, np.float32), (1433, np.float32), (768, np.float16),
                                        (6, np.float16),      # 12-byte rows: under one 16-byte unit
                                        (5, np.float32),      # 20 bytes: two units that overlap by 12
                                        (17, np.float32),     # 68 bytes: four whole units and a 4-byte tail
                                        (102, np.float32),    # 408 bytes: 8-byte aligned rows
                                        (4, np.float32)])     # 16 bytes: one unit per row
def test_static_cache_parity(lmi, oracle, table, dim, dtype):
    rng = np.random.default_rng(dim + table)
    n_nodes, batch, fanout = 4000, 96, [10, 5]
    indptr, indices = random_graph(rng, n_nodes, 8, hubs=10, hub_deg=300)
    feats = make_features(lmi, rng, n_nodes, dim, dtype)
    srv = lmi.Server(batch, fanout, dim, feat_dtype=lmi.F16 if dtype == np.float16 else lmi.F32)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        for cap in (1, 1200, n_nodes):
            srv.build_static_cache(cap, table)
            slot_ref = oracle.static_cache_build(indptr, cap)
            np.testing.assert_array_equal(srv.cache_dump(n_nodes), slot_ref)
            seeds = rng.choice(n_nodes, batch, replace=False).astype(np.int32)
            srv.run_once(seeds, rng_seed=cap)
            g = srv.fetch()
            o = oracle.sample_batch(indptr, indices, seeds, fanout, cap)
            assert_batch_equal(g, o)
            np.testing.assert_array_equal(g.cache_index, slot_ref[o.ids])
            assert g.features.tobytes() == feats.array[o.ids].tobytes()
    finally:
        srv.close()
        feats.free()


def test_operator_chain_matches_run_once(lmi, oracle):
    """The five reference operator slots, called one by one, give the same batch."""
    rng = np.random.default_rng(11)
    n_nodes, batch, fanout, dim = 3000, 50, [6, 4, 3], 32
    indptr, indices = random_graph(rng, n_nodes, 10)
    feats = make_features(lmi, rng, n_nodes, dim)
    train = rng.permutation(n_nodes)[:230].astype(np.int32)
    labels = (train % 7).astype(np.int32)
    srv = lmi.Server(batch, fanout, dim, seed=5)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.load_idset(lmi.MODE_TRAIN, train, labels)
        srv.build_static_cache(1000)
        slot_ref = oracle.static_cache_build(indptr, 1000)
        for it in range(5):  # 230 ids / 50 -> last batch has 30 seeds
            srv.op_batch_generate(None, batch_counter=it)
            srv.op_cache_lookup(0)
            srv.op_io_submit()
            for k in range(3):
                srv.op_random_sample(k)
                srv.op_cache_lookup(k + 1)
                srv.op_io_submit()
            srv.op_io_complete()
            g = srv.fetch()
            seeds = train[it * batch:(it + 1) * batch]
            o = oracle.sample_batch(indptr, indices, seeds, fanout, 5 + it)
            assert_batch_equal(g, o)
            np.testing.assert_array_equal(g.labels, labels[it * batch:(it + 1) * batch])
            np.testing.assert_array_equal(g.cache_index, slot_ref[o.ids])
            assert g.features.tobytes() == feats.array[o.ids].tobytes()
        with pytest.raises(lmi.LegionError):
            srv.op_batch_generate(None, batch_counter=5)  # past the end of the id set
    finally:
        srv.close()
        feats.free()


def test_id_set_sliced_at_its_own_batch_size(lmi, oracle):
    """Validation / test sets are served in batches of their own size (the reference's
    GetCurrentBatchsize): 130 ids at 40 a batch -> 40, 40, 40, 10."""
    rng = np.random.default_rng(12)
    n_nodes, batch, fanout, dim = 2000, 64, [5, 3], 8
    indptr, indices = random_graph(rng, n_nodes, 8)
    feats = make_features(lmi, rng, n_nodes, dim)
    valid = rng.permutation(n_nodes)[:130].astype(np.int32)
    labels = (valid % 5).astype(np.int32)
    srv = lmi.Server(batch, fanout, dim, seed=3)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.load_idset(lmi.MODE_VALID, valid, labels)
        with pytest.raises(lmi.LegionError):
            srv.idset_batch(lmi.MODE_VALID, batch + 1)   # more than the output buffers hold
        with pytest.raises(lmi.LegionError):
            srv.idset_batch(lmi.MODE_VALID, 0)
        srv.idset_batch(lmi.MODE_VALID, 40)
        for it in range(4):
            srv.run_once(None, batch_counter=it, mode=lmi.MODE_VALID)
            g = srv.fetch()
            assert_batch_equal(g, oracle.sample_batch(indptr, indices, valid[it * 40:(it + 1) * 40], fanout, 3 + it))
            np.testing.assert_array_equal(g.labels, labels[it * 40:(it + 1) * 40])
        with pytest.raises(lmi.LegionError):
            srv.run_once(None, batch_counter=4, mode=lmi.MODE_VALID)
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("cache", ["static", "int8", "lru"])
@pytest.mark.parametrize("dim,dtype", [(128, np.float32), (100, np.float32), (768, np.float16)])
def test_hits_come_from_hbm_and_misses_from_the_host(lmi, oracle, cache, dim, dtype):
    """A cached fp32 row equals its host row byte for byte, so equality with the host table cannot
    tell which copy a hit was served from.  Here every host row is overwritten AFTER the cache was
    filled: hits must still return what was cached, misses must return the new host bytes."""
    rng = np.random.default_rng(dim + len(cache))
    n_nodes, batch, fanout = 6000, 200, [10, 5]
    indptr, indices = random_graph(rng, n_nodes, 9, hubs=5, hub_deg=700)
    feats = make_features(lmi, rng, n_nodes, dim, dtype)
    orig = feats.array.copy()
    srv = lmi.Server(batch, fanout, dim, feat_dtype=lmi.F16 if dtype == np.float16 else lmi.F32)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        seeds = rng.choice(n_nodes, batch, replace=False).astype(np.int32)
        if cache == "lru":
            srv.build_lru_cache(1024, 8)              # room for every row of the batches below
            srv.run_once(seeds[:batch // 2], rng_seed=5)   # cold: every row misses and is inserted
            first = srv.fetch()
            assert (first.cache_index < 0).all() and first.features.tobytes() == orig[first.ids].tobytes()
        elif cache == "static":
            srv.build_static_cache(2000, lmi.TABLE_RANK)
        else:
            srv.build_int8_cache(2000, lmi.TABLE_RANK)
        # poison: no host row keeps a single one of its bytes
        feats.array[...] = (orig.astype(np.float32) + 100.0).astype(dtype)
        poisoned = feats.array.copy()
        assert not (poisoned == orig).any()
        srv.run_once(seeds, rng_seed=5)
        g = srv.fetch()
        hit = g.cache_index >= 0
        assert hit.any() and (~hit).any()
        assert g.features[~hit].tobytes() == poisoned[g.ids[~hit]].tobytes()      # over the host link
        if cache == "int8":
            q, sc = oracle.quantize_rows(orig[g.ids[hit]])
            want = oracle.dequant_rows(q, sc, dtype)
        else:
            want = orig[g.ids[hit]]
        assert g.features[hit].tobytes() == want.tobytes()                          # from the copy in HBM
        if cache == "lru":
            # what the second batch inserted was gathered from the poisoned host rows
            srv.run_once(seeds, rng_seed=5)
            g3 = srv.fetch()
            was_miss = ~hit
            now_hit = g3.cache_index >= 0
            assert (now_hit & was_miss).any()
            assert g3.features[now_hit & was_miss].tobytes() == poisoned[g3.ids[now_hit & was_miss]].tobytes()
            assert g3.features[now_hit & hit].tobytes() == orig[g3.ids[now_hit & hit]].tobytes()
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("n_sets,ways", [(64, 8), (16, 4), (1, 32), (500, 2)])
def test_lru_cache_parity(lmi, oracle, n_sets, ways):
    """Reference-shaped toy workload (comp_cache/tests/test_cache.cu:4-9,48-53):
    1000 nodes, 130 hot ones, 90 % of the seeds hot -- replayed on both sides."""
    rng = np.random.default_rng(n_sets * 100 + ways)
    n_nodes, batch, fanout, dim = 1000, 128, [3, 2], 32
    indptr, indices = random_graph(rng, n_nodes, 6)
    feats = make_features(lmi, rng, n_nodes, dim)
    hot = rng.choice(n_nodes, 130, replace=False)
    srv = lmi.Server(batch, fanout, dim)
    lru = oracle.Lru(n_sets, ways, dim * 4)
    host_rows = feats.array.view(np.uint8).reshape(n_nodes, dim * 4)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.build_lru_cache(n_sets, ways)
        for it in range(12):
            k_hot = int(batch * 0.9)
            seeds = np.concatenate([rng.choice(hot, k_hot, replace=False),
                                    rng.choice(n_nodes, batch - k_hot, replace=False)]).astype(np.int32)
            seeds = np.array(list(dict.fromkeys(seeds.tolist())), np.int32)
            srv.run_once(seeds, rng_seed=it + 1)
            g = srv.fetch()
            o = oracle.sample_batch(indptr, indices, seeds, fanout, it + 1)
            assert_batch_equal(g, o)
            hit, fill, out = lru.access(o.ids, host_rows)
            np.testing.assert_array_equal(g.cache_index, hit)
            assert g.features.tobytes() == out.tobytes()
            keys, use = srv.cache_dump(n_sets * ways, with_aux=True)
            okeys, ouse = lru.state()
            np.testing.assert_array_equal(keys, okeys)
            np.testing.assert_array_equal(use, ouse)
        assert (hit >= 0).sum() > 0
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("schedule", [0, 1, 2])
def test_lru_batches_in_flight_on_two_pipes(lmi, oracle, schedule):
    """Four batches are issued back to back on alternating pipes before any is read: the
    sampling of a batch may overlap the host-link gather and the insertion of the one before
    it, but every lookup sees the cache after the previous batch's insertion."""
    rng = np.random.default_rng(77 + schedule)
    n_nodes, batch, fanout, dim = 4000, 256, [6, 4], 64
    indptr, indices = random_graph(rng, n_nodes, 8, hubs=4, hub_deg=300)
    feats = make_features(lmi, rng, n_nodes, dim)
    hot = rng.choice(n_nodes, 400, replace=False)
    srv = lmi.Server(batch, fanout, dim, pipes=2)
    lru = oracle.Lru(96, 4, dim * 4)
    host_rows = feats.array.view(np.uint8).reshape(n_nodes, dim * 4)
    stream = lmi.stream_create()
    try:
        srv.tune("split_miss", schedule)
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.build_lru_cache(96, 4)
        for rnd in range(5):
            group = []
            for k in range(4):
                seeds = np.concatenate([rng.choice(hot, 200, replace=False), rng.choice(n_nodes, 56, replace=False)])
                seeds = np.array(list(dict.fromkeys(seeds.tolist())), np.int32)
                group.append(seeds)
            # two in flight at a time (a pipe's buffers are reused by the batch after next)
            for half in (0, 2):
                for k in (half, half + 1):
                    srv.run_once(group[k], rng_seed=100 + rnd * 4 + k, pipe=k % 2, stream=stream)
                for k in (half, half + 1):
                    g = srv.fetch(pipe=k % 2, stream=stream)
                    o = oracle.sample_batch(indptr, indices, group[k], fanout, 100 + rnd * 4 + k)
                    assert_batch_equal(g, o)
                    hit, fill, out = lru.access(o.ids, host_rows)
                    np.testing.assert_array_equal(g.cache_index, hit)
                    assert g.features.tobytes() == out.tobytes()
        keys, use = srv.cache_dump(96 * 4, with_aux=True)
        okeys, ouse = lru.state()
        np.testing.assert_array_equal(keys, okeys)
        np.testing.assert_array_equal(use, ouse)
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("n_sets,ways", [(1, 2), (3, 4), (40, 2)])
def test_lru_with_repeated_seeds(lmi, oracle, n_sets, ways):
    """A repeated seed keeps both of its rows, but its id is offered to the cache once."""
    rng = np.random.default_rng(n_sets + ways)
    n_nodes, batch, fanout, dim = 600, 64, [4, 2], 8
    indptr, indices = random_graph(rng, n_nodes, 5)
    feats = make_features(lmi, rng, n_nodes, dim)
    srv = lmi.Server(batch, fanout, dim)
    lru = oracle.Lru(n_sets, ways, dim * 4)
    host_rows = feats.array.view(np.uint8).reshape(n_nodes, dim * 4)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.build_lru_cache(n_sets, ways)
        for it in range(8):
            seeds = rng.integers(0, 60, batch).astype(np.int32)      # 64 draws from 60 ids: many repeats
            srv.run_once(seeds, rng_seed=it + 1)
            g = srv.fetch()
            o = oracle.sample_batch(indptr, indices, seeds, fanout, it + 1)
            assert_batch_equal(g, o)
            hit, fill, out = lru.access(o.ids, host_rows)
            np.testing.assert_array_equal(g.cache_index, hit)
            assert g.features.tobytes() == out.tobytes()
            keys, use = srv.cache_dump(n_sets * ways, with_aux=True)
            okeys, ouse = lru.state()
            np.testing.assert_array_equal(keys, okeys)
            np.testing.assert_array_equal(use, ouse)
            live = keys[keys >= 0]
            assert len(set(live.tolist())) == len(live)              # no id cached twice
    finally:
        srv.close()
        feats.free()


def test_lru_operator_chain(lmi, oracle):
    rng = np.random.default_rng(3)
    n_nodes, batch, fanout, dim = 800, 40, [4, 3], 16
    indptr, indices = random_graph(rng, n_nodes, 6)
    feats = make_features(lmi, rng, n_nodes, dim)
    srv = lmi.Server(batch, fanout, dim)
    lru = oracle.Lru(32, 4, dim * 4)
    host_rows = feats.array.view(np.uint8).reshape(n_nodes, dim * 4)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.build_lru_cache(32, 4)
        for it in range(6):
            seeds = rng.choice(200, batch, replace=False).astype(np.int32)
            srv.op_batch_generate(seeds, rng_seed=it + 1)
            srv.op_cache_lookup(0)
            for k in range(2):
                srv.op_random_sample(k)
                srv.op_cache_lookup(k + 1)
            srv.op_io_complete()
            g = srv.fetch()
            o = oracle.sample_batch(indptr, indices, seeds, fanout, it + 1)
            assert_batch_equal(g, o)
            hit, fill, out = lru.access(o.ids, host_rows)
            np.testing.assert_array_equal(g.cache_index, hit)
            assert g.features.tobytes() == out.tobytes()
            keys, use = srv.cache_dump(128, with_aux=True)
            okeys, ouse = lru.state()
            np.testing.assert_array_equal(keys, okeys)
            np.testing.assert_array_equal(use, ouse)
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("dim,dtype", [(768, np.float16), (128, np.float32), (100, np.float32), (48, np.float16),
                                        (6, np.float16)])
def test_int8_cache_parity(lmi, oracle, dim, dtype):
    rng = np.random.default_rng(dim)
    n_nodes, batch, fanout = 3000, 64, [8, 4]
    indptr, indices = random_graph(rng, n_nodes, 8, hubs=4, hub_deg=200)
    feats = make_features(lmi, rng, n_nodes, dim, dtype)
    feats.array[7] = 0            # all-zero row: scale 0
    feats.array[11, 0] = 3.0      # clear absmax
    srv = lmi.Server(batch, fanout, dim, feat_dtype=lmi.F16 if dtype == np.float16 else lmi.F32)
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        cap = 2000
        srv.build_int8_cache(cap)
        slot_ref = oracle.static_cache_build(indptr, cap)
        np.testing.assert_array_equal(srv.cache_dump(n_nodes), slot_ref)
        cached = np.flatnonzero(slot_ref >= 0)
        q, sc = oracle.quantize_rows(feats.array[cached])
        for it in range(3):
            seeds = rng.choice(n_nodes, batch, replace=False).astype(np.int32)
            if it == 0:
                seeds[:2] = [7, 11]
            srv.run_once(seeds, rng_seed=it + 1)
            g = srv.fetch()
            o = oracle.sample_batch(indptr, indices, seeds, fanout, it + 1)
            assert_batch_equal(g, o)
            np.testing.assert_array_equal(g.cache_index, slot_ref[o.ids])
            ref = oracle.gather_rows_int8(o.ids, slot_ref[o.ids], q, sc, feats.array)
            # tolerance: the specification allows 1 ulp on dequantised rows; both sides do one IEEE
            # multiply (+ RNE to fp16), so the expected difference is 0
            assert g.features.tobytes() == ref.tobytes()
    finally:
        srv.close()
        feats.free()


def test_synth_graph_matches_oracle(lmi, oracle):
    cdf = lmi.zipf_cdf(2.0, 500, 9.0)
    for mode in (0, 1):
        ip, ix, ne = lmi.synth_graph(42, cdf, 20000, mode)
        indptr = lmi.to_host(ip, 20001, np.int64)
        indices = lmi.to_host(ix, ne, np.int32)
        o_indptr, o_indices = oracle.synth_graph(42, cdf, 20000, mode)
        np.testing.assert_array_equal(indptr, o_indptr)
        np.testing.assert_array_equal(indices, o_indices)
        lmi.check(lmi.lib().lmi_device_free(ip))
        lmi.check(lmi.lib().lmi_device_free(ix))
    np.testing.assert_array_equal(lmi.synth_trainset(7, 20000, 1500), oracle.synth_trainset(7, 20000, 1500))
    mean = np.diff(indptr).mean()
    assert 8.0 < mean < 10.0


@pytest.mark.parametrize("schedule", [0, 1, 2])
@pytest.mark.parametrize("cache", ["static", "lru", "int8"])
def test_graph_replay_matches_eager_and_oracle(lmi, oracle, cache, schedule):
    """lmi_run_once on a real stream replays a captured HIP graph; every replay is
    checked against the oracle, with eager batches and synchronisations in between."""
    rng = np.random.default_rng(21)
    n_nodes, batch, fanout, dim = 6000, 200, [10, 5, 3], 64
    indptr, indices = random_graph(rng, n_nodes, 9, hubs=6, hub_deg=400)
    feats = make_features(lmi, rng, n_nodes, dim)
    host_rows = feats.array.view(np.uint8).reshape(n_nodes, dim * 4)
    train = rng.permutation(n_nodes)[:1000].astype(np.int32)
    srv = lmi.Server(batch, fanout, dim, pipes=2, seed=9)
    streams = [lmi.stream_create(), lmi.stream_create()]
    lru = oracle.Lru(128, 4, dim * 4)
    try:
        srv.tune("split_miss", schedule)   # where the HBM and host-link gathers run (caller / side stream)
        srv.tune("use_graph", 1)           # batches on a real stream replay a captured graph
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.load_idset(lmi.MODE_TRAIN, train)
        if cache == "static":
            srv.build_static_cache(2500, lmi.TABLE_RANK)
            slot_ref = oracle.static_cache_build(indptr, 2500)
        elif cache == "int8":
            srv.build_int8_cache(2500, lmi.TABLE_RANK)
            slot_ref = oracle.static_cache_build(indptr, 2500)
            q, sc = oracle.quantize_rows(feats.array[np.flatnonzero(slot_ref >= 0)])
        else:
            srv.build_lru_cache(128, 4)
        for it in range(10):
            pipe = it % 2
            graph = it % 3 != 2          # every third batch runs eagerly on the default stream
            if it == 6:
                seeds = rng.choice(n_nodes, 77, replace=False).astype(np.int32)   # caller seeds, short batch
                ref_seeds = seeds
            else:
                seeds = None
                ref_seeds = train[(it % 5) * batch:(it % 5 + 1) * batch]
            st = streams[pipe] if graph else None
            srv.run_once(seeds, batch_counter=it % 5, rng_seed=50 + it, pipe=pipe, stream=st)
            g = srv.fetch(pipe=pipe, stream=st)
            o = oracle.sample_batch(indptr, indices, ref_seeds, fanout, 50 + it)
            assert_batch_equal(g, o)
            if cache == "static":
                np.testing.assert_array_equal(g.cache_index, slot_ref[o.ids])
                assert g.features.tobytes() == feats.array[o.ids].tobytes()
            elif cache == "int8":
                ref = oracle.gather_rows_int8(o.ids, slot_ref[o.ids], q, sc, feats.array)
                assert g.features.tobytes() == ref.tobytes()
            else:
                hit, fill, out = lru.access(o.ids, host_rows)
                np.testing.assert_array_equal(g.cache_index, hit)
                assert g.features.tobytes() == out.tobytes()
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("int8", [False, True])
def test_presampled_hot_set_policy(lmi, oracle, int8):
    """The reference's own cache policy: presample the training batches, count how often every
    node is sampled, cache the most frequently sampled rows (ties by id)."""
    rng = np.random.default_rng(17)
    n_nodes, batch, fanout, dim, n_train = 4000, 80, [10, 5], 32, 400
    indptr, indices = random_graph(rng, n_nodes, 9, hubs=6, hub_deg=500)
    feats = make_features(lmi, rng, n_nodes, dim)
    train = rng.permutation(n_nodes)[:n_train].astype(np.int32)
    srv = lmi.Server(batch, fanout, dim, seed=23)
    stream = lmi.stream_create()
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.load_idset(lmi.MODE_TRAIN, train)
        with pytest.raises(lmi.LegionError):
            srv.cache_policy(lmi.POLICY_PRESAMPLED)
            srv.build_static_cache(500)            # nothing presampled yet
        srv.presample(3, first_batch=0, stream=stream)
        srv.presample(2, first_batch=3, stream=stream)
        counts = np.zeros(n_nodes, np.int64)
        for b in range(5):
            o = oracle.sample_batch(indptr, indices, train[b * batch:(b + 1) * batch], fanout, 23 + b)
            counts += np.bincount(o.ids, minlength=n_nodes)
        assert np.array_equal(srv.hotness(n_nodes).astype(np.int64), counts)
        cap = 700
        slot_ref = oracle.static_cache_build_keys(counts, cap)
        if int8:
            srv.build_int8_cache(cap, lmi.TABLE_RANK)
            q, sc = oracle.quantize_rows(feats.array[np.flatnonzero(slot_ref >= 0)])
        else:
            srv.build_static_cache(cap, lmi.TABLE_HASH)
        assert np.array_equal(srv.cache_dump(n_nodes), slot_ref)
        assert not np.array_equal(slot_ref >= 0, oracle.static_cache_build(indptr, cap) >= 0)  # differs from degree order
        srv.run_once(None, batch_counter=1, stream=stream)
        g = srv.fetch(stream=stream)
        o = oracle.sample_batch(indptr, indices, train[batch:2 * batch], fanout, 24)
        assert_batch_equal(g, o)
        assert np.array_equal(g.cache_index, slot_ref[o.ids])
        ref = oracle.gather_rows_int8(o.ids, slot_ref[o.ids], q, sc, feats.array) if int8 else feats.array[o.ids]
        assert g.features.tobytes() == ref.tobytes()
        # a served batch of the presampled set hits more often than under degree order would guarantee
        assert (g.cache_index >= 0).mean() > cap / n_nodes
    finally:
        srv.close()
        feats.free()


def test_rebuilding_cache_or_graph_after_graph_capture(lmi, oracle):
    """The captured batch graph holds table pointers and graph pointers; rebuilding either
    afterwards must take effect on the next batch."""
    rng = np.random.default_rng(31)
    n_nodes, batch, fanout, dim = 3000, 64, [8, 4], 16
    indptr, indices = random_graph(rng, n_nodes, 8, hubs=4, hub_deg=200)
    indptr2, indices2 = random_graph(rng, n_nodes, 5, hubs=2, hub_deg=400)
    feats = make_features(lmi, rng, n_nodes, dim)
    srv = lmi.Server(batch, fanout, dim)
    stream = lmi.stream_create()
    seeds = rng.choice(n_nodes, batch, replace=False).astype(np.int32)
    try:
        srv.tune("use_graph", 1)
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        for step, (cap, table, gp, gi) in enumerate([(500, lmi.TABLE_HASH, indptr, indices),
                                                     (1500, lmi.TABLE_RANK, indptr, indices),
                                                     (900, lmi.TABLE_DIRECT, indptr2, indices2)]):
            if step == 2:
                srv.load_graph(gp, gi)
            srv.build_static_cache(cap, table)
            slot_ref = oracle.static_cache_build(gp, cap)
            for rep in range(2):
                srv.run_once(seeds, rng_seed=5 + rep, stream=stream)
                g = srv.fetch(stream=stream)
                o = oracle.sample_batch(gp, gi, seeds, fanout, 5 + rep)
                assert_batch_equal(g, o)
                assert np.array_equal(g.cache_index, slot_ref[o.ids])
                assert g.features.tobytes() == feats.array[o.ids].tobytes()
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("cache", ["static", "int8", "lru"])
@pytest.mark.parametrize("level,every", [(1, 1), (2, 1), (2, 3)])
def test_profiled_batches_come_out_the_same_and_count_their_rows(lmi, oracle, level, every, cache):
    """Profiling changes how kernels are launched (event-carrying launches, marker events between
    phases, device row counters): the batches must not change, and the counters must add up to the
    rows of the batches that were profiled (one in `every`)."""
    rng = np.random.default_rng(level * 7 + every)
    n_nodes, batch, dim, fanout = 4000, 120, 16, [8, 5]
    indptr, indices = random_graph(rng, n_nodes, 12, hubs=4, hub_deg=400)
    feats = make_features(lmi, rng, n_nodes, dim)
    train = rng.permutation(n_nodes)[:3600].astype(np.int32)
    group = 1 if cache == "lru" else 3
    srv = lmi.Server(batch, fanout, dim, pipes=group, seed=4)
    stream = lmi.stream_create()
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.load_idset(lmi.MODE_TRAIN, train)
        if cache == "static":
            srv.build_static_cache(1200, lmi.TABLE_RANK)
        elif cache == "int8":
            srv.build_int8_cache(1200, lmi.TABLE_RANK)
        else:
            srv.build_lru_cache(96, 4)
        srv.tune("profile_every", every)
        srv.profile_enable(level)
        rows_profiled = hits_profiled = 0
        n_calls = 6
        for call in range(n_calls):
            counters = [call * group + k for k in range(group)]
            if group == 1:
                srv.run_once(batch_counter=counters[0], pipe=0, stream=stream)
            else:
                srv.run_group(list(range(group)), counters, stream=stream)
            for k, c in enumerate(counters):
                g = srv.fetch(pipe=k, stream=stream)
                o = oracle.sample_batch(indptr, indices, train[c * batch:(c + 1) * batch], fanout, 4 + c)
                assert_batch_equal(g, o)
                if cache != "int8":
                    assert g.features.tobytes() == feats.array[o.ids].tobytes()
                if call % every == 0:   # the first call after profile_enable is profiled, then one in `every`
                    rows_profiled += len(o.ids)
                    hits_profiled += int((g.cache_index >= 0).sum())
        prof = srv.profile_read()
        assert prof.gather_hit_rows + prof.gather_miss_rows == rows_profiled
        assert prof.gather_hit_rows == hits_profiled
        calls_profiled = len(range(0, n_calls, every))
        assert prof.gather_hit_launches == calls_profiled          # one HBM gather launch per call
        assert prof.gather_miss_launches == calls_profiled         # and one host-link gather launch
        assert prof.gather_hit_ms > 0 and prof.gather_miss_ms > 0
        if level == 1:
            assert prof.sample_launches == calls_profiled and prof.sample_ms > 0
        srv.profile_enable(0)
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("fanout,batch,n_nodes,deg", [([25, 10], 64, 1_000_000, 40), ([64, 64], 16, 2_000_000, 72),
                                                      ([8, 8, 8], 128, 600_000, 160)])
def test_batches_that_nearly_fill_their_buffers(lmi, oracle, fanout, batch, n_nodes, deg):
    """Every node has more neighbours than the fan-out and they are spread over a graph far larger
    than a batch, so almost every sampled edge brings a new node: the batch comes within a few
    percent of the worst case the buffers and the dedup table are sized for, with both pipes of a
    group at that size."""
    rng = np.random.default_rng(len(fanout) * 1000 + batch)
    indptr = np.arange(n_nodes + 1, dtype=np.int64) * deg
    indices = rng.integers(0, n_nodes, n_nodes * deg, dtype=np.int32)
    dim = 4
    feats = lmi.HostBuffer((n_nodes, dim), np.float32)
    feats.array[...] = np.arange(n_nodes, dtype=np.float32)[:, None]
    worst = batch
    for f in fanout:
        worst *= 1 + f
    srv = lmi.Server(batch, fanout, dim, pipes=2, seed=11)
    stream = lmi.stream_create()
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.build_static_cache(n_nodes // 3, lmi.TABLE_RANK)
        seeds = [rng.choice(n_nodes, batch, replace=False).astype(np.int32) for _ in range(2)]
        srv.run_group([0, 1], [0, 0], seeds=seeds, rng_seeds=[5, 6], stream=stream)
        for k in range(2):
            g = srv.fetch(pipe=k, stream=stream)
            o = oracle.sample_batch(indptr, indices, seeds[k], fanout, 5 + k)
            assert_batch_equal(g, o)
            assert g.n_nodes[-1] > 0.9 * worst
            assert g.features.tobytes() == feats.array[o.ids].tobytes()
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("case", range(48))
def test_random_groups_sweep(lmi, oracle, case):
    """Seeded sweep through lmi_run_group: random group sizes on random subsets of 2..16 pipes,
    ragged seed lists, every launch shape and gather schedule the tuning keys select."""
    rng = np.random.default_rng(31000 + case)
    hops = int(rng.integers(1, 4))
    fanout = [int(rng.choice([1, 2, 3, 5, 8, 16, 25, 33, 64])) for _ in range(hops)]
    n_nodes = int(rng.choice([2, 50, 1000, 20000, 200000]))
    batch = int(rng.choice([1, 7, 64, 500]))
    hubs = int(rng.integers(0, 3)) if n_nodes >= 1000 else 0
    indptr, indices = random_graph(rng, n_nodes, float(rng.choice([0, 1, 5, 40])), hubs=hubs,
                                   hub_deg=int(rng.choice([300, 70000])), zero_frac=float(rng.choice([0.0, 0.3])))
    dim = int(rng.choice([4, 20, 128]))
    pipes = int(rng.choice([2, 4, 8, 16]))
    worst = batch
    for f in fanout:
        worst *= 1 + f
    while worst * (dim * 4 + 64) * pipes > 4e9 and batch > 1:   # keep the output buffers of all pipes modest
        batch = max(1, batch // 4)
        worst = batch
        for f in fanout:
            worst *= 1 + f
    feats = make_features(lmi, rng, n_nodes, dim)
    srv = lmi.Server(batch, fanout, dim, pipes=pipes, seed=5)
    stream = lmi.stream_create() if case % 2 else None
    kind = ["static", "int8", "none"][case % 3]
    slot_ref = q = sc = None
    try:
        for key, vals in (("group_miss", [0, 1]), ("protect_hits", [0, 1]), ("fuse_count", [0, 1]),
                          ("table_epochs", [0, 2, 1 << 30]), ("miss_blocks", [1, 8, 32]), ("split_miss", [0, 1, 2]),
                          ("early_fork", [0, 1]), ("split_lookup", [0, 1, 2]), ("miss_blocks_early", [0, 1, 16])):
            srv.tune(key, int(rng.choice(vals)))
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        cap = int(rng.integers(1, n_nodes + 1))
        if kind == "static":
            srv.build_static_cache(cap, int(rng.integers(0, 3)))
            slot_ref = oracle.static_cache_build(indptr, cap)
        elif kind == "int8":
            srv.build_int8_cache(cap, int(rng.integers(0, 3)))
            slot_ref = oracle.static_cache_build(indptr, cap)
            q, sc = oracle.quantize_rows(feats.array[np.flatnonzero(slot_ref >= 0)])
        issued = 0
        for rnd in range(4):
            n = int(rng.integers(1, min(8, pipes) + 1))
            plist = [int(x) for x in rng.choice(pipes, n, replace=False)]
            seeds = [rng.integers(0, n_nodes, int(rng.integers(1, batch + 1))).astype(np.int32) for _ in plist]
            rs = [500 + issued + k for k in range(n)]
            issued += n
            srv.run_group(plist, [0] * n, seeds=seeds, rng_seeds=rs, stream=stream)
            for k, pipe in enumerate(plist):
                g = srv.fetch(pipe=pipe, stream=stream)
                o = oracle.sample_batch(indptr, indices, seeds[k], fanout, rs[k])
                assert_batch_equal(g, o)
                if kind == "int8":
                    np.testing.assert_array_equal(g.cache_index, slot_ref[o.ids])
                    assert g.features.tobytes() == oracle.gather_rows_int8(o.ids, slot_ref[o.ids], q, sc, feats.array).tobytes()
                else:
                    assert g.features.tobytes() == feats.array[o.ids].tobytes()
                    if slot_ref is not None:
                        np.testing.assert_array_equal(g.cache_index, slot_ref[o.ids])
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("early_fork", [0, 1, 2])
@pytest.mark.parametrize("streams", [1, 2])
@pytest.mark.parametrize("split_lookup", [0, 1])
def test_groups_that_reuse_pipes_wait_for_the_host_link_gather_before(lmi, oracle, streams, early_fork, split_lookup):
    """Groups issued back to back on overlapping sets of pipes, nothing fetched in between: a pipe's
    next batch may only start once the side stream has finished the host-link gather of the one
    before (one event per group marks that, whichever pipes of it are reused first).  The host-link
    gather is slowed to one block and most rows miss, so a batch that started early would be
    overwritten by the rows of its predecessor.  With the side stream released ahead of the HBM gather
    (early_fork) that event does not cover the HBM gather: a pipe taken over by the other caller's
    stream is ordered behind the stream that carried its batch.  With split lookups a batch has two host-link
    gathers, the first released before its second hop is sampled; the one event still marks the end of both."""
    rng = np.random.default_rng(77 + streams)
    n_nodes, batch, dim, fanout, pipes = 40_000, 500, 128, [10, 5], 8
    indptr, indices = random_graph(rng, n_nodes, 12, hubs=4, hub_deg=2000)
    feats = make_features(lmi, rng, n_nodes, dim)
    srv = lmi.Server(batch, fanout, dim, pipes=pipes, seed=3)
    ss = [lmi.stream_create() for _ in range(streams)]
    try:
        srv.tune("miss_blocks", 1)
        srv.tune("early_fork", early_fork)
        srv.tune("split_lookup", split_lookup)
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.build_static_cache(n_nodes // 10, lmi.TABLE_RANK)
        last, issued = {}, 0
        for rnd in range(14):
            n = int(rng.integers(1, pipes + 1))
            plist = [int(x) for x in rng.choice(pipes, n, replace=False)]
            seeds = [rng.choice(n_nodes, int(rng.integers(batch // 2, batch + 1)), replace=False).astype(np.int32)
                     for _ in plist]
            rs = [900 + issued + k for k in range(n)]
            issued += n
            if n == 1 and rnd % 2:
                srv.run_once(seeds[0], rng_seed=rs[0], pipe=plist[0], stream=ss[rnd % streams])
            else:
                srv.run_group(plist, [0] * n, seeds=seeds, rng_seeds=rs, stream=ss[rnd % streams])
            for k, pipe in enumerate(plist):
                last[pipe] = (seeds[k], rs[k])
        for pipe, (seeds, r) in sorted(last.items()):
            g = srv.fetch(pipe=pipe, stream=ss[0])
            o = oracle.sample_batch(indptr, indices, seeds, fanout, r)
            assert_batch_equal(g, o)
            assert g.features.tobytes() == feats.array[o.ids].tobytes(), "pipe %d" % pipe
        srv.status()
    finally:
        srv.close()
        feats.free()


@pytest.mark.parametrize("cache", ["none", "static-early", "static-late"])
def test_a_pipe_read_from_another_stream_sees_the_whole_batch(lmi, oracle, cache):
    """A batch issued on one stream and waited for (lmi_batch_wait, and the read-back that follows)
    on another: without a cache the whole batch sits on the issuing stream, with the side stream
    released early its HBM gather does -- the waiting stream must be ordered behind that too."""
    rng = np.random.default_rng(5150)
    n_nodes, batch, dim, fanout = 60_000, 1500, 128, [15, 8]
    indptr, indices = random_graph(rng, n_nodes, 14, hubs=3, hub_deg=3000)
    feats = make_features(lmi, rng, n_nodes, dim)
    srv = lmi.Server(batch, fanout, dim, pipes=2, seed=9)
    a, b = lmi.stream_create(), lmi.stream_create()
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        if cache != "none":
            srv.build_static_cache(n_nodes * 9 // 10, lmi.TABLE_RANK)   # nearly everything is an HBM hit
            srv.tune("early_fork", 1 if cache == "static-early" else 0)
        for it in range(6):
            seeds = rng.choice(n_nodes, batch, replace=False).astype(np.int32)
            srv.run_once(seeds, rng_seed=40 + it, pipe=it % 2, stream=a if it % 2 == 0 else b)
            srv.batch_wait(it % 2, b if it % 2 == 0 else a)              # the OTHER stream waits ...
            g = srv.fetch(pipe=it % 2, stream=b if it % 2 == 0 else a)   # ... and reads
            o = oracle.sample_batch(indptr, indices, seeds, fanout, 40 + it)
            assert_batch_equal(g, o)
            assert g.features.tobytes() == feats.array[o.ids].tobytes(), "batch %d" % it
    finally:
        srv.close()
        feats.free()


def test_a_wait_on_one_stream_does_not_release_another(lmi, oracle):
    """The host-link gather of a batch is slowed to one block; a second stream waits for the batch
    (lmi_batch_wait), then the pipe's NEXT batch is issued on the first stream at once.  That stream
    has not waited yet: it must still be held until the first batch's rows are in, or they would land
    among the second batch's."""
    rng = np.random.default_rng(616)
    n_nodes, batch, dim, fanout = 50_000, 800, 128, [10, 6]
    indptr, indices = random_graph(rng, n_nodes, 12, hubs=3, hub_deg=2500)
    feats = make_features(lmi, rng, n_nodes, dim)
    srv = lmi.Server(batch, fanout, dim, pipes=1, seed=2)
    a, b = lmi.stream_create(), lmi.stream_create()
    try:
        srv.tune("miss_blocks", 1)
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.build_static_cache(n_nodes // 20, lmi.TABLE_RANK)            # most rows cross the host link
        for it in range(4):
            s1 = rng.choice(n_nodes, batch, replace=False).astype(np.int32)
            s2 = rng.choice(n_nodes, batch // 2, replace=False).astype(np.int32)
            srv.run_once(s1, rng_seed=70 + it, pipe=0, stream=a)
            srv.batch_wait(0, b)                                         # stream b is now behind the batch
            srv.run_once(s2, rng_seed=170 + it, pipe=0, stream=a)        # stream a is not, unless the call sees to it
            g = srv.fetch(pipe=0, stream=a)
            o = oracle.sample_batch(indptr, indices, s2, fanout, 170 + it)
            assert_batch_equal(g, o)
            assert g.features.tobytes() == feats.array[o.ids].tobytes(), "round %d" % it
        srv.status()
    finally:
        srv.close()
        feats.free()
