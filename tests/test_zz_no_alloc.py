"""The entry point that allocates nothing (lmi_run_once_static): same outputs as lmi_run_once,
bit for bit, on two calls in a row, the second with a smaller input; plus its refusals."""
import ctypes as C

import numpy as np
import pytest

from conftest import random_graph

pytestmark = pytest.mark.gpu


class DeviceOutputs:
    """Caller-owned device buffers for one batch, as an lmi_batch_view."""

    def __init__(self, lmi, srv, poison=0xA5):
        v0 = srv.view(0)   # only for the worst-case sizes
        self.lmi, self.max_nodes, self.max_edges = lmi, int(v0.max_nodes), int(v0.max_edges)
        self.dim, self.np_dtype = srv.cfg.feat_dim, srv.np_dtype
        esz = np.dtype(self.np_dtype).itemsize
        hops, batch = srv.cfg.hops, srv.cfg.batch_size
        caps = [batch]
        for k in range(hops):
            caps.append(caps[-1] * (1 + srv.fanout[k]))
        sizes = dict(ids=self.max_nodes * 4, features=self.max_nodes * self.dim * esz, labels=batch * 4,
                     agg_src_ids=self.max_edges * 4, agg_src_off=self.max_edges * 4, agg_dst_off=self.max_edges * 4,
                     node_counter=64, edge_counter=64, cache_index=self.max_nodes * 4)
        for k in range(hops):
            sizes["blk%d" % k] = (caps[k] + 1) * 4
        self.ptr = {}
        for name, nbytes in sizes.items():
            p = C.c_void_p()
            lmi.check(lmi.lib().lmi_device_alloc(nbytes, C.byref(p)))
            junk = np.full(nbytes, poison, np.uint8)   # whatever a caller's buffer held before
            lmi.check(lmi.lib().lmi_copy_to_device(p, junk.ctypes.data, nbytes))
            self.ptr[name] = p
        v = lmi.BatchView()
        for name in ("ids", "features", "labels", "agg_src_ids", "agg_src_off", "agg_dst_off", "node_counter",
                     "edge_counter", "cache_index"):
            setattr(v, name, self.ptr[name])
        for k in range(hops):
            v.blk_indptr[k] = self.ptr["blk%d" % k]
        v.max_nodes, v.max_edges = self.max_nodes, self.max_edges
        self.view = v

    def fetch(self):
        lmi = self.lmi
        nc = lmi.to_host(self.ptr["node_counter"], 16, np.int32)
        ec = lmi.to_host(self.ptr["edge_counter"], 16, np.int32)
        hops = int(nc[8])
        b = lmi.Batch()
        b.node_counter, b.edge_counter = nc, ec
        b.n_nodes = [int(nc[9 + k]) for k in range(hops + 1)]
        n, e = b.n_nodes[-1], int(sum(ec[9 + k] for k in range(1, hops + 1)))
        b.ids = lmi.to_host(self.ptr["ids"], n, np.int32)
        b.labels = lmi.to_host(self.ptr["labels"], b.n_nodes[0], np.int32)
        for name in ("agg_src_ids", "agg_src_off", "agg_dst_off"):
            setattr(b, name, lmi.to_host(self.ptr[name], e, np.int32))
        b.blk_indptr = [lmi.to_host(self.ptr["blk%d" % k], b.n_nodes[k] + 1, np.int32) for k in range(hops)]
        b.cache_index = lmi.to_host(self.ptr["cache_index"], n, np.int32)
        b.features = lmi.to_host(self.ptr["features"], n * self.dim, self.np_dtype).reshape(n, self.dim)
        return b

    def free(self):
        for p in self.ptr.values():
            self.lmi.check(self.lmi.lib().lmi_device_free(p))


def device_seeds(lmi, seeds):
    p = C.c_void_p()
    lmi.check(lmi.lib().lmi_device_alloc(max(4, seeds.nbytes), C.byref(p)))
    if len(seeds):
        lmi.check(lmi.lib().lmi_copy_to_device(p, seeds.ctypes.data, seeds.nbytes))
    return p


def assert_same(a, b):
    assert list(a.node_counter) == list(b.node_counter) and list(a.edge_counter) == list(b.edge_counter)
    for name in ("ids", "labels", "agg_src_ids", "agg_src_off", "agg_dst_off", "cache_index"):
        assert np.array_equal(getattr(a, name), getattr(b, name)), name
    for x, y in zip(a.blk_indptr, b.blk_indptr):
        assert np.array_equal(x, y)
    assert a.features.tobytes() == b.features.tobytes()


@pytest.mark.parametrize("cache,dim,dtype,fanout,batch", [
    ("static", 128, np.float32, [25, 10], 300),
    ("int8", 768, np.float16, [25, 15], 64),
    ("static", 100, np.float32, [5, 4, 3], 700),
    ("none", 64, np.float32, [64, 2], 128),
])
def test_static_entry_point_matches_run_once_twice_in_a_row(lmi, oracle, cache, dim, dtype, fanout, batch):
    rng = np.random.default_rng(11)
    n_nodes = 30_000
    indptr, indices = random_graph(rng, n_nodes, 14, hubs=8, hub_deg=3000)
    feats = lmi.HostBuffer((n_nodes, dim), dtype)
    feats.array[...] = rng.standard_normal((n_nodes, dim)).astype(dtype)
    srv = lmi.Server(batch, fanout, dim, feat_dtype=lmi.F16 if dtype == np.float16 else lmi.F32, pipes=1, seed=5)
    stream = lmi.stream_create()
    outs, dseeds = None, []
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        if cache == "static":
            srv.build_static_cache(9000, lmi.TABLE_RANK)
        elif cache == "int8":
            srv.build_int8_cache(9000, lmi.TABLE_HASH)
        outs = DeviceOutputs(lmi, srv)
        # two calls in a row on the same scratch, the second with a smaller input, then a third
        # as large as the first again
        for call, n in enumerate([batch, max(1, batch // 5), batch]):
            seeds = rng.choice(n_nodes, n, replace=False).astype(np.int32)
            d = device_seeds(lmi, seeds)
            dseeds.append(d)
            srv.run_once_static(d, n, outs.view, rng_seed=100 + call, stream=stream)
            lmi.check(lmi.lib().lmi_stream_sync(stream))
            got = outs.fetch()
            srv.run_once(seeds, rng_seed=100 + call, pipe=0, stream=stream)
            ref = srv.fetch(pipe=0, stream=stream)
            assert_same(got, ref)
            # and both are what the oracle says
            o = oracle.sample_batch(indptr, indices, seeds, fanout, 100 + call)
            assert np.array_equal(got.ids, o.ids) and np.array_equal(got.agg_src_off, o.agg_src_off)
            assert len(got.ids) > n
    finally:
        srv.close()
        if outs:
            outs.free()
        for d in dseeds:
            lmi.check(lmi.lib().lmi_device_free(d))
        feats.free()


def test_static_entry_point_at_the_largest_server_it_takes(lmi, oracle):
    """Batch 800 with fan-out [25, 10]: 228 800 rows and 208 000 edges of a hop in the worst case, just
    inside the limits (2^18 each), on a graph dense enough that a batch comes close to them; a second
    server on the same GPU uses the entry point in between (the scratch array is shared, nothing on the
    host is)."""
    rng = np.random.default_rng(41)
    n_nodes, dim, batch, fanout = 400_000, 100, 800, [25, 10]
    indptr, indices = random_graph(rng, n_nodes, 30, hubs=4, hub_deg=5000, zero_frac=0.02)
    feats = lmi.HostBuffer((n_nodes, dim), np.float32)
    feats.array[...] = rng.standard_normal((n_nodes, dim)).astype(np.float32)
    srv = lmi.Server(batch, fanout, dim, pipes=1, seed=5)
    other = lmi.Server(64, [5, 4], dim, pipes=1, seed=6)
    stream = lmi.stream_create()
    outs = outs2 = None
    dseeds = []
    try:
        assert int(srv.view(0).max_nodes) == 228_800 <= lmi.STATIC_MAX_NODES
        for sv in (srv, other):
            sv.load_graph(indptr, indices)
            sv.attach_features(feats)
            sv.build_static_cache(120_000, lmi.TABLE_RANK)
        outs, outs2 = DeviceOutputs(lmi, srv), DeviceOutputs(lmi, other)
        for call, n in enumerate([batch, 37, batch]):
            seeds = rng.choice(n_nodes, n, replace=False).astype(np.int32)
            d = device_seeds(lmi, seeds)
            dseeds.append(d)
            srv.run_once_static(d, n, outs.view, rng_seed=300 + call, stream=stream)
            # the other server takes the same scratch right behind it, on the same stream (no overlap)
            small = seeds[:min(n, 64)]
            other.run_once_static(d, len(small), outs2.view, rng_seed=900 + call, stream=stream)
            lmi.check(lmi.lib().lmi_stream_sync(stream))
            got, got2 = outs.fetch(), outs2.fetch()
            srv.run_once(seeds, rng_seed=300 + call, pipe=0, stream=stream)
            assert_same(got, srv.fetch(pipe=0, stream=stream))
            other.run_once(small, rng_seed=900 + call, pipe=0, stream=stream)
            assert_same(got2, other.fetch(pipe=0, stream=stream))
            o = oracle.sample_batch(indptr, indices, seeds, fanout, 300 + call)
            assert np.array_equal(got.ids, o.ids) and np.array_equal(got.agg_src_off, o.agg_src_off)
            if n == batch:
                assert len(got.ids) > 150_000      # the batch comes close to the worst case
    finally:
        srv.close()
        other.close()
        for o_ in (outs, outs2):
            if o_:
                o_.free()
        for d in dseeds:
            lmi.check(lmi.lib().lmi_device_free(d))
        feats.free()


def test_static_entry_point_refuses_what_it_cannot_hold(lmi):
    rng = np.random.default_rng(3)
    n_nodes, dim = 5000, 32
    indptr, indices = random_graph(rng, n_nodes, 10)
    feats = lmi.HostBuffer((n_nodes, dim), np.float32)
    feats.array[...] = 1.0
    seeds = np.arange(10, dtype=np.int32)
    d = device_seeds(lmi, seeds)
    try:
        # worst case beyond the scratch: 8000 x 26 x 11 rows
        big = lmi.Server(8000, [25, 10], dim, pipes=1)
        try:
            big.load_graph(indptr, indices)
            big.attach_features(feats)
            with pytest.raises(lmi.LegionError) as e:
                big.run_once_static(d, 10, big.view(0))
            assert e.value.code == -4 and "static scratch" in str(e.value)
        finally:
            big.close()
        small = lmi.Server(64, [5, 5], dim, pipes=1)
        try:
            small.load_graph(indptr, indices)
            small.attach_features(feats)
            v = small.view(0)
            v.max_nodes = 10   # buffers said to be too small
            with pytest.raises(lmi.LegionError) as e:
                small.run_once_static(d, 10, v)
            assert e.value.code == -4
            v = small.view(0)
            v.cache_index = None
            with pytest.raises(lmi.LegionError) as e:
                small.run_once_static(d, 10, v)
            assert e.value.code == -1
            small.build_lru_cache(16, 4)
            with pytest.raises(lmi.LegionError) as e:
                small.run_once_static(d, 10, small.view(0))
            assert e.value.code == -3
        finally:
            small.close()
    finally:
        lmi.check(lmi.lib().lmi_device_free(d))
        feats.free()


def hip_runtime():
    """The HIP runtime the library itself is linked against (already loaded with it)."""
    hip = C.CDLL("libamdhip64.so.7")
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    return hip


def test_static_entry_point_replayed_from_a_captured_graph(lmi, oracle):
    """The callers the entry point is for: its launches captured once in a HIP graph and replayed
    with other seeds in the same buffer; eager batches and synchronisations between the replays,
    every replay checked.  Captured in the global mode, in which an allocation by the capturing
    thread is an error."""
    hip = hip_runtime()
    rng = np.random.default_rng(23)
    n_nodes, dim, batch, fanout = 30_000, 128, 256, [25, 10]
    indptr, indices = random_graph(rng, n_nodes, 14, hubs=8, hub_deg=3000)
    feats = lmi.HostBuffer((n_nodes, dim), np.float32)
    feats.array[...] = rng.standard_normal((n_nodes, dim)).astype(np.float32)
    srv = lmi.Server(batch, fanout, dim, pipes=1, seed=5)
    stream, other = lmi.stream_create(), lmi.stream_create()
    outs = d = None
    graph, graph_exec = C.c_void_p(), C.c_void_p()
    try:
        srv.load_graph(indptr, indices)
        srv.attach_features(feats)
        srv.build_static_cache(9000, lmi.TABLE_RANK)
        outs = DeviceOutputs(lmi, srv)
        d = device_seeds(lmi, np.zeros(batch, np.int32))
        lmi.check(lmi.lib().lmi_device_sync())
        assert hip.hipStreamBeginCapture(stream, 0) == 0          # hipStreamCaptureModeGlobal
        try:
            srv.run_once_static(d, batch, outs.view, rng_seed=77, stream=stream)
        finally:
            rc = hip.hipStreamEndCapture(stream, C.byref(graph))
        assert rc == 0 and graph.value
        assert hip.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, 0) == 0
        for rep in range(4):
            seeds = rng.choice(n_nodes, batch, replace=False).astype(np.int32)
            lmi.check(lmi.lib().lmi_copy_to_device(d, seeds.ctypes.data, seeds.nbytes))
            assert hip.hipGraphLaunch(graph_exec, stream) == 0
            lmi.check(lmi.lib().lmi_stream_sync(stream))
            got = outs.fetch()
            srv.run_once(seeds, rng_seed=77, pipe=0, stream=other)   # eager work between the replays
            assert_same(got, srv.fetch(pipe=0, stream=other))
            o = oracle.sample_batch(indptr, indices, seeds, fanout, 77)
            assert np.array_equal(got.ids, o.ids) and np.array_equal(got.agg_src_off, o.agg_src_off)
        srv.status()
    finally:
        if graph_exec.value:
            hip.hipGraphExecDestroy(graph_exec)
        if graph.value:
            hip.hipGraphDestroy(graph)
        srv.close()
        if outs:
            outs.free()
        if d:
            lmi.check(lmi.lib().lmi_device_free(d))
        feats.free()
