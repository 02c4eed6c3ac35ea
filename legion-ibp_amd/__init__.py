"""ctypes view of liblegion_mi.so -- the MI355X sampling-server hot path.

Thin by design: every call goes straight through the C ABI declared in
include/legion_mi.h.  There is no CPU fallback; loading fails loudly when the
HIP library has not been built (run `make -C legion-ibp_amd` or
`python -c "import __graft_entry__ as g; g.build()"`).
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblegion_mi.so")

MAX_HOPS, MAX_FANOUT, MAX_PIPES, MAX_GROUP = 3, 64, 16, 8
STATIC_MAX_NODES, STATIC_MAX_HOP_EDGES = 1 << 18, 1 << 18   # limits of lmi_run_once_static
F32, F16 = 0, 1
LOC_HOST, LOC_DEVICE = 0, 1
MODE_TRAIN, MODE_VALID, MODE_TEST = 0, 1, 2
TABLE_HASH, TABLE_DIRECT, TABLE_RANK = 0, 1, 2
CACHE_NONE, CACHE_STATIC, CACHE_LRU, CACHE_INT8 = 0, 1, 2, 3
POLICY_DEGREE, POLICY_PRESAMPLED = 0, 1

# every symbol include/legion_mi.h declares
ABI_SYMBOLS = [
    "lmi_abi_version", "lmi_last_error", "lmi_server_create", "lmi_server_destroy", "lmi_server_pipes",
    "lmi_host_alloc", "lmi_host_free", "lmi_device_alloc", "lmi_device_free",
    "lmi_copy_to_host", "lmi_copy_to_device", "lmi_copy_device", "lmi_ipc_export", "lmi_ipc_open", "lmi_ipc_close",
    "lmi_stream_create", "lmi_stream_destroy",
    "lmi_stream_sync", "lmi_device_sync", "lmi_graph_load", "lmi_features_attach",
    "lmi_idset_load", "lmi_idset_batch", "lmi_presample", "lmi_op_hotness", "lmi_presample_reset", "lmi_hotness_dump",
    "lmi_cache_policy", "lmi_cache_build_static", "lmi_cache_build_lru", "lmi_cache_build_int8",
    "lmi_cache_info_get", "lmi_cache_dump", "lmi_op_batch_generate", "lmi_op_random_sample",
    "lmi_op_cache_lookup", "lmi_op_io_submit", "lmi_op_io_complete", "lmi_run_once",
    "lmi_run_group", "lmi_run_once_static", "lmi_batch_wait", "lmi_server_status", "lmi_batch_view_get", "lmi_batch_counters", "lmi_steps_per_epoch", "lmi_profile_enable",
    "lmi_profile_read", "lmi_tune", "lmi_bench_copy", "lmi_bench_copy_launch", "lmi_bench_stream", "lmi_bench_row_stream", "lmi_bench_row_stream_shape", "lmi_bench_host_read", "lmi_bench_random_read", "lmi_synth_graph", "lmi_synth_trainset",
    "lmi_synth_features",
]


class Config(C.Structure):
    _fields_ = [("device_id", C.c_int32), ("batch_size", C.c_int32), ("hops", C.c_int32),
                ("fanout", C.c_int32 * MAX_HOPS), ("feat_dim", C.c_int32), ("feat_dtype", C.c_int32),
                ("pipes", C.c_int32), ("reserved", C.c_int32), ("seed", C.c_uint64)]


class BatchView(C.Structure):
    _fields_ = [("ids", C.c_void_p), ("features", C.c_void_p), ("labels", C.c_void_p),
                ("agg_src_ids", C.c_void_p), ("agg_src_off", C.c_void_p), ("agg_dst_off", C.c_void_p),
                ("node_counter", C.c_void_p), ("edge_counter", C.c_void_p),
                ("blk_indptr", C.c_void_p * MAX_HOPS), ("cache_index", C.c_void_p),
                ("max_nodes", C.c_int64), ("max_edges", C.c_int64), ("row_bytes", C.c_int64)]


class CacheInfo(C.Structure):
    _fields_ = [("kind", C.c_int32), ("table_kind", C.c_int32), ("capacity_rows", C.c_int64),
                ("row_bytes", C.c_int64), ("table_bytes", C.c_int64), ("n_sets", C.c_int64),
                ("ways", C.c_int32), ("lru_tick", C.c_int32)]


class Profile(C.Structure):
    _fields_ = [("gather_hit_ms", C.c_double), ("gather_hit_launches", C.c_int64), ("gather_hit_rows", C.c_int64),
                ("gather_miss_ms", C.c_double), ("gather_miss_launches", C.c_int64), ("gather_miss_rows", C.c_int64),
                ("sample_ms", C.c_double), ("sample_launches", C.c_int64),
                ("lookup_ms", C.c_double), ("lookup_launches", C.c_int64),
                ("batch_ms", C.c_double), ("batches", C.c_int64)]


class LegionError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("legion_mi error %d: %s" % (code, text))
        self.code = code


_lib = None


def lib():
    """Load the C-ABI library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("liblegion_mi.so is missing: build it with `make -C %s` "
                              "(there is no CPU fallback)" % _HERE)
        # RTLD_GLOBAL: a HIP runtime loaded later by another package (PyTorch brings its own copy)
        # then resolves to the one this library already initialised; two runtimes in one process
        # cannot both open the GPU
        L = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
        L.lmi_last_error.restype = C.c_char_p
        L.lmi_host_alloc.argtypes = [C.c_size_t, C.POINTER(C.c_void_p)]
        L.lmi_host_free.argtypes = [C.c_void_p]
        L.lmi_device_alloc.argtypes = [C.c_size_t, C.POINTER(C.c_void_p)]
        L.lmi_device_free.argtypes = [C.c_void_p]
        L.lmi_copy_to_host.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.lmi_copy_to_device.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.lmi_copy_device.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        L.lmi_ipc_export.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
        L.lmi_ipc_open.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.lmi_ipc_close.argtypes = [C.c_void_p]
        L.lmi_stream_create.argtypes = [C.POINTER(C.c_void_p)]
        L.lmi_stream_destroy.argtypes = [C.c_void_p]
        L.lmi_stream_sync.argtypes = [C.c_void_p]
        L.lmi_server_create.argtypes = [C.POINTER(Config), C.POINTER(C.c_void_p)]
        L.lmi_server_destroy.argtypes = [C.c_void_p]
        L.lmi_server_pipes.argtypes = [C.c_void_p, C.c_int32]
        L.lmi_graph_load.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int]
        L.lmi_features_attach.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
        L.lmi_idset_load.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
        L.lmi_idset_batch.argtypes = [C.c_void_p, C.c_int, C.c_int32]
        L.lmi_presample.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int32, C.c_int32]
        L.lmi_op_hotness.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
        L.lmi_presample_reset.argtypes = [C.c_void_p]
        L.lmi_hotness_dump.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        L.lmi_cache_policy.argtypes = [C.c_void_p, C.c_int]
        L.lmi_cache_build_static.argtypes = [C.c_void_p, C.c_int64, C.c_int]
        L.lmi_cache_build_int8.argtypes = [C.c_void_p, C.c_int64, C.c_int]
        L.lmi_cache_build_lru.argtypes = [C.c_void_p, C.c_int64, C.c_int32]
        L.lmi_cache_info_get.argtypes = [C.c_void_p, C.POINTER(CacheInfo)]
        L.lmi_cache_dump.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]
        L.lmi_op_batch_generate.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int32, C.c_int,
                                            C.c_int32, C.c_int, C.c_uint64]
        L.lmi_op_random_sample.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int]
        L.lmi_op_cache_lookup.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int]
        L.lmi_op_io_submit.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
        L.lmi_op_io_complete.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
        L.lmi_run_once.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int32, C.c_int, C.c_int32,
                                   C.c_int, C.c_uint64]
        L.lmi_batch_wait.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
        L.lmi_server_status.argtypes = [C.c_void_p, C.c_int]
        L.lmi_batch_view_get.argtypes = [C.c_void_p, C.c_int, C.POINTER(BatchView)]
        L.lmi_batch_counters.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.lmi_run_group.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                    C.c_void_p, C.c_int, C.c_void_p]
        L.lmi_run_once_static.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_uint64,
                                          C.POINTER(BatchView)]
        L.lmi_steps_per_epoch.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_int32)]
        L.lmi_profile_enable.argtypes = [C.c_void_p, C.c_int]
        L.lmi_profile_read.argtypes = [C.c_void_p, C.POINTER(Profile), C.c_int]
        L.lmi_tune.argtypes = [C.c_void_p, C.c_char_p, C.c_int64]
        L.lmi_bench_copy.argtypes = [C.c_size_t, C.c_int, C.POINTER(C.c_double)]
        L.lmi_bench_copy_launch.argtypes = [C.c_size_t, C.c_int, C.POINTER(C.c_double)]
        L.lmi_bench_stream.argtypes = [C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double)]
        L.lmi_bench_row_stream.argtypes = [C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_int64, C.c_int, C.c_int,
                                           C.POINTER(C.c_double)]
        L.lmi_bench_row_stream_shape.argtypes = [C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_int64, C.c_int, C.c_int, C.c_int,
                                                 C.c_int, C.c_int, C.POINTER(C.c_double)]
        L.lmi_bench_host_read.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.POINTER(C.c_double)]
        L.lmi_bench_random_read.argtypes = [C.c_void_p, C.c_size_t, C.c_int64, C.c_int, C.POINTER(C.c_double)]
        L.lmi_synth_graph.argtypes = [C.c_uint64, C.c_void_p, C.c_int32, C.c_int64, C.c_int32,
                                      C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.POINTER(C.c_int64)]
        L.lmi_synth_trainset.argtypes = [C.c_uint64, C.c_int64, C.c_int32, C.c_void_p]
        L.lmi_synth_features.argtypes = [C.c_uint64, C.c_void_p, C.c_int64, C.c_int32, C.c_int32]
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise LegionError(rc, lib().lmi_last_error().decode())


class HostBuffer:
    """Pinned + mapped host memory (lmi_host_alloc) exposed as a numpy array."""

    def __init__(self, shape, dtype):
        self.shape, self.dtype = tuple(shape), np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        p = C.c_void_p()
        check(lib().lmi_host_alloc(self.nbytes, C.byref(p)))
        self.ptr = p.value
        buf = (C.c_uint8 * self.nbytes).from_address(self.ptr)
        self.array = np.frombuffer(buf, dtype=self.dtype).reshape(self.shape)

    def free(self):
        if self.ptr:
            self.array = None
            check(lib().lmi_host_free(self.ptr))
            self.ptr = None


def to_host(dev_ptr, count, dtype):
    out = np.empty(count, dtype)
    if count:
        check(lib().lmi_copy_to_host(out.ctypes.data, dev_ptr, out.nbytes))
    return out


class Batch:
    """Host copy of one pipe's outputs, trimmed to the real sizes."""


class Server:
    """One sampling server on one GPU (reference: GPUServer + GPURunner)."""

    def __init__(self, batch_size, fanout, feat_dim, feat_dtype=F32, pipes=1, seed=1, device_id=0):
        cfg = Config()
        cfg.device_id, cfg.batch_size, cfg.hops = device_id, batch_size, len(fanout)
        for k, f in enumerate(fanout[:MAX_HOPS]):
            cfg.fanout[k] = f
        if len(fanout) > MAX_HOPS:
            cfg.hops = len(fanout)
        cfg.feat_dim, cfg.feat_dtype, cfg.pipes, cfg.seed = feat_dim, feat_dtype, pipes, seed
        self.cfg, self.fanout = cfg, list(fanout)
        self.np_dtype = np.float16 if feat_dtype == F16 else np.float32
        self.h = C.c_void_p()
        check(lib().lmi_server_create(C.byref(cfg), C.byref(self.h)))
        self._keep = []

    def close(self):
        if self.h:
            check(lib().lmi_server_destroy(self.h))
            self.h = None

    def add_pipes(self, pipes):
        """Grow the server to `pipes` output buffer sets (lmi_server_pipes)."""
        check(lib().lmi_server_pipes(self.h, pipes))
        self.cfg.pipes = max(int(self.cfg.pipes), pipes)

    # storage -----------------------------------------------------------------
    def load_graph(self, indptr, indices):
        indptr = np.ascontiguousarray(indptr, dtype=np.int64)
        indices = np.ascontiguousarray(indices, dtype=np.int32)
        check(lib().lmi_graph_load(self.h, indptr.ctypes.data, indices.ctypes.data, len(indptr) - 1,
                                   len(indices), LOC_HOST))

    def attach_graph_device(self, d_indptr, d_indices, n_nodes, n_edges):
        check(lib().lmi_graph_load(self.h, d_indptr, d_indices, n_nodes, n_edges, LOC_DEVICE))

    def attach_features(self, host_buffer):
        self._keep.append(host_buffer)
        check(lib().lmi_features_attach(self.h, host_buffer.ptr, host_buffer.shape[0], LOC_HOST))

    def attach_features_device(self, dev_ptr, n_rows):
        check(lib().lmi_features_attach(self.h, dev_ptr, n_rows, LOC_DEVICE))

    def load_idset(self, mode, ids, labels=None):
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        lp = None
        if labels is not None:
            labels = np.ascontiguousarray(labels, dtype=np.int32)
            lp = labels.ctypes.data
        check(lib().lmi_idset_load(self.h, mode, ids.ctypes.data, lp, len(ids), LOC_HOST))

    def idset_batch(self, mode, ids_per_batch):
        """Ids per sliced batch of id set `mode` (default: the server's batch size)."""
        check(lib().lmi_idset_batch(self.h, mode, ids_per_batch))

    # presampling -------------------------------------------------------------
    def presample(self, n_batches, first_batch=0, mode=MODE_TRAIN, pipe=0, stream=None):
        check(lib().lmi_presample(self.h, pipe, stream, mode, first_batch, n_batches))

    def hotness(self, n_nodes):
        out = np.empty(n_nodes, np.uint32)
        check(lib().lmi_hotness_dump(self.h, out.ctypes.data, n_nodes))
        return out

    def cache_policy(self, policy):
        check(lib().lmi_cache_policy(self.h, policy))

    # caches ------------------------------------------------------------------
    def build_static_cache(self, rows, table=TABLE_HASH):
        check(lib().lmi_cache_build_static(self.h, rows, table))

    def build_int8_cache(self, rows, table=TABLE_HASH):
        check(lib().lmi_cache_build_int8(self.h, rows, table))

    def build_lru_cache(self, n_sets, ways):
        check(lib().lmi_cache_build_lru(self.h, n_sets, ways))

    def cache_info(self):
        ci = CacheInfo()
        check(lib().lmi_cache_info_get(self.h, C.byref(ci)))
        return ci

    def cache_dump(self, n, with_aux=False):
        out = np.empty(n, np.int32)
        aux = np.empty(n, np.int32) if with_aux else None
        check(lib().lmi_cache_dump(self.h, out.ctypes.data, n, aux.ctypes.data if with_aux else None))
        return (out, aux) if with_aux else out

    # operators ---------------------------------------------------------------
    def _seed_args(self, seeds):
        if seeds is None:
            return None, 0, None
        seeds = np.ascontiguousarray(seeds, dtype=np.int32)
        return seeds.ctypes.data, len(seeds), seeds

    def op_batch_generate(self, seeds=None, batch_counter=0, mode=MODE_TRAIN, rng_seed=0, pipe=0, stream=None):
        p, n, keep = self._seed_args(seeds)
        check(lib().lmi_op_batch_generate(self.h, pipe, stream, p, n, LOC_HOST, batch_counter, mode, rng_seed))

    def op_random_sample(self, hop, pipe=0, stream=None):
        check(lib().lmi_op_random_sample(self.h, pipe, stream, hop))

    def op_cache_lookup(self, segment, pipe=0, stream=None):
        check(lib().lmi_op_cache_lookup(self.h, pipe, stream, segment))

    def op_io_submit(self, pipe=0, stream=None):
        check(lib().lmi_op_io_submit(self.h, pipe, stream))

    def op_io_complete(self, pipe=0, stream=None):
        check(lib().lmi_op_io_complete(self.h, pipe, stream))

    def run_once(self, seeds=None, batch_counter=0, mode=MODE_TRAIN, rng_seed=0, pipe=0, stream=None):
        p, n, keep = self._seed_args(seeds)
        check(lib().lmi_run_once(self.h, pipe, stream, p, n, LOC_HOST, batch_counter, mode, rng_seed))

    def run_group(self, pipes, batch_counters, seeds=None, mode=MODE_TRAIN, rng_seeds=None, stream=None):
        """One batch per listed pipe, all served by the same launches (lmi_run_group)."""
        n = len(pipes)
        pa = (C.c_int32 * n)(*pipes)
        bc = (C.c_int32 * n)(*batch_counters)
        rs = (C.c_uint64 * n)(*rng_seeds) if rng_seeds is not None else None
        sp = ns = keep = None
        if seeds is not None:
            keep = [np.ascontiguousarray(x, dtype=np.int32) for x in seeds]
            sp = (C.c_void_p * n)(*[x.ctypes.data for x in keep])
            ns = (C.c_int32 * n)(*[len(x) for x in keep])
        check(lib().lmi_run_group(self.h, n, pa, stream, sp, ns, LOC_HOST, bc, mode, rs))

    def run_once_static(self, seeds_dev, n, view, rng_seed=0, stream=None):
        """lmi_run_once_static: `seeds_dev` is device memory holding n seed ids, `view` a BatchView of
        caller-owned device buffers; nothing is allocated by the call."""
        check(lib().lmi_run_once_static(self.h, stream, seeds_dev, n, rng_seed, C.byref(view)))

    # outputs -----------------------------------------------------------------
    def batch_wait(self, pipe=0, stream=None):
        check(lib().lmi_batch_wait(self.h, pipe, stream))

    def status(self, clear=False):
        """Raises if a kernel of any batch so far reported a bad seed id or a scan that gave up."""
        check(lib().lmi_server_status(self.h, int(clear)))

    def counters(self, pipe=0, stream=None):
        nc = np.zeros(16, np.int32)
        ec = np.zeros(16, np.int32)
        check(lib().lmi_batch_counters(self.h, pipe, stream, nc.ctypes.data, ec.ctypes.data))
        return nc, ec

    def view(self, pipe=0):
        v = BatchView()
        check(lib().lmi_batch_view_get(self.h, pipe, C.byref(v)))
        return v

    def fetch(self, pipe=0, stream=None, features=True):
        """Synchronise and copy the pipe's outputs to the host."""
        nc, ec = self.counters(pipe, stream)
        v = self.view(pipe)
        hops = int(nc[8])
        b = Batch()
        b.node_counter, b.edge_counter, b.hops = nc, ec, hops
        b.n_nodes = [int(nc[9 + k]) for k in range(hops + 1)]
        b.n_edges = [int(ec[9 + k]) for k in range(1, hops + 1)]
        b.edge_off = [int(ec[12 + k]) for k in range(1, hops + 1)]
        n, e = b.n_nodes[-1], sum(b.n_edges)
        b.ids = to_host(v.ids, n, np.int32)
        b.labels = to_host(v.labels, b.n_nodes[0], np.int32)
        b.agg_src_ids = to_host(v.agg_src_ids, e, np.int32)
        b.agg_src_off = to_host(v.agg_src_off, e, np.int32)
        b.agg_dst_off = to_host(v.agg_dst_off, e, np.int32)
        b.blk_indptr = [to_host(v.blk_indptr[k], b.n_nodes[k] + 1, np.int32) for k in range(hops)]
        b.cache_index = to_host(v.cache_index, n, np.int32)
        if features:
            d = self.cfg.feat_dim
            b.features = to_host(v.features, n * d, self.np_dtype).reshape(n, d)
        return b

    def fetch_ids(self, pipe=0, stream=None):
        """Synchronise and copy only the batch's node ids (its frontier) to the host."""
        nc, _ = self.counters(pipe, stream)
        return to_host(self.view(pipe).ids, int(nc[9 + int(nc[8])]), np.int32)

    # measurement -------------------------------------------------------------
    def profile_enable(self, level=1):
        """0 / False: off; 1 / True: events around every phase; 2: around the gather kernels only."""
        check(lib().lmi_profile_enable(self.h, int(level)))

    def profile_read(self, reset=True):
        p = Profile()
        check(lib().lmi_profile_read(self.h, C.byref(p), int(reset)))
        return p

    def tune(self, key, value):
        check(lib().lmi_tune(self.h, key.encode(), int(value)))


def bench_copy(nbytes, repeats=10):
    ms = C.c_double()
    check(lib().lmi_bench_copy(nbytes, repeats, C.byref(ms)))
    return ms.value


def bench_copy_launch(nbytes, repeats=10):
    """Mean ms of one copy launch of nbytes, each launch alone on the device and timed by its own events."""
    ms = C.c_double()
    check(lib().lmi_bench_copy_launch(nbytes, repeats, C.byref(ms)))
    return ms.value


def bench_stream(units, read_bytes, write_bytes, misalign=0, repeats=10, launch_by_launch=False):
    """Mean ms of one launch of the streaming kernel that reads read_bytes and writes write_bytes per unit."""
    ms = C.c_double()
    check(lib().lmi_bench_stream(int(units), read_bytes, write_bytes, misalign, repeats, int(launch_by_launch), C.byref(ms)))
    return ms.value


def bench_row_stream(rows, src_pitch, read_bytes, write_bytes, table_rows, repeats=10, launch_by_launch=False):
    """Mean ms of one launch of the row-streaming kernel: `rows` rows of src_pitch bytes taken from hashed
    places of a table of (a power of two <=) table_rows rows, written one after the other."""
    ms = C.c_double()
    check(lib().lmi_bench_row_stream(int(rows), int(src_pitch), read_bytes, write_bytes, int(table_rows), repeats,
                                     int(launch_by_launch), C.byref(ms)))
    return ms.value


def bench_row_stream_shape(rows, src_pitch, read_bytes, write_bytes, table_rows, rows_per_block=0, grid_blocks=0,
                           every_lane_loads=False, repeats=10, launch_by_launch=True):
    """bench_row_stream with the rows per block visit, the grid and the treatment of idle lanes chosen by the caller."""
    ms = C.c_double()
    check(lib().lmi_bench_row_stream_shape(int(rows), int(src_pitch), read_bytes, write_bytes, int(table_rows),
                                           int(rows_per_block), int(grid_blocks), int(every_lane_loads), repeats,
                                           int(launch_by_launch), C.byref(ms)))
    return ms.value


def bench_random_read(device_ptr, nbytes, n_reads=1 << 24, repeats=5):
    """Mean ms of n_reads independent random 4-byte reads of a device array of nbytes bytes."""
    ms = C.c_double()
    check(lib().lmi_bench_random_read(device_ptr, int(nbytes), int(n_reads), repeats, C.byref(ms)))
    return ms.value


def bench_host_read(host_buffer, nbytes, repeats=5):
    """Mean ms of one streaming zero-copy read of the first nbytes of a HostBuffer into HBM."""
    ms = C.c_double()
    check(lib().lmi_bench_host_read(host_buffer.ptr, min(int(nbytes), host_buffer.nbytes) // 16 * 16, repeats, C.byref(ms)))
    return ms.value


def stream_create():
    s = C.c_void_p()
    check(lib().lmi_stream_create(C.byref(s)))
    return s


def synth_graph(seed, cdf_u32, n_nodes, mode=1):
    """Generate a power-law CSR graph in HBM; returns (d_indptr, d_indices, n_edges)."""
    cdf = np.ascontiguousarray(cdf_u32, dtype=np.uint32)
    ip, ix, ne = C.c_void_p(), C.c_void_p(), C.c_int64()
    check(lib().lmi_synth_graph(seed, cdf.ctypes.data, len(cdf), n_nodes, mode, C.byref(ip), C.byref(ix),
                                C.byref(ne)))
    return ip, ix, ne.value


def synth_trainset(seed, n_nodes, n_train):
    ids = np.empty(n_train, np.int32)
    check(lib().lmi_synth_trainset(seed, n_nodes, n_train, ids.ctypes.data))
    return ids


def synth_features(seed, host_buffer):
    dt = F16 if host_buffer.dtype == np.float16 else F32
    check(lib().lmi_synth_features(seed, host_buffer.ptr, host_buffer.shape[0], host_buffer.shape[1], dt))


def zipf_cdf(alpha, d_max, mean_degree):
    """uint32 inverse-CDF table of P(d) ~ (d + q)^-alpha on d = 1..d_max, with the
    shift q chosen by bisection so that the mean is `mean_degree` (entry 0, degree
    0, has probability 0)."""
    d = np.arange(1, d_max + 1, dtype=np.float64)

    def mean(q):
        w = (d + q) ** (-alpha)
        return float((w * d).sum() / w.sum())

    lo, hi = 0.0, 1.0
    if mean(0.0) < mean_degree:
        while mean(hi) < mean_degree and hi < 1e9:
            hi *= 2
        for _ in range(80):
            mid = 0.5 * (lo + hi)
            if mean(mid) < mean_degree:
                lo = mid
            else:
                hi = mid
    q = 0.5 * (lo + hi) if mean(0.0) < mean_degree else 0.0
    w = (d + q) ** (-alpha)
    cdf = np.cumsum(w) / w.sum()
    t = np.minimum(np.floor(cdf * 4294967296.0), 4294967295.0).astype(np.uint64)
    t[-1] = 4294967295
    return np.concatenate([[0], t]).astype(np.uint32)
