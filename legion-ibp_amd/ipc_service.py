"""Trainer-side consumer of the sampling server's mini-batches.

Same functions as the reference's `ipc_service` extension module (Legion-IBP
training_backend/ipc_service.cpp:15-97: initialize, get_next, get_block_size, get_steps,
synchronize, finalize; used by training_backend/legion_graphsage.py), over
liblegion_trainer.so.  The sampling server is another process (the `sampling_server`
binary with LEGION_MI_HANDOFF=1, as the reference deploys it: `initialize` opens its output
buffers through inter-process memory handles and must come before any other GPU work of
this process) or a background thread of this one (`start_server`).

    start_server(dyn_cache=0, fanout=[25, 10])      # reads ./meta_config, builds the cache
    initialize()
    train_steps, valid_steps, test_steps = get_steps()
    for _ in range(...):
        ids, features, labels, src2, dst2, src1, dst1 = get_next(feature_dim)   # torch tensors on the GPU
        sizes = get_block_size()
        ...train...
        synchronize()                                # hands the buffers back to the sampler
    finalize(); join_server()

`get_next` returns torch tensors that alias the server's device buffers (features are a
fresh copy, as in the reference); `get_next_numpy` returns host copies and needs no torch.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
MAX_HOPS = 3


class Batch(C.Structure):
    _fields_ = [("ids", C.c_void_p), ("n_ids", C.c_int64), ("features", C.c_void_p),
                ("labels", C.c_void_p), ("n_labels", C.c_int64), ("hop_num", C.c_int32),
                ("agg_src", C.c_void_p * MAX_HOPS), ("agg_dst", C.c_void_p * MAX_HOPS),
                ("n_edges", C.c_int64 * MAX_HOPS),
                ("node_counter", C.c_int32 * 16), ("edge_counter", C.c_int32 * 16)]


_libs = None


def _load():
    global _libs
    if _libs is None:
        paths = [os.path.join(_HERE, n) for n in ("liblegion_mi.so", "liblegion_server.so", "liblegion_trainer.so")]
        for p in paths:
            if not os.path.exists(p):
                raise ImportError("%s is missing: build it with `make -C %s`" % (p, _HERE))
        mi = C.CDLL(paths[0], mode=C.RTLD_GLOBAL)
        srv = C.CDLL(paths[1], mode=C.RTLD_GLOBAL)
        tr = C.CDLL(paths[2], mode=C.RTLD_GLOBAL)
        srv.legion_server_start.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int32), C.c_int, C.c_int, C.c_double]
        srv.legion_schedule.argtypes = [C.c_int32] * 5 + [C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
        srv.legion_schedule.restype = None
        srv.legion_schedule_batch.argtypes = [C.c_int32] * 6 + [C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
        srv.legion_schedule_batch.restype = None
        tr.legion_ipc_last_error.restype = C.c_char_p
        tr.legion_ipc_get_next.argtypes = [C.POINTER(Batch), C.c_double]
        tr.legion_ipc_get_block_size.argtypes = [C.POINTER(C.c_int32), C.c_int]
        tr.legion_ipc_get_steps.argtypes = [C.POINTER(C.c_int32)]
        tr.legion_ipc_get_steps.restype = None
        tr.legion_ipc_synchronize.restype = None
        tr.legion_ipc_finalize.restype = None
        mi.lmi_copy_to_host.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        _libs = (mi, srv, tr)
    return _libs


class HandoffError(RuntimeError):
    pass


# ------------------------------------------------------------------ the server thread
def start_server(dyn_cache=0, fanout=(25, 10), cache_agg_mode=0, wait_seconds=600.0, handoff=True):
    """Initialize + PreSc of a sampling server on a background thread (returns once the
    server is ready to serve); its Run loop then waits for this process's trainer."""
    _, srv, _ = _load()
    fan = (C.c_int32 * len(fanout))(*fanout)
    if srv.legion_server_start(1, cache_agg_mode, dyn_cache, fan, len(fanout), int(handoff), float(wait_seconds)) != 0:
        raise HandoffError("a sampling server is already running in this process")


def join_server():
    _, srv, _ = _load()
    srv.legion_server_join()


def schedule(train_n, valid_n, test_n, raw_batch, epoch):
    """The reference's batch schedule: (steps[3], ids per batch[3], total batches)."""
    _, srv, _ = _load()
    steps, sizes, total = (C.c_int32 * 3)(), (C.c_int32 * 3)(), C.c_int32()
    srv.legion_schedule(train_n, valid_n, test_n, raw_batch, epoch, steps, sizes, C.byref(total))
    return list(steps), list(sizes), total.value


def schedule_batch(train_n, valid_n, test_n, raw_batch, epoch, global_batch_id):
    """(mode, place in the id set) of one batch of the schedule."""
    _, srv, _ = _load()
    mode, local = C.c_int32(), C.c_int32()
    srv.legion_schedule_batch(train_n, valid_n, test_n, raw_batch, epoch, global_batch_id, C.byref(mode), C.byref(local))
    return mode.value, local.value


# ------------------------------------------------------------- the reference's module
def initialize():
    _, _, tr = _load()
    if tr.legion_ipc_initialize() != 0:
        raise HandoffError(tr.legion_ipc_last_error().decode())


def _next(wait_seconds):
    _, _, tr = _load()
    b = Batch()
    if tr.legion_ipc_get_next(C.byref(b), float(wait_seconds)) != 0:
        raise HandoffError(tr.legion_ipc_last_error().decode())
    return b


class _DeviceArray:
    """Exposes a raw device address through the CUDA array interface (torch reads it on ROCm too)."""

    def __init__(self, ptr, shape, typestr):
        self.__cuda_array_interface__ = {"data": (int(ptr), False), "shape": tuple(shape), "typestr": typestr,
                                         "version": 2, "strides": None}


def get_next(feature_dim, wait_seconds=600.0, feature_typestr="<f4"):
    """[ids, features, labels, src_L, dst_L, ..., src_1, dst_1] as torch tensors on the GPU
    (blocks from the last hop to the first, training_backend/ipc_cuda_kernel.cu:194-240)."""
    import torch

    b = _next(wait_seconds)
    dev = torch.device("cuda", 0)

    def view(ptr, shape, typestr="<i4"):
        if int(np.prod(shape)) == 0:
            return torch.empty(shape, dtype=torch.float32 if typestr == "<f4" else
                               (torch.float16 if typestr == "<f2" else torch.int32), device=dev)
        return torch.as_tensor(_DeviceArray(ptr, shape, typestr), device=dev)

    out = [view(b.ids, (b.n_ids,)), view(b.features, (b.n_ids, feature_dim), feature_typestr).clone(),
           view(b.labels, (b.n_labels,))]
    for k in range(b.hop_num):
        out.append(view(b.agg_src[k], (b.n_edges[k],)))
        out.append(view(b.agg_dst[k], (b.n_edges[k],)))
    return out


def get_next_numpy(feature_dim, wait_seconds=600.0, feature_dtype=np.float32):
    """The same list as host copies (numpy), for consumers without torch."""
    mi, _, _ = _load()
    b = _next(wait_seconds)

    def copy(ptr, shape, dtype=np.int32):
        a = np.empty(shape, dtype)
        if a.size and mi.lmi_copy_to_host(a.ctypes.data_as(C.c_void_p), C.c_void_p(ptr), a.nbytes) != 0:
            raise HandoffError("device to host copy failed")
        return a

    out = [copy(b.ids, (b.n_ids,)), copy(b.features, (b.n_ids, feature_dim), feature_dtype), copy(b.labels, (b.n_labels,))]
    for k in range(b.hop_num):
        out.append(copy(b.agg_src[k], (b.n_edges[k],)))
        out.append(copy(b.agg_dst[k], (b.n_edges[k],)))
    return out


def get_block_size():
    """[src nodes, dst nodes] per block of the batch get_next returned last, last hop first."""
    _, _, tr = _load()
    buf = (C.c_int32 * (2 * MAX_HOPS))()
    n = tr.legion_ipc_get_block_size(buf, 2 * MAX_HOPS)
    return list(buf[:n])


def get_steps():
    _, _, tr = _load()
    s = (C.c_int32 * 3)()
    tr.legion_ipc_get_steps(s)
    return list(s)


def synchronize():
    _, _, tr = _load()
    tr.legion_ipc_synchronize()


def finalize():
    _, _, tr = _load()
    tr.legion_ipc_finalize()
