"""ctypes binding of the CPU oracle (oracle/liblegion_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py -- never by the product package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblegion_oracle.so")
MAX_HOPS = 3
F32, F16 = 0, 1


def build(force=False):
    """Compile the oracle with its Makefile (g++)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])


def _ptr(a, ctype):
    return a.ctypes.data_as(C.POINTER(ctype)) if a is not None else None


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.orc_draw.restype = C.c_uint32
        L.orc_draw.argtypes = [C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint32]
        L.orc_sample_positions.restype = C.c_int32
        L.orc_sample_positions.argtypes = [C.c_uint64, C.c_int32, C.c_int32, C.c_int64, C.c_int32,
                                           C.POINTER(C.c_int64)]
        L.orc_sample_batch.restype = C.c_int
        L.orc_lru_create.restype = C.c_void_p
        L.orc_lru_create.argtypes = [C.c_int64, C.c_int32, C.c_int64]
        L.orc_lru_destroy.argtypes = [C.c_void_p]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        _lib = L
    return _lib


def philox4x32_10(ctr, key):
    c = np.asarray(ctr, dtype=np.uint32)
    k = np.asarray(key, dtype=np.uint32)
    o = np.zeros(4, dtype=np.uint32)
    lib().orc_philox4x32_10(_ptr(c, C.c_uint32), _ptr(k, C.c_uint32), _ptr(o, C.c_uint32))
    return o


def draw(seed, hop, node, slot):
    return lib().orc_draw(seed, hop, node, slot)


def sample_positions(seed, hop, node, deg, fanout):
    pos = np.zeros(max(fanout, 1), dtype=np.int64)
    n = lib().orc_sample_positions(seed, hop, node, deg, fanout, _ptr(pos, C.c_int64))
    return pos[:n].copy()


def batch_caps(n_seeds, fanout):
    """Worst-case node / edge / indptr counts: n_k <= n_{k-1}(1+f_k)."""
    n, e_tot, ip = n_seeds, 0, 0
    for f in fanout:
        ip += n + 1
        e = n * f
        e_tot += e
        n += e
    return n, e_tot, ip


class Batch:
    """Result of one oracle mini-batch (numpy views trimmed to the real sizes)."""


def sample_batch(indptr, indices, seeds, fanout, seed, threads=0):
    indptr = np.ascontiguousarray(indptr, dtype=np.int64)
    indices = np.ascontiguousarray(indices, dtype=np.int32)
    seeds = np.ascontiguousarray(seeds, dtype=np.int32)
    fan = np.ascontiguousarray(fanout, dtype=np.int32)
    hops = len(fan)
    ncap, ecap, ipcap = batch_caps(len(seeds), list(fan))
    ids = np.empty(max(ncap, 1), np.int32)
    src_g = np.empty(max(ecap, 1), np.int32)
    src_l = np.empty(max(ecap, 1), np.int32)
    dst_l = np.empty(max(ecap, 1), np.int32)
    ipt = np.empty(max(ipcap, 1), np.int32)
    nc = np.zeros(16, np.int32)
    ec = np.zeros(16, np.int32)
    rc = lib().orc_sample_batch(
        _ptr(indptr, C.c_int64), _ptr(indices, C.c_int32), C.c_int64(len(indptr) - 1),
        _ptr(seeds, C.c_int32), C.c_int32(len(seeds)), _ptr(fan, C.c_int32), C.c_int32(hops),
        C.c_uint64(seed), _ptr(ids, C.c_int32), C.c_int64(ncap),
        _ptr(src_g, C.c_int32), _ptr(src_l, C.c_int32), _ptr(dst_l, C.c_int32), C.c_int64(ecap),
        _ptr(ipt, C.c_int32), C.c_int64(ipcap), _ptr(nc, C.c_int32), _ptr(ec, C.c_int32),
        C.c_int(threads))
    if rc != 0:
        raise RuntimeError("orc_sample_batch failed: %d" % rc)
    b = Batch()
    b.node_counter, b.edge_counter = nc, ec
    b.hops = hops
    b.n_nodes = [int(nc[9 + k]) for k in range(hops + 1)]
    b.n_edges = [int(ec[9 + k]) for k in range(1, hops + 1)]
    b.edge_off = [int(ec[12 + k]) for k in range(1, hops + 1)]
    tot_e = sum(b.n_edges)
    b.ids = ids[:b.n_nodes[-1]]
    b.agg_src_ids = src_g[:tot_e]
    b.agg_src_off = src_l[:tot_e]
    b.agg_dst_off = dst_l[:tot_e]
    b.blk_indptr, off = [], 0
    for k in range(hops):
        b.blk_indptr.append(ipt[off:off + b.n_nodes[k] + 1])
        off += b.n_nodes[k] + 1
    return b


def static_cache_build(indptr, cap_rows):
    indptr = np.ascontiguousarray(indptr, dtype=np.int64)
    n = len(indptr) - 1
    slot_of = np.empty(n, np.int32)
    lib().orc_static_cache_build(_ptr(indptr, C.c_int64), C.c_int64(n), C.c_int64(cap_rows),
                                 _ptr(slot_of, C.c_int32))
    return slot_of


def static_cache_build_keys(keys, cap_rows):
    keys = np.ascontiguousarray(keys, dtype=np.int64)
    slot_of = np.empty(len(keys), np.int32)
    lib().orc_static_cache_build_keys(_ptr(keys, C.c_int64), C.c_int64(len(keys)), C.c_int64(cap_rows),
                                      _ptr(slot_of, C.c_int32))
    return slot_of


class Lru:
    def __init__(self, n_sets, ways, row_bytes):
        self.n_sets, self.ways, self.row_bytes = n_sets, ways, row_bytes
        self.h = C.c_void_p(lib().orc_lru_create(n_sets, ways, row_bytes))

    def access(self, ids, host_rows=None):
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        n = len(ids)
        hit = np.empty(n, np.int32)
        fill = np.empty(n, np.int32)
        out = None
        hp = None
        op = None
        if host_rows is not None:
            out = np.empty((n, self.row_bytes), np.uint8)
            hp = host_rows.ctypes.data_as(C.c_void_p)
            op = out.ctypes.data_as(C.c_void_p)
        lib().orc_lru_access(self.h, _ptr(ids, C.c_int32), C.c_int64(n), _ptr(hit, C.c_int32),
                             _ptr(fill, C.c_int32), hp, op)
        return hit, fill, out

    def state(self):
        k = np.empty(self.n_sets * self.ways, np.int32)
        u = np.empty(self.n_sets * self.ways, np.int32)
        lib().orc_lru_state(self.h, _ptr(k, C.c_int32), _ptr(u, C.c_int32))
        return k, u

    def __del__(self):
        try:
            lib().orc_lru_destroy(self.h)
        except Exception:
            pass


def f32_to_f16(x):
    return lib().orc_f32_to_f16(float(x))


def f16_to_f32(h):
    return lib().orc_f16_to_f32(int(h))


def quantize_rows(rows):
    rows = np.ascontiguousarray(rows)
    dt = F16 if rows.dtype == np.float16 else F32
    n, d = rows.shape
    q = np.empty((n, d), np.int8)
    sc = np.empty(n, np.float32)
    lib().orc_quantize_rows(rows.ctypes.data_as(C.c_void_p), C.c_int32(dt), C.c_int64(n),
                            C.c_int32(d), _ptr(q, C.c_int8), _ptr(sc, C.c_float))
    return q, sc


def dequant_rows(q, scale, out_dtype):
    q = np.ascontiguousarray(q, dtype=np.int8)
    scale = np.ascontiguousarray(scale, dtype=np.float32)
    n, d = q.shape
    out = np.empty((n, d), out_dtype)
    dt = F16 if out.dtype == np.float16 else F32
    lib().orc_dequant_rows(_ptr(q, C.c_int8), _ptr(scale, C.c_float), C.c_int64(n), C.c_int32(d),
                           out.ctypes.data_as(C.c_void_p), C.c_int32(dt))
    return out


def gather_rows(ids, slot, cache_rows, host_rows, threads=0):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    slot = np.ascontiguousarray(slot, dtype=np.int32)
    rb = host_rows.shape[1] * host_rows.dtype.itemsize
    out = np.empty((len(ids), host_rows.shape[1]), host_rows.dtype)
    cp = cache_rows.ctypes.data_as(C.c_void_p) if cache_rows is not None else None
    lib().orc_gather_rows(_ptr(ids, C.c_int32), _ptr(slot, C.c_int32), C.c_int64(len(ids)), cp,
                          host_rows.ctypes.data_as(C.c_void_p), C.c_int64(rb),
                          out.ctypes.data_as(C.c_void_p), C.c_int(threads))
    return out


def gather_rows_int8(ids, slot, q_rows, scales, host_rows, threads=0):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    slot = np.ascontiguousarray(slot, dtype=np.int32)
    dt = F16 if host_rows.dtype == np.float16 else F32
    out = np.empty((len(ids), host_rows.shape[1]), host_rows.dtype)
    lib().orc_gather_rows_int8(_ptr(ids, C.c_int32), _ptr(slot, C.c_int32), C.c_int64(len(ids)),
                               _ptr(q_rows, C.c_int8), _ptr(scales, C.c_float),
                               host_rows.ctypes.data_as(C.c_void_p), C.c_int32(host_rows.shape[1]),
                               C.c_int32(dt), out.ctypes.data_as(C.c_void_p), C.c_int(threads))
    return out


def synth_graph(seed, cdf_u32, n_nodes, mode=1, threads=0):
    cdf = np.ascontiguousarray(cdf_u32, dtype=np.uint32)
    indptr = np.empty(n_nodes + 1, np.int64)
    lib().orc_synth_degrees(C.c_uint64(seed), _ptr(cdf, C.c_uint32), C.c_int32(len(cdf)),
                            C.c_int64(n_nodes), _ptr(indptr, C.c_int64))
    indices = np.empty(max(int(indptr[-1]), 1), np.int32)
    lib().orc_synth_indices(C.c_uint64(seed), _ptr(indptr, C.c_int64), C.c_int64(n_nodes),
                            C.c_int32(mode), _ptr(indices, C.c_int32), C.c_int(threads))
    return indptr, indices[:int(indptr[-1])]


def synth_trainset(seed, n_nodes, n_train):
    ids = np.empty(n_train, np.int32)
    lib().orc_synth_trainset(C.c_uint64(seed), C.c_int64(n_nodes), C.c_int32(n_train),
                             _ptr(ids, C.c_int32))
    return ids
