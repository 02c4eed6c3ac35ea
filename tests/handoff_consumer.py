"""Trainer process of the hand-off test (run by test_gpu_handoff.py as a subprocess, so that
a failure inside the server thread, which ends the process like the reference's error checks
do, cannot take the test runner with it).

Starts the sampling server on a background thread -- or, with `attach`, takes the batches of a
`sampling_server` process that is already up (the reference's two-process deployment: the
buffers are then opened through inter-process memory handles, before this process does any
other GPU work) --, consumes every batch of the reference's schedule through the `ipc_service`
functions and checks each against the CPU oracle.
usage: handoff_consumer.py <dataset dir> <batch> <dim> <epochs> <dyn_cache> <numpy|torch> [attach]
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from conftest import load_ipc_service  # noqa: E402
from oracle import binding as oracle  # noqa: E402


def main():
    data, batch, dim, epochs, dyn_cache, flavour = sys.argv[1], int(sys.argv[2]), int(sys.argv[3]), int(sys.argv[4]), \
        int(sys.argv[5]), sys.argv[6]
    fanout = [7, 4]
    indptr = np.fromfile(os.path.join(data, "edge_src"), np.int64)
    indices = np.fromfile(os.path.join(data, "edge_dst"), np.int32)
    n_nodes = len(indptr) - 1
    # element type of the `features` file: the server and this consumer learn it the same way
    f16 = os.environ.get("LEGION_MI_FEAT_DTYPE") == "f16"
    np_dtype = np.float16 if f16 else np.float32
    feats = np.fromfile(os.path.join(data, "features"), np_dtype).reshape(n_nodes, dim)
    labels = np.fromfile(os.path.join(data, "labels"), np.int32)
    sets = [np.fromfile(os.path.join(data, n), np.int32) for n in ("trainingset", "validationset", "testingset")]
    ipc = load_ipc_service()
    steps_ref, sizes, total = ipc.schedule(len(sets[0]), len(sets[1]), len(sets[2]), batch, epochs)

    if dyn_cache == 8:   # int8 cache: hits arrive dequantised; the oracle's codec says what they must be
        cache_bytes = int(open(os.environ.get("LEGION_MI_META_CONFIG", "meta_config")).read().split()[8])
        slot = oracle.static_cache_build(indptr, cache_bytes // (dim + 4))
        q, sc = oracle.quantize_rows(feats[np.flatnonzero(slot >= 0)])
    attach = len(sys.argv) > 7 and sys.argv[7] == "attach"
    if not attach:
        ipc.start_server(dyn_cache=dyn_cache, fanout=fanout, wait_seconds=60.0)
    ipc.initialize()
    assert ipc.get_steps() == steps_ref, (ipc.get_steps(), steps_ref)
    for g in range(total):
        mode, local = ipc.schedule_batch(len(sets[0]), len(sets[1]), len(sets[2]), batch, epochs, g)
        seeds = sets[mode][local * sizes[mode]:(local + 1) * sizes[mode]]
        if flavour == "torch":
            out = [t.cpu().numpy() for t in ipc.get_next(dim, wait_seconds=60.0, feature_typestr="<f2" if f16 else "<f4")]
        else:
            out = ipc.get_next_numpy(dim, wait_seconds=60.0, feature_dtype=np_dtype)
        o = oracle.sample_batch(indptr, indices, seeds, fanout, 1 + local)
        ids, f, lab = out[0], out[1], out[2]
        assert np.array_equal(ids, o.ids), "ids of batch %d" % g
        want = oracle.gather_rows_int8(o.ids, slot[o.ids], q, sc, feats) if dyn_cache == 8 else feats[o.ids]
        assert f.tobytes() == want.tobytes(), "features of batch %d" % g
        assert np.array_equal(lab, labels[seeds]), "labels of batch %d" % g
        hops = len(fanout)
        sizes_ref = []
        for k in range(hops):                 # blocks arrive from the last hop to the first
            h = hops - 1 - k
            lo, n = o.edge_off[h], o.n_edges[h]
            assert np.array_equal(out[3 + 2 * k], o.agg_src_off[lo:lo + n]), "src of block %d, batch %d" % (h, g)
            assert np.array_equal(out[4 + 2 * k], o.agg_dst_off[lo:lo + n]), "dst of block %d, batch %d" % (h, g)
            sizes_ref += [o.n_nodes[h + 1], o.n_nodes[h]]
        assert ipc.get_block_size() == sizes_ref, (ipc.get_block_size(), sizes_ref)
        ipc.synchronize()
    ipc.finalize()
    if not attach:
        ipc.join_server()
    print("HANDOFF_OK %d batches" % total, flush=True)


if __name__ == "__main__":
    main()
