"""The reference-shaped entry point: the `sampling_server` binary (same argv as the
reference's main.cu) reading ./meta_config and a dataset in the Legion on-disk
format, driven through the C++ Server/Runner/Operator shim.  Its dumped batches are
compared with the CPU oracle."""
import os
import subprocess

import numpy as np
import pytest

from conftest import ROOT, random_graph

pytestmark = pytest.mark.gpu
BIN = os.path.join(ROOT, "legion-ibp_amd", "sampling_server")


def write_dataset(d, rng, n_nodes, dim, n_train, dtype=np.float32):
    indptr, indices = random_graph(rng, n_nodes, 10, hubs=4, hub_deg=300)
    feats = rng.standard_normal((n_nodes, dim)).astype(dtype)
    labels = rng.integers(0, 40, n_nodes).astype(np.int32)
    perm = rng.permutation(n_nodes).astype(np.int32)
    train, valid, test = perm[:n_train], perm[n_train:n_train + 50], perm[n_train + 50:n_train + 90]
    indptr.astype(np.int64).tofile(os.path.join(d, "edge_src"))
    indices.astype(np.int32).tofile(os.path.join(d, "edge_dst"))
    feats.tofile(os.path.join(d, "features"))
    labels.tofile(os.path.join(d, "labels"))
    train.tofile(os.path.join(d, "trainingset"))
    valid.tofile(os.path.join(d, "validationset"))
    test.tofile(os.path.join(d, "testingset"))
    return indptr, indices, feats, train


def read_sets(d):
    return [np.fromfile(os.path.join(d, n), np.int32) for n in ("trainingset", "validationset", "testingset")]


def read_dump(path, dim, dtype=np.float32):
    raw = np.fromfile(path, np.uint8)
    words = dim * np.dtype(dtype).itemsize // 4     # 4-byte words of a feature row
    raw, dim = raw.view(np.int32), words
    nc, ec = raw[:16], raw[16:32]
    hops = int(nc[8])
    n, e = int(nc[9 + hops]), int(sum(ec[10:10 + hops]))
    o = 32
    ids = raw[o:o + n]; o += n
    src = raw[o:o + e]; o += e
    dst = raw[o:o + e]; o += e
    feat = raw[o:o + n * dim].view(dtype).reshape(n, -1)
    assert o + n * dim == len(raw)
    return nc, ec, ids, src, dst, feat


@pytest.mark.parametrize("dyn_cache,table_mode,presample,dtype", [
    (0, False, False, "f32"), (0, True, False, "f32"), (1, False, False, "f32"), (1, True, False, "f32"),
    (8, False, False, "f32"), (0, True, True, "f32"),
    (0, False, False, "f16"), (1, False, False, "f16"), (8, False, False, "f16")])   # fp16 `features` file
def test_sampling_server_binary(tmp_path, oracle, dyn_cache, table_mode, presample, dtype):
    assert os.path.exists(BIN), "build the host shim first (make -C legion-ibp_amd)"
    rng = np.random.default_rng(dyn_cache * 2 + table_mode)
    n_nodes, dim, batch, n_train, fanout = 5000, 64, 100, 350, [25, 10]
    data = tmp_path / "data"
    data.mkdir()
    np_dtype = np.float16 if dtype == "f16" else np.float32
    indptr, indices, feats, train = write_dataset(str(data), rng, n_nodes, dim, n_train, np_dtype)
    cache_bytes = 1500 * dim * 4
    (tmp_path / "meta_config").write_text("%s/ %d %d %d %d %d %d %d %d %d" % (
        data, batch, n_nodes, len(indices), dim, n_train, 50, 40, cache_bytes, 2))
    dump = tmp_path / "dump"
    dump.mkdir()
    env = dict(os.environ, LEGION_MI_DUMP=str(dump), LEGION_MI_DUMP_BATCHES="4")
    if dtype == "f16":
        env["LEGION_MI_FEAT_DTYPE"] = "f16"
    if table_mode:
        env["LEGION_MI_OPERATOR_TABLE"] = "1"
    if presample:
        env["LEGION_MI_PRESAMPLE"] = "1"   # rank the hot set by a presampling pass, as the reference does
    out = subprocess.run([BIN, "1", "0", str(dyn_cache), "25,10"], cwd=str(tmp_path), env=env, timeout=100,
                         capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    # the reference's schedule: (350-1)/100 = 3 training steps and 1 validation step per epoch,
    # 1 test step after the last epoch
    assert "System is ready for serving" in out.stdout and "batches: 9" in out.stdout
    if dyn_cache == 8:
        slot = oracle.static_cache_build(indptr, cache_bytes // (dim + 4))
        q, sc = oracle.quantize_rows(feats[np.flatnonzero(slot >= 0)])
    valid = read_sets(str(data))[1]
    for i in range(4):   # three training batches of 100, then the validation batch of 50
        nc, ec, ids, src, dst, feat = read_dump(str(dump / ("batch_%d.bin" % i)), dim, np_dtype)
        seeds, local = (train[i * batch:(i + 1) * batch], i) if i < 3 else (valid, 0)
        o = oracle.sample_batch(indptr, indices, seeds, fanout, 1 + local)
        assert list(nc) == list(o.node_counter) and list(ec) == list(o.edge_counter)
        assert np.array_equal(ids, o.ids) and np.array_equal(src, o.agg_src_off) and np.array_equal(dst, o.agg_dst_off)
        if dyn_cache == 8:
            ref = oracle.gather_rows_int8(o.ids, slot[o.ids], q, sc, feats)
            assert feat.tobytes() == ref.tobytes()
        else:
            assert feat.tobytes() == feats[o.ids].tobytes()


def test_sampling_server_rejects_two_gpus(tmp_path):
    (tmp_path / "meta_config").write_text("/nonexistent/ 10 10 10 4 1 0 0 100 1")
    out = subprocess.run([BIN, "2", "0", "0"], cwd=str(tmp_path), timeout=60, capture_output=True, text=True)
    assert out.returncode != 0 and "one GPU" in out.stderr


def test_sampling_server_stops_on_a_seed_outside_the_graph(tmp_path):
    """A training set that names a node the graph does not have: the reference would abort on the
    resulting device error (engine/memorypool.cuh:9-17); the shim exits non-zero and says why
    instead of reporting a served epoch."""
    rng = np.random.default_rng(77)
    n_nodes, dim, batch, n_train = 3000, 16, 50, 160
    data = tmp_path / "data"
    data.mkdir()
    indptr, indices, feats, train = write_dataset(str(data), rng, n_nodes, dim, n_train)
    train = train.copy()
    train[60] = n_nodes + 5          # second batch
    train.tofile(str(data / "trainingset"))
    (tmp_path / "meta_config").write_text("%s/ %d %d %d %d %d %d %d %d %d" % (
        data, batch, n_nodes, len(indices), dim, n_train, 50, 40, 500 * dim * 4, 1))
    out = subprocess.run([BIN, "1", "0", "0", "25,10"], cwd=str(tmp_path), timeout=100, capture_output=True, text=True)
    assert out.returncode != 0, out.stdout + out.stderr
    assert "seed id outside" in out.stderr, out.stdout + out.stderr
    assert "batches:" not in out.stdout       # the run did not report a throughput
