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


# group: None = the server's own choice (groups of up to 8 batches of one mode when nothing takes the batches
# one by one -- here the static and int8 caches without the operator table), 1 = one batch per RunOnce as in
# the reference, 2 = small groups, so that the three training steps of an epoch go out as 2 + 1
@pytest.mark.parametrize("dyn_cache,table_mode,presample,dtype,group", [
    (0, False, False, "f32", None), (0, False, False, "f32", 1), (0, False, False, "f32", 2),
    (0, True, False, "f32", None), (1, False, False, "f32", None), (1, True, False, "f32", None),
    (8, False, False, "f32", None), (0, True, True, "f32", None), (0, False, True, "f32", None),
    (0, False, False, "f16", None), (1, False, False, "f16", None), (8, False, False, "f16", None),   # fp16 `features` file
    (0, False, False, "f32", "tuned"), (8, False, False, "f16", "tuned")])   # knobs through LEGION_MI_TUNE: split lookups
def test_sampling_server_binary(tmp_path, oracle, dyn_cache, table_mode, presample, dtype, group):
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
    env = dict(os.environ, LEGION_MI_DUMP=str(dump), LEGION_MI_DUMP_BATCHES="9")
    if group == "tuned":
        env["LEGION_MI_TUNE"] = "split_lookup=2,miss_blocks=16,miss_blocks_early=8"
    elif group:
        env["LEGION_MI_GROUP"] = str(group)
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
    _, valid, test = read_sets(str(data))
    # every batch of the schedule, in order: per epoch three training batches of 100 and the validation
    # batch of 50, the test batch of 40 at the end
    schedule = ([(train[k * batch:(k + 1) * batch], k) for k in range(3)] + [(valid, 0)]) * 2 + [(test, 0)]
    for i, (seeds, local) in enumerate(schedule):
        nc, ec, ids, src, dst, feat = read_dump(str(dump / ("batch_%d.bin" % i)), dim, np_dtype)
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


@pytest.fixture(scope="module")
def products_on_disk(tmp_path_factory, lmi):
    """A products-sized dataset in the reference's on-disk format (2.45 M nodes, 61.9 M edges, 100-d
    fp32 rows, batch 800, cache = 30 % of the rows, 8 epochs of 245 training steps), written from
    bench.py's synthetic graph."""
    import sys
    sys.path.insert(0, ROOT)
    import bench
    if bench.mem_available_gb() < 16:
        pytest.skip("needs a few GB of host memory and of /tmp")
    root = tmp_path_factory.mktemp("products")
    w = dict(bench.WORKLOADS["products"])
    inputs = bench.build_inputs(lmi, w, 20260101, 8.0)
    data = root / "data"
    data.mkdir()
    try:
        n_nodes, n_edges, n_train = inputs["n_nodes"], inputs["n_edges"], inputs["n_train"]
        lmi.to_host(inputs["d_indptr"], n_nodes + 1, np.int64).tofile(str(data / "edge_src"))
        lmi.to_host(inputs["d_indices"], n_edges, np.int32).tofile(str(data / "edge_dst"))
        inputs["feats"].array.tofile(str(data / "features"))
        inputs["train"].astype(np.int32).tofile(str(data / "trainingset"))
    finally:
        bench.free_inputs(lmi, inputs)
    epochs = 8
    cache_bytes = int(n_nodes * 0.30) * w["dim"] * 4
    (root / "meta_config").write_text("%s/ %d %d %d %d %d %d %d %d %d" % (
        data, w["batch"], n_nodes, n_edges, w["dim"], n_train, 0, 0, cache_bytes, epochs))
    return dict(root=root, steps=(n_train - 1) // w["batch"] * epochs, batch=w["batch"])


def test_server_run_reaches_the_rate_of_the_grouped_path(products_on_disk):
    """The products-sized dataset served by the `sampling_server` binary through Server::Run, which
    issues groups of eight batches on sixteen buffer sets when nothing takes the batches one by one: its
    own batches/s line against bench.py's products figure (the same graph, the same issue pattern through
    the Python binding)."""
    import json
    import re
    import sys
    root, steps = products_on_disk["root"], products_on_disk["steps"]
    out = subprocess.run([BIN, "1", "0", "0", "25,10"], cwd=str(root), timeout=300, capture_output=True, text=True)
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-2000:]
    m = re.search(r"batches: (\d+) .*\(([0-9.]+) batches/s\)", out.stdout)
    assert m and int(m.group(1)) == steps, out.stdout[-2000:]
    served = float(m.group(2))
    one = subprocess.run([BIN, "1", "0", "0", "25,10"], cwd=str(root), timeout=300, capture_output=True, text=True,
                         env=dict(os.environ, LEGION_MI_GROUP="1"))
    assert one.returncode == 0, one.stdout[-2000:] + one.stderr[-2000:]
    one_by_one = float(re.search(r"\(([0-9.]+) batches/s\)", one.stdout).group(1))
    table = subprocess.run([BIN, "1", "0", "0", "25,10"], cwd=str(root), timeout=300, capture_output=True, text=True,
                           env=dict(os.environ, LEGION_MI_OPERATOR_TABLE="1"))
    assert table.returncode == 0, table.stdout[-2000:] + table.stderr[-2000:]
    by_operator = float(re.search(r"\(([0-9.]+) batches/s\)", table.stdout).group(1))
    ref = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "products", "--steps", str(steps),
                          "--warmup", "16", "--cpu-seconds", "0", "--runner-steps", "0", "--companion-steps", "0"],
                         timeout=600, capture_output=True, text=True)
    assert ref.returncode == 0, ref.stderr[-3000:]
    line = json.loads(ref.stdout.strip().splitlines()[-1])
    print("Server::Run %.0f batches/s (one batch per RunOnce: %.0f, operator by operator: %.0f); "
          "bench.py --workload products %.0f batches/s" % (served, one_by_one, by_operator, line["value"]))
    assert served >= 0.90 * line["value"], (served, line["value"])   # 0.96 measured, box after box
    assert served > one_by_one


def test_handoff_rate_with_a_trainer_that_only_takes_the_batches(products_on_disk):
    """The same dataset through the two-process hand-off (two buffer sets, two semaphores each, as the
    reference deploys it) with a trainer that releases every batch at once: what the sampler side of the
    hand-off sustains.  The runner posts batch i while batch i + 1 is already queued, so the rate stays
    near that of the free-running one-batch-per-call loop."""
    import re
    import sys
    import time
    root, steps = products_on_disk["root"], products_on_disk["steps"]
    env = dict(os.environ, LEGION_MI_HANDOFF="1", LEGION_MI_WAIT_SECONDS="120")
    log_path = root / "handoff_server.log"
    with open(log_path, "w") as log:
        server = subprocess.Popen([BIN, "1", "0", "0", "25,10"], cwd=str(root), env=env, stdout=log, stderr=subprocess.STDOUT)
    try:
        deadline = time.time() + 200
        while "System is ready for serving" not in log_path.read_text():
            assert server.poll() is None, "the server ended early:\n" + log_path.read_text()[-3000:]
            assert time.time() < deadline, "the server did not come up:\n" + log_path.read_text()[-3000:]
            time.sleep(0.2)
        out = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "handoff_drain.py"), str(steps)], timeout=300,
                             capture_output=True, text=True, cwd=str(root), env=env)
        assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-3000:] + log_path.read_text()[-2000:]
        m = re.search(r"DRAIN_OK (\d+) batches, ([0-9.]+) batches/s", out.stdout)
        assert m and int(m.group(1)) == steps, out.stdout
        assert server.wait(timeout=120) == 0, log_path.read_text()[-3000:]
        print("hand-off, trainer that only takes the batches: %s batches/s" % m.group(2))
        assert float(m.group(2)) > 1000.0
    finally:
        if server.poll() is None:
            server.kill()       # this test's own child, by its handle
            server.wait()
