"""Sampler -> trainer hand-off: the sampling server serves the reference's schedule (training
and validation steps per epoch, test steps at the end) through the shared-memory slab and the
two semaphores per buffer set; the consumer takes every batch through the `ipc_service`
functions and checks it against the CPU oracle (in tests/handoff_consumer.py, run as a
subprocess).  Once with the server on a background thread of the consumer's process, once
as the reference deploys it: the `sampling_server` binary in one process, the trainer in
another, the buffers opened through inter-process memory handles."""
import os
import subprocess
import sys
import time

import numpy as np
import pytest

from conftest import ROOT
from test_gpu_server_binary import write_dataset

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dyn_cache,flavour", [(0, "numpy"), (1, "numpy"), (0, "torch")])
def test_every_scheduled_batch_reaches_the_trainer(tmp_path, dyn_cache, flavour):
    rng = np.random.default_rng(3 + dyn_cache)
    n_nodes, dim, batch, n_train, epochs = 4000, 32, 64, 300, 2
    data = tmp_path / "data"
    data.mkdir()
    indptr, indices, feats, train = write_dataset(str(data), rng, n_nodes, dim, n_train)
    meta = tmp_path / "meta_config"
    meta.write_text("%s/ %d %d %d %d %d %d %d %d %d" % (data, batch, n_nodes, len(indices), dim, n_train, 50, 40,
                                                       600 * dim * 4, epochs))
    env = dict(os.environ, LEGION_MI_META_CONFIG=str(meta))
    out = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "handoff_consumer.py"), str(data), str(batch),
                          str(dim), str(epochs), str(dyn_cache), flavour], env=env, timeout=600, capture_output=True,
                         text=True, cwd=str(tmp_path))
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-3000:]
    # (300-1)/64 = 4 training steps + 1 validation step per epoch, 1 test step
    assert "HANDOFF_OK %d batches" % ((4 + 1) * epochs + 1) in out.stdout
    assert not os.path.exists("/dev/shm/simpleIPCshm") and not os.path.exists("/dev/shm/sem.sem_r_0_0")


def leftovers():
    return [n for n in ("simpleIPCshm", "sem.sem_r_0_0", "sem.sem_w_0_0", "sem.sem_r_0_1", "sem.sem_w_0_1")
            if os.path.exists("/dev/shm/" + n)]


@pytest.mark.parametrize("dyn_cache,part_bytes,flavour,dtype", [
    (0, None, "numpy", "f32"), (1, None, "numpy", "f32"), (0, 65536, "numpy", "f32"), (0, None, "torch", "f32"),
    (0, 65536, "torch", "f32"), (0, 40000, "numpy", "f16"), (8, None, "torch", "f16")])
def test_trainer_in_a_process_of_its_own(tmp_path, dyn_cache, part_bytes, flavour, dtype):
    """part_bytes: the largest allocation the server shares whole.  The real limit (2 GiB) only
    matters for feature buffers of the largest configurations; a small one makes this test's
    feature buffer (2560 rows of 128 bytes) go over in five pieces, re-assembled by the trainer."""
    binary = os.path.join(ROOT, "legion-ibp_amd", "sampling_server")
    assert os.path.exists(binary), "build the host shim first (make -C legion-ibp_amd)"
    assert not leftovers(), "a previous run left %s in /dev/shm" % leftovers()
    rng = np.random.default_rng(31 + dyn_cache)
    n_nodes, dim, batch, n_train, epochs = 4000, 32, 64, 300, 2
    data = tmp_path / "data"
    data.mkdir()
    indptr, indices, feats, train = write_dataset(str(data), rng, n_nodes, dim, n_train,
                                                  np.float16 if dtype == "f16" else np.float32)
    (tmp_path / "meta_config").write_text("%s/ %d %d %d %d %d %d %d %d %d" % (
        data, batch, n_nodes, len(indices), dim, n_train, 50, 40, 600 * dim * 4, epochs))
    env = dict(os.environ, LEGION_MI_HANDOFF="1", LEGION_MI_WAIT_SECONDS="90", LEGION_MI_FEAT_DTYPE=dtype)
    if part_bytes:
        env["LEGION_MI_IPC_PART_BYTES"] = str(part_bytes)
    log_path = tmp_path / "server.log"
    with open(log_path, "w") as log:
        server = subprocess.Popen([binary, "1", "0", str(dyn_cache), "7,4"], cwd=str(tmp_path), env=env, stdout=log,
                                  stderr=subprocess.STDOUT)
    try:
        deadline = time.time() + 150
        while "System is ready for serving" not in log_path.read_text():
            assert server.poll() is None, "the server ended early:\n" + log_path.read_text()[-3000:]
            assert time.time() < deadline, "the server did not come up:\n" + log_path.read_text()[-3000:]
            time.sleep(0.2)
        # the trainer: a fresh process whose first GPU work is opening the server's buffers
        out = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "handoff_consumer.py"), str(data), str(batch),
                              str(dim), str(epochs), str(dyn_cache), flavour, "attach"], timeout=300,
                             capture_output=True, text=True, cwd=str(tmp_path), env=env)
        assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-3000:] + log_path.read_text()[-2000:]
        assert "HANDOFF_OK %d batches" % ((4 + 1) * epochs + 1) in out.stdout
        assert server.wait(timeout=120) == 0, log_path.read_text()[-3000:]
        assert "batches: %d" % ((4 + 1) * epochs + 1) in log_path.read_text()
    finally:
        if server.poll() is None:
            server.kill()       # this test's own child, by its handle
            server.wait()
    assert not leftovers(), "left in /dev/shm: %s" % leftovers()
