"""Sampler -> trainer hand-off inside one process: the sampling server on a background
thread serves the reference's schedule (training and validation steps per epoch, test steps
at the end) through the shared-memory slab and the two semaphores per buffer set; the
consumer takes every batch through the `ipc_service` functions and checks it against the
CPU oracle (in tests/handoff_consumer.py, run as a subprocess)."""
import os
import subprocess
import sys

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
