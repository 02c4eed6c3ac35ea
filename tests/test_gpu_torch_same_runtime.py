"""A trainer process uses PyTorch and this library together: both must end up on ONE HIP runtime
(PyTorch's wheel brings its own copy; the second runtime to open the GPU in a process finds no
device).  Either load order works: torch first (the library binds to torch's copy), or the
library first through its Python bindings (RTLD_GLOBAL, torch resolves to the copy already
running).  Each order in a process of its own; a torch tensor laid over a buffer of the library
must read and write the same memory."""
import os
import subprocess
import sys

import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu

SCRIPT = r"""
import ctypes as C, os, sys
import numpy as np
sys.path.insert(0, os.path.join(%(root)r, "tests"))
from conftest import load_package, load_ipc_service
order = sys.argv[1]
if order == "torch_first":
    import torch
    assert torch.ones(4, device="cuda").sum().item() == 4.0
lmi = load_package()
p = C.c_void_p()
lmi.check(lmi.lib().lmi_device_alloc(64, C.byref(p)))
src = np.arange(16, dtype=np.int32)
lmi.check(lmi.lib().lmi_copy_to_device(p, src.ctypes.data, 64))
import torch
ipc = load_ipc_service()
t = torch.as_tensor(ipc._DeviceArray(p.value, (16,), "<i4"), device="cuda")
assert t.cpu().numpy().tolist() == src.tolist()          # torch reads what the library wrote
t.mul_(3)
torch.cuda.synchronize()
assert lmi.to_host(p, 16, np.int32).tolist() == (src * 3).tolist()   # and the library what torch wrote
lmi.check(lmi.lib().lmi_device_free(p))
print("SAME_RUNTIME_OK", order, flush=True)
"""


@pytest.mark.parametrize("order", ["torch_first", "library_first"])
def test_torch_and_the_library_share_one_runtime(order):
    out = subprocess.run([sys.executable, "-c", SCRIPT % {"root": ROOT}, order], capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-3000:]
    assert "SAME_RUNTIME_OK " + order in out.stdout
