"""CPU checks of the boundary: the C-ABI library loads without a GPU, exports
every symbol include/legion_mi.h declares, and the Python mirror agrees with the
header.  No compute call is made here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "legion_mi.h")


def header_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lmi_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lmi):
    lib = lmi.lib()
    declared = header_symbols()
    assert len(declared) >= 35
    missing = [s for s in declared if not hasattr(lib, s)]
    assert not missing, "declared in legion_mi.h but not exported: %s" % missing
    assert sorted(lmi.ABI_SYMBOLS) == declared, "python mirror out of sync with the header"
    assert lib.lmi_abi_version() == 3


def test_struct_layouts_match_header(lmi):
    # sizes computed by hand from include/legion_mi.h (LP64)
    assert ctypes.sizeof(lmi.Config) == 48
    assert ctypes.sizeof(lmi.BatchView) == 8 * 8 + 3 * 8 + 8 + 24
    assert ctypes.sizeof(lmi.CacheInfo) == 48
    assert ctypes.sizeof(lmi.Profile) == 12 * 8


def test_bad_arguments_are_rejected_without_a_gpu(lmi):
    lib = lmi.lib()
    assert lib.lmi_server_create(None, None) == -1
    assert b"null" in lib.lmi_last_error()
    cfg = lmi.Config()
    cfg.hops, cfg.batch_size, cfg.feat_dim, cfg.pipes = 9, 8, 4, 1
    h = ctypes.c_void_p()
    assert lib.lmi_server_create(ctypes.byref(cfg), ctypes.byref(h)) == -1   # too many hops
    cfg.hops = 1
    cfg.fanout[0] = 65
    assert lib.lmi_server_create(ctypes.byref(cfg), ctypes.byref(h)) == -1   # fanout > LMI_MAX_FANOUT
    assert lib.lmi_server_destroy(None) == 0
    # the measurement kernels check their shapes before they touch a device
    ms = ctypes.c_double()
    assert lib.lmi_bench_stream(1 << 20, 12, 16, 0, 1, 0, ctypes.byref(ms)) == -1          # no 12:16 shape
    assert lib.lmi_bench_stream(1 << 20, 8, 16, 4, 1, 0, ctypes.byref(ms)) == -1           # misaligned only as 16:16
    assert lib.lmi_bench_row_stream_shape(1000, 512, 16, 16, 4096, 5000, 0, 0, 1, 1, ctypes.byref(ms)) == -1   # rows per visit
    assert lib.lmi_bench_row_stream_shape(1000, 510, 16, 16, 4096, 0, 0, 0, 1, 1, ctypes.byref(ms)) == -1      # rows of 4 k bytes
    assert lib.lmi_bench_row_stream_shape(1000, 404, 8, 16, 4096, 0, 0, 0, 1, 1, ctypes.byref(ms)) == -1       # 8:16 wants 16-byte rows
    assert lib.lmi_server_pipes(None, 4) == -1


def test_header_cites_the_reference_for_every_group():
    text = open(HEADER).read()
    for cite in ["engine/server.cu", "engine/operator_impl.cuh", "engine/server_imp.cuh", "cache/cache.cu",
                 "storage/graph_storage.cu", "storage/feature_storage.cu", "engine/memorypool.cuh"]:
        assert cite in text


def test_missing_library_fails_loudly(lmi, monkeypatch):
    monkeypatch.setattr(lmi, "_lib", None)
    monkeypatch.setattr(lmi, "LIB_PATH", "/nonexistent/liblegion_mi.so")
    with pytest.raises(ImportError):
        lmi.lib()


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""
