"""The window logic of the single-pass scan's look-back, in a CPU build: from any mix of
published sums, published inclusive prefixes and unpublished words it must return the exact
exclusive prefix, or ask for another read -- never a partial sum."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from conftest import ROOT


@pytest.fixture(scope="module")
def lookback(tmp_path_factory):
    so = str(tmp_path_factory.mktemp("lookback") / "liblookback.so")
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-o", so,
                           os.path.join(ROOT, "tests", "lookback_host.cpp")])
    lib = C.CDLL(so)
    lib.lookback_prefix.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_int64), C.POINTER(C.c_int)]
    return lib


def walk_back(flags, sums, tile):
    """Plain statement: going back from tile-1, add sums until an inclusive prefix is met."""
    total = 0
    for j in range(tile - 1, -1, -1):
        if flags[j] == 0:
            return None
        if flags[j] == 2:
            return total + int(sums[:j + 1].sum())
        total += int(sums[j])
    return total


@pytest.mark.parametrize("n_tiles", [1, 2, 63, 64, 65, 128, 129, 1000])
def test_lookback_gives_the_exact_prefix_or_waits(lookback, n_tiles):
    rng = np.random.default_rng(n_tiles)
    for trial in range(60):
        sums = rng.integers(0, 5000, n_tiles).astype(np.int64)
        # tile 0 only ever publishes an inclusive prefix; the others any of the three states
        p_unpub = [0.0, 0.02, 0.3][trial % 3]
        flags = rng.choice([0, 1, 2], n_tiles, p=[p_unpub, 0.75 - p_unpub, 0.25])
        if trial % 5 == 0:
            flags[:] = 1           # long chains of plain sums, back to tile 0
        flags[0] = 2 if rng.random() < 0.9 else 0
        inclusive = np.cumsum(sums)
        status = np.where(flags == 2, (2 << 32) | inclusive, np.where(flags == 1, (1 << 32) | sums, 0)).astype(np.uint64)
        for tile in sorted(set([0, 1, n_tiles - 1, n_tiles // 2] + rng.integers(0, n_tiles, 8).tolist())):
            got, windows = C.c_int64(-1), C.c_int(0)
            done = lookback.lookback_prefix(status.ctypes.data, tile, C.byref(got), C.byref(windows))
            want = walk_back(flags, sums, tile)
            if want is None:
                assert done == 0
            else:
                assert done == 1 and got.value == want == int(sums[:tile].sum())
                assert windows.value <= (tile + 63) // 64 + 1


@pytest.mark.parametrize("n", range(1, 9))
def test_blocks_of_a_shared_launch_map_onto_pipes(lookback, n):
    """What the look-back needs of the mapping: every pipe's blocks are numbered 0, 1, 2, ... in
    launch order, block k of every pipe lies in the k-th run of n blocks (so the pipes advance in
    step).  What the hardware wants: with workgroups dealt to 8 XCDs round robin, every pipe's blocks
    visit all 8."""
    lookback.grid_row_of.argtypes = [C.c_uint, C.c_uint, C.POINTER(C.c_int), C.POINTER(C.c_int)]
    row, bx = C.c_int(), C.c_int()
    seen = {p: [] for p in range(n)}
    xcds = {p: set() for p in range(n)}
    for b in range(n * 8 * 50):
        lookback.grid_row_of(b, n, C.byref(row), C.byref(bx))
        assert 0 <= row.value < n and bx.value == b // n
        seen[row.value].append(bx.value)
        xcds[row.value].add(b % 8)
    for p in range(n):
        assert seen[p] == list(range(8 * 50)), "pipe %d of %d" % (p, n)
        assert len(xcds[p]) == 8
