"""The tile kernels' map from a workgroup id to (batch, tile row, tile column) (hodu_amd/csrc/tile_walk.hpp) is plain
C++: compiled here for the host and held against the same walk written out in Python integers -- every workgroup of
a spread of grids, including the BASELINE configurations' -- and against what the walk must be whatever its order: a
bijection between the grid and the tiles."""
import ctypes
import os
import subprocess
import tempfile

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SRC = r"""
#include "tile_walk.hpp"
extern "C" void walk_all(unsigned total, unsigned tiles_m, unsigned tiles_n, unsigned *batch, unsigned *tm, unsigned *tn) {
    for (unsigned pid = 0; pid < total; pid++) hodu::tile_walk(pid, total, tiles_m, tiles_n, batch[pid], tm[pid], tn[pid]);
}
"""


@pytest.fixture(scope="module")
def lib():
    with tempfile.TemporaryDirectory() as d:
        src, so = os.path.join(d, "walk.cpp"), os.path.join(d, "walk.so")
        with open(src, "w") as f:
            f.write(SRC)
        subprocess.run(["g++", "-O2", "-shared", "-fPIC", "-I", os.path.join(ROOT, "hodu_amd", "csrc"), src, "-o", so], check=True)
        yield ctypes.CDLL(so)


def reference_walk(pid, total, tiles_m, tiles_n):
    """the walk in unbounded integers: XCD x (ids x, x + 8, ...) owns a contiguous range; groups of 8 tile rows,
    column by column inside a group"""
    if total % 8 == 0:
        pid = (pid % 8) * (total // 8) + pid // 8
    per_batch = tiles_m * tiles_n
    batch, t = divmod(pid, per_batch)
    width = 8 * tiles_n
    first_m = (t // width) * 8
    gsize = min(tiles_m - first_m, 8)
    return batch, first_m + (t % width) % gsize, (t % width) // gsize


GRIDS = [(1, 1, 1), (1, 16, 16), (16, 4, 4), (1, 16, 56), (1, 2, 32), (1, 8, 8), (3, 5, 7), (1, 17, 16), (5, 8, 7), (1, 18, 15),
         (7, 1, 1), (1, 1, 300), (1, 300, 1), (2, 9, 9), (1, 33, 3), (4096, 1, 1), (1, 181, 182)]


@pytest.mark.parametrize("batches,tiles_m,tiles_n", GRIDS)
def test_walk_matches_the_integer_formula_and_is_a_bijection(lib, batches, tiles_m, tiles_n):
    total = batches * tiles_m * tiles_n
    b, m, n = (np.zeros(total, dtype=np.uint32) for _ in range(3))
    ptr = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint))
    lib.walk_all(ctypes.c_uint(total), ctypes.c_uint(tiles_m), ctypes.c_uint(tiles_n), ptr(b), ptr(m), ptr(n))
    want = np.array([reference_walk(p, total, tiles_m, tiles_n) for p in range(total)], dtype=np.int64).reshape(total, 3)
    assert np.array_equal(b, want[:, 0]) and np.array_equal(m, want[:, 1]) and np.array_equal(n, want[:, 2])
    assert b.max() < batches and m.max() < tiles_m and n.max() < tiles_n
    flat = (b.astype(np.int64) * tiles_m + m) * tiles_n + n
    assert np.array_equal(np.sort(flat), np.arange(total))  # every tile exactly once


def test_walk_near_the_largest_grid(lib):
    """ids near 2^31: the arithmetic stays inside 32 unsigned bits"""
    total, tiles_m, tiles_n = 0x7FFFFFF8, 4, 8
    batch, tm, tn = ctypes.c_uint(), ctypes.c_uint(), ctypes.c_uint()
    src = r"""
#include "tile_walk.hpp"
extern "C" void walk_one(unsigned pid, unsigned total, unsigned tiles_m, unsigned tiles_n, unsigned *b, unsigned *m, unsigned *n) {
    hodu::tile_walk(pid, total, tiles_m, tiles_n, *b, *m, *n);
}
"""
    with tempfile.TemporaryDirectory() as d:
        s, so = os.path.join(d, "one.cpp"), os.path.join(d, "one.so")
        with open(s, "w") as f:
            f.write(src)
        subprocess.run(["g++", "-O2", "-shared", "-fPIC", "-I", os.path.join(ROOT, "hodu_amd", "csrc"), s, "-o", so], check=True)
        one = ctypes.CDLL(so)
        for pid in (0, 1, 7, 8, total // 2, total - 9, total - 8, total - 1):
            one.walk_one(ctypes.c_uint(pid), ctypes.c_uint(total), ctypes.c_uint(tiles_m), ctypes.c_uint(tiles_n),
                         ctypes.byref(batch), ctypes.byref(tm), ctypes.byref(tn))
            assert (batch.value, tm.value, tn.value) == reference_walk(pid, total, tiles_m, tiles_n), pid
