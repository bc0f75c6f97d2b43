"""The softmax kernels' unmodified source, compiled for the host (tests/emu, tests/emu_util.py) and run there through
the real entry points, against the oracle's comparator.  Two jobs: the plain kernels, which the GPU tests hold to the
same comparator on the hardware (tests/test_gpu_softmax.py), show that the CPU build executes this source faithfully --
every launcher of softmax.hip is reached; and hodu_rocm_softmax_masked (attention's attn_mask), on the shapes its GPU
test uses, is held to oracle.softmax_masked_spec.  Tolerances are the GPU tests': f32 1e-5, bf16 / f16 2e-2, f64 1e-12
relative, with the output format's floor; masked entries exact zeros."""
import numpy as np
import pytest

import emu_util
import helpers as H
import oracle

V = H.View
TOL = {"f32": 1e-5, "bf16": 2e-2, "f16": 2e-2, "f64": 1e-12}
FLOOR = {"f32": 1e-30, "bf16": 1e-30, "f16": 2.0 ** -24, "f64": 1e-30}

pytestmark = pytest.mark.skipif(emu_util.compiler() is None, reason="no host clang++ for the CPU build")


@pytest.fixture(scope="module")
def emu():
    e = emu_util.Emu()
    yield e
    e.close()


def check_softmax(emu, dt, v, dim, causal=False, seed=0, expect=None):
    x = H.random_storage(dt, v.span(), 900 + seed, 3.0)
    md = H.reduce_md(v, [dim], True)
    out = np.zeros(v.size, dtype=oracle.STORAGE[dt])
    emu.softmax(dt, x, out, md, causal)
    if expect:
        assert emu.last_kernel() == expect, emu.last_kernel()
    _, want = oracle.softmax_spec(dt, x, md, causal)
    got = H.widen(dt, out)
    assert np.all(np.isfinite(got)) and np.all(got[want == 0.0] == 0.0)
    assert np.all(np.abs(got - want) <= TOL[dt] * np.abs(want) + FLOOR[dt])


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64"])
def test_every_plain_softmax_kernel_runs_faithfully_on_the_cpu_build(emu, dt):
    check_softmax(emu, dt, V([3, 5, 129]), 2, seed=1, expect="softmax_row")
    check_softmax(emu, dt, V([7, 512]), 1, seed=2, expect="softmax_row_vec")
    check_softmax(emu, dt, V([37, 64]), 1, seed=3, expect="softmax_row_vec")          # rows sharing a wavefront
    check_softmax(emu, dt, V([2, 20, 64]), 2, causal=True, seed=4, expect="softmax_row_vec")
    check_softmax(emu, dt, V([2, 9, 33]), 2, causal=True, seed=5, expect="softmax_row")
    check_softmax(emu, dt, V([2, 5000]), 1, seed=6, expect="softmax_long_vec")
    check_softmax(emu, dt, V([2, 4099]), 1, seed=7, expect="softmax_long")
    check_softmax(emu, dt, V([6, 10]).t(), 1, seed=8, expect="softmax_strided")
    check_softmax(emu, dt, V([4, 9, 33]), 1, seed=9, expect="softmax_cols")


def mask_strides(mask_shape, full_shape):
    ms = [1] * (len(full_shape) - len(mask_shape)) + list(mask_shape)
    strides, acc = [0] * len(ms), 1
    for d in range(len(ms) - 1, -1, -1):
        strides[d] = 0 if ms[d] == 1 and full_shape[d] != 1 else acc
        acc *= ms[d]
    return strides


def check_masked(emu, dt, v, mask_shape, causal=False, seed=0, closed_rows=(), mask_dt="u8", mask_offset=0):
    full = v.shape
    g = np.random.default_rng(1234 + seed)
    x = H.random_storage(dt, v.span(), 900 + seed, 3.0)
    mask = (g.random(mask_shape) > 0.4).astype(np.uint8)
    mask[..., 0] = 1
    for r in closed_rows:
        mask.reshape(-1, mask_shape[-1])[r, :] = 0
    strides = mask_strides(mask_shape, full)
    flat = np.concatenate([np.zeros(mask_offset, np.uint8), mask.ravel()])
    md = H.reduce_md(v, [len(full) - 1], True)
    out = np.zeros(v.size, dtype=oracle.STORAGE[dt])
    emu.softmax_masked(dt, x, out, md, flat, strides, mask_offset, causal, mask_dt)
    assert emu.last_kernel() == "softmax_masked"
    _, want = oracle.softmax_masked_spec(dt, x, md, flat, strides, mask_offset, causal)
    got = H.widen(dt, out)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.all(got[~nan][want[~nan] == 0.0] == 0.0)
    assert np.all(np.abs(got[~nan] - want[~nan]) <= TOL[dt] * np.abs(want[~nan]) + FLOOR[dt])
    return int(nan.sum())


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64"])
def test_masked_softmax_with_masks_of_every_broadcast_shape(emu, dt):
    full = [2, 3, 20, 70]
    for n, ms in enumerate(([2, 3, 20, 70], [1, 1, 20, 70], [2, 1, 1, 70], [20, 70], [70])):
        check_masked(emu, dt, V(full), ms, seed=n)
        check_masked(emu, dt, V(full), ms, causal=True, seed=10 + n)
    check_masked(emu, dt, V([5, 1]), [5, 1], seed=20)            # rows of one entry
    check_masked(emu, dt, V([3, 4100]), [3, 4100], seed=21)      # many passes of a wavefront over a row
    check_masked(emu, dt, V([70, 50]).t(), [50, 70], seed=22)    # scores as a transposed view
    check_masked(emu, dt, V([6, 40]), [6, 40], seed=23, mask_offset=5)


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64"])
def test_masked_softmax_rows_masked_entirely(emu, dt):
    """uniform in the 16-bit types (the reference's fill is finite there), NaN in f32 / f64"""
    nans = check_masked(emu, dt, V([4, 6, 33]), [4, 6, 33], seed=30, closed_rows=(0, 7, 23))
    assert nans == (0 if dt in ("bf16", "f16") else 3 * 33)
    nans = check_masked(emu, dt, V([4, 6, 33]), [4, 1, 33], seed=31, closed_rows=(2,))
    assert nans == (0 if dt in ("bf16", "f16") else 6 * 33)


def test_masked_softmax_argument_checks(emu):
    x = np.zeros(12, np.float32)
    out = np.zeros(12, np.float32)
    mask = np.ones(12, np.uint8)
    md = H.reduce_md(V([3, 4]), [1], True)
    check = lambda **kw: emu.softmax_masked("f32", x, out, kw.get("md", md), mask, kw.get("strides", [4, 1]), 0, False, kw.get("mask_dt", "u8"))  # noqa: E731
    check()
    with pytest.raises(RuntimeError, match="one byte per element"):
        check(mask_dt="f32")
    with pytest.raises(RuntimeError, match="mask layout"):
        check(strides=[1])
    with pytest.raises(RuntimeError, match="last dim"):
        check(md=H.reduce_md(V([3, 4]), [0], True))
