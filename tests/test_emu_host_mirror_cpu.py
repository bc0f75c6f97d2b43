"""The Tensor-level path in the CPU build: hodu_amd.tensor over the host mirror's compiled library
(hodu_amd/host/capi.cpp, unmodified) linked against the CPU build of the kernels (tests/emu_util.py) instead of the
real kernel library.  Every test function of tests/test_gpu_host_tensor.py -- Tensor::matmul's rank routing, broadcast
batches, deferred casts, the copy / no-copy equivalence, Linear, the VJP products, sum_to_shape, attention, .hdt
ingestion -- runs unchanged, plus scaled_dot_product_attention with an attn_mask (which has not run on a GPU)."""
import inspect

import pytest

import emu_util
from hodu_amd import tensor as T

pytestmark = pytest.mark.skipif(emu_util.compiler() is None, reason="no host clang++ for the CPU build")


@pytest.fixture(scope="module", autouse=True)
def host_mirror_over_the_cpu_build():
    saved_path, saved_lib = T.HOST_LIB_PATH, T._lib
    T.HOST_LIB_PATH, T._lib = emu_util.build_host(), None
    yield
    T.HOST_LIB_PATH, T._lib = saved_path, saved_lib


def _cases():
    import test_gpu_host_tensor as suite
    import test_zx_softmax_masked
    for mod, names in ((suite, None), (test_zx_softmax_masked, {"test_attention_with_a_padding_mask_against_float64",
                                                                  "test_a_mask_of_another_dtype_is_its_nonzero_pattern"})):
        for name, fn in inspect.getmembers(mod, inspect.isfunction):
            if not name.startswith("test_") or fn.__module__ != mod.__name__ or (names is not None and name not in names):
                continue
            marks = [m for m in getattr(fn, "pytestmark", []) if m.name == "parametrize"]
            assert len(marks) <= 1
            if not marks:
                yield pytest.param(fn, {}, id=name)
                continue
            argnames = [a.strip() for a in marks[0].args[0].split(",")]
            for value in marks[0].args[1]:
                values = value if len(argnames) > 1 else (value,)
                yield pytest.param(fn, dict(zip(argnames, values)), id=f"{name}[{'-'.join(str(v) for v in values)}]")


def _collected():
    """(a failure to collect must not take the other test files' collection down with it: it becomes one failing case)"""
    try:
        return list(_cases())
    except Exception as e:  # noqa: BLE001
        message = f"{type(e).__name__}: {e}"

        def collection_failed():
            raise RuntimeError(f"collecting the Tensor-level test functions failed: {message}")
        return [pytest.param(collection_failed, {}, id="collection")]


@pytest.mark.parametrize("fn,kwargs", _collected())
def test_tensor_level_test_passes_in_the_cpu_build(fn, kwargs, tmp_path):
    params = inspect.signature(fn).parameters
    if "tmp_path" in params:
        kwargs = dict(kwargs, tmp_path=tmp_path)
    if "ctx" in params:
        kwargs = dict(kwargs, ctx=None)  # (the masked-attention test takes the fixture and does not use it)
    fn(**kwargs)


def test_reference_sums_through_the_tensor_api():
    """Tensor::matmul of bf16 tensors with the device switched to the reference's arithmetic stores the bytes of
    hodu_cpu_matmul_bf16 (the oracle's reference-faithful product); switched back, the f32-accumulated ones"""
    import numpy as np

    import helpers as H
    import oracle
    a = H.random_storage("bf16", 3 * 20 * 48, 1)
    b = H.random_storage("bf16", 48 * 24, 2)
    ta, tb = T.Tensor.from_bits(a, "bf16", [3, 20, 48]), T.Tensor.from_bits(b, "bf16", [48, 24])
    md = H.matmul_md(H.View([3, 20, 48]), H.View([48, 24]).broadcast_to([3, 48, 24]))
    T.set_reference_sums(True)
    try:
        got = ta.matmul(tb).to_bits()
    finally:
        T.set_reference_sums(False)
    assert np.array_equal(got, oracle.matmul_asis("bf16", a, b, md))
    own = ta.matmul(tb).to_bits()
    assert not np.array_equal(own, got)
