"""No-GPU checks of the host-side mirror of hodu's Tensor / Layout / metadata layer."""
import ctypes
import os
import subprocess

import pytest

from hodu_amd import ffi, tensor

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("sanitized", [False, True])
def test_layout_algebra_and_metadata_encoders(tmp_path, sanitized):
    """The C++ checks hold the reference tests' metadata literals and brute-force view enumeration; once more with the
    address and undefined-behaviour sanitizers on the host code."""
    exe = tmp_path / "host_layout_tests"
    extra = ["-fsanitize=address,undefined", "-fno-sanitize-recover=all"] if sanitized else []
    built = subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-O1", *extra, f"-I{ROOT}/hodu_amd/host",
                            "-o", str(exe), f"{ROOT}/tests/host/host_layout_tests.cpp"], capture_output=True, text=True)
    if sanitized and built.returncode != 0 and ("sanitize" in built.stderr or "asan" in built.stderr):
        pytest.skip("this g++ has no sanitizer runtimes")
    assert built.returncode == 0, built.stderr[-3000:]
    out = subprocess.run([str(exe)], capture_output=True, text=True, env={**os.environ, "ASAN_OPTIONS": "verify_asan_link_order=0"})
    assert out.returncode == 0, out.stdout + out.stderr
    assert "passed" in out.stdout


def test_host_library_loads_and_exports_the_tensor_interface():
    lib = tensor.load()
    for name in ("tensor_from_bytes", "tensor_free", "tensor_to_bytes", "tensor_layout", "matmul", "dot", "to_dtype",
                 "contiguous", "transpose", "broadcast", "reshape", "squeeze", "unsqueeze", "slice", "view",
                 "set_matmul_mode", "stats", "last_error", "matmul_then", "linear", "sum", "sum_to_shape", "matmul_vjp",
                 "dot_vjp", "softmax", "attention", "scalar_bits"):
        assert hasattr(lib, f"hodu_host_{name}"), name


@pytest.mark.skipif(ffi.device_count() > 0, reason="a GPU is present")
def test_tensor_creation_without_a_gpu_is_a_clean_error():
    import numpy as np
    with pytest.raises(tensor.HoduError) as e:
        tensor.Tensor.from_bits(np.zeros(4, np.uint32), "f32", [2, 2])
    assert e.value.kind == "RocmKernelError"


def test_from_bits_checks_the_element_width():
    import numpy as np
    with pytest.raises(ValueError):
        tensor.Tensor.from_bits(np.zeros(4, np.uint8), "f32", [2, 2])


def test_scalar_bits_round_to_nearest_even():
    """the scalar a mul_scalar step carries: f64 -> tensor dtype as Scalar::to_dtype does (crates/hodu_core/src/
    scalar.rs:391-404); f16 / bf16 against numpy's and the test helpers' independent RNE conversions, ties, subnormals
    and overflow included"""
    import numpy as np
    import helpers as H
    from hodu_amd import tensor as T
    g = np.random.default_rng(3)
    vals = np.concatenate([g.standard_normal(300) * np.exp2(g.uniform(-30, 17, 300)),
                           [0.0, -0.0, 1.0, 65504.0, 65519.9, 65520.0, 1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                            2.0 ** -14, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 1.0 / np.sqrt(128.0), np.inf, -np.inf]])
    for v in vals:
        f = np.float32(v)
        with np.errstate(over="ignore"):
            want16 = np.array([f], np.float32).astype(np.float16).view(np.uint16)[0]
        assert T.scalar_bits("f16", float(v))[0] == want16, (v, hex(want16))
        assert T.scalar_bits("bf16", float(v))[0] == H.f32_to_bf16_rne(np.array([f]))[0], v
        assert T.scalar_bits("f32", float(v)).view(np.float32)[0] == f or np.isnan(f)
        assert T.scalar_bits("f64", float(v)).view(np.float64)[0] == v
