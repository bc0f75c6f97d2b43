"""No-GPU checks of the host-side mirror of hodu's Tensor / Layout / metadata layer."""
import ctypes
import os
import subprocess

import pytest

from hodu_amd import ffi, tensor

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_layout_algebra_and_metadata_encoders(tmp_path):
    """The C++ checks hold the reference tests' metadata literals and brute-force view enumeration."""
    exe = tmp_path / "host_layout_tests"
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-O1", f"-I{ROOT}/hodu_amd/host",
                           "-o", str(exe), f"{ROOT}/tests/host/host_layout_tests.cpp"])
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "passed" in out.stdout


def test_host_library_loads_and_exports_the_tensor_interface():
    lib = tensor.load()
    for name in ("tensor_from_bytes", "tensor_free", "tensor_to_bytes", "tensor_layout", "matmul", "dot", "to_dtype",
                 "contiguous", "transpose", "broadcast", "reshape", "squeeze", "unsqueeze", "slice", "view",
                 "set_matmul_mode", "stats", "last_error"):
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
