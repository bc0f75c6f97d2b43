"""No-GPU checks of the C-ABI library: it loads, exports every symbol the header declares, and its
host-side entry points fail with a status code (never a crash) when there is no device."""
import ctypes
import os
import re
import subprocess

import pytest

from hodu_amd import ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hodu_rocm_kernels.h")
DEBUG_HEADER = os.path.join(ROOT, "include", "hodu_rocm_debug.h")


def declared_symbols(header=HEADER):
    text = subprocess.check_output(["gcc", "-E", "-P", f"-I{ROOT}/include", header], text=True)
    return sorted(set(re.findall(r"\b(hodu_rocm_\w+)\s*\(", text)))


def exported_symbols(path):
    out = subprocess.check_output(["nm", "-D", "--defined-only", path], text=True)
    return sorted({line.split()[-1] for line in out.splitlines() if " T " in line and "hodu_rocm_" in line
                   and not line.split()[-1].startswith("_Z")})


def test_library_exports_every_declared_symbol():
    lib = ffi.load()
    names = declared_symbols()
    assert len(names) >= 50
    for op in ("matmul", "dot"):
        for dt in ffi.PRODUCT_DTYPES + list(ffi.FUSED_PRODUCTS):
            assert f"hodu_rocm_{op}_{dt}" in names
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    # and nothing else: the kernel library is the drop-in boundary, so every extern "C" hodu_rocm_* symbol it
    # exports is one the header declares (test and measurement hooks live in the hooks library)
    assert not [n for n in names if "debug" in n]
    extra = sorted(set(exported_symbols(ffi.LIB_PATH)) - set(names))
    assert not extra, extra


def test_hooks_library_exports_what_its_header_declares():
    lib = ffi.load_debug()
    names = sorted(set(declared_symbols(DEBUG_HEADER)) - set(declared_symbols()))
    assert names and all(n.startswith("hodu_rocm_debug_") for n in names), names
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    assert sorted(exported_symbols(ffi.DEBUG_LIB_PATH)) == names


def test_header_compiles_as_c_and_cxx(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "hodu_rocm_kernels.h"\nint main(void){return HODU_ROCM_OK;}\n')
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Werror", "-fsyntax-only", f"-I{ROOT}/include", str(src)])
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", f"-I{ROOT}/include", str(src)])


def test_null_arguments_are_rejected_without_a_device():
    lib = ffi.load()
    md = (ctypes.c_size_t * 9)(2, 3, 2, 3, 1, 2, 1, 0, 0)
    assert lib.hodu_rocm_dot_f32(None, None, None, None, md, 9) == ffi.INVALID_ARG
    assert b"context is null" in lib.hodu_rocm_last_error(None)
    assert lib.hodu_rocm_cast(None, 5, 3, None, None, md, 9) == ffi.INVALID_ARG
    assert lib.hodu_rocm_ctx_create(0, None) == ffi.INVALID_ARG
    assert lib.hodu_rocm_ctx_destroy(None) == ffi.OK


@pytest.mark.skipif(ffi.device_count() > 0, reason="a GPU is present")
def test_context_creation_fails_cleanly_without_a_gpu():
    with pytest.raises(ffi.HoduRocmError):
        ffi.Context(0)


def test_host_binding_refuses_metadata_that_reaches_past_a_buffer():
    """The C ABI takes bare pointers like the reference's kernels; the binding that owns the buffers
    checks that a metadata vector stays inside them before anything is launched."""
    class Buf:
        def __init__(self, n):
            self.nbytes, self.ptr = n, 0

    chk = ffi.Context._check_extents
    md = [4, 8, 4, 8, 1, 1, 8, 0, 0]  # dot: [4,8] x [8,4] with the rhs a transposed view of [4,8]
    chk("dot", "bf16", Buf(64), [Buf(64)], Buf(32), md)
    with pytest.raises(ffi.HoduRocmError):
        chk("dot", "bf16", Buf(64), [Buf(62)], Buf(32), md)
    with pytest.raises(ffi.HoduRocmError):
        chk("dot", "bf16", Buf(64), [Buf(64)], Buf(30), md)
    with pytest.raises(ffi.HoduRocmError):
        chk("dot", "bf16_f8e4m3w", Buf(64), [Buf(31)], Buf(32), md)
    # matmul with a stride-0 batch-broadcast rhs only needs one copy of it
    mm = [64, 3, 3, 1, 4, 4, 8, 4, 8, 4, 4, 32, 8, 1, 0, 1, 8, 0, 0, 4, 8, 4]
    assert ffi.product_spans("matmul", mm) == (128, 32, 64)
    with pytest.raises(ffi.HoduRocmError):
        ffi.Context._check_strided("cast", 1, 2, Buf(15), Buf(32), [16, 2, 4, 4, 1, 4, 0])
