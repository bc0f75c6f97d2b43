"""The CPU build and the host mirror under AddressSanitizer (opt-in: HODU_EMU_ALL=2, most of an hour).

The guard pages of the CPU build's allocator catch an access that leaves an operand at the end it is tight against;
AddressSanitizer adds the other end, the heap blocks of the host code (metadata, the host mirror's tensors and layouts,
use after free of a storage a view still holds), the globals (the LDS array, the static scratch of the entry point
that allocates nothing) and the kernels' fixed-size register arrays on the lanes' stacks.  The pytest files that drive
the CPU build run under a Python that carries the sanitizer's runtime (tests/emu/python_host.cpp), with the library
built by HODU_EMU_SANITIZE=address; a finding aborts the run with a report."""
import os
import subprocess
import sys

import pytest

import emu_util

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FILES = ["test_emu_random_tensors_cpu.py", "test_emu_host_mirror_cpu.py", "test_emu_mfma_cpu.py", "test_emu_random_layouts_cpu.py"]


@pytest.mark.skipif(emu_util.compiler() is None, reason="no host clang for the CPU build")
@pytest.mark.skipif(os.environ.get("HODU_EMU_ALL", "") != "2", reason="most of an hour; set HODU_EMU_ALL=2")
def test_tensor_level_and_random_layouts_under_the_address_sanitizer():
    python = emu_util.build_race_checked_python("address")
    if python is None:
        pytest.skip("no Python headers or library to link the sanitizer-carrying interpreter")
    # not the stack-use-after-return check: a lane's frames live on a stack of its own that the sanitizer's fake frames
    # do not follow; leaks are the interpreter's own
    env = {**os.environ, "HODU_EMU_SANITIZE": "address", "HODU_EMU_ALL": "0", "PYTHONPATH": os.pathsep.join(p for p in sys.path if p),
           "ASAN_OPTIONS": "detect_stack_use_after_return=0:detect_leaks=0:verify_asan_link_order=0"}
    # (the no-alloc entry point's shapes and the masked softmax's rows, thousands of workgroups each, take too long
    # under this sanitizer; both run in the plain and the race-checked CPU build)
    r = subprocess.run([python, "-m", "pytest", *[os.path.join("tests", f) for f in FILES], "-q", "-x", "-p", "no:cacheprovider",
                        "-k", "not allocates_nothing and not masked_softmax"],
                       capture_output=True, text=True, cwd=ROOT, env=env)
    assert "AddressSanitizer" not in r.stderr and "AddressSanitizer" not in r.stdout, (r.stdout[-3000:] + r.stderr[-3000:])
    assert r.returncode == 0 and " passed" in r.stdout, r.stdout[-3000:] + r.stderr[-3000:]
