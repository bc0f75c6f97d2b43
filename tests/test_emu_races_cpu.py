"""Data races between the wavefronts of a workgroup, looked for with ThreadSanitizer in the CPU build of the kernels.

In the CPU build a wavefront is a host thread and LDS is ordinary memory, so two wavefronts race on LDS exactly where
the kernel's source lacks a barrier between one's write and the other's access, or waits too late for an LDS-DMA whose
bytes another wavefront reads.  ThreadSanitizer records every access of the (unmodified) kernel source per thread and
reports such a pair from ONE run, whether or not the schedule of that run made it visible in the result -- which is
what the result-comparing tests cannot do: they only see the interleavings the host's scheduler happens to produce.
(The lanes of one wavefront are contexts on one thread: they cannot race, as they cannot on the GPU.)

 * tests/emu/race_driver.cpp, a native program: products through the C ABI, the testing hook pinning each tile kernel
   (general, pipelined 32x32x16, 16x16x32 and its respaced form; bf16 and f8e4m3 weights; both right-operand layouts;
   K cut across workgroups; the few-rows kernel) and the one-kernel attention with and without a mask, under the
   earliest and the latest model of LDS-DMA arrival;
 * the same program's hand-offs with the barrier left out, or the wait placed behind the barrier, must be reported:
   the detector has teeth;
 * opt-in (HODU_EMU_ALL=1): every pytest file that drives the CPU build, run by a Python that carries the sanitizer
   (tests/emu/python_host.cpp), i.e. every kernel family the GPU tests cover, at the case set those files run by
   default (ten minutes); HODU_EMU_ALL=2: at their own HODU_EMU_ALL=1 set (more than an hour).
"""
import glob
import os
import subprocess
import sys

import pytest

import emu_util

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.skipif(emu_util.compiler() is None, reason="no host clang for the CPU build")
# the suppressions name the uninstrumented libraries (numpy, its BLAS, the oracle's OpenMP loops) whose interceptor
# calls are none of the sanitizer's business; nothing of the CPU build is suppressed
OPTIONS = "halt_on_error=0 exitcode=66 suppressions=" + os.path.join(ROOT, "tests", "emu", "tsan_suppressions.txt")


@pytest.fixture(scope="module")
def driver():
    exe = emu_util.build_race_driver()
    assert exe is not None
    return exe


def run(cmd, **env):
    return subprocess.run(cmd, capture_output=True, text=True, cwd=ROOT, env={**os.environ, "TSAN_OPTIONS": OPTIONS, **env})


def test_tile_kernels_have_no_race_between_wavefronts(driver):
    r = run([driver])
    assert "ThreadSanitizer" not in r.stderr, r.stderr[:3000]
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    lines = [ln for ln in r.stdout.split("\n") if ln.endswith(" ok")]
    assert len(lines) == 40 and not any("WRONG" in ln for ln in r.stdout.split("\n"))
    for kernel in ("mfma_bf16_256x256_KK", "mfma_bf16_pipe256x256_KK_splitk3", "mfma_bf16_pipe256x256mi16_KM", "mfma_bf16_pipe256x256mi16_KK_r",
                   "mfma_bf16_f8w_pipe256x256mi16_KM_r", "skinny_bf16_f8w", "attention_fwd_bf16", "attention_masked_fwd_bf16_d64"):
        assert sum(kernel in ln.split() for ln in lines) == 2, kernel  # once per arrival model


@pytest.mark.parametrize("fault", ["missing-barrier", "late-wait"])
def test_a_hand_off_without_its_barrier_or_wait_is_reported(driver, fault):
    assert run([driver, "handoff"]).returncode == 0
    r = run([driver, fault])
    assert r.returncode == 66 and "ThreadSanitizer: data race" in r.stderr and "g_lds" in r.stderr, r.stderr[:2000]


SUITES = ["test_emu_mfma_cpu.py", "test_emu_kernel_families_cpu.py", "test_emu_plain_kernels_cpu.py", "test_emu_softmax_cpu.py",
          "test_emu_reference_sums_cpu.py", "test_emu_gpu_suites_cpu.py", "test_emu_host_mirror_cpu.py", "test_emu_random_layouts_cpu.py", "test_emu_random_tensors_cpu.py"]


@pytest.mark.skipif(os.environ.get("HODU_EMU_ALL", "") in ("", "0"), reason="ten minutes; set HODU_EMU_ALL=1")
def test_every_kernel_family_under_the_race_detector(tmp_path):
    python = emu_util.build_race_checked_python()
    if python is None:
        pytest.skip("no Python headers or library to link the sanitizer-carrying interpreter")
    log = str(tmp_path / "report")
    env = dict(TSAN_OPTIONS=OPTIONS + f" exitcode=0 log_path={log}", HODU_EMU_SANITIZE="thread", PYTHONPATH=os.pathsep.join(p for p in sys.path if p),
               HODU_EMU_ALL="1" if os.environ.get("HODU_EMU_ALL") == "2" else "0")
    pytest_args = ["-q", "-x", "-p", "no:cacheprovider"]
    # the test that runs kernels under a deliberately wrong arrival model must be reported: the detector sees the kernels
    r = run([python, "-m", "pytest", os.path.join("tests", "test_emu_mfma_cpu.py"), *pytest_args, "-k", "one_load_too_late"], **env)
    reports = "".join(open(p).read() for p in glob.glob(log + ".*"))
    assert " passed" in r.stdout and "data race" in reports and "dma16_now" in reports, r.stdout[-2000:] + reports[:2000]
    for p in glob.glob(log + ".*"):
        os.remove(p)
    # everything else must be clean
    r = run([python, "-m", "pytest", *[os.path.join("tests", s) for s in SUITES], *pytest_args, "-k", "not one_load_too_late"], **env)
    reports = "".join(open(p).read() for p in glob.glob(log + ".*"))
    assert "ThreadSanitizer" not in reports, reports[:4000]
    assert " passed" in r.stdout and " failed" not in r.stdout, r.stdout[-3000:]
