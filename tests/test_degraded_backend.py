"""The drop-in without a usable GPU backend, on the CPU only. The reference's CI builds with a
GPU backend and runs its test program on a runner that has no driver
(/root/reference/.github/workflows/ci.yml:29-61): every op must decline and the evaluator's CPU
path must carry the whole suite. oracle/_ref/refprogs/tensorlib_test is the reference's own
test/test_array.cpp + test_qwen.cpp, compiled unmodified on cpp-tensorlib_amd/include/tl/hip.h
(oracle/Makefile refprogs). It is run in --gpu and --auto mode
  - with TENSORLIB_HIP_LIB naming a file that does not exist (dlopen fails), and
  - with the real library on a machine without a device (tlhip_init fails),
and must pass every assertion both ways. The seam check program, which insists on a device,
must say so and exit non-zero rather than compute anything."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "oracle", "_ref", "refprogs", "tensorlib_test")
LIB = os.path.join(ROOT, "cpp-tensorlib_amd", "lib", "libtensorlib_hip.so")
HAVE_GPU = os.path.exists("/dev/kfd")


def _run(mode, lib):
    r = subprocess.run([EXE, mode], env=dict(os.environ, TENSORLIB_HIP_LIB=lib), stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, timeout=280)
    out = r.stdout.decode(errors="replace")
    assert r.returncode == 0, out[-3000:]
    m = re.search(r"assertions:\s+(\d+)\s+\|\s+(\d+) passed\s+\|\s+(\d+) failed", out)
    assert m, out[-1000:]
    total, passed, failed = map(int, m.groups())
    assert failed == 0 and passed == total and total >= 275, out[-1000:]


@pytest.mark.parametrize("mode", ["--gpu", "--auto", "--cpu"])
def test_reference_suite_passes_when_the_library_cannot_be_loaded(mode):
    if not os.path.exists(EXE):
        pytest.skip("oracle/_ref/refprogs not built (needs /root/reference at build time: make -C oracle refprogs)")
    _run(mode, "/nonexistent/libtensorlib_hip.so")


@pytest.mark.parametrize("mode", ["--gpu", "--auto"])
def test_reference_suite_passes_when_there_is_no_device(mode):
    if not os.path.exists(EXE):
        pytest.skip("oracle/_ref/refprogs not built (needs /root/reference at build time: make -C oracle refprogs)")
    if HAVE_GPU:
        pytest.skip("a GPU is present; the no-device path is what this checks")
    _run(mode, LIB)


def test_seam_check_program_refuses_to_run_without_a_backend():
    exe = os.path.join(ROOT, "tests", "bin", "tl_seam_check")
    if not os.path.exists(exe):
        pytest.skip("tests/bin/tl_seam_check not built (python tests/build_programs.py)")
    r = subprocess.run([exe], env=dict(os.environ, TENSORLIB_HIP_LIB="/nonexistent/libtensorlib_hip.so"),
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=60)
    out = r.stdout.decode(errors="replace")
    assert r.returncode != 0, out
    assert "unavailable" in out.lower() or "not found" in out.lower() or "cannot open" in out.lower(), out
