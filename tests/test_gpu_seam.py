"""GPU: the tl::hip backend header driven the way the reference's evaluator drives a backend
(byte-offset views, affine epilogues, the rmsnorm composition, the GEMV arms with the scales
inside the weight allocation, attention/rope, the cpu_barrier/sync_to_host protocol, the pool).
The program is tests/seam_check.cpp, compiled by tests/build_programs.py; every case is checked
against host loops inside it."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "bin", "tl_seam_check")
HIP_LIB = os.path.join(ROOT, "cpp-tensorlib_amd", "lib", "libtensorlib_hip.so")


def test_backend_header_seam_check():
    assert os.path.exists(EXE), "build it with `python tests/build_programs.py`"
    env = dict(os.environ, TENSORLIB_HIP_LIB=HIP_LIB)
    r = subprocess.run([EXE], env=env, capture_output=True, text=True, timeout=120)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "0 failed" in r.stdout
