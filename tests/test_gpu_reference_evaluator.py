"""The reference's REAL evaluator on this backend. oracle/_ref/array_on_hip is the reference's
unmodified array.h / storage.h / types.h compiled (in the build container, by oracle/Makefile)
on top of cpp-tensorlib_amd/include/tl/hip.h through the gpu.h arm INTEGRATION.md describes.
It evaluates every case twice with the reference's own code - use_cpu() and use_gpu() - and
compares with allclose(rtol 1e-4, atol 1e-5); the dispatch census shows that the GPU run
launched kernels. This is the drop-in claim itself: dot (int4 / bf16 / f32, with and without
the fused affine epilogue), gemm, attn_decode, rope, the rmsnorm / silu / swiglu / softmax
compositions with their lazy-graph fusion, broadcasts, and a decoder block."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "oracle", "_ref", "array_on_hip")
LIB = os.path.join(ROOT, "cpp-tensorlib_amd", "lib", "libtensorlib_hip.so")


def test_reference_array_ops_on_the_hip_backend():
    if not os.path.exists(EXE):
        pytest.skip("oracle/_ref/array_on_hip not built (needs /root/reference at build time: make -C oracle seam)")
    env = dict(os.environ, TENSORLIB_HIP_LIB=LIB)
    print("running", EXE, flush=True)
    r = subprocess.run([EXE], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=100)
    out = r.stdout.decode(errors="replace")
    print(out)
    assert r.returncode == 0, out[-3000:]
    assert "ALL OK" in out and "FAIL" not in out
    assert out.count("PASS") >= 35
