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


QWEN_EXE = os.path.join(ROOT, "oracle", "_ref", "qwen_on_hip")


@pytest.mark.timeout(400)
def test_reference_decode_harness_on_the_hip_backend(tmp_path):
    """bench/cuda/qwen_model.h, unmodified, on tl::hip (oracle/qwen_on_hip.cpp): the reference's own
    GGUF loading, array-path forward, imperative step, batched prefill and graph-captured decoder,
    compared against each other on a synthetic Qwen2.5-0.5B-shaped F16 file (the harness hard-codes
    those dimensions: 24 layers, 896 hidden, 14/2 heads of 64, vocab 151936; a 1.26 GB file)."""
    if not os.path.exists(QWEN_EXE):
        pytest.skip("oracle/_ref/qwen_on_hip not built (needs /root/reference at build time: make -C oracle seam)")
    import numpy as np
    import ggufwriter as W
    NL, E, NH, NKV, HD, FF, V = 24, 896, 14, 2, 64, 4864, 151936
    rng = np.random.default_rng(17)
    block = (rng.standard_normal(1 << 21) * 0.02).astype(np.float16)

    def lin(out, inn, k):
        return np.resize(np.roll(block, 7919 * k), out * inn).reshape(out, inn)

    def vec(n, mean, k):
        return (mean + np.resize(np.roll(block, 104729 * k), n).astype(np.float32)).astype(np.float32)
    kv = [("general.architecture", W.STRING, "qwen2"), ("qwen2.block_count", W.U32, NL),
          ("qwen2.embedding_length", W.U32, E), ("qwen2.feed_forward_length", W.U32, FF),
          ("qwen2.attention.head_count", W.U32, NH), ("qwen2.attention.head_count_kv", W.U32, NKV)]
    f16, f32 = W.GGML["f16"], W.GGML["f32"]
    t = [("token_embd.weight", f16, [E, V], lin(V, E, 1)), ("output.weight", f16, [E, V], lin(V, E, 2)),
         ("output_norm.weight", f32, [E], vec(E, 1.0, 3))]
    for l in range(NL):
        p, k = "blk.%d." % l, 10 * l + 5
        t += [(p + "attn_q.weight", f16, [E, NH * HD], lin(NH * HD, E, k)), (p + "attn_q.bias", f32, [NH * HD], vec(NH * HD, 0.0, k + 1)),
              (p + "attn_k.weight", f16, [E, NKV * HD], lin(NKV * HD, E, k + 2)), (p + "attn_k.bias", f32, [NKV * HD], vec(NKV * HD, 0.0, k + 3)),
              (p + "attn_v.weight", f16, [E, NKV * HD], lin(NKV * HD, E, k + 4)), (p + "attn_v.bias", f32, [NKV * HD], vec(NKV * HD, 0.0, k + 5)),
              (p + "attn_output.weight", f16, [NH * HD, E], lin(E, NH * HD, k + 6)),
              (p + "ffn_gate.weight", f16, [E, FF], lin(FF, E, k + 7)), (p + "ffn_up.weight", f16, [E, FF], lin(FF, E, k + 8)),
              (p + "ffn_down.weight", f16, [FF, E], lin(E, FF, k + 9)),
              (p + "attn_norm.weight", f32, [E], vec(E, 1.0, k + 10)), (p + "ffn_norm.weight", f32, [E], vec(E, 1.0, k + 11))]
    path = str(tmp_path / "qwen05b_synthetic_f16.gguf")
    print("writing", path, flush=True)
    W.write_streaming(path, kv, t)
    print("file written: %.2f GB; running %s" % (os.path.getsize(path) / 1e9, QWEN_EXE), flush=True)
    env = dict(os.environ, TENSORLIB_HIP_LIB=LIB)
    r = subprocess.run([QWEN_EXE, path], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=330)
    out = r.stdout.decode(errors="replace")
    print(out, flush=True)
    os.remove(path)
    assert r.returncode == 0, out[-3000:]
    assert "ALL OK" in out and "FAIL" not in out
