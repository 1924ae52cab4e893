"""CPU: pins of the oracle that do not need the reference at all — the known
answers the reference's own tests hold, closed forms, and fp64 brute force — plus
agreement with the compiled reference where oracle/_ref was built."""
import numpy as np
import pytest

from oraclelib import allclose


# ---- bf16 (test_array.cpp:705-719; types.h:35-46) ---------------------------------
def test_bf16_known_answers(orc):
    exact = np.array([0.0, 1.0, -2.0, 0.5, 256.0, -0.15625], np.float32)
    assert np.array_equal(orc.bf16_widen(orc.to_bf16(exact)), exact)          # representable values survive
    v = np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -7], np.float32)
    # ties to even: 1+2^-8 -> 1.0 ; 1+3*2^-8 -> 1+2^-6 ; 1+2^-7 is representable
    assert np.array_equal(orc.bf16_widen(orc.to_bf16(v)), np.array([1.0, 1.0 + 2.0 ** -6, 1.0 + 2.0 ** -7], np.float32))


def test_bf16_exhaustive_roundtrip(orc):
    h = np.arange(1 << 16, dtype=np.uint16)
    f = orc.bf16_widen(h)
    keep = ~np.isnan(f)
    assert np.array_equal(orc.to_bf16(f)[keep], h[keep])                      # narrow(widen(h)) == h


# ---- q4 (array.h:703-742; test_array.cpp:809-856) --------------------------------------
def test_f16_widen_exhaustive(orc):
    """orc_f16_to_f32 (the model loader's widening, qwen_model.h:41-60) on all 2^16 patterns
    against an independent IEEE half implementation (numpy's float16): equal bits for every
    number incl. subnormals, zeros and infinities; a NaN keeps sign and mantissa bits (payload
    shifted up by 13, no quieting)."""
    h = np.arange(65536, dtype=np.uint16)
    got = orc.f16_widen(h).view(np.uint32)
    want = h.view(np.float16).astype(np.float32).view(np.uint32)
    nan = ((h >> 10) & 31 == 31) & (h & 0x3ff != 0)
    assert np.array_equal(got[~nan], want[~nan])
    hn = h[nan].astype(np.uint32)
    assert np.array_equal(got[nan], ((hn & 0x8000) << 16) | 0x7f800000 | ((hn & 0x3ff) << 13))
    # known answers: 1.0, -2.0, the largest half, the smallest subnormal, the smallest normal
    ka = orc.f16_widen(np.array([0x3c00, 0xc000, 0x7bff, 0x0001, 0x0400], np.uint16))
    assert list(ka) == [1.0, -2.0, 65504.0, 2.0 ** -24, 2.0 ** -14]


def test_q4_bytes_and_layout(orc):
    assert orc.q4_bytes(48, 256) == 48 * 128 + 48 * 8 * 4 == 7680
    K, N = 64, 3
    w = np.zeros((K, N), np.float32)
    w[0, 1] = 7.0          # group 0 of row n=1: maxabs 7 -> scale 1 -> q=7 at k=0 (low nibble of byte 0)
    w[33, 2] = -3.5        # group 1 of row n=2: scale .5 -> q=-7 at k=33 (high nibble of byte 16)
    buf = orc.to_q4(w)
    packed = buf[:N * K // 2].reshape(N, K // 2)
    scales = buf[N * K // 2:].view(np.float32).reshape(N, K // 32)
    assert packed[1, 0] == (8 << 4 | 15) and packed[2, 16] == (1 << 4 | 8)
    assert scales[1, 0] == np.float32(1.0) and scales[2, 1] == np.float32(0.5)
    assert scales[0, 0] == np.float32(1e-8) / np.float32(7.0)               # all-zero group: floor, q = 0
    assert np.all(packed[0] == 0x88)


def test_q4_quantiser_rounding(orc):
    """lround = half away from zero, clamp to [-8, 7], scale = maxabs/7."""
    K, N = 32, 1
    w = np.zeros((K, N), np.float32)
    w[0, 0] = 7.0                    # scale = 1
    w[1, 0], w[2, 0], w[3, 0], w[4, 0] = 0.5, -0.5, 1.5, -2.5   # ties -> 1, -1, 2, -3
    w[5, 0] = -7.0                   # -7 (the -8 code is only reached by clamping)
    q = (orc.q4_to_f32(orc.to_q4(w), K, N)[:, 0]).astype(int)
    assert list(q[:6]) == [7, 1, -1, 2, -3, -7]


def test_q4_dequant_error_bound(orc):
    K, N = 256, 48                    # test_array.cpp:839-844
    st = 5
    vals = []
    for _ in range(K + K * N):
        st = (st * 1664525 + 1013904223) & 0xFFFFFFFF
        vals.append(np.float32(np.int32(st >> 9)) / np.float32(1 << 22) - np.float32(1.0))
    a = np.array(vals[:K], np.float32)
    w = np.array(vals[K:], np.float32).reshape(K, N)
    buf = orc.to_q4(w)
    deq = orc.q4_to_f32(buf, K, N)
    assert np.max(np.abs(deq - w)) < 0.2
    got = orc.gemv_q4(a, buf, N, K)
    want = a.astype(np.float64) @ deq.astype(np.float64)
    assert allclose(got, want, 1e-3, 1e-5)                                   # epsilon(1e-3), :836


def test_gemv_q4_fp64_bruteforce_odd_shapes(orc):
    rng = np.random.default_rng(0)
    for (N, K) in [(1, 32), (5, 896), (7, 96), (3, 1056)]:
        buf = orc.fill_q4(N, K, N + K)
        x = orc.normal(K, 9)
        pk = buf[:N * K // 2].reshape(N, K // 2)
        sc = buf[N * K // 2:].view(np.float32).reshape(N, K // 32).astype(np.float64)
        nib = np.empty((N, K), np.int64)
        nib[:, 0::2], nib[:, 1::2] = pk & 0xF, pk >> 4
        want = ((nib - 8) * np.repeat(sc, 32, axis=1)) @ x.astype(np.float64)
        assert allclose(orc.gemv_q4(x, buf, N, K), want, 1e-5, 1e-6)
    del rng


def test_dot_epilogue_and_tiny_path(orc):
    A = np.array([[1, 2, 3]], np.float32)
    B = np.array([[1, 0], [0, 1], [1, 1]], np.float32)
    assert np.array_equal(orc.dot(A, B, 2.0, 1.0), np.array([[9.0, 11.0]], np.float32))   # (A.B)*2+1
    assert np.array_equal(orc.ref_dot(A, B), np.array([[4.0, 5.0]], np.float32))


def test_sgemm_slab_order_is_visible(orc):
    """K > 512 is summed in 512-wide slabs (cpu.h:89-91): a case where slab order and a
    single left-to-right fp32 chain differ, against an explicit numpy restatement."""
    K, N = 1500, 4
    A = orc.normal(K, 1).reshape(1, K)
    B = orc.normal(K * N, 2).reshape(K, N)
    want = np.zeros(N, np.float32)
    for s in range(0, K, 512):
        acc = np.zeros(N, np.float64)
        # an fp32 FMA chain == exact product added then rounded once per step
        accf = np.zeros(N, np.float32)
        for p in range(s, min(K, s + 512)):
            accf = (accf.astype(np.float64) + np.float64(A[0, p]) * B[p].astype(np.float64)).astype(np.float32)
        want = want + accf
        del acc
    assert np.array_equal(orc.sgemm(A, B)[0], want)


# ---- attention (test_array.cpp:763-807, 273-274) -----------------------------------------
def test_attn_closed_forms(orc):
    H, D, ctx = 2, 128, 5
    q = orc.normal(H * D, 1).reshape(H, D)
    K = orc.normal(H * ctx * D, 2).reshape(H, ctx, D)
    V = orc.normal(H * ctx * D, 3).reshape(H, ctx, D)
    out = orc.attn_decode(q, K, V, 0.3)
    s = np.einsum("hd,hjd->hj", q.astype(np.float64), K.astype(np.float64)) * 0.3
    p = np.exp(s - s.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    assert allclose(out, np.einsum("hj,hjd->hd", p, V.astype(np.float64)), 1e-5, 1e-6)
    assert np.array_equal(orc.attn_decode(q, np.ascontiguousarray(K[:, :1]), np.ascontiguousarray(V[:, :1]), 0.3), V[:, 0])        # ctx == 1
    assert allclose(orc.attn_decode(q, K, V, 0.0), V.mean(axis=1), 1e-6, 1e-6)         # scale 0 => mean
    # GQA head map: query head h reads kv head h // group
    q4 = orc.normal(4 * D, 4).reshape(4, D)
    g = orc.attn_decode(q4, K, V, 0.2)
    for h in range(4):
        assert np.array_equal(g[h], orc.attn_decode(np.ascontiguousarray(q4[h:h + 1]), np.ascontiguousarray(K[h // 2:h // 2 + 1]), np.ascontiguousarray(V[h // 2:h // 2 + 1]), 0.2)[0])
    # cache prefix: rows past ctx are ignored
    Kp = np.concatenate([K, np.full((H, 3, D), 1e30, np.float32)], axis=1)
    Vp = np.concatenate([V, np.full((H, 3, D), np.nan, np.float32)], axis=1)
    assert np.array_equal(orc.attn_decode(q, Kp, Vp, 0.3, ctx=ctx), out)


def test_softmax_stability(orc):
    x = np.array([[1000.0, 1001.0]], np.float32)
    e = np.exp(-1.0)
    assert allclose(orc.softmax(x), [[e / (1 + e), 1 / (1 + e)]], 1e-6, 1e-7)


# ---- rope / rmsnorm / swiglu (check_llm_block.cpp:62-92, 134-144) ---------------------------
def test_rope_properties(orc):
    x = orc.normal(6 * 64, 1).reshape(6, 64)
    assert np.array_equal(orc.rope(x, 0, 1e4), x)                                       # pos 0
    y = orc.rope(x, 3, 1e4)
    c, s = np.float32(np.cos(3.0)), np.float32(np.sin(3.0))                             # j = 0 rotates by pos rad
    assert np.array_equal(y[:, 0], x[:, 0] * c - x[:, 32] * s)
    assert allclose(y[:, :32] ** 2 + y[:, 32:] ** 2, x[:, :32] ** 2 + x[:, 32:] ** 2, 1e-5, 1e-6)
    j = np.arange(32)
    ang = 777.0 * np.power(1e6, -2.0 * j / 64.0)
    want0 = x[:, :32].astype(np.float64) * np.cos(ang) - x[:, 32:].astype(np.float64) * np.sin(ang)
    assert allclose(orc.rope(x, 777, 1e6)[:, :32], want0, 1e-5, 1e-6)                   # fp64 reference
    b = orc.normal(6 * 64, 2).reshape(6, 64)
    assert np.array_equal(orc.rope(x, 5, 1e4, bias=b), orc.rope(x + b, 5, 1e4))


def test_rmsnorm_swiglu_closed_forms(orc):
    n = 896
    w = orc.normal(n, 3, 1.0, 0.02)
    xc = np.full((1, n), 3.0, np.float32)
    assert allclose(orc.rmsnorm(xc, w, 1e-6)[0], 3.0 / np.sqrt(9.0 + 1e-6) * w.astype(np.float64), 1e-6, 1e-7)
    x = orc.normal(n, 4).reshape(1, n)
    ms = np.mean(x.astype(np.float64) ** 2)
    assert allclose(orc.rmsnorm(x, w, 1e-5)[0], x[0] / np.sqrt(ms + 1e-5) * w, 1e-5, 1e-6)
    assert abs(orc.silu(np.array([1.0], np.float32))[0] - 0.7310586) < 1e-6
    assert np.all(orc.swiglu(np.zeros(8, np.float32), np.full(8, 5.0, np.float32)) == 0.0)
    g, u = orc.normal(100, 5), orc.normal(100, 6)
    assert np.array_equal(orc.swiglu_fused(np.concatenate([g, u]).reshape(1, 200), 100)[0], orc.swiglu(g, u))


def test_argmax_ties(orc):
    v = np.array([1, 5, 5, 2, 5], np.float32)
    assert orc.argmax(v) == 1
    assert orc.argmax(np.full(9, -3.0, np.float32)) == 0


def test_cache_and_head_moves(orc):
    import ctypes as C
    Hkv, D, kv_max, T = 2, 64, 10, 3
    Kc, Vc = np.zeros((Hkv, kv_max, D), np.float32), np.zeros((Hkv, kv_max, D), np.float32)
    k, v = orc.normal(Hkv * T * D, 1).reshape(Hkv, T, D), orc.normal(Hkv * T * D, 2).reshape(Hkv, T, D)
    P = lambda a: a.ctypes.data_as(C.c_void_p)
    orc.lib.orc_kv_fill(P(Kc), P(Vc), P(k), P(v), T, kv_max, Hkv, D, 4)
    assert np.array_equal(Kc[:, 4:7], k) and np.array_equal(Vc[:, 4:7], v) and not Kc[:, :4].any()
    k1, v1 = np.ascontiguousarray(k[:, 0]), np.ascontiguousarray(v[:, 0])
    orc.lib.orc_kv_append(P(Kc), P(Vc), P(k1), P(v1), 9, kv_max, Hkv, D)
    assert np.array_equal(Kc[:, 9], k1)


# ---- agreement with the compiled reference (where built) -------------------------------------
def test_oracle_equals_reference_bitwise(orc, refimpl):
    r = refimpl
    K, N = 896, 96
    w = orc.normal(K * N, 1, 0, 0.02).reshape(K, N)
    assert np.array_equal(orc.to_q4(w), r.to_q4(w)) and np.array_equal(orc.to_bf16(w), r.to_bf16(w))
    buf, x = orc.to_q4(w), orc.normal(K, 2)
    assert np.array_equal(orc.q4_to_f32(buf, K, N), r.q4_to_f32(buf, K, N))
    assert np.array_equal(orc.gemv_q4(x, buf, N, K), r.gemv_q4(x, buf, N, K))
    assert np.array_equal(orc.gemv_bf16(x, orc.to_bf16(w)), r.gemv_bf16(x, orc.to_bf16(w)))
    for (m, n, k) in [(1, 8, 16), (3, 40, 100), (2, 300, 700), (5, 64, 1030)]:
        A, B = orc.normal(m * k, 11).reshape(m, k), orc.normal(k * n, 12).reshape(k, n)
        assert np.array_equal(orc.dot(A, B, 2.0, 1.0), r.dot(A, B, 2.0, 1.0))
    H, ctx, D = 4, 300, 128
    q = orc.normal(H * D, 21).reshape(H, D)
    Kk, V = orc.normal(H * ctx * D, 22).reshape(H, ctx, D), orc.normal(H * ctx * D, 23).reshape(H, ctx, D)
    assert np.array_equal(orc.attn_decode(q, Kk, V, 0.088), r.attn_decode(q, Kk, V, 0.088))
    xr = orc.normal(6 * 64, 31).reshape(6, 64)
    assert np.array_equal(orc.rope(xr, 4095, 1e6), r.rope(xr, 4095, 1e6))
    xx, ww = orc.normal(2 * 3584, 41).reshape(2, 3584), orc.normal(3584, 42, 1, 0.02)
    assert np.array_equal(orc.rmsnorm(xx, ww, 1e-6), r.rmsnorm(xx, ww, 1e-6))
    g, u = orc.normal(4864, 51), orc.normal(4864, 52)
    assert np.array_equal(orc.swiglu(g, u), r.swiglu(g, u))
    v = np.abs(orc.normal(5000, 71)) + np.float32(0.1)
    for op in ("exp", "log", "sqrt", "sigmoid", "relu", "recip"):
        assert np.array_equal(orc.unary(op, v, 1.5, -0.25), r.unary(op, v, 1.5, -0.25)), op
    assert orc.argmax(g) == r.argmax(g)


def test_oracle_model_equals_reference_model(orc, refimpl):
    dims = dict(n_layers=2, hidden=256, n_q_heads=4, n_kv_heads=2, head_dim=64, ff=512, vocab=320,
                max_ctx=16, eps=1e-6, rope_base=1e6)
    om = orc.qwen_create(dims, seed=11, q4=True)
    rm = refimpl.qwen_from_oracle(om, predeq=False)
    tok = 3
    for pos in range(6):
        t1, l1 = om.step(tok, pos)
        t2, l2 = rm.step(tok, pos)
        assert t1 == t2 and np.array_equal(l1, l2), pos
        tok = t1
    rm.close(); om.close()
