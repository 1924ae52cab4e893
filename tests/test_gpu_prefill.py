"""GPU parity: the prefill pair (MFMA GEMM against bf16 weights, causal attention over a
cache) through the C ABI vs the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

from oraclelib import allclose, maxrel

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-4, 1e-5


def _gemm(lib, A, Wb):
    M, K = A.shape
    N = Wb.shape[0]
    da, dw, dc = lib.to_device(A), lib.to_device(Wb), lib.empty((M, N))
    lib.gemm_bf16_nt(da, dw, dc, M, N, K)
    out = dc.numpy()
    for b in (da, dw, dc):
        b.free()
    return out


@pytest.mark.parametrize("M,N,K", [
    (512, 512, 3584),      # a prompt chunk against a kv-sized projection: 8 wide tiles, K split 14 ways
    (512, 4608, 896),      # 72 wide tiles, K split 3 ways
    (1024, 4864, 896),     # 152 wide tiles, K split 3 ways
    (128, 1152, 896),      # 0.5B fused q|k|v
    (33, 200, 40),         # short prompt: 64-row tiles; ragged in M, N and K (K % 32 != 0)
    (64, 4608, 896),       # short prompt, K split
    (1, 64, 8),            # smallest legal
    (257, 129, 264),       # N % 4 != 0: no K split possible
])
def test_gemm_bf16_nt_matches_oracle(lib, orc, M, N, K):
    """out[M,N] = A[M,K] . W[N,K]^T, W bf16 (cuda.h:786-840). Weights N(0,0.02) as in the
    decode model, A ~ N(0,1)."""
    print("case gemm_bf16_nt", M, N, K, flush=True)
    A = orc.normal(M * K, 11).reshape(M, K)
    Wb = orc.to_bf16(orc.normal(N * K, 12, std=0.02)).reshape(N, K)
    before = lib.census()["gemm_bf16_nt"]
    got = _gemm(lib, A, Wb)
    assert lib.census()["gemm_bf16_nt"] == before + 1
    want = orc.gemm_bf16_nt(A, Wb)
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)


def test_gemm_bf16_nt_exact_cases(lib, orc):
    """What the arithmetic fixes without an oracle: the three-way bf16 split of A loses
    nothing, so integer-valued operands give exact integers, and a one-hot A row copies
    a weight column out bit for bit (a transposed operand or a wrong accumulator lane
    map fails here)."""
    M, N, K = 96, 160, 64
    rng = np.random.default_rng(5)
    A = rng.integers(-500, 500, (M, K)).astype(np.float32) + 0.5   # needs > 8 mantissa bits
    Wf = rng.integers(-64, 64, (N, K)).astype(np.float32)
    Wb = orc.to_bf16(Wf).reshape(N, K)
    got = _gemm(lib, A, Wb)
    want = (A.astype(np.float64) @ Wf.astype(np.float64).T)
    assert np.array_equal(got.astype(np.float64), want)
    # one-hot rows: out[m, n] == W[n, m % K]
    A = np.zeros((M, K), np.float32)
    A[np.arange(M), np.arange(M) % K] = 1.0
    Wf = orc.bf16_widen(orc.to_bf16(orc.normal(N * K, 3))).reshape(N, K)
    got = _gemm(lib, A, orc.to_bf16(Wf).reshape(N, K))
    assert np.array_equal(got, Wf[:, np.arange(M) % K].T)
    # 24-bit mantissas survive: a = 1 + 2^-23, w = 1 -> the sum of K copies is exact in f32
    A = np.full((32, 8), np.float32(1.0) + np.float32(2.0 ** -23), np.float32)
    got = _gemm(lib, A, orc.to_bf16(np.ones((32, 8), np.float32)).reshape(32, 8))
    assert np.all(got == np.float32(8.0 * (1.0 + 2.0 ** -23)))


def test_gemm_bf16_nt_whole_rounds_plus_split_tail(lib, orc):
    """More tiles than the chip runs at once: the columns that make whole rounds of tiles run
    with full K, the rest (here 9 tile columns, the last one ragged) is split over K into scratch
    parts and summed into its column range of the result. Integer-valued operands make every
    partial sum exact, so the result must equal the float64 product bit for bit wherever a
    column lands."""
    M, N, K = 640, 256 * 110 + 100, 1024
    rng = np.random.default_rng(17)
    A = rng.integers(-100, 100, (M, K)).astype(np.float32) + 0.5
    Wf = rng.integers(-16, 16, (N, K)).astype(np.float32)
    got = _gemm(lib, A, orc.to_bf16(Wf).reshape(N, K))
    want = A.astype(np.float64) @ Wf.astype(np.float64).T
    assert np.array_equal(got.astype(np.float64), want)


def test_gemm_bf16_nt_random_shapes_exact(lib, orc):
    """Forty random shapes (every tile variant, K-split counts from 1 to 16, ragged edges in M, N
    and K, N % 4 != 0 where K cannot be split) with integer-valued operands: each result must
    equal the float64 product exactly, whatever the launch shape chosen for it."""
    rng = np.random.default_rng(23)
    for case in range(40):
        M = int(rng.choice([1, 7, 33, 64, 65, 128, 200, 257, 512, 640]))
        N = int(rng.integers(1, 1400)) if case % 3 else int(rng.integers(1, 350)) * 4
        K = int(rng.integers(1, 260)) * 8
        print("case gemm random", M, N, K, flush=True)
        A = rng.integers(-60, 60, (M, K)).astype(np.float32) + 0.25
        Wf = rng.integers(-12, 12, (N, K)).astype(np.float32)
        got = _gemm(lib, A, orc.to_bf16(Wf).reshape(N, K))
        want = A.astype(np.float64) @ Wf.astype(np.float64).T
        assert np.array_equal(got.astype(np.float64), want), (M, N, K)


@pytest.mark.parametrize("M,N,K,room", [
    (512, 3584, 3584, 16),    # o-proj of the 7B shape: 56 tiles, 9 parts
    (512, 3584, 18944, 16),   # down
    (512, 3584, 3584, 4),     # the caller's buffer holds 4 parts: the split stops there
    (512, 3584, 3584, 1),     # room for the product only: one part
    (200, 896, 4864, 16),     # 0.5B down, ragged M
    (33, 896, 896, 16),       # short prompt: 64-row tiles
    (257, 130, 264, 16),      # N % 4 != 0: never split
])
def test_gemm_parts_then_residual_norm_is_gemm_then_residual_norm(lib, orc, M, N, K, room):
    """The product left as its K-split parts and summed by the residual norm while it reads them
    is, bit for bit, the product summed by the GEMM's own part-sum launch and then normalised:
    same parts, same order of addition (when the caller's buffer has room for the split the plain
    GEMM picks - 16 parts always is). Checked on the residual stream and on the normalised rows."""
    print("case gemm parts", M, N, K, room, flush=True)
    A = orc.normal(M * K, 41).reshape(M, K)
    Wb = orc.to_bf16(orc.normal(N * K, 42, std=0.02)).reshape(N, K)
    res = orc.normal(M * N, 43).reshape(M, N)
    nw = orc.normal(N, 44) + 1.0
    da, dw, dres, dnw = (lib.to_device(a) for a in (A, Wb, res, nw))
    dc, x1, h1, x2, h2 = (lib.empty((M, N)) for _ in range(5))
    parts = lib.empty((room, M, N))
    lib.gemm_bf16_nt(da, dw, dc, M, N, K)
    lib.rmsnorm_res(dc, dres, dnw, x1, h1, N, 1e-6, M)
    n = lib.gemm_bf16_nt_parts(da, dw, parts, M, N, K)
    assert 1 <= n <= room
    if room == 16 and N % 4 == 0 and M * N < 4 * 512 * 3584:
        assert n > 1          # these shapes do split: the test is not vacuous
    if N % 4 != 0:
        assert n == 1
    lib.rmsnorm_res_parts(dres, parts, n, dnw, x2, h2, N, 1e-6, M)
    if room == 16:            # room for the split the plain GEMM picks: the same parts
        assert np.array_equal(x1.numpy(), x2.numpy())
        assert np.array_equal(h1.numpy(), h2.numpy())
    else:                     # fewer, longer parts: the same product to summation-order noise
        assert allclose(x2.numpy(), x1.numpy(), RTOL, ATOL)
        assert allclose(h2.numpy(), h1.numpy(), RTOL, ATOL)
    x1n, h1n = x2.numpy(), h2.numpy()
    # and the parts do add up to the product the oracle computes
    p = parts.numpy()[:n].astype(np.float64).sum(axis=0)
    want = orc.gemm_bf16_nt(A[:8], Wb)
    assert allclose(p[:8].astype(np.float32), want, RTOL, ATOL)
    # in place on the residual stream, as the model's second norm of a layer does
    lib.rmsnorm_res_parts(dres, parts, n, dnw, dres, h2, N, 1e-6, M)
    assert np.array_equal(dres.numpy(), x1n) and np.array_equal(h2.numpy(), h1n)
    for b in (da, dw, dres, dnw, dc, x1, h1, x2, h2, parts):
        b.free()


@pytest.mark.parametrize("M,ff,K", [
    (512, 18944, 3584),    # 7B chunk: 128 whole-round tile columns + 20 split over K
    (512, 4864, 896),      # 0.5B chunk: 152 tiles, split over K
    (200, 1000, 264),      # ragged in M and in the last tile's features
    (64, 4864, 896),       # short prompt: 64-row tiles
    (7, 36, 40),           # less than one tile
    (130, 130, 64),        # ff % 4 != 0: never split
])
def test_gemm_swiglu_epilogue(lib, orc, M, ff, K):
    """act = swiglu(A . Wg^T, A . Wu^T) from one launch over the fused [gate rows | up rows] matrix:
    against the oracle's product and gate, and against this library's gemm_bf16_nt followed by
    swiglu (the same products; the K split may fall on other columns, hence not bit for bit)."""
    print("case gemm swiglu", M, ff, K, flush=True)
    A = orc.normal(M * K, 51).reshape(M, K)
    Wb = orc.to_bf16(orc.normal(2 * ff * K, 52, std=0.05)).reshape(2 * ff, K)
    da, dw = lib.to_device(A), lib.to_device(Wb)
    act, gu, act2 = lib.empty((M, ff)), lib.empty((M, 2 * ff)), lib.empty((M, ff))
    lib.gemm_bf16_nt_swiglu(da, dw, act, M, ff, K)
    lib.gemm_bf16_nt(da, dw, gu, M, 2 * ff, K)
    lib.swiglu(gu, act2, ff, M)
    got, two = act.numpy(), act2.numpy()

    def within(got, want, prod):
        # the GEMM's tolerance on each product, carried through act = (g * sigmoid(g)) * u:
        # |d act| <= |u| * 1.1 * |dg| + |g * sigmoid(g)| * |du|   (|d(g * sigmoid(g)) / dg| < 1.1)
        g, u = prod[:, :ff].astype(np.float64), prod[:, ff:].astype(np.float64)
        dg, du = RTOL * np.abs(g) + ATOL, RTOL * np.abs(u) + ATOL
        tol = 1.1 * np.abs(u) * dg + np.abs(g / (1.0 + np.exp(-g))) * du + ATOL
        return bool(np.all(np.abs(got.astype(np.float64) - want) <= tol))

    assert within(got, two, gu.numpy()), maxrel(got, two)
    rows = [0, M // 2, M - 1]
    p = orc.gemm_bf16_nt(A[rows], Wb)
    want = orc.swiglu_fused(np.ascontiguousarray(p), ff)
    assert within(got[rows], want, p), maxrel(got[rows], want)
    assert maxrel(got, two) < 1e-4
    for b in (da, dw, act, gu, act2):
        b.free()


def test_gemm_swiglu_exact_cases(lib, orc):
    """What the layout fixes without an oracle. A gate product of exactly 0 gives act = 0 * 0.5 * up
    = 0 whatever up is, and a gate product large enough that sigmoid rounds to 1 gives act = g * up
    exactly; with a one-hot A row both products are weight entries, so every (row, feature) pair
    must land where its gate AND its up row say - a feature gated with another feature's up
    value, or stored under another feature's index, fails."""
    M, ff, K = 96, 320, 64
    rng = np.random.default_rng(9)
    Wg = rng.integers(20, 40, (ff, K)).astype(np.float32)           # sigmoid(g >= 20) == 1 in f32
    Wu = rng.integers(-64, 64, (ff, K)).astype(np.float32)
    A = np.zeros((M, K), np.float32)
    A[np.arange(M), np.arange(M) % K] = 1.0
    Wb = orc.to_bf16(np.concatenate([Wg, Wu])).reshape(2 * ff, K)
    da, dw, act = lib.to_device(A), lib.to_device(Wb), lib.empty((M, ff))
    lib.gemm_bf16_nt_swiglu(da, dw, act, M, ff, K)
    cols = np.arange(M) % K
    assert np.array_equal(act.numpy(), (Wg[:, cols] * Wu[:, cols]).T)
    for b in (da, dw, act):
        b.free()


@pytest.mark.parametrize("M,N,K", [
    (512, 3584, 3584),     # 7B o-proj: 128 x 128 tiles, K split
    (512, 1152, 896),      # 0.5B q|k|v
    (300, 4864, 896),      # ragged M
    (64, 896, 4864),       # short prompt (64-row tiles), long K
    (5, 130, 64),          # less than one tile, N % 4 != 0: never split
    (130, 520, 32),        # one scale group
])
def test_gemm_q4_nt_matches_oracle_and_the_decode_gemv(lib, orc, M, N, K):
    """C = A . dequant(Wq)^T over the int4 weight of the decode path: every row against the CPU
    path's int4 dot (array.h:1980-1984) and against this library's decode GEMV on the same buffer."""
    print("case gemm_q4_nt", M, N, K, flush=True)
    A = orc.normal(M * K, 91).reshape(M, K)
    buf = orc.fill_q4(N, K, 92) if K > 64 else orc.to_q4(orc.normal(K * N, 92, 0.0, 0.02).reshape(K, N))
    da, dw, dc, dy = lib.to_device(A), lib.to_device(buf), lib.empty((M, N)), lib.empty(N)
    lib.gemm_q4_nt(da, dw, dc, M, N, K)
    got = dc.numpy()
    for m in sorted({0, M // 3, M - 1}):
        want = orc.gemv_q4(A[m], buf, N, K)
        assert allclose(got[m], want, RTOL, ATOL), (m, maxrel(got[m], want))
        dx = lib.to_device(A[m])
        lib.gemv_q4(dx, dw, dy, N, K)
        assert allclose(got[m], dy.numpy(), RTOL, ATOL), (m, maxrel(got[m], dy.numpy()))
        dx.free()
    # the K-split parts add up to the product
    parts = lib.empty((16, M, N))
    n = lib.gemm_q4_nt_parts(da, dw, parts, M, N, K)
    assert 1 <= n <= 16
    total = parts.numpy()[:n].astype(np.float64).sum(axis=0).astype(np.float32)
    assert allclose(total, got, RTOL, ATOL), maxrel(total, got)
    for b in (da, dw, dc, dy, parts):
        b.free()


def test_gemm_q4_nt_exact_cases(lib, orc):
    """What the arithmetic fixes without an oracle: integer-valued activations, every nibble value
    and power-of-two scales make each group sum and each scaled sum exact, so the result must equal
    the float64 value of sum_g scale_g * (a . (nibble - 8)) bit for bit - a wrong nibble order,
    a scale taken from the neighbouring group or row, or a transposed tile fails."""
    M, N, K = 130, 200, 128
    rng = np.random.default_rng(31)
    A = rng.integers(-300, 300, (M, K)).astype(np.float32) + 0.5
    q = rng.integers(0, 16, (N, K)).astype(np.uint8)
    scales = (2.0 ** rng.integers(-6, 2, (N, K // 32))).astype(np.float32)
    packed = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)         # even k in the low nibble
    buf = np.concatenate([packed.reshape(-1), scales.reshape(-1).view(np.uint8)])
    da, dw, dc = lib.to_device(A), lib.to_device(buf), lib.empty((M, N))
    lib.gemm_q4_nt(da, dw, dc, M, N, K)
    w = (q.astype(np.float64) - 8.0) * np.repeat(scales.astype(np.float64), 32, axis=1)
    want = A.astype(np.float64) @ w.T
    assert np.array_equal(dc.numpy().astype(np.float64), want)
    for b in (da, dw, dc):
        b.free()


@pytest.mark.parametrize("M,ff,K", [(512, 4864, 896), (200, 1000, 64), (64, 4864, 896), (512, 18944, 3584)])
def test_gemm_q4_nt_swiglu_epilogue(lib, orc, M, ff, K):
    """The gated activation from one launch over the fused int4 [gate rows | up rows] weight against
    gemm_q4_nt followed by swiglu, with the GEMM's tolerance carried through the gate."""
    print("case gemm_q4 swiglu", M, ff, K, flush=True)
    A = orc.normal(M * K, 95).reshape(M, K)
    buf = orc.fill_q4(2 * ff, K, 96)
    da, dw = lib.to_device(A), lib.to_device(buf)
    act, gu, act2 = lib.empty((M, ff)), lib.empty((M, 2 * ff)), lib.empty((M, ff))
    lib.gemm_q4_nt_swiglu(da, dw, act, M, ff, K)
    lib.gemm_q4_nt(da, dw, gu, M, 2 * ff, K)
    lib.swiglu(gu, act2, ff, M)
    got, two, prod = act.numpy().astype(np.float64), act2.numpy(), gu.numpy()
    g, u = prod[:, :ff].astype(np.float64), prod[:, ff:].astype(np.float64)
    dg, du = RTOL * np.abs(g) + ATOL, RTOL * np.abs(u) + ATOL
    tol = 1.1 * np.abs(u) * dg + np.abs(g / (1.0 + np.exp(-g))) * du + ATOL
    assert np.all(np.abs(got - two) <= tol), maxrel(got, two)
    for b in (da, dw, act, gu, act2):
        b.free()


def test_gemm_q4_nt_rejects(lib):
    """The int4 GEMM refuses what its kernel does not cover instead of computing something else:
    a scale group other than 32, K that is not whole groups, missing scales."""
    a, w, c_ = lib.empty((8, 64)), lib.empty_bytes(64 * 64), lib.empty((8, 64))
    n = C.c_int(0)
    with pytest.raises(RuntimeError):
        lib._chk(lib.c.tlhip_gemm_q4_nt(a.ptr, w.ptr, w.ptr + 2048, c_.ptr, 8, 64, 64, 64))      # group 64
    with pytest.raises(RuntimeError):
        lib._chk(lib.c.tlhip_gemm_q4_nt(a.ptr, w.ptr, w.ptr + 2048, c_.ptr, 8, 64, 48, 32))      # K % 32 != 0
    with pytest.raises(RuntimeError):
        lib._chk(lib.c.tlhip_gemm_q4_nt(a.ptr, w.ptr, None, c_.ptr, 8, 64, 64, 32))              # no scales
    with pytest.raises(RuntimeError):
        lib._chk(lib.c.tlhip_gemm_q4_nt_parts(a.ptr, w.ptr, w.ptr + 2048, c_.ptr, 16, 8, 64, 64, 32, C.byref(n)))  # no room
    with pytest.raises(RuntimeError):
        lib._chk(lib.c.tlhip_gemm_q4_nt_swiglu(a.ptr, w.ptr, w.ptr + 2048, c_.ptr, 8, 32, 64, 16))  # group 16
    for b in (a, w, c_):
        b.free()


def test_gemm_parts_rejects(lib):
    a, w = lib.empty((64, 64)), lib.empty((64, 32))
    small = lib.empty(16)
    with pytest.raises(RuntimeError):
        lib.gemm_bf16_nt_parts(a, w, small, 64, 64, 64)          # no room for one [M, N] part
    x = lib.empty((64, 64))
    with pytest.raises(RuntimeError):
        lib.rmsnorm_res_parts(a, x, 0, w, small, small, 64, 1e-6, 64)   # S = 0
    with pytest.raises(RuntimeError):
        lib.rmsnorm_res_parts(a, x, 1, w, x, small, 64, 1e-6, 64)       # xout is the parts
    for b in (a, w, small, x):
        b.free()


def test_gemm_bf16_nt_row_equals_gemv(lib, orc):
    """Row m of the GEMM and the decode GEMV over the same [N,K] bf16 weights agree to
    summation-order noise."""
    M, N, K = 8, 1024, 896
    A = orc.normal(M * K, 21).reshape(M, K)
    Wb = orc.to_bf16(orc.normal(N * K, 22, std=0.02)).reshape(N, K)
    got = _gemm(lib, A, Wb)
    dw, dy = lib.to_device(Wb), lib.empty(N)
    for m in (0, 7):
        da = lib.to_device(A[m])
        lib.gemv_bf16_row(da, dw, dy, N, K)
        assert allclose(got[m], dy.numpy(), RTOL, ATOL)
        da.free()
    dw.free(), dy.free()


def test_gemm_bf16_nt_declines(lib):
    from importlib import import_module
    err = import_module("cpp-tensorlib_amd.capi").TlHipError
    a, w, c = lib.empty((4, 12)), lib.empty((4, 12), np.uint16), lib.empty((4, 4))
    with pytest.raises(err):
        lib.gemm_bf16_nt(a, w, c, 4, 4, 12)      # K % 8 != 0
    for b in (a, w, c):
        b.free()


KERNELS = {"auto": 0, "valu": 1, "fp32pipe": 2, "f16terms": 4}


def _prefill(lib, q, K, V, scale, pos0, kv_bf16=False, kernel="auto"):
    """kernel (tlhip_tune_attn_prefill): the library's own choice, the VALU kernel, the fp32
    matrix-pipe kernel, or the f16-term kernels on the matrix cores (two f16 terms per operand; what
    the library's own choice takes deep in a context)."""
    Hq, T, D = q.shape
    Hkv, kv_max, _ = K.shape
    dq, dk, dv, do = lib.to_device(q), lib.to_device(K), lib.to_device(V), lib.empty((Hq, T, D))
    lib.tune_attn_prefill(KERNELS[kernel])
    try:
        lib.attn_prefill(dq, dk, dv, do, Hq, Hkv, T, kv_max, D, scale, kv_bf16, pos0)
    finally:
        lib.tune_attn_prefill(0)
    out = do.numpy()
    for b in (dq, dk, dv, do):
        b.free()
    return out


@pytest.mark.parametrize("kernel", list(KERNELS))
@pytest.mark.parametrize("D,Hq,Hkv,T,pos0", [
    (128, 28, 4, 64, 0), (64, 14, 2, 100, 0), (128, 4, 2, 7, 0), (128, 8, 8, 33, 300),
    (64, 6, 2, 257, 19), (128, 2, 1, 1, 0), (128, 2, 1, 1, 77), (64, 4, 4, 130, 513),
    (128, 7, 1, 512, 0), (64, 2, 2, 512, 0), (128, 2, 1, 200, 1000), (128, 1, 1, 31, 32), (64, 3, 1, 32, 31),
    (128, 7, 1, 512, 3584), (128, 4, 4, 256, 7680),      # deep in a context: > 120 key tiles per wavefront
    (128, 12, 1, 50, 1500), (128, 3, 1, 100, 990), (128, 16, 2, 17, 2047),   # head groups of 12, 3 and 8; ragged chunk lengths
    (64, 14, 2, 512, 1536), (64, 5, 1, 33, 3000),                            # head size 64 deep in a context (0.5B shape)
])
def test_attn_prefill_matches_oracle(lib, orc, D, Hq, Hkv, T, pos0, kernel):
    """Causal prefill over a cache: query p at absolute position pos0+p sees keys
    0..pos0+p (cuda.h:1165-1200). Rows past pos0+T hold poison that must not leak; so
    must, per query, the chunk's own later keys."""
    print("case attn_prefill", D, Hq, Hkv, T, pos0, flush=True)
    kv_max = pos0 + T + 5
    q = orc.normal(Hq * T * D, 31).reshape(Hq, T, D)
    K = orc.normal(Hkv * kv_max * D, 32).reshape(Hkv, kv_max, D)
    V = orc.normal(Hkv * kv_max * D, 33).reshape(Hkv, kv_max, D)
    K[:, pos0 + T:, :] = 1e30
    V[:, pos0 + T:, :] = np.nan
    scale = 1.0 / np.sqrt(float(D))
    got = _prefill(lib, q, K, V, scale, pos0, kernel=kernel)
    want = orc.attn_prefill(q, K, V, scale, pos0)
    assert np.all(np.isfinite(got))
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)


def _attn_f64(q, K, V, scale, pos0):
    """Causal attention in float64: what the arithmetic fixes, independent of any summation order."""
    Hq, T, D = q.shape
    Hkv = K.shape[0]
    out = np.empty((Hq, T, D))
    for h in range(Hq):
        kh, vh = K[h // (Hq // Hkv)].astype(np.float64), V[h // (Hq // Hkv)].astype(np.float64)
        for t in range(T):
            s = (kh[:pos0 + t + 1] @ q[h, t].astype(np.float64)) * scale
            p = np.exp(s - s.max())
            out[h, t] = (p / p.sum()) @ vh[:pos0 + t + 1]
    return out


@pytest.mark.parametrize("kernel", ["fp32pipe", "f16terms"])
@pytest.mark.parametrize("case", ["one_dominant_key", "equal_scores", "large_values", "tiny_values", "cancelling_values",
                                  "value_scale_by_tile"])
def test_attn_prefill_adversarial_rows(lib, orc, case, kernel):
    """Rows chosen against the f16-term products (two terms per operand, scaled per query row and
    per 32-key tile, three term pairs: what is dropped is below 2^-24 of |a b|) and the online softmax:
      one_dominant_key    one key's score exceeds the others by ~40: the softmax is one-hot to
                          fp32 and the output must be that key's value row;
      equal_scores        every key of a row scores the same to 1e-6: the output is a plain mean,
                          where an error in the scores is not damped by a peaked softmax;
      large_values        |q|, |k|, |v| around 2^10 (scores around 1e5 before the maximum is
                          taken): plane residuals of large numbers;
      tiny_values         values around 2^-40: far below f16's range before the per-tile scaling;
      cancelling_values   V alternates +-(1000 + small) so that the output is a small difference
                          of large terms (tests the value terms and the fp32 accumulation);
      value_scale_by_tile every run of 32 keys has its V rows scaled by its own power of two between
                          2^-24 and 2^24 and its K rows by one between 2^-2 and 2^2 (the f16 form
                          scales K and V per 32-key tile and carries the output accumulators from
                          one tile's unit to the next).
    Both matrix kernels against the CPU oracle at allclose(1e-4, 1e-5) and against float64 with the
    bound an fp32 evaluation obeys: 2^-22 (4 + max_k sum_i |q_i k_i| scale) sum_k p_k |v_k| (the
    CPU oracle itself uses up to 0.7 of it on these rows; the plane kernel measured at or below the
    oracle's error on every case)."""
    print("case attn_prefill adversarial", case, kernel, flush=True)
    D, Hq, Hkv, T, pos0 = 128, 7, 1, 48, 1200
    kv_max = pos0 + T
    rng = np.random.default_rng(17)
    q = rng.standard_normal((Hq, T, D)).astype(np.float32)
    K = rng.standard_normal((Hkv, kv_max, D)).astype(np.float32)
    V = rng.standard_normal((Hkv, kv_max, D)).astype(np.float32)
    scale = np.float32(1.0 / np.sqrt(float(D)))
    if case == "one_dominant_key":
        # key 777 is 4 q-directions long for every row: its score leads by ~ 4 |q|^2 scale ~ 45
        K[0, 777] = 0.0
        q[:] = np.abs(q)
        K[0, 777] = 4.0 * np.sign(q.mean(axis=(0, 1)))
    elif case == "equal_scores":
        K[0, :] = K[0, 0] + (1e-6 * rng.standard_normal((kv_max, D))).astype(np.float32)
    elif case == "large_values":
        q *= np.float32(1024.0); K *= np.float32(1024.0); V *= np.float32(1024.0)
        scale = np.float32(scale / 1024.0 / 1024.0 * 8.0)
    elif case == "tiny_values":
        q *= np.float32(2.0 ** -40); K *= np.float32(2.0 ** -40); V *= np.float32(2.0 ** -40)
        scale = np.float32(scale * 2.0 ** 80)
    elif case == "cancelling_values":
        sign = np.where(np.arange(kv_max) % 2 == 0, 1.0, -1.0).astype(np.float32)
        V[0] = sign[:, None] * (1000.0 + V[0])
        K[0, :] = K[0, 0] + (1e-3 * rng.standard_normal((kv_max, D))).astype(np.float32)   # near-uniform softmax
    elif case == "value_scale_by_tile":
        tiles = (kv_max + 31) // 32
        ev = np.repeat(rng.integers(-24, 25, tiles), 32)[:kv_max]
        ek = np.repeat(rng.integers(-2, 3, tiles), 32)[:kv_max]
        V[0] *= np.exp2(ev).astype(np.float32)[:, None]
        K[0] *= np.exp2(ek).astype(np.float32)[:, None]
    got = _prefill(lib, q, K, V, float(scale), pos0, kernel=kernel)
    want = orc.attn_prefill(q, K, V, float(scale), pos0)
    assert np.all(np.isfinite(got))
    exact = _attn_f64(q, K, V, float(scale), pos0)
    # sum_k p_k |v_k| per output element, the scale an fp32 evaluation's error goes with
    mag = _attn_f64(q, K, np.abs(V), float(scale), pos0)
    err, err_ref = np.abs(got - exact), np.abs(want - exact)
    # An fp32 score carries up to 2^-24 sum_i |q_i k_i| scale of rounding per product, and an error
    # d in a score is a relative error d in its probability: the bound grows with the largest
    # sum_i |q_i k_i| scale of a row (its own dot products are what the terms must reproduce).
    absdot = np.einsum("htd,kd->htk", np.abs(q).astype(np.float64), np.abs(K[0]).astype(np.float64)).max(axis=2) * float(scale)
    bound = 2.0 ** -22 * (4.0 + absdot)[:, :, None] * mag + 1e-37
    print("   max err / bound: kernel %.3f, CPU oracle %.3f" % ((err / bound).max(), (err_ref / bound).max()), flush=True)
    assert np.all(err <= bound), float((err / bound).max())
    # (with sharp softmaxes over large scores, or outputs that are small differences of large
    # terms, two correct fp32 evaluations differ by more than allclose(1e-4, 1e-5) allows)
    if case in ("one_dominant_key", "equal_scores"):
        assert allclose(got, want, RTOL, ATOL), maxrel(got, want)
    if case == "one_dominant_key":
        assert allclose(got, np.broadcast_to(V[0, 777], got.shape), 1e-6, 1e-6)


@pytest.mark.parametrize("kernel", list(KERNELS))
def test_attn_prefill_rows_equal_decode(lib, orc, kernel):
    """Row p of a prefill equals a decode step with ctx = pos0 + p + 1 (the equivalence the
    reference's prefill bench relies on, bench_qwen_prefill.cpp:283-310), and the first query
    of a fresh cache returns V[0] (exactly; to one rounding from the f16 form)."""
    D, Hq, Hkv, T, pos0 = 128, 8, 2, 40, 24
    kv_max = pos0 + T
    q = orc.normal(Hq * T * D, 41).reshape(Hq, T, D)
    K = orc.normal(Hkv * kv_max * D, 42).reshape(Hkv, kv_max, D)
    V = orc.normal(Hkv * kv_max * D, 43).reshape(Hkv, kv_max, D)
    scale = 1.0 / np.sqrt(float(D))
    got = _prefill(lib, q, K, V, scale, pos0, kernel=kernel)
    dk, dv, do = lib.to_device(K), lib.to_device(V), lib.empty((Hq, D))
    for p in (0, 1, 17, T - 1):
        dq = lib.to_device(np.ascontiguousarray(q[:, p, :]))
        lib.attn_decode(dq, dk, dv, do, Hq, Hkv, pos0 + p + 1, kv_max, D, scale)
        assert allclose(got[:, p, :], do.numpy(), RTOL, ATOL)
        dq.free()
    for b in (dk, dv, do):
        b.free()
    fresh = _prefill(lib, q, K, V, scale, 0, kernel=kernel)
    v0 = np.repeat(V[:, 0, :], Hq // Hkv, axis=0)
    if kernel == "f16terms":   # two f16 terms carry 23 bits of a value, not 24: one rounding, like any fp32 operation
        assert np.all(np.abs(fresh[:, 0, :] - v0) <= 2.0 ** -23 * np.abs(v0))
    else:
        assert np.array_equal(fresh[:, 0, :], v0)


@pytest.mark.parametrize("kernel", list(KERNELS))
@pytest.mark.parametrize("pos0", [10, 2100])
@pytest.mark.parametrize("D", [128, 64])
def test_attn_prefill_bf16_cache(lib, orc, D, pos0, kernel):
    """A bf16 cache, fresh and deep in a context (one plane / one term of K and V in the matrix-core kernels)."""
    Hq, Hkv, T = 4, 2, 70
    kv_max = pos0 + T
    q = orc.normal(Hq * T * D, 51).reshape(Hq, T, D)
    Kb = orc.to_bf16(orc.normal(Hkv * kv_max * D, 52)).reshape(Hkv, kv_max, D)
    Vb = orc.to_bf16(orc.normal(Hkv * kv_max * D, 53)).reshape(Hkv, kv_max, D)
    scale = 1.0 / np.sqrt(float(D))
    got = _prefill(lib, q, Kb, Vb, scale, pos0, kv_bf16=True, kernel=kernel)
    want = orc.attn_prefill(q, orc.bf16_widen(Kb).reshape(Kb.shape),
                            orc.bf16_widen(Vb).reshape(Vb.shape), scale, pos0)
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)


@pytest.mark.parametrize("D,T,pos0,expect", [
    (128, 64, 100, "fp32pipe"), (128, 64, 576, "f16terms"), (128, 512, 0, "f16terms"), (128, 256, 256, "fp32pipe"),
    (64, 64, 700, "fp32pipe"), (64, 64, 960, "f16terms"), (64, 256, 512, "f16terms"), (128, 8, 4000, "fp32pipe"),
])
def test_attn_prefill_builtin_choice(lib, orc, D, T, pos0, expect):
    """Which kernel the library picks by itself: the f16-term kernels from 640 keys on at head size
    128 (512 for a chunk of 512) and from 1024 at head size 64 (768 for chunks of 256 up), chunks
    of at least 16 tokens; the fp32 matrix-pipe kernel otherwise. Checked bit for bit against the
    forced kernel."""
    Hq, Hkv = 4, 2
    kv_max = pos0 + T
    q = orc.normal(Hq * T * D, 81).reshape(Hq, T, D)
    K = orc.normal(Hkv * kv_max * D, 82).reshape(Hkv, kv_max, D)
    V = orc.normal(Hkv * kv_max * D, 83).reshape(Hkv, kv_max, D)
    scale = 1.0 / np.sqrt(float(D))
    auto = _prefill(lib, q, K, V, scale, pos0, kernel="auto")
    forced = _prefill(lib, q, K, V, scale, pos0, kernel=expect)
    assert np.array_equal(auto, forced)
    other = _prefill(lib, q, K, V, scale, pos0, kernel="fp32pipe" if expect == "f16terms" else "f16terms")
    assert not np.array_equal(auto, other)      # (the two kernels differ in the last bits, so the check above tells them apart)


@pytest.mark.parametrize("kernel", list(KERNELS))
def test_attn_prefill_negative_scale(lib, orc, kernel):
    """The scale is an argument like any other: a negative one turns the softmax towards the
    smallest dot products (the matrix-core kernels fold its sign into Q)."""
    D, Hq, Hkv, T, pos0 = 128, 4, 2, 40, 1100
    kv_max = pos0 + T
    q = orc.normal(Hq * T * D, 71).reshape(Hq, T, D)
    K = orc.normal(Hkv * kv_max * D, 72).reshape(Hkv, kv_max, D)
    V = orc.normal(Hkv * kv_max * D, 73).reshape(Hkv, kv_max, D)
    got = _prefill(lib, q, K, V, -0.07, pos0, kernel=kernel)
    want = orc.attn_prefill(q, K, V, -0.07, pos0)
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)


@pytest.mark.parametrize("kv_bf16", [False, True])
@pytest.mark.parametrize("D,Hq,Hkv,T,pos0", [(128, 28, 4, 64, 0), (64, 14, 2, 100, 7), (128, 4, 2, 1, 300), (64, 3, 1, 5, 2)])
def test_qkv_rope_fill_equals_the_separate_ops(lib, orc, D, Hq, Hkv, T, pos0, kv_bf16):
    """tlhip_rope_table_range + tlhip_qkv_rope_fill against split_heads (with bias) + rope(q) +
    rope(k) + kv_fill: rotated queries and both caches bit for bit (f32 and bf16 caches), cache rows
    outside [pos0, pos0 + T) untouched."""
    print("case qkv_rope_fill", D, Hq, Hkv, T, pos0, kv_bf16, flush=True)
    base, kv_max = 1e6, pos0 + T + 3
    qd, kvd = Hq * D, Hkv * D
    ld = qd + 2 * kvd
    qkv = orc.normal(T * ld, 61).reshape(T, ld)
    bias = orc.normal(ld, 62, 0.0, 0.1)
    cdt = np.uint16 if kv_bf16 else np.float32
    fill = np.full(Hkv * kv_max * D, 0x7fc0 if kv_bf16 else np.nan, cdt)
    dqkv, db = lib.to_device(qkv), lib.to_device(bias)
    # the separate ops
    dh = lib.empty((Hq + 2 * Hkv, T, D))
    lib.split_heads(dqkv, db, dh, T, ld, 0, Hq + 2 * Hkv, D)
    lib.rope(dh, dh, Hq * T, T, D, pos0, base)
    c = lib.c
    kh, vh = dh.ptr + qd * T * 4, dh.ptr + (qd + kvd) * T * 4
    lib._chk(c.tlhip_rope(kh, kh, Hkv * T, T, D, pos0, base, None))
    K1, V1 = lib.to_device(fill), lib.to_device(fill)
    lib._chk(c.tlhip_kv_fill(K1.ptr, V1.ptr, kh, vh, T, kv_max, Hkv, D, int(kv_bf16), pos0))
    want_q = dh.numpy().reshape(-1)[:qd * T]
    # the fused launch
    tab, qh = lib.empty(T * D), lib.to_device(np.full(qd * T, np.nan, np.float32))
    K2, V2 = lib.to_device(fill), lib.to_device(fill)
    lib.rope_table_range(tab, D, pos0, T, base)
    lib._chk(c.tlhip_qkv_rope_fill(dqkv.ptr, db.ptr, db.ptr + qd * 4, db.ptr + (qd + kvd) * 4, tab.ptr, qh.ptr,
                                   K2.ptr, V2.ptr, T, Hq, Hkv, D, pos0, kv_max, int(kv_bf16)))
    assert np.array_equal(qh.numpy(), want_q)
    assert np.array_equal(K2.numpy(cdt).view(np.uint16 if kv_bf16 else np.uint32),
                          K1.numpy(cdt).view(np.uint16 if kv_bf16 else np.uint32))
    assert np.array_equal(V2.numpy(cdt).view(np.uint16 if kv_bf16 else np.uint32),
                          V1.numpy(cdt).view(np.uint16 if kv_bf16 else np.uint32))
    assert np.array_equal(dqkv.numpy().reshape(T, ld), qkv)        # the projection is left untouched
    for b in (dqkv, db, dh, K1, V1, K2, V2, tab, qh):
        b.free()


@pytest.mark.parametrize("kv_bf16", [False, True])
@pytest.mark.parametrize("D,Hq,Hkv,T,pos0,S", [(128, 28, 4, 64, 0, 7), (64, 14, 2, 100, 7, 2), (64, 3, 1, 5, 2, 16)])
def test_qkv_rope_fill_from_k_split_parts(lib, orc, D, Hq, Hkv, T, pos0, S, kv_bf16):
    """tlhip_qkv_rope_fill_parts on S parts equals tlhip_qkv_rope_fill on their sum, taken in
    ascending order in fp32 (what the GEMM's part-sum launch stores): queries and caches bit for bit."""
    print("case qkv_rope_fill_parts", D, Hq, Hkv, T, pos0, S, kv_bf16, flush=True)
    base, kv_max = 1e6, pos0 + T + 1
    qd, kvd = Hq * D, Hkv * D
    ld = qd + 2 * kvd
    parts = orc.normal(S * T * ld, 81).reshape(S, T, ld)
    total = parts[0].copy()
    for sidx in range(1, S):
        total = total + parts[sidx]            # fp32, one rounding per part, ascending
    bias = orc.normal(ld, 82, 0.0, 0.1)
    cdt = np.uint16 if kv_bf16 else np.float32
    bits = np.uint16 if kv_bf16 else np.uint32
    fill = np.zeros(Hkv * kv_max * D, cdt)
    db, tab = lib.to_device(bias), lib.empty(T * D)
    lib.rope_table_range(tab, D, pos0, T, base)
    view = lambda off: type("View", (), {"ptr": db.ptr + off * 4})()
    bq, bk, bv = db, view(qd), view(qd + kvd)
    out = []
    for src, n in ((total, 1), (parts, S)):
        dsrc, qh = lib.to_device(src), lib.empty(qd * T)
        Kc, Vc = lib.to_device(fill), lib.to_device(fill)
        lib.qkv_rope_fill(dsrc, bq, bk, bv, tab, qh, Kc, Vc, T, Hq, Hkv, D, pos0, kv_max, kv_bf16, n_parts=n)
        out.append((qh.numpy().view(np.uint32), Kc.numpy(cdt).view(bits), Vc.numpy(cdt).view(bits)))
        for b in (dsrc, qh, Kc, Vc):
            b.free()
    for a, b in zip(*out):
        assert np.array_equal(a, b)
    db.free()
    tab.free()


def test_attn_prefill_tok_is_the_merged_layout(lib, orc):
    """tlhip_attn_prefill_tok writes [T, Hq*D]: exactly merge_heads of tlhip_attn_prefill's result."""
    D, Hq, Hkv, T, pos0 = 128, 6, 2, 75, 11
    kv_max = pos0 + T
    q = orc.normal(Hq * T * D, 71).reshape(Hq, T, D)
    K = orc.normal(Hkv * kv_max * D, 72).reshape(Hkv, kv_max, D)
    V = orc.normal(Hkv * kv_max * D, 73).reshape(Hkv, kv_max, D)
    scale = 1.0 / np.sqrt(float(D))
    head_major = _prefill(lib, q, K, V, scale, pos0)
    dq, dk, dv, do = lib.to_device(q), lib.to_device(K), lib.to_device(V), lib.empty((T, Hq * D))
    lib.attn_prefill_tok(dq, dk, dv, do, Hq, Hkv, T, kv_max, D, scale, False, pos0)
    assert np.array_equal(do.numpy(), head_major.transpose(1, 0, 2).reshape(T, Hq * D))
    for b in (dq, dk, dv, do):
        b.free()


def test_prefill_chunk_pipeline(lib, orc):
    """The attention half of a prompt chunk as the reference harness runs it
    (bench/cuda/qwen_model.h:357-383): fused q|k|v GEMM -> split_heads (+bias) -> rope at pos0
    -> kv_fill -> attn_prefill -> merge_heads, against the same chain in the oracle."""
    D, Hq, Hkv, T, pos0, H = 64, 4, 2, 24, 8, 256
    kv_max = 64
    qd, kvd = Hq * D, Hkv * D
    x = orc.normal(T * H, 61).reshape(T, H)
    Wb = orc.to_bf16(orc.normal((qd + 2 * kvd) * H, 62, std=0.05)).reshape(qd + 2 * kvd, H)
    bias = orc.normal(qd + 2 * kvd, 63, std=0.1)
    Kc = orc.normal(Hkv * kv_max * D, 64).reshape(Hkv, kv_max, D)
    Vc = orc.normal(Hkv * kv_max * D, 65).reshape(Hkv, kv_max, D)
    scale = 1.0 / np.sqrt(float(D))
    # oracle chain
    qkv = orc.gemm_bf16_nt(x, Wb) + bias[None, :]
    def heads(off, Hn):
        return np.ascontiguousarray(qkv[:, off:off + Hn * D].reshape(T, Hn, D).transpose(1, 0, 2))
    qh = orc.rope(heads(0, Hq), pos0, 1e6, T=T)
    kh = orc.rope(heads(qd, Hkv), pos0, 1e6, T=T)
    vh = heads(qd + kvd, Hkv)
    Kw, Vw = Kc.copy(), Vc.copy()
    Kw[:, pos0:pos0 + T] = kh
    Vw[:, pos0:pos0 + T] = vh
    want = orc.attn_prefill(qh, Kw, Vw, scale, pos0).transpose(1, 0, 2).reshape(T, qd)
    # device chain
    dx, dw = lib.to_device(x), lib.to_device(Wb)
    dbq, dbk, dbv = (lib.to_device(bias[:qd]), lib.to_device(bias[qd:qd + kvd]),
                     lib.to_device(bias[qd + kvd:]))
    dqkv = lib.empty((T, qd + 2 * kvd))
    dq, dk, dv = lib.empty((Hq, T, D)), lib.empty((Hkv, T, D)), lib.empty((Hkv, T, D))
    dKc, dVc = lib.to_device(Kc), lib.to_device(Vc)
    dah, dat = lib.empty((Hq, T, D)), lib.empty((T, qd))
    lib.gemm_bf16_nt(dx, dw, dqkv, T, qd + 2 * kvd, H)
    lib.split_heads(dqkv, dbq, dq, T, qd + 2 * kvd, 0, Hq, D)
    lib.split_heads(dqkv, dbk, dk, T, qd + 2 * kvd, qd, Hkv, D)
    lib.split_heads(dqkv, dbv, dv, T, qd + 2 * kvd, qd + kvd, Hkv, D)
    lib.rope(dq, dq, Hq * T, T, D, pos0, 1e6)
    lib.rope(dk, dk, Hkv * T, T, D, pos0, 1e6)
    lib.kv_fill(dKc, dVc, dk, dv, T, kv_max, Hkv, D, False, pos0)
    lib.attn_prefill(dq, dKc, dVc, dah, Hq, Hkv, T, kv_max, D, scale, False, pos0)
    lib.merge_heads(dah, dat, T, Hq, D)
    got = dat.numpy()
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)
    for b in (dx, dw, dbq, dbk, dbv, dqkv, dq, dk, dv, dKc, dVc, dah, dat):
        b.free()
