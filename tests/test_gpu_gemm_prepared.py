"""GPU parity: the prompt-chunk products over a PREPARED bf16 weight (tlhip_gemm_f16w_*: f16 slab
images of the weight, two f16 terms per activation) through the C ABI vs the CPU oracle's
gemm_bf16_nt (cuda.h:787-841 / tensorlib_cuda.cu:509-519) on the bf16 weight itself."""
import numpy as np
import pytest

from oraclelib import allclose, maxrel

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-4, 1e-5


class Prepared:
    """A bf16 weight on the device with its prepared form."""

    def __init__(self, lib, Wb, gated=False):
        rows, self.K = Wb.shape
        self.N = rows // 2 if gated else rows
        self.lib, self.gated = lib, gated
        self.w = lib.to_device(Wb)
        self.image, self.exps = lib.gemm_f16w_prepare(self.w, self.N, self.K, gated=gated)

    def product(self, A):
        M = A.shape[0]
        da, dc = self.lib.to_device(A), self.lib.empty((M, self.N))
        if self.gated:
            self.lib.gemm_f16w_nt_swiglu(da, self.image, self.exps, dc, M, self.N, self.K)
        else:
            self.lib.gemm_f16w_nt(da, self.image, self.exps, dc, M, self.N, self.K)
        out = dc.numpy()
        da.free(); dc.free()
        return out

    def free(self):
        for b in (self.w, self.image, self.exps):
            b.free()


@pytest.mark.parametrize("M,N,K", [
    (512, 3584, 3584),     # 7B o-proj: 128-row tiles, K split 4 ways
    (512, 1152, 896),      # 0.5B q|k|v: 20 tiles, K split
    (300, 4864, 896),      # ragged M
    (512, 33024, 64),      # more 256-row tiles than CUs: whole rounds with full K, the rest split
    (130, 520, 32),        # one slab
    (1, 64, 32),           # one row
    (65, 129, 96),         # N % 4 != 0: never split; ragged everywhere
    (1000, 256, 18944),    # long K at the 7B down shape's depth
])
def test_gemm_f16w_matches_oracle(lib, orc, M, N, K):
    """out[M,N] = A[M,K] . W[N,K]^T with A ~ N(0,1), W ~ N(0,0.02) bf16: sampled rows against the
    oracle's f32 product over the bf16 weight."""
    print("case gemm_f16w", M, N, K, flush=True)
    A = orc.normal(M * K, 11).reshape(M, K)
    Wb = orc.to_bf16(orc.normal(N * K, 12, std=0.02)).reshape(N, K)
    P = Prepared(lib, Wb)
    before = lib.census()["gemm_bf16_nt"]
    got = P.product(A)
    assert lib.census()["gemm_bf16_nt"] == before + 1
    rows = sorted({r for r in (0, 1, M // 3, M // 2, M - 2, M - 1) if 0 <= r < M})
    want = orc.gemm_bf16_nt(np.ascontiguousarray(A[rows]), Wb)
    assert np.all(np.isfinite(got))
    assert allclose(got[rows], want, RTOL, ATOL), maxrel(got[rows], want)
    P.free()


def test_gemm_f16w_exact_cases(lib, orc):
    """What the arithmetic fixes without an oracle. The two f16 terms of a scaled activation hold
    22 significant bits and a bf16 weight is an exact f16 after its row's scaling, so integer-valued
    operands whose products and sums fit fp32 give exact integers (these activations need 13 bits:
    the second term carries part of each); a one-hot A row copies a weight column out bit for bit
    (a transposed operand, a wrong accumulator lane map or a wrong exponent on the way back fails);
    and a one-hot weight row copies an activation out with both of its terms."""
    M, N, K = 300, 520, 64
    rng = np.random.default_rng(5)
    A = rng.integers(-2000, 2000, (M, K)).astype(np.float32) + 0.25
    Wf = rng.integers(-32, 32, (N, K)).astype(np.float32)
    P = Prepared(lib, orc.to_bf16(Wf).reshape(N, K))
    got = P.product(A)
    want = A.astype(np.float64) @ Wf.astype(np.float64).T
    assert np.array_equal(got.astype(np.float64), want)
    P.free()
    # one-hot rows: out[m, n] == W[n, m % K]
    A = np.zeros((M, K), np.float32)
    A[np.arange(M), np.arange(M) % K] = 1.0
    Wf = orc.bf16_widen(orc.to_bf16(orc.normal(N * K, 3))).reshape(N, K)
    P = Prepared(lib, orc.to_bf16(Wf).reshape(N, K))
    got = P.product(A)
    assert np.array_equal(got, Wf[:, np.arange(M) % K].T)
    P.free()
    # one-hot weight rows copy activations out: 20-bit mantissas (11 in the first term, the rest in
    # the second) and 1 + 2^-23 (a second term of one bit, 2^-23 of the first) come back bit for bit
    K2 = 64
    A = (1.0 + rng.integers(0, 1 << 19, (40, K2)) * 2.0 ** -19).astype(np.float32) * np.exp2(rng.integers(-3, 4, (40, K2))).astype(np.float32)
    A[:, 5] = np.float32(1.0) + np.float32(2.0 ** -23)
    Wf = np.zeros((96, K2), np.float32)
    Wf[np.arange(96), np.arange(96) % K2] = 1.0
    P = Prepared(lib, orc.to_bf16(Wf).reshape(96, K2))
    got = P.product(A)
    assert np.array_equal(got, A[:, np.arange(96) % K2])
    P.free()


def test_gemm_f16w_whole_rounds_plus_split_tail_exact(lib, orc):
    """More 256 x 256 tiles than CUs: the columns that make whole rounds run with full K, the rest
    (the last tile column ragged) is split over K and summed into its column range. Integer-valued
    operands make every partial sum exact, so the result equals the float64 product bit for bit
    wherever a column lands."""
    M, N, K = 640, 256 * 90 + 100, 512
    rng = np.random.default_rng(17)
    A = rng.integers(-100, 100, (M, K)).astype(np.float32) + 0.5
    Wf = rng.integers(-16, 16, (N, K)).astype(np.float32)
    P = Prepared(lib, orc.to_bf16(Wf).reshape(N, K))
    got = P.product(A)
    want = A.astype(np.float64) @ Wf.astype(np.float64).T
    assert np.array_equal(got.astype(np.float64), want)
    P.free()


def test_gemm_f16w_random_shapes_exact(lib, orc):
    """Thirty random shapes (both tile heights, K-split counts from 1 up, ragged edges in M and N,
    N % 4 != 0 where K cannot be split) with integer-valued operands: each result equals the
    float64 product exactly, whatever the launch shape chosen for it."""
    rng = np.random.default_rng(23)
    for case in range(30):
        M = int(rng.choice([1, 7, 65, 128, 129, 200, 257, 512, 640]))
        N = int(rng.integers(1, 1400)) if case % 3 else int(rng.integers(1, 350)) * 4
        K = int(rng.integers(1, 66)) * 32
        print("case gemm_f16w random", M, N, K, flush=True)
        A = rng.integers(-60, 60, (M, K)).astype(np.float32) + 0.25
        Wf = rng.integers(-12, 12, (N, K)).astype(np.float32)
        P = Prepared(lib, orc.to_bf16(Wf).reshape(N, K))
        got = P.product(A)
        want = A.astype(np.float64) @ Wf.astype(np.float64).T
        assert np.array_equal(got.astype(np.float64), want), (M, N, K)
        P.free()


def test_gemm_f16w_wide_ranges(lib, orc):
    """Rows whose magnitudes are far apart, in A and in W, against float64. The scaling is per row,
    so a row of 1e-30 or 1e+20 is as accurate as a row of ones. Bound per result:
      (K/8 + 4) 2^-24 sum_k |a w|      fp32 accumulation in K/16 steps per plane, at most one ulp of the
                                       running sum each (the reference's own chain has K such steps),
                                       plus the split's 2^-24 and the product's rounding;
      2^-38 max|a_row| sum_k |w|       inside a row, an activation more than 2^23 below the row's
                                       largest keeps an absolute error of 2^-39.5 of that largest
                                       (its second f16 term is a subnormal);
      2^-39 sum_k |a| max|w_row|       a weight more than 2^29 below its row's largest likewise.
    Results below the f32 normal range are not compared."""
    M, N, K = 260, 516, 512
    rng = np.random.default_rng(31)
    A = rng.standard_normal((M, K)).astype(np.float32)
    Wf = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    A[3] *= np.float32(1e20); A[4] *= np.float32(1e-30); A[5] = 0.0
    A[6, 17] = 3e7                      # one outlier 10^7 times the rest of its row
    A[7] *= np.exp2(rng.integers(-12, 12, K)).astype(np.float32)   # 2^24 between elements of a row
    Wf[2] *= np.float32(1e-20); Wf[3] *= np.float32(1e15); Wf[4] = 0.0
    Wf[5] *= np.exp2(rng.integers(-14, 14, K)).astype(np.float32)
    Wf[6, 100] = 5e4
    Wb = orc.to_bf16(Wf).reshape(N, K)
    Ww = orc.bf16_widen(Wb).reshape(N, K).astype(np.float64)
    P = Prepared(lib, Wb)
    got = P.product(A).astype(np.float64)
    a64 = A.astype(np.float64)
    with np.errstate(over="ignore", invalid="ignore"):
        want = a64 @ Ww.T
        bound = ((K / 8 + 4) * 2.0 ** -24 * (np.abs(a64) @ np.abs(Ww).T)
                 + 2.0 ** -38 * np.abs(a64).max(axis=1)[:, None] * np.abs(Ww).sum(axis=1)[None, :]
                 + 2.0 ** -39 * np.abs(a64).sum(axis=1)[:, None] * np.abs(Ww).max(axis=1)[None, :])
    ok = np.isfinite(want) & (np.abs(want) < 3e38) & ((np.abs(want) > 1e-37) | (want == 0.0))
    assert np.all(np.isfinite(got[ok]))
    err = np.abs(got - want)
    assert np.all(err[ok] <= bound[ok]), float((err[ok] / (bound[ok] + 1e-300)).max())
    print("   worst error / bound: %.3f" % float((err[ok] / (bound[ok] + 1e-300)).max()), flush=True)
    assert np.all(got[5] == 0.0) and np.all(got[:, 4] == 0.0)
    # and the plain rows meet the GEMM's tolerance against the oracle
    plain = [0, 1, 2, 100, 259]
    w2 = orc.gemm_bf16_nt(np.ascontiguousarray(A[plain]), Wb)
    cols = np.array([c for c in range(N) if c not in (2, 3, 4, 5, 6)])
    assert allclose(got[plain][:, cols].astype(np.float32), w2[:, cols], RTOL, ATOL)
    P.free()


@pytest.mark.parametrize("M,N,K,room", [
    (512, 3584, 3584, 16),    # o-proj of the 7B shape
    (512, 3584, 18944, 16),   # down
    (512, 3584, 3584, 2),     # the caller's buffer holds 2 parts: the split stops there
    (512, 3584, 3584, 1),     # room for the product only: one part
    (200, 896, 4864, 16),     # 0.5B down, ragged M
    (257, 130, 64, 16),       # N % 4 != 0: never split
])
def test_gemm_f16w_parts_feed_the_residual_norm(lib, orc, M, N, K, room):
    """The product left as its K-split parts: they add up to the product the oracle computes, and
    the residual norm that sums them as it reads gives what the plain product followed by the
    residual norm gives (same products; another split, hence summation-order noise)."""
    print("case gemm_f16w parts", M, N, K, room, flush=True)
    A = orc.normal(M * K, 41).reshape(M, K)
    Wb = orc.to_bf16(orc.normal(N * K, 42, std=0.02)).reshape(N, K)
    res = orc.normal(M * N, 43).reshape(M, N)
    nw = orc.normal(N, 44) + 1.0
    P = Prepared(lib, Wb)
    da, dres, dnw = (lib.to_device(a) for a in (A, res, nw))
    dc, x1, h1, x2, h2 = (lib.empty((M, N)) for _ in range(5))
    parts = lib.empty((room, M, N))
    lib.gemm_f16w_nt(da, P.image, P.exps, dc, M, N, K)
    lib.rmsnorm_res(dc, dres, dnw, x1, h1, N, 1e-6, M)
    n = lib.gemm_f16w_nt_parts(da, P.image, P.exps, parts, M, N, K)
    assert 1 <= n <= room
    if room == 16 and N % 4 == 0:
        assert n > 1          # these shapes do split: the test is not vacuous
    if N % 4 != 0:
        assert n == 1
    lib.rmsnorm_res_parts(dres, parts, n, dnw, x2, h2, N, 1e-6, M)
    assert allclose(x2.numpy(), x1.numpy(), RTOL, ATOL)
    assert allclose(h2.numpy(), h1.numpy(), RTOL, 2 * ATOL)
    p = parts.numpy()[:n].astype(np.float64).sum(axis=0)
    want = orc.gemm_bf16_nt(A[:8], Wb)
    assert allclose(p[:8].astype(np.float32), want, RTOL, ATOL)
    for b in (da, dres, dnw, dc, x1, h1, x2, h2, parts):
        b.free()
    P.free()


@pytest.mark.parametrize("M,ff,K", [
    (512, 18944, 3584),    # 7B chunk: 256 whole-round tiles + 40 split over K
    (512, 4864, 896),      # 0.5B chunk
    (200, 1000, 256),      # ragged in M and in the last tile's features
    (65, 130, 64),         # ff % 4 != 0: never split
])
def test_gemm_f16w_swiglu_epilogue(lib, orc, M, ff, K):
    """act = swiglu(A . Wg^T, A . Wu^T) from the prepared [gate rows | up rows] weight: sampled rows
    against the oracle's product and gate, with the GEMM's tolerance on each product carried
    through the gate."""
    print("case gemm_f16w swiglu", M, ff, K, flush=True)
    A = orc.normal(M * K, 51).reshape(M, K)
    Wb = orc.to_bf16(orc.normal(2 * ff * K, 52, std=0.05)).reshape(2 * ff, K)
    P = Prepared(lib, Wb, gated=True)
    got = P.product(A)
    rows = [0, M // 2, M - 1]
    p = orc.gemm_bf16_nt(np.ascontiguousarray(A[rows]), Wb)
    want = orc.swiglu_fused(np.ascontiguousarray(p), ff)
    g, u = p[:, :ff].astype(np.float64), p[:, ff:].astype(np.float64)
    dg, du = RTOL * np.abs(g) + ATOL, RTOL * np.abs(u) + ATOL
    tol = 1.1 * np.abs(u) * dg + np.abs(g / (1.0 + np.exp(-g))) * du + ATOL
    assert np.all(np.isfinite(got))
    assert np.all(np.abs(got[rows].astype(np.float64) - want) <= tol), maxrel(got[rows], want)
    P.free()


def test_gemm_f16w_swiglu_exact_cases(lib, orc):
    """A gate product large enough that sigmoid rounds to 1 gives act = g * up exactly; with a
    one-hot A row both products are weight entries, so every (row, feature) pair must land where its
    gate AND its up row say - a feature gated with another feature's up value, or stored under
    another feature's index, fails. 300 features: three 128-feature tile columns, the last ragged."""
    M, ff, K = 140, 300, 64
    rng = np.random.default_rng(9)
    Wg = rng.integers(20, 40, (ff, K)).astype(np.float32)           # sigmoid(g >= 20) == 1 in f32
    Wu = rng.integers(-64, 64, (ff, K)).astype(np.float32)
    A = np.zeros((M, K), np.float32)
    A[np.arange(M), np.arange(M) % K] = 1.0
    P = Prepared(lib, orc.to_bf16(np.concatenate([Wg, Wu])).reshape(2 * ff, K), gated=True)
    got = P.product(A)
    cols = np.arange(M) % K
    assert np.array_equal(got, (Wg[:, cols] * Wu[:, cols]).T)
    P.free()


def test_gemm_f16w_agrees_with_the_plain_entries(lib, orc):
    """The same products as tlhip_gemm_bf16_nt / _swiglu on the bf16 rows, to fp32 summation order."""
    M, N, K = 384, 2048, 1024
    A = orc.normal(M * K, 61).reshape(M, K)
    Wb = orc.to_bf16(orc.normal(N * K, 62, std=0.02)).reshape(N, K)
    P = Prepared(lib, Wb)
    da, dc = lib.to_device(A), lib.empty((M, N))
    lib.gemm_bf16_nt(da, P.w, dc, M, N, K)
    assert allclose(P.product(A), dc.numpy(), RTOL, ATOL)
    G = Prepared(lib, Wb, gated=True)
    act = lib.empty((M, N // 2))
    lib.gemm_bf16_nt_swiglu(da, G.w, act, M, N // 2, K)
    assert maxrel(G.product(A), act.numpy()) < 1e-4
    for b in (da, dc, act):
        b.free()
    P.free(); G.free()


def test_gemm_f16w_declines(lib):
    """K must be whole slabs of 32 and at most 32768; nulls and misaligned operands are refused;
    the library stays usable."""
    a, w, c = lib.empty((8, 40)), lib.empty_bytes(64 * 40 * 2), lib.empty((8, 64))
    img, ex = lib.empty_bytes(1 << 16), lib.empty_bytes(64)
    assert lib.c.tlhip_gemm_f16w_bytes(64, 40, 0) == 0
    assert lib.c.tlhip_gemm_f16w_bytes(64, 64, 0) == 2 * 16384          # one column tile, two slabs
    assert lib.c.tlhip_gemm_f16w_bytes(130, 64, 1) == 2 * 2 * 16384     # gated: 128 features per tile
    assert lib.c.tlhip_gemm_f16w_prepare(w.ptr, 64, 40, 0, img.ptr, ex.ptr) == -3
    assert lib.c.tlhip_gemm_f16w_prepare(None, 64, 64, 0, img.ptr, ex.ptr) == -2
    assert lib.c.tlhip_gemm_f16w_nt(a.ptr, img.ptr, ex.ptr, c.ptr, 8, 64, 40) == -3
    assert lib.c.tlhip_gemm_f16w_nt(a.ptr, img.ptr, ex.ptr, c.ptr, 8, 64, 32800) == -3
    assert lib.c.tlhip_gemm_f16w_nt(a.ptr, None, ex.ptr, c.ptr, 8, 64, 64) == -2
    assert lib.c.tlhip_gemm_f16w_nt(a.ptr + 4, img.ptr, ex.ptr, c.ptr, 8, 64, 64) == -2
    import ctypes as C
    n = C.c_int(7)
    assert lib.c.tlhip_gemm_f16w_nt_parts(a.ptr, img.ptr, ex.ptr, c.ptr, 4, 8, 64, 64, C.byref(n)) == -2   # no room for one part
    assert lib.c.tlhip_gemm_f16w_nt_parts(a.ptr, img.ptr, ex.ptr, c.ptr, c.nbytes, 8, 64, 64, None) == -2
    lib.last_error()
    for b in (a, w, c, img, ex):
        b.free()
