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


def _same_as_fp32_chain(got, want, A=None, Ww=None):
    """allclose(1e-4, 1e-5) against the oracle's fp32 chain where that is finite; the same infinity
    or a NaN where it is not. Two fp32 evaluations of a sum whose terms cancel can differ by more than
    rtol of the (small) result without either being wrong: with the operands given (A f32, Ww the
    widened weight), an element outside allclose passes only if it is within twice the oracle's own
    distance from the float64 product - no worse an evaluation than the reference's chain, which is
    itself off by more than the tolerance there. Returns (ok, worst element in tolerances, elements
    judged against float64 that way)."""
    fin = np.isfinite(want)
    with np.errstate(over="ignore", invalid="ignore"):
        units = np.where(fin, np.abs(got.astype(np.float64) - want) / (ATOL + RTOL * np.abs(want.astype(np.float64))), 0.0)
    units = np.nan_to_num(units, nan=np.inf)
    out = fin & (units > 1.0)
    by_bound = 0
    if out.any() and A is not None:
        a64, w64 = A.astype(np.float64), Ww.astype(np.float64)
        with np.errstate(over="ignore", invalid="ignore"):
            truth = a64 @ w64.T
        with np.errstate(over="ignore", invalid="ignore"):
            excused = out & (np.abs(got - truth) <= 2.0 * np.abs(want - truth))
        by_bound = int(excused.sum())
        out = out & ~excused
    same_inf = np.array_equal(np.isnan(want), np.isnan(got)) and np.array_equal(want[np.isinf(want)], got[np.isinf(want)])
    return (not out.any()) and same_inf, float(units.max()) if units.size else 0.0, by_bound


def test_gemm_f16w_wide_ranges(lib, orc):
    """Rows whose magnitudes are far apart, in A and between the rows of W: EVERY row against the
    oracle's fp32 product at allclose(1e-4, 1e-5), the adversarial ones included. The scaling is per
    row, so a row of 1e-30 or 1e+20 is as accurate as a row of ones. Inside a row, an activation more
    than 2^24 below the row's largest is carried with an absolute error only; rows 6, 8 and 9 are
    built so that this would show - an outlier 10^7 to 10^8 above the rest that meets zero or tiny
    weights, so that the results are made of the small elements alone - and the kernel has to notice
    and work those results out with the reference's fp32 chain. Rows with an infinity or a NaN come
    out as the reference's chain leaves them (+-inf, NaN where inf meets a zero weight)."""
    M, N, K = 260, 516, 512
    rng = np.random.default_rng(31)
    A = rng.standard_normal((M, K)).astype(np.float32)
    Wf = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    A[3] *= np.float32(1e20); A[4] *= np.float32(1e-30); A[5] = 0.0
    A[6, 17] = 3e7                      # one outlier 10^7 times the rest of its row
    A[7] *= np.exp2(rng.integers(-12, 12, K)).astype(np.float32)   # 2^24 between elements of a row
    A[8, 5] = 1e8                       # an outlier that meets only zero weights (column 5 of W below)
    A[9, 5] = -4e9; A[9] *= np.float32(1e-3)
    A[10, 3] = np.inf
    A[11, 7] = np.nan
    A[12, 3] = np.inf; A[12, 9] = -np.inf
    Wf[2] *= np.float32(1e-20); Wf[3] *= np.float32(1e15); Wf[4] = 0.0
    Wf[5] *= np.exp2(rng.integers(-6, 6, K)).astype(np.float32)
    Wf[6, 100] = 5e4
    Wf[:, 5] = 0.0
    Wf[7:40, 17] *= np.float32(1e-6)    # the outlier of row 6 meets tiny weights in these columns
    Wb = orc.to_bf16(Wf).reshape(N, K)
    Ww = orc.bf16_widen(Wb).reshape(N, K)
    P = Prepared(lib, Wb)
    got = P.product(A)
    with np.errstate(over="ignore", invalid="ignore"):
        want = orc.gemm_bf16_nt(A, Wb)
    for r in range(14):
        ok, worst, nb = _same_as_fp32_chain(got[r:r + 1], want[r:r + 1], A[r:r + 1], Ww)
        print("   row %2d: worst %.3f tolerances, %d elements judged against float64%s"
              % (r, worst, nb, "" if np.all(np.isfinite(want[r])) else "  (not finite in the reference)"), flush=True)
        assert ok, (r, worst)
    ok, worst, nb = _same_as_fp32_chain(got, want, A, Ww)
    assert ok and nb <= 8, (worst, nb)
    assert np.all(got[5] == 0.0) and np.all(got[:13, 4][np.isfinite(want[:13, 4])] == 0.0)
    # the same rows through the gated product and through K-split parts
    P.free()


def test_gemm_f16w_wide_ranges_under_a_k_split_and_gated(lib, orc):
    """The same kind of rows where the product is split over K (each part works out its own K range
    exactly) and through the gated epilogue."""
    M, ff, K = 130, 256, 1024
    rng = np.random.default_rng(33)
    A = rng.standard_normal((M, K)).astype(np.float32)
    A[2, 700] = 2e8
    A[3, 5] = np.inf
    Wf = (rng.standard_normal((2 * ff, K)) * 0.02).astype(np.float32)
    Wf[:, 700] = 0.0
    Wb = orc.to_bf16(Wf).reshape(2 * ff, K)
    with np.errstate(over="ignore", invalid="ignore"):
        both = orc.gemm_bf16_nt(A, Wb)
    Pp = Prepared(lib, Wb)                         # plain: [M, 2 ff], few tiles -> K split
    got = Pp.product(A)
    ok, worst, nb = _same_as_fp32_chain(got, both, A, orc.bf16_widen(Wb).reshape(2 * ff, K))
    assert ok and nb <= 4, (worst, nb)
    Pp.free()
    Pg = Prepared(lib, Wb, gated=True)
    got = Pg.product(A)
    with np.errstate(over="ignore", invalid="ignore"):
        want = orc.swiglu(np.ascontiguousarray(both[:, :ff]), np.ascontiguousarray(both[:, ff:]))
    fin = np.isfinite(want)
    assert np.all(np.abs(got[fin] - want[fin]) <= 2e-5 + 2e-4 * np.abs(want[fin])), "gated rows"
    assert np.array_equal(np.isnan(got[3]), np.isnan(want[3]))
    Pg.free()


def test_gemm_f16w_weights_the_image_cannot_hold(lib, orc):
    """Weight rows whose nonzero elements span more than 2^31, or that hold an infinity: the f16 image
    is not exact there, the preparation counts such elements per row, and the products work out from
    W itself the results in which that could show. Here it does show: row 3 of A is a single huge
    activation at the k of a tiny weight, so the results of that row ARE those tiny weights."""
    M, N, K = 70, 96, 128
    rng = np.random.default_rng(35)
    A = rng.standard_normal((M, K)).astype(np.float32)
    Wf = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    Wf[3] *= np.float32(1e-25); Wf[4] *= np.float32(1e20)       # rows may differ by any factor
    Wf[7, 11] = 1e-12                  # 2^-34 of its row's largest
    Wf[8, 11] = -3e-13
    Wf[9, 1] = np.inf
    A[3] = 0.0; A[3, 11] = 2e9         # picks out column 11 of W
    A[5, 11] = 1e7
    Wb = orc.to_bf16(Wf).reshape(N, K)
    P = Prepared(lib, Wb)
    got = P.product(A)
    with np.errstate(over="ignore", invalid="ignore"):
        want = orc.gemm_bf16_nt(A, Wb)
    ok, worst, nb = _same_as_fp32_chain(got, want, A, orc.bf16_widen(Wb).reshape(N, K))
    assert ok and nb == 0, (worst, nb)
    assert want[3, 7] != 0.0 and abs(got[3, 7] - want[3, 7]) <= 1e-4 * abs(want[3, 7])     # 2e9 * 1e-12, from W itself
    assert np.all(np.isinf(got[:, 9]) | np.isnan(got[:, 9]))
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
    img, ex = lib.empty_bytes(1 << 16), lib.empty_bytes(lib.c.tlhip_gemm_f16w_exps_bytes(64, 0))
    assert lib.c.tlhip_gemm_f16w_exps_bytes(64, 0) == 3 * 64 + 16 and lib.c.tlhip_gemm_f16w_exps_bytes(70, 1) == 3 * 144 + 16
    assert lib.c.tlhip_gemm_f16w_bytes(64, 32800, 0) == 0 and lib.c.tlhip_gemm_f16w_bytes(64, 32768 + 32, 0) == 0   # deeper than the products go
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


@pytest.mark.parametrize("rows,n,S", [(512, 3584, 4), (300, 896, 3), (77, 8192, 1), (512, 4096, 2), (1, 64, 1)])
def test_norm_leaves_the_activation_image(lib, orc, rows, n, S):
    """tlhip_rmsnorm_res_parts_aimage: the residual norm of a prompt chunk that writes the activation
    image of its own output. xout and hout are the bits of tlhip_rmsnorm_res_parts, and the three
    products over that image are the bits of the products that cut the activations themselves -
    plain, K-split parts and gated - on ordinary rows and on rows with tiny elements under a large
    one, a zero row and a row with an infinity (the image's small-element marks decide which
    results the GEMM works out again)."""
    print("case norm aimage", rows, n, S, flush=True)
    x = orc.normal(rows * n, 201).reshape(rows, n)
    parts = orc.normal(S * rows * n, 202, std=0.3).reshape(S, rows, n)
    w = orc.normal(n, 203, 1.0, 0.1)
    if rows > 8:
        x[3, :] = 0.0
        parts[:, 3, :] = 0.0                      # a zero row
        x[5, ::7] *= 1e-9                         # elements far below their row's largest
        x[5, 1] = 3e4
        parts[:, 5, :] = 0.0
        x[6, 2] = np.inf                          # a row that is not finite
    dx, dp, dw = lib.to_device(x), lib.to_device(parts), lib.to_device(w)
    xo1, h1, xo2, h2 = (lib.empty((rows, n)) for _ in range(4))
    nb = lib.gemm_f16w_aimage_bytes(rows, n)
    assert nb > 0
    aimg = lib.empty_bytes(nb)
    lib.rmsnorm_res_parts(dx, dp, S, dw, xo1, h1, n, 1e-6, rows)
    lib.rmsnorm_res_parts_aimage(dx, dp, S, dw, xo2, h2, n, 1e-6, rows, aimg)
    assert np.array_equal(xo1.numpy(), xo2.numpy(), equal_nan=True)
    H1, H2 = h1.numpy(), h2.numpy()
    assert np.array_equal(H1, H2, equal_nan=True)
    # the products over the image against the products that make their own
    N, ff = 384, 256
    Wb = orc.to_bf16(orc.normal(N * n, 204, std=0.02)).reshape(N, n)
    Wg = orc.to_bf16(orc.normal(2 * ff * n, 205, std=0.02)).reshape(2 * ff, n)
    P, G = Prepared(lib, Wb), Prepared(lib, Wg, gated=True)
    c1, c2 = lib.empty((rows, N)), lib.empty((rows, N))
    lib.gemm_f16w_nt(h1, P.image, P.exps, c1, rows, N, n)
    lib.gemm_f16w_nt_aimage(h2, aimg, P.image, P.exps, c2, rows, N, n)
    assert np.array_equal(c1.numpy(), c2.numpy(), equal_nan=True)
    a1, a2 = lib.empty((rows, ff)), lib.empty((rows, ff))
    lib.gemm_f16w_nt_swiglu(h1, G.image, G.exps, a1, rows, ff, n)
    lib.gemm_f16w_nt_swiglu_aimage(h2, aimg, G.image, G.exps, a2, rows, ff, n)
    assert np.array_equal(a1.numpy(), a2.numpy(), equal_nan=True)
    p1, p2 = lib.empty((8, rows, N)), lib.empty((8, rows, N))
    s1 = lib.gemm_f16w_nt_parts(h1, P.image, P.exps, p1, rows, N, n)
    s2 = lib.gemm_f16w_nt_parts_aimage(h2, aimg, P.image, P.exps, p2, rows, N, n)
    assert s1 == s2 and np.array_equal(p1.numpy()[:s1], p2.numpy()[:s2], equal_nan=True)
    # and against the oracle on the finite rows
    fin = np.all(np.isfinite(H1), axis=1)
    want = orc.gemm_bf16_nt(np.ascontiguousarray(H1[fin]), Wb)
    got = c2.numpy()[fin]
    ok, worst, _ = _same_as_fp32_chain(got, want, H1[fin], orc.bf16_widen(Wb).reshape(N, n))
    assert ok, (worst, maxrel(got, want))
    for b in (dx, dp, dw, xo1, h1, xo2, h2, aimg, c1, c2, a1, a2, p1, p2):
        b.free()
    P.free(); G.free()


def test_norm_aimage_declines(lib):
    """Shapes without an image: n not a multiple of 32, n beyond the register-resident norm."""
    assert lib.gemm_f16w_aimage_bytes(512, 100) == 0
    assert lib.gemm_f16w_aimage_bytes(512, 65536) == 0
    x, p, w, o, h = (lib.empty((4, 16384)) for _ in range(5))
    a = lib.empty_bytes(lib.gemm_f16w_aimage_bytes(4, 16384))
    with pytest.raises(Exception):
        lib.rmsnorm_res_parts_aimage(x, p, 1, w, o, h, 16384, 1e-6, 4, a)
    for b in (x, p, w, o, h, a):
        b.free()
