"""GPU parity: decode GEMVs through the C ABI vs the CPU oracle.

Bar (BASELINE.json): allclose(rtol=1e-4, atol=1e-5) against the reference CPU
path with fp32 accumulation — |gpu - ref| <= 1e-5 + 1e-4*|ref|, the reference's
own allclose (array.h:2538-2547).
"""
import numpy as np
import pytest

from oraclelib import allclose, maxrel

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-4, 1e-5


def _q4_case(lib, orc, N, K, seed, from_weights):
    x = orc.normal(K, seed + 1)
    if from_weights:   # config 2: N(0,0.02) weights quantised with group-32 scales
        w = orc.normal(K * N, seed, 0.0, 0.02).reshape(K, N)
        buf = orc.to_q4(w)
    else:              # config 1: uniform nibbles, scales ~ U(0.005, 0.02)
        buf = orc.fill_q4(N, K, seed)
    want = orc.gemv_q4(x, buf, N, K)
    dx, dw, dy = lib.to_device(x), lib.to_device(buf), lib.empty(N)
    lib.gemv_q4(dx, dw, dy, N, K)
    got = dy.numpy()
    for b in (dx, dw, dy):
        b.free()
    return got, want


@pytest.mark.parametrize("N,K", [(4864, 896), (3584, 3584), (512, 3584), (18944, 3584), (3584, 18944),
                                 (1024, 18944),
                                 (4608, 3584), (4097, 512), (8191, 256)])   # the last three: 17..31 rows per CU
def test_gemv_q4_baseline_shapes(lib, orc, N, K):
    print("case gemv_q4", N, K, flush=True)
    got, want = _q4_case(lib, orc, N, K, 100 + N % 97, from_weights=(K != 896))
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)


@pytest.mark.parametrize("N,K", [(1, 32), (3, 64), (7, 96), (48, 256), (130, 2048 + 32),
                                 (257, 4096), (33, 160), (5, 32768 - 32)])
def test_gemv_q4_ragged(lib, orc, N, K):
    print("case gemv_q4 ragged", N, K, flush=True)
    got, want = _q4_case(lib, orc, N, K, 7 + N + K, from_weights=True)
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)


@pytest.mark.parametrize("lpr", [64, 16])
@pytest.mark.parametrize("rows,kw", [(1, 1), (2, 1), (4, 1), (8, 1), (1, 2), (2, 4), (1, 8), (4, 2)])
def test_gemv_q4_every_launch_shape(lib, orc, rows, kw, lpr):
    """All (rows per wavefront, K-split, lanes per row) variants compute the same product."""
    N, K = 777, 3584
    print("case gemv_q4 tuned", rows, kw, lpr, flush=True)
    lib.tune_gemv_q4(rows, kw, 0, 0, lpr)
    try:
        got, want = _q4_case(lib, orc, N, K, 31, from_weights=True)
    finally:
        lib.tune_gemv_q4(0, 0, 0, 0, 0)
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)


def test_gemv_q4_closed_forms(lib, orc):
    """One-hot weight => y = scale*q*x_k; all q == 1 => y = s*sum(x).

    The kernel evaluates sum((nib-8)*x) as sum(nib*x) - 8*sum(x), so a row of
    q == 0 carries fp32 rounding noise of the size of eps*8*sum|x| instead of an
    exact zero; the bound is BASELINE's atol."""
    N, K = 8, 256
    buf = np.zeros(orc.q4_bytes(N, K), np.uint8)
    buf[:N * K // 2] = 0x88                      # every nibble 8 => q = 0
    sc = buf[N * K // 2:].view(np.float32)
    sc[:] = 0.5
    # row 2: k=37 (odd => high nibble of byte 18) gets q=+3 ; row 5: k=200 (even) gets q=-8
    buf[2 * (K // 2) + 18] = (8 + 3) << 4 | 8
    buf[5 * (K // 2) + 100] = 0x80 | 0
    x = orc.normal(K, 5)
    dx, dw, dy = lib.to_device(x), lib.to_device(buf), lib.empty(N)
    lib.gemv_q4(dx, dw, dy, N, K)
    y = dy.numpy()
    want = np.zeros(N, np.float32)
    want[2] = np.float32(0.5) * np.float32(3.0) * x[37]
    want[5] = np.float32(0.5) * np.float32(-8.0) * x[200]
    assert allclose(y, want, 1e-5, 1e-5), (y, want)
    buf[:N * K // 2] = 0x99                      # every q = 1
    sc[:] = 0.25
    dw.upload(buf)
    lib.gemv_q4(dx, dw, dy, N, K)
    y = dy.numpy()
    s = np.float32(0.25 * float(np.sum(x.astype(np.float64))))
    assert allclose(y, np.full(N, s), 1e-5, 1e-5), (y, s)


@pytest.mark.parametrize("group", [8, 16, 64, 128])
def test_gemv_q4_other_groups(lib, orc, group):
    """group != 32 is legal at the C ABI (cuda.h:889-890); checked against an fp64
    dequant-dot like bench_q4_gemv.cpp:98-104."""
    N, K = 19, 512
    rng = np.random.default_rng(group)
    packed = rng.integers(0, 256, N * K // 2, dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, (N, K // group)).astype(np.float32)
    x = orc.normal(K, 3)
    nib = np.empty((N, K), np.int32)
    pk = packed.reshape(N, K // 2)
    nib[:, 0::2] = pk & 0xF
    nib[:, 1::2] = pk >> 4
    deq = (nib - 8).astype(np.float64) * np.repeat(scales.astype(np.float64), group, axis=1)
    want = deq @ x.astype(np.float64)
    buf = np.concatenate([packed, scales.view(np.uint8).ravel()])
    dx, dw, dy = lib.to_device(x), lib.to_device(buf), lib.empty(N)
    lib.gemv_q4(dx, dw, dy, N, K, group=group)
    assert allclose(dy.numpy(), want, RTOL, ATOL)


def test_gemv_q4_declines(lib, pkg):
    a, w, y = lib.empty(64), lib.empty_bytes(4096), lib.empty(8)
    for N, K, g in [(8, 48, 32), (8, 64, 12), (8, 64, 0)]:
        with pytest.raises(pkg.TlHipError) as e:
            lib.gemv_q4(a, w, y, N, K, group=g)
        assert e.value.code == -3   # TLHIP_EUNSUPPORTED => the backend header declines


@pytest.mark.parametrize("N,K", [(3584, 3584), (512, 3584), (18944, 3584), (3584, 18944), (4864, 896),
                                 (40, 64), (1000, 520),
                                 (9, 8), (151936 // 8, 896), (4608, 3584), (7001, 1024)])
def test_gemv_bf16_row(lib, orc, N, K):
    print("case gemv_bf16_row", N, K, flush=True)
    w = orc.to_bf16(orc.normal(N * K, 11 + N, 0.0, 0.02).reshape(N, K))
    x = orc.normal(K, 12)
    want = orc.gemv_bf16_row(x, w)
    dx, dw, dy = lib.to_device(x), lib.to_device(w), lib.empty(N)
    lib.gemv_bf16_row(dx, dw, dy, N, K)
    got = dy.numpy()
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)


@pytest.mark.parametrize("N,K", [(3584, 3584), (512, 3584), (18944, 3584), (3584, 18944), (4864, 896),
                                 (48, 256), (1001, 300),
                                 (8, 5), (18944, 1024)])
def test_gemv_bf16_and_f32_kn(lib, orc, N, K):
    print("case gemv [K,N]", N, K, flush=True)
    wf = orc.normal(K * N, 21 + N, 0.0, 0.02).reshape(K, N)
    wb = orc.to_bf16(wf)
    x = orc.normal(K, 22)
    dx, dy = lib.to_device(x), lib.empty(N)
    dwb = lib.to_device(wb)
    lib.gemv_bf16(dx, dwb, dy, N, K)
    got = dy.numpy()
    want = orc.gemv_bf16(x, wb)
    assert allclose(got, want, RTOL, ATOL), ("bf16", maxrel(got, want))
    dwf = lib.to_device(wf)
    lib.gemv_f32(dx, dwf, dy, N, K)
    got = dy.numpy()
    want = orc.dot(x.reshape(1, K), wf).ravel()
    assert allclose(got, want, RTOL, ATOL), ("f32", maxrel(got, want))


def test_gemv_is_deterministic(lib, orc):
    N, K = 3584, 3584
    buf = orc.fill_q4(N, K, 9)
    x = orc.normal(K, 10)
    dx, dw, dy = lib.to_device(x), lib.to_device(buf), lib.empty(N)
    lib.gemv_q4(dx, dw, dy, N, K)
    first = dy.numpy().copy()
    for _ in range(3):
        lib.gemv_q4(dx, dw, dy, N, K)
        assert np.array_equal(dy.numpy(), first)


def test_census_counts_launches(lib, orc):
    lib.census_reset()
    N, K = 64, 64
    dx, dw, dy = lib.to_device(orc.normal(K, 1)), lib.to_device(orc.fill_q4(N, K, 2)), lib.empty(N)
    lib.gemv_q4(dx, dw, dy, N, K)
    lib.gemv_q4(dx, dw, dy, N, K)
    assert lib.census()["gemv_q4"] == 2


# ---- GEMVs that evaluate the producer of their activation vector ---------------------------

@pytest.mark.parametrize("fmt", ["q4", "bf16"])
@pytest.mark.parametrize("N,K", [(896, 4864), (3584, 18944), (40, 64), (777, 2048 + 32)])
def test_gemv_swiglu_fused(lib, orc, fmt, N, K):
    """y = W . swiglu(gu) in one launch equals swiglu (array.h:2435-2439) followed by the GEMV,
    both taken from the oracle."""
    print("case gemv_swiglu", fmt, N, K, flush=True)
    gu = orc.normal(2 * K, 70 + N, 0.0, 1.5)
    x = orc.swiglu_fused(gu, K).reshape(K)
    dgu, dy = lib.to_device(gu), lib.empty(N)
    if fmt == "q4":
        buf = orc.to_q4(orc.normal(K * N, 71, 0.0, 0.02).reshape(K, N))
        want = orc.gemv_q4(x, buf, N, K)
        dw = lib.to_device(buf)
        lib.gemv_q4_swiglu(dgu, dw, dy, N, K)
    else:
        w = orc.to_bf16(orc.normal(N * K, 72, 0.0, 0.02).reshape(N, K))
        want = orc.gemv_bf16_row(x, w)
        dw = lib.to_device(w)
        lib.gemv_bf16_row_swiglu(dgu, dw, dy, N, K)
    got = dy.numpy()
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)
    for b in (dgu, dw, dy):
        b.free()


@pytest.mark.parametrize("fmt", ["q4", "bf16"])
@pytest.mark.parametrize("with_delta,with_xout", [(True, True), (False, True), (True, False), (False, False)])
@pytest.mark.parametrize("N,K", [(4608, 3584), (1152, 896), (33, 160), (152064 // 16, 3584)])
def test_gemv_rmsnorm_fused(lib, orc, fmt, N, K, with_delta, with_xout):
    """s = x (+ delta) -> xout; y = W . rmsnorm(s) in one launch equals the oracle's rmsnorm_res
    (array.h:2429-2433) followed by the GEMV; xout is the exact fp32 sum."""
    print("case gemv_rmsnorm", fmt, N, K, with_delta, with_xout, flush=True)
    eps = 1e-6
    x = orc.normal(K, 80 + N, 0.0, 2.0)
    delta = orc.normal(K, 81, 0.0, 0.5) if with_delta else np.zeros(K, np.float32)
    nw = (1.0 + orc.normal(K, 82, 0.0, 0.1)).astype(np.float32)
    s, h = orc.rmsnorm_res(x.reshape(1, K), delta.reshape(1, K), nw, eps)
    dx, dn, dy = lib.to_device(x), lib.to_device(nw), lib.empty(N)
    dd = lib.to_device(delta) if with_delta else None
    dxo = lib.to_device(np.full(K, np.nan, np.float32)) if with_xout else None
    if fmt == "q4":
        buf = orc.to_q4(orc.normal(K * N, 83, 0.0, 0.02).reshape(K, N))
        want = orc.gemv_q4(h.reshape(K), buf, N, K)
        dw = lib.to_device(buf)
        lib.gemv_q4_rmsnorm(dx, dd, dn, dxo, dw, dy, N, K, eps)
    else:
        w = orc.to_bf16(orc.normal(N * K, 84, 0.0, 0.02).reshape(N, K))
        want = orc.gemv_bf16_row(h.reshape(K), w)
        dw = lib.to_device(w)
        lib.gemv_bf16_row_rmsnorm(dx, dd, dn, dxo, dw, dy, N, K, eps)
    got = dy.numpy()
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)
    if with_xout:
        assert np.array_equal(dxo.numpy(), s.reshape(K))
    assert np.array_equal(dx.numpy(), x)          # inputs untouched
    for b in (dx, dn, dy, dw, dd, dxo):
        if b is not None:
            b.free()


@pytest.mark.parametrize("fmt", ["q4", "bf16"])
@pytest.mark.parametrize("FF,K,with_delta", [(18944, 3584, True), (4864, 896, True), (4864, 896, False),
                                             (33, 160, True), (7, 64, False), (1000, 18944, True),
                                             (256 * 3, 3584, False)])
def test_gemv_rmsnorm_gateup_epilogue(lib, orc, fmt, FF, K, with_delta):
    """W = [gate rows | up rows]; act = swiglu(gate . n, up . n), n = rmsnorm(x + delta): the one
    launch equals the oracle's rmsnorm_res, GEMV and swiglu (array.h:2429-2439) in sequence, and
    the library's own two-launch form (GEMV, then tlhip_swiglu); xout is the exact fp32 sum.
    Shapes: the 7B and 0.5B gate|up, ragged ones (odd FF, one tile), a long-K one whose launch
    shape splits K over wavefronts, and a few rows per CU."""
    print("case gemv_rmsnorm_gateup", fmt, FF, K, with_delta, flush=True)
    eps, N2 = 1e-6, 2 * FF
    x = orc.normal(K, 90 + FF, 0.0, 2.0)
    delta = orc.normal(K, 91, 0.0, 0.5) if with_delta else np.zeros(K, np.float32)
    nw = (1.0 + orc.normal(K, 92, 0.0, 0.1)).astype(np.float32)
    s, h = orc.rmsnorm_res(x.reshape(1, K), delta.reshape(1, K), nw, eps)
    dx, dn = lib.to_device(x), lib.to_device(nw)
    dd = lib.to_device(delta) if with_delta else None
    dxo = lib.to_device(np.full(K, np.nan, np.float32))
    dact = lib.to_device(np.full(FF, np.nan, np.float32))
    dgu, dact2 = lib.empty(N2), lib.empty(FF)
    # weights with a spread that puts gate values on both sides of zero
    if fmt == "q4":
        buf = orc.to_q4(orc.normal(K * N2, 93, 0.0, 0.05).reshape(K, N2))
        gu = orc.gemv_q4(h.reshape(K), buf, N2, K)
        dw = lib.to_device(buf)
        lib.gemv_q4_rmsnorm_gateup(dx, dd, dn, dxo, dw, dact, N2, K, eps)
        lib.gemv_q4_rmsnorm(dx, dd, dn, None, dw, dgu, N2, K, eps)
    else:
        w = orc.to_bf16(orc.normal(N2 * K, 94, 0.0, 0.05).reshape(N2, K))
        gu = orc.gemv_bf16_row(h.reshape(K), w)
        dw = lib.to_device(w)
        lib.gemv_bf16_row_rmsnorm_gateup(dx, dd, dn, dxo, dw, dact, N2, K, eps)
        lib.gemv_bf16_row_rmsnorm(dx, dd, dn, None, dw, dgu, N2, K, eps)
    lib.swiglu(dgu, dact2, FF)
    want = orc.swiglu_fused(gu, FF).reshape(FF)
    got, two = dact.numpy(), dact2.numpy()
    assert not np.isnan(got).any()
    # the GEMV bar (|dg| <= ATOL + RTOL |g|, same for u) carried through silu(g) * u, |silu'| <= 1.1
    g, u = np.abs(gu[:FF]), np.abs(gu[FF:])
    tol = ATOL * (1.1 * u + g + 1.0) + 2.1 * RTOL * g * u
    assert np.all(np.abs(got - want) <= tol), maxrel(got, want)
    assert np.all(np.abs(got - two) <= tol), maxrel(got, two)
    assert np.array_equal(dxo.numpy(), s.reshape(K))
    assert np.array_equal(dx.numpy(), x)
    for b in (dx, dn, dw, dd, dxo, dact, dgu, dact2):
        if b is not None:
            b.free()


def test_gemv_fused_rejects_aliasing_and_other_groups(lib, pkg):
    x, n, y, w = lib.empty(64), lib.empty(64), lib.empty(8), lib.empty_bytes(4096)
    with pytest.raises(pkg.TlHipError) as e:
        lib.gemv_q4_rmsnorm(x, None, n, x, w, y, 8, 64, 1e-6)          # xout aliases x
    assert e.value.code == -2
    with pytest.raises(pkg.TlHipError) as e:
        lib.gemv_q4_rmsnorm(x, None, n, None, w, y, 8, 64, 1e-6, group=16)
    assert e.value.code == -3
    with pytest.raises(pkg.TlHipError) as e:
        lib.gemv_q4_swiglu(x, w, y, 8, 32, group=8)
    assert e.value.code == -3
    with pytest.raises(pkg.TlHipError) as e:
        lib.gemv_q4_rmsnorm_gateup(x, None, n, None, w, y, 7, 64, 1e-6)     # odd row count
    assert e.value.code == -2
    with pytest.raises(pkg.TlHipError) as e:
        lib.gemv_q4_rmsnorm_gateup(x, None, n, x, w, y, 8, 64, 1e-6)        # xout aliases x
    assert e.value.code == -2


def test_gemv_q4_full_size_linearity(lib, orc):
    """The LM-head shape of BASELINE config 2 (152064x3584, 340 MB) through size-independent
    properties: y(a + b) = y(a) + y(b), y(2a) = 2 y(a) exactly, y(0) = 0 exactly, and a one-hot
    a picks column k of the dequantised matrix (checked against the stored nibbles and scales
    of a few rows)."""
    N, K = 152064, 3584
    buf = orc.fill_q4(N, K, 5)
    dw = lib.to_device(buf)
    def run(a):
        da, dy = lib.to_device(a.astype(np.float32)), lib.empty(N)
        lib.gemv_q4(da, dw, dy, N, K)
        out = dy.numpy()
        da.free(); dy.free()
        return out
    a, b = orc.normal(K, 6), orc.normal(K, 7)
    ya, yb, yab = run(a), run(b), run(a + b)
    assert allclose(yab, ya + yb, 1e-4, 2e-5), maxrel(yab, ya + yb)
    assert np.array_equal(run(2.0 * a), 2.0 * ya)
    assert not run(np.zeros(K)).any()
    k = 1234
    col = run(np.eye(1, K, k).reshape(K))
    packed = buf[:N * K // 2].reshape(N, K // 2)
    scales = buf[N * K // 2:].view(np.float32).reshape(N, K // 32)
    rows = np.array([0, 1, 77, N // 2, N - 1])
    byte = packed[rows, k // 2]
    nib = (byte >> 4) if (k & 1) else (byte & 15)
    want = scales[rows, k // 32] * (nib.astype(np.float32) - 8.0)
    assert np.allclose(col[rows], want, rtol=1e-6, atol=1e-7)
    dw.free()


# ---- the reference's own results at BASELINE configs 1 and 2 ---------------------------------

def _golden():
    import json
    import os
    g = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    return np.load(os.path.join(g, "gemv.npz")), json.load(open(os.path.join(g, "gemv.json")))


def test_config1_gemv_q4_against_reference_golden(lib, orc):
    """BASELINE config 1 (4864x896, uniform nibbles, scales ~U(0.005,0.02)): the plain entry point
    against what the compiled reference's CPU path returned for the same seeded inputs
    (tests/golden/make_golden.py; inputs regenerated and CRC-checked)."""
    z, meta = _golden()
    m = meta["c1"]
    N, K = m["N"], m["K"]
    buf, x = orc.fill_q4(N, K, m["seed_w"]), orc.normal(K, m["seed_x"])
    assert orc.crc32(buf) == m["crc_w"] and orc.crc32(x) == m["crc_x"], "inputs not regenerated identically"
    dx, dw, dy = lib.to_device(x), lib.to_device(buf), lib.empty(N)
    lib.gemv_q4(dx, dw, dy, N, K)
    got = dy.numpy()
    assert allclose(got, z["c1_y"], RTOL, ATOL), maxrel(got, z["c1_y"])
    for b in (dx, dw, dy):
        b.free()


@pytest.mark.parametrize("i", [0, 1, 2, 3])
def test_config2_gemv_against_reference_golden(lib, orc, i):
    """BASELINE config 2, shapes 3584x3584, 512x3584, 18944x3584, 3584x18944: tlhip_gemv_q4,
    tlhip_gemv_bf16 ([K,N]) and tlhip_gemv_bf16_row ([N,K]) - the plain entry points, in the
    launch shapes the benchmark times - against the golden vectors the compiled reference wrote
    for N(0,0.02) weights quantised by its own to_q4 / to_bf16 (inputs regenerated from the
    seeds, CRC-checked, quantised here by the oracle whose output CRCs equal the reference's)."""
    z, meta = _golden()
    m = meta["c2_%d" % i]
    N, K, st = m["N"], m["K"], m["stride"]
    print("case golden config 2", N, K, flush=True)
    w = orc.normal(K * N, m["seed_w"], 0.0, 0.02).reshape(K, N)
    x = orc.normal(K, m["seed_x"])
    assert orc.crc32(w) == m["crc_w"] and orc.crc32(x) == m["crc_x"], "inputs not regenerated identically"
    q, b = orc.to_q4(w), orc.to_bf16(w)
    assert orc.crc32(q) == m["crc_q4"] and orc.crc32(b) == m["crc_bf16"]
    dx, dy = lib.to_device(x), lib.empty(N)
    dq = lib.to_device(q)
    lib.gemv_q4(dx, dq, dy, N, K)
    got = dy.numpy()[::st]
    assert allclose(got, z["c2_q4_%d" % i], RTOL, ATOL), ("q4", maxrel(got, z["c2_q4_%d" % i]))
    dq.free()
    db = lib.to_device(b)
    lib.gemv_bf16(dx, db, dy, N, K)
    got = dy.numpy()[::st]
    assert allclose(got, z["c2_bf16_%d" % i], RTOL, ATOL), ("bf16 [K,N]", maxrel(got, z["c2_bf16_%d" % i]))
    db.free()
    dr = lib.to_device(np.ascontiguousarray(b.T))          # the same weights as [N,K] rows
    lib.gemv_bf16_row(dx, dr, dy, N, K)
    got = dy.numpy()[::st]
    assert allclose(got, z["c2_bf16_%d" % i], RTOL, ATOL), ("bf16 rows", maxrel(got, z["c2_bf16_%d" % i]))
    for d in (dr, dx, dy):
        d.free()


def test_lm_head_rows_against_oracle(lib, orc):
    """The LM-head shape of BASELINE config 2 (152064x3584) at full size, in the launch shape the
    benchmark times: rows are independent, so every 97th output is compared with the oracle run
    on the gathered sub-matrix (int4 rows, bf16 rows, and columns of the [K,N] bf16 layout)."""
    N, K, st = 152064, 3584, 97
    rng = np.random.default_rng(97)
    x = orc.normal(K, 98)
    dx, dy = lib.to_device(x), lib.empty(N)
    n_sub = len(range(0, N, st))
    # int4: seeded nibbles and scales in the reference's one-buffer layout
    buf = orc.fill_q4(N, K, 99)
    packed = buf[:N * K // 2].reshape(N, K // 2)
    scales = buf[N * K // 2:].reshape(N, K // 32 * 4)
    sub = np.concatenate([packed[::st].ravel(), scales[::st].ravel()])
    want = orc.gemv_q4(x, sub, n_sub, K)
    dw = lib.to_device(buf)
    lib.gemv_q4(dx, dw, dy, N, K)
    got = dy.numpy()[::st]
    assert allclose(got, want, RTOL, ATOL), ("q4", maxrel(got, want))
    dw.free()
    del buf, packed, scales
    # bf16 rows [N,K]
    wr = orc.to_bf16((0.02 * rng.standard_normal((N, K), dtype=np.float32)))
    want = orc.gemv_bf16_row(x, np.ascontiguousarray(wr[::st]))
    dw = lib.to_device(wr)
    lib.gemv_bf16_row(dx, dw, dy, N, K)
    got = dy.numpy()[::st]
    assert allclose(got, want, RTOL, ATOL), ("bf16 rows", maxrel(got, want))
    # the same bytes read as the seam layout [K', N'] = [N, K] would be another matrix; build the
    # [K,N] one by transposing, and compare columns
    wkn = np.ascontiguousarray(wr.T)
    dw.upload(wkn)
    lib.gemv_bf16(dx, dw, dy, N, K)
    got = dy.numpy()[::st]
    want = orc.gemv_bf16(x, np.ascontiguousarray(wkn[:, ::st]))
    assert allclose(got, want, RTOL, ATOL), ("bf16 [K,N]", maxrel(got, want))
    for b in (dw, dx, dy):
        b.free()
