"""GPU parity: rope, rmsnorm, swiglu, argmax, cache writes, elementwise and row
ops through the C ABI vs the CPU oracle."""
import numpy as np
import pytest

from oraclelib import allclose, maxrel

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-4, 1e-5


@pytest.mark.parametrize("rows,T,D,pos,base", [(16, 1, 64, 0, 1e6), (16, 1, 64, 4095, 1e6),
                                               (32, 1, 128, 4096, 1e6), (6, 3, 64, 77, 1e4),
                                               (28 * 16, 16, 128, 32000, 1e6), (2, 1, 2, 5, 1e4)])
def test_rope(lib, orc, rows, T, D, pos, base):
    x = orc.normal(rows * D, 1 + rows).reshape(rows, D)
    dx, do = lib.to_device(x), lib.empty((rows, D))
    lib.rope(dx, do, rows, T, D, pos, base)
    got = do.numpy()
    want = orc.rope(x, pos, base, T=T)
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)
    if pos == 0 and T == 1:
        assert np.array_equal(got, x)          # pos 0 is the identity
    half = D // 2                              # rotations preserve each pair's norm
    n_in = x[:, :half] ** 2 + x[:, half:] ** 2
    n_out = got[:, :half] ** 2 + got[:, half:] ** 2
    assert allclose(n_out, n_in, 1e-5, 1e-6)


def test_rope_bias_and_inplace(lib, orc):
    rows, D, pos = 14, 64, 1234
    x = orc.normal(rows * D, 3).reshape(rows, D)
    b = orc.normal(rows * D, 4, 0, 0.02).reshape(rows, D)
    dx, db = lib.to_device(x), lib.to_device(b)
    lib.rope(dx, dx, rows, 1, D, pos, 1e6, bias=db)
    want = orc.rope(x, pos, 1e6, bias=b)
    assert allclose(dx.numpy(), want, RTOL, ATOL)


@pytest.mark.parametrize("rows,n", [(1, 896), (1, 3584), (5, 3584), (3, 1000), (2, 7), (512, 896)])
def test_rmsnorm(lib, orc, rows, n):
    x = orc.normal(rows * n, 5 + n).reshape(rows, n)
    w = orc.normal(n, 6, 1.0, 0.02)
    dx, dw, do = lib.to_device(x), lib.to_device(w), lib.empty((rows, n))
    lib.rmsnorm(dx, dw, do, n, 1e-6, rows)
    got, want = do.numpy(), orc.rmsnorm(x, w, 1e-6)
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)
    # constant row c => c/sqrt(c^2+eps) * w
    xc = np.full((1, n), 3.0, np.float32)
    dxc = lib.to_device(xc)
    lib.rmsnorm(dxc, dw, do, n, 1e-6, 1)
    assert allclose(do.numpy()[0], 3.0 / np.sqrt(9.0 + 1e-6) * w.astype(np.float64), 1e-6, 1e-6)


@pytest.mark.parametrize("rows,n", [(1, 896), (1, 3584), (4, 1001)])
def test_rmsnorm_res(lib, orc, rows, n):
    x = orc.normal(rows * n, 7).reshape(rows, n)
    d = orc.normal(rows * n, 8).reshape(rows, n)
    w = orc.normal(n, 9, 1.0, 0.02)
    dx, dd, dw, dh = lib.to_device(x), lib.to_device(d), lib.to_device(w), lib.empty((rows, n))
    lib.rmsnorm_res(dx, dd, dw, dx, dh, n, 1e-6, rows)      # xout aliases x
    xo, ho = orc.rmsnorm_res(x, d, w, 1e-6)
    assert np.array_equal(dx.numpy(), xo)
    assert allclose(dh.numpy(), ho, RTOL, ATOL)


@pytest.mark.parametrize("rows,ff", [(1, 4864), (1, 18944), (3, 1000), (2, 1)])
def test_swiglu(lib, orc, rows, ff):
    gu = orc.normal(rows * 2 * ff, 10, 0, 3.0).reshape(rows, 2 * ff)
    dg, do = lib.to_device(gu), lib.empty((rows, ff))
    lib.swiglu(dg, do, ff, rows)
    got, want = do.numpy(), orc.swiglu_fused(gu, ff)
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)
    z = np.zeros((1, 2 * ff), np.float32); z[0, ff:] = 5.0
    dz = lib.to_device(z)
    lib.swiglu(dz, do, ff, 1)
    assert np.all(do.numpy()[0] == 0.0)                      # g = 0 => 0


@pytest.mark.parametrize("n", [1, 5, 256, 4097, 151936, 152064])
def test_argmax(lib, orc, n):
    v = orc.normal(n, 11 + n)
    dv = lib.to_device(v)
    assert lib.argmax(dv, n) == orc.argmax(v)
    v[:] = -3.0                                             # all ties => index 0
    dv.upload(v)
    assert lib.argmax(dv, n) == 0
    if n > 300:
        v[n - 7] = 2.0; v[123] = 2.0; v[299] = 2.0          # ties => smallest index
        dv.upload(v)
        assert lib.argmax(dv, n) == 123 == orc.argmax(v)


def test_kv_append_fill(lib, orc):
    Hkv, D, kv_max = 4, 128, 50
    Kc = np.zeros((Hkv, kv_max, D), np.float32); Vc = Kc.copy()
    dK, dV = lib.to_device(Kc), lib.to_device(Vc)
    for pos in (0, 1, 49):
        k = orc.normal(Hkv * D, 20 + pos).reshape(Hkv, D); v = orc.normal(Hkv * D, 30 + pos).reshape(Hkv, D)
        lib.kv_append(dK, dV, lib.to_device(k), lib.to_device(v), pos, kv_max, Hkv, D)
        Kc[:, pos] = k; Vc[:, pos] = v
    T = 9
    k = orc.normal(Hkv * T * D, 40).reshape(Hkv, T, D); v = orc.normal(Hkv * T * D, 41).reshape(Hkv, T, D)
    lib.kv_fill(dK, dV, lib.to_device(k), lib.to_device(v), T, kv_max, Hkv, D, pos0=10)
    Kc[:, 10:19] = k; Vc[:, 10:19] = v
    assert np.array_equal(dK.numpy(), Kc) and np.array_equal(dV.numpy(), Vc)
    with pytest.raises(RuntimeError):                        # full cache => refused
        lib.kv_append(dK, dV, lib.to_device(k), lib.to_device(v), kv_max, kv_max, Hkv, D)


def test_split_merge_heads(lib, orc):
    T, H, D, ld, off = 7, 6, 64, 6 * 64 + 128, 128
    src = orc.normal(T * ld, 50).reshape(T, ld)
    bias = orc.normal(H * D, 51)
    ds, db, dd = lib.to_device(src), lib.to_device(bias), lib.empty((H, T, D))
    lib.split_heads(ds, db, dd, T, ld, off, H, D)
    want = (src[:, off:off + H * D].reshape(T, H, D) + bias.reshape(1, H, D)).transpose(1, 0, 2)
    assert np.array_equal(dd.numpy(), want)
    dm = lib.empty((T, H * D))
    lib.merge_heads(dd, dm, T, H, D)
    assert np.array_equal(dm.numpy(), want.transpose(1, 0, 2).reshape(T, H * D))


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
@pytest.mark.parametrize("epi", [(1.0, 0.0), (2.0, 1.0)])
def test_binary(lib, orc, op, epi):
    n = 70001
    a = orc.normal(n, 60); b = orc.normal(n, 61) + np.float32(3.0)
    da, db, do = lib.to_device(a), lib.to_device(b), lib.empty(n)
    lib.binary(op, da, db, do, n, *epi)
    want = orc.binary(op, a, b, *epi)
    assert allclose(do.numpy(), want, 1e-6, 1e-7)
    lib.binary(op, da, db, do, n - 5, *epi, ao=8, bo=12, oo=4)     # byte offsets
    assert allclose(do.numpy()[1:n - 4], orc.binary(op, a[2:n - 3], b[3:n - 2], *epi), 1e-6, 1e-7)


@pytest.mark.parametrize("op", ["exp", "log", "sqrt", "sigmoid", "relu", "affine", "recip"])
def test_unary(lib, orc, op):
    n = 5000
    a = np.abs(orc.normal(n, 62)) + np.float32(0.1)
    if op == "relu":
        a = orc.normal(n, 63)
    da, do = lib.to_device(a), lib.empty(n)
    for epi in [(1.0, 0.0), (1.5, -0.25)]:
        lib.unary(op, da, do, n, *epi)
        assert allclose(do.numpy(), orc.unary(op, a, *epi), 2e-6, 1e-6), op


def test_binary_bcast(lib, orc):
    m, n = 5, 896
    x = orc.normal(m * n, 64).reshape(m, n)
    col = orc.normal(m, 65).reshape(m, 1) + np.float32(2.0)
    row = orc.normal(n, 66).reshape(1, n)
    dx, dc, dr, do = lib.to_device(x), lib.to_device(col), lib.to_device(row), lib.empty((m, n))
    lib.binary_bcast("bmul", dx, (n, 1), dc, (1, 0), do, m, n)          # x * inv  (rmsnorm)
    assert np.array_equal(do.numpy(), x * col)
    lib.binary_bcast("badd", dx, (n, 1), dr, (0, 1), do, m, n, 2.0, 1.0)  # + bias row, epilogue
    assert allclose(do.numpy(), orc.binary_bcast("add", x, (n, 1), row, (0, 1), m, n, 2.0, 1.0), 1e-6, 1e-7)
    lib.binary_bcast("bdiv", dx, (n, 1), dc, (1, 0), do, m, n)
    assert allclose(do.numpy(), x / col, 1e-6, 1e-7)


def test_row_ops(lib, orc):
    rows, cols = 9, 1500
    x = orc.normal(rows * cols, 67).reshape(rows, cols)
    dx, dr, ds = lib.to_device(x), lib.empty(rows), lib.empty((rows, cols))
    lib.row_op("row_sum", dx, dr, rows, cols, 1.0 / cols, 1e-6)      # mean + eps, as rmsnorm lowers it
    assert allclose(dr.numpy(), orc.row_sum(x, 1.0 / cols, 1e-6), 1e-5, 1e-6)
    lib.row_op("row_max", dx, dr, rows, cols)
    assert np.array_equal(dr.numpy(), orc.row_max(x))
    lib.row_op("softmax", dx, ds, rows, cols)
    got = ds.numpy()
    assert allclose(got, orc.softmax(x), RTOL, 1e-7)
    assert allclose(got.sum(axis=1), np.ones(rows), 1e-5, 1e-5)


@pytest.mark.parametrize("m,n,k,ta,tb", [(3, 40, 100, 0, 0), (2, 300, 700, 0, 1), (65, 64, 1030, 1, 0),
                                         (1, 17, 33, 1, 1),
                                         # from 128 x 128 outputs on: the fp32 matrix-pipe kernel, all four
                                         # operand forms, whole tiles and ragged edges, K not a slab multiple
                                         (128, 128, 16, 0, 0), (256, 384, 512, 0, 0), (256, 384, 512, 0, 1),
                                         (256, 384, 512, 1, 0), (256, 384, 512, 1, 1), (130, 257, 75, 0, 0),
                                         (130, 257, 75, 0, 1), (131, 258, 77, 1, 0), (129, 129, 17, 1, 1),
                                         (512, 640, 1001, 0, 1), (300, 128, 19, 0, 0)])
def test_gemm_seam(lib, orc, m, n, k, ta, tb):
    A = orc.normal(m * k, 70).reshape(m, k); B = orc.normal(k * n, 71).reshape(k, n)
    As = np.ascontiguousarray(A.T) if ta else A
    Bs = np.ascontiguousarray(B.T) if tb else B
    da, db, do = lib.to_device(As), lib.to_device(Bs), lib.empty((m, n))
    lib.gemm(da, As.shape[1], ta, db, Bs.shape[1], tb, do, m, n, k, 2.0, 1.0)
    want = orc.dot(A, B, 2.0, 1.0)
    assert allclose(do.numpy(), want, RTOL, 1e-4), maxrel(do.numpy(), want)
    lib.gemm(da, As.shape[1], ta, db, Bs.shape[1], tb, do, m, n, k)          # identity epilogue
    assert allclose(do.numpy(), orc.dot(A, B), RTOL, 1e-4)


def test_gemm_seam_exact_and_strided(lib, orc):
    """Integer-valued operands make every partial sum exact, so any summation order gives the same
    bits: the matrix-pipe GEMM must equal the integer product exactly. Then operands that are
    views into larger buffers (row strides larger than the row, byte offsets, unaligned bases)."""
    rng = np.random.default_rng(4)
    m, n, k = 256, 256, 96
    A = rng.integers(-8, 9, (m, k)).astype(np.float32); B = rng.integers(-8, 9, (k, n)).astype(np.float32)
    da, db, do = lib.to_device(A), lib.to_device(B), lib.empty((m, n))
    lib.gemm(da, k, 0, db, n, 0, do, m, n, k)
    assert np.array_equal(do.numpy(), (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32))
    # A = rows 3.. of a [m+5, k+7] buffer starting at column 1 (unaligned, lda = k + 7); B transposed view
    big = orc.normal((m + 5) * (k + 7), 72).reshape(m + 5, k + 7)
    Bt = orc.normal(n * (k + 4), 73).reshape(n, k + 4)
    dbig, dbt = lib.to_device(big), lib.to_device(Bt)
    lib._chk(lib.c.tlhip_gemm(dbig.ptr, (3 * (k + 7) + 1) * 4, k + 7, 0, dbt.ptr, 2 * 4, k + 4, 1, do.ptr, 0, m, n, k, 1.0, 0.0))
    want = orc.dot(np.ascontiguousarray(big[3:3 + m, 1:1 + k]), np.ascontiguousarray(Bt[:, 2:2 + k].T))
    assert allclose(do.numpy(), want, RTOL, 1e-4)


@pytest.mark.parametrize("Hq,Hkv,D", [(14, 2, 64), (28, 4, 128)])
def test_qkv_rope_append_equals_unfused(lib, orc, Hq, Hkv, D):
    """The fused q/k/v epilogue is bit-identical to rope + rope + add + kv_append."""
    kv_max, pos = 40, 17
    n = (Hq + 2 * Hkv) * D
    qkv = orc.normal(n, 80)
    bq, bk, bv = orc.normal(Hq * D, 81, 0, 0.02), orc.normal(Hkv * D, 82, 0, 0.02), orc.normal(Hkv * D, 83, 0, 0.02)
    zeros = np.zeros((Hkv, kv_max, D), np.float32)
    d1, K1, V1 = lib.to_device(qkv), lib.to_device(zeros), lib.to_device(zeros)
    dbq, dbk, dbv = lib.to_device(bq), lib.to_device(bk), lib.to_device(bv)
    lib.qkv_rope_append(d1, dbq, dbk, dbv, K1, V1, Hq, Hkv, D, pos, kv_max, 1e6)
    q = orc.rope(qkv[:Hq * D].reshape(Hq, D), pos, 1e6, bias=bq.reshape(Hq, D))
    k = orc.rope(qkv[Hq * D:(Hq + Hkv) * D].reshape(Hkv, D), pos, 1e6, bias=bk.reshape(Hkv, D))
    v = (qkv[(Hq + Hkv) * D:] + bv).reshape(Hkv, D)
    got = d1.numpy()
    assert allclose(got[:Hq * D], q.ravel(), RTOL, ATOL) and allclose(got[Hq * D:(Hq + Hkv) * D], k.ravel(), RTOL, ATOL)
    assert np.array_equal(got[(Hq + Hkv) * D:], v.ravel())
    Kc, Vc = K1.numpy(), V1.numpy()
    assert np.array_equal(Kc[:, pos], got[Hq * D:(Hq + Hkv) * D].reshape(Hkv, D)) and np.array_equal(Vc[:, pos], v)
    Kc[:, pos] = 0; Vc[:, pos] = 0
    assert not Kc.any() and not Vc.any()
    with pytest.raises(RuntimeError):
        lib.qkv_rope_append(d1, dbq, dbk, dbv, K1, V1, Hq, Hkv, D, kv_max, kv_max, 1e6)


def test_device_position_twins_equal_host_position_calls(lib, orc):
    """rope_dpos / kv_append_dpos / qkv_rope_append_dpos read the position from a device
    scalar and are otherwise the host-position kernels: bit-identical results, and
    incr_u32 advances the scalar (cuda.h:1011-1060)."""
    Hq, Hkv, D, kv_max, base = 6, 2, 64, 50, 1e6
    dpos = lib.to_device(np.array([0], np.uint32))
    for pos in (0, 7, 49):
        dpos.upload(np.array([pos], np.uint32))
        x = orc.normal(Hq * D, 300 + pos).reshape(Hq, D)
        bias = orc.normal(Hq * D, 301).reshape(Hq, D)
        dx, db, o1, o2 = lib.to_device(x), lib.to_device(bias), lib.empty((Hq, D)), lib.empty((Hq, D))
        lib.rope(dx, o1, Hq, 1, D, pos, base, bias=db)
        lib.rope_dpos(dx, o2, Hq, 1, D, dpos, base, bias=db)
        assert np.array_equal(o1.numpy(), o2.numpy())
        k, v = orc.normal(Hkv * D, 302).reshape(Hkv, D), orc.normal(Hkv * D, 303).reshape(Hkv, D)
        dk, dv = lib.to_device(k), lib.to_device(v)
        caches = [lib.to_device(np.zeros((Hkv, kv_max, D), np.float32)) for _ in range(4)]
        lib.kv_append(caches[0], caches[1], dk, dv, pos, kv_max, Hkv, D)
        lib.kv_append_dpos(caches[2], caches[3], dk, dv, dpos, kv_max, Hkv, D)
        assert np.array_equal(caches[0].numpy(), caches[2].numpy())
        assert np.array_equal(caches[1].numpy(), caches[3].numpy())
        assert np.array_equal(caches[0].numpy()[:, pos, :], k)
        qkv = orc.normal((Hq + 2 * Hkv) * D, 304)
        bq, bk, bv = (lib.to_device(orc.normal(n, 305 + i)) for i, n in enumerate((Hq * D, Hkv * D, Hkv * D)))
        q1, q2 = lib.to_device(qkv), lib.to_device(qkv)
        lib.qkv_rope_append(q1, bq, bk, bv, caches[0], caches[1], Hq, Hkv, D, pos, kv_max, base)
        lib.qkv_rope_append_dpos(q2, bq, bk, bv, caches[2], caches[3], Hq, Hkv, D, dpos, kv_max, base)
        assert np.array_equal(q1.numpy(), q2.numpy())
        assert np.array_equal(caches[0].numpy(), caches[2].numpy())
        assert np.array_equal(caches[1].numpy(), caches[3].numpy())
        for b in [dx, db, o1, o2, dk, dv, q1, q2, bq, bk, bv] + caches:
            b.free()
    dpos.upload(np.array([41], np.uint32))
    lib.incr_u32(dpos)
    lib.incr_u32(dpos)
    assert int(dpos.numpy()[0]) == 43
    # a full cache drops the write instead of running past the end
    dpos.upload(np.array([kv_max], np.uint32))
    Kc, Vc = lib.to_device(np.zeros((Hkv, kv_max, D), np.float32)), lib.to_device(np.zeros((Hkv, kv_max, D), np.float32))
    dk = lib.to_device(np.ones((Hkv, D), np.float32))
    lib.kv_append_dpos(Kc, Vc, dk, dk, dpos, kv_max, Hkv, D)
    assert not Kc.numpy().any() and not Vc.numpy().any()
    for b in (dpos, Kc, Vc, dk):
        b.free()


@pytest.mark.parametrize("D", [64, 128])
def test_rope_table_form_is_bit_identical(lib, orc, D):
    """The per-step rotary table (cos, sin formed once, fp64 like array.h:1719-1727) and the fused
    epilogue that reads it give exactly what the table-less epilogue gives, with the position on
    the host or on the device."""
    Hq, Hkv, kv_max, base = 6, 2, 5000, 1e6
    dpos = lib.to_device(np.array([0], np.uint32))
    tab = lib.empty(D)                       # D/2 float2
    for pos in (0, 1, 777, 4095):
        qkv = orc.normal((Hq + 2 * Hkv) * D, 400 + pos)
        bq, bk, bv = (lib.to_device(orc.normal(n, 401 + i)) for i, n in enumerate((Hq * D, Hkv * D, Hkv * D)))
        q1, q2, q3 = lib.to_device(qkv), lib.to_device(qkv), lib.to_device(qkv)
        big = [lib.to_device(np.zeros((Hkv, kv_max, D), np.float32)) for _ in range(6)]
        lib.qkv_rope_append(q1, bq, bk, bv, big[0], big[1], Hq, Hkv, D, pos, kv_max, base)
        lib.rope_table(tab, D, pos, base)
        lib.qkv_rope_append_tab(q2, bq, bk, bv, big[2], big[3], Hq, Hkv, D, pos, kv_max, tab)
        dpos.upload(np.array([pos], np.uint32))
        lib.rope_table(tab, D, 0, base, d_pos=dpos)
        lib.qkv_rope_append_tab(q3, bq, bk, bv, big[4], big[5], Hq, Hkv, D, 0, kv_max, tab, d_pos=dpos)
        a = q1.numpy()
        assert np.array_equal(a, q2.numpy()) and np.array_equal(a, q3.numpy())
        k1, v1 = big[0].numpy(), big[1].numpy()
        assert np.array_equal(k1, big[2].numpy()) and np.array_equal(k1, big[4].numpy())
        assert np.array_equal(v1, big[3].numpy()) and np.array_equal(v1, big[5].numpy())
        assert k1[:, pos, :].any()
        for b in [q1, q2, q3, bq, bk, bv] + big:
            b.free()
    dpos.free(); tab.free()
