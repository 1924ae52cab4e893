"""GPU parity: decode attention through the C ABI vs the CPU oracle."""
import numpy as np
import pytest

from oraclelib import allclose, maxrel

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-4, 1e-5


def _run(lib, q, K, V, ctx, scale, kv_bf16=False):
    Hq, D = q.shape
    Hkv, kv_max, _ = K.shape
    dq, dk, dv, do = lib.to_device(q), lib.to_device(K), lib.to_device(V), lib.empty((Hq, D))
    lib.attn_decode(dq, dk, dv, do, Hq, Hkv, ctx, kv_max, D, scale, kv_bf16)
    out = do.numpy()
    for b in (dq, dk, dv, do):
        b.free()
    return out


@pytest.mark.parametrize("ctx", [512, 2048, 8192, 32768])
def test_attn_config3(lib, orc, ctx):
    """BASELINE config 3: q[28,128], K/V[28,ctx,128] ~ N(0,1), scale 1/sqrt(128)."""
    H, D = 28, 128
    print("case attn config3", ctx, flush=True)
    q = orc.normal(H * D, 1).reshape(H, D)
    K = orc.normal(H * ctx * D, 2).reshape(H, ctx, D)
    V = orc.normal(H * ctx * D, 3).reshape(H, ctx, D)
    scale = 1.0 / np.sqrt(128.0)
    got = _run(lib, q, K, V, ctx, scale)
    want = orc.attn_decode(q, K, V, scale)
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)


@pytest.mark.parametrize("D,Hq,Hkv", [(64, 14, 2), (128, 28, 4), (128, 4, 2), (64, 6, 2),
                                      (128, 3, 1), (64, 16, 1), (128, 5, 5),
                                      (128, 32, 8), (64, 10, 2), (128, 12, 2), (64, 16, 2)])   # groups of 4, 5, 6, 8
@pytest.mark.parametrize("ctx", [1, 2, 63, 64, 65, 127, 128, 129, 255, 256, 257, 1000, 2047])
@pytest.mark.parametrize("kernel", ["built-in", "key-slot"])
def test_attn_gqa_and_split_boundaries(lib, orc, D, Hq, Hkv, ctx, kernel):
    """GQA head map h/group and the split/tile boundaries (check_attn64.cpp:65-66),
    reading a cache prefix: kv_max > ctx, rows past ctx hold garbage that must not leak.
    kernel: the library's choice (groups of 3 to 8 heads over an f32 cache take the kernel that
    stages 64-key tiles in LDS, one wavefront per head) or the key-slot kernel forced for every shape."""
    print("case attn gqa", D, Hq, Hkv, ctx, kernel, flush=True)
    lib.tune_attn_decode(1 if kernel == "key-slot" else 0)
    kv_max = ctx + 37
    q = orc.normal(Hq * D, 4 + ctx).reshape(Hq, D)
    K = orc.normal(Hkv * kv_max * D, 5 + ctx).reshape(Hkv, kv_max, D)
    V = orc.normal(Hkv * kv_max * D, 6 + ctx).reshape(Hkv, kv_max, D)
    K[:, ctx:, :] = 1e30
    V[:, ctx:, :] = np.nan
    scale = 1.0 / np.sqrt(float(D))
    try:
        got = _run(lib, q, K, V, ctx, scale)
    finally:
        lib.tune_attn_decode(0)
    want = orc.attn_decode(q, K, V, scale, ctx=ctx)
    assert np.all(np.isfinite(got))
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)


def test_attn_closed_forms(lib, orc):
    H, D, ctx = 4, 128, 300
    q = orc.normal(H * D, 1).reshape(H, D)
    K = orc.normal(H * ctx * D, 2).reshape(H, ctx, D)
    V = orc.normal(H * ctx * D, 3).reshape(H, ctx, D)
    # ctx == 1 => out == V[:,0]
    got = _run(lib, q, K, V, 1, 0.3)
    assert allclose(got, V[:, 0, :], 1e-6, 1e-6)
    # scale == 0 => uniform weights => mean of V
    got = _run(lib, q, K, V, ctx, 0.0)
    assert allclose(got, V.astype(np.float64).mean(axis=1), 1e-5, 1e-5)
    # identical keys => mean of V as well
    K2 = np.repeat(K[:, :1, :], ctx, axis=1).copy()
    got = _run(lib, q, K2, V, ctx, 0.7)
    assert allclose(got, V.astype(np.float64).mean(axis=1), 1e-5, 1e-5)
    # large scores stay finite ({1000,1001} stability, test_array.cpp:273-274)
    q3 = np.zeros((1, 128), np.float32); q3[0, 0] = 1.0
    K3 = np.zeros((1, 2, 128), np.float32); K3[0, 0, 0] = 1000.0; K3[0, 1, 0] = 1001.0
    V3 = np.zeros((1, 2, 128), np.float32); V3[0, 0, :] = 1.0; V3[0, 1, :] = 3.0
    got = _run(lib, q3, K3, V3, 2, 1.0)
    e = np.exp(-1.0)
    assert allclose(got, np.full((1, 128), (1 * e + 3) / (1 + e)), 1e-5, 1e-5)


@pytest.mark.parametrize("D", [64, 128])
def test_attn_bf16_cache(lib, orc, D):
    Hq, Hkv, ctx = 8, 2, 700
    q = orc.normal(Hq * D, 1).reshape(Hq, D)
    Kb = orc.to_bf16(orc.normal(Hkv * ctx * D, 2).reshape(Hkv, ctx, D))
    Vb = orc.to_bf16(orc.normal(Hkv * ctx * D, 3).reshape(Hkv, ctx, D))
    scale = 1.0 / np.sqrt(float(D))
    got = _run(lib, q, Kb, Vb, ctx, scale, kv_bf16=True)
    want = orc.attn_decode(q, orc.bf16_widen(Kb), orc.bf16_widen(Vb), scale)
    assert allclose(got, want, RTOL, ATOL), maxrel(got, want)


def test_attn_declines(lib, pkg):
    b = lib.empty(4096)
    for args in [(4, 4, 8, 8, 96), (5, 2, 8, 8, 128), (4, 0, 8, 8, 128)]:
        with pytest.raises(pkg.TlHipError) as e:
            lib.attn_decode(b, b, b, b, *args, 1.0)
        assert e.value.code == -3


@pytest.mark.parametrize("D,Hq,Hkv,kv_max", [(128, 28, 4, 4352), (64, 14, 2, 700), (128, 4, 4, 96),
                                             (128, 28, 4, 20000)])
def test_attn_decode_device_position(lib, orc, D, Hq, Hkv, kv_max):
    """Position on the device (cuda.h:1073-1114): the grid is planned once for the cache
    capacity, ctx = *d_pos + 1 is read by the kernel, and splits past the live context
    contribute exact zeros. The same launch must be right at every position."""
    rng = np.random.default_rng(3)
    q = orc.normal(Hq * D, 90).reshape(Hq, D)
    K = orc.normal(Hkv * kv_max * D, 91).reshape(Hkv, kv_max, D)
    V = orc.normal(Hkv * kv_max * D, 92).reshape(Hkv, kv_max, D)
    scale = 1.0 / np.sqrt(float(D))
    dq, dk, dv, do = lib.to_device(q), lib.to_device(K), lib.to_device(V), lib.empty((Hq, D))
    dhost = lib.empty((Hq, D))
    nb = lib.attn_partials_bytes(Hq, Hkv, kv_max, D)
    assert nb > 0
    part = lib.empty_bytes(nb)
    dpos = lib.to_device(np.zeros(1, np.uint32))
    positions = sorted(set([0, 1, 15, 16, 63, 64, 255, 256, 257, kv_max // 2, kv_max - 2, kv_max - 1]))
    for pos in [p for p in positions if 0 <= p < kv_max]:
        print("case attn dpos", D, Hq, Hkv, kv_max, pos, flush=True)
        dpos.upload(np.array([pos], np.uint32))
        do.upload(np.full((Hq, D), np.nan, np.float32))
        lib.attn_decode_dpos(dq, dk, dv, do, Hq, Hkv, dpos, kv_max, D, scale, part)
        got = do.numpy()
        want = orc.attn_decode(q, K, V, scale, ctx=pos + 1)
        assert np.all(np.isfinite(got)), pos
        assert allclose(got, want, RTOL, ATOL), (pos, maxrel(got, want))
        # the host-position call plans its grid for the live context, this one for the capacity:
        # the same bits all the same (check_attn64.cpp:94-103), splits without keys add exact zeros
        lib.attn_decode(dq, dk, dv, dhost, Hq, Hkv, pos + 1, kv_max, D, scale)
        assert np.array_equal(got, dhost.numpy()), pos
    # too small a partials buffer is refused, not overrun
    if nb > 64:
        small = lib.empty_bytes(32)
        with pytest.raises(Exception):
            lib.attn_decode_dpos(dq, dk, dv, do, Hq, Hkv, dpos, kv_max, D, scale, small)
        small.free()
    for b in (dq, dk, dv, do, part, dpos):
        b.free()


def test_attn_full_size_properties(lib, orc):
    """BASELINE config 3 at its largest context (ctx 32768, 0.94 GB of f32 K/V) through
    properties that need no oracle run: constant keys make the output the plain mean of V
    for every head; adding a constant to all scores (a key offset along q) leaves the
    output unchanged; the result does not depend on rows of the cache past ctx."""
    H, D, ctx = 28, 128, 32768
    q = orc.normal(H * D, 1).reshape(H, D)
    V = orc.normal(H * ctx * D, 3).reshape(H, ctx, D)
    K = np.tile(orc.normal(H * D, 2).reshape(H, 1, D), (1, ctx, 1))       # every key of a head identical
    scale = 1.0 / np.sqrt(128.0)
    got = _run(lib, q, K, V, ctx, scale)
    want = V.astype(np.float64).mean(axis=1)
    assert allclose(got, want, 1e-4, 2e-5), maxrel(got, want)
    K2 = orc.normal(H * ctx * D, 4).reshape(H, ctx, D)
    base = _run(lib, q, K2, V, ctx, scale)
    shifted = _run(lib, q, K2 + (q / np.sum(q * q, axis=1, keepdims=True))[:, None, :] * 3.0, V, ctx, scale)
    assert allclose(shifted, base, 2e-4, 2e-5), maxrel(shifted, base)


@pytest.mark.parametrize("kv_bf16", [False, True])
@pytest.mark.parametrize("D,Hq,Hkv,kv_max", [(128, 28, 4, 4352), (64, 14, 2, 700), (128, 4, 4, 96),
                                             (64, 16, 1, 300), (128, 3, 1, 130)])
def test_attn_decode_qkv_fused_prologue(lib, orc, D, Hq, Hkv, kv_max, kv_bf16):
    """Bias + rope + cache append + attention in one launch (the raw [q|k|v] projection goes in)
    against the oracle's rope and attention, and against the two-launch path: the appended cache
    rows are bit-identical, no other cache row changes, the projection is left untouched and the
    output agrees to the attention tolerance. Position on the host and on the device; the last
    case has a full cache (device position == capacity: no row is taken)."""
    base, scale = 1e6, 1.0 / np.sqrt(float(D))
    n = (Hq + 2 * Hkv) * D
    cache_dt = np.uint16 if kv_bf16 else np.float32
    K0 = orc.normal(Hkv * kv_max * D, 501).reshape(Hkv, kv_max, D)
    V0 = orc.normal(Hkv * kv_max * D, 502).reshape(Hkv, kv_max, D)
    if kv_bf16:
        K0, V0 = orc.to_bf16(K0), orc.to_bf16(V0)
    widen = (lambda a: orc.bf16_widen(a)) if kv_bf16 else (lambda a: a)
    bq, bk, bv = orc.normal(Hq * D, 503, 0, 0.5), orc.normal(Hkv * D, 504, 0, 0.5), orc.normal(Hkv * D, 505, 0, 0.5)
    dbq, dbk, dbv = lib.to_device(bq), lib.to_device(bk), lib.to_device(bv)
    tab = lib.empty(D)
    dpos = lib.to_device(np.zeros(1, np.uint32))
    part = lib.empty_bytes(lib.attn_partials_bytes(Hq, Hkv, kv_max, D))
    positions = sorted(set([0, 1, 15, 16, 63, 64, 65, 127, 128, kv_max // 2, kv_max - 2, kv_max - 1]))
    for pos in [p for p in positions if 0 <= p < kv_max]:
        for on_device, with_bias in ((False, True), (True, True), (True, False)):
            print("case attn qkv", D, Hq, Hkv, kv_max, kv_bf16, pos, on_device, with_bias, flush=True)
            qkv = orc.normal(n, 510 + pos)
            b3 = (dbq, dbk, dbv) if with_bias else (None, None, None)
            # two launches
            q1, K1, V1, o1 = lib.to_device(qkv), lib.to_device(K0), lib.to_device(V0), lib.empty((Hq, D))
            lib.rope_table(tab, D, pos, base)
            if with_bias:
                lib.qkv_rope_append_tab(q1, dbq, dbk, dbv, K1, V1, Hq, Hkv, D, pos, kv_max, tab, kv_bf16=kv_bf16)
            else:
                zq, zk, zv = (lib.to_device(np.zeros(m, np.float32)) for m in (Hq * D, Hkv * D, Hkv * D))
                lib.qkv_rope_append_tab(q1, zq, zk, zv, K1, V1, Hq, Hkv, D, pos, kv_max, tab, kv_bf16=kv_bf16)
                for z in (zq, zk, zv):
                    z.free()
            lib.attn_decode(q1, K1, V1, o1, Hq, Hkv, pos + 1, kv_max, D, scale, kv_bf16)
            # one launch
            q2, K2, V2, o2 = lib.to_device(qkv), lib.to_device(K0), lib.to_device(V0), lib.empty((Hq, D))
            o2.upload(np.full((Hq, D), np.nan, np.float32))
            if on_device:
                dpos.upload(np.array([pos], np.uint32))
                lib.rope_table(tab, D, 0, base, d_pos=dpos)
                lib.attn_decode_qkv(q2, *b3, K2, V2, o2, Hq, Hkv, 0, kv_max, D, scale, tab, d_pos=dpos,
                                    partials=part, kv_bf16=kv_bf16)
            else:
                lib.attn_decode_qkv(q2, *b3, K2, V2, o2, Hq, Hkv, pos, kv_max, D, scale, tab, kv_bf16=kv_bf16)
            k1, v1, k2, v2 = K1.numpy(cache_dt), V1.numpy(cache_dt), K2.numpy(cache_dt), V2.numpy(cache_dt)
            assert np.array_equal(k1, k2) and np.array_equal(v1, v2), pos
            assert not np.array_equal(k2[:, pos], K0[:, pos])
            assert np.array_equal(q2.numpy(), qkv)
            got, two = o2.numpy(), o1.numpy()
            assert np.all(np.isfinite(got)), pos
            assert allclose(got, two, RTOL, ATOL), (pos, maxrel(got, two))
            # the oracle on the same cache contents
            zero = np.zeros_like
            qr = orc.rope(qkv[:Hq * D].reshape(Hq, D), pos, base, bias=(bq if with_bias else zero(bq)).reshape(Hq, D))
            want = orc.attn_decode(qr, widen(k2), widen(v2), scale, ctx=pos + 1)
            assert allclose(got, want, RTOL, ATOL), (pos, maxrel(got, want))
            for b in (q1, K1, V1, o1, q2, K2, V2, o2):
                b.free()
    # full cache: the device position has run past the capacity
    qkv = orc.normal(n, 599)
    q2, K2, V2, o2 = lib.to_device(qkv), lib.to_device(K0), lib.to_device(V0), lib.empty((Hq, D))
    dpos.upload(np.array([kv_max], np.uint32))
    lib.rope_table(tab, D, 0, base, d_pos=dpos)
    lib.attn_decode_qkv(q2, dbq, dbk, dbv, K2, V2, o2, Hq, Hkv, 0, kv_max, D, scale, tab, d_pos=dpos,
                        partials=part, kv_bf16=kv_bf16)
    assert np.array_equal(K2.numpy(cache_dt), K0) and np.array_equal(V2.numpy(cache_dt), V0)
    qr = orc.rope(qkv[:Hq * D].reshape(Hq, D), kv_max, base, bias=bq.reshape(Hq, D))
    want = orc.attn_decode(qr, widen(K0), widen(V0), scale, ctx=kv_max)
    assert allclose(o2.numpy(), want, RTOL, ATOL)
    with pytest.raises(Exception):
        lib.attn_decode_qkv(q2, dbq, dbk, dbv, K2, V2, o2, Hq, Hkv, kv_max, kv_max, D, scale, tab, kv_bf16=kv_bf16)
    for b in (q2, K2, V2, o2, dbq, dbk, dbv, tab, dpos, part):
        b.free()


@pytest.mark.parametrize("fmt", ["q4", "bf16"])
@pytest.mark.parametrize("D,Hq,Hkv,kv_max,E", [(64, 14, 2, 1024, 896), (128, 28, 4, 512, 256), (64, 16, 2, 640, 160),
                                               (128, 6, 2, 300, 96)])
def test_attn_splits_merged_by_the_o_projection(lib, orc, fmt, D, Hq, Hkv, kv_max, E):
    """The fused decode attention leaving its split partials (1 to 16 of them) and the o-projection's
    GEMV merging them while it stages its input, against the path with the merge launch: the same
    cache rows and the same projection bit for bit, and both within the tolerance of the oracle's
    attention followed by its GEMV. Position on the host and, where the capacity's plan is served,
    on the device."""
    base, scale = 1e6, 1.0 / np.sqrt(float(D))
    n, QD = (Hq + 2 * Hkv) * D, Hq * D
    K0 = orc.normal(Hkv * kv_max * D, 521).reshape(Hkv, kv_max, D)
    V0 = orc.normal(Hkv * kv_max * D, 522).reshape(Hkv, kv_max, D)
    bq, bk, bv = orc.normal(Hq * D, 523, 0, 0.5), orc.normal(Hkv * D, 524, 0, 0.5), orc.normal(Hkv * D, 525, 0, 0.5)
    dbq, dbk, dbv = lib.to_device(bq), lib.to_device(bk), lib.to_device(bv)
    if fmt == "q4":
        wbuf = orc.to_q4(orc.normal(QD * E, 526, 0.0, 0.05).reshape(QD, E))
        gemv_o = lambda x: orc.gemv_q4(x, wbuf, E, QD)
    else:
        wbuf = orc.to_bf16(orc.normal(E * QD, 527, 0.0, 0.05).reshape(E, QD))
        gemv_o = lambda x: orc.gemv_bf16_row(x, wbuf)
    dw = lib.to_device(wbuf)
    tab, dpos = lib.empty(D), lib.to_device(np.zeros(1, np.uint32))
    part = lib.empty_bytes(lib.attn_partials_bytes(Hq, Hkv, kv_max, D))
    assert lib.attn_parts_splits(Hq, Hkv, kv_max, D, kv_bf16=True) == 0
    seen = set()
    positions = sorted(set([0, 1, 63, 64, 65, 127, 128, 191, 300, kv_max // 2, kv_max - 65, kv_max - 2, kv_max - 1]))
    for pos in [p for p in positions if 0 <= p < kv_max]:
        for on_device in (False, True):
            S = lib.attn_parts_splits(Hq, Hkv, kv_max if on_device else pos + 1, D)
            if S == 0:
                continue
            print("case attn parts", fmt, D, Hq, Hkv, kv_max, pos, on_device, S, flush=True)
            qkv = orc.normal(n, 530 + pos)
            q1, K1, V1, o1, y1 = lib.to_device(qkv), lib.to_device(K0), lib.to_device(V0), lib.empty((Hq, D)), lib.empty(E)
            q2, K2, V2, y2 = lib.to_device(qkv), lib.to_device(K0), lib.to_device(V0), lib.empty(E)
            part.upload(np.full(part.nbytes // 4, np.nan, np.float32).view(np.uint8))
            if on_device:
                dpos.upload(np.array([pos], np.uint32))
                lib.rope_table(tab, D, 0, base, d_pos=dpos)
                lib.attn_decode_qkv(q1, dbq, dbk, dbv, K1, V1, o1, Hq, Hkv, 0, kv_max, D, scale, tab, d_pos=dpos, partials=part)
                got_S = lib.attn_decode_qkv_parts(q2, dbq, dbk, dbv, K2, V2, Hq, Hkv, 0, kv_max, D, scale, tab, part, d_pos=dpos)
            else:
                lib.rope_table(tab, D, pos, base)
                lib.attn_decode_qkv(q1, dbq, dbk, dbv, K1, V1, o1, Hq, Hkv, pos, kv_max, D, scale, tab)
                got_S = lib.attn_decode_qkv_parts(q2, dbq, dbk, dbv, K2, V2, Hq, Hkv, pos, kv_max, D, scale, tab, part)
            assert got_S == S
            seen.add(S)
            if fmt == "q4":
                lib.gemv_q4(o1, dw, y1, E, QD)
                lib.gemv_q4_attn(part, S, Hq, D, dw, y2, E, QD)
            else:
                lib.gemv_bf16_row(o1, dw, y1, E, QD)
                lib.gemv_bf16_row_attn(part, S, Hq, D, dw, y2, E, QD)
            assert np.array_equal(K1.numpy(), K2.numpy()) and np.array_equal(V1.numpy(), V2.numpy()), pos
            two, got = y1.numpy(), y2.numpy()
            assert np.array_equal(two, got), (pos, S, maxrel(got, two))
            qr = orc.rope(qkv[:QD].reshape(Hq, D), pos, base, bias=bq.reshape(Hq, D))
            want = gemv_o(orc.attn_decode(qr, K2.numpy(), V2.numpy(), scale, ctx=pos + 1).reshape(QD))
            assert allclose(got, want, RTOL, ATOL), (pos, S, maxrel(got, want))
            for b in (q1, K1, V1, o1, y1, q2, K2, V2, y2):
                b.free()
    assert len(seen) >= 3, seen          # one split, a few, and the most the shape's plan makes
    # refusals: more parts than the merge sums in order, a K that is not heads x head_dim
    y = lib.empty(E)
    with pytest.raises(Exception):
        (lib.gemv_q4_attn if fmt == "q4" else lib.gemv_bf16_row_attn)(part, 17 if D == 64 else 9, Hq, D, dw, y, E, QD)
    with pytest.raises(Exception):
        (lib.gemv_q4_attn if fmt == "q4" else lib.gemv_bf16_row_attn)(part, 1, Hq - 1, D, dw, y, E, QD)
    for b in (dbq, dbk, dbv, dw, tab, dpos, part, y):
        b.free()


@pytest.mark.parametrize("D,heads,S", [(64, 14, 16), (64, 14, 5), (128, 28, 8), (128, 2, 3), (64, 4, 1)])
def test_gemv_attn_merge_of_made_up_partials(lib, orc, D, heads, S):
    """The merge alone, on partials no attention produced: maxima spread over 60 units (weights down
    to e^-60), splits that held no key (maximum -inf, sum 0, accumulator 0), against the formula
    x[h,d] = sum_s e^(m_s - M) acc_s[d] / sum_s e^(m_s - M) l_s in float64, through an identity-like
    bf16 weight so that y is x itself."""
    rng = np.random.default_rng(D + heads + S)
    m = rng.uniform(-30, 30, (heads, S)).astype(np.float32)
    l = rng.uniform(0.5, 64, (heads, S)).astype(np.float32)
    acc = (rng.standard_normal((heads, S, D)) * l[:, :, None]).astype(np.float32)
    if S > 2:
        dead = rng.integers(1, S, heads)                   # one empty split per head, never split 0
        for h in range(heads):
            m[h, dead[h]], l[h, dead[h]], acc[h, dead[h]] = -np.inf, 0.0, 0.0
    K = heads * D
    w64 = np.exp(m.astype(np.float64) - m.max(axis=1, keepdims=True))
    want = ((w64[:, :, None] * acc).sum(axis=1) / (w64 * l).sum(axis=1)[:, None]).reshape(K).astype(np.float32)
    eye = orc.to_bf16(np.eye(K, dtype=np.float32))
    part = lib.to_device(np.concatenate([m.ravel(), l.ravel(), acc.ravel()]))
    dw, y = lib.to_device(eye), lib.empty(K)
    lib.gemv_bf16_row_attn(part, S, heads, D, dw, y, K, K)
    got = y.numpy()
    assert allclose(got, want, 1e-5, 1e-6), maxrel(got, want)
    for b in (part, dw, y):
        b.free()
