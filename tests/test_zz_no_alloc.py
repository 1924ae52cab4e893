"""GPU: tlhip_attn_decode_static, the decode attention entry point that allocates nothing (its
split partials live in a fixed 1 MiB array inside the library), gives the results of
tlhip_attn_decode bit for bit - same kernels, same launch plan - and against the oracle within
the bar of BASELINE (allclose rtol 1e-4 / atol 1e-5). Two calls in a row share the array, the
second on a smaller input; a shape whose partials exceed the array is refused. That the calls
allocate nothing is checked twice: the library's count of allocation and release calls does not
move across them, and they run inside a graph capture, where the library's growable scratch
refuses to grow, with every replay of the graph equal to the eager result."""
import numpy as np
import pytest

from oraclelib import allclose, maxrel

pytestmark = pytest.mark.gpu


def _inputs(orc, Hq, Hkv, ctx, kv_max, D, seed):
    q = orc.normal(Hq * D, seed).reshape(Hq, D)
    K = orc.normal(Hkv * kv_max * D, seed + 1).reshape(Hkv, kv_max, D)
    V = orc.normal(Hkv * kv_max * D, seed + 2).reshape(Hkv, kv_max, D)
    K[:, ctx:, :] = 1e30          # rows past the context must not be read
    V[:, ctx:, :] = np.nan
    return q, K, V


def test_static_entry_equals_attn_decode_on_two_calls_in_a_row(lib, orc):
    """First the 7B decode shape at ctx 4096 (28 query heads over 4 kv heads, 64-way split:
    932 KB of partials), then at once a smaller one (14 over 2 heads of 64, ctx 700), then a
    one-split call that uses no partials; each against tlhip_attn_decode and the oracle."""
    cases = [(28, 4, 4096, 4352, 128, 11), (14, 2, 700, 1024, 64, 21), (4, 4, 40, 64, 128, 31)]
    bufs = []
    for Hq, Hkv, ctx, kv_max, D, seed in cases:
        q, K, V = _inputs(orc, Hq, Hkv, ctx, kv_max, D, seed)
        bufs.append((q, K, V, lib.to_device(q), lib.to_device(K), lib.to_device(V),
                     lib.to_device(np.full((Hq, D), np.nan, np.float32)), lib.empty((Hq, D))))
    lib.sync()
    # the calls under test, back to back on the library's stream
    allocs = lib.alloc_calls()
    for (Hq, Hkv, ctx, kv_max, D, _), (q, K, V, dq, dk, dv, do, _ref) in zip(cases, bufs):
        print("case attn_decode_static", Hq, Hkv, ctx, D, flush=True)
        lib.attn_decode_static(dq, dk, dv, do, Hq, Hkv, ctx, kv_max, D, float(1.0 / np.sqrt(D)))
    lib.sync()
    assert lib.alloc_calls() == allocs, "the static entry point allocated or released memory"
    for (Hq, Hkv, ctx, kv_max, D, _), (q, K, V, dq, dk, dv, do, dref) in zip(cases, bufs):
        scale = float(1.0 / np.sqrt(D))
        lib.attn_decode(dq, dk, dv, dref, Hq, Hkv, ctx, kv_max, D, scale)
        got, ref = do.numpy(), dref.numpy()
        assert np.all(np.isfinite(got))
        assert np.array_equal(got, ref), maxrel(got, ref)
        want = orc.attn_decode(q, K, V, scale, ctx=ctx)
        assert allclose(got, want, 1e-4, 1e-5), maxrel(got, want)
    # the larger shape again after the smaller ones: the array's old contents do not matter
    (Hq, Hkv, ctx, kv_max, D, _), (q, K, V, dq, dk, dv, do, dref) = cases[0], bufs[0]
    do.upload(np.full((Hq, D), np.nan, np.float32))
    lib.attn_decode_static(dq, dk, dv, do, Hq, Hkv, ctx, kv_max, D, float(1.0 / np.sqrt(D)))
    assert np.array_equal(do.numpy(), dref.numpy())
    for b in bufs:
        for d in b[3:]:
            d.free()


def test_static_entry_inside_a_graph_capture(lib, orc):
    """The 7B decode shape recorded into a graph (where growing the library's scratch is refused, so
    a fallback to it would fail the call) and replayed three times with eager work and syncs in
    between: every replay equals the eager call bit for bit, and nothing was allocated."""
    Hq, Hkv, ctx, kv_max, D = 28, 4, 4096, 4352, 128
    q, K, V = _inputs(orc, Hq, Hkv, ctx, kv_max, D, 51)
    dq, dk, dv = lib.to_device(q), lib.to_device(K), lib.to_device(V)
    do, dref = lib.empty((Hq, D)), lib.empty((Hq, D))
    scale = float(1.0 / np.sqrt(D))
    lib.attn_decode_static(dq, dk, dv, dref, Hq, Hkv, ctx, kv_max, D, scale)
    ref = dref.numpy()
    allocs = lib.alloc_calls()
    lib.graph_begin()
    lib.attn_decode_static(dq, dk, dv, do, Hq, Hkv, ctx, kv_max, D, scale)
    g = lib.graph_end()
    assert lib.alloc_calls() == allocs
    nan = np.full((Hq, D), np.nan, np.float32)
    for i in range(3):
        do.upload(nan)                      # eager work and a sync between the replays
        lib.graph_launch(g)
        assert np.array_equal(do.numpy(), ref), i
    lib.graph_destroy(g)
    for d in (dq, dk, dv, do, dref):
        d.free()


def test_static_entry_bf16_cache(lib, orc):
    Hq, Hkv, ctx, kv_max, D = 8, 2, 3000, 3072, 128
    q = orc.normal(Hq * D, 41).reshape(Hq, D)
    Kb = orc.to_bf16(orc.normal(Hkv * kv_max * D, 42)).reshape(Hkv, kv_max, D)
    Vb = orc.to_bf16(orc.normal(Hkv * kv_max * D, 43)).reshape(Hkv, kv_max, D)
    dq, dk, dv, do, dref = (lib.to_device(q), lib.to_device(Kb), lib.to_device(Vb), lib.empty((Hq, D)),
                            lib.empty((Hq, D)))
    scale = float(1.0 / np.sqrt(D))
    lib.attn_decode_static(dq, dk, dv, do, Hq, Hkv, ctx, kv_max, D, scale, kv_bf16=True)
    lib.attn_decode(dq, dk, dv, dref, Hq, Hkv, ctx, kv_max, D, scale, kv_bf16=True)
    assert np.array_equal(do.numpy(), dref.numpy())
    want = orc.attn_decode(q, orc.bf16_widen(Kb), orc.bf16_widen(Vb), scale, ctx=ctx)
    assert allclose(do.numpy(), want, 1e-4, 1e-5)
    for d in (dq, dk, dv, do, dref):
        d.free()


def test_static_entry_refuses_what_does_not_fit(lib, pkg):
    """64 query heads over 8 kv heads at ctx 32768 splits 32 ways: 2048 x 130 floats of partials,
    1.06 MB, more than the 1 MiB array. The call is refused before anything is launched (the
    growable-scratch entry point serves that shape); bad arguments are refused as in
    tlhip_attn_decode."""
    Hq, Hkv, ctx, D = 64, 8, 32768, 128
    dq, do = lib.empty((Hq, D)), lib.empty((Hq, D))
    dk, dv = lib.empty((Hkv, ctx, D)), lib.empty((Hkv, ctx, D))
    with pytest.raises(pkg.TlHipError) as e:
        lib.attn_decode_static(dq, dk, dv, do, Hq, Hkv, ctx, ctx, D, 0.1)
    assert e.value.code == -3 and "fixed buffer" in str(e.value)
    with pytest.raises(pkg.TlHipError) as e:
        lib.attn_decode_static(dq, dk, dv, do, Hq, Hkv, 64, ctx, 96, 0.1)       # head_dim 96
    assert e.value.code == -3
    with pytest.raises(pkg.TlHipError) as e:
        lib.attn_decode_static(dq, dk, dv, do, Hq, Hkv, ctx + 1, ctx, D, 0.1)   # ctx > kv_max
    assert e.value.code == -2
    lib.attn_decode(dq, dk, dv, do, Hq, Hkv, ctx, ctx, D, 0.1)                   # the allocating entry takes it
    lib.sync()
    for d in (dq, dk, dv, do):
        d.free()
