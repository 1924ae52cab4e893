#!/usr/bin/env python3
"""Headline benchmark: int4 decode GEMV on one MI355X (BASELINE.json configs[1]).

One "step" is one pass over the five Qwen2.5-7B-shape int4 GEMVs
(3584x3584, 512x3584, 18944x3584, 3584x18944, 152064x3584; batch 1, group-32
scales), each call reading a different device copy of its weight so that no
call is served by the 256 MB Infinity Cache. `value` is algorithmic weight
bytes (0.625 B/weight, the reference's own accounting, bench_q4_gemv.cpp:121)
per second over the whole pass, inputs resident in HBM.

Extra fields: the roofline of the dominant kernel (the 152064x3584 LM-head
GEMV, timed with HIP events on the library's stream inside the same steps),
the reference CPU path timed on this box's host cores on a bounded sample, and
the Qwen2.5-7B-shape int4 decode step at ctx 4096 (tok/s, hipGraph replay).

  python bench.py --gpus 1 --steps K --warmup W
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

SHAPES = [(3584, 3584), (512, 3584), (18944, 3584), (3584, 18944), (152064, 3584)]  # (N, K)
HBM_PEAK_GBS = 8000.0
RING_BYTES = 1.2e9      # distinct weight bytes per shape, > 4x the Infinity Cache
LMHEAD_HBM_BYTES_PER_LAUNCH = 341_917_491   # (166654.9 KiB * 2.000 + 594.0 KiB) * 1024


def q4_nbytes(N, K):
    return N * K // 2 + N * (K // 32) * 4


def normal(n, seed, mean=0.0, std=1.0):
    return (np.random.default_rng(seed).standard_normal(n, dtype=np.float32) * np.float32(std)
            + np.float32(mean)).astype(np.float32)


def make_q4_host(lib, N, K, seed):
    """Seeded N(0,0.02) weight rows in the int4 group format (what array::to_q4 produces),
    quantised by the library's own load-time converter on the device. A block of rows is
    quantised and tiled along N: kernel time does not depend on the values."""
    rows = min(N, 2048)
    src = lib.to_device(normal(rows * K, seed, 0.0, 0.02))
    q4 = lib.empty_bytes(q4_nbytes(rows, K))
    lib.quantize_q4(src, lib.T_F32, q4, rows, K)
    blk = q4.numpy(np.uint8)
    src.free(); q4.free()
    packed, scales = blk[:rows * K // 2], blk[rows * K // 2:]
    reps = -(-N // rows)
    out = np.empty(q4_nbytes(N, K), np.uint8)
    out[:N * K // 2] = np.tile(packed, reps)[:N * K // 2]
    out[N * K // 2:] = np.tile(scales, reps)[:N * (K // 32) * 4]
    return out


def cpu_baseline(guards, budget_s=25.0):
    """The only leg that touches oracle/. It first checks the GPU result of EVERY sweep shape
    (`guards` = x, q4 buffer, N, K, y from the GPU; rows [::stride] of the big ones, whose rows
    are independent) against the CPU checker, then times the reference CPU path (x.dot(Wq) in
    use_cpu() mode: per-call widening to f32 plus cpu::sgemm on ONE thread, array.h:1980-1984,
    cpu.h:436-438) on the sweep's own shapes, smallest first: median of 3 calls (after a
    warm-up call for the four smaller ones); a shape is skipped once the time budget is spent
    (the sample says which were timed). Then the other ops of a decode step at the 7B shape -
    attn_decode over 28 heads at ctx 4096, rope, rmsnorm, swiglu - are timed the same way and
    summed per layer the way the reference's bench_llm.cpp:167-176 sums per-op times into ms per
    token. Falls back to the plain-C restatement when oracle/_ref was not built."""
    import ctypes as C
    from oraclelib import oracle, ref
    orc = oracle()
    refl = ref()            # None when oracle/_ref was not built
    checked = []
    for (gx, gbuf, gN, gK, got) in guards:
        st = 1 if gN <= 4096 else 97
        packed = gbuf[:gN * gK // 2].reshape(gN, gK // 2)[::st]
        scales = gbuf[gN * gK // 2:].reshape(gN, gK // 32 * 4)[::st]
        sub = np.concatenate([packed.ravel(), scales.ravel()])
        want = orc.gemv_q4(gx, sub, packed.shape[0], gK)
        if not np.all(np.abs(got[::st] - want) <= 1e-5 + 1e-4 * np.abs(want)):
            print("bench.py: GPU result of %dx%d differs from the CPU oracle" % (gN, gK), file=sys.stderr)
            sys.exit(3)
        checked.append("%dx%d%s" % (gN, gK, "" if st == 1 else " rows[::%d]" % st))
    P = C.c_void_p
    ptr = lambda a: a.ctypes.data_as(P)

    def med3(run, warm=True):
        if warm:
            run()
        ts = []
        for _ in range(3):
            t = time.perf_counter()
            run()
            ts.append(time.perf_counter() - t)
        return float(np.median(ts))

    total_bytes, total_s, timed, per_shape_s = 0, 0.0, [], {}
    t_start = time.time()
    for (N, K) in [(4864, 896)] + sorted(SHAPES, key=lambda s: s[0] * s[1]):
        big = N * K > 10 ** 8
        est = 0.62 * N * K / 0.1e9 * (3.3 if big else 4.2)     # ~0.1 GB/s, calls incl. warm-up
        if time.time() - t_start + est > budget_s and timed:
            continue
        buf = orc.fill_q4(N, K, 77)
        x = orc.normal(K, 78)
        y = np.empty(N, np.float32)
        if refl is not None:
            h = refl.lib.tlref_gemv_q4_prepare(ptr(x), ptr(buf), N, K)
            run = lambda: refl.lib.tlref_gemv_run(h, ptr(y))
        else:
            ws = np.empty(K * N, np.float32)
            run = lambda: orc.lib.orc_gemv_q4(ptr(x), ptr(buf), ptr(y), N, K, 1.0, 0.0, ptr(ws))
        sec = med3(run, warm=not big)
        if refl is not None:
            refl.lib.tlref_gemv_free(h)
        if (N, K) not in SHAPES:        # BASELINE configs[0]: reported beside the sweep, not in it
            config0_ms = sec * 1e3
            continue
        total_bytes += q4_nbytes(N, K)
        total_s += sec
        per_shape_s["%dx%d" % (N, K)] = sec
        timed.append("%dx%d" % (N, K))
    out = {
        "value": round(total_bytes / total_s / 1e9, 4), "unit": "GB/s", "cores": 1,
        "kind": "reference" if refl is not None else "port",
        "gpu_result_checked": "allclose(1e-4, 1e-5) at " + ", ".join(checked),
        "sample": "int4 x.dot(Wq) at %s (%d of the 5 sweep shapes; median of 3 calls, after a warm-up "
                  "call except for the LM head); the reference's dot at M=1 runs on one thread whatever the core "
                  "count" % (", ".join(timed), len(timed)),
        "ms": round(total_s * 1e3, 2), "host_cores_online": os.cpu_count(),
        "config0_4864x896_ms": round(config0_ms, 3),
    }
    # ---- the other ops of a 7B-shape decode step at ctx 4096, one thread like the dots
    if len(timed) == len(SHAPES):
        L, E, HQ, HKV, D, FF, ctx = 28, 3584, 28, 4, 128, 18944, 4096
        impl = refl if refl is not None else orc
        q = orc.normal(HQ * D, 81).reshape(HQ, D)
        # the array op has no GQA (array.h:1380-1381: one K/V head per query head)
        Kc = np.tile(orc.normal(HKV * ctx * D, 82).reshape(HKV, 1, ctx, D), (1, HQ // HKV, 1, 1)).reshape(HQ, ctx, D)
        Vc = np.tile(orc.normal(HKV * ctx * D, 83).reshape(HKV, 1, ctx, D), (1, HQ // HKV, 1, 1)).reshape(HQ, ctx, D)
        scale = float(1.0 / np.sqrt(128.0))
        t_attn = med3(lambda: impl.attn_decode(q, Kc, Vc, scale), warm=False)
        qk = orc.normal((HQ + HKV) * D, 84).reshape(HQ + HKV, D)
        t_rope = med3(lambda: impl.rope(qk, 4095, 1e6))
        xr, wn = orc.normal(E, 85).reshape(1, E), orc.normal(E, 86, 1.0, 0.02)
        t_norm = med3(lambda: impl.rmsnorm(xr, wn, 1e-6))
        g_, u_ = orc.normal(FF, 87), orc.normal(FF, 88)
        t_swiglu = med3(lambda: impl.swiglu(g_, u_))
        ps = per_shape_s
        # per layer: wq, wo (3584x3584), wk, wv (512x3584), wg, wu (18944x3584), wd (3584x18944)
        dots = 2 * ps["3584x3584"] + 2 * ps["512x3584"] + 2 * ps["18944x3584"] + ps["3584x18944"]
        layer = dots + t_attn + t_rope + 2 * t_norm + t_swiglu
        token = L * layer + t_norm + ps["152064x3584"]
        out["decode_7b_ctx4096"] = {
            "kind": "summed per-op, measured (bench_llm.cpp:167-176)",
            "ms_per_token": round(token * 1e3, 1), "tok_s": round(1.0 / token, 5),
            "per_layer_ms": {"int4 dots": round(dots * 1e3, 2), "attn_decode 28 heads x ctx 4096": round(t_attn * 1e3, 2),
                             "rope q+k": round(t_rope * 1e3, 4), "rmsnorm x2": round(2 * t_norm * 1e3, 4),
                             "swiglu": round(t_swiglu * 1e3, 4)},
            "lm_head_ms": round(ps["152064x3584"] * 1e3, 1),
            "left_out": "bias adds, residual adds, cache append, embedding gather, argmax (microseconds)"}
    out["cpu_seconds_spent"] = round(time.time() - t_start, 1)
    return out


def decode_guard(lib):
    """One decode step at the 7B layer shape against the CPU oracle before anything is timed: a
    one-layer model with the 7B dimensions (hidden 3584, 28/4 heads of 128, MLP 18944; a small
    vocabulary - the LM-head shape is checked by the sweep's guard) built from the oracle's
    seeded weights, caches of 4352 rows seeded up to row 4095 on both sides, one fused step at
    position 4095 eagerly and one from a recorded graph with the position on the device. Bar:
    logits max |d| / (1 + |ref|) < 1e-4 (a few times what the step measures; the reference's own
    bar for a decode loop is 2e-3, check_llm_decode.cpp:268-276); the share of logits inside
    allclose(rtol 1e-4, atol 1e-5) is reported beside it."""
    from oraclelib import QWEN_7B, maxrel, oracle
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    orc = oracle()
    om = orc.qwen_create(dict(QWEN_7B, n_layers=1, vocab=4096), seed=9, q4=True)
    g = qwen.QwenGPU.from_blobs(om)
    d, pos = om.d, 4095
    Kc, Vc = om.cache(0)
    n = d.n_kv_heads * pos * d.head_dim
    Kc[:, :pos, :] = orc.normal(n, 901).reshape(d.n_kv_heads, pos, d.head_dim)
    Vc[:, :pos, :] = orc.normal(n, 902).reshape(d.n_kv_heads, pos, d.head_dim)
    g.cache_upload(0, Kc, Vc, pos)
    want_tok, want = om.step(1234, pos)
    _, eager = g.step(1234, pos, want_logits=True)
    ok = g.decoder_init(1234, pos)
    _, replay = g.decoder_step(1234, want_logits=True)
    worst = max(maxrel(eager, want), maxrel(replay, want))
    inside = min(float(np.mean(np.abs(r.astype(np.float64) - want) <= 1e-5 + 1e-4 * np.abs(want))) for r in (eager, replay))
    g.close(); om.close()
    if not (worst < 1e-4):
        print("bench.py: 7B-shape decode step differs from the CPU oracle (maxrel %.2e)" % worst, file=sys.stderr)
        sys.exit(3)
    return {"what": "one-layer 7B-dims model, step at position 4095, eager and recorded graph, vs the CPU oracle",
            "logits_maxrel": float("%.3g" % worst), "bar": 1e-4, "logits_inside_allclose_1e-4_1e-5": round(inside, 5),
            "graph_captured": bool(ok)}


def decode_7b(lib, steps, eager=False, warm=None):
    """Qwen2.5-7B-shape int4 decode step at ctx 4096 (BASELINE configs[4], decode half):
    random-init weights, cache rows [0,4095) pre-filled, one step captured as a hipGraph
    at position 4095 and replayed. eager=True launches the same kernels one by one, without
    a graph: the form a kernel trace is taken from."""
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    g = qwen.QwenGPU(dict(qwen.QWEN_7B))
    g.set_random(1)
    ctx = 4096
    g.fill_cache_random(ctx - 1, 2)
    pos = ctx - 1
    if warm:        # (mode, blocks): weight warm-up reads on a second stream beside each layer
        g.set_warm(warm[1], False, warm[0])
    for _ in range(2):
        g.step(11, pos)
    if eager:
        t = time.perf_counter()
        for _ in range(steps):
            g.run_layers(11, pos)
        g.flush()
        ms = (time.perf_counter() - t) / steps * 1e3
        g.close()
        return {"workload": "Qwen2.5-7B-shape int4 decode step, ctx 4096, eager launches",
                "ms_per_token": round(ms, 4), "tok_s": round(1e3 / ms, 1)}
    # where the step's GPU time goes: events between the launches of five eager steps (the role
    # of the reference's StepProf, bench_qwen_decode.cpp:212-237); the events cost a little themselves
    layer_us = {k: round(v, 2) for k, v in g.profile_steps(11, pos, 5).items()}
    # what an event costs: the same eager step without them, timed by two events around five steps
    pe0, pe1 = lib.event(), lib.event()
    lib.record(pe0)
    for _ in range(5):
        g.run_layers(11, pos)
    lib.record(pe1)
    g.flush()
    plain_us = lib.elapsed_ms(pe0, pe1) * 1e3 / 5
    n_events = 5 * g.d.n_layers + 2
    layer_us["event_cost"] = round(max(0.0, (layer_us["step"] - plain_us) / n_events), 2)
    layer_us["step_without_events"] = round(plain_us, 2)
    g.capture(11, pos)
    for _ in range(3):
        g.replay()
    g.flush()
    e0, e1 = lib.event(), lib.event()
    best = None
    for _ in range(3):                      # min of rounds, bench_qwen_decode.cpp:95-116
        lib.record(e0)
        for _ in range(steps):
            g.replay()
        lib.record(e1)
        ms = lib.elapsed_ms(e0, e1) / steps
        best = ms if best is None else min(best, ms)
    # The real loop: ONE graph recorded with the position on the device, replayed for
    # successive tokens ending at position 4095 (ctx 4096); each token stages its embedding
    # row (host gather + 14 KB copy) and, in the greedy form, reads the argmax back.
    n_loop = max(steps, 32)
    start = ctx - 2 * n_loop
    g.set_cache_pos(start - 1)
    captured = g.decoder_init(11, start - 1)
    g.decoder_feed(11)                      # the first launch of a new graph pays its upload
    g.flush()
    t = time.perf_counter()
    for i in range(n_loop):
        g.decoder_feed(11 + i)
    g.flush()
    loop_feed = (time.perf_counter() - t) / n_loop * 1e3
    tok = 11
    t = time.perf_counter()
    for i in range(n_loop):
        tok = g.decoder_step(tok)
    with_argmax = (time.perf_counter() - t) / n_loop * 1e3
    assert g.decoder_pos() == ctx
    # Greedy decoding with the token loop on the device: embedding gather, argmax and the
    # token hand-over are kernels of the recorded step, so n tokens are queued back to back
    # and the ids are read once at the end.
    g.set_cache_pos(start - 1)
    g.greedy_init(11, start - 1)
    g.greedy_run(1)
    g.flush()
    t = time.perf_counter()
    queued = g.greedy_run(2 * n_loop)
    g.flush()                                     # the last token exists
    greedy_dev = (time.perf_counter() - t) / queued * 1e3
    ids = g.greedy_tokens(start, queued)          # one read-back of the whole history
    assert queued == 2 * n_loop and len(ids) == queued
    d = g.d
    wbytes = 0.625 * (d.n_layers * (d.hidden * (d.n_q_heads + 2 * d.n_kv_heads) * d.head_dim
                                    + d.hidden * d.n_q_heads * d.head_dim + 3 * d.hidden * d.ff)
                      + d.vocab * d.hidden)
    kvbytes = d.n_layers * 2 * d.n_kv_heads * ctx * d.head_dim * 4
    g.close()
    return {
        "workload": "Qwen2.5-7B-shape int4 decode step, ctx 4096, f32 KV, hipGraph replay",
        "ms_per_token": round(best, 4), "tok_s": round(1e3 / best, 1),
        "loop": {"what": "one recorded graph, position on the device, %d successive tokens ending at "
                         "ctx 4096, wall clock incl. embedding staging" % n_loop,
                 "graph_captured": bool(captured),
                 "ms_per_token_feed_only": round(loop_feed, 4),
                 "ms_per_token_greedy_with_argmax_readback": round(with_argmax, 4),
                 "tok_s_greedy": round(1e3 / with_argmax, 1),
                 "ms_per_token_greedy_token_loop_on_device": round(greedy_dev, 4),
                 "tok_s_greedy_token_loop_on_device": round(1e3 / greedy_dev, 1)},
        "algorithmic_bytes": int(wbytes + kvbytes),
        "hbm_frac": round((wbytes + kvbytes) / (best * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "layer_us": dict(layer_us, what="eager step with an event between its regions: microseconds per layer, each region including one event's cost (event_cost, from the same step without events) "
                                        "(lm_head, step: per token); attention = q/k/v epilogue + attention + split combine"),
    }


def decode_05b(lib, steps):
    """Qwen2.5-0.5B-shape decode (BASELINE configs[3]'s architecture; the shape the reference's
    published RTX 3090 figures are quoted on, README.md:310-311) through tl/qwen_decode.h's fused
    step: graph replay at a fixed position after a 128-token context, and the greedy loop with
    an argmax read-back per token (one recorded graph, position on the device)."""
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    out = {"workload": "Qwen2.5-0.5B-shape decode after a 128-token context, f32 KV"}
    e0, e1 = lib.event(), lib.event()
    for fmt in ("q4", "bf16"):
        g = qwen.QwenGPU(dict(qwen.QWEN_05B))
        g.set_random(5, fmt=fmt)
        g.fill_cache_random(127, 6)
        for _ in range(2):
            g.step(11, 127)
        g.capture(11, 127)
        for _ in range(3):
            g.replay()
        g.flush()
        best = None
        for _ in range(3):
            lib.record(e0)
            for _ in range(steps):
                g.replay()
            lib.record(e1)
            ms = lib.elapsed_ms(e0, e1) / steps
            best = ms if best is None else min(best, ms)
        n_loop = 64
        g.set_cache_pos(127)
        g.decoder_init(11, 127)
        g.decoder_feed(11)
        g.flush()
        tok = 11
        t = time.perf_counter()
        for _ in range(n_loop):
            tok = g.decoder_step(tok)
        loop = (time.perf_counter() - t) / n_loop * 1e3
        g.close()
        out[fmt] = {"ms_per_token_graph_replay": round(best, 4), "tok_s_graph_replay": round(1e3 / best, 1),
                    "ms_per_token_greedy_with_argmax_readback": round(loop, 4), "tok_s_greedy": round(1e3 / loop, 1)}
    return out


def side_kernels(lib):
    """The other bandwidth-bound kernels of the path at their BASELINE shapes: the bf16 GEMV in
    both layouts (configs[1] weights as bf16; [N,K] rows for the harness, [K,N] at the array
    seam) and decode attention (configs[2]: q[28,128], K/V[28,ctx,128] f32). Bytes counted the
    reference's way: 2*N*K per GEMV (bench_bf16_gemv.cpp:119), 2*H*ctx*D*4 per attention call
    (bench_attn_decode.cpp:129). Buffers rotate so that no call re-reads what the previous one
    left in the caches."""
    rng = np.random.default_rng(7)
    e0, e1 = lib.event(), lib.event()
    out = {"gemv_bf16_row": {}, "gemv_bf16_kn": {}, "attn_decode_f32": {}, "load_convert_f16": {}}

    def timed(calls, n):
        for i in range(min(n, 3)):
            calls(i)
        lib.record(e0)
        for i in range(n):
            calls(i)
        lib.record(e1)
        return lib.elapsed_ms(e0, e1) / n

    for (N, K) in [(3584, 3584), (18944, 3584), (3584, 18944), (152064, 3584)]:
        nb = 2 * N * K
        copies = max(2, int(1.2e9 // nb) + 1)
        w = lib.empty_bytes(nb * copies)
        host = (rng.integers(0, 65536, N * K, dtype=np.uint16) & 0x807f) | 0x3c00
        w.upload(host)
        for c in range(1, copies):
            lib._chk(lib.c.tlhip_memcpy_d2d_async(w.ptr + c * nb, w.ptr, nb))
        x, y = lib.to_device(normal(K, 5)), lib.empty(N)
        for name, fn in (("gemv_bf16_row", lib.c.tlhip_gemv_bf16_row), ("gemv_bf16_kn", lib.c.tlhip_gemv_bf16)):
            ms = timed(lambda i: lib._chk(fn(x.ptr, w.ptr + (i % copies) * nb, y.ptr, N, K)), max(10, copies))
            out[name]["%dx%d" % (N, K)] = {"us": round(ms * 1e3, 2), "GB/s": round(nb / ms / 1e6, 1)}
        for b in (w, x, y):
            b.free()

    # Load-time conversion of a model file's f16 rows (the 7B LM head, 1.09 GB of f16): into the
    # int4 group format and into bf16 rows. GB/s over bytes read + bytes written.
    N, K = 152064, 3584
    src = lib.empty_bytes(2 * N * K)
    host = (rng.integers(0, 65536, 1 << 22, dtype=np.uint16) & 0x83ff) | 0x2000      # |w| ~ 0.01
    for o in range(0, 2 * N * K, host.nbytes):
        lib._chk(lib.c.tlhip_memcpy_h2d(src.ptr + o, host.ctypes.data, min(host.nbytes, 2 * N * K - o)))
    q4, b16 = lib.empty_bytes(N * K // 2 + N * (K // 32) * 4), lib.empty_bytes(2 * N * K)
    ms = timed(lambda i: lib.quantize_q4(src, lib.T_F16, q4, N, K), 5)
    nb = 2 * N * K + q4.nbytes
    out["load_convert_f16"]["to_q4_152064x3584"] = {"us": round(ms * 1e3, 1), "GB/s": round(nb / ms / 1e6, 1)}
    ms = timed(lambda i: lib.convert(src, lib.T_F16, b16, lib.T_BF16, N * K), 5)
    out["load_convert_f16"]["to_bf16_152064x3584"] = {"us": round(ms * 1e3, 1), "GB/s": round(4 * N * K / ms / 1e6, 1)}
    for b in (src, q4, b16):
        b.free()

    H, D = 28, 128
    for ctx in (512, 2048, 8192, 32768):
        per = H * ctx * D
        copies = max(2, min(8, int(1.2e9 // (8 * per)) + 1))
        Ks, Vs = lib.empty(per * copies), lib.empty(per * copies)
        blk = normal(min(per, 1 << 22), 9)
        for b in (Ks, Vs):
            for o in range(0, per * copies, len(blk)):
                n = min(len(blk), per * copies - o)
                lib._chk(lib.c.tlhip_memcpy_h2d(b.ptr + o * 4, blk.ctypes.data, n * 4))
        q, o_ = lib.to_device(normal(H * D, 10)), lib.empty(H * D)
        scale = 1.0 / np.sqrt(128.0)
        ms = timed(lambda i: lib._chk(lib.c.tlhip_attn_decode(
            q.ptr, Ks.ptr + (i % copies) * per * 4, Vs.ptr + (i % copies) * per * 4, o_.ptr,
            H, H, ctx, ctx, D, scale, 0)), 20)
        nb = 2 * per * 4
        out["attn_decode_f32"]["ctx%d" % ctx] = {"us": round(ms * 1e3, 2), "GB/s": round(nb / ms / 1e6, 1)}
        for b in (Ks, Vs, q, o_):
            b.free()
    return out


def prefill_7b(lib, rounds=3):
    """Qwen2.5-7B-shape 512-token prompt chunk with bf16 weights (BASELINE configs[4],
    prefill half): every linear layer is the MFMA GEMM C[512,N] = A[512,K] . W[N,K]^T.
    Flops are counted the reference's way, 2*M*N*K over the four GEMMs of a layer
    (bench_llm.cpp:109); the harness runs them over the prepared f16 form of its weights, two f16
    MFMAs per product (two f16 terms per f32 activation), so the matrix-core rate it sustains is
    twice that."""
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    dims = dict(qwen.QWEN_7B)
    dims["max_ctx"] = 1024
    g = qwen.QwenGPU(dims)
    g.set_random(3, fmt="bf16")
    T = 512
    rng = np.random.default_rng(4)
    g.stage_chunk(rng.integers(0, dims["vocab"], T))
    for _ in range(2):
        g.prefill_layers(T, 0)
    g.flush()
    e0, e1 = lib.event(), lib.event()
    best = None
    for _ in range(rounds):
        lib.record(e0)
        g.prefill_layers(T, 0)
        lib.record(e1)
        ms = lib.elapsed_ms(e0, e1)
        best = ms if best is None else min(best, ms)
    d = g.d
    qkvn = (d.n_q_heads + 2 * d.n_kv_heads) * d.head_dim
    shapes = [(qkvn, d.hidden), (d.hidden, d.n_q_heads * d.head_dim), (2 * d.ff, d.hidden), (d.hidden, d.ff)]
    flops = 2.0 * T * sum(n * k for n, k in shapes) * d.n_layers
    g.close()
    # the same chunk over the decode path's int4 weights (the reference feeds an int4 model its
    # prompt token by token, qwen_model.h:419)
    g = qwen.QwenGPU(dims)
    g.set_random(3, fmt="q4")
    g.stage_chunk(rng.integers(0, dims["vocab"], T))
    for _ in range(2):
        g.prefill_layers(T, 0)
    g.flush()
    best_q4 = None
    for _ in range(rounds):
        lib.record(e0)
        g.prefill_layers(T, 0)
        lib.record(e1)
        ms = lib.elapsed_ms(e0, e1)
        best_q4 = ms if best_q4 is None else min(best_q4, ms)
    g.close()
    # the four GEMMs alone, back to back: over the prepared weight (what the chunk above runs:
    # activation planes + product + part sum where K is split) and over the bf16 rows
    per_gemm, gemm_ms, rows_ms = {}, 0.0, 0.0
    for (N, K) in shapes:
        A = lib.to_device(rng.standard_normal((T, K)).astype(np.float32))
        # random sign and mantissa, exponent pinned so that |w| is in [2^-7, 2^-6)
        W = lib.to_device((rng.integers(0, 65536, (N, K), dtype=np.uint16) & 0x807f) | 0x3c00)
        image, exps = lib.gemm_f16w_prepare(W, N, K)
        C = lib.empty((T, N))
        times = []
        for fn in (lambda: lib.gemm_f16w_nt(A, image, exps, C, T, N, K), lambda: lib.gemm_bf16_nt(A, W, C, T, N, K)):
            for _ in range(2):
                fn()
            lib.record(e0)
            for _ in range(10):
                fn()
            lib.record(e1)
            times.append(lib.elapsed_ms(e0, e1) / 10)
        gemm_ms += times[0]
        rows_ms += times[1]
        per_gemm["%dx%dx%d" % (T, N, K)] = {"us": round(times[0] * 1e3, 1),
                                            "TFLOP/s": round(2.0 * T * N * K / times[0] / 1e9, 1),
                                            "bf16_rows_us": round(times[1] * 1e3, 1)}
        for b in (A, W, C, image, exps):
            b.free()
    gemm_tf = flops / d.n_layers / gemm_ms / 1e9
    rows_tf = flops / d.n_layers / rows_ms / 1e9
    # one layer's causal attention for the chunk at three depths of the context (f32 cache)
    attn = {}
    Hq, Hkv, D = d.n_q_heads, d.n_kv_heads, d.head_dim
    scale = float(1.0 / np.sqrt(D))
    for pos0 in (0, 3584, 7680):
        kv_max = pos0 + T
        K = lib.to_device(rng.standard_normal(Hkv * kv_max * D, dtype=np.float32))
        V = lib.to_device(rng.standard_normal(Hkv * kv_max * D, dtype=np.float32))
        q = lib.to_device(rng.standard_normal(Hq * T * D, dtype=np.float32))
        out = lib.empty(Hq * T * D)
        for _ in range(2):
            lib.attn_prefill(q, K, V, out, Hq, Hkv, T, kv_max, D, scale, pos0=pos0)
        lib.record(e0)
        for _ in range(10):
            lib.attn_prefill(q, K, V, out, Hq, Hkv, T, kv_max, D, scale, pos0=pos0)
        lib.record(e1)
        ms = lib.elapsed_ms(e0, e1) / 10
        fl = 4.0 * Hq * D * (T * pos0 + T * (T + 1) / 2)
        attn["pos0_%d" % pos0] = {"us": round(ms * 1e3, 1), "TFLOP/s": round(fl / ms / 1e9, 1)}
        for b in (K, V, q, out):
            b.free()
    return {
        "workload": "Qwen2.5-7B-shape 512-token prompt chunk at pos0 0, bf16 weights, f32 KV",
        "ms_per_chunk": round(best, 3), "tok_s": round(T / best * 1e3, 1),
        "tflops_chunk": round(flops / best / 1e9, 1),
        "int4_weights": {"ms_per_chunk": round(best_q4, 3), "tok_s": round(T / best_q4 * 1e3, 1)},
        "attention_per_layer": dict(attn, note="causal attention of the 512-token chunk, 28/4 heads of 128, f32 cache; "
                                               "deep in a context: two f16 terms per operand on the matrix cores, three term products per "
                                               "fp32 product (157.3 TFLOP/s is the fp32 matrix-pipe peak)"),
        "gemm": {"per_shape": per_gemm, "TFLOP/s": round(gemm_tf, 1), "bf16_rows_TFLOP/s": round(rows_tf, 1),
                 "roofline": {"bound": "mfma", "achieved": round(2 * gemm_tf, 1), "peak": 2500.0,
                              "unit": "TFLOP/s", "frac": round(2 * gemm_tf / 2500.0, 4),
                              "note": "prepared weight (tlhip_gemm_f16w_nt): f16 MFMA rate issued = 2 x algorithmic "
                                      "(two f16 terms per f32 activation), timed with the activation-plane pass "
                                      "and the K-split part sums; tlhip_gemm_bf16_nt on the bf16 rows issues 3 x "
                                      "(bf16_rows_*); fp32-MFMA peak would be 157.3"}},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-decode", action="store_true", help="skip the 7B-shape decode leg")
    ap.add_argument("--eager-decode", action="store_true",
                    help="decode leg without the hipGraph (for kernel traces)")
    ap.add_argument("--decode-warm", default="", metavar="MODE:BLOCKS",
                    help="decode leg with weight warm-up reads on a second stream beside each layer "
                         "(an experiment that does not pay; off by default). MODE 0: o-proj, gate|up, down "
                         "and the next q|k|v from the layer's start; 3: o-proj and gate|up beside attention. "
                         "BLOCKS < 0: short-lived 32 KB blocks")
    ap.add_argument("--no-side", action="store_true",
                    help="skip the bf16 GEMV and decode attention legs")
    ap.add_argument("--no-prefill", action="store_true", help="skip the 7B-shape prompt-chunk leg")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch the plain 1 GiB copy kernel 3 times (scale for --pmc runs)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU; every GPU box of this run has one. "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    pkg = importlib.import_module("cpp-tensorlib_amd")
    lib = pkg.load()                      # raises when the HIP library or the GPU is missing

    # ---- device-resident inputs: a ring of weight copies per shape -----------------
    def make_ring(N, K, wseed, xseed):
        nb = q4_nbytes(N, K)
        stride = (nb + 255) // 256 * 256
        copies = max(2, int(RING_BYTES // nb) + 1)
        host = make_q4_host(lib, N, K, wseed)
        first = lib.empty_bytes(stride * copies)
        first.upload(host)
        for c in range(1, copies):
            lib._chk(lib.c.tlhip_memcpy_d2d_async(first.ptr + c * stride, first.ptr, nb))
        x = lib.to_device(normal(K, xseed))
        y = lib.empty(N)
        return dict(N=N, K=K, nb=nb, stride=stride, copies=copies, buf=first, x=x, y=y, it=0,
                    host=None if a.no_cpu else host)

    rings = [make_ring(N, K, 100 + si, 200 + si) for si, (N, K) in enumerate(SHAPES)]
    lib.sync()

    # every shape's GPU result (through the last copy of its ring), kept for the CPU leg's check
    guards = []
    if not a.no_cpu:
        for r in rings:
            lib.gemv_q4(r["x"], r["buf"], r["y"], r["N"], r["K"], wq_off=(r["copies"] - 1) * r["stride"])
            guards.append((r["x"].numpy(), r["host"], r["N"], r["K"], r["y"].numpy()))
            r["host"] = None

    def one_step(ev=None):
        for r in rings:
            off = (r["it"] % r["copies"]) * r["stride"]
            r["it"] += 1
            dominant = r["N"] == 152064
            if ev is not None and dominant:
                lib.record(ev[0])
            lib.gemv_q4(r["x"], r["buf"], r["y"], r["N"], r["K"], wq_off=off)
            if ev is not None and dominant:
                lib.record(ev[1])

    for _ in range(a.warmup):
        one_step()
    lib.sync()
    evs = [(lib.event(), lib.event()) for _ in range(a.steps)]
    t0 = time.perf_counter()
    for i in range(a.steps):
        one_step(evs[i])
    lib.sync()
    dt = time.perf_counter() - t0
    ms_per_step = dt / a.steps * 1e3
    step_bytes = sum(r["nb"] for r in rings)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    dom = rings[-1]
    in_step_ms = float(np.mean([lib.elapsed_ms(e0, e1) for (e0, e1) in evs]))

    # per-shape rates (events around R back-to-back launches, rotating copies), and beside each:
    # a kernel that only READS the same bytes of the same rotating copies (the floor any GEMV
    # launch over them has, launch included) and the GEMV over ONE copy read again and again
    # (what it would take if its weights already waited in the last-level cache)
    per_shape = {}
    e0, e1 = lib.event(), lib.event()
    sink = lib.empty(4)

    def median_us(call, n):
        rounds = []
        for _ in range(5):      # median of 5 rounds, the reference's discipline (bench_q4_gemv.cpp:106-119)
            lib.record(e0)
            for i in range(n):
                call(i)
            lib.record(e1)
            rounds.append(lib.elapsed_ms(e0, e1) / n * 1e3)
        return float(np.median(rounds))

    def shape_line(r):
        n = max(10, min(r["copies"], 60))
        off = lambda i: ((r["it"] + i) % r["copies"]) * r["stride"]
        us = median_us(lambda i: lib.gemv_q4(r["x"], r["buf"], r["y"], r["N"], r["K"], wq_off=off(i)), n)
        r["it"] += n
        nb16 = r["nb"] & ~15
        floor = min(median_us(lambda i: lib.bench_read(r["buf"], nb16, sink, blocks, off=off(i)), n)
                    for blocks in (256, 512, 1024))
        line = {"us": round(us, 2), "GB/s": round(r["nb"] / us / 1e3, 1),
                "read_floor_us": round(floor, 2), "frac_of_read": round(floor / us, 3)}
        if r["nb"] <= 100e6:
            line["resident_us"] = round(median_us(lambda i: lib.gemv_q4(r["x"], r["buf"], r["y"], r["N"], r["K"]), n), 2)
        return line

    for r in rings:
        per_shape["%dx%d" % (r["N"], r["K"])] = shape_line(r)
    # BASELINE configs[0], the reference's own CPU-runnable case (bench_q4_gemv.cpp's first shape):
    # a 2.7 MB weight, i.e. a launch and little else; outside `value`, which is configs[1]'s sweep
    r0 = make_ring(4864, 896, 99, 299)
    config0 = shape_line(r0)
    if not a.no_cpu:
        lib.gemv_q4(r0["x"], r0["buf"], r0["y"], r0["N"], r0["K"], wq_off=(r0["copies"] - 1) * r0["stride"])
        guards.append((r0["x"].numpy(), r0["host"], r0["N"], r0["K"], r0["y"].numpy()))
    r0["buf"].free()
    sink.free()
    # dominant kernel: average launch duration over back-to-back launches of the LM-head
    # GEMV (events on the library's stream), the figure rocprofv3 --kernel-trace reports too
    dom_ms = per_shape["152064x3584"]["us"] * 1e-3
    achieved = dom["nb"] / (dom_ms * 1e-3) / 1e9
    if a.copy_probe:
        gib = 1 << 30
        src, dst = lib.empty_bytes(gib), lib.empty_bytes(gib)
        lib._chk(lib.c.tlhip_fill_u32(src.ptr, 0x01020304, gib // 4))
        for _ in range(3):
            lib.bench_copy(dst, src, gib)
        lib.sync()
        src.free(); dst.free()
    for r in rings:
        r["buf"].free()

    out = {
        "metric": "int4_gemv_hbm_gbps", "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "int4 GEMV sweep at Qwen2.5-7B shapes (BASELINE configs[1]): "
                               "3584x3584, 512x3584, 18944x3584, 3584x18944, 152064x3584, batch 1, "
                               "group-32 scales, weights rotated through >1.2 GB of copies per shape",
                   "bytes_per_step": step_bytes, "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
                   "per_shape": per_shape,
                   "config0_4864x896": config0},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "gemv_rows_kernel<FmtQ4,4,0,64,0> on 152064x3584 (LM head)",
                     "bytes_per_launch": dom["nb"], "avg_launch_us": round(dom_ms * 1e3, 2),
                     "avg_us_between_events_inside_step": round(in_step_ms * 1e3, 2)},
    }
    # HBM bytes per LM-head launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled
    # by what the same counter reads for a plain 1 GiB copy kernel (x2.000 and x1.000 here)
    out["roofline"]["traffic"] = LMHEAD_HBM_BYTES_PER_LAUNCH
    out["roofline"]["traffic_source"] = ("profiles/gemv_q4_lmhead_hbm_traffic.md (rocprofv3 --pmc runs of this "
                                         "command; a constant of the kernel, not measured by this run)")
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline(guards)
    if not a.no_decode:
        guard7b = None if a.no_cpu else decode_guard(lib)
        warm = tuple(int(v) for v in a.decode_warm.split(":")) if a.decode_warm else None
        out["decode"] = decode_7b(lib, max(10, a.steps), eager=a.eager_decode, warm=warm)
        if warm:
            out["decode"]["warm"] = {"mode": warm[0], "blocks": warm[1]}
        if guard7b is not None:
            out["decode"]["checked_against_oracle"] = guard7b
        cpu_dec = out.get("cpu_baseline", {}).get("decode_7b_ctx4096")
        if cpu_dec is not None:
            # the reference's CPU kernels on this box's host cores (one thread: its M=1 dot and its
            # attention are single-threaded), per-op times summed into ms per token
            d = out["decode"]
            d["cpu_reference_ms_per_token"] = cpu_dec["ms_per_token"]
            d["cpu_reference_kind"] = cpu_dec["kind"]
            d["speedup_vs_cpu_reference"] = round(cpu_dec["ms_per_token"] / d["ms_per_token"], 1)
        if not a.eager_decode:
            out["decode_05b"] = decode_05b(lib, max(20, a.steps))
    if not a.no_side:
        out["side_kernels"] = side_kernels(lib)
    if not a.no_prefill:
        out["prefill"] = prefill_7b(lib)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
