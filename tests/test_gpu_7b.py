"""GPU parity at the Qwen2.5-7B dimensions of BASELINE config 5, through the chained harness
(tl::qwen over tl::hip), not kernel by kernel: a decode step at position 4095 of a 2-layer
model with the full 152064-row LM head, and one layer's 512-token prompt chunk at position 0
and deep in a context, against the CPU oracle on the same weight bytes and the same seeded
cache rows.

The reference checks these with logits maxrel < 2e-3 and identical greedy ids for a decode loop
(check_llm_decode.cpp:268-276; ids may differ only where the top-2 logits are within
rtol 1e-4 / atol 1e-5), maxrel < 2e-4 for one decoder block (check_llm_block.cpp:94-98, 242);
the bars asserted here are tighter (below) and the share of elements inside allclose(rtol 1e-4,
atol 1e-5) is asserted beside them."""
import importlib

import numpy as np
import pytest

from oraclelib import QWEN_7B, check_logits

pytestmark = pytest.mark.gpu

# Bars: max |d| / (1 + |ref|) at under five times what these tests measure on the MI355X (3.8e-5
# for the step two tokens past position 4095; the reference's own bars for the same checks are
# 2e-3 and 2e-4), and the least fraction of elements that must sit inside allclose(rtol 1e-4,
# atol 1e-5) of the oracle. Random-init logits are a few hundredths in size, so it is the atol that
# binds: the fp32 chains of the two sides differ by up to 4e-5 on them (98.9 % inside, the worst
# element 3.1 tolerances out). The chunk's final-norm rows divide a residual of size ~0.03 by its
# rms, which magnifies the two sides' 1e-6 differences thirty times: 4.6e-5 measured, 5.2e-5 on the
# logits of the step that follows the chunk (97.5 % inside).
STEP_BAR, STEP_FRAC = 1.5e-4, 0.97
CHUNK_BAR, CHUNK_FRAC = 2e-4, 0.95


def _near_tie(logits, rtol=1e-4, atol=1e-5):
    top2 = np.sort(logits)[-2:]
    return (top2[1] - top2[0]) <= atol + rtol * abs(top2[1])


def _seed_caches(orc, om, g, upto, seed):
    """Rows [0, upto) of every layer's K and V: N(0,1), the same on both sides."""
    d = om.d
    for l in range(d.n_layers):
        K, V = om.cache(l)
        n = d.n_kv_heads * upto * d.head_dim
        K[:, :upto, :] = orc.normal(n, seed + 2 * l).reshape(d.n_kv_heads, upto, d.head_dim)
        V[:, :upto, :] = orc.normal(n, seed + 2 * l + 1).reshape(d.n_kv_heads, upto, d.head_dim)
        g.cache_upload(l, K, V, upto)


def test_decode_step_at_7b_dims_deep_in_a_context(orc):
    """2 layers of the 7B shape (hidden 3584, 28/4 heads of 128, MLP 18944, vocab 152064, int4
    weights, f32 caches of 4352 rows pre-filled with seeded N(0,1) up to row 4095). One step at
    position 4095 in every form of the step - all fused, q/k/v epilogue apart, swiglu in the
    down GEMV, one launch per reference op - then the recorded graph with the position on the
    device for two more tokens and the on-device greedy loop for three, the oracle stepping the
    same tokens. This is the launch plan the benchmark times: fused [q|k|v] rows 4608, gate|up rows
    37888, K = 18944 down projection, capacity-planned split attention at kv_max 4352."""
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    dims = dict(QWEN_7B, n_layers=2)
    print("building the 2-layer 7B-shape oracle model", flush=True)
    om = orc.qwen_create(dims, seed=5, q4=True)
    g = qwen.QwenGPU.from_blobs(om)
    pos = 4095
    _seed_caches(orc, om, g, pos, 700)
    tok = 4321
    want_tok, want_logits = om.step(tok, pos)
    modes = {"fused": (True, True, True), "fused_attn_apart": (True, False, True),
             "fused_swiglu_in_down": (True, True, False), "plain": (False, True, True)}
    for name, (fused, fattn, gu) in modes.items():
        print("case 7B step", name, flush=True)
        g.set_fused(fused); g.set_fused_attn(fattn); g.set_gateup_epilogue(gu)
        got_tok, got_logits = g.step(tok, pos, want_logits=True)      # rewrites cache row 4095 identically
        check_logits(got_logits, want_logits, STEP_BAR, "logits " + name, STEP_FRAC)
        assert got_tok == want_tok or _near_tie(want_logits), (name, got_tok, want_tok)
    g.set_fused(True); g.set_fused_attn(True); g.set_gateup_epilogue(True)
    # one recorded graph, position on the device: positions 4095 (again), 4096, 4097
    print("case 7B step recorded graph", flush=True)
    assert g.decoder_init(tok, pos), "graph capture unavailable"
    feed = tok
    for p in range(pos, pos + 3):
        if p > pos:
            want_tok, want_logits = om.step(feed, p)
        got_tok, got_logits = g.decoder_step(feed, want_logits=True)
        check_logits(got_logits, want_logits, STEP_BAR, "logits pos %d" % p, STEP_FRAC)
        assert got_tok == want_tok or _near_tie(want_logits), (p, got_tok, want_tok)
        feed = want_tok
    g.decoder_sync_host_pos()
    # token loop on the device from position 4098
    print("case 7B greedy loop on the device", flush=True)
    start, n = pos + 3, 3
    g.greedy_init(feed, start)
    assert g.greedy_run(n) == n
    got = g.greedy_tokens(start, n)
    for i in range(n):
        want_tok, want_logits = om.step(feed, start + i)
        assert int(got[i]) == want_tok or _near_tie(want_logits), (i, int(got[i]), want_tok)
        feed = int(got[i])
    c = g.census()
    assert c["gemv_q4"] > 0 and c["attn_decode"] > 0
    g.close(); om.close()


def _lin_f32(orc, om, layer, name):
    """A linear weight of the oracle model widened to f32 [K,N], as its CPU dot would see it."""
    K, N = om.lin_shape(name)
    raw = om.weight(layer, name)
    if om.q4:
        return orc.q4_to_f32(np.ascontiguousarray(raw), K, N)
    return orc.bf16_widen(np.ascontiguousarray(raw).view(np.uint16)).reshape(K, N)


def _oracle_chunk_rows(orc, om, tokens, pos0, rows):
    """Final-norm output of a one-layer model for the chunk rows `rows`, built from the oracle's
    ops in the order of the reference's forward (bench/cuda/qwen_model.h:559-599): projections of
    the whole chunk (every row's k and v enter the cache), attention / o-proj / MLP for the
    sampled rows only. Leaves the chunk's keys and values in the oracle model's cache."""
    d = om.d
    T, E, Hq, Hkv, D = len(tokens), d.hidden, d.n_q_heads, d.n_kv_heads, d.head_dim
    emb = om.weight(-1, "embed").view(np.uint16).reshape(d.vocab, E)
    X = orc.bf16_widen(np.ascontiguousarray(emb[tokens]))
    vec = lambda n: om.weight(0, n).copy()
    H = orc.rmsnorm(X, vec("an"), d.eps)
    q = orc.sgemm(H, _lin_f32(orc, om, 0, "wq")) + vec("bq")
    k = orc.sgemm(H, _lin_f32(orc, om, 0, "wk")) + vec("bk")
    v = orc.sgemm(H, _lin_f32(orc, om, 0, "wv")) + vec("bv")
    heads = lambda a, h: np.ascontiguousarray(a.reshape(T, h, D).transpose(1, 0, 2))
    qh = orc.rope(heads(q, Hq), pos0, d.rope_base, T=T)
    kh = orc.rope(heads(k, Hkv), pos0, d.rope_base, T=T)
    Kc, Vc = om.cache(0)
    Kc[:, pos0:pos0 + T, :] = kh
    Vc[:, pos0:pos0 + T, :] = heads(v, Hkv)
    scale = float(1.0 / np.sqrt(np.float32(D)))
    A = np.stack([orc.attn_decode(np.ascontiguousarray(qh[:, t, :]), Kc, Vc, scale, ctx=pos0 + t + 1).reshape(Hq * D)
                  for t in rows])
    x1 = X[rows] + orc.sgemm(A, _lin_f32(orc, om, 0, "wo"))
    h2 = orc.rmsnorm(x1, vec("fn"), d.eps)
    gate = orc.sgemm(h2, _lin_f32(orc, om, 0, "wg"))
    up = orc.sgemm(h2, _lin_f32(orc, om, 0, "wu"))
    x2 = x1 + orc.sgemm(orc.swiglu(gate, up), _lin_f32(orc, om, 0, "wd"))
    return orc.rmsnorm(x2, om.weight(-1, "onorm").copy(), d.eps)


@pytest.mark.parametrize("q4", [False, True])
def test_prefill_chunk_at_7b_dims(orc, q4):
    """One layer of the 7B shape, bf16 and int4 weights, a 512-token chunk at position 0 and at
    position 3584 of a seeded cache, in the fused and the one-launch-per-op form: sampled rows of
    the chunk's final-norm output against the oracle chain. Exercises the K-split plan of every
    product at M = 512 (q|k|v 4608, o-proj, gate|up 37888 with the gate as epilogue, down
    K = 18944), the q/k/v epilogue that fills the cache, and causal attention 3584 rows deep."""
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    dims = dict(QWEN_7B, n_layers=1, vocab=1024)      # the lm_head is not part of a chunk's layers
    om = orc.qwen_create(dims, seed=6, q4=q4)
    g = qwen.QwenGPU.from_blobs(om, fmt="q4" if q4 else "bf16")
    rng = np.random.default_rng(11)
    T = 512
    rows = np.array([0, 1, 31, 32, 127, 128, 255, 300, 383, 447, 510, 511])
    for pos0 in (0, 3584):
        tokens = rng.integers(0, dims["vocab"], T)
        Kc, Vc = om.cache(0)
        Kc[:] = 0.0
        Vc[:] = 0.0
        _seed_caches(orc, om, g, pos0, 800 + pos0)
        want = _oracle_chunk_rows(orc, om, tokens, pos0, rows)
        # fused twice for bf16 weights: on their prepared f16 images (the default) and on the bf16 rows
        for fused, f16 in ((True, True), (True, False), (False, True)) if not q4 else ((True, True), (False, True)):
            print("case 7B chunk", "q4" if q4 else "bf16", "pos0", pos0, "fused" if fused else "plain",
                  "f16 images" if f16 else "bf16 rows", flush=True)
            g.set_fused_prefill(fused)
            g.set_prompt_f16(f16)
            g.set_cache_pos(pos0)
            g.prefill(tokens, chunk=T, want_logits=False)
            got = g.prefill_hidden(T)[rows]
            check_logits(got, want, CHUNK_BAR, "final-norm rows", CHUNK_FRAC)
            if fused and f16 and not q4:
                # the residual norms leave the activation images of their outputs (the default) or
                # every product cuts its own: the same bits
                g.set_norm_images(False)
                g.set_cache_pos(pos0)
                g.prefill(tokens, chunk=T, want_logits=False)
                assert np.array_equal(g.prefill_hidden(T)[rows], got)
                g.set_norm_images(True)
        # decode continues on the caches the chunk filled
        tok = int(tokens[-1])
        want_tok, want_logits = om.step(tok, pos0 + T)
        got_tok, got_logits = g.step(tok, pos0 + T, want_logits=True)
        check_logits(got_logits, want_logits, CHUNK_BAR, "logits of the step after the chunk", CHUNK_FRAC)
        assert got_tok == want_tok or _near_tie(want_logits)
    g.close(); om.close()
