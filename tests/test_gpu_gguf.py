"""GPU parity for the model-file path: the load-time converters (f16 / f32 / bf16 file rows ->
bf16 rows, [K,N], int4 groups) are bit-exact against the oracle's restatement of the reference's
host loops, and a synthetic Qwen2-architecture GGUF file loaded through tl::qwen::load_gguf
decodes like the oracle model built from the same tensors."""
import importlib

import numpy as np
import pytest

import ggufwriter as W
from oraclelib import check_logits

pytestmark = pytest.mark.gpu

F32, F16, BF16 = 0, 1, 2


def test_f16_widen_exhaustive_on_device(lib, orc):
    """Every half bit pattern (subnormals, infinities, NaN payloads) widens to the oracle's bits."""
    h = np.arange(65536, dtype=np.uint16)
    src, dst = lib.to_device(h), lib.empty(65536)
    lib.convert(src, F16, dst, F32, 65536)
    assert np.array_equal(dst.numpy().view(np.uint32), orc.f16_widen(h).view(np.uint32))
    src.free(); dst.free()


@pytest.mark.parametrize("n", [8, 1, 7, 9, 2048, 2049, 4095, 3584 * 19, 1000003])
@pytest.mark.parametrize("st", [F32, F16, BF16])
def test_convert_to_bf16_and_f32(lib, orc, st, n):
    """dst = narrow(widen(src)) for every source type, bf16 (RNE, types.h:35-41) and f32
    destinations, ragged lengths (the 8-wide body and the scalar tail)."""
    print("case convert", st, n, flush=True)
    rng = np.random.default_rng(n + st)
    if st == F32:
        host = (rng.standard_normal(n) * 10.0 ** rng.integers(-6, 6, n)).astype(np.float32)
        wide = host
    else:
        host = rng.integers(0, 65536, n, dtype=np.uint16)
        if st == F16:
            host[((host >> 10) & 31) == 31] = 0x3c00          # NaN/inf patterns are covered exhaustively above
            wide = orc.f16_widen(host)
        else:
            host[((host >> 7) & 255) == 255] = 0x3f80
            wide = orc.bf16_widen(host)
    src = lib.to_device(host)
    d16, d32 = lib.to_device(np.full(n + 8, 0xdead, np.uint16)), lib.to_device(np.full(n + 8, np.nan, np.float32))
    lib.convert(src, st, d16, BF16, n)
    lib.convert(src, st, d32, F32, n)
    got16, got32 = d16.numpy(), d32.numpy()
    assert np.array_equal(got16[:n], orc.to_bf16(wide))
    assert np.array_equal(got32[:n].view(np.uint32), wide.view(np.uint32))
    assert np.all(got16[n:] == 0xdead) and np.all(np.isnan(got32[n:]))      # nothing written past n
    for b in (src, d16, d32):
        b.free()


@pytest.mark.parametrize("rows,cols,ld,base", [(64, 64, 64, 0), (70, 130, 200, 17), (1, 5, 3, 2),
                                               (512, 896, 1152, 640), (333, 64, 333, 0)])
@pytest.mark.parametrize("st,dt", [(F16, F32), (F16, BF16), (F32, F32), (BF16, BF16)])
def test_convert_transpose_into_kn(lib, orc, rows, cols, ld, base, st, dt):
    """File rows [out, in] into the seam's [K, N] layout at a column block (qwen_model.h:88-106)."""
    print("case transpose", rows, cols, ld, base, st, dt, flush=True)
    rng = np.random.default_rng(rows * 7 + cols)
    if st == F32:
        host = rng.standard_normal((rows, cols)).astype(np.float32)
        wide = host
    else:
        host = rng.integers(0, 0x7c00 if st == F16 else 0x7f80, (rows, cols), dtype=np.uint16)
        wide = orc.f16_widen(host) if st == F16 else orc.bf16_widen(host)
    src = lib.to_device(host)
    fill = np.full((cols, ld), 0x1234, np.uint16) if dt == BF16 else np.full((cols, ld), 7.0, np.float32)
    dst = lib.to_device(fill)
    lib.convert_transpose(src, st, dst, dt, rows, cols, ld, base)
    got = dst.numpy()
    want = fill.copy()
    want[:, base:base + rows] = orc.to_bf16(wide.T.copy()) if dt == BF16 else wide.T
    assert np.array_equal(got.view(np.uint16 if dt == BF16 else np.uint32), want.view(np.uint16 if dt == BF16 else np.uint32))
    src.free(); dst.free()


@pytest.mark.parametrize("st", [F16, F32, BF16])
def test_quantize_q4_is_bit_exact(lib, orc, st):
    """array::to_q4 of the widened rows (array.h:703-742): packed nibbles and scales bit for bit,
    incl. rounding ties, all-zero groups, a group of one huge value, and row blocks stacked into a
    fused buffer (q|k|v)."""
    rng = np.random.default_rng(11 + st)
    K = 256
    parts = [96, 32, 32]
    Ntot = sum(parts)

    def rows(n):
        w = (rng.standard_normal((n, K)) * 0.02).astype(np.float32)
        w[0, :32] = 0.0                                   # all-zero group: scale = 1e-8 / 7
        w[1, 32:64] = np.arange(32, dtype=np.float32) * 0.5 - 8.0   # exact half steps of scale 8/7... ties in w/scale
        w[2, 64:96] = 0.0; w[2, 70] = 3.0e4                # one dominant value
        w[3, :32] = np.where(np.arange(32) % 2, -7.0, 7.0) * 0.125
        if st == F16:
            return w.astype(np.float16).view(np.uint16)
        if st == BF16:
            return orc.to_bf16(w)
        return w
    q4 = lib.to_device(np.zeros(orc.q4_bytes(Ntot, K), np.uint8))
    wide_rows = []
    base = 0
    for n in parts:
        host = rows(n)
        src = lib.to_device(host)
        lib.quantize_q4(src, st, q4, n, K, row_base=base, total_rows=Ntot)
        src.free()
        wide_rows.append(host if st == F32 else orc.f16_widen(host) if st == F16 else orc.bf16_widen(host))
        base += n
    wide = np.concatenate(wide_rows, axis=0)             # [N, K]
    want = orc.to_q4(np.ascontiguousarray(wide.T))       # the reference quantises the logical [K, N] array
    got = q4.numpy(np.uint8)
    assert np.array_equal(got[:Ntot * K // 2], want[:Ntot * K // 2])
    assert np.array_equal(got[Ntot * K // 2:].view(np.uint32), want[Ntot * K // 2:].view(np.uint32))
    q4.free()


def test_quantize_q4_declines(lib, pkg):
    b = lib.empty(4096)
    for rows, K, group in [(4, 48, 32), (0, 64, 32), (4, 64, 16)]:
        with pytest.raises(pkg.TlHipError):
            lib._chk(lib.c.tlhip_quantize_q4(b.ptr, F32, b.ptr, b.ptr, rows, K, group))
    b.free()


# ---- a whole model from a file -----------------------------------------------------------------
SMALL = dict(n_layers=3, hidden=512, n_q_heads=8, n_kv_heads=2, head_dim=64, ff=1024, vocab=1000,
             max_ctx=96, eps=1e-6, rope_base=1e6)
WIDE_HEAD = dict(n_layers=2, hidden=256, n_q_heads=4, n_kv_heads=2, head_dim=128, ff=512, vocab=320,
                 max_ctx=80, eps=1e-5, rope_base=1e4)


def synth_weights(d, seed, tied=False):
    """File-layout tensors: linear layers [out, in] float16, vectors float32."""
    rng = np.random.default_rng(seed)
    E, QD, KD, FF = d["hidden"], d["n_q_heads"] * d["head_dim"], d["n_kv_heads"] * d["head_dim"], d["ff"]
    lin = lambda o, i: (rng.standard_normal((o, i)) * 0.02).astype(np.float16)
    vec = lambda n, m, s: (m + s * rng.standard_normal(n)).astype(np.float32)
    w = {"token_embd.weight": (rng.standard_normal((d["vocab"], E)) * 0.02).astype(np.float16),
         "output_norm.weight": vec(E, 1.0, 0.02)}
    w["output.weight"] = w["token_embd.weight"] if tied else lin(d["vocab"], E)
    for l in range(d["n_layers"]):
        p = "blk.%d." % l
        w.update({p + "attn_q.weight": lin(QD, E), p + "attn_k.weight": lin(KD, E), p + "attn_v.weight": lin(KD, E),
                  p + "attn_output.weight": lin(E, QD), p + "ffn_gate.weight": lin(FF, E), p + "ffn_up.weight": lin(FF, E),
                  p + "ffn_down.weight": lin(E, FF), p + "attn_q.bias": vec(QD, 0, 0.02), p + "attn_k.bias": vec(KD, 0, 0.02),
                  p + "attn_v.bias": vec(KD, 0, 0.02), p + "attn_norm.weight": vec(E, 1, 0.02), p + "ffn_norm.weight": vec(E, 1, 0.02)})
    return w


def oracle_from_weights(orc, d, w, q4, with_bias=True):
    """The oracle model holding the same tensors: file rows [out, in] widened and transposed to the
    logical [K, N] the reference's build() feeds to to_q4 / to_bf16 (qwen_model.h:449-505)."""
    om = orc.qwen_create(d, seed=1, q4=q4)
    kn = lambda a: np.ascontiguousarray(orc.f16_widen(a.view(np.uint16)).T)
    names = dict(wq="attn_q.weight", wk="attn_k.weight", wv="attn_v.weight", wo="attn_output.weight",
                 wg="ffn_gate.weight", wu="ffn_up.weight", wd="ffn_down.weight")
    vecs = dict(bq="attn_q.bias", bk="attn_k.bias", bv="attn_v.bias", an="attn_norm.weight", fn="ffn_norm.weight")
    for l in range(d["n_layers"]):
        p = "blk.%d." % l
        for k, n in names.items():
            om.set(l, k, kn(w[p + n]))
        for k, n in vecs.items():
            v = w[p + n]
            om.set(l, k, v if with_bias or not n.endswith(".bias") else np.zeros_like(v))
    om.set(-1, "embed", orc.f16_widen(w["token_embd.weight"].view(np.uint16)))
    om.set(-1, "onorm", w["output_norm.weight"])
    om.set(-1, "outw", kn(w["output.weight"]))
    return om


def _near_tie(logits, rtol=1e-4, atol=1e-5):
    top2 = np.sort(logits)[-2:]
    return (top2[1] - top2[0]) <= atol + rtol * abs(top2[1])


@pytest.mark.parametrize("fmt", ["q4", "bf16"])
@pytest.mark.parametrize("dims,variant", [(SMALL, "plain"), (SMALL, "tied"), (SMALL, "no_bias"), (WIDE_HEAD, "plain")])
def test_model_from_gguf_decodes_like_the_oracle(orc, tmp_path, fmt, dims, variant):
    """load_gguf: metadata -> dims, f16 tensors uploaded as stored and converted on the device into
    fused int4 / bf16-row weights, f16 embedding rows gathered per token. 40 greedy steps against
    the oracle model built from the same tensors: every logit inside allclose(rtol 1e-4, atol 1e-5),
    max |d| / (1 + |ref|) < 1e-5, same token unless the oracle's top two are a near tie (the
    reference's own bar for such a loop is maxrel < 2e-3, check_llm_decode.cpp:268-276)."""
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    tied, with_bias = variant == "tied", variant != "no_bias"
    w = synth_weights(dims, seed=5, tied=tied)
    path = str(tmp_path / "model.gguf")
    W.qwen2_file(path, dims, w, tied=tied, with_bias=with_bias)
    g = qwen.QwenGPU.from_gguf(path, fmt=fmt, max_ctx=dims["max_ctx"])
    for k in ("n_layers", "hidden", "n_q_heads", "n_kv_heads", "head_dim", "ff", "vocab", "max_ctx"):
        assert getattr(g.d, k) == dims[k], k
    om = oracle_from_weights(orc, dims, w, q4=(fmt == "q4"), with_bias=with_bias)
    rng = np.random.default_rng(9)
    tok, worst = int(rng.integers(0, dims["vocab"])), 0.0
    for pos in range(40):
        want_tok, want_logits = om.step(tok, pos)
        got_tok, got_logits = g.step(tok, pos, want_logits=True)
        worst = max(worst, check_logits(got_logits, want_logits, 1e-5, "pos %d" % pos, 1.0)[0])
        if got_tok != want_tok:
            assert _near_tie(want_logits), (pos, got_tok, want_tok)
        tok = want_tok if pos >= 8 else int(rng.integers(0, dims["vocab"]))
    print("gguf %s %s worst logits maxrel %.2e" % (fmt, variant, worst))
    c = g.census()
    assert c["quantize_q4" if fmt == "q4" else "convert"] > 0
    g.close(); om.close()


def test_model_from_gguf_greedy_loop_on_device(orc, tmp_path):
    """The device-resident token loop on a file-loaded model gathers f16 embedding rows on the
    device (tlhip_embed_gather_f16): same tokens as stepping from the host."""
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    w = synth_weights(SMALL, seed=6)
    path = str(tmp_path / "model.gguf")
    W.qwen2_file(path, SMALL, w)
    g = qwen.QwenGPU.from_gguf(path, fmt="q4", max_ctx=SMALL["max_ctx"])
    tok, toks = 17, []
    for pos in range(24):
        tok = g.step(tok, pos)
        toks.append(tok)
    g2 = qwen.QwenGPU.from_gguf(path, fmt="q4", max_ctx=SMALL["max_ctx"])
    g2.greedy_init(17, 0)
    assert g2.greedy_run(24) == 24
    assert list(g2.greedy_tokens(0, 24)) == toks
    g.close(); g2.close()


@pytest.mark.parametrize("what", ["missing_tensor", "bad_shape", "quantised", "f32_embedding"])
def test_load_gguf_refuses_what_it_cannot_take(tmp_path, what):
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    d = dict(WIDE_HEAD, n_layers=1)
    w = synth_weights(d, seed=2)
    if what == "missing_tensor":
        del w["blk.0.ffn_up.weight"]
    elif what == "bad_shape":
        w["blk.0.attn_k.weight"] = w["blk.0.attn_k.weight"][:-1]
    elif what == "f32_embedding":
        w["token_embd.weight"] = w["token_embd.weight"].astype(np.float32)
    path = str(tmp_path / "bad.gguf")
    if what == "quantised":
        # ffn_down stored as q8_0 blocks of the right element count
        blocks = bytes(w["blk.0.ffn_down.weight"].size // 32 * 34)
        tensors = []
        for name, a in w.items():
            a = np.ascontiguousarray(a)
            if name == "blk.0.ffn_down.weight":
                tensors.append((name, W.GGML["q8_0"], list(a.shape[::-1]), blocks))
            else:
                code = W.GGML["f16"] if a.dtype == np.float16 else W.GGML["f32"]
                tensors.append((name, code, list(a.shape[::-1]), a.tobytes()))
        kv = [("general.architecture", W.STRING, "qwen2"), ("qwen2.block_count", W.U32, 1),
              ("qwen2.embedding_length", W.U32, d["hidden"]), ("qwen2.feed_forward_length", W.U32, d["ff"]),
              ("qwen2.attention.head_count", W.U32, d["n_q_heads"]), ("qwen2.attention.head_count_kv", W.U32, d["n_kv_heads"]),
              ("qwen2.attention.key_length", W.U32, d["head_dim"])]
        W.write(path, kv, tensors)
    else:
        W.qwen2_file(path, d, w)
    with pytest.raises(RuntimeError, match="load_gguf failed"):
        qwen.QwenGPU.from_gguf(path, fmt="q4", max_ctx=64)
