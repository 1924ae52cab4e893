"""Writes the golden vectors under tests/golden/ by running the REAL reference
(cpp-tensorlib's CPU path, compiled into oracle/_ref/libtlref.so from the sources
under /root/reference by oracle/Makefile) on seeded inputs.

Inputs are not stored: every test regenerates them with the checker's own PRNG
(oracle.c: xorshift32 + Box-Muller) and proves it did so with the CRC-32 recorded
here. Outputs are stored as float32 (sub-sampled where large).

    python tests/golden/make_golden.py            # everything but the 0.5B decode
    python tests/golden/make_golden.py qwen05b     # BASELINE config 4 token sequence (~10 min)
    python tests/golden/make_golden.py gguf        # a small GGUF file + the reference reader's view of it
    python tests/golden/make_golden.py tokenizer   # a synthetic BPE vocabulary + the reference tokenizer's ids
"""
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from oraclelib import QWEN_05B, oracle, ref  # noqa: E402

orc, R = oracle(), ref()
assert R is not None, "build oracle/_ref first: make -C oracle ref"


def save(name, meta, **arrays):
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
    json.dump(meta, open(os.path.join(HERE, name + ".json"), "w"), indent=1, sort_keys=True)
    print("wrote", name, {k: v.shape for k, v in arrays.items()})


def gemv_cases():
    meta, arrs = {}, {}
    # BASELINE config 1: uniform nibbles, scales ~U(0.005,0.02), x ~ N(0,1)
    N, K = 4864, 896
    buf, x = orc.fill_q4(N, K, 1001), orc.normal(K, 1002)
    arrs["c1_y"] = R.gemv_q4(x, buf, N, K)
    meta["c1"] = dict(N=N, K=K, seed_w=1001, seed_x=1002, crc_w=orc.crc32(buf), crc_x=orc.crc32(x), stride=1)
    # BASELINE config 2 (four of the five shapes; the LM head is covered on the GPU by
    # the oracle, whose arithmetic these cases pin): N(0,0.02) weights -> to_q4 / to_bf16
    for i, (N, K) in enumerate([(3584, 3584), (512, 3584), (18944, 3584), (3584, 18944)]):
        w = orc.normal(K * N, 2000 + i, 0.0, 0.02).reshape(K, N)
        x = orc.normal(K, 2100 + i)
        q = R.to_q4(w)
        b = R.to_bf16(w)
        stride = 1 if N <= 4096 else 7
        arrs["c2_q4_%d" % i] = R.gemv_q4(x, q, N, K)[::stride]
        arrs["c2_bf16_%d" % i] = R.gemv_bf16(x, b)[::stride]
        meta["c2_%d" % i] = dict(N=N, K=K, seed_w=2000 + i, seed_x=2100 + i, crc_w=orc.crc32(w),
                                 crc_x=orc.crc32(x), crc_q4=orc.crc32(q), crc_bf16=orc.crc32(b), stride=stride)
    save("gemv", meta, **arrs)


def attn_cases():
    meta, arrs = {}, {}
    H, D = 28, 128
    for ctx in (512, 2048):
        q = orc.normal(H * D, 3000).reshape(H, D)
        K = orc.normal(H * ctx * D, 3001 + ctx).reshape(H, ctx, D)
        V = orc.normal(H * ctx * D, 3002 + ctx).reshape(H, ctx, D)
        arrs["c3_%d" % ctx] = R.attn_decode(q, K, V, float(1.0 / np.sqrt(128.0)))
        meta["c3_%d" % ctx] = dict(H=H, D=D, ctx=ctx, seeds=[3000, 3001 + ctx, 3002 + ctx],
                                   crc=[orc.crc32(q), orc.crc32(K), orc.crc32(V)])
    save("attn", meta, **arrs)


def op_cases():
    meta, arrs = {}, {}
    x = orc.normal(32 * 128, 4000).reshape(32, 128)
    arrs["rope_4095"] = R.rope(x, 4095, 1e6)
    x3 = orc.normal(4 * 6 * 64, 4001).reshape(4, 6, 64)
    arrs["rope_T6"] = R.rope(x3, 1000, 1e4)
    for n in (896, 3584):
        xr = orc.normal(2 * n, 4002 + n).reshape(2, n)
        w = orc.normal(n, 4003 + n, 1.0, 0.02)
        arrs["rmsnorm_%d" % n] = R.rmsnorm(xr, w, 1e-6)
    g, u = orc.normal(4864, 4010, 0, 2.0), orc.normal(4864, 4011)
    arrs["swiglu"] = R.swiglu(g, u)
    arrs["silu"] = R.silu(g)
    sm = orc.normal(5 * 777, 4012, 0, 3.0).reshape(5, 777)
    arrs["softmax"] = R.softmax(sm)
    arrs["row_mean"] = R.row_mean(sm)
    A, B = orc.normal(3 * 700, 4013).reshape(3, 700), orc.normal(700 * 50, 4014).reshape(700, 50)
    arrs["dot_epi"] = R.dot(A, B, 2.0, 1.0)
    meta["ops"] = dict(crc_rope=orc.crc32(x), crc_g=orc.crc32(g))
    save("ops", meta, **arrs)


def decode_small():
    dims = dict(n_layers=3, hidden=512, n_q_heads=8, n_kv_heads=2, head_dim=64, ff=1024, vocab=1000,
                max_ctx=96, eps=1e-6, rope_base=1e6)
    om = orc.qwen_create(dims, seed=3, q4=True)
    rm = R.qwen_from_oracle(om, predeq=False)      # the reference widens int4 on every call
    toks, logit_rows = [], []
    tok = 17
    for pos in range(24):
        t, lg = rm.step(tok, pos)
        toks.append(t)
        logit_rows.append(lg[::13].copy())
        tok = t
    meta = dict(dims=dims, seed=3, first_token=17, crc_outw=orc.crc32(om.weight(-1, "outw")),
                crc_wq0=orc.crc32(om.weight(0, "wq")))
    save("decode_small", meta, tokens=np.array(toks, np.int64), logits_sub=np.array(logit_rows))
    rm.close(); om.close()


def qwen05b():
    """BASELINE config 4: Qwen2.5-0.5B architecture, int4 weights, 128 random prompt ids,
    256 greedy tokens, from the reference's CPU path (weights widened once up front, which
    yields bit-identical values to its per-call widening)."""
    dims = dict(QWEN_05B, max_ctx=384)
    t0 = time.time()
    om = orc.qwen_create(dims, seed=7, q4=True)
    rm = R.qwen_from_oracle(om, predeq=True)
    print("model built in %.0fs" % (time.time() - t0), flush=True)
    prompt = [int(v % dims["vocab"]) for v in np.frombuffer(orc.uniform(128, 99).tobytes(), np.uint32)]
    toks, margins, top1 = [], [], []
    tok = prompt[0]
    for pos in range(128 + 256 - 1):
        t, lg = rm.step(tok, pos)
        two = np.partition(lg, -2)[-2:]
        toks.append(t); margins.append(float(two[1] - two[0])); top1.append(float(two[1]))
        tok = prompt[pos + 1] if pos + 1 < 128 else t
        if pos % 16 == 0:
            print("pos", pos, "tok", t, "%.0fs" % (time.time() - t0), flush=True)
    meta = dict(dims=dims, seed=7, prompt=prompt, crc_outw=orc.crc32(om.weight(-1, "outw")))
    save("qwen05b_decode", meta, argmax=np.array(toks, np.int64), margin=np.array(margins, np.float32),
         top1=np.array(top1, np.float32))


def gguf():
    """gguf_small.gguf (written by tests/ggufwriter.py) and gguf_small.dump.txt: what the
    REFERENCE's reader (include/gguf.h) reports for it, rendered by tl/gguf_dump.h."""
    sys.path.insert(0, os.path.join(HERE, ".."))
    import ggufwriter as W
    from test_gguf_reader import rich_file
    kv, t = rich_file()
    path = os.path.join(HERE, "gguf_small.gguf")
    W.write(path, kv, t, alignment=64)
    text = R.gguf_dump(path)
    assert text is not None
    with open(os.path.join(HERE, "gguf_small.dump.txt"), "w", encoding="latin-1") as f:
        f.write(text)
    print("wrote gguf_small.gguf (%d bytes) and its reference dump (%d chars)" % (os.path.getsize(path), len(text)))


def tokenizer():
    """tok_vocab.gguf (the synthetic vocabulary of tests/test_tokenizer.py) and tok_cases.json: ids
    the REFERENCE's tokenizer (include/tokenizer.h) gives for that file's CASES plus byte strings
    with malformed UTF-8."""
    sys.path.insert(0, os.path.join(HERE, ".."))
    import test_tokenizer as T
    path = os.path.join(HERE, "tok_vocab.gguf")
    T.write_vocab(path)
    tok = R.tokenizer(path)
    rng = np.random.default_rng(3)
    raws = [t.encode() for t in T.CASES] + [b"\x80", b"\xc3", b"\xe3\x81", b"\xaa\xb5 x", b"ok \xe2\x82 ok"]
    raws += [bytes(rng.integers(0, 256, int(rng.integers(1, 40)), dtype=np.uint8)) for _ in range(40)]
    cases = []
    for raw in raws:
        ids = tok.encode(raw)
        assert ids is not None and tok.decode(ids) == raw
        cases.append({"text_hex": raw.hex(), "ids": ids})
    json.dump(cases, open(os.path.join(HERE, "tok_cases.json"), "w"))
    print("wrote tok_vocab.gguf (%d bytes) and %d cases" % (os.path.getsize(path), len(cases)))


if __name__ == "__main__":
    if "tokenizer" in sys.argv[1:]:
        tokenizer()
    elif "gguf" in sys.argv[1:]:
        gguf()
    elif "qwen05b" in sys.argv[1:]:
        qwen05b()
    else:
        gemv_cases(); attn_cases(); op_cases(); decode_small()
