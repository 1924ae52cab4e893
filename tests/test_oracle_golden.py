"""CPU: the plain-C oracle reproduces the golden vectors written by the real
reference (tests/golden/make_golden.py) on inputs regenerated from seeds."""
import json
import os

import numpy as np
import pytest

from oraclelib import allclose

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(G, name + ".npz")), json.load(open(os.path.join(G, name + ".json")))


def test_config1_int4_gemv(orc):
    z, meta = load("gemv")
    m = meta["c1"]
    buf, x = orc.fill_q4(m["N"], m["K"], m["seed_w"]), orc.normal(m["K"], m["seed_x"])
    assert orc.crc32(buf) == m["crc_w"] and orc.crc32(x) == m["crc_x"], "inputs not regenerated identically"
    assert np.array_equal(orc.gemv_q4(x, buf, m["N"], m["K"]), z["c1_y"])     # bit-exact


@pytest.mark.parametrize("i", [0, 1, 2, 3])
def test_config2_int4_and_bf16_gemv(orc, i):
    z, meta = load("gemv")
    m = meta["c2_%d" % i]
    N, K = m["N"], m["K"]
    w = orc.normal(K * N, m["seed_w"], 0.0, 0.02).reshape(K, N)
    x = orc.normal(K, m["seed_x"])
    assert orc.crc32(w) == m["crc_w"] and orc.crc32(x) == m["crc_x"]
    q, b = orc.to_q4(w), orc.to_bf16(w)
    assert orc.crc32(q) == m["crc_q4"] and orc.crc32(b) == m["crc_bf16"]        # quantisers bit-exact
    assert np.array_equal(orc.gemv_q4(x, q, N, K)[::m["stride"]], z["c2_q4_%d" % i])
    assert np.array_equal(orc.gemv_bf16(x, b)[::m["stride"]], z["c2_bf16_%d" % i])


@pytest.mark.parametrize("ctx", [512, 2048])
def test_config3_attn_decode(orc, ctx):
    z, meta = load("attn")
    m = meta["c3_%d" % ctx]
    H, D = m["H"], m["D"]
    q = orc.normal(H * D, m["seeds"][0]).reshape(H, D)
    K = orc.normal(H * ctx * D, m["seeds"][1]).reshape(H, ctx, D)
    V = orc.normal(H * ctx * D, m["seeds"][2]).reshape(H, ctx, D)
    assert [orc.crc32(q), orc.crc32(K), orc.crc32(V)] == m["crc"]
    assert np.array_equal(orc.attn_decode(q, K, V, float(1.0 / np.sqrt(128.0))), z["c3_%d" % ctx])


def test_model_ops(orc):
    z, meta = load("ops")
    x = orc.normal(32 * 128, 4000).reshape(32, 128)
    assert orc.crc32(x) == meta["ops"]["crc_rope"]
    assert np.array_equal(orc.rope(x, 4095, 1e6), z["rope_4095"])
    x3 = orc.normal(4 * 6 * 64, 4001).reshape(4, 6, 64)
    assert np.array_equal(orc.rope(x3, 1000, 1e4, T=6), z["rope_T6"])
    for n in (896, 3584):
        xr = orc.normal(2 * n, 4002 + n).reshape(2, n)
        w = orc.normal(n, 4003 + n, 1.0, 0.02)
        assert np.array_equal(orc.rmsnorm(xr, w, 1e-6), z["rmsnorm_%d" % n])
    g, u = orc.normal(4864, 4010, 0, 2.0), orc.normal(4864, 4011)
    assert np.array_equal(orc.swiglu(g, u), z["swiglu"]) and np.array_equal(orc.silu(g), z["silu"])
    sm = orc.normal(5 * 777, 4012, 0, 3.0).reshape(5, 777)
    assert np.array_equal(orc.softmax(sm), z["softmax"])
    assert np.array_equal(orc.row_sum(sm, 1.0) * np.float32(1.0 / 777), z["row_mean"])
    A, B = orc.normal(3 * 700, 4013).reshape(3, 700), orc.normal(700 * 50, 4014).reshape(700, 50)
    assert np.array_equal(orc.dot(A, B, 2.0, 1.0), z["dot_epi"])


def test_small_decode_loop(orc):
    z, meta = load("decode_small")
    om = orc.qwen_create(meta["dims"], seed=meta["seed"], q4=True)
    assert orc.crc32(om.weight(-1, "outw")) == meta["crc_outw"] and orc.crc32(om.weight(0, "wq")) == meta["crc_wq0"]
    tok = meta["first_token"]
    for pos in range(len(z["tokens"])):
        t, lg = om.step(tok, pos)
        assert t == int(z["tokens"][pos]), pos
        assert np.array_equal(lg[::13], z["logits_sub"][pos]), pos             # bit-exact logits
        tok = t
    om.close()


def test_qwen05b_golden_is_well_formed():
    p = os.path.join(G, "qwen05b_decode.npz")
    if not os.path.exists(p):
        pytest.skip("tests/golden/qwen05b_decode.npz not generated yet")
    z, meta = load("qwen05b_decode")
    assert len(meta["prompt"]) == 128 and z["argmax"].shape == (383,) and np.all(z["margin"] >= 0)
