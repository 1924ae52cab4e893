"""The GGUF v3 reader (tl/gguf.h) against the reference's reader (include/gguf.h, compiled
into oracle/_ref) on files written by tests/ggufwriter.py: both parse results are rendered by
one generic text dump and must be identical; every malformed file one of them rejects the
other rejects too. Host logic only: no GPU needed."""
import importlib
import os
import struct

import numpy as np
import pytest

import ggufwriter as W

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = os.path.join(HERE, "golden")


@pytest.fixture(scope="module")
def qwen():
    return importlib.import_module("cpp-tensorlib_amd.qwen")


def rich_file():
    rng = np.random.default_rng(7)
    kv = [("general.architecture", W.STRING, "qwen2"), ("general.alignment", W.U32, 64),
          ("a.u8", W.U8, 250), ("a.i8", W.I8, -128), ("a.u16", W.U16, 65535), ("a.i16", W.I16, -32768),
          ("a.u32", W.U32, 4000000000), ("a.i32", W.I32, -2000000000), ("a.f32", W.F32, 1e-6),
          ("a.true", W.BOOL, 1), ("a.false", W.BOOL, 0), ("a.odd_bool", W.BOOL, 7),
          ("a.u64", W.U64, 2 ** 63 + 5), ("a.i64", W.I64, -2 ** 62), ("a.f64", W.F64, 3.141592653589793),
          ("a.empty", W.STRING, ""), ("a.bytes", W.STRING, bytes([0, 255, 34, 92, 10, 200])),
          ("tokenizer.ggml.tokens", W.ARRAY, (W.STRING, ["<|endoftext|>", "Ġhello", "", "日本"])),
          ("tokenizer.ggml.token_type", W.ARRAY, (W.I32, [1, 1, 3, -4])),
          ("tokenizer.ggml.scores", W.ARRAY, (W.F32, [0.5, -1.25, 3e38])),
          ("a.empty_array", W.ARRAY, (W.U8, [])), ("a.u64s", W.ARRAY, (W.U64, [0, 2 ** 64 - 1])),
          ("a.bools", W.ARRAY, (W.BOOL, [1, 0, 1])), ("a.f64s", W.ARRAY, (W.F64, [1e300, -0.0])),
          ("dup", W.U32, 1), ("dup", W.U32, 2)]
    t = [("token_embd.weight", W.GGML["f16"], [64, 10], rng.integers(0, 65536, 640, dtype=np.uint16).tobytes()),
         ("blk.0.attn_norm.weight", W.GGML["f32"], [64], rng.standard_normal(64).astype(np.float32).tobytes()),
         ("q4_0.blocks", W.GGML["q4_0"], [64, 3], rng.integers(0, 256, 6 * 18, dtype=np.uint8).tobytes()),
         ("q6_k.blocks", W.GGML["q6_k"], [256, 2], rng.integers(0, 256, 2 * 210, dtype=np.uint8).tobytes()),
         ("q8_0.blocks", W.GGML["q8_0"], [32], rng.integers(0, 256, 34, dtype=np.uint8).tobytes()),
         ("scalar", W.GGML["f32"], [], struct.pack("<f", 2.5)),
         ("three_d", W.GGML["f16"], [4, 3, 2], rng.integers(0, 65536, 24, dtype=np.uint16).tobytes()),
         ("token_embd.weight", W.GGML["f32"], [2], struct.pack("<ff", 1.0, 2.0))]     # duplicate name
    return kv, t


def ours(qwen, path):
    try:
        g = qwen.GgufFile(path)
    except RuntimeError as e:
        return None, str(e)
    text = g.dump()
    g.close()
    return text, None


def test_reader_equals_reference_on_a_rich_file(qwen, refimpl, tmp_path):
    kv, t = rich_file()
    for align_kv in (("general.alignment", W.U32, 64), ("general.alignment", W.U64, 128), None):
        kv2 = [e for e in kv if e[0] != "general.alignment"] + ([align_kv] if align_kv else [])
        path = str(tmp_path / "rich.gguf")
        W.write(path, kv2, t, alignment=align_kv[2] if align_kv else 32)
        mine, err = ours(qwen, path)
        assert mine is not None, err
        theirs = refimpl.gguf_dump(path)
        assert theirs is not None and mine == theirs
        assert "alignment=%d" % (align_kv[2] if align_kv else 32) in mine
        assert 'kv 3:"dup" t4=1' in mine            # a repeated key keeps its first value
        assert mine.count("tensor ") == len(t)


def test_reader_golden_dump(qwen):
    """The committed fixture and the dump the REFERENCE's reader produced for it
    (tests/golden/make_golden.py gguf): holds where oracle/_ref is not built."""
    mine, err = ours(qwen, os.path.join(GOLD, "gguf_small.gguf"))
    assert mine is not None, err
    with open(os.path.join(GOLD, "gguf_small.dump.txt"), encoding="latin-1") as f:
        assert mine == f.read()


def test_every_truncation_is_rejected_like_the_reference(qwen, refimpl, tmp_path):
    kv, t = rich_file()
    data = W.build(kv[:8], t[:3])
    path = str(tmp_path / "cut.gguf")
    cuts = sorted(set(list(range(0, 64)) + list(range(64, len(data), 7)) + [len(data) - 1, len(data)]))
    rejected = 0
    for n in cuts:
        with open(path, "wb") as f:
            f.write(data[:n])
        mine, _ = ours(qwen, path)
        theirs = refimpl.gguf_dump(path)
        assert (mine is None) == (theirs is None), n
        if mine is not None:
            assert mine == theirs
        else:
            rejected += 1
    assert rejected >= len(cuts) - 2        # only the complete file (and nothing shorter) parses


@pytest.mark.parametrize("what", ["magic", "version2", "version4", "nested_array", "value_type",
                                  "tensor_type", "offset_past_end", "huge_string", "huge_array"])
def test_malformed_files_are_rejected_by_both(qwen, refimpl, tmp_path, what):
    kv = [("k", W.U32, 1)]
    t = [("w", W.GGML["f32"], [4], struct.pack("<4f", 1, 2, 3, 4))]
    data = bytearray(W.build(kv, t))
    if what == "magic":
        data[:4] = b"GGML"
    elif what == "version2":
        data[4:8] = struct.pack("<I", 2)
    elif what == "version4":
        data[4:8] = struct.pack("<I", 4)
    elif what == "nested_array":
        data = bytearray(W.build([("k", W.ARRAY, (W.U32, []))], t))
        i = data.index(struct.pack("<IQ", W.U32, 0), 24)
        data[i:i + 4] = struct.pack("<I", W.ARRAY)
    elif what == "value_type":
        i = data.index(b"k", 24) + 1
        data[i:i + 4] = struct.pack("<I", 13)
    elif what == "tensor_type":
        i = data.index(b"w", 40) + 1 + 4 + 8
        data[i:i + 4] = struct.pack("<I", 99)
    elif what == "offset_past_end":
        i = data.index(b"w", 40) + 1 + 4 + 8 + 4
        data[i:i + 8] = struct.pack("<Q", 1 << 40)
    elif what == "huge_string":
        data[24:32] = struct.pack("<Q", 1 << 60)       # length of the first key
    elif what == "huge_array":
        data = bytearray(W.build([("k", W.ARRAY, (W.U8, [1, 2]))], t))
        i = data.index(struct.pack("<IQ", W.U8, 2), 24)
        data[i + 4:i + 12] = struct.pack("<Q", 1 << 40)
    path = str(tmp_path / "bad.gguf")
    with open(path, "wb") as f:
        f.write(data)
    mine, err = ours(qwen, path)
    assert mine is None and err.startswith("gguf:"), (what, err)
    if what != "huge_array":    # the reference tries to reserve 2^40 elements before it reads any
        assert refimpl.gguf_dump(path) is None


def test_missing_file_and_empty_file(qwen, tmp_path):
    assert ours(qwen, str(tmp_path / "nope.gguf"))[0] is None
    p = str(tmp_path / "empty.gguf")
    open(p, "wb").close()
    assert ours(qwen, p)[0] is None


def test_bf16_storage_is_an_extension(qwen, refimpl, tmp_path):
    """Storage code 30 (bf16) is accepted here; the reference's reader rejects it (gguf.h:56-76)."""
    path = str(tmp_path / "bf16.gguf")
    W.write(path, [], [("w", W.GGML["bf16"], [8], bytes(16))])
    mine, err = ours(qwen, path)
    assert mine is not None and "type=30" in mine and "nbytes=16" in mine, err
    assert refimpl.gguf_dump(path) is None


def test_hyperparameters_from_metadata(qwen, tmp_path):
    d = dict(n_layers=3, hidden=512, n_q_heads=8, n_kv_heads=2, head_dim=64, ff=1024, vocab=300,
             max_ctx=96, eps=1e-5, rope_base=1e4)
    w = {"token_embd.weight": np.zeros((300, 512), np.float16)}
    path = str(tmp_path / "hp.gguf")
    W.qwen2_file(path, d, w)
    g = qwen.GgufFile(path)
    got = g.dims(max_ctx=96)
    for k in ("n_layers", "hidden", "n_q_heads", "n_kv_heads", "head_dim", "ff", "vocab", "max_ctx"):
        assert getattr(got, k) == d[k], k
    assert got.eps == np.float32(1e-5) and got.rope_base == np.float32(1e4)
    assert g.dims(max_ctx=10 ** 6).max_ctx == 32768          # clipped to the file's context_length
    g.close()
    # head_dim from attention.key_length when it is not hidden / heads; another architecture name
    d2 = dict(d, head_dim=128)
    W.qwen2_file(path, d2, w, arch="llama")
    g = qwen.GgufFile(path)
    assert g.dims().head_dim == 128
    g.close()
    # a missing key is reported, not guessed
    W.write(path, [("general.architecture", W.STRING, "qwen2")], [])
    g = qwen.GgufFile(path)
    with pytest.raises(RuntimeError, match="no metadata key"):
        g.dims()
    g.close()
