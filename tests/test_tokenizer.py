"""tl::tokenizer (byte-level BPE) against the reference's tokenizer (include/tokenizer.h,
compiled into oracle/_ref) on a synthetic vocabulary: a GGUF file whose tokenizer.ggml.* metadata
holds the 256 byte pieces, merges learnt from a small multilingual corpus and three control
tokens. Same ids, same decoded bytes, same refusals. Host logic only."""
import importlib
import os
import unicodedata

import numpy as np
import pytest

import ggufwriter as W

CORPUS = (
    "The quick brown fox jumps over the lazy dog. I'm sure you're right, they'll see; we've done it, he'd say.\n"
    "Give me a short introduction to large language models. Large language models are trained on text.\n"
    "def encode(self, text):\n    return [self.vocab[t] for t in text.split()]  # 123 456 7890\n"
    "日本語のテスト です。 これは 日本語 の テスト。 中文 测试 文本。 한국어 테스트 문장.\n"
    "Привет, мир! Это тест. Ελληνικά κείμενο. naïve café über straße.\n"
    "    leading spaces\tand\ttabs   trailing   \r\n\r\n\n  \n"
    "!!! ??? ... --- *** $100.00 (a+b)*c == d; x<=y && y>=z || !w\n"
) * 3


def byte_pieces():
    keep = list(range(33, 127)) + list(range(161, 173)) + list(range(174, 256))
    out, nxt = {}, 256
    for b in range(256):
        if b in keep:
            out[b] = chr(b)
        else:
            out[b] = chr(nxt)
            nxt += 1
    return out


def train_bpe(corpus, n_merges):
    """A small BPE trainer over space-led words: any consistent merge list exercises the merger."""
    bp = byte_pieces()
    words = {}
    for w in corpus.replace("\n", " \n").split(" "):
        if w:
            key = tuple(bp[b] for b in (" " + w).encode())
            words[key] = words.get(key, 0) + 1
    merges = []
    for _ in range(n_merges):
        pairs = {}
        for w, c in words.items():
            for a, b in zip(w, w[1:]):
                pairs[(a, b)] = pairs.get((a, b), 0) + c
        if not pairs:
            break
        (a, b), _ = max(pairs.items(), key=lambda kv: (kv[1], kv[0]))
        merges.append((a, b))
        new = {}
        for w, c in words.items():
            out, i = [], 0
            while i < len(w):
                if i + 1 < len(w) and w[i] == a and w[i + 1] == b:
                    out.append(a + b)
                    i += 2
                else:
                    out.append(w[i])
                    i += 1
            new[tuple(out)] = new.get(tuple(out), 0) + c
        words = new
    return merges


def write_vocab(path):
    bp = byte_pieces()
    merges = train_bpe(CORPUS, 400)
    tokens = [bp[b] for b in range(256)]
    seen = set(tokens)
    for a, b in merges:
        if a + b not in seen:
            tokens.append(a + b)
            seen.add(a + b)
    controls = ["<|endoftext|>", "<|im_start|>", "<|im_end|>", "<|im_start|>system"]   # one is a prefix of another
    types = [1] * len(tokens) + [3] * len(controls)
    tokens += controls
    tokens.append("<|not_control|>")          # looks like a control token but is a normal one: never matched atomically
    types.append(1)
    kv = [("general.architecture", W.STRING, "qwen2"),
          ("tokenizer.ggml.model", W.STRING, "gpt2"),
          ("tokenizer.ggml.tokens", W.ARRAY, (W.STRING, tokens)),
          ("tokenizer.ggml.token_type", W.ARRAY, (W.I32, types)),
          ("tokenizer.ggml.merges", W.ARRAY, (W.STRING, [a + " " + b for a, b in merges])),
          ("tokenizer.ggml.eos_token_id", W.U32, len(tokens) - 3),
          ("tokenizer.ggml.bos_token_id", W.U32, len(tokens) - 5)]
    W.write(path, kv, [])
    return tokens


@pytest.fixture(scope="module")
def vocab_file(tmp_path_factory):
    path = str(tmp_path_factory.mktemp("tok") / "vocab.gguf")
    return path, write_vocab(path)


@pytest.fixture(scope="module")
def toks(vocab_file, refimpl):
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    mine, theirs = qwen.Tokenizer(vocab_file[0]), refimpl.tokenizer(vocab_file[0])
    yield mine, theirs
    mine.close(); theirs.close()


CASES = [
    "Hello, world!", "The quick brown fox jumps over the lazy dog.", "日本語のテスト", "123  456\n789",
    "  leading spaces and\ttab", "I'm you're THEY'LL we'Ve he'D it's don't 'tis ' 's' ''ll", "a'", "'", "'r", "'l",
    "<|im_start|>system\nYou are a helpful assistant.<|im_end|>\n<|im_start|>user\nHi<|im_end|>\n<|im_start|>assistant\n",
    "<|endoftext|>", "<|endoftext|><|endoftext|>x<|im_end|", "<|not_control|> and <|im_start|>system2", "<|im_start|>syste",
    "", " ", "  ", "   x", "x   ", "\n", "\n\n", " \n \n ", "\r\n\r\n", "a\r\nb", "\t\t\tx", " \t\n", "x \n y", "x y", "x　　y",
    "!!!\n\n\n???", " !!!", "  !!!", "a !b", "$100.00", "...\r\n", "1234567890", "٣٤٥ ४५६ ⅓ ²", "x²y", "é ñ", "🙂🙃 👍🏽",
    "naïve café ÜBER straße", "Привет, мир!", "中文，测试。", "한국어 테스트", "ªº µ ǅ ʰ", "​​zero​width", "\x00\x01\x7f",
    "tab\tseparated\tvalues", "under_score snake_case camelCase", "https://example.com/a?b=c&d=e#f", "a b c", "\x1c\x1d\x1e\x1f end",
]


def test_encode_decode_equal_the_reference(toks):
    mine, theirs = toks
    assert (mine.bos_id, mine.eos_id) == (theirs.bos_id, theirs.eos_id)
    for text in CASES:
        raw = text.encode()
        ids = mine.encode(raw)
        assert ids == theirs.encode(raw), text
        assert mine.decode(ids) == raw == theirs.decode(ids), text


def test_golden_ids_from_the_reference():
    """tests/golden/tok_vocab.gguf + tok_cases.json: ids and decoded bytes the REFERENCE's tokenizer
    produced for CASES (tests/golden/make_golden.py tokenizer); holds where oracle/_ref is not built."""
    import json
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    gold = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    mine = qwen.Tokenizer(os.path.join(gold, "tok_vocab.gguf"))
    cases = json.load(open(os.path.join(gold, "tok_cases.json")))
    assert len(cases) >= len(CASES)
    for c in cases:
        raw = bytes.fromhex(c["text_hex"])
        assert mine.encode(raw) == c["ids"], raw
        assert mine.decode(c["ids"]) == raw
    mine.close()


def test_control_tokens_are_atomic_and_longest_wins(toks, vocab_file):
    mine, _ = toks
    tokens = vocab_file[1]
    ids = mine.encode("<|im_start|>system")
    assert ids == [tokens.index("<|im_start|>system")]
    ids = mine.encode("<|im_start|>user")
    assert ids[0] == tokens.index("<|im_start|>") and len(ids) > 1
    assert tokens.index("<|not_control|>") not in mine.encode("<|not_control|>")


def test_malformed_utf8_and_random_bytes(toks):
    """Stray continuation bytes, truncated sequences, 0xF8+ bytes: every byte still maps to a byte
    piece, and the pre-token boundaries (hence the ids) agree with the reference."""
    mine, theirs = toks
    rng = np.random.default_rng(3)
    fixed = [b"\x80", b"\xff\xfe", b"\xc3", b"\xe3\x81", b"\xf0\x9f\x99", b"a\xc3", b"\xaa\xb5 x", b"\xc3\x28", b"\xed\xa0\x80",
             b"ok \xe2\x82 ok", b"\xf8\x88\x80\x80\x80", b"x\xf0\x9f", b"\xc0\x80", b"\xe0\x80\xaf"]
    for raw in fixed + [bytes(rng.integers(0, 256, int(rng.integers(1, 40)), dtype=np.uint8)) for _ in range(400)]:
        ids = mine.encode(raw)
        assert ids == theirs.encode(raw), raw
        assert mine.decode(ids) == raw


def test_random_text_fuzz(toks):
    mine, theirs = toks
    rng = np.random.default_rng(5)
    alphabet = list("abcXYZ  \t\n\r'.,!?-_019") + ["'s", "'LL", "é", "ß", "я", "日", "本", "한", "٣", "²", "🙂", " ", "　", "́",
                                                      "<|im_end|>", "<|endoftext|>", "<|", "|>", " the", " language", "models"]
    for _ in range(600):
        text = "".join(alphabet[i] for i in rng.integers(0, len(alphabet), int(rng.integers(0, 60))))
        raw = text.encode()
        ids = mine.encode(raw)
        assert ids == theirs.encode(raw), text
        assert mine.decode(ids) == raw


def test_long_pretoken_merges_like_the_quadratic_reference(toks):
    """One pre-token of several thousand letters: the heap-ordered merger must pick the same merges
    (lowest rank, leftmost among equals) as the reference's rescan of all pairs after every merge."""
    mine, theirs = toks
    rng = np.random.default_rng(8)
    for n in (257, 3000):
        raw = "".join("language models the of"[i] for i in rng.integers(0, 22, n)).replace(" ", "e").encode()
        assert mine.encode(raw) == theirs.encode(raw)
    raw = b"a" * 1001
    assert mine.encode(raw) == theirs.encode(raw)


def test_refusals_equal_the_reference(toks, vocab_file):
    mine, theirs = toks
    n = len(vocab_file[1])
    for ids in ([n], [-1], [0, n + 5]):
        assert theirs.decode(ids) is None
        with pytest.raises(RuntimeError, match="id out of range"):
            mine.decode(ids)
    # a control token's text is not made of byte pieces: decoding it alone is refused by both
    ctl = vocab_file[1].index("<|im_end|>")
    got = theirs.decode([ctl])
    if got is None:
        with pytest.raises(RuntimeError):
            mine.decode([ctl])
    else:
        assert mine.decode([ctl]) == got


def test_vocabulary_without_a_byte_piece_is_reported(tmp_path, refimpl):
    """A vocabulary that lacks a byte piece cannot spell every text: both tokenizers refuse such a text."""
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    bp = byte_pieces()
    tokens = [bp[b] for b in range(256) if b != ord("z")]
    kv = [("tokenizer.ggml.tokens", W.ARRAY, (W.STRING, tokens)), ("tokenizer.ggml.token_type", W.ARRAY, (W.I32, [1] * len(tokens))),
          ("tokenizer.ggml.merges", W.ARRAY, (W.STRING, [])), ("tokenizer.ggml.eos_token_id", W.U32, 0),
          ("tokenizer.ggml.bos_token_id", W.U32, 0)]
    path = str(tmp_path / "holes.gguf")
    W.write(path, kv, [])
    mine, theirs = qwen.Tokenizer(path), refimpl.tokenizer(path)
    assert mine.encode(b"abc") == theirs.encode(b"abc")
    assert theirs.encode(b"xyz") is None
    with pytest.raises(RuntimeError, match="symbol not in vocab"):
        mine.encode(b"xyz")
    # a file without tokenizer metadata is refused at construction
    W.write(path, [("general.architecture", W.STRING, "qwen2")], [])
    with pytest.raises(RuntimeError, match="no metadata key"):
        qwen.Tokenizer(path)


def test_code_point_classes_against_the_reference_and_unicodedata(refimpl):
    """\\p{L}, \\p{N}, \\s for every code point: equal to this interpreter's unicodedata (the tables'
    source) everywhere, and equal to the reference's tables except on code points that Unicode %s
    leaves unassigned (the reference's tables come from a later Unicode, tokenizer_data.h:2-4)."""
    qwen = importlib.import_module("cpp-tensorlib_amd.qwen")
    L = qwen._load()
    differ = 0
    for cp in range(0x110000):
        c = chr(cp)
        cat = unicodedata.category(c)
        want = (1 if cat[0] == "L" else 0) | (2 if cat[0] == "N" else 0) | (4 if c.isspace() else 0)
        got = L.tlq_unicode_class(cp)
        assert got == want, hex(cp)
        theirs = refimpl.unicode_class(cp)
        if theirs != got:
            assert cat == "Cn", (hex(cp), cat, got, theirs)     # assigned after this Unicode version
            differ += 1
    print("code points classified differently (all unassigned in Unicode %s): %d" % (unicodedata.unidata_version, differ))
    assert differ < 12000
