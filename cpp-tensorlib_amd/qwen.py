"""ctypes binding of libtl_qwen.so: the C++ decode harness (include/tl/qwen_decode.h)
as seen from Python tests and benchmarks. The harness finds the HIP library through
tl::hip's dlopen, so TENSORLIB_HIP_LIB is pointed at the in-tree build first."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
QWEN_LIB_PATH = os.path.join(HERE, "lib", "libtl_qwen.so")
HIP_LIB_PATH = os.path.join(HERE, "lib", "libtensorlib_hip.so")

i64, f32, u32, cint = C.c_int64, C.c_float, C.c_uint32, C.c_int
P = C.c_void_p


class Dims(C.Structure):
    _fields_ = [("n_layers", i64), ("hidden", i64), ("n_q_heads", i64), ("n_kv_heads", i64),
                ("head_dim", i64), ("ff", i64), ("vocab", i64), ("max_ctx", i64),
                ("eps", f32), ("rope_base", f32)]


QWEN_05B = dict(n_layers=24, hidden=896, n_q_heads=14, n_kv_heads=2, head_dim=64, ff=4864,
                vocab=151936, max_ctx=512, eps=1e-6, rope_base=1e6)
QWEN_7B = dict(n_layers=28, hidden=3584, n_q_heads=28, n_kv_heads=4, head_dim=128, ff=18944,
               vocab=152064, max_ctx=4352, eps=1e-6, rope_base=1e6)

_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(QWEN_LIB_PATH):
            raise FileNotFoundError("%s is missing: run `python cpp-tensorlib_amd/build.py`" % QWEN_LIB_PATH)
        os.environ.setdefault("TENSORLIB_HIP_LIB", HIP_LIB_PATH)
        L = C.CDLL(QWEN_LIB_PATH)
        sig = {
            "tlq_available": (cint, []),
            "tlq_unavailable_reason": (C.c_char_p, []),
            "tlq_create": (P, [C.POINTER(Dims)]),
            "tlq_destroy": (None, [P]),
            "tlq_set_layer_q4": (cint, [P, i64] + [P] * 12),
            "tlq_set_head_q4": (cint, [P, P, P, P]),
            "tlq_set_random_q4": (cint, [P, u32]),
            "tlq_set_layer_bf16": (cint, [P, i64] + [P] * 12),
            "tlq_set_head_bf16": (cint, [P, P, P, P]),
            "tlq_set_random_bf16": (cint, [P, u32]),
            "tlq_prefill": (cint, [P, P, i64, i64, P]),
            "tlq_stage_chunk": (cint, [P, P, i64]),
            "tlq_prefill_layers": (cint, [P, i64, i64]),
            "tlq_set_cache_pos": (None, [P, i64]),
            "tlq_fill_cache_random": (cint, [P, i64, u32]),
            "tlq_cache_upload": (cint, [P, i64, P, P, i64]),
            "tlq_prefill_hidden": (cint, [P, P, i64]),
            "tlq_step": (i64, [P, i64, i64, P]),
            "tlq_run_layers": (cint, [P, i64, i64]),
            "tlq_argmax": (i64, [P]),
            "tlq_capture": (cint, [P, i64, i64]),
            "tlq_replay": (cint, [P]),
            "tlq_set_fused": (None, [P, cint]),
            "tlq_set_warm": (None, [P, cint, cint, cint]),
            "tlq_profile_steps": (cint, [P, i64, i64, i64, C.POINTER(C.c_double)]),
            "tlq_set_fused_attn": (None, [P, cint]),
            "tlq_set_merge_in_oproj": (None, [P, cint]),
            "tlq_set_norm_images": (None, [P, cint]),
            "tlq_set_gateup_epilogue": (None, [P, cint]),
            "tlq_set_fused_prefill": (None, [P, cint]),
            "tlq_set_prompt_f16": (None, [P, cint]),
            "tlq_greedy_init": (cint, [P, i64, i64]),
            "tlq_greedy_run": (i64, [P, i64]),
            "tlq_greedy_tokens": (cint, [P, i64, i64, P]),
            "tlq_greedy_sync_host_pos": (None, [P]),
            "tlq_decoder_init": (cint, [P, i64, i64]),
            "tlq_decoder_feed": (cint, [P, i64]),
            "tlq_decoder_step": (i64, [P, i64, P]),
            "tlq_decoder_pos": (i64, [P]),
            "tlq_decoder_captured": (cint, [P]),
            "tlq_decoder_sync_host_pos": (None, [P]),
            "tlq_flush": (None, []),
            "tlq_census": (cint, [C.POINTER(C.c_uint64), cint]),
            "tlq_file_error": (C.c_char_p, []),
            "tlq_gguf_open": (P, [C.c_char_p]),
            "tlq_gguf_close": (None, [P]),
            "tlq_gguf_dump": (i64, [P, C.c_char_p, i64]),
            "tlq_gguf_dims": (cint, [P, i64, C.POINTER(Dims)]),
            "tlq_create_from_gguf": (P, [C.c_char_p, cint, i64]),
            "tlq_tok_open": (P, [C.c_char_p]),
            "tlq_tok_close": (None, [P]),
            "tlq_tok_special_ids": (None, [P, C.POINTER(cint), C.POINTER(cint)]),
            "tlq_tok_encode": (i64, [P, C.c_char_p, i64, P, i64]),
            "tlq_tok_decode": (i64, [P, P, i64, C.c_char_p, i64]),
            "tlq_unicode_class": (cint, [u32]),
            "tlq_get_dims": (None, [P, C.POINTER(Dims)]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _p(a):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(P)


class GgufFile:
    """A GGUF v3 file parsed by tl/gguf.h (host only: no GPU is needed to read a file)."""

    def __init__(self, path):
        self.L = _load()
        self.h = self.L.tlq_gguf_open(os.fsencode(path))
        if not self.h:
            raise RuntimeError(self.L.tlq_file_error().decode())

    def dump(self):
        """Canonical rendering of header, metadata and tensor directory (tl/gguf_dump.h)."""
        n = self.L.tlq_gguf_dump(self.h, None, 0)
        buf = C.create_string_buffer(n + 1)
        self.L.tlq_gguf_dump(self.h, buf, n + 1)
        return buf.value.decode("latin-1")

    def dims(self, max_ctx=4096):
        d = Dims()
        if self.L.tlq_gguf_dims(self.h, max_ctx, C.byref(d)) != 0:
            raise RuntimeError(self.L.tlq_file_error().decode())
        return d

    def close(self):
        if self.h:
            self.L.tlq_gguf_close(self.h)
            self.h = None


class Tokenizer:
    """tl::tokenizer (byte-level BPE, vocabulary from a GGUF file's metadata). Host only."""

    def __init__(self, path):
        self.L = _load()
        self.h = self.L.tlq_tok_open(os.fsencode(path))
        if not self.h:
            raise RuntimeError(self.L.tlq_file_error().decode("latin-1"))
        bos, eos = cint(), cint()
        self.L.tlq_tok_special_ids(self.h, C.byref(bos), C.byref(eos))
        self.bos_id, self.eos_id = bos.value, eos.value

    def encode(self, text):
        raw = text.encode() if isinstance(text, str) else bytes(text)
        cap = 4 * len(raw) + 16
        out = np.empty(cap, np.int32)
        n = self.L.tlq_tok_encode(self.h, raw, len(raw), _p(out), cap)
        if n < 0:
            raise RuntimeError(self.L.tlq_file_error().decode("latin-1"))
        return [int(v) for v in out[:n]]

    def decode(self, ids):
        a = np.ascontiguousarray(ids, np.int32)
        cap = 64 * max(1, len(a)) + 64
        buf = C.create_string_buffer(cap)
        n = self.L.tlq_tok_decode(self.h, _p(a), len(a), buf, cap)
        if n < 0:
            raise RuntimeError(self.L.tlq_file_error().decode("latin-1"))
        assert n <= cap
        return buf.raw[:n]

    def close(self):
        if self.h:
            self.L.tlq_tok_close(self.h)
            self.h = None


class QwenGPU:
    """A decoder on the GPU. No CPU fallback: construction raises when the HIP
    backend is unavailable."""

    def __init__(self, dims):
        self.L = _load()
        if not self.L.tlq_available():
            raise RuntimeError("tl::hip backend unavailable: %s" % self.L.tlq_unavailable_reason().decode())
        self.d = Dims(**dims) if isinstance(dims, dict) else dims
        self.h = self.L.tlq_create(C.byref(self.d))
        if not self.h:
            raise RuntimeError("tlq_create failed")
        self._keep = []

    @classmethod
    def from_blobs(cls, om, fmt="q4"):
        """Build from a weight source: any object with `.d` (the dims) and
        `.weight(layer, name)` returning the stored bytes of wq/wk/wv/wo/wg/wu/wd (q4
        buffers, or bf16 in the logical [K,N] layout when fmt == "bf16"), bq/bk/bv/an/fn
        (f32) and, for layer -1, embed (bf16), onorm, outw."""
        d = om.d
        g = cls(dict((f, getattr(d, f)) for f, _ in Dims._fields_))
        set_layer = g.L.tlq_set_layer_q4 if fmt == "q4" else g.L.tlq_set_layer_bf16
        set_head = g.L.tlq_set_head_q4 if fmt == "q4" else g.L.tlq_set_head_bf16
        for li in range(d.n_layers):
            w = [np.ascontiguousarray(om.weight(li, n)) for n in ("wq", "wk", "wv", "wo", "wg", "wu", "wd")]
            v = [np.ascontiguousarray(om.weight(li, n)) for n in ("bq", "bk", "bv", "an", "fn")]
            if set_layer(g.h, li, *[_p(a) for a in w + v]) != 0:
                raise RuntimeError("set_layer(%d) failed" % li)
        emb = np.ascontiguousarray(om.weight(-1, "embed"))
        onorm = np.ascontiguousarray(om.weight(-1, "onorm"))
        outw = np.ascontiguousarray(om.weight(-1, "outw"))
        if set_head(g.h, _p(emb), _p(onorm), _p(outw)) != 0:
            raise RuntimeError("set_head failed")
        return g

    @classmethod
    def from_gguf(cls, path, fmt="q4", max_ctx=4096):
        """Build from a GGUF file: f16 / f32 / bf16 tensors are uploaded as stored and converted to
        int4 groups (fmt "q4") or bf16 rows (fmt "bf16") on the device."""
        g = cls.__new__(cls)
        g.L = _load()
        if not g.L.tlq_available():
            raise RuntimeError("tl::hip backend unavailable: %s" % g.L.tlq_unavailable_reason().decode())
        g.h = g.L.tlq_create_from_gguf(os.fsencode(path), 0 if fmt == "q4" else 1, max_ctx)
        if not g.h:
            raise RuntimeError("load_gguf failed: %s" % g.L.tlq_file_error().decode())
        g.d = Dims()
        g.L.tlq_get_dims(g.h, C.byref(g.d))
        g._keep = []
        return g

    def set_random(self, seed=1, fmt="q4"):
        fn = self.L.tlq_set_random_q4 if fmt == "q4" else self.L.tlq_set_random_bf16
        if fn(self.h, seed) != 0:
            raise RuntimeError("set_random failed")

    def prefill(self, tokens, chunk=512, want_logits=True):
        """Consume prompt tokens in chunks at the caches' current position; returns the
        last token's logits."""
        t = np.ascontiguousarray(tokens, np.int64)
        logits = np.empty(self.d.vocab, np.float32) if want_logits else None
        if self.L.tlq_prefill(self.h, _p(t), len(t), chunk, _p(logits) if want_logits else None) != 0:
            raise RuntimeError("prefill declined by the backend")
        return logits

    def stage_chunk(self, tokens):
        t = np.ascontiguousarray(tokens, np.int64)
        if self.L.tlq_stage_chunk(self.h, _p(t), len(t)) != 0:
            raise RuntimeError("stage_chunk failed")

    def prefill_layers(self, T, pos0):
        if self.L.tlq_prefill_layers(self.h, T, pos0) != 0:
            raise RuntimeError("prefill_layers declined by the backend")

    def set_cache_pos(self, pos):
        self.L.tlq_set_cache_pos(self.h, pos)

    def fill_cache_random(self, upto, seed=2):
        if self.L.tlq_fill_cache_random(self.h, upto, seed) != 0:
            raise RuntimeError("tlq_fill_cache_random failed")

    def cache_upload(self, layer, K, V, pos):
        """Overwrite a layer's f32 caches with [n_kv_heads, max_ctx, head_dim] arrays; every
        cache's position becomes pos."""
        K, V = np.ascontiguousarray(K, np.float32), np.ascontiguousarray(V, np.float32)
        want = self.d.n_kv_heads * self.d.max_ctx * self.d.head_dim
        assert K.size == want and V.size == want
        if self.L.tlq_cache_upload(self.h, layer, _p(K), _p(V), pos) != 0:
            raise RuntimeError("cache_upload failed")

    def prefill_hidden(self, T):
        """Final-norm rows [T, hidden] of the last chunk run."""
        out = np.empty((T, self.d.hidden), np.float32)
        if self.L.tlq_prefill_hidden(self.h, _p(out), T) != 0:
            raise RuntimeError("prefill_hidden: no chunk of that length was run")
        return out

    def step(self, token, pos, want_logits=False):
        logits = np.empty(self.d.vocab, np.float32) if want_logits else None
        tok = self.L.tlq_step(self.h, token, pos, _p(logits) if want_logits else None)
        if tok < 0:
            raise RuntimeError("decode step declined by the backend")
        return (int(tok), logits) if want_logits else int(tok)

    def run_layers(self, token, pos):
        if self.L.tlq_run_layers(self.h, token, pos) != 0:
            raise RuntimeError("run_layers declined by the backend")

    def argmax(self):
        return int(self.L.tlq_argmax(self.h))

    def capture(self, token, pos):
        if self.L.tlq_capture(self.h, token, pos) != 0:
            raise RuntimeError("graph capture failed")

    def replay(self):
        if self.L.tlq_replay(self.h) != 0:
            raise RuntimeError("graph replay failed")

    # ---- greedy decoding with the token loop on the device -----------------------------
    def greedy_init(self, first_id, pos):
        """Record ONE graph: embedding gather of the device token -> layers -> lm_head ->
        argmax -> device token; position and token history stay on the device."""
        if self.L.tlq_greedy_init(self.h, first_id, pos) != 0:
            raise RuntimeError("greedy loop: graph capture failed")

    def greedy_run(self, n):
        """Queue n greedy steps back to back (no sync); returns how many were queued."""
        return int(self.L.tlq_greedy_run(self.h, n))

    def greedy_tokens(self, start, n):
        """Tokens generated at positions [start, start+n) (blocks until they exist)."""
        out = np.empty(n, np.int32)
        if self.L.tlq_greedy_tokens(self.h, start, n, _p(out)) != 0:
            raise RuntimeError("greedy_tokens: range not generated yet")
        return out

    def greedy_sync_host_pos(self):
        self.L.tlq_greedy_sync_host_pos(self.h)

    # ---- a decode loop on ONE recorded graph, position kept on the device ----------
    def decoder_init(self, first_id, pos):
        """Record the forward at `pos`; returns True when a graph was captured (otherwise
        feed/step run the imperative path)."""
        self.L.tlq_decoder_init(self.h, first_id, pos)
        return bool(self.L.tlq_decoder_captured(self.h))

    def decoder_feed(self, token):
        if self.L.tlq_decoder_feed(self.h, token) != 0:
            raise RuntimeError("decoder feed failed (cache full or launch declined)")

    def decoder_step(self, token, want_logits=False):
        logits = np.empty(self.d.vocab, np.float32) if want_logits else None
        tok = self.L.tlq_decoder_step(self.h, token, _p(logits) if want_logits else None)
        if tok < 0:
            raise RuntimeError("decoder step failed (cache full or launch declined)")
        return (int(tok), logits) if want_logits else int(tok)

    def decoder_pos(self):
        return int(self.L.tlq_decoder_pos(self.h))

    def decoder_sync_host_pos(self):
        self.L.tlq_decoder_sync_host_pos(self.h)

    def set_fused(self, on):
        self.L.tlq_set_fused(self.h, 1 if on else 0)

    def profile_steps(self, token, pos, n=5):
        """GPU microseconds per region of the fused decode step (events between the launches of
        n eager steps): per layer qkv / attention / o-proj / gate|up / down, then the LM head and the step."""
        out = (C.c_double * 7)()
        if self.L.tlq_profile_steps(self.h, token, pos, n, out) != 0:
            raise RuntimeError("profile_steps: a launch or an event was declined")
        names = ("qkv_gemv", "attention", "o_proj_gemv", "gateup_gemv", "down_gemv", "lm_head", "step")
        return {k: float(v) for k, v in zip(names, out)}

    def set_warm(self, blocks, nt=False, mode=0):
        """Within the fused path: weight warm-up reads on a second stream beside each layer (0 blocks = off)."""
        self.L.tlq_set_warm(self.h, int(blocks), 1 if nt else 0, int(mode))

    def set_fused_attn(self, on):
        """Within the fused path: run the q/k/v epilogue inside the attention launch (default) or alone."""
        self.L.tlq_set_fused_attn(self.h, 1 if on else 0)

    def set_norm_images(self, on):
        """Prompt chunks: let the residual norms leave the activation image of their output for the
        prepared-weight product that reads it (default), or let every product cut its own."""
        self.L.tlq_set_norm_images(self.h, 1 if on else 0)

    def set_merge_in_oproj(self, on):
        """Within the fused attention: let the o-projection's GEMV merge the attention's splits where
        the launch plan makes few of them (default), or always run the merge launch."""
        self.L.tlq_set_merge_in_oproj(self.h, 1 if on else 0)

    def set_fused_prefill(self, on):
        """Prompt chunks: one launch for split_heads + rope + kv_fill and token-major attention output (default), or the reference's op sequence."""
        self.L.tlq_set_fused_prefill(self.h, 1 if on else 0)

    def set_prompt_f16(self, on):
        """Prompt chunks of bf16 weights: on their prepared f16 images (default; a second copy of the weights, made on the first chunk) or on the bf16 rows."""
        self.L.tlq_set_prompt_f16(self.h, 1 if on else 0)

    def set_gateup_epilogue(self, on):
        """Within the fused path: swiglu as the epilogue of the gate|up GEMV (default) or as the producer of the down GEMV."""
        self.L.tlq_set_gateup_epilogue(self.h, 1 if on else 0)

    def flush(self):
        self.L.tlq_flush()

    def census(self):
        from .capi import CENSUS
        buf = (C.c_uint64 * len(CENSUS))()
        self.L.tlq_census(buf, len(CENSUS))
        return dict(zip(CENSUS, [int(v) for v in buf]))

    def close(self):
        if self.h:
            self.L.tlq_destroy(self.h)
            self.h = None
