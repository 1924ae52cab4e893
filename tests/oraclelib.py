"""ctypes bindings for the CHECKER libraries (test infrastructure only).

`oracle`  -> oracle/liboracle.so, the plain-C restatement of the reference CPU
             path (oracle/oracle.c).
`ref`     -> oracle/_ref/libtlref.so, the real reference's CPU path behind a C
             ABI (oracle/ref_shim.cpp); None where it has not been built.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import
this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")

i64, f32, u32, cint = C.c_int64, C.c_float, C.c_uint32, C.c_int
P = C.c_void_p


def _ptr(a):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"], "need contiguous ndarray"
    return a.ctypes.data_as(P)


class QwenDims(C.Structure):
    _fields_ = [("n_layers", i64), ("hidden", i64), ("n_q_heads", i64), ("n_kv_heads", i64),
                ("head_dim", i64), ("ff", i64), ("vocab", i64), ("max_ctx", i64),
                ("eps", f32), ("rope_base", f32)]


QWEN_05B = dict(n_layers=24, hidden=896, n_q_heads=14, n_kv_heads=2, head_dim=64, ff=4864,
                vocab=151936, max_ctx=512, eps=1e-6, rope_base=1e6)
QWEN_7B = dict(n_layers=28, hidden=3584, n_q_heads=28, n_kv_heads=4, head_dim=128, ff=18944,
               vocab=152064, max_ctx=4352, eps=1e-6, rope_base=1e6)


def build_oracle(force=False):
    so = os.path.join(ORACLE_DIR, "liboracle.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "liboracle.so"])
    return so


class Oracle:
    def __init__(self):
        self.lib = L = C.CDLL(build_oracle())
        sig = {
            "orc_fill_normal": (None, [P, i64, u32, f32, f32]),
            "orc_fill_uniform": (None, [P, i64, u32, f32, f32]),
            "orc_fill_q4": (None, [P, i64, i64, u32, f32, f32]),
            "orc_crc32": (u32, [P, i64]),
            "orc_to_bf16": (None, [P, P, i64]),
            "orc_bf16_widen": (None, [P, P, i64]),
            "orc_q4_bytes": (i64, [i64, i64]),
            "orc_to_q4": (cint, [P, i64, i64, i64, i64, P]),
            "orc_q4_to_f32": (None, [P, i64, i64, P]),
            "orc_sgemm": (None, [P, i64, i64, P, i64, i64, P, i64, i64, i64, f32]),
            "orc_ref_dot": (None, [P, i64, i64, P, i64, i64, P, i64, i64, i64]),
            "orc_dot": (None, [P, P, P, i64, i64, i64, f32, f32]),
            "orc_gemv_q4": (None, [P, P, P, i64, i64, f32, f32, P]),
            "orc_gemv_bf16": (None, [P, P, P, i64, i64, f32, f32, P]),
            "orc_gemv_bf16_row": (None, [P, P, P, i64, i64, P]),
            "orc_gemm_bf16_nt": (None, [P, P, P, i64, i64, i64, P]),
            "orc_attn_decode": (None, [P, P, P, P, i64, i64, i64, i64, i64, f32]),
            "orc_attn_prefill": (None, [P, P, P, P, i64, i64, i64, i64, i64, f32, i64]),
            "orc_rope": (None, [P, P, P, i64, i64, i64, i64, f32]),
            "orc_binary": (None, [cint, P, P, P, i64, f32, f32]),
            "orc_binary_bcast": (None, [cint, P, i64, i64, P, i64, i64, P, i64, i64, f32, f32]),
            "orc_unary": (None, [cint, P, P, i64, f32, f32]),
            "orc_row_sum": (None, [P, P, i64, i64, f32, f32]),
            "orc_row_max": (None, [P, P, i64, i64, f32, f32]),
            "orc_softmax": (None, [P, P, i64, i64]),
            "orc_rmsnorm": (None, [P, P, P, i64, i64, f32]),
            "orc_rmsnorm_res": (None, [P, P, P, P, P, i64, i64, f32]),
            "orc_silu": (None, [P, P, i64]),
            "orc_swiglu": (None, [P, P, P, i64]),
            "orc_swiglu_fused": (None, [P, P, i64, i64]),
            "orc_argmax": (i64, [P, i64]),
            "orc_kv_append": (None, [P, P, P, P, i64, i64, i64, i64]),
            "orc_kv_fill": (None, [P, P, P, P, i64, i64, i64, i64, i64]),
            "orc_split_heads": (None, [P, P, P, i64, i64, i64, i64, i64]),
            "orc_merge_heads": (None, [P, P, i64, i64, i64]),
            "orc_qwen_create": (P, [C.POINTER(QwenDims), u32, cint]),
            "orc_qwen_destroy": (None, [P]),
            "orc_qwen_step": (i64, [P, i64, i64, P]),
            "orc_qwen_weight": (P, [P, i64, C.c_char_p, C.POINTER(i64)]),
            "orc_qwen_set": (cint, [P, i64, C.c_char_p, P]),
            "orc_qwen_cache": (P, [P, i64, cint]),
            "orc_f16_widen": (None, [P, P, i64]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args

    # ---- seeded inputs --------------------------------------------------
    def normal(self, n, seed, mean=0.0, std=1.0):
        a = np.empty(int(n), np.float32)
        self.lib.orc_fill_normal(_ptr(a), a.size, seed, mean, std)
        return a

    def uniform(self, n, seed, lo=0.0, hi=1.0):
        a = np.empty(int(n), np.float32)
        self.lib.orc_fill_uniform(_ptr(a), a.size, seed, lo, hi)
        return a

    def fill_q4(self, N, K, seed, lo=0.005, hi=0.02):
        buf = np.empty(self.q4_bytes(N, K), np.uint8)
        self.lib.orc_fill_q4(_ptr(buf), N, K, seed, lo, hi)
        return buf

    def crc32(self, a):
        a = np.ascontiguousarray(a)
        return int(self.lib.orc_crc32(_ptr(a), a.nbytes))

    # ---- formats ---------------------------------------------------------
    def q4_bytes(self, N, K):
        return int(self.lib.orc_q4_bytes(N, K))

    def to_q4(self, w):
        """w: [K,N] f32 (any strides) -> packed buffer (uint8)."""
        K, N = w.shape
        out = np.empty(self.q4_bytes(N, K), np.uint8)
        s0, s1 = (s // 4 for s in w.strides)
        rc = self.lib.orc_to_q4(C.c_void_p(w.ctypes.data), s0, s1, K, N, _ptr(out))
        if rc != 0:
            raise ValueError("to_q4: K must be a multiple of 32")
        return out

    def q4_to_f32(self, buf, K, N):
        out = np.empty((K, N), np.float32)
        self.lib.orc_q4_to_f32(_ptr(buf), K, N, _ptr(out))
        return out

    def to_bf16(self, a):
        a = np.ascontiguousarray(a, np.float32)
        out = np.empty(a.shape, np.uint16)
        self.lib.orc_to_bf16(_ptr(a), _ptr(out), a.size)
        return out

    def f16_widen(self, a):
        """IEEE half bit patterns (uint16) -> float32, the model loader's widening."""
        a = np.ascontiguousarray(a, np.uint16)
        out = np.empty(a.shape, np.float32)
        self.lib.orc_f16_widen(_ptr(a), _ptr(out), a.size)
        return out

    def bf16_widen(self, a):
        a = np.ascontiguousarray(a, np.uint16)
        out = np.empty(a.shape, np.float32)
        self.lib.orc_bf16_widen(_ptr(a), _ptr(out), a.size)
        return out

    # ---- matmul ----------------------------------------------------------
    def sgemm(self, A, B, alpha=1.0):
        m, k = A.shape
        n = B.shape[1]
        Cc = np.empty((m, n), np.float32)
        self.lib.orc_sgemm(C.c_void_p(A.ctypes.data), A.strides[0] // 4, A.strides[1] // 4,
                           C.c_void_p(B.ctypes.data), B.strides[0] // 4, B.strides[1] // 4,
                           _ptr(Cc), m, n, k, alpha)
        return Cc

    def ref_dot(self, A, B):
        m, k = A.shape
        n = B.shape[1]
        Cc = np.empty((m, n), np.float32)
        self.lib.orc_ref_dot(C.c_void_p(A.ctypes.data), A.strides[0] // 4, A.strides[1] // 4,
                             C.c_void_p(B.ctypes.data), B.strides[0] // 4, B.strides[1] // 4,
                             _ptr(Cc), m, n, k)
        return Cc

    def dot(self, A, B, scale=1.0, offset=0.0):
        A = np.ascontiguousarray(A, np.float32)
        B = np.ascontiguousarray(B, np.float32)
        m, k = A.shape
        n = B.shape[1]
        Cc = np.empty((m, n), np.float32)
        self.lib.orc_dot(_ptr(A), _ptr(B), _ptr(Cc), m, n, k, scale, offset)
        return Cc

    def gemv_q4(self, a, buf, N, K, scale=1.0, offset=0.0):
        y = np.empty(N, np.float32)
        self.lib.orc_gemv_q4(_ptr(a), _ptr(buf), _ptr(y), N, K, scale, offset, None)
        return y

    def gemv_bf16(self, a, B, scale=1.0, offset=0.0):
        K, N = B.shape
        y = np.empty(N, np.float32)
        self.lib.orc_gemv_bf16(_ptr(a), _ptr(B), _ptr(y), N, K, scale, offset, None)
        return y

    def gemv_bf16_row(self, a, W):
        N, K = W.shape
        y = np.empty(N, np.float32)
        self.lib.orc_gemv_bf16_row(_ptr(a), _ptr(W), _ptr(y), N, K, None)
        return y

    def gemm_bf16_nt(self, A, W):
        M, K = A.shape
        N = W.shape[0]
        out = np.empty((M, N), np.float32)
        self.lib.orc_gemm_bf16_nt(_ptr(A), _ptr(W), _ptr(out), M, N, K, None)
        return out

    # ---- attention / rope --------------------------------------------------
    def attn_decode(self, q, K, V, scale, ctx=None):
        Hq, D = q.shape
        Hkv, kv_max, _ = K.shape
        ctx = kv_max if ctx is None else ctx
        out = np.empty((Hq, D), np.float32)
        self.lib.orc_attn_decode(_ptr(q), _ptr(K), _ptr(V), _ptr(out), Hq, Hkv, ctx, kv_max, D,
                                 scale)
        return out

    def attn_prefill(self, q, K, V, scale, pos0=0):
        Hq, T, D = q.shape
        Hkv, kv_max, _ = K.shape
        out = np.empty((Hq, T, D), np.float32)
        self.lib.orc_attn_prefill(_ptr(q), _ptr(K), _ptr(V), _ptr(out), Hq, Hkv, T, kv_max, D,
                                  scale, pos0)
        return out

    def rope(self, x, pos, base, T=1, bias=None):
        D = x.shape[-1]
        rows = x.size // D
        out = np.empty_like(x)
        self.lib.orc_rope(_ptr(x), _ptr(bias), _ptr(out), rows, T, D, pos, base)
        return out

    # ---- elementwise -------------------------------------------------------
    OPS = dict(add=0, sub=1, mul=2, div=3, pow=4, exp=5, log=6, sqrt=7, sigmoid=8, relu=9,
               affine=10, recip=11)

    def binary(self, op, a, b, scale=1.0, offset=0.0):
        out = np.empty_like(a)
        self.lib.orc_binary(self.OPS[op], _ptr(a), _ptr(b), _ptr(out), a.size, scale, offset)
        return out

    def binary_bcast(self, op, a, astr, b, bstr, m, n, scale=1.0, offset=0.0):
        out = np.empty((m, n), np.float32)
        self.lib.orc_binary_bcast(self.OPS[op], _ptr(a), astr[0], astr[1], _ptr(b), bstr[0],
                                  bstr[1], _ptr(out), m, n, scale, offset)
        return out

    def unary(self, op, a, scale=1.0, offset=0.0):
        out = np.empty_like(a)
        self.lib.orc_unary(self.OPS[op], _ptr(a), _ptr(out), a.size, scale, offset)
        return out

    def row_sum(self, x, scale=1.0, offset=0.0):
        rows, cols = x.shape
        out = np.empty(rows, np.float32)
        self.lib.orc_row_sum(_ptr(x), _ptr(out), rows, cols, scale, offset)
        return out

    def row_max(self, x, scale=1.0, offset=0.0):
        rows, cols = x.shape
        out = np.empty(rows, np.float32)
        self.lib.orc_row_max(_ptr(x), _ptr(out), rows, cols, scale, offset)
        return out

    def softmax(self, x):
        rows, cols = x.shape
        out = np.empty_like(x)
        self.lib.orc_softmax(_ptr(x), _ptr(out), rows, cols)
        return out

    def rmsnorm(self, x, w, eps):
        rows, n = x.shape
        out = np.empty_like(x)
        self.lib.orc_rmsnorm(_ptr(x), _ptr(w), _ptr(out), rows, n, eps)
        return out

    def rmsnorm_res(self, x, delta, w, eps):
        rows, n = x.shape
        xo, ho = np.empty_like(x), np.empty_like(x)
        self.lib.orc_rmsnorm_res(_ptr(x), _ptr(delta), _ptr(w), _ptr(xo), _ptr(ho), rows, n, eps)
        return xo, ho

    def silu(self, x):
        out = np.empty_like(x)
        self.lib.orc_silu(_ptr(x), _ptr(out), x.size)
        return out

    def swiglu(self, g, u):
        out = np.empty_like(g)
        self.lib.orc_swiglu(_ptr(g), _ptr(u), _ptr(out), g.size)
        return out

    def swiglu_fused(self, gu, ff):
        rows = gu.size // (2 * ff)
        out = np.empty((rows, ff), np.float32)
        self.lib.orc_swiglu_fused(_ptr(gu), _ptr(out), ff, rows)
        return out

    def argmax(self, v):
        return int(self.lib.orc_argmax(_ptr(v), v.size))

    # ---- decode model --------------------------------------------------------
    def qwen_create(self, dims, seed, q4=True):
        d = QwenDims(**dims)
        return OracleQwen(self, d, self.lib.orc_qwen_create(C.byref(d), seed, 1 if q4 else 0), q4)


class OracleQwen:
    LIN = ("wq", "wk", "wv", "wo", "wg", "wu", "wd")
    VEC = ("bq", "bk", "bv", "an", "fn")

    def __init__(self, orc, dims, handle, q4):
        self.orc, self.d, self.h, self.q4 = orc, dims, handle, q4

    def close(self):
        if self.h:
            self.orc.lib.orc_qwen_destroy(self.h)
            self.h = None

    def step(self, token, pos):
        logits = np.empty(self.d.vocab, np.float32)
        tok = self.orc.lib.orc_qwen_step(self.h, token, pos, _ptr(logits))
        return int(tok), logits

    def cache(self, layer):
        """The host K and V caches of a layer as writable [n_kv_heads, max_ctx, head_dim] views."""
        d = self.d
        n = d.n_kv_heads * d.max_ctx * d.head_dim
        out = []
        for which in (0, 1):
            p = self.orc.lib.orc_qwen_cache(self.h, layer, which)
            buf = (C.c_float * n).from_address(p)
            out.append(np.frombuffer(buf, np.float32).reshape(d.n_kv_heads, d.max_ctx, d.head_dim))
        return out

    def set(self, layer, name, data):
        """Replace a weight: linear layers as f32 in the logical [K,N] layout (stored in the model's
        format like the seeded ones), vectors f32, layer -1: embed f32 [vocab, hidden], onorm, outw."""
        a = np.ascontiguousarray(data, np.float32)
        if self.orc.lib.orc_qwen_set(self.h, layer, name.encode(), _ptr(a)) != 0:
            raise KeyError(name)

    def weight(self, layer, name):
        """Stored bytes of a weight as a numpy view (uint8 for linear weights and the
        bf16 embedding, float32 for vectors)."""
        nb = i64(0)
        p = self.orc.lib.orc_qwen_weight(self.h, layer, name.encode(), C.byref(nb))
        if not p:
            raise KeyError(name)
        buf = (C.c_uint8 * nb.value).from_address(p)
        a = np.frombuffer(buf, np.uint8)
        if name in self.VEC or name == "onorm":
            return a.view(np.float32)
        return a

    def lin_shape(self, name):
        d = self.d
        QD, KD = d.n_q_heads * d.head_dim, d.n_kv_heads * d.head_dim
        return {"wq": (d.hidden, QD), "wk": (d.hidden, KD), "wv": (d.hidden, KD),
                "wo": (QD, d.hidden), "wg": (d.hidden, d.ff), "wu": (d.hidden, d.ff),
                "wd": (d.ff, d.hidden), "outw": (d.hidden, d.vocab)}[name]


class Ref:
    """The real reference CPU path (oracle/_ref/libtlref.so)."""

    def __init__(self, path):
        self.lib = L = C.CDLL(path)
        sig = {
            "tlref_init": (cint, []),
            "tlref_set_cpu_gemm": (None, [cint]),
            "tlref_q4_bytes": (i64, [i64, i64]),
            "tlref_to_q4": (None, [P, i64, i64, P]),
            "tlref_q4_to_f32": (None, [P, i64, i64, P]),
            "tlref_to_bf16": (None, [P, P, i64]),
            "tlref_bf16_to_f32": (None, [P, P, i64]),
            "tlref_dot": (None, [P, P, P, i64, i64, i64, f32, f32]),
            "tlref_gemv_q4": (None, [P, P, P, i64, i64]),
            "tlref_gemv_bf16": (None, [P, P, P, i64, i64]),
            "tlref_gemv_q4_prepare": (P, [P, P, i64, i64]),
            "tlref_gemv_bf16_prepare": (P, [P, P, i64, i64]),
            "tlref_gemv_run": (None, [P, P]),
            "tlref_gemv_free": (None, [P]),
            "tlref_attn_decode": (None, [P, P, P, P, i64, i64, i64, f32]),
            "tlref_rope": (None, [P, P, i64, i64, i64, i64, f32]),
            "tlref_rmsnorm": (None, [P, P, P, i64, i64, f32]),
            "tlref_silu": (None, [P, P, i64]),
            "tlref_swiglu": (None, [P, P, P, i64]),
            "tlref_softmax": (None, [P, P, i64, i64]),
            "tlref_row_sum": (None, [P, P, i64, i64, f32, f32]),
            "tlref_row_mean": (None, [P, P, i64, i64]),
            "tlref_row_max": (None, [P, P, i64, i64]),
            "tlref_binary": (None, [cint, P, i64, i64, P, i64, i64, P, f32, f32]),
            "tlref_unary": (None, [cint, P, P, i64, f32, f32]),
            "tlref_argmax": (i64, [P, i64]),
            "tlref_qwen_create": (P, [C.POINTER(QwenDims)]),
            "tlref_qwen_destroy": (None, [P]),
            "tlref_qwen_set": (cint, [P, i64, C.c_char_p, P, cint, i64, i64, cint]),
            "tlref_qwen_step": (i64, [P, i64, i64, P]),
            "tlref_gguf_dump": (i64, [C.c_char_p, C.c_char_p, i64]),
            "tlref_tok_open": (P, [C.c_char_p]),
            "tlref_tok_close": (None, [P]),
            "tlref_tok_special_ids": (None, [P, C.POINTER(cint), C.POINTER(cint)]),
            "tlref_tok_encode": (i64, [P, C.c_char_p, i64, P, i64]),
            "tlref_tok_decode": (i64, [P, P, i64, C.c_char_p, i64]),
            "tlref_unicode_class": (cint, [u32]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        L.tlref_init()

    def tokenizer(self, path):
        return RefTokenizer(self, path)

    def unicode_class(self, cp):
        return int(self.lib.tlref_unicode_class(cp))

    def gguf_dump(self, path):
        """Canonical text of a GGUF file as the reference's reader parses it; None when it throws."""
        n = self.lib.tlref_gguf_dump(os.fsencode(path), None, 0)
        if n < 0:
            return None
        buf = C.create_string_buffer(n + 1)
        self.lib.tlref_gguf_dump(os.fsencode(path), buf, n + 1)
        return buf.value.decode("latin-1")

    def to_q4(self, w):
        w = np.ascontiguousarray(w, np.float32)
        K, N = w.shape
        out = np.empty(int(self.lib.tlref_q4_bytes(N, K)), np.uint8)
        self.lib.tlref_to_q4(_ptr(w), K, N, _ptr(out))
        return out

    def q4_to_f32(self, buf, K, N):
        out = np.empty((K, N), np.float32)
        self.lib.tlref_q4_to_f32(_ptr(buf), K, N, _ptr(out))
        return out

    def to_bf16(self, a):
        a = np.ascontiguousarray(a, np.float32)
        out = np.empty(a.shape, np.uint16)
        self.lib.tlref_to_bf16(_ptr(a), _ptr(out), a.size)
        return out

    def bf16_to_f32(self, a):
        out = np.empty(a.shape, np.float32)
        self.lib.tlref_bf16_to_f32(_ptr(a), _ptr(out), a.size)
        return out

    def dot(self, A, B, scale=1.0, offset=0.0):
        A = np.ascontiguousarray(A, np.float32)
        B = np.ascontiguousarray(B, np.float32)
        m, k = A.shape
        n = B.shape[1]
        out = np.empty((m, n), np.float32)
        self.lib.tlref_dot(_ptr(A), _ptr(B), _ptr(out), m, n, k, scale, offset)
        return out

    def gemv_q4(self, a, buf, N, K):
        y = np.empty(N, np.float32)
        self.lib.tlref_gemv_q4(_ptr(a), _ptr(buf), _ptr(y), N, K)
        return y

    def gemv_bf16(self, a, B):
        K, N = B.shape
        y = np.empty(N, np.float32)
        self.lib.tlref_gemv_bf16(_ptr(a), _ptr(B), _ptr(y), N, K)
        return y

    def attn_decode(self, q, K, V, scale):
        H, D = q.shape
        ctx = K.shape[1]
        out = np.empty((H, D), np.float32)
        self.lib.tlref_attn_decode(_ptr(q), _ptr(K), _ptr(V), _ptr(out), H, ctx, D, scale)
        return out

    def rope(self, x, pos, base):
        H, D = x.shape[0], x.shape[-1]
        T = x.shape[1] if x.ndim == 3 else 1
        out = np.empty_like(x)
        self.lib.tlref_rope(_ptr(x), _ptr(out), H, T, D, pos, base)
        return out

    def rmsnorm(self, x, w, eps):
        rows, n = x.shape
        out = np.empty_like(x)
        self.lib.tlref_rmsnorm(_ptr(x), _ptr(w), _ptr(out), rows, n, eps)
        return out

    def silu(self, x):
        out = np.empty_like(x)
        self.lib.tlref_silu(_ptr(x), _ptr(out), x.size)
        return out

    def swiglu(self, g, u):
        out = np.empty_like(g)
        self.lib.tlref_swiglu(_ptr(g), _ptr(u), _ptr(out), g.size)
        return out

    def softmax(self, x):
        out = np.empty_like(x)
        self.lib.tlref_softmax(_ptr(x), _ptr(out), x.shape[0], x.shape[1])
        return out

    def row_sum(self, x, scale=1.0, offset=0.0):
        out = np.empty(x.shape[0], np.float32)
        self.lib.tlref_row_sum(_ptr(x), _ptr(out), x.shape[0], x.shape[1], scale, offset)
        return out

    def row_mean(self, x):
        out = np.empty(x.shape[0], np.float32)
        self.lib.tlref_row_mean(_ptr(x), _ptr(out), x.shape[0], x.shape[1])
        return out

    def row_max(self, x):
        out = np.empty(x.shape[0], np.float32)
        self.lib.tlref_row_max(_ptr(x), _ptr(out), x.shape[0], x.shape[1])
        return out

    def binary(self, op, a, b, scale=1.0, offset=0.0):
        a2 = a.reshape(1, -1) if a.ndim == 1 else a
        b2 = b.reshape(1, -1) if b.ndim == 1 else b
        m = max(a2.shape[0], b2.shape[0])
        n = max(a2.shape[1], b2.shape[1])
        out = np.empty((m, n), np.float32)
        self.lib.tlref_binary(Oracle.OPS[op], _ptr(a2), a2.shape[0], a2.shape[1], _ptr(b2),
                              b2.shape[0], b2.shape[1], _ptr(out), scale, offset)
        return out

    def unary(self, op, a, scale=1.0, offset=0.0):
        out = np.empty_like(a)
        self.lib.tlref_unary(Oracle.OPS[op], _ptr(a), _ptr(out), a.size, scale, offset)
        return out

    def argmax(self, v):
        return int(self.lib.tlref_argmax(_ptr(v), v.size))

    def qwen_from_oracle(self, om, predeq=True):
        """Build the reference-side decode model around the oracle model's weight bytes."""
        d = om.d
        h = self.lib.tlref_qwen_create(C.byref(d))
        kind = 1 if om.q4 else 2
        keep = []

        def put(li, name, arr, k, K=0, N=0):
            keep.append(arr)
            rc = self.lib.tlref_qwen_set(h, li, name.encode(), _ptr(arr), k, K, N, 1 if predeq else 0)
            assert rc == 0, name

        put(-1, "embed", om.weight(-1, "embed").copy(), 3, d.vocab, d.hidden)
        put(-1, "onorm", om.weight(-1, "onorm").copy(), 0, 0, d.hidden)
        K, N = om.lin_shape("outw")
        put(-1, "outw", om.weight(-1, "outw").copy(), kind, K, N)
        for li in range(d.n_layers):
            for nm in OracleQwen.LIN:
                K, N = om.lin_shape(nm)
                put(li, nm, om.weight(li, nm).copy(), kind, K, N)
            for nm in OracleQwen.VEC:
                v = om.weight(li, nm).copy()
                put(li, nm, v, 0, 0, v.size)
        return RefQwen(self, h, d)


class RefTokenizer:
    """The reference's tl::tokenizer; encode / decode return None where it throws."""

    def __init__(self, ref, path):
        self.lib = ref.lib
        self.h = self.lib.tlref_tok_open(os.fsencode(path))
        if not self.h:
            raise RuntimeError("reference tokenizer rejected " + path)
        bos, eos = cint(), cint()
        self.lib.tlref_tok_special_ids(self.h, C.byref(bos), C.byref(eos))
        self.bos_id, self.eos_id = bos.value, eos.value

    def encode(self, raw):
        cap = 4 * len(raw) + 16
        out = np.empty(cap, np.int32)
        n = self.lib.tlref_tok_encode(self.h, raw, len(raw), _ptr(out), cap)
        return None if n < 0 else [int(v) for v in out[:n]]

    def decode(self, ids):
        a = np.ascontiguousarray(ids, np.int32)
        cap = 64 * max(1, len(a)) + 64
        buf = C.create_string_buffer(cap)
        n = self.lib.tlref_tok_decode(self.h, _ptr(a), len(a), buf, cap)
        return None if n < 0 else buf.raw[:n]

    def close(self):
        self.lib.tlref_tok_close(self.h)


class RefQwen:
    def __init__(self, ref, h, d):
        self.ref, self.h, self.d = ref, h, d

    def step(self, token, pos):
        logits = np.empty(self.d.vocab, np.float32)
        tok = self.ref.lib.tlref_qwen_step(self.h, token, pos, _ptr(logits))
        return int(tok), logits

    def close(self):
        if self.h:
            self.ref.lib.tlref_qwen_destroy(self.h)
            self.h = None


_oracle = None
_ref = False


def oracle():
    global _oracle
    if _oracle is None:
        _oracle = Oracle()
    return _oracle


def ref():
    """The compiled reference, or None when oracle/_ref has not been built."""
    global _ref
    if _ref is False:
        path = os.path.join(ORACLE_DIR, "_ref", "libtlref.so")
        _ref = Ref(path) if os.path.exists(path) else None
    return _ref


def allclose(got, want, rtol=1e-4, atol=1e-5):
    """The reference's allclose (array.h:2538-2547): |a-b| <= atol + rtol*|b|."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return bool(np.all(np.abs(got - want) <= atol + rtol * np.abs(want)))


def maxrel(got, want):
    """check_attn64.cpp:122: max |d| / (1 + |ref|)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float(np.max(np.abs(got - want) / (1.0 + np.abs(want)))) if got.size else 0.0


def check_logits(got, want, maxrel_bar, label="", min_frac=0.0, rtol=1e-4, atol=1e-5):
    """A model-level result against the oracle, at two bars. The task's bar is allclose(rtol 1e-4,
    atol 1e-5) element by element: the fraction of elements inside it and the worst element (in units
    of its own tolerance) are printed, and the fraction must reach min_frac. The reference's own bar
    for chained layers is max |d| / (1 + |ref|) (check_llm_decode.cpp:268-276, check_llm_block.cpp:242):
    it must stay under maxrel_bar, which each test sets to a few times the value it measures. Both
    sides are fp32 evaluations of the same chain in different summation orders, so an element near
    zero can miss its atol on either side without anything being wrong; that is why the fraction, not
    every element, is asserted at model level (the kernel-level tests assert allclose on everything)."""
    got = np.asarray(got, np.float64).ravel()
    want = np.asarray(want, np.float64).ravel()
    d = np.abs(got - want)
    units = d / (atol + rtol * np.abs(want))
    frac = float(np.mean(units <= 1.0))
    i = int(np.argmax(units))
    mr = float(np.max(d / (1.0 + np.abs(want))))
    print("   %s maxrel %.2e (bar %.1e)  allclose(%.0e, %.0e): %.5f of %d, worst %.2f tolerances at [%d] got %.6g want %.6g"
          % (label, mr, maxrel_bar, rtol, atol, frac, got.size, float(units[i]), i, got[i], want[i]), flush=True)
    assert np.all(np.isfinite(got)), label
    assert mr < maxrel_bar, (label, mr, maxrel_bar)
    assert frac >= min_frac, (label, frac, min_frac)
    return mr, frac
