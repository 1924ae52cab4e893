"""ctypes binding of libtensorlib_hip.so (include/tensorlib_hip.h).

This is the Python-side view of the C ABI used by the tests, bench.py and
__graft_entry__.py. It adds nothing to the library: every method is one C call
plus error translation. There is no CPU fallback here or anywhere below it — a
missing library or a missing GPU raises.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libtensorlib_hip.so")

i64, f32, cint, u32, u64, sz = C.c_int64, C.c_float, C.c_int, C.c_uint32, C.c_uint64, C.c_size_t
P = C.c_void_p

OK, ENODEVICE, EINVAL, EUNSUPPORTED, ENOMEM, ERUNTIME = 0, -1, -2, -3, -4, -5

OPS = dict(add=0, sub=1, mul=2, div=3, pow=4, exp=5, log=6, sqrt=7, sigmoid=8, relu=9, affine=10,
           badd=11, bsub=12, bmul=13, bdiv=14, bpow=15, softmax=26, row_sum=27, row_max=28,
           recip=64)

CENSUS = ["binary", "bcast", "unary", "row_op", "gemm", "gemv_f32", "gemv_bf16", "gemv_bf16_row",
          "gemv_q4", "attn_decode", "rope", "rmsnorm", "rmsnorm_res", "swiglu", "argmax",
          "kv_append", "kv_fill", "split_heads", "merge_heads", "gemm_bf16_nt", "attn_prefill",
          "convert", "quantize_q4"]

# name -> (restype, argtypes): exactly the declarations of include/tensorlib_hip.h
SIGNATURES = {
    "tlhip_init": (cint, [cint]),
    "tlhip_abi_version": (cint, []),
    "tlhip_arch": (C.c_char_p, []),
    "tlhip_last_error": (C.c_char_p, []),
    "tlhip_device_info": (cint, [C.POINTER(cint), C.POINTER(i64), C.POINTER(cint)]),
    "tlhip_malloc": (cint, [C.POINTER(P), sz]),
    "tlhip_free": (cint, [P]),
    "tlhip_host_alloc": (cint, [C.POINTER(P), sz]),
    "tlhip_host_free": (cint, [P]),
    "tlhip_memcpy_h2d": (cint, [P, P, sz]),
    "tlhip_memcpy_d2h": (cint, [P, P, sz]),
    "tlhip_memcpy_h2d_async": (cint, [P, P, sz]),
    "tlhip_memcpy_d2d_async": (cint, [P, P, sz]),
    "tlhip_fill_u32": (cint, [P, u32, sz]),
    "tlhip_sync": (cint, []),
    "tlhip_graph_begin": (cint, []),
    "tlhip_graph_end": (cint, [C.POINTER(P)]),
    "tlhip_graph_launch": (cint, [P]),
    "tlhip_graph_destroy": (cint, [P]),
    "tlhip_event_create": (cint, [C.POINTER(P)]),
    "tlhip_event_record": (cint, [P]),
    "tlhip_event_elapsed_ms": (cint, [P, P, C.POINTER(f32)]),
    "tlhip_event_destroy": (cint, [P]),
    "tlhip_census": (cint, [C.POINTER(u64), cint]),
    "tlhip_census_reset": (cint, []),
    "tlhip_binary": (cint, [cint, P, i64, P, i64, P, i64, i64, f32, f32]),
    "tlhip_binary_bcast": (cint, [cint, P, i64, i64, i64, P, i64, i64, i64, P, i64, i64, i64, f32, f32]),
    "tlhip_unary": (cint, [cint, P, i64, P, i64, i64, f32, f32]),
    "tlhip_row_op": (cint, [cint, P, i64, P, i64, i64, i64, f32, f32]),
    "tlhip_gemm": (cint, [P, i64, i64, cint, P, i64, i64, cint, P, i64, i64, i64, i64, f32, f32]),
    "tlhip_gemv_f32": (cint, [P, P, P, i64, i64]),
    "tlhip_gemv_bf16": (cint, [P, P, P, i64, i64]),
    "tlhip_gemv_bf16_row": (cint, [P, P, P, i64, i64]),
    "tlhip_gemv_q4": (cint, [P, P, P, P, i64, i64, i64]),
    "tlhip_attn_decode": (cint, [P, P, P, P, i64, i64, i64, i64, i64, f32, cint]),
    "tlhip_attn_decode_static": (cint, [P, P, P, P, i64, i64, i64, i64, i64, f32, cint]),
    "tlhip_attn_prefill": (cint, [P, P, P, P, i64, i64, i64, i64, i64, f32, cint, i64]),
    "tlhip_kv_append": (cint, [P, P, P, P, i64, i64, i64, i64, cint]),
    "tlhip_kv_fill": (cint, [P, P, P, P, i64, i64, i64, i64, cint, i64]),
    "tlhip_rope": (cint, [P, P, i64, i64, i64, i64, f32, P]),
    "tlhip_rmsnorm": (cint, [P, P, P, i64, f32, i64]),
    "tlhip_rmsnorm_res": (cint, [P, P, P, P, P, i64, f32, i64]),
    "tlhip_swiglu": (cint, [P, P, i64, i64]),
    "tlhip_argmax": (cint, [P, i64, C.POINTER(i64)]),
    "tlhip_argmax_async": (cint, [P, i64, P]),
    "tlhip_gemm_bf16_nt": (cint, [P, P, P, i64, i64, i64]),
    "tlhip_gemm_q4_nt": (cint, [P, P, P, P, i64, i64, i64, i64]),
    "tlhip_gemm_q4_nt_parts": (cint, [P, P, P, P, i64, i64, i64, i64, i64, P]),
    "tlhip_gemm_q4_nt_swiglu": (cint, [P, P, P, P, i64, i64, i64, i64]),
    "tlhip_gemm_bf16_nt_swiglu": (cint, [P, P, P, i64, i64, i64]),
    "tlhip_gemm_bf16_nt_parts": (cint, [P, P, P, i64, i64, i64, i64, P]),
    "tlhip_gemm_f16w_bytes": (i64, [i64, i64, cint]),
    "tlhip_gemm_f16w_exps_bytes": (i64, [i64, cint]),
    "tlhip_gemm_f16w_prepare": (cint, [P, i64, i64, cint, P, P]),
    "tlhip_gemm_f16w_nt": (cint, [P, P, P, P, i64, i64, i64]),
    "tlhip_gemm_f16w_nt_parts": (cint, [P, P, P, P, i64, i64, i64, i64, P]),
    "tlhip_gemm_f16w_nt_swiglu": (cint, [P, P, P, P, i64, i64, i64]),
    "tlhip_rmsnorm_res_parts": (cint, [P, P, i64, P, P, P, i64, f32, i64]),
    "tlhip_split_heads": (cint, [P, P, P, i64, i64, i64, i64, i64]),
    "tlhip_merge_heads": (cint, [P, P, i64, i64, i64]),
    "tlhip_qkv_rope_append": (cint, [P, P, P, P, P, P, i64, i64, i64, i64, i64, f32, cint]),
    "tlhip_rope_dpos": (cint, [P, P, i64, i64, i64, P, f32, P]),
    "tlhip_incr_u32": (cint, [P]),
    "tlhip_kv_append_dpos": (cint, [P, P, P, P, P, i64, i64, i64, cint]),
    "tlhip_attn_partials_bytes": (i64, [i64, i64, i64, i64]),
    "tlhip_attn_decode_dpos": (cint, [P, P, P, P, i64, i64, P, i64, i64, f32, cint, P, i64]),
    "tlhip_qkv_rope_append_dpos": (cint, [P, P, P, P, P, P, i64, i64, i64, P, i64, f32, cint]),
    "tlhip_rope_table": (cint, [P, i64, i64, P, f32]),
    "tlhip_rope_table_range": (cint, [P, i64, i64, i64, f32]),
    "tlhip_qkv_rope_fill": (cint, [P, P, P, P, P, P, P, P, i64, i64, i64, i64, i64, i64, cint]),
    "tlhip_qkv_rope_fill_parts": (cint, [P, i64, P, P, P, P, P, P, P, i64, i64, i64, i64, i64, i64, cint]),
    "tlhip_attn_prefill_tok": (cint, [P, P, P, P, i64, i64, i64, i64, i64, f32, cint, i64]),
    "tlhip_qkv_rope_append_tab": (cint, [P, P, P, P, P, P, i64, i64, i64, i64, P, i64, P, cint]),
    "tlhip_convert": (cint, [P, cint, P, cint, i64]),
    "tlhip_convert_transpose": (cint, [P, cint, P, cint, i64, i64, i64, i64]),
    "tlhip_quantize_q4": (cint, [P, cint, P, P, i64, i64, i64]),
    "tlhip_embed_gather_f16": (cint, [P, P, P, i64, i64]),
    "tlhip_attn_decode_qkv": (cint, [P, P, P, P, P, P, P, i64, i64, i64, P, i64, i64, f32, P, cint, P, i64]),
    "tlhip_embed_gather_bf16": (cint, [P, P, P, i64, i64]),
    "tlhip_token_advance": (cint, [P, P, P, i64]),
    "tlhip_gemm_f16w_aimage_bytes": (i64, [i64, i64]),
    "tlhip_rmsnorm_res_parts_aimage": (cint, [P, P, i64, P, P, P, i64, f32, i64, P]),
    "tlhip_gemm_f16w_nt_aimage": (cint, [P, P, P, P, P, i64, i64, i64]),
    "tlhip_gemm_f16w_nt_parts_aimage": (cint, [P, P, P, P, P, i64, i64, i64, i64, P]),
    "tlhip_gemm_f16w_nt_swiglu_aimage": (cint, [P, P, P, P, P, i64, i64, i64]),
    "tlhip_attn_parts_splits": (cint, [i64, i64, i64, i64, cint]),
    "tlhip_attn_decode_qkv_parts": (cint, [P, P, P, P, P, P, i64, i64, i64, P, i64, i64, f32, P, P, i64, P]),
    "tlhip_gemv_q4_attn": (cint, [P, i64, i64, i64, P, P, P, i64, i64, i64]),
    "tlhip_gemv_bf16_row_attn": (cint, [P, i64, i64, i64, P, P, i64, i64]),
    "tlhip_gemv_q4_swiglu": (cint, [P, P, P, P, i64, i64, i64]),
    "tlhip_gemv_bf16_row_swiglu": (cint, [P, P, P, i64, i64]),
    "tlhip_gemv_q4_rmsnorm": (cint, [P, P, P, P, P, P, P, i64, i64, i64, f32]),
    "tlhip_gemv_bf16_row_rmsnorm": (cint, [P, P, P, P, P, P, i64, i64, f32]),
    "tlhip_gemv_q4_rmsnorm_gateup": (cint, [P, P, P, P, P, P, P, i64, i64, i64, f32]),
    "tlhip_gemv_bf16_row_rmsnorm_gateup": (cint, [P, P, P, P, P, P, i64, i64, f32]),
    "tlhip_tune_gemv_q4": (cint, [cint, cint, cint, cint, cint]),
    "tlhip_tune_gemv_cols": (cint, [cint]),
    "tlhip_tune_attn_prefill": (cint, [cint]),
    "tlhip_tune_gemm_planes": (cint, [cint]),
    "tlhip_tune_reset": (cint, []),
    "tlhip_bench_copy": (cint, [P, P, sz, cint]),
    "tlhip_bench_read": (cint, [P, sz, P, cint]),
    "tlhip_alloc_calls": (cint, [C.POINTER(u64)]),
    "tlhip_tune_attn_decode": (cint, [cint]),
    "tlhip_warm_fork": (cint, [P, P, cint, cint, cint]),
    "tlhip_warm_join": (cint, []),
}


class TlHipError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("tlhip error %d: %s" % (code, msg))
        self.code = code


class DevBuf:
    """A device allocation with its logical numpy dtype/shape."""

    def __init__(self, lib, nbytes, dtype=np.float32, shape=None):
        self.lib, self.nbytes = lib, int(nbytes)
        self.dtype = np.dtype(dtype)
        self.shape = tuple(shape) if shape is not None else (self.nbytes // self.dtype.itemsize,)
        p = P()
        lib._chk(lib.c.tlhip_malloc(C.byref(p), self.nbytes))
        self.ptr = p.value

    def at(self, byte_off):
        return C.c_void_p(self.ptr + int(byte_off))

    def upload(self, arr):
        a = np.ascontiguousarray(arr)
        assert a.nbytes <= self.nbytes, (a.nbytes, self.nbytes)
        self.lib._chk(self.lib.c.tlhip_memcpy_h2d(self.ptr, a.ctypes.data_as(P), a.nbytes))
        return self

    def numpy(self, dtype=None, shape=None):
        dtype = np.dtype(dtype or self.dtype)
        out = np.empty(self.nbytes // dtype.itemsize, dtype)
        self.lib._chk(self.lib.c.tlhip_memcpy_d2h(out.ctypes.data_as(P), self.ptr, out.nbytes))
        shape = shape or (self.shape if dtype == self.dtype else None)
        return out.reshape(shape) if shape is not None else out

    def free(self):
        if self.ptr:
            self.lib.c.tlhip_free(self.ptr)
            self.ptr = None


class TlHip:
    def __init__(self, path=LIB_PATH, init=True):
        if not os.path.exists(path):
            raise FileNotFoundError(
                "%s is missing: build it with `python cpp-tensorlib_amd/build.py`" % path)
        self.path = path
        self.c = C.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(self.c, name)
            fn.restype, fn.argtypes = res, args
        if init:
            self._chk(self.c.tlhip_init(0))

    # ---- plumbing -----------------------------------------------------------
    def _chk(self, rc):
        if rc != 0:
            raise TlHipError(rc, self.c.tlhip_last_error().decode())
        return rc

    def last_error(self):
        return self.c.tlhip_last_error().decode()

    def device_info(self):
        cu, hbm, lds = cint(), i64(), cint()
        self._chk(self.c.tlhip_device_info(C.byref(cu), C.byref(hbm), C.byref(lds)))
        return dict(compute_units=cu.value, hbm_bytes=hbm.value, lds_bytes_per_cu=lds.value,
                    arch=self.c.tlhip_arch().decode())

    def empty(self, shape, dtype=np.float32):
        shape = (shape,) if isinstance(shape, int) else tuple(shape)
        n = int(np.prod(shape)) if shape else 1
        return DevBuf(self, max(n, 1) * np.dtype(dtype).itemsize, dtype, shape)

    def empty_bytes(self, nbytes):
        return DevBuf(self, nbytes, np.uint8, (int(nbytes),))

    def to_device(self, arr):
        a = np.ascontiguousarray(arr)
        return DevBuf(self, max(a.nbytes, 4), a.dtype, a.shape).upload(a)

    def sync(self):
        self._chk(self.c.tlhip_sync())

    def census(self):
        buf = (u64 * len(CENSUS))()
        self._chk(self.c.tlhip_census(buf, len(CENSUS)))
        return dict(zip(CENSUS, [int(v) for v in buf]))

    def census_reset(self):
        self.c.tlhip_census_reset()

    # events
    def event(self):
        e = P()
        self._chk(self.c.tlhip_event_create(C.byref(e)))
        return e

    def record(self, ev):
        self._chk(self.c.tlhip_event_record(ev))

    def elapsed_ms(self, a, b):
        ms = f32()
        self._chk(self.c.tlhip_event_elapsed_ms(a, b, C.byref(ms)))
        return ms.value

    # graphs
    def graph_begin(self):
        self._chk(self.c.tlhip_graph_begin())

    def graph_end(self):
        g = P()
        self._chk(self.c.tlhip_graph_end(C.byref(g)))
        return g

    def graph_launch(self, g):
        self._chk(self.c.tlhip_graph_launch(g))

    def graph_destroy(self, g):
        self._chk(self.c.tlhip_graph_destroy(g))

    # ---- ops (thin; raise on any non-zero status) -----------------------------
    def binary(self, op, a, b, out, n, scale=1.0, offset=0.0, ao=0, bo=0, oo=0):
        self._chk(self.c.tlhip_binary(OPS[op], a.ptr, ao, b.ptr, bo, out.ptr, oo, n, scale, offset))

    def binary_bcast(self, op, a, astr, b, bstr, out, m, n, scale=1.0, offset=0.0):
        self._chk(self.c.tlhip_binary_bcast(OPS[op], a.ptr, 0, astr[0], astr[1], b.ptr, 0, bstr[0],
                                            bstr[1], out.ptr, 0, m, n, scale, offset))

    def unary(self, op, a, out, n, scale=1.0, offset=0.0, ao=0, oo=0):
        self._chk(self.c.tlhip_unary(OPS[op], a.ptr, ao, out.ptr, oo, n, scale, offset))

    def row_op(self, op, a, out, rows, cols, scale=1.0, offset=0.0):
        self._chk(self.c.tlhip_row_op(OPS[op], a.ptr, 0, out.ptr, 0, rows, cols, scale, offset))

    def gemm(self, a, lda, ta, b, ldb, tb, out, m, n, k, scale=1.0, offset=0.0):
        self._chk(self.c.tlhip_gemm(a.ptr, 0, lda, int(ta), b.ptr, 0, ldb, int(tb), out.ptr, 0, m, n,
                                    k, scale, offset))

    def gemv_f32(self, a, B, y, n, k):
        self._chk(self.c.tlhip_gemv_f32(a.ptr, B.ptr, y.ptr, n, k))

    def gemv_bf16(self, a, B, y, n, k):
        self._chk(self.c.tlhip_gemv_bf16(a.ptr, B.ptr, y.ptr, n, k))

    def gemv_bf16_row(self, a, W, y, n, k):
        self._chk(self.c.tlhip_gemv_bf16_row(a.ptr, W.ptr, y.ptr, n, k))

    def gemv_q4(self, a, wq, y, N, K, group=32, wq_off=0):
        """wq: one buffer [packed N*K/2 bytes | scales], as the reference stores it."""
        qp = wq.ptr + wq_off
        self._chk(self.c.tlhip_gemv_q4(a.ptr, qp, qp + N * K // 2, y.ptr, N, K, group))

    def attn_decode(self, q, K, V, out, Hq, Hkv, ctx, kv_max, D, scale, kv_bf16=False):
        self._chk(self.c.tlhip_attn_decode(q.ptr, K.ptr, V.ptr, out.ptr, Hq, Hkv, ctx, kv_max, D,
                                           scale, int(kv_bf16)))

    def attn_decode_static(self, q, K, V, out, Hq, Hkv, ctx, kv_max, D, scale, kv_bf16=False):
        self._chk(self.c.tlhip_attn_decode_static(q.ptr, K.ptr, V.ptr, out.ptr, Hq, Hkv, ctx, kv_max, D,
                                                  scale, 1 if kv_bf16 else 0))

    def attn_prefill(self, q, K, V, out, Hq, Hkv, T, kv_max, D, scale, kv_bf16=False, pos0=0):
        self._chk(self.c.tlhip_attn_prefill(q.ptr, K.ptr, V.ptr, out.ptr, Hq, Hkv, T, kv_max, D,
                                            scale, int(kv_bf16), pos0))

    def kv_append(self, Kc, Vc, k, v, pos, kv_max, Hkv, D, kv_bf16=False):
        self._chk(self.c.tlhip_kv_append(Kc.ptr, Vc.ptr, k.ptr, v.ptr, pos, kv_max, Hkv, D,
                                         int(kv_bf16)))

    def kv_fill(self, Kc, Vc, K, V, T, kv_max, Hkv, D, kv_bf16=False, pos0=0):
        self._chk(self.c.tlhip_kv_fill(Kc.ptr, Vc.ptr, K.ptr, V.ptr, T, kv_max, Hkv, D,
                                       int(kv_bf16), pos0))

    def rope(self, x, out, rows, T, D, pos, base, bias=None):
        self._chk(self.c.tlhip_rope(x.ptr, out.ptr, rows, T, D, pos, base,
                                    bias.ptr if bias is not None else None))

    def rmsnorm(self, x, w, out, n, eps, rows=1):
        self._chk(self.c.tlhip_rmsnorm(x.ptr, w.ptr, out.ptr, n, eps, rows))

    def rmsnorm_res(self, x, delta, w, xout, hout, n, eps, rows=1):
        self._chk(self.c.tlhip_rmsnorm_res(x.ptr, delta.ptr, w.ptr, xout.ptr, hout.ptr, n, eps, rows))

    def swiglu(self, gu, out, ff, rows=1):
        self._chk(self.c.tlhip_swiglu(gu.ptr, out.ptr, ff, rows))

    def argmax(self, x, n):
        idx = i64()
        self._chk(self.c.tlhip_argmax(x.ptr, n, C.byref(idx)))
        return idx.value

    def gemm_bf16_nt(self, A, W, out, M, N, K):
        self._chk(self.c.tlhip_gemm_bf16_nt(A.ptr, W.ptr, out.ptr, M, N, K))

    def gemm_q4_nt(self, A, q4, out, M, N, K):
        """q4: the one-buffer int4 weight (packed nibbles, then scales) that gemv_q4 takes."""
        self._chk(self.c.tlhip_gemm_q4_nt(A.ptr, q4.ptr, q4.ptr + N * K // 2, out.ptr, M, N, K, 32))

    def gemm_q4_nt_swiglu(self, A, q4, act, M, ff, K):
        self._chk(self.c.tlhip_gemm_q4_nt_swiglu(A.ptr, q4.ptr, q4.ptr + 2 * ff * K // 2, act.ptr, M, ff, K, 32))

    def gemm_q4_nt_parts(self, A, q4, parts, M, N, K):
        n = C.c_int(0)
        self._chk(self.c.tlhip_gemm_q4_nt_parts(A.ptr, q4.ptr, q4.ptr + N * K // 2, parts.ptr, parts.nbytes,
                                                M, N, K, 32, C.byref(n)))
        return n.value

    def gemm_bf16_nt_swiglu(self, A, W, act, M, ff, K):
        self._chk(self.c.tlhip_gemm_bf16_nt_swiglu(A.ptr, W.ptr, act.ptr, M, ff, K))

    def gemm_bf16_nt_parts(self, A, W, parts, M, N, K):
        """The product as its K-split parts in `parts`; returns how many there are."""
        n = C.c_int(0)
        self._chk(self.c.tlhip_gemm_bf16_nt_parts(A.ptr, W.ptr, parts.ptr, parts.nbytes, M, N, K, C.byref(n)))
        return n.value

    def gemm_f16w_prepare(self, W, N, K, gated=False):
        """The prepared form of the bf16 weight W ([N, K], or [2 * N, K] = gate rows | up rows when
        gated): returns (image, exps) device buffers for the gemm_f16w_* products."""
        nbytes = self.c.tlhip_gemm_f16w_bytes(N, K, int(gated))
        if nbytes <= 0:
            raise ValueError("gemm_f16w_prepare: need positive N, K and K % 32 == 0")
        image = self.empty_bytes(nbytes)
        exps = self.empty_bytes(self.c.tlhip_gemm_f16w_exps_bytes(N, int(gated)))
        self._chk(self.c.tlhip_gemm_f16w_prepare(W.ptr, N, K, int(gated), image.ptr, exps.ptr))
        return image, exps

    def gemm_f16w_nt(self, A, image, exps, out, M, N, K):
        self._chk(self.c.tlhip_gemm_f16w_nt(A.ptr, image.ptr, exps.ptr, out.ptr, M, N, K))

    def gemm_f16w_nt_swiglu(self, A, image, exps, act, M, ff, K):
        self._chk(self.c.tlhip_gemm_f16w_nt_swiglu(A.ptr, image.ptr, exps.ptr, act.ptr, M, ff, K))

    def gemm_f16w_nt_parts(self, A, image, exps, parts, M, N, K):
        n = C.c_int(0)
        self._chk(self.c.tlhip_gemm_f16w_nt_parts(A.ptr, image.ptr, exps.ptr, parts.ptr, parts.nbytes, M, N, K,
                                                  C.byref(n)))
        return n.value

    def rmsnorm_res_parts(self, x, parts, n_parts, w, xout, hout, n, eps, rows=1):
        self._chk(self.c.tlhip_rmsnorm_res_parts(x.ptr, parts.ptr, n_parts, w.ptr, xout.ptr, hout.ptr,
                                                 n, eps, rows))

    def gemm_f16w_aimage_bytes(self, M, K):
        return int(self.c.tlhip_gemm_f16w_aimage_bytes(M, K))

    def rmsnorm_res_parts_aimage(self, x, parts, n_parts, w, xout, hout, n, eps, rows, aimage):
        """rmsnorm_res_parts that also leaves hout's activation image (gemm_f16w_aimage_bytes(rows, n) bytes)."""
        self._chk(self.c.tlhip_rmsnorm_res_parts_aimage(x.ptr, parts.ptr, n_parts, w.ptr, xout.ptr, hout.ptr,
                                                        n, eps, rows, aimage.ptr))

    def gemm_f16w_nt_aimage(self, A, aimage, image, exps, out, M, N, K):
        self._chk(self.c.tlhip_gemm_f16w_nt_aimage(A.ptr, aimage.ptr, image.ptr, exps.ptr, out.ptr, M, N, K))

    def gemm_f16w_nt_swiglu_aimage(self, A, aimage, image, exps, act, M, ff, K):
        self._chk(self.c.tlhip_gemm_f16w_nt_swiglu_aimage(A.ptr, aimage.ptr, image.ptr, exps.ptr, act.ptr, M, ff, K))

    def gemm_f16w_nt_parts_aimage(self, A, aimage, image, exps, parts, M, N, K):
        n = C.c_int(0)
        self._chk(self.c.tlhip_gemm_f16w_nt_parts_aimage(A.ptr, aimage.ptr, image.ptr, exps.ptr, parts.ptr,
                                                         parts.nbytes, M, N, K, C.byref(n)))
        return n.value

    def split_heads(self, src, bias, dst, T, ld, off, H, D):
        self._chk(self.c.tlhip_split_heads(src.ptr, bias.ptr if bias is not None else None, dst.ptr,
                                           T, ld, off, H, D))

    def merge_heads(self, src, dst, T, H, D):
        self._chk(self.c.tlhip_merge_heads(src.ptr, dst.ptr, T, H, D))

    def alloc_calls(self):
        """Allocation and release calls the library has made so far (device and pinned host)."""
        n = u64(0)
        self._chk(self.c.tlhip_alloc_calls(C.byref(n)))
        return int(n.value)

    def bench_copy(self, dst, src, nbytes, blocks=0):
        self._chk(self.c.tlhip_bench_copy(dst.ptr, src.ptr, nbytes, blocks))

    def bench_read(self, src, nbytes, sink, blocks=0, off=0):
        self._chk(self.c.tlhip_bench_read(src.ptr + off, nbytes, sink.ptr, blocks))

    def qkv_rope_append(self, qkv, bq, bk, bv, Kc, Vc, Hq, Hkv, D, pos, kv_max, base, kv_bf16=False):
        self._chk(self.c.tlhip_qkv_rope_append(qkv.ptr, bq.ptr, bk.ptr, bv.ptr if bv is not None else None,
                                               Kc.ptr, Vc.ptr, Hq, Hkv, D, pos, kv_max, base, int(kv_bf16)))

    def rope_dpos(self, x, out, rows, T, D, d_pos, base, bias=None):
        self._chk(self.c.tlhip_rope_dpos(x.ptr, out.ptr, rows, T, D, d_pos.ptr, base,
                                         bias.ptr if bias is not None else None))

    def incr_u32(self, d_pos):
        self._chk(self.c.tlhip_incr_u32(d_pos.ptr))

    def kv_append_dpos(self, Kc, Vc, k, v, d_pos, kv_max, Hkv, D, kv_bf16=False):
        self._chk(self.c.tlhip_kv_append_dpos(Kc.ptr, Vc.ptr, k.ptr, v.ptr, d_pos.ptr, kv_max, Hkv, D,
                                              int(kv_bf16)))

    def attn_partials_bytes(self, Hq, Hkv, kv_max, D):
        return int(self.c.tlhip_attn_partials_bytes(Hq, Hkv, kv_max, D))

    def attn_decode_dpos(self, q, K, V, out, Hq, Hkv, d_pos, kv_max, D, scale, partials, kv_bf16=False):
        self._chk(self.c.tlhip_attn_decode_dpos(q.ptr, K.ptr, V.ptr, out.ptr, Hq, Hkv, d_pos.ptr, kv_max,
                                                D, scale, int(kv_bf16), partials.ptr, partials.nbytes))

    def qkv_rope_append_dpos(self, qkv, bq, bk, bv, Kc, Vc, Hq, Hkv, D, d_pos, kv_max, base, kv_bf16=False):
        self._chk(self.c.tlhip_qkv_rope_append_dpos(
            qkv.ptr, bq.ptr, bk.ptr, bv.ptr if bv is not None else None, Kc.ptr, Vc.ptr, Hq, Hkv, D,
            d_pos.ptr, kv_max, base, int(kv_bf16)))

    def rope_table(self, table, D, pos, base, d_pos=None):
        self._chk(self.c.tlhip_rope_table(table.ptr, D, pos, d_pos.ptr if d_pos is not None else None, base))

    def qkv_rope_append_tab(self, qkv, bq, bk, bv, Kc, Vc, Hq, Hkv, D, pos, kv_max, table, d_pos=None,
                            kv_bf16=False):
        self._chk(self.c.tlhip_qkv_rope_append_tab(
            qkv.ptr, bq.ptr, bk.ptr, bv.ptr if bv is not None else None, Kc.ptr, Vc.ptr, Hq, Hkv, D, pos,
            d_pos.ptr if d_pos is not None else None, kv_max, table.ptr, int(kv_bf16)))

    def attn_decode_qkv(self, qkv, bq, bk, bv, Kc, Vc, out, Hq, Hkv, pos, kv_max, D, scale, table,
                        d_pos=None, partials=None, kv_bf16=False):
        opt = lambda b: b.ptr if b is not None else None
        self._chk(self.c.tlhip_attn_decode_qkv(
            qkv.ptr, opt(bq), opt(bk), opt(bv), Kc.ptr, Vc.ptr, out.ptr, Hq, Hkv, pos, opt(d_pos), kv_max,
            D, scale, table.ptr, int(kv_bf16), opt(partials), partials.nbytes if partials is not None else 0))

    def attn_parts_splits(self, Hq, Hkv, plan_ctx, D, kv_bf16=False):
        """Splits tlhip_attn_decode_qkv_parts would leave for a grid planned for plan_ctx keys; 0: shape not served."""
        return int(self.c.tlhip_attn_parts_splits(Hq, Hkv, plan_ctx, D, int(kv_bf16)))

    def attn_decode_qkv_parts(self, qkv, bq, bk, bv, Kc, Vc, Hq, Hkv, pos, kv_max, D, scale, table, partials,
                              d_pos=None):
        """The fused decode attention with the split merge left to gemv_*_attn; returns the number of splits."""
        opt = lambda b: b.ptr if b is not None else None
        n = C.c_int(0)
        self._chk(self.c.tlhip_attn_decode_qkv_parts(
            qkv.ptr, opt(bq), opt(bk), opt(bv), Kc.ptr, Vc.ptr, Hq, Hkv, pos, opt(d_pos), kv_max, D, scale,
            table.ptr, partials.ptr, partials.nbytes, C.byref(n)))
        return n.value

    def gemv_q4_attn(self, parts, n_parts, heads, D, wq, y, N, K, group=32):
        self._chk(self.c.tlhip_gemv_q4_attn(parts.ptr, n_parts, heads, D, wq.ptr, wq.ptr + N * K // 2, y.ptr, N, K, group))

    def gemv_bf16_row_attn(self, parts, n_parts, heads, D, W, y, N, K):
        self._chk(self.c.tlhip_gemv_bf16_row_attn(parts.ptr, n_parts, heads, D, W.ptr, y.ptr, N, K))

    # element types of the load-time converters
    T_F32, T_F16, T_BF16 = 0, 1, 2

    def convert(self, src, src_type, dst, dst_type, n):
        self._chk(self.c.tlhip_convert(src.ptr, src_type, dst.ptr, dst_type, n))

    def convert_transpose(self, src, src_type, dst, dst_type, rows, cols, ld_dst, col_base=0):
        self._chk(self.c.tlhip_convert_transpose(src.ptr, src_type, dst.ptr, dst_type, rows, cols, ld_dst, col_base))

    def quantize_q4(self, src, src_type, q4buf, rows, K, row_base=0, total_rows=None, group=32):
        """Quantise `rows` file rows into rows [row_base, row_base + rows) of a q4 buffer of total_rows."""
        total = rows if total_rows is None else total_rows
        self._chk(self.c.tlhip_quantize_q4(src.ptr, src_type, q4buf.ptr + row_base * K // 2,
                                           q4buf.ptr + total * K // 2 + row_base * (K // 32) * 4, rows, K, group))

    def embed_gather_f16(self, table, d_token, out, hidden, vocab):
        self._chk(self.c.tlhip_embed_gather_f16(table.ptr, d_token.ptr, out.ptr, hidden, vocab))

    def embed_gather_bf16(self, table, d_token, out, hidden, vocab):
        self._chk(self.c.tlhip_embed_gather_bf16(table.ptr, d_token.ptr, out.ptr, hidden, vocab))

    def token_advance(self, d_pos, d_token, history, capacity):
        self._chk(self.c.tlhip_token_advance(d_pos.ptr, d_token.ptr,
                                             history.ptr if history is not None else None, capacity))

    def gemv_q4_swiglu(self, gu, wq, y, N, K, group=32):
        self._chk(self.c.tlhip_gemv_q4_swiglu(gu.ptr, wq.ptr, wq.ptr + N * K // 2, y.ptr, N, K, group))

    def gemv_bf16_row_swiglu(self, gu, W, y, N, K):
        self._chk(self.c.tlhip_gemv_bf16_row_swiglu(gu.ptr, W.ptr, y.ptr, N, K))

    def gemv_q4_rmsnorm(self, x, delta, norm_w, xout, wq, y, N, K, eps, group=32):
        self._chk(self.c.tlhip_gemv_q4_rmsnorm(
            x.ptr, delta.ptr if delta is not None else None, norm_w.ptr,
            xout.ptr if xout is not None else None, wq.ptr, wq.ptr + N * K // 2, y.ptr, N, K, group, eps))

    def gemv_bf16_row_rmsnorm(self, x, delta, norm_w, xout, W, y, N, K, eps):
        self._chk(self.c.tlhip_gemv_bf16_row_rmsnorm(
            x.ptr, delta.ptr if delta is not None else None, norm_w.ptr,
            xout.ptr if xout is not None else None, W.ptr, y.ptr, N, K, eps))

    def gemv_q4_rmsnorm_gateup(self, x, delta, norm_w, xout, wq, act, N2, K, eps, group=32):
        self._chk(self.c.tlhip_gemv_q4_rmsnorm_gateup(
            x.ptr, delta.ptr if delta is not None else None, norm_w.ptr,
            xout.ptr if xout is not None else None, wq.ptr, wq.ptr + N2 * K // 2, act.ptr, N2, K, group, eps))

    def gemv_bf16_row_rmsnorm_gateup(self, x, delta, norm_w, xout, W, act, N2, K, eps):
        self._chk(self.c.tlhip_gemv_bf16_row_rmsnorm_gateup(
            x.ptr, delta.ptr if delta is not None else None, norm_w.ptr,
            xout.ptr if xout is not None else None, W.ptr, act.ptr, N2, K, eps))

    def rope_table_range(self, table, D, pos0, T, base):
        self._chk(self.c.tlhip_rope_table_range(table.ptr, D, pos0, T, base))

    def qkv_rope_fill(self, qkv, bq, bk, bv, table, qh, Kc, Vc, T, Hq, Hkv, D, pos0, kv_max, kv_bf16=False,
                      n_parts=1):
        """n_parts > 1: qkv holds the projection's K-split parts, [n_parts][T][(Hq + 2 Hkv) D]."""
        opt = lambda b: b.ptr if b is not None else None
        self._chk(self.c.tlhip_qkv_rope_fill_parts(qkv.ptr, n_parts, opt(bq), opt(bk), opt(bv), table.ptr,
                                                   qh.ptr, Kc.ptr, Vc.ptr, T, Hq, Hkv, D, pos0, kv_max,
                                                   1 if kv_bf16 else 0))

    def attn_prefill_tok(self, q, K, V, out, Hq, Hkv, T, kv_max, D, scale, kv_bf16=False, pos0=0):
        self._chk(self.c.tlhip_attn_prefill_tok(q.ptr, K.ptr, V.ptr, out.ptr, Hq, Hkv, T, kv_max, D, scale,
                                                1 if kv_bf16 else 0, pos0))

    def tune_attn_prefill(self, kernel):
        """0 / False: built-in choice, 1 / True: VALU kernel, 2: fp32 matrix pipe, 4: f16 terms."""
        self._chk(self.c.tlhip_tune_attn_prefill(int(kernel)))

    def tune_attn_decode(self, kernel):
        """0: built-in choice, 1: the key-slot decode attention kernel for every shape."""
        self._chk(self.c.tlhip_tune_attn_decode(int(kernel)))

    def tune_gemm_planes(self, planes):
        """3: the int4 prompt GEMMs cut activations into three bf16 terms; 0: built-in choice (two f16)."""
        self._chk(self.c.tlhip_tune_gemm_planes(int(planes)))

    def tune_reset(self):
        self._chk(self.c.tlhip_tune_reset())

    def tune_gemv_q4(self, rows=0, kw=0, bpc=0, nw=0, lpr=0):
        self._chk(self.c.tlhip_tune_gemv_q4(rows, kw, bpc, nw, lpr))


_lib = None


def load():
    """The process-wide library handle (initialises device 0). Raises when the
    library has not been built or no gfx950 GPU is present."""
    global _lib
    if _lib is None:
        _lib = TlHip()
    return _lib
