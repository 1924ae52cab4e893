"""Where the time goes inside a kernel: accumulated phase clocks per wavefront.

The kernels carry TLHIP_MARK points that compile to nothing in the product library. The trace
build (python cpp-tensorlib_amd/build.py --trace -> lib/libtensorlib_hip_trace.so) makes lane 0 of
every wavefront record the shader clock (s_memtime) there; this script runs one launch and prints
the distribution over wavefronts. Times are clocks of the 100 MHz-referenced shader counter
divided by the frequency given with --ghz (default 2.1).

  python cpp-tensorlib_amd/trace_phases.py attn_decode [pos]      7B decode attention (fused q/k/v, device position)
  python cpp-tensorlib_amd/trace_phases.py attn_prefill [pos0 [bf16]]  7B causal prefill attention of a 512-token chunk: f16 terms, or bf16 planes
  python cpp-tensorlib_amd/trace_phases.py gemm [f16w|bf16|q4]    a 512 x 32768 x 3584 prompt GEMM: prepared weight, plain bf16, or int4
"""
import ctypes as C
import importlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
SLOTS, WAVES, BLOCKS = 8, 16, 1024


def load():
    capi = importlib.import_module("cpp-tensorlib_amd.capi")
    path = os.path.join(HERE, "lib", "libtensorlib_hip_trace.so")
    if not os.path.exists(path):
        sys.exit("build the trace library first: python cpp-tensorlib_amd/build.py --trace")
    lib = capi.TlHip(path=path)
    lib.c.tlhip_trace_read.restype = C.c_int
    lib.c.tlhip_trace_read.argtypes = [C.c_void_p, C.c_size_t, C.c_int]
    return lib


def read_trace(lib, clear=True):
    tr = np.zeros(BLOCKS * WAVES * SLOTS, np.uint64)
    if lib.c.tlhip_trace_read(tr.ctypes.data, tr.nbytes, 1 if clear else 0) != 0:
        sys.exit("tlhip_trace_read failed")
    return tr.reshape(BLOCKS, WAVES, SLOTS).astype(np.float64)


def pct(name, d):
    print("   %-58s p10 %7.2f  med %7.2f  p90 %7.2f  max %7.2f us" % (name, np.percentile(d, 10), np.median(d), np.percentile(d, 90), d.max()))


def attn_decode(lib, pos, ghz):
    Hq, Hkv, D, kv_max = 28, 4, 128, 4352
    rng = np.random.default_rng(1)
    qkv = lib.to_device(rng.standard_normal((Hq + 2 * Hkv) * D, dtype=np.float32))
    layers = 8
    Ks = [lib.to_device(rng.standard_normal((Hkv, kv_max, D), dtype=np.float32)) for _ in range(layers)]
    Vs = [lib.to_device(rng.standard_normal((Hkv, kv_max, D), dtype=np.float32)) for _ in range(layers)]
    bq, bk, bv = (lib.to_device(np.zeros(m, np.float32)) for m in (Hq * D, Hkv * D, Hkv * D))
    tab, out = lib.empty(D), lib.empty((Hq, D))
    dpos = lib.to_device(np.array([pos], np.uint32))
    part = lib.empty_bytes(lib.attn_partials_bytes(Hq, Hkv, kv_max, D))
    lib.rope_table(tab, D, pos, 1e6)
    scale = float(1 / np.sqrt(D))
    run = lambda i: lib.attn_decode_qkv(qkv, bq, bk, bv, Ks[i % layers], Vs[i % layers], out, Hq, Hkv, pos, kv_max, D,
                                        scale, tab, d_pos=dpos, partials=part)
    for i in range(layers):
        run(i)
    lib.sync()
    e0, e1 = lib.event(), lib.event()
    lib.record(e0)
    for i in range(4 * layers):
        run(i)
    lib.record(e1)
    lib.sync()
    print("tlhip_attn_decode_qkv (attention + combine), position %d, caches rotating: %.2f us per call"
          % (pos, lib.elapsed_ms(e0, e1) * 1e3 / (4 * layers)))
    read_trace(lib)
    run(0)
    lib.sync()
    t = read_trace(lib)
    live = t[:, :, 0] > 0
    print("%d wavefronts; time since the wavefront's first instruction:" % int(live.sum()))
    names = {7: "all requests issued (query rows, rotary table, first K/V tile)",
             1: "query rows staged in LDS, rotated; position read",
             2: "new key/value row formed (wavefront 0 of split 0)",
             3: "tile loop done (scores, softmax, P.V)",
             4: "wave totals (sums over lanes and key slots) in LDS",
             5: "block barrier passed",
             6: "block merge done, partials stored"}
    for sl in (7, 1, 2, 3, 4, 5, 6):
        ok = live & (t[:, :, sl] > 0)
        pct(names[sl], ((t[:, :, sl] - t[:, :, 0])[ok]) / (ghz * 1e3))


def attn_prefill(lib, pos0, ghz, mode=4):
    Hq, Hkv, D, T = 28, 4, 128, 512
    rng = np.random.default_rng(3)
    kv_max = pos0 + T
    scale = float(1 / np.sqrt(D))
    K = lib.to_device(rng.standard_normal(Hkv * kv_max * D, dtype=np.float32))
    V = lib.to_device(rng.standard_normal(Hkv * kv_max * D, dtype=np.float32))
    q = lib.to_device(rng.standard_normal(Hq * T * D, dtype=np.float32))
    out = lib.empty(Hq * T * D)
    lib.tune_attn_prefill(mode)
    for _ in range(2):
        lib.attn_prefill(q, K, V, out, Hq, Hkv, T, kv_max, D, scale, pos0=pos0)
    lib.sync()
    read_trace(lib)
    e0, e1 = lib.event(), lib.event()
    lib.record(e0)
    lib.attn_prefill(q, K, V, out, Hq, Hkv, T, kv_max, D, scale, pos0=pos0)
    lib.record(e1)
    lib.sync()
    print("tlhip_attn_prefill, %s (planes + attention + merge), pos0 %d: %.1f us"
          % ("f16-term kernels" if mode == 4 else "bf16-plane kernels", pos0, lib.elapsed_ms(e0, e1) * 1e3))
    t = read_trace(lib)
    for grp, ws in (("wavefronts 0-3 (matrix phase, then softmax)", range(0, 4)), ("wavefronts 4-6 (softmax, then matrix phase)", range(4, 7))):
        tt = t[:, list(ws), :]
        live = tt[:, :, 4] > 0
        iv = tt[:, :, 4][live]
        print("%s: %d wavefronts, %d barrier intervals each (median); per interval:" % (grp, int(live.sum()), int(np.median(iv))))
        for k, nm in ((1, "softmax phase"), (2, "matrix phase (P.V of the tile before, Q.K^T of this one)"), (3, "barrier wait")):
            pct(nm, tt[:, :, k][live] / iv / (ghz * 1e3))
        pct("whole interval", (tt[:, :, 6] - tt[:, :, 0])[live] / iv / (ghz * 1e3))


def gemm(lib, kind, ghz):
    M, N, K = 512, 32768, 3584
    rng = np.random.default_rng(5)
    A = lib.to_device(rng.standard_normal((M, K), dtype=np.float32))
    w = (rng.standard_normal((N, K), dtype=np.float32) * 0.02).view(np.uint32) >> 16
    W = lib.to_device(w.astype(np.uint16))
    Cm = lib.empty((M, N))
    us = lambda x: x / (ghz * 1e3)
    if kind == "f16w":
        img, ex = lib.gemm_f16w_prepare(W, N, K)
        run = lambda: lib.gemm_f16w_nt(A, img, ex, Cm, M, N, K)
    elif kind == "q4":
        host = np.empty(N * K // 2 + N * (K // 32) * 4, np.uint8)       # packed nibbles, then f32 scales
        host[:N * K // 2] = rng.integers(0, 256, N * K // 2, dtype=np.uint8)
        host[N * K // 2:] = rng.uniform(0.005, 0.02, N * (K // 32)).astype(np.float32).view(np.uint8)
        q4 = lib.to_device(host)
        run = lambda: lib.gemm_q4_nt(A, q4, Cm, M, N, K)
    else:
        run = lambda: lib.gemm_bf16_nt(A, W, Cm, M, N, K)
    for _ in range(2):
        run()
    lib.sync()
    read_trace(lib)
    e0, e1 = lib.event(), lib.event()
    lib.record(e0)
    run()
    lib.record(e1)
    lib.sync()
    print("prompt GEMM %d x %d x %d, %s: %.1f us" % (M, N, K, kind, lib.elapsed_ms(e0, e1) * 1e3))
    t = read_trace(lib)
    if kind != "f16w":
        t = t[:, :4, :]
        live = t[:, :, 7] > 0
        slabs = t[:, :, 7][live]
        print("%d wavefronts, %d K slabs each; per slab:" % (int(live.sum()), int(np.median(slabs))))
        for k, nm in ((1, "barrier: the slab before consumed by every wavefront"), (2, "wait for the slab's global loads"),
                      (3, "convert and store to LDS"), (4, "barrier: slab complete in LDS"),
                      (5, "next slab requested, fragments read, matrix products")):
            pct(nm, us(t[:, :, k][live] / slabs))
        pct("whole slab", us((t[:, :, 6] - t[:, :, 0])[live] / slabs))
        return
    t = t[:, :8, :]
    live = t[:, :, 7] > 0
    slabs = t[:, :, 7][live]
    print("%d wavefronts, %d K slabs each" % (int(live.sum()), int(np.median(slabs))))
    pct("first three slab copies issued -> slab 0 landed everywhere", us((t[:, :, 1] - t[:, :, 0])[live]))
    pct("per slab: fragment reads, matrix products, copy requests", us(t[:, :, 2][live] / slabs))
    pct("per slab: wait for own reads and copies, barrier", us(t[:, :, 3][live] / slabs))
    pct("loop", us((t[:, :, 5] - t[:, :, 1])[live]))
    pct("result scaled and stored", us((t[:, :, 6] - t[:, :, 5])[live]))


if __name__ == "__main__":
    args = [a for a in sys.argv[1:] if not a.startswith("--ghz")]
    ghz = next((float(a.split("=")[1]) for a in sys.argv[1:] if a.startswith("--ghz=")), 2.1)
    if not args or args[0] not in ("attn_decode", "attn_prefill", "gemm"):
        sys.exit(__doc__)
    lib = load()
    if args[0] == "gemm":
        gemm(lib, args[1] if len(args) > 1 else "f16w", ghz)
    elif args[0] == "attn_decode":
        attn_decode(lib, int(args[1]) if len(args) > 1 else 4095, ghz)
    else:
        attn_prefill(lib, int(args[1]) if len(args) > 1 else 7680, ghz, 3 if "bf16" in args[2:] else 4)
