"""TEST INFRASTRUCTURE: writes GGUF v3 files (the llama.cpp model container) from Python, so
the reader and the loader can be exercised without a downloaded model. Wire format: magic,
version, tensor count, kv count, metadata (key string, u32 type, value), tensor directory (name,
n_dims, dims in ne order, u32 storage code, u64 offset into the data section), padding to the
alignment, tensor bytes (each padded to the alignment). Everything little-endian."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
GGML = dict(f32=0, f16=1, q4_0=2, q4_1=3, q5_0=6, q5_1=7, q8_0=8, q8_1=9, q2_k=10, q3_k=11, q4_k=12,
            q5_k=13, q6_k=14, q8_k=15, bf16=30)
_SCALAR = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B",
           U64: "<Q", I64: "<q", F64: "<d"}


def _string(b):
    b = b.encode() if isinstance(b, str) else bytes(b)
    return struct.pack("<Q", len(b)) + b


def _value(t, v):
    if t in _SCALAR:
        return struct.pack(_SCALAR[t], v)
    if t == STRING:
        return _string(v)
    if t == ARRAY:                      # v = (elem_type, [values])
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(_value(et, x) for x in items)
    raise ValueError(t)


def build(kv, tensors, alignment=32, version=3, magic=b"GGUF"):
    """kv: [(key, type, value)], tensors: [(name, storage_code, dims_ne, raw_bytes)] -> bytes."""
    head = magic + struct.pack("<IQQ", version, len(tensors), len(kv))
    for key, t, v in kv:
        head += _string(key) + struct.pack("<I", t) + _value(t, v)
    offsets, at = [], 0
    for _, _, _, raw in tensors:
        offsets.append(at)
        at = (at + len(raw) + alignment - 1) // alignment * alignment
    for (name, code, dims, _), off in zip(tensors, offsets):
        head += _string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", code, off)
    head += b"\0" * ((-len(head)) % alignment)
    body = b""
    for (_, _, _, raw), off in zip(tensors, offsets):
        body += b"\0" * (off - len(body)) + bytes(raw)
    return head + body


def write(path, kv, tensors, **kw):
    data = build(kv, tensors, **kw)
    with open(path, "wb") as f:
        f.write(data)
    return data


def write_streaming(path, kv, tensors, alignment=32):
    """Like write() for files too large to assemble in memory: tensors = [(name, storage_code,
    dims_ne, ndarray)], each array written straight to the file."""
    sizes = [int(a.nbytes) for _, _, _, a in tensors]
    directory = [(n, c, d, b"") for n, c, d, _ in tensors]
    head = bytearray(build(kv, directory, alignment=alignment))
    # build() laid the (empty) tensors out at offset 0: patch the real offsets in
    offsets, at = [], 0
    for nb in sizes:
        offsets.append(at)
        at = (at + nb + alignment - 1) // alignment * alignment
    pos = 24
    for key, t, v in kv:
        pos += len(_string(key)) + 4 + len(_value(t, v))
    for (name, _, dims, _), off in zip(tensors, offsets):
        pos += len(_string(name)) + 4 + 8 * len(dims) + 4
        head[pos:pos + 8] = struct.pack("<Q", off)
        pos += 8
    with open(path, "wb") as f:
        f.write(head)
        written = 0
        for (_, _, _, a), off in zip(tensors, offsets):
            f.write(b"\0" * (off - written))
            f.write(np.ascontiguousarray(a).data)
            written = off + int(a.nbytes)


def qwen2_file(path, dims, weights, arch="qwen2", tied=False, with_bias=True, linear_type="f16",
               extra_kv=()):
    """A Qwen2-architecture file. weights: dict name -> ndarray in the FILE's layout: linear layers
    [out, in] (float16 / float32 / uint16 holding bf16 per linear_type), vectors float32,
    'token_embd.weight' [vocab, hidden] float16."""
    d = dims
    kv = [("general.architecture", STRING, arch), ("general.name", STRING, "synthetic"),
          (arch + ".block_count", U32, d["n_layers"]), (arch + ".embedding_length", U32, d["hidden"]),
          (arch + ".feed_forward_length", U32, d["ff"]), (arch + ".attention.head_count", U32, d["n_q_heads"]),
          (arch + ".attention.head_count_kv", U32, d["n_kv_heads"]),
          (arch + ".attention.layer_norm_rms_epsilon", F32, d["eps"]), (arch + ".rope.freq_base", F32, d["rope_base"]),
          (arch + ".context_length", U32, 32768)] + list(extra_kv)
    if d["head_dim"] * d["n_q_heads"] != d["hidden"]:
        kv.append((arch + ".attention.key_length", U32, d["head_dim"]))
    tensors = []
    for name, a in weights.items():
        if tied and name == "output.weight":
            continue
        if not with_bias and name.endswith(".bias"):
            continue
        a = np.ascontiguousarray(a)
        if a.ndim == 2 and name != "token_embd.weight":
            code = GGML[linear_type]
        else:
            code = {np.dtype(np.float32): GGML["f32"], np.dtype(np.float16): GGML["f16"]}[a.dtype]
        tensors.append((name, code, list(a.shape[::-1]), a.tobytes()))
    return write(path, kv, tensors)


def qwen05b_synthetic(path, seed=17):
    """A Qwen2.5-0.5B-shaped F16 file (24 layers, hidden 896, 14/2 heads of 64, FF 4864, vocab 151936;
    1.26 GB) with seeded ~N(0, 0.02) weights: the shape the reference's harness hard-codes
    (bench/cuda/qwen_model.h:27-28). Tensors are tiled from one random block, each at its own shift."""
    NL, E, NH, NKV, HD, FF, V = 24, 896, 14, 2, 64, 4864, 151936
    rng = np.random.default_rng(seed)
    block = (rng.standard_normal(1 << 21) * 0.02).astype(np.float16)

    def lin(out, inn, k):
        return np.resize(np.roll(block, 7919 * k), out * inn).reshape(out, inn)

    def vec(n, mean, k):
        return (mean + np.resize(np.roll(block, 104729 * k), n).astype(np.float32)).astype(np.float32)
    kv = [("general.architecture", STRING, "qwen2"), ("qwen2.block_count", U32, NL),
          ("qwen2.embedding_length", U32, E), ("qwen2.feed_forward_length", U32, FF),
          ("qwen2.attention.head_count", U32, NH), ("qwen2.attention.head_count_kv", U32, NKV)]
    f16, f32 = GGML["f16"], GGML["f32"]
    t = [("token_embd.weight", f16, [E, V], lin(V, E, 1)), ("output.weight", f16, [E, V], lin(V, E, 2)),
         ("output_norm.weight", f32, [E], vec(E, 1.0, 3))]
    for l in range(NL):
        p, k = "blk.%d." % l, 10 * l + 5
        t += [(p + "attn_q.weight", f16, [E, NH * HD], lin(NH * HD, E, k)), (p + "attn_q.bias", f32, [NH * HD], vec(NH * HD, 0.0, k + 1)),
              (p + "attn_k.weight", f16, [E, NKV * HD], lin(NKV * HD, E, k + 2)), (p + "attn_k.bias", f32, [NKV * HD], vec(NKV * HD, 0.0, k + 3)),
              (p + "attn_v.weight", f16, [E, NKV * HD], lin(NKV * HD, E, k + 4)), (p + "attn_v.bias", f32, [NKV * HD], vec(NKV * HD, 0.0, k + 5)),
              (p + "attn_output.weight", f16, [NH * HD, E], lin(E, NH * HD, k + 6)),
              (p + "ffn_gate.weight", f16, [E, FF], lin(FF, E, k + 7)), (p + "ffn_up.weight", f16, [E, FF], lin(FF, E, k + 8)),
              (p + "ffn_down.weight", f16, [FF, E], lin(E, FF, k + 9)),
              (p + "attn_norm.weight", f32, [E], vec(E, 1.0, k + 10)), (p + "ffn_norm.weight", f32, [E], vec(E, 1.0, k + 11))]
    write_streaming(path, kv, t)
