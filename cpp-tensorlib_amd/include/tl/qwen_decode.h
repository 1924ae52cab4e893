#pragma once

// A Qwen2.5-architecture decoder driven imperatively through the tl::hip
// backend: the counterpart of the reference's bench/cuda/qwen_model.h
// (Layer/Scratch/Model: 175-308; run_layers_: 673-740; step_imperative:
// 747-752; captured_decoder: 791-905), with two differences that the task
// asks for: the dimensions are parameters (0.5B and 7B shapes), and weights
// come from memory blobs or from a GGUF file whose tensors are converted on the
// device (load_gguf).
//
// Per token and layer the step issues, in stream order and with no host sync:
//   fused QKV GEMV -> rope(q,+bias) , rope(k,+bias) , v += bias -> cache append
//   -> decode attention over the cache prefix -> o-proj GEMV
//   -> rmsnorm_res (x1 = x + attn ; h2 = norm(x1)) -> fused gate|up GEMV
//   -> swiglu -> down GEMV -> rmsnorm_res (x2 = x1 + mlp ; next layer's input norm)
// then the lm_head GEMV and a device argmax whose 4-byte copy is the single
// blocking call of the step. With model::fused (the default) the q/k/v epilogue is
// one launch and the norms and swiglu are evaluated inside the GEMV that consumes
// them: 6 launches per layer instead of 12.
//
// A prompt is consumed in chunks of T tokens (prefill_chunk, the counterpart of
// qm:357-395): the same layer wiring with every GEMV replaced by the MFMA GEMM
// over [T, hidden] activations, split_heads/rope/kv_fill/attn_prefill/merge_heads
// around the cache, and multi-row norms. Like the reference's, it needs bf16
// row-major weights.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include "gguf.h"
#include "hip.h"
#include "types.h"

namespace tl {
namespace qwen {

struct dims {
  int64_t n_layers, hidden, n_q_heads, n_kv_heads, head_dim, ff, vocab, max_ctx;
  float eps, rope_base;
  int64_t q_dim() const { return n_q_heads * head_dim; }
  int64_t kv_dim() const { return n_kv_heads * head_dim; }
  int64_t qkv_dim() const { return q_dim() + 2 * kv_dim(); }
};

inline dims qwen25_05b(int64_t max_ctx = 4096) {
  return dims{24, 896, 14, 2, 64, 4864, 151936, max_ctx, 1e-6f, 1e6f};
}
inline dims qwen25_7b(int64_t max_ctx = 4352) {
  return dims{28, 3584, 28, 4, 128, 18944, 152064, max_ctx, 1e-6f, 1e6f};
}

// A linear weight resident on the device. q4: the reference's one-buffer layout
// [packed [N][K/2] | scales [N][K/32]] (types.h:25-31). bf16_row: [N][K] bf16,
// the layout gemv_bf16_row and gemm_bf16_nt share (cuda.h:765-841).
enum class wfmt { q4, bf16_row };
struct linear {
  void* w = nullptr;
  int64_t N = 0, K = 0;
  wfmt fmt = wfmt::q4;
  int64_t bytes() const { return fmt == wfmt::q4 ? q4_bytes(N, K) : N * K * 2; }
};

// y[N] = a[K] . W
inline bool gemv(const linear& L, void* a, void* y) {
  if (L.fmt == wfmt::q4) {
    void* scales = static_cast<char*>(L.w) + L.N * L.K / 2;
    return hip::gemv_q4(a, L.w, scales, y, L.N, L.K, kQ4Group);
  }
  return hip::gemv_bf16_row(a, L.w, y, L.N, L.K);
}

// y = W . (attention output merged from n_parts split partials)
inline bool gemv_attn(const linear& L, void* parts, int n_parts, int64_t heads, int64_t head_dim, void* y) {
  if (L.fmt == wfmt::q4)
    return hip::gemv_q4_attn(parts, n_parts, heads, head_dim, L.w, static_cast<char*>(L.w) + L.N * L.K / 2, y, L.N,
                             L.K, kQ4Group);
  return hip::gemv_bf16_row_attn(parts, n_parts, heads, head_dim, L.w, y, L.N, L.K);
}

// Prompt-chunk products, T rows at a time: out[T, N] = a[T, K] . W^T for either weight format
// (bf16 rows or int4); `_parts` leaves the K-split parts for the launch that consumes them,
// `_swiglu` takes the fused [gate | up] weight and writes the gated activation [T, N / 2].
inline bool gemm(const linear& L, void* a, void* out, int64_t T) {
  if (L.fmt == wfmt::q4)
    return hip::gemm_q4_nt(a, L.w, static_cast<char*>(L.w) + L.N * L.K / 2, out, T, L.N, L.K, kQ4Group);
  return hip::gemm_bf16_nt(a, L.w, out, T, L.N, L.K);
}
inline bool gemm_parts(const linear& L, void* a, void* parts, int64_t parts_bytes, int64_t T, int* n_parts) {
  if (L.fmt == wfmt::q4)
    return hip::gemm_q4_nt_parts(a, L.w, static_cast<char*>(L.w) + L.N * L.K / 2, parts, parts_bytes, T, L.N,
                                 L.K, n_parts, kQ4Group);
  return hip::gemm_bf16_nt_parts(a, L.w, parts, parts_bytes, T, L.N, L.K, n_parts);
}
inline bool gemm_swiglu(const linear& L, void* a, void* act, int64_t T) {
  if (L.fmt == wfmt::q4)
    return hip::gemm_q4_nt_swiglu(a, L.w, static_cast<char*>(L.w) + L.N * L.K / 2, act, T, L.N / 2, L.K,
                                  kQ4Group);
  return hip::gemm_bf16_nt_swiglu(a, L.w, act, T, L.N / 2, L.K);
}

// y = W . swiglu(gu)
inline bool gemv_swiglu(const linear& L, void* gu, void* y) {
  if (L.fmt == wfmt::q4) {
    void* scales = static_cast<char*>(L.w) + L.N * L.K / 2;
    return hip::gemv_q4_swiglu(gu, L.w, scales, y, L.N, L.K, kQ4Group);
  }
  return hip::gemv_bf16_row_swiglu(gu, L.w, y, L.N, L.K);
}
// s = x (+ delta) -> xout ; y = W . rmsnorm(s, norm_w)
inline bool gemv_rmsnorm(const linear& L, void* x, void* delta, void* norm_w, void* xout, void* y,
                         float eps) {
  if (L.fmt == wfmt::q4) {
    void* scales = static_cast<char*>(L.w) + L.N * L.K / 2;
    return hip::gemv_q4_rmsnorm(x, delta, norm_w, xout, L.w, scales, y, L.N, L.K, kQ4Group, eps);
  }
  return hip::gemv_bf16_row_rmsnorm(x, delta, norm_w, xout, L.w, y, L.N, L.K, eps);
}

// L = [gate rows | up rows]; s = x (+ delta) -> xout ; act = swiglu(gate . n, up . n), n = rmsnorm(s, norm_w)
inline bool gemv_rmsnorm_gateup(const linear& L, void* x, void* delta, void* norm_w, void* xout, void* act,
                                float eps) {
  if (L.fmt == wfmt::q4) {
    void* scales = static_cast<char*>(L.w) + L.N * L.K / 2;
    return hip::gemv_q4_rmsnorm_gateup(x, delta, norm_w, xout, L.w, scales, act, L.N, L.K, kQ4Group, eps);
  }
  return hip::gemv_bf16_row_rmsnorm_gateup(x, delta, norm_w, xout, L.w, act, L.N, L.K, eps);
}

struct layer {
  linear wqkv, wo, wgu, wd;          // fused [wq|wk|wv] and [wg|wu] (qm:188-199)
  void* bqkv = nullptr;                              // fused bias [q_dim + 2 kv_dim] (qm:196)
  void *bq = nullptr, *bk = nullptr, *bv = nullptr;  // its three parts
  void *an = nullptr, *fn = nullptr;                 // attention / ffn norm weights [hidden]
  hip::kv_cache cache;
};

// Every per-step intermediate, allocated once (qm:208-246).
struct scratch {
  void* res[2] = {nullptr, nullptr};
  void *hb = nullptr, *h2b = nullptr, *qkvb = nullptr, *ab = nullptr, *mb = nullptr, *gub = nullptr,
       *mdb = nullptr, *logitsb = nullptr, *embedb = nullptr;
  float* embed_host = nullptr;
  float* logits_host = nullptr;
};

// Intermediates of a prompt chunk of up to T rows (qm:248-283), allocated on first use.
struct prefill_scratch {
  int64_t T = 0;
  void *emb = nullptr, *h = nullptr, *h2 = nullptr, *qkv = nullptr, *qkvh = nullptr, *ah = nullptr,
       *at = nullptr, *gu = nullptr, *mb = nullptr, *md = nullptr;
  void* res[2] = {nullptr, nullptr};
  void* rope = nullptr;         // (cos, sin)[T][head_dim/2] of the chunk being run
  void* parts = nullptr;        // K-split parts of the o-proj / down products, read by the residual norm
  int64_t parts_bytes = 0;
  float* emb_host = nullptr;
};

// GPU time per region of a decode step, from events on the library's stream around the launches
// of each region (the role of the reference harness's StepProf, qm:543-552, whose regions are
// host-side because its step is host-bound; this step is a chain of launches, so the regions are
// the launches). Sums over layers and steps, in milliseconds; `n` counts steps. The events cost
// a little GPU time themselves: read the shares, not the total, against an unprofiled step.
struct step_prof {
  double qkv = 0, attn = 0, oproj = 0, gateup = 0, down = 0, head = 0, total = 0;
  int64_t n = 0;
};

struct model {
  dims d{};
  prefill_scratch ps;
  std::vector<uint16_t> embed;  // [vocab, hidden] bf16 or f16 rows, gathered on the host (qm:530-535)
  bool embed_f16 = false;       // rows are IEEE half, as a model file stores token_embd (qm:297)
  void* onorm = nullptr;
  linear lm_head;
  std::vector<layer> layers;
  scratch s;
  void* rope_tab = nullptr;            // (cos, sin)[head_dim/2] of the step being run
  void* embed_dev = nullptr;           // the embedding table on the device (greedy_loop only)
  void* attn_partials = nullptr;       // split partials of the device-position attention
  int64_t attn_partials_bytes = 0;
  bool ready = false;
  // true: fused launches (q/k/v epilogue + append; norms and swiglu evaluated inside the
  // GEMV that consumes them). false: the reference's call sequence, one launch per op.
  bool fused = true;
  bool fused_attn = true;   // within the fused path: q/k/v epilogue + append inside the attention launch
  // within fused_attn: where the launch plan cuts the context into few splits (short contexts, small
  // models), the o-projection's GEMV merges them while it stages its input: no merge launch
  bool merge_in_oproj = true;
  bool fused_prefill = true;     // prompt chunks: one launch for split_heads + rope + kv_fill, attention writes token-major
  bool norm_images = true;       // prompt chunks: the residual norms leave the activation image of their output for the prepared-weight product that reads it
  bool prompt_f16 = true;        // prompt chunks of bf16 weights on the backend's prepared f16 form of them (a second copy, made on first use)
  bool gateup_epilogue = true;   // within the fused path: swiglu as the gate|up GEMV's epilogue, not the down GEMV's producer
  // within the fused path: blocks of the weight warm-up that runs beside each layer on a second
  // stream (0 = none); warm_nt: with streaming loads; warm_mode picks what is read when
  int warm_blocks = 0;
  bool warm_nt = false;
  int warm_mode = 0;
  std::vector<void*> prof_events;   // profile_step's events: 5 per layer + 2, recorded by run_layers when set
};

namespace detail {

inline void* dev_from_host(const void* src, int64_t bytes) {
  float* host = nullptr;
  void* n = hip::alloc(bytes, &host);
  if (!n) return nullptr;
  std::memcpy(host, src, (size_t)bytes);
  hip::upload(n, host, (bytes + 3) / 4);  // device copy current from now on
  return n;
}

// Rows of several q4 matrices with the same K, stacked: packed parts first,
// then the scale parts, which is again a valid q4 buffer of N = sum(N_i).
inline std::vector<uint8_t> fuse_q4(const std::vector<const uint8_t*>& parts,
                                    const std::vector<int64_t>& Ns, int64_t K) {
  int64_t N = 0;
  for (auto n : Ns) N += n;
  std::vector<uint8_t> out((size_t)q4_bytes(N, K));
  uint8_t* pk = out.data();
  uint8_t* sc = out.data() + N * K / 2;
  for (size_t i = 0; i < parts.size(); i++) {
    const int64_t pb = Ns[i] * K / 2, sb = Ns[i] * (K / kQ4Group) * 4;
    std::memcpy(pk, parts[i], (size_t)pb);
    std::memcpy(sc, parts[i] + pb, (size_t)sb);
    pk += pb;
    sc += sb;
  }
  return out;
}

// [K,N] -> [N,K]
inline void transpose_kn(const uint16_t* src, uint16_t* dst, int64_t K, int64_t N) {
  for (int64_t k = 0; k < K; k++)
    for (int64_t n = 0; n < N; n++) dst[n * K + k] = src[k * N + n];
}

}  // namespace detail

// Host-side description of one layer's weights in the reference's storage
// forms: q4 buffers of logical [K,N] weights (array.h:703-742) and f32 vectors.
struct layer_blobs {
  const uint8_t *wq, *wk, *wv, *wo, *wg, *wu, *wd;
  const float *bq, *bk, *bv, *an, *fn;
};

namespace detail {
// Biases (one fused buffer, as the prefill path wants it) and norm weights.
inline bool set_vectors(model& M, layer& L, const float* bq, const float* bk, const float* bv,
                        const float* an, const float* fn) {
  const dims& d = M.d;
  std::vector<float> fused((size_t)d.qkv_dim());
  std::memcpy(fused.data(), bq, (size_t)d.q_dim() * 4);
  std::memcpy(fused.data() + d.q_dim(), bk, (size_t)d.kv_dim() * 4);
  std::memcpy(fused.data() + d.q_dim() + d.kv_dim(), bv, (size_t)d.kv_dim() * 4);
  L.bqkv = dev_from_host(fused.data(), d.qkv_dim() * 4);
  if (!L.bqkv) return false;
  L.bq = L.bqkv;
  L.bk = static_cast<char*>(L.bqkv) + d.q_dim() * 4;
  L.bv = static_cast<char*>(L.bqkv) + (d.q_dim() + d.kv_dim()) * 4;
  L.an = dev_from_host(an, d.hidden * 4);
  L.fn = dev_from_host(fn, d.hidden * 4);
  return L.an && L.fn;
}
}  // namespace detail

inline bool init(model& M, const dims& d) {
  if (!hip::available()) return false;
  M.d = d;
  M.layers.assign((size_t)d.n_layers, layer{});
  auto A = [](int64_t n) { return hip::alloc(n * 4, nullptr); };
  scratch& S = M.s;
  S.embedb = hip::alloc(d.hidden * 4, &S.embed_host);
  S.res[0] = A(d.hidden);
  S.res[1] = A(d.hidden);
  S.hb = A(d.hidden);
  S.h2b = A(d.hidden);
  S.qkvb = A(d.qkv_dim());
  S.ab = A(d.q_dim());
  S.mb = A(d.ff);
  S.gub = A(2 * d.ff);
  S.mdb = A(d.hidden);
  S.logitsb = hip::alloc(d.vocab * 4, &S.logits_host);
  for (auto& L : M.layers)
    if (!L.cache.init(d.n_kv_heads, d.max_ctx, d.head_dim)) return false;
  M.attn_partials_bytes = hip::attn_partials_bytes(d.n_q_heads, d.n_kv_heads, d.max_ctx, d.head_dim);
  M.attn_partials = hip::alloc_device(M.attn_partials_bytes);
  return S.logitsb != nullptr && S.embedb != nullptr && M.attn_partials != nullptr;
}

inline bool set_layer_q4(model& M, int64_t li, const layer_blobs& b) {
  const dims& d = M.d;
  layer& L = M.layers[(size_t)li];
  const int64_t E = d.hidden;
  auto fused_qkv = detail::fuse_q4({b.wq, b.wk, b.wv}, {d.q_dim(), d.kv_dim(), d.kv_dim()}, E);
  auto fused_gu = detail::fuse_q4({b.wg, b.wu}, {d.ff, d.ff}, E);
  L.wqkv = linear{detail::dev_from_host(fused_qkv.data(), (int64_t)fused_qkv.size()), d.qkv_dim(), E,
                  wfmt::q4};
  L.wgu = linear{detail::dev_from_host(fused_gu.data(), (int64_t)fused_gu.size()), 2 * d.ff, E,
                 wfmt::q4};
  L.wo = linear{detail::dev_from_host(b.wo, q4_bytes(E, d.q_dim())), E, d.q_dim(), wfmt::q4};
  L.wd = linear{detail::dev_from_host(b.wd, q4_bytes(E, d.ff)), E, d.ff, wfmt::q4};
  return detail::set_vectors(M, L, b.bq, b.bk, b.bv, b.an, b.fn) && L.wqkv.w && L.wgu.w && L.wo.w &&
         L.wd.w;
}

// The same layer from bf16 blobs in the reference's logical [K,N] layout
// (array.h:639-658): transposed on the host to [N,K] rows, the layout the decode
// GEMV and the prefill GEMM share (qm:118-146 does this transpose at load).
struct layer_blobs_bf16 {
  const uint16_t *wq, *wk, *wv, *wo, *wg, *wu, *wd;
  const float *bq, *bk, *bv, *an, *fn;
};

inline bool set_layer_bf16(model& M, int64_t li, const layer_blobs_bf16& b) {
  const dims& d = M.d;
  layer& L = M.layers[(size_t)li];
  const int64_t E = d.hidden;
  std::vector<uint16_t> rows;
  auto put = [&](std::vector<const uint16_t*> parts, std::vector<int64_t> Ns, int64_t K) {
    int64_t N = 0;
    for (auto n : Ns) N += n;
    rows.resize((size_t)(N * K));
    int64_t n0 = 0;
    for (size_t i = 0; i < parts.size(); i++) {
      detail::transpose_kn(parts[i], rows.data() + n0 * K, K, Ns[i]);
      n0 += Ns[i];
    }
    return linear{detail::dev_from_host(rows.data(), N * K * 2), N, K, wfmt::bf16_row};
  };
  L.wqkv = put({b.wq, b.wk, b.wv}, {d.q_dim(), d.kv_dim(), d.kv_dim()}, E);
  L.wgu = put({b.wg, b.wu}, {d.ff, d.ff}, E);
  L.wo = put({b.wo}, {E}, d.q_dim());
  L.wd = put({b.wd}, {E}, d.ff);
  return detail::set_vectors(M, L, b.bq, b.bk, b.bv, b.an, b.fn) && L.wqkv.w && L.wgu.w && L.wo.w &&
         L.wd.w;
}

inline bool set_head_bf16(model& M, const uint16_t* embed_bf16, const float* onorm,
                          const uint16_t* outw_kn) {
  const dims& d = M.d;
  M.embed.assign(embed_bf16, embed_bf16 + d.vocab * d.hidden);
  M.onorm = detail::dev_from_host(onorm, d.hidden * 4);
  std::vector<uint16_t> rows((size_t)(d.vocab * d.hidden));
  detail::transpose_kn(outw_kn, rows.data(), d.hidden, d.vocab);
  M.lm_head = linear{detail::dev_from_host(rows.data(), d.vocab * d.hidden * 2), d.vocab, d.hidden,
                     wfmt::bf16_row};
  M.ready = M.onorm && M.lm_head.w;
  return M.ready;
}

inline bool set_head_q4(model& M, const uint16_t* embed_bf16, const float* onorm,
                        const uint8_t* outw_q4) {
  const dims& d = M.d;
  M.embed.assign(embed_bf16, embed_bf16 + d.vocab * d.hidden);
  M.onorm = detail::dev_from_host(onorm, d.hidden * 4);
  M.lm_head = linear{detail::dev_from_host(outw_q4, q4_bytes(d.vocab, d.hidden)), d.vocab, d.hidden,
                     wfmt::q4};
  M.ready = M.onorm && M.lm_head.w;
  return M.ready;
}

// Synthetic weights for throughput runs (a 7B-shape model is 4.4 GB of int4):
// one 32 MB block of seeded random nibbles and one of scales ~U(0.002,0.006) are
// uploaded once and tiled into device-only weight buffers with device copies.
// Values do not affect kernel time; they keep activations finite.
inline bool set_random(model& M, uint32_t seed, wfmt fmt) {
  const dims& d = M.d;
  const int64_t blk = int64_t(32) << 20;
  std::vector<uint32_t> nib((size_t)blk / 4);
  std::vector<float> scl((size_t)blk / 4);
  uint32_t s = seed * 2654435761u + 1u;
  auto next = [&s] { s ^= s << 13; s ^= s >> 17; s ^= s << 5; return s; };
  for (auto& v : nib) v = next();
  for (auto& v : scl) v = 0.002f + 0.004f * (float)(next() >> 8) * (1.0f / 16777216.0f);
  void* dn = detail::dev_from_host(nib.data(), blk);
  void* ds = detail::dev_from_host(scl.data(), blk);
  if (!dn || !ds) return false;
  bool ok = true;
  // bf16: the scale block doubles as the weight pattern once its exponent bits are
  // pinned to [2^-7, 2^-6) with random sign, so |w| ~ 0.01
  std::vector<uint32_t> bfw((size_t)blk / 4);
  for (auto& v : bfw) v = (next() & 0x807f807fu) | 0x3c003c00u;
  void* db = fmt == wfmt::bf16_row ? detail::dev_from_host(bfw.data(), blk) : nullptr;
  auto make = [&](int64_t N, int64_t K) {
    if (fmt == wfmt::bf16_row) {
      linear L{hip::alloc_device(N * K * 2), N, K, wfmt::bf16_row};
      if (!L.w || !db) { ok = false; return L; }
      for (int64_t o = 0; o < N * K * 2; o += blk)
        ok &= hip::copy_d2d(static_cast<char*>(L.w) + o, db, std::min(blk, N * K * 2 - o));
      return L;
    }
    linear L{hip::alloc_device(q4_bytes(N, K)), N, K, wfmt::q4};
    if (!L.w) { ok = false; return L; }
    const int64_t pb = N * K / 2, sb = N * (K / kQ4Group) * 4;
    for (int64_t o = 0; o < pb; o += blk)
      ok &= hip::copy_d2d(static_cast<char*>(L.w) + o, dn, std::min(blk, pb - o));
    for (int64_t o = 0; o < sb; o += blk)
      ok &= hip::copy_d2d(static_cast<char*>(L.w) + pb + o, ds, std::min(blk, sb - o));
    return L;
  };
  auto hvec = [&](int64_t n, float mean, float std_) {
    std::vector<float> v((size_t)n);
    for (auto& e : v) e = mean + std_ * ((float)(int32_t)next() * (1.0f / 2147483648.0f));
    return v;
  };
  for (auto& L : M.layers) {
    L.wqkv = make(d.qkv_dim(), d.hidden);
    L.wo = make(d.hidden, d.q_dim());
    L.wgu = make(2 * d.ff, d.hidden);
    L.wd = make(d.hidden, d.ff);
    const auto bq = hvec(d.q_dim(), 0.f, 0.02f), bk = hvec(d.kv_dim(), 0.f, 0.02f),
               bv = hvec(d.kv_dim(), 0.f, 0.02f), an = hvec(d.hidden, 1.f, 0.02f),
               fn = hvec(d.hidden, 1.f, 0.02f);
    ok = ok && detail::set_vectors(M, L, bq.data(), bk.data(), bv.data(), an.data(), fn.data());
  }
  M.lm_head = make(d.vocab, d.hidden);
  M.onorm = detail::dev_from_host(hvec(d.hidden, 1.f, 0.02f).data(), d.hidden * 4);
  M.embed.resize((size_t)(d.vocab * d.hidden));
  for (size_t i = 0; i < M.embed.size(); i++)
    M.embed[i] = f32_to_bf16(0.02f * ((float)(int32_t)next() * (1.0f / 2147483648.0f)));
  hip::flush();
  M.ready = ok && M.onorm;
  return M.ready;
}
inline bool set_random_q4(model& M, uint32_t seed) { return set_random(M, seed, wfmt::q4); }
inline bool set_random_bf16(model& M, uint32_t seed) { return set_random(M, seed, wfmt::bf16_row); }

// Fill every layer's cache rows [0, upto) with seeded N(0,1)-like values so a
// decode step at a deep position reads a realistic cache.
inline bool fill_cache_random(model& M, int64_t upto, uint32_t seed) {
  const dims& d = M.d;
  const int64_t per = d.n_kv_heads * d.max_ctx * d.head_dim;
  std::vector<float> blkv((size_t)per);
  uint32_t s = seed * 2654435761u + 7u;
  auto next = [&s] { s ^= s << 13; s ^= s >> 17; s ^= s << 5; return s; };
  for (auto& e : blkv) {  // sum of 4 uniforms: variance 1, near-normal
    float a = 0.f;
    for (int i = 0; i < 4; i++) a += (float)(int32_t)next() * (1.0f / 2147483648.0f);
    e = a * 0.8660254f;
  }
  void* stage = detail::dev_from_host(blkv.data(), per * 4);
  if (!stage) return false;
  bool ok = true;
  for (auto& L : M.layers) {
    ok &= hip::copy_d2d(L.cache.K, stage, per * 4);
    ok &= hip::copy_d2d(L.cache.V, stage, per * 4);
    L.cache.pos = upto;
  }
  hip::flush();
  hip::release(stage, 0, nullptr);
  return ok;
}

// ---- a model file as the source of the weights (qm:449-505 build) ---------------------------
// The reference widens every f16 tensor to f32 on the host, transposes or stacks it there,
// narrows to bf16 / quantises to int4 and uploads the result. Here the mapped file bytes go
// to the device as they are, through one staging buffer, and tlhip_convert /
// tlhip_quantize_q4 write the decode formats straight into the fused weight buffers:
// the same values bit for bit, with the element loops on the GPU.
namespace detail {

inline bool why_(std::string* why, const std::string& msg) {
  if (why) *why = msg;
  return false;
}

inline bool elem_of(gguf::ggml_type t, hip::elem& e) {
  switch (t) {
    case gguf::ggml_type::f32: e = hip::elem::f32; return true;
    case gguf::ggml_type::f16: e = hip::elem::f16; return true;
    case gguf::ggml_type::bf16: e = hip::elem::bf16; return true;
    default: return false;   // block-quantised files: dequantisation is the consumer's job, not built
  }
}
inline int64_t elem_bytes(hip::elem e) { return e == hip::elem::f32 ? 4 : 2; }

// Uploads file tensors through one device staging buffer and converts them in place.
struct converter {
  void* stage = nullptr;
  int64_t stage_bytes = 0;
  bool init(int64_t bytes = int64_t(64) << 20) {
    stage_bytes = bytes;
    stage = hip::alloc_device(bytes);
    return stage != nullptr;
  }
  void destroy() {
    if (stage) hip::release(stage, 0, nullptr);
    stage = nullptr;
  }
  // Rows [out, in] of one file tensor into rows [row_base, row_base + out) of `dst`.
  bool rows_into(const gguf::tensor_info& t, int64_t out, int64_t in, const linear& dst, int64_t row_base) {
    hip::elem e;
    if (!elem_of(t.type, e)) return false;
    const int64_t row_bytes = in * elem_bytes(e);
    int64_t per = stage_bytes / row_bytes;      // whole rows per staged piece
    if (per < 1) return false;
    const char* src = static_cast<const char*>(t.data);
    char* w = static_cast<char*>(dst.w);
    for (int64_t r = 0; r < out; r += per) {
      const int64_t n = std::min(per, out - r);
      if (!hip::upload_raw(stage, src + r * row_bytes, n * row_bytes)) return false;
      const int64_t row = row_base + r;
      bool ok;
      if (dst.fmt == wfmt::q4)
        ok = hip::quantize_q4(stage, e, w + row * in / 2,
                              w + dst.N * in / 2 + row * (in / kQ4Group) * 4, n, in);
      else
        ok = hip::convert(stage, e, w + row * in * 2, hip::elem::bf16, n * in);
      if (!ok) return false;
    }
    return true;
  }
};

// A linear layer's file tensor must be 2-D with dims {in, out} (dims[0] is the contiguous axis).
inline const gguf::tensor_info* linear_tensor(const gguf::model& g, const std::string& name, int64_t in,
                                              int64_t out, std::string* why) {
  const gguf::tensor_info* t = g.tensor(name);
  if (!t) { why_(why, "missing tensor " + name); return nullptr; }
  hip::elem e;
  if (!elem_of(t->type, e)) { why_(why, name + ": storage type not supported (f32, f16, bf16 only)"); return nullptr; }
  if (t->dims.size() != 2 || (int64_t)t->dims[0] != in || (int64_t)t->dims[1] != out) {
    why_(why, name + ": shape does not match the hyperparameters");
    return nullptr;
  }
  return t;
}

// An f32 vector of the file (norm weights, biases); `optional` ones default to a constant.
inline bool vector_f32(const gguf::model& g, const std::string& name, int64_t len, bool optional,
                       float fill, std::vector<float>& out, std::string* why) {
  out.assign((size_t)len, fill);
  const gguf::tensor_info* t = g.tensor(name);
  if (!t) return optional ? true : why_(why, "missing tensor " + name);
  if (t->type != gguf::ggml_type::f32 || (int64_t)t->n_elements() != len)
    return why_(why, name + ": expected " + std::to_string(len) + " f32 values");
  std::memcpy(out.data(), t->data, (size_t)len * 4);
  return true;
}

}  // namespace detail

// Hyperparameters from the metadata (`<arch>.block_count` ..., arch = general.architecture,
// "qwen2" when absent: qm:918-922 checks exactly these keys) and from token_embd's shape.
inline bool dims_from_gguf(const gguf::model& g, int64_t max_ctx, dims& d, std::string* why = nullptr) {
  try {
    const std::string a = (g.has("general.architecture") ? g.kv("general.architecture").as_str() : "qwen2") + ".";
    d.n_layers = (int64_t)g.kv(a + "block_count").as_count();
    d.hidden = (int64_t)g.kv(a + "embedding_length").as_count();
    d.ff = (int64_t)g.kv(a + "feed_forward_length").as_count();
    d.n_q_heads = (int64_t)g.kv(a + "attention.head_count").as_count();
    d.n_kv_heads = g.has(a + "attention.head_count_kv") ? (int64_t)g.kv(a + "attention.head_count_kv").as_count()
                                                         : d.n_q_heads;
    if (d.n_q_heads <= 0) return detail::why_(why, "attention.head_count is zero");
    d.head_dim = g.has(a + "attention.key_length") ? (int64_t)g.kv(a + "attention.key_length").as_count()
                                                   : d.hidden / d.n_q_heads;
    d.eps = g.has(a + "attention.layer_norm_rms_epsilon") ? g.kv(a + "attention.layer_norm_rms_epsilon").as_f32() : 1e-6f;
    d.rope_base = g.has(a + "rope.freq_base") ? g.kv(a + "rope.freq_base").as_f32() : 1e6f;
    const gguf::tensor_info* emb = g.tensor("token_embd.weight");
    if (!emb || emb->dims.size() != 2 || (int64_t)emb->dims[0] != d.hidden)
      return detail::why_(why, "token_embd.weight missing or not [vocab, hidden]");
    d.vocab = (int64_t)emb->dims[1];
    d.max_ctx = max_ctx;
    if (g.has(a + "context_length")) d.max_ctx = std::min<int64_t>(max_ctx, (int64_t)g.kv(a + "context_length").as_count());
  } catch (const std::exception& e) {
    return detail::why_(why, e.what());
  }
  if (d.n_layers <= 0 || d.hidden <= 0 || d.ff <= 0 || d.n_kv_heads <= 0 || d.n_q_heads % d.n_kv_heads != 0 ||
      (d.head_dim != 64 && d.head_dim != 128) || d.max_ctx <= 0 || d.hidden % kQ4Group != 0 ||
      d.ff % kQ4Group != 0 || d.q_dim() % kQ4Group != 0)
    return detail::why_(why, "hyperparameters outside what the decode path takes");
  return true;
}

// Builds the model from a mapped file: linear layers into `fmt` (int4 groups or bf16 rows),
// fused [q|k|v] and [gate|up] by stacking row blocks; norms and biases f32; the embedding
// stays in the file's f16 (bf16 accepted) and is gathered per token. output.weight may be
// absent (tied to token_embd.weight).
inline bool load_gguf(model& M, const gguf::model& g, wfmt fmt, int64_t max_ctx = 4096,
                      std::string* why = nullptr) {
  dims d{};
  if (!dims_from_gguf(g, max_ctx, d, why)) return false;
  if (!init(M, d)) return detail::why_(why, "GPU backend unavailable or out of memory");
  detail::converter cv;
  if (!cv.init()) return detail::why_(why, "no staging buffer");
  const int64_t E = d.hidden;
  auto make = [&](int64_t N, int64_t K) {
    linear L{nullptr, N, K, fmt};
    L.w = hip::alloc_device(L.bytes());
    return L;
  };
  struct part { std::string name; int64_t out; };
  auto fill = [&](linear& L, std::vector<part> parts) {
    if (!L.w) return detail::why_(why, "out of device memory");
    int64_t row = 0;
    for (const auto& p : parts) {
      const gguf::tensor_info* t = detail::linear_tensor(g, p.name, L.K, p.out, why);
      if (!t) return false;
      if (!cv.rows_into(*t, p.out, L.K, L, row)) return detail::why_(why, p.name + ": conversion failed");
      row += p.out;
    }
    return true;
  };
  bool ok = true;
  std::vector<float> bq, bk, bv, an, fn;
  for (int64_t l = 0; l < d.n_layers && ok; l++) {
    layer& L = M.layers[(size_t)l];
    const std::string p = "blk." + std::to_string(l) + ".";
    L.wqkv = make(d.qkv_dim(), E);
    L.wo = make(E, d.q_dim());
    L.wgu = make(2 * d.ff, E);
    L.wd = make(E, d.ff);
    ok = fill(L.wqkv, {{p + "attn_q.weight", d.q_dim()}, {p + "attn_k.weight", d.kv_dim()}, {p + "attn_v.weight", d.kv_dim()}}) &&
         fill(L.wo, {{p + "attn_output.weight", E}}) &&
         fill(L.wgu, {{p + "ffn_gate.weight", d.ff}, {p + "ffn_up.weight", d.ff}}) &&
         fill(L.wd, {{p + "ffn_down.weight", E}}) &&
         detail::vector_f32(g, p + "attn_q.bias", d.q_dim(), true, 0.f, bq, why) &&
         detail::vector_f32(g, p + "attn_k.bias", d.kv_dim(), true, 0.f, bk, why) &&
         detail::vector_f32(g, p + "attn_v.bias", d.kv_dim(), true, 0.f, bv, why) &&
         detail::vector_f32(g, p + "attn_norm.weight", E, false, 1.f, an, why) &&
         detail::vector_f32(g, p + "ffn_norm.weight", E, false, 1.f, fn, why) &&
         detail::set_vectors(M, L, bq.data(), bk.data(), bv.data(), an.data(), fn.data());
  }
  if (ok) {
    std::vector<float> on;
    ok = detail::vector_f32(g, "output_norm.weight", E, false, 1.f, on, why);
    if (ok) M.onorm = detail::dev_from_host(on.data(), E * 4);
    M.lm_head = make(d.vocab, E);
    const char* head = g.tensor("output.weight") ? "output.weight" : "token_embd.weight";
    ok = ok && M.onorm && fill(M.lm_head, {{head, d.vocab}});
  }
  if (ok) {
    const gguf::tensor_info* emb = g.tensor("token_embd.weight");
    if (emb->type == gguf::ggml_type::f16) M.embed_f16 = true;
    else if (emb->type == gguf::ggml_type::bf16) M.embed_f16 = false;
    else ok = detail::why_(why, "token_embd.weight: f16 or bf16 expected");
    if (ok) {
      const uint16_t* rows = static_cast<const uint16_t*>(emb->data);
      M.embed.assign(rows, rows + d.vocab * E);
    }
  }
  hip::flush();
  cv.destroy();
  M.ready = ok;
  return ok;
}

inline void reset_cache(model& M) {
  for (auto& L : M.layers) L.cache.pos = 0;
}
inline void set_cache_pos(model& M, int64_t p) {
  for (auto& L : M.layers) L.cache.pos = p;
}

// Widen one embedding row into the staged input (host gather, one small H2D).
// false for a token id outside [0, vocab): nothing is read or uploaded.
inline bool stage_embed(model& M, int64_t token) {
  const dims& d = M.d;
  if (token < 0 || token >= d.vocab) return false;
  const uint16_t* r = M.embed.data() + (size_t)token * d.hidden;
  if (M.embed_f16)
    for (int64_t j = 0; j < d.hidden; j++) M.s.embed_host[j] = f16_to_f32(r[j]);
  else
    for (int64_t j = 0; j < d.hidden; j++) M.s.embed_host[j] = bf16_to_f32(r[j]);
  hip::upload(M.s.embedb, M.s.embed_host, d.hidden);
  return true;
}

// All layers + final norm + lm_head on the scratch buffers, no allocation, no
// sync: capturable as one graph. Reads the layer-0 residual from x0, writes
// logits to S.logitsb (or logits_out).
// With d_pos (a 4-byte device scalar holding the position) the cache append and the
// attention take the position from the device on position-independent grids, and the
// scalar is advanced at the end: the launch sequence is then the same for every
// token and one recorded graph serves a whole decode loop (qm:673-740 with d_pos).
inline bool run_layers(model& M, void* x0, int64_t pos, void* logits_out = nullptr,
                       void* d_pos = nullptr, bool advance = true) {
  const dims& d = M.d;
  scratch& S = M.s;
  const float scale = 1.0f / std::sqrt((float)d.head_dim);
  const int64_t E = d.hidden, QD = d.q_dim(), KD = d.kv_dim();
  bool ok = true;
  if (M.fused) {
    // 5 launches per layer (+1 when attention splits the context and the o-projection does not merge):
    //   [norm -> qkv GEMV] , [q/k/v epilogue + append -> attention] , o-proj GEMV ,
    //   [residual + norm -> gate|up GEMV] , [swiglu -> down GEMV]
    // (fused_attn = false runs the q/k/v epilogue as a launch of its own)
    // The residual stream ping-pongs between res[0] and res[1] because a fused GEMV
    // may not write the residual over a vector its other blocks still read.
    void* rin = x0;          // residual entering the layer
    void* din = nullptr;     // MLP output of the previous layer, not yet added
    if (!M.rope_tab) M.rope_tab = hip::alloc_device(d.head_dim * 4);
    ok &= M.rope_tab && hip::rope_table(M.rope_tab, d.head_dim, pos, d_pos, d.rope_base);
    // the attention's splits merged by the o-projection: decided once per step from the launch plan
    const bool merge = M.fused_attn && M.merge_in_oproj && M.attn_partials &&
                       hip::attn_parts_splits(d.n_q_heads, d.n_kv_heads, d_pos ? M.layers[0].cache.max_ctx : pos + 1,
                                              d.head_dim, M.layers[0].cache.kv_bf16) > 0;
    size_t marks = 0;
    auto mark = [&] { if (marks < M.prof_events.size()) ok &= hip::event_record(M.prof_events[marks++]); };
    for (int64_t l = 0; l < d.n_layers; l++) {
      layer& L = M.layers[(size_t)l];
      mark();
      auto warm = [&](int mode) {
        if (M.warm_blocks == 0 || M.warm_mode != mode) return;
        const linear& nx = (l + 1 < d.n_layers) ? M.layers[(size_t)l + 1].wqkv : M.lm_head;
        const void* p[4] = {L.wo.w, L.wgu.w, L.wd.w, nx.w};
        int64_t b[4] = {L.wo.bytes(), L.wgu.bytes(), L.wd.bytes(), std::min<int64_t>(nx.bytes(), int64_t(16) << 20)};
        for (auto& x : b) x &= ~int64_t(15);
        ok &= hip::warm_fork(p, b, mode == 1 || mode == 3 ? 2 : mode == 4 ? 3 : 4, M.warm_blocks, M.warm_nt);
      };
      warm(0); warm(1);            // beside the whole layer: everything / o-proj and gate|up only
      ok &= gemv_rmsnorm(L.wqkv, rin, din, L.an, S.res[0], S.qkvb, d.eps);
      warm(2); warm(3); warm(4);   // beside attention: everything / o-proj and gate|up / + down
      mark();
      int n_parts = 0;
      if (merge) {
        if (!d_pos) L.cache.pos = pos;
        ok &= L.cache.attn_qkv_parts(S.qkvb, L.bq, L.bk, L.bv, d.n_q_heads, scale, M.rope_tab, d_pos, M.attn_partials,
                                     M.attn_partials_bytes, &n_parts);
      } else if (M.fused_attn) {
        if (!d_pos) L.cache.pos = pos;
        ok &= L.cache.attn_qkv(S.qkvb, L.bq, L.bk, L.bv, S.ab, d.n_q_heads, scale, M.rope_tab, d_pos,
                               d_pos ? M.attn_partials : nullptr, d_pos ? M.attn_partials_bytes : 0);
      } else if (d_pos) {
        ok &= L.cache.rope_append_tab(S.qkvb, L.bq, L.bk, L.bv, d.n_q_heads, M.rope_tab, d_pos);
        ok &= L.cache.attn_dpos(S.qkvb, S.ab, d.n_q_heads, scale, d_pos, M.attn_partials,
                                M.attn_partials_bytes);
      } else {
        L.cache.pos = pos;
        ok &= L.cache.rope_append_tab(S.qkvb, L.bq, L.bk, L.bv, d.n_q_heads, M.rope_tab);
        ok &= L.cache.attn(S.qkvb, S.ab, d.n_q_heads, scale);
      }
      mark();
      ok &= merge ? gemv_attn(L.wo, M.attn_partials, n_parts, d.n_q_heads, d.head_dim, S.hb) : gemv(L.wo, S.ab, S.hb);
      mark();
      if (M.gateup_epilogue) {
        ok &= gemv_rmsnorm_gateup(L.wgu, S.res[0], S.hb, L.fn, S.res[1], S.mb, d.eps);
        mark();
        ok &= gemv(L.wd, S.mb, S.mdb);
      } else {
        ok &= gemv_rmsnorm(L.wgu, S.res[0], S.hb, L.fn, S.res[1], S.gub, d.eps);
        mark();
        ok &= gemv_swiglu(L.wd, S.gub, S.mdb);
      }
      rin = S.res[1];
      din = S.mdb;
    }
    mark();
    ok &= gemv_rmsnorm(M.lm_head, rin, din, M.onorm, nullptr, logits_out ? logits_out : S.logitsb, d.eps);
    mark();
    if (M.warm_blocks != 0) ok &= hip::warm_join();
    if (d_pos && advance) ok &= hip::incr_u32(d_pos);
    return ok;
  }
  if (d_pos) return false;  // the one-launch-per-op sequence is kept on the host position
  void* x = x0;
  ok &= hip::rmsnorm(x, M.layers[0].an, S.hb, E, d.eps);
  for (int64_t l = 0; l < d.n_layers; l++) {
    layer& L = M.layers[(size_t)l];
    void* ro = S.res[l & 1];
    ok &= gemv(L.wqkv, S.hb, S.qkvb);
    void* qp = S.qkvb;
    void* kp = static_cast<char*>(S.qkvb) + QD * 4;
    void* vp = static_cast<char*>(S.qkvb) + (QD + KD) * 4;
    L.cache.pos = pos;
    // the reference's call sequence, one launch per op (qm:703-716)
    ok &= hip::rope(qp, qp, d.n_q_heads, 1, d.head_dim, pos, d.rope_base, L.bq);
    ok &= hip::rope(kp, kp, d.n_kv_heads, 1, d.head_dim, pos, d.rope_base, L.bk);
    ok &= hip::binary(hip::kop::add, vp, 0, L.bv, 0, vp, 0, KD, 1.0f, 0.0f);
    ok &= L.cache.append(kp, vp);
    ok &= L.cache.attn(qp, S.ab, d.n_q_heads, scale);
    ok &= gemv(L.wo, S.ab, ro);
    ok &= hip::rmsnorm_res(ro, x, L.fn, ro, S.h2b, E, d.eps);
    ok &= gemv(L.wgu, S.h2b, S.gub);
    ok &= hip::swiglu(S.gub, S.mb, d.ff);
    ok &= gemv(L.wd, S.mb, S.mdb);
    void* nextw = (l + 1 < d.n_layers) ? M.layers[(size_t)l + 1].an : M.onorm;
    ok &= hip::rmsnorm_res(ro, S.mdb, nextw, ro, S.hb, E, d.eps);
    x = ro;
  }
  ok &= gemv(M.lm_head, S.hb, logits_out ? logits_out : S.logitsb);
  return ok;
}

// One eager step of the fused launch sequence with an event between its regions; the regions'
// GPU times are added to `p`. false when a launch or an event was declined.
inline bool profile_step(model& M, int64_t token, int64_t pos, step_prof& p) {
  if (!M.fused || !stage_embed(M, token)) return false;
  const size_t L = (size_t)M.d.n_layers, want = 5 * L + 2;
  while (M.prof_events.size() < want) {
    void* ev = hip::event_create();
    if (!ev) break;
    M.prof_events.push_back(ev);
  }
  bool ok = M.prof_events.size() == want && run_layers(M, M.s.embedb, pos);
  hip::flush();
  std::vector<void*> ev;
  ev.swap(M.prof_events);          // later steps run without marks
  if (ok) {
    auto ms = [&](size_t a, size_t b) { return (double)hip::event_elapsed_ms(ev[a], ev[b]); };
    for (size_t l = 0; l < L; l++) {
      p.qkv += ms(5 * l, 5 * l + 1);
      p.attn += ms(5 * l + 1, 5 * l + 2);
      p.oproj += ms(5 * l + 2, 5 * l + 3);
      p.gateup += ms(5 * l + 3, 5 * l + 4);
      p.down += ms(5 * l + 4, 5 * l + 5);
    }
    p.head += ms(5 * L, 5 * L + 1);
    p.total += ms(0, 5 * L + 1);
    p.n++;
  }
  for (void* e : ev) hip::event_destroy(e);
  return ok;
}

// embed -> layers -> device argmax. Returns the greedy token, or -1 when any
// launch was declined.
inline int64_t step_greedy(model& M, int64_t token, int64_t pos) {
  if (!stage_embed(M, token) || !run_layers(M, M.s.embedb, pos)) return -1;
  int64_t idx = -1;
  if (!hip::argmax(M.s.logitsb, M.d.vocab, &idx)) return -1;
  return idx;
}

// Host view of the logits the last step left on the device.
inline const float* logits(model& M) {
  hip::sync_to_host(M.s.logitsb, false);
  return M.s.logits_host;
}

// ---- prompt chunks ---------------------------------------------------------------------------

inline bool prefill_reserve(model& M, int64_t T) {
  prefill_scratch& P = M.ps;
  if (P.T >= T) return true;
  const dims& d = M.d;
  auto A = [](int64_t n) { return hip::alloc_device(n * 4); };
  for (void* b : {P.emb, P.h, P.h2, P.qkv, P.qkvh, P.ah, P.at, P.gu, P.mb, P.md, P.res[0], P.res[1], P.rope, P.parts})
    if (b) hip::release(b, 0, nullptr);
  P.emb = hip::alloc(T * d.hidden * 4, &P.emb_host);
  P.h = A(T * d.hidden);
  P.h2 = A(T * d.hidden);
  P.qkv = A(T * d.qkv_dim());
  P.qkvh = A(T * d.qkv_dim());
  P.ah = A(T * d.q_dim());
  P.at = A(T * d.q_dim());
  P.gu = A(T * 2 * d.ff);
  P.mb = A(T * d.ff);
  P.md = A(T * d.hidden);
  P.res[0] = A(T * d.hidden);
  P.res[1] = A(T * d.hidden);
  P.rope = A(T * d.head_dim);
  P.parts_bytes = 16 * T * std::max(d.hidden, d.qkv_dim()) * 4;   // the GEMM splits K at most 16 ways
  P.parts = hip::alloc_device(P.parts_bytes);
  const bool ok = P.emb && P.h && P.h2 && P.qkv && P.qkvh && P.ah && P.at && P.gu && P.mb && P.md &&
                  P.res[0] && P.res[1] && P.rope && P.parts;
  P.T = ok ? T : 0;
  return ok;
}

// All layers over the T rows staged in ps.emb, appended to the caches at their
// current position (qm:357-395). Leaves the final norm of every row in ps.h.
inline bool prefill_layers(model& M, int64_t T) {
  const dims& d = M.d;
  prefill_scratch& P = M.ps;
  if (T <= 0 || T > P.T) return false;
  for (const layer& L : M.layers)   // the MFMA GEMM reads bf16 rows or int4, not [K,N] bf16
    if (L.wqkv.fmt != wfmt::bf16_row && L.wqkv.fmt != wfmt::q4) return false;
  const float scale = 1.0f / std::sqrt((float)d.head_dim);
  const int64_t E = d.hidden, QD = d.q_dim(), KD = d.kv_dim(), QKVN = d.qkv_dim(), HD = d.head_dim;
  const int64_t pos0 = M.layers[0].cache.pos;
  bool ok = true;
  void* x = P.emb;
  ok &= hip::rmsnorm(x, M.layers[0].an, P.h, E, d.eps, T);
  const bool fused = M.fused_prefill;
  hip::set_prompt_f16(M.prompt_f16);
  if (fused) ok &= hip::rope_table_range(P.rope, HD, pos0, T, d.rope_base);   // once for all layers
  for (int64_t l = 0; l < d.n_layers; l++) {
    layer& L = M.layers[(size_t)l];
    void* ro = P.res[l & 1];
    if (fused) {
      // the projection's K-split parts are added up by the launch that does bias + rope +
      // head-major q + cache rows; attention writes [T, Hq*D]
      int np = 0;
      ok &= gemm_parts(L.wqkv, P.h, P.parts, P.parts_bytes, T, &np);
      L.cache.pos = pos0;
      ok = ok && L.cache.prefill_qkv(P.parts, L.bq, L.bk, L.bv, P.rope, P.qkvh, P.at, T, d.n_q_heads, scale, np);
    } else {
    ok &= gemm(L.wqkv, P.h, P.qkv, T);
    // [T, q|k|v] -> head-major [Hq + 2 Hkv, T, D], bias added on the way
    ok &= hip::split_heads(P.qkv, L.bqkv, P.qkvh, T, QKVN, 0, d.n_q_heads + 2 * d.n_kv_heads, HD);
    void* kh = static_cast<char*>(P.qkvh) + QD * T * 4;
    void* vh = static_cast<char*>(P.qkvh) + (QD + KD) * T * 4;
    // row r = h*T + t, so rope's position pos0 + r % T is pos0 + t
    ok &= hip::rope(P.qkvh, P.qkvh, d.n_q_heads * T, T, HD, pos0, d.rope_base);
    ok &= hip::rope(kh, kh, d.n_kv_heads * T, T, HD, pos0, d.rope_base);
    L.cache.pos = pos0;
    ok &= L.cache.prefill(P.qkvh, kh, vh, P.ah, T, d.n_q_heads, scale);
    ok &= hip::merge_heads(P.ah, P.at, T, d.n_q_heads, HD);
    }
    void* nextw = (l + 1 < d.n_layers) ? M.layers[(size_t)l + 1].an : M.onorm;
    if (fused) {
      // o-proj and down leave their K-split parts; the residual norm adds them up as it reads
      int np = 0;
      ok &= gemm_parts(L.wo, P.at, P.parts, P.parts_bytes, T, &np);
      // (the norms are told which bf16 product reads their output: where that one runs over a
      // prepared weight, the norm leaves the activation image it would otherwise make itself)
      const auto cols = [&](const linear& W) { return W.fmt == wfmt::q4 || !M.norm_images ? int64_t(0) : W.N; };
      ok = ok && hip::rmsnorm_res_parts(x, P.parts, np, L.fn, ro, P.h2, E, d.eps, T, cols(L.wgu));
      ok &= gemm_swiglu(L.wgu, P.h2, P.mb, T);   // the gate as the epilogue
      ok &= gemm_parts(L.wd, P.mb, P.parts, P.parts_bytes, T, &np);
      ok = ok && hip::rmsnorm_res_parts(ro, P.parts, np, nextw, ro, P.h, E, d.eps, T,
                                        l + 1 < d.n_layers ? cols(M.layers[(size_t)l + 1].wqkv) : int64_t(0));
    } else {
    ok &= gemm(L.wo, P.at, ro, T);
    ok &= hip::rmsnorm_res(ro, x, L.fn, ro, P.h2, E, d.eps, T);
    ok &= gemm(L.wgu, P.h2, P.gu, T);
    ok &= hip::swiglu(P.gu, P.mb, d.ff, T);
    ok &= gemm(L.wd, P.mb, P.md, T);
    ok &= hip::rmsnorm_res(ro, P.md, nextw, ro, P.h, E, d.eps, T);
    }
    x = ro;
  }
  return ok;
}

// Gather T embedding rows on the host and upload them as the chunk input.
// false for a token id outside [0, vocab), before anything is read.
inline bool stage_chunk(model& M, const int64_t* tokens, int64_t T) {
  const dims& d = M.d;
  for (int64_t t = 0; t < T; t++)
    if (tokens[t] < 0 || tokens[t] >= d.vocab) return false;
  if (!prefill_reserve(M, T)) return false;
  for (int64_t t = 0; t < T; t++) {
    const uint16_t* r = M.embed.data() + (size_t)tokens[t] * d.hidden;
    float* o = M.ps.emb_host + t * d.hidden;
    if (M.embed_f16)
      for (int64_t j = 0; j < d.hidden; j++) o[j] = f16_to_f32(r[j]);
    else
      for (int64_t j = 0; j < d.hidden; j++) o[j] = bf16_to_f32(r[j]);
  }
  hip::upload(M.ps.emb, M.ps.emb_host, T * d.hidden);
  return true;
}

// Consume a prompt in chunks; logits of its LAST token land in s.logitsb (only
// that row is ever read, so only it meets the lm_head: qm:396-401).
inline bool prefill(model& M, const int64_t* tokens, int64_t n, int64_t chunk = 512) {
  if (n <= 0 || chunk <= 0) return false;
  bool ok = true;
  int64_t last_T = 0;
  for (int64_t t0 = 0; t0 < n && ok; t0 += chunk) {
    last_T = std::min(chunk, n - t0);
    ok = stage_chunk(M, tokens + t0, last_T) && prefill_layers(M, last_T);
  }
  if (!ok) return false;
  void* last = static_cast<char*>(M.ps.h) + (last_T - 1) * M.d.hidden * 4;
  return gemv(M.lm_head, last, M.s.logitsb);
}

// One decode step recorded as a hipGraph at a FIXED position (the throughput
// measurement replays the same step; replaying re-writes the same cache row).
struct captured_step {
  void* graph = nullptr;
  bool capture(model& M, int64_t pos) {
    // warm: lets the library size its scratch before the capture opens
    if (!run_layers(M, M.s.embedb, pos)) return false;
    hip::flush();
    if (!hip::capture_begin()) return false;
    const bool ok = run_layers(M, M.s.embedb, pos);
    graph = hip::capture_end();
    return ok && graph != nullptr;
  }
  bool replay() { return hip::graph_launch(graph); }
  void destroy() {
    hip::graph_destroy(graph);
    graph = nullptr;
  }
};

// Copy the host embedding table to the device once, through a pinned staging block.
inline bool upload_embed(model& M) {
  if (M.embed_dev) return true;
  const int64_t bytes = (int64_t)M.embed.size() * 2;
  if (bytes <= 0) return false;
  M.embed_dev = hip::alloc_device(bytes);
  if (!M.embed_dev) return false;
  const int64_t blk = int64_t(32) << 20;
  float* stage_host = nullptr;
  void* stage = hip::alloc(blk, &stage_host);
  if (!stage) return false;
  bool ok = true;
  for (int64_t o = 0; o < bytes && ok; o += blk) {
    const int64_t n = std::min(blk, bytes - o);
    std::memcpy(stage_host, reinterpret_cast<const char*>(M.embed.data()) + o, (size_t)n);
    hip::upload(stage, stage_host, (n + 3) / 4);
    ok = hip::copy_d2d(static_cast<char*>(M.embed_dev) + o, stage, n);
    hip::flush();   // the staging block is reused
  }
  hip::release(stage, blk, stage_host);
  return ok;
}

// Greedy decoding with the whole token loop on the device: one recorded graph does
//   embedding gather of *d_tok -> layers at *d_pos -> lm_head -> argmax -> *d_tok,
//   history[*d_pos] = *d_tok, *d_pos += 1
// so consecutive tokens are queued back to back with no host round trip between them
// (the reference stages each embedding on the host and reads every argmax back:
// qm:530-535, 642-647). The host reads the generated ids from the history afterwards.
struct greedy_loop {
  void *d_pos = nullptr, *d_tok = nullptr, *history = nullptr, *graph = nullptr;
  float* history_host = nullptr;
  int64_t cur_pos = 0, max_ctx = 0;

  bool init(model& M, int64_t first_id, int64_t pos) {
    if (M.layers.empty() || !M.fused || !hip::graph_available()) return false;
    const dims& d = M.d;
    if (first_id < 0 || first_id >= d.vocab) return false;   // later ids are argmax results, in range by construction
    max_ctx = M.layers[0].cache.max_ctx;
    cur_pos = pos;
    if (!upload_embed(M)) return false;
    if (!M.attn_partials) {
      M.attn_partials_bytes = hip::attn_partials_bytes(d.n_q_heads, d.n_kv_heads, max_ctx, d.head_dim);
      M.attn_partials = hip::alloc_device(M.attn_partials_bytes);
      if (!M.attn_partials) return false;
    }
    d_pos = hip::alloc(4, nullptr);
    d_tok = hip::alloc(4, nullptr);
    history = hip::alloc(max_ctx * 4, &history_host);
    if (!d_pos || !d_tok || !history) return false;
    auto one = [&]() {
      bool ok = M.embed_f16 ? hip::embed_gather_f16(M.embed_dev, d_tok, M.s.embedb, d.hidden, d.vocab)
                            : hip::embed_gather_bf16(M.embed_dev, d_tok, M.s.embedb, d.hidden, d.vocab);
      ok = ok && run_layers(M, M.s.embedb, 0, nullptr, d_pos, /*advance=*/false);
      ok = ok && hip::argmax_async(M.s.logitsb, d.vocab, d_tok);
      return ok && hip::token_advance(d_pos, d_tok, history, max_ctx);
    };
    hip::upload_u32(d_pos, (unsigned)pos);
    hip::upload_u32(d_tok, (unsigned)first_id);
    if (!one()) return false;            // warm run (sizes the library's scratch)
    hip::flush();
    hip::upload_u32(d_pos, (unsigned)pos);
    hip::upload_u32(d_tok, (unsigned)first_id);
    if (!hip::capture_begin()) return false;
    const bool ok = one();
    graph = hip::capture_end();
    if (!ok && graph) { hip::graph_destroy(graph); graph = nullptr; }
    return graph != nullptr;
  }
  // Queue n greedy steps (no sync). Returns how many were queued before the cache filled.
  int64_t run(int64_t n) {
    int64_t done = 0;
    while (done < n && cur_pos < max_ctx && graph && hip::graph_launch(graph)) {
      cur_pos++;
      done++;
    }
    return done;
  }
  // The token generated at position p (p in [first pos, cur_pos)); blocks until the queue drained.
  const int32_t* tokens() {
    hip::sync_to_host(history, false);
    return reinterpret_cast<const int32_t*>(history_host);
  }
  void sync_host_pos(model& M) const { set_cache_pos(M, cur_pos); }
  void destroy() {
    if (graph) hip::graph_destroy(graph);
    for (void* b : {d_pos, d_tok, history})
      if (b) hip::release(b, 0, nullptr);
    graph = d_pos = d_tok = history = nullptr;
  }
};

// A decode loop on ONE recorded graph (qm:791-905): the position lives in a device
// scalar that the recorded forward advances itself, so feed()/step() replay the same
// graph for every token. Falls back to the imperative path when capture is not
// available; callers never branch on ok().
struct captured_decoder {
  void* d_pos = nullptr;
  void* graph = nullptr;
  int64_t cur_pos = 0, max_ctx = 0;

  // Record the forward at `pos` (the first position this decoder will process).
  bool init(model& M, int64_t first_id, int64_t pos) {
    if (M.layers.empty()) return false;
    max_ctx = M.layers[0].cache.max_ctx;
    cur_pos = pos;
    if (!hip::graph_available() || !M.fused) return false;
    const dims& d = M.d;
    if (!M.attn_partials) {
      M.attn_partials_bytes = hip::attn_partials_bytes(d.n_q_heads, d.n_kv_heads, max_ctx, d.head_dim);
      M.attn_partials = hip::alloc_device(M.attn_partials_bytes);
      if (!M.attn_partials) return false;
    }
    d_pos = hip::alloc(4, nullptr);
    if (!d_pos) return false;
    if (!stage_embed(M, first_id)) return false;
    hip::upload_u32(d_pos, (unsigned)pos);
    // warm run: real launches (they also size the library's scratch); it advances d_pos
    // and writes cache row pos, which the first recorded step rewrites identically
    if (!run_layers(M, M.s.embedb, pos, nullptr, d_pos)) return false;
    hip::flush();
    hip::upload_u32(d_pos, (unsigned)pos);
    if (!hip::capture_begin()) return false;
    const bool ok = run_layers(M, M.s.embedb, pos, nullptr, d_pos);  // recorded, not executed
    graph = hip::capture_end();
    if (!ok && graph) { hip::graph_destroy(graph); graph = nullptr; }
    return graph != nullptr;
  }
  // Feed token `id` at the current position without reading a token back.
  bool feed(model& M, int64_t id) {
    if (cur_pos >= max_ctx || !stage_embed(M, id)) return false;
    bool ok;
    if (graph) ok = hip::graph_launch(graph);
    else ok = run_layers(M, M.s.embedb, cur_pos);
    cur_pos++;
    return ok;
  }
  // One decode step: feed + greedy token (-1 when the cache is full or a launch failed).
  int64_t step(model& M, int64_t id) {
    if (!feed(M, id)) return -1;
    int64_t idx = -1;
    return hip::argmax(M.s.logitsb, M.d.vocab, &idx) ? idx : -1;
  }
  // Replays advance only the device counter; bring the host cache position up to date
  // before switching to a host-position call.
  void sync_host_pos(model& M) const {
    if (graph) set_cache_pos(M, cur_pos);
  }
  bool ok() const { return graph != nullptr; }
  void destroy() {
    if (graph) hip::graph_destroy(graph);
    if (d_pos) hip::release(d_pos, 0, nullptr);
    graph = nullptr;
    d_pos = nullptr;
  }
};

}  // namespace qwen
}  // namespace tl
