// TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// A C-ABI window onto the REAL reference's CPU path. This file holds no
// arithmetic of its own: it includes the reference's header-only library from
// where it lies (/root/reference/include, passed with -I by the Makefile),
// builds tl::array objects around caller buffers and evaluates the reference's
// own array ops in use_cpu() mode. The result (oracle/_ref/libtlref.so) is used
// to (1) validate the plain-C restatement in oracle.c, (2) write the golden
// vectors under tests/golden/, and (3) time the reference's CPU path beside the
// GPU numbers. It only exists where /root/reference exists at build time.
#include <algorithm>
#include <array>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <functional>
#include <limits>
#include <memory>
#include <numeric>
#include <optional>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

// The reference keeps q4/bf16 bytes behind private storage and offers no
// public way to wrap existing packed bytes in an array; the checker needs that
// to feed the reference the exact weight bytes the GPU sees.
#define private public
#include <tensorlib.h>
#undef private

// The reference's GGUF reader, parsed results rendered by the same generic text dump the
// product's reader is rendered with (the dump touches only the surface both share).
#include <gguf.h>
#include <tokenizer.h>
#include <tl/gguf_dump.h>

using tl::array;

namespace {

array f32_array(const float* p, tl::shape_t shape) {
  int64_t n = 1;
  for (auto s : shape) n *= s;
  return array::from(std::vector<float>(p, p + n), std::move(shape));
}

// q4 array [K,N] whose storage holds exactly `buf` (packed rows + scales).
array q4_array(const uint8_t* buf, int64_t K, int64_t N) {
  array out;
  out.shape_ = {K, N};
  out.strides_ = tl::detail::contiguous_strides(out.shape_);
  out.storage_ = tl::storage::make_bytes_(N * K, tl::q4_bytes(N, K), tl::dtype::q4);
  std::memcpy(out.storage_.data(), buf, (size_t)tl::q4_bytes(N, K));
  return out;
}

array bf16_array(const uint16_t* p, tl::shape_t shape) {
  array out;
  out.shape_ = shape;
  out.strides_ = tl::detail::contiguous_strides(out.shape_);
  int64_t n = 1;
  for (auto s : shape) n *= s;
  out.storage_ = tl::storage::make(n, tl::dtype::bf16);
  std::memcpy(out.storage_.data(), p, (size_t)n * 2);
  return out;
}

void copy_out(const array& a, float* dst) {
  array c = a.contiguous() ? a : a.clone();
  c.eval();
  const float* p = c.raw();
  std::copy(p, p + c.size(), dst);
}

}  // namespace

extern "C" {

int tlref_init() {
  tl::use_cpu();
  return 1;
}

// toggles the reference's own in-process oracle switch (test_array.cpp:23-68):
// 0 => ref:: loops only, 1 => cpu::sgemm path (the default CPU path).
void tlref_set_cpu_gemm(int on) { tl::cpu::enabled_ = on != 0; }

int64_t tlref_q4_bytes(int64_t N, int64_t K) { return tl::q4_bytes(N, K); }

void tlref_to_q4(const float* w, int64_t K, int64_t N, uint8_t* out) {
  array q = f32_array(w, {K, N}).to_q4();
  std::memcpy(out, q.storage_.data(), (size_t)tl::q4_bytes(N, K));
}

void tlref_q4_to_f32(const uint8_t* buf, int64_t K, int64_t N, float* out) {
  copy_out(q4_array(buf, K, N).to_f32(), out);
}

void tlref_to_bf16(const float* src, uint16_t* dst, int64_t n) {
  array b = f32_array(src, {n}).to_bf16();
  std::memcpy(dst, b.storage_.data(), (size_t)n * 2);
}

void tlref_bf16_to_f32(const uint16_t* src, float* dst, int64_t n) {
  copy_out(bf16_array(src, {n}).to_f32(), dst);
}

// (A[m,k] . B[k,n]) * scale + offset through the lazy graph (fused epilogue).
void tlref_dot(const float* A, const float* B, float* C, int64_t m, int64_t n, int64_t k,
               float scale, float offset) {
  array a = f32_array(A, {m, k}), b = f32_array(B, {k, n});
  array r = a.dot(b);
  if (scale != 1.0f) r = r * scale;
  if (offset != 0.0f) r = r + offset;
  copy_out(r, C);
}

void tlref_gemv_q4(const float* a, const uint8_t* q4buf, float* y, int64_t N, int64_t K) {
  copy_out(f32_array(a, {1, K}).dot(q4_array(q4buf, K, N)), y);
}

void tlref_gemv_bf16(const float* a, const uint16_t* B, float* y, int64_t N, int64_t K) {
  copy_out(f32_array(a, {1, K}).dot(bf16_array(B, {K, N})), y);
}

// Handles for timing: build the arrays once, then evaluate the dot repeatedly
// (each evaluation re-widens the weight, as the reference does).
struct tlref_gemv { array a, W; };
void* tlref_gemv_q4_prepare(const float* a, const uint8_t* q4buf, int64_t N, int64_t K) {
  return new tlref_gemv{f32_array(a, {1, K}), q4_array(q4buf, K, N)};
}
void* tlref_gemv_bf16_prepare(const float* a, const uint16_t* B, int64_t N, int64_t K) {
  return new tlref_gemv{f32_array(a, {1, K}), bf16_array(B, {K, N})};
}
void tlref_gemv_run(void* h, float* y) {
  auto* g = static_cast<tlref_gemv*>(h);
  array r = g->a.dot(g->W);
  r.eval();
  if (y) std::copy(r.raw(), r.raw() + r.size(), y);
}
void tlref_gemv_free(void* h) { delete static_cast<tlref_gemv*>(h); }

void tlref_attn_decode(const float* q, const float* K, const float* V, float* out,
                       int64_t H, int64_t ctx, int64_t D, float scale) {
  copy_out(array::attn_decode(f32_array(q, {H, D}), f32_array(K, {H, ctx, D}),
                              f32_array(V, {H, ctx, D}), scale),
           out);
}

void tlref_rope(const float* x, float* out, int64_t H, int64_t T, int64_t D, int64_t pos,
                float base) {
  array a = T > 1 ? f32_array(x, {H, T, D}) : f32_array(x, {H, D});
  copy_out(array::rope(a, pos, base), out);
}

void tlref_rmsnorm(const float* x, const float* w, float* out, int64_t rows, int64_t n,
                   float eps) {
  copy_out(array::rmsnorm(f32_array(x, {rows, n}), f32_array(w, {n}), eps), out);
}

void tlref_silu(const float* x, float* out, int64_t n) {
  copy_out(array::silu(f32_array(x, {1, n})), out);
}

void tlref_swiglu(const float* g, const float* u, float* out, int64_t n) {
  copy_out(array::swiglu(f32_array(g, {1, n}), f32_array(u, {1, n})), out);
}

void tlref_softmax(const float* x, float* out, int64_t rows, int64_t cols) {
  copy_out(f32_array(x, {rows, cols}).softmax(), out);
}

void tlref_row_sum(const float* x, float* out, int64_t rows, int64_t cols, float scale,
                   float offset) {
  array r = f32_array(x, {rows, cols}).sum(-1);
  if (scale != 1.0f) r = r * scale;
  if (offset != 0.0f) r = r + offset;
  copy_out(r, out);
}

void tlref_row_mean(const float* x, float* out, int64_t rows, int64_t cols) {
  copy_out(f32_array(x, {rows, cols}).mean(-1), out);
}

void tlref_row_max(const float* x, float* out, int64_t rows, int64_t cols) {
  copy_out(f32_array(x, {rows, cols}).max(-1), out);
}

// op: 0 add 1 sub 2 mul 3 div; b broadcasts numpy-style from [bm,bn] to [m,n]
void tlref_binary(int op, const float* a, int64_t am, int64_t an, const float* b, int64_t bm,
                  int64_t bn, float* out, float scale, float offset) {
  array x = f32_array(a, {am, an}), y = f32_array(b, {bm, bn});
  array r = op == 0 ? x + y : op == 1 ? x - y : op == 2 ? x * y : x / y;
  if (scale != 1.0f) r = r * scale;
  if (offset != 0.0f) r = r + offset;
  copy_out(r, out);
}

// op: 5 exp 6 log 7 sqrt 8 sigmoid 9 relu 10 affine 11 recip (oracle.h numbering)
void tlref_unary(int op, const float* a, float* out, int64_t n, float scale, float offset) {
  // [2, n/2]-free: keep rank 1 but larger than the eager-tiny cutoff is not
  // required; values are identical on the eager and lazy routes.
  array x = f32_array(a, {n});
  array r;
  switch (op) {
    case 5: r = x.exp(); break;
    case 6: r = x.log(); break;
    case 7: r = x.sqrt(); break;
    case 8: r = x.sigmoid(); break;
    case 9: r = x.relu(); break;
    case 11: r = 1.0f / x; break;
    default: r = x * 1.0f; break;
  }
  if (scale != 1.0f) r = r * scale;
  if (offset != 0.0f) r = r + offset;
  copy_out(r, out);
}

int64_t tlref_argmax(const float* v, int64_t n) { return f32_array(v, {n}).argmax(); }

// ---- decode model assembled from array ops (bench/cuda/qwen_model.h:559-599),
// with a host-side cache and one attn_decode call per query head, since the
// array op has no GQA (array.h:1380-1381).
struct dims {
  int64_t n_layers, hidden, n_q_heads, n_kv_heads, head_dim, ff, vocab, max_ctx;
  float eps, rope_base;
};
struct layer {
  array wq, wk, wv, wo, wg, wu, wd, bq, bk, bv, an, fn;
  std::vector<float> Kc, Vc;
};
struct model {
  dims d;
  std::vector<uint16_t> embed;
  array onorm, outw;
  std::vector<layer> layers;
};

void* tlref_qwen_create(const dims* d) {
  auto* m = new model();
  m->d = *d;
  m->layers.resize((size_t)d->n_layers);
  for (auto& L : m->layers) {
    L.Kc.assign((size_t)(d->n_kv_heads * d->max_ctx * d->head_dim), 0.0f);
    L.Vc.assign((size_t)(d->n_kv_heads * d->max_ctx * d->head_dim), 0.0f);
  }
  return m;
}
void tlref_qwen_destroy(void* h) { delete static_cast<model*>(h); }

// kind: 0 f32 vector, 1 q4 [K,N], 2 bf16 [K,N], 3 bf16 embedding table.
// predeq != 0 widens q4/bf16 once (values identical to the per-call widening).
int tlref_qwen_set(void* h, int64_t li, const char* name, const void* p, int kind, int64_t K,
                   int64_t N, int predeq) {
  auto* m = static_cast<model*>(h);
  std::string s(name);
  array a;
  if (kind == 0) a = f32_array(static_cast<const float*>(p), {1, N});
  else if (kind == 1) a = q4_array(static_cast<const uint8_t*>(p), K, N);
  else if (kind == 2) a = bf16_array(static_cast<const uint16_t*>(p), {K, N});
  if ((kind == 1 || kind == 2) && predeq) a = a.to_f32();
  if (li < 0) {
    if (s == "embed") {
      auto* e = static_cast<const uint16_t*>(p);
      m->embed.assign(e, e + K * N);
    } else if (s == "onorm") m->onorm = a;
    else if (s == "outw") m->outw = a;
    else return -1;
    return 0;
  }
  layer& L = m->layers[(size_t)li];
  if (s == "wq") L.wq = a; else if (s == "wk") L.wk = a; else if (s == "wv") L.wv = a;
  else if (s == "wo") L.wo = a; else if (s == "wg") L.wg = a; else if (s == "wu") L.wu = a;
  else if (s == "wd") L.wd = a; else if (s == "bq") L.bq = a; else if (s == "bk") L.bk = a;
  else if (s == "bv") L.bv = a; else if (s == "an") L.an = a; else if (s == "fn") L.fn = a;
  else return -1;
  return 0;
}

int64_t tlref_qwen_step(void* h, int64_t token, int64_t pos, float* logits) {
  auto* m = static_cast<model*>(h);
  const dims& d = m->d;
  const int64_t E = d.hidden, HQ = d.n_q_heads, HKV = d.n_kv_heads, HD = d.head_dim;
  const int64_t group = HQ / HKV, ctx = pos + 1;
  const float scale = 1.0f / std::sqrt((float)HD);
  std::vector<float> xe((size_t)E);
  for (int64_t j = 0; j < E; j++) xe[(size_t)j] = tl::bf16_to_f32(m->embed[(size_t)(token * E + j)]);
  array x = array::from(xe, {1, E});
  for (auto& L : m->layers) {
    array hh = array::rmsnorm(x, L.an, d.eps);
    array q = array::rope((hh.dot(L.wq) + L.bq).reshape({HQ, HD}), pos, d.rope_base);
    array k = array::rope((hh.dot(L.wk) + L.bk).reshape({HKV, HD}), pos, d.rope_base);
    array v = hh.dot(L.wv) + L.bv;
    tl::eval(q, k, v);
    const float* pk = k.raw();
    const float* pv = v.raw();
    for (int64_t g = 0; g < HKV; g++) {
      std::copy(pk + g * HD, pk + (g + 1) * HD, L.Kc.begin() + (g * d.max_ctx + pos) * HD);
      std::copy(pv + g * HD, pv + (g + 1) * HD, L.Vc.begin() + (g * d.max_ctx + pos) * HD);
    }
    std::vector<float> ao((size_t)(HQ * HD));
    for (int64_t g = 0; g < HKV; g++) {
      array Kg = f32_array(L.Kc.data() + g * d.max_ctx * HD, {1, ctx, HD});
      array Vg = f32_array(L.Vc.data() + g * d.max_ctx * HD, {1, ctx, HD});
      for (int64_t j = 0; j < group; j++) {
        int64_t hq = g * group + j;
        array o = array::attn_decode(q.slice(hq, 1), Kg, Vg, scale);
        copy_out(o, ao.data() + hq * HD);
      }
    }
    array a_out = array::from(ao, {1, HQ * HD});
    array x1 = x + a_out.dot(L.wo);
    array h2 = array::rmsnorm(x1, L.fn, d.eps);
    array mlp = array::swiglu(h2.dot(L.wg), h2.dot(L.wu)).dot(L.wd);
    array x2 = x1 + mlp;
    x2.eval();
    x = x2;
  }
  array xf = array::rmsnorm(x, m->onorm, d.eps);
  array lg = xf.dot(m->outw);
  lg.eval();
  const float* p = lg.raw();
  if (logits) std::copy(p, p + d.vocab, logits);
  int64_t bi = 0;
  for (int64_t i = 1; i < d.vocab; i++)
    if (p[i] > p[bi]) bi = i;
  return bi;
}

}  // extern "C"

extern "C" {

// Canonical rendering of a GGUF file as the REFERENCE's reader parses it. Returns the text
// length (buf is filled and NUL-terminated when it fits), or -1 with the exception text in
// buf when the reader throws.
int64_t tlref_gguf_dump(const char* path, char* buf, int64_t cap) {
  try {
    tl::gguf::model m(path);
    const std::string text = tl::gguf_dump::render(m);
    if (buf && cap > (int64_t)text.size()) std::memcpy(buf, text.c_str(), text.size() + 1);
    return (int64_t)text.size();
  } catch (const std::exception& e) {
    if (buf && cap > 0) {
      std::strncpy(buf, e.what(), (size_t)cap - 1);
      buf[cap - 1] = 0;
    }
    return -1;
  }
}


// The REFERENCE's tokenizer (include/tokenizer.h) and its code-point classes.
void* tlref_tok_open(const char* path) {
  try {
    return new tl::tokenizer(std::string(path));
  } catch (const std::exception&) {
    return nullptr;
  }
}
void tlref_tok_close(void* t) { delete static_cast<tl::tokenizer*>(t); }
void tlref_tok_special_ids(void* t, int* bos, int* eos) {
  *bos = static_cast<tl::tokenizer*>(t)->bos_id();
  *eos = static_cast<tl::tokenizer*>(t)->eos_id();
}
int64_t tlref_tok_encode(void* t, const char* text, int64_t n, int32_t* out, int64_t cap) {
  try {
    const std::vector<int> ids = static_cast<tl::tokenizer*>(t)->encode(std::string(text, (size_t)n));
    for (size_t i = 0; i < ids.size() && (int64_t)i < cap; i++) out[i] = ids[i];
    return (int64_t)ids.size();
  } catch (const std::exception&) {
    return -1;
  }
}
int64_t tlref_tok_decode(void* t, const int32_t* ids, int64_t n, char* out, int64_t cap) {
  try {
    const std::string s = static_cast<tl::tokenizer*>(t)->decode(std::vector<int>(ids, ids + n));
    std::memcpy(out, s.data(), (size_t)std::min<int64_t>(cap, (int64_t)s.size()));
    return (int64_t)s.size();
  } catch (const std::exception&) {
    return -1;
  }
}
int tlref_unicode_class(uint32_t cp) {
  return (tl::tokdata::is_L(cp) ? 1 : 0) | (tl::tokdata::is_N(cp) ? 2 : 0) | (tl::tokdata::is_WS(cp) ? 4 : 0);
}

}  // extern "C"
