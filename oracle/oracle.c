/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE — see oracle.h.
 *
 * Plain-C restatement of the reference CPU path for the decode hot path.
 * Built with -ffp-contract=off so every multiply-add below is exactly what is
 * written: fmaf() where the reference's AVX2 microkernel issues an FMA,
 * separate multiply and add where its scalar loops do.
 */
#include "oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

/* ------------------------------------------------------------------------ */
/* seeded inputs                                                             */
/* ------------------------------------------------------------------------ */

void orc_rng_seed(orc_rng* r, uint32_t seed) {
  /* multiplicative scramble so that small consecutive seeds diverge at once;
   * same idea as check_llm_decode.cpp:33 */
  r->s = seed * 2654435761u + 1u;
  if (r->s == 0) r->s = 0x9E3779B9u;
  r->has_spare = 0;
  r->spare = 0.0;
}

uint32_t orc_rng_u32(orc_rng* r) {
  /* xorshift32, the generator of check_llm_block.cpp:24-34 */
  uint32_t s = r->s;
  s ^= s << 13;
  s ^= s >> 17;
  s ^= s << 5;
  r->s = s;
  return s;
}

double orc_rng_uniform(orc_rng* r) { return orc_rng_u32(r) * (1.0 / 4294967296.0); }

double orc_rng_normal(orc_rng* r) {
  if (r->has_spare) {
    r->has_spare = 0;
    return r->spare;
  }
  double u1;
  do { u1 = orc_rng_uniform(r); } while (u1 <= 0.0);
  double u2 = orc_rng_uniform(r);
  double rad = sqrt(-2.0 * log(u1));
  double ang = 6.283185307179586476925 * u2;
  r->spare = rad * sin(ang);
  r->has_spare = 1;
  return rad * cos(ang);
}

void orc_fill_normal(float* dst, int64_t n, uint32_t seed, float mean, float std) {
  orc_rng r;
  orc_rng_seed(&r, seed);
  for (int64_t i = 0; i < n; i++) dst[i] = (float)(mean + std * orc_rng_normal(&r));
}

void orc_fill_uniform(float* dst, int64_t n, uint32_t seed, float lo, float hi) {
  orc_rng r;
  orc_rng_seed(&r, seed);
  for (int64_t i = 0; i < n; i++) dst[i] = (float)(lo + (hi - lo) * orc_rng_uniform(&r));
}

void orc_fill_q4(uint8_t* buf, int64_t N, int64_t K, uint32_t seed, float lo, float hi) {
  orc_rng r;
  orc_rng_seed(&r, seed);
  int64_t nb = N * K / 2;
  for (int64_t i = 0; i < nb; i += 4) {
    uint32_t w = orc_rng_u32(&r);
    for (int j = 0; j < 4 && i + j < nb; j++) buf[i + j] = (uint8_t)(w >> (8 * j));
  }
  float* sc = (float*)(buf + nb);
  int64_t ns = N * (K / 32);
  for (int64_t i = 0; i < ns; i++) sc[i] = (float)(lo + (hi - lo) * orc_rng_uniform(&r));
}

uint32_t orc_crc32(const void* data, int64_t bytes) {
  static uint32_t table[256];
  static int init = 0;
  if (!init) {
    for (uint32_t i = 0; i < 256; i++) {
      uint32_t c = i;
      for (int k = 0; k < 8; k++) c = (c & 1) ? 0xEDB88320u ^ (c >> 1) : c >> 1;
      table[i] = c;
    }
    init = 1;
  }
  const uint8_t* p = (const uint8_t*)data;
  uint32_t c = 0xFFFFFFFFu;
  for (int64_t i = 0; i < bytes; i++) c = table[(c ^ p[i]) & 0xFF] ^ (c >> 8);
  return c ^ 0xFFFFFFFFu;
}

/* ------------------------------------------------------------------------ */
/* storage formats                                                           */
/* ------------------------------------------------------------------------ */

uint16_t orc_f32_to_bf16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  x += 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}

float orc_bf16_to_f32(uint16_t h) {
  uint32_t x = (uint32_t)h << 16;
  float f;
  memcpy(&f, &x, 4);
  return f;
}

void orc_to_bf16(const float* src, uint16_t* dst, int64_t n) {
  for (int64_t i = 0; i < n; i++) dst[i] = orc_f32_to_bf16(src[i]);
}

void orc_bf16_widen(const uint16_t* src, float* dst, int64_t n) {
  for (int64_t i = 0; i < n; i++) dst[i] = orc_bf16_to_f32(src[i]);
}

/* IEEE half -> float as the model loader widens GGUF F16 tensors
 * (bench/cuda/qwen_model.h:41-60): subnormals are renormalised by shifting the
 * mantissa up, inf/nan keep their mantissa bits, everything else rebiases the
 * exponent by 127 - 15. */
float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1Fu, mant = h & 0x3FFu, bits;
  if (e == 0x1Fu) {
    bits = sign | 0x7F800000u | (mant << 13);
  } else if (e != 0) {
    bits = sign | ((e + 112u) << 23) | (mant << 13);
  } else if (mant == 0) {
    bits = sign;
  } else {
    e = 113; /* 127 - 15 + 1 */
    while (!(mant & 0x400u)) {
      mant <<= 1;
      e--;
    }
    bits = sign | (e << 23) | ((mant & 0x3FFu) << 13);
  }
  float out;
  memcpy(&out, &bits, 4);
  return out;
}

void orc_f16_widen(const uint16_t* src, float* dst, int64_t n) {
  for (int64_t i = 0; i < n; i++) dst[i] = orc_f16_to_f32(src[i]);
}

int64_t orc_q4_bytes(int64_t N, int64_t K) { return N * K / 2 + N * (K / 32) * 4; }

int orc_to_q4(const float* w, int64_t s0, int64_t s1, int64_t K, int64_t N, uint8_t* out) {
  const int64_t G = 32;
  if (K % G != 0) return -1;
  memset(out, 0, (size_t)orc_q4_bytes(N, K));
  float* sc = (float*)(out + N * K / 2);
  for (int64_t n = 0; n < N; n++) {
    uint8_t* qrow = out + n * (K / 2);
    float* srow = sc + n * (K / G);
    for (int64_t g = 0; g < K / G; g++) {
      float maxabs = 1e-8f;
      for (int64_t j = 0; j < G; j++) {
        float a = fabsf(w[(g * G + j) * s0 + n * s1]);
        if (a > maxabs) maxabs = a;
      }
      float scale = maxabs / 7.0f;
      srow[g] = scale;
      for (int64_t j = 0; j < G; j++) {
        int64_t k = g * G + j;
        long q = lroundf(w[k * s0 + n * s1] / scale); /* half away from zero */
        if (q < -8) q = -8;
        if (q > 7) q = 7;
        unsigned nib = (unsigned)(q + 8);
        uint8_t* byte = &qrow[k / 2];
        *byte = (k & 1) ? (uint8_t)((*byte & 0x0F) | (nib << 4))
                        : (uint8_t)((*byte & 0xF0) | nib);
      }
    }
  }
  return 0;
}

void orc_q4_to_f32(const uint8_t* buf, int64_t K, int64_t N, float* out) {
  const int64_t G = 32;
  const float* sc = (const float*)(buf + N * K / 2);
  for (int64_t n = 0; n < N; n++) {
    const uint8_t* qrow = buf + n * (K / 2);
    const float* srow = sc + n * (K / G);
    for (int64_t k = 0; k < K; k++) {
      uint8_t byte = qrow[k / 2];
      int nib = (k & 1) ? (byte >> 4) : (byte & 0xF);
      out[k * N + n] = srow[k / G] * (float)(nib - 8);
    }
  }
}

/* ------------------------------------------------------------------------ */
/* matmul                                                                    */
/* ------------------------------------------------------------------------ */

void orc_sgemm(const float* A, int64_t as0, int64_t as1, const float* B, int64_t bs0,
               int64_t bs1, float* C, int64_t m, int64_t n, int64_t k, float alpha) {
  /* cpu.h:393-466 with the AVX2 6x16 microkernel (285-346): C is zeroed, the
   * K axis is cut in KC=512 slabs (cpu.h:89-91, 422-423), each C element gets
   * one FMA chain per slab starting from 0 (ab registers), alpha is folded
   * into the packed A panel (cpu.h:104-110), and the slab result is added
   * into C (cpu.h:330-345). The NC/MC blocking and the tile shape do not
   * change any element's operation order. */
  const int64_t KC = 512;
  if (m == 0 || n == 0) return;
  memset(C, 0, (size_t)m * (size_t)n * sizeof(float));
  if (k == 0) return;
  float* ap = (float*)malloc((size_t)KC * sizeof(float));
  float* acc = (float*)malloc((size_t)n * sizeof(float));
  for (int64_t pc = 0; pc < k; pc += KC) {
    int64_t kc = k - pc < KC ? k - pc : KC;
    for (int64_t i = 0; i < m; i++) {
      for (int64_t p = 0; p < kc; p++) ap[p] = alpha * A[i * as0 + (pc + p) * as1];
      for (int64_t j = 0; j < n; j++) acc[j] = 0.0f;
      for (int64_t p = 0; p < kc; p++) {
        const float a = ap[p];
        const float* brow = B + (pc + p) * bs0;
        if (bs1 == 1) {
          for (int64_t j = 0; j < n; j++) acc[j] = fmaf(a, brow[j], acc[j]);
        } else {
          for (int64_t j = 0; j < n; j++) acc[j] = fmaf(a, brow[j * bs1], acc[j]);
        }
      }
      float* crow = C + i * n;
      for (int64_t j = 0; j < n; j++) crow[j] += acc[j];
    }
  }
  free(acc);
  free(ap);
}

void orc_ref_dot(const float* A, int64_t as0, int64_t as1, const float* B, int64_t bs0,
                 int64_t bs1, float* C, int64_t m, int64_t n, int64_t k) {
  /* array.h:946-970 */
  memset(C, 0, (size_t)m * (size_t)n * sizeof(float));
  for (int64_t i = 0; i < m; i++)
    for (int64_t l = 0; l < k; l++) {
      float av = A[i * as0 + l * as1];
      for (int64_t j = 0; j < n; j++) C[i * n + j] += av * B[l * bs0 + j * bs1];
    }
}

static void dot_strided(const float* A, int64_t as0, int64_t as1, const float* B,
                        int64_t bs0, int64_t bs1, float* C, int64_t m, int64_t n, int64_t k,
                        float scale, float offset) {
  /* array.h:1943-1972: M*N*K <= 16384 takes a plain triple loop with the
   * epilogue in the store. */
  if (m * n * k <= 16384 && m * n != 0) {
    for (int64_t i = 0; i < m; i++)
      for (int64_t j = 0; j < n; j++) {
        float acc = 0.0f;
        for (int64_t l = 0; l < k; l++) acc += A[i * as0 + l * as1] * B[l * bs0 + j * bs1];
        C[i * n + j] = acc * scale + offset;
      }
    return;
  }
  /* array.h:2126-2136: cpu::sgemm with the epilogue scale as alpha, then the
   * offset as a post-pass (1511-1518). */
  orc_sgemm(A, as0, as1, B, bs0, bs1, C, m, n, k, scale);
  if (offset != 0.0f)
    for (int64_t i = 0; i < m * n; i++) C[i] = C[i] + offset;
}

void orc_dot(const float* A, const float* B, float* C, int64_t m, int64_t n, int64_t k,
             float scale, float offset) {
  dot_strided(A, k, 1, B, n, 1, C, m, n, k, scale, offset);
}

void orc_gemv_q4(const float* a, const uint8_t* q4buf, float* y, int64_t N, int64_t K,
                 float scale, float offset, float* workspace) {
  /* array.h:1980-1984 funnel: the q4 operand is widened to an f32 [K,N] copy
   * (666-684), then the dot ladder runs on f32. The tiny fast path is closed
   * to non-f32 operands (1947-1948), so sgemm is always taken. */
  float* W = workspace ? workspace : (float*)malloc((size_t)K * (size_t)N * sizeof(float));
  orc_q4_to_f32(q4buf, K, N, W);
  orc_sgemm(a, K, 1, W, N, 1, y, 1, N, K, scale);
  if (offset != 0.0f)
    for (int64_t i = 0; i < N; i++) y[i] = y[i] + offset;
  if (!workspace) free(W);
}

void orc_gemv_bf16(const float* a, const uint16_t* B, float* y, int64_t N, int64_t K,
                   float scale, float offset, float* workspace) {
  float* W = workspace ? workspace : (float*)malloc((size_t)K * (size_t)N * sizeof(float));
  orc_bf16_widen(B, W, K * N);
  orc_sgemm(a, K, 1, W, N, 1, y, 1, N, K, scale);
  if (offset != 0.0f)
    for (int64_t i = 0; i < N; i++) y[i] = y[i] + offset;
  if (!workspace) free(W);
}

void orc_gemv_bf16_row(const float* a, const uint16_t* Wb, float* y, int64_t N, int64_t K,
                       float* workspace) {
  float* W = workspace ? workspace : (float*)malloc((size_t)K * (size_t)N * sizeof(float));
  orc_bf16_widen(Wb, W, K * N);
  orc_sgemm(a, K, 1, W, 1, K, y, 1, N, K, 1.0f);
  if (!workspace) free(W);
}

void orc_gemm_bf16_nt(const float* A, const uint16_t* Wb, float* C, int64_t M, int64_t N,
                      int64_t K, float* workspace) {
  float* W = workspace ? workspace : (float*)malloc((size_t)K * (size_t)N * sizeof(float));
  orc_bf16_widen(Wb, W, K * N);
  dot_strided(A, K, 1, W, 1, K, C, M, N, K, 1.0f, 0.0f);
  if (!workspace) free(W);
}

/* ------------------------------------------------------------------------ */
/* attention                                                                 */
/* ------------------------------------------------------------------------ */

static void attn_one(const float* qh, const float* Kh, const float* Vh, float* oh,
                     int64_t ctx, int64_t D, float scale, float* s) {
  /* array.h:1663-1685, one head */
  float mx = -INFINITY;
  for (int64_t j = 0; j < ctx; j++) {
    float acc = 0;
    for (int64_t d = 0; d < D; d++) acc += qh[d] * Kh[j * D + d];
    s[j] = acc * scale;
    if (s[j] > mx) mx = s[j];
  }
  float sum = 0;
  for (int64_t j = 0; j < ctx; j++) {
    s[j] = expf(s[j] - mx);
    sum += s[j];
  }
  for (int64_t d = 0; d < D; d++) {
    float acc = 0;
    for (int64_t j = 0; j < ctx; j++) acc += s[j] * Vh[j * D + d];
    oh[d] = acc / sum;
  }
}

void orc_attn_decode(const float* q, const float* K, const float* V, float* out,
                     int64_t n_q_heads, int64_t n_kv_heads, int64_t ctx, int64_t kv_max,
                     int64_t D, float scale) {
  /* array.h:1654-1687 with the head map of cuda.h:962-1009: query head h reads
   * kv head h/(Hq/Hkv); a head's keys start at kv*kv_max*D and the first ctx
   * rows are live. With Hq==Hkv and kv_max==ctx this is ref_attn_ verbatim. */
  int64_t group = n_q_heads / n_kv_heads;
  float* s = (float*)malloc((size_t)(ctx > 0 ? ctx : 1) * sizeof(float));
  for (int64_t h = 0; h < n_q_heads; h++) {
    int64_t kv = h / group;
    attn_one(q + h * D, K + kv * kv_max * D, V + kv * kv_max * D, out + h * D, ctx, D,
             scale, s);
  }
  free(s);
}

void orc_attn_prefill(const float* q, const float* K, const float* V, float* out,
                      int64_t n_q_heads, int64_t n_kv_heads, int64_t T, int64_t kv_max,
                      int64_t D, float scale, int64_t pos0) {
  int64_t group = n_q_heads / n_kv_heads;
  float* s = (float*)malloc((size_t)(pos0 + T) * sizeof(float));
  for (int64_t h = 0; h < n_q_heads; h++) {
    int64_t kv = h / group;
    for (int64_t p = 0; p < T; p++)
      attn_one(q + (h * T + p) * D, K + kv * kv_max * D, V + kv * kv_max * D,
               out + (h * T + p) * D, pos0 + p + 1, D, scale, s);
  }
  free(s);
}

/* ------------------------------------------------------------------------ */
/* rope                                                                      */
/* ------------------------------------------------------------------------ */

void orc_rope(const float* x, const float* bias, float* out, int64_t rows, int64_t T,
              int64_t D, int64_t pos, float base) {
  /* array.h:1709-1734: fp64 angle, fp32 rotation; bias (cu:1374-1377) is added
   * to both halves before rotating, indexed like x. */
  int64_t half = D / 2;
  for (int64_t r = 0; r < rows; r++) {
    int64_t t = T ? r % T : 0;
    double position = (double)(pos + t);
    const float* xr = x + r * D;
    float* orr = out + r * D;
    for (int64_t j = 0; j < half; j++) {
      double theta = pow((double)base, -2.0 * (double)j / (double)D);
      double ang = position * theta;
      float c = (float)cos(ang);
      float s = (float)sin(ang);
      float x0 = xr[j], x1 = xr[j + half];
      if (bias) {
        x0 += bias[r * D + j];
        x1 += bias[r * D + j + half];
      }
      orr[j] = x0 * c - x1 * s;
      orr[j + half] = x0 * s + x1 * c;
    }
  }
}

/* ------------------------------------------------------------------------ */
/* elementwise / rows                                                        */
/* ------------------------------------------------------------------------ */

static inline float bin_(int op, float x, float y) {
  switch (op) {
    case ORC_ADD: return x + y;
    case ORC_SUB: return x - y;
    case ORC_MUL: return x * y;
    case ORC_DIV: return x / y;
    default: return powf(x, y);
  }
}

static inline float un_(int op, float x) {
  switch (op) {
    case ORC_EXP: return expf(x);
    case ORC_LOG: return logf(x);
    case ORC_SQRT: return sqrtf(x);
    case ORC_SIGMOID: return 1.0f / (1.0f + expf(-x));
    case ORC_RELU: return x > 0 ? x : 0.0f;
    case ORC_RECIP: return 1.0f / x;
    default: return x;
  }
}

static inline float epi_(float v, float scale, float offset) {
  /* array.h:1872-1882 / 2218-2225: identity epilogues are skipped */
  if (scale == 1.0f && offset == 0.0f) return v;
  return v * scale + offset;
}

void orc_binary(int op, const float* a, const float* b, float* out, int64_t n,
                float scale, float offset) {
  for (int64_t i = 0; i < n; i++) out[i] = epi_(bin_(op, a[i], b[i]), scale, offset);
}

void orc_binary_bcast(int op, const float* a, int64_t ars, int64_t acs, const float* b,
                      int64_t brs, int64_t bcs, float* out, int64_t m, int64_t n,
                      float scale, float offset) {
  for (int64_t i = 0; i < m; i++)
    for (int64_t j = 0; j < n; j++)
      out[i * n + j] =
          epi_(bin_(op, a[i * ars + j * acs], b[i * brs + j * bcs]), scale, offset);
}

void orc_unary(int op, const float* a, float* out, int64_t n, float scale, float offset) {
  for (int64_t i = 0; i < n; i++) out[i] = epi_(un_(op, a[i]), scale, offset);
}

void orc_row_sum(const float* in, float* out, int64_t rows, int64_t cols, float scale,
                 float offset) {
  /* array.h:849-880 last-axis fast path: sequential f32 accumulator */
  for (int64_t r = 0; r < rows; r++) {
    float acc = 0.0f;
    for (int64_t c = 0; c < cols; c++) acc += in[r * cols + c];
    out[r] = epi_(acc, scale, offset);
  }
}

void orc_row_max(const float* in, float* out, int64_t rows, int64_t cols, float scale,
                 float offset) {
  for (int64_t r = 0; r < rows; r++) {
    float acc = -INFINITY;
    for (int64_t c = 0; c < cols; c++)
      if (in[r * cols + c] > acc) acc = in[r * cols + c];
    out[r] = epi_(acc, scale, offset);
  }
}

void orc_softmax(const float* in, float* out, int64_t rows, int64_t cols) {
  /* array.h:915-944 */
  for (int64_t r = 0; r < rows; r++) {
    const float* src = in + r * cols;
    float* dst = out + r * cols;
    float m = src[0];
    for (int64_t c = 1; c < cols; c++)
      if (src[c] > m) m = src[c];
    float denom = 0;
    for (int64_t c = 0; c < cols; c++) {
      dst[c] = expf(src[c] - m);
      denom += dst[c];
    }
    for (int64_t c = 0; c < cols; c++) dst[c] /= denom;
  }
}

/* ------------------------------------------------------------------------ */
/* model ops                                                                 */
/* ------------------------------------------------------------------------ */

void orc_rmsnorm(const float* x, const float* w, float* out, int64_t rows, int64_t n,
                 float eps) {
  /* array.h:2429-2433 step by step in CPU mode:
   *   ms  = mean(x*x, -1, keepdims)  -> ref::mean (977-983): sequential f32 sum,
   *                                     then * (1.0f/n); "+eps" rides the node's
   *                                     epilogue (1305-1311): ms*1 + eps
   *   inv = 1.0f / sqrt(.)           -> sqrtf, then recip 1.0f/x (scale 1)
   *   out = (x*inv)*weight */
  const float invn = 1.0f / (float)n;
  for (int64_t r = 0; r < rows; r++) {
    const float* xr = x + r * n;
    float acc = 0.0f;
    for (int64_t i = 0; i < n; i++) acc += xr[i] * xr[i];
    float ms = acc * invn;
    ms = ms * 1.0f + eps;
    float inv = 1.0f / sqrtf(ms);
    for (int64_t i = 0; i < n; i++) out[r * n + i] = (xr[i] * inv) * w[i];
  }
}

void orc_rmsnorm_res(const float* x, const float* delta, const float* w, float* xout,
                     float* hout, int64_t rows, int64_t n, float eps) {
  /* qm:586-590: x1 = x + delta (binary add), then rmsnorm(x1, w) */
  for (int64_t i = 0; i < rows * n; i++) xout[i] = x[i] + delta[i];
  orc_rmsnorm(xout, w, hout, rows, n, eps);
}

void orc_silu(const float* x, float* out, int64_t n) {
  /* array.h:2435: x * sigmoid(x) */
  for (int64_t i = 0; i < n; i++) out[i] = x[i] * (1.0f / (1.0f + expf(-x[i])));
}

void orc_swiglu(const float* gate, const float* up, float* out, int64_t n) {
  /* array.h:2437-2439: silu(gate) * up */
  for (int64_t i = 0; i < n; i++)
    out[i] = (gate[i] * (1.0f / (1.0f + expf(-gate[i])))) * up[i];
}

void orc_swiglu_fused(const float* gu, float* out, int64_t ff, int64_t rows) {
  for (int64_t r = 0; r < rows; r++)
    orc_swiglu(gu + r * 2 * ff, gu + r * 2 * ff + ff, out + r * ff, ff);
}

int64_t orc_argmax(const float* v, int64_t n) {
  int64_t best = 0;
  float m = v[0];
  for (int64_t i = 0; i < n; i++)
    if (v[i] > m) {
      m = v[i];
      best = i;
    }
  return best;
}

/* ------------------------------------------------------------------------ */
/* cache + layout moves                                                      */
/* ------------------------------------------------------------------------ */

void orc_kv_append(float* Kc, float* Vc, const float* k_new, const float* v_new,
                   int64_t pos, int64_t kv_max, int64_t n_kv_heads, int64_t D) {
  for (int64_t h = 0; h < n_kv_heads; h++) {
    memcpy(Kc + (h * kv_max + pos) * D, k_new + h * D, (size_t)D * sizeof(float));
    memcpy(Vc + (h * kv_max + pos) * D, v_new + h * D, (size_t)D * sizeof(float));
  }
}

void orc_kv_fill(float* Kc, float* Vc, const float* K, const float* V, int64_t T,
                 int64_t kv_max, int64_t n_kv_heads, int64_t D, int64_t pos0) {
  for (int64_t h = 0; h < n_kv_heads; h++)
    for (int64_t p = 0; p < T; p++) {
      memcpy(Kc + (h * kv_max + pos0 + p) * D, K + (h * T + p) * D, (size_t)D * sizeof(float));
      memcpy(Vc + (h * kv_max + pos0 + p) * D, V + (h * T + p) * D, (size_t)D * sizeof(float));
    }
}

void orc_split_heads(const float* src, const float* bias, float* dst, int64_t T,
                     int64_t ld, int64_t off, int64_t H, int64_t D) {
  for (int64_t h = 0; h < H; h++)
    for (int64_t t = 0; t < T; t++)
      for (int64_t d = 0; d < D; d++) {
        float v = src[t * ld + off + h * D + d];
        if (bias) v += bias[h * D + d];
        dst[(h * T + t) * D + d] = v;
      }
}

void orc_merge_heads(const float* src, float* dst, int64_t T, int64_t H, int64_t D) {
  for (int64_t h = 0; h < H; h++)
    for (int64_t t = 0; t < T; t++)
      for (int64_t d = 0; d < D; d++) dst[t * H * D + h * D + d] = src[(h * T + t) * D + d];
}

/* ------------------------------------------------------------------------ */
/* decode model                                                              */
/* ------------------------------------------------------------------------ */

typedef struct {
  /* stored form (q4 buffer or bf16 [K,N]) + the f32 widening used to compute */
  void* stored;
  int64_t stored_bytes;
  float* f32; /* [K,N] */
  int64_t K, N;
} orc_lin;

typedef struct {
  orc_lin wq, wk, wv, wo, wg, wu, wd;
  float *bq, *bk, *bv, *an, *fn;
  float *Kc, *Vc;
} orc_layer;

struct orc_qwen {
  orc_qwen_dims d;
  int q4;
  uint16_t* embed; /* bf16 [vocab, hidden] */
  float* embed_f32; /* when set (a model file's f16 table, widened): used instead of embed */
  float* onorm;
  orc_lin outw; /* [hidden, vocab] */
  orc_layer* layers;
};

static void lin_init(orc_lin* L, int64_t K, int64_t N, uint32_t seed, int q4) {
  L->K = K;
  L->N = N;
  float* w = (float*)malloc((size_t)K * (size_t)N * sizeof(float));
  orc_fill_normal(w, K * N, seed, 0.0f, 0.02f);
  if (q4) {
    L->stored_bytes = orc_q4_bytes(N, K);
    L->stored = malloc((size_t)L->stored_bytes);
    orc_to_q4(w, N, 1, K, N, (uint8_t*)L->stored);
    orc_q4_to_f32((const uint8_t*)L->stored, K, N, w);
  } else {
    L->stored_bytes = K * N * 2;
    L->stored = malloc((size_t)L->stored_bytes);
    orc_to_bf16(w, (uint16_t*)L->stored, K * N);
    orc_bf16_widen((const uint16_t*)L->stored, w, K * N);
  }
  L->f32 = w;
}

static void lin_free(orc_lin* L) {
  free(L->stored);
  free(L->f32);
}

static float* vec_normal(int64_t n, uint32_t seed, float mean, float std) {
  float* v = (float*)malloc((size_t)n * sizeof(float));
  orc_fill_normal(v, n, seed, mean, std);
  return v;
}

/* Weight generation is a set of independent seeded streams (one per matrix), so it is
 * spread over a few threads; every value is what the serial order produces. */
typedef struct {
  orc_lin* lin;         /* a linear weight ... */
  int64_t K, N;
  uint16_t* embed;      /* ... or the bf16 embedding table of n values */
  int64_t n;
  uint32_t seed;
  int q4;
} gen_task;

typedef struct {
  gen_task* tasks;
  int n_tasks;
  int next;
  pthread_mutex_t mu;
} gen_queue;

static void* gen_worker(void* qv) {
  gen_queue* q = (gen_queue*)qv;
  for (;;) {
    pthread_mutex_lock(&q->mu);
    int i = q->next < q->n_tasks ? q->next++ : -1;
    pthread_mutex_unlock(&q->mu);
    if (i < 0) return NULL;
    gen_task* t = &q->tasks[i];
    if (t->lin) {
      lin_init(t->lin, t->K, t->N, t->seed, t->q4);
    } else {
      float* emb = vec_normal(t->n, t->seed, 0.0f, 0.02f);
      orc_to_bf16(emb, t->embed, t->n);
      free(emb);
    }
  }
}

static int by_size_desc(const void* a, const void* b) {
  const gen_task *x = (const gen_task*)a, *y = (const gen_task*)b;
  int64_t sx = x->lin ? x->K * x->N : x->n, sy = y->lin ? y->K * y->N : y->n;
  return sx < sy ? 1 : sx > sy ? -1 : 0;
}

orc_qwen* orc_qwen_create(const orc_qwen_dims* d, uint32_t seed, int q4) {
  orc_qwen* m = (orc_qwen*)calloc(1, sizeof(orc_qwen));
  m->d = *d;
  m->q4 = q4;
  const int64_t E = d->hidden, QD = d->n_q_heads * d->head_dim,
                KD = d->n_kv_heads * d->head_dim;
  gen_task* tasks = (gen_task*)calloc((size_t)(2 + 7 * d->n_layers), sizeof(gen_task));
  int nt = 0;
#define LIN(ptr, k, n, sd) do { gen_task t = {(ptr), (k), (n), NULL, 0, (sd), q4}; tasks[nt++] = t; } while (0)
  m->embed = (uint16_t*)malloc((size_t)(d->vocab * E) * 2);
  { gen_task t = {NULL, 0, 0, m->embed, d->vocab * E, seed * 1000u + 1u, q4}; tasks[nt++] = t; }
  m->onorm = vec_normal(E, seed * 1000u + 2u, 1.0f, 0.02f);
  LIN(&m->outw, E, d->vocab, seed * 1000u + 3u);
  m->layers = (orc_layer*)calloc((size_t)d->n_layers, sizeof(orc_layer));
  for (int64_t l = 0; l < d->n_layers; l++) {
    orc_layer* L = &m->layers[l];
    uint32_t b = seed * 1000u + 100u + (uint32_t)l * 20u;
    LIN(&L->wq, E, QD, b + 1);
    LIN(&L->wk, E, KD, b + 2);
    LIN(&L->wv, E, KD, b + 3);
    LIN(&L->wo, QD, E, b + 4);
    LIN(&L->wg, E, d->ff, b + 5);
    LIN(&L->wu, E, d->ff, b + 6);
    LIN(&L->wd, d->ff, E, b + 7);
    L->bq = vec_normal(QD, b + 8, 0.0f, 0.02f);
    L->bk = vec_normal(KD, b + 9, 0.0f, 0.02f);
    L->bv = vec_normal(KD, b + 10, 0.0f, 0.02f);
    L->an = vec_normal(E, b + 11, 1.0f, 0.02f);
    L->fn = vec_normal(E, b + 12, 1.0f, 0.02f);
    L->Kc = (float*)calloc((size_t)(d->n_kv_heads * d->max_ctx * d->head_dim), sizeof(float));
    L->Vc = (float*)calloc((size_t)(d->n_kv_heads * d->max_ctx * d->head_dim), sizeof(float));
  }
#undef LIN
  qsort(tasks, (size_t)nt, sizeof(gen_task), by_size_desc);   /* largest first */
  gen_queue q = {tasks, nt, 0, PTHREAD_MUTEX_INITIALIZER};
  long cpus = sysconf(_SC_NPROCESSORS_ONLN);
  int n_thr = (int)(cpus < 1 ? 1 : cpus > 8 ? 8 : cpus);
  if (n_thr > nt) n_thr = nt;
  pthread_t thr[8];
  int started = 0;
  for (int i = 1; i < n_thr; i++)
    if (pthread_create(&thr[started], NULL, gen_worker, &q) == 0) started++;
  gen_worker(&q);
  for (int i = 0; i < started; i++) pthread_join(thr[i], NULL);
  free(tasks);
  return m;
}

/* The host K (which = 0) or V (which = 1) cache of a layer, [n_kv_heads, max_ctx, head_dim]:
 * lets a test start a step deep in a context from seeded cache rows. */
float* orc_qwen_cache(orc_qwen* m, int64_t layer, int which) {
  if (layer < 0 || layer >= m->d.n_layers) return NULL;
  return which ? m->layers[layer].Vc : m->layers[layer].Kc;
}

void orc_qwen_destroy(orc_qwen* m) {
  if (!m) return;
  for (int64_t l = 0; l < m->d.n_layers; l++) {
    orc_layer* L = &m->layers[l];
    lin_free(&L->wq); lin_free(&L->wk); lin_free(&L->wv); lin_free(&L->wo);
    lin_free(&L->wg); lin_free(&L->wu); lin_free(&L->wd);
    free(L->bq); free(L->bk); free(L->bv); free(L->an); free(L->fn);
    free(L->Kc); free(L->Vc);
  }
  free(m->layers);
  lin_free(&m->outw);
  free(m->onorm);
  free(m->embed);
  free(m->embed_f32);
  free(m);
}

void orc_qwen_reset(orc_qwen* m) { (void)m; /* positions are passed per step */ }

static void lin_apply(const orc_lin* L, const float* x, float* y) {
  /* x[1,K].dot(W) in CPU mode: widen (done once at create) + cpu::sgemm */
  orc_sgemm(x, L->K, 1, L->f32, L->N, 1, y, 1, L->N, L->K, 1.0f);
}

int64_t orc_qwen_step(orc_qwen* m, int64_t token, int64_t pos, float* logits) {
  /* bench/cuda/qwen_model.h:559-599 (the array-path forward), with the cache
   * held on the host and attention over its prefix. */
  const orc_qwen_dims* d = &m->d;
  const int64_t E = d->hidden, HQ = d->n_q_heads, HKV = d->n_kv_heads, HD = d->head_dim,
                FF = d->ff;
  const float scale = 1.0f / sqrtf((float)HD);
  float* x = (float*)malloc((size_t)E * 4);
  float* h = (float*)malloc((size_t)E * 4);
  float* x1 = (float*)malloc((size_t)E * 4);
  float* q = (float*)malloc((size_t)(HQ * HD) * 4);
  float* k = (float*)malloc((size_t)(HKV * HD) * 4);
  float* v = (float*)malloc((size_t)(HKV * HD) * 4);
  float* a = (float*)malloc((size_t)(HQ * HD) * 4);
  float* t = (float*)malloc((size_t)E * 4);
  float* g = (float*)malloc((size_t)FF * 4);
  float* u = (float*)malloc((size_t)FF * 4);
  float* mm = (float*)malloc((size_t)FF * 4);
  if (m->embed_f32) memcpy(x, m->embed_f32 + token * E, (size_t)E * 4);
  else orc_bf16_widen(m->embed + token * E, x, E);
  for (int64_t l = 0; l < d->n_layers; l++) {
    orc_layer* L = &m->layers[l];
    orc_rmsnorm(x, L->an, h, 1, E, d->eps);
    lin_apply(&L->wq, h, q);
    orc_binary(ORC_ADD, q, L->bq, q, HQ * HD, 1.0f, 0.0f);
    orc_rope(q, NULL, q, HQ, 1, HD, pos, d->rope_base);
    lin_apply(&L->wk, h, k);
    orc_binary(ORC_ADD, k, L->bk, k, HKV * HD, 1.0f, 0.0f);
    orc_rope(k, NULL, k, HKV, 1, HD, pos, d->rope_base);
    lin_apply(&L->wv, h, v);
    orc_binary(ORC_ADD, v, L->bv, v, HKV * HD, 1.0f, 0.0f);
    orc_kv_append(L->Kc, L->Vc, k, v, pos, d->max_ctx, HKV, HD);
    orc_attn_decode(q, L->Kc, L->Vc, a, HQ, HKV, pos + 1, d->max_ctx, HD, scale);
    lin_apply(&L->wo, a, t);
    orc_binary(ORC_ADD, x, t, x1, E, 1.0f, 0.0f);
    orc_rmsnorm(x1, L->fn, h, 1, E, d->eps);
    lin_apply(&L->wg, h, g);
    lin_apply(&L->wu, h, u);
    orc_swiglu(g, u, mm, FF);
    lin_apply(&L->wd, mm, t);
    orc_binary(ORC_ADD, x1, t, x, E, 1.0f, 0.0f);
  }
  orc_rmsnorm(x, m->onorm, h, 1, E, d->eps);
  lin_apply(&m->outw, h, logits);
  int64_t id = orc_argmax(logits, d->vocab);
  free(x); free(h); free(x1); free(q); free(k); free(v); free(a); free(t);
  free(g); free(u); free(mm);
  return id;
}

/* Replace one weight of the model with caller data (a model built from a file instead
 * of from the seeded generator). Linear weights come as f32 in the logical [K,N] layout and are
 * stored in the model's format exactly as lin_init does: to_q4 / to_bf16, then widened back
 * (what the reference's build() does with the widened file tensors,
 * bench/cuda/qwen_model.h:449-505). Vectors are copied. "embed" takes f32 [vocab, hidden]. */
static void lin_set(orc_lin* L, const float* w_kn, int q4) {
  const int64_t K = L->K, N = L->N;
  memcpy(L->f32, w_kn, (size_t)(K * N) * 4);
  if (q4) {
    orc_to_q4(L->f32, N, 1, K, N, (uint8_t*)L->stored);
    orc_q4_to_f32((const uint8_t*)L->stored, K, N, L->f32);
  } else {
    orc_to_bf16(L->f32, (uint16_t*)L->stored, K * N);
    orc_bf16_widen((const uint16_t*)L->stored, L->f32, K * N);
  }
}

int orc_qwen_set(orc_qwen* m, int64_t layer, const char* name, const float* data) {
  const orc_qwen_dims* d = &m->d;
  const int64_t E = d->hidden, QD = d->n_q_heads * d->head_dim, KD = d->n_kv_heads * d->head_dim;
  if (layer < 0) {
    if (!strcmp(name, "embed")) {
      if (!m->embed_f32) m->embed_f32 = (float*)malloc((size_t)(d->vocab * E) * 4);
      memcpy(m->embed_f32, data, (size_t)(d->vocab * E) * 4);
      return 0;
    }
    if (!strcmp(name, "onorm")) { memcpy(m->onorm, data, (size_t)E * 4); return 0; }
    if (!strcmp(name, "outw")) { lin_set(&m->outw, data, m->q4); return 0; }
    return -1;
  }
  if (layer >= d->n_layers) return -1;
  orc_layer* L = &m->layers[layer];
  orc_lin* lin = !strcmp(name, "wq") ? &L->wq : !strcmp(name, "wk") ? &L->wk : !strcmp(name, "wv") ? &L->wv
               : !strcmp(name, "wo") ? &L->wo : !strcmp(name, "wg") ? &L->wg : !strcmp(name, "wu") ? &L->wu
               : !strcmp(name, "wd") ? &L->wd : NULL;
  if (lin) { lin_set(lin, data, m->q4); return 0; }
  if (!strcmp(name, "bq")) { memcpy(L->bq, data, (size_t)QD * 4); return 0; }
  if (!strcmp(name, "bk")) { memcpy(L->bk, data, (size_t)KD * 4); return 0; }
  if (!strcmp(name, "bv")) { memcpy(L->bv, data, (size_t)KD * 4); return 0; }
  if (!strcmp(name, "an")) { memcpy(L->an, data, (size_t)E * 4); return 0; }
  if (!strcmp(name, "fn")) { memcpy(L->fn, data, (size_t)E * 4); return 0; }
  return -1;
}

const void* orc_qwen_weight(const orc_qwen* m, int64_t layer, const char* name,
                            int64_t* bytes) {
  const orc_qwen_dims* d = &m->d;
  const int64_t E = d->hidden, QD = d->n_q_heads * d->head_dim,
                KD = d->n_kv_heads * d->head_dim;
#define RET(p, b) do { if (bytes) *bytes = (b); return (p); } while (0)
  if (layer < 0) {
    if (!strcmp(name, "embed")) RET(m->embed, d->vocab * E * 2);
    if (!strcmp(name, "onorm")) RET(m->onorm, E * 4);
    if (!strcmp(name, "outw")) RET(m->outw.stored, m->outw.stored_bytes);
    return NULL;
  }
  if (layer >= d->n_layers) return NULL;
  const orc_layer* L = &m->layers[layer];
  if (!strcmp(name, "wq")) RET(L->wq.stored, L->wq.stored_bytes);
  if (!strcmp(name, "wk")) RET(L->wk.stored, L->wk.stored_bytes);
  if (!strcmp(name, "wv")) RET(L->wv.stored, L->wv.stored_bytes);
  if (!strcmp(name, "wo")) RET(L->wo.stored, L->wo.stored_bytes);
  if (!strcmp(name, "wg")) RET(L->wg.stored, L->wg.stored_bytes);
  if (!strcmp(name, "wu")) RET(L->wu.stored, L->wu.stored_bytes);
  if (!strcmp(name, "wd")) RET(L->wd.stored, L->wd.stored_bytes);
  if (!strcmp(name, "bq")) RET(L->bq, QD * 4);
  if (!strcmp(name, "bk")) RET(L->bk, KD * 4);
  if (!strcmp(name, "bv")) RET(L->bv, KD * 4);
  if (!strcmp(name, "an")) RET(L->an, E * 4);
  if (!strcmp(name, "fn")) RET(L->fn, E * 4);
#undef RET
  return NULL;
}
