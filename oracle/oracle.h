/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Plain-C restatement of the reference's CPU arithmetic for the LLM decode
 * hot path (cpp-tensorlib, files under /root/reference/include). It is the
 * checker the HIP kernels are compared with; nothing in the shipped library
 * or its host headers may include, link or call it.
 *
 * Every function names the reference lines it restates. All of them are
 * pinned by the reference's own known-answer cases, by the compiled
 * reference (oracle/_ref, when built) and by closed forms / fp64 brute
 * force in tests/test_oracle_*.py; none is "parity unpinned".
 */
#ifndef TL_ORACLE_H
#define TL_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- seeded inputs (own PRNG: xorshift32 + Box-Muller in fp64) ---------- */
typedef struct { uint32_t s; double spare; int has_spare; } orc_rng;
void     orc_rng_seed(orc_rng* r, uint32_t seed);
uint32_t orc_rng_u32(orc_rng* r);
double   orc_rng_uniform(orc_rng* r);               /* [0,1) */
double   orc_rng_normal(orc_rng* r);                /* N(0,1) */
void     orc_fill_normal(float* dst, int64_t n, uint32_t seed, float mean, float std);
void     orc_fill_uniform(float* dst, int64_t n, uint32_t seed, float lo, float hi);
/* packed int4 weight buffer with arbitrary seeded scales (BASELINE config 1):
 * nibbles q+8 with q ~ U{-8..7}, scales ~ U(lo,hi). buf has orc_q4_bytes(N,K). */
void     orc_fill_q4(uint8_t* buf, int64_t N, int64_t K, uint32_t seed, float lo, float hi);
uint32_t orc_crc32(const void* data, int64_t bytes);

/* ---- storage formats (types.h:20-46, array.h:639-742) -------------------- */
uint16_t orc_f32_to_bf16(float f);                  /* types.h:35-40, RNE */
float    orc_bf16_to_f32(uint16_t h);               /* types.h:41-46 */
void     orc_to_bf16(const float* src, uint16_t* dst, int64_t n);   /* array.h:639-658 */
void     orc_bf16_widen(const uint16_t* src, float* dst, int64_t n);/* array.h:685-697 */
/* GGUF F16 widening of the model loader; pinned exhaustively (2^16 patterns) against an
 * independent IEEE half implementation (numpy float16) in tests/test_oracle_pins.py */
float    orc_f16_to_f32(uint16_t h);                                 /* bench/cuda/qwen_model.h:41-60 */
void     orc_f16_widen(const uint16_t* src, float* dst, int64_t n);
int64_t  orc_q4_bytes(int64_t N, int64_t K);        /* types.h:28-31 */
/* w is logical [K,N] with element strides (s0,s1); out = packed [N][K/2] bytes
 * then f32 scales [N][K/32]. array.h:703-742 */
int      orc_to_q4(const float* w, int64_t s0, int64_t s1, int64_t K, int64_t N, uint8_t* out);
/* dequantise to logical [K,N] f32 contiguous. array.h:666-684 */
void     orc_q4_to_f32(const uint8_t* buf, int64_t K, int64_t N, float* out);

/* ---- matmul (cpu.h:393-466, array.h:946-970, 1943-1972, 2109-2141) ------- */
/* cpu::sgemm summation order: per KC=512 slab an FMA chain from 0, slabs
 * added into C in order, alpha folded into A. Strides in elements. */
void orc_sgemm(const float* A, int64_t as0, int64_t as1, const float* B, int64_t bs0,
               int64_t bs1, float* C, int64_t m, int64_t n, int64_t k, float alpha);
/* ref::dot order (cpu::enabled_ == false): C zeroed, for l, for j: C += a*b. */
void orc_ref_dot(const float* A, int64_t as0, int64_t as1, const float* B, int64_t bs0,
                 int64_t bs1, float* C, int64_t m, int64_t n, int64_t k);
/* the CPU-mode `dot` node on f32 operands incl. the tiny fast path and the
 * fused epilogue (out = A.B*scale+offset). */
void orc_dot(const float* A, const float* B, float* C, int64_t m, int64_t n, int64_t k,
             float scale, float offset);
/* a[1,K] . Wq (q4 buffer, logical [K,N]): widen, then orc_dot. workspace: K*N floats
 * (NULL => malloc). */
void orc_gemv_q4(const float* a, const uint8_t* q4buf, float* y, int64_t N, int64_t K,
                 float scale, float offset, float* workspace);
/* a[1,K] . B (bf16, [K,N] contiguous) */
void orc_gemv_bf16(const float* a, const uint16_t* B, float* y, int64_t N, int64_t K,
                   float scale, float offset, float* workspace);
/* harness layout: W bf16 [N,K] row-major (cuda.h:770-785); the CPU restatement
 * is the same dot with B strides (1,K). */
void orc_gemv_bf16_row(const float* a, const uint16_t* W, float* y, int64_t N, int64_t K,
                       float* workspace);
/* prefill: C[M,N] = A[M,K] f32 . W[N,K]^T bf16 (cuda.h:790-841) via the dot ladder */
void orc_gemm_bf16_nt(const float* A, const uint16_t* W, float* C, int64_t M, int64_t N,
                      int64_t K, float* workspace);

/* ---- attention (array.h:1654-1687; GQA + cache prefix per cuda.h:962-1009) */
void orc_attn_decode(const float* q, const float* K, const float* V, float* out,
                     int64_t n_q_heads, int64_t n_kv_heads, int64_t ctx, int64_t kv_max,
                     int64_t D, float scale);
/* causal prefill attention (cuda.h:1166-1201): q,out [Hq,T,D]; query p sits at
 * absolute position pos0+p and sees keys 0..pos0+p. Same three-loop softmax. */
void orc_attn_prefill(const float* q, const float* K, const float* V, float* out,
                      int64_t n_q_heads, int64_t n_kv_heads, int64_t T, int64_t kv_max,
                      int64_t D, float scale, int64_t pos0);

/* ---- rope (array.h:1709-1734; optional bias per cu:1360-1380) ------------ */
void orc_rope(const float* x, const float* bias, float* out, int64_t rows, int64_t T,
              int64_t D, int64_t pos, float base);

/* ---- elementwise / rows (array.h:1974-2108, 913-983; metal.h:41-47 kop) -- */
enum { ORC_ADD, ORC_SUB, ORC_MUL, ORC_DIV, ORC_POW, ORC_EXP, ORC_LOG, ORC_SQRT,
       ORC_SIGMOID, ORC_RELU, ORC_AFFINE, ORC_RECIP };
void orc_binary(int op, const float* a, const float* b, float* out, int64_t n,
                float scale, float offset);
/* rank-2 broadcast: element (i,j) reads a[i*ars+j*acs], b[i*brs+j*bcs] */
void orc_binary_bcast(int op, const float* a, int64_t ars, int64_t acs, const float* b,
                      int64_t brs, int64_t bcs, float* out, int64_t m, int64_t n,
                      float scale, float offset);
void orc_unary(int op, const float* a, float* out, int64_t n, float scale, float offset);
void orc_row_sum(const float* in, float* out, int64_t rows, int64_t cols, float scale, float offset);
void orc_row_max(const float* in, float* out, int64_t rows, int64_t cols, float scale, float offset);
void orc_softmax(const float* in, float* out, int64_t rows, int64_t cols);

/* ---- model ops as array compositions (array.h:2429-2439) ----------------- */
void orc_rmsnorm(const float* x, const float* w, float* out, int64_t rows, int64_t n, float eps);
/* xout = x + delta; hout = rmsnorm(xout)*w  (cuda.h:1229-1252 as array ops) */
void orc_rmsnorm_res(const float* x, const float* delta, const float* w, float* xout,
                     float* hout, int64_t rows, int64_t n, float eps);
void orc_silu(const float* x, float* out, int64_t n);
void orc_swiglu(const float* gate, const float* up, float* out, int64_t n);
/* fused-buffer form: gu [rows, 2*ff] -> out [rows, ff] (cuda.h:1304-1319) */
void orc_swiglu_fused(const float* gu, float* out, int64_t ff, int64_t rows);
int64_t orc_argmax(const float* v, int64_t n);      /* array.h:2481-2494 */

/* ---- cache + layout moves (cuda.h:1116-1164, 843-879) --------------------- */
void orc_kv_append(float* Kc, float* Vc, const float* k_new, const float* v_new,
                   int64_t pos, int64_t kv_max, int64_t n_kv_heads, int64_t D);
void orc_kv_fill(float* Kc, float* Vc, const float* K, const float* V, int64_t T,
                 int64_t kv_max, int64_t n_kv_heads, int64_t D, int64_t pos0);
void orc_split_heads(const float* src, const float* bias, float* dst, int64_t T,
                     int64_t ld, int64_t off, int64_t H, int64_t D);
void orc_merge_heads(const float* src, float* dst, int64_t T, int64_t H, int64_t D);

/* ---- decode model (bench/cuda/qwen_model.h:559-599 wiring, host cache) ---- */
typedef struct {
  int64_t n_layers, hidden, n_q_heads, n_kv_heads, head_dim, ff, vocab, max_ctx;
  float eps, rope_base;
} orc_qwen_dims;

typedef struct orc_qwen orc_qwen;
/* Random-init model: linear weights N(0,0.02) stored int4 (group 32) when
 * q4 != 0 else bf16 [K,N]; embeddings bf16; norm weights 1+N(0,0.02); q/k/v
 * biases N(0,0.02). Weights are dequantised ONCE into f32 (bit-identical to the
 * per-call widening of array.h:1980-1984). */
orc_qwen* orc_qwen_create(const orc_qwen_dims* d, uint32_t seed, int q4);
void      orc_qwen_destroy(orc_qwen* m);
void      orc_qwen_reset(orc_qwen* m);
/* one decode step at position pos; logits [vocab] out; returns greedy id */
int64_t   orc_qwen_step(orc_qwen* m, int64_t token, int64_t pos, float* logits);
/* accessors so the GPU harness can upload the very same weight bytes */
int       orc_qwen_set(orc_qwen* m, int64_t layer, const char* name, const float* data);
const void*  orc_qwen_weight(const orc_qwen* m, int64_t layer, const char* name, int64_t* bytes);
/* host K (which = 0) / V (which = 1) cache of a layer, [n_kv_heads, max_ctx, head_dim] */
float*    orc_qwen_cache(orc_qwen* m, int64_t layer, int which);

#ifdef __cplusplus
}
#endif
#endif
