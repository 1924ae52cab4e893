/*
 * libtensorlib_hip.so — C ABI of the MI355X (gfx950) backend for the
 * cpp-tensorlib LLM decode path.
 *
 * This is the boundary a cpp-tensorlib backend header binds with
 * dlopen()/dlsym(), the way the reference's cuda.h binds libcuda
 * (include/cuda.h:240-321) — except that the kernels live behind this ABI too,
 * so the header above it is a thin launch/coherence layer. Plain C types only.
 *
 * Conventions
 *  - Every function returns 0 on success and a negative tlhip_status on
 *    failure; tlhip_last_error() describes the last failure of the calling
 *    thread. Nothing throws, nothing aborts.
 *  - All tensor pointers are DEVICE pointers obtained from tlhip_malloc.
 *    `*_off` arguments are byte offsets added to the base (the reference passes
 *    element offsets * 4, array.h:1480).
 *  - Launchers enqueue on the library's stream and return immediately;
 *    tlhip_sync() is the only blocking call besides the synchronous copies and
 *    tlhip_argmax. While a capture is open (tlhip_graph_begin) launches are
 *    recorded instead of run.
 *  - Shapes a kernel does not support are refused with TLHIP_EUNSUPPORTED
 *    before anything is launched; the caller (the backend header) turns that
 *    into the reference's "declined" (`false`).
 *  - One device, one stream, single-threaded use, as the reference's evaluator
 *    (README.md:182).
 */
#ifndef TENSORLIB_HIP_H
#define TENSORLIB_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TLHIP_ABI_VERSION 1

typedef enum {
  TLHIP_OK = 0,
  TLHIP_ENODEVICE = -1,    /* no usable gfx950 device / HIP runtime failure at init */
  TLHIP_EINVAL = -2,       /* null pointer, negative size, misaligned operand */
  TLHIP_EUNSUPPORTED = -3, /* shape/dtype outside what the kernels cover: caller falls back */
  TLHIP_ENOMEM = -4,
  TLHIP_ERUNTIME = -5      /* a HIP call failed; see tlhip_last_error() */
} tlhip_status;

/* Elementwise / row op codes. Values are those of the reference's shared
 * tl::metal::kop enum (include/metal.h:41-47) so a backend header can pass
 * static_cast<int>(op) straight through. */
typedef enum {
  TLHIP_ADD = 0, TLHIP_SUB = 1, TLHIP_MUL = 2, TLHIP_DIV = 3, TLHIP_POW = 4,
  TLHIP_EXP = 5, TLHIP_LOG = 6, TLHIP_SQRT = 7, TLHIP_SIGMOID = 8, TLHIP_RELU = 9,
  TLHIP_AFFINE = 10,
  TLHIP_BADD = 11, TLHIP_BSUB = 12, TLHIP_BMUL = 13, TLHIP_BDIV = 14, TLHIP_BPOW = 15,
  TLHIP_SOFTMAX = 26, TLHIP_ROW_SUM = 27, TLHIP_ROW_MAX = 28,
  TLHIP_RECIP = 64 /* extension: 1/x, so array::rmsnorm's `1.0f / sqrt` stays on device
                      (the reference evaluates recip on the CPU, array.h:2064-2066) */
} tlhip_op;

/* ---- lifecycle ------------------------------------------------------------
 * replaces cuda.h:240-321 (context ctor: driver load, device 0, module load) */
int tlhip_init(int device);               /* idempotent; device must be gfx950 */
int tlhip_abi_version(void);
const char* tlhip_arch(void);             /* "gfx950" once initialised, else "" */
const char* tlhip_last_error(void);
int tlhip_device_info(int* compute_units, int64_t* hbm_bytes, int* lds_bytes_per_cu);

/* ---- memory -----------------------------------------------------------------
 * replaces cuMemAlloc/cuMemFree/cuMemcpy* as used by cuda.h:553-637 */
int tlhip_malloc(void** dptr, size_t bytes);
int tlhip_free(void* dptr);
int tlhip_host_alloc(void** hptr, size_t bytes);    /* pinned, for the mirror's host side */
int tlhip_host_free(void* hptr);
int tlhip_memcpy_h2d(void* dst, const void* src, size_t bytes);       /* blocking */
int tlhip_memcpy_d2h(void* dst, const void* src, size_t bytes);       /* blocking, drains stream */
int tlhip_memcpy_h2d_async(void* dst, const void* src, size_t bytes); /* src must stay valid */
int tlhip_memcpy_d2d_async(void* dst, const void* src, size_t bytes);
int tlhip_fill_u32(void* dst, uint32_t value, size_t count);          /* fill kernel, capturable */
int tlhip_sync(void);                     /* cuda.h:501-506 flush() */

/* ---- graph capture (cuda.h:508-551) and timing events ----------------------- */
int tlhip_graph_begin(void);
int tlhip_graph_end(void** graph_exec);
int tlhip_graph_launch(void* graph_exec);
int tlhip_graph_destroy(void* graph_exec);
int tlhip_event_create(void** ev);
int tlhip_event_record(void* ev);         /* on the library's stream */
int tlhip_event_elapsed_ms(void* start, void* stop, float* ms); /* waits for stop */
int tlhip_event_destroy(void* ev);

/* ---- dispatch census ----------------------------------------------------------
 * Per-entry-point launch counters, so a test can assert that kernels ran
 * (the reference's WebGPU backend keeps the same census, webgpu.h:197-202). */
typedef enum {
  TLHIP_C_BINARY = 0, TLHIP_C_BCAST, TLHIP_C_UNARY, TLHIP_C_ROW_OP, TLHIP_C_GEMM,
  TLHIP_C_GEMV_F32, TLHIP_C_GEMV_BF16, TLHIP_C_GEMV_BF16_ROW, TLHIP_C_GEMV_Q4,
  TLHIP_C_ATTN_DECODE, TLHIP_C_ROPE, TLHIP_C_RMSNORM, TLHIP_C_RMSNORM_RES, TLHIP_C_SWIGLU,
  TLHIP_C_ARGMAX, TLHIP_C_KV_APPEND, TLHIP_C_KV_FILL, TLHIP_C_SPLIT_HEADS,
  TLHIP_C_MERGE_HEADS, TLHIP_C_GEMM_BF16_NT, TLHIP_C_ATTN_PREFILL, TLHIP_C_CONVERT,
  TLHIP_C_QUANTIZE_Q4, TLHIP_C_COUNT
} tlhip_census_id;
int tlhip_census(uint64_t* counts, int n);  /* copies min(n, TLHIP_C_COUNT) counters */
int tlhip_census_reset(void);

/* ---- elementwise / rows (the gpu:: seam of array.h:1470-1507, 1738-1773) ------ */
/* out = (a OP b)*scale + offset, n contiguous f32.  cuda.h:640-654 */
int tlhip_binary(int op, const void* a, int64_t a_off, const void* b, int64_t b_off,
                 void* out, int64_t out_off, int64_t n, float scale, float offset);
/* rank-2 broadcast, op in TLHIP_BADD..TLHIP_BPOW; element (i,j) reads
 * a[i*ars+j*acs], b[i*brs+j*bcs] (strides in elements, 0 = broadcast).
 * cuda.h:656-662 declines this; metal.h has it — implemented here. */
int tlhip_binary_bcast(int op, const void* a, int64_t a_off, int64_t ars, int64_t acs,
                       const void* b, int64_t b_off, int64_t brs, int64_t bcs, void* out,
                       int64_t out_off, int64_t m, int64_t n, float scale, float offset);
/* out = f(a)*scale + offset.  cuda.h:664-675 */
int tlhip_unary(int op, const void* a, int64_t a_off, void* out, int64_t out_off, int64_t n,
                float scale, float offset);
/* last-axis softmax (rows x cols out) or row_sum/row_max (rows out, affine epilogue).
 * cuda.h:1487-1503 */
int tlhip_row_op(int op, const void* in, int64_t in_off, void* out, int64_t out_off,
                 int64_t rows, int64_t cols, float scale, float offset);
/* C[m,n] = (A.B)*scale + offset, f32; lda/ldb row strides, ta/tb read a transposed
 * view in place.  cuda.h:1409-1483 */
int tlhip_gemm(const void* a, int64_t a_off, int64_t lda, int ta, const void* b, int64_t b_off,
               int64_t ldb, int tb, void* out, int64_t out_off, int64_t m, int64_t n,
               int64_t k, float scale, float offset);

/* ---- decode GEMV -------------------------------------------------------------- */
/* y[n] = sum_k a[k]*B[k,n], B f32 [K,N] row-major.  cuda.h:719-728 */
int tlhip_gemv_f32(const void* a, const void* B, void* y, int64_t n, int64_t k);
/* same, B bf16 [K,N].  cuda.h:729-742 */
int tlhip_gemv_bf16(const void* a, const void* B, void* y, int64_t n, int64_t k);
/* y[n] = sum_k a[k]*W[n,k], W bf16 [N,K] row-major; K % 8 == 0.  cuda.h:770-785 */
int tlhip_gemv_bf16_row(const void* a, const void* W, void* y, int64_t n, int64_t k);
/* y[n] = sum_k a[k] * scales[n][k/group] * (nibble(n,k) - 8).
 * qw: packed int4 [N][K/2] bytes, even k in the low nibble (array.h:735-737);
 * scales: f32 [N][K/group]. group > 0, K % group == 0, group % 8 == 0.
 * cuda.h:886-905 */
int tlhip_gemv_q4(const void* a, const void* qw, const void* scales, void* y, int64_t N,
                  int64_t K, int64_t group);

/* ---- attention ---------------------------------------------------------------- */
/* out[h,:] = softmax(scale * q[h,:].K[kv(h)]^T) . V[kv(h)],  kv(h) = h/(Hq/Hkv);
 * q,out [Hq,D] f32; K,V [Hkv,kv_max,D] read over rows [0,ctx); D in {64,128};
 * kv_bf16 != 0: K,V hold bf16.  cuda.h:962-1009 */
int tlhip_attn_decode(const void* q, const void* K, const void* V, void* out,
                      int64_t n_q_heads, int64_t n_kv_heads, int64_t ctx, int64_t kv_max,
                      int64_t D, float scale, int kv_bf16);
/* tlhip_attn_decode for callers that cannot allocate device memory (code under hipGraph
 * capture, serving loops and harnesses that forbid hipMalloc). No counterpart in the reference.
 * Same arguments, same launch plan and bit-identical results; the split partials live in a
 * 1 MiB array that is part of the library's code object (one copy per GPU, held until the process
 * ends) instead of the library's growable scratch, and the call itself allocates and frees
 * nothing. Needs a prior tlhip_init (which does allocate). A shape whose partials exceed 1 MiB
 * (Hq * splits * (D + 2) * 4 bytes; the 7B decode shape at ctx 4096 needs 932 KB) is refused with
 * TLHIP_EUNSUPPORTED. Every call on a GPU shares that GPU's array: calls that overlap on one
 * GPU race. Nothing in the array has to start at zero (each call writes every partial it reads). */
int tlhip_attn_decode_static(const void* q, const void* K, const void* V, void* out,
                             int64_t n_q_heads, int64_t n_kv_heads, int64_t ctx, int64_t kv_max,
                             int64_t D, float scale, int kv_bf16);
/* causal prefill: q,out [Hq,T,D]; query p is at position pos0+p and sees keys
 * [0,pos0+p].  cuda.h:1166-1201 */
int tlhip_attn_prefill(const void* q, const void* K, const void* V, void* out,
                       int64_t n_q_heads, int64_t n_kv_heads, int64_t T, int64_t kv_max,
                       int64_t D, float scale, int kv_bf16, int64_t pos0);
/* scatter one token's k,v [Hkv,D] into the cache row pos.  cuda.h:1116-1138 */
int tlhip_kv_append(void* Kc, void* Vc, const void* k_new, const void* v_new, int64_t pos,
                    int64_t kv_max, int64_t n_kv_heads, int64_t D, int kv_bf16);
/* bulk copy k,v [Hkv,T,D] into cache rows [pos0,pos0+T).  cuda.h:1140-1164 */
int tlhip_kv_fill(void* Kc, void* Vc, const void* K, const void* V, int64_t T, int64_t kv_max,
                  int64_t n_kv_heads, int64_t D, int kv_bf16, int64_t pos0);

/* ---- model ops ---------------------------------------------------------------- */
/* half-split rotary on [rows,D]; row r sits at position pos + r%T; bias (may be
 * NULL, [rows,D]) is added before rotating. Angles are computed in fp64 like the
 * reference CPU path (array.h:1709-1734).  cuda.h:1203-1222 */
int tlhip_rope(const void* x, void* out, int64_t rows, int64_t T, int64_t D, int64_t pos,
               float base, const void* bias);
/* out = x * 1/sqrt(mean(x^2)+eps) * w per row of n.  cuda.h:1284-1302 */
int tlhip_rmsnorm(const void* x, const void* w, void* out, int64_t n, float eps, int64_t rows);
/* xout = x + delta; hout = rmsnorm(xout)*w.  xout may alias x.  cuda.h:1229-1252 */
int tlhip_rmsnorm_res(const void* x, const void* delta, const void* w, void* xout, void* hout,
                      int64_t n, float eps, int64_t rows);
/* tlhip_rmsnorm_res with delta = parts[0] + ... + parts[S-1] (ascending, each [rows][n], rows*n
 * floats apart): the K-split parts of tlhip_gemm_bf16_nt_parts. xout must not be the parts. */
int tlhip_rmsnorm_res_parts(const void* x, const void* parts, int64_t S, const void* w, void* xout,
                            void* hout, int64_t n, float eps, int64_t rows);
/* out[rows,ff] = silu(gu[:, :ff]) * gu[:, ff:], gu [rows,2*ff].  cuda.h:1304-1319 */
int tlhip_swiglu(const void* gu, void* out, int64_t ff, int64_t rows);
/* index of the maximum of in[0..n), ties to the smallest index; blocks until the
 * result is on the host.  cuda.h:1254-1282 */
int tlhip_argmax(const void* in, int64_t n, int64_t* out_idx);
/* same reduction, result left in a device int32 (no sync; capturable) */
int tlhip_argmax_async(const void* in, int64_t n, void* out_idx_dev);

/* ---- fused decode-step epilogues (no single reference counterpart) -------------
 * q/k bias + rope, v bias and the cache append of one token in ONE launch; the
 * arithmetic is that of tlhip_rope (bias form), tlhip_binary(ADD) and
 * tlhip_kv_append, i.e. cuda.h:1203-1222, 640-654 and 1116-1138 as the reference's
 * run_layers_ chains them (bench/cuda/qwen_model.h:703-716).
 * qkv = [q (Hq*D) | k (Hkv*D) | v (Hkv*D)] f32, updated in place. */
int tlhip_qkv_rope_append(void* qkv, const void* bq, const void* bk, const void* bv, void* Kc,
                          void* Vc, int64_t n_q_heads, int64_t n_kv_heads, int64_t D, int64_t pos,
                          int64_t kv_max, float base, int kv_bf16);

/* ---- position on the device: capturable decode loops -----------------------------
 * Twins of tlhip_rope / tlhip_kv_append / tlhip_attn_decode / tlhip_qkv_rope_append that read
 * the position from a 4-byte device scalar the caller owns, so that ONE recorded hipGraph
 * serves every token (cuda.h:1011-1114). Grids do not depend on the position:
 * attention is planned for the cache CAPACITY kv_max and bounds its work by *d_pos
 * (ctx = *d_pos + 1); splits past the live context write neutral partials. `partials` is a
 * caller-owned device buffer of tlhip_attn_partials_bytes(...) bytes: like d_pos it is
 * graph-lifetime state, so it cannot be the library's growable scratch. */
int tlhip_rope_dpos(const void* x, void* out, int64_t rows, int64_t T, int64_t D, const void* d_pos,
                    float base, const void* bias);
/* *d_pos += 1 (tail of a recorded forward).  cuda.h:1037-1047 */
int tlhip_incr_u32(void* d_pos);
int tlhip_kv_append_dpos(void* Kc, void* Vc, const void* k_new, const void* v_new, const void* d_pos,
                         int64_t kv_max, int64_t n_kv_heads, int64_t D, int kv_bf16);
int64_t tlhip_attn_partials_bytes(int64_t n_q_heads, int64_t n_kv_heads, int64_t kv_max, int64_t D);
int tlhip_attn_decode_dpos(const void* q, const void* K, const void* V, void* out, int64_t n_q_heads,
                           int64_t n_kv_heads, const void* d_pos, int64_t kv_max, int64_t D,
                           float scale, int kv_bf16, void* partials, int64_t partials_bytes);
int tlhip_qkv_rope_append_dpos(void* qkv, const void* bq, const void* bk, const void* bv, void* Kc,
                               void* Vc, int64_t n_q_heads, int64_t n_kv_heads, int64_t D,
                               const void* d_pos, int64_t kv_max, float base, int kv_bf16);

/* ---- rotary angles formed once per step (no reference counterpart) -------------------
 * table[D/2] of float2 (cos, sin) at position pos (or *d_pos when d_pos is non-NULL), the fp64
 * expression of tlhip_rope. All layers of a decode step rotate by the same angles. */
int tlhip_rope_table(void* table, int64_t D, int64_t pos, const void* d_pos, float base);
/* tlhip_qkv_rope_append(_dpos) reading the angles from such a table; the cache row is pos, or
 * *d_pos when d_pos is non-NULL. Bit-identical to the table-less forms. */
int tlhip_qkv_rope_append_tab(void* qkv, const void* bq, const void* bk, const void* bv, void* Kc,
                              void* Vc, int64_t n_q_heads, int64_t n_kv_heads, int64_t D, int64_t pos,
                              const void* d_pos, int64_t kv_max, const void* table, int kv_bf16);

/* ---- q/k/v epilogue of a prompt chunk in one launch (no reference counterpart: the reference runs
 * split_heads with bias, rope of q, rope of k and kv_fill as separate ops, qwen_model.h:367-382) --
 * tlhip_rope_table_range: table[T][D/2] of float2 (cos, sin) at positions pos0 .. pos0 + T - 1, the
 * fp64 expression of tlhip_rope; every layer and head of the chunk rotates by these.
 * tlhip_qkv_rope_fill: qkv = the chunk's raw [T, (Hq + 2 Hkv) D] projection (token-major, left
 * untouched); adds the biases (each may be NULL), rotates q and k by `table`; q lands head-major in
 * qh [Hq, T, D], k and v go into cache rows pos0 .. pos0 + T - 1. Bit-identical to the separate
 * ops. D in {64, 128}, like the cache ops. */
int tlhip_rope_table_range(void* table, int64_t D, int64_t pos0, int64_t T, float base);
int tlhip_qkv_rope_fill(const void* qkv, const void* bq, const void* bk, const void* bv, const void* table,
                        void* qh, void* Kc, void* Vc, int64_t T, int64_t n_q_heads, int64_t n_kv_heads,
                        int64_t D, int64_t pos0, int64_t kv_max, int kv_bf16);
/* The same with qkv = the n_parts K-split parts of the projection (tlhip_gemm_bf16_nt_parts:
 * [n_parts][T][(Hq + 2 Hkv) D]), added up in ascending order as they are read. */
int tlhip_qkv_rope_fill_parts(const void* qkv, int64_t n_parts, const void* bq, const void* bk,
                              const void* bv, const void* table, void* qh, void* Kc, void* Vc, int64_t T,
                              int64_t n_q_heads, int64_t n_kv_heads, int64_t D, int64_t pos0,
                              int64_t kv_max, int kv_bf16);
/* tlhip_attn_prefill writing out token-major, [T, Hq*D] - what merge_heads (cuda.h:862-880) would
 * make of the head-major result, so that launch is not needed. */
int tlhip_attn_prefill_tok(const void* q, const void* K, const void* V, void* out,
                           int64_t n_q_heads, int64_t n_kv_heads, int64_t T, int64_t kv_max,
                           int64_t D, float scale, int kv_bf16, int64_t pos0);

/* ---- decode attention with the step's prologue fused in (no reference counterpart: the
 * reference runs bias, rope, cache append and attention as separate ops, qwen_model.h:560-600) --
 * qkv = the step's raw [q (Hq*D) | k (Hkv*D) | v (Hkv*D)] projection, left untouched. Adds the
 * biases (each may be NULL), rotates q and k by `table` (tlhip_rope_table), stores the new k, v
 * row at cache row pos (or *d_pos when d_pos is non-NULL; a full cache takes no row) and writes
 * out[Hq*D] = attention of the rotated q over keys [0, pos]. Same values as
 * tlhip_qkv_rope_append_tab followed by tlhip_attn_decode(_dpos); the new key enters the softmax
 * in a different position of the summation order. With d_pos the grid is planned for kv_max and
 * `partials` (tlhip_attn_partials_bytes) is required; without it partials may be NULL. */
int tlhip_attn_decode_qkv(const void* qkv, const void* bq, const void* bk, const void* bv, void* Kc,
                          void* Vc, void* out, int64_t n_q_heads, int64_t n_kv_heads, int64_t pos,
                          const void* d_pos, int64_t kv_max, int64_t D, float scale,
                          const void* table, int kv_bf16, void* partials, int64_t partials_bytes);

/* The same step with the split merge left to the o-projection (tlhip_gemv_*_attn below): nothing
 * is written but the cache row and `partials`, laid out [Hq*S] running maxima | [Hq*S] sums |
 * [Hq*S][D] accumulators for the S = *n_parts splits of the context that the launch plan chose
 * (also when S is 1). Served: f32 caches, 3 to 8 query heads per kv head, an even head count, and
 * contexts (capacities, with d_pos) that the plan cuts into at most 1024 / D, and at most 16,
 * splits - tlhip_attn_parts_splits tells (0: not served, call tlhip_attn_decode_qkv). `partials`
 * is required: tlhip_attn_partials_bytes. For small models: their merge launch costs as much as
 * a projection. */
int tlhip_attn_parts_splits(int64_t n_q_heads, int64_t n_kv_heads, int64_t plan_ctx, int64_t D, int kv_bf16);
int tlhip_attn_decode_qkv_parts(const void* qkv, const void* bq, const void* bk, const void* bv, void* Kc,
                                void* Vc, int64_t n_q_heads, int64_t n_kv_heads, int64_t pos,
                                const void* d_pos, int64_t kv_max, int64_t D, float scale,
                                const void* table, void* partials, int64_t partials_bytes, int* n_parts);

/* ---- device-resident greedy loop (no reference counterpart: the reference gathers the
 * embedding row on the host and reads every token back, qwen_model.h:530-535, 642-647) ----
 * out[hidden] f32 = widened row *d_token of a bf16 [vocab, hidden] table; d_token is a device
 * int32 (what tlhip_argmax_async wrote), clamped to [0, vocab). */
int tlhip_embed_gather_bf16(const void* table, const void* d_token, void* out, int64_t hidden,
                            int64_t vocab);
/* history[*d_pos] = *d_token when *d_pos < capacity (history may be NULL), then *d_pos += 1 */
int tlhip_token_advance(void* d_pos, const void* d_token, void* history, int64_t capacity);

/* ---- load-time weight conversion on the device ------------------------------------------
 * A model file (GGUF) stores linear layers as f16 / f32 / bf16 rows [out, in]. The reference
 * widens, transposes, narrows and quantises them on the host, element by element, and
 * uploads the result (bench/cuda/qwen_model.h:40-131); here the file's bytes are uploaded as
 * they are and converted on the device, bit-identically to that host arithmetic. */
typedef enum { TLHIP_T_F32 = 0, TLHIP_T_F16 = 1, TLHIP_T_BF16 = 2 } tlhip_elem_type;
/* dst[i] = narrow(widen(src[i])), i < n; dst_type f32 or bf16 (round to nearest even,
 * types.h:35-41); f16 widening is exact for every bit pattern (qwen_model.h:41-60). Same
 * layout both sides: file rows [out, in] ARE the row layout [N, K] of tlhip_gemv_bf16_row
 * (qwen_model.h:114-131 load_w_T_cat_row; stack parts by pointing dst at their row block). */
int tlhip_convert(const void* src, int src_type, void* dst, int dst_type, int64_t n);
/* dst[c * ld_dst + col_base + r] = src[r * cols + c]: file rows [out = rows, in = cols] into the
 * seam's [K, N] layout, N = ld_dst, this tensor's outputs at columns [col_base, col_base + rows)
 * (qwen_model.h:88-106 load_w_T_cat). dst_type f32 or bf16. */
int tlhip_convert_transpose(const void* src, int src_type, void* dst, int dst_type, int64_t rows,
                            int64_t cols, int64_t ld_dst, int64_t col_base);
/* array::to_q4 (array.h:703-742) applied to the widened rows: per group of 32 consecutive k of a
 * row, scale = max(1e-8, maxabs) / 7, q = clamp(lround(w / scale), -8, 7), nibble q + 8, even k
 * low. packed: rows x K/2 bytes, scales: rows x K/32 floats - the two sections of a q4 buffer
 * (point them at a row block of a fused buffer to stack parts). group must be 32. */
int tlhip_quantize_q4(const void* src, int src_type, void* packed, void* scales, int64_t rows,
                      int64_t K, int64_t group);
/* tlhip_embed_gather_bf16 for an f16 [vocab, hidden] table, as the file stores token_embd and
 * the reference gathers it (qwen_model.h:297, 531-540). */
int tlhip_embed_gather_f16(const void* table, const void* d_token, void* out, int64_t hidden,
                           int64_t vocab);

/* ---- GEMVs that produce their own activation vector (no single reference
 * counterpart) -----------------------------------------------------------------
 * The producer of x is evaluated by every block while it stages x, which removes a
 * launch and a memory round trip per fused pair. Arithmetic is that of the separate
 * entry points: tlhip_swiglu then tlhip_gemv_*, and tlhip_rmsnorm_res then
 * tlhip_gemv_*, as run_layers_ chains them (bench/cuda/qwen_model.h:717-737); the split merge of
 * tlhip_attn_decode_qkv then tlhip_gemv_*.
 * Row layouts only (int4 group 32, bf16 [N,K]); other shapes return
 * TLHIP_EUNSUPPORTED and the caller issues the two separate calls. */
/* y = W . swiglu(gu), gu = [gate (K) | up (K)] f32 */
int tlhip_gemv_q4_swiglu(const void* gu, const void* qw, const void* scales, void* y, int64_t N,
                         int64_t K, int64_t group);
int tlhip_gemv_bf16_row_swiglu(const void* gu, const void* W, void* y, int64_t n, int64_t k);
/* y = W . x, x[h*D + d] = sum_s e^(m_s - M) acc_s[d] / sum_s e^(m_s - M) l_s: the decode attention's
 * output, merged from the n_parts split partials tlhip_attn_decode_qkv_parts left (its layout;
 * K = heads * head_dim), bit for bit what tlhip_attn_decode_qkv writes to `out`. */
int tlhip_gemv_q4_attn(const void* parts, int64_t n_parts, int64_t heads, int64_t head_dim, const void* qw,
                       const void* scales, void* y, int64_t N, int64_t K, int64_t group);
int tlhip_gemv_bf16_row_attn(const void* parts, int64_t n_parts, int64_t heads, int64_t head_dim,
                             const void* W, void* y, int64_t n, int64_t k);
/* s = x (+ delta when non-NULL); xout (when non-NULL) receives s; y = W . rmsnorm(s, norm_w, eps).
 * xout must not alias x or delta. */
int tlhip_gemv_q4_rmsnorm(const void* x, const void* delta, const void* norm_w, void* xout,
                          const void* qw, const void* scales, void* y, int64_t N, int64_t K,
                          int64_t group, float eps);
int tlhip_gemv_bf16_row_rmsnorm(const void* x, const void* delta, const void* norm_w, void* xout,
                                const void* W, void* y, int64_t n, int64_t k, float eps);
/* The same with the gated activation as the GEMV's epilogue: W = [gate rows | up rows], N2 / 2
 * rows each (the fused [wg|wu] of qwen_model.h:194-199); act[i] = swiglu(gate_i, up_i) for
 * i < N2 / 2, arithmetic of tlhip_swiglu. The activation is then formed once per element by the
 * GEMV that produces it, and the down projection is a plain tlhip_gemv_*. */
int tlhip_gemv_q4_rmsnorm_gateup(const void* x, const void* delta, const void* norm_w, void* xout,
                                 const void* qw, const void* scales, void* act, int64_t N2, int64_t K,
                                 int64_t group, float eps);
int tlhip_gemv_bf16_row_rmsnorm_gateup(const void* x, const void* delta, const void* norm_w, void* xout,
                                       const void* W, void* act, int64_t n2, int64_t k, float eps);

/* ---- prefill ------------------------------------------------------------------ */
/* C[M,N] = A[M,K] f32 . W[N,K]^T bf16, fp32 accumulate; K % 8 == 0.  cuda.h:787-841 */
int tlhip_gemm_bf16_nt(const void* A, const void* W, void* C, int64_t M, int64_t N, int64_t K);
/* The same product left as its K-split parts: parts = [*n_parts][M][N] f32, dense, in a buffer
 * of the caller's (parts_bytes >= M*N*4; it also bounds the split), no part-sum launch. The
 * product is parts[0] + parts[1] + ... in that order - exactly what tlhip_gemm_bf16_nt stores
 * when it splits - and tlhip_rmsnorm_res_parts forms it while it reads. For the products whose
 * consumer is the residual norm (o-proj and down, qwen_model.h:382-383, 386-388). */
int tlhip_gemm_bf16_nt_parts(const void* A, const void* W, void* parts, int64_t parts_bytes, int64_t M,
                             int64_t N, int64_t K, int* n_parts);
/* The gate|up product of a prompt chunk with the gated activation as its epilogue:
 * W = [gate rows | up rows], [2*ff, K] bf16 (the fused [wg|wu] of qwen_model.h:194-199),
 * act[M, ff] = swiglu(A . gate^T, A . up^T) with tlhip_swiglu's arithmetic - the two launches of
 * qwen_model.h:384-385 in one; the [M, 2*ff] products are never written. Same products as
 * tlhip_gemm_bf16_nt on the same W; where K is split, it is split for other columns than there,
 * so the two agree to fp32 summation order, not bit for bit. */
int tlhip_gemm_bf16_nt_swiglu(const void* A, const void* W, void* act, int64_t M, int64_t ff, int64_t K);
/* The same three products over a PREPARED weight, for a harness that owns its weights (no reference
 * counterpart: gemm_bf16_nt of cuda.h:787-841 takes the weight alone). tlhip_gemm_f16w_prepare, once
 * when the weight is loaded, writes
 *   exps (tlhip_gemm_f16w_exps_bytes(N, gated) bytes, 16-byte aligned): per row of W the int8
 *     exponent 14 - floor(log2(max_k |W[r][k]|)), what brings the row's largest magnitude into
 *     [2^14, 2^15) (0 for a row of zeros); per row the count of its nonzero weights that lie more than
 *     2^31 below the row's largest (0xffff: the row holds an infinity or a NaN); and W's own address, and
 *   image (tlhip_gemm_f16w_bytes(N, K, gated) bytes; 0 = no image for this shape, K > 32768 included)
 *     = every weight times 2^exponent as f16, laid out slab by slab (256 rows x 32 k, 16 KB) in the
 *     order the kernel's LDS reads expect. A bf16 weight has 8 significant bits and an f16 holds 11,
 *     so each weight is exact unless it is one of the counted ones (then its absolute error is below
 *     2^-40 of the row's largest).
 * gated != 0: W = [gate rows | up rows], [2*N, K], N = features (the operand of
 * tlhip_gemm_bf16_nt_swiglu); the image then serves tlhip_gemm_f16w_nt_swiglu only, a plain image
 * the other two. K % 32 == 0.
 * The products cut every activation row, scaled the same way, into two f16 terms, both rounded to
 * nearest (2^-24 relative), and run two matrix-core products per weight instead of three, fp32
 * sums, the result scaled back exactly: the error is that of one fp32 rounding per product, as in
 * tlhip_gemm_bf16_nt, which these agree with to fp32 summation order. An activation more than 2^24
 * below its row's largest (like a counted weight) is carried with an absolute error only; the
 * products count those too and work out again, from A and W themselves with the fp32 FMA chain of
 * tensorlib_cuda.cu:509-519, every result in which such errors could reach a quarter of an absolute
 * tolerance of 1e-5, and every result of a row of A or W that holds an infinity or a NaN (which then
 * comes out as that chain leaves it). So the results meet allclose(rtol 1e-4, atol 1e-5) against
 * the fp32 chain whatever the spread of the operands; ordinary operands never take that path.
 * The image and exps are DERIVED from W and exps refers to it: W must stay allocated and unchanged
 * while they are in use (the decode GEMV keeps reading the bf16 weight anyway), and they must be
 * prepared again when W changes. */
int64_t tlhip_gemm_f16w_bytes(int64_t N, int64_t K, int gated);
int64_t tlhip_gemm_f16w_exps_bytes(int64_t N, int gated);
int tlhip_gemm_f16w_prepare(const void* W, int64_t N, int64_t K, int gated, void* image, void* exps);
int tlhip_gemm_f16w_nt(const void* A, const void* image, const void* exps, void* C, int64_t M, int64_t N,
                       int64_t K);
int tlhip_gemm_f16w_nt_parts(const void* A, const void* image, const void* exps, void* parts,
                             int64_t parts_bytes, int64_t M, int64_t N, int64_t K, int* n_parts);
int tlhip_gemm_f16w_nt_swiglu(const void* A, const void* image, const void* exps, void* act, int64_t M,
                              int64_t ff, int64_t K);
/* The same three products over an ACTIVATION IMAGE made beforehand: the row exponents and the two
 * f16 terms of A as slab images (tlhip_gemm_f16w_aimage_bytes(M, K) bytes, 16-byte aligned; 0: no
 * image for this shape), which the products above make on every call and the producer of A can
 * make while it still holds A's rows. One producer does: tlhip_rmsnorm_res_parts_aimage is
 * tlhip_rmsnorm_res_parts (same arguments, same bits in xout and hout; n % 32 == 0, n <= 8192)
 * that also leaves hout's image in `aimage`, saving the products' own pass over A (one launch and
 * one read of A per product: the two norms of a layer feed q|k|v and gate|up). A must still be
 * passed, and must be the rows the image was made from, unchanged: wide-range results are worked
 * out from them (above). Same results bit for bit as the calls without an image. No counterpart
 * in the reference (the products and the norm are separate ops, qwen_model.h:559-599). */
int64_t tlhip_gemm_f16w_aimage_bytes(int64_t M, int64_t K);
int tlhip_rmsnorm_res_parts_aimage(const void* x, const void* parts, int64_t S, const void* w, void* xout,
                                   void* hout, int64_t n, float eps, int64_t rows, void* aimage);
int tlhip_gemm_f16w_nt_aimage(const void* A, const void* aimage, const void* image, const void* exps, void* C,
                              int64_t M, int64_t N, int64_t K);
int tlhip_gemm_f16w_nt_parts_aimage(const void* A, const void* aimage, const void* image, const void* exps,
                                    void* parts, int64_t parts_bytes, int64_t M, int64_t N, int64_t K,
                                    int* n_parts);
int tlhip_gemm_f16w_nt_swiglu_aimage(const void* A, const void* aimage, const void* image, const void* exps,
                                     void* act, int64_t M, int64_t ff, int64_t K);
/* The three prompt-chunk products over an int4 weight (qw = packed nibbles [N][K/2], scales
 * [N][K/32], group 32 - the operand of tlhip_gemv_q4): C = A . dequant(W)^T formed as
 * sum over groups of scale * (A . q) with exact products on the matrix pipe, fp32 sums - the decode
 * GEMV's arithmetic, M rows at a time. No reference counterpart: the reference feeds prompts to
 * an int4 model one token at a time (qwen_model.h:419 gates its batched prefill on bf16 weights);
 * parity is against tlhip_gemv_q4 / the CPU path row by row. For M > 64 the activations enter as two
 * f16 terms of each row scaled by a power of two (nibbles are exact in f16): an activation more than
 * 2^24 below its row's largest keeps an absolute, not a relative, error (2^-39.5 of that largest),
 * and a row that holds an infinity comes out as NaN where the decode GEMV gives +-inf - parity
 * unpinned for such rows (no reference test feeds them); tlhip_gemv_q4 row by row is exact there. */
int tlhip_gemm_q4_nt(const void* A, const void* qw, const void* scales, void* C, int64_t M, int64_t N,
                     int64_t K, int64_t group);
int tlhip_gemm_q4_nt_parts(const void* A, const void* qw, const void* scales, void* parts,
                           int64_t parts_bytes, int64_t M, int64_t N, int64_t K, int64_t group,
                           int* n_parts);
int tlhip_gemm_q4_nt_swiglu(const void* A, const void* qw, const void* scales, void* act, int64_t M,
                            int64_t ff, int64_t K, int64_t group);
/* [T,ld] token-major (+ optional bias [H*D]) -> [H,T,D]; `off` selects a column
 * block of a fused projection.  cuda.h:846-864 */
int tlhip_split_heads(const void* src, const void* bias, void* dst, int64_t T, int64_t ld,
                      int64_t off, int64_t H, int64_t D);
/* [H,T,D] -> [T,H*D].  cuda.h:866-879 */
int tlhip_merge_heads(const void* src, void* dst, int64_t T, int64_t H, int64_t D);

/* Upper bound on the K splits of the [K,N] GEMVs (tlhip_gemv_f32 / tlhip_gemv_bf16); 1 = no
 * split, 0 = the built-in choice. The reference's diagnostic knob set_no_splitk (cuda.h:193-197,
 * 496-497), which its GEMV benchmark toggles through the backend header. */
int tlhip_tune_gemv_cols(int max_k_splits);

#ifdef __cplusplus
}
#endif
#endif /* TENSORLIB_HIP_H */
