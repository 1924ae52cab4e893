/* Benchmark and tuning entry points of libtensorlib_hip.so.
 *
 * Not part of the backend boundary: a backend header binds include/tensorlib_hip.h only.
 * These serve bench.py, the profiles and the tests that force a launch shape. They set
 * process-wide state: a caller that changes a launch shape restores it with the same call
 * (zeros) or with tlhip_tune_reset(). None has a counterpart in the reference.
 */
#ifndef TENSORLIB_HIP_BENCH_H
#define TENSORLIB_HIP_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- measurement yardsticks ---------------------------------------------------------
 * A plain 16-byte-per-lane streaming copy / read of `bytes` bytes, used to find
 * the HBM rate this GPU really sustains and to scale the profiler's traffic
 * counters. blocks <= 0 picks 8 blocks per CU. */
int tlhip_bench_copy(void* dst, const void* src, size_t bytes, int blocks);
int tlhip_bench_read(const void* src, size_t bytes, void* sink4, int blocks);

/* How many device / pinned-host allocation and release calls (hipMalloc, hipFree, hipHostMalloc,
 * hipHostFree) the library has made since it was loaded: its own scratch growth and the
 * tlhip_malloc / tlhip_free / tlhip_host_* calls of its users. A caller that must not allocate
 * (tlhip_attn_decode_static) can be checked against it. */
int tlhip_alloc_calls(uint64_t* calls);

/* ---- weight warm-up on a second stream ---------------------------------------------------
 * tlhip_warm_fork: up to four byte ranges (16-byte aligned) are read once, in the order given, by
 * `blocks` blocks of 256 threads (<= 0: 32) on a second stream of the same priority that starts
 * where the main stream stands now; nothing is written. What the reads leave behind is the
 * ranges' lines in the last-level cache, so that a later launch on the main stream finds them
 * there. nontemporal != 0 reads with streaming loads. tlhip_warm_join makes the main stream wait
 * for every fork since the last join (a capture must join before it ends; tlhip_graph_end does it
 * if the caller did not). Both record into an open capture as a parallel branch. */
int tlhip_warm_fork(const void* const* ptrs, const int64_t* bytes, int n, int blocks, int nontemporal);
int tlhip_warm_join(void);

/* ---- launch-shape overrides ----------------------------------------------------------
 * The int4 GEMV launch shape: rows per wavefront (1,2,4,8), wavefronts sharing one row's K
 * range, resident blocks per CU, wavefronts per block (<= 16; rounded down to a multiple of
 * the K-sharing wavefronts) and lanes that share a weight row (64 or 16); 0 restores the
 * built-in choice for that field. Results do not depend on it beyond fp32 summation order. */
int tlhip_tune_gemv_q4(int rows_per_wave, int k_waves, int blocks_per_cu, int waves_per_block,
                       int lanes_per_row);
/* Which kernel serves tlhip_attn_prefill: 0 = the built-in choice (the f16-term kernels on the
 * matrix cores from about 640 keys on at head size 128 and 1024 at head size 64, else the fp32
 * matrix pipe), 1 = the VALU kernel that shares its code with decode attention,
 * 2 = the fp32 matrix-pipe kernel, 4 = the f16-term kernels (two f16 terms per operand, scaled per
 * query row and per 32-key tile); 3 is not in use.
 * Same results within fp32 summation order; for A/B timing and tests. */
int tlhip_tune_attn_prefill(int kernel);
/* Which kernel serves decode attention: 0 = the built-in choice (for f32 caches with 3 to 8 query
 * heads per kv head the kernel that gives every query head a wavefront over K/V tiles staged in
 * LDS; otherwise the key-slot kernel), 1 = the key-slot kernel for every shape. Same results
 * within fp32 summation order; for A/B timing and tests. */
int tlhip_tune_attn_decode(int kernel);
/* How the prompt GEMMs over an int4 weight (M > 64) cut the f32 activations: 0 = the built-in
 * choice (two f16 terms), 3 = three bf16 terms. Same results within fp32 summation order; for A/B
 * timing and tests. */
int tlhip_tune_gemm_planes(int planes);
/* Every override back to the built-in choice (tlhip_tune_gemv_cols included). */
int tlhip_tune_reset(void);

#ifdef __cplusplus
}
#endif
#endif /* TENSORLIB_HIP_BENCH_H */
