// Shared host/device helpers for the gfx950 kernels behind the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <vector>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/tensorlib_hip.h"

namespace tlhip {

constexpr int kWave = 64;  // CDNA wavefront width; every tiling below assumes it

// ---- library state (one device, one stream) -------------------------------
struct Context {
  bool ready = false;
  int device = -1;
  int cus = 0;
  int lds_per_cu = 0;
  int64_t hbm_bytes = 0;
  hipStream_t stream = nullptr;   // every launch and async copy goes here
  // A second stream of the same priority that only ever runs weight warm-up reads
  // (tlhip_warm_fork / tlhip_warm_join); created on first use.
  hipStream_t side = nullptr;
  hipEvent_t ev_fork = nullptr, ev_join = nullptr;
  bool side_open = false;         // reads queued on `side` that the main stream has not joined yet
  bool capturing = false;
  // grow-only device scratch (split-K / split-KV partials, argmax partials)
  void* scratch = nullptr;
  size_t scratch_bytes = 0;
  // A recorded graph bakes the scratch address into its kernel nodes: once any graph
  // exists, an outgrown scratch buffer is retired (kept allocated), never freed.
  int graphs_recorded = 0;
  std::vector<void*> retired_scratch;
  int* argmax_dev = nullptr;      // one int32 result slot
  int* argmax_host = nullptr;     // pinned landing slot for the 4-byte result
  uint64_t census[TLHIP_C_COUNT] = {};
  uint64_t alloc_calls = 0;       // hipMalloc / hipFree / hipHostMalloc / hipHostFree calls the library has made
  // int4 GEMV launch-shape override (tlhip_tune_gemv_q4)
  int tune_q4_rows = 0, tune_q4_kw = 0, tune_q4_bpc = 0, tune_q4_nw = 0, tune_q4_lpr = 0;
  int tune_cols_max_splits = 0;   // [K,N] GEMV K-split bound (tlhip_tune_gemv_cols), 0 = automatic
  int tune_gemm_planes = 0;       // tlhip_tune_gemm_planes: 0 = automatic, 3 = int4 prompt GEMMs on three bf16 planes of A
  int tune_attn_decode = 0;       // tlhip_tune_attn_decode: 0 = automatic, 1 = the key-slot kernel for every shape
  int tune_prefill_valu = 0;      // tlhip_tune_attn_prefill: 0 = automatic, 1 = VALU kernel, 2 = fp32 matrix pipe, 4 = f16 terms
};

Context& ctx();
int fail(int code, const char* fmt, ...);   // records the message, returns code
int hip_fail(hipError_t e, const char* what);
void* scratch(size_t bytes);                // nullptr on allocation failure
int attn_static_setup(int device);          // attn.hip: address of the allocation-free entry point's array

inline const char* at(const void* base, int64_t byte_off) {
  return static_cast<const char*>(base) + byte_off;
}
inline char* at(void* base, int64_t byte_off) { return static_cast<char*>(base) + byte_off; }

#define TLHIP_REQUIRE_READY()                                                   \
  do {                                                                          \
    if (!::tlhip::ctx().ready) {                                                \
      int rc_ = tlhip_init(0);                                                  \
      if (rc_ != 0) return rc_;                                                 \
    }                                                                           \
  } while (0)

#define TLHIP_CHECK_LAUNCH(id)                                                  \
  do {                                                                          \
    hipError_t e_ = hipGetLastError();                                          \
    if (e_ != hipSuccess) return ::tlhip::hip_fail(e_, "kernel launch");        \
    ::tlhip::ctx().census[id]++;                                                \
    return TLHIP_OK;                                                            \
  } while (0)

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- device helpers ----------------------------------------------------------
#if defined(__HIPCC__)

// Phase timestamps for kernel tuning. Off in the library build; a single-translation-unit
// build with TLHIP_TRACE defined makes lane 0 of every wavefront record the shader clock at
// the marks, into g_trace[block][wave][slot].
#ifdef TLHIP_TRACE
constexpr int kTraceSlots = 8, kTraceWaves = 16, kTraceBlocks = 1024;
static __device__ unsigned long long g_trace[kTraceBlocks * kTraceWaves * kTraceSlots];
__device__ __forceinline__ void trace_mark(int slot) {
  const unsigned b = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  if ((threadIdx.x & 63) == 0 && b < kTraceBlocks)
    g_trace[(b * kTraceWaves + (threadIdx.x >> 6)) * kTraceSlots + slot] = __builtin_readcyclecounter();
}
#define TLHIP_MARK(slot) ::tlhip::trace_mark(slot)
#else
#define TLHIP_MARK(slot)
#endif

// One rounding each, never contracted into an FMA with a neighbouring operation: the CPU path
// multiplies and adds separately (its loops are compiled without FMA contraction). hipcc's
// __fmul_rn / __fadd_rn are plain `*` / `+` and do NOT prevent contraction; these do, because
// the operations are built in a scope where contraction is off and keep that property when inlined.
__device__ __forceinline__ float mul_rn(float a, float b) {
#pragma clang fp contract(off)
  return a * b;
}
__device__ __forceinline__ float add_rn(float a, float b) {
#pragma clang fp contract(off)
  return a + b;
}
__device__ __forceinline__ float sub_rn(float a, float b) {
#pragma clang fp contract(off)
  return a - b;
}

// Cross-lane exchanges without the LDS crossbar (gfx950).
//   swap32(x, y): lanes 0-31 get (x.lo, x.hi), lanes 32-63 get (y.lo, y.hi) as (first, second):
//   v_permlane32_swap trades x's upper half with y's lower half.
//   swap16(x, y): the same per pair of 16-lane rows (v_permlane16_swap).
// With x == y == v, first + second is v[l] + v[l ^ 32] (resp. ^ 16) in every lane.
struct LanePair { float first, second; };
__device__ __forceinline__ LanePair swap32(float x, float y) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(y), false, false);
  return LanePair{__uint_as_float(r[0]), __uint_as_float(r[1])};
}
__device__ __forceinline__ LanePair swap16(float x, float y) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(y), false, false);
  return LanePair{__uint_as_float(r[0]), __uint_as_float(r[1])};
}
template <int CTRL>
__device__ __forceinline__ float dpp_read(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// Butterfly over the wavefront: the pairings of xor 32, 16, 8, 4, 2, 1 in that order (row_ror n
// reads the xor-n partner's value once the values have period 2n within a row), so the sums
// are those of the shuffle form bit for bit.
__device__ __forceinline__ float wave_sum(float v) {
  LanePair p = swap32(v, v);
  v = p.first + p.second;
  p = swap16(v, v);
  v = p.first + p.second;
  v += dpp_read<0x128>(v);   // row_ror:8
  v += dpp_read<0x124>(v);   // row_ror:4
  v += dpp_read<0x122>(v);   // row_ror:2
  v += dpp_read<0x121>(v);   // row_ror:1
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
  LanePair p = swap32(v, v);
  v = fmaxf(p.first, p.second);
  p = swap16(v, v);
  v = fmaxf(p.first, p.second);
  v = fmaxf(v, dpp_read<0x128>(v));
  v = fmaxf(v, dpp_read<0x124>(v));
  v = fmaxf(v, dpp_read<0x122>(v));
  v = fmaxf(v, dpp_read<0x121>(v));
  return v;
}

// Block-wide sum for blocks of NW wavefronts; `red` is NW floats of LDS.
// Every thread gets the result. Summation order is fixed (wave 0..NW-1).
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NW; i++) t += red[i];
  __syncthreads();
  return t;
}

__device__ __forceinline__ float bf16_lo(uint32_t packed) {  // element 0 of a pair
  return __uint_as_float(packed << 16);
}
__device__ __forceinline__ float bf16_hi(uint32_t packed) {  // element 1 of a pair
  return __uint_as_float(packed & 0xffff0000u);
}
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
  uint32_t x = __float_as_uint(f);
  x += 0x7fffu + ((x >> 16) & 1u);
  return static_cast<uint16_t>(x >> 16);
}

#endif  // __HIPCC__

}  // namespace tlhip
