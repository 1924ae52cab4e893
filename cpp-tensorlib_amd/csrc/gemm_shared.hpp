// What the two prompt-GEMM files share: the K-split sums, the row exponents, the f16 split.
#pragma once
#include "common.hpp"

namespace tlhip {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t frag16 __attribute__((ext_vector_type(4)));   // eight 16-bit operands of one lane

// defined in prefill.hip
__global__ void splitk_sum_kernel(const float4* __restrict__ part, float4* __restrict__ C, int M, int n4,
                                  int ldc4, int S);
__global__ void splitk_sum_swiglu_kernel(const float4* __restrict__ part, float4* __restrict__ out, int M,
                                         int pf4, int nv4, int ldc4, int S, int hw4);
__global__ void row_exponent_f32_kernel(const float* __restrict__ A, int K, int* __restrict__ ea);
__global__ void row_exponent_bf16_kernel(const uint16_t* __restrict__ W, int K, int8_t* __restrict__ ew);

#if defined(__HIPCC__)
// Exponent that brings the largest magnitude of a row into [2^14, 2^15): 14 - floor(log2(max)),
// kept within [-126, 126] so that 2^e is a normal float; 0 for a row of zeros. `field` is the
// biased exponent field of the row's largest magnitude (255 for inf / NaN: they stay what they are).
__device__ __forceinline__ int row_exponent(int field, bool all_zero) {
  return all_zero ? 0 : max(-126, min(126, 14 - (field - 127)));
}
__device__ __forceinline__ float pow2f(int e) { return __uint_as_float((uint32_t)(e + 127) << 23); }   // e in [-126, 127]

// What is left of x after its first f16 term; 0 where that is not a number: an infinite x has an
// infinite first term and inf - inf, and a NaN second term would turn the +-inf that an fp32
// product chain gives there into NaN (a NaN x stays NaN through its first term).
__device__ __forceinline__ f32x2 rest_or_zero(f32x2 d) {
  d.x = d.x == d.x ? d.x : 0.f;
  d.y = d.y == d.y ? d.y : 0.f;
  return d;
}
// two scaled floats -> their f16 terms, both round-to-nearest; x - hi is exact in fp32.
// GUARD = false leaves out the two instructions per element that keep an infinity an infinity
// (for a loop that is bound by its vector instructions; an infinite x then gives NaN terms).
template <bool GUARD = true>
__device__ __forceinline__ void split2_f16(float x0, float x1, uint32_t& hi, uint32_t& lo) {
  const f32x2 x = {x0, x1};
  const f16x2 h = __builtin_convertvector(x, f16x2);
  const f32x2 rest = x - __builtin_convertvector(h, f32x2);
  const f16x2 l = __builtin_convertvector(GUARD ? rest_or_zero(rest) : rest, f16x2);
  hi = __builtin_bit_cast(uint32_t, h);
  lo = __builtin_bit_cast(uint32_t, l);
}
// 8 bf16 weights times 2^exponent -> 8 f16
__device__ __forceinline__ frag16 bf16x8_to_f16(frag16 r, float s) {
  frag16 o;
#pragma unroll
  for (int b = 0; b < 4; b++) {
    const f32x2 x = {__uint_as_float(r[b] << 16) * s, __uint_as_float(r[b] & 0xffff0000u) * s};
    o[b] = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2));
  }
  return o;
}
#endif

}  // namespace tlhip
