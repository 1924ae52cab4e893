// Pieces the GEMV kernels share: the streaming load, wavefront row sums on DPP / permlane
// swaps, and the producer / epilogue vocabulary of the fused forms.
#pragma once

#include "common.hpp"

namespace tlhip {

// 16-byte streaming load: weights are read exactly once per GEMV, so they are
// marked non-temporal and do not displace x and the scales in the caches.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_stream16(const uint4* p) {
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

// ---- weight formats of the row kernels ----------------------------------------------------
// int4: a byte of a packed row holds k even in its low nibble and k+1 in its
// high nibble. Instead of isolating the high nibble, the kernel converts the
// WHOLE byte (lo + 16*hi) and the masked low nibble, and folds the difference
// into the activations when they are staged:
//     lo*x_e + hi*x_o  =  lo*(x_e - x_o/16) + (lo + 16*hi)*(x_o/16)
// so a 32-bit word of 8 weights costs one v_and, eight v_cvt_f32_ubyteN and
// eight FMAs. The "-8" of the offset-binary nibbles becomes -8*sum(x) per
// group, also formed once at staging.
__device__ __forceinline__ uint32_t low_nibbles(uint32_t v) {
  uint32_t r;  // opaque to the optimiser so the byte converts below stay byte converts
  asm("v_and_b32 %0, 0x0f0f0f0f, %1" : "=v"(r) : "v"(v));
  return r;
}
__device__ __forceinline__ float byte0(uint32_t v) { return (float)(v & 0xffu); }
__device__ __forceinline__ float byte1(uint32_t v) { return (float)((v >> 8) & 0xffu); }
__device__ __forceinline__ float byte2(uint32_t v) { return (float)((v >> 16) & 0xffu); }
__device__ __forceinline__ float byte3(uint32_t v) { return (float)(v >> 24); }

// acc + h * x in one instruction, h the low (HI = false) or high half of `pair` read as an f16.
// A half that holds only mantissa bits is an f16 subnormal, value bits * 2^-24: four weight bits
// masked out of a word need no conversion to become a number.
template <bool HI>
__device__ __forceinline__ float fma_half(uint32_t pair, float x, float acc) {
  float d;
  if constexpr (HI)
    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(d) : "v"(pair), "v"(x), "v"(acc));
  else
    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel_hi:[1,0,0]" : "=v"(d) : "v"(pair), "v"(x), "v"(acc));
  return d;
}

struct FmtQ4 {
  static constexpr int E = 32;  // weights per 16-byte unit == one scale group
  static constexpr bool kScaled = true;
  // staged form of (x_even, x_odd, x_even, x_odd): the odd ones over 16 (exact), because their
  // nibbles are read where they sit, four bits up
  static __device__ __forceinline__ float4 stage(const float4 v) {
    return make_float4(v.x, v.y * 0.0625f, v.z, v.w * 0.0625f);
  }
  // sum_k nib_k * x_k over the unit, x in staged form. A 32-bit word holds weights 8i .. 8i+7,
  // byte j the pair (2j, 2j+1), even in the low nibble. Masked in place, the nibbles of bytes 0
  // and 2 (and, from the word shifted down a byte, 1 and 3) are the two f16 halves of a
  // register: five integer instructions and eight mixed-precision FMAs per eight weights. The
  // products are nib * 2^-24 * x, exact scalings of what the CPU loop adds (array.h:735-737), and
  // the factor comes off the unit's sum; only activations below 2^-120 lose bits to it.
  static __device__ __forceinline__ float dot(const uint4 w, const float4 (&x)[8]) {
    const uint32_t d[4] = {w.x, w.y, w.z, w.w};
    float a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t full = d[i], up = full >> 8;
      const uint32_t e02 = full & 0x000f000fu, o02 = full & 0x00f000f0u;
      const uint32_t e13 = up & 0x000f000fu, o13 = up & 0x00f000f0u;
      const float4 xa = x[2 * i], xb = x[2 * i + 1];
      a0 = fma_half<false>(e02, xa.x, a0);
      a1 = fma_half<false>(o02, xa.y, a1);
      a0 = fma_half<false>(e13, xa.z, a0);
      a1 = fma_half<false>(o13, xa.w, a1);
      a0 = fma_half<true>(e02, xb.x, a0);
      a1 = fma_half<true>(o02, xb.y, a1);
      a0 = fma_half<true>(e13, xb.z, a0);
      a1 = fma_half<true>(o13, xb.w, a1);
    }
    return (a0 + a1) * 16777216.0f;
  }
};

struct FmtBf16 {
  static constexpr int E = 8;
  static constexpr bool kScaled = false;
  static __device__ __forceinline__ float4 stage(const float4 v) { return v; }
  static __device__ __forceinline__ float dot(const uint4 w, const float4 (&x)[2]) {
    float a0 = 0.f, a1 = 0.f;
    a0 = fmaf(bf16_lo(w.x), x[0].x, a0);
    a1 = fmaf(bf16_hi(w.x), x[0].y, a1);
    a0 = fmaf(bf16_lo(w.y), x[0].z, a0);
    a1 = fmaf(bf16_hi(w.y), x[0].w, a1);
    a0 = fmaf(bf16_lo(w.z), x[1].x, a0);
    a1 = fmaf(bf16_hi(w.z), x[1].y, a1);
    a0 = fmaf(bf16_lo(w.w), x[1].z, a0);
    a1 = fmaf(bf16_hi(w.w), x[1].w, a1);
    return a0 + a1;
  }
};

// ---- 16-lane sum on DPP: every lane of a DPP row ends up with the row's total ----
template <int CTRL>
__device__ __forceinline__ float dpp_add_f32(float v) {
  const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true);
  return v + __int_as_float(t);
}

// Sum R per-lane partials over the wavefront at once. Halving steps trade
// values for lanes (lane bit m clear keeps the lower half of the values and
// receives the partner's contribution to them), so R values cost R-1 exchanges
// instead of 6R; what is left is one value per lane, finished inside its lane
// group on DPP. Returns, in every lane, the total of row (lane * R) >> 6.
template <int N, int M, int R>
__device__ __forceinline__ void halve_rows(float (&a)[R], int lane) {  // N live values -> N/2
  if constexpr (M == 32 || M == 16) {
    // one v_permlane swap hands the lower lanes both halves' a[i] and the upper lanes both
    // halves' a[i + N/2]: the same two operands the shuffle form adds
#pragma unroll
    for (int i = 0; i < N / 2; i++) {
      const LanePair p = M == 32 ? swap32(a[i], a[i + N / 2]) : swap16(a[i], a[i + N / 2]);
      a[i] = p.first + p.second;
    }
  } else {
    const bool up = (lane & M) != 0;
#pragma unroll
    for (int i = 0; i < N / 2; i++) {
      const float keep = up ? a[i + N / 2] : a[i];
      const float send = up ? a[i] : a[i + N / 2];
      a[i] = keep + __shfl_xor(send, M, kWave);
    }
  }
}

template <int R>
__device__ __forceinline__ float wave_sum_rows(float (&a)[R], int lane) {
  static_assert(R == 1 || R == 2 || R == 4 || R == 8, "rows per wavefront");
  if constexpr (R == 8) { halve_rows<8, 32>(a, lane); halve_rows<4, 16>(a, lane); halve_rows<2, 8>(a, lane); }
  if constexpr (R == 4) { halve_rows<4, 32>(a, lane); halve_rows<2, 16>(a, lane); }
  if constexpr (R == 2) { halve_rows<2, 32>(a, lane); }
  float v = a[0];
  // lanes that differ only in bits below the last halving mask share a row
  if (R <= 1) { const LanePair p = swap32(v, v); v = p.first + p.second; }
  if (R <= 2) { const LanePair p = swap16(v, v); v = p.first + p.second; }
  v = dpp_add_f32<0xB1>(v);                 // quad_perm [1,0,3,2]
  v = dpp_add_f32<0x4E>(v);                 // quad_perm [2,3,0,1]
  v = dpp_add_f32<0x141>(v);                // row_half_mirror: the two quads of 8 lanes
  if (R <= 4) v = dpp_add_f32<0x140>(v);    // row_mirror: the two halves of 16 lanes
  return v;
}

// How a block obtains the activation vector while it stages it. Folding the
// producer of x into the GEMV removes a launch and a round trip through memory;
// every block recomputes the (tiny) producer redundantly.
//   kPlain:   x is read as is.
//   kSwiglu:  x[k] = (g*sigmoid(g))*u with g = in[k], u = in[K + k]   (array.h:2435-2439)
//   kRmsnorm: s = in (+ delta); x = (s * 1/sqrt(mean(s*s) + eps)) * norm_w   (array.h:2429-2433);
//             block 0 also writes s to xout (the residual stream), which therefore
//             must not alias in or delta: other blocks still read them.
//   kAttnMerge: x is the decode attention's output, still in the split partials the attention
//             kernel left (per head and split: running maximum m, sum l, accumulator acc[D]):
//             x[h*D + d] = sum_s e^(m_s - M) acc_s[d] / sum_s e^(m_s - M) l_s, at most 16 splits,
//             in the summation order of the stand-alone merge kernel (same bits). The merge's
//             launch goes; what it read (a few KB per head) every block now reads from L2.
// How a block leaves its results (EPI):
//   kStore:  y[row] = dot.
//   kGateUp: W is [gate rows | up rows] (N/2 each); a lane group owns R/2 gate rows and the
//            matching up rows, and writes y[i] = (g*sigmoid(g))*u for i < N/2 - the gated
//            activation in the GEMV that produces it, once per element, instead of in every
//            block of the GEMV that consumes it.
enum { kPlain = 0, kSwiglu = 1, kRmsnorm = 2, kAttnMerge = 3 };
constexpr int kMergeMax = 16;  // splits the kAttnMerge producer takes (its lanes per head)
enum { kStore = 0, kGateUp = 1 };
__device__ __forceinline__ float gated(float g, float u) { return (g * (1.0f / (1.0f + expf(-g)))) * u; }
struct Producer {
  const float* delta;
  const float* norm_w;
  float* xout;
  float eps;
  // kAttnMerge: x points at the partials [heads*S] m | [heads*S] l | [heads*S][D] acc
  int S = 0, heads = 0, D = 0;
};

}  // namespace tlhip
