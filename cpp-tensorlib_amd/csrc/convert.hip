// Load-time weight conversion on the device.
//
// A model file stores linear layers as f16 (or f32 / bf16) rows [out, in]. The decode
// path wants bf16 rows [N, K], the int4 group format, or [K, N] for the seam's GEMV.
// The reference converts on the host, one element at a time, before uploading
// (bench/cuda/qwen_model.h:40-131, array.h:639-658, 703-742); here the file's bytes are
// uploaded as they are and these kernels write the decode formats straight into the
// weight buffers. All of it is byte/integer work at HBM speed, bit-identical to the
// host arithmetic.
#include "common.hpp"

namespace tlhip {

// ---- element formats -----------------------------------------------------------------
// IEEE half -> float, every bit pattern (subnormals exact, NaN payload kept, no quieting):
// the values of bench/cuda/qwen_model.h:41-60.
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  const uint32_t sign = (h & 0x8000u) << 16, exp = (h >> 10) & 31u, man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    // zero or subnormal: man * 2^-24, exact in f32 (and a normal f32, so no flush applies)
    bits = __float_as_uint(static_cast<float>(man) * 5.9604644775390625e-8f);
  } else if (exp == 31) {
    bits = 0x7f800000u | (man << 13);
  } else {
    bits = ((exp + 112u) << 23) | (man << 13);
  }
  return __uint_as_float(sign | bits);
}

template <int T> struct Elem;   // T: TLHIP_T_F32 / F16 / BF16
template <> struct Elem<TLHIP_T_F32> {
  using type = float;
  static __device__ __forceinline__ float load(const float* p, int64_t i) { return p[i]; }
  static __device__ __forceinline__ void store(float* p, int64_t i, float v) { p[i] = v; }
};
template <> struct Elem<TLHIP_T_F16> {
  using type = uint16_t;
  static __device__ __forceinline__ float load(const uint16_t* p, int64_t i) { return f16_bits_to_f32(p[i]); }
};
template <> struct Elem<TLHIP_T_BF16> {
  using type = uint16_t;
  static __device__ __forceinline__ float load(const uint16_t* p, int64_t i) {
    return __uint_as_float(static_cast<uint32_t>(p[i]) << 16);
  }
  static __device__ __forceinline__ void store(uint16_t* p, int64_t i, float v) { p[i] = f32_to_bf16_rne(v); }
};

// Eight consecutive source elements as floats (16-byte loads where the type allows).
template <int S>
__device__ __forceinline__ void load8(const typename Elem<S>::type* src, int64_t i, float (&v)[8]) {
  if constexpr (S == TLHIP_T_F32) {
    const float4 a = *reinterpret_cast<const float4*>(src + i), b = *reinterpret_cast<const float4*>(src + i + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
    const uint4 r = *reinterpret_cast<const uint4*>(src + i);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int k = 0; k < 4; k++) {
      if constexpr (S == TLHIP_T_F16) {
        v[2 * k] = f16_bits_to_f32(w[k] & 0xffffu);
        v[2 * k + 1] = f16_bits_to_f32(w[k] >> 16);
      } else {
        v[2 * k] = bf16_lo(w[k]);
        v[2 * k + 1] = bf16_hi(w[k]);
      }
    }
  }
}

// ---- dst[i] = narrow(widen(src[i])): same layout, other element type ---------------------
template <int S, int T>
__global__ __launch_bounds__(256) void convert_kernel(const typename Elem<S>::type* __restrict__ src,
                                                      typename Elem<T>::type* __restrict__ dst, int64_t n) {
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 8;
  if (i + 8 <= n) {
    float v[8];
    load8<S>(src, i, v);
    if constexpr (T == TLHIP_T_F32) {
      *reinterpret_cast<float4*>(dst + i) = make_float4(v[0], v[1], v[2], v[3]);
      *reinterpret_cast<float4*>(dst + i + 4) = make_float4(v[4], v[5], v[6], v[7]);
    } else {
      uint32_t w[4];
#pragma unroll
      for (int k = 0; k < 4; k++)
        w[k] = static_cast<uint32_t>(f32_to_bf16_rne(v[2 * k])) |
               (static_cast<uint32_t>(f32_to_bf16_rne(v[2 * k + 1])) << 16);
      *reinterpret_cast<uint4*>(dst + i) = make_uint4(w[0], w[1], w[2], w[3]);
    }
  } else {
    for (int64_t j = i; j < n; j++) Elem<T>::store(dst, j, Elem<S>::load(src, j));
  }
}

// ---- dst[c * ld + col_base + r] = src[r * cols + c]: file rows [out, in] -> [K, N] -------------
// 64 x 64 tiles through LDS so that both sides move whole cache lines.
template <int S, int T>
__global__ __launch_bounds__(256) void convert_transpose_kernel(
    const typename Elem<S>::type* __restrict__ src, typename Elem<T>::type* __restrict__ dst,
    int64_t rows, int64_t cols, int64_t ld, int64_t col_base) {
  __shared__ float tile[64][65];
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * 64, c0 = static_cast<int64_t>(blockIdx.x) * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;   // 64 x 4
  for (int j = ty; j < 64; j += 4) {
    const int64_t r = r0 + j, c = c0 + tx;
    if (r < rows && c < cols) tile[j][tx] = Elem<S>::load(src, r * cols + c);
  }
  __syncthreads();
  for (int j = ty; j < 64; j += 4) {
    const int64_t c = c0 + j, r = r0 + tx;   // output row = source column
    if (r < rows && c < cols) Elem<T>::store(dst, c * ld + col_base + r, tile[tx][j]);
  }
}

// ---- int4 group quantiser (array.h:703-742 on the widened rows) ----------------------------
// One thread owns one group of 32 consecutive weights of a row: scale = max(1e-8, maxabs) / 7,
// q = clamp(lround(w / scale), -8, 7), stored nibble q + 8, even k in the low nibble. Rows
// are contiguous on both sides, so group t reads elements [32 t, 32 t + 32) and writes
// packed bytes [16 t, 16 t + 16) and scale t.
template <int S>
__global__ __launch_bounds__(256) void quantize_q4_kernel(const typename Elem<S>::type* __restrict__ src,
                                                          uint4* __restrict__ packed,
                                                          float* __restrict__ scales, int64_t groups) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (t >= groups) return;
  float w[32];
#pragma unroll
  for (int k = 0; k < 4; k++) {
    float v[8];
    load8<S>(src, t * 32 + k * 8, v);
#pragma unroll
    for (int j = 0; j < 8; j++) w[k * 8 + j] = v[j];
  }
  float maxabs = 1e-8f;
#pragma unroll
  for (int k = 0; k < 32; k++) {
    const float a = fabsf(w[k]);
    if (a > maxabs) maxabs = a;
  }
  const float scale = __fdiv_rn(maxabs, 7.0f);
  uint32_t out[4] = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int k = 0; k < 32; k++) {
    float q = roundf(__fdiv_rn(w[k], scale));   // half away from zero, like lround
    q = fminf(fmaxf(q, -8.0f), 7.0f);
    const uint32_t nib = static_cast<uint32_t>(static_cast<int>(q) + 8);
    out[k >> 3] |= nib << ((k & 7) * 4);        // bytes in memory order, even k low
  }
  packed[t] = make_uint4(out[0], out[1], out[2], out[3]);
  scales[t] = scale;
}

// out[j] = widen(table[tok][j]) for an f16 embedding table, tok read from the device
// (the row gather of bench/cuda/qwen_model.h:531-540 without the host in between).
__global__ __launch_bounds__(256) void embed_gather_f16_kernel(const uint16_t* __restrict__ table,
                                                               const int* __restrict__ d_token,
                                                               float* __restrict__ out, int hidden,
                                                               int vocab) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= hidden) return;
  int tok = *d_token;
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  out[j] = f16_bits_to_f32(table[static_cast<size_t>(tok) * hidden + j]);
}

static bool known_type(int t) { return t == TLHIP_T_F32 || t == TLHIP_T_F16 || t == TLHIP_T_BF16; }

}  // namespace tlhip

using namespace tlhip;

// (S, T) dispatch: sources f32 / f16 / bf16, destinations f32 / bf16
#define TLHIP_CONVERT_DISPATCH(S_, T_, CALL)                                             \
  do {                                                                                   \
    if ((T_) == TLHIP_T_F32) {                                                           \
      if ((S_) == TLHIP_T_F32) { CALL(TLHIP_T_F32, TLHIP_T_F32); }                       \
      else if ((S_) == TLHIP_T_F16) { CALL(TLHIP_T_F16, TLHIP_T_F32); }                  \
      else { CALL(TLHIP_T_BF16, TLHIP_T_F32); }                                          \
    } else {                                                                             \
      if ((S_) == TLHIP_T_F32) { CALL(TLHIP_T_F32, TLHIP_T_BF16); }                      \
      else if ((S_) == TLHIP_T_F16) { CALL(TLHIP_T_F16, TLHIP_T_BF16); }                 \
      else { CALL(TLHIP_T_BF16, TLHIP_T_BF16); }                                         \
    }                                                                                    \
  } while (0)

extern "C" {

int tlhip_convert(const void* src, int src_type, void* dst, int dst_type, int64_t n) {
  TLHIP_REQUIRE_READY();
  if (!src || !dst) return fail(TLHIP_EINVAL, "tlhip_convert: null pointer");
  if (!known_type(src_type) || (dst_type != TLHIP_T_F32 && dst_type != TLHIP_T_BF16))
    return fail(TLHIP_EUNSUPPORTED, "tlhip_convert: element types %d -> %d", src_type, dst_type);
  if (n <= 0) return fail(TLHIP_EINVAL, "tlhip_convert: n must be positive");
  if (!aligned16(src) || !aligned16(dst)) return fail(TLHIP_EINVAL, "tlhip_convert: operands must be 16-byte aligned");
  const int64_t blocks = (n + 2047) / 2048;
  if (blocks > 0x7fffffff) return fail(TLHIP_EUNSUPPORTED, "tlhip_convert: too many elements");
#define CALL(S, T)                                                                              \
  convert_kernel<S, T><<<dim3((unsigned)blocks), dim3(256), 0, ctx().stream>>>(                 \
      static_cast<const Elem<S>::type*>(src), static_cast<Elem<T>::type*>(dst), n)
  TLHIP_CONVERT_DISPATCH(src_type, dst_type, CALL);
#undef CALL
  TLHIP_CHECK_LAUNCH(TLHIP_C_CONVERT);
}

int tlhip_convert_transpose(const void* src, int src_type, void* dst, int dst_type, int64_t rows,
                            int64_t cols, int64_t ld_dst, int64_t col_base) {
  TLHIP_REQUIRE_READY();
  if (!src || !dst) return fail(TLHIP_EINVAL, "tlhip_convert_transpose: null pointer");
  if (!known_type(src_type) || (dst_type != TLHIP_T_F32 && dst_type != TLHIP_T_BF16))
    return fail(TLHIP_EUNSUPPORTED, "tlhip_convert_transpose: element types %d -> %d", src_type, dst_type);
  if (rows <= 0 || cols <= 0 || col_base < 0 || col_base + rows > ld_dst)
    return fail(TLHIP_EINVAL, "tlhip_convert_transpose: need rows, cols > 0 and col_base + rows <= ld_dst");
  const int64_t gx = (cols + 63) / 64, gy = (rows + 63) / 64;
  if (gx > 0x7fffffff || gy > 65535) return fail(TLHIP_EUNSUPPORTED, "tlhip_convert_transpose: shape too large");
#define CALL(S, T)                                                                              \
  convert_transpose_kernel<S, T><<<dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, ctx().stream>>>( \
      static_cast<const Elem<S>::type*>(src), static_cast<Elem<T>::type*>(dst), rows, cols, ld_dst, col_base)
  TLHIP_CONVERT_DISPATCH(src_type, dst_type, CALL);
#undef CALL
  TLHIP_CHECK_LAUNCH(TLHIP_C_CONVERT);
}

int tlhip_quantize_q4(const void* src, int src_type, void* packed, void* scales, int64_t rows,
                      int64_t K, int64_t group) {
  TLHIP_REQUIRE_READY();
  if (!src || !packed || !scales) return fail(TLHIP_EINVAL, "tlhip_quantize_q4: null pointer");
  if (!known_type(src_type)) return fail(TLHIP_EUNSUPPORTED, "tlhip_quantize_q4: element type %d", src_type);
  if (group != 32) return fail(TLHIP_EUNSUPPORTED, "tlhip_quantize_q4: group must be 32");   // types.h:20
  if (rows <= 0 || K <= 0 || K % 32 != 0) return fail(TLHIP_EINVAL, "tlhip_quantize_q4: need rows > 0, K a positive multiple of 32");
  if (!aligned16(src) || !aligned16(packed) || (reinterpret_cast<uintptr_t>(scales) & 3u))
    return fail(TLHIP_EINVAL, "tlhip_quantize_q4: src and packed must be 16-byte aligned, scales 4-byte");
  const int64_t groups = rows * (K / 32);
  const int64_t blocks = (groups + 255) / 256;
  if (blocks > 0x7fffffff) return fail(TLHIP_EUNSUPPORTED, "tlhip_quantize_q4: too many groups");
  uint4* pk = static_cast<uint4*>(packed);
  float* sc = static_cast<float*>(scales);
  const dim3 grid((unsigned)blocks), block(256);
  if (src_type == TLHIP_T_F32)
    quantize_q4_kernel<TLHIP_T_F32><<<grid, block, 0, ctx().stream>>>(static_cast<const float*>(src), pk, sc, groups);
  else if (src_type == TLHIP_T_F16)
    quantize_q4_kernel<TLHIP_T_F16><<<grid, block, 0, ctx().stream>>>(static_cast<const uint16_t*>(src), pk, sc, groups);
  else
    quantize_q4_kernel<TLHIP_T_BF16><<<grid, block, 0, ctx().stream>>>(static_cast<const uint16_t*>(src), pk, sc, groups);
  TLHIP_CHECK_LAUNCH(TLHIP_C_QUANTIZE_Q4);
}

int tlhip_embed_gather_f16(const void* table, const void* d_token, void* out, int64_t hidden,
                           int64_t vocab) {
  TLHIP_REQUIRE_READY();
  if (!table || !d_token || !out) return fail(TLHIP_EINVAL, "tlhip_embed_gather_f16: null pointer");
  if (hidden <= 0 || vocab <= 0 || hidden > 0x7fffffff || vocab > 0x7fffffff)
    return fail(TLHIP_EINVAL, "tlhip_embed_gather_f16: bad shape");
  embed_gather_f16_kernel<<<dim3((unsigned)((hidden + 255) / 256)), dim3(256), 0, ctx().stream>>>(
      static_cast<const uint16_t*>(table), static_cast<const int*>(d_token), static_cast<float*>(out),
      (int)hidden, (int)vocab);
  hipError_t e_ = hipGetLastError();
  if (e_ != hipSuccess) return hip_fail(e_, "kernel launch");
  return TLHIP_OK;
}

}  // extern "C"
