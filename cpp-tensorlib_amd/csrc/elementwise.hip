// Elementwise maps, rank-2 broadcast, last-axis row ops and the general f32
// GEMM of the array seam. All are tiny next to the GEMVs; they exist so that
// array-level compositions (rmsnorm, swiglu, bias adds) never leave the device.
#include "common.hpp"

namespace tlhip {

template <int OP>
__device__ __forceinline__ float bin_op(float a, float b) {
  if constexpr (OP == TLHIP_ADD) return a + b;
  else if constexpr (OP == TLHIP_SUB) return a - b;
  else if constexpr (OP == TLHIP_MUL) return a * b;
  else if constexpr (OP == TLHIP_DIV) return a / b;
  else return powf(a, b);
}

template <int OP>
__device__ __forceinline__ float un_op(float a) {
  if constexpr (OP == TLHIP_EXP) return expf(a);
  else if constexpr (OP == TLHIP_LOG) return logf(a);
  else if constexpr (OP == TLHIP_SQRT) return sqrtf(a);
  else if constexpr (OP == TLHIP_SIGMOID) return 1.0f / (1.0f + expf(-a));
  else if constexpr (OP == TLHIP_RELU) return a > 0.0f ? a : 0.0f;
  else if constexpr (OP == TLHIP_RECIP) return 1.0f / a;
  else return a;
}

// out = f(...)*scale + offset with separate multiply and add, like the CPU
// loops (array.h:1879, 2223); identity epilogues leave the value untouched.
__device__ __forceinline__ float epilogue(float v, float scale, float offset) {
  return add_rn(mul_rn(v, scale), offset);
}

template <int OP>
__global__ __launch_bounds__(256) void binary_kernel(const float* __restrict__ a,
                                                     const float* __restrict__ b,
                                                     float* __restrict__ out, int64_t n,
                                                     float scale, float offset, int epi) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    float v = bin_op<OP>(a[i], b[i]);
    out[i] = epi ? epilogue(v, scale, offset) : v;
  }
}

template <int OP>
__global__ __launch_bounds__(256) void bcast_kernel(const float* __restrict__ a, int64_t ars,
                                                    int64_t acs, const float* __restrict__ b,
                                                    int64_t brs, int64_t bcs,
                                                    float* __restrict__ out, int64_t m, int64_t n,
                                                    float scale, float offset, int epi) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = m * n, stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += stride) {
    const int64_t r = i / n, c = i - r * n;
    float v = bin_op<OP>(a[r * ars + c * acs], b[r * brs + c * bcs]);
    out[i] = epi ? epilogue(v, scale, offset) : v;
  }
}

template <int OP>
__global__ __launch_bounds__(256) void unary_kernel(const float* __restrict__ a,
                                                    float* __restrict__ out, int64_t n,
                                                    float scale, float offset, int epi) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    float v = un_op<OP>(a[i]);
    out[i] = epi ? epilogue(v, scale, offset) : v;
  }
}

// one block per row
template <bool MAX>
__global__ __launch_bounds__(256) void row_reduce_kernel(const float* __restrict__ in,
                                                         float* __restrict__ out, int64_t cols,
                                                         float scale, float offset, int epi) {
  __shared__ float red[4];
  const float* src = in + (size_t)blockIdx.x * cols;
  float acc = MAX ? -INFINITY : 0.0f;
  for (int64_t c = threadIdx.x; c < cols; c += 256) {
    float v = src[c];
    acc = MAX ? fmaxf(acc, v) : acc + v;
  }
  acc = MAX ? wave_max(acc) : wave_sum(acc);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float v = MAX ? fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]))
                  : ((red[0] + red[1]) + red[2]) + red[3];
    out[blockIdx.x] = epi ? epilogue(v, scale, offset) : v;
  }
}

__global__ __launch_bounds__(256) void softmax_kernel(const float* __restrict__ in,
                                                      float* __restrict__ out, int64_t cols) {
  __shared__ float red[4];
  const float* src = in + (size_t)blockIdx.x * cols;
  float* dst = out + (size_t)blockIdx.x * cols;
  float m = -INFINITY;
  for (int64_t c = threadIdx.x; c < cols; c += 256) m = fmaxf(m, src[c]);
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float s = 0.0f;
  for (int64_t c = threadIdx.x; c < cols; c += 256) {
    float e = expf(src[c] - m);
    dst[c] = e;
    s += e;
  }
  s = block_sum<4>(s, red);
  for (int64_t c = threadIdx.x; c < cols; c += 256) dst[c] = dst[c] / s;
}

// General f32 GEMM with transposed-view operands and an affine epilogue, VALU form:
// 64x64 tile, 16-wide K slab through LDS, 4x4 outputs per thread. Serves the small
// products; from 128 x 128 outputs on the matrix-pipe kernel of sgemm.hip takes over.
__global__ __launch_bounds__(256) void sgemm_kernel(const float* __restrict__ A, int64_t lda,
                                                    int ta, const float* __restrict__ B,
                                                    int64_t ldb, int tb, float* __restrict__ C,
                                                    int M, int N, int K, float scale,
                                                    float offset, int epi) {
  __shared__ float As[16][64 + 1];
  __shared__ float Bs[16][64 + 1];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += 16) {
    for (int i = threadIdx.x; i < 64 * 16; i += 256) {
      const int kk = i & 15, r = i >> 4;
      const int gm = m0 + r, gk = k0 + kk;
      As[kk][r] = (gm < M && gk < K) ? (ta ? A[(size_t)gk * lda + gm] : A[(size_t)gm * lda + gk]) : 0.f;
      const int gn = n0 + r;
      Bs[kk][r] = (gn < N && gk < K) ? (tb ? B[(size_t)gn * ldb + gk] : B[(size_t)gk * ldb + gn]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; kk++) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; i++) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; j++) bv[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int gn = n0 + tx * 4 + j;
      if (gn < N) C[(size_t)gm * N + gn] = epi ? epilogue(acc[i][j], scale, offset) : acc[i][j];
    }
  }
}

int launch_sgemm_mfma(const float* pa, int64_t lda, int ta, const float* pb, int64_t ldb, int tb, float* pc,
                      int M, int N, int K, float scale, float offset, int epi);   // sgemm.hip

static unsigned grid1d(int64_t n) {
  int64_t b = (n + 255) / 256;
  if (b > 65535 * 16) b = 65535 * 16;
  return (unsigned)(b > 0 ? b : 1);
}

}  // namespace tlhip

using namespace tlhip;

extern "C" {

int tlhip_binary(int op, const void* a, int64_t a_off, const void* b, int64_t b_off, void* out,
                 int64_t out_off, int64_t n, float scale, float offset) {
  TLHIP_REQUIRE_READY();
  if (!a || !b || !out || n < 0) return fail(TLHIP_EINVAL, "tlhip_binary: bad arguments");
  if (n == 0) return TLHIP_OK;
  const float* pa = reinterpret_cast<const float*>(at(a, a_off));
  const float* pb = reinterpret_cast<const float*>(at(b, b_off));
  float* po = reinterpret_cast<float*>(at(out, out_off));
  const int epi = !(scale == 1.0f && offset == 0.0f);
  hipStream_t s = ctx().stream;
  dim3 g(grid1d(n)), blk(256);
  switch (op) {
    case TLHIP_ADD: binary_kernel<TLHIP_ADD><<<g, blk, 0, s>>>(pa, pb, po, n, scale, offset, epi); break;
    case TLHIP_SUB: binary_kernel<TLHIP_SUB><<<g, blk, 0, s>>>(pa, pb, po, n, scale, offset, epi); break;
    case TLHIP_MUL: binary_kernel<TLHIP_MUL><<<g, blk, 0, s>>>(pa, pb, po, n, scale, offset, epi); break;
    case TLHIP_DIV: binary_kernel<TLHIP_DIV><<<g, blk, 0, s>>>(pa, pb, po, n, scale, offset, epi); break;
    case TLHIP_POW: binary_kernel<TLHIP_POW><<<g, blk, 0, s>>>(pa, pb, po, n, scale, offset, epi); break;
    default: return fail(TLHIP_EUNSUPPORTED, "tlhip_binary: op %d", op);
  }
  TLHIP_CHECK_LAUNCH(TLHIP_C_BINARY);
}

int tlhip_binary_bcast(int op, const void* a, int64_t a_off, int64_t ars, int64_t acs,
                       const void* b, int64_t b_off, int64_t brs, int64_t bcs, void* out,
                       int64_t out_off, int64_t m, int64_t n, float scale, float offset) {
  TLHIP_REQUIRE_READY();
  if (!a || !b || !out || m < 0 || n < 0) return fail(TLHIP_EINVAL, "tlhip_binary_bcast: bad arguments");
  if (m * n == 0) return TLHIP_OK;
  const float* pa = reinterpret_cast<const float*>(at(a, a_off));
  const float* pb = reinterpret_cast<const float*>(at(b, b_off));
  float* po = reinterpret_cast<float*>(at(out, out_off));
  const int epi = !(scale == 1.0f && offset == 0.0f);
  hipStream_t s = ctx().stream;
  dim3 g(grid1d(m * n)), blk(256);
#define TLHIP_BC(OP) bcast_kernel<OP><<<g, blk, 0, s>>>(pa, ars, acs, pb, brs, bcs, po, m, n, scale, offset, epi)
  switch (op) {
    case TLHIP_BADD: TLHIP_BC(TLHIP_ADD); break;
    case TLHIP_BSUB: TLHIP_BC(TLHIP_SUB); break;
    case TLHIP_BMUL: TLHIP_BC(TLHIP_MUL); break;
    case TLHIP_BDIV: TLHIP_BC(TLHIP_DIV); break;
    case TLHIP_BPOW: TLHIP_BC(TLHIP_POW); break;
    default: return fail(TLHIP_EUNSUPPORTED, "tlhip_binary_bcast: op %d", op);
  }
#undef TLHIP_BC
  TLHIP_CHECK_LAUNCH(TLHIP_C_BCAST);
}

int tlhip_unary(int op, const void* a, int64_t a_off, void* out, int64_t out_off, int64_t n,
                float scale, float offset) {
  TLHIP_REQUIRE_READY();
  if (!a || !out || n < 0) return fail(TLHIP_EINVAL, "tlhip_unary: bad arguments");
  if (n == 0) return TLHIP_OK;
  const float* pa = reinterpret_cast<const float*>(at(a, a_off));
  float* po = reinterpret_cast<float*>(at(out, out_off));
  // an `affine` node IS its epilogue (array.h:2051-2062): always applied
  const int epi = op == TLHIP_AFFINE ? 1 : !(scale == 1.0f && offset == 0.0f);
  hipStream_t s = ctx().stream;
  dim3 g(grid1d(n)), blk(256);
#define TLHIP_UN(OP) unary_kernel<OP><<<g, blk, 0, s>>>(pa, po, n, scale, offset, epi)
  switch (op) {
    case TLHIP_EXP: TLHIP_UN(TLHIP_EXP); break;
    case TLHIP_LOG: TLHIP_UN(TLHIP_LOG); break;
    case TLHIP_SQRT: TLHIP_UN(TLHIP_SQRT); break;
    case TLHIP_SIGMOID: TLHIP_UN(TLHIP_SIGMOID); break;
    case TLHIP_RELU: TLHIP_UN(TLHIP_RELU); break;
    case TLHIP_AFFINE: TLHIP_UN(TLHIP_AFFINE); break;
    case TLHIP_RECIP: TLHIP_UN(TLHIP_RECIP); break;
    default: return fail(TLHIP_EUNSUPPORTED, "tlhip_unary: op %d", op);
  }
#undef TLHIP_UN
  TLHIP_CHECK_LAUNCH(TLHIP_C_UNARY);
}

int tlhip_row_op(int op, const void* in, int64_t in_off, void* out, int64_t out_off, int64_t rows,
                 int64_t cols, float scale, float offset) {
  TLHIP_REQUIRE_READY();
  if (!in || !out || rows < 0 || cols < 0) return fail(TLHIP_EINVAL, "tlhip_row_op: bad arguments");
  if (rows == 0) return TLHIP_OK;
  if (cols == 0) return fail(TLHIP_EUNSUPPORTED, "tlhip_row_op: empty rows");
  if (rows > 0x7fffffff) return fail(TLHIP_EUNSUPPORTED, "tlhip_row_op: too many rows");
  const float* pi = reinterpret_cast<const float*>(at(in, in_off));
  float* po = reinterpret_cast<float*>(at(out, out_off));
  const int epi = !(scale == 1.0f && offset == 0.0f);
  hipStream_t s = ctx().stream;
  dim3 g((unsigned)rows), blk(256);
  switch (op) {
    case TLHIP_ROW_SUM: row_reduce_kernel<false><<<g, blk, 0, s>>>(pi, po, cols, scale, offset, epi); break;
    case TLHIP_ROW_MAX: row_reduce_kernel<true><<<g, blk, 0, s>>>(pi, po, cols, scale, offset, epi); break;
    case TLHIP_SOFTMAX: softmax_kernel<<<g, blk, 0, s>>>(pi, po, cols); break;
    default: return fail(TLHIP_EUNSUPPORTED, "tlhip_row_op: op %d", op);
  }
  TLHIP_CHECK_LAUNCH(TLHIP_C_ROW_OP);
}

int tlhip_gemm(const void* a, int64_t a_off, int64_t lda, int ta, const void* b, int64_t b_off,
               int64_t ldb, int tb, void* out, int64_t out_off, int64_t m, int64_t n, int64_t k,
               float scale, float offset) {
  TLHIP_REQUIRE_READY();
  if (!a || !b || !out || m < 0 || n < 0 || k < 0) return fail(TLHIP_EINVAL, "tlhip_gemm: bad arguments");
  if (m == 0 || n == 0) return TLHIP_OK;
  if (m > 0x3fffffff || n > 0x3fffffff || k > 0x3fffffff)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm: dimension too large");
  const float* pa = reinterpret_cast<const float*>(at(a, a_off));
  const float* pb = reinterpret_cast<const float*>(at(b, b_off));
  float* po = reinterpret_cast<float*>(at(out, out_off));
  const int epi = !(scale == 1.0f && offset == 0.0f);
  if (m >= 128 && n >= 128 && k >= 16 && (m + 127) / 128 <= 65535) {
    const int rc = launch_sgemm_mfma(pa, lda, ta, pb, ldb, tb, po, (int)m, (int)n, (int)k, scale, offset, epi);
    if (rc != 0) return rc;
    TLHIP_CHECK_LAUNCH(TLHIP_C_GEMM);
  }
  dim3 g((unsigned)((n + 63) / 64), (unsigned)((m + 63) / 64));
  if (g.y > 65535) return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm: M too large for the grid");
  sgemm_kernel<<<g, dim3(256), 0, ctx().stream>>>(pa, lda, ta, pb, ldb, tb, po, (int)m, (int)n,
                                                  (int)k, scale, offset, epi);
  TLHIP_CHECK_LAUNCH(TLHIP_C_GEMM);
}

}  // extern "C"
