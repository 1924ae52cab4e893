// General f32 GEMM of the tl::gpu seam on the fp32 matrix pipe:
//   C[M,N] = (op(A) . op(B)) * scale + offset,  op = identity or transposed view
// (cuda.h:1408-1460 `gemm`: lda / ldb row strides, ta / tb read a transposed view in
// place). This is what `array::dot` issues for rank-2 f32 operands with M > 1 (prompt-side
// matmuls of the array path, training-style graphs); the decode path never reaches it.
//
// v_mfma_f32_32x32x2_f32 multiplies f32 by f32 exactly and accumulates in fp32, so the
// result differs from the reference's FMA loops in summation order only. One instruction
// consumes ONE float per lane per operand - lane l supplies A[l % 32][l / 32] and
// B[l / 32][l % 32] - so both tiles sit in LDS k-major (As[k][m], Bs[k][n]): the 32 lanes of a
// half-wave then read 32 consecutive floats, conflict-free. An operand whose k index is
// contiguous in memory ([m][k] A, [n][k] B) is transposed on its way into LDS.
//
// 4 wavefronts (2 x 2) per block, 128 x 128 block tile, 64 x 64 per wavefront (2 x 2 MFMA
// tiles, 64 accumulator registers), K slabs of 16; the next slab's global loads are in
// flight while the current one is multiplied.
#include "common.hpp"

namespace tlhip {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kSgBM = 128, kSgBN = 128, kSgBK = 16, kSgPad = 4;

// One 128 x 16 operand tile, moved global -> registers -> LDS (k-major).
//   KC = true : k is the contiguous index in memory  (element (r, k) at base[r * ld + k])
//   KC = false: the tile's row index is contiguous   (element (r, k) at base[k * ld + r])
// r = row of A (m) or column of B (n). `fast` (block-uniform): the whole tile is inside the
// matrix and 16-byte loads are aligned; otherwise every element is bounds-checked.
template <bool KC>
struct TileMover {
  float4 reg[2];
  __device__ __forceinline__ void load(const float* __restrict__ base, int64_t ld, int r0, int k0, int R,
                                       int K, bool fast, int tid) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int idx = tid + i * 256;
      if constexpr (KC) {
        const int r = idx >> 2, c4 = (idx & 3) * 4;          // 4 float4 along k per row
        const float* p = base + (int64_t)(r0 + r) * ld + k0 + c4;
        if (fast) {
          reg[i] = *reinterpret_cast<const float4*>(p);
        } else {
          float v[4];
#pragma unroll
          for (int j = 0; j < 4; j++) v[j] = (r0 + r < R && k0 + c4 + j < K) ? p[j] : 0.f;
          reg[i] = make_float4(v[0], v[1], v[2], v[3]);
        }
      } else {
        const int kk = idx >> 5, r4 = (idx & 31) * 4;        // 32 float4 along r per k row
        const float* p = base + (int64_t)(k0 + kk) * ld + r0 + r4;
        if (fast) {
          reg[i] = *reinterpret_cast<const float4*>(p);
        } else {
          float v[4];
#pragma unroll
          for (int j = 0; j < 4; j++) v[j] = (k0 + kk < K && r0 + r4 + j < R) ? p[j] : 0.f;
          reg[i] = make_float4(v[0], v[1], v[2], v[3]);
        }
      }
    }
  }
  __device__ __forceinline__ void store(float (*tile)[kSgBM + kSgPad], int tid) const {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int idx = tid + i * 256;
      if constexpr (KC) {
        const int r = idx >> 2, c4 = (idx & 3) * 4;
        tile[c4 + 0][r] = reg[i].x;
        tile[c4 + 1][r] = reg[i].y;
        tile[c4 + 2][r] = reg[i].z;
        tile[c4 + 3][r] = reg[i].w;
      } else {
        const int kk = idx >> 5, r4 = (idx & 31) * 4;
        *reinterpret_cast<float4*>(&tile[kk][r4]) = reg[i];
      }
    }
  }
};

// TA / TB as the seam passes them: TA = 0 means A is [M][K] (k contiguous), TA = 1 means the
// buffer holds [K][M]; TB = 0 means B is [K][N] (n contiguous), TB = 1 means [N][K].
template <int TA, int TB>
__global__ __launch_bounds__(256, 2) void sgemm_mfma_kernel(const float* __restrict__ A, int64_t lda,
                                                           const float* __restrict__ B, int64_t ldb,
                                                           float* __restrict__ C, int M, int N, int K,
                                                           float scale, float offset, int epi,
                                                           int aligned, int kchunk) {
  __shared__ __attribute__((aligned(16))) float As[kSgBK][kSgBM + kSgPad];
  __shared__ __attribute__((aligned(16))) float Bs[kSgBK][kSgBN + kSgPad];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * kSgBM, n0 = blockIdx.x * kSgBN;
  const bool inside = aligned && m0 + kSgBM <= M && n0 + kSgBN <= N;
  // gridDim.z > 1 is split-K: slice z takes K range [z * kchunk, (z + 1) * kchunk) (kchunk a
  // multiple of the slab) and writes its partial product, without the epilogue, to
  // C + z * M * N, a scratch area that sgemm_sum_kernel adds up in slice order.
  const int kbeg = blockIdx.z * kchunk;
  K = min(K, kbeg + kchunk);
  C += (size_t)blockIdx.z * M * N;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  TileMover<TA == 0> ma;   // A: k contiguous unless transposed
  TileMover<TB != 0> mb;   // B: k contiguous only when transposed
  ma.load(A, lda, m0, kbeg, M, K, inside && kbeg + kSgBK <= K, tid);
  mb.load(B, ldb, n0, kbeg, N, K, inside && kbeg + kSgBK <= K, tid);
  for (int k0 = kbeg; k0 < K; k0 += kSgBK) {
    __syncthreads();   // the previous slab has been consumed
    ma.store(As, tid);
    mb.store(Bs, tid);
    __syncthreads();
    if (k0 + kSgBK < K) {
      const bool fast = inside && k0 + 2 * kSgBK <= K;
      ma.load(A, lda, m0, k0 + kSgBK, M, K, fast, tid);
      mb.load(B, ldb, n0, k0 + kSgBK, N, K, fast, tid);
    }
    const int kh = lane >> 5, l32 = lane & 31;
#pragma unroll
    for (int s = 0; s < kSgBK / 2; s++) {
      float a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; i++) a[i] = As[2 * s + kh][wm * 64 + i * 32 + l32];
#pragma unroll
      for (int j = 0; j < 2; j++) b[j] = Bs[2 * s + kh][wn * 64 + j * 32 + l32];
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
  }

  // acc[v] of lane l: row 8 * (v / 4) + 4 * (l / 32) + v % 4, column l % 32 of the 32 x 32 tile
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int gn = n0 + wn * 64 + j * 32 + (lane & 31);
      if (gn >= N) continue;
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int gm = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (gm < M) {
          const float r = acc[i][j][v];
          // separate multiply and add, like the CPU loops (array.h:1879, 2223)
          C[(size_t)gm * N + gn] = epi ? add_rn(mul_rn(r, scale), offset) : r;
        }
      }
    }
}

// C[i] = (sum over slices of part[s][i]) * scale + offset, slices in ascending order.
__global__ __launch_bounds__(256) void sgemm_sum_kernel(const float* __restrict__ part, float* __restrict__ C,
                                                        size_t n, int S, float scale, float offset, int epi) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float a = part[i];
  for (int s = 1; s < S; s++) a += part[(size_t)s * n + i];
  C[i] = epi ? add_rn(mul_rn(a, scale), offset) : a;
}

// Launches the matrix-pipe GEMM; the caller has checked the arguments.
int launch_sgemm_mfma(const float* pa, int64_t lda, int ta, const float* pb, int64_t ldb, int tb, float* pc,
                      int M, int N, int K, float scale, float offset, int epi) {
  const int64_t tiles = (int64_t)((N + kSgBN - 1) / kSgBN) * ((M + kSgBM - 1) / kSgBM);
  // Too few tiles to fill the chip: split K over gridDim.z (at least 256 of K per slice) into
  // scratch parts that are summed in a fixed order - deterministic, no atomics.
  int S = 1;
  if (tiles < ctx().cus) {
    S = (int)((2 * (int64_t)ctx().cus + tiles - 1) / tiles);
    if (S > 8) S = 8;
    while (S > 1 && K / S < 256) S--;
  }
  int kchunk = K;
  float* dst = pc;
  if (S > 1) {
    kchunk = ((K + S - 1) / S + kSgBK - 1) / kSgBK * kSgBK;
    S = (K + kchunk - 1) / kchunk;
    dst = S > 1 ? static_cast<float*>(scratch((size_t)S * M * N * sizeof(float))) : pc;
    if (!dst) return fail(TLHIP_ENOMEM, "tlhip_gemm: no scratch for %d K-splits", S);
  }
  const dim3 grid((unsigned)((N + kSgBN - 1) / kSgBN), (unsigned)((M + kSgBM - 1) / kSgBM), (unsigned)S);
  // 16-byte loads need aligned bases and row strides that keep every row aligned
  const int aligned = aligned16(pa) && aligned16(pb) && (lda % 4) == 0 && (ldb % 4) == 0;
  hipStream_t st = ctx().stream;
  const int kepi = S > 1 ? 0 : epi;   // the part sum applies the epilogue when K is split
#define TLHIP_SGEMM(TA_, TB_)                                                                         \
  sgemm_mfma_kernel<TA_, TB_><<<grid, dim3(256), 0, st>>>(pa, lda, pb, ldb, dst, M, N, K, scale, offset, \
                                                          kepi, aligned, kchunk)
  if (!ta && !tb) TLHIP_SGEMM(0, 0);
  else if (!ta && tb) TLHIP_SGEMM(0, 1);
  else if (ta && !tb) TLHIP_SGEMM(1, 0);
  else TLHIP_SGEMM(1, 1);
#undef TLHIP_SGEMM
  if (S > 1) {
    const size_t n = (size_t)M * N;
    sgemm_sum_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st>>>(dst, pc, n, S, scale, offset, epi);
  }
  return 0;
}

}  // namespace tlhip
