// Prompt-chunk GEMM over a PREPARED bf16 weight: C[M,N] = A[M,K] f32 . W[N,K]^T, on f16 operands
// copied global -> LDS without passing through registers.
//
// Why a second GEMM. Measured per K slab, gemm_bf16_nt_kernel (prefill.hip) is not bound by the
// matrix pipe: its 128 x 256 tile pulls 32 KB per slab through the CU's vector memory path, which
// moves about 45 bytes a clock for rows that are 64 or 128 bytes long and kilobytes apart, and it
// spends 100-140 vector ALU instructions per lane and slab on cutting activations into planes -
// together more clocks than the slab's MFMAs. Both costs are removed here by doing the work once,
// outside the loop:
//   * the weight is prepared when it is loaded (tlhip_gemm_f16w_prepare): every row times
//     2^ew[n], converted to f16 (a bf16 weight has 8 significant bits, an f16 holds 11; ew[n]
//     brings the row's largest magnitude into [2^14, 2^15), so every weight within 2^-29 of it
//     converts exactly and smaller ones carry an absolute error below 2^-40 of it), stored as the
//     LDS image of each (256 rows, 32 k) slab: 16 KB, rows already in the bank-conflict-free order
//     the fragment reads expect;
//   * the activations are cut once per call (a_image_kernel): row m times 2^ea[m], then TWO f16
//     terms, both rounded to nearest - a * 2^ea = hi + lo + r with |r| <= 2^-24 |a * 2^ea| where lo
//     is a normal f16 (<= 2^-39 of the row's largest where it is not): the accuracy of one fp32
//     rounding, from two MFMAs per product instead of the three of the bf16 split - again stored
//     as slab images, 32 KB per (256 rows, 32 k).
// The GEMM then has no vector ALU work and no address arithmetic in its loop: a slab is 48
// contiguous kilobytes, copied by 48 global_load_lds_dwordx4 (1 KB each, whole cache lines, no
// registers), six per wavefront. A block is eight wavefronts (4 x 2) on a 256 x 256 tile, 64 x 128
// per wavefront (128 x 256 and 32 x 128 where N is small), one block per CU, a ring of three slabs
// in LDS (144 KB), one barrier per slab; a copy has two slab times to land. Products of f16 are exact in fp32, the MFMA sums in fp32, and
// the result leaves as acc * 2^-(ea[m] + ew[n]), an exact scaling: the error is fp32 summation
// error plus one fp32-rounding-sized term per product, as in the reference's fp32 FMA loop
// (tensorlib_cuda.cu:509-519).
#include "gemm_shared.hpp"

namespace tlhip {
namespace f16t {

template <int N> struct Idx { static constexpr int value = N; };

constexpr int kBK = 32;                 // K slab
constexpr int kTile = 256;              // block tile, both ways
constexpr int kRing = 3;
constexpr int kRowBytes = kBK * 2;      // one row of one plane of a slab: 64 bytes, four 16-byte chunks
constexpr int kPlaneBytes = kTile * kRowBytes;          // 16 KB
constexpr int kAImage = 2 * kPlaneBytes;                // hi plane, lo plane
constexpr int kWImage = kPlaneBytes;

// Byte offset of 16-byte chunk `chunk` (8 k) of row `row` inside a plane image: the chunk index is
// XORed with bits of the row so that both the fragment reads (32 consecutive rows, same chunk) and
// linear copies spread over all LDS banks.
__host__ __device__ __forceinline__ int image_off(int row, int chunk) {
  return row * kRowBytes + ((chunk ^ ((row >> 1) & 3)) << 4);
}

// W row behind tile column `col` (0..255) of column tile `tn`; -1 past the edge. Gated: the tile's
// two 128-column strips are 64 gate features followed by the same features' up rows (ff rows
// further down), so that a lane of the GEMM holds both accumulators of a feature.
__host__ __device__ __forceinline__ int weight_row(bool gated, int tn, int col, int n, int ff) {
  if (gated) {
    const int j = col & 127, f = tn * 128 + (col >> 7) * 64 + (j & 63);
    return f < n ? f + (j >= 64 ? ff : 0) : -1;
  }
  const int r = tn * kTile + col;
  return r < n ? r : -1;
}

// One block per (column tile, slab): 256 rows x 32 k of the bf16 weight -> its f16 slab image.
// n = rows of W (plain) or features (gated: W has 2 * ff rows).
__global__ __launch_bounds__(256) void w_image_kernel(const uint16_t* __restrict__ W,
                                                      const int8_t* __restrict__ ew, char* __restrict__ img,
                                                      int n, int K, int ff, int gated) {
  const int tn = blockIdx.x, slab = blockIdx.y, nslab = gridDim.y, t = threadIdx.x;
  char* dst = img + ((size_t)tn * nslab + slab) * kWImage;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int col = (t >> 2) + 64 * i, c8 = t & 3;
    const int r = weight_row(gated != 0, tn, col, n, ff);
    frag16 v = {0u, 0u, 0u, 0u};
    if (r >= 0)
      v = bf16x8_to_f16(*reinterpret_cast<const frag16*>(W + (size_t)r * K + slab * kBK + c8 * 8), pow2f(ew[r]));
    *reinterpret_cast<frag16*>(dst + image_off(col, c8)) = v;
  }
}

// The exponents buffer a preparation fills, `exps`: [pad] int8 row exponents, [pad] uint16 counts,
// then the weight's own address and depth (pad = rows rounded up to 16). The count of a row is the
// number of its nonzero elements that, times 2^ew[row], lie below 2^-17 - their eight significant
// bits no longer fit above the f16 subnormal step of 2^-24, so the image holds them with an absolute
// error of up to 2^-25 - or 0xffff for a row that holds an infinity or a NaN. The products weigh the
// counts against the scale of each result and work out from W itself, exactly, the results in which
// those errors could show; that is why the buffer remembers where W is.
struct WHeader { const uint16_t* W; int64_t K; };
__host__ __device__ inline int64_t exps_pad(int64_t rows) { return (rows + 15) & ~int64_t(15); }
constexpr uint32_t kWSmallMax = 0xffffu;

__global__ __launch_bounds__(256) void w_range_kernel(const uint16_t* __restrict__ W, const int8_t* __restrict__ ew,
                                                      int K, uint16_t* __restrict__ counts, WHeader* __restrict__ hdr) {
  __shared__ uint32_t cnt[4], inf[4];
  const uint4* row = reinterpret_cast<const uint4*>(W + (size_t)blockIdx.x * K);
  const int lim = 127 - 17 - (int)ew[blockIdx.x];      // biased exponent below which an element is too small
  uint32_t small = 0;
  bool nonfinite = false;
  for (int i = threadIdx.x; i < K / 8; i += 256) {
    const uint4 v = row[i];
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const uint32_t m = (w[j] >> (16 * h)) & 0x7fffu;
        const int field = (int)(m >> 7);
        small += (m != 0u && field < lim) ? 1u : 0u;
        nonfinite |= field == 255;
      }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) small += (uint32_t)__shfl_xor((int)small, d);
  const bool anyinf = __any(nonfinite);
  if ((threadIdx.x & 63) == 0) { cnt[threadIdx.x >> 6] = small; inf[threadIdx.x >> 6] = anyinf ? 1u : 0u; }
  __syncthreads();
  if (threadIdx.x == 0) {
    small = cnt[0] + cnt[1] + cnt[2] + cnt[3];
    if (small > kWSmallMax - 1) small = kWSmallMax - 1;
    if (inf[0] | inf[1] | inf[2] | inf[3]) small = kWSmallMax;
    counts[blockIdx.x] = (uint16_t)small;
    if (blockIdx.x == 0) { hdr->W = W; hdr->K = K; }
  }
}

// One block per row of the activation images (rows past M are zero rows): the row's largest
// magnitude and from it the exponent e, then its two f16 terms into the slab images - one read of A.
// The row stays in registers between the two steps: up to kRowRegs float4s per thread.
// ea[m] = (e & 0xff) | (n << 8). n bounds the number of the row's nonzero elements that, scaled, lie
// below 2^-10 (more than 2^24 below the row's largest): their second term is an f16 subnormal with
// fewer than three bits left, so they are carried with an ABSOLUTE error of up to 2^-25 each (scaled)
// instead of a relative one. The bound is K as soon as the row's smallest nonzero magnitude is that
// small (a minimum costs less per element than a count, and this pass is bound by its memory
// traffic only just), 0 otherwise. The GEMM weighs n against the scale of each result and works
// out exactly the results for which those errors could show (gemm_f16t_kernel's epilogue). A row
// that holds an infinity or a NaN gets the largest n: all of its results are worked out exactly.
constexpr int kRowRegs = 32;            // K <= 256 * 4 * 32 = 32768
constexpr uint32_t kSmallMax = 0x7fffffu;
__global__ __launch_bounds__(256) void a_image_kernel(const float* __restrict__ A, int* __restrict__ ea,
                                                      char* __restrict__ img, int M, int K) {
  __shared__ uint32_t part[4], cnt[4];
  const int gm = blockIdx.x, t = threadIdx.x, nslab = K / kBK, k4 = K / 4;
  const int tm = gm / kTile, row = gm % kTile;
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  f32x4 v[kRowRegs];
  uint32_t mx = 0;
  if (gm < M) {
    const f32x4* src = reinterpret_cast<const f32x4*>(A + (size_t)gm * K);
#pragma unroll
    for (int i = 0; i < kRowRegs; i++) {
      const int q = t + 256 * i;
      v[i] = q < k4 ? src[q] : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int e = 0; e < 4; e++) mx = max(mx, __float_as_uint(v[i][e]) & 0x7fffffffu);
    }
  } else {
#pragma unroll
    for (int i = 0; i < kRowRegs; i++) v[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, d));
  if ((t & 63) == 0) part[t >> 6] = mx;
  __syncthreads();
  mx = max(max(part[0], part[1]), max(part[2], part[3]));
  const int e = row_exponent((int)(mx >> 23), mx == 0);
  const float s = pow2f(e);
  char* dst = img + (size_t)tm * nslab * kAImage;
  uint32_t least = 0xffffffffu;                    // smallest nonzero magnitude's bits, minus one
#pragma unroll
  for (int i = 0; i < kRowRegs; i++) {
    const int q = t + 256 * i;               // float4 q of the row: slab q / 8, 8-byte piece q % 8 of its 64 bytes
    if (q >= k4) break;
    const f32x4 x = v[i] * s;
#pragma unroll
    for (int j = 0; j < 4; j++) least = min(least, (__float_as_uint(x[j]) & 0x7fffffffu) - 1u);   // 0 wraps to the top
    uint32_t h01, l01, h23, l23;
    split2_f16(x[0], x[1], h01, l01);
    split2_f16(x[2], x[3], h23, l23);
    const int c4 = q & 7;
    char* o = dst + (size_t)(q >> 3) * kAImage + image_off(row, c4 >> 1) + (c4 & 1) * 8;
    *reinterpret_cast<uint2*>(o) = make_uint2(h01, h23);
    *reinterpret_cast<uint2*>(o + kPlaneBytes) = make_uint2(l01, l23);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) least = min(least, (uint32_t)__shfl_xor((int)least, d));
  if ((t & 63) == 0) cnt[t >> 6] = least;
  __syncthreads();
  if (t == 0 && gm < M) {
    least = min(min(cnt[0], cnt[1]), min(cnt[2], cnt[3]));
    uint32_t small = least < 0x3a800000u - 1u ? (uint32_t)K : 0u;          // 0 < |x| < 2^-10 somewhere
    if (mx >= 0x7f800000u) small = kSmallMax;
    ea[gm] = (e & 0xff) | (int)(small << 8);
  }
}

// The residual norm of a prompt chunk writing the activation image of its own output: what
// rmsnorm_wide_kernel<true, RV> (modelops.hip) followed by a_image_kernel would leave - the same
// arithmetic in the same order for s = x + parts, hout = (s / rms) w, and the same exponent, terms
// and small-element mark for the row of hout, which is still in registers - in one launch and
// without reading hout back. One block of 1024 threads per image row (rows past M are zero rows).
// x and xout may be the same buffer (a thread writes only what it has read).
template <int RV>
__global__ __launch_bounds__(1024) void rmsnorm_aimage_kernel(const float* x, const float* __restrict__ delta,
                                                              const float* __restrict__ w, float* xout,
                                                              float* __restrict__ hout, int n, float eps, int S,
                                                              size_t part_stride, int* __restrict__ ea,
                                                              char* __restrict__ img, int M) {
  __shared__ float red[16];
  __shared__ uint32_t part[16], cnt[16];
  const int gm = blockIdx.x, t = threadIdx.x, n4 = n >> 2, nslab = n / kBK;
  const int tm = gm / kTile, row = gm % kTile;
  float4 o[RV];
#pragma unroll
  for (int k = 0; k < RV; k++) o[k] = make_float4(0.f, 0.f, 0.f, 0.f);
  uint32_t mx = 0;
  if (gm < M) {                                    // (the same for every thread of the block)
    const size_t base = (size_t)gm * n;
    const float4* x4 = reinterpret_cast<const float4*>(x + base);
    const float4* d4 = reinterpret_cast<const float4*>(delta + base);
    const float4* w4 = reinterpret_cast<const float4*>(w);
    float4 v[RV], wv[RV];
    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < RV; k++) {
      const int i = t + k * 1024;
      if (i < n4) {
        v[k] = x4[i];
        wv[k] = w4[i];
        float4 d = d4[i];
        for (int sidx = 1; sidx < S; sidx++) {     // K-split parts, ascending
          const float4 e = d4[sidx * (part_stride >> 2) + i];
          d.x += e.x; d.y += e.y; d.z += e.z; d.w += e.w;
        }
        v[k].x += d.x; v[k].y += d.y; v[k].z += d.z; v[k].w += d.w;
      }
    }
#pragma unroll
    for (int k = 0; k < RV; k++) {
      const int i = t + k * 1024;
      if (i < n4) {
        reinterpret_cast<float4*>(xout + base)[i] = v[k];
        acc += (v[k].x * v[k].x + v[k].y * v[k].y) + (v[k].z * v[k].z + v[k].w * v[k].w);
      }
    }
    const float sum = block_sum<16>(acc, red);
    const float inv = 1.0f / sqrtf(sum * (1.0f / (float)n) + eps);
#pragma unroll
    for (int k = 0; k < RV; k++) {
      const int i = t + k * 1024;
      if (i < n4) {
        o[k].x = (v[k].x * inv) * wv[k].x; o[k].y = (v[k].y * inv) * wv[k].y;
        o[k].z = (v[k].z * inv) * wv[k].z; o[k].w = (v[k].w * inv) * wv[k].w;
        reinterpret_cast<float4*>(hout + base)[i] = o[k];
        mx = max(mx, __float_as_uint(o[k].x) & 0x7fffffffu);
        mx = max(mx, __float_as_uint(o[k].y) & 0x7fffffffu);
        mx = max(mx, __float_as_uint(o[k].z) & 0x7fffffffu);
        mx = max(mx, __float_as_uint(o[k].w) & 0x7fffffffu);
      }
    }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, d));
  if ((t & 63) == 0) part[t >> 6] = mx;
  __syncthreads();
  mx = part[0];
#pragma unroll
  for (int k = 1; k < 16; k++) mx = max(mx, part[k]);
  const int e = row_exponent((int)(mx >> 23), mx == 0);
  const float sc = pow2f(e);
  char* dst = img + (size_t)tm * nslab * kAImage;
  uint32_t least = 0xffffffffu;                    // smallest nonzero magnitude's bits, minus one
#pragma unroll
  for (int k = 0; k < RV; k++) {
    const int q = t + k * 1024;                    // float4 q of the row: slab q / 8, 8-byte piece q % 8 of its 64 bytes
    if (q < n4) {
      const float xs[4] = {o[k].x * sc, o[k].y * sc, o[k].z * sc, o[k].w * sc};
#pragma unroll
      for (int j = 0; j < 4; j++) least = min(least, (__float_as_uint(xs[j]) & 0x7fffffffu) - 1u);   // 0 wraps to the top
      uint32_t h01, l01, h23, l23;
      split2_f16(xs[0], xs[1], h01, l01);
      split2_f16(xs[2], xs[3], h23, l23);
      const int c4 = q & 7;
      char* op = dst + (size_t)(q >> 3) * kAImage + image_off(row, c4 >> 1) + (c4 & 1) * 8;
      *reinterpret_cast<uint2*>(op) = make_uint2(h01, h23);
      *reinterpret_cast<uint2*>(op + kPlaneBytes) = make_uint2(l01, l23);
    }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) least = min(least, (uint32_t)__shfl_xor((int)least, d));
  if ((t & 63) == 0) cnt[t >> 6] = least;
  __syncthreads();
  if (t == 0 && gm < M) {
    least = cnt[0];
    for (int k = 1; k < 16; k++) least = min(least, cnt[k]);
    uint32_t small = least < 0x3a800000u - 1u ? (uint32_t)n : 0u;          // 0 < |x| < 2^-10 somewhere
    if (mx >= 0x7f800000u) small = kSmallMax;
    ea[gm] = (e & 0xff) | (int)(small << 8);
  }
}

// Grid: x = tiles (row tiles fastest, one contiguous run of tiles per XCD), y = K-split parts of
// `part_slabs` slabs each; part y goes to C + y * M * ldc. N = columns of this launch (gated:
// features), tn0 = first column tile (the launch may cover a column range of the weight).
// TM = 2: a 256 x 256 tile, 64 x 128 per wavefront. TM = 1: 128 x 256 (32 x 128 per wavefront, one
// half of an activation image): twice the tiles for the products whose N is a few thousand, which
// then need half the K splits and write half the parts.
// GU: the result is the gated activation act[m][f] = swiglu(A . gate_f, A . up_f)
// (array.h:2435-2439) when K is not split; under a split the raw parts are stored in tile column
// order and splitk_sum_swiglu_kernel gates after the sum.
template <int TM, bool GU>
__global__ __launch_bounds__(512, 1) void gemm_f16t_kernel(const char* __restrict__ Aimg,
                                                           const char* __restrict__ Wimg,
                                                           float* __restrict__ C, int M, int N, int nslab,
                                                           int part_slabs, int ldc, int tn0, int ff,
                                                           const int* __restrict__ ea,
                                                           const int8_t* __restrict__ ew, int wpad,
                                                           const float* __restrict__ A) {
  constexpr int BM = 128 * TM;
  constexpr int kAPlane = BM * kRowBytes;            // one plane of this block's rows in a stage
  constexpr int kStage = 2 * kAPlane + kWImage;
  constexpr int kCopies = 2 * TM + 2;                // 1 KB copies per wavefront and slab
  extern __shared__ __attribute__((aligned(1024))) char ring[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;           // 4 x 2 wavefronts, (32 * TM) x 128 each
  const int mt = (M + BM - 1) / BM;
  const int nb = gridDim.x, xcd = blockIdx.x & 7, within = blockIdx.x >> 3;
  const int q8 = nb >> 3, r8 = nb & 7;
  const int lid = xcd * q8 + min(xcd, r8) + within;
  const int tm = lid % mt, tn = tn0 + lid / mt;
  const int sbeg = blockIdx.y * part_slabs, ns = min(nslab, sbeg + part_slabs) - sbeg;
  C += (size_t)blockIdx.y * M * ldc;

  // this wavefront's share of a slab copy: TM KB of each plane of A (TM = 1: of the half image
  // that holds this block's rows), two of the 16 KB of W
  // Everything but the lane's 16-byte slot is uniform over the wavefront and kept in scalars.
  const int img = TM == 2 ? tm : tm >> 1, half = TM == 2 ? 0 : (tm & 1) * kAPlane;
  const int uw = __builtin_amdgcn_readfirstlane(wave);
  const char* asrc = Aimg + ((size_t)img * nslab + sbeg) * kAImage + half + (uw * TM) * 1024;
  const char* wsrc = Wimg + ((size_t)tn * nslab + sbeg) * kWImage + (uw * 2) * 1024;
  const uint32_t slot = lane * 16;
  // copy C of this wavefront's kCopies for slab `slab` into ring stage `stage`
  // (past the end: the last slab again, into a stage nobody reads)
  auto copy = [&](int slab, int stage, auto CI) {
    constexpr int ci = decltype(CI)::value;
    const int s = min(slab, ns - 1);
    char* base = ring + stage * kStage;
    if (ci < 2 * TM) {
      constexpr int p = ci / TM, j = ci % TM;
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(asrc + (size_t)s * kAImage + p * kPlaneBytes + j * 1024 + slot),
          (__attribute__((address_space(3))) void*)(base + p * kAPlane + (uw * TM + j) * 1024), 16, 0, 0);
    } else {
      constexpr int j = ci - 2 * TM;
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(wsrc + (size_t)s * kWImage + j * 1024 + slot),
          (__attribute__((address_space(3))) void*)(base + 2 * kAPlane + (uw * 2 + j) * 1024), 16, 0, 0);
    }
  };
  auto issue = [&](int slab, int stage) {
    copy(slab, stage, Idx<0>{});
    copy(slab, stage, Idx<1>{});
    copy(slab, stage, Idx<2>{});
    copy(slab, stage, Idx<3>{});
    if (TM == 2) {
      copy(slab, stage, Idx<4>{});
      copy(slab, stage, Idx<5>{});
    }
  };

  f32x16 acc[TM][4];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  // this lane's first fragment of A (hi plane, tile row 0) and of W (tile column 0) within a
  // stage, per 16-k step; the other fragments are constant offsets from these
  int aoff[2], boff[2];
#pragma unroll
  for (int ks = 0; ks < 2; ks++) {
    const int kc = ks * 2 + (lane >> 5);
    aoff[ks] = image_off(wm * 32 * TM + (lane & 31), kc);
    boff[ks] = 2 * kAPlane + image_off(wn * 128 + (lane & 31), kc);
  }
  // fragment sets: F[0] for the first 16 k of a slab, F[1] for the second
  frag16 af[2][TM][2], bf[2][4];
  auto fetch = [&](const char* stage, auto KS) {
    constexpr int ks = decltype(KS)::value;
#pragma unroll
    for (int j = 0; j < 4; j++) bf[ks][j] = *reinterpret_cast<const frag16*>(stage + boff[ks] + j * 32 * kRowBytes);
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int p = 0; p < 2; p++)
        af[ks][i][p] = *reinterpret_cast<const frag16*>(stage + aoff[ks] + p * kAPlane + i * 32 * kRowBytes);
  };
  // four products: fragment set KS, (tile row, plane) pair Q against the four tile columns. The
  // weight fragment is the MFMA's first operand: the tile comes out transposed, D[n][m], so that a
  // lane ends up with four consecutive COLUMNS of one row of C - a 16-byte store, not four 4-byte ones.
  auto mul4 = [&](auto KS, auto Q) {
    constexpr int ks = decltype(KS)::value, q = decltype(Q)::value;
#pragma unroll
    for (int j = 0; j < 4; j++)
      acc[q >> 1][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, bf[ks][j]),
                                                              __builtin_bit_cast(f16x8, af[ks][q >> 1][q & 1]), acc[q >> 1][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  };
  // The block's barrier without the fence __syncthreads() puts before it: that fence would wait for
  // EVERY copy in flight (they write LDS). What has to be complete is waited for by count instead.
  auto barrier = [] {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  // Three slabs in flight. Invariant at the top of iteration k: slab k has landed in stage k % 3
  // for every wavefront and its first fragment set is on its way to registers; slabs k + 1 and
  // k + 2 are being copied.
  issue(0, 0);
  issue(1, 1);
  issue(2, 2);
#ifdef TLHIP_TRACE
  unsigned long long ph[2] = {0, 0}, tc = __builtin_readcyclecounter();
  TLHIP_MARK(0);
#define TLHIP_PHASE(i) do { const unsigned long long n_ = __builtin_readcyclecounter(); ph[i] += n_ - tc; tc = n_; } while (0)
#else
#define TLHIP_PHASE(i)
#endif
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kCopies) : "memory");   // my copies of slab 0
  barrier();
  fetch(ring, Idx<0>{});
  TLHIP_MARK(1);
  // A fragment set is requested a few MFMAs before the set that uses it starts, and nothing
  // younger is outstanding when it is waited for. The copies of slab k + 3 go out one or two at a
  // time between groups of MFMAs: issued together, the 48 of a block queue up in front of the
  // CU's one vector memory path and hold back the MFMAs that follow them in each wavefront.
  int st = 0;
  for (int k = 0; k < ns; k++) {
    const char* stage = ring + st * kStage;
    const int nx = st == 2 ? 0 : st + 1;
    mul4(Idx<0>{}, Idx<0>{});
    fetch(stage, Idx<1>{});
    __builtin_amdgcn_sched_barrier(0);
    mul4(Idx<0>{}, Idx<1>{});
    if constexpr (TM == 2) {
      mul4(Idx<0>{}, Idx<2>{});
      mul4(Idx<0>{}, Idx<3>{});
    }
    TLHIP_PHASE(0);
    // my reads of slab k are complete and my copies of slab k + 1 have landed (those of slab
    // k + 2 may still be in flight); past the barrier that holds for every wavefront
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kCopies) : "memory");
    barrier();
    TLHIP_PHASE(1);
    // slab k + 3 into the stage slab k has just left
    mul4(Idx<1>{}, Idx<0>{});
    copy(k + 3, st, Idx<0>{});
    if (TM == 1) copy(k + 3, st, Idx<1>{});
    if (k + 1 < ns) fetch(ring + nx * kStage, Idx<0>{});
    __builtin_amdgcn_sched_barrier(0);
    mul4(Idx<1>{}, Idx<1>{});
    if constexpr (TM == 1) {
      copy(k + 3, st, Idx<2>{});
      copy(k + 3, st, Idx<3>{});
    } else {
      copy(k + 3, st, Idx<1>{});
      copy(k + 3, st, Idx<2>{});
      __builtin_amdgcn_sched_barrier(0);
      mul4(Idx<1>{}, Idx<2>{});
      copy(k + 3, st, Idx<3>{});
      copy(k + 3, st, Idx<4>{});
      __builtin_amdgcn_sched_barrier(0);
      mul4(Idx<1>{}, Idx<3>{});
      copy(k + 3, st, Idx<5>{});
    }
    __builtin_amdgcn_sched_barrier(0);
    st = nx;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the copies past the end
#ifdef TLHIP_TRACE
  {
    const unsigned b = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    if (lane == 0 && b < kTraceBlocks) {
      unsigned long long* g = &g_trace[(b * kTraceWaves + wave) * kTraceSlots];
      g[2] = ph[0]; g[3] = ph[1]; g[7] = ns;
    }
  }
  TLHIP_MARK(5);
#endif
#undef TLHIP_PHASE

  // acc[v] of lane l (transposed tile): column of C 8*(v/4) + 4*(l/32) + v%4 of the tile, row of C
  // l%32. Four consecutive v are four consecutive columns: one 16-byte store where the row stride
  // allows it. The exponents come back out, -(ea[row] + ew[W row of the column]); ldexpf is exact.
  const int ltn = tn - tn0;                          // column tile within this launch
  const int nlim = N + (GU ? tn0 * 128 : tn0 * kTile);   // first unit of N past this launch, absolute
  const bool wide = (ldc & 3) == 0;
  // exponents of the W rows behind tile columns c .. c + 3 of this block
  auto wexp4 = [&](int c, int e4[4]) {
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const int r = weight_row(GU, tn, c + e, nlim, ff);
      e4[e] = r >= 0 ? (int)ew[r] : 0;
    }
  };
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  // Where small elements were counted - in a row of A (a_image_kernel) or in a row of W
  // (w_range_kernel) - their absolute errors add up to at most n 2^-10 in the units of acc, i.e.
  // n 2^-10 2^-(ea + ew) in the result's. After the tile has been stored, a result for which that
  // could reach a quarter of the absolute tolerance of 1e-5 (and every result of a row that is not
  // finite) is worked out again from the operands themselves, the f32 activations and the bf16
  // weight - an fp32 FMA chain over this block's K range in k order, the arithmetic of the
  // reference's loop (tensorlib_cuda.cu:509-519) - and stored over the first one by the lane that
  // stored that. Ordinary operands never get here: it takes an element 2^24 (of W: 2^31) below its
  // row's largest AND a row-times-column scale above 2^14. The pass is per lane and serial; the
  // kernel's time is not its concern.
  const uint16_t* wcount = reinterpret_cast<const uint16_t*>(ew + wpad);
  const WHeader* whdr = reinterpret_cast<const WHeader*>(ew + 3 * (size_t)wpad);
  auto again = [&](bool gated_out) {
    bool wsome = false;                 // does any of this wavefront's 128 columns carry a count?
#pragma unroll
    for (int e = 0; e < 2; e++) {
      const int r = weight_row(GU, tn, wn * 128 + lane * 2 + e, nlim, ff);
      wsome |= r >= 0 && wcount[r] != 0;
    }
    wsome = __any(wsome);
#pragma unroll 1
    for (int i = 0; i < TM; i++) {
      const int gm = tm * BM + wm * 32 * TM + i * 32 + (lane & 31);
      const int raw = gm < M ? ea[gm] : 0;
      const uint32_t nsm = (uint32_t)raw >> 8;
      if (!wsome && !__any(nsm != 0u)) continue;      // the ordinary case: nothing to weigh
      if (gm >= M) continue;
      const int em = (int)(int8_t)(raw & 0xff);
      const int64_t K = whdr->K;
      const float* arow = A + (size_t)gm * K + (size_t)sbeg * kBK;
      auto needs = [&](int r) {
        const uint32_t nw = wcount[r];
        return (nsm | nw) != 0u && (nsm == kSmallMax || nw == kWSmallMax ||
                                    ldexpf((float)(nsm + nw), -(em + (int)ew[r])) > 0x1p-8f);
      };
      auto chain = [&](int r) {         // row gm of A against row r of W over this block's K range
        const uint16_t* wrow = whdr->W + (size_t)r * K + (size_t)sbeg * kBK;
        float x = 0.f;
#pragma unroll 1
        for (int k = 0; k < ns * kBK; k += 2) {
          const uint32_t w = *reinterpret_cast<const uint32_t*>(wrow + k);
          x = fmaf(arow[k], bf16_lo(w), x);
          x = fmaf(arow[k + 1], bf16_hi(w), x);
        }
        return x;
      };
#pragma unroll 1
      for (int idx = 0; idx < (gated_out ? 32 : 64); idx++) {
        const int j = idx >> 4, v = idx & 15;
        const int c = wn * 128 + j * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (gated_out) {
          const int f = ltn * 128 + wn * 64 + j * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
          const int rg = weight_row(GU, tn, c, nlim, ff), ru = weight_row(GU, tn, c + 64, nlim, ff);
          if (f >= N || rg < 0 || ru < 0 || !(needs(rg) || needs(ru))) continue;
          const float gt = chain(rg), sg = 1.0f / (1.0f + expf(-gt));
          C[(size_t)gm * ldc + f] = (gt * sg) * chain(ru);
        } else {
          const int gn = ltn * kTile + c;
          const int r = weight_row(GU, tn, c, nlim, ff);
          if ((!GU && gn >= N) || r < 0 || !needs(r)) continue;
          C[(size_t)gm * ldc + gn] = chain(r);
        }
      }
    }
  };
  if (GU && gridDim.y == 1) {
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int gm = tm * BM + wm * 32 * TM + i * 32 + (lane & 31);
      if (gm >= M) continue;
      const int em = (int)(int8_t)(ea[gm] & 0xff);
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const int c = wn * 128 + j * 32 + 8 * g + 4 * (lane >> 5);      // gate column of the tile; its up value is 64 further
          const int f = ltn * 128 + wn * 64 + j * 32 + 8 * g + 4 * (lane >> 5);
          if (f >= N) continue;
          int eg[4], eu[4];
          wexp4(c, eg);
          wexp4(c + 64, eu);
          f32x4 o;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float gt = ldexpf(acc[i][j][4 * g + e], -(em + eg[e])), sg = 1.0f / (1.0f + expf(-gt));
            o[e] = (gt * sg) * ldexpf(acc[i][j + 2][4 * g + e], -(em + eu[e]));
          }
          float* dst = C + (size_t)gm * ldc + f;
          if (wide && f + 3 < N) {
            *reinterpret_cast<f32x4*>(dst) = o;
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
              if (f + e < N) dst[e] = o[e];
          }
        }
    }
    again(true);
    TLHIP_MARK(6);
    return;
  }
#pragma unroll
  for (int i = 0; i < TM; i++) {
    const int gm = tm * BM + wm * 32 * TM + i * 32 + (lane & 31);
    if (gm >= M) continue;
    const int em = (int)(int8_t)(ea[gm] & 0xff);
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int c = wn * 128 + j * 32 + 8 * g + 4 * (lane >> 5);
        const int gn = ltn * kTile + c;
        if (!GU && gn >= N) continue;   // gated parts are whole tiles wide
        int e4[4];
        wexp4(c, e4);
        f32x4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = ldexpf(acc[i][j][4 * g + e], -(em + e4[e]));
        float* dst = C + (size_t)gm * ldc + gn;
        if (wide && (GU || gn + 3 < N)) {
          *reinterpret_cast<f32x4*>(dst) = o;
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++)
            if (GU || gn + e < N) dst[e] = o[e];
        }
      }
  }
  again(false);
  TLHIP_MARK(6);
}

}  // namespace f16t
}  // namespace tlhip

using namespace tlhip;

namespace {

int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// plain: C[M][N]; parts (S_out != nullptr): C is the caller's [S][M][N]; gated: N = features, C[M][N] the activation
// aimg_in: the activation image of A made before (tlhip_rmsnorm_res_parts_aimage), or nullptr: made here
int gemm_f16w_impl(const void* A, const void* image, const void* exps, void* C, int64_t M, int64_t N, int64_t K,
                   size_t parts_bytes, int* S_out, bool gu, const void* aimg_in = nullptr) {
  TLHIP_REQUIRE_READY();
  const bool want_parts = S_out != nullptr;
  if (!A || !image || !exps || !C) return fail(TLHIP_EINVAL, "tlhip_gemm_f16w_nt: null pointer");
  if (M <= 0 || N <= 0 || K <= 0 || (K % f16t::kBK) != 0 || K > 256 * 4 * f16t::kRowRegs)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm_f16w_nt: need positive M, N, K, K %% 32 == 0 and K <= 32768");
  if (M > 0x3fffffff || N > 0x3fffffff || K > 0x3fffffff)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm_f16w_nt: dimension too large");
  if (!aligned16(A) || !aligned16(image) || !aligned16(C))
    return fail(TLHIP_EINVAL, "tlhip_gemm_f16w_nt: operands must be 16-byte aligned");
  Context& c = ctx();
  const int per = gu ? 2 : 1;                       // tile columns per unit of N
  const int64_t w = f16t::kTile / per;              // units of N per column tile
  const int64_t nslab = K / f16t::kBK, tn = cdiv64(N, w);
  const int64_t slots = c.cus;                      // one block per CU
  const int64_t tm256 = cdiv64(M, 256), tm128 = cdiv64(M, 128);
  const bool can_split = (N % 4) == 0;              // the part sums work on float4s
  // Work is shaped to whole rounds of the block slots, as in tlhip_gemm_bf16_nt: fewer tiles than
  // slots -> K split so that tiles * S comes close to the slots; more -> the columns that make
  // whole rounds with full K, the remaining columns split over K in a second launch. A piece runs
  // on 256-row tiles unless those would leave more than half of the CUs to K splits; then on
  // 128-row tiles: twice the tiles, half the splits, half the parts to write and add up.
  struct Piece { int64_t tn0, tcols; int S; int tmh; };
  Piece pieces[2];
  int npieces = 0;
  auto pick_S = [&](int64_t t) {
    if (!can_split || t >= slots) return 1;
    int64_t S = slots / t;
    if (S > 16) S = 16;
    while (S > 1 && nslab / S < 8) S--;             // at least 256 k per part
    if (want_parts)
      while (S > 1 && (size_t)S * M * N * sizeof(float) > parts_bytes) S--;
    return (int)S;
  };
  auto piece = [&](int64_t tn0, int64_t tcols, bool split) {
    const int tmh = tm256 * tcols * 2 <= slots ? 1 : 2;
    return Piece{tn0, tcols, split ? pick_S((tmh == 1 ? tm128 : tm256) * tcols) : 1, tmh};
  };
  const int64_t cols_per_round = slots / tm256;
  if (tm256 * tn <= slots || cols_per_round == 0 || !can_split || want_parts) {
    pieces[npieces++] = piece(0, tn, true);
  } else {
    const int64_t main_tn = tn / cols_per_round * cols_per_round;
    pieces[npieces++] = Piece{0, main_tn, 1, 2};
    if (main_tn < tn) pieces[npieces++] = piece(main_tn, tn - main_tn, true);
  }
  // scratch: exponents of A's rows, the slab images of A, room for the largest piece's parts
  const size_t ea_bytes = ((size_t)M * sizeof(int) + 1023) & ~(size_t)1023;
  const int64_t timg = cdiv64(M, f16t::kTile);      // activation images are 256 rows tall
  const size_t aimg_bytes = (size_t)timg * nslab * f16t::kAImage;
  size_t parts_need = 0;
  if (!want_parts)
    for (int pi = 0; pi < npieces; pi++)
      if (pieces[pi].S > 1) {
        const int64_t part_w = gu ? pieces[pi].tcols * f16t::kTile : std::min<int64_t>(pieces[pi].tcols * w, N - pieces[pi].tn0 * w);
        parts_need = std::max(parts_need, (size_t)pieces[pi].S * M * part_w * sizeof(float));
      }
  char* sbase = static_cast<char*>(scratch(ea_bytes + aimg_bytes + parts_need));
  if (!sbase) return fail(TLHIP_ENOMEM, "tlhip_gemm_f16w_nt: no scratch for the activation planes and K-split parts");
  const int* ea = reinterpret_cast<const int*>(sbase);
  const char* aimg = sbase + ea_bytes;
  const float* pa = static_cast<const float*>(A);
  if (aimg_in) {
    if (!aligned16(aimg_in)) return fail(TLHIP_EINVAL, "tlhip_gemm_f16w_nt: activation image not 16-byte aligned");
    ea = static_cast<const int*>(aimg_in);
    aimg = static_cast<const char*>(aimg_in) + ea_bytes;
  } else {
    f16t::a_image_kernel<<<dim3((unsigned)(timg * f16t::kTile)), dim3(256), 0, c.stream>>>(
        pa, reinterpret_cast<int*>(sbase), sbase + ea_bytes, (int)M, (int)K);
  }
  float* pc = static_cast<float*>(C);
  for (int pi = 0; pi < npieces; pi++) {
    const Piece& P = pieces[pi];
    const int64_t n0 = P.tn0 * w, pn = std::min<int64_t>(P.tcols * w, N - n0);   // units of N in this piece
    const int64_t part_w = gu ? P.tcols * f16t::kTile : pn;
    int S = P.S, part_slabs = (int)nslab;
    float* dst = pc + n0;
    int ldc = (int)N;
    if (S > 1) {
      part_slabs = (int)cdiv64(nslab, S);
      S = (int)cdiv64(nslab, part_slabs);
    }
    if (want_parts) {
      *S_out = S;
      dst = pc;
    } else if (S > 1) {
      dst = reinterpret_cast<float*>(sbase + ea_bytes + aimg_bytes);
      ldc = (int)part_w;
    }
    const int64_t nblk = (P.tmh == 1 ? tm128 : tm256) * P.tcols;
    const size_t lds = (size_t)f16t::kRing * (2 * 128 * P.tmh * f16t::kRowBytes + f16t::kWImage);
    if (nblk > 0x7fffffff || part_w > 0x7fffffff)
      return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm_f16w_nt: too many tiles for one grid");
    const dim3 grid((unsigned)nblk, (unsigned)S);
    auto launch = [&](auto fn) -> hipError_t {
      // more than 64 KB of LDS per block has to be asked for once per kernel (and device); the
      // four kernels share this one lambda instantiation (same function-pointer type), so the
      // note of who has asked is kept per kernel: [gated][tile height - 1]
      static int asked[2][2] = {{-1, -1}, {-1, -1}};
      int& asked_on_ = asked[gu ? 1 : 0][P.tmh - 1];
      if (asked_on_ != c.device) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)((size_t)f16t::kRing * (2 * 128 * P.tmh * f16t::kRowBytes + f16t::kWImage)));
        if (e != hipSuccess) return e;
        asked_on_ = c.device;
      }
      fn<<<grid, dim3(512), lds, c.stream>>>(aimg, static_cast<const char*>(image), dst, (int)M, (int)pn, (int)nslab,
                                             part_slabs, ldc, (int)P.tn0, (int)N, ea, static_cast<const int8_t*>(exps),
                                             (int)f16t::exps_pad(gu ? 2 * N : N), pa);
      return hipSuccess;
    };
    const hipError_t e = P.tmh == 2 ? (gu ? launch(f16t::gemm_f16t_kernel<2, true>) : launch(f16t::gemm_f16t_kernel<2, false>))
                                  : (gu ? launch(f16t::gemm_f16t_kernel<1, true>) : launch(f16t::gemm_f16t_kernel<1, false>));
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(LDS)");
    if (S > 1 && !want_parts) {
      const size_t total4 = (size_t)M * pn / 4;
      const dim3 sgrid((unsigned)((total4 + 255) / 256));
      if (gu)
        splitk_sum_swiglu_kernel<<<sgrid, dim3(256), 0, c.stream>>>(
            reinterpret_cast<const float4*>(dst), reinterpret_cast<float4*>(pc + n0), (int)M, (int)(pn / 4),
            (int)(part_w / 4), (int)(N / 4), S, 64 / 4);
      else
        splitk_sum_kernel<<<sgrid, dim3(256), 0, c.stream>>>(reinterpret_cast<const float4*>(dst),
                                                              reinterpret_cast<float4*>(pc + n0), (int)M,
                                                              (int)(pn / 4), (int)(N / 4), S);
    }
  }
  TLHIP_CHECK_LAUNCH(TLHIP_C_GEMM_BF16_NT);
}

}  // namespace

extern "C" {

int64_t tlhip_gemm_f16w_bytes(int64_t N, int64_t K, int gated) {
  if (N <= 0 || K <= 0 || (K % f16t::kBK) != 0) return 0;
  if (K > 256 * 4 * f16t::kRowRegs) return 0;    // deeper than the products over an image go: no image
  const int64_t tn = cdiv64(N, gated ? 128 : f16t::kTile);
  return tn * (K / f16t::kBK) * f16t::kWImage;
}

int tlhip_gemm_f16w_prepare(const void* W, int64_t N, int64_t K, int gated, void* image, void* exps) {
  TLHIP_REQUIRE_READY();
  if (!W || !image || !exps) return fail(TLHIP_EINVAL, "tlhip_gemm_f16w_prepare: null pointer");
  const int64_t rows = gated ? 2 * N : N;
  if (N <= 0 || K <= 0 || (K % f16t::kBK) != 0 || rows > 0x7fffffff || K > 0x3fffffff)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm_f16w_prepare: need positive N, K and K %% 32 == 0");
  if (!aligned16(W) || !aligned16(image) || !aligned16(exps))
    return fail(TLHIP_EINVAL, "tlhip_gemm_f16w_prepare: weight, image and exps must be 16-byte aligned");
  Context& c = ctx();
  const uint16_t* pw = static_cast<const uint16_t*>(W);
  int8_t* pe = static_cast<int8_t*>(exps);
  const int64_t tn = cdiv64(N, gated ? 128 : f16t::kTile), nslab = K / f16t::kBK;
  if (tn > 0x7fffffff || nslab > 65535)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm_f16w_prepare: weight too large for one grid");
  const int64_t pad = f16t::exps_pad(rows);
  row_exponent_bf16_kernel<<<dim3((unsigned)rows), dim3(256), 0, c.stream>>>(pw, (int)K, pe);
  f16t::w_range_kernel<<<dim3((unsigned)rows), dim3(256), 0, c.stream>>>(
      pw, pe, (int)K, reinterpret_cast<uint16_t*>(pe + pad), reinterpret_cast<f16t::WHeader*>(pe + 3 * pad));
  f16t::w_image_kernel<<<dim3((unsigned)tn, (unsigned)nslab), dim3(256), 0, c.stream>>>(
      pw, pe, static_cast<char*>(image), (int)N, (int)K, (int)N, gated ? 1 : 0);
  const hipError_t e = hipGetLastError();   // a preparation is not a product: not in the census
  return e == hipSuccess ? TLHIP_OK : hip_fail(e, "kernel launch");
}

int64_t tlhip_gemm_f16w_exps_bytes(int64_t N, int gated) {
  if (N <= 0) return 0;
  return 3 * f16t::exps_pad(gated ? 2 * N : N) + (int64_t)sizeof(f16t::WHeader);
}

int tlhip_gemm_f16w_nt(const void* A, const void* image, const void* exps, void* C, int64_t M, int64_t N,
                       int64_t K) {
  return gemm_f16w_impl(A, image, exps, C, M, N, K, 0, nullptr, false);
}

int tlhip_gemm_f16w_nt_swiglu(const void* A, const void* image, const void* exps, void* act, int64_t M,
                              int64_t ff, int64_t K) {
  return gemm_f16w_impl(A, image, exps, act, M, ff, K, 0, nullptr, true);
}

int64_t tlhip_gemm_f16w_aimage_bytes(int64_t M, int64_t K) {
  if (M <= 0 || K <= 0 || (K % f16t::kBK) != 0 || K > 256 * 4 * f16t::kRowRegs || M > 0x3fffffff) return 0;
  const int64_t ea_bytes = (M * (int64_t)sizeof(int) + 1023) & ~(int64_t)1023;
  return ea_bytes + cdiv64(M, f16t::kTile) * (K / f16t::kBK) * f16t::kAImage;
}

int tlhip_rmsnorm_res_parts_aimage(const void* x, const void* parts, int64_t S, const void* w, void* xout,
                                   void* hout, int64_t n, float eps, int64_t rows, void* aimage) {
  TLHIP_REQUIRE_READY();
  if (!x || !parts || !w || !xout || !hout || !aimage)
    return fail(TLHIP_EINVAL, "tlhip_rmsnorm_res_parts_aimage: null pointer");
  if (n <= 0 || rows <= 0 || rows > 0x3fffffff || S <= 0 || S > 64 || (n % f16t::kBK) != 0 || n > 8192)
    return fail(TLHIP_EUNSUPPORTED,
                "tlhip_rmsnorm_res_parts_aimage: need positive rows, 1 <= S <= 64, n %% 32 == 0 and n <= 8192");
  if (!aligned16(x) || !aligned16(parts) || !aligned16(xout) || !aligned16(w) || !aligned16(hout) || !aligned16(aimage))
    return fail(TLHIP_EINVAL, "tlhip_rmsnorm_res_parts_aimage: misaligned");
  if (xout == parts) return fail(TLHIP_EINVAL, "tlhip_rmsnorm_res_parts_aimage: xout must not alias the parts");
  const int64_t timg = cdiv64(rows, f16t::kTile);
  if (timg * f16t::kTile > 0x7fffffff) return fail(TLHIP_EUNSUPPORTED, "tlhip_rmsnorm_res_parts_aimage: too many rows");
  const size_t ea_bytes = ((size_t)rows * sizeof(int) + 1023) & ~(size_t)1023;
  int* ea = static_cast<int*>(aimage);
  char* img = static_cast<char*>(aimage) + ea_bytes;
  const dim3 grid((unsigned)(timg * f16t::kTile)), block(1024);
  const size_t ps = (size_t)(rows * n);
  hipStream_t st = ctx().stream;
  if (n <= 4096)
    f16t::rmsnorm_aimage_kernel<1><<<grid, block, 0, st>>>(static_cast<const float*>(x), static_cast<const float*>(parts),
                                                         static_cast<const float*>(w), static_cast<float*>(xout),
                                                         static_cast<float*>(hout), (int)n, eps, (int)S, ps, ea, img, (int)rows);
  else
    f16t::rmsnorm_aimage_kernel<2><<<grid, block, 0, st>>>(static_cast<const float*>(x), static_cast<const float*>(parts),
                                                         static_cast<const float*>(w), static_cast<float*>(xout),
                                                         static_cast<float*>(hout), (int)n, eps, (int)S, ps, ea, img, (int)rows);
  TLHIP_CHECK_LAUNCH(TLHIP_C_RMSNORM_RES);
}

int tlhip_gemm_f16w_nt_aimage(const void* A, const void* aimage, const void* image, const void* exps, void* C,
                              int64_t M, int64_t N, int64_t K) {
  if (!aimage) return fail(TLHIP_EINVAL, "tlhip_gemm_f16w_nt_aimage: null activation image");
  return gemm_f16w_impl(A, image, exps, C, M, N, K, 0, nullptr, false, aimage);
}

int tlhip_gemm_f16w_nt_swiglu_aimage(const void* A, const void* aimage, const void* image, const void* exps,
                                     void* act, int64_t M, int64_t ff, int64_t K) {
  if (!aimage) return fail(TLHIP_EINVAL, "tlhip_gemm_f16w_nt_swiglu_aimage: null activation image");
  return gemm_f16w_impl(A, image, exps, act, M, ff, K, 0, nullptr, true, aimage);
}

int tlhip_gemm_f16w_nt_parts_aimage(const void* A, const void* aimage, const void* image, const void* exps,
                                    void* parts, int64_t parts_bytes, int64_t M, int64_t N, int64_t K, int* n_parts) {
  if (!n_parts || !aimage) return fail(TLHIP_EINVAL, "tlhip_gemm_f16w_nt_parts_aimage: null n_parts or activation image");
  if (M > 0 && N > 0 && parts_bytes < (int64_t)(M * N * sizeof(float)))
    return fail(TLHIP_EINVAL, "tlhip_gemm_f16w_nt_parts_aimage: the buffer must hold at least one [M, N] part");
  *n_parts = 0;
  return gemm_f16w_impl(A, image, exps, parts, M, N, K, (size_t)parts_bytes, n_parts, false, aimage);
}

int tlhip_gemm_f16w_nt_parts(const void* A, const void* image, const void* exps, void* parts,
                             int64_t parts_bytes, int64_t M, int64_t N, int64_t K, int* n_parts) {
  if (!n_parts) return fail(TLHIP_EINVAL, "tlhip_gemm_f16w_nt_parts: null n_parts");
  if (M > 0 && N > 0 && parts_bytes < (int64_t)(M * N * sizeof(float)))
    return fail(TLHIP_EINVAL, "tlhip_gemm_f16w_nt_parts: the buffer must hold at least one [M, N] part");
  *n_parts = 0;
  return gemm_f16w_impl(A, image, exps, parts, M, N, K, (size_t)parts_bytes, n_parts, false);
}

}  // extern "C"
