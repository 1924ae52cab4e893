// Causal prefill attention on the fp32 matrix pipe (tlhip_attn_prefill, cuda.h:1165-1201).
//
//   out[h, p, :] = softmax_k( scale * q[h, p, :] . K[kv(h), k, :] ) . V[kv(h), k, :],  k <= pos0 + p
//
// v_mfma_f32_32x32x2_f32 multiplies f32 by f32 exactly and accumulates in fp32, so scores and
// outputs differ from the reference's loops in summation order only.
//
// A block owns one query head and 32 consecutive query positions; its 8 wavefronts deal the
// 32-key tiles of the causal range round-robin and each keeps a running (max, sum, output) state
// for all 32 queries (online softmax), merged through LDS at the end. Per key tile a wavefront
// issues 2 x D/2 MFMAs (Q.K^T, then P.V):
//   * S[32 q x 32 k] : A = the Q tile (in LDS, shared by the block), B = the K tile from LDS;
//   * the score tile leaves the MFMA as one column (key) per lane and 16 rows (queries) per
//     lane, so row maxima and sums are lane reductions over half a wavefront;
//   * P goes through a 32 x 32 LDS tile to become the A operand of P.V; the output
//     accumulators share the score tile's row layout, so the softmax rescale needs no exchange.
// One MFMA consumes one float per lane per operand: lane l supplies A[l % 32][l / 32] and
// B[l / 32][l % 32]. The reduction index is consumed in the order 8m + 4(l/32) + j, which
// makes a lane's four consecutive steps one 16-byte LDS read (Q and K, or P and V, use the
// same order, and a sum does not care).
//
// K, P and V tiles are private to their wavefront and take turns in ONE LDS region (no block
// barriers inside the loop): K is dead once the scores exist, P once it sits in registers.
// Eight wavefronts are two per SIMD: one's softmax (~750 VALU instructions a tile) and load
// latency run under the other's 64-cycle MFMAs. One block per CU (9 regions of 32 x (D+4) floats).
#include "common.hpp"

namespace tlhip {

typedef float f32x16 __attribute__((ext_vector_type(16)));

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// max / sum over the 32 lanes of a half wavefront (lanes that share lane / 32); result in every
// lane. Four DPP steps finish a 16-lane row; v_permlane16_swap (gfx950) then hands each row of a
// pair the other row's value: with both operands = v it returns (rows 0,0,2,2 ; rows 1,1,3,3).
__device__ __forceinline__ float half_max(float v) {
  v = fmaxf(v, dpp_mov<0xB1>(v));    // quad_perm [1,0,3,2]
  v = fmaxf(v, dpp_mov<0x4E>(v));    // quad_perm [2,3,0,1]
  v = fmaxf(v, dpp_mov<0x141>(v));   // row_half_mirror
  v = fmaxf(v, dpp_mov<0x140>(v));   // row_mirror
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_sum(float v) {
  v += dpp_mov<0xB1>(v);
  v += dpp_mov<0x4E>(v);
  v += dpp_mov<0x141>(v);
  v += dpp_mov<0x140>(v);
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ float4 load_kv4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load_kv4(const uint16_t* p) {   // 4 bf16, widened exactly
  const uint2 r = *reinterpret_cast<const uint2*>(p);
  return make_float4(bf16_lo(r.x), bf16_hi(r.x), bf16_lo(r.y), bf16_hi(r.y));
}

// LDS: the Q tile (shared by the block) and one 32 x (D+4) region per wavefront that holds the K
// tile, then P, then the V tile.
template <int D>
struct PrefillLds {
  static constexpr int KS = D + 4;
  static constexpr int PS = 36;
  static constexpr int kRegion = 32 * KS;                 // floats: Q, and one region per wavefront
  static constexpr size_t kBytes = (size_t)9 * kRegion * sizeof(float);
};

template <int D, typename KT>
__global__ __launch_bounds__(512, 1) void attn_prefill_mfma_kernel(const float* __restrict__ q,
                                                                    const KT* __restrict__ K,
                                                                    const KT* __restrict__ V,
                                                                    float* __restrict__ out, int group, int T,
                                                                    int pos0, int64_t kv_stride, float scale,
                                                                    int64_t o_head, int64_t o_row) {
  using L = PrefillLds<D>;
  constexpr int KS = L::KS, PS = L::PS;
  constexpr int kLoads = 32 * D / 4 / 64;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l31 = lane & 31, hi = lane >> 5;
  const int h = blockIdx.x;
  const int nqt = (T + 31) >> 5;
  const int p0 = (nqt - 1 - (int)blockIdx.y) * 32;
  const KT* Kh = K + (size_t)(h / group) * kv_stride;
  const KT* Vh = V + (size_t)(h / group) * kv_stride;
  float* Qs = lds;
  float* R = lds + (1 + wave) * L::kRegion;
  const int kend = min(pos0 + p0 + 32, pos0 + T);
  const int nkt = (kend + 31) >> 5;

  for (int slot = tid; slot < 32 * D / 4; slot += 512) {   // Q tile -> LDS (rows beyond T clamped, never stored)
    const int row = slot / (D / 4), c4 = slot % (D / 4);
    *reinterpret_cast<float4*>(Qs + row * KS + 4 * c4) =
        *reinterpret_cast<const float4*>(q + ((size_t)h * T + min(p0 + row, T - 1)) * D + 4 * c4);
  }
  __syncthreads();

  f32x16 o[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
    for (int v = 0; v < 16; v++) o[dt][v] = 0.f;
  float mrow[16], lrow[16];
#pragma unroll
  for (int v = 0; v < 16; v++) { mrow[v] = -INFINITY; lrow[v] = 0.f; }

  // K and V rows of a tile travel through registers into the wavefront's LDS region. The
  // registers are free again as soon as the tile has been written to LDS, so the NEXT tile's
  // rows are requested at that point - K right after the K tile is stored, V right after the V
  // tile is stored - and have a whole tile's arithmetic to arrive in. (Rows past the causal
  // range are clamped to its last row: mapped memory, masked when used.)
  float4 kreg[kLoads], vreg[kLoads];
  const auto request = [&](float4* dst, const KT* base, int tile) {
#pragma unroll
    for (int i = 0; i < kLoads; i++) {
      const int slot = lane + 64 * i, key = slot / (D / 4), c4 = slot % (D / 4);
      dst[i] = load_kv4(base + (size_t)min(tile * 32 + key, kend - 1) * D + 4 * c4);
    }
  };
  request(kreg, Kh, wave);
  request(vreg, Vh, wave);
#ifdef TLHIP_TRACE
  unsigned long long ph[5] = {0, 0, 0, 0, 0}, tc = __builtin_readcyclecounter();
  TLHIP_MARK(0);
#define TLHIP_PHASE(i) do { const unsigned long long n_ = __builtin_readcyclecounter(); ph[i] += n_ - tc; tc = n_; } while (0)
#else
#define TLHIP_PHASE(i)
#endif
  for (int kt = wave; kt < nkt; kt += 8) {
    const int k0 = kt * 32;
#pragma unroll
    for (int i = 0; i < kLoads; i++) {
      const int slot = lane + 64 * i, key = slot / (D / 4), c4 = slot % (D / 4);
      *reinterpret_cast<float4*>(R + key * KS + 4 * c4) = kreg[i];
    }
    request(kreg, Kh, kt + 8);
    TLHIP_PHASE(0);
    f32x16 s;
#pragma unroll
    for (int v = 0; v < 16; v++) s[v] = 0.f;
#pragma unroll
    for (int m = 0; m < D / 8; m++) {
      const float4 qa = *reinterpret_cast<const float4*>(Qs + l31 * KS + 8 * m + 4 * hi);
      const float4 kf = *reinterpret_cast<const float4*>(R + l31 * KS + 8 * m + 4 * hi);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(qa.x, kf.x, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(qa.y, kf.y, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(qa.z, kf.z, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(qa.w, kf.w, s, 0, 0, 0);
    }
    TLHIP_PHASE(1);
    const int key = k0 + l31;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int r = 8 * (v >> 2) + 4 * hi + (v & 3);
      const bool seen = key <= pos0 + p0 + r && key < kend;
      const float sv = seen ? s[v] * scale : -INFINITY;
      const float mnew = fmaxf(mrow[v], half_max(sv));
      const float mref = mnew == -INFINITY ? 0.f : mnew;
      const float corr = __expf(mrow[v] - mref);
      const float p = __expf(sv - mref);
      lrow[v] = lrow[v] * corr + half_sum(p);
      mrow[v] = mnew;
#pragma unroll
      for (int dt = 0; dt < D / 32; dt++) o[dt][v] *= corr;
      R[r * PS + l31] = p;                      // the K tile is dead: P takes its place
    }
    float4 pf[4];
#pragma unroll
    for (int m = 0; m < 4; m++) pf[m] = *reinterpret_cast<const float4*>(R + l31 * PS + 8 * m + 4 * hi);
#pragma unroll
    for (int i = 0; i < kLoads; i++) {          // P is in registers: V takes the region
      const int slot = lane + 64 * i, vkey = slot / (D / 4), c4 = slot % (D / 4);
      *reinterpret_cast<float4*>(R + vkey * D + 4 * c4) = vreg[i];
    }
    request(vreg, Vh, kt + 8);
    TLHIP_PHASE(2);
    // (the D/32 output tiles take turns, so consecutive MFMAs never wait for each other's result)
#pragma unroll
    for (int m = 0; m < 4; m++) {
      const float pj[4] = {pf[m].x, pf[m].y, pf[m].z, pf[m].w};
#pragma unroll
      for (int j = 0; j < 4; j++) {
#pragma unroll
        for (int dt = 0; dt < D / 32; dt++) {
          const float* vp = R + (8 * m + 4 * hi + j) * D + dt * 32 + l31;
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(pj[j], vp[0], o[dt], 0, 0, 0);
        }
      }
    }
    TLHIP_PHASE(3);
  }
#ifdef TLHIP_TRACE
  {
    const unsigned b = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    if (lane == 0 && b < kTraceBlocks) {
      unsigned long long* g = &g_trace[(b * kTraceWaves + wave) * kTraceSlots];
      g[1] = ph[0]; g[2] = ph[1]; g[3] = ph[2]; g[4] = ph[3]; g[5] = (nkt - wave + 7) / 8;
    }
  }
  TLHIP_MARK(6);
#endif
#undef TLHIP_PHASE

  // merge: each wavefront leaves O [32][D], m [32], l [32] in its region; 16 threads finish a row
  float* Mw = R + 32 * D;
#pragma unroll
  for (int v = 0; v < 16; v++) {
    const int r = 8 * (v >> 2) + 4 * hi + (v & 3);
#pragma unroll
    for (int dt = 0; dt < D / 32; dt++) R[r * D + dt * 32 + l31] = o[dt][v];
    if (l31 == 0) { Mw[r] = mrow[v]; Mw[32 + r] = lrow[v]; }
  }
  __syncthreads();
  {
    const int row = tid >> 4, d0 = (tid & 15) * (D / 16);
    const float* base = lds + L::kRegion;
    float f[8], M = -INFINITY, Lsum = 0.f;
#pragma unroll
    for (int w = 0; w < 8; w++) M = fmaxf(M, base[w * L::kRegion + 32 * D + row]);
#pragma unroll
    for (int w = 0; w < 8; w++) {
      const float mw = base[w * L::kRegion + 32 * D + row];
      f[w] = mw == -INFINITY ? 0.f : __expf(mw - M);
      Lsum += f[w] * base[w * L::kRegion + 32 * D + 32 + row];
    }
    if (p0 + row < T) {
      const float inv = 1.0f / Lsum;
      float* op = out + (size_t)h * o_head + (size_t)(p0 + row) * o_row + d0;   // [Hq,T,D] or [T,Hq*D]
#pragma unroll
      for (int d = 0; d < D / 16; d += 4) {
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int w = 0; w < 8; w++) {
          const float4 ow = *reinterpret_cast<const float4*>(base + w * L::kRegion + row * D + d0 + d);
          a.x += f[w] * ow.x; a.y += f[w] * ow.y; a.z += f[w] * ow.z; a.w += f[w] * ow.w;
        }
        *reinterpret_cast<float4*>(op + d) = make_float4(a.x * inv, a.y * inv, a.z * inv, a.w * inv);
      }
    }
  }
}

template <int D, typename KT>
int launch_prefill_mfma(const float* q, const KT* K, const KT* V, float* out, int Hq, int Hkv, int T,
                        int64_t kv_max, float scale, int pos0, int token_major) {
  Context& c = ctx();
  auto fn = attn_prefill_mfma_kernel<D, KT>;
  const int lds = (int)PrefillLds<D>::kBytes;
  if ((size_t)lds > (size_t)c.lds_per_cu) return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_prefill: not enough LDS");
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(LDS)");
  const dim3 grid((unsigned)Hq, (unsigned)((T + 31) / 32)), block(512);
  const int64_t o_head = token_major ? D : (int64_t)T * D, o_row = token_major ? (int64_t)Hq * D : D;
  hipLaunchKernelGGL(fn, grid, block, (size_t)lds, c.stream, q, K, V, out, Hq / Hkv, T, pos0, kv_max * (int64_t)D, scale,
                     o_head, o_row);
  return 0;
}

template int launch_prefill_mfma<128, float>(const float*, const float*, const float*, float*, int, int, int, int64_t, float, int, int);
template int launch_prefill_mfma<64, float>(const float*, const float*, const float*, float*, int, int, int, int64_t, float, int, int);
template int launch_prefill_mfma<128, uint16_t>(const float*, const uint16_t*, const uint16_t*, float*, int, int, int, int64_t, float, int, int);
template int launch_prefill_mfma<64, uint16_t>(const float*, const uint16_t*, const uint16_t*, float*, int, int, int, int64_t, float, int, int);

}  // namespace tlhip
