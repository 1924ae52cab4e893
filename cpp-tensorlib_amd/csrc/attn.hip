// Decode attention over a [Hkv, kv_max, D] cache: flash-decoding on wave64.
//
// One block serves ONE kv head and up to G of its query heads, so with GQA the
// K/V rows are fetched from HBM once per group instead of once per query head.
// Keys are split over gridDim.y (split-KV) and over the wavefronts of a block
// in tiles of 64 keys. Inside a wavefront a key row is spread over LPK = D/4
// lanes (one 128-bit load per lane, 64/LPK keys per load instruction, fully
// coalesced); scores are reduced over those lanes, parked one-key-per-lane so
// that the softmax exponentials cost one instruction per 64 keys, and fed back
// to the P.V pass through a per-wave LDS line. Running (max, sum, acc) states
// are merged wave -> block -> split in a fixed order: no atomics.
#include "common.hpp"

namespace tlhip {

template <typename KT> struct KvLoad;
template <> struct KvLoad<float> {
  static __device__ __forceinline__ float4 ld(const float* p) { return *reinterpret_cast<const float4*>(p); }
};
template <> struct KvLoad<uint16_t> {
  static __device__ __forceinline__ float4 ld(const uint16_t* p) {
    const uint2 r = *reinterpret_cast<const uint2*>(p);
    return make_float4(bf16_lo(r.x), bf16_hi(r.x), bf16_lo(r.y), bf16_hi(r.y));
  }
};

__device__ __forceinline__ void wave_lds_sync() {
  // order this wavefront's LDS writes before its later LDS reads (other lanes' data)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// grid = (Hkv, S, ceil(group/G)); block = nw*64 threads (nw in 1,2,4).
// part_m/part_l: [Hq*S], part_acc: [Hq*S*D]; used when S > 1, else `out` is final.
template <int D, int G, typename KT>
__global__ __launch_bounds__(256) void attn_decode_kernel(
    const float* __restrict__ q, const KT* __restrict__ K, const KT* __restrict__ V,
    float* __restrict__ out, float* __restrict__ part_m, float* __restrict__ part_l,
    float* __restrict__ part_acc, int group, int ctx, int64_t kv_stride, int chunk, float scale,
    int S) {
  constexpr int LPK = D / 4;        // lanes per key row
  constexpr int KPS = 64 / LPK;     // keys per load step
  constexpr int UNR = 8;            // loads in flight per lane
  __shared__ float pbuf[4][G][64];              // per-wave probabilities of the current tile
  __shared__ float st_m[4][G], st_l[4][G];      // per-wave softmax state for the block merge
  __shared__ float st_acc[4][G][D];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int slot = lane / LPK, c = lane % LPK;
  const int kvh = blockIdx.x, split = blockIdx.y;
  const int g0 = blockIdx.z * G;                // first query head (within the group) of this block
  const int ng = min(G, group - g0);
  const int h0 = kvh * group + g0;              // absolute query head of g == 0
  const KT* Kh = K + (size_t)kvh * kv_stride;
  const KT* Vh = V + (size_t)kvh * kv_stride;
  const int k_begin = split * chunk, k_end = min(ctx, k_begin + chunk);

  float4 qv[G];
#pragma unroll
  for (int g = 0; g < G; g++) {
    qv[g] = g < ng ? *reinterpret_cast<const float4*>(q + (size_t)(h0 + g) * D + c * 4)
                   : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float m[G], l[G];
  float4 acc[G];
#pragma unroll
  for (int g = 0; g < G; g++) {
    m[g] = -INFINITY;
    l[g] = 0.f;
    acc[g] = make_float4(0.f, 0.f, 0.f, 0.f);
  }

  for (int kb = k_begin + wave * 64; kb < k_end; kb += nw * 64) {
    // ---- scores: lane (slot,c) ends up holding key kb + c*KPS + slot ----------
    float sreg[G];
#pragma unroll
    for (int g = 0; g < G; g++) sreg[g] = -INFINITY;
#pragma unroll
    for (int i0 = 0; i0 < LPK; i0 += UNR) {
      float4 kv[UNR];
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        const int key = kb + (i0 + u) * KPS + slot;
        kv[u] = key < k_end ? KvLoad<KT>::ld(Kh + (size_t)key * D + c * 4)
                            : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        const int key = kb + (i0 + u) * KPS + slot;
#pragma unroll
        for (int g = 0; g < G; g++) {
          float p = qv[g].x * kv[u].x;
          p = fmaf(qv[g].y, kv[u].y, p);
          p = fmaf(qv[g].z, kv[u].z, p);
          p = fmaf(qv[g].w, kv[u].w, p);
#pragma unroll
          for (int msk = LPK / 2; msk >= 1; msk >>= 1) p += __shfl_xor(p, msk, kWave);
          if (c == i0 + u) sreg[g] = key < k_end ? p * scale : -INFINITY;
        }
      }
    }
    // ---- online softmax update for the tile ---------------------------------------
#pragma unroll
    for (int g = 0; g < G; g++) {
      const float tmax = wave_max(sreg[g]);      // finite: the tile holds >= 1 live key
      const float mnew = fmaxf(m[g], tmax);
      const float corr = __expf(m[g] - mnew);    // 0 on the first tile (m = -inf)
      const float p = __expf(sreg[g] - mnew);    // 0 for masked keys
      l[g] = fmaf(l[g], corr, p);
      acc[g].x *= corr; acc[g].y *= corr; acc[g].z *= corr; acc[g].w *= corr;
      m[g] = mnew;
      pbuf[wave][g][lane] = p;
    }
    wave_lds_sync();
    // ---- P.V: lane (slot,c) accumulates its 4 output columns over its slot's keys ----
#pragma unroll
    for (int i0 = 0; i0 < LPK; i0 += UNR) {
      float4 vv[UNR];
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        const int key = kb + (i0 + u) * KPS + slot;
        vv[u] = key < k_end ? KvLoad<KT>::ld(Vh + (size_t)key * D + c * 4)
                            : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int g = 0; g < G; g++) {
        // key (i, slot) was parked in lane slot*LPK + i
        const float4 p0 = *reinterpret_cast<const float4*>(&pbuf[wave][g][slot * LPK + i0]);
        const float4 p1 = *reinterpret_cast<const float4*>(&pbuf[wave][g][slot * LPK + i0 + 4]);
        const float pp[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
#pragma unroll
        for (int u = 0; u < UNR; u++) {
          acc[g].x = fmaf(pp[u], vv[u].x, acc[g].x);
          acc[g].y = fmaf(pp[u], vv[u].y, acc[g].y);
          acc[g].z = fmaf(pp[u], vv[u].z, acc[g].z);
          acc[g].w = fmaf(pp[u], vv[u].w, acc[g].w);
        }
      }
    }
    wave_lds_sync();  // pbuf is rewritten by the next tile
  }

  // ---- wave totals: sum l over lanes, acc over the key slots -----------------------------
#pragma unroll
  for (int g = 0; g < G; g++) {
    l[g] = wave_sum(l[g]);
#pragma unroll
    for (int msk = LPK; msk < 64; msk <<= 1) {
      acc[g].x += __shfl_xor(acc[g].x, msk, kWave);
      acc[g].y += __shfl_xor(acc[g].y, msk, kWave);
      acc[g].z += __shfl_xor(acc[g].z, msk, kWave);
      acc[g].w += __shfl_xor(acc[g].w, msk, kWave);
    }
    if (lane == 0) { st_m[wave][g] = m[g]; st_l[wave][g] = l[g]; }
    if (slot == 0) *reinterpret_cast<float4*>(&st_acc[wave][g][c * 4]) = acc[g];
  }
  __syncthreads();

  // ---- block merge (fixed wave order) and store ---------------------------------------------
  for (int e = threadIdx.x; e < ng * D; e += blockDim.x) {
    const int g = e / D, d = e - g * D;
    float M = st_m[0][g];
    for (int w = 1; w < nw; w++) M = fmaxf(M, st_m[w][g]);
    float L = 0.f, A = 0.f;
    for (int w = 0; w < nw; w++) {
      const float f = __expf(st_m[w][g] - M);   // idle waves: exp(-inf) = 0
      L = fmaf(st_l[w][g], f, L);
      A = fmaf(st_acc[w][g][d], f, A);
    }
    const int h = h0 + g;
    if (S == 1) {
      out[(size_t)h * D + d] = A / L;
    } else {
      const size_t ps = (size_t)h * S + split;
      part_acc[ps * D + d] = A;
      if (d == 0) { part_m[ps] = M; part_l[ps] = L; }
    }
  }
}

// grid = Hq, block = D: merge the S split partials of one head.
__global__ void attn_combine_kernel(const float* __restrict__ part_m,
                                    const float* __restrict__ part_l,
                                    const float* __restrict__ part_acc, float* __restrict__ out,
                                    int S, int D) {
  const int h = blockIdx.x, d = threadIdx.x;
  const float* pm = part_m + (size_t)h * S;
  const float* pl = part_l + (size_t)h * S;
  float M = pm[0];
  for (int s = 1; s < S; s++) M = fmaxf(M, pm[s]);
  float L = 0.f, A = 0.f;
  for (int s = 0; s < S; s++) {
    const float f = __expf(pm[s] - M);
    L = fmaf(pl[s], f, L);
    A = fmaf(part_acc[((size_t)h * S + s) * D + d], f, A);
  }
  out[(size_t)h * D + d] = A / L;
}

struct AttnPlan { int G, gz, nw, S, chunk; };

// Split-KV plan: enough blocks to cover the CUs about twice, and never less
// than one 64-key tile per wavefront.
static AttnPlan plan_attn(int Hkv, int group, int ctx, int cus) {
  AttnPlan p{};
  p.G = group > 4 ? 8 : group > 2 ? 4 : group > 1 ? 2 : 1;
  p.gz = (group + p.G - 1) / p.G;
  const int base = Hkv * p.gz;
  const int tiles = (ctx + 63) / 64;
  int want = (2 * cus + base - 1) / base;  // splits wanted to fill the chip
  if (want < 1) want = 1;
  if (want > tiles) want = tiles;
  int tiles_per_split = (tiles + want - 1) / want;
  p.nw = tiles_per_split >= 4 ? 4 : tiles_per_split >= 2 ? 2 : 1;
  tiles_per_split = (tiles_per_split + p.nw - 1) / p.nw * p.nw;
  p.chunk = tiles_per_split * 64;
  p.S = (ctx + p.chunk - 1) / p.chunk;
  return p;
}

template <int D, typename KT>
static int launch_attn(const float* q, const KT* K, const KT* V, float* out, int Hq, int Hkv,
                       int ctx, int64_t kv_max, float scale) {
  Context& c = tlhip::ctx();
  const int group = Hq / Hkv;
  const AttnPlan p = plan_attn(Hkv, group, ctx, c.cus);
  float *pm = nullptr, *pl = nullptr, *pacc = nullptr;
  if (p.S > 1) {
    const size_t hs = (size_t)Hq * p.S;
    float* base = static_cast<float*>(scratch((hs * 2 + hs * D) * sizeof(float)));
    if (!base) return fail(TLHIP_ENOMEM, "tlhip_attn_decode: no scratch for %d splits", p.S);
    pm = base;
    pl = pm + hs;
    pacc = pl + hs;
  }
  const dim3 grid(Hkv, p.S, p.gz), block(p.nw * 64);
  const int64_t kv_stride = kv_max * D;
#define TLHIP_ATTN(GG)                                                                         \
  hipLaunchKernelGGL((attn_decode_kernel<D, GG, KT>), grid, block, 0, c.stream, q, K, V, out, \
                     pm, pl, pacc, group, ctx, kv_stride, p.chunk, scale, p.S)
  switch (p.G) {
    case 1: TLHIP_ATTN(1); break;
    case 2: TLHIP_ATTN(2); break;
    case 4: TLHIP_ATTN(4); break;
    default: TLHIP_ATTN(8); break;
  }
#undef TLHIP_ATTN
  if (p.S > 1)
    hipLaunchKernelGGL(attn_combine_kernel, dim3(Hq), dim3(D), 0, c.stream, pm, pl, pacc, out, p.S, D);
  TLHIP_CHECK_LAUNCH(TLHIP_C_ATTN_DECODE);
}

}  // namespace tlhip

using namespace tlhip;

extern "C" {

int tlhip_attn_decode(const void* q, const void* K, const void* V, void* out, int64_t n_q_heads,
                      int64_t n_kv_heads, int64_t ctx_len, int64_t kv_max, int64_t D, float scale,
                      int kv_bf16) {
  TLHIP_REQUIRE_READY();
  if (!q || !K || !V || !out) return fail(TLHIP_EINVAL, "tlhip_attn_decode: null pointer");
  // the reference's gates (cuda.h:970-971)
  if (D != 64 && D != 128) return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode: head_dim must be 64 or 128");
  if (n_kv_heads <= 0 || n_q_heads <= 0 || n_q_heads % n_kv_heads != 0)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode: Hq must be a positive multiple of Hkv");
  if (ctx_len <= 0 || ctx_len > kv_max) return fail(TLHIP_EINVAL, "tlhip_attn_decode: need 0 < ctx <= kv_max");
  if (ctx_len > 0x3fffffff || n_kv_heads > 65535 || kv_max * D > ((int64_t)1 << 40))
    return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode: shape too large");
  if (!aligned16(q) || !aligned16(K) || !aligned16(V) || !aligned16(out))
    return fail(TLHIP_EINVAL, "tlhip_attn_decode: operands must be 16-byte aligned");
  const float* pq = static_cast<const float*>(q);
  float* po = static_cast<float*>(out);
  const int Hq = (int)n_q_heads, Hkv = (int)n_kv_heads, cx = (int)ctx_len;
  if (kv_bf16) {
    const uint16_t* pk = static_cast<const uint16_t*>(K);
    const uint16_t* pv = static_cast<const uint16_t*>(V);
    return D == 128 ? launch_attn<128, uint16_t>(pq, pk, pv, po, Hq, Hkv, cx, kv_max, scale)
                    : launch_attn<64, uint16_t>(pq, pk, pv, po, Hq, Hkv, cx, kv_max, scale);
  }
  const float* pk = static_cast<const float*>(K);
  const float* pv = static_cast<const float*>(V);
  return D == 128 ? launch_attn<128, float>(pq, pk, pv, po, Hq, Hkv, cx, kv_max, scale)
                  : launch_attn<64, float>(pq, pk, pv, po, Hq, Hkv, cx, kv_max, scale);
}

}  // extern "C"
