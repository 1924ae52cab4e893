// Decode attention over a [Hkv, kv_max, D] cache: flash-decoding on wave64.
//
// One block serves ONE kv head and up to G of its query heads, so with GQA the
// K/V rows are fetched from HBM once per group instead of once per query head.
// Keys are split over gridDim.y (split-KV) and over the wavefronts of a block
// in tiles of 16-64 keys. Inside a wavefront a key row is spread over the 16
// lanes of a DPP row (one or two 128-bit loads per lane, 4 keys per load step,
// fully coalesced); scores are reduced inside the row with DPP adds, parked
// one-key-per-lane so that the softmax exponentials cost one instruction per
// tile, and fed back to the P.V pass through a per-wave LDS line. Running (max, sum, acc) states
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

// ---- 16-lane reductions on DPP (no LDS round trips) ------------------------------
// A key row is spread over the 16 lanes of one DPP row, so a score is finished
// with four v_add_f32 carrying DPP modifiers: xor-1 and xor-2 inside a quad,
// then mirroring the half row and the row. Every lane of the row ends up with
// the full sum.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true);
  return v + __int_as_float(t);
}
__device__ __forceinline__ float row16_sum(float v) {
  v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);  // row_half_mirror
  v = dpp_add<0x140>(v);  // row_mirror
  return v;
}

// grid = (Hkv, S, ceil(group/G)); block = nw*64 threads (nw in 1,2,4).
// A wavefront works on tiles of TK keys (16, 32 or 64): 4 keys per load step
// (one per DPP row), each lane holding EPL = D/16 consecutive floats of its key.
// part_m/part_l: [Hq*S], part_acc: [Hq*S*D]; used when S > 1, else `out` is final.
//
// PRE = true is causal prefill over q/out [Hq, T, D]: grid = (Hq, 1, ceil(T/(4G))).
// A WAVEFRONT owns G consecutive query positions of one head, which share the K/V
// stream exactly like the query heads of a GQA group do in decode, and walks all
// of their keys itself (no merge between wavefronts). Row g sees keys
// [0, pos0 + p_g]; later keys of a tile are masked per row. Longest rows first.
template <int D, int G, typename KT, bool PRE>
__global__ __launch_bounds__(256) void attn_decode_kernel(
    const float* __restrict__ q, const KT* __restrict__ K, const KT* __restrict__ V,
    float* __restrict__ out, float* __restrict__ part_m, float* __restrict__ part_l,
    float* __restrict__ part_acc, int group, int ctx, int64_t kv_stride, int chunk, int TK,
    float scale, int S, int T, int pos0, const uint32_t* __restrict__ dpos) {
  constexpr int EPL = D / 16;        // floats of a key row per lane (4 or 8)
  constexpr int NV = EPL / 4;        // float4 loads per lane per key
  constexpr int UNR = 4;             // key steps in flight per lane
  __shared__ float pbuf[4][G][64];               // per-wave probabilities of the current tile
  __shared__ float st_m[4][G], st_l[4][G];       // per-wave softmax state for the block merge
  __shared__ float st_acc[4][G][D];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int slot = lane >> 4, c = lane & 15;     // DPP row = key slot, c = position in the row
  const int split = blockIdx.y;
  // Position kept on the device (captured decode loops): the grid was planned for
  // the cache capacity, the live context is *dpos + 1. Splits past it find no keys
  // and write neutral partials (m = -inf, l = 0, acc = 0).
  if (!PRE && dpos) ctx = min(ctx, (int)*dpos + 1);
  int kvh, g0, ng, k_begin, k_end;
  size_t row0;                                   // index of row g = 0 in q / out, in rows of D
  if constexpr (PRE) {
    const int h = blockIdx.x;
    kvh = h / group;
    // every wavefront owns G query rows of its own and walks ALL of their keys: no
    // merge between wavefronts, and the four of a block read the same K/V rows at
    // about the same time (the later ones hit in L1/L2)
    g0 = ((gridDim.z - 1 - blockIdx.z) * nw + wave) * G;   // first query position of this wavefront
    if (g0 >= T) return;                                   // (no block-wide barrier follows in this mode)
    ng = min(G, T - g0);
    row0 = (size_t)h * T + g0;
    k_begin = 0;
    k_end = pos0 + g0 + ng;                      // the last row's limit
    TK = k_end >= 64 ? 64 : k_end >= 32 ? 32 : 16;
  } else {
    kvh = blockIdx.x;
    g0 = blockIdx.z * G;
    ng = min(G, group - g0);
    row0 = (size_t)kvh * group + g0;
    k_begin = split * chunk;
    k_end = min(ctx, k_begin + chunk);
  }
  const int lim0 = pos0 + g0 + 1;                // PRE: row g sees keys < lim0 + g
  const KT* Kh = K + (size_t)kvh * kv_stride;
  const KT* Vh = V + (size_t)kvh * kv_stride;
  const int steps = TK >> 2;                     // load steps per tile

  float4 qv[G][NV];
#pragma unroll
  for (int g = 0; g < G; g++)
#pragma unroll
    for (int v = 0; v < NV; v++)
      qv[g][v] = g < ng ? *reinterpret_cast<const float4*>(q + (row0 + g) * D + c * EPL + v * 4)
                        : make_float4(0.f, 0.f, 0.f, 0.f);
  float m[G], l[G];
  float4 acc[G][NV];
#pragma unroll
  for (int g = 0; g < G; g++) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int v = 0; v < NV; v++) acc[g][v] = make_float4(0.f, 0.f, 0.f, 0.f);
  }

  const int kb_first = PRE ? 0 : k_begin + wave * TK, kb_step = PRE ? TK : nw * TK;
  for (int kb = kb_first; kb < k_end; kb += kb_step) {
    // ---- scores: lane (slot,c) ends up holding key kb + c*4 + slot (c < steps) ----
    float sreg[G];
#pragma unroll
    for (int g = 0; g < G; g++) sreg[g] = -INFINITY;
    // The tile's first V rows do not depend on the scores: request them with the K
    // rows so that one memory latency covers both.
    float4 vfirst[UNR][NV];
    for (int i0 = 0; i0 < steps; i0 += UNR) {
      float4 kv[UNR][NV];
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        const int key = kb + (i0 + u) * 4 + slot;
#pragma unroll
        for (int v = 0; v < NV; v++)
          kv[u][v] = key < k_end ? KvLoad<KT>::ld(Kh + (size_t)key * D + c * EPL + v * 4)
                                 : make_float4(0.f, 0.f, 0.f, 0.f);
      }
      if (i0 == 0) {
#pragma unroll
        for (int u = 0; u < UNR; u++) {
          const int key = kb + u * 4 + slot;
#pragma unroll
          for (int v = 0; v < NV; v++)
            vfirst[u][v] = key < k_end ? KvLoad<KT>::ld(Vh + (size_t)key * D + c * EPL + v * 4)
                                       : make_float4(0.f, 0.f, 0.f, 0.f);
        }
      }
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        const int key = kb + (i0 + u) * 4 + slot;
#pragma unroll
        for (int g = 0; g < G; g++) {
          float p = qv[g][0].x * kv[u][0].x;
          p = fmaf(qv[g][0].y, kv[u][0].y, p);
          p = fmaf(qv[g][0].z, kv[u][0].z, p);
          p = fmaf(qv[g][0].w, kv[u][0].w, p);
          if (NV > 1) {
            p = fmaf(qv[g][NV - 1].x, kv[u][NV - 1].x, p);
            p = fmaf(qv[g][NV - 1].y, kv[u][NV - 1].y, p);
            p = fmaf(qv[g][NV - 1].z, kv[u][NV - 1].z, p);
            p = fmaf(qv[g][NV - 1].w, kv[u][NV - 1].w, p);
          }
          p = row16_sum(p);
          if (c == i0 + u) sreg[g] = key < (PRE ? min(k_end, lim0 + g) : k_end) ? p * scale : -INFINITY;
        }
      }
    }
    // ---- online softmax update for the tile ---------------------------------------
#pragma unroll
    for (int g = 0; g < G; g++) {
      const float tmax = wave_max(sreg[g]);      // decode: finite, the tile holds >= 1 live key
      const float mnew = fmaxf(m[g], tmax);
      // prefill: a row may have seen no key yet (mnew = -inf); keep exp() away from inf - inf
      const float mref = (PRE && mnew == -INFINITY) ? 0.f : mnew;
      const float corr = __expf(m[g] - mref);    // 0 on the first tile (m = -inf)
      const float p = __expf(sreg[g] - mref);    // 0 for masked keys and idle lanes
      l[g] = fmaf(l[g], corr, p);
#pragma unroll
      for (int v = 0; v < NV; v++) {
        acc[g][v].x *= corr; acc[g][v].y *= corr; acc[g][v].z *= corr; acc[g][v].w *= corr;
      }
      m[g] = mnew;
      pbuf[wave][g][lane] = p;
    }
    wave_lds_sync();
    // ---- P.V: lane (slot,c) accumulates its EPL output columns over its slot's keys ----
    for (int i0 = 0; i0 < steps; i0 += UNR) {
      float4 vv[UNR][NV];
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        const int key = kb + (i0 + u) * 4 + slot;
#pragma unroll
        for (int v = 0; v < NV; v++)
          vv[u][v] = i0 == 0 ? vfirst[u][v]
                     : key < k_end ? KvLoad<KT>::ld(Vh + (size_t)key * D + c * EPL + v * 4)
                                   : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int g = 0; g < G; g++) {
        // key (step i, slot) was parked in lane slot*16 + i
        const float4 p4 = *reinterpret_cast<const float4*>(&pbuf[wave][g][slot * 16 + i0]);
        const float pp[4] = {p4.x, p4.y, p4.z, p4.w};
#pragma unroll
        for (int u = 0; u < UNR; u++)
#pragma unroll
          for (int v = 0; v < NV; v++) {
            acc[g][v].x = fmaf(pp[u], vv[u][v].x, acc[g][v].x);
            acc[g][v].y = fmaf(pp[u], vv[u][v].y, acc[g][v].y);
            acc[g][v].z = fmaf(pp[u], vv[u][v].z, acc[g][v].z);
            acc[g][v].w = fmaf(pp[u], vv[u][v].w, acc[g][v].w);
          }
      }
    }
    wave_lds_sync();  // pbuf is rewritten by the next tile
  }

  // ---- wave totals: sum l over lanes, acc over the four key slots --------------------------
#pragma unroll
  for (int g = 0; g < G; g++) {
    l[g] = wave_sum(l[g]);
#pragma unroll
    for (int v = 0; v < NV; v++) {
#pragma unroll
      for (int msk = 16; msk < 64; msk <<= 1) {
        acc[g][v].x += __shfl_xor(acc[g][v].x, msk, kWave);
        acc[g][v].y += __shfl_xor(acc[g][v].y, msk, kWave);
        acc[g][v].z += __shfl_xor(acc[g][v].z, msk, kWave);
        acc[g][v].w += __shfl_xor(acc[g][v].w, msk, kWave);
      }
      if constexpr (PRE) {   // this wavefront's rows are complete: normalise and store
        if (slot == 0 && g < ng) {
          const float inv = 1.0f / l[g];
          float4 o = acc[g][v];
          o.x *= inv; o.y *= inv; o.z *= inv; o.w *= inv;
          *reinterpret_cast<float4*>(out + (row0 + g) * D + c * EPL + v * 4) = o;
        }
      } else {
        if (slot == 0) *reinterpret_cast<float4*>(&st_acc[wave][g][c * EPL + v * 4]) = acc[g][v];
      }
    }
    if (!PRE && lane == 0) { st_m[wave][g] = m[g]; st_l[wave][g] = l[g]; }
  }
  if constexpr (PRE) return;
  __syncthreads();

  // ---- block merge (fixed wave order) and store ---------------------------------------------
  for (int e = threadIdx.x; e < ng * D; e += blockDim.x) {
    const int g = e / D, d = e - g * D;
    float M = st_m[0][g];
    for (int w = 1; w < nw; w++) M = fmaxf(M, st_m[w][g]);
    float L = 0.f, A = 0.f;
    for (int w = 0; w < nw; w++) {
      // waves (or whole blocks, with a device-side position) that saw no key weigh 0
      const float f = st_m[w][g] == -INFINITY ? 0.f : __expf(st_m[w][g] - M);
      L = fmaf(st_l[w][g], f, L);
      A = fmaf(st_acc[w][g][d], f, A);
    }
    const size_t h = row0 + g;
    if (PRE || S == 1) {
      out[h * D + d] = A / L;
    } else {
      const size_t ps = h * S + split;
      part_acc[ps * D + d] = A;
      if (d == 0) { part_m[ps] = M; part_l[ps] = L; }
    }
  }
}

// grid = Hq, block = 1024: merge the S split partials of one head. The split
// weights exp(m_s - M) are formed once per split in LDS; the threads are D
// columns x (1024/D) split groups, each summing its splits in a fixed order with
// the loads of four splits in flight, then the groups are summed in a fixed order.
__global__ __launch_bounds__(1024) void attn_combine_kernel(const float* __restrict__ part_m,
                                                            const float* __restrict__ part_l,
                                                            const float* __restrict__ part_acc,
                                                            float* __restrict__ out, int S, int D) {
  extern __shared__ float sm[];   // f[S] | red[1024]
  float* f = sm;
  float* red = sm + S;
  const int h = blockIdx.x, tid = threadIdx.x;
  const float* pm = part_m + (size_t)h * S;
  const float* pl = part_l + (size_t)h * S;
  float mx = -INFINITY;
  for (int s = tid; s < S; s += 1024) mx = fmaxf(mx, pm[s]);
  mx = wave_max(mx);
  if ((tid & 63) == 0) red[tid >> 6] = mx;
  __syncthreads();
  float M = red[0];
#pragma unroll
  for (int w = 1; w < 16; w++) M = fmaxf(M, red[w]);
  __syncthreads();
  float lsum = 0.f;
  for (int s = tid; s < S; s += 1024) {
    const float w = __expf(pm[s] - M);
    f[s] = w;
    lsum = fmaf(pl[s], w, lsum);
  }
  lsum = wave_sum(lsum);
  if ((tid & 63) == 0) red[tid >> 6] = lsum;
  __syncthreads();
  float L = red[0];
#pragma unroll
  for (int w = 1; w < 16; w++) L += red[w];
  __syncthreads();
  const int groups = 1024 / D, d = tid % D, sg = tid / D;
  const float* pa = part_acc + (size_t)h * S * D + d;
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  int s = sg;
  for (; s + 3 * groups < S; s += 4 * groups) {
    const float v0 = pa[(size_t)s * D], v1 = pa[(size_t)(s + groups) * D],
                v2 = pa[(size_t)(s + 2 * groups) * D], v3 = pa[(size_t)(s + 3 * groups) * D];
    a0 = fmaf(f[s], v0, a0);
    a1 = fmaf(f[s + groups], v1, a1);
    a2 = fmaf(f[s + 2 * groups], v2, a2);
    a3 = fmaf(f[s + 3 * groups], v3, a3);
  }
  for (; s < S; s += groups) a0 = fmaf(f[s], pa[(size_t)s * D], a0);
  red[tid] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  if (sg == 0) {
    float A = red[d];
    for (int k = 1; k < groups; k++) A += red[k * D + d];
    out[(size_t)h * D + d] = A / L;
  }
}

struct AttnPlan { int G, gz, nw, TK, S, chunk; };

// Split-KV plan. Work is cut into wave tiles of TK keys; the chip wants at least
// ~4 wavefronts per CU, so short contexts use small tiles and 4-wave blocks, and
// long contexts give every wavefront several 64-key tiles.
static AttnPlan plan_attn(int Hkv, int group, int ctx, int cus) {
  AttnPlan p{};
  // Query heads per block. A wavefront's instruction stream grows with G and, at
  // short and medium contexts, that serial stream (not bandwidth) is what a step
  // waits for: up to 4 heads per block there, and the whole group (up to 8) only
  // when the context is long enough for K/V traffic to dominate.
  const int gmax = ctx >= 16384 ? 8 : 4;
  p.G = group > 4 ? gmax : group > 2 ? 4 : group > 1 ? 2 : 1;
  p.gz = (group + p.G - 1) / p.G;
  const int base = Hkv * p.gz;
  const int64_t want_waves = (int64_t)cus * 4;
  p.TK = 64;
  while (p.TK > 16 && (int64_t)base * ((ctx + p.TK - 1) / p.TK) < want_waves) p.TK >>= 1;
  const int tiles = (ctx + p.TK - 1) / p.TK;
  p.nw = tiles >= 4 ? 4 : tiles >= 2 ? 2 : 1;
  const int block_tiles = (tiles + p.nw - 1) / p.nw;       // tiles per wave if S == 1
  int want_s = (int)((want_waves + (int64_t)base * p.nw - 1) / ((int64_t)base * p.nw));
  if (want_s < 1) want_s = 1;
  if (want_s > block_tiles) want_s = block_tiles;
  // nearest, not ceiling: 34 tiles for 32 wanted splits is 34 splits of one tile per
  // wave, not 17 of two
  int tiles_per_wave = (block_tiles + want_s / 2) / want_s;
  if (tiles_per_wave < 1) tiles_per_wave = 1;
  p.chunk = tiles_per_wave * p.nw * p.TK;
  p.S = (ctx + p.chunk - 1) / p.chunk;
  return p;
}

static size_t attn_partials_floats(int Hq, int S, int D) {
  const size_t hs = (size_t)Hq * S;
  return hs * 2 + hs * D;
}

// dpos != nullptr: ctx is the cache CAPACITY the grid is planned for, the live
// context is read from the device, and the split partials live in a buffer the
// caller owns (a captured graph bakes the address in).
template <int D, typename KT>
static int launch_attn(const float* q, const KT* K, const KT* V, float* out, int Hq, int Hkv,
                       int ctx, int64_t kv_max, float scale, const uint32_t* dpos = nullptr,
                       float* partials = nullptr, size_t partials_bytes = 0) {
  Context& c = tlhip::ctx();
  const int group = Hq / Hkv;
  const AttnPlan p = plan_attn(Hkv, group, ctx, c.cus);
  float *pm = nullptr, *pl = nullptr, *pacc = nullptr;
  if (p.S > 1) {
    const size_t hs = (size_t)Hq * p.S;
    const size_t need = attn_partials_floats(Hq, p.S, D) * sizeof(float);
    float* base;
    if (dpos) {
      if (!partials || partials_bytes < need)
        return fail(TLHIP_EINVAL, "tlhip_attn_decode_dpos: partials buffer of %zu bytes needed", need);
      base = partials;
    } else {
      base = static_cast<float*>(scratch(need));
    }
    if (!base) return fail(TLHIP_ENOMEM, "tlhip_attn_decode: no scratch for %d splits", p.S);
    pm = base;
    pl = pm + hs;
    pacc = pl + hs;
  }
  if (p.S > 65535) return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode: context too long");
  const dim3 grid(Hkv, p.S, p.gz), block(p.nw * 64);
  const int64_t kv_stride = kv_max * D;
#define TLHIP_ATTN(GG)                                                                         \
  hipLaunchKernelGGL((attn_decode_kernel<D, GG, KT, false>), grid, block, 0, c.stream, q, K, V, \
                     out, pm, pl, pacc, group, ctx, kv_stride, p.chunk, p.TK, scale, p.S, 1, 0, dpos)
  switch (p.G) {
    case 1: TLHIP_ATTN(1); break;
    case 2: TLHIP_ATTN(2); break;
    case 4: TLHIP_ATTN(4); break;
    default: TLHIP_ATTN(8); break;
  }
#undef TLHIP_ATTN
  if (p.S > 1)
    hipLaunchKernelGGL(attn_combine_kernel, dim3(Hq), dim3(1024), (size_t)(p.S + 1024) * sizeof(float),
                       c.stream, pm, pl, pacc, out, p.S, D);
  TLHIP_CHECK_LAUNCH(TLHIP_C_ATTN_DECODE);
}

template <int D, typename KT>
static int launch_prefill(const float* q, const KT* K, const KT* V, float* out, int Hq, int Hkv,
                          int T, int64_t kv_max, float scale, int pos0) {
  Context& c = tlhip::ctx();
  constexpr int G = 8;   // query positions per block
  const dim3 grid(Hq, 1, (T + 4 * G - 1) / (4 * G)), block(256);   // 4 wavefronts x G query rows
  hipLaunchKernelGGL((attn_decode_kernel<D, G, KT, true>), grid, block, 0, c.stream, q, K, V, out,
                     (float*)nullptr, (float*)nullptr, (float*)nullptr, Hq / Hkv, pos0 + T,
                     kv_max * D, 0, 64, scale, 1, T, pos0, (const uint32_t*)nullptr);
  TLHIP_CHECK_LAUNCH(TLHIP_C_ATTN_PREFILL);
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

int tlhip_attn_prefill(const void* q, const void* K, const void* V, void* out, int64_t n_q_heads,
                       int64_t n_kv_heads, int64_t T, int64_t kv_max, int64_t D, float scale,
                       int kv_bf16, int64_t pos0) {
  TLHIP_REQUIRE_READY();
  if (!q || !K || !V || !out) return fail(TLHIP_EINVAL, "tlhip_attn_prefill: null pointer");
  // the reference's gates (cuda.h:1171-1177)
  if (D != 64 && D != 128) return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_prefill: head_dim must be 64 or 128");
  if (n_kv_heads <= 0 || n_q_heads <= 0 || n_q_heads % n_kv_heads != 0)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_prefill: Hq must be a positive multiple of Hkv");
  if (T <= 0 || T > 65535) return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_prefill: need 0 < T <= 65535");
  if (pos0 < 0 || pos0 + T > kv_max) return fail(TLHIP_EINVAL, "tlhip_attn_prefill: need 0 <= pos0, pos0 + T <= kv_max");
  if (kv_max > 0x3fffffff || n_q_heads > 0x7fffffff || kv_max * D > ((int64_t)1 << 40))
    return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_prefill: shape too large");
  if (!aligned16(q) || !aligned16(K) || !aligned16(V) || !aligned16(out))
    return fail(TLHIP_EINVAL, "tlhip_attn_prefill: operands must be 16-byte aligned");
  const float* pq = static_cast<const float*>(q);
  float* po = static_cast<float*>(out);
  const int Hq = (int)n_q_heads, Hkv = (int)n_kv_heads, t = (int)T, p0 = (int)pos0;
  if (kv_bf16) {
    const uint16_t* pk = static_cast<const uint16_t*>(K);
    const uint16_t* pv = static_cast<const uint16_t*>(V);
    return D == 128 ? launch_prefill<128, uint16_t>(pq, pk, pv, po, Hq, Hkv, t, kv_max, scale, p0)
                    : launch_prefill<64, uint16_t>(pq, pk, pv, po, Hq, Hkv, t, kv_max, scale, p0);
  }
  const float* pk = static_cast<const float*>(K);
  const float* pv = static_cast<const float*>(V);
  return D == 128 ? launch_prefill<128, float>(pq, pk, pv, po, Hq, Hkv, t, kv_max, scale, p0)
                  : launch_prefill<64, float>(pq, pk, pv, po, Hq, Hkv, t, kv_max, scale, p0);
}

int64_t tlhip_attn_partials_bytes(int64_t n_q_heads, int64_t n_kv_heads, int64_t kv_max, int64_t D) {
  if (!ctx().ready || n_q_heads <= 0 || n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0 || kv_max <= 0 ||
      kv_max > 0x3fffffff || (D != 64 && D != 128))
    return 0;
  const AttnPlan p = plan_attn((int)n_kv_heads, (int)(n_q_heads / n_kv_heads), (int)kv_max, ctx().cus);
  return (int64_t)(attn_partials_floats((int)n_q_heads, p.S, (int)D) * sizeof(float)) + 16;
}

int tlhip_attn_decode_dpos(const void* q, const void* K, const void* V, void* out, int64_t n_q_heads,
                           int64_t n_kv_heads, const void* d_pos, int64_t kv_max, int64_t D,
                           float scale, int kv_bf16, void* partials, int64_t partials_bytes) {
  TLHIP_REQUIRE_READY();
  if (!q || !K || !V || !out || !d_pos) return fail(TLHIP_EINVAL, "tlhip_attn_decode_dpos: null pointer");
  if (D != 64 && D != 128) return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode_dpos: head_dim must be 64 or 128");
  if (n_kv_heads <= 0 || n_q_heads <= 0 || n_q_heads % n_kv_heads != 0)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode_dpos: Hq must be a positive multiple of Hkv");
  if (kv_max <= 0 || kv_max > 0x3fffffff || n_kv_heads > 65535 || kv_max * D > ((int64_t)1 << 40))
    return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode_dpos: shape too large");
  if (!aligned16(q) || !aligned16(K) || !aligned16(V) || !aligned16(out) || (partials && !aligned16(partials)))
    return fail(TLHIP_EINVAL, "tlhip_attn_decode_dpos: operands must be 16-byte aligned");
  const float* pq = static_cast<const float*>(q);
  float* po = static_cast<float*>(out);
  const uint32_t* dp = static_cast<const uint32_t*>(d_pos);
  float* pp = static_cast<float*>(partials);
  const size_t pb = partials_bytes > 0 ? (size_t)partials_bytes : 0;
  const int Hq = (int)n_q_heads, Hkv = (int)n_kv_heads, cap = (int)kv_max;
  if (kv_bf16) {
    const uint16_t* pk = static_cast<const uint16_t*>(K);
    const uint16_t* pv = static_cast<const uint16_t*>(V);
    return D == 128 ? launch_attn<128, uint16_t>(pq, pk, pv, po, Hq, Hkv, cap, kv_max, scale, dp, pp, pb)
                    : launch_attn<64, uint16_t>(pq, pk, pv, po, Hq, Hkv, cap, kv_max, scale, dp, pp, pb);
  }
  const float* pk = static_cast<const float*>(K);
  const float* pv = static_cast<const float*>(V);
  return D == 128 ? launch_attn<128, float>(pq, pk, pv, po, Hq, Hkv, cap, kv_max, scale, dp, pp, pb)
                  : launch_attn<64, float>(pq, pk, pv, po, Hq, Hkv, cap, kv_max, scale, dp, pp, pb);
}

}  // extern "C"
