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

// ---- fused step prologue (QKV = true) ------------------------------------------------------
// The kernel then takes the raw [q | k | v] vector of the step's projection instead of a
// finished q: every block adds the bias to its own query heads and rotates them in
// registers, and the step's new key/value row (bias, rotation, narrowing to the cache
// type) is formed in registers by wavefront 0 of split 0, which starts its running
// softmax state from it as key number one; its loads are requested together with the
// query's, so the row costs that wavefront some arithmetic and no extra memory latency.
// The block of head group 0 stores the row into the cache. Keys [0, pos) come from the cache as usual, so no block
// reads the row that is being written. The arithmetic (unfused multiplies, then one add/sub) is that of
// qkv_rope_append_kernel, so the rotated values are bit-identical to the two-kernel path.
struct QkvFuse {
  const float *bq, *bk, *bv;   // biases or nullptr
  const float2* table;         // (cos, sin) of this step's position, D/2 entries
  void *Kw, *Vw;               // the caches, writable
  int64_t kv_max;
};

// Rotates four consecutive elements of a head row. `own` holds elements d0 .. d0+3 with the bias
// added, `oth` their rotation partners (elements d -+ D/2), t0/t1 the four (cos, sin) pairs of
// j = d mod D/2, lo says whether `own` is the lower half. The arithmetic - two unfused
// multiplies, then one add or subtract - is that of the stand-alone rotation kernels.
__device__ __forceinline__ float4 rope4_pair(float4 own, float4 oth, float4 t0, float4 t1, bool lo) {
  const float4 a = lo ? own : oth;   // x0: elements j
  const float4 b = lo ? oth : own;   // x1: elements j + half
  float4 o;
  if (lo) {
    o.x = sub_rn(mul_rn(a.x, t0.x), mul_rn(b.x, t0.y));
    o.y = sub_rn(mul_rn(a.y, t0.z), mul_rn(b.y, t0.w));
    o.z = sub_rn(mul_rn(a.z, t1.x), mul_rn(b.z, t1.y));
    o.w = sub_rn(mul_rn(a.w, t1.z), mul_rn(b.w, t1.w));
  } else {
    o.x = add_rn(mul_rn(a.x, t0.y), mul_rn(b.x, t0.x));
    o.y = add_rn(mul_rn(a.y, t0.w), mul_rn(b.y, t0.z));
    o.z = add_rn(mul_rn(a.z, t1.y), mul_rn(b.z, t1.x));
    o.w = add_rn(mul_rn(a.w, t1.w), mul_rn(b.w, t1.z));
  }
  return o;
}
// x[d0..d0+4) + bias[d0..d0+4) (bias may be nullptr)
__device__ __forceinline__ float4 load_biased4(const float* __restrict__ x, const float* __restrict__ bias, int d0) {
  float4 a = *reinterpret_cast<const float4*>(x + d0);
  if (bias) {
    const float4 b4 = *reinterpret_cast<const float4*>(bias + d0);
    a.x += b4.x; a.y += b4.y; a.z += b4.z; a.w += b4.w;
  }
  return a;
}

// Stores four consecutive elements into a cache row and returns them as the cache holds them.
__device__ __forceinline__ float4 kv_store4(float* p, float4 v, bool store) {
  if (store) *reinterpret_cast<float4*>(p) = v;
  return v;
}
__device__ __forceinline__ float4 kv_store4(uint16_t* p, float4 v, bool store) {
  const uint32_t a = f32_to_bf16_rne(v.x), b = f32_to_bf16_rne(v.y), c = f32_to_bf16_rne(v.z),
                 d = f32_to_bf16_rne(v.w);
  const uint2 r = make_uint2(a | (b << 16), c | (d << 16));
  if (store) *reinterpret_cast<uint2*>(p) = r;
  return make_float4(bf16_lo(r.x), bf16_hi(r.x), bf16_lo(r.y), bf16_hi(r.y));
}

// grid = (Hkv, S, ceil(group/G)); block = nw*64 threads (nw in 1,2,4).
// A wavefront works on tiles of TK keys (16, 32 or 64): 4 keys per load step
// (one per DPP row), each lane holding EPL = D/16 floats of its key: four consecutive
// ones of each 64-element part of the row.
// part_m/part_l: [Hq*S], part_acc: [Hq*S*D]; used when S > 1, else `out` is final.
//
// PRE = true is causal prefill over q/out [Hq, T, D]: grid = (Hq, 1, ceil(T/(4G))).
// A WAVEFRONT owns G consecutive query positions of one head, which share the K/V
// stream exactly like the query heads of a GQA group do in decode, and walks all
// of their keys itself (no merge between wavefronts). Row g sees keys
// [0, pos0 + p_g]; later keys of a tile are masked per row. Longest rows first.
template <int D, int G, typename KT, bool PRE, bool QKV = false>
__global__ __launch_bounds__((!PRE && G <= 4) ? 512 : 256) void attn_decode_kernel(
    const float* __restrict__ q, const KT* __restrict__ K, const KT* __restrict__ V,
    float* __restrict__ out, float* __restrict__ part_m, float* __restrict__ part_l,
    float* __restrict__ part_acc, int group, int ctx, int64_t kv_stride, int chunk, int TK,
    float scale, int S, int T, int pos0, const uint32_t* __restrict__ dpos, QkvFuse fz, int kv_rows,
    int n_kv_heads, int n_head_groups) {
  constexpr int EPL = D / 16;        // floats of a key row per lane (4 or 8)
  constexpr int NV = EPL / 4;        // float4 loads per lane per key
  // Lane c of a row holds elements [4c, 4c+4) of each of the NV consecutive 64-element
  // parts of a key row, so that one load instruction of the 16 lanes covers 256 contiguous
  // bytes of the row (64 elements) - and, with D = 128, a rotation pair (d, d + 64) in one lane.
  const auto dim0 = [](int cc, int v) { return v * 64 + cc * 4; };
  constexpr int UNR = 4;             // key steps in flight per lane
  // Decode at short and medium contexts gives a wavefront one or two tiles, and the step
  // is a chain of memory latencies. The first K and V rows of the wavefront's first tile
  // depend on nothing but the block and wave indices (rows are clamped to the cache's
  // capacity, which is mapped memory whatever it holds), so they are requested at the very
  // top, ahead of the device-side position and of the query prologue, and masked when used.
  constexpr bool kPre = !PRE && G <= 4;
  constexpr int NWMAX = (!PRE && G <= 4) ? 8 : 4;   // wavefronts per block, at most
  __shared__ float pbuf[NWMAX][G][64];              // per-wave probabilities of the current tile
  __shared__ float st_m[NWMAX][G], st_l[NWMAX][G];  // per-wave softmax state for the block merge
  __shared__ float st_acc[NWMAX][G][D];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int slot = lane >> 4, c = lane & 15;     // DPP row = key slot, c = position in the row
  // Decode launches a 1-D grid and deals (kv head, split, head group) from the block number so
  // that the head groups of one (kv head, split) - which read the same K/V rows - run on the
  // same XCD back to back: workgroups go to the 8 XCDs round-robin by number, each XCD has an L2
  // of its own, and the second reader of a tile then finds it there instead of in HBM.
  // Block b runs on XCD b % 8 as that XCD's workgroup number b / 8; the XCD's sequence is
  // (pair, head group) with the head group fastest. Blocks past the last pair exit.
  int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
  if constexpr (!PRE) {
    const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
    bz = seq % n_head_groups;
    const int pair = (seq / n_head_groups) * 8 + xcd;
    if (pair >= n_kv_heads * S) return;          // (uniform for the block; no barrier was passed)
    bx = pair % n_kv_heads;
    by = pair / n_kv_heads;
  }
  const int split = by;
  TLHIP_MARK(0);
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
    kvh = bx;
    g0 = bz * G;
    ng = min(G, group - g0);
    row0 = (size_t)kvh * group + g0;
    k_begin = k_end = 0;                         // set below, once the position is known
  }
  const int lim0 = pos0 + g0 + 1;                // PRE: row g sees keys < lim0 + g
  const KT* Kh = K + (size_t)kvh * kv_stride;
  const KT* Vh = V + (size_t)kvh * kv_stride;
  const int steps = TK >> 2;                     // load steps per tile

  // ---- requests. A CU accepts roughly one vector memory instruction per 10 ns while misses are
  // outstanding, so at decode sizes the number of load instructions is what the first microseconds
  // cost. Decode: the block's G query rows (with bias) and the rotary table are fetched ONCE per
  // block - one float4 per thread of the first wavefronts - and reach the other wavefronts
  // through LDS; then every wavefront requests the first K and V rows of its first tile.
  // Prefill (PRE): every wavefront has query rows of its own and loads them itself.
  __shared__ float qs[PRE ? 1 : G][PRE ? 4 : D];   // decode: the block's query rows, bias added, not yet rotated
  __shared__ float tabs[PRE ? 4 : D];              // decode, QKV: (cos, sin) pairs of the step
  float4 qraw[PRE ? G : 1][NV];
  float4 q_own = make_float4(0.f, 0.f, 0.f, 0.f), q_bias = q_own, t_own = q_own;
  constexpr int QT = G * (D / 4);                  // float4s of the block's query rows
  const int tq = threadIdx.x;
  if constexpr (PRE) {
#pragma unroll
    for (int g = 0; g < G; g++) {
      const size_t r = (row0 + (size_t)min(g, ng - 1)) * D;
#pragma unroll
      for (int v = 0; v < NV; v++) qraw[g][v] = *reinterpret_cast<const float4*>(q + r + dim0(c, v));
    }
  } else {
    if (tq < QT) {
      const int gq = tq / (D / 4), dq = (tq - gq * (D / 4)) * 4;
      const size_t r = (row0 + (size_t)min(gq, ng - 1)) * D;
      q_own = *reinterpret_cast<const float4*>(q + r + dq);
      if constexpr (QKV) {
        const float* bsrc = fz.bq ? fz.bq : q;   // without a bias: any mapped address, the values are not used
        q_bias = *reinterpret_cast<const float4*>(bsrc + r + dq);
      }
    } else if (QKV && tq < QT + D / 4) {
      t_own = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(fz.table) + (tq - QT) * 4);
    }
  }
  __builtin_amdgcn_sched_barrier(0);   // (the scheduler may not move the K/V requests ahead of these)
  float4 kpre[UNR][NV], vpre[UNR][NV];
  if constexpr (kPre) {
    const size_t hoff = (size_t)bx * kv_stride;
    const int kb0 = chunk ? split * chunk + wave * TK : (split * nw + wave) * TK;
#pragma unroll
    for (int u = 0; u < UNR; u++) {
      const int key = min(kb0 + u * 4 + slot, kv_rows - 1);
#pragma unroll
      for (int v = 0; v < NV; v++) {
        kpre[u][v] = KvLoad<KT>::ld(K + hoff + (size_t)key * D + dim0(c, v));
        vpre[u][v] = KvLoad<KT>::ld(V + hoff + (size_t)key * D + dim0(c, v));
      }
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  TLHIP_MARK(7);
  float4 qv[G][NV];
  if constexpr (PRE) {
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
      for (int v = 0; v < NV; v++) qv[g][v] = g < ng ? qraw[g][v] : make_float4(0.f, 0.f, 0.f, 0.f);
  } else {
    if (tq < QT) {
      const int gq = tq / (D / 4), dq = (tq - gq * (D / 4)) * 4;
      if constexpr (QKV) {
        if (fz.bq) { q_own.x += q_bias.x; q_own.y += q_bias.y; q_own.z += q_bias.z; q_own.w += q_bias.w; }
      }
      if (gq >= ng) q_own = make_float4(0.f, 0.f, 0.f, 0.f);
      *reinterpret_cast<float4*>(&qs[gq][dq]) = q_own;
    } else if (QKV && tq < QT + D / 4) {
      *reinterpret_cast<float4*>(&tabs[(tq - QT) * 4]) = t_own;
    }
    // blocks of one or two wavefronts (short contexts) have fewer threads than there are float4s
    for (int t2 = tq + (int)blockDim.x; t2 < QT + (QKV ? D / 4 : 0); t2 += (int)blockDim.x) {
      if (t2 < QT) {
        const int gq = t2 / (D / 4), dq = (t2 - gq * (D / 4)) * 4;
        const size_t r = (row0 + (size_t)min(gq, ng - 1)) * D;
        float4 a = *reinterpret_cast<const float4*>(q + r + dq);
        if constexpr (QKV) {
          if (fz.bq) {
            const float4 b4 = *reinterpret_cast<const float4*>(fz.bq + r + dq);
            a.x += b4.x; a.y += b4.y; a.z += b4.z; a.w += b4.w;
          }
        }
        if (gq >= ng) a = make_float4(0.f, 0.f, 0.f, 0.f);
        *reinterpret_cast<float4*>(&qs[gq][dq]) = a;
      } else {
        *reinterpret_cast<float4*>(&tabs[(t2 - QT) * 4]) =
            *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(fz.table) + (t2 - QT) * 4);
      }
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
      for (int v = 0; v < NV; v++) {
        const int d0 = dim0(c, v);
        const float4 own = *reinterpret_cast<const float4*>(&qs[g][d0]);
        if constexpr (QKV) {
          const bool lo = d0 < D / 2;
          const int j0 = lo ? d0 : d0 - D / 2;
          const float4 oth = *reinterpret_cast<const float4*>(&qs[g][lo ? d0 + D / 2 : d0 - D / 2]);
          const float4 t0 = *reinterpret_cast<const float4*>(&tabs[2 * j0]);       // (c0, s0, c1, s1)
          const float4 t1 = *reinterpret_cast<const float4*>(&tabs[2 * j0 + 4]);   // (c2, s2, c3, s3)
          qv[g][v] = rope4_pair(own, oth, t0, t1, lo);
        } else {
          qv[g][v] = own;
        }
      }
  }
  // Position kept on the device (captured decode loops): the grid was planned for
  // the cache capacity, the live context is *dpos + 1. Splits past it find no keys
  // and write neutral partials (m = -inf, l = 0, acc = 0).
  if (!PRE && !QKV && dpos) ctx = min(ctx, (int)*dpos + 1);
  // QKV: the step's position; keys [0, pos) are in the cache, key pos is formed here
  // (a full cache takes no new row: the step attends to what the cache holds).
  int64_t new_pos = 0;
  bool has_new = false;
  if constexpr (QKV) {
    new_pos = dpos ? (int64_t)*dpos : (int64_t)ctx - 1;
    has_new = new_pos < fz.kv_max;
    ctx = (int)min(new_pos, fz.kv_max);
  }
  if constexpr (!PRE) {
    // Two ways to deal tiles. chunk > 0: split s owns keys [s * chunk, (s + 1) * chunk) and its
    // wavefronts alternate over the tiles of that range (long per-head streams read best
    // this way). chunk == 0: round-robin over all wavefronts of all splits, wavefront w of
    // split s takes tiles (s * nw + w) + j * (S * nw); that deal does not depend on the
    // context length, so a grid planned for the cache capacity (position on the device)
    // keeps every split busy at any live context.
    k_begin = split * chunk;
    k_end = chunk ? min(ctx, k_begin + chunk) : ctx;
  }
  TLHIP_MARK(1);
  float m[G], l[G];
  float4 acc[G][NV];
#pragma unroll
  for (int g = 0; g < G; g++) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int v = 0; v < NV; v++) acc[g][v] = make_float4(0.f, 0.f, 0.f, 0.f);
  }

  // ---- the step's own key/value row: the first key of split 0's first wavefront -----------
  // (its loads travel with the query's, so it costs that wavefront arithmetic only)
  if constexpr (QKV) {
    if (split == 0 && wave == 0 && has_new) {
      const int Hkv = n_kv_heads, Hq = Hkv * group;
      const float* kraw = q + (size_t)(Hq + kvh) * D;
      const float* vraw = q + (size_t)(Hq + Hkv + kvh) * D;
      KT* krow = static_cast<KT*>(fz.Kw) + (size_t)kvh * kv_stride + (size_t)new_pos * D;
      KT* vrow = static_cast<KT*>(fz.Vw) + (size_t)kvh * kv_stride + (size_t)new_pos * D;
      const bool store = bz == 0 && slot == 0;
      float4 kn[NV], vn[NV];
#pragma unroll
      for (int v = 0; v < NV; v++) {
        const int d0 = dim0(c, v);
        const bool lo = d0 < D / 2;
        const int j0 = lo ? d0 : d0 - D / 2;
        const float* kb = fz.bk ? fz.bk + (size_t)kvh * D : nullptr;
        const float4 kr = rope4_pair(load_biased4(kraw, kb, d0), load_biased4(kraw, kb, lo ? d0 + D / 2 : d0 - D / 2),
                                     *reinterpret_cast<const float4*>(fz.table + j0),
                                     *reinterpret_cast<const float4*>(fz.table + j0 + 2), lo);
        const float4 vr = load_biased4(vraw, fz.bv ? fz.bv + (size_t)kvh * D : nullptr, d0);
        kn[v] = kv_store4(krow + d0, kr, store);
        vn[v] = kv_store4(vrow + d0, vr, store);
      }
#pragma unroll
      for (int g = 0; g < G; g++) {
        float p = qv[g][0].x * kn[0].x;
        p = fmaf(qv[g][0].y, kn[0].y, p);
        p = fmaf(qv[g][0].z, kn[0].z, p);
        p = fmaf(qv[g][0].w, kn[0].w, p);
        if (NV > 1) {
          p = fmaf(qv[g][NV - 1].x, kn[NV - 1].x, p);
          p = fmaf(qv[g][NV - 1].y, kn[NV - 1].y, p);
          p = fmaf(qv[g][NV - 1].z, kn[NV - 1].z, p);
          p = fmaf(qv[g][NV - 1].w, kn[NV - 1].w, p);
        }
        // the state is still empty: the key's weight is exp(0) = 1 (l, acc are per-lane and
        // per-slot partials that are summed later, so one lane and one slot carry it)
        m[g] = row16_sum(p) * scale;               // the same in all four slots
        l[g] = lane == 0 ? 1.f : 0.f;
#pragma unroll
        for (int v = 0; v < NV; v++)
          acc[g][v] = slot == 0 ? vn[v] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
  }

  TLHIP_MARK(2);
  const int kb_first = PRE ? 0 : chunk ? k_begin + wave * TK : (split * nw + wave) * TK;
  const int kb_step = PRE ? TK : chunk ? nw * TK : S * nw * TK;
  for (int kb = kb_first; kb < k_end; kb += kb_step) {
    // ---- scores: lane (slot,c) ends up holding key kb + c*4 + slot (c < steps) ----
    float sreg[G];
#pragma unroll
    for (int g = 0; g < G; g++) sreg[g] = -INFINITY;
    // The tile's first V rows do not depend on the scores: request them with the K
    // rows so that one memory latency covers both.
    float4 vfirst[UNR][NV];
    const bool pre_tile = kPre && kb == kb_first;   // its first rows were requested at the top
    for (int i0 = 0; i0 < steps; i0 += UNR) {
      float4 kv[UNR][NV];
      if (pre_tile && i0 == 0) {
#pragma unroll
        for (int u = 0; u < UNR; u++) {
          const bool live = kb + u * 4 + slot < k_end;   // masked keys: finite K, zero V
#pragma unroll
          for (int v = 0; v < NV; v++) {
            kv[u][v] = live ? kpre[u][v] : make_float4(0.f, 0.f, 0.f, 0.f);
            vfirst[u][v] = live ? vpre[u][v] : make_float4(0.f, 0.f, 0.f, 0.f);
          }
        }
      } else {
#pragma unroll
        for (int u = 0; u < UNR; u++) {
          const int key = kb + (i0 + u) * 4 + slot;
#pragma unroll
          for (int v = 0; v < NV; v++)
            kv[u][v] = key < k_end ? KvLoad<KT>::ld(Kh + (size_t)key * D + dim0(c, v))
                                   : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        if (i0 == 0) {
#pragma unroll
          for (int u = 0; u < UNR; u++) {
            const int key = kb + u * 4 + slot;
#pragma unroll
            for (int v = 0; v < NV; v++)
              vfirst[u][v] = key < k_end ? KvLoad<KT>::ld(Vh + (size_t)key * D + dim0(c, v))
                                         : make_float4(0.f, 0.f, 0.f, 0.f);
          }
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
                     : key < k_end ? KvLoad<KT>::ld(Vh + (size_t)key * D + dim0(c, v))
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

  TLHIP_MARK(3);
  // ---- wave totals: sum l over lanes, acc over the four key slots --------------------------
#pragma unroll
  for (int g = 0; g < G; g++) {
    l[g] = wave_sum(l[g]);
#pragma unroll
    for (int v = 0; v < NV; v++) {
      {   // + the value 16 lanes away, then + the value 32 lanes away
        const auto both = [](float a) {
          LanePair p = swap16(a, a);
          a = p.first + p.second;
          p = swap32(a, a);
          return p.first + p.second;
        };
        acc[g][v].x = both(acc[g][v].x);
        acc[g][v].y = both(acc[g][v].y);
        acc[g][v].z = both(acc[g][v].z);
        acc[g][v].w = both(acc[g][v].w);
      }
      if constexpr (PRE) {   // this wavefront's rows are complete: normalise and store
        if (slot == 0 && g < ng) {
          const float inv = 1.0f / l[g];
          float4 o = acc[g][v];
          o.x *= inv; o.y *= inv; o.z *= inv; o.w *= inv;
          *reinterpret_cast<float4*>(out + (row0 + g) * D + dim0(c, v)) = o;
        }
      } else {
        if (slot == 0) *reinterpret_cast<float4*>(&st_acc[wave][g][dim0(c, v)]) = acc[g][v];
      }
    }
    if (!PRE && lane == 0) { st_m[wave][g] = m[g]; st_l[wave][g] = l[g]; }
  }
  if constexpr (PRE) return;
  TLHIP_MARK(4);
  __syncthreads();
  TLHIP_MARK(5);

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
  TLHIP_MARK(6);
}

// grid = Hq, block = 1024: merge the S split partials of one head. The threads are D
// columns x (1024/D) split groups. The kernel is a chain of memory latencies and little
// else, so with up to 8 splits per group (S <= 64 at D = 128) every load - the partial
// maxima and sums and the thread's own accumulator values - is requested at the top and
// waited for once; the split weights exp(m_s - M) are formed once per split in LDS, each
// thread sums its splits in a fixed order and the groups are summed in a fixed order.
__global__ __launch_bounds__(1024) void attn_combine_kernel(const float* __restrict__ part_m,
                                                            const float* __restrict__ part_l,
                                                            const float* __restrict__ part_acc,
                                                            float* __restrict__ out, int S, int D) {
  extern __shared__ float sm[];   // f[S] | red[1024]
  float* f = sm;
  float* red = sm + S;
  constexpr int kUp = 8;          // accumulator loads a thread issues up front
  const int h = blockIdx.x, tid = threadIdx.x;
  const float* pm = part_m + (size_t)h * S;
  const float* pl = part_l + (size_t)h * S;
  const int groups = 1024 / D, d = tid % D, sg = tid / D;
  const float* pa = part_acc + (size_t)h * S * D + d;
  const bool upfront = S <= kUp * groups;        // (then S <= 1024 as well)
  float pv[kUp], my_m = -INFINITY, my_l = 0.f;
  if (upfront) {
#pragma unroll
    for (int u = 0; u < kUp; u++) {
      const int s = sg + u * groups;
      pv[u] = s < S ? pa[(size_t)s * D] : 0.f;
    }
    if (tid < S) { my_m = pm[tid]; my_l = pl[tid]; }
  }
  float mx = my_m;
  if (!upfront)
    for (int s = tid; s < S; s += 1024) mx = fmaxf(mx, pm[s]);
  mx = wave_max(mx);
  if ((tid & 63) == 0) red[tid >> 6] = mx;
  __syncthreads();
  float M = red[0];
#pragma unroll
  for (int w = 1; w < 16; w++) M = fmaxf(M, red[w]);
  __syncthreads();
  float lsum = 0.f;
  if (upfront) {
    if (tid < S) {
      const float w = __expf(my_m - M);
      f[tid] = w;
      lsum = my_l * w;
    }
  } else {
    for (int s = tid; s < S; s += 1024) {
      const float w = __expf(pm[s] - M);
      f[s] = w;
      lsum = fmaf(pl[s], w, lsum);
    }
  }
  lsum = wave_sum(lsum);
  if ((tid & 63) == 0) red[tid >> 6] = lsum;
  __syncthreads();
  float L = red[0];
#pragma unroll
  for (int w = 1; w < 16; w++) L += red[w];
  __syncthreads();
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  if (upfront) {
#pragma unroll
    for (int u = 0; u < kUp; u += 4) {
      const int s = sg + u * groups;
      a0 = fmaf(s < S ? f[s] : 0.f, pv[u], a0);
      a1 = fmaf(s + groups < S ? f[s + groups] : 0.f, pv[u + 1], a1);
      a2 = fmaf(s + 2 * groups < S ? f[s + 2 * groups] : 0.f, pv[u + 2], a2);
      a3 = fmaf(s + 3 * groups < S ? f[s + 3 * groups] : 0.f, pv[u + 3], a3);
    }
  } else {
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
  }
  red[tid] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  if (sg == 0) {
    float A = red[d];
    for (int k = 1; k < groups; k++) A += red[k * D + d];
    out[(size_t)h * D + d] = A / L;
  }
}

// ---- decode attention for a GQA group: one block per (kv head, split), one wavefront per head ----
//
// At the decode sizes of a GQA model (7 query heads per kv head, a few thousand keys) a step is
// not bound by bandwidth but by two other things: how many load instructions a CU has to issue
// (about one 1 KB instruction per 10 ns while misses are outstanding) and how long each
// wavefront's own instruction stream is. The kernel above lets two blocks fetch the K/V rows of a
// kv head (one per half of the head group) and pays the per-head costs - the softmax update, the
// sums over key slots at the end - once per head AND wavefront, then merges the wavefronts of a
// block through LDS. Here:
//   * a block owns a (kv head, split) pair and ALL of the group's query heads: a 64-key tile of K
//     and of V is copied global -> LDS once per CU, without passing through registers
//     (global_load_lds, 1 KB of whole rows per instruction, requested before anything else);
//   * wavefront h of the block serves query head h over the whole tile, so the running softmax
//     state of a (head, split) lives in ONE wavefront: nothing is merged inside the block, and the
//     per-head costs are paid once per head; the last wavefront serves no head: it copies, and in
//     the fused form it makes the step's new key/value row;
//   * scores: lane = key. A lane walks its key's row in LDS 16 bytes at a time against the query
//     row, which every lane reads from the same LDS address (a broadcast): 4 FMAs per two LDS
//     reads and no cross-lane step at all. The row's 16-byte chunks are stored XOR-swizzled by the
//     key number (chunk j of key k at position j ^ (k mod CH)) - the copy chooses which global
//     chunk each lane fetches, so this costs nothing - which spreads the 64 lanes' reads, 512 bytes
//     apart, over all banks;
//   * the softmax maximum and sum are plain wavefront reductions over the 64 keys;
//   * P.V: lane = (key group, 4 output columns): CH = D/4 lanes cover a V row (a contiguous,
//     conflict-free LDS read), the 64/CH key groups take KPG = CH keys each, probabilities are
//     read from a per-head LDS line (the lanes of a group read the same address), and the key
//     groups are added up at the very end with one or two register swaps per column.
// Tiles are dealt round-robin over the splits (tile t to split t mod S); a block whose split holds
// several tiles (long contexts, or a context past what the planned grid covers at one tile each)
// copies the next tile into a second LDS stage while it works on the current one. The deal does
// not depend on the live context, so a grid planned for the cache capacity (position on the
// device) and one planned for the live context give the same bits: splits without keys write
// neutral partials, which add exact zeros in the combine.
// QKV: as in the kernel above, the raw [q | k | v] projection comes in; the block's query rows get
// their bias and rotation on the way into LDS, and the block whose tile holds the step's position
// forms the new key/value row (same arithmetic as the stand-alone epilogue, so cache rows are
// bit-identical), stores it into the cache and uses it from LDS in place of the stale cache row.
namespace gqa {

constexpr int kKeys = 64;   // keys per tile: the lanes of a wavefront

template <int D> struct Geo {
  static constexpr int CH = D / 4;               // 16-byte chunks per row
  static constexpr int RB = D * 4;               // bytes per row
  static constexpr int KG = 64 / CH;             // key groups of the P.V pass
  static constexpr int TILE = kKeys * RB;        // bytes of a tile's K (or V) rows
  static constexpr int RPI = 1024 / RB;          // rows per 1 KB copy
  static constexpr int COPIES = 2 * kKeys / RPI; // 1 KB copies per tile (K and V)
};

template <int D> inline size_t lds_bytes(int group, int stages) {
  return (size_t)stages * 2 * Geo<D>::TILE + (size_t)(2 * D + 2 * group * D + D + group * 64) * sizeof(float);
}

template <int D, int GRP, bool QKV>
__global__ __launch_bounds__(64 * (GRP + 1)) void attn_gqa_kernel(
    const float* __restrict__ q, const float* __restrict__ K, const float* __restrict__ V,
    float* __restrict__ out, float* __restrict__ part_m, float* __restrict__ part_l,
    float* __restrict__ part_acc, int ctx, int64_t kv_stride, float scale, int S,
    const uint32_t* __restrict__ dpos, QkvFuse fz, int kv_rows, int n_kv_heads, int stages) {
  using Gm = Geo<D>;
  constexpr int CH = Gm::CH, RB = Gm::RB, KG = Gm::KG, TILE = Gm::TILE, RPI = Gm::RPI;
  constexpr int NW = GRP + 1;
  constexpr int CPW = (Gm::COPIES / 2 + NW - 1) / NW;        // 1 KB copies per wavefront and tile, of K and again of V
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int lane = threadIdx.x & 63, tq = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kvh = blockIdx.x % n_kv_heads, split = blockIdx.x / n_kv_heads;
  char* extra = smem + (size_t)stages * 2 * TILE;
  float* newk = reinterpret_cast<float*>(extra);             // the step's own key / value row (QKV)
  float* newv = newk + D;
  float* qs = newv + D;                                      // QKV: the query rows with bias, not yet rotated
  float* qrot = qs + GRP * D;                                // the query rows the scores use
  float* tabs = qrot + GRP * D;                              // QKV: (cos, sin) pairs of the step
  float* pb = tabs + D;                                      // [GRP][64] probabilities of the current tile
  const float* Kh = K + (size_t)kvh * kv_stride;
  const float* Vh = V + (size_t)kvh * kv_stride;

  // A block barrier without the fence __syncthreads() carries: that fence waits for every copy
  // in flight (they write LDS). What has to be complete is waited for by count instead.
  auto barrier = [] {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  // this wavefront's copies of tile t into `stage`: rows past the cache's capacity are clamped
  // (mapped memory whatever it holds; such keys are masked where they are used)
  // (all of a wavefront's K copies go out before its V copies: loads land in order, so the scores
  // can start when "all but my CPW youngest" have landed)
  auto copy_tile = [&](int t, char* stage) {
#pragma unroll
    for (int half = 0; half < 2; half++)
#pragma unroll
      for (int i = 0; i < CPW; i++) {
        const int rp = min(wave + i * NW, Gm::COPIES / 2 - 1);   // (a spare slot repeats the last copy)
        const int r = rp * RPI + lane / CH;                      // row of the tile
        const int j = (lane % CH) ^ (r & (CH - 1));              // the chunk that belongs at this lane's position
        const int key = min(t * kKeys + r, kv_rows - 1);
        const float* src = (half ? Vh : Kh) + (size_t)key * D + j * 4;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)(stage + half * TILE + rp * 1024),
                                         16, 0, 0);
      }
  };

  // ---- requests, oldest first: the query rows (a few), then the first tile -----------------------
  TLHIP_MARK(0);
  constexpr int QT = GRP * CH;                               // float4s of the block's query rows
  float4 q_own = make_float4(0.f, 0.f, 0.f, 0.f), q_bias = q_own;
  if (tq < QT) {
    const size_t r = ((size_t)kvh * GRP + tq / CH) * D + (tq % CH) * 4;
    q_own = *reinterpret_cast<const float4*>(q + r);
    if (QKV && fz.bq) q_bias = *reinterpret_cast<const float4*>(fz.bq + r);
  } else if (QKV && tq < QT + D / 4) {
    q_own = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(fz.table) + (tq - QT) * 4);
  }
  // QKV: what the step's own key/value row is made of, requested now by the wavefront that serves
  // no head (in every block: which block needs it depends on the position, which may live on the
  // device and is not known yet)
  float4 nk_own = q_own, nk_oth = q_own, nv_own = q_own, nt0 = q_own, nt1 = q_own;
  const int nd0 = (lane % CH) * 4;
  const bool nlo = nd0 < D / 2;
  if (QKV && wave == GRP) {
    const int Hq = n_kv_heads * GRP;
    const float* kraw = q + (size_t)(Hq + kvh) * D;
    const float* vraw = q + (size_t)(Hq + n_kv_heads + kvh) * D;
    const int j0 = nlo ? nd0 : nd0 - D / 2;
    nk_own = load_biased4(kraw, fz.bk ? fz.bk + (size_t)kvh * D : nullptr, nd0);
    nk_oth = load_biased4(kraw, fz.bk ? fz.bk + (size_t)kvh * D : nullptr, nlo ? nd0 + D / 2 : nd0 - D / 2);
    nv_own = load_biased4(vraw, fz.bv ? fz.bv + (size_t)kvh * D : nullptr, nd0);
    nt0 = *reinterpret_cast<const float4*>(fz.table + j0);
    nt1 = *reinterpret_cast<const float4*>(fz.table + j0 + 2);
  }
  __builtin_amdgcn_sched_barrier(0);
  copy_tile(split, smem);
  __builtin_amdgcn_sched_barrier(0);
  TLHIP_MARK(7);

  // ---- the position, the live context, who makes the new row -------------------------------------
  int64_t new_pos = 0;
  bool has_new = false;
  if constexpr (QKV) {
    new_pos = dpos ? (int64_t)*dpos : (int64_t)ctx - 1;
    has_new = new_pos < fz.kv_max;
    ctx = (int)min(new_pos, fz.kv_max) + (has_new ? 1 : 0);  // keys [0, pos) of the cache and the new one
  } else if (dpos) {
    ctx = min(ctx, (int)*dpos + 1);
  }
  const int newt = (int)(new_pos / kKeys), newj = (int)(new_pos % kKeys);
  const bool owner = QKV && has_new && newt % S == split;    // this block's tiles include the step's position

  // ---- query rows into LDS (the copies stay in flight: wait for what is older than them) ----------
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * CPW) : "memory");
  if (tq < QT) {
    if constexpr (QKV) {
      q_own.x += q_bias.x; q_own.y += q_bias.y; q_own.z += q_bias.z; q_own.w += q_bias.w;
      *reinterpret_cast<float4*>(qs + (tq / CH) * D + (tq % CH) * 4) = q_own;
    } else {
      *reinterpret_cast<float4*>(qrot + (tq / CH) * D + (tq % CH) * 4) = q_own;
    }
  } else if (QKV && tq < QT + D / 4) {
    *reinterpret_cast<float4*>(tabs + (tq - QT) * 4) = q_own;
  }
  if constexpr (QKV) {
    barrier();
    if (tq < QT) {
      const int g = tq / CH, d0 = (tq % CH) * 4;
      const bool lo = d0 < D / 2;
      const int j0 = lo ? d0 : d0 - D / 2;
      const float4 own = *reinterpret_cast<const float4*>(qs + g * D + d0);
      const float4 oth = *reinterpret_cast<const float4*>(qs + g * D + (lo ? d0 + D / 2 : d0 - D / 2));
      const float4 t0 = *reinterpret_cast<const float4*>(tabs + 2 * j0);        // (c0, s0, c1, s1)
      const float4 t1 = *reinterpret_cast<const float4*>(tabs + 2 * j0 + 4);    // (c2, s2, c3, s3)
      *reinterpret_cast<float4*>(qrot + g * D + d0) = rope4_pair(own, oth, t0, t1, lo);
    }
    // the step's own key/value row: formed by the wavefront that serves no head, kept in LDS for
    // this block's scores and stored into the cache (rows of other tiles belong to other blocks)
    if (owner && wave == GRP && lane < CH) {
      float* krow = static_cast<float*>(fz.Kw) + (size_t)kvh * kv_stride + (size_t)new_pos * D;
      float* vrow = static_cast<float*>(fz.Vw) + (size_t)kvh * kv_stride + (size_t)new_pos * D;
      const float4 kr = rope4_pair(nk_own, nk_oth, nt0, nt1, nlo);
      *reinterpret_cast<float4*>(krow + nd0) = kr;
      *reinterpret_cast<float4*>(vrow + nd0) = nv_own;
      *reinterpret_cast<float4*>(newk + nd0) = kr;
      *reinterpret_cast<float4*>(newv + nd0) = nv_own;
    }
  }
  // ---- the tiles of this split ---------------------------------------------------------------------
  const int h = wave;                                        // the query head this wavefront serves (wave GRP: none)
  const int cg = lane % CH, kg = lane / CH;
  // While the tile is on its way: every lane of a head's wavefront takes the whole query row
  // into registers (reads of one LDS address by all lanes). The scores then read LDS for the keys
  // only - they are bound by the LDS pipe, and the query reads were half of its traffic. (Blocks
  // of more than eight wavefronts leave a lane fewer registers than the row needs at head size
  // 128; they read the row from LDS as they go.)
  constexpr bool QREG = D == 64 || NW <= 8;
  float4 qreg[QREG ? CH : 1];
  barrier();                                                 // the rotated query rows (and the new row) are in LDS
  if (QREG && h < GRP) {
#pragma unroll
    for (int j = 0; j < CH; j++) qreg[j] = *reinterpret_cast<const float4*>(qrot + h * D + j * 4);
  }
  TLHIP_MARK(1);
  float m = -INFINITY, l = 0.f;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  int st = 0;
  bool first = true;
  // The first tile is used as it lands: its K rows (and the query rows, and the new row) are
  // waited for, the scores and the softmax run while its V rows are still on their way. A later
  // tile has landed whole by the time its turn comes (it was copied during the tile before it).
  for (int t = split; t * kKeys < ctx; t += S) {
    char* stage = smem + (size_t)st * 2 * TILE;
    const int tn = t + S;
    const bool more = tn * kKeys < ctx;
    if (first) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(CPW) : "memory");     // my K copies of the first tile
      TLHIP_MARK(5);
      barrier();                                                     // ... and everyone's; query rows and the new row too
      TLHIP_MARK(2);
    }
    if (more) copy_tile(tn, smem + (size_t)(st ^ 1) * 2 * TILE);   // (stages == 2 whenever a split holds two tiles)
    const int nvalid = min(kKeys, ctx - t * kKeys);          // >= 1
    const bool with_new = QKV && has_new && t == newt;       // key newj of this tile is the new row
    const bool plain = nvalid == kKeys && !with_new;
    if (h < GRP) {
      // scores: lane = key
      // (rows start at multiples of the row size, so "row + (chunk position)" is an XOR: one
      // instruction per read for the swizzle and the address together)
      const bool mine_new = with_new && lane == newj;
      const uint32_t kx = mine_new ? (uint32_t)(reinterpret_cast<const char*>(newk) - smem)
                                   : ((uint32_t)(stage - smem) + lane * RB) ^ ((lane & (CH - 1)) << 4);
      const float* qh = qrot + h * D;
      float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
      for (int j = 0; j < CH; j += 4) {
        const float4 k0 = *reinterpret_cast<const float4*>(smem + (kx ^ ((j + 0) << 4)));
        const float4 k1 = *reinterpret_cast<const float4*>(smem + (kx ^ ((j + 1) << 4)));
        const float4 k2 = *reinterpret_cast<const float4*>(smem + (kx ^ ((j + 2) << 4)));
        const float4 k3 = *reinterpret_cast<const float4*>(smem + (kx ^ ((j + 3) << 4)));
        const float4 q0 = QREG ? qreg[QREG ? j + 0 : 0] : *reinterpret_cast<const float4*>(qh + (j + 0) * 4);
        const float4 q1 = QREG ? qreg[QREG ? j + 1 : 0] : *reinterpret_cast<const float4*>(qh + (j + 1) * 4);
        const float4 q2 = QREG ? qreg[QREG ? j + 2 : 0] : *reinterpret_cast<const float4*>(qh + (j + 2) * 4);
        const float4 q3 = QREG ? qreg[QREG ? j + 3 : 0] : *reinterpret_cast<const float4*>(qh + (j + 3) * 4);
        s0 = fmaf(q0.x, k0.x, s0); s0 = fmaf(q0.y, k0.y, s0); s0 = fmaf(q0.z, k0.z, s0); s0 = fmaf(q0.w, k0.w, s0);
        s1 = fmaf(q1.x, k1.x, s1); s1 = fmaf(q1.y, k1.y, s1); s1 = fmaf(q1.z, k1.z, s1); s1 = fmaf(q1.w, k1.w, s1);
        s2 = fmaf(q2.x, k2.x, s2); s2 = fmaf(q2.y, k2.y, s2); s2 = fmaf(q2.z, k2.z, s2); s2 = fmaf(q2.w, k2.w, s2);
        s3 = fmaf(q3.x, k3.x, s3); s3 = fmaf(q3.y, k3.y, s3); s3 = fmaf(q3.z, k3.z, s3); s3 = fmaf(q3.w, k3.w, s3);
      }
      const float sc = lane < nvalid ? ((s0 + s1) + (s2 + s3)) * scale : -INFINITY;
      // online softmax over the tile's keys: m and l are the same in every lane
      const float mnew = fmaxf(m, wave_max(sc));             // finite: the tile holds a live key
      const float corr = __expf(m - mnew);                   // 0 on the first tile (m = -inf)
      const float p = __expf(sc - mnew);                     // 0 for masked keys
      l = fmaf(l, corr, wave_sum(p));
      acc.x *= corr; acc.y *= corr; acc.z *= corr; acc.w *= corr;
      m = mnew;
      pb[h * 64 + lane] = p;
      wave_lds_sync();
      TLHIP_MARK(3);
    }
    if (first) {                                             // the first tile's V rows
      if (more) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * CPW) : "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      barrier();
      first = false;
    }
    if (h < GRP) {
      // P.V: lane = (key group kg, columns 4 cg .. 4 cg + 3)
      const char* vt = stage + TILE;
      const float* ph = pb + h * 64 + kg * CH;
      if (plain) {
        const uint32_t vx = ((uint32_t)(vt - smem) + kg * CH * RB) ^ (cg << 4);   // the group's first row, this lane's chunk
#pragma unroll
        for (int i = 0; i < CH; i += 4) {
          const float4 p4 = *reinterpret_cast<const float4*>(ph + i);
          const float pp[4] = {p4.x, p4.y, p4.z, p4.w};
#pragma unroll
          for (int u = 0; u < 4; u++) {
            const float4 v = *reinterpret_cast<const float4*>(smem + (vx ^ ((i + u) << 4)) + (i + u) * RB);
            acc.x = fmaf(pp[u], v.x, acc.x); acc.y = fmaf(pp[u], v.y, acc.y);
            acc.z = fmaf(pp[u], v.z, acc.z); acc.w = fmaf(pp[u], v.w, acc.w);
          }
        }
      } else {
        // the tile at the end of the context, or the one that holds the new row: a masked key
        // (weight 0) reads the last live row instead of its own, which may hold anything
#pragma unroll 4
        for (int i = 0; i < CH; i++) {
          const int row = min(kg * CH + i, nvalid - 1);
          const char* vrow = with_new && row == newj ? reinterpret_cast<const char*>(newv) + (cg << 4)
                                                     : vt + row * RB + ((cg ^ (row & (CH - 1))) << 4);
          const float4 v = *reinterpret_cast<const float4*>(vrow);
          const float pp = ph[i];
          acc.x = fmaf(pp, v.x, acc.x); acc.y = fmaf(pp, v.y, acc.y);
          acc.z = fmaf(pp, v.z, acc.z); acc.w = fmaf(pp, v.w, acc.w);
        }
      }
    }
    if (more) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // the next tile has landed (my copies) ...
      barrier();                                             // ... everyone's; and this stage is free again
    }
    st ^= 1;
  }

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");           // (a block without keys still has its copies in flight)
  // ---- add up the key groups and store ----------------------------------------------------------------
  TLHIP_MARK(4);
  if (h < GRP) {
    const auto across = [](float a) {
      if (KG == 4) {
        const LanePair p16 = swap16(a, a);
        a = p16.first + p16.second;
      }
      const LanePair p32 = swap32(a, a);
      return p32.first + p32.second;
    };
    acc.x = across(acc.x); acc.y = across(acc.y); acc.z = across(acc.z); acc.w = across(acc.w);
    if (lane < CH) {
      const size_t head = (size_t)kvh * GRP + h;
      if (S == 1 && out) {
        // (divisions, as in the combine kernel: a grid with one split and one with more give the same bits)
        *reinterpret_cast<float4*>(out + head * D + lane * 4) = make_float4(acc.x / l, acc.y / l, acc.z / l, acc.w / l);
      } else {
        const size_t ps = head * S + split;
        *reinterpret_cast<float4*>(part_acc + ps * D + lane * 4) = acc;   // zeros, -inf, 0 where the split held no key
        if (lane == 0) { part_m[ps] = m; part_l[ps] = l; }
      }
    }
  }
  TLHIP_MARK(6);
}

}  // namespace gqa

struct AttnPlan { int G, gz, nw, TK, S, chunk; };

// Split-KV plan. Work is cut into wave tiles of TK keys; the chip wants 4 to 8
// wavefronts per CU, so short contexts use small tiles and 4-wave blocks, and
// long contexts give every wavefront several 64-key tiles. chunk == 0: tiles are
// dealt round-robin over the S * nw wavefronts of a kv head.
static AttnPlan plan_attn(int Hkv, int group, int ctx, int cus, bool fixed_grid) {
  AttnPlan p{};
  // Query heads per block. A wavefront's instruction stream grows with G and, at
  // short and medium contexts, that serial stream (not bandwidth) is what a step
  // waits for: up to 4 heads per block there, and the whole group (up to 8) only
  // when the context is long enough for K/V traffic to dominate.
  const int gmax = ctx >= 16384 ? 8 : 4;
  p.G = group > 4 ? gmax : group > 2 ? 4 : group > 1 ? 2 : 1;
  p.gz = (group + p.G - 1) / p.G;
  const int base = Hkv * p.gz;
  // 8-wavefront blocks of 16-key tiles (every K/V row of a tile is then requested at the
  // top of the kernel and the tile costs one memory latency) once such blocks still cover
  // every CU; below that, 4-wavefront blocks spread a short context over more CUs.
  const bool wide = p.G <= 4 && (int64_t)base * ((ctx + 127) / 128) >= cus;
  const int64_t want_waves = (int64_t)cus * (wide ? 8 : 4);
  p.TK = 64;
  while (p.TK > 16 && (int64_t)base * ((ctx + p.TK - 1) / p.TK) < want_waves) p.TK >>= 1;
  const int tiles = (ctx + p.TK - 1) / p.TK;
  p.nw = wide && tiles >= 8 ? 8 : tiles >= 4 ? 4 : tiles >= 2 ? 2 : 1;
  // Splits: enough for want_waves wavefronts, no more than there are rows of nw tiles, and
  // no more blocks than run at once (a block left for a second round would double the
  // step): 8-wavefront blocks and the 8-head kernel fill a CU's registers alone, the
  // smaller 4-wavefront blocks fit two to a CU.
  const int tile_rows = (tiles + p.nw - 1) / p.nw;
  const int at_once = cus * ((wide || p.G > 4) ? 1 : 2);
  int S = (int)((want_waves + (int64_t)base * p.nw - 1) / ((int64_t)base * p.nw));
  if (S > tile_rows) S = tile_rows;
  if (S > at_once / base) S = at_once / base;
  p.S = S < 1 ? 1 : S;
  // Many kv heads with one query head each (no GQA sharing) at a long context is a plain
  // bandwidth problem, and there long contiguous per-split streams measured best: 8 x 64-key
  // tiles per block round, at least 1024 keys per split, at most two blocks per CU. (Needs
  // the context length when the grid is built, so not with a device-side position.)
  if (!fixed_grid && p.G == 1 && wide && ctx >= 4096 && (int64_t)base * (ctx / 1024) >= cus / 2) {
    p.TK = 64;
    p.nw = 8;
    const int rows = (ctx + 511) / 512;                        // rounds of 8 tiles
    int want = ctx / 1024 < 2 * cus / base ? ctx / 1024 : 2 * cus / base;
    const int one_round = rows < cus / base ? rows : cus / base;
    if (want < one_round) want = one_round;
    if (want < 1) want = 1;
    const int per_split = (rows + want - 1) / want;
    p.chunk = per_split * 512;
    p.S = (ctx + p.chunk - 1) / p.chunk;
  }
  return p;
}

static size_t attn_partials_floats(int Hq, int S, int D) {
  const size_t hs = (size_t)Hq * S;
  return hs * 2 + hs * D;
}

// ---- the GQA kernel's plan and launch ----------------------------------------------------------
// Which calls it serves: f32 caches, 3 to 8 query heads per kv head (one wavefront each).
template <typename KT> static bool gqa_applies(int group) { return false; }
template <> bool gqa_applies<float>(int group) { return group >= 3 && group <= 8; }

// Splits: one tile each while there are CUs for them (a block per CU and kv head), never more
// than the combine kernel sums in one pass (8 per column group; beyond that its summation order
// would depend on the count). stages: 2 when a split holds more than one tile.
struct GqaPlan { int S, stages; };
static GqaPlan plan_gqa(int Hkv, int ctx, int cus, int D) {
  const int tiles = (ctx + gqa::kKeys - 1) / gqa::kKeys;
  int S = cus / Hkv;
  if (S > 8 * (1024 / D)) S = 8 * (1024 / D);
  if (S > tiles) S = tiles;
  if (S < 1) S = 1;
  return GqaPlan{S, (tiles + S - 1) / S > 1 ? 2 : 1};
}

static size_t attn_partials_floats(int Hq, int S, int D);

template <int D>
static int launch_gqa(const float* q, const float* K, const float* V, float* out, int Hq, int Hkv, int ctx,
                      int64_t kv_max, float scale, const uint32_t* dpos, float* partials, size_t partials_bytes,
                      const QkvFuse* fuse) {
  // out == nullptr: the partials are the result (also of a single split); whoever reads them merges
  Context& c = tlhip::ctx();
  const int group = Hq / Hkv;
  const GqaPlan p = plan_gqa(Hkv, ctx, c.cus, D);
  const int S = p.S;
  float *pm = nullptr, *pl = nullptr, *pacc = nullptr;
  if (S > 1 || !out) {
    const size_t hs = (size_t)Hq * S;
    const size_t need = attn_partials_floats(Hq, S, D) * sizeof(float);
    float* base;
    if (dpos || partials) {   // a buffer the caller named: never the library's growable scratch
      if (!partials || partials_bytes < need)
        return fail(TLHIP_EINVAL, "attention: %zu bytes of split partials needed, the buffer given holds %zu",
                    need, partials_bytes);
      base = partials;
    } else {
      base = static_cast<float*>(scratch(need));
    }
    if (!base) return fail(TLHIP_ENOMEM, "tlhip_attn_decode: no scratch for %d splits", S);
    pm = base;
    pl = pm + hs;
    pacc = pl + hs;
  }
  const size_t lds = gqa::lds_bytes<D>(group, p.stages);
  const dim3 grid((unsigned)(Hkv * S)), block(64 * (group + 1));
  const int64_t kv_stride = kv_max * D;
  const QkvFuse fz = fuse ? *fuse : QkvFuse{};
  hipError_t e = hipSuccess;
  auto go = [&](auto kernel) {
    // more than 64 KB of LDS per block has to be asked for; asking is cheap next to a launch
    if (lds > 64 * 1024)
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e == hipSuccess)
      hipLaunchKernelGGL(kernel, grid, block, lds, c.stream, q, K, V, out, pm, pl, pacc, ctx, kv_stride, scale, S, dpos,
                         fz, (int)kv_max, Hkv, p.stages);
  };
#define TLHIP_GQA(GG) \
  if (fuse) go(gqa::attn_gqa_kernel<D, GG, true>); else go(gqa::attn_gqa_kernel<D, GG, false>)
  switch (group) {
    case 3: TLHIP_GQA(3); break;
    case 4: TLHIP_GQA(4); break;
    case 5: TLHIP_GQA(5); break;
    case 6: TLHIP_GQA(6); break;
    case 7: TLHIP_GQA(7); break;
    default: TLHIP_GQA(8); break;
  }
#undef TLHIP_GQA
  if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(LDS)");
  if (S > 1 && out)
    hipLaunchKernelGGL(attn_combine_kernel, dim3(Hq), dim3(1024), (size_t)(S + 1024) * sizeof(float),
                       c.stream, pm, pl, pacc, out, S, D);
  TLHIP_CHECK_LAUNCH(TLHIP_C_ATTN_DECODE);
}

// dpos != nullptr: ctx is the cache CAPACITY the grid is planned for, the live
// context is read from the device, and the split partials live in a buffer the
// caller owns (a captured graph bakes the address in).
template <int D, typename KT>
static int launch_attn(const float* q, const KT* K, const KT* V, float* out, int Hq, int Hkv,
                       int ctx, int64_t kv_max, float scale, const uint32_t* dpos = nullptr,
                       float* partials = nullptr, size_t partials_bytes = 0,
                       const QkvFuse* fuse = nullptr) {
  Context& c = tlhip::ctx();
  const int group = Hq / Hkv;
  if (gqa_applies<KT>(group) && c.tune_attn_decode != 1)
    return launch_gqa<D>(q, reinterpret_cast<const float*>(K), reinterpret_cast<const float*>(V), out, Hq, Hkv, ctx,
                         kv_max, scale, dpos, partials, partials_bytes, fuse);
  const AttnPlan p = plan_attn(Hkv, group, ctx, c.cus, dpos != nullptr);
  float *pm = nullptr, *pl = nullptr, *pacc = nullptr;
  const int S = p.S;
  if (S > 1) {
    const size_t hs = (size_t)Hq * S;
    const size_t need = attn_partials_floats(Hq, S, D) * sizeof(float);
    float* base;
    if (dpos || partials) {   // a buffer the caller named: never the library's growable scratch
      if (!partials || partials_bytes < need)
        return fail(TLHIP_EINVAL, "attention: %zu bytes of split partials needed, the buffer given holds %zu",
                    need, partials_bytes);
      base = partials;
    } else {
      base = static_cast<float*>(scratch(need));
    }
    if (!base) return fail(TLHIP_ENOMEM, "tlhip_attn_decode: no scratch for %d splits", p.S);
    pm = base;
    pl = pm + hs;
    pacc = pl + hs;
  }
  if (S > 65535) return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode: context too long");
  const int pairs8 = (Hkv * S + 7) / 8 * 8;       // (kv head, split) pairs, padded to whole rounds of the 8 XCDs
  const dim3 grid(pairs8 * p.gz), block(p.nw * 64);
  const int64_t kv_stride = kv_max * D;
  const QkvFuse fz = fuse ? *fuse : QkvFuse{};
#define TLHIP_ATTN(GG)                                                                            \
  if (fuse)                                                                                       \
    hipLaunchKernelGGL((attn_decode_kernel<D, GG, KT, false, true>), grid, block, 0, c.stream, q, \
                       K, V, out, pm, pl, pacc, group, ctx, kv_stride, p.chunk, p.TK, scale, S,   \
                       1, 0, dpos, fz, (int)kv_max, Hkv, p.gz);                                   \
  else                                                                                            \
    hipLaunchKernelGGL((attn_decode_kernel<D, GG, KT, false>), grid, block, 0, c.stream, q, K, V, \
                       out, pm, pl, pacc, group, ctx, kv_stride, p.chunk, p.TK, scale, p.S, 1, 0, \
                       dpos, fz, (int)kv_max, Hkv, p.gz)
  switch (p.G) {
    case 1: TLHIP_ATTN(1); break;
    case 2: TLHIP_ATTN(2); break;
    case 4: TLHIP_ATTN(4); break;
    default: TLHIP_ATTN(8); break;
  }
#undef TLHIP_ATTN
  if (S > 1)
    hipLaunchKernelGGL(attn_combine_kernel, dim3(Hq), dim3(1024), (size_t)(S + 1024) * sizeof(float),
                       c.stream, pm, pl, pacc, out, S, D);
  TLHIP_CHECK_LAUNCH(TLHIP_C_ATTN_DECODE);
}

// attn_prefill_mfma.hip
template <int D, typename KT>
int launch_prefill_mfma(const float* q, const KT* K, const KT* V, float* out, int Hq, int Hkv, int T,
                        int64_t kv_max, float scale, int pos0, int token_major);

// attn_prefill_f16.hip
bool prefill_x3_applies(int D, int T, int pos0);
template <int D, typename KT>
int launch_prefill_x3(const float* q, const KT* K, const KT* V, float* out, int Hq, int Hkv, int T,
                      int64_t kv_max, float scale, int pos0, int token_major);

// Three kernels serve causal prefill attention. Deep in a context the f16-term kernels on the
// matrix cores; otherwise the fp32 matrix-pipe kernel; the VALU kernel that shares its code with
// decode attention on request. tune_prefill: 0 = that choice, 1 = VALU, 2 = fp32 matrix pipe,
// 4 = f16 terms (what the choice takes deep in a context).
template <int D, typename KT>
static int launch_prefill(const float* q, const KT* K, const KT* V, float* out, int Hq, int Hkv,
                          int T, int64_t kv_max, float scale, int pos0, int token_major) {
  Context& c = tlhip::ctx();
  const int mode = c.tune_prefill_valu;
  if (mode == 4 || (mode == 0 && prefill_x3_applies(D, T, pos0))) {
    const int rc = launch_prefill_x3<D, KT>(q, K, V, out, Hq, Hkv, T, kv_max, scale, pos0, token_major);
    if (rc < 0) return rc;
    if (rc == 0) TLHIP_CHECK_LAUNCH(TLHIP_C_ATTN_PREFILL);
    if (mode != 0) return fail(TLHIP_ENOMEM, "tlhip_attn_prefill: no scratch for the key/value planes");
    // no scratch for the planes: the fp32 matrix-pipe kernel needs none
  }
  if (mode != 1) {
    if (int rc = launch_prefill_mfma<D, KT>(q, K, V, out, Hq, Hkv, T, kv_max, scale, pos0, token_major)) return rc;
    TLHIP_CHECK_LAUNCH(TLHIP_C_ATTN_PREFILL);
  }
  if (token_major) return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_prefill_tok: the VALU kernel writes head-major only");
  constexpr int G = 8;   // query positions per block
  const dim3 grid(Hq, 1, (T + 4 * G - 1) / (4 * G)), block(256);   // 4 wavefronts x G query rows
  hipLaunchKernelGGL((attn_decode_kernel<D, G, KT, true>), grid, block, 0, c.stream, q, K, V, out,
                     (float*)nullptr, (float*)nullptr, (float*)nullptr, Hq / Hkv, pos0 + T,
                     kv_max * D, 0, 64, scale, 1, T, pos0, (const uint32_t*)nullptr, QkvFuse{}, (int)kv_max, 0, 1);
  TLHIP_CHECK_LAUNCH(TLHIP_C_ATTN_PREFILL);
}

// ---- memory of the entry point that allocates nothing -------------------------------------
// tlhip_attn_decode_static keeps its split partials in this array instead of the library's
// growable scratch. Each GPU holds its own copy at its own address; host code never uses the
// array's name as an address, only the pointer hipGetSymbolAddress returned for that device.
namespace fixed {
constexpr size_t kBytes = size_t(1) << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kBytes];
static void* dev_ptr[kMaxDevices] = {};   // per device: where that device's copy lives
}  // namespace fixed

// Resolves the array's address on `device`, which must be the current one. Called by tlhip_init.
int attn_static_setup(int device) {
  if (device < 0 || device >= fixed::kMaxDevices) return fail(TLHIP_EINVAL, "device %d out of range", device);
  if (fixed::dev_ptr[device]) return TLHIP_OK;
  void* p = nullptr;
  const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(fixed::scratch));
  if (e != hipSuccess || !p) return hip_fail(e, "hipGetSymbolAddress");
  fixed::dev_ptr[device] = p;
  return TLHIP_OK;
}

}  // namespace tlhip

using namespace tlhip;

extern "C" {

int tlhip_attn_decode_static(const void* q, const void* K, const void* V, void* out, int64_t n_q_heads,
                             int64_t n_kv_heads, int64_t ctx_len, int64_t kv_max, int64_t D, float scale,
                             int kv_bf16) {
  Context& c = ctx();
  if (!c.ready)   // tlhip_init allocates (stream, result slots); this entry point may not
    return fail(TLHIP_ERUNTIME, "tlhip_attn_decode_static: call tlhip_init first");
  void* fixed_ptr = c.device >= 0 && c.device < fixed::kMaxDevices ? fixed::dev_ptr[c.device] : nullptr;
  if (!fixed_ptr) return fail(TLHIP_ERUNTIME, "tlhip_attn_decode_static: fixed buffer not resolved on device %d", c.device);
  if (!q || !K || !V || !out) return fail(TLHIP_EINVAL, "tlhip_attn_decode_static: null pointer");
  if (D != 64 && D != 128) return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode_static: head_dim must be 64 or 128");
  if (n_kv_heads <= 0 || n_q_heads <= 0 || n_q_heads % n_kv_heads != 0)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode_static: Hq must be a positive multiple of Hkv");
  if (ctx_len <= 0 || ctx_len > kv_max) return fail(TLHIP_EINVAL, "tlhip_attn_decode_static: need 0 < ctx <= kv_max");
  if (ctx_len > 0x3fffffff || n_kv_heads > 65535 || n_q_heads > 0x7fffffff || kv_max * D > ((int64_t)1 << 40))
    return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode_static: shape too large");
  if (!aligned16(q) || !aligned16(K) || !aligned16(V) || !aligned16(out))
    return fail(TLHIP_EINVAL, "tlhip_attn_decode_static: operands must be 16-byte aligned");
  const int Hq = (int)n_q_heads, Hkv = (int)n_kv_heads, cx = (int)ctx_len;
  // the same launch plan as tlhip_attn_decode; its split partials must fit the fixed array
  AttnPlan p = plan_attn(Hkv, Hq / Hkv, cx, c.cus, false);
  if (!kv_bf16 && gqa_applies<float>(Hq / Hkv) && c.tune_attn_decode != 1) p.S = plan_gqa(Hkv, cx, c.cus, (int)D).S;
  const size_t need = p.S > 1 ? attn_partials_floats(Hq, p.S, (int)D) * sizeof(float) : 0;
  if (need > fixed::kBytes)
    return fail(TLHIP_EUNSUPPORTED,
                "tlhip_attn_decode_static: this shape splits the context %d ways and needs %zu bytes of "
                "partials; the fixed buffer holds %zu (use tlhip_attn_decode)", p.S, need, fixed::kBytes);
  const float* pq = static_cast<const float*>(q);
  float* po = static_cast<float*>(out);
  float* part = static_cast<float*>(fixed_ptr);
  if (kv_bf16) {
    const uint16_t* pk = static_cast<const uint16_t*>(K);
    const uint16_t* pv = static_cast<const uint16_t*>(V);
    return D == 128 ? launch_attn<128, uint16_t>(pq, pk, pv, po, Hq, Hkv, cx, kv_max, scale, nullptr, part, fixed::kBytes)
                    : launch_attn<64, uint16_t>(pq, pk, pv, po, Hq, Hkv, cx, kv_max, scale, nullptr, part, fixed::kBytes);
  }
  const float* pk = static_cast<const float*>(K);
  const float* pv = static_cast<const float*>(V);
  return D == 128 ? launch_attn<128, float>(pq, pk, pv, po, Hq, Hkv, cx, kv_max, scale, nullptr, part, fixed::kBytes)
                  : launch_attn<64, float>(pq, pk, pv, po, Hq, Hkv, cx, kv_max, scale, nullptr, part, fixed::kBytes);
}

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

static int attn_prefill_entry(const void* q, const void* K, const void* V, void* out, int64_t n_q_heads,
                              int64_t n_kv_heads, int64_t T, int64_t kv_max, int64_t D, float scale,
                              int kv_bf16, int64_t pos0, int token_major) {
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
    return D == 128 ? launch_prefill<128, uint16_t>(pq, pk, pv, po, Hq, Hkv, t, kv_max, scale, p0, token_major)
                    : launch_prefill<64, uint16_t>(pq, pk, pv, po, Hq, Hkv, t, kv_max, scale, p0, token_major);
  }
  const float* pk = static_cast<const float*>(K);
  const float* pv = static_cast<const float*>(V);
  return D == 128 ? launch_prefill<128, float>(pq, pk, pv, po, Hq, Hkv, t, kv_max, scale, p0, token_major)
                  : launch_prefill<64, float>(pq, pk, pv, po, Hq, Hkv, t, kv_max, scale, p0, token_major);
}

int tlhip_attn_prefill(const void* q, const void* K, const void* V, void* out, int64_t n_q_heads,
                       int64_t n_kv_heads, int64_t T, int64_t kv_max, int64_t D, float scale,
                       int kv_bf16, int64_t pos0) {
  return attn_prefill_entry(q, K, V, out, n_q_heads, n_kv_heads, T, kv_max, D, scale, kv_bf16, pos0, 0);
}

int tlhip_attn_prefill_tok(const void* q, const void* K, const void* V, void* out, int64_t n_q_heads,
                           int64_t n_kv_heads, int64_t T, int64_t kv_max, int64_t D, float scale,
                           int kv_bf16, int64_t pos0) {
  return attn_prefill_entry(q, K, V, out, n_q_heads, n_kv_heads, T, kv_max, D, scale, kv_bf16, pos0, 1);
}

int64_t tlhip_attn_partials_bytes(int64_t n_q_heads, int64_t n_kv_heads, int64_t kv_max, int64_t D) {
  if (!ctx().ready || n_q_heads <= 0 || n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0 || kv_max <= 0 ||
      kv_max > 0x3fffffff || (D != 64 && D != 128))
    return 0;
  const AttnPlan p = plan_attn((int)n_kv_heads, (int)(n_q_heads / n_kv_heads), (int)kv_max, ctx().cus, true);
  const GqaPlan g = plan_gqa((int)n_kv_heads, (int)kv_max, ctx().cus, (int)D);   // whichever kernel serves the cache type
  return (int64_t)(attn_partials_floats((int)n_q_heads, p.S > g.S ? p.S : g.S, (int)D) * sizeof(float)) + 16;
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

// The step's raw [q | k | v] projection goes in; bias, rotation, the cache append
// and the attention over keys [0, pos] happen in one launch (plus the split merge).
int tlhip_attn_decode_qkv(const void* qkv, const void* bq, const void* bk, const void* bv, void* Kc,
                          void* Vc, void* out, int64_t n_q_heads, int64_t n_kv_heads, int64_t pos,
                          const void* d_pos, int64_t kv_max, int64_t D, float scale,
                          const void* table, int kv_bf16, void* partials, int64_t partials_bytes) {
  TLHIP_REQUIRE_READY();
  if (!qkv || !Kc || !Vc || !out || !table) return fail(TLHIP_EINVAL, "tlhip_attn_decode_qkv: null pointer");
  if (D != 64 && D != 128) return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode_qkv: head_dim must be 64 or 128");
  if (n_kv_heads <= 0 || n_q_heads <= 0 || n_q_heads % n_kv_heads != 0)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode_qkv: Hq must be a positive multiple of Hkv");
  if (kv_max <= 0 || kv_max > 0x3fffffff || n_kv_heads > 65535 || kv_max * D > ((int64_t)1 << 40))
    return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode_qkv: shape too large");
  if (!d_pos && (pos < 0 || pos >= kv_max)) return fail(TLHIP_EINVAL, "tlhip_attn_decode_qkv: need 0 <= pos < kv_max");
  if (!aligned16(qkv) || !aligned16(Kc) || !aligned16(Vc) || !aligned16(out) || !aligned16(table) ||
      (bq && !aligned16(bq)) || (bk && !aligned16(bk)) || (bv && !aligned16(bv)) ||
      (partials && !aligned16(partials)))
    return fail(TLHIP_EINVAL, "tlhip_attn_decode_qkv: operands must be 16-byte aligned");
  const QkvFuse fz{static_cast<const float*>(bq), static_cast<const float*>(bk),
                   static_cast<const float*>(bv), static_cast<const float2*>(table), Kc, Vc, kv_max};
  const float* pq = static_cast<const float*>(qkv);
  float* po = static_cast<float*>(out);
  const uint32_t* dp = static_cast<const uint32_t*>(d_pos);
  float* pp = static_cast<float*>(partials);
  const size_t pb = partials_bytes > 0 ? (size_t)partials_bytes : 0;
  const int Hq = (int)n_q_heads, Hkv = (int)n_kv_heads;
  const int cx = dp ? (int)kv_max : (int)pos + 1;   // the grid is planned for this many keys
  int rc;
  if (kv_bf16) {
    const uint16_t* pk = static_cast<const uint16_t*>(Kc);
    const uint16_t* pv = static_cast<const uint16_t*>(Vc);
    rc = D == 128 ? launch_attn<128, uint16_t>(pq, pk, pv, po, Hq, Hkv, cx, kv_max, scale, dp, pp, pb, &fz)
                  : launch_attn<64, uint16_t>(pq, pk, pv, po, Hq, Hkv, cx, kv_max, scale, dp, pp, pb, &fz);
  } else {
    const float* pk = static_cast<const float*>(Kc);
    const float* pv = static_cast<const float*>(Vc);
    rc = D == 128 ? launch_attn<128, float>(pq, pk, pv, po, Hq, Hkv, cx, kv_max, scale, dp, pp, pb, &fz)
                  : launch_attn<64, float>(pq, pk, pv, po, Hq, Hkv, cx, kv_max, scale, dp, pp, pb, &fz);
  }
  if (rc == TLHIP_OK) {
    ctx().census[TLHIP_C_ROPE]++;
    ctx().census[TLHIP_C_KV_APPEND]++;
  }
  return rc;
}

// Splits whose partials a GEMV's staging pass merges in the summation order of the merge kernel:
// one per column group of that kernel (1024 / D), 16 at most.
static int parts_limit(int64_t D) { return D == 64 ? 16 : 8; }

int tlhip_attn_parts_splits(int64_t n_q_heads, int64_t n_kv_heads, int64_t plan_ctx, int64_t D, int kv_bf16) {
  if (!ctx().ready || kv_bf16 || (D != 64 && D != 128) || n_kv_heads <= 0 || n_kv_heads > 65535 || n_q_heads <= 0 ||
      n_q_heads % n_kv_heads != 0 || plan_ctx <= 0 || plan_ctx > 0x3fffffff)
    return 0;
  if (!gqa_applies<float>((int)(n_q_heads / n_kv_heads)) || ctx().tune_attn_decode == 1) return 0;
  if ((n_q_heads & 1) != 0) return 0;   // the accumulators follow 2 * heads * splits floats and are read 16 bytes at a time
  const int S = plan_gqa((int)n_kv_heads, (int)plan_ctx, ctx().cus, (int)D).S;
  return S <= parts_limit(D) ? S : 0;
}

int tlhip_attn_decode_qkv_parts(const void* qkv, const void* bq, const void* bk, const void* bv, void* Kc,
                                void* Vc, int64_t n_q_heads, int64_t n_kv_heads, int64_t pos,
                                const void* d_pos, int64_t kv_max, int64_t D, float scale,
                                const void* table, void* partials, int64_t partials_bytes, int* n_parts) {
  TLHIP_REQUIRE_READY();
  if (!qkv || !Kc || !Vc || !table || !partials || !n_parts)
    return fail(TLHIP_EINVAL, "tlhip_attn_decode_qkv_parts: null pointer");
  if (D != 64 && D != 128) return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode_qkv_parts: head_dim must be 64 or 128");
  if (n_kv_heads <= 0 || n_q_heads <= 0 || n_q_heads % n_kv_heads != 0)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode_qkv_parts: Hq must be a positive multiple of Hkv");
  if (kv_max <= 0 || kv_max > 0x3fffffff || n_kv_heads > 65535 || kv_max * D > ((int64_t)1 << 40))
    return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_decode_qkv_parts: shape too large");
  if (!d_pos && (pos < 0 || pos >= kv_max))
    return fail(TLHIP_EINVAL, "tlhip_attn_decode_qkv_parts: need 0 <= pos < kv_max");
  if (!aligned16(qkv) || !aligned16(Kc) || !aligned16(Vc) || !aligned16(table) || (bq && !aligned16(bq)) ||
      (bk && !aligned16(bk)) || (bv && !aligned16(bv)) || !aligned16(partials))
    return fail(TLHIP_EINVAL, "tlhip_attn_decode_qkv_parts: operands must be 16-byte aligned");
  const int cx = d_pos ? (int)kv_max : (int)pos + 1;   // the grid is planned for this many keys
  const int S = tlhip_attn_parts_splits(n_q_heads, n_kv_heads, cx, D, 0);
  if (S <= 0)
    return fail(TLHIP_EUNSUPPORTED,
                "tlhip_attn_decode_qkv_parts: f32 cache, 3 to 8 query heads per kv head, an even head count and a "
                "context of at most %d splits (ask tlhip_attn_parts_splits)", parts_limit(D));
  const QkvFuse fz{static_cast<const float*>(bq), static_cast<const float*>(bk),
                   static_cast<const float*>(bv), static_cast<const float2*>(table), Kc, Vc, kv_max};
  const float* pq = static_cast<const float*>(qkv);
  const uint32_t* dp = static_cast<const uint32_t*>(d_pos);
  const size_t pb = partials_bytes > 0 ? (size_t)partials_bytes : 0;
  const int Hq = (int)n_q_heads, Hkv = (int)n_kv_heads;
  const float* pk = static_cast<const float*>(Kc);
  const float* pv = static_cast<const float*>(Vc);
  float* pp = static_cast<float*>(partials);
  const int rc = D == 128 ? launch_gqa<128>(pq, pk, pv, nullptr, Hq, Hkv, cx, kv_max, scale, dp, pp, pb, &fz)
                          : launch_gqa<64>(pq, pk, pv, nullptr, Hq, Hkv, cx, kv_max, scale, dp, pp, pb, &fz);
  if (rc == TLHIP_OK) {
    *n_parts = S;
    ctx().census[TLHIP_C_ROPE]++;
    ctx().census[TLHIP_C_KV_APPEND]++;
  }
  return rc;
}

}  // extern "C"
