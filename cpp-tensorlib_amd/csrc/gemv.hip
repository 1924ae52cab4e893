// Decode GEMV kernels (batch 1, weight-stationary, HBM-bound).
//
// Row layouts (int4 [N][K/2] + scales, bf16 [N][K]): gemv_rows_kernel.
//   * persistent blocks: the activation vector x is staged ONCE per block into
//     LDS in a lane-interleaved layout, then the block walks row tiles;
//   * every lane streams 16-byte units of a weight row (32 int4 weights = one
//     scale group, or 8 bf16 weights) with global_load_dwordx4, fully
//     coalesced along K, R rows in flight per wavefront so that one x fragment
//     (held in VGPRs) is reused R times;
//   * nibbles are unpacked and scaled in registers, fp32 accumulate;
//   * K is split over the lanes of a wavefront and, for short-N shapes, over
//     KW wavefronts of the block; partial sums are combined with wave
//     shuffles and a fixed-order LDS pass: no atomics, deterministic.
//
// Column layouts (f32/bf16 [K][N], the array seam's layout): gemv_cols_kernel.
//   * a lane owns 16 bytes of consecutive columns, a wavefront 64 of those,
//     K is split over the 4 wavefronts of a block and over gridDim.y; split
//     partials go to scratch and are summed in a fixed order by a second
//     kernel.
#include "common.hpp"
#include "gemv_shared.hpp"

namespace tlhip {

// ---------------------------------------------------------------------------
// row kernel
// ---------------------------------------------------------------------------
// W: [N][upr] 16-byte units. scales: [N][upr] f32 (int4 only).
// Block = nw wavefronts arranged as (nw/KW row groups) x (KW K-splits).
// LDS: x as float4 xs[(chunk*J + j)*XS + lane], J = E/4, XS = LPR + a few (see the kernel), so that lane l's j-th
// fragment of chunk c is one conflict-free ds_read_b128; then KW*rows floats.
template <typename Fmt, int R>
struct RowFrag {          // one (row tile, chunk) work item of a lane: R weight units in flight
  uint4 w[R];
  float sc[R];
};

// Weight and scale addresses are formed as a uniform base plus a 32-bit byte
// offset per lane (the launcher checks that the matrix is below 4 GiB), which is
// the cheapest global addressing form: one 24-bit multiply-add per row.
//
// PAIR: the matrix is two stacked halves of N/2 rows (gate rows, then up rows) and the R
// fragments are R/2 consecutive rows of the first half followed by the same rows of the
// second; row0 counts rows of a half.
template <typename Fmt, int R, bool PAIR = false>
__device__ __forceinline__ void load_frag(RowFrag<Fmt, R>& f, const uint4* __restrict__ W,
                                          const float* __restrict__ scales, int N, int upr,
                                          int row0, int u) {
  // Branch-free: a lane past the end of the row re-reads the row's last unit (its result is
  // never used). Loads under a condition would make the compiler's wait counters
  // conservative - every wait would also cover the loads issued after the ones it needs.
  u = min(u, upr - 1);
  const char* wb = reinterpret_cast<const char*>(W);
  const char* sb = reinterpret_cast<const char*>(scales);
#pragma unroll
  for (int r = 0; r < R; r++) {
    const uint32_t row = PAIR ? (uint32_t)(min(row0 + (r % (R / 2 > 0 ? R / 2 : 1)), N / 2 - 1) +
                                           (r >= R / 2 ? N / 2 : 0))
                              : (uint32_t)min(row0 + r, N - 1);
    const uint32_t idx = __umul24(row, (uint32_t)upr) + (uint32_t)u;
    f.w[r] = load_stream16(reinterpret_cast<const uint4*>(wb + (idx << 4)));
    if (Fmt::kScaled)
      f.sc[r] = __builtin_nontemporal_load(reinterpret_cast<const float*>(sb + (idx << 2)));
  }
}

// LPR = lanes that share a weight row: 64 (a row segment of 64 units per
// wavefront step) or 16 (the wavefront works on 4 row groups at once, 16 units
// of each per step). Rows whose unit count is not close to a multiple of 64 leave
// lanes idle in the 64-lane form (K = 3584 is 112 units: 12.5 % idle; K = 896 is
// 28 units: 56 % idle); the 16-lane form wastes at most 15 units per row and
// finishes a row sum inside one DPP row.
template <typename Fmt, int R, int PRO, int LPR, int EPI = kStore>
__global__ __launch_bounds__(R >= 8 ? 512 : 1024) void gemv_rows_kernel(
    const float* x, const uint4* __restrict__ W, const float* __restrict__ scales,
    float* __restrict__ y, int N, int upr, int KW, int ntiles, const Producer pro) {
  constexpr int J = Fmt::E / 4;
  constexpr int QN = 64 / LPR;       // row groups a wavefront works on at once
  extern __shared__ float4 smem4[];
  const int tid = threadIdx.x, lane = tid & 63;
  // wavefront-uniform, and known to be: the loop over work items then runs on scalar
  // branches, which also keeps the compiler's wait counters exact
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & (LPR - 1), q = lane / LPR;
  const int nw = blockDim.x >> 6;
  const int chunks = (upr + LPR - 1) / LPR;
  // Row stride of the staged x: LPR float4s plus padding chosen so that the staging writes
  // spread over all banks as well (the J threads of a unit write J rows at the same column:
  // with a stride of exactly LPR float4s they would all hit one group of four banks).
  constexpr int XS = LPR + (J == 8 ? 2 : 8);
  float4* xs = smem4;
  float* xsum = reinterpret_cast<float*>(smem4 + (size_t)chunks * J * XS);  // [chunks*LPR], int4 only
  float* red = xsum + (Fmt::kScaled ? chunks * LPR : 0);   // [nw * QN * 8] K-split partials
  float* nsum = red + nw * QN * 8;                          // [16] per-wavefront sums of squares (norm producer)
  float* fw = nsum + 16;                                    // [heads * 8] split weights (attention-merge producer)
  float* fL = fw + (PRO == kAttnMerge ? pro.heads * kMergeMax : 0);   // [heads] the heads' sums

  const int kw = wave % KW;          // which K split this wavefront takes
  const int wn = wave / KW;          // which row group of the block tile
  const int groups = nw / KW;        // wavefront row groups per block tile
  const int rows_per_tile = groups * QN * R;
  const int wrow = (wn * QN + q) * R;  // this lane's first row inside a tile
  constexpr bool kPair = EPI == kGateUp;
  static_assert(!kPair || R >= 2, "a gate/up pair needs two rows per lane group");
  // first row of work item (tile tt): a row of W, or with kPair a row of each half
  const auto item_row = [&](int tt) { return kPair ? (tt * rows_per_tile + wrow) >> 1 : tt * rows_per_tile + wrow; };

  // Requests go out in this order: the activations (and what their producer reads) first, then
  // the first work item's weights. A wavefront's loads return in order, so x requested after
  // the weights would keep the staging pass waiting for them.
  TLHIP_MARK(0);
  const float4* x4 = reinterpret_cast<const float4*>(x);
  const int n4 = upr * J;
  const float4* d4 = reinterpret_cast<const float4*>(pro.delta);
  // float4s a thread requests up front: all of x up to 20 floats per thread (K = 18944 on 1024
  // threads), 8 per thread in the norm form, whose vector is the hidden size (registers)
  constexpr int PL = PRO == kRmsnorm ? 2 : 5;
  float4 px[PL], pa[PL], pn[PL];
  // attention-merge producer: this thread's first float4 of the first kPre splits' accumulators, and
  // the (head, split) pair whose maximum and sum it weighs
  constexpr int kPre = 8;
  float4 pre[kPre];
  float pre_m = -INFINITY, pre_l = 0.f;
  if constexpr (PRO == kAttnMerge) {
    const int S = pro.S, D4 = pro.D >> 2;
    const int i = min(tid, n4 - 1), h = i / D4;
    const float4* pacc = reinterpret_cast<const float4*>(x + 2 * pro.heads * S) + (size_t)h * S * D4 + (i - h * D4);
#pragma unroll
    for (int sp = 0; sp < kPre; sp++)
      if (sp < S) pre[sp] = pacc[(size_t)sp * D4];
    const int hh = tid / kMergeMax, sp = tid % kMergeMax;
    if (hh < pro.heads && sp < S) { pre_m = x[hh * S + sp]; pre_l = x[pro.heads * S + hh * S + sp]; }
  }
  {
    const float4* aux4 = PRO == kSwiglu ? x4 + n4 : (d4 ? d4 : x4);   // up half, or delta (x when none: ignored)
#pragma unroll
    for (int k = 0; k < PL; k++) {
      const int i = min(tid + k * (int)blockDim.x, n4 - 1);
      if (PRO != kAttnMerge) px[k] = x4[i];
      if (PRO != kPlain && PRO != kAttnMerge) pa[k] = aux4[i];
      if (PRO == kRmsnorm) pn[k] = reinterpret_cast<const float4*>(pro.norm_w)[i];
    }
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
  // This wavefront's work items, numbered i = 0, 1, ...: item i is chunk kw + (i % cpw) * KW of
  // the block's tile number i / cpw. Two items are kept in flight (NS).
  constexpr int NS = 2;
  // chunks per tile for this wavefront; one (idle) when KW exceeds the chunk count, so that
  // the wavefront still meets the block's barriers at every tile end
  const int cpw = max((chunks - kw + KW - 1) / KW, 1);
  const int my_tiles = (int)blockIdx.x < ntiles ? (ntiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x : 0;
  const int n_items = my_tiles * cpw;
  const auto load_item = [&](RowFrag<Fmt, R>& f, int i) {
    const int ti = i / cpw, ci = i - ti * cpw;
    const int tt = min((int)blockIdx.x + ti * (int)gridDim.x, ntiles - 1);
    load_frag<Fmt, R, kPair>(f, W, scales, N, upr, item_row(tt), (kw + ci * KW) * LPR + li);
  };
  RowFrag<Fmt, R> frag[NS];
  load_item(frag[0], 0);
  TLHIP_MARK(1);

  if constexpr (PRO == kAttnMerge) {
    // The splits' weights e^(m_s - M) and each head's sum, once per block into LDS: sixteen adjacent
    // lanes hold the (up to) sixteen splits of a head. Sums in the order of attn_combine_kernel's
    // wavefront sum over its first sixteen lanes: partners 8, 4, 2 and 1 lanes away in turn.
    const int S = pro.S, hs = pro.heads * S;
    const int nl = (pro.heads * kMergeMax + 63) & ~63;
    for (int e = tid; e < nl; e += blockDim.x) {
      const int h = e / kMergeMax, sp = e % kMergeMax;
      const bool live = h < pro.heads && sp < S;
      const float m = e == tid ? pre_m : (live ? x[h * S + sp] : -INFINITY);
      const float l = e == tid ? pre_l : (live ? x[hs + h * S + sp] : 0.f);
      float M = fmaxf(m, __shfl_xor(m, 8, kWave));
      M = fmaxf(M, __shfl_xor(M, 4, kWave));
      M = fmaxf(M, __shfl_xor(M, 2, kWave));
      M = fmaxf(M, __shfl_xor(M, 1, kWave));
      const float w = live ? __expf(m - M) : 0.f;
      float t = mul_rn(l, w);   // (a product left to the compiler could fuse with the first sum)
      t = add_rn(t, __shfl_xor(t, 8, kWave));
      t += __shfl_xor(t, 4, kWave);
      t += __shfl_xor(t, 2, kWave);
      t += __shfl_xor(t, 1, kWave);
      if (h < pro.heads) {
        fw[e] = w;
        if (sp == 0) fL[h] = t;
      }
    }
    __syncthreads();
  }

  {  // stage x (K = upr*E floats) into the interleaved layout, one pass:
     // thread i owns float4 i; the J threads of a unit are adjacent lanes, so the
     // unit's sum(x) is a J-lane shuffle reduction (J is 8 or 2, both divide 64).
    const int n4_padded = (n4 + 63) & ~63;   // whole wavefronts take part in the shuffles
    // float4 number k of this thread before the norm: x (+ delta), or swiglu(gate, up);
    // nv receives its norm weights. The first PL come from the registers requested above.
    const auto raw = [&](int k, int i, float4& nv) -> float4 {
      if constexpr (PRO == kAttnMerge) {
        const int D4 = pro.D >> 2, h = i / D4, d4i = i - h * D4, S = pro.S;
        const float4* pacc = reinterpret_cast<const float4*>(x + 2 * pro.heads * S) + (size_t)h * S * D4 + d4i;
        const float* fh = fw + h * kMergeMax;
        // split 0's product, then the others' added one by one: the merge kernel's order
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        const auto add = [&](float f, const float4 a, bool first) {
          const float4 p = make_float4(mul_rn(f, a.x), mul_rn(f, a.y), mul_rn(f, a.z), mul_rn(f, a.w));
          v = first ? p : make_float4(add_rn(v.x, p.x), add_rn(v.y, p.y), add_rn(v.z, p.z), add_rn(v.w, p.w));
        };
#pragma unroll
        for (int sp = 0; sp < kPre; sp++)
          if (sp < S) add(fh[sp], k == 0 ? pre[sp] : pacc[(size_t)sp * D4], sp == 0);
        for (int sp = kPre; sp < S; sp++) add(fh[sp], pacc[(size_t)sp * D4], false);
        const float L = fL[h];
        return make_float4(v.x / L, v.y / L, v.z / L, v.w / L);
      }
      float4 v, aux;
      bool have = false;
#pragma unroll
      for (int kk = 0; kk < PL; kk++)
        if (k == kk) { v = px[kk]; aux = pa[kk]; nv = pn[kk]; have = true; }
      if (!have) {
        v = x4[i];
        if (PRO == kSwiglu) aux = x4[n4 + i];
        if (PRO == kRmsnorm) { nv = reinterpret_cast<const float4*>(pro.norm_w)[i]; if (d4) aux = d4[i]; }
      }
      if (PRO == kRmsnorm && d4) { v.x += aux.x; v.y += aux.y; v.z += aux.z; v.w += aux.w; }
      if (PRO == kSwiglu) { v.x = gated(v.x, aux.x); v.y = gated(v.y, aux.y); v.z = gated(v.z, aux.z); v.w = gated(v.w, aux.w); }
      return v;
    };
    if (PRO == kRmsnorm) {
      // Mean square of the row, summed in a fixed order. The row goes into LDS as x * w without
      // the 1 / rms factor, which is one number for the whole row: every row total is multiplied
      // by it at the end instead (W . (x w / rms) = (W . (x w)) / rms), so the staging pass does
      // not wait for this sum and the block needs no barrier of its own for it.
      float ss = 0.f;
      int k = 0;
      for (int i = tid; i < n4; i += blockDim.x, k++) {
        float4 nv;
        const float4 v = raw(k, i, nv);
        ss += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
      }
      ss = wave_sum(ss);
      if (lane == 0) nsum[wave] = ss;
    }
    int k2 = 0;
    for (int i = tid; i < n4_padded; i += blockDim.x, k2++) {
      const bool live = i < n4;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (live) {
        float4 nv;
        v = raw(k2, i, nv);
        if (PRO == kRmsnorm) {
          if (pro.xout && blockIdx.x == 0) reinterpret_cast<float4*>(pro.xout)[i] = v;
          v.x *= nv.x; v.y *= nv.y; v.z *= nv.z; v.w *= nv.w;
        }
      }
      const int u = i / J, j = i - u * J;
      if (live) xs[((u / LPR) * J + j) * XS + (u & (LPR - 1))] = Fmt::stage(v);
      if (Fmt::kScaled) {
        float sx = (v.x + v.y) + (v.z + v.w);
        if constexpr (J == 8) {   // the unit's 8 adjacent lanes, on DPP: quads, then the other quad of the 8
          sx = dpp_add_f32<0xB1>(sx);
          sx = dpp_add_f32<0x4E>(sx);
          sx = dpp_add_f32<0x141>(sx);
        } else {
#pragma unroll
          for (int msk = J / 2; msk >= 1; msk >>= 1) sx += __shfl_xor(sx, msk, kWave);
        }
        if (live && j == 0) xsum[u] = -8.0f * sx;  // sum_k (nib_k-8) x_k = sum nib_k x_k - 8 sum x_k
      }
    }
  }
  __syncthreads();
  TLHIP_MARK(2);
  float inv = 1.0f;
  if (PRO == kRmsnorm) {
    float tot = nsum[0];
    for (int w = 1; w < nw; w++) tot += nsum[w];
    inv = 1.0f / sqrtf(tot * (1.0f / (float)(upr * Fmt::E)) + pro.eps);
  }

  float acc[R];
#pragma unroll
  for (int r = 0; r < R; r++) acc[r] = 0.f;

  // Software pipeline over the items: NS fragments in flight, each requested again right after
  // it has been consumed. Loads are branch-free in the steady-state loop, so the waits of a
  // compute cover exactly its own fragment.
  int t = 0, c = 0, nt = 0;   // the item being computed: tile, chunk; nt != t at a tile's last chunk
  const auto compute = [&](const RowFrag<Fmt, R>& cur) {   // item (t, c); nt != t ends its tile
    const int u = c * LPR + li;
    if (u < upr) {
      float4 xv[J];
#pragma unroll
      for (int j = 0; j < J; j++) xv[j] = xs[(c * J + j) * XS + li];
      if (Fmt::kScaled) {
        const float bias = xsum[u];
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = fmaf(cur.sc[r], Fmt::dot(cur.w[r], xv) + bias, acc[r]);
      } else {
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] += Fmt::dot(cur.w[r], xv);
      }
    }

    if (nt != t) {  // last chunk of tile t for this wavefront: reduce and store
      const int row0 = item_row(t);
      float v;
      int r;
      bool writer;
      if constexpr (LPR == 64) {
        v = wave_sum_rows<R>(acc, lane);   // total of row (lane*R)>>6, in every lane
        r = (lane * R) >> 6;
        writer = (lane & (64 / R - 1)) == 0;
      } else {
        // every lane of the DPP row gets every row total; lane r keeps row r
        v = 0.f;
#pragma unroll
        for (int rr = 0; rr < R; rr++) {
          const float tot = dpp_add_f32<0x140>(dpp_add_f32<0x141>(dpp_add_f32<0x4E>(dpp_add_f32<0xB1>(acc[rr]))));
          v = (li == rr) ? tot : v;
        }
        r = li;
        writer = li < R;
      }
      if (PRO == kRmsnorm) v *= inv;
      if (KW == 1) {
        if constexpr (kPair) {
          // the up row's total sits half a wavefront (64-lane form) or R/2 lanes (16-lane form) away
          const float up = LPR == 64 ? swap32(v, v).second : __shfl_down(v, R / 2, kWave);   // .second: the upper half's value in the lower lanes
          if (writer && r < R / 2 && row0 + r < N / 2) y[row0 + r] = gated(v, up);
        } else {
          if (writer && row0 + r < N) y[row0 + r] = v;
        }
      } else {
        // every wavefront of the block passes these two barriers once per tile
        if (writer) red[(wrow / R * KW + kw) * R + r] = v;
        __syncthreads();
        if constexpr (kPair) {
          float sum = 0.f;
          if (kw == 0 && li < R)
            for (int sidx = 0; sidx < KW; sidx++) sum += red[(wrow / R * KW + sidx) * R + li];
          const float up = __shfl_down(sum, R / 2, kWave);
          if (kw == 0 && li < R / 2 && row0 + li < N / 2) y[row0 + li] = gated(sum, up);
        } else if (kw == 0 && li < R && row0 + li < N) {
          float sum = 0.f;
          for (int sidx = 0; sidx < KW; sidx++) sum += red[(wrow / R * KW + sidx) * R + li];
          y[row0 + li] = sum;
        }
        __syncthreads();
      }
#pragma unroll
      for (int r2 = 0; r2 < R; r2++) acc[r2] = 0.f;
    }
  };
  const auto compute_item = [&](const RowFrag<Fmt, R>& f, int i) {
    const int ti = i / cpw, ci = i - ti * cpw;
    t = (int)blockIdx.x + ti * (int)gridDim.x;
    c = kw + ci * KW;
    nt = ci == cpw - 1 ? -1 : t;
    compute(f);
  };
  if (n_items >= NS) {
#pragma unroll
    for (int k = 1; k < NS; k++) load_item(frag[k], k);
    int it = 0;
    for (; it + 2 * NS <= n_items; it += NS) {
#pragma unroll
      for (int k = 0; k < NS; k++) {
        compute_item(frag[k], it + k);
        load_item(frag[k], it + k + NS);
      }
    }
    TLHIP_MARK(3);
    // two or three items left, two of them in flight; each case is straight-line code so that
    // its waits stay exact
    static_assert(NS == 2, "the tail below is written for two fragments");
    if (n_items - it == 2) {
      compute_item(frag[0], it);
      compute_item(frag[1], it + 1);
    } else {
      compute_item(frag[0], it);
      load_item(frag[0], it + 2);
      compute_item(frag[1], it + 1);
      compute_item(frag[0], it + 2);
    }
  } else if (n_items == 1) {   // a single item: nothing more to request
    compute_item(frag[0], 0);
  }
  TLHIP_MARK(4);
}

// Generic int4 kernel for group sizes other than 32 (group % 8 == 0): one
// wavefront per row, a lane eats one 32-bit word (8 nibbles, all in one group).
__global__ __launch_bounds__(256) void gemv_q4_generic_kernel(
    const float* __restrict__ x, const uint32_t* __restrict__ qw,
    const float* __restrict__ scales, float* __restrict__ y, int N, int K, int group) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= N) return;
  const int words = K >> 3, gpr = K / group;
  const uint32_t* wr = qw + (size_t)row * words;
  const float* sr = scales + (size_t)row * gpr;
  float acc = 0.f;
  for (int wi = lane; wi < words; wi += 64) {
    const uint32_t v = wr[wi];
    const float s = sr[(wi << 3) / group];
    const float* xp = x + (wi << 3);
    float d = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) d = fmaf((float)((int)((v >> (4 * j)) & 0xf) - 8), xp[j], d);
    acc = fmaf(s, d, acc);
  }
  acc = wave_sum(acc);
  if (lane == 0) y[row] = acc;
}

// ---------------------------------------------------------------------------
// column kernel: B is [K][N], N contiguous
// ---------------------------------------------------------------------------
template <typename T> struct ColVec;
template <> struct ColVec<float> {
  static constexpr int V = 4;
  using Raw = float4;
  static __device__ __forceinline__ void fma(float (&acc)[4], float a, const Raw b) {
    acc[0] = fmaf(a, b.x, acc[0]); acc[1] = fmaf(a, b.y, acc[1]);
    acc[2] = fmaf(a, b.z, acc[2]); acc[3] = fmaf(a, b.w, acc[3]);
  }
};
template <> struct ColVec<uint16_t> {
  static constexpr int V = 8;
  using Raw = uint4;
  static __device__ __forceinline__ void fma(float (&acc)[8], float a, const Raw b) {
    acc[0] = fmaf(a, bf16_lo(b.x), acc[0]); acc[1] = fmaf(a, bf16_hi(b.x), acc[1]);
    acc[2] = fmaf(a, bf16_lo(b.y), acc[2]); acc[3] = fmaf(a, bf16_hi(b.y), acc[3]);
    acc[4] = fmaf(a, bf16_lo(b.z), acc[4]); acc[5] = fmaf(a, bf16_hi(b.z), acc[5]);
    acc[6] = fmaf(a, bf16_lo(b.w), acc[6]); acc[7] = fmaf(a, bf16_hi(b.w), acc[7]);
  }
};

// grid = (ceil(N/(64*V)), S). Block = 4 wavefronts on the same 64*V columns,
// wavefront w takes rows k0+w, k0+w+4, ... of this block's K range.
// out = y when S == 1, else partials [S][N].
template <typename T>
__global__ __launch_bounds__(256) void gemv_cols_kernel(const float* __restrict__ a,
                                                        const T* __restrict__ B,
                                                        float* __restrict__ out, int N, int K,
                                                        int kchunk) {
  constexpr int V = ColVec<T>::V;
  using Raw = typename ColVec<T>::Raw;
  __shared__ float red[3][64][V + 1];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = (blockIdx.x * 64 + lane) * V;
  const int k0 = blockIdx.y * kchunk;
  const int k1 = min(K, k0 + kchunk);
  float acc[V];
#pragma unroll
  for (int v = 0; v < V; v++) acc[v] = 0.f;
  if (col < N) {  // N % V == 0 is guaranteed by the launcher
    const T* bp = B + col;
    int k = k0 + w;
    for (; k + 28 < k1; k += 32) {  // 8 rows in flight per lane
      Raw b[8];
#pragma unroll
      for (int u = 0; u < 8; u++) b[u] = *reinterpret_cast<const Raw*>(bp + (size_t)(k + 4 * u) * N);
#pragma unroll
      for (int u = 0; u < 8; u++) ColVec<T>::fma(acc, a[k + 4 * u], b[u]);
    }
    for (; k < k1; k += 4) {
      const Raw b0 = *reinterpret_cast<const Raw*>(bp + (size_t)k * N);
      ColVec<T>::fma(acc, a[k], b0);
    }
  }
  if (w > 0) {
#pragma unroll
    for (int v = 0; v < V; v++) red[w - 1][lane][v] = acc[v];
  }
  __syncthreads();
  if (w == 0 && col < N) {
    float* o = out + (size_t)blockIdx.y * N + col;
#pragma unroll
    for (int v = 0; v < V; v++) o[v] = ((acc[v] + red[0][lane][v]) + red[1][lane][v]) + red[2][lane][v];
  }
}

// scalar-column fallback (N not a multiple of the vector width): one lane per column
template <typename T>
__global__ __launch_bounds__(256) void gemv_cols_scalar_kernel(const float* __restrict__ a,
                                                               const T* __restrict__ B,
                                                               float* __restrict__ out, int N,
                                                               int K, int kchunk) {
  const int col = blockIdx.x * blockDim.x + threadIdx.x;
  if (col >= N) return;
  const int k0 = blockIdx.y * kchunk, k1 = min(K, k0 + kchunk);
  float acc = 0.f;
  for (int k = k0; k < k1; k++) {
    float b;
    if constexpr (sizeof(T) == 2) b = __uint_as_float((uint32_t)B[(size_t)k * N + col] << 16);
    else b = B[(size_t)k * N + col];
    acc = fmaf(a[k], b, acc);
  }
  out[(size_t)blockIdx.y * N + col] = acc;
}

// y[i] = sum over s of part[s][i], fixed order. The kernel is latency, not bytes: a block is
// 64 columns x 16 split groups, a thread requests up to eight of its splits at once (s = g,
// g + 16, ...), and the 16 group sums meet in LDS in group order.
__global__ __launch_bounds__(1024) void reduce_partials_kernel(const float* __restrict__ part,
                                                               float* __restrict__ y, int N,
                                                               int S) {
  __shared__ float red[16][64];
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int i = blockIdx.x * 64 + lane;
  float acc = 0.f;
  if (i < N) {
    for (int s0 = g; s0 < S; s0 += 128) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int s = s0 + 16 * u;
        v[u] = s < S ? part[(size_t)s * N + i] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 8; u++) acc += v[u];
    }
  }
  red[g][lane] = acc;
  __syncthreads();
  if (g == 0 && i < N) {
    float t = red[0][lane];
#pragma unroll
    for (int k = 1; k < 16; k++) t += red[k][lane];
    y[i] = t;
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

struct RowCfg { int R, KW, nw, lpr, blocks; size_t lds; };
struct RowTune { int R, KW, bpc, nw, lpr; };

// Launch shape for the row kernel, from sweeps on MI355X. With two work items in flight per
// wavefront the memory pipe saturates at 8 to 16 wavefronts per CU, and HBM runs best when the
// blocks that are active at one time cover a narrow band of the matrix, so the shapes below are
// smaller than occupancy alone would suggest:
//  * lanes per row: 16 when the 64-lane form would leave a large part of the lanes without
//    a unit (K = 896 is 28 units per row), else 64;
//  * many rows per CU: whole rows per wavefront (KW = 1), 2 to 4 rows in flight per lane group;
//  * few rows per CU: K is split over KW wavefronts of a block so that every CU still has a
//    tile, one chunk per wavefront where the chunks allow it.
static RowCfg pick_rows_cfg(int64_t N, int upr, int E, int cus, int lds_per_cu, const RowTune& tn) {
  RowCfg c{};
  const double waste64 = (double)((upr + 63) / 64 * 64) / upr, waste16 = (double)((upr + 15) / 16 * 16) / upr;
  int lpr = (waste64 >= 1.3 && waste16 < waste64) ? 16 : 64;
  if (tn.lpr == 16 || tn.lpr == 64) lpr = tn.lpr;
  const int qn = 64 / lpr;
  const int chunks = (upr + lpr - 1) / lpr;
  const int xs_stride = lpr + (E == 32 ? 2 : 8);   // float4s per staged row, as in the kernel
  const size_t xbytes = (size_t)chunks * (E / 4) * xs_stride * 16 + (size_t)chunks * lpr * 4;
  const int64_t rows_per_cu = N / cus;
  int nw, R, KW, want_bpc;
  if (lpr == 64) {
    if (rows_per_cu >= 512) { nw = 16; R = 4; KW = 2; want_bpc = 1; }        // LM head
    else if (rows_per_cu >= 128) { nw = 8; R = 4; KW = 1; want_bpc = 1; }    // 7B gate|up
    else if (rows_per_cu >= 32) { nw = 8; R = 2; KW = 1; want_bpc = 1; }     // 7B up-projection alone
    else if (rows_per_cu >= 17) {                                            // 7B q|k|v
      // one tile per CU: as many 4-row groups as a CU's share of the rows needs, K over two wavefronts
      const int groups = (int)(((N + cus - 1) / cus + 3) / 4);
      R = 4; KW = 2; nw = 2 * (groups < 8 ? groups : 8); want_bpc = 2;
    } else if (rows_per_cu >= 8) {
      if (chunks <= 3) { nw = 8; R = 4; KW = 2; want_bpc = 2; }              // 7B o-projection
      else { nw = 16; R = 2; KW = 2; want_bpc = 1; }                         // 7B down-projection (K = 18944)
    } else {                                                                 // a few rows per CU
      KW = chunks < 3 ? chunks : 3;
      nw = 2 * KW; want_bpc = 2;
      R = N / 4 >= cus ? 2 : 1;                                              // two row groups a block: keep every CU busy
    }
  } else {
    if (rows_per_cu >= 256) { nw = 8; R = 1; KW = 1; want_bpc = 2; }         // 0.5B LM head
    else if (rows_per_cu >= 32) { nw = 4; R = 1; KW = 2; want_bpc = 4; }     // 0.5B gate|up
    else if (rows_per_cu >= 8) { nw = 8; R = 1; KW = 2; want_bpc = 2; }
    else { nw = 4; R = 1; KW = 1; want_bpc = 4; }
  }
  while (KW > chunks) {  // not enough K to split that far: more row groups instead
    KW /= 2;
    if (R > 1) R /= 2; else if (nw > 4) nw /= 2;
  }
  if (tn.nw > 0) nw = tn.nw;
  if (tn.R > 0) R = tn.R;
  if (tn.KW > 0) KW = tn.KW;
  if (R >= 8 && nw > 8) nw = 8;  // the 8-row variant is built for <= 512 threads
  if (KW > nw) KW = nw;
  if (nw % KW) nw -= nw % KW;    // whole row groups only (an override may ask for anything)
  int bpc = (int)((size_t)lds_per_cu / (xbytes + 4096));
  const int max_by_waves = 32 / nw > 0 ? 32 / nw : 1;
  if (tn.nw > 0) want_bpc = nw >= 16 ? 1 : nw == 8 ? 2 : 4;   // an overridden block size: the old default
  if (bpc > max_by_waves) bpc = max_by_waves;
  if (bpc > want_bpc) bpc = want_bpc;
  if (bpc < 1) bpc = 1;
  if (tn.bpc > 0) bpc = tn.bpc;
  c.R = R;
  c.KW = KW;
  c.nw = nw;
  c.lpr = lpr;
  const int rows_per_tile = (nw / KW) * qn * R;
  const int64_t ntiles = (N + rows_per_tile - 1) / rows_per_tile;
  const int64_t maxb = (int64_t)cus * bpc;
  c.blocks = (int)(ntiles < maxb ? ntiles : maxb);
  c.lds = xbytes + (size_t)nw * qn * 8 * 4 + 64;   // x, per-unit sums, K-split partials
  return c;
}

template <typename Fmt, int PRO, int LPR, int EPI>
static auto pick_rows_fn(int R) -> void (*)(const float*, const uint4*, const float*, float*, int, int,
                                            int, int, const Producer) {
  switch (R) {
    case 1:
      if constexpr (EPI == kStore) return gemv_rows_kernel<Fmt, 1, PRO, LPR, EPI>;
      else return nullptr;
    case 2: return gemv_rows_kernel<Fmt, 2, PRO, LPR, EPI>;
    case 4: return gemv_rows_kernel<Fmt, 4, PRO, LPR, EPI>;
    case 8: return gemv_rows_kernel<Fmt, 8, PRO, LPR, EPI>;
    default: return nullptr;
  }
}

// N counts the rows of W; with EPI = kGateUp, y has N / 2 entries.
template <typename Fmt, int PRO = kPlain, int EPI = kStore>
static int launch_rows(const float* x, const void* W, const float* scales, float* y, int64_t N,
                       int64_t K, int census_id, const RowTune tn = RowTune{0, 0, 0, 0, 0},
                       const Producer pro = Producer{nullptr, nullptr, nullptr, 0.f, 0, 0, 0}) {
  Context& c = ctx();
  const int upr = (int)(K / Fmt::E);
  if (upr >= (1 << 24)) return fail(TLHIP_EUNSUPPORTED, "gemv: K too large");
  // The kernel addresses a matrix with 32-bit byte offsets and 24-bit row numbers:
  // larger ones are walked in row ranges of < 4 GiB, one launch each.
  int64_t max_rows = (((int64_t)1 << 32) - 16) / ((int64_t)upr * 16);
  if (max_rows >= (1 << 24)) max_rows = (1 << 24) - 1;
  max_rows &= ~(int64_t)255;
  if (max_rows <= 0) return fail(TLHIP_EUNSUPPORTED, "gemv: K too large");
  if (EPI == kGateUp && N > max_rows) return fail(TLHIP_EUNSUPPORTED, "gemv: gate|up matrix too large for one launch");
  for (int64_t n0 = 0; n0 < N; n0 += max_rows) {
    const int64_t n = N - n0 < max_rows ? N - n0 : max_rows;
    RowCfg cfg = pick_rows_cfg(n, upr, Fmt::E, c.cus, c.lds_per_cu, tn);
    if (EPI == kGateUp && cfg.R == 1) {   // a lane group needs a gate row and its up row
      RowTune two = tn;
      two.R = 2;
      if (cfg.nw / cfg.KW >= 2 && cfg.nw > 4) two.nw = cfg.nw / 2;   // keeps the rows of a block tile
      cfg = pick_rows_cfg(n, upr, Fmt::E, c.cus, c.lds_per_cu, two);
    }
    if (PRO == kAttnMerge) cfg.lds += (size_t)pro.heads * (kMergeMax + 1) * sizeof(float);
    if (cfg.lds > (size_t)c.lds_per_cu) return fail(TLHIP_EUNSUPPORTED, "gemv: K too large for the LDS-staged kernel");
    const int rows_per_tile = (cfg.nw / cfg.KW) * (64 / cfg.lpr) * cfg.R;
    const int ntiles = (int)((n + rows_per_tile - 1) / rows_per_tile);
    auto fn = cfg.lpr == 16 ? pick_rows_fn<Fmt, PRO, 16, EPI>(cfg.R) : pick_rows_fn<Fmt, PRO, 64, EPI>(cfg.R);
    if (!fn) return fail(TLHIP_EINVAL, "rows per wavefront must be 1, 2, 4 or 8");
    if (cfg.lds > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)cfg.lds);
      if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(LDS)");
    }
    const uint4* Wn = static_cast<const uint4*>(W) + (size_t)n0 * upr;
    const float* sn = scales ? scales + (size_t)n0 * upr : nullptr;
    hipLaunchKernelGGL(fn, dim3(cfg.blocks), dim3(cfg.nw * 64), cfg.lds, c.stream, x, Wn, sn, y + n0,
                       (int)n, upr, cfg.KW, ntiles, pro);
  }
  TLHIP_CHECK_LAUNCH(census_id);
}

template <typename T>
static int launch_cols(const float* a, const T* B, float* y, int64_t N, int64_t K, int census_id) {
  Context& c = ctx();
  constexpr int V = ColVec<T>::V;
  const bool vec = (N % V) == 0 && aligned16(B);
  const int64_t ctiles = vec ? (N + 64 * V - 1) / (64 * V) : (N + 255) / 256;
  // K splits: fill ~4 blocks per CU, keep >= 128 rows per split (32 per wavefront)
  int64_t S = ((int64_t)c.cus * 4 + ctiles - 1) / ctiles;
  if (S > K / 128) S = K / 128;
  if (c.tune_cols_max_splits > 0 && S > c.tune_cols_max_splits) S = c.tune_cols_max_splits;
  if (S < 1) S = 1;
  int kchunk = (int)((K + S - 1) / S);
  kchunk = (kchunk + 3) & ~3;
  S = (K + kchunk - 1) / kchunk;
  float* out = y;
  if (S > 1) {
    out = static_cast<float*>(scratch((size_t)S * N * sizeof(float)));
    if (!out) return fail(TLHIP_ENOMEM, "gemv: no scratch for %lld K-splits", (long long)S);
  }
  if (vec)
    hipLaunchKernelGGL(gemv_cols_kernel<T>, dim3((unsigned)ctiles, (unsigned)S), dim3(256), 0,
                       c.stream, a, B, out, (int)N, (int)K, kchunk);
  else
    hipLaunchKernelGGL(gemv_cols_scalar_kernel<T>, dim3((unsigned)ctiles, (unsigned)S), dim3(256),
                       0, c.stream, a, B, out, (int)N, (int)K, kchunk);
  if (S > 1)
    hipLaunchKernelGGL(reduce_partials_kernel, dim3((unsigned)((N + 63) / 64)), dim3(1024), 0,
                       c.stream, out, y, (int)N, (int)S);
  TLHIP_CHECK_LAUNCH(census_id);
}

static RowTune q4_tune(const Context& c) {
  return RowTune{c.tune_q4_rows, c.tune_q4_kw, c.tune_q4_bpc, c.tune_q4_nw, c.tune_q4_lpr};
}

// int4, group 32, through the row kernel.
template <int PRO, int EPI>
static int launch_q4(const float* x, const void* W, const float* scales, float* y, int64_t N, int64_t K,
                     const Producer pro = Producer{nullptr, nullptr, nullptr, 0.f, 0, 0, 0}) {
  return launch_rows<FmtQ4, PRO, EPI>(x, W, scales, y, N, K, TLHIP_C_GEMV_Q4, q4_tune(ctx()), pro);
}

static int check_gemv_args(const void* a, const void* B, const void* y, int64_t n, int64_t k,
                           const char* who) {
  if (!a || !B || !y) return fail(TLHIP_EINVAL, "%s: null pointer", who);
  if (n <= 0 || k <= 0) return fail(TLHIP_EINVAL, "%s: n and k must be positive", who);
  if (n > (int64_t)1 << 30 || k > (int64_t)1 << 30)
    return fail(TLHIP_EUNSUPPORTED, "%s: dimension beyond 2^30", who);
  if (!aligned16(a)) return fail(TLHIP_EINVAL, "%s: activation pointer not 16-byte aligned", who);
  return 0;
}

}  // namespace tlhip

using namespace tlhip;

extern "C" {

int tlhip_gemv_q4(const void* a, const void* qw, const void* scales, void* y, int64_t N,
                  int64_t K, int64_t group) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(a, qw, y, N, K, "tlhip_gemv_q4")) return rc;
  if (!scales) return fail(TLHIP_EINVAL, "tlhip_gemv_q4: null scales");
  // the reference's gate (cuda.h:889-890)
  if (group <= 0 || (K % group) != 0 || (group % 8) != 0)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemv_q4: need group>0, K%%group==0, group%%8==0");
  Context& c = ctx();
  const size_t xbytes = (size_t)((K / 32 + 63) / 64) * 66 * 32 * 4;
  if (group == 32 && aligned16(qw) && xbytes + 2048 <= (size_t)c.lds_per_cu)
    return launch_q4<kPlain, kStore>(static_cast<const float*>(a), qw, static_cast<const float*>(scales),
                                     static_cast<float*>(y), N, K);
  hipLaunchKernelGGL(gemv_q4_generic_kernel, dim3((unsigned)((N + 3) / 4)), dim3(256), 0, c.stream,
                     static_cast<const float*>(a), static_cast<const uint32_t*>(qw),
                     static_cast<const float*>(scales), static_cast<float*>(y), (int)N, (int)K,
                     (int)group);
  TLHIP_CHECK_LAUNCH(TLHIP_C_GEMV_Q4);
}

int tlhip_gemv_bf16_row(const void* a, const void* W, void* y, int64_t n, int64_t k) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(a, W, y, n, k, "tlhip_gemv_bf16_row")) return rc;
  if ((k % 8) != 0) return fail(TLHIP_EUNSUPPORTED, "tlhip_gemv_bf16_row: K %% 8 != 0");  // cuda.h:772
  if (!aligned16(W)) return fail(TLHIP_EINVAL, "tlhip_gemv_bf16_row: weight pointer not 16-byte aligned");
  const size_t xbytes = (size_t)((k / 8 + 63) / 64) * 72 * 8 * 4;
  if (xbytes + 2048 > (size_t)ctx().lds_per_cu)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemv_bf16_row: K too large for the LDS-staged kernel");
  return launch_rows<FmtBf16>(static_cast<const float*>(a), W, nullptr, static_cast<float*>(y), n, k,
                              TLHIP_C_GEMV_BF16_ROW);
}

static int check_attn_merge(const void* parts, int64_t n_parts, int64_t heads, int64_t D, int64_t K, const char* who) {
  if (!parts || !aligned16(parts)) return fail(TLHIP_EINVAL, "%s: partials pointer null or not 16-byte aligned", who);
  if (heads <= 0 || heads > 4096 || (D != 64 && D != 128) || heads * D != K)
    return fail(TLHIP_EINVAL, "%s: K must be heads x head_dim, head_dim 64 or 128", who);
  // as many splits as the merge kernel sums one after the other: one per column group of its 1024 threads
  const int64_t most = D == 64 ? kMergeMax : kMergeMax / 2;
  if (n_parts < 1 || n_parts > most) return fail(TLHIP_EUNSUPPORTED, "%s: 1 to %d split partials", who, (int)most);
  if (((2 * heads * n_parts) % 4) != 0) return fail(TLHIP_EUNSUPPORTED, "%s: heads x splits must be even", who);
  return 0;
}

int tlhip_gemv_q4_attn(const void* parts, int64_t n_parts, int64_t heads, int64_t head_dim, const void* qw,
                       const void* scales, void* y, int64_t N, int64_t K, int64_t group) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(parts, qw, y, N, K, "tlhip_gemv_q4_attn")) return rc;
  if (int rc = check_attn_merge(parts, n_parts, heads, head_dim, K, "tlhip_gemv_q4_attn")) return rc;
  if (!scales || group != 32 || !aligned16(qw)) return fail(TLHIP_EUNSUPPORTED, "tlhip_gemv_q4_attn: group 32, aligned weights");
  const size_t xbytes = (size_t)((K / 32 + 63) / 64) * 66 * 32 * 4;
  if (xbytes + 2048 + (size_t)heads * 68 > (size_t)ctx().lds_per_cu)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemv_q4_attn: K too large for the LDS-staged kernel");
  Producer pro{nullptr, nullptr, nullptr, 0.f, (int)n_parts, (int)heads, (int)head_dim};
  return launch_q4<kAttnMerge, kStore>(static_cast<const float*>(parts), qw, static_cast<const float*>(scales),
                                       static_cast<float*>(y), N, K, pro);
}

int tlhip_gemv_bf16_row_attn(const void* parts, int64_t n_parts, int64_t heads, int64_t head_dim, const void* W,
                             void* y, int64_t n, int64_t k) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(parts, W, y, n, k, "tlhip_gemv_bf16_row_attn")) return rc;
  if (int rc = check_attn_merge(parts, n_parts, heads, head_dim, k, "tlhip_gemv_bf16_row_attn")) return rc;
  if (!aligned16(W)) return fail(TLHIP_EINVAL, "tlhip_gemv_bf16_row_attn: weight pointer not 16-byte aligned");
  const size_t xbytes = (size_t)((k / 8 + 63) / 64) * 72 * 8 * 4;
  if (xbytes + 2048 + (size_t)heads * 68 > (size_t)ctx().lds_per_cu)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemv_bf16_row_attn: K too large for the LDS-staged kernel");
  Producer pro{nullptr, nullptr, nullptr, 0.f, (int)n_parts, (int)heads, (int)head_dim};
  return launch_rows<FmtBf16, kAttnMerge>(static_cast<const float*>(parts), W, nullptr, static_cast<float*>(y), n, k,
                                          TLHIP_C_GEMV_BF16_ROW, RowTune{0, 0, 0, 0, 0}, pro);
}

int tlhip_gemv_f32(const void* a, const void* B, void* y, int64_t n, int64_t k) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(a, B, y, n, k, "tlhip_gemv_f32")) return rc;
  return launch_cols<float>(static_cast<const float*>(a), static_cast<const float*>(B),
                            static_cast<float*>(y), n, k, TLHIP_C_GEMV_F32);
}

int tlhip_gemv_bf16(const void* a, const void* B, void* y, int64_t n, int64_t k) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(a, B, y, n, k, "tlhip_gemv_bf16")) return rc;
  return launch_cols<uint16_t>(static_cast<const float*>(a), static_cast<const uint16_t*>(B),
                               static_cast<float*>(y), n, k, TLHIP_C_GEMV_BF16);
}

// ---- GEMVs that produce their own activation vector ------------------------------------------

static int check_fused_q4(const void* qw, const void* scales, int64_t K, int64_t group, size_t in_floats,
                          const char* who) {
  if (!scales) return fail(TLHIP_EINVAL, "%s: null scales", who);
  if (group != 32 || (K % 32) != 0 || !aligned16(qw))
    return fail(TLHIP_EUNSUPPORTED, "%s: fused form needs group 32, K %% 32 == 0, aligned weights", who);
  const size_t xbytes = (size_t)((K / 32 + 63) / 64) * 66 * 32 * 4;
  if (xbytes + 2048 > (size_t)ctx().lds_per_cu)
    return fail(TLHIP_EUNSUPPORTED, "%s: K too large for the LDS-staged kernel", who);
  (void)in_floats;
  return 0;
}

static int check_fused_bf16(const void* W, int64_t K, const char* who) {
  if ((K % 8) != 0 || !aligned16(W))
    return fail(TLHIP_EUNSUPPORTED, "%s: need K %% 8 == 0 and aligned weights", who);
  const size_t xbytes = (size_t)((K / 8 + 63) / 64) * 72 * 8 * 4;
  if (xbytes + 2048 > (size_t)ctx().lds_per_cu)
    return fail(TLHIP_EUNSUPPORTED, "%s: K too large for the LDS-staged kernel", who);
  return 0;
}

static int check_norm_args(const void* x, const void* delta, const void* norm_w, const void* xout,
                           const char* who) {
  if (!norm_w) return fail(TLHIP_EINVAL, "%s: null norm weight", who);
  if (!aligned16(norm_w) || (delta && !aligned16(delta)) || (xout && !aligned16(xout)))
    return fail(TLHIP_EINVAL, "%s: vectors must be 16-byte aligned", who);
  if (xout && (xout == x || xout == delta))
    return fail(TLHIP_EINVAL, "%s: xout must not alias x or delta (other blocks still read them)", who);
  return 0;
}

int tlhip_gemv_q4_swiglu(const void* gu, const void* qw, const void* scales, void* y, int64_t N,
                         int64_t K, int64_t group) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(gu, qw, y, N, K, "tlhip_gemv_q4_swiglu")) return rc;
  if (int rc = check_fused_q4(qw, scales, K, group, 2 * K, "tlhip_gemv_q4_swiglu")) return rc;
  return launch_q4<kSwiglu, kStore>(static_cast<const float*>(gu), qw, static_cast<const float*>(scales),
                                    static_cast<float*>(y), N, K);
}

int tlhip_gemv_q4_rmsnorm(const void* x, const void* delta, const void* norm_w, void* xout,
                          const void* qw, const void* scales, void* y, int64_t N, int64_t K,
                          int64_t group, float eps) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(x, qw, y, N, K, "tlhip_gemv_q4_rmsnorm")) return rc;
  if (int rc = check_fused_q4(qw, scales, K, group, K, "tlhip_gemv_q4_rmsnorm")) return rc;
  if (int rc = check_norm_args(x, delta, norm_w, xout, "tlhip_gemv_q4_rmsnorm")) return rc;
  const Producer pro{static_cast<const float*>(delta), static_cast<const float*>(norm_w),
                     static_cast<float*>(xout), eps};
  return launch_q4<kRmsnorm, kStore>(static_cast<const float*>(x), qw, static_cast<const float*>(scales),
                                     static_cast<float*>(y), N, K, pro);
}

int tlhip_gemv_q4_rmsnorm_gateup(const void* x, const void* delta, const void* norm_w, void* xout,
                                 const void* qw, const void* scales, void* act, int64_t N2, int64_t K,
                                 int64_t group, float eps) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(x, qw, act, N2, K, "tlhip_gemv_q4_rmsnorm_gateup")) return rc;
  if (N2 % 2) return fail(TLHIP_EINVAL, "tlhip_gemv_q4_rmsnorm_gateup: odd row count %lld", (long long)N2);
  if (int rc = check_fused_q4(qw, scales, K, group, K, "tlhip_gemv_q4_rmsnorm_gateup")) return rc;
  if (int rc = check_norm_args(x, delta, norm_w, xout, "tlhip_gemv_q4_rmsnorm_gateup")) return rc;
  const Producer pro{static_cast<const float*>(delta), static_cast<const float*>(norm_w),
                     static_cast<float*>(xout), eps};
  return launch_q4<kRmsnorm, kGateUp>(static_cast<const float*>(x), qw, static_cast<const float*>(scales),
                                      static_cast<float*>(act), N2, K, pro);
}

int tlhip_gemv_bf16_row_rmsnorm_gateup(const void* x, const void* delta, const void* norm_w, void* xout,
                                       const void* W, void* act, int64_t n2, int64_t k, float eps) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(x, W, act, n2, k, "tlhip_gemv_bf16_row_rmsnorm_gateup")) return rc;
  if (n2 % 2) return fail(TLHIP_EINVAL, "tlhip_gemv_bf16_row_rmsnorm_gateup: odd row count %lld", (long long)n2);
  if (int rc = check_fused_bf16(W, k, "tlhip_gemv_bf16_row_rmsnorm_gateup")) return rc;
  if (int rc = check_norm_args(x, delta, norm_w, xout, "tlhip_gemv_bf16_row_rmsnorm_gateup")) return rc;
  const Producer pro{static_cast<const float*>(delta), static_cast<const float*>(norm_w),
                     static_cast<float*>(xout), eps};
  return launch_rows<FmtBf16, kRmsnorm, kGateUp>(static_cast<const float*>(x), W, nullptr,
                                                 static_cast<float*>(act), n2, k, TLHIP_C_GEMV_BF16_ROW,
                                                 RowTune{0, 0, 0, 0, 0}, pro);
}

int tlhip_gemv_bf16_row_swiglu(const void* gu, const void* W, void* y, int64_t n, int64_t k) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(gu, W, y, n, k, "tlhip_gemv_bf16_row_swiglu")) return rc;
  if (int rc = check_fused_bf16(W, k, "tlhip_gemv_bf16_row_swiglu")) return rc;
  return launch_rows<FmtBf16, kSwiglu>(static_cast<const float*>(gu), W, nullptr, static_cast<float*>(y),
                                       n, k, TLHIP_C_GEMV_BF16_ROW);
}

int tlhip_gemv_bf16_row_rmsnorm(const void* x, const void* delta, const void* norm_w, void* xout,
                                const void* W, void* y, int64_t n, int64_t k, float eps) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(x, W, y, n, k, "tlhip_gemv_bf16_row_rmsnorm")) return rc;
  if (int rc = check_fused_bf16(W, k, "tlhip_gemv_bf16_row_rmsnorm")) return rc;
  if (int rc = check_norm_args(x, delta, norm_w, xout, "tlhip_gemv_bf16_row_rmsnorm")) return rc;
  const Producer pro{static_cast<const float*>(delta), static_cast<const float*>(norm_w),
                     static_cast<float*>(xout), eps};
  return launch_rows<FmtBf16, kRmsnorm>(static_cast<const float*>(x), W, nullptr, static_cast<float*>(y),
                                        n, k, TLHIP_C_GEMV_BF16_ROW, RowTune{0, 0, 0, 0, 0}, pro);
}

}  // extern "C"
