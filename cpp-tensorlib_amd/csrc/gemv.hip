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

namespace tlhip {

// ---------------------------------------------------------------------------
// weight formats for the row kernel
// ---------------------------------------------------------------------------

// 16-byte streaming load: weights are read exactly once per GEMV, so they are
// marked non-temporal and do not displace x and the scales in the caches.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_stream16(const uint4* p) {
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

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

struct FmtQ4 {
  static constexpr int E = 32;  // weights per 16-byte unit == one scale group
  static constexpr bool kScaled = true;
  // staged form of (x_even, x_odd, x_even, x_odd)
  static __device__ __forceinline__ float4 stage(const float4 v) {
    const float o0 = v.y * 0.0625f, o1 = v.w * 0.0625f;
    return make_float4(v.x - o0, o0, v.z - o1, o1);
  }
  // sum_k nib_k * x_k over the unit, x in staged form
  static __device__ __forceinline__ float dot(const uint4 w, const float4 (&x)[8]) {
    const uint32_t d[4] = {w.x, w.y, w.z, w.w};
    float a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t full = d[i], lo = low_nibbles(full);
      const float4 xa = x[2 * i], xb = x[2 * i + 1];
      a0 = fmaf(byte0(lo), xa.x, a0);
      a1 = fmaf(byte0(full), xa.y, a1);
      a0 = fmaf(byte1(lo), xa.z, a0);
      a1 = fmaf(byte1(full), xa.w, a1);
      a0 = fmaf(byte2(lo), xb.x, a0);
      a1 = fmaf(byte2(full), xb.y, a1);
      a0 = fmaf(byte3(lo), xb.z, a0);
      a1 = fmaf(byte3(full), xb.w, a1);
    }
    return a0 + a1;
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

// ---------------------------------------------------------------------------
// row kernel
// ---------------------------------------------------------------------------
// W: [N][upr] 16-byte units. scales: [N][upr] f32 (int4 only).
// Block = nw wavefronts arranged as (nw/KW row groups) x (KW K-splits).
// LDS: x as float4 xs[(chunk*J + j)*64 + lane], J = E/4, so that lane l's j-th
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
  if (u < upr) {
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
}

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
// How a block leaves its results (EPI):
//   kStore:  y[row] = dot.
//   kGateUp: W is [gate rows | up rows] (N/2 each); a lane group owns R/2 gate rows and the
//            matching up rows, and writes y[i] = (g*sigmoid(g))*u for i < N/2 - the gated
//            activation in the GEMV that produces it, once per element, instead of in every
//            block of the GEMV that consumes it.
enum { kPlain = 0, kSwiglu = 1, kRmsnorm = 2 };
enum { kStore = 0, kGateUp = 1 };
__device__ __forceinline__ float gated(float g, float u) { return (g * (1.0f / (1.0f + expf(-g)))) * u; }
struct Producer {
  const float* delta;
  const float* norm_w;
  float* xout;
  float eps;
};

// LPR = lanes that share a weight row: 64 (a row segment of 64 units per
// wavefront step) or 16 (the wavefront works on 4 row groups at once, 16 units
// of each per step). Rows whose unit count is not close to a multiple of 64 leave
// lanes idle in the 64-lane form (K = 3584 is 112 units: 12.5 % idle; K = 896 is
// 28 units: 56 % idle); the 16-lane form wastes at most 15 units per row and
// finishes a row sum inside one DPP row.
template <typename Fmt, int R, int PRO, int LPR, int EPI = kStore>
__global__ __launch_bounds__(R >= 8 ? 512 : 1024) void gemv_rows_kernel(
    const float* __restrict__ x, const uint4* __restrict__ W, const float* __restrict__ scales,
    float* __restrict__ y, int N, int upr, int KW, int ntiles, const Producer pro) {
  constexpr int J = Fmt::E / 4;
  constexpr int QN = 64 / LPR;       // row groups a wavefront works on at once
  extern __shared__ float4 smem4[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & (LPR - 1), q = lane / LPR;
  const int nw = blockDim.x >> 6;
  const int chunks = (upr + LPR - 1) / LPR;
  float4* xs = smem4;
  float* xsum = reinterpret_cast<float*>(smem4 + (size_t)chunks * J * LPR);  // [chunks*LPR], int4 only
  float* red = xsum + (Fmt::kScaled ? chunks * LPR : 0);

  const int kw = wave % KW;          // which K split this wavefront takes
  const int wn = wave / KW;          // which row group of the block tile
  const int groups = nw / KW;        // wavefront row groups per block tile
  const int rows_per_tile = groups * QN * R;
  const int wrow = (wn * QN + q) * R;  // this lane's first row inside a tile
  constexpr bool kPair = EPI == kGateUp;
  static_assert(!kPair || R >= 2, "a gate/up pair needs two rows per lane group");
  // first row of work item (tile tt): a row of W, or with kPair a row of each half
  const auto item_row = [&](int tt) { return kPair ? (tt * rows_per_tile + wrow) >> 1 : tt * rows_per_tile + wrow; };

  // The first work item's weights are requested before x is staged, so that the
  // HBM latency of the weights and the L2 latency of x overlap.
  int t = blockIdx.x, c = kw;
  RowFrag<Fmt, R> cur;
  if (t < ntiles) load_frag<Fmt, R, kPair>(cur, W, scales, N, upr, item_row(t), c * LPR + li);

  {  // stage x (K = upr*E floats) into the interleaved layout, one pass:
     // thread i owns float4 i; the J threads of a unit are adjacent lanes, so the
     // unit's sum(x) is a J-lane shuffle reduction (J is 8 or 2, both divide 64).
    const float4* x4 = reinterpret_cast<const float4*>(x);
    const int n4 = upr * J;
    const int n4_padded = (n4 + 63) & ~63;   // whole wavefronts take part in the shuffles
    const float4* d4 = reinterpret_cast<const float4*>(pro.delta);
    float inv = 0.f;
    // the first two float4s a thread owns (all of them for rows up to 2 * blockDim * 4
    // floats) stay in registers between the two passes of the norm
    float4 kept0 = make_float4(0.f, 0.f, 0.f, 0.f), kept1 = kept0;
    float4 keptw0 = kept0, keptw1 = kept0;   // their norm weights, requested ahead of the block sum
    if (PRO == kRmsnorm) {   // mean square of the row, summed in a fixed order
      float ss = 0.f;
      int it = 0;
      for (int i = tid; i < n4; i += blockDim.x, it++) {
        float4 v = x4[i];
        if (it == 0) keptw0 = reinterpret_cast<const float4*>(pro.norm_w)[i];
        if (it == 1) keptw1 = reinterpret_cast<const float4*>(pro.norm_w)[i];
        if (d4) { const float4 d = d4[i]; v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w; }
        if (it == 0) kept0 = v;
        if (it == 1) kept1 = v;
        ss += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
      }
      ss = wave_sum(ss);
      if (lane == 0) red[wave] = ss;
      __syncthreads();
      float tot = red[0];
      for (int w = 1; w < nw; w++) tot += red[w];
      inv = 1.0f / sqrtf(tot * (1.0f / (float)(n4 * 4)) + pro.eps);
      // red is reused only after the barrier that ends the staging pass
    }
    int it2 = 0;
    for (int i = tid; i < n4_padded; i += blockDim.x, it2++) {
      const bool live = i < n4;
      const bool have = PRO == kRmsnorm && it2 < 2;   // already summed with delta, in registers
      float4 v = have ? (it2 == 0 ? kept0 : kept1)
                      : live ? x4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
      if (PRO == kSwiglu && live) {
        const float4 up = x4[n4 + i];
        v.x = (v.x * (1.0f / (1.0f + expf(-v.x)))) * up.x;
        v.y = (v.y * (1.0f / (1.0f + expf(-v.y)))) * up.y;
        v.z = (v.z * (1.0f / (1.0f + expf(-v.z)))) * up.z;
        v.w = (v.w * (1.0f / (1.0f + expf(-v.w)))) * up.w;
      }
      if (PRO == kRmsnorm && live) {
        if (d4 && !have) { const float4 d = d4[i]; v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w; }
        if (pro.xout && blockIdx.x == 0) reinterpret_cast<float4*>(pro.xout)[i] = v;
        const float4 w4 = have ? (it2 == 0 ? keptw0 : keptw1) : reinterpret_cast<const float4*>(pro.norm_w)[i];
        v.x = (v.x * inv) * w4.x; v.y = (v.y * inv) * w4.y;
        v.z = (v.z * inv) * w4.z; v.w = (v.w * inv) * w4.w;
      }
      const int u = i / J, j = i - u * J;
      if (live) xs[((u / LPR) * J + j) * LPR + (u & (LPR - 1))] = Fmt::stage(v);
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

  float acc[R];
#pragma unroll
  for (int r = 0; r < R; r++) acc[r] = 0.f;

  // Software pipeline over this wavefront's (tile, chunk) items: the next item's
  // loads are in flight while the current one is unpacked and accumulated. The
  // two fragments swap roles every step (no register copies).
  auto step = [&](const RowFrag<Fmt, R>& cur, RowFrag<Fmt, R>& nxt) -> bool {
    int nc = c + KW, nt = t;
    if (nc >= chunks) { nc = kw; nt = t + gridDim.x; }
    if (nt < ntiles)
      load_frag<Fmt, R, kPair>(nxt, W, scales, N, upr, item_row(nt), nc * LPR + li);

    const int u = c * LPR + li;
    if (u < upr) {
      float4 xv[J];
#pragma unroll
      for (int j = 0; j < J; j++) xv[j] = xs[(c * J + j) * LPR + li];
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
    t = nt;
    c = nc;
    return t < ntiles;
  };
  RowFrag<Fmt, R> other;
  if (t < ntiles) {
    while (step(cur, other) && step(other, cur)) {
    }
  }
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

// Launch shape for the row kernel, from sweeps on MI355X:
//  * lanes per row: 16 when the 64-lane form would leave a large part of the
//    lanes without a unit (K = 896 is 28 units per row), else 64;
//  * big matrices: two 8-wavefront blocks per CU, 4 rows per wavefront;
//    otherwise one fat block per CU (16 wavefronts) so x is staged once per CU;
//  * rows per block tile grow with the rows a CU owns (the x fragment held in
//    VGPRs is reused for every row a lane group owns);
//  * K is split over KW wavefronts of a block only when rows alone cannot give
//    every CU a tile.
static RowCfg pick_rows_cfg(int64_t N, int upr, int E, int cus, int lds_per_cu, const RowTune& tn) {
  RowCfg c{};
  const double waste64 = (double)((upr + 63) / 64 * 64) / upr, waste16 = (double)((upr + 15) / 16 * 16) / upr;
  int lpr = (waste64 >= 1.3 && waste16 < waste64) ? 16 : 64;
  if (tn.lpr == 16 || tn.lpr == 64) lpr = tn.lpr;
  const int qn = 64 / lpr;
  const int chunks = (upr + lpr - 1) / lpr;
  const size_t xbytes = (size_t)chunks * lpr * E * 4 + (size_t)chunks * lpr * 4;
  const int64_t rows_per_cu = N / cus;
  int nw = 16, R, KW;
  if (lpr == 64) {
    if (rows_per_cu >= 128) { nw = 8; R = 4; KW = 1; }  // two 8-wave blocks per CU, 32-row tiles
    else if (rows_per_cu >= 64) { nw = 8; R = 4; KW = 2; }  // same blocks, 16-row tiles
    else if (rows_per_cu >= 32) { R = 2; KW = 1; }    // 32
    else if (N > 16 * (int64_t)cus) {
      // 17..31 rows per CU: 16-row tiles would leave a second, nearly empty round. Two blocks
      // per CU, one row per wavefront, as many wavefronts as make the rows one round.
      R = 1; KW = 1;
      nw = (int)((N + 2 * (int64_t)cus - 1) / (2 * (int64_t)cus));
      if (nw < 4) nw = 4;
    }
    else if (rows_per_cu >= 8) { R = 2; KW = 2; }     // 16
    else { nw = 8; R = 1; KW = 2; }                   // 4
  } else {
    if (rows_per_cu >= 256) { R = 2; KW = 1; }        // 128 rows per block tile
    else if (rows_per_cu >= 64) { R = 1; KW = 1; }    // 64
    else if (rows_per_cu >= 16) { R = 1; KW = 2; }    // 32
    else if (rows_per_cu >= 8) { R = 1; KW = 4; }     // 16
    else { nw = 8; R = 1; KW = 4; }                   // 8
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
  int bpc = (int)((size_t)lds_per_cu / (xbytes + 4096));
  const int max_by_waves = 32 / nw > 0 ? 32 / nw : 1;
  const int want_bpc = nw >= 16 ? 1 : nw == 8 ? 2 : 4;
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
                       const Producer pro = Producer{nullptr, nullptr, nullptr, 0.f}) {
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
  const size_t xbytes = (size_t)((K / 32 + 63) / 64) * 64 * 32 * 4;
  if (group == 32 && aligned16(qw) && xbytes + 2048 <= (size_t)c.lds_per_cu)
    return launch_rows<FmtQ4>(static_cast<const float*>(a), qw, static_cast<const float*>(scales),
                              static_cast<float*>(y), N, K, TLHIP_C_GEMV_Q4, q4_tune(c));
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
  const size_t xbytes = (size_t)((k / 8 + 63) / 64) * 64 * 8 * 4;
  if (xbytes + 2048 > (size_t)ctx().lds_per_cu)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemv_bf16_row: K too large for the LDS-staged kernel");
  return launch_rows<FmtBf16>(static_cast<const float*>(a), W, nullptr, static_cast<float*>(y), n, k,
                              TLHIP_C_GEMV_BF16_ROW);
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
  const size_t xbytes = (size_t)((K / 32 + 63) / 64) * 64 * 32 * 4;
  if (xbytes + 2048 > (size_t)ctx().lds_per_cu)
    return fail(TLHIP_EUNSUPPORTED, "%s: K too large for the LDS-staged kernel", who);
  (void)in_floats;
  return 0;
}

static int check_fused_bf16(const void* W, int64_t K, const char* who) {
  if ((K % 8) != 0 || !aligned16(W))
    return fail(TLHIP_EUNSUPPORTED, "%s: need K %% 8 == 0 and aligned weights", who);
  const size_t xbytes = (size_t)((K / 8 + 63) / 64) * 64 * 8 * 4;
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
  Context& c = ctx();
  return launch_rows<FmtQ4, kSwiglu>(static_cast<const float*>(gu), qw, static_cast<const float*>(scales),
                                     static_cast<float*>(y), N, K, TLHIP_C_GEMV_Q4, q4_tune(c));
}

int tlhip_gemv_q4_rmsnorm(const void* x, const void* delta, const void* norm_w, void* xout,
                          const void* qw, const void* scales, void* y, int64_t N, int64_t K,
                          int64_t group, float eps) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(x, qw, y, N, K, "tlhip_gemv_q4_rmsnorm")) return rc;
  if (int rc = check_fused_q4(qw, scales, K, group, K, "tlhip_gemv_q4_rmsnorm")) return rc;
  if (int rc = check_norm_args(x, delta, norm_w, xout, "tlhip_gemv_q4_rmsnorm")) return rc;
  Context& c = ctx();
  const Producer pro{static_cast<const float*>(delta), static_cast<const float*>(norm_w),
                     static_cast<float*>(xout), eps};
  return launch_rows<FmtQ4, kRmsnorm>(static_cast<const float*>(x), qw, static_cast<const float*>(scales),
                                      static_cast<float*>(y), N, K, TLHIP_C_GEMV_Q4, q4_tune(c), pro);
}

int tlhip_gemv_q4_rmsnorm_gateup(const void* x, const void* delta, const void* norm_w, void* xout,
                                 const void* qw, const void* scales, void* act, int64_t N2, int64_t K,
                                 int64_t group, float eps) {
  TLHIP_REQUIRE_READY();
  if (int rc = check_gemv_args(x, qw, act, N2, K, "tlhip_gemv_q4_rmsnorm_gateup")) return rc;
  if (N2 % 2) return fail(TLHIP_EINVAL, "tlhip_gemv_q4_rmsnorm_gateup: odd row count %lld", (long long)N2);
  if (int rc = check_fused_q4(qw, scales, K, group, K, "tlhip_gemv_q4_rmsnorm_gateup")) return rc;
  if (int rc = check_norm_args(x, delta, norm_w, xout, "tlhip_gemv_q4_rmsnorm_gateup")) return rc;
  Context& c = ctx();
  const Producer pro{static_cast<const float*>(delta), static_cast<const float*>(norm_w),
                     static_cast<float*>(xout), eps};
  return launch_rows<FmtQ4, kRmsnorm, kGateUp>(static_cast<const float*>(x), qw,
                                               static_cast<const float*>(scales), static_cast<float*>(act),
                                               N2, K, TLHIP_C_GEMV_Q4, q4_tune(c), pro);
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
