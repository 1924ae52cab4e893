// Causal prefill attention on the 16-bit matrix cores with fp32-level products
// (tlhip_attn_prefill deep in a context, cuda.h:1165-1201).
//
//   out[h, p, :] = softmax_k( scale * q[h, p, :] . K[kv(h), k, :] ) . V[kv(h), k, :],  k <= pos0 + p
//
// The fp32 matrix instructions share the vector ALU's multipliers: a kernel built on them runs
// its softmax and its products one after the other. v_mfma_f32_32x32x16_f16 runs on the matrix
// cores proper, 16 times faster and beside the vector ALU, but multiplies f16. Every f32 operand
// is therefore cut into TWO f16 terms, each rounded to nearest, and a product a.b is formed from
// the three term pairs that hold a first term, a1b1 + (a1b2 + a2b1), smallest first, accumulated
// in fp32 inside the MFMA; a2b2 <= 2^-24 |ab|, an fp32 rounding, is dropped. (A cache that already
// holds bf16 needs one term for K and V and two products.) f16 has 11 significant bits but a
// narrow exponent, so an operand is first multiplied by a power of two that brings its block's
// largest magnitude into [2^14, 2^15): one exponent per query row, one each for K and V per
// 32-key tile (kept beside the terms). Two terms then carry 23 bits of a value whose magnitude is
// within 2^14 of its block's largest and an absolute 2^-39 of that largest below. The Q and K
// exponents leave through the score scale; P enters as p * 2^14 and the output accumulators move
// from one tile's V exponent to the next in the multiplication that applies the softmax
// correction. Scores and outputs then differ from an fp32 loop by what a different summation
// order would give.
//
// Three kernels per call:
//  1. kv_planes_kernel cuts the cache rows [0, pos0 + T) of every kv head into terms, written as
//     the exact register image of the MFMA operands, one 32-key tile after the other (layouts at
//     the kernel), so that the attention kernel copies a tile to LDS verbatim and every operand is
//     one conflict-free 16-byte LDS read per lane. Keys at and past pos0 + T are written as zeros.
//  2. attn_w32_kernel: a block serves ONE kv head and up to 7 wavefronts of 32 query rows each
//     that all read the same K/V tiles: with grouped-query attention the query heads of the group
//     (32 positions each), else consecutive runs of positions. The 32-key tiles of the block's
//     causal range are dealt round-robin over `S` blocks (key splits); a tile is staged into LDS
//     once per block (double buffered, one barrier per tile) by an eighth wavefront and read by
//     every computing wavefront. Both products are formed transposed (S^T = K . Q^T,
//     O^T = V^T . P^T): a lane's scores, probabilities and output columns all belong to one query
//     row, so the softmax needs no exchange through LDS and P goes from the score registers - cut
//     into terms - straight back into the matrix core. Per tile and wavefront (head size 128, f32
//     cache): 24 + 24 MFMAs of 32x32x16 and an online-softmax update on 16 scores per lane.
//     S == 1 writes the normalised rows; S > 1 leaves (max, sum, accumulator) per split and
//  3. attn_x3_merge_kernel combines them in split order.
#include "common.hpp"

namespace tlhip {

namespace x3 {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // a 16-byte unit in registers

constexpr int kTile = 32;                    // keys per tile
// 16-byte units of one K term of a tile (D/16 dim steps x 64 lanes) and of one V term (D/32 column
// tiles x 2 key steps x 64 lanes): 4 D either way. Head sizes 64 and 128 are built.
// The 32x32x16 MFMA leaves the scores of a 32-key tile with lane (g = l/32, c = l%32) holding, for
// query row c, the keys 8a + 4g + b (a, b = 0..3) in accumulator register 4a + b. Registers
// 8u .. 8u + 7 are the lane's 8 elements of key step u of P.V, so element j of lane half g in
// step u is key 8 (2u + j / 4) + 4 g + j % 4.
__host__ __device__ constexpr int wide_key(int u, int g, int j) { return 8 * (2 * u + (j >> 2)) + 4 * g + (j & 3); }

template <int D> struct Img { static constexpr int kKUnits = (D / 32) * 2 * 64, kVUnits = (D / 16) * 64; };

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// An operand, first multiplied by a power of two that brings it into the f16 range, is cut into
// TWO f16 terms, both rounded to nearest (2^-24 relative while the second term is a normal f16).
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
// what is left after the first term, 0 where that is inf - inf (an infinite operand): a NaN second
// term would turn the infinity an fp32 product gives there into NaN
__device__ __forceinline__ f32x2 rest_or_zero(f32x2 d) {
  d.x = d.x == d.x ? d.x : 0.f;
  d.y = d.y == d.y ? d.y : 0.f;
  return d;
}
__device__ __forceinline__ void split2x8_f16(const float (&x)[8], float s, uint4& p1, uint4& p2) {
  uint32_t a[4], b[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const f32x2 v = {x[2 * j] * s, x[2 * j + 1] * s};
    const f16x2 h = __builtin_convertvector(v, f16x2);
    const f16x2 l = __builtin_convertvector(rest_or_zero(v - __builtin_convertvector(h, f32x2)), f16x2);
    a[j] = __builtin_bit_cast(uint32_t, h);
    b[j] = __builtin_bit_cast(uint32_t, l);
  }
  p1 = make_uint4(a[0], a[1], a[2], a[3]);
  p2 = make_uint4(b[0], b[1], b[2], b[3]);
}
__device__ __forceinline__ void split2x8_f16(const float (&x)[8], uint4& p1, uint4& p2) {   // (already in range)
  uint32_t a[4], b[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const f32x2 v = {x[2 * j], x[2 * j + 1]};
    const f16x2 h = __builtin_convertvector(v, f16x2);
    const f16x2 l = __builtin_convertvector(v - __builtin_convertvector(h, f32x2), f16x2);
    a[j] = __builtin_bit_cast(uint32_t, h);
    b[j] = __builtin_bit_cast(uint32_t, l);
  }
  p1 = make_uint4(a[0], a[1], a[2], a[3]);
  p2 = make_uint4(b[0], b[1], b[2], b[3]);
}
// exponent that brings a largest magnitude (as f32 bits, sign cleared) into [2^14, 2^15); 0 for 0
__device__ __forceinline__ int f16_exponent(uint32_t maxbits) {
  return maxbits == 0 ? 0 : max(-100, min(100, 14 - ((int)(maxbits >> 23) - 127)));
}
__device__ __forceinline__ float pow2i(int e) { return __uint_as_float((uint32_t)(e + 127) << 23); }   // e in [-126, 127]
__device__ __forceinline__ u32x4 as_u32x4(const uint4& u) { return u32x4{u.x, u.y, u.z, u.w}; }

__device__ __forceinline__ float cache_elem(const float* p) { return *p; }
__device__ __forceinline__ float cache_elem(const uint16_t* p) { return bf16_bits_to_f32(*p); }

// ---- 1. terms ----------------------------------------------------------------------------
// grid = (tiles, Hkv), block = 256. NP terms per element: 2 for an f32 cache, 1 for a bf16 cache.
// planes: per (kv head, tile) a K image of NP * kKUnits uint4, then a V image of NP * kVUnits uint4.
// K and V of a tile are scaled by 2^ek and 2^ev, one exponent each per tile (from the tile's
// largest magnitude), left in texp[(kv head * tiles + tile) * 2 + {0, 1}]; the attention kernel
// folds them into its score scale and its running output scale.
// The operand images are those of the 32x32x16 MFMA:
//   K image [term][16-dim step s][lane][8]        = K[32t + l%32][16s + 8(l/32) + j]
//   V image [term][32-column tile][key step u][lane][8] = V[32t + wide_key(u, l/32, j)][32d + l%32]
template <typename KT, int NP, int D>
__global__ __launch_bounds__(256) void kv_planes_kernel(const KT* __restrict__ K, const KT* __restrict__ V,
                                                        uint4* __restrict__ planes, int* __restrict__ texp,
                                                        int64_t kv_stride, int kend, int ntiles) {
  constexpr int kD = D, kKUnits = Img<D>::kKUnits, kVUnits = Img<D>::kVUnits;
  constexpr int kPer = (kKUnits + kVUnits) / 256;       // units per thread: the first half of them K, the rest V
  static_assert(kKUnits % 256 == 0 && kVUnits % 256 == 0, "a thread's units are all K or all V per step");
  __shared__ uint32_t red[2][4];
  const int t = blockIdx.x, kvh = blockIdx.y;
  const KT* Kh = K + (size_t)kvh * kv_stride;
  const KT* Vh = V + (size_t)kvh * kv_stride;
  uint4* img = planes + ((size_t)kvh * ntiles + t) * (size_t)(NP * (kKUnits + kVUnits));
  float x[kPer][8];
  uint32_t mxk = 0, mxv = 0;
#pragma unroll
  for (int i = 0; i < kPer; i++) {
    const int u = threadIdx.x + 256 * i;
    if (u < kKUnits) {
      const int l = u & 63;
      const int key = t * kTile + (l & 31);
      const int dim = 16 * (u >> 6) + 8 * (l >> 5);
      const bool live = key < kend;
      const KT* src = Kh + (size_t)min(key, kend - 1) * kD + dim;
#pragma unroll
      for (int j = 0; j < 8; j++) x[i][j] = live ? cache_elem(src + j) : 0.f;
#pragma unroll
      for (int j = 0; j < 8; j++) mxk = max(mxk, __float_as_uint(x[i][j]) & 0x7fffffffu);
    } else {
      const int v = u - kKUnits, l = v & 63;
      const int dim = 32 * (v >> 7) + (l & 31);
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const int key = t * kTile + wide_key((v >> 6) & 1, l >> 5, j);
        x[i][j] = key < kend ? cache_elem(Vh + (size_t)key * kD + dim) : 0.f;
      }
#pragma unroll
      for (int j = 0; j < 8; j++) mxv = max(mxv, __float_as_uint(x[i][j]) & 0x7fffffffu);
    }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    mxk = max(mxk, (uint32_t)__shfl_xor((int)mxk, d));
    mxv = max(mxv, (uint32_t)__shfl_xor((int)mxv, d));
  }
  if ((threadIdx.x & 63) == 0) { red[0][threadIdx.x >> 6] = mxk; red[1][threadIdx.x >> 6] = mxv; }
  __syncthreads();
  mxk = max(max(red[0][0], red[0][1]), max(red[0][2], red[0][3]));
  mxv = max(max(red[1][0], red[1][1]), max(red[1][2], red[1][3]));
  const int ek = f16_exponent(mxk), ev = f16_exponent(mxv);
  if (threadIdx.x == 0) {
    texp[((size_t)kvh * ntiles + t) * 2] = ek;
    texp[((size_t)kvh * ntiles + t) * 2 + 1] = ev;
  }
  const float sk = pow2i(ek), sv = pow2i(ev);
#pragma unroll
  for (int i = 0; i < kPer; i++) {
    const int u = threadIdx.x + 256 * i;
    const bool isk = u < kKUnits;
    uint4* dst = isk ? img + u : img + NP * kKUnits + (u - kKUnits);
    const int plane_stride = isk ? kKUnits : kVUnits;
    uint4 p1, p2;
    split2x8_f16(x[i], isk ? sk : sv, p1, p2);
    dst[0] = p1;
    if (NP == 2) dst[plane_stride] = p2;
  }
}

struct Geometry {
  int group;        // query heads per kv head
  int nh, np;       // computing wavefronts of a block: nh heads x np runs of 32 positions (nh * np <= 7)
  int head_chunks;  // ceil(group / nh)
  int T, pos0, S, ntiles;
  int64_t rows;     // Hq * T
  int64_t o_head, o_row;   // output strides in floats: [Hq,T,D] or [T,Hq*D]
};

// ---- 2. attention ------------------------------------------------------------------------
// grid = (Hkv * head_chunks, position blocks, S), block = 512: seven computing wavefronts and
// one that moves tiles.
//
// A computing wavefront owns TWO 16-row tiles - 32 consecutive positions of one head - and uses
// every K/V operand it reads from LDS twice (with one tile per wavefront the operand reads took
// as long as the MFMAs they feed). Its registers then hold 96 for the query planes and 64 for
// the output accumulators, which leaves no room for tiles in transit: wavefront 7 does nothing
// but copy, K of the next tile and V of this one, global -> registers -> LDS, one 16-byte unit
// per lane and instruction.
//
// A step of the loop is one barrier interval. In interval i a computing wavefront runs one
// matrix phase - P.V of tile i-1, then Q.K^T of tile i - and one vector phase, the online
// softmax of one tile. Wavefronts 0-3 run the softmax of tile i AFTER their matrix phase,
// wavefronts 4-6 run the softmax of tile i-1 BEFORE it. The two wavefronts that share a SIMD
// (w and w + 4) are therefore never in the same kind of phase: one feeds the matrix core while
// the other is on the vector ALU. Interval i needs K of tile i and V of tile i-1 in LDS.
constexpr int kRT = 2;          // 16-row tiles per computing wavefront
constexpr int kF16Weight = 1;   // f16 form: term pairs (a, b) with a + b <= this; 1 leaves out lo x lo, <= 2^-24 |a b|
constexpr int kCompute = 7;     // computing wavefronts per block

// ---- 2. attention on 32x32x16 MFMAs (f16 terms) -------------------------------------------
// A computing wavefront's 32 query rows are ONE 32-column tile of both transposed products:
//   S^T[32 keys x 32 rows] = K[32 keys x D] . Q^T      D/16 steps, A = K image, B = the row's Q terms
//   O^T[D x 32 rows]      += V^T[D x 32 keys] . P^T    D/32 column tiles x 2 key steps
// Lane (g = l/32, c = l%32) holds, for query row c, 16 scores of a tile (keys 8a + 4g + b) and,
// per 32-column tile of the output, the 16 columns 8a + 4g + b; the row's other half is lane
// l ^ 32 - one register swap for the row maximum, one for the sum at the end. A wavefront
// issues half as many matrix instructions for the same products as with 16x16x32 tiles, and a
// matrix instruction of this shape takes a third of the issue cycles away from the vector-ALU
// wavefront that shares its SIMD.
template <int NP, int D>
__global__ __launch_bounds__(512, 1) void attn_w32_kernel(const float* __restrict__ q, const uint4* __restrict__ planes,
                                                           const int* __restrict__ texp,
                                                           float* __restrict__ out, float* __restrict__ part_o,
                                                           float* __restrict__ part_ml, float scale, const Geometry g) {
  typedef float f32x16 __attribute__((ext_vector_type(16)));
  constexpr int kD = D, kKUnits = Img<D>::kKUnits, kVUnits = Img<D>::kVUnits;
  constexpr int kKS = D / 16, kDT = D / 32;                   // steps of Q.K^T, 32-column tiles of P.V
  constexpr int kKImg = NP * kKUnits, kVImg = NP * kVUnits;
  constexpr int kImg = kKImg + kVImg;
  constexpr int kCopyK = kKImg / 64, kCopyV = kVImg / 64;
  constexpr int kRows = 16 * kRT;                             // query rows of a computing wavefront
  static_assert(kRows == 32, "one 32-column tile per wavefront");
  extern __shared__ u32x4 lds4[];
  u32x4* kbuf = lds4;
  u32x4* vbuf = lds4 + 2 * kKImg;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l31 = lane & 31, lh = lane >> 5;
  const int kvh = blockIdx.x / g.head_chunks, hc = blockIdx.x - kvh * g.head_chunks;
  const int nblk = gridDim.y;
  const int pblock = nblk - 1 - (int)blockIdx.y;
  const int split = blockIdx.z;
  const int blk_last = min((pblock + 1) * g.np * kRows, g.T) - 1;
  const int nkt_blk = (g.pos0 + blk_last) / kTile + 1;
  const int n = nkt_blk > split ? (nkt_blk - split + g.S - 1) / g.S : 0;
  const auto tile_of = [&](int i) { return split + i * g.S; };
  const u32x4* img0 = reinterpret_cast<const u32x4*>(planes) + (size_t)kvh * g.ntiles * kImg;
  const int* texp0 = texp + (size_t)kvh * g.ntiles * 2;

  if (wave == kCompute) {   // the copying wavefront
    u32x4 stk[kCopyK], stv[kCopyV];
    const auto request = [&](int ik, int iv) {
      const u32x4* srck = img0 + (size_t)min(tile_of(ik), g.ntiles - 1) * kImg;
      const u32x4* srcv = img0 + (size_t)min(tile_of(iv), g.ntiles - 1) * kImg + kKImg;
#pragma unroll
      for (int c = 0; c < kCopyK; c++) stk[c] = srck[lane + 64 * c];
#pragma unroll
      for (int c = 0; c < kCopyV; c++) stv[c] = srcv[lane + 64 * c];
    };
    request(0, 0);
#pragma unroll
    for (int c = 0; c < kCopyK; c++) kbuf[lane + 64 * c] = stk[c];
    request(1, 0);
    __syncthreads();
    for (int i = 0; i <= n; i++) {
#pragma unroll
      for (int c = 0; c < kCopyK; c++) kbuf[((i + 1) & 1) * kKImg + lane + 64 * c] = stk[c];
#pragma unroll
      for (int c = 0; c < kCopyV; c++) vbuf[(i & 1) * kVImg + lane + 64 * c] = stv[c];
      request(i + 2, i + 1);
      __syncthreads();
    }
    return;
  }

  const int hh = wave % g.nh, pt = wave / g.nh;
  const int hloc = hc * g.nh + hh;
  const int p_first = (pblock * g.np + pt) * kRows;
  const bool active = pt < g.np && hloc < g.group && p_first < g.T;
  const bool late = wave >= 4;
  const int h = kvh * g.group + min(hloc, g.group - 1);
  const int my_last_key = g.pos0 + min(p_first + kRows - 1, g.T - 1);
  const int kend = g.pos0 + g.T;

  // ---- query row l%32 as two f16 terms: dims 16s + 8(l/32) + j ----
  uint4 qa[2][kKS];
  int eq;
  {
    const float* qrow = q + ((size_t)h * g.T + min(p_first + l31, g.T - 1)) * kD;
    float x[kKS][8];
    uint32_t mx = 0;
#pragma unroll
    for (int ks = 0; ks < kKS; ks++) {
      const float4 a = *reinterpret_cast<const float4*>(qrow + 16 * ks + 8 * lh);
      const float4 b = *reinterpret_cast<const float4*>(qrow + 16 * ks + 8 * lh + 4);
      x[ks][0] = a.x; x[ks][1] = a.y; x[ks][2] = a.z; x[ks][3] = a.w;
      x[ks][4] = b.x; x[ks][5] = b.y; x[ks][6] = b.z; x[ks][7] = b.w;
      if (scale < 0.f) {   // the sign of the scale goes into Q
#pragma unroll
        for (int j = 0; j < 8; j++) x[ks][j] = -x[ks][j];
      }
#pragma unroll
      for (int j = 0; j < 8; j++) mx = max(mx, __float_as_uint(x[ks][j]) & 0x7fffffffu);
    }
    const LanePair e = swap32(__uint_as_float(mx), __uint_as_float(mx));   // the row's other 64 dims
    eq = f16_exponent(max(__float_as_uint(e.first), __float_as_uint(e.second)));
#pragma unroll
    for (int ks = 0; ks < kKS; ks++) split2x8_f16(x[ks], pow2i(eq), qa[0][ks], qa[1][ks]);
  }

  f32x16 o[kDT];                      // O^T: columns 32 dt + 8a + 4(l/32) + b of row l%32 in register 4a + b
  float mrow = -INFINITY, lrow = 0.f; // row l%32: running maximum (base-2 units); this lane's share of the running sum
  f32x16 s;                           // S^T of the tile whose softmax is pending
  uint4 pa[2][2];                     // P terms of the tile whose P.V is pending, per key step
  // P of a tile enters its MFMAs as p * 2^14 against V * 2^ev(tile), so the tile's products come
  // in units of 2^-(14 + ev(tile)). The output accumulators are kept in the unit of the tile last
  // added, 2^-(14 + unit): moving on to the next tile multiplies them by 2^(unit' - unit) in the
  // same multiplication as the softmax correction. unit = ev(tile), except that it stays within
  // kUnitSpan of the smallest ev seen (the largest V): a tile whose values are more than 2^64 below
  // an earlier tile's gets its P scaled down instead, which keeps the accumulators far from overflow.
  constexpr int kUnitSpan = 64;
  int evmin = 1 << 20, unit = 0;
  // (ek, ev) of the tile whose softmax comes next: asked for one tile ahead, so that the load's
  // latency passes behind a matrix phase
  int2 next_exp = *reinterpret_cast<const int2*>(texp0 + 2 * min(tile_of(0), g.ntiles - 1));
#pragma unroll
  for (int dt = 0; dt < kDT; dt++)
#pragma unroll
    for (int v = 0; v < 16; v++) o[dt][v] = 0.f;
#pragma unroll
  for (int v = 0; v < 16; v++) s[v] = 0.f;
  pa[0][0] = pa[0][1] = pa[1][0] = pa[1][1] = make_uint4(0, 0, 0, 0);

  const float ascale = fabsf(scale) * 1.44269504088896341f;
  const auto softmax_tile = [&](int i) {
    const int kt = tile_of(i);
    const bool masked = (kt + 1) * kTile - 1 > min(g.pos0 + p_first, kend - 1);   // (uniform for the wavefront)
    const int ek = next_exp.x, ev = next_exp.y;
    next_exp = *reinterpret_cast<const int2*>(texp0 + 2 * min(tile_of(i + 1), g.ntiles - 1));
    evmin = min(evmin, ev);
    const int nunit = min(ev, evmin + kUnitSpan);
    const int down = max(nunit - unit, -200);
    const int pexp = max(14 + nunit - ev, -120);
    unit = nunit;
    const float c2 = ldexpf(ascale, -(eq + ek));
    float v[16], mx;
    if (masked) {
      const int limit = min(g.pos0 + p_first + l31, kend - 1);   // last key the row sees
#pragma unroll
      for (int r = 0; r < 16; r++) v[r] = kt * kTile + 8 * (r >> 2) + 4 * lh + (r & 3) <= limit ? s[r] * c2 : -INFINITY;
    } else {
#pragma unroll
      for (int r = 0; r < 16; r++) v[r] = s[r];
    }
    mx = fmaxf(fmaxf(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])), fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7]))),
               fmaxf(fmaxf(fmaxf(v[8], v[9]), fmaxf(v[10], v[11])), fmaxf(fmaxf(v[12], v[13]), fmaxf(v[14], v[15]))));
    if (!masked) mx *= c2;   // c2 >= 0
    const LanePair e = swap32(mx, mx);
    mx = fmaxf(e.first, e.second);                 // over the row's 32 keys
    const float mnew = fmaxf(mrow, mx);
    const float mref = mnew == -INFINITY ? 0.f : mnew;
    const float lcorr = __builtin_amdgcn_exp2f(mrow - mref);
    const float off = (float)pexp - mref;
    float p[16];
    if (masked) {
#pragma unroll
      for (int r = 0; r < 16; r++) p[r] = __builtin_amdgcn_exp2f(v[r] + off);
    } else {
#pragma unroll
      for (int r = 0; r < 16; r++) p[r] = __builtin_amdgcn_exp2f(fmaf(v[r], c2, off));
    }
    const float psum = (((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]))) +
                       (((p[8] + p[9]) + (p[10] + p[11])) + ((p[12] + p[13]) + (p[14] + p[15])));
    lrow = fmaf(lrow, lcorr, ldexpf(psum, -pexp));
    mrow = mnew;
    const float corr = ldexpf(lcorr, down);
    if (__builtin_amdgcn_ballot_w64(corr != 1.0f) != 0) {
#pragma unroll
      for (int dt = 0; dt < kDT; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[dt][r] *= corr;
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const float pu[8] = {p[8 * u], p[8 * u + 1], p[8 * u + 2], p[8 * u + 3], p[8 * u + 4], p[8 * u + 5], p[8 * u + 6], p[8 * u + 7]};
      split2x8_f16(pu, pa[0][u], pa[1][u]);
    }
  };
  const auto mine = [&](int i) { return active && i >= 0 && i < n && tile_of(i) * kTile <= my_last_key; };
  const auto mma = [](const u32x4 a, const uint4& b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, as_u32x4(b)), c, 0, 0, 0);
  };

#ifdef TLHIP_TRACE
  unsigned long long ph[4] = {0, 0, 0, 0}, tc;
  TLHIP_MARK(0);
#define TLHIP_X3_T0() tc = __builtin_readcyclecounter()
#define TLHIP_X3_T(k) do { const unsigned long long n_ = __builtin_readcyclecounter(); ph[k] += n_ - tc; tc = n_; } while (0)
#else
#define TLHIP_X3_T0()
#define TLHIP_X3_T(k)
#endif
  __syncthreads();   // K of tile 0 is in LDS
  TLHIP_X3_T0();
  for (int i = 0; i <= n; i++) {
    if (late && mine(i - 1)) softmax_tile(i - 1);
    TLHIP_X3_T(0);
    // ---- matrix phase; term pairs (a, b) with a + b <= 1, smallest products first ----
    if (mine(i - 1)) {   // P.V of tile i-1: two column tiles at a time so that two accumulators take turns
      const u32x4* vimg = vbuf + ((i - 1) & 1) * kVImg;
#pragma unroll
      for (int dt = 0; dt < kDT; dt += 2) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
          u32x4 vb[2][NP];
#pragma unroll
          for (int d2 = 0; d2 < 2; d2++)
#pragma unroll
            for (int pl = 0; pl < NP; pl++) vb[d2][pl] = vimg[pl * kVUnits + ((dt + d2) * 2 + u) * 64 + lane];
#pragma unroll
          for (int w = kF16Weight; w >= 0; w--)
#pragma unroll
            for (int pb = NP - 1; pb >= 0; pb--) {
              const int pp = w - pb;
              if (pp >= 0 && pp < 2) {
#pragma unroll
                for (int d2 = 0; d2 < 2; d2++) o[dt + d2] = mma(vb[d2][pb], pa[pp][u], o[dt + d2]);
              }
            }
        }
      }
    }
    if (mine(i)) {       // S^T of tile i: even and odd dim steps into two accumulators
      const u32x4* kimg = kbuf + (i & 1) * kKImg;
      f32x16 s2;
#pragma unroll
      for (int v = 0; v < 16; v++) { s[v] = 0.f; s2[v] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < kKS; ks += 2) {
        u32x4 kb[2][NP];
#pragma unroll
        for (int k2 = 0; k2 < 2; k2++)
#pragma unroll
          for (int pl = 0; pl < NP; pl++) kb[k2][pl] = kimg[pl * kKUnits + (ks + k2) * 64 + lane];
#pragma unroll
        for (int w = kF16Weight; w >= 0; w--)
#pragma unroll
          for (int pb = NP - 1; pb >= 0; pb--) {
            const int pp = w - pb;
            if (pp >= 0 && pp < 2) {
              s = mma(kb[0][pb], qa[pp][ks], s);
              s2 = mma(kb[1][pb], qa[pp][ks + 1], s2);
            }
          }
      }
#pragma unroll
      for (int v = 0; v < 16; v++) s[v] += s2[v];
    }
    TLHIP_X3_T(1);
    if (!late && mine(i)) softmax_tile(i);
    TLHIP_X3_T(0);
    __syncthreads();
    TLHIP_X3_T(2);
  }
#ifdef TLHIP_TRACE
  {
    const unsigned b = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    if (lane == 0 && b < kTraceBlocks) {
      unsigned long long* gt = &g_trace[(b * kTraceWaves + wave) * kTraceSlots];
      gt[1] = ph[0]; gt[2] = ph[1]; gt[3] = ph[2]; gt[4] = n + 1;
    }
  }
  TLHIP_MARK(6);
#endif
#undef TLHIP_X3_T0
#undef TLHIP_X3_T

  if (!active) return;
  const int p = p_first + l31;
  const LanePair e = swap32(lrow, lrow);
  const float lsum = e.first + e.second;
  if (p >= g.T) return;
  const int back = -(14 + unit);   // the accumulators are in units of 2^-(14 + unit)
  if (g.S == 1) {
    const float inv = ldexpf(1.0f / lsum, back);
    float* op = out + (size_t)h * g.o_head + (size_t)p * g.o_row + 4 * lh;
#pragma unroll
    for (int dt = 0; dt < kDT; dt++)
#pragma unroll
      for (int a = 0; a < 4; a++)
        *reinterpret_cast<float4*>(op + 32 * dt + 8 * a) =
            make_float4(o[dt][4 * a] * inv, o[dt][4 * a + 1] * inv, o[dt][4 * a + 2] * inv, o[dt][4 * a + 3] * inv);
  } else {
    const size_t row = (size_t)h * g.T + p, rows = (size_t)g.rows;
    float* po = part_o + ((size_t)split * rows + row) * kD + 4 * lh;
#pragma unroll
    for (int dt = 0; dt < kDT; dt++)
#pragma unroll
      for (int a = 0; a < 4; a++)
        *reinterpret_cast<float4*>(po + 32 * dt + 8 * a) =
            make_float4(ldexpf(o[dt][4 * a], back), ldexpf(o[dt][4 * a + 1], back), ldexpf(o[dt][4 * a + 2], back),
                        ldexpf(o[dt][4 * a + 3], back));
    if (lh == 0) {
      part_ml[((size_t)split * rows + row) * 2] = mrow;
      part_ml[((size_t)split * rows + row) * 2 + 1] = lsum;
    }
  }
}


// ---- 3. merge of the key splits ---------------------------------------------------------------
// One thread per (row, 4 columns); splits are combined in split order.
template <int D>
__global__ __launch_bounds__(256) void attn_x3_merge_kernel(const float* __restrict__ part_o,
                                                            const float* __restrict__ part_ml,
                                                            float* __restrict__ out, int rows, int T, int S,
                                                            int64_t o_head, int64_t o_row) {
  constexpr int kD = D;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = i / (kD / 4);
  const int c4 = (int)(i - row * (kD / 4)) * 4;
  if (row >= rows) return;
  float M = -INFINITY;
  for (int s = 0; s < S; s++) M = fmaxf(M, part_ml[((size_t)s * rows + row) * 2]);
  float L = 0.f;
  float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int s = 0; s < S; s++) {
    const float m = part_ml[((size_t)s * rows + row) * 2];
    const float f = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - M);   // maxima are in base-2 units
    L = fmaf(part_ml[((size_t)s * rows + row) * 2 + 1], f, L);
    const float4 v = *reinterpret_cast<const float4*>(part_o + ((size_t)s * rows + row) * kD + c4);
    a.x = fmaf(v.x, f, a.x); a.y = fmaf(v.y, f, a.y); a.z = fmaf(v.z, f, a.z); a.w = fmaf(v.w, f, a.w);
  }
  const float inv = 1.0f / L;
  const int64_t h = row / T, p = row - h * T;
  *reinterpret_cast<float4*>(out + h * o_head + p * o_row + c4) = make_float4(a.x * inv, a.y * inv, a.z * inv, a.w * inv);
}

}  // namespace x3

// Whether the matrix-core kernels serve this call: head size 64 or 128 and enough keys for the
// extra passes (planes, merge) to pay. Measured crossover of the f16 form against the fp32
// matrix-pipe kernel at the 7B and 0.5B head shapes, chunks of 32 to 512 tokens: from 640 keys on
// at head size 128 (512 for a chunk of 512), from 1024 at head size 64 (768 for chunks of 256 up).
bool prefill_x3_applies(int D, int T, int pos0) {
  if (T < 16) return false;
  const int64_t keys = (int64_t)pos0 + T;
  if (D == 128) return keys >= 640 || (keys >= 512 && T >= 512);
  if (D == 64) return keys >= 1024 || (keys >= 768 && T >= 256);
  return false;
}

// Launches the three kernels. Returns 0 when launched, a negative status on failure, 1 when the
// scratch for the planes could not be had (the caller then uses the fp32 matrix-pipe kernel).
template <int D, typename KT>
static int launch_x3(const float* q, const KT* K, const KT* V, float* out, int Hq, int Hkv, int T,
                     int64_t kv_max, float scale, int pos0, int token_major) {
  using namespace x3;
  constexpr int NP = sizeof(KT) == 4 ? 2 : 1;
  constexpr int kD = D, kKUnits = Img<D>::kKUnits, kVUnits = Img<D>::kVUnits;
  Context& c = ctx();
  Geometry g{};
  g.group = Hq / Hkv;
  g.nh = g.group < kCompute ? g.group : kCompute;
  g.np = kCompute / g.nh;
  if (g.np * 16 * kRT > T) g.np = (T + 16 * kRT - 1) / (16 * kRT);
  g.head_chunks = (g.group + g.nh - 1) / g.nh;
  g.T = T;
  g.pos0 = pos0;
  const int kend = pos0 + T;
  g.ntiles = (kend + kTile - 1) / kTile;
  g.o_head = token_major ? kD : (int64_t)T * kD;
  g.o_row = token_major ? (int64_t)Hq * kD : kD;
  g.rows = (int64_t)Hq * T;
  const int pblocks = (T + g.np * 16 * kRT - 1) / (g.np * 16 * kRT);
  const int base = Hkv * g.head_chunks * pblocks;
  // key splits: fill the chip once, keep at least 4 tiles per block
  int S = (c.cus + base - 1) / base;
  if (S > g.ntiles / 4) S = g.ntiles / 4;
  if (S < 1) S = 1;
  if (S > 64) S = 64;
  g.S = S;
  constexpr size_t kImgBytes = (size_t)NP * (kKUnits + kVUnits) * 16;
  const size_t plane_bytes = (size_t)Hkv * g.ntiles * kImgBytes;
  const size_t rows = (size_t)Hq * T;
  const size_t part_o_bytes = S > 1 ? (size_t)S * rows * kD * 4 : 0;
  const size_t part_ml_bytes = S > 1 ? (size_t)S * rows * 2 * 4 : 0;
  const size_t texp_bytes = ((size_t)Hkv * g.ntiles * 2 * sizeof(int) + 255) & ~(size_t)255;
  char* buf = static_cast<char*>(scratch(plane_bytes + part_o_bytes + part_ml_bytes + texp_bytes + 256));
  if (!buf) return 1;   // no room for the planes: the caller takes the kernel that needs none
  uint4* planes = reinterpret_cast<uint4*>(buf);
  float* part_o = reinterpret_cast<float*>(buf + plane_bytes);
  float* part_ml = reinterpret_cast<float*>(buf + plane_bytes + part_o_bytes);
  int* texp = reinterpret_cast<int*>(buf + plane_bytes + part_o_bytes + part_ml_bytes);
  const size_t lds = 2 * kImgBytes;
  if (lds > (size_t)c.lds_per_cu) return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_prefill: not enough LDS");
  const void* fn = reinterpret_cast<const void*>(attn_w32_kernel<NP, D>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(LDS)");
  hipLaunchKernelGGL((kv_planes_kernel<KT, NP, D>), dim3(g.ntiles, Hkv), dim3(256), 0, c.stream, K, V, planes, texp,
                     kv_max * (int64_t)kD, kend, g.ntiles);
  const dim3 grid(Hkv * g.head_chunks, pblocks, S);
  hipLaunchKernelGGL((attn_w32_kernel<NP, D>), grid, dim3(512), lds, c.stream, q, planes, texp, out, part_o, part_ml, scale, g);
  if (S > 1) {
    const int64_t threads = (int64_t)rows * (kD / 4);
    hipLaunchKernelGGL(attn_x3_merge_kernel<D>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, c.stream, part_o,
                       part_ml, out, (int)rows, T, S, g.o_head, g.o_row);
  }
  return 0;
}

template <int D, typename KT>
int launch_prefill_x3(const float* q, const KT* K, const KT* V, float* out, int Hq, int Hkv, int T,
                      int64_t kv_max, float scale, int pos0, int token_major) {
  return launch_x3<D, KT>(q, K, V, out, Hq, Hkv, T, kv_max, scale, pos0, token_major);
}

template int launch_prefill_x3<128, float>(const float*, const float*, const float*, float*, int, int, int, int64_t, float, int, int);
template int launch_prefill_x3<128, uint16_t>(const float*, const uint16_t*, const uint16_t*, float*, int, int, int, int64_t, float, int, int);
template int launch_prefill_x3<64, float>(const float*, const float*, const float*, float*, int, int, int, int64_t, float, int, int);
template int launch_prefill_x3<64, uint16_t>(const float*, const uint16_t*, const uint16_t*, float*, int, int, int, int64_t, float, int, int);

}  // namespace tlhip
