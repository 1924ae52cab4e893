// Prefill GEMM: C[M,N] = A[M,K] (f32) . W[N,K]^T (bf16), fp32 accumulate, on MFMA.
//
// This is the one dense contraction of the path, so it is the one MFMA kernel.
// The reference multiplies f32 activations by widened bf16 weights in fp32
// (tensorlib_cuda.cu:509-519); rounding A to bf16 would miss rtol 1e-4. Instead
// every f32 activation is split EXACTLY into three bf16 terms
//     a = a_hi + a_mid + a_lo        (8 + 8 + 8 mantissa bits, by truncation)
// and the product is formed as three v_mfma_f32_32x32x16_bf16 per weight
// fragment. bf16 x bf16 products are exact in fp32 and the MFMA accumulates in
// fp32, so the result carries ordinary fp32 summation error only, at a third of
// the bf16 matrix rate (still ~5x the fp32 MFMA rate).
//
// Tiling: a block of 4 wavefronts (2x2) owns a (64*TM) x (64*TN) tile of C; each
// wavefront TM x TN MFMA tiles of 32x32 (2 x 4 for prompt chunks: an A fragment costs three
// LDS reads, one per plane, so tiles are wide in N, where a fragment costs one).
// K advances in slabs of 32 through LDS:
// the A slab is split into its three bf16 planes while it is written to LDS, the
// W slab is copied as is (rows XOR-swizzled against bank conflicts). Both operands are K-contiguous per lane (A is [M,K],
// W is [N,K]), which is exactly the MFMA operand layout: one ds_read_b128 per
// fragment. Global loads of the next slab are in flight while the current one is
// multiplied.
#include "gemm_shared.hpp"

namespace tlhip {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kBK = 32;        // K slab: an LDS row is 32 bf16 = four 16-byte chunks

// LDS rows are not padded; instead the 16-byte chunk index is XORed with bits of
// the row number. Both the fragment reads (8 consecutive rows, same chunk) and the
// tile stores (consecutive chunks of one row, then the next row) then spread over
// all 32 banks.
__device__ __forceinline__ int lds_off(int row, int chunk) {   // in bf16 elements
  return row * kBK + ((chunk ^ ((row >> 1) & 3)) << 3);
}

// gridDim.y > 1 is split-K: block row y takes K range [y*kchunk, (y+1)*kchunk) and
// writes its partial product to C + y*M*N (a scratch area); splitk_sum_kernel adds
// the parts in a fixed order. ldc = row stride of C (N for a scratch part; the full
// width when the launch covers a column range of a wider result).
//
// GU = true: W is a fused [gate rows | up rows] matrix ([2*ff, K], qwen_model.h:194-199) and the
// result is the gated activation act[m][f] = swiglu(A.gate_f, A.up_f), never the two products.
// Each wavefront's 32*TN tile columns are then 16*TN gate features followed by the SAME features'
// up rows (`ff` rows further down in W), so a lane holds both accumulators of a feature
// (MFMA tile j and j + TN/2) and the epilogue gates in registers. N counts features, n0 still
// counts tile columns (two per feature). Under split-K the raw parts are stored in that tile
// column order ([M][tiles * BN]) and splitk_sum_swiglu_kernel gates after the sum.
//
// Q4 = true: W is the int4 weight of the decode path - packed nibbles [rows][K/2] (even k in the
// low nibble, value = nibble - 8) with f32 scales [rows][K/32] (types.h:25-31). A slab of 32 k is
// exactly one scale group: the nibbles go to LDS as the bf16 integers they stand for (exact), the
// slab's MFMAs run into a second set of accumulators that starts at zero, and
// acc += group sum * scale closes the slab - sum over groups of scale * (a . q), the decode GEMV's
// arithmetic on the matrix pipe. The second set holds one row block of MFMA tiles at a time; with
// it, 64-column wavefront tiles (TN = 2) fit the registers, 128-column ones spill (and then run
// at half the speed).
//
// H = true (int4 weights): the operands go to the matrix cores as f16 instead. Row m of A is first
// multiplied by 2^ea[m], which brings its largest magnitude into [2^14, 2^15), and then cut into
// TWO f16 terms, both rounded to nearest: a * 2^ea = hi + lo + r with |r| <= 2^-24 |a * 2^ea|
// wherever lo is a normal f16 (and <= 2^-25 absolute, 2^-39 of the row's largest, where it is not)
// - the accuracy of one fp32 rounding, from two MFMAs per product instead of three. The nibbles
// are small integers, exact in f16; the result leaves as acc * 2^-ea[m], an exact scaling.
template <int TM, int TN, int WM = 2, int WN = 2, bool GU = false, bool Q4 = false, bool H = false>
__global__ __launch_bounds__(64 * WM * WN, 2) void gemm_bf16_nt_kernel(const float* __restrict__ A,
                                                           const uint16_t* __restrict__ W,
                                                           float* __restrict__ C, int M, int N,
                                                           int K, int kchunk, int ldc, int ff,
                                                           const float* __restrict__ scales,
                                                           const int* __restrict__ ea) {
  static_assert(!H || Q4, "f16 planes here are for int4 weights; prepared bf16 weights have their own kernel");
  constexpr int PL = H ? 2 : 3;                 // planes of A
  static_assert(!GU || TN % 2 == 0, "gate and up accumulators of a feature must share a lane");
  static_assert(!Q4 || ((32 * TN * WN == 128 || 32 * TN * WN == 256) && 64 * WM * WN == 256),
                "int4 slab copy: one or two threads per tile column");
  constexpr int TPC = Q4 ? 256 / (32 * TN * WN) : 1;   // Q4: threads per tile column of the slab copy
  constexpr int WT = 32 * TN, HW = WT / 2;      // a wavefront's tile columns; GU: gate half, up half
  constexpr int NT = 64 * WM * WN;              // threads: WM x WN wavefronts
  constexpr int BM = 32 * TM * WM, BN = 32 * TN * WN;
  constexpr int A_LOADS = BM * kBK / 4 / NT;    // float4 per thread per slab
  constexpr int B_LOADS = BN * kBK / 8 / NT;    // uint4 (8 bf16) per thread per slab
  static_assert(A_LOADS >= 1 && B_LOADS >= 1 && BM * kBK / 4 % NT == 0 && BN * kBK / 8 % NT == 0, "tile vs threads");
  __shared__ __attribute__((aligned(16))) uint16_t As[PL][BM * kBK];
  __shared__ __attribute__((aligned(16))) uint16_t Bs[BN * kBK];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  // Block order. Hardware deals consecutive block ids round-robin to the 8 XCDs,
  // each with a private L2. Give every XCD one contiguous run of tiles, M fastest,
  // so the blocks that share a weight tile run together on one L2 and W is
  // streamed from HBM once.
  const int mt = (M + BM - 1) / BM;
  const int nb = gridDim.x, xcd = blockIdx.x & 7, within = blockIdx.x >> 3;
  const int q8 = nb >> 3, r8 = nb & 7;
  const int lid = xcd * q8 + min(xcd, r8) + within;
  const int m0 = (lid % mt) * BM, n0 = (lid / mt) * BN;
  const int kbeg = blockIdx.y * kchunk, kend = min(K, kbeg + kchunk);
  C += (size_t)blockIdx.y * M * ldc;   // split parts are dense [M][N] (ldc == N there)

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  float4 ra[A_LOADS];
  uint4 rb[Q4 ? 1 : B_LOADS];
  uint32_t rq[4 / TPC] = {};          // Q4: 32 / TPC nibbles of one tile column
  float sc[TN], sc_next[TN];          // Q4: this lane's scale per MFMA tile column, this slab / next
  // W row of tile column `col` of this block (-1: past the edge)
  auto wrow = [&](int col) {
    if (GU) {
      const int j = col % WT, f = (n0 >> 1) + (col / WT) * HW + j % HW;
      return f < N ? f + (j >= HW ? ff : 0) : -1;
    }
    return n0 + col < N ? n0 + col : -1;
  };
  // H: 2^exponent of the rows of A this thread copies (the same rows in every slab)
  float sa[H ? A_LOADS : 1];
  if (H) {
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
      const int gm = m0 + ((tid + i * NT) >> 3);
      sa[i] = gm < M ? pow2f(ea[gm]) : 1.0f;
    }
  }
  // Q4: where this thread's loads of a slab start at k = 0 (the same rows in every slab). Every
  // address is clamped into the operands and what lies past an edge is replaced when the slab is
  // stored to LDS, so that no load sits under a condition and nothing waits for a load where it
  // is issued: the requests of a slab go out back to back, in front of the products.
  const float* a_src[Q4 ? A_LOADS : 1];
  const uint8_t* q_src = nullptr;
  const float* s_src[Q4 ? TN : 1];
  bool a_in[Q4 ? A_LOADS : 1], s_in[Q4 ? TN : 1], q_in = false;
  if constexpr (Q4) {
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
      const int idx = tid + i * NT, row = idx >> 3, c4 = idx & 7;
      a_in[i] = m0 + row < M;
      a_src[i] = A + (size_t)min(m0 + row, M - 1) * K + c4 * 4;
    }
    const int gn = wrow(tid / TPC);
    q_in = gn >= 0;
    q_src = reinterpret_cast<const uint8_t*>(W) + ((size_t)max(gn, 0) * K + (tid % TPC) * (32 / TPC)) / 2;
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int gn2 = wrow(wn * WT + j * 32 + (lane & 31));
      s_in[j] = gn2 >= 0;
      s_src[j] = scales + (size_t)max(gn2, 0) * (K >> 5);
    }
  }
  auto gload = [&](int k0) {
    if constexpr (Q4) {   // (k0 < kend: the loop asks for slabs that exist)
#pragma unroll
      for (int i = 0; i < A_LOADS; i++) ra[i] = *reinterpret_cast<const float4*>(a_src[i] + k0);
      // thread t: tile column t / TPC, nibbles of k0 + (32 / TPC) * (t % TPC) .. (16 / TPC bytes)
      const uint32_t* src = reinterpret_cast<const uint32_t*>(q_src + (k0 >> 1));
#pragma unroll
      for (int u = 0; u < 4 / TPC; u++) rq[u] = src[u];
#pragma unroll
      for (int j = 0; j < TN; j++) sc_next[j] = s_src[j][k0 >> 5];
      return;
    }
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
      const int idx = tid + i * NT, row = idx >> 3, c4 = idx & 7;
      const int gm = m0 + row, gk = k0 + c4 * 4;
      ra[i] = (gm < M && gk < kend) ? *reinterpret_cast<const float4*>(A + (size_t)gm * K + gk)
                                 : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; i++) {
      const int idx = tid + i * NT, row = idx >> 2, c8 = idx & 3;
      const int gk = k0 + c8 * 8, gn = wrow(row);
      rb[i] = (gn >= 0 && gk < kend) ? *reinterpret_cast<const uint4*>(W + (size_t)gn * K + gk)
                                     : make_uint4(0u, 0u, 0u, 0u);
    }
  };
  // 4 bytes = 8 nibbles -> 8 bf16 (k ascending): float(nibble) - 8 is an integer in [-8, 7], exact in bf16
  auto nib8 = [](uint32_t w) {
    const uint32_t lo = w & 0x0f0f0f0fu, hi = (w >> 4) & 0x0f0f0f0fu;   // even k, odd k
    uint4 o;
    uint32_t* po = reinterpret_cast<uint32_t*>(&o);
#pragma unroll
    for (int b = 0; b < 4; b++) {
      const float e = (float)((lo >> (8 * b)) & 0xffu) - 8.0f, d = (float)((hi >> (8 * b)) & 0xffu) - 8.0f;
      po[b] = (__float_as_uint(e) >> 16) | (__float_as_uint(d) & 0xffff0000u);
    }
    return o;
  };
  // the same as f16: 0x6400 | n is the f16 number 1024 + n (one unit in the last place there), so
  // a nibble becomes its weight n - 8 by a byte permute, an OR and one packed f16 subtraction
  auto nib8h = [](uint32_t w) {
    const uint32_t lo = w & 0x0f0f0f0fu, hi = (w >> 4) & 0x0f0f0f0fu;   // even k, odd k
    uint4 o;
    uint32_t* po = reinterpret_cast<uint32_t*>(&o);
    const f16x2 bias = {(_Float16)1032.0f, (_Float16)1032.0f};
#pragma unroll
    for (int b = 0; b < 4; b++) {
      // bytes of the pair: [lo.byte b, 0, hi.byte b, 0]
      const uint32_t pair = __builtin_amdgcn_perm(hi, lo, (uint32_t)b | 0x0c00u | ((uint32_t)(4 + b) << 16) | 0x0c000000u);
      po[b] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, pair | 0x64006400u) - bias);
    }
    return o;
  };
  auto split3 = [](float a, uint32_t& hi, uint32_t& mid, uint32_t& lo) {
    const uint32_t h = __float_as_uint(a) & 0xffff0000u;
    const float r1 = a - __uint_as_float(h);            // exact
    const uint32_t m = __float_as_uint(r1) & 0xffff0000u;
    const float r2 = r1 - __uint_as_float(m);           // exact, <= 8 significant bits
    hi = h >> 16;
    mid = m >> 16;
    lo = __float_as_uint(r2) >> 16;
  };
  auto lstore = [&]() {
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
      const int idx = tid + i * NT, row = idx >> 3, c4 = idx & 7;
      if (Q4 && !a_in[Q4 ? i : 0]) ra[i] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (H) {
        uint32_t h01, l01, h23, l23;
        const float s = sa[H ? i : 0];
        split2_f16<false>(ra[i].x * s, ra[i].y * s, h01, l01);   // every block cuts its rows again, slab by slab:
        split2_f16<false>(ra[i].z * s, ra[i].w * s, h23, l23);   // the loop is bound by these instructions
        const int o = lds_off(row, c4 >> 1) + (c4 & 1) * 4;
        *reinterpret_cast<uint2*>(&As[0][o]) = make_uint2(h01, h23);
        *reinterpret_cast<uint2*>(&As[1][o]) = make_uint2(l01, l23);
        continue;
      }
      uint32_t h[4], m[4], l[4];
      split3(ra[i].x, h[0], m[0], l[0]);
      split3(ra[i].y, h[1], m[1], l[1]);
      split3(ra[i].z, h[2], m[2], l[2]);
      split3(ra[i].w, h[3], m[3], l[3]);
      const int o = lds_off(row, c4 >> 1) + (c4 & 1) * 4;
      *reinterpret_cast<uint2*>(&As[0][o]) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
      *reinterpret_cast<uint2*>(&As[1][o]) = make_uint2(m[0] | (m[1] << 16), m[2] | (m[3] << 16));
      *reinterpret_cast<uint2*>(&As[PL - 1][o]) = make_uint2(l[0] | (l[1] << 16), l[2] | (l[3] << 16));
    }
    if (Q4) {
      const int row = tid / TPC, c8 = (tid % TPC) * (4 / TPC);
#pragma unroll
      for (int u = 0; u < 4 / TPC; u++) {
        const uint32_t w = q_in ? rq[u] : 0x88888888u;   // nibble 8 = weight 0
        *reinterpret_cast<uint4*>(&Bs[lds_off(row, c8 + u)]) = H ? nib8h(w) : nib8(w);
      }
#pragma unroll
      for (int j = 0; j < TN; j++) sc[j] = s_in[Q4 ? j : 0] ? sc_next[j] : 0.f;
    } else {
#pragma unroll
    for (int i = 0; i < B_LOADS; i++) {
      const int idx = tid + i * NT, row = idx >> 2, c8 = idx & 3;
      *reinterpret_cast<uint4*>(&Bs[lds_off(row, c8)]) = rb[i];
    }
    }
  };

  // one 32x32x16 product step on two 16-byte fragments
  auto mma = [](frag16 a, frag16 b, f32x16 c) {
    if (H)
      return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  };
  gload(kbeg);
#ifdef TLHIP_TRACE
  unsigned long long ph[6] = {0, 0, 0, 0, 0, 0}, tc = __builtin_readcyclecounter();
  TLHIP_MARK(0);
#define TLHIP_PHASE(i) do { const unsigned long long n_ = __builtin_readcyclecounter(); ph[i] += n_ - tc; tc = n_; } while (0)
#else
#define TLHIP_PHASE(i)
#endif
  for (int k0 = kbeg; k0 < kend; k0 += kBK) {
    TLHIP_PHASE(4);           // products of the slab before
    __syncthreads();          // the previous slab has been consumed
    TLHIP_PHASE(0);
#ifdef TLHIP_TRACE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    TLHIP_PHASE(1);
#endif
    lstore();
    TLHIP_PHASE(2);
    __syncthreads();
    TLHIP_PHASE(3);
    if (k0 + kBK < kend) gload(k0 + kBK);
    if (Q4) {
      // one row block of MFMA tiles at a time: its sums over this slab (= this scale group) in a
      // second accumulator set that starts at zero, then acc += sums * scale
#pragma unroll
      for (int i = 0; i < TM; i++) {
        f32x16 grp[TN];
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int v = 0; v < 16; v++) grp[j][v] = 0.f;
        const int row = wm * 32 * TM + i * 32 + (lane & 31);
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ks++) {
          const int kc = ks * 2 + (lane >> 5);
          frag16 bfrag[TN];
#pragma unroll
          for (int j = 0; j < TN; j++)
            bfrag[j] = *reinterpret_cast<const frag16*>(&Bs[lds_off(wn * 32 * TN + j * 32 + (lane & 31), kc)]);
#pragma unroll
          for (int p = 0; p < PL; p++) {
            const frag16 afrag = *reinterpret_cast<const frag16*>(&As[p][lds_off(row, kc)]);
#pragma unroll
            for (int j = 0; j < TN; j++)
              grp[j] = mma(afrag, bfrag[j], grp[j]);
          }
        }
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int v = 0; v < 16; v++) acc[i][j][v] = fmaf(grp[j][v], sc[j], acc[i][j][v]);
      }
      continue;
    }
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ks++) {
      const int kc = ks * 2 + (lane >> 5);   // 16-byte chunk of the slab this lane multiplies
      frag16 bfrag[TN];
#pragma unroll
      for (int j = 0; j < TN; j++)
        bfrag[j] = *reinterpret_cast<const frag16*>(&Bs[lds_off(wn * 32 * TN + j * 32 + (lane & 31), kc)]);
#pragma unroll
      for (int i = 0; i < TM; i++) {
        const int row = wm * 32 * TM + i * 32 + (lane & 31);
#pragma unroll
        for (int p = 0; p < PL; p++) {
          const frag16 afrag = *reinterpret_cast<const frag16*>(&As[p][lds_off(row, kc)]);
#pragma unroll
          for (int j = 0; j < TN; j++)
            acc[i][j] = mma(afrag, bfrag[j], acc[i][j]);
        }
      }
    }
  }

#ifdef TLHIP_TRACE
  {
    TLHIP_PHASE(4);
    const unsigned b = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    if (lane == 0 && b < kTraceBlocks) {
      unsigned long long* g = &g_trace[(b * kTraceWaves + wave) * kTraceSlots];
      g[1] = ph[0]; g[2] = ph[1]; g[3] = ph[2]; g[4] = ph[3]; g[5] = ph[4]; g[7] = (kend - kbeg + kBK - 1) / kBK;
    }
  }
  TLHIP_MARK(6);
#endif
#undef TLHIP_PHASE
  // acc[v] of lane l: row 8*(v/4) + 4*(l/32) + v%4, column l%32 of the 32x32 tile.
  // H: the exponent of the row comes back out; ldexpf is exact.
  auto out = [&](float x, int e) { return H ? ldexpf(x, -e) : x; };
  if (GU && gridDim.y == 1) {
    // act = (g * sigmoid(g)) * u, the arithmetic of swiglu_kernel (array.h:2435-2439)
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int gm = m0 + wm * 32 * TM + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (gm >= M) continue;
        const int em = H ? ea[gm] : 0;
#pragma unroll
        for (int j = 0; j < TN / 2; j++) {
          const int f = (n0 >> 1) + wn * HW + j * 32 + (lane & 31);
          if (f >= N) continue;
          const float g = out(acc[i][j][v], em), sg = 1.0f / (1.0f + expf(-g));
          C[(size_t)gm * ldc + f] = (g * sg) * out(acc[i][j + TN / 2][v], em);
        }
      }
    return;
  }
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int gm = m0 + wm * 32 * TM + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
      if (gm >= M) continue;
      const int em = H ? ea[gm] : 0;
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const int gn = n0 + wn * 32 * TN + j * 32 + (lane & 31);
        if (!GU && gn >= N) continue;   // GU parts are whole tiles wide
        C[(size_t)gm * ldc + gn] = out(acc[i][j][v], em);
      }
    }
}

// ea[m] for the rows of an f32 matrix [M][K] (K % 4 == 0, rows 16-byte aligned). One block per row.
__global__ __launch_bounds__(256) void row_exponent_f32_kernel(const float* __restrict__ A, int K,
                                                               int* __restrict__ ea) {
  __shared__ uint32_t part[4];
  const uint4* row = reinterpret_cast<const uint4*>(A + (size_t)blockIdx.x * K);
  uint32_t mx = 0;
  for (int i = threadIdx.x; i < K / 4; i += 256) {
    const uint4 v = row[i];
    mx = max(max(mx, v.x & 0x7fffffffu), max(max(v.y & 0x7fffffffu, v.z & 0x7fffffffu), v.w & 0x7fffffffu));
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, d));
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x == 0) {
    mx = max(max(part[0], part[1]), max(part[2], part[3]));
    ea[blockIdx.x] = row_exponent((int)(mx >> 23), mx == 0);
  }
}

// ew[n] for the rows of a bf16 matrix [N][K] (K % 8 == 0, rows 16-byte aligned). One block per row.
__global__ __launch_bounds__(256) void row_exponent_bf16_kernel(const uint16_t* __restrict__ W, int K,
                                                                int8_t* __restrict__ ew) {
  __shared__ uint32_t part[4];
  const uint4* row = reinterpret_cast<const uint4*>(W + (size_t)blockIdx.x * K);
  uint32_t mx = 0;   // two 15-bit magnitudes, compared half by half
  auto both = [](uint32_t a, uint32_t b) {
    return max(a & 0x7fff0000u, b & 0x7fff0000u) | max(a & 0x7fffu, b & 0x7fffu);
  };
  for (int i = threadIdx.x; i < K / 8; i += 256) {
    const uint4 v = row[i];
    mx = both(both(mx, v.x), both(both(v.y, v.z), v.w));
  }
  mx = max(mx >> 16, mx & 0x7fffu);
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, d));
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x == 0) {
    mx = max(max(part[0], part[1]), max(part[2], part[3]));
    ew[blockIdx.x] = (int8_t)row_exponent((int)(mx >> 7), mx == 0);
  }
}

// C[m][n] = sum_s part[s][m][n], s in ascending order. Parts are dense [M][n4 * 4]; C rows
// are ldc4 float4s apart (the result may be a column range of a wider matrix).
__global__ __launch_bounds__(256) void splitk_sum_kernel(const float4* __restrict__ part,
                                                         float4* __restrict__ C, int M, int n4,
                                                         int ldc4, int S) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, total = (size_t)M * n4;
  if (i >= total) return;
  float4 a = part[i];
  for (int sidx = 1; sidx < S; sidx++) {
    const float4 b = part[sidx * total + i];
    a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
  }
  const size_t m = i / n4;
  C[m * ldc4 + (i - m * n4)] = a;
}

// The same for the parts of a GU launch: out[m][f] = swiglu(sum_s gate part, sum_s up part). Parts are
// [M][nv] in tile column order: per wavefront strip of 2 * HW columns, HW gate features then their
// up values. pf4 = features / 4 of this piece, ldc4 = row stride of out in float4s.
__global__ __launch_bounds__(256) void splitk_sum_swiglu_kernel(const float4* __restrict__ part,
                                                                float4* __restrict__ out, int M, int pf4,
                                                                int nv4, int ldc4, int S, int hw4) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)M * pf4) return;
  const size_t m = i / pf4;
  const int f4 = (int)(i - m * pf4);
  const size_t gi = m * nv4 + (size_t)(f4 / hw4) * 2 * hw4 + f4 % hw4, total = (size_t)M * nv4;
  float4 g = part[gi], u = part[gi + hw4];
  for (int sidx = 1; sidx < S; sidx++) {
    const float4 a = part[sidx * total + gi], b = part[sidx * total + gi + hw4];
    g.x += a.x; g.y += a.y; g.z += a.z; g.w += a.w;
    u.x += b.x; u.y += b.y; u.z += b.z; u.w += b.w;
  }
  float4 o;
  o.x = (g.x * (1.0f / (1.0f + expf(-g.x)))) * u.x;
  o.y = (g.y * (1.0f / (1.0f + expf(-g.y)))) * u.y;
  o.z = (g.z * (1.0f / (1.0f + expf(-g.z)))) * u.z;
  o.w = (g.w * (1.0f / (1.0f + expf(-g.w)))) * u.w;
  out[m * ldc4 + f4] = o;
}

}  // namespace tlhip

using namespace tlhip;

extern "C" {

// Three forms of one launcher.
//   plain: C[M][N] is the product.
//   parts (S_out != nullptr): the K-split parts are the result - C is then the caller's buffer,
//     [S][M][N], no part sum is launched and *S_out says how many there are (1: the plain
//     product); one piece, so that the layout is uniform.
//   gu: W = [gate rows | up rows], N = features (rows of each), C[M][N] = the gated activation.
//   scales != nullptr: W is an int4 weight (packed nibbles [rows][K/2], scales [rows][K/32]); any of
//     the three forms above.
//     Prompt chunks (M > 64) of an int4 weight run on two f16 planes of A instead of three bf16
//     ones (the nibbles are exact in either format); the exponents of A's rows are taken here.
static int gemm_bf16_nt_impl(const void* A, const void* W, void* C, int64_t M, int64_t N, int64_t K,
                             size_t parts_bytes, int* S_out, bool gu, const void* scales = nullptr) {
  TLHIP_REQUIRE_READY();
  const bool want_parts = S_out != nullptr;
  const bool q4 = scales != nullptr;
  if (!A || !W || !C) return fail(TLHIP_EINVAL, "tlhip_gemm_bf16_nt: null pointer");
  if (q4 && ((K % 32) != 0 || !aligned16(scales)))
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm_q4_nt: need K %% 32 == 0 (one scale per 32 weights) and aligned scales");
  // the reference's gate: K a multiple of 8
  if ((K % 8) != 0 || M <= 0 || N <= 0 || K <= 0)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm_bf16_nt: need K %% 8 == 0 and positive M, N, K");
  if (M > 0x3fffffff || N > 0x3fffffff || K > 0x3fffffff)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm_bf16_nt: dimension too large");
  if (!aligned16(A) || !aligned16(W)) return fail(TLHIP_EINVAL, "tlhip_gemm_bf16_nt: operands must be 16-byte aligned");
  Context& c = ctx();
  const float* pa = static_cast<const float*>(A);
  const uint16_t* pw = static_cast<const uint16_t*>(W);
  float* pc = static_cast<float*>(C);
  // Tile variants {MFMA tiles per wavefront in M, in N}, 2 x 2 wavefronts each. The wide one
  // (128 x 256 block tile, 64 x 128 per wavefront) needs fewest LDS reads per MFMA - the three
  // A planes make LDS, not the matrix pipe, the first limit - and runs 2 blocks per CU.
  // Work is shaped to fill those 2 * CUs block slots in whole rounds:
  //   * fewer tiles than slots: K is split over gridDim.y so that tiles * S comes close to
  //     the slots; parts go to scratch and are summed in a fixed order (no atomics);
  //   * more tiles than slots: the columns that make whole rounds run with full K, the
  //     remaining columns (less than one round of tiles) are split over K the same way.
  // gu: a tile column of bn is bn / 2 features wide (gate and up of each), so all widths below
  // are in units of N - columns, or features.
  auto cdiv = [](int64_t a, int64_t b) { return (a + b - 1) / b; };
  const int64_t slots = (int64_t)c.cus * 2;
  const int per = gu ? 2 : 1;                             // tile columns per unit of N
  const bool can_split = (N % 4) == 0 && aligned16(C);   // the part sum works on float4s
  const bool half = q4 && M > 64 && c.tune_gemm_planes != 3;
  const size_t ea_bytes = half ? (((size_t)M * sizeof(int) + 255) & ~(size_t)255) : 0;
  struct Piece { int64_t n0, n; int S; int variant; };    // columns (features) [n0, n0 + n)
  Piece pieces[2];
  int npieces = 0;
  auto pick_S = [&](int64_t tiles) {   // K splits that bring `tiles` blocks up to the slots
    if (!can_split || tiles >= slots) return 1;
    int64_t S = slots / tiles;   // never past the slots: a few blocks left for a second round double the launch
    if (S > 16) S = 16;
    while (S > 1 && K / S < 256) S--;
    if (want_parts)   // the caller's buffer bounds the parts
      while (S > 1 && (size_t)S * M * N * sizeof(float) > parts_bytes) S--;
    return (int)S;
  };
  if (M > 64) {
    // int4: two accumulator sets per wavefront, so 64 x 64 wavefront tiles (128 x 128 per block)
    const int64_t w = (q4 ? 128 : 256) / per;
    const int wide = q4 ? 3 : 0;
    const int64_t tm = cdiv(M, 128), tn = cdiv(N, w), tiles = tm * tn;
    const int64_t cols_per_round = slots / tm;            // whole tile columns in one round
    if (tiles <= slots || cols_per_round == 0 || !can_split || want_parts) {
      pieces[npieces++] = Piece{0, N, pick_S(tiles), wide};
    } else {
      const int64_t main_tn = tn / cols_per_round * cols_per_round;   // whole rounds
      const int64_t n_main = main_tn * w;
      pieces[npieces++] = Piece{0, n_main, 1, wide};
      if (n_main < N) pieces[npieces++] = Piece{n_main, N - n_main, pick_S(tm * (tn - main_tn)), wide};
    }
  } else {
    // short prompts: 64-row tiles; narrow ones when that is what fills the chip (a gated
    // tile needs two MFMA tiles per wavefront in N, so the narrow one is not for gu)
    const int64_t t128 = cdiv(N, 128 / per), t64 = cdiv(N, 64 / per);
    if (gu || q4 || t128 >= slots || pick_S(t128) > 1) pieces[npieces++] = Piece{0, N, pick_S(t128), 1};
    else pieces[npieces++] = Piece{0, N, pick_S(t64), 2};
  }
  static const int kBm[4] = {128, 64, 64, 128}, kBn[4] = {256, 128, 64, 128};
  // One scratch request for the whole call (a second, larger one could move the buffer): the
  // exponents of A's rows first, then room for the largest piece's K-split parts.
  size_t parts_need = 0;
  if (!want_parts)
    for (int pi = 0; pi < npieces; pi++) {
      const Piece& P = pieces[pi];
      const int bn = kBn[P.variant];
      const int64_t part_w = gu ? cdiv(P.n, bn / per) * bn : P.n;
      if (P.S > 1) parts_need = std::max(parts_need, (size_t)P.S * M * part_w * sizeof(float));
    }
  char* sbase = nullptr;
  if (ea_bytes + parts_need > 0) {
    sbase = static_cast<char*>(scratch(ea_bytes + parts_need));
    if (!sbase) return fail(TLHIP_ENOMEM, "tlhip_gemm_bf16_nt: no scratch for row exponents and K-split parts");
  }
  int* ea = reinterpret_cast<int*>(sbase);
  if (half) row_exponent_f32_kernel<<<dim3((unsigned)M), dim3(256), 0, c.stream>>>(pa, (int)K, ea);
  for (int pi = 0; pi < npieces; pi++) {
    const Piece& P = pieces[pi];
    const int bm = kBm[P.variant], bn = kBn[P.variant];
    const int64_t tcols = cdiv(P.n, bn / per);            // tile columns of this piece
    const int64_t part_w = gu ? tcols * bn : P.n;         // row width of a K-split part
    int S = P.S, kchunk = (int)K;
    float* dst = pc + P.n0;
    int ldc = (int)N;
    if (S > 1) {
      kchunk = (int)(cdiv(cdiv(K, S), kBK) * kBK);
      S = (int)cdiv(K, kchunk);
    }
    if (want_parts) {
      *S_out = S;             // one piece: dst is the caller's parts, [S][M][N]
      if (S == 1) kchunk = (int)K;
    } else if (S > 1) {
      dst = reinterpret_cast<float*>(sbase + ea_bytes);
      ldc = (int)part_w;
    } else {
      kchunk = (int)K;
    }
    const int64_t nblk = cdiv(M, bm) * tcols;
    if (nblk > 0x7fffffff || part_w > 0x7fffffff)
      return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm_bf16_nt: too many tiles for one grid");
    const dim3 grid((unsigned)nblk, (unsigned)S);
    // first row of the piece: bf16 rows are K elements, int4 rows K / 2 bytes + K / 32 scales
    const uint16_t* wp = q4 ? reinterpret_cast<const uint16_t*>(static_cast<const uint8_t*>(W) + (size_t)P.n0 * K / 2)
                            : pw + (size_t)P.n0 * K;
    const float* sp = q4 ? static_cast<const float*>(scales) + (size_t)P.n0 * (K / 32) : nullptr;
#define TLHIP_GEMM(TM_, TN_, GU_, Q4_, H_)                                                     \
  gemm_bf16_nt_kernel<TM_, TN_, 2, 2, GU_, Q4_, H_><<<grid, dim3(256), 0, c.stream>>>(         \
      pa, wp, dst, (int)M, (int)P.n, (int)K, kchunk, ldc, (int)N, sp, ea)
    switch (P.variant + (gu ? 4 : 0) + (q4 ? 8 : 0) + (half ? 16 : 0)) {
      case 0: TLHIP_GEMM(2, 4, false, false, false); break;
      case 1: TLHIP_GEMM(1, 2, false, false, false); break;
      case 2: TLHIP_GEMM(1, 1, false, false, false); break;
      case 4: TLHIP_GEMM(2, 4, true, false, false); break;
      case 5: TLHIP_GEMM(1, 2, true, false, false); break;
      case 9: TLHIP_GEMM(1, 2, false, true, false); break;
      case 11: TLHIP_GEMM(2, 2, false, true, false); break;
      case 13: TLHIP_GEMM(1, 2, true, true, false); break;
      case 15: TLHIP_GEMM(2, 2, true, true, false); break;
      case 27: TLHIP_GEMM(2, 2, false, true, true); break;
      case 31: TLHIP_GEMM(2, 2, true, true, true); break;
      default: return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm_bf16_nt: no kernel for this plan");
    }
#undef TLHIP_GEMM
    if (S > 1 && !want_parts) {
      const size_t total4 = (size_t)M * P.n / 4;
      const dim3 sgrid((unsigned)((total4 + 255) / 256));
      if (gu)
        splitk_sum_swiglu_kernel<<<sgrid, dim3(256), 0, c.stream>>>(
            reinterpret_cast<const float4*>(dst), reinterpret_cast<float4*>(pc + P.n0), (int)M,
            (int)(P.n / 4), (int)(part_w / 4), (int)(N / 4), S, bn / 4 / 4);
      else
        splitk_sum_kernel<<<sgrid, dim3(256), 0, c.stream>>>(
            reinterpret_cast<const float4*>(dst), reinterpret_cast<float4*>(pc + P.n0), (int)M,
            (int)(P.n / 4), (int)(N / 4), S);
    }
  }
  TLHIP_CHECK_LAUNCH(TLHIP_C_GEMM_BF16_NT);
}

int tlhip_gemm_bf16_nt(const void* A, const void* W, void* C, int64_t M, int64_t N, int64_t K) {
  return gemm_bf16_nt_impl(A, W, C, M, N, K, 0, nullptr, false);
}

int tlhip_gemm_bf16_nt_swiglu(const void* A, const void* W, void* act, int64_t M, int64_t ff, int64_t K) {
  return gemm_bf16_nt_impl(A, W, act, M, ff, K, 0, nullptr, true);
}

static int gemm_parts_entry(const void* A, const void* W, const void* scales, void* parts,
                            int64_t parts_bytes, int64_t M, int64_t N, int64_t K, int* n_parts) {
  if (!n_parts) return fail(TLHIP_EINVAL, "tlhip_gemm_*_nt_parts: null n_parts");
  if (M > 0 && N > 0 && parts_bytes < (int64_t)(M * N * sizeof(float)))
    return fail(TLHIP_EINVAL, "tlhip_gemm_*_nt_parts: the buffer must hold at least one [M, N] part");
  if (parts && !aligned16(parts)) return fail(TLHIP_EINVAL, "tlhip_gemm_*_nt_parts: parts must be 16-byte aligned");
  *n_parts = 0;
  return gemm_bf16_nt_impl(A, W, parts, M, N, K, (size_t)parts_bytes, n_parts, false, scales);
}

int tlhip_gemm_bf16_nt_parts(const void* A, const void* W, void* parts, int64_t parts_bytes, int64_t M,
                             int64_t N, int64_t K, int* n_parts) {
  return gemm_parts_entry(A, W, nullptr, parts, parts_bytes, M, N, K, n_parts);
}

// ---- the same three forms over an int4 weight (no reference counterpart: the reference feeds
// prompts to an int4 model token by token, qwen_model.h:419) ----
static int q4_gate(const void* scales, int64_t group) {
  if (!scales) return fail(TLHIP_EINVAL, "tlhip_gemm_q4_nt: null scales");
  if (group != 32) return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm_q4_nt: group must be 32");   // types.h:30
  return TLHIP_OK;
}

int tlhip_gemm_q4_nt(const void* A, const void* qw, const void* scales, void* C, int64_t M, int64_t N,
                     int64_t K, int64_t group) {
  if (int rc = q4_gate(scales, group)) return rc;
  return gemm_bf16_nt_impl(A, qw, C, M, N, K, 0, nullptr, false, scales);
}

int tlhip_gemm_q4_nt_swiglu(const void* A, const void* qw, const void* scales, void* act, int64_t M,
                            int64_t ff, int64_t K, int64_t group) {
  if (int rc = q4_gate(scales, group)) return rc;
  return gemm_bf16_nt_impl(A, qw, act, M, ff, K, 0, nullptr, true, scales);
}

int tlhip_gemm_q4_nt_parts(const void* A, const void* qw, const void* scales, void* parts,
                           int64_t parts_bytes, int64_t M, int64_t N, int64_t K, int64_t group,
                           int* n_parts) {
  if (int rc = q4_gate(scales, group)) return rc;
  return gemm_parts_entry(A, qw, scales, parts, parts_bytes, M, N, K, n_parts);
}

}  // extern "C"
