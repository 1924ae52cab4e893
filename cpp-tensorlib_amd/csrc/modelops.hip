// Model ops of the decode step: rope, rmsnorm (+fused residual), swiglu,
// argmax, KV-cache writes and the token-major/head-major moves of prefill.
// All are launch- or latency-bound at decode sizes; rows are processed with
// 128-bit accesses where the layout allows.
#include "common.hpp"

namespace tlhip {

// ---- rope ---------------------------------------------------------------------
// The angle is formed in fp64 exactly as the CPU path does (array.h:1719-1727):
// theta = pow((double)base, -2j/D), ang = position*theta, then cos/sin are
// rounded to f32 and the rotation runs in f32. Fast f32 intrinsics lose 1e-4
// at positions in the thousands with base 1e6.
__global__ __launch_bounds__(256) void rope_kernel(const float* __restrict__ x,
                                                   const float* __restrict__ bias,
                                                   float* __restrict__ out, int64_t rows, int T,
                                                   int D, int64_t pos, float base,
                                                   const uint32_t* __restrict__ dpos) {
  const int half = D >> 1;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * half) return;
  if (dpos) pos = (int64_t)*dpos;   // position kept on the device (captured decode loops)
  const int64_t r = i / half;
  const int j = (int)(i - r * half);
  const int64_t t = T ? r % T : 0;
  const double position = (double)(pos + t);
  const double theta = pow((double)base, -2.0 * (double)j / (double)D);
  const double ang = position * theta;
  const float c = (float)cos(ang), s = (float)sin(ang);
  const size_t bi = (size_t)r * D;
  float x0 = x[bi + j], x1 = x[bi + j + half];
  if (bias) {
    x0 += bias[bi + j];
    x1 += bias[bi + j + half];
  }
  out[bi + j] = sub_rn(mul_rn(x0, c), mul_rn(x1, s));
  out[bi + j + half] = add_rn(mul_rn(x0, s), mul_rn(x1, c));
}

// ---- rmsnorm --------------------------------------------------------------------
// One block per row. Follows the array composition (array.h:2429-2433):
// ms = sum(x*x) * (1/n); inv = 1/sqrt(ms + eps); out = (x*inv)*w.
// S > 1: delta is S parts, `part_stride` floats apart (the K-split parts of a GEMM), added up in
// ascending order before the residual add - what a part-sum launch followed by this one computes.
template <bool RES>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x,
                                                      const float* __restrict__ delta,
                                                      const float* __restrict__ w,
                                                      float* __restrict__ xout,
                                                      float* __restrict__ hout, int n, float eps,
                                                      int S = 1, size_t part_stride = 0) {
  __shared__ float red[4];
  const size_t base = (size_t)blockIdx.x * n;
  float acc = 0.f;
  if ((n & 3) == 0) {
    const float4* x4 = reinterpret_cast<const float4*>(x + base);
    const float4* d4 = RES ? reinterpret_cast<const float4*>(delta + base) : nullptr;
    float4* xo4 = RES ? reinterpret_cast<float4*>(xout + base) : nullptr;
    const size_t ps4 = part_stride >> 2;
    for (int i = threadIdx.x; i < (n >> 2); i += 256) {
      float4 v = x4[i];
      if (RES) {
        float4 d = d4[i];
        int sidx = 1;
        for (; sidx + 4 <= S; sidx += 4) {   // four loads in flight, added in ascending order
          float4 e[4];
#pragma unroll
          for (int u = 0; u < 4; u++) e[u] = d4[(sidx + u) * ps4 + i];
#pragma unroll
          for (int u = 0; u < 4; u++) { d.x += e[u].x; d.y += e[u].y; d.z += e[u].z; d.w += e[u].w; }
        }
        for (; sidx < S; sidx++) {
          const float4 e = d4[sidx * ps4 + i];
          d.x += e.x; d.y += e.y; d.z += e.z; d.w += e.w;
        }
        v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
        xo4[i] = v;
      }
      acc += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
    }
  } else {
    for (int i = threadIdx.x; i < n; i += 256) {
      float v = x[base + i];
      if (RES) {
        float d = delta[base + i];
        for (int sidx = 1; sidx < S; sidx++) d += delta[sidx * part_stride + base + i];
        v += d;
        xout[base + i] = v;
      }
      acc += v * v;
    }
  }
  if (RES) __threadfence_block();
  const float sum = block_sum<4>(acc, red);  // also orders the xout stores before the re-read
  const float inv = 1.0f / sqrtf(sum * (1.0f / (float)n) + eps);
  const float* src = RES ? xout : x;
  for (int i = threadIdx.x; i < n; i += 256) hout[base + i] = (src[base + i] * inv) * w[i];
}

// Wide variant for rows that fit the registers of one 1024-thread block
// (n % 4 == 0, n <= 4*1024*RV): every thread keeps its float4s of the row and of
// the weight in VGPRs, so the row is read once and nothing waits on a second
// pass. This is the model shape (n = 896 ... 8192), for one row of a decode step and for
// the 512 rows of a prompt chunk alike (6.6 us against 11.1 us for 512 x 3584).
template <bool RES, int RV>
__global__ __launch_bounds__(1024) void rmsnorm_wide_kernel(const float* __restrict__ x,
                                                            const float* __restrict__ delta,
                                                            const float* __restrict__ w,
                                                            float* __restrict__ xout,
                                                            float* __restrict__ hout, int n,
                                                            float eps, int S = 1,
                                                            size_t part_stride = 0) {
  __shared__ float red[16];
  const size_t base = (size_t)blockIdx.x * n;
  const int n4 = n >> 2;
  const float4* x4 = reinterpret_cast<const float4*>(x + base);
  const float4* d4 = RES ? reinterpret_cast<const float4*>(delta + base) : nullptr;
  const float4* w4 = reinterpret_cast<const float4*>(w);
  float4 v[RV], wv[RV];
  float acc = 0.f;
#pragma unroll
  for (int k = 0; k < RV; k++) {
    const int i = threadIdx.x + k * 1024;
    if (i < n4) {
      v[k] = x4[i];
      wv[k] = w4[i];
      if (RES) {
        float4 d = d4[i];
        for (int sidx = 1; sidx < S; sidx++) {   // K-split parts, ascending
          const float4 e = d4[sidx * (part_stride >> 2) + i];
          d.x += e.x; d.y += e.y; d.z += e.z; d.w += e.w;
        }
        v[k].x += d.x; v[k].y += d.y; v[k].z += d.z; v[k].w += d.w;
      }
    }
  }
#pragma unroll
  for (int k = 0; k < RV; k++) {
    const int i = threadIdx.x + k * 1024;
    if (i < n4) {
      if (RES) reinterpret_cast<float4*>(xout + base)[i] = v[k];
      acc += (v[k].x * v[k].x + v[k].y * v[k].y) + (v[k].z * v[k].z + v[k].w * v[k].w);
    }
  }
  const float sum = block_sum<16>(acc, red);
  const float inv = 1.0f / sqrtf(sum * (1.0f / (float)n) + eps);
#pragma unroll
  for (int k = 0; k < RV; k++) {
    const int i = threadIdx.x + k * 1024;
    if (i < n4) {
      float4 o;
      o.x = (v[k].x * inv) * wv[k].x; o.y = (v[k].y * inv) * wv[k].y;
      o.z = (v[k].z * inv) * wv[k].z; o.w = (v[k].w * inv) * wv[k].w;
      reinterpret_cast<float4*>(hout + base)[i] = o;
    }
  }
}

template <bool RES>
static void launch_rmsnorm(const float* x, const float* delta, const float* w, float* xout,
                           float* hout, int64_t n, float eps, int64_t rows, int S = 1) {
  hipStream_t st = ctx().stream;
  const size_t ps = (size_t)(rows * n);   // delta parts, when S > 1
  const bool wide_ok = (n % 4) == 0 && aligned16(w) && aligned16(hout);
  if (wide_ok && n <= 4096)
    rmsnorm_wide_kernel<RES, 1><<<dim3((unsigned)rows), dim3(1024), 0, st>>>(x, delta, w, xout, hout, (int)n, eps, S, ps);
  else if (wide_ok && n <= 8192)
    rmsnorm_wide_kernel<RES, 2><<<dim3((unsigned)rows), dim3(1024), 0, st>>>(x, delta, w, xout, hout, (int)n, eps, S, ps);
  else
    rmsnorm_kernel<RES><<<dim3((unsigned)rows), dim3(256), 0, st>>>(x, delta, w, xout, hout, (int)n, eps, S, ps);
}

// ---- swiglu -----------------------------------------------------------------------
// out = (g * sigmoid(g)) * u, the order of array.h:2435-2439.
__global__ __launch_bounds__(256) void swiglu_kernel(const float* __restrict__ gu,
                                                     float* __restrict__ out, int64_t ff) {
  const int64_t f = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (f >= ff) return;
  const size_t src = (size_t)blockIdx.y * 2 * ff + f;
  const float g = gu[src];
  const float sg = 1.0f / (1.0f + expf(-g));
  out[(size_t)blockIdx.y * ff + f] = (g * sg) * gu[src + ff];
}

// ---- argmax ---------------------------------------------------------------------------
// Stage 1: each block scans a slice and keeps (max, smallest index attaining it).
// Stage 2: one block merges the slices. Ties always go to the smallest index
// (array.h:2481-2494 uses a strict '>').
__device__ __forceinline__ void argmax_merge(float& v, int& i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

__device__ __forceinline__ void argmax_block(float& v, int& i, float* sv, int* si) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    const float ov = __shfl_xor(v, m, kWave);
    const int oi = __shfl_xor(i, m, kWave);
    argmax_merge(v, i, ov, oi);
  }
  const int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { sv[w] = v; si[w] = i; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < 4; k++) argmax_merge(v, i, sv[k], si[k]);
  }
}

__global__ __launch_bounds__(256) void argmax_stage1(const float* __restrict__ in, int64_t n,
                                                     float* __restrict__ pv, int* __restrict__ pi) {
  __shared__ float sv[4];
  __shared__ int si[4];
  float v = -INFINITY;
  int idx = 0x7fffffff;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const float x = in[i];
    if (x > v || idx == 0x7fffffff) { v = x; idx = (int)i; }
  }
  argmax_block(v, idx, sv, si);
  if (threadIdx.x == 0) { pv[blockIdx.x] = v; pi[blockIdx.x] = idx; }
}

__global__ __launch_bounds__(256) void argmax_stage2(const float* __restrict__ pv,
                                                     const int* __restrict__ pi, int nparts,
                                                     int* __restrict__ out) {
  __shared__ float sv[4];
  __shared__ int si[4];
  float v = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = threadIdx.x; i < nparts; i += 256) argmax_merge(v, idx, pv[i], pi[i]);
  argmax_block(v, idx, sv, si);
  if (threadIdx.x == 0) out[0] = idx == 0x7fffffff ? 0 : idx;
}

// ---- cache writes and head moves -----------------------------------------------------------
template <typename KT>
__device__ __forceinline__ KT kv_narrow(float v);
template <> __device__ __forceinline__ float kv_narrow<float>(float v) { return v; }
template <> __device__ __forceinline__ uint16_t kv_narrow<uint16_t>(float v) { return f32_to_bf16_rne(v); }

// k,v [Hkv,T,D] -> cache [Hkv,kv_max,D] rows pos0..pos0+T (T == 1: append)
template <typename KT>
__global__ __launch_bounds__(256) void kv_write_kernel(KT* __restrict__ Kc, KT* __restrict__ Vc,
                                                       const float* __restrict__ k,
                                                       const float* __restrict__ v, int64_t T,
                                                       int64_t kv_max, int D, int64_t pos0,
                                                       int64_t total,
                                                       const uint32_t* __restrict__ dpos) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  if (dpos) {
    pos0 = (int64_t)*dpos;
    if (pos0 + T > kv_max) return;   // a full cache drops the write instead of leaving it
  }
  const int d = (int)(i % D);
  const int64_t hp = i / D;
  const int64_t p = hp % T, h = hp / T;
  const size_t dst = ((size_t)h * kv_max + pos0 + p) * D + d;
  Kc[dst] = kv_narrow<KT>(k[i]);
  Vc[dst] = kv_narrow<KT>(v[i]);
}

__global__ __launch_bounds__(256) void split_heads_kernel(const float* __restrict__ src,
                                                          const float* __restrict__ bias,
                                                          float* __restrict__ dst, int64_t T,
                                                          int64_t ld, int64_t off, int D,
                                                          int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;  // i indexes dst [H,T,D]
  const int d = (int)(i % D);
  const int64_t ht = i / D;
  const int64_t t = ht % T, h = ht / T;
  float v = src[(size_t)t * ld + off + h * D + d];
  if (bias) v += bias[h * D + d];
  dst[i] = v;
}

__global__ __launch_bounds__(256) void merge_heads_kernel(const float* __restrict__ src,
                                                          float* __restrict__ dst, int64_t T,
                                                          int64_t H, int D, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;  // i indexes dst [T,H*D]
  const int d = (int)(i % D);
  const int64_t th = i / D;
  const int64_t h = th % H, t = th / H;
  dst[i] = src[((size_t)h * T + t) * D + d];
}

// ---- fused q/k/v epilogue of a decode step --------------------------------------------
// One launch for what the step otherwise does in four: q and k get their bias
// and rotary embedding (written back in place), v gets its bias, and the new k, v
// rows go straight into the cache at row `pos`. qkv = [q (Hq*D) | k (Hkv*D) | v (Hkv*D)].
template <typename KT>
__global__ __launch_bounds__(256) void qkv_rope_append_kernel(
    float* __restrict__ qkv, const float* __restrict__ bq, const float* __restrict__ bk,
    const float* __restrict__ bv, KT* __restrict__ Kc, KT* __restrict__ Vc, int Hq, int Hkv, int D,
    int64_t pos, int64_t kv_max, float base, const uint32_t* __restrict__ dpos,
    const float2* __restrict__ table) {
  if (dpos) {   // position kept on the device; a full cache drops the step's writes
    pos = (int64_t)*dpos;
    if (pos >= kv_max) return;
  }
  const int half = D >> 1;
  const int n_rot = (Hq + Hkv) * half;       // rotary pairs of q and k
  const int n_v = Hkv * D;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_rot) {
    const int r = i / half, j = i - r * half;   // r: head row within [q heads | k heads]
    float c, s;
    if (table) {   // (cos, sin) of this step's position, formed once per step by rope_table_kernel
      const float2 cs = table[j];
      c = cs.x;
      s = cs.y;
    } else {
      const double theta = pow((double)base, -2.0 * (double)j / (double)D);
      const double ang = (double)pos * theta;
      c = (float)cos(ang);
      s = (float)sin(ang);
    }
    const size_t bi = (size_t)r * D;
    const bool is_k = r >= Hq;
    const float* bias = is_k ? (bk ? bk + (size_t)(r - Hq) * D : nullptr) : (bq ? bq + bi : nullptr);
    float x0 = qkv[bi + j], x1 = qkv[bi + j + half];
    if (bias) { x0 += bias[j]; x1 += bias[j + half]; }
    const float o0 = sub_rn(mul_rn(x0, c), mul_rn(x1, s));
    const float o1 = add_rn(mul_rn(x0, s), mul_rn(x1, c));
    qkv[bi + j] = o0;
    qkv[bi + j + half] = o1;
    if (is_k) {
      const size_t dst = ((size_t)(r - Hq) * kv_max + pos) * D;
      Kc[dst + j] = kv_narrow<KT>(o0);
      Kc[dst + j + half] = kv_narrow<KT>(o1);
    }
  } else if (i < n_rot + n_v) {
    const int e = i - n_rot, h = e / D, d = e - h * D;
    float* vp = qkv + (size_t)(Hq + Hkv) * D;
    float v = vp[e];
    if (bv) v += bv[e];
    vp[e] = v;
    Vc[((size_t)h * kv_max + pos) * D + d] = kv_narrow<KT>(v);
  }
}

__global__ void incr_u32_kernel(uint32_t* p) { *p += 1u; }

// table[j] = (cos, sin)(pos * base^(-2j/D)), the same fp64 expression as rope_kernel:
// every layer of a decode step rotates by the same angles, so a step forms them once.
__global__ void rope_table_kernel(float2* __restrict__ table, int D, int64_t pos, float base,
                                  const uint32_t* __restrict__ dpos) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= (D >> 1)) return;
  if (dpos) pos = (int64_t)*dpos;
  const double theta = pow((double)base, -2.0 * (double)j / (double)D);
  const double ang = (double)pos * theta;
  table[j] = make_float2((float)cos(ang), (float)sin(ang));
}

// table[t][j] = (cos, sin)((pos0 + t) * base^(-2j/D)), t < T: the angles of a prompt chunk, the
// same for every layer and every head (rope_kernel forms each of them once per head and layer).
__global__ __launch_bounds__(256) void rope_table_range_kernel(float2* __restrict__ table, int D,
                                                               int64_t pos0, int T, float base) {
  const int half = D >> 1;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T * half) return;
  const int t = i / half, j = i - t * half;
  const double theta = pow((double)base, -2.0 * (double)j / (double)D);
  const double ang = (double)(pos0 + t) * theta;
  table[i] = make_float2((float)cos(ang), (float)sin(ang));
}

// ---- fused q/k/v epilogue of a prompt chunk --------------------------------------------------
// One launch for what the chunk otherwise does in five (split_heads with bias, rope of q, rope
// of k, and the two cache fills): qkv [T, (Hq + 2 Hkv) D] token-major from the projection GEMM;
// q gets bias and rotation and lands head-major in qh [Hq, T, D]; k gets bias and rotation,
// v its bias, and both go straight into cache rows pos0 .. pos0 + T. Same arithmetic as the
// separate kernels (bias add, unfused multiplies, one add / sub), so results are bit-identical.
// A thread owns 4 consecutive rotary pairs (j .. j+3 with j + D/2 ..) or 4 consecutive v values.
template <typename KT>
__device__ __forceinline__ void kv_store4(KT* p, const float4 v);
template <> __device__ __forceinline__ void kv_store4<float>(float* p, const float4 v) {
  *reinterpret_cast<float4*>(p) = v;
}
template <> __device__ __forceinline__ void kv_store4<uint16_t>(uint16_t* p, const float4 v) {
  const uint32_t lo = (uint32_t)f32_to_bf16_rne(v.x) | ((uint32_t)f32_to_bf16_rne(v.y) << 16);
  const uint32_t hi = (uint32_t)f32_to_bf16_rne(v.z) | ((uint32_t)f32_to_bf16_rne(v.w) << 16);
  *reinterpret_cast<uint2*>(p) = make_uint2(lo, hi);
}

template <typename KT>
__global__ __launch_bounds__(256) void qkv_rope_fill_kernel(
    const float* __restrict__ qkv, const float* __restrict__ bq, const float* __restrict__ bk,
    const float* __restrict__ bv, const float2* __restrict__ table, float* __restrict__ qh,
    KT* __restrict__ Kc, KT* __restrict__ Vc, int T, int Hq, int Hkv, int D, int64_t pos0,
    int64_t kv_max, int S, size_t part_stride) {
  // S > 1: qkv is the S K-split parts of the projection, part_stride floats apart, added up in
  // ascending order as the part-sum launch would have
  auto ld4 = [&](const float* p) {
    float4 a = *reinterpret_cast<const float4*>(p);
    for (int sidx = 1; sidx < S; sidx++) {
      const float4 b = *reinterpret_cast<const float4*>(p + sidx * part_stride);
      a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
    }
    return a;
  };
  const int half = D >> 1, q4 = half >> 2;            // float4 groups per half row
  const int rot_per_t = (Hq + Hkv) * q4, v_per_t = Hkv * (D >> 2);
  const int per_t = rot_per_t + v_per_t;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)T * per_t) return;
  const int t = (int)(i / per_t), e = (int)(i - (int64_t)t * per_t);
  const float* row = qkv + (size_t)t * (Hq + 2 * Hkv) * D;
  if (e < rot_per_t) {
    const int r = e / q4, j = (e - r * q4) * 4;       // r: head within [q heads | k heads]
    const bool is_k = r >= Hq;
    const float* bias = is_k ? (bk ? bk + (size_t)(r - Hq) * D : nullptr) : (bq ? bq + (size_t)r * D : nullptr);
    float4 x0 = ld4(row + (size_t)r * D + j);
    float4 x1 = ld4(row + (size_t)r * D + j + half);
    if (bias) {
      const float4 b0 = *reinterpret_cast<const float4*>(bias + j);
      const float4 b1 = *reinterpret_cast<const float4*>(bias + j + half);
      x0.x += b0.x; x0.y += b0.y; x0.z += b0.z; x0.w += b0.w;
      x1.x += b1.x; x1.y += b1.y; x1.z += b1.z; x1.w += b1.w;
    }
    const float2* cs = table + (size_t)t * half + j;
    const float2 c0 = cs[0], c1 = cs[1], c2 = cs[2], c3 = cs[3];
    float4 o0, o1;
    o0.x = sub_rn(mul_rn(x0.x, c0.x), mul_rn(x1.x, c0.y));
    o1.x = add_rn(mul_rn(x0.x, c0.y), mul_rn(x1.x, c0.x));
    o0.y = sub_rn(mul_rn(x0.y, c1.x), mul_rn(x1.y, c1.y));
    o1.y = add_rn(mul_rn(x0.y, c1.y), mul_rn(x1.y, c1.x));
    o0.z = sub_rn(mul_rn(x0.z, c2.x), mul_rn(x1.z, c2.y));
    o1.z = add_rn(mul_rn(x0.z, c2.y), mul_rn(x1.z, c2.x));
    o0.w = sub_rn(mul_rn(x0.w, c3.x), mul_rn(x1.w, c3.y));
    o1.w = add_rn(mul_rn(x0.w, c3.y), mul_rn(x1.w, c3.x));
    if (is_k) {
      KT* dst = Kc + ((size_t)(r - Hq) * kv_max + pos0 + t) * D;
      kv_store4<KT>(dst + j, o0);
      kv_store4<KT>(dst + j + half, o1);
    } else {
      float* dst = qh + ((size_t)r * T + t) * D;
      *reinterpret_cast<float4*>(dst + j) = o0;
      *reinterpret_cast<float4*>(dst + j + half) = o1;
    }
  } else {
    const int ev = e - rot_per_t, h = ev / (D >> 2), d = (ev - h * (D >> 2)) * 4;
    float4 v = ld4(row + (size_t)(Hq + Hkv) * D + (size_t)h * D + d);
    if (bv) {
      const float4 b = *reinterpret_cast<const float4*>(bv + (size_t)h * D + d);
      v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w;
    }
    kv_store4<KT>(Vc + ((size_t)h * kv_max + pos0 + t) * D + d, v);
  }
}

// ---- device-resident greedy loop --------------------------------------------------------
// out[j] = widen(table[tok][j]) with tok read from the device (the previous step's argmax).
__global__ __launch_bounds__(256) void embed_gather_bf16_kernel(const uint16_t* __restrict__ table,
                                                                const int* __restrict__ d_token,
                                                                float* __restrict__ out, int hidden,
                                                                int vocab) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= hidden) return;
  int tok = *d_token;
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  out[j] = __uint_as_float((uint32_t)table[(size_t)tok * hidden + j] << 16);
}

// history[*d_pos] = *d_token (when it fits), then *d_pos += 1: the tail of a recorded greedy step.
__global__ void token_advance_kernel(uint32_t* d_pos, const int* d_token, int* history, uint32_t capacity) {
  const uint32_t p = *d_pos;
  if (history && p < capacity) history[p] = *d_token;
  *d_pos = p + 1u;
}

static unsigned blocks_for(int64_t n) { return (unsigned)((n + 255) / 256); }

}  // namespace tlhip

using namespace tlhip;

extern "C" {

static int rope_launch(const void* x, void* out, int64_t rows, int64_t T, int64_t D, int64_t pos,
                       float base, const void* bias, const void* d_pos) {
  if (!x || !out || rows < 0 || T < 0) return fail(TLHIP_EINVAL, "tlhip_rope: bad arguments");
  if (D <= 0 || (D & 1)) return fail(TLHIP_EUNSUPPORTED, "tlhip_rope: head_dim must be even");  // cuda.h:1208
  if (rows == 0) return TLHIP_OK;
  const int64_t n = rows * (D / 2);
  if (n > (int64_t)0x7fffffff * 128) return fail(TLHIP_EUNSUPPORTED, "tlhip_rope: too large");
  rope_kernel<<<dim3(blocks_for(n)), dim3(256), 0, ctx().stream>>>(
      static_cast<const float*>(x), static_cast<const float*>(bias), static_cast<float*>(out), rows,
      (int)T, (int)D, pos, base, static_cast<const uint32_t*>(d_pos));
  TLHIP_CHECK_LAUNCH(TLHIP_C_ROPE);
}

int tlhip_rope(const void* x, void* out, int64_t rows, int64_t T, int64_t D, int64_t pos,
               float base, const void* bias) {
  TLHIP_REQUIRE_READY();
  return rope_launch(x, out, rows, T, D, pos, base, bias, nullptr);
}

int tlhip_rope_dpos(const void* x, void* out, int64_t rows, int64_t T, int64_t D, const void* d_pos,
                    float base, const void* bias) {
  TLHIP_REQUIRE_READY();
  if (!d_pos) return fail(TLHIP_EINVAL, "tlhip_rope_dpos: null position pointer");
  return rope_launch(x, out, rows, T, D, 0, base, bias, d_pos);
}

int tlhip_incr_u32(void* d_pos) {
  TLHIP_REQUIRE_READY();
  if (!d_pos) return fail(TLHIP_EINVAL, "tlhip_incr_u32: null pointer");
  incr_u32_kernel<<<dim3(1), dim3(1), 0, ctx().stream>>>(static_cast<uint32_t*>(d_pos));
  hipError_t e_ = hipGetLastError();
  if (e_ != hipSuccess) return hip_fail(e_, "kernel launch");
  return TLHIP_OK;
}

int tlhip_rmsnorm(const void* x, const void* w, void* out, int64_t n, float eps, int64_t rows) {
  TLHIP_REQUIRE_READY();
  if (!x || !w || !out) return fail(TLHIP_EINVAL, "tlhip_rmsnorm: null pointer");
  if (n <= 0 || rows <= 0 || n > 0x7fffffff || rows > 0x7fffffff)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_rmsnorm: n and rows must be positive");  // cuda.h:1290
  if (!aligned16(x) || !aligned16(out)) return fail(TLHIP_EINVAL, "tlhip_rmsnorm: misaligned");
  launch_rmsnorm<false>(static_cast<const float*>(x), nullptr, static_cast<const float*>(w), nullptr,
                        static_cast<float*>(out), n, eps, rows);
  TLHIP_CHECK_LAUNCH(TLHIP_C_RMSNORM);
}

int tlhip_rmsnorm_res(const void* x, const void* delta, const void* w, void* xout, void* hout,
                      int64_t n, float eps, int64_t rows) {
  TLHIP_REQUIRE_READY();
  if (!x || !delta || !w || !xout || !hout) return fail(TLHIP_EINVAL, "tlhip_rmsnorm_res: null pointer");
  if (n <= 0 || rows <= 0 || n > 0x7fffffff || rows > 0x7fffffff)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_rmsnorm_res: n and rows must be positive");
  if (!aligned16(x) || !aligned16(delta) || !aligned16(xout))
    return fail(TLHIP_EINVAL, "tlhip_rmsnorm_res: misaligned");
  launch_rmsnorm<true>(static_cast<const float*>(x), static_cast<const float*>(delta),
                       static_cast<const float*>(w), static_cast<float*>(xout),
                       static_cast<float*>(hout), n, eps, rows);
  TLHIP_CHECK_LAUNCH(TLHIP_C_RMSNORM_RES);
}

int tlhip_rmsnorm_res_parts(const void* x, const void* parts, int64_t S, const void* w, void* xout,
                            void* hout, int64_t n, float eps, int64_t rows) {
  TLHIP_REQUIRE_READY();
  if (!x || !parts || !w || !xout || !hout) return fail(TLHIP_EINVAL, "tlhip_rmsnorm_res_parts: null pointer");
  if (n <= 0 || rows <= 0 || n > 0x7fffffff || rows > 0x7fffffff || S <= 0 || S > 64)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_rmsnorm_res_parts: need positive n, rows and 1 <= S <= 64");
  if (!aligned16(x) || !aligned16(parts) || !aligned16(xout))
    return fail(TLHIP_EINVAL, "tlhip_rmsnorm_res_parts: misaligned");
  if (xout == parts) return fail(TLHIP_EINVAL, "tlhip_rmsnorm_res_parts: xout must not alias the parts");
  launch_rmsnorm<true>(static_cast<const float*>(x), static_cast<const float*>(parts),
                       static_cast<const float*>(w), static_cast<float*>(xout),
                       static_cast<float*>(hout), n, eps, rows, (int)S);
  TLHIP_CHECK_LAUNCH(TLHIP_C_RMSNORM_RES);
}

int tlhip_swiglu(const void* gu, void* out, int64_t ff, int64_t rows) {
  TLHIP_REQUIRE_READY();
  if (!gu || !out) return fail(TLHIP_EINVAL, "tlhip_swiglu: null pointer");
  if (ff <= 0 || rows <= 0 || rows > 65535)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_swiglu: ff>0 and 0<rows<=65535 required");
  swiglu_kernel<<<dim3(blocks_for(ff), (unsigned)rows), dim3(256), 0, ctx().stream>>>(
      static_cast<const float*>(gu), static_cast<float*>(out), ff);
  TLHIP_CHECK_LAUNCH(TLHIP_C_SWIGLU);
}

int tlhip_argmax_async(const void* in, int64_t n, void* out_idx_dev) {
  TLHIP_REQUIRE_READY();
  if (!in || !out_idx_dev || n <= 0 || n > 0x7fffffff)
    return fail(TLHIP_EINVAL, "tlhip_argmax: bad arguments");  // cuda.h:1263
  int parts = (int)((n + 2047) / 2048);
  if (parts > 1024) parts = 1024;
  char* s = static_cast<char*>(scratch(2 * 1024 * sizeof(float)));
  if (!s) return fail(TLHIP_ENOMEM, "tlhip_argmax: no scratch");
  float* pv = reinterpret_cast<float*>(s);
  int* pi = reinterpret_cast<int*>(s + 1024 * sizeof(float));
  argmax_stage1<<<dim3(parts), dim3(256), 0, ctx().stream>>>(static_cast<const float*>(in), n, pv, pi);
  argmax_stage2<<<dim3(1), dim3(256), 0, ctx().stream>>>(pv, pi, parts, static_cast<int*>(out_idx_dev));
  TLHIP_CHECK_LAUNCH(TLHIP_C_ARGMAX);
}

int tlhip_argmax(const void* in, int64_t n, int64_t* out_idx) {
  TLHIP_REQUIRE_READY();
  if (!out_idx) return fail(TLHIP_EINVAL, "tlhip_argmax: null out pointer");
  Context& c = ctx();
  if (int rc = tlhip_argmax_async(in, n, c.argmax_dev)) return rc;
  hipError_t e = hipMemcpyAsync(c.argmax_host, c.argmax_dev, sizeof(int), hipMemcpyDeviceToHost, c.stream);
  if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
  if (e != hipSuccess) return hip_fail(e, "argmax result copy");
  *out_idx = *c.argmax_host;
  return TLHIP_OK;
}

static int kv_write(void* Kc, void* Vc, const void* k, const void* v, int64_t T, int64_t kv_max,
                    int64_t n_kv_heads, int64_t D, int kv_bf16, int64_t pos0, int census_id,
                    const char* who, const void* d_pos = nullptr) {
  if (!Kc || !Vc || !k || !v) return fail(TLHIP_EINVAL, "%s: null pointer", who);
  const uint32_t* dp = static_cast<const uint32_t*>(d_pos);
  if (D != 64 && D != 128) return fail(TLHIP_EUNSUPPORTED, "%s: head_dim must be 64 or 128", who);  // cuda.h:1122
  if (T <= 0 || n_kv_heads <= 0 || pos0 < 0 || pos0 + T > kv_max)
    return fail(TLHIP_EINVAL, "%s: rows [%lld,%lld) outside the cache of %lld", who, (long long)pos0,
                (long long)(pos0 + T), (long long)kv_max);
  const int64_t total = n_kv_heads * T * D;
  if (kv_bf16)
    kv_write_kernel<uint16_t><<<dim3(blocks_for(total)), dim3(256), 0, ctx().stream>>>(
        static_cast<uint16_t*>(Kc), static_cast<uint16_t*>(Vc), static_cast<const float*>(k),
        static_cast<const float*>(v), T, kv_max, (int)D, pos0, total, dp);
  else
    kv_write_kernel<float><<<dim3(blocks_for(total)), dim3(256), 0, ctx().stream>>>(
        static_cast<float*>(Kc), static_cast<float*>(Vc), static_cast<const float*>(k),
        static_cast<const float*>(v), T, kv_max, (int)D, pos0, total, dp);
  TLHIP_CHECK_LAUNCH(census_id);
}

int tlhip_embed_gather_bf16(const void* table, const void* d_token, void* out, int64_t hidden,
                            int64_t vocab) {
  TLHIP_REQUIRE_READY();
  if (!table || !d_token || !out) return fail(TLHIP_EINVAL, "tlhip_embed_gather_bf16: null pointer");
  if (hidden <= 0 || vocab <= 0 || hidden > 0x7fffffff || vocab > 0x7fffffff)
    return fail(TLHIP_EINVAL, "tlhip_embed_gather_bf16: bad sizes");
  embed_gather_bf16_kernel<<<dim3(blocks_for(hidden)), dim3(256), 0, ctx().stream>>>(
      static_cast<const uint16_t*>(table), static_cast<const int*>(d_token), static_cast<float*>(out),
      (int)hidden, (int)vocab);
  hipError_t e_ = hipGetLastError();
  if (e_ != hipSuccess) return hip_fail(e_, "kernel launch");
  return TLHIP_OK;
}

int tlhip_token_advance(void* d_pos, const void* d_token, void* history, int64_t capacity) {
  TLHIP_REQUIRE_READY();
  if (!d_pos || !d_token) return fail(TLHIP_EINVAL, "tlhip_token_advance: null pointer");
  if (capacity < 0 || capacity > 0xffffffffll) return fail(TLHIP_EINVAL, "tlhip_token_advance: bad capacity");
  token_advance_kernel<<<dim3(1), dim3(1), 0, ctx().stream>>>(
      static_cast<uint32_t*>(d_pos), static_cast<const int*>(d_token), static_cast<int*>(history),
      (uint32_t)capacity);
  hipError_t e_ = hipGetLastError();
  if (e_ != hipSuccess) return hip_fail(e_, "kernel launch");
  return TLHIP_OK;
}

int tlhip_kv_append_dpos(void* Kc, void* Vc, const void* k_new, const void* v_new, const void* d_pos,
                         int64_t kv_max, int64_t n_kv_heads, int64_t D, int kv_bf16) {
  TLHIP_REQUIRE_READY();
  if (!d_pos) return fail(TLHIP_EINVAL, "tlhip_kv_append_dpos: null position pointer");
  return kv_write(Kc, Vc, k_new, v_new, 1, kv_max, n_kv_heads, D, kv_bf16, 0, TLHIP_C_KV_APPEND,
                  "tlhip_kv_append_dpos", d_pos);
}

int tlhip_kv_append(void* Kc, void* Vc, const void* k_new, const void* v_new, int64_t pos,
                    int64_t kv_max, int64_t n_kv_heads, int64_t D, int kv_bf16) {
  TLHIP_REQUIRE_READY();
  return kv_write(Kc, Vc, k_new, v_new, 1, kv_max, n_kv_heads, D, kv_bf16, pos, TLHIP_C_KV_APPEND,
                  "tlhip_kv_append");
}

static int qkv_rope_append_launch(void* qkv, const void* bq, const void* bk, const void* bv, void* Kc,
                                  void* Vc, int64_t n_q_heads, int64_t n_kv_heads, int64_t D,
                                  int64_t pos, int64_t kv_max, float base, int kv_bf16,
                                  const void* d_pos, const void* table = nullptr) {
  if (!qkv || !Kc || !Vc) return fail(TLHIP_EINVAL, "tlhip_qkv_rope_append: null pointer");
  if (D != 64 && D != 128) return fail(TLHIP_EUNSUPPORTED, "tlhip_qkv_rope_append: head_dim must be 64 or 128");
  if (n_q_heads <= 0 || n_kv_heads <= 0 || n_q_heads > 4096)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_qkv_rope_append: bad head counts");
  if (!d_pos && (pos < 0 || pos >= kv_max))
    return fail(TLHIP_EINVAL, "tlhip_qkv_rope_append: row %lld outside the cache of %lld",
                (long long)pos, (long long)kv_max);
  const int64_t total = (n_q_heads + n_kv_heads) * (D / 2) + n_kv_heads * D;
  const float* pbq = static_cast<const float*>(bq);
  const float* pbk = static_cast<const float*>(bk);
  const uint32_t* dp = static_cast<const uint32_t*>(d_pos);
  const float2* tb = static_cast<const float2*>(table);
  if (kv_bf16)
    qkv_rope_append_kernel<uint16_t><<<dim3(blocks_for(total)), dim3(256), 0, ctx().stream>>>(
        static_cast<float*>(qkv), pbq, pbk, static_cast<const float*>(bv), static_cast<uint16_t*>(Kc),
        static_cast<uint16_t*>(Vc), (int)n_q_heads, (int)n_kv_heads, (int)D, pos, kv_max, base, dp, tb);
  else
    qkv_rope_append_kernel<float><<<dim3(blocks_for(total)), dim3(256), 0, ctx().stream>>>(
        static_cast<float*>(qkv), pbq, pbk, static_cast<const float*>(bv), static_cast<float*>(Kc),
        static_cast<float*>(Vc), (int)n_q_heads, (int)n_kv_heads, (int)D, pos, kv_max, base, dp, tb);
  hipError_t e_ = hipGetLastError();
  if (e_ != hipSuccess) return hip_fail(e_, "kernel launch");
  ctx().census[TLHIP_C_ROPE]++;
  ctx().census[TLHIP_C_KV_APPEND]++;
  return TLHIP_OK;
}

int tlhip_qkv_rope_append(void* qkv, const void* bq, const void* bk, const void* bv, void* Kc,
                          void* Vc, int64_t n_q_heads, int64_t n_kv_heads, int64_t D, int64_t pos,
                          int64_t kv_max, float base, int kv_bf16) {
  TLHIP_REQUIRE_READY();
  return qkv_rope_append_launch(qkv, bq, bk, bv, Kc, Vc, n_q_heads, n_kv_heads, D, pos, kv_max, base,
                                kv_bf16, nullptr);
}

int tlhip_rope_table(void* table, int64_t D, int64_t pos, const void* d_pos, float base) {
  TLHIP_REQUIRE_READY();
  if (!table || D <= 0 || (D & 1) || D > 65536) return fail(TLHIP_EINVAL, "tlhip_rope_table: bad arguments");
  rope_table_kernel<<<dim3(blocks_for(D / 2)), dim3(256), 0, ctx().stream>>>(
      static_cast<float2*>(table), (int)D, pos, base, static_cast<const uint32_t*>(d_pos));
  hipError_t e_ = hipGetLastError();
  if (e_ != hipSuccess) return hip_fail(e_, "kernel launch");
  return TLHIP_OK;
}

int tlhip_rope_table_range(void* table, int64_t D, int64_t pos0, int64_t T, float base) {
  TLHIP_REQUIRE_READY();
  if (!table || D <= 0 || (D & 1) || D > 65536 || T <= 0 || T > 65535 || pos0 < 0)
    return fail(TLHIP_EINVAL, "tlhip_rope_table_range: bad arguments");
  rope_table_range_kernel<<<dim3(blocks_for(T * (D / 2))), dim3(256), 0, ctx().stream>>>(
      static_cast<float2*>(table), (int)D, pos0, (int)T, base);
  hipError_t e_ = hipGetLastError();
  if (e_ != hipSuccess) return hip_fail(e_, "kernel launch");
  return TLHIP_OK;
}

int tlhip_qkv_rope_fill(const void* qkv, const void* bq, const void* bk, const void* bv, const void* table,
                        void* qh, void* Kc, void* Vc, int64_t T, int64_t n_q_heads, int64_t n_kv_heads,
                        int64_t D, int64_t pos0, int64_t kv_max, int kv_bf16) {
  return tlhip_qkv_rope_fill_parts(qkv, 1, bq, bk, bv, table, qh, Kc, Vc, T, n_q_heads, n_kv_heads, D, pos0,
                                   kv_max, kv_bf16);
}

int tlhip_qkv_rope_fill_parts(const void* qkv, int64_t n_parts, const void* bq, const void* bk,
                              const void* bv, const void* table, void* qh, void* Kc, void* Vc, int64_t T,
                              int64_t n_q_heads, int64_t n_kv_heads, int64_t D, int64_t pos0,
                              int64_t kv_max, int kv_bf16) {
  TLHIP_REQUIRE_READY();
  if (n_parts <= 0 || n_parts > 64) return fail(TLHIP_EUNSUPPORTED, "tlhip_qkv_rope_fill: need 1 <= n_parts <= 64");
  if (!qkv || !table || !qh || !Kc || !Vc) return fail(TLHIP_EINVAL, "tlhip_qkv_rope_fill: null pointer");
  if (T <= 0 || T > 65535 || n_q_heads <= 0 || n_kv_heads <= 0 || n_q_heads > 65535 || n_kv_heads > 65535)
    return fail(TLHIP_EUNSUPPORTED, "tlhip_qkv_rope_fill: bad shape");
  if (D != 64 && D != 128) return fail(TLHIP_EUNSUPPORTED, "tlhip_qkv_rope_fill: head_dim must be 64 or 128");   // the cache ops' gate
  if (pos0 < 0 || pos0 + T > kv_max) return fail(TLHIP_EINVAL, "tlhip_qkv_rope_fill: need 0 <= pos0, pos0 + T <= kv_max");
  if (!aligned16(qkv) || !aligned16(qh) || !aligned16(Kc) || !aligned16(Vc) || (bq && !aligned16(bq)) ||
      (bk && !aligned16(bk)) || (bv && !aligned16(bv)) || !aligned16(table))
    return fail(TLHIP_EINVAL, "tlhip_qkv_rope_fill: operands must be 16-byte aligned");
  const int Hq = (int)n_q_heads, Hkv = (int)n_kv_heads;
  const int64_t total = T * ((int64_t)(Hq + Hkv) * (D / 8) + (int64_t)Hkv * (D / 4));
#define TLHIP_FILL(KT_)                                                                              \
  qkv_rope_fill_kernel<KT_><<<dim3(blocks_for(total)), dim3(256), 0, ctx().stream>>>(                \
      static_cast<const float*>(qkv), static_cast<const float*>(bq), static_cast<const float*>(bk), \
      static_cast<const float*>(bv), static_cast<const float2*>(table), static_cast<float*>(qh),    \
      static_cast<KT_*>(Kc), static_cast<KT_*>(Vc), (int)T, Hq, Hkv, (int)D, pos0, kv_max,        \
      (int)n_parts, (size_t)(T * (Hq + 2 * Hkv) * D))
  if (kv_bf16) TLHIP_FILL(uint16_t);
  else TLHIP_FILL(float);
#undef TLHIP_FILL
  TLHIP_CHECK_LAUNCH(TLHIP_C_KV_FILL);
}

int tlhip_qkv_rope_append_tab(void* qkv, const void* bq, const void* bk, const void* bv, void* Kc,
                              void* Vc, int64_t n_q_heads, int64_t n_kv_heads, int64_t D, int64_t pos,
                              const void* d_pos, int64_t kv_max, const void* table, int kv_bf16) {
  TLHIP_REQUIRE_READY();
  if (!table) return fail(TLHIP_EINVAL, "tlhip_qkv_rope_append_tab: null table");
  return qkv_rope_append_launch(qkv, bq, bk, bv, Kc, Vc, n_q_heads, n_kv_heads, D, pos, kv_max, 0.f,
                                kv_bf16, d_pos, table);
}

int tlhip_qkv_rope_append_dpos(void* qkv, const void* bq, const void* bk, const void* bv, void* Kc,
                               void* Vc, int64_t n_q_heads, int64_t n_kv_heads, int64_t D,
                               const void* d_pos, int64_t kv_max, float base, int kv_bf16) {
  TLHIP_REQUIRE_READY();
  if (!d_pos) return fail(TLHIP_EINVAL, "tlhip_qkv_rope_append_dpos: null position pointer");
  return qkv_rope_append_launch(qkv, bq, bk, bv, Kc, Vc, n_q_heads, n_kv_heads, D, 0, kv_max, base,
                                kv_bf16, d_pos);
}

int tlhip_kv_fill(void* Kc, void* Vc, const void* K, const void* V, int64_t T, int64_t kv_max,
                  int64_t n_kv_heads, int64_t D, int kv_bf16, int64_t pos0) {
  TLHIP_REQUIRE_READY();
  return kv_write(Kc, Vc, K, V, T, kv_max, n_kv_heads, D, kv_bf16, pos0, TLHIP_C_KV_FILL,
                  "tlhip_kv_fill");
}

int tlhip_split_heads(const void* src, const void* bias, void* dst, int64_t T, int64_t ld,
                      int64_t off, int64_t H, int64_t D) {
  TLHIP_REQUIRE_READY();
  if (!src || !dst) return fail(TLHIP_EINVAL, "tlhip_split_heads: null pointer");
  if (T <= 0 || H <= 0 || D <= 0) return fail(TLHIP_EUNSUPPORTED, "tlhip_split_heads: empty");  // cuda.h:851
  if (off < 0 || off + H * D > ld) return fail(TLHIP_EINVAL, "tlhip_split_heads: column block outside ld");
  const int64_t total = H * T * D;
  split_heads_kernel<<<dim3(blocks_for(total)), dim3(256), 0, ctx().stream>>>(
      static_cast<const float*>(src), static_cast<const float*>(bias), static_cast<float*>(dst), T, ld,
      off, (int)D, total);
  TLHIP_CHECK_LAUNCH(TLHIP_C_SPLIT_HEADS);
}

int tlhip_merge_heads(const void* src, void* dst, int64_t T, int64_t H, int64_t D) {
  TLHIP_REQUIRE_READY();
  if (!src || !dst) return fail(TLHIP_EINVAL, "tlhip_merge_heads: null pointer");
  if (T <= 0 || H <= 0 || D <= 0) return fail(TLHIP_EUNSUPPORTED, "tlhip_merge_heads: empty");
  const int64_t total = H * T * D;
  merge_heads_kernel<<<dim3(blocks_for(total)), dim3(256), 0, ctx().stream>>>(
      static_cast<const float*>(src), static_cast<float*>(dst), T, H, (int)D, total);
  TLHIP_CHECK_LAUNCH(TLHIP_C_MERGE_HEADS);
}

}  // extern "C"
