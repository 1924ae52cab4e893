#pragma once

// Storage dtypes, the int4/bf16 formats and the process-wide device switch of
// the cpp-tensorlib array API, as this host layer sees them. Semantics follow
// the reference's include/types.h (dtype: 20; q4 layout: 25-31; bf16 RNE: 35-46;
// device switch: 48-54; auto thresholds: 67-149; batch bias: 161-191); the
// auto-mode numbers are an MI355X arm of their own.

#include <cstdint>
#include <cstdlib>
#include <cstring>

namespace tl {

// Compute is f32 everywhere. bf16 and q4 are weight STORAGE types: the decode
// GEMV reads them natively, every other op widens them to an f32 copy first.
enum class dtype : uint8_t { f32, bf16, q4 };

inline int64_t dtype_size(dtype dt) { return dt == dtype::bf16 ? 2 : 4; }

// q4: logical [K,N] weight stored as one buffer
//   [ packed int4, row-major [N][K/2], even k in the low nibble | f32 scales [N][K/32] ]
// value(k,n) = scale[n][k/32] * (nibble - 8).
inline constexpr int64_t kQ4Group = 32;
inline int64_t q4_bytes(int64_t N, int64_t K) { return N * K / 2 + N * (K / kQ4Group) * 4; }

// bf16 = the top 16 bits of the f32 pattern; narrowing rounds to nearest even.
inline uint16_t f32_to_bf16(float f) {
  uint32_t bits;
  std::memcpy(&bits, &f, sizeof bits);
  bits += 0x7fffu + ((bits >> 16) & 1u);
  return static_cast<uint16_t>(bits >> 16);
}
inline float bf16_to_f32(uint16_t h) {
  const uint32_t bits = static_cast<uint32_t>(h) << 16;
  float f;
  std::memcpy(&f, &bits, sizeof f);
  return f;
}

// IEEE half -> float, exact for every bit pattern (model files store f16): a subnormal
// is mantissa * 2^-24, a NaN keeps its payload.
inline float f16_to_f32(uint16_t h) {
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16, exp = (h >> 10) & 31u, man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    const float sub = static_cast<float>(man) * 5.9604644775390625e-8f;   // exact, and a normal f32
    std::memcpy(&bits, &sub, sizeof bits);
  } else if (exp == 31) {
    bits = 0x7f800000u | (man << 13);
  } else {
    bits = ((exp + 112u) << 23) | (man << 13);
  }
  bits |= sign;
  float f;
  std::memcpy(&f, &bits, sizeof f);
  return f;
}

enum class device_type { cpu, gpu, auto_ };
inline device_type device_ = device_type::cpu;
inline void use_cpu() { device_ = device_type::cpu; }
inline void use_gpu() { device_ = device_type::gpu; }
inline void use_auto() { device_ = device_type::auto_; }

// Test/benchmark switch: false routes CPU evaluation through the plain
// reference loops only (no blocked GEMM), so a backend can be compared with
// them in-process.
inline bool use_accelerate_ = true;

enum class kernel_class { elementwise, reduction, matmul };

// auto_ mode: the op size from which GPU-total (single op + flush) beats the CPU path.
// MI355X census with the reference's own tool (misc/census.cpp compiled against this backend,
// host = the GPU box's Xeon cores, CPU side = the reference's blocked SGEMM / loops); a
// launch plus a flush costs ~12 us here:
//   matmul      64^3 = 2.6e5 already GPU (0.022 vs cpu 0.035 ms), 512^3 0.091 vs 0.446 ms:
//               the crossover lies at or below the smallest measured size.
//   elementwise 16K cpu (0.004 vs 0.012 ms), 64K GPU (0.012 vs 0.014), 256K 0.012 vs 0.055
//               -> ~5e4.
//   reduction   softmax 64x256 = 16K already GPU (0.013 vs 0.054 ms): GPU from the smallest
//               measured size.
inline int64_t auto_threshold_(kernel_class kc) {
  switch (kc) {
    case kernel_class::matmul: return 200'000;        // ~58^3; GPU by 64^3
    case kernel_class::elementwise: return 50'000;    // cpu at 16K, GPU from 64K
    case kernel_class::reduction: return 16'000;      // GPU from ~16K
  }
  return INT64_MAX;
}

// auto_ mode, whole-batch bias: when the summed M*N*K of the dots in one
// evaluation batch crosses this, every op of the batch goes to the GPU so the
// pipeline is not broken by small ops. TL_BATCH_MATMUL_BIAS overrides.
inline int64_t batch_matmul_bias_threshold_() {
  static const int64_t v = [] {
    if (const char* e = std::getenv("TL_BATCH_MATMUL_BIAS")) {
      char* end = nullptr;
      const long long x = std::strtoll(e, &end, 10);
      if (end != e && x > 0) return static_cast<int64_t>(x);
    }
    return static_cast<int64_t>(1'000'000);
  }();
  return v;
}

}  // namespace tl
