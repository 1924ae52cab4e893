// Drives the tl::hip backend header the way the reference's evaluator drives a
// backend (array.h:1470-1507 binary/unary/row launches with BYTE offsets,
// 1578-1628 the GEMV arms, 1632-1705 attention and rope, 510-533 the
// cpu_barrier / sync_to_host protocol around host reads and writes), with
// storage-like buffers obtained from alloc(bytes, &contents). Every case is
// checked against plain host loops written here. Exit status 0 = all cases ok.
//
// Built by tests/build_programs.py into tests/bin/tl_seam_check; needs a gfx950 GPU to run.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "tl/hip.h"

namespace hip = tl::hip;
using tl::hip::kop;

namespace {

int g_failed = 0, g_cases = 0;

struct buf {  // what storage::make keeps: the native handle and the host pointer
  void* native = nullptr;
  float* host = nullptr;
  int64_t n = 0;
  explicit buf(int64_t count) : n(count) { native = hip::alloc(count * 4, &host); }
  ~buf() { hip::release(native, n * 4, host); }
  // CPU reader: barrier, bring the bytes home (array.h:510-520)
  const float* read() {
    hip::cpu_barrier();
    hip::sync_to_host(native, false);
    return host;
  }
  // CPU writer (array.h:522-533)
  float* write() {
    hip::cpu_barrier();
    hip::sync_to_host(native, true);
    return host;
  }
};

uint32_t rng_state = 12345;
float rnd() {  // uniform in [-1, 1)
  rng_state ^= rng_state << 13; rng_state ^= rng_state >> 17; rng_state ^= rng_state << 5;
  return (float)(int32_t)rng_state * (1.0f / 2147483648.0f);
}
void fill(buf& b, float scale = 1.0f) {
  float* p = b.write();
  for (int64_t i = 0; i < b.n; i++) p[i] = scale * rnd();
}

bool close(float got, double want) { return std::fabs(got - want) <= 1e-5 + 1e-4 * std::fabs(want); }

void check(const char* name, bool ok) {
  g_cases++;
  if (!ok) { g_failed++; std::printf("FAILED: %s\n", name); }
  else std::printf("ok: %s\n", name);
  std::fflush(stdout);
}

template <typename F>
bool all_close(buf& got, int64_t n, F want, int64_t off = 0) {
  const float* p = got.read();
  for (int64_t i = 0; i < n; i++)
    if (!close(p[off + i], want(i))) {
      std::printf("  at %lld: got %.9g want %.9g\n", (long long)i, p[off + i], (double)want(i));
      return false;
    }
  return true;
}

}  // namespace

int main() {
  if (!hip::available()) {
    std::printf("tl::hip unavailable: %s\n", hip::unavailable_reason());
    return 2;
  }
  const auto census0 = hip::census();

  {  // elementwise on views: byte offsets and the affine epilogue (scale, offset)
    const int64_t n = 1000;
    buf a(n + 8), b(n + 16), o(n + 4);
    fill(a); fill(b);
    std::vector<float> ha(a.host, a.host + a.n), hb(b.host, b.host + b.n);
    bool ok = hip::binary(kop::mul, a.native, 8 * 4, b.native, 16 * 4, o.native, 4 * 4, n, 2.0f, 1.0f);
    ok = ok && hip::pending();  // enqueued, not drained
    ok = ok && all_close(o, n, [&](int64_t i) { return (double)(ha[8 + i] * hb[16 + i]) * 2.0 + 1.0; }, 4);
    check("binary mul on views with affine epilogue", ok);
    ok = hip::unary(kop::sigmoid, a.native, 0, o.native, 0, n, 1.0f, 0.0f);
    ok = ok && all_close(o, n, [&](int64_t i) { return 1.0 / (1.0 + std::exp(-(double)ha[i])); });
    check("unary sigmoid", ok);
    ok = hip::unary(kop::affine, a.native, 0, o.native, 0, n, -3.0f, 0.5f);
    ok = ok && all_close(o, n, [&](int64_t i) { return (double)ha[i] * -3.0 + 0.5; });
    check("unary affine", ok);
  }

  {  // coherence: a host write after a device write must reach the next kernel
    const int64_t n = 256;
    buf a(n), o(n);
    fill(a);
    bool ok = hip::unary(kop::affine, a.native, 0, a.native, 0, n, 2.0f, 0.0f);  // device owns a now
    float* w = a.write();                                                      // comes home doubled
    std::vector<float> doubled(w, w + n);
    for (int64_t i = 0; i < n; i++) w[i] += 1.0f;                               // host edit
    ok = ok && hip::unary(kop::affine, a.native, 0, o.native, 0, n, 1.0f, 0.0f);
    ok = ok && all_close(o, n, [&](int64_t i) { return (double)doubled[i] + 1.0; });
    check("host write after device write is seen by the next launch", ok);
  }

  {  // array::rmsnorm as the composition of array.h:2429-2433, all through the seam
    const int64_t rows = 3, n = 896;
    buf x(rows * n), w(n), sq(rows * n), ms(rows), inv(rows), xn(rows * n), out(rows * n);
    fill(x, 2.0f); fill(w);
    std::vector<float> hx(x.host, x.host + x.n), hw(w.host, w.host + n);
    const float eps = 1e-6f;
    bool ok = hip::binary(kop::mul, x.native, 0, x.native, 0, sq.native, 0, rows * n, 1.0f, 0.0f);
    ok = ok && hip::row_op(kop::row_sum, sq.native, 0, ms.native, 0, rows, n, 1.0f / (float)n, eps);
    ok = ok && hip::unary(kop::sqrt_, ms.native, 0, ms.native, 0, rows, 1.0f, 0.0f);
    ok = ok && hip::recip(ms.native, 0, inv.native, 0, rows, 1.0f, 0.0f);
    // x [rows,n] * inv [rows,1] : strides (n,1) and (1,0)
    ok = ok && hip::binary_bcast(kop::bmul, x.native, 0, n, 1, inv.native, 0, 1, 0, xn.native, 0, rows, n, 1.0f, 0.0f);
    // * w [1,n] : strides (0,1)
    ok = ok && hip::binary_bcast(kop::bmul, xn.native, 0, n, 1, w.native, 0, 0, 1, out.native, 0, rows, n, 1.0f, 0.0f);
    ok = ok && all_close(out, rows * n, [&](int64_t i) {
      const int64_t r = i / n;
      double s = 0;
      for (int64_t j = 0; j < n; j++) s += (double)hx[r * n + j] * hx[r * n + j];
      return hx[i] / std::sqrt(s / n + eps) * hw[i % n];
    });
    check("rmsnorm composed from seam ops", ok);
    // the fused harness op gives the same
    buf fused(rows * n);
    ok = hip::rmsnorm(x.native, w.native, fused.native, n, eps, rows);
    const float* po = out.read();
    std::vector<float> comp(po, po + rows * n);
    ok = ok && all_close(fused, rows * n, [&](int64_t i) { return (double)comp[i]; });
    check("fused rmsnorm equals the composition", ok);
    ok = hip::row_op(kop::softmax, x.native, 0, out.native, 0, rows, n, 1.0f, 0.0f);
    ok = ok && all_close(out, rows * n, [&](int64_t i) {
      const int64_t r = i / n;
      double mx = -1e30, s = 0;
      for (int64_t j = 0; j < n; j++) mx = std::max(mx, (double)hx[r * n + j]);
      for (int64_t j = 0; j < n; j++) s += std::exp(hx[r * n + j] - mx);
      return std::exp(hx[i] - mx) / s;
    });
    check("row softmax", ok);
  }

  {  // dot at M = 1: the int4 arm with the scales INSIDE the weight allocation
     // (array.h:1607-1628), and the bf16 [K,N] arm (1578-1601)
    const int64_t N = 200, K = 256;
    buf a(K), y(N);
    fill(a);
    std::vector<float> ha(a.host, a.host + K);
    const int64_t qbytes = tl::q4_bytes(N, K);
    buf wq((qbytes + 3) / 4);
    {
      uint8_t* p = reinterpret_cast<uint8_t*>(wq.write());
      for (int64_t i = 0; i < N * K / 2; i++) { rng_state ^= rng_state << 13; rng_state ^= rng_state >> 17; rng_state ^= rng_state << 5; p[i] = (uint8_t)rng_state; }
      float* sc = reinterpret_cast<float*>(p + N * K / 2);
      for (int64_t i = 0; i < N * (K / 32); i++) sc[i] = 0.005f + 0.01f * std::fabs(rnd());
    }
    std::vector<uint8_t> hq(reinterpret_cast<uint8_t*>(wq.host), reinterpret_cast<uint8_t*>(wq.host) + qbytes);
    void* scales = static_cast<char*>(wq.native) + N * K / 2;
    bool ok = hip::gemv_q4(a.native, wq.native, scales, y.native, N, K, tl::kQ4Group);
    const float* hs = reinterpret_cast<const float*>(hq.data() + N * K / 2);
    ok = ok && all_close(y, N, [&](int64_t n) {
      double s = 0;
      for (int64_t k = 0; k < K; k++) {
        const uint8_t byte = hq[(n * K + k) / 2];
        const int nib = (k & 1) ? (byte >> 4) : (byte & 15);   // even k in the low nibble
        s += (double)hs[n * (K / 32) + k / 32] * (nib - 8) * ha[k];
      }
      return s;
    });
    check("gemv_q4 with interior scale pointer", ok);
    check("gemv_q4 declines a group that does not divide K",
          !hip::gemv_q4(a.native, wq.native, scales, y.native, N, K, 48));

    buf wb((K * N + 1) / 2);  // bf16 [K,N]
    std::vector<float> hwf((size_t)(K * N));
    {
      uint16_t* p = reinterpret_cast<uint16_t*>(wb.write());
      for (int64_t i = 0; i < K * N; i++) { p[i] = tl::f32_to_bf16(0.05f * rnd()); hwf[(size_t)i] = tl::bf16_to_f32(p[i]); }
    }
    ok = hip::gemv_bf16(a.native, wb.native, y.native, N, K);
    ok = ok && all_close(y, N, [&](int64_t n) {
      double s = 0;
      for (int64_t k = 0; k < K; k++) s += (double)ha[k] * hwf[(size_t)(k * N + n)];
      return s;
    });
    check("gemv_bf16 [K,N]", ok);
  }

  {  // attn_decode over a cache prefix + rope, as array.h:1632-1705 launches them
    const int64_t Hq = 4, Hkv = 2, D = 64, ctx = 70, kvmax = 96;
    buf q(Hq * D), K(Hkv * kvmax * D), V(Hkv * kvmax * D), o(Hq * D);
    fill(q); fill(K); fill(V);
    std::vector<float> hq(q.host, q.host + q.n), hk(K.host, K.host + K.n), hv(V.host, V.host + V.n);
    const float scale = 0.125f;
    bool ok = hip::attn_decode(q.native, K.native, V.native, o.native, Hq, Hkv, ctx, kvmax, D, scale);
    ok = ok && all_close(o, Hq * D, [&](int64_t i) {
      const int64_t h = i / D, d = i % D, kv = h / (Hq / Hkv);
      std::vector<double> s((size_t)ctx);
      double mx = -1e30, sum = 0, acc = 0;
      for (int64_t j = 0; j < ctx; j++) {
        double dot = 0;
        for (int64_t e = 0; e < D; e++) dot += (double)hq[h * D + e] * hk[(kv * kvmax + j) * D + e];
        s[(size_t)j] = dot * scale;
        mx = std::max(mx, s[(size_t)j]);
      }
      for (int64_t j = 0; j < ctx; j++) { s[(size_t)j] = std::exp(s[(size_t)j] - mx); sum += s[(size_t)j]; }
      for (int64_t j = 0; j < ctx; j++) acc += s[(size_t)j] * hv[(kv * kvmax + j) * D + d];
      return acc / sum;
    });
    check("attn_decode with GQA over a cache prefix", ok);
    const int64_t pos = 1234;
    ok = hip::rope(q.native, o.native, Hq, 1, D, pos, 1e6f);
    ok = ok && all_close(o, Hq * D, [&](int64_t i) {
      const int64_t h = i / D, d = i % D, half = D / 2, j = d % half;
      const double ang = (double)pos * std::pow(1e6, -2.0 * (double)j / (double)D);
      const double x0 = hq[h * D + j], x1 = hq[h * D + j + half];
      return d < half ? x0 * std::cos(ang) - x1 * std::sin(ang) : x0 * std::sin(ang) + x1 * std::cos(ang);
    });
    check("rope", ok);
  }

  {  // a large prompt product runs on a form of the bf16 weight the header prepares once and keeps
     // with the buffer: a host edit of the weight and a device-side overwrite must both reach the
     // next product, and switching the prepared form off must give the same rows
    const int64_t m = 512, n = 1024, k = 8192;      // m * n * k = 4.3e9: large enough to be prepared
    buf a(m * k), w(n * k / 2), w2(n * k / 2), o(m * n);
    fill(a);
    auto fill_bf16 = [&](buf& b, float scale) {     // two bf16 per float slot
      uint16_t* p = reinterpret_cast<uint16_t*>(b.write());
      for (int64_t i = 0; i < n * k; i++) {
        const float v = scale * rnd();
        uint32_t u;
        std::memcpy(&u, &v, 4);
        p[i] = (uint16_t)(u >> 16);
      }
    };
    auto widen = [](uint16_t h) { const uint32_t u = (uint32_t)h << 16; float f; std::memcpy(&f, &u, 4); return f; };
    auto rows_match = [&](buf& wb, const char* what) {
      std::vector<uint16_t> hw(reinterpret_cast<const uint16_t*>(wb.host), reinterpret_cast<const uint16_t*>(wb.host) + n * k);
      std::vector<float> ha(a.host, a.host + a.n);
      const float* got = o.read();
      for (int64_t r : {int64_t(0), m / 2, m - 1})
        for (int64_t c : {int64_t(0), int64_t(17), n - 1}) {
          double want = 0;
          for (int64_t i = 0; i < k; i++) want += (double)ha[r * k + i] * (double)widen(hw[c * k + i]);
          if (!close(got[r * n + c], want)) {
            std::printf("  %s at (%lld, %lld): got %.9g want %.9g\n", what, (long long)r, (long long)c, got[r * n + c], want);
            return false;
          }
        }
      return true;
    };
    fill_bf16(w, 0.05f);
    fill_bf16(w2, 0.3f);
    bool ok = hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k) && rows_match(w, "first product");
    ok = ok && hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k) && rows_match(w, "second product (cached form)");
    reinterpret_cast<uint16_t*>(w.write())[17 * k + 5] = 0x4080;          // host edit: one weight becomes 4.0
    ok = ok && hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k) && rows_match(w, "after a host edit");
    w2.read();                                                              // keep w2's host half current for the comparison
    ok = ok && hip::copy_d2d(w.native, w2.native, n * k * 2);             // device-side overwrite
    ok = ok && hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k) && rows_match(w2, "after a device copy into the weight");
    hip::set_prompt_f16(false);
    ok = ok && hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k) && rows_match(w2, "on the bf16 rows");
    hip::set_prompt_f16(true);
    check("prepared weight follows host edits and device writes of its buffer", ok);

    // a raw upload into the weight (the loader's way of writing device bytes) drops the cached form too
    ok = hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k);          // prepares again
    std::vector<uint16_t> fresh(n * k);
    for (auto& h : fresh) { const float v = 0.11f * rnd(); uint32_t u; std::memcpy(&u, &v, 4); h = (uint16_t)(u >> 16); }
    ok = ok && hip::upload_raw(w.native, fresh.data(), n * k * 2);
    std::memcpy(w.host, fresh.data(), (size_t)n * k * 2);                    // the comparison reads the host half
    ok = ok && hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k) && rows_match(w, "after upload_raw into the weight");
    check("prepared weight follows a raw upload into its buffer", ok);

    // a recorded graph that writes the weight: every replay drops the cached form, and the
    // drop recorded while the capture was open waits for the capture's end
    ok = hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k);          // prepared form exists
    w2.read();
    ok = ok && hip::capture_begin();
    ok = ok && hip::copy_d2d(w.native, w2.native, n * k * 2);             // recorded: claims the weight, drops the form
    void* g = hip::capture_end();
    ok = ok && g != nullptr;
    ok = ok && hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k) && rows_match(w, "capture alone changes nothing");
    ok = ok && hip::graph_launch(g);
    ok = ok && hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k) && rows_match(w2, "after a replay that overwrites the weight");
    hip::graph_destroy(g);
    check("prepared weight follows a graph replay that writes its buffer", ok);

    // a weight row that spans 2^40: its image is not exact for the tiny element, and a row of A
    // that is one huge activation at that element's k makes the result that element alone
    reinterpret_cast<uint16_t*>(w.write())[3 * k + 9] = 0x2b80;             // 2^-40
    {
      float* pa = a.write();
      for (int64_t i = 0; i < k; i++) pa[(m / 2) * k + i] = 0.0f;
      pa[(m / 2) * k + 9] = 3.0e9f;
    }
    ok = hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k) && rows_match(w, "tiny weight under a huge activation");
    {
      const float got = o.read()[(m / 2) * n + 3];
      const double want = 3.0e9 * std::ldexp(1.0, -40);
      ok = ok && close(got, want) && std::fabs(got - want) <= 1e-4 * want;
      if (!ok) std::printf("  tiny weight: got %.9g want %.9g\n", got, want);
    }
    check("a weight element its f16 image cannot hold is taken from the weight itself where it shows", ok);
  }

  {  // the residual norm of a prompt chunk leaves the activation image of its output with the
     // output's buffer, and the product that follows uses it instead of cutting the rows itself:
     // a host edit or a device write of the norm's output between the two must reach the product
    const int64_t m = 512, n = 4096, k = 2048;      // m * n * k = 4.3e9: the product is prepared
    buf x(m * k), parts(2 * m * k), nw(k), xo(m * k), h(m * k), w(n * k / 2), o(m * n), other(m * k);
    fill(x); fill(parts, 0.25f); fill(other, 3.0f);
    { float* p = nw.write(); for (int64_t i = 0; i < k; i++) p[i] = 1.0f + 0.1f * rnd(); }
    uint16_t* pw = reinterpret_cast<uint16_t*>(w.write());
    for (int64_t i = 0; i < n * k; i++) { const float v = 0.05f * rnd(); uint32_t u; std::memcpy(&u, &v, 4); pw[i] = (uint16_t)(u >> 16); }
    auto rows_match = [&](const char* what) {        // o against h (read back) times w, in float64
      std::vector<float> hh(h.read(), h.read() + m * k);
      const float* got = o.read();
      for (int64_t r : {int64_t(0), m / 2, m - 1})
        for (int64_t c : {int64_t(0), int64_t(33), n - 1}) {
          double want = 0;
          for (int64_t i = 0; i < k; i++) {
            const uint32_t u = (uint32_t)reinterpret_cast<const uint16_t*>(w.host)[c * k + i] << 16;
            float f; std::memcpy(&f, &u, 4);
            want += (double)hh[r * k + i] * (double)f;
          }
          if (!close(got[r * n + c], want)) {
            std::printf("  %s at (%lld, %lld): got %.9g want %.9g\n", what, (long long)r, (long long)c, got[r * n + c], want);
            return false;
          }
        }
      return true;
    };
    auto norm = [&] { return hip::rmsnorm_res_parts(x.native, parts.native, 2, nw.native, xo.native, h.native, k, 1e-6f, m, n); };
    bool ok = norm() && hip::gemm_bf16_nt(h.native, w.native, o.native, m, n, k) && rows_match("product after the norm");
    ok = ok && norm();
    h.write()[(m / 2) * k + 7] = 1000.0f;                                    // host edit of the norm's output
    ok = ok && hip::gemm_bf16_nt(h.native, w.native, o.native, m, n, k) && rows_match("after a host edit of the rows");
    ok = ok && norm();
    other.read();
    ok = ok && hip::copy_d2d(h.native, other.native, m * k * 4);             // device write of the norm's output
    ok = ok && hip::gemm_bf16_nt(h.native, w.native, o.native, m, n, k) && rows_match("after a device copy into the rows");
    hip::set_prompt_f16(false);
    ok = ok && norm() && hip::gemm_bf16_nt(h.native, w.native, o.native, m, n, k) && rows_match("on the bf16 rows");
    hip::set_prompt_f16(true);
    check("the norm's activation image follows host edits and device writes of the norm's output", ok);
  }

  {  // a product deeper than the prepared form goes (K > 32768) has no image and runs on the bf16 rows
    const int64_t m = 96, n = 1280, k = 32768 + 64;                          // m * n * k = 4.03e9: "large"
    buf a(m * k), w(n * k / 2), o(m * n);
    fill(a);
    uint16_t* pw = reinterpret_cast<uint16_t*>(w.write());
    for (int64_t i = 0; i < n * k; i++) { const float v = 0.05f * rnd(); uint32_t u; std::memcpy(&u, &v, 4); pw[i] = (uint16_t)(u >> 16); }
    bool ok = hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k);
    ok = ok && hip::gemm_bf16_nt(a.native, w.native, o.native, m, n, k);
    const float* got = o.read();
    for (int64_t r : {int64_t(0), m - 1})
      for (int64_t c : {int64_t(0), n - 1}) {
        double want = 0;
        for (int64_t i = 0; i < k; i++) {
          const uint32_t u = (uint32_t)reinterpret_cast<const uint16_t*>(w.host)[c * k + i] << 16;
          float f; std::memcpy(&f, &u, 4);
          want += (double)a.host[r * k + i] * (double)f;
        }
        ok = ok && close(got[r * n + c], want);
      }
    check("a prompt product deeper than the prepared form runs on the bf16 rows", ok);
  }

  {  // pool: a released buffer comes back for the same size, contents pointer included
    float* h1 = nullptr;
    void* n1 = hip::alloc(4096, &h1);
    hip::release(n1, 4096, h1);
    float* h2 = nullptr;
    void* n2 = hip::alloc(4096, &h2);
    check("release recycles into the size-keyed pool", n1 == n2 && h1 == h2);
    hip::release(n2, 4096, h2);
  }

  const auto census1 = hip::census();
  uint64_t launches = 0;
  for (size_t i = 0; i < census1.size(); i++) launches += census1[i] - census0[i];
  check("kernels were launched (census moved)", launches >= 15);
  std::printf("seam check: %d cases, %d failed\n", g_cases, g_failed);
  return g_failed ? 1 : 0;
}
