// TEST INFRASTRUCTURE. The reference's REAL decode harness (bench/cuda/qwen_model.h, unmodified:
// GGUF loading, array-path forward, imperative run_layers_, batched prefill, graph-captured
// decoder with the position on the device) compiled on top of this repository's backend. The
// harness spells its backend `tl::cuda` throughout; the one-line rename a maintainer would make
// (namespace cu = tl::hip) is done here with a macro, and the graph handle type it names gets an
// alias. Everything else - kv_cache, gemv_bf16_row, gemm_bf16_nt, rmsnorm_res, swiglu, rope(_dpos),
// attn(_dpos), argmax, capture_begin/end, graph_launch - resolves to tl::hip as is.
//
// argv[1] = a Qwen2.5-0.5B-shaped F16 GGUF file (the harness hard-codes those dimensions); the
// test writes a synthetic one. Paths compared, all on the GPU backend, with the reference's own
// bar for a decode loop (logits maxrel < 2e-3, same greedy id unless the top two are a near tie):
//   A  array path (forward(): lazy graph through the tl::gpu seam)      - the harness's oracle
//   B  imperative path (run_layers_)                                    vs A, every step
//   C  batched prefill (GEMM) + captured decoder (hipGraph, d_pos)      vs A, next-token ids
//   D  int4 MLP + int4 lm_head model, imperative                         runs on gemv_q4, stays close to A
#include <tensorlib.h>

namespace tl { namespace hip { using CUgraphExec = void*; } }
#define cuda hip
#include <qwen_model.h>
#undef cuda

#include <cmath>
#include <cstdio>
#include <vector>

namespace qm = qwenmodel;

static int failures = 0;
static void expect(bool ok, const char* what) {
  std::printf("%s  %s\n", ok ? "PASS" : "FAIL", what);
  std::fflush(stdout);
  if (!ok) failures++;
}
static double maxrel(const float* got, const float* want, int64_t n) {
  double d = 0, m = 0;
  for (int64_t i = 0; i < n; i++) {
    d = std::max(d, (double)std::fabs(got[i] - want[i]));
    m = std::max(m, (double)std::fabs(want[i]));
  }
  return d / (m + 1e-30);
}
static bool near_tie(const std::vector<float>& v) {
  float a = -INFINITY, b = -INFINITY;
  for (float x : v) {
    if (x > a) { b = a; a = x; } else if (x > b) b = x;
  }
  return a - b <= 1e-5f + 1e-4f * std::fabs(a);
}

int main(int argc, char** argv) {
  if (argc < 2) return 2;
  if (!tl::gpu_available()) {
    std::printf("no GPU backend: %s\n", tl::hip::unavailable_reason());
    return 77;
  }
  tl::use_gpu();
  qm::gg::model file(argv[1]);
  expect(qm::check_config(file), "file metadata matches the harness's dimensions");
  const int64_t P = 12, N = 24;   // prompt tokens, total steps
  std::vector<int> ids;
  uint32_t s = 2463534242u;
  for (int64_t i = 0; i < P; i++) { s ^= s << 13; s ^= s >> 17; s ^= s << 5; ids.push_back((int)(s % (uint32_t)qm::VOCAB)); }
  std::vector<std::vector<float>> A;
  {
    std::printf("building the bf16 model (reference build(): host widen/transpose/narrow, prefill warm-up)\n");
    std::fflush(stdout);
    qm::Model M = qm::build(file, tl::dtype::bf16);
    expect(M.row && M.scratch.ready, "model built in row mode, scratch ready");
    // A: array path, also the teacher for the continuation
    qm::reset_cache(M);
    for (int64_t t = 0; t < N; t++) {
      A.push_back(qm::step(M, ids[(size_t)t], t));
      if (t + 1 >= P && t + 1 < N) ids.push_back((int)qm::argmax(A.back()));
    }
    std::printf("array path: %lld steps done\n", (long long)N);
    // B: imperative path
    qm::reset_cache(M);
    double worst = 0;
    bool ids_ok = true;
    for (int64_t t = 0; t < N; t++) {
      const float* L = qm::imperative_logits(M, ids[(size_t)t], t);
      worst = std::max(worst, maxrel(L, A[(size_t)t].data(), qm::VOCAB));
      std::vector<float> v(L, L + qm::VOCAB);
      if (qm::argmax(v) != qm::argmax(A[(size_t)t]) && !near_tie(A[(size_t)t])) ids_ok = false;
    }
    std::printf("imperative vs array path: worst logits maxrel %.2e\n", worst);
    expect(worst < 2e-3 && ids_ok, "B imperative run_layers_ == array path (24 steps)");
    // C: batched prefill + captured decoder
    qm::reset_cache(M);
    qm::captured_decoder dec;
    std::vector<int> prompt(ids.begin(), ids.begin() + P);
    const int64_t next = dec.begin(M, prompt);
    expect(dec.batched, "C prompt went through the batched (GEMM) prefill");
    expect(dec.ok(), "C decode graph captured");
    expect(next == qm::argmax(A[(size_t)P - 1]) || near_tie(A[(size_t)P - 1]), "C prefill's next token == array path");
    bool graph_ok = true;
    for (int64_t t = P; t < N; t++) {
      const int64_t tok = dec.step(M, ids[(size_t)t]);
      if (tok != qm::argmax(A[(size_t)t]) && !near_tie(A[(size_t)t])) graph_ok = false;
    }
    expect(graph_ok && dec.cur_pos == N, "C captured decoder (graph replay, position on the device) == array path");
    dec.sync_host_pos(M);
    expect(M.layers[0].cache.pos == N, "C host cache position reconciled");
    dec.destroy();
  }
  {
    std::printf("building the int4 model (q4 MLP + q4 lm_head)\n");
    std::fflush(stdout);
    const std::vector<uint64_t> before = tl::hip::census();
    qm::Model M = qm::build(file, tl::dtype::bf16, /*q4_mlp=*/true, /*q4_lmhead=*/true);
    qm::reset_cache(M);
    double dot = 0, na = 0, nb = 0;
    bool finite = true;
    for (int64_t t = 0; t < 6; t++) {
      const float* L = qm::imperative_logits(M, ids[(size_t)t], t);
      for (int64_t i = 0; i < qm::VOCAB; i++) {
        if (!std::isfinite(L[i])) finite = false;
        dot += (double)L[i] * A[(size_t)t][(size_t)i];
        na += (double)L[i] * L[i];
        nb += (double)A[(size_t)t][(size_t)i] * A[(size_t)t][(size_t)i];
      }
    }
    const std::vector<uint64_t> after = tl::hip::census();
    const double cosine = dot / std::sqrt(na * nb);
    std::printf("int4 vs bf16 logits: cosine %.5f, gemv_q4 launches %lld\n", cosine, (long long)(after[8] - before[8]));
    expect(finite && cosine > 0.9 && after[8] - before[8] >= 6 * (2 * 24 + 1), "D int4 model decodes on gemv_q4 and stays close to bf16");
  }
  std::printf(failures ? "%d check(s) FAILED\n" : "ALL OK\n", failures);
  return failures ? 1 : 0;
}
