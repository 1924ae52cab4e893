// Prefill-side kernels: bf16-weight GEMM and causal attention over a chunk.
#include "common.hpp"

using namespace tlhip;

extern "C" {

int tlhip_gemm_bf16_nt(const void* A, const void* W, void* C, int64_t M, int64_t N, int64_t K) {
  (void)A; (void)W; (void)C; (void)M; (void)N; (void)K;
  return fail(TLHIP_EUNSUPPORTED, "tlhip_gemm_bf16_nt: not built yet");
}

int tlhip_attn_prefill(const void* q, const void* K, const void* V, void* out, int64_t n_q_heads,
                       int64_t n_kv_heads, int64_t T, int64_t kv_max, int64_t D, float scale,
                       int kv_bf16, int64_t pos0) {
  (void)q; (void)K; (void)V; (void)out; (void)n_q_heads; (void)n_kv_heads; (void)T; (void)kv_max;
  (void)D; (void)scale; (void)kv_bf16; (void)pos0;
  return fail(TLHIP_EUNSUPPORTED, "tlhip_attn_prefill: not built yet");
}

}  // extern "C"
