// C entry points over the header-only decode harness (include/tl/qwen_decode.h),
// so that tests and benchmarks written in Python can drive the C++ host layer.
// Built with plain g++ into libtl_qwen.so: it links nothing but libdl, the HIP
// library is reached through tl::hip's dlopen like any other client would.
#include <cstdint>
#include <cstring>
#include <map>
#include <string>

#include "../include/tl/qwen_decode.h"

using namespace tl;

namespace {
struct handle {
  qwen::model M;
  qwen::captured_step cap;
  std::map<std::string, const void*> pending;  // weight blobs of the layer being assembled
};
}  // namespace

extern "C" {

int tlq_available() { return hip::available() ? 1 : 0; }
const char* tlq_unavailable_reason() { return hip::unavailable_reason(); }

void* tlq_create(const qwen::dims* d) {
  auto* h = new handle();
  if (!qwen::init(h->M, *d)) {
    delete h;
    return nullptr;
  }
  return h;
}

void tlq_destroy(void* hv) { delete static_cast<handle*>(hv); }

// One layer's blobs in the reference's storage forms (q4 buffers, f32 vectors).
int tlq_set_layer_q4(void* hv, int64_t li, const uint8_t* wq, const uint8_t* wk, const uint8_t* wv,
                     const uint8_t* wo, const uint8_t* wg, const uint8_t* wu, const uint8_t* wd,
                     const float* bq, const float* bk, const float* bv, const float* an,
                     const float* fn) {
  auto* h = static_cast<handle*>(hv);
  qwen::layer_blobs b{wq, wk, wv, wo, wg, wu, wd, bq, bk, bv, an, fn};
  return qwen::set_layer_q4(h->M, li, b) ? 0 : -1;
}

int tlq_set_head_q4(void* hv, const uint16_t* embed, const float* onorm, const uint8_t* outw) {
  return qwen::set_head_q4(static_cast<handle*>(hv)->M, embed, onorm, outw) ? 0 : -1;
}

int tlq_set_random_q4(void* hv, uint32_t seed) {
  return qwen::set_random_q4(static_cast<handle*>(hv)->M, seed) ? 0 : -1;
}

int tlq_fill_cache_random(void* hv, int64_t upto, uint32_t seed) {
  return qwen::fill_cache_random(static_cast<handle*>(hv)->M, upto, seed) ? 0 : -1;
}

// Greedy step; logits_out (may be NULL) receives the [vocab] logits.
int64_t tlq_step(void* hv, int64_t token, int64_t pos, float* logits_out) {
  auto* h = static_cast<handle*>(hv);
  const int64_t id = qwen::step_greedy(h->M, token, pos);
  if (id >= 0 && logits_out)
    std::memcpy(logits_out, qwen::logits(h->M), (size_t)h->M.d.vocab * sizeof(float));
  return id;
}

// Enqueue one step's launches without the argmax and without any sync.
int tlq_run_layers(void* hv, int64_t token, int64_t pos) {
  auto* h = static_cast<handle*>(hv);
  qwen::stage_embed(h->M, token);
  return qwen::run_layers(h->M, h->M.s.embedb, pos) ? 0 : -1;
}

int64_t tlq_argmax(void* hv) {
  auto* h = static_cast<handle*>(hv);
  int64_t idx = -1;
  return hip::argmax(h->M.s.logitsb, h->M.d.vocab, &idx) ? idx : -1;
}

int tlq_capture(void* hv, int64_t token, int64_t pos) {
  auto* h = static_cast<handle*>(hv);
  qwen::stage_embed(h->M, token);
  return h->cap.capture(h->M, pos) ? 0 : -1;
}
void tlq_set_fused(void* hv, int on) { static_cast<handle*>(hv)->M.fused = on != 0; }
int tlq_replay(void* hv) { return static_cast<handle*>(hv)->cap.replay() ? 0 : -1; }
void tlq_flush() { hip::flush(); }

int tlq_census(uint64_t* out, int n) {
  auto v = hip::census();
  for (int i = 0; i < n && i < (int)v.size(); i++) out[i] = v[(size_t)i];
  return 0;
}

}  // extern "C"
