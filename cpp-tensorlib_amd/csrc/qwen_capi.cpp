// C entry points over the header-only decode harness (include/tl/qwen_decode.h),
// so that tests and benchmarks written in Python can drive the C++ host layer.
// Built with plain g++ into libtl_qwen.so: it links nothing but libdl, the HIP
// library is reached through tl::hip's dlopen like any other client would.
#include <cstdint>
#include <cstring>
#include <map>
#include <string>

#include "../include/tl/gguf_dump.h"
#include "../include/tl/qwen_decode.h"
#include "../include/tl/tokenizer.h"

using namespace tl;

namespace {
struct handle {
  qwen::model M;
  qwen::captured_step cap;
  qwen::captured_decoder dec;
  qwen::greedy_loop loop;
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

// ---- model files ------------------------------------------------------------------------------
// The last error of tlq_gguf_* / tlq_create_from_gguf on this thread ("" when none).
static thread_local std::string g_file_error;
const char* tlq_file_error() { return g_file_error.c_str(); }

// Parses a GGUF file on the host (no GPU involved). NULL on error.
void* tlq_gguf_open(const char* path) {
  g_file_error.clear();
  try {
    return new gguf::model(path);
  } catch (const std::exception& e) {
    g_file_error = e.what();
    return nullptr;
  }
}
void tlq_gguf_close(void* g) { delete static_cast<gguf::model*>(g); }
// Writes the canonical rendering (tl/gguf_dump.h) into buf (cap bytes, NUL-terminated when it
// fits) and returns its length without the NUL.
int64_t tlq_gguf_dump(void* g, char* buf, int64_t cap) {
  const std::string text = gguf_dump::render(*static_cast<gguf::model*>(g));
  if (buf && cap > (int64_t)text.size()) std::memcpy(buf, text.c_str(), text.size() + 1);
  return (int64_t)text.size();
}
// Hyperparameters a loader would use; 0 on success.
int tlq_gguf_dims(void* g, int64_t max_ctx, qwen::dims* out) {
  g_file_error.clear();
  return qwen::dims_from_gguf(*static_cast<gguf::model*>(g), max_ctx, *out, &g_file_error) ? 0 : -1;
}

// ---- tokenizer (host only) --------------------------------------------------------------------
void* tlq_tok_open(const char* path) {
  g_file_error.clear();
  try {
    return new tokenizer(std::string(path));
  } catch (const std::exception& e) {
    g_file_error = e.what();
    return nullptr;
  }
}
void tlq_tok_close(void* t) { delete static_cast<tokenizer*>(t); }
void tlq_tok_special_ids(void* t, int* bos, int* eos) {
  *bos = static_cast<tokenizer*>(t)->bos_id();
  *eos = static_cast<tokenizer*>(t)->eos_id();
}
// ids of text[0, n) into out (cap entries); returns the count, or -1 when encode throws.
int64_t tlq_tok_encode(void* t, const char* text, int64_t n, int32_t* out, int64_t cap) {
  g_file_error.clear();
  try {
    const std::vector<int> ids = static_cast<tokenizer*>(t)->encode(std::string(text, (size_t)n));
    for (size_t i = 0; i < ids.size() && (int64_t)i < cap; i++) out[i] = ids[i];
    return (int64_t)ids.size();
  } catch (const std::exception& e) {
    g_file_error = e.what();
    return -1;
  }
}
// bytes of ids[0, n) into out (cap bytes); returns the length, or -1 when decode throws.
int64_t tlq_tok_decode(void* t, const int32_t* ids, int64_t n, char* out, int64_t cap) {
  g_file_error.clear();
  try {
    const std::string s = static_cast<tokenizer*>(t)->decode(std::vector<int>(ids, ids + n));
    std::memcpy(out, s.data(), (size_t)std::min<int64_t>(cap, (int64_t)s.size()));
    return (int64_t)s.size();
  } catch (const std::exception& e) {
    g_file_error = e.what();
    return -1;
  }
}
// bit 0: letter, bit 1: number, bit 2: whitespace - the classes the pre-tokenizer uses
int tlq_unicode_class(uint32_t cp) {
  return (unicode::is_letter(cp) ? 1 : 0) | (unicode::is_number(cp) ? 2 : 0) | (unicode::is_space(cp) ? 4 : 0);
}

// A model built from a GGUF file: fmt 0 = int4 groups, 1 = bf16 rows. NULL on error.
void* tlq_create_from_gguf(const char* path, int fmt, int64_t max_ctx) {
  g_file_error.clear();
  auto* h = new handle();
  try {
    gguf::model g(path);
    if (qwen::load_gguf(h->M, g, fmt == 0 ? qwen::wfmt::q4 : qwen::wfmt::bf16_row, max_ctx, &g_file_error))
      return h;
  } catch (const std::exception& e) {
    g_file_error = e.what();
  }
  delete h;
  return nullptr;
}
void tlq_get_dims(void* hv, qwen::dims* out) { *out = static_cast<handle*>(hv)->M.d; }

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

// The same from bf16 blobs in the logical [K,N] layout.
int tlq_set_layer_bf16(void* hv, int64_t li, const uint16_t* wq, const uint16_t* wk,
                       const uint16_t* wv, const uint16_t* wo, const uint16_t* wg, const uint16_t* wu,
                       const uint16_t* wd, const float* bq, const float* bk, const float* bv,
                       const float* an, const float* fn) {
  auto* h = static_cast<handle*>(hv);
  qwen::layer_blobs_bf16 b{wq, wk, wv, wo, wg, wu, wd, bq, bk, bv, an, fn};
  return qwen::set_layer_bf16(h->M, li, b) ? 0 : -1;
}

int tlq_set_head_bf16(void* hv, const uint16_t* embed, const float* onorm, const uint16_t* outw) {
  return qwen::set_head_bf16(static_cast<handle*>(hv)->M, embed, onorm, outw) ? 0 : -1;
}

int tlq_set_random_bf16(void* hv, uint32_t seed) {
  return qwen::set_random_bf16(static_cast<handle*>(hv)->M, seed) ? 0 : -1;
}

// Consume n prompt tokens in chunks, appending to the caches at their current
// position; logits_out (may be NULL) receives the last token's [vocab] logits.
int tlq_prefill(void* hv, const int64_t* tokens, int64_t n, int64_t chunk, float* logits_out) {
  auto* h = static_cast<handle*>(hv);
  if (!qwen::prefill(h->M, tokens, n, chunk)) return -1;
  if (logits_out)
    std::memcpy(logits_out, qwen::logits(h->M), (size_t)h->M.d.vocab * sizeof(float));
  return 0;
}

// Throughput form: stage one chunk, then enqueue its layers with the caches
// rewound to pos0, no lm_head and no sync.
int tlq_stage_chunk(void* hv, const int64_t* tokens, int64_t T) {
  return qwen::stage_chunk(static_cast<handle*>(hv)->M, tokens, T) ? 0 : -1;
}
int tlq_prefill_layers(void* hv, int64_t T, int64_t pos0) {
  auto* h = static_cast<handle*>(hv);
  qwen::set_cache_pos(h->M, pos0);
  return qwen::prefill_layers(h->M, T) ? 0 : -1;
}
void tlq_set_cache_pos(void* hv, int64_t pos) { qwen::set_cache_pos(static_cast<handle*>(hv)->M, pos); }

int tlq_fill_cache_random(void* hv, int64_t upto, uint32_t seed) {
  return qwen::fill_cache_random(static_cast<handle*>(hv)->M, upto, seed) ? 0 : -1;
}

// Overwrite a layer's f32 K and V caches with host arrays [n_kv_heads, max_ctx, head_dim] and set
// every cache's position: a step or a chunk can then start deep in a context whose rows the caller
// chose.
int tlq_cache_upload(void* hv, int64_t layer, const float* K, const float* V, int64_t pos) {
  auto* h = static_cast<handle*>(hv);
  if (layer < 0 || layer >= (int64_t)h->M.layers.size()) return -1;
  hip::kv_cache& c = h->M.layers[(size_t)layer].cache;
  if (c.kv_bf16) return -1;
  const int64_t bytes = c.n_kv_heads * c.max_ctx * c.D * 4;
  hip::flush();
  if (!hip::upload_raw(c.K, K, bytes) || !hip::upload_raw(c.V, V, bytes)) return -1;
  qwen::set_cache_pos(h->M, pos);
  return 0;
}

// The last chunk's final-norm rows [T, hidden] (what the lm_head would read), copied to out.
int tlq_prefill_hidden(void* hv, float* out, int64_t T) {
  auto* h = static_cast<handle*>(hv);
  if (T <= 0 || T > h->M.ps.T) return -1;
  hip::flush();
  return hip::download_raw(out, h->M.ps.h, T * h->M.d.hidden * 4) ? 0 : -1;
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
  if (!qwen::stage_embed(h->M, token)) return -1;
  return qwen::run_layers(h->M, h->M.s.embedb, pos) ? 0 : -1;
}

// n eager steps at one position with events between the regions of the step; out[0..6] = qkv,
// attention, o-proj, gate|up, down (each per layer), LM head and the whole step, microseconds.
int tlq_profile_steps(void* hv, int64_t token, int64_t pos, int64_t n, double* out) {
  auto* h = static_cast<handle*>(hv);
  qwen::step_prof p;
  for (int64_t i = 0; i < n; i++)
    if (!qwen::profile_step(h->M, token, pos, p)) return -1;
  if (p.n == 0) return -1;
  const double per_layer = 1e3 / ((double)p.n * (double)h->M.d.n_layers), per_step = 1e3 / (double)p.n;
  out[0] = p.qkv * per_layer; out[1] = p.attn * per_layer; out[2] = p.oproj * per_layer;
  out[3] = p.gateup * per_layer; out[4] = p.down * per_layer; out[5] = p.head * per_step;
  out[6] = p.total * per_step;
  return 0;
}

int64_t tlq_argmax(void* hv) {
  auto* h = static_cast<handle*>(hv);
  int64_t idx = -1;
  return hip::argmax(h->M.s.logitsb, h->M.d.vocab, &idx) ? idx : -1;
}

int tlq_capture(void* hv, int64_t token, int64_t pos) {
  auto* h = static_cast<handle*>(hv);
  if (!qwen::stage_embed(h->M, token)) return -1;
  return h->cap.capture(h->M, pos) ? 0 : -1;
}
// A decode loop on one recorded graph with the position on the device.
int tlq_decoder_init(void* hv, int64_t first_id, int64_t pos) {
  auto* h = static_cast<handle*>(hv);
  h->dec.destroy();
  return h->dec.init(h->M, first_id, pos) ? 0 : -1;
}
int tlq_decoder_feed(void* hv, int64_t id) {
  auto* h = static_cast<handle*>(hv);
  return h->dec.feed(h->M, id) ? 0 : -1;
}
int64_t tlq_decoder_step(void* hv, int64_t id, float* logits_out) {
  auto* h = static_cast<handle*>(hv);
  const int64_t tok = h->dec.step(h->M, id);
  if (tok >= 0 && logits_out)
    std::memcpy(logits_out, qwen::logits(h->M), (size_t)h->M.d.vocab * sizeof(float));
  return tok;
}
int64_t tlq_decoder_pos(void* hv) { return static_cast<handle*>(hv)->dec.cur_pos; }
int tlq_decoder_captured(void* hv) { return static_cast<handle*>(hv)->dec.ok() ? 1 : 0; }
void tlq_decoder_sync_host_pos(void* hv) {
  auto* h = static_cast<handle*>(hv);
  h->dec.sync_host_pos(h->M);
}

// Greedy decoding with the token loop on the device.
int tlq_greedy_init(void* hv, int64_t first_id, int64_t pos) {
  auto* h = static_cast<handle*>(hv);
  h->loop.destroy();
  return h->loop.init(h->M, first_id, pos) ? 0 : -1;
}
int64_t tlq_greedy_run(void* hv, int64_t n) { return static_cast<handle*>(hv)->loop.run(n); }
// Copies the tokens generated at positions [from, from + n) into out (blocks until done).
int tlq_greedy_tokens(void* hv, int64_t from, int64_t n, int32_t* out) {
  auto* h = static_cast<handle*>(hv);
  if (from < 0 || from + n > h->loop.cur_pos) return -1;
  const int32_t* t = h->loop.tokens();
  std::memcpy(out, t + from, (size_t)n * sizeof(int32_t));
  return 0;
}
void tlq_greedy_sync_host_pos(void* hv) {
  auto* h = static_cast<handle*>(hv);
  h->loop.sync_host_pos(h->M);
}

void tlq_set_fused(void* hv, int on) { static_cast<handle*>(hv)->M.fused = on != 0; }
void tlq_set_fused_attn(void* hv, int on) { static_cast<handle*>(hv)->M.fused_attn = on != 0; }
void tlq_set_norm_images(void* hv, int on) { static_cast<handle*>(hv)->M.norm_images = on != 0; }
void tlq_set_merge_in_oproj(void* hv, int on) { static_cast<handle*>(hv)->M.merge_in_oproj = on != 0; }
void tlq_set_fused_prefill(void* hv, int on) { static_cast<handle*>(hv)->M.fused_prefill = on != 0; }
// prompt chunks of bf16 weights on their prepared f16 images (default) or on the bf16 rows
void tlq_set_prompt_f16(void* hv, int on) { static_cast<handle*>(hv)->M.prompt_f16 = on != 0; }
void tlq_set_gateup_epilogue(void* hv, int on) { static_cast<handle*>(hv)->M.gateup_epilogue = on != 0; }
void tlq_set_warm(void* hv, int blocks, int nt, int mode) {
  auto& M = static_cast<handle*>(hv)->M;
  M.warm_blocks = blocks; M.warm_nt = nt != 0; M.warm_mode = mode;
}
int tlq_replay(void* hv) { return static_cast<handle*>(hv)->cap.replay() ? 0 : -1; }
void tlq_flush() { hip::flush(); }

int tlq_census(uint64_t* out, int n) {
  auto v = hip::census();
  for (int i = 0; i < n && i < (int)v.size(); i++) out[i] = v[(size_t)i];
  return 0;
}

}  // extern "C"
