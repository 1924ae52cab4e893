#pragma once

// tl::hip — the MI355X (gfx950) backend header for cpp-tensorlib's tl::gpu seam.
//
// It exposes the free-function set every backend of the reference exposes
// (reference include/gpu.h:1-12; signatures as include/cuda.h:494-506, 586-675,
// 719-742, 886-905, 962-1009, 1203-1222, 1487-1503 and the stubs of
// include/metal.h:434-484), plus the harness-level calls of include/cuda.h
// (gemv_bf16_row, gemm_bf16_nt, rmsnorm, rmsnorm_res, swiglu, argmax,
// split/merge_heads, kv_append, kv_fill, attn_prefill, kv_cache, upload,
// graph capture). array.h / storage.h call it as tl::gpu::X after
// `namespace gpu = hip;`.
//
// Unlike cuda.h, which dlopens the driver and loads an embedded PTX blob, this
// header dlopens ONE shared object, libtensorlib_hip.so, that holds the gfx950
// code objects and a plain C ABI (include/tensorlib_hip.h). What stays here is
// the host policy the reference keeps in its backend header: a ledger of buffers
// with a device half and a pinned host half and a note of which one is current,
// reuse of idle buffers by size, the `pending` flag, and turning every refusal of the library into the seam's
// "declined" (`false` / nullptr) so the evaluator takes its CPU path. No
// exception and no error code crosses the seam.
//
// Header-only C++17, single-threaded use like the rest of the evaluator.

#include <dlfcn.h>

#include <cstdint>
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "types.h"

namespace tl {

// The op enum all backends share. The reference declares it in metal.h:41-47
// as tl::metal::kop; a build that includes that header picks it up, a
// standalone build of this host layer gets the identical enumerator order.
#ifndef TL_HIP_USE_METAL_KOP
namespace metal {
enum class kop {
  add, sub, mul, div, pow_, exp_, log_, sqrt_, sigmoid, relu, affine,
  badd, bsub, bmul, bdiv, bpow,
  sgemm32, sgemm32x64, sgemm64x32, sgemm64,
  steel, steel32x64, steel_ta, steel_tb, steel32x64_ta, steel32x64_tb,
  softmax, row_sum, row_max
};
}  // namespace metal
#endif

namespace hip {

using kop = tl::metal::kop;

// ---- the C ABI, bound by name ------------------------------------------------
struct api {
  int (*init)(int) = nullptr;
  int (*abi_version)() = nullptr;
  const char* (*last_error)() = nullptr;
  int (*malloc_)(void**, size_t) = nullptr;
  int (*free_)(void*) = nullptr;
  int (*host_alloc)(void**, size_t) = nullptr;
  int (*host_free)(void*) = nullptr;
  int (*memcpy_h2d)(void*, const void*, size_t) = nullptr;
  int (*memcpy_d2h)(void*, const void*, size_t) = nullptr;
  int (*memcpy_h2d_async)(void*, const void*, size_t) = nullptr;
  int (*memcpy_d2d_async)(void*, const void*, size_t) = nullptr;
  int (*fill_u32)(void*, uint32_t, size_t) = nullptr;
  int (*sync)() = nullptr;
  int (*graph_begin)() = nullptr;
  int (*graph_end)(void**) = nullptr;
  int (*graph_launch)(void*) = nullptr;
  int (*graph_destroy)(void*) = nullptr;
  int (*census)(uint64_t*, int) = nullptr;
  int (*binary)(int, const void*, int64_t, const void*, int64_t, void*, int64_t, int64_t, float,
                float) = nullptr;
  int (*binary_bcast)(int, const void*, int64_t, int64_t, int64_t, const void*, int64_t, int64_t,
                      int64_t, void*, int64_t, int64_t, int64_t, float, float) = nullptr;
  int (*unary)(int, const void*, int64_t, void*, int64_t, int64_t, float, float) = nullptr;
  int (*row_op)(int, const void*, int64_t, void*, int64_t, int64_t, int64_t, float, float) = nullptr;
  int (*gemm)(const void*, int64_t, int64_t, int, const void*, int64_t, int64_t, int, void*, int64_t,
              int64_t, int64_t, int64_t, float, float) = nullptr;
  int (*gemv_f32)(const void*, const void*, void*, int64_t, int64_t) = nullptr;
  int (*gemv_bf16)(const void*, const void*, void*, int64_t, int64_t) = nullptr;
  int (*gemv_bf16_row)(const void*, const void*, void*, int64_t, int64_t) = nullptr;
  int (*gemv_q4)(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t) = nullptr;
  int (*attn_decode)(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t, int64_t,
                     int64_t, float, int) = nullptr;
  int (*attn_prefill)(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t,
                      int64_t, int64_t, float, int, int64_t) = nullptr;
  int (*kv_append)(void*, void*, const void*, const void*, int64_t, int64_t, int64_t, int64_t,
                   int) = nullptr;
  int (*kv_fill)(void*, void*, const void*, const void*, int64_t, int64_t, int64_t, int64_t, int,
                 int64_t) = nullptr;
  int (*rope)(const void*, void*, int64_t, int64_t, int64_t, int64_t, float, const void*) = nullptr;
  int (*rmsnorm)(const void*, const void*, void*, int64_t, float, int64_t) = nullptr;
  int (*rmsnorm_res)(const void*, const void*, const void*, void*, void*, int64_t, float,
                     int64_t) = nullptr;
  int (*swiglu)(const void*, void*, int64_t, int64_t) = nullptr;
  int (*argmax)(const void*, int64_t, int64_t*) = nullptr;
  int (*argmax_async)(const void*, int64_t, void*) = nullptr;
  int (*gemm_bf16_nt)(const void*, const void*, void*, int64_t, int64_t, int64_t) = nullptr;
  int (*gemm_q4_nt)(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t, int64_t) = nullptr;
  int (*gemm_q4_nt_parts)(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t, int64_t,
                          int64_t, int*) = nullptr;
  int (*gemm_q4_nt_swiglu)(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t,
                           int64_t) = nullptr;
  int (*gemm_bf16_nt_swiglu)(const void*, const void*, void*, int64_t, int64_t, int64_t) = nullptr;
  int64_t (*gemm_f16w_bytes)(int64_t, int64_t, int) = nullptr;
  int64_t (*gemm_f16w_exps_bytes)(int64_t, int) = nullptr;
  int (*gemm_f16w_prepare)(const void*, int64_t, int64_t, int, void*, void*) = nullptr;
  int (*gemm_f16w_nt)(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t) = nullptr;
  int (*gemm_f16w_nt_parts)(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t, int64_t,
                            int*) = nullptr;
  int (*gemm_f16w_nt_swiglu)(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t) = nullptr;
  int (*gemm_bf16_nt_parts)(const void*, const void*, void*, int64_t, int64_t, int64_t, int64_t,
                            int*) = nullptr;
  int (*rmsnorm_res_parts)(const void*, const void*, int64_t, const void*, void*, void*, int64_t, float,
                           int64_t) = nullptr;
  int (*split_heads)(const void*, const void*, void*, int64_t, int64_t, int64_t, int64_t,
                     int64_t) = nullptr;
  int (*merge_heads)(const void*, void*, int64_t, int64_t, int64_t) = nullptr;
  int (*qkv_rope_append)(void*, const void*, const void*, const void*, void*, void*, int64_t, int64_t,
                         int64_t, int64_t, int64_t, float, int) = nullptr;
  int (*rope_dpos)(const void*, void*, int64_t, int64_t, int64_t, const void*, float, const void*) = nullptr;
  int (*incr_u32)(void*) = nullptr;
  int (*kv_append_dpos)(void*, void*, const void*, const void*, const void*, int64_t, int64_t, int64_t,
                        int) = nullptr;
  int64_t (*attn_partials_bytes)(int64_t, int64_t, int64_t, int64_t) = nullptr;
  int (*attn_decode_dpos)(const void*, const void*, const void*, void*, int64_t, int64_t, const void*,
                          int64_t, int64_t, float, int, void*, int64_t) = nullptr;
  int (*qkv_rope_append_dpos)(void*, const void*, const void*, const void*, void*, void*, int64_t,
                              int64_t, int64_t, const void*, int64_t, float, int) = nullptr;
  int (*rope_table)(void*, int64_t, int64_t, const void*, float) = nullptr;
  int (*rope_table_range)(void*, int64_t, int64_t, int64_t, float) = nullptr;
  int (*qkv_rope_fill_parts)(const void*, int64_t, const void*, const void*, const void*, const void*, void*,
                             void*, void*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int) = nullptr;
  int (*qkv_rope_fill)(const void*, const void*, const void*, const void*, const void*, void*, void*, void*,
                       int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int) = nullptr;
  int (*attn_prefill_tok)(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t,
                          int64_t, int64_t, float, int, int64_t) = nullptr;
  int (*tune_gemv_cols)(int) = nullptr;
  int (*convert)(const void*, int, void*, int, int64_t) = nullptr;
  int (*convert_transpose)(const void*, int, void*, int, int64_t, int64_t, int64_t, int64_t) = nullptr;
  int (*quantize_q4)(const void*, int, void*, void*, int64_t, int64_t, int64_t) = nullptr;
  int (*embed_gather_f16)(const void*, const void*, void*, int64_t, int64_t) = nullptr;
  int (*attn_decode_qkv)(const void*, const void*, const void*, const void*, void*, void*, void*, int64_t,
                        int64_t, int64_t, const void*, int64_t, int64_t, float, const void*, int, void*,
                        int64_t);
  int (*qkv_rope_append_tab)(void*, const void*, const void*, const void*, void*, void*, int64_t, int64_t,
                             int64_t, int64_t, const void*, int64_t, const void*, int) = nullptr;
  int (*embed_gather_bf16)(const void*, const void*, void*, int64_t, int64_t) = nullptr;
  int (*token_advance)(void*, const void*, void*, int64_t) = nullptr;
  int (*gemv_q4_swiglu)(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t) = nullptr;
  int (*gemv_bf16_row_swiglu)(const void*, const void*, void*, int64_t, int64_t) = nullptr;
  int (*gemv_q4_rmsnorm)(const void*, const void*, const void*, void*, const void*, const void*, void*,
                         int64_t, int64_t, int64_t, float) = nullptr;
  int (*gemv_bf16_row_rmsnorm)(const void*, const void*, const void*, void*, const void*, void*,
                               int64_t, int64_t, float) = nullptr;
  int (*gemv_q4_rmsnorm_gateup)(const void*, const void*, const void*, void*, const void*, const void*,
                                void*, int64_t, int64_t, int64_t, float) = nullptr;
  int (*gemv_bf16_row_rmsnorm_gateup)(const void*, const void*, const void*, void*, const void*, void*,
                                      int64_t, int64_t, float) = nullptr;
  int64_t (*gemm_f16w_aimage_bytes)(int64_t, int64_t) = nullptr;
  int (*rmsnorm_res_parts_aimage)(const void*, const void*, int64_t, const void*, void*, void*, int64_t, float,
                                  int64_t, void*) = nullptr;
  int (*gemm_f16w_nt_aimage)(const void*, const void*, const void*, const void*, void*, int64_t, int64_t,
                             int64_t) = nullptr;
  int (*gemm_f16w_nt_parts_aimage)(const void*, const void*, const void*, const void*, void*, int64_t, int64_t,
                                   int64_t, int64_t, int*) = nullptr;
  int (*gemm_f16w_nt_swiglu_aimage)(const void*, const void*, const void*, const void*, void*, int64_t, int64_t,
                                    int64_t) = nullptr;
  int (*attn_parts_splits)(int64_t, int64_t, int64_t, int64_t, int) = nullptr;
  int (*attn_decode_qkv_parts)(const void*, const void*, const void*, const void*, void*, void*, int64_t, int64_t,
                              int64_t, const void*, int64_t, int64_t, float, const void*, void*, int64_t,
                              int*) = nullptr;
  int (*gemv_q4_attn)(const void*, int64_t, int64_t, int64_t, const void*, const void*, void*, int64_t, int64_t,
                      int64_t) = nullptr;
  int (*gemv_bf16_row_attn)(const void*, int64_t, int64_t, int64_t, const void*, void*, int64_t, int64_t) = nullptr;
  int (*warm_fork)(const void* const*, const int64_t*, int, int, int) = nullptr;
  int (*warm_join)() = nullptr;
  int (*event_create)(void**) = nullptr;
  int (*event_record)(void*) = nullptr;
  int (*event_elapsed_ms)(void*, void*, float*) = nullptr;
  int (*event_destroy)(void*) = nullptr;
};

// ---- buffer ledger ----------------------------------------------------------------
// A buffer handed to tensorlib's storage is an extent: device bytes at `base` (the handle
// storage keeps) and, unless it is device-only, a pinned host half of the same size (the
// `contents` pointer storage keeps). `live` names the half that holds the current bytes.
struct extent {
  enum class side : unsigned char { staging, device, either };
  char* base = nullptr;
  float* staging = nullptr;
  size_t size = 0;
  side live = side::staging;
  // What the library derived from a bf16 weight inside this extent for prompt-chunk products
  // (its f16 slab images and row exponents): made on the first such product, dropped as soon as
  // the extent's device bytes can change (an upload, a launch that writes it, its release).
  struct prepared {
    size_t off = 0;            // of the weight inside the extent
    int64_t n = 0, k = 0;      // rows (gated: features) and depth
    bool gated = false;
    void* image = nullptr;     // one allocation: the images, then the exponents
    void* exps = nullptr;
  };
  std::vector<prepared> derived;
  // (offset, rows, depth, gated) of weights whose preparation failed (no memory, or the library
  // refused the product): not tried again until the extent's device bytes change.
  struct unprepared { size_t off; int64_t n, k; bool gated; };
  std::vector<unprepared> refused;
  // The activation image of `rows` f32 rows of `k` at offset `off` of this extent (row exponents
  // and two f16 terms, the operand form of the prompt products over a prepared weight), written
  // by the launch that produced the rows. `valid` ends as soon as the extent's device bytes can
  // change; the allocation stays with the extent for the next producer (a layer's norm output is
  // the same buffer every layer) and goes when the extent is released.
  struct act_image {
    void* buf = nullptr;
    size_t bytes = 0, off = 0;
    int64_t rows = 0, k = 0;
    bool valid = false;
  };
  act_image act;
};

// The extents in use, ordered by base address so that an address INSIDE one (q4 scales at
// base + N*K/2, one projection of a fused weight) resolves to it, and the idle ones, filed by
// exact size. Idle extents are reused, never returned to the driver: the evaluator allocates
// the same few sizes over and over (the policy of cuda.h:211-216).
class ledger {
  std::map<uintptr_t, extent> in_use_;
  std::unordered_map<size_t, std::vector<extent>> idle_;

 public:
  extent* containing(const void* p) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    auto after = in_use_.upper_bound(a);
    if (!a || after == in_use_.begin()) return nullptr;
    extent& e = std::prev(after)->second;
    return a - reinterpret_cast<uintptr_t>(e.base) < e.size ? &e : nullptr;
  }
  extent* at_base(uintptr_t base) {
    auto it = in_use_.find(base);
    return it == in_use_.end() ? nullptr : &it->second;
  }
  bool reuse(size_t size, extent& out) {
    auto it = idle_.find(size);
    if (it == idle_.end() || it->second.empty()) return false;
    out = it->second.back();
    it->second.pop_back();
    return true;
  }
  void enter(const extent& e) { in_use_[reinterpret_cast<uintptr_t>(e.base)] = e; }
  bool leave(const void* base, extent& out) {
    auto it = in_use_.find(reinterpret_cast<uintptr_t>(base));
    if (it == in_use_.end()) return false;
    out = it->second;
    in_use_.erase(it);
    return true;
  }
  void park(const extent& e) { idle_[e.size].push_back(e); }
};

struct context {
  void* lib = nullptr;
  api f;
  bool ready = false;
  bool pending = false;
  bool capturing = false;
  // Buffers a capture recorded writes to. A replay runs no launcher, so it is
  // graph_launch that marks them device-owned again: a host reader after a replay
  // must fetch, not trust the copy it made after the previous one.
  std::vector<uintptr_t> capture_writes;
  std::unordered_map<void*, std::vector<uintptr_t>> graph_writes;
  // Images dropped while a capture is open: freeing synchronises the device, which a capture
  // forbids, so they are freed when the capture ends.
  std::vector<void*> deferred_free;
  std::string why;  // why the backend is unavailable (diagnostics only)
  // Prompt-chunk products over bf16 weights run on the library's prepared f16 form of the weight
  // (a second copy of it, made on first use). TENSORLIB_HIP_PROMPT_F16=0 keeps them on the bf16 rows.
  bool prompt_f16 = true;

  ledger buffers;   // every extent handed out, and the idle ones waiting for reuse

  static context& get() {
    static auto* c = new context();  // leaked: outlives every storage deleter
    return *c;
  }

  template <typename T>
  bool bind(T& slot, const char* name) {
    slot = reinterpret_cast<T>(dlsym(lib, name));
    if (!slot) why = std::string("missing symbol ") + name;
    return slot != nullptr;
  }

  context() {
    // TENSORLIB_HIP_LIB names the library explicitly; otherwise the usual
    // dynamic-loader search applies.
    std::vector<std::string> paths;
    if (const char* e = std::getenv("TENSORLIB_HIP_PROMPT_F16")) prompt_f16 = std::strcmp(e, "0") != 0;
    if (const char* e = std::getenv("TENSORLIB_HIP_LIB")) paths.emplace_back(e);
    paths.emplace_back("libtensorlib_hip.so");
    for (const auto& p : paths) {
      lib = dlopen(p.c_str(), RTLD_NOW | RTLD_LOCAL);
      if (lib) break;
    }
    if (!lib) {
      const char* e = dlerror();
      why = e ? e : "libtensorlib_hip.so not found";
      return;  // available() == false: every op declines, the CPU path runs
    }
    bool ok = bind(f.init, "tlhip_init") && bind(f.abi_version, "tlhip_abi_version") &&
              bind(f.last_error, "tlhip_last_error") && bind(f.malloc_, "tlhip_malloc") &&
              bind(f.free_, "tlhip_free") && bind(f.host_alloc, "tlhip_host_alloc") &&
              bind(f.host_free, "tlhip_host_free") && bind(f.memcpy_h2d, "tlhip_memcpy_h2d") &&
              bind(f.memcpy_d2h, "tlhip_memcpy_d2h") &&
              bind(f.memcpy_h2d_async, "tlhip_memcpy_h2d_async") &&
              bind(f.memcpy_d2d_async, "tlhip_memcpy_d2d_async") &&
              bind(f.fill_u32, "tlhip_fill_u32") && bind(f.sync, "tlhip_sync") &&
              bind(f.graph_begin, "tlhip_graph_begin") && bind(f.graph_end, "tlhip_graph_end") &&
              bind(f.graph_launch, "tlhip_graph_launch") &&
              bind(f.graph_destroy, "tlhip_graph_destroy") && bind(f.census, "tlhip_census") &&
              bind(f.binary, "tlhip_binary") && bind(f.binary_bcast, "tlhip_binary_bcast") &&
              bind(f.unary, "tlhip_unary") && bind(f.row_op, "tlhip_row_op") &&
              bind(f.gemm, "tlhip_gemm") && bind(f.gemv_f32, "tlhip_gemv_f32") &&
              bind(f.gemv_bf16, "tlhip_gemv_bf16") && bind(f.gemv_bf16_row, "tlhip_gemv_bf16_row") &&
              bind(f.gemv_q4, "tlhip_gemv_q4") && bind(f.attn_decode, "tlhip_attn_decode") &&
              bind(f.attn_prefill, "tlhip_attn_prefill") && bind(f.kv_append, "tlhip_kv_append") &&
              bind(f.kv_fill, "tlhip_kv_fill") && bind(f.rope, "tlhip_rope") &&
              bind(f.rmsnorm, "tlhip_rmsnorm") && bind(f.rmsnorm_res, "tlhip_rmsnorm_res") &&
              bind(f.swiglu, "tlhip_swiglu") && bind(f.argmax, "tlhip_argmax") &&
              bind(f.argmax_async, "tlhip_argmax_async") &&
              bind(f.gemm_bf16_nt, "tlhip_gemm_bf16_nt") &&
              bind(f.gemm_bf16_nt_parts, "tlhip_gemm_bf16_nt_parts") &&
              bind(f.gemm_bf16_nt_swiglu, "tlhip_gemm_bf16_nt_swiglu") &&
              bind(f.gemm_f16w_bytes, "tlhip_gemm_f16w_bytes") && bind(f.gemm_f16w_exps_bytes, "tlhip_gemm_f16w_exps_bytes") &&
              bind(f.gemm_f16w_prepare, "tlhip_gemm_f16w_prepare") &&
              bind(f.gemm_f16w_nt, "tlhip_gemm_f16w_nt") && bind(f.gemm_f16w_nt_parts, "tlhip_gemm_f16w_nt_parts") &&
              bind(f.gemm_f16w_nt_swiglu, "tlhip_gemm_f16w_nt_swiglu") &&
              bind(f.gemm_q4_nt, "tlhip_gemm_q4_nt") && bind(f.gemm_q4_nt_parts, "tlhip_gemm_q4_nt_parts") &&
              bind(f.gemm_q4_nt_swiglu, "tlhip_gemm_q4_nt_swiglu") &&
              bind(f.rmsnorm_res_parts, "tlhip_rmsnorm_res_parts") &&
              bind(f.split_heads, "tlhip_split_heads") && bind(f.merge_heads, "tlhip_merge_heads") &&
              bind(f.qkv_rope_append, "tlhip_qkv_rope_append") &&
              bind(f.rope_dpos, "tlhip_rope_dpos") && bind(f.incr_u32, "tlhip_incr_u32") &&
              bind(f.kv_append_dpos, "tlhip_kv_append_dpos") &&
              bind(f.attn_partials_bytes, "tlhip_attn_partials_bytes") &&
              bind(f.attn_decode_dpos, "tlhip_attn_decode_dpos") &&
              bind(f.qkv_rope_append_dpos, "tlhip_qkv_rope_append_dpos") &&
              bind(f.rope_table, "tlhip_rope_table") &&
              bind(f.rope_table_range, "tlhip_rope_table_range") &&
              bind(f.qkv_rope_fill, "tlhip_qkv_rope_fill") &&
              bind(f.qkv_rope_fill_parts, "tlhip_qkv_rope_fill_parts") &&
              bind(f.attn_prefill_tok, "tlhip_attn_prefill_tok") &&
              bind(f.qkv_rope_append_tab, "tlhip_qkv_rope_append_tab") &&
              bind(f.attn_decode_qkv, "tlhip_attn_decode_qkv") &&
              bind(f.tune_gemv_cols, "tlhip_tune_gemv_cols") && bind(f.convert, "tlhip_convert") && bind(f.convert_transpose, "tlhip_convert_transpose") &&
              bind(f.quantize_q4, "tlhip_quantize_q4") && bind(f.embed_gather_f16, "tlhip_embed_gather_f16") &&
              bind(f.embed_gather_bf16, "tlhip_embed_gather_bf16") &&
              bind(f.token_advance, "tlhip_token_advance") &&
              bind(f.gemv_q4_swiglu, "tlhip_gemv_q4_swiglu") &&
              bind(f.gemv_bf16_row_swiglu, "tlhip_gemv_bf16_row_swiglu") &&
              bind(f.gemv_q4_rmsnorm, "tlhip_gemv_q4_rmsnorm") &&
              bind(f.gemv_bf16_row_rmsnorm, "tlhip_gemv_bf16_row_rmsnorm") &&
              bind(f.gemv_q4_rmsnorm_gateup, "tlhip_gemv_q4_rmsnorm_gateup") &&
              bind(f.gemv_bf16_row_rmsnorm_gateup, "tlhip_gemv_bf16_row_rmsnorm_gateup") &&
              bind(f.gemm_f16w_aimage_bytes, "tlhip_gemm_f16w_aimage_bytes") &&
              bind(f.rmsnorm_res_parts_aimage, "tlhip_rmsnorm_res_parts_aimage") &&
              bind(f.gemm_f16w_nt_aimage, "tlhip_gemm_f16w_nt_aimage") &&
              bind(f.gemm_f16w_nt_parts_aimage, "tlhip_gemm_f16w_nt_parts_aimage") &&
              bind(f.gemm_f16w_nt_swiglu_aimage, "tlhip_gemm_f16w_nt_swiglu_aimage") &&
              bind(f.attn_parts_splits, "tlhip_attn_parts_splits") &&
              bind(f.attn_decode_qkv_parts, "tlhip_attn_decode_qkv_parts") &&
              bind(f.gemv_q4_attn, "tlhip_gemv_q4_attn") &&
              bind(f.gemv_bf16_row_attn, "tlhip_gemv_bf16_row_attn");
    if (!ok) return;
    bind(f.warm_fork, "tlhip_warm_fork") && bind(f.warm_join, "tlhip_warm_join");   // optional
    why.clear();
    ok = bind(f.event_create, "tlhip_event_create") && bind(f.event_record, "tlhip_event_record") &&
         bind(f.event_elapsed_ms, "tlhip_event_elapsed_ms") && bind(f.event_destroy, "tlhip_event_destroy");
    if (!ok) return;
    if (f.abi_version() != 1) {
      why = "libtensorlib_hip.so has a different ABI version";
      return;
    }
    if (f.init(0) != 0) {
      why = f.last_error();
      return;  // no gfx950 device: stay unavailable
    }
    ready = true;
  }

  // ---- keeping the two halves of an extent coherent ---------------------------------
  // The device half is about to be read by a launch: bring it up to date.
  void refresh_device(const void* p) {
    extent* e = buffers.containing(p);
    if (e && e->live == extent::side::staging) push(*e, e->size);
  }
  // The device half is about to be written by a launch (at p, possibly inside the extent).
  // A launch that starts past the extent's base may leave the bytes before it untouched, so a
  // staging-live extent is pushed whole first. Recorded while a graph capture is open.
  void claim_device(void* p) {
    extent* e = buffers.containing(p);
    if (!e) return;
    if (e->live == extent::side::staging && static_cast<char*>(p) != e->base) push(*e, e->size);
    forget_derived(*e);
    e->live = extent::side::device;
    if (capturing) capture_writes.push_back(reinterpret_cast<uintptr_t>(e->base));
  }
  // staging -> device, blocking and ordered after the queued launches
  void push(extent& e, size_t n) {
    f.memcpy_h2d(e.base, e.staging, n < e.size ? n : e.size);
    forget_derived(e);
    e.live = extent::side::either;
  }
  // The extent's device bytes are changing: what was derived from them goes. (free_ drains the
  // device first, so a queued product that still reads an image finishes with it.)
  void forget_derived(extent& e) {
    for (auto& d : e.derived) {
      if (capturing) deferred_free.push_back(d.image);
      else f.free_(d.image);
    }
    e.derived.clear();
    e.refused.clear();
    e.act.valid = false;
  }
  // Room for the activation image of the `rows` rows of `k` at `p` that a launch is about to
  // write, kept with p's extent (allocated on first use, reused afterwards). nullptr: not a
  // managed buffer, not a shape that has an image, a capture is open, or no memory.
  void* act_image_room(void* p, int64_t rows, int64_t k) {
    if (!prompt_f16 || capturing) return nullptr;
    extent* e = buffers.containing(p);
    if (!e) return nullptr;
    const int64_t bytes = f.gemm_f16w_aimage_bytes(rows, k);
    const size_t off = static_cast<size_t>(static_cast<char*>(p) - e->base);
    if (bytes <= 0 || off + static_cast<size_t>(rows * k * 4) > e->size) return nullptr;
    extent::act_image& a = e->act;
    a.valid = false;
    if (a.bytes < static_cast<size_t>(bytes)) {
      if (a.buf) f.free_(a.buf);
      a.buf = nullptr;
      a.bytes = 0;
      if (f.malloc_(&a.buf, static_cast<size_t>(bytes)) != 0) { a.buf = nullptr; return nullptr; }
      a.bytes = static_cast<size_t>(bytes);
    }
    a.off = off; a.rows = rows; a.k = k;
    return a.buf;
  }
  void act_image_made(void* p) {
    if (extent* e = buffers.containing(p)) e->act.valid = e->act.buf != nullptr;
  }
  // The image of exactly these rows, if the launch that wrote them left one and nothing has
  // written the extent since.
  const void* act_image_of(const void* p, int64_t rows, int64_t k) {
    if (!prompt_f16) return nullptr;
    extent* e = buffers.containing(p);
    if (!e || !e->act.valid) return nullptr;
    const size_t off = static_cast<size_t>(static_cast<const char*>(p) - e->base);
    return e->act.off == off && e->act.rows == rows && e->act.k == k ? e->act.buf : nullptr;
  }
  void drop_act_image(extent& e) {
    if (e.act.buf) {
      if (capturing) deferred_free.push_back(e.act.buf);
      else f.free_(e.act.buf);
    }
    e.act = extent::act_image{};
  }
  void free_deferred() {
    for (void* p : deferred_free) f.free_(p);
    deferred_free.clear();
  }
  // The prepared product over `d` was refused by the library: drop the image and do not prepare
  // this weight again (the caller runs the product on the bf16 rows).
  void refuse_prepared(void* B, const extent::prepared* d) {
    extent* e = buffers.containing(B);
    if (!e) return;
    for (size_t i = 0; i < e->derived.size(); i++)
      if (&e->derived[i] == d) {
        e->refused.push_back({d->off, d->n, d->k, d->gated});
        if (capturing) deferred_free.push_back(d->image);
        else f.free_(d->image);
        e->derived.erase(e->derived.begin() + (long)i);
        return;
      }
  }
  // The prepared form of the bf16 weight B [n, k] (gated: [2n, k], gate rows | up rows), made now
  // if this is its first prompt-chunk product. nullptr: not a managed buffer, not a shape the
  // prepared products take, no memory (remembered: not tried again until the buffer changes), or
  // a capture is open - the caller uses the bf16 rows.
  // Cost: the image is a SECOND copy of the weight (2 bytes per element plus one byte per row),
  // held until the extent's device bytes can change. The pointer returned points into the
  // extent's list and is valid only until the next call that prepares or drops a weight of the
  // same extent: use it for the one product at hand, do not keep it.
  const extent::prepared* prepared_weight(void* B, int64_t n, int64_t k, bool gated) {
    if (!prompt_f16 || capturing) return nullptr;
    extent* e = buffers.containing(B);
    if (!e) return nullptr;
    const size_t off = static_cast<size_t>(static_cast<char*>(B) - e->base);
    for (const auto& d : e->derived)
      if (d.off == off && d.n == n && d.k == k && d.gated == gated) return &d;
    for (const auto& r : e->refused)
      if (r.off == off && r.n == n && r.k == k && r.gated == gated) return nullptr;
    const int64_t rows = gated ? 2 * n : n, bytes = f.gemm_f16w_bytes(n, k, gated ? 1 : 0);
    if (bytes <= 0 || off + static_cast<size_t>(rows * k * 2) > e->size) return nullptr;
    extent::prepared d;
    d.off = off; d.n = n; d.k = k; d.gated = gated;
    if (f.malloc_(&d.image, static_cast<size_t>(bytes + f.gemm_f16w_exps_bytes(n, gated ? 1 : 0))) != 0) {
      e->refused.push_back({off, n, k, gated});
      return nullptr;
    }
    d.exps = static_cast<char*>(d.image) + bytes;
    if (f.gemm_f16w_prepare(B, n, k, gated ? 1 : 0, d.image, d.exps) != 0) {
      f.free_(d.image);
      e->refused.push_back({off, n, k, gated});
      return nullptr;
    }
    pending = true;
    e->derived.push_back(d);
    return &e->derived.back();
  }
  // device -> staging
  void pull(extent& e) {
    f.memcpy_d2h(e.staging, e.base, e.size);
    e.live = extent::side::either;
  }
};

// One submission to the library. The caller names what the call reads and writes - stale device
// halves are refreshed, written extents become device-live - and hands the library's return
// code to sent(), which also notes that work is now queued.
class launch {
  context& c_;

 public:
  const api& lib;
  const bool ok;   // false: no library or no device, the caller declines
  launch() : c_(context::get()), lib(c_.f), ok(c_.ready) {}
  template <class... P>
  void reads(P... p) { (c_.refresh_device(p), ...); }
  template <class... P>
  void writes(P... p) { (c_.claim_device(p), ...); }
  // see context::prepared_weight; call after reads() has brought the weight up to date
  const extent::prepared* prepared(void* B, int64_t n, int64_t k, bool gated) { return c_.prepared_weight(B, n, k, gated); }
  // the library refused the product over the prepared form: the caller goes on to the bf16 rows
  void refused(void* B, const extent::prepared* p) { c_.refuse_prepared(B, p); }
  // see context::act_image_room / act_image_made / act_image_of; room() after writes(), made() after a good launch
  void* act_room(void* p, int64_t rows, int64_t k) { return c_.act_image_room(p, rows, k); }
  void act_made(void* p) { c_.act_image_made(p); }
  const void* act_of(const void* p, int64_t rows, int64_t k) { return c_.act_image_of(p, rows, k); }
  bool sent(int rc) {
    if (rc != 0) return false;   // declined or failed: the caller falls back
    c_.pending = true;
    return true;
  }
};

inline bool available() { return context::get().ready; }
inline const char* unavailable_reason() { return context::get().why.c_str(); }
inline bool pending() { return context::get().pending; }

// End the batch: block until the GPU has drained (cuda.h:501-506).
inline void flush() {
  auto& c = context::get();
  if (!c.ready || !c.pending) return;
  c.f.sync();
  c.pending = false;
}

// Diagnostic knob of the reference (cuda.h:496-497): true forces the [K,N] GEMVs to run
// without K splits, false restores the built-in choice.
inline void set_no_splitk(bool v) {
  auto& c = context::get();
  if (c.ready) c.f.tune_gemv_cols(v ? 1 : 0);
}

inline void cpu_barrier() {
  if (pending()) flush();
}

// Dispatch census of the library (launches per entry point), so a caller can
// assert that a green result was computed on the GPU (webgpu.h:197-202).
inline std::vector<uint64_t> census() {
  auto& c = context::get();
  std::vector<uint64_t> v(32, 0);
  if (c.ready) c.f.census(v.data(), (int)v.size());
  return v;
}

// ---- memory: the storage hooks of the seam (cuda.h:553-637) ----------------------------
// A buffer of `bytes` bytes: returns the device handle, *contents gets the host half.
// The host half starts as the live one (storage fills it before any launch).
inline void* alloc(int64_t bytes, float** contents) {
  auto& c = context::get();
  if (!c.ready) return nullptr;
  extent e;
  e.size = bytes > 0 ? static_cast<size_t>(bytes) : 4;
  if (!c.buffers.reuse(e.size, e)) {
    void *d = nullptr, *h = nullptr;
    if (c.f.malloc_(&d, e.size) != 0) return nullptr;
    if (c.f.host_alloc(&h, e.size) != 0) {   // pinned, so both copy directions run at the link rate
      c.f.free_(d);
      return nullptr;
    }
    e.base = static_cast<char*>(d);
    e.staging = static_cast<float*>(h);
  }
  e.live = extent::side::staging;
  c.buffers.enter(e);
  if (contents) *contents = e.staging;
  return e.base;
}

// A buffer that never visits the host (weights written by device copies, KV caches): no
// host half is pinned for it and sync_to_host leaves it alone.
inline void* alloc_device(int64_t bytes) {
  auto& c = context::get();
  if (!c.ready) return nullptr;
  extent e;
  e.size = bytes > 0 ? static_cast<size_t>(bytes) : 4;
  void* d = nullptr;
  if (c.f.malloc_(&d, e.size) != 0) return nullptr;
  e.base = static_cast<char*>(d);
  e.live = extent::side::device;
  c.buffers.enter(e);
  return d;
}

// Stream-ordered device-to-device copy between two managed buffers.
inline bool copy_d2d(void* dst, const void* src, int64_t bytes) {
  launch L;
  if (!L.ok || !dst || !src || bytes < 0) return false;
  L.reads(src);
  L.writes(dst);
  return L.sent(L.lib.memcpy_d2d_async(dst, src, (size_t)bytes));
}

inline void release(void* buf, int64_t, float*) {
  auto& c = context::get();
  if (!c.ready || !buf) return;
  if (!c.buffers.at_base(reinterpret_cast<uintptr_t>(buf))) return;
  // a queued launch may still use the buffer: it may change hands only after the drain
  if (c.pending && !c.capturing) flush();
  extent e;
  c.buffers.leave(buf, e);
  c.forget_derived(e);
  c.drop_act_image(e);
  if (e.staging) c.buffers.park(e);
  else c.f.free_(e.base);   // device-only extents are not kept for reuse
}

// The host is about to read (for_write: and then modify) the buffer through its host half.
inline void sync_to_host(void* native, bool for_write) {
  auto& c = context::get();
  extent* e = c.ready ? c.buffers.containing(native) : nullptr;
  if (!e) return;
  if (c.pending) flush();
  if (!e->staging) return;
  if (e->live == extent::side::device) c.pull(*e);
  if (for_write) e->live = extent::side::staging;
}

// Blocking copy of n floats from src into the buffer, both halves (cuda.h:553-568).
inline void upload(void* native, const float* src, int64_t n) {
  auto& c = context::get();
  extent* e = c.ready ? c.buffers.containing(native) : nullptr;
  if (!e || !e->staging) return;
  const size_t nb = std::min(static_cast<size_t>(n) * sizeof(float), e->size);
  if (src != e->staging) std::memcpy(e->staging, src, nb);
  c.push(*e, nb);
}

// Blocking H2D from any host memory (pageable or a file mapping) to a device address, which
// may lie inside a managed buffer; ordered after the launches queued so far.
inline bool upload_raw(void* dst_dev, const void* src_host, int64_t bytes) {
  auto& c = context::get();
  if (!c.ready || !dst_dev || !src_host || bytes < 0) return false;
  if (bytes == 0) return true;
  if (extent* e = c.buffers.containing(dst_dev)) {
    // a managed buffer: bring a staging-live one to the device first (the copy may cover only part
    // of it), then the device half is the current one and what was derived from it is stale
    if (e->live == extent::side::staging) c.push(*e, e->size);
    c.forget_derived(*e);
    e->live = extent::side::device;
  }
  return c.f.memcpy_h2d(dst_dev, src_host, (size_t)bytes) == 0;
}

// Blocking D2H from a device address (which may lie inside a managed buffer) into any host
// memory; ordered after the launches queued so far.
inline bool download_raw(void* dst_host, const void* src_dev, int64_t bytes) {
  auto& c = context::get();
  if (!c.ready || !dst_host || !src_dev || bytes < 0) return false;
  return bytes == 0 || c.f.memcpy_d2h(dst_host, src_dev, (size_t)bytes) == 0;
}

// A 4-byte device scalar (a position, a token id) set from the host.
inline void upload_u32(void* native, unsigned val) {
  auto& c = context::get();
  extent* e = c.ready ? c.buffers.containing(native) : nullptr;
  if (!e || !e->staging || e->size < sizeof val) return;
  std::memcpy(e->staging, &val, sizeof val);
  c.push(*e, sizeof val);
}

// ---- the seam ------------------------------------------------------------------
inline bool binary(kop op, void* a, int64_t ao, void* b, int64_t bo, void* out, int64_t oo,
                   int64_t n, float scale, float offset) {
  launch L;
  if (!L.ok) return false;
  L.reads(a, b);
  L.writes(out);
  return L.sent(L.lib.binary(static_cast<int>(op), a, ao, b, bo, out, oo, n, scale, offset));
}

inline bool binary_bcast(kop op, void* a, int64_t ao, int64_t ars, int64_t acs, void* b, int64_t bo,
                         int64_t brs, int64_t bcs, void* out, int64_t oo, int64_t m, int64_t n,
                         float scale, float offset) {
  launch L;
  if (!L.ok) return false;
  L.reads(a, b);
  L.writes(out);
  return L.sent(L.lib.binary_bcast(static_cast<int>(op), a, ao, ars, acs, b, bo, brs, bcs,
                                           out, oo, m, n, scale, offset));
}

inline bool unary(kop op, void* a, int64_t ao, void* out, int64_t oo, int64_t n, float scale,
                  float offset) {
  launch L;
  if (!L.ok) return false;
  L.reads(a);
  L.writes(out);
  return L.sent(L.lib.unary(static_cast<int>(op), a, ao, out, oo, n, scale, offset));
}

// 1/x with an affine epilogue: an op the reference's seam lacks (its `recip`
// node always runs on the CPU, array.h:2064-2066); offered so a host layer that
// knows about it can keep array::rmsnorm on the device.
inline bool recip(void* a, int64_t ao, void* out, int64_t oo, int64_t n, float scale, float offset) {
  launch L;
  if (!L.ok) return false;
  L.reads(a);
  L.writes(out);
  return L.sent(L.lib.unary(64 /* TLHIP_RECIP */, a, ao, out, oo, n, scale, offset));
}

inline bool gemm(void* a, int64_t ao, int64_t lda, bool ta, void* b, int64_t bo, int64_t ldb, bool tb,
                 void* out, int64_t oo, int64_t m, int64_t n, int64_t k, float scale, float offset) {
  launch L;
  if (!L.ok) return false;
  L.reads(a, b);
  L.writes(out);
  return L.sent(L.lib.gemm(a, ao, lda, ta ? 1 : 0, b, bo, ldb, tb ? 1 : 0, out, oo, m, n, k,
                                   scale, offset));
}

inline bool row_op(kop op, void* in, int64_t io, void* out, int64_t oo, int64_t rows, int64_t cols,
                   float scale, float offset) {
  launch L;
  if (!L.ok) return false;
  L.reads(in);
  L.writes(out);
  return L.sent(L.lib.row_op(static_cast<int>(op), in, io, out, oo, rows, cols, scale, offset));
}

inline bool gemv_f32(void* a, void* B, void* y, int64_t n, int64_t k) {
  launch L;
  if (!L.ok) return false;
  L.reads(a, B);
  L.writes(y);
  return L.sent(L.lib.gemv_f32(a, B, y, n, k));
}

inline bool gemv_bf16(void* a, void* B, void* y, int64_t n, int64_t k) {
  launch L;
  if (!L.ok) return false;
  L.reads(a, B);
  L.writes(y);
  return L.sent(L.lib.gemv_bf16(a, B, y, n, k));
}

inline bool gemv_bf16_row(void* a, void* B, void* y, int64_t n, int64_t k) {
  launch L;
  if (!L.ok || (k % 8) != 0) return false;
  L.reads(a, B);
  L.writes(y);
  return L.sent(L.lib.gemv_bf16_row(a, B, y, n, k));
}

inline bool gemv_q4(void* a, void* qw, void* scales, void* y, int64_t N, int64_t K, int64_t group) {
  launch L;
  if (!L.ok || group <= 0 || (K % group) != 0 || (group % 8) != 0) return false;
  L.reads(a, qw, scales);
  L.writes(y);
  return L.sent(L.lib.gemv_q4(a, qw, scales, y, N, K, group));
}

// The prepared-weight products pay one more launch (the activation planes) and win it back on the
// matrix cores only when the product is large: measured, from about 4 * 10^9 multiply-adds on
// (512 x 4608 x 3584 gains 13 %, 512 x 896 x 4864 loses 10 %).
inline bool prompt_product_is_large(int64_t m, int64_t n, int64_t k) {
  return m > 64 && (double)m * (double)n * (double)k >= 4e9;
}

inline bool gemm_bf16_nt(void* a, void* B, void* out, int64_t m, int64_t n, int64_t k) {
  launch L;
  if (!L.ok || (k % 8) != 0 || m <= 0 || n <= 0) return false;
  L.reads(a, B);
  L.writes(out);
  if (prompt_product_is_large(m, n, k))   // on the weight's prepared f16 form where there is one
    if (const auto* p = L.prepared(B, n, k, false)) {
      const void* ai = L.act_of(a, m, k);   // the activation image a's producer left, if any
      if (L.sent(ai ? L.lib.gemm_f16w_nt_aimage(a, ai, p->image, p->exps, out, m, n, k)
                    : L.lib.gemm_f16w_nt(a, p->image, p->exps, out, m, n, k)))
        return true;
      L.refused(B, p);                    // the bf16 rows serve what the prepared product declined
    }
  return L.sent(L.lib.gemm_bf16_nt(a, B, out, m, n, k));
}

// gemm_bf16_nt + swiglu in one launch.
inline bool gemm_bf16_nt_swiglu(void* a, void* B, void* act, int64_t m, int64_t ff, int64_t k) {
  launch L;
  if (!L.ok || (k % 8) != 0 || m <= 0 || ff <= 0) return false;
  L.reads(a, B);
  L.writes(act);
  if (prompt_product_is_large(m, 2 * ff, k))
    if (const auto* p = L.prepared(B, ff, k, true)) {
      const void* ai = L.act_of(a, m, k);
      if (L.sent(ai ? L.lib.gemm_f16w_nt_swiglu_aimage(a, ai, p->image, p->exps, act, m, ff, k)
                    : L.lib.gemm_f16w_nt_swiglu(a, p->image, p->exps, act, m, ff, k)))
        return true;
      L.refused(B, p);
    }
  return L.sent(L.lib.gemm_bf16_nt_swiglu(a, B, act, m, ff, k));
}

// The prompt-chunk products over an int4 weight (packed nibbles + scales, group 32), M rows at a
// time on the matrix pipe; plain, gated and parts forms like the bf16 ones.
inline bool gemm_q4_nt(void* a, void* qw, void* scales, void* out, int64_t m, int64_t n, int64_t k,
                       int64_t group = 32) {
  launch L;
  if (!L.ok || (k % 32) != 0 || m <= 0 || n <= 0) return false;
  L.reads(a, qw);
  L.writes(out);
  return L.sent(L.lib.gemm_q4_nt(a, qw, scales, out, m, n, k, group));
}
inline bool gemm_q4_nt_swiglu(void* a, void* qw, void* scales, void* act, int64_t m, int64_t ff, int64_t k,
                              int64_t group = 32) {
  launch L;
  if (!L.ok || (k % 32) != 0 || m <= 0 || ff <= 0) return false;
  L.reads(a, qw);
  L.writes(act);
  return L.sent(L.lib.gemm_q4_nt_swiglu(a, qw, scales, act, m, ff, k, group));
}
inline bool gemm_q4_nt_parts(void* a, void* qw, void* scales, void* parts, int64_t parts_bytes, int64_t m,
                             int64_t n, int64_t k, int* n_parts, int64_t group = 32) {
  launch L;
  if (!L.ok || (k % 32) != 0 || m <= 0 || n <= 0 || !n_parts) return false;
  L.reads(a, qw);
  L.writes(parts);
  return L.sent(L.lib.gemm_q4_nt_parts(a, qw, scales, parts, parts_bytes, m, n, k, group, n_parts));
}

// The product left as its K-split parts ([*n_parts][m][n] in `parts`), for rmsnorm_res_parts.
inline bool gemm_bf16_nt_parts(void* a, void* B, void* parts, int64_t parts_bytes, int64_t m, int64_t n,
                               int64_t k, int* n_parts) {
  launch L;
  if (!L.ok || (k % 8) != 0 || m <= 0 || n <= 0 || !n_parts) return false;
  L.reads(a, B);
  L.writes(parts);
  if (prompt_product_is_large(m, n, k))
    if (const auto* p = L.prepared(B, n, k, false)) {
      const void* ai = L.act_of(a, m, k);
      if (L.sent(ai ? L.lib.gemm_f16w_nt_parts_aimage(a, ai, p->image, p->exps, parts, parts_bytes, m, n, k, n_parts)
                    : L.lib.gemm_f16w_nt_parts(a, p->image, p->exps, parts, parts_bytes, m, n, k, n_parts)))
        return true;
      L.refused(B, p);
    }
  return L.sent(L.lib.gemm_bf16_nt_parts(a, B, parts, parts_bytes, m, n, k, n_parts));
}

// Prompt-chunk products over bf16 weights (the three above, m > 64) run on the library's prepared
// f16 form of the weight, made and cached per weight on first use: `false` keeps them on the bf16
// rows (and stops new images; existing ones stay until their buffer changes).
inline void set_prompt_f16(bool on) { context::get().prompt_f16 = on; }

inline bool attn_decode(void* q, void* K, void* V, void* out, int64_t n_q_heads, int64_t n_kv_heads,
                        int64_t ctx, int64_t kv_max, int64_t D, float scale, bool kv_bf16 = false) {
  launch L;
  if (!L.ok || (D != 128 && D != 64)) return false;
  if (n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0) return false;
  L.reads(q, K, V);
  L.writes(out);
  return L.sent(L.lib.attn_decode(q, K, V, out, n_q_heads, n_kv_heads, ctx, kv_max, D, scale,
                                          kv_bf16 ? 1 : 0));
}

inline bool attn_prefill(void* q, void* K, void* V, void* out, int64_t n_q_heads, int64_t n_kv_heads,
                         int64_t T, int64_t kv_max, int64_t D, float scale, bool kv_bf16 = false,
                         int64_t pos0 = 0) {
  launch L;
  if (!L.ok || (D != 128 && D != 64)) return false;
  if (n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0) return false;
  if (T <= 0 || T > 65535) return false;
  L.reads(q, K, V);
  L.writes(out);
  return L.sent(L.lib.attn_prefill(q, K, V, out, n_q_heads, n_kv_heads, T, kv_max, D, scale,
                                           kv_bf16 ? 1 : 0, pos0));
}

inline bool kv_append(void* Kc, void* Vc, void* k_new, void* v_new, int64_t pos, int64_t kv_max,
                      int64_t n_kv_heads, int64_t D, bool kv_bf16 = false) {
  launch L;
  if (!L.ok || (D != 128 && D != 64)) return false;
  L.reads(k_new, v_new);
  L.writes(Kc, Vc);
  return L.sent(L.lib.kv_append(Kc, Vc, k_new, v_new, pos, kv_max, n_kv_heads, D,
                                        kv_bf16 ? 1 : 0));
}

inline bool kv_fill(void* Kc, void* Vc, void* K, void* V, int64_t T, int64_t kv_max,
                    int64_t n_kv_heads, int64_t D, bool kv_bf16 = false, int64_t pos0 = 0) {
  launch L;
  if (!L.ok || (D != 128 && D != 64)) return false;
  L.reads(K, V);
  L.writes(Kc, Vc);
  return L.sent(L.lib.kv_fill(Kc, Vc, K, V, T, kv_max, n_kv_heads, D, kv_bf16 ? 1 : 0, pos0));
}

inline bool rope(void* x, void* out, int64_t rows, int64_t T, int64_t D, int64_t pos, float base,
                 void* bias = nullptr) {
  launch L;
  if (!L.ok || D <= 0 || (D & 1)) return false;
  L.reads(x);
  if (bias) L.reads(bias);
  L.writes(out);
  return L.sent(L.lib.rope(x, out, rows, T, D, pos, base, bias));
}

inline bool rmsnorm(void* x, void* w, void* out, int64_t n, float eps, int64_t rows = 1) {
  launch L;
  if (!L.ok || n <= 0 || rows <= 0) return false;
  L.reads(x, w);
  L.writes(out);
  return L.sent(L.lib.rmsnorm(x, w, out, n, eps, rows));
}

inline bool rmsnorm_res(void* x, void* delta, void* w, void* xout, void* hout, int64_t n, float eps,
                        int64_t rows = 1) {
  launch L;
  if (!L.ok || n <= 0 || rows <= 0) return false;
  L.reads(x, delta, w);
  L.writes(xout, hout);
  return L.sent(L.lib.rmsnorm_res(x, delta, w, xout, hout, n, eps, rows));
}

// rmsnorm_res with delta = parts[0] + ... + parts[n_parts-1], rows * n floats apart.
// next_n: columns of the bf16 product that will consume hout (0: unknown or none). Where that
// product will run over the weight's prepared form, the norm leaves hout's activation image with
// hout's buffer and the product skips its own pass over hout (same bits either way).
inline bool rmsnorm_res_parts(void* x, void* parts, int64_t n_parts, void* w, void* xout, void* hout,
                              int64_t n, float eps, int64_t rows = 1, int64_t next_n = 0) {
  launch L;
  if (!L.ok || n <= 0 || rows <= 0 || n_parts <= 0) return false;
  L.reads(x, parts, w);
  L.writes(xout, hout);
  if (next_n > 0 && prompt_product_is_large(rows, next_n, n) && (n % 32) == 0 && n <= 8192)
    if (void* room = L.act_room(hout, rows, n)) {
      if (L.sent(L.lib.rmsnorm_res_parts_aimage(x, parts, n_parts, w, xout, hout, n, eps, rows, room))) {
        L.act_made(hout);
        return true;
      }
    }
  return L.sent(L.lib.rmsnorm_res_parts(x, parts, n_parts, w, xout, hout, n, eps, rows));
}

inline bool swiglu(void* gu, void* out, int64_t ff, int64_t rows = 1) {
  launch L;
  if (!L.ok || ff <= 0 || rows <= 0) return false;
  L.reads(gu);
  L.writes(out);
  return L.sent(L.lib.swiglu(gu, out, ff, rows));
}

// Greedy token: reduces on the device, copies 4 bytes back; the one blocking
// call of a decode step (cuda.h:1254-1282).
inline bool argmax(void* in, int64_t n, int64_t* out_idx) {
  auto& c = context::get();
  if (!c.ready || !in || n <= 0 || !out_idx) return false;
  c.refresh_device(in);
  if (c.f.argmax(in, n, out_idx) != 0) return false;
  c.pending = false;  // the library drained the stream to deliver the index
  return true;
}

inline bool split_heads(void* src, void* bias, void* dst, int64_t T, int64_t ld, int64_t off,
                        int64_t H, int64_t D) {
  launch L;
  if (!L.ok || T <= 0 || H <= 0 || D <= 0) return false;
  L.reads(src);
  if (bias) L.reads(bias);
  L.writes(dst);
  return L.sent(L.lib.split_heads(src, bias, dst, T, ld, off, H, D));
}

inline bool merge_heads(void* src, void* dst, int64_t T, int64_t H, int64_t D) {
  launch L;
  if (!L.ok || T <= 0 || H <= 0 || D <= 0) return false;
  L.reads(src);
  L.writes(dst);
  return L.sent(L.lib.merge_heads(src, dst, T, H, D));
}

// One launch for the q/k/v epilogue of a decode step: rope(q,+bq), rope(k,+bk),
// v += bv and the cache append at row pos — the four calls the reference's
// run_layers_ issues per layer (qm:703-716), fused. qkv = [q | k | v] in place.
inline bool qkv_rope_append(void* qkv, void* bq, void* bk, void* bv, void* Kc, void* Vc,
                            int64_t n_q_heads, int64_t n_kv_heads, int64_t D, int64_t pos,
                            int64_t kv_max, float base, bool kv_bf16 = false) {
  launch L;
  if (!L.ok || (D != 128 && D != 64) || pos < 0 || pos >= kv_max) return false;
  L.reads(qkv);
  if (bq) L.reads(bq);
  if (bk) L.reads(bk);
  if (bv) L.reads(bv);
  L.writes(qkv, Kc, Vc);
  return L.sent(L.lib.qkv_rope_append(qkv, bq, bk, bv, Kc, Vc, n_q_heads, n_kv_heads, D, pos,
                                              kv_max, base, kv_bf16 ? 1 : 0));
}

// ---- device-side position (cuda.h:1011-1114) ------------------------------------------
// Twins of rope / kv_append / attn_decode that take the position from a 4-byte
// device scalar `d_pos`, on grids that do not depend on it, so one recorded graph
// serves every token of a decode loop.
inline bool rope_dpos(void* x, void* out, int64_t rows, int64_t T, int64_t D, void* d_pos, float base,
                      void* bias = nullptr) {
  launch L;
  if (!L.ok || D <= 0 || (D & 1) || !d_pos) return false;
  L.reads(x);
  if (bias) L.reads(bias);
  L.reads(d_pos);
  L.writes(out);
  return L.sent(L.lib.rope_dpos(x, out, rows, T, D, d_pos, base, bias));
}
inline bool incr_u32(void* d_pos) {
  launch L;
  if (!L.ok || !d_pos) return false;
  L.reads(d_pos);
  L.writes(d_pos);
  return L.sent(L.lib.incr_u32(d_pos));
}
// Weights that launches further down the stream will stream: read them now on a second stream
// (up to four device ranges, in the order given) so that they wait in the last-level cache.
// No counterpart in the reference. warm_join makes the stream wait for the reads.
inline bool warm_fork(const void* const* ptrs, const int64_t* bytes, int n, int blocks, bool nontemporal) {
  launch L;
  if (!L.ok || !L.lib.warm_fork) return false;
  for (int i = 0; i < n; i++) L.reads(ptrs[i]);
  return L.sent(L.lib.warm_fork(ptrs, bytes, n, blocks, nontemporal ? 1 : 0));
}
inline bool warm_join() {
  launch L;
  return L.ok && L.lib.warm_join && L.sent(L.lib.warm_join());
}
inline bool kv_append_dpos(void* Kc, void* Vc, void* k_new, void* v_new, void* d_pos, int64_t kv_max,
                           int64_t n_kv_heads, int64_t D, bool kv_bf16 = false) {
  launch L;
  if (!L.ok || (D != 128 && D != 64) || !d_pos) return false;
  L.reads(k_new, v_new, d_pos);
  L.writes(Kc, Vc);
  return L.sent(L.lib.kv_append_dpos(Kc, Vc, k_new, v_new, d_pos, kv_max, n_kv_heads, D,
                                             kv_bf16 ? 1 : 0));
}
// Bytes of the caller-owned split-partials buffer attn_decode_dpos needs for a cache.
inline int64_t attn_partials_bytes(int64_t n_q_heads, int64_t n_kv_heads, int64_t kv_max, int64_t D) {
  auto& c = context::get();
  return c.ready ? c.f.attn_partials_bytes(n_q_heads, n_kv_heads, kv_max, D) : 0;
}
inline bool attn_decode_dpos(void* q, void* K, void* V, void* out, int64_t n_q_heads,
                             int64_t n_kv_heads, void* d_pos, int64_t kv_max, int64_t D, float scale,
                             void* partials, int64_t partials_bytes, bool kv_bf16 = false) {
  launch L;
  if (!L.ok || (D != 128 && D != 64) || !partials || !d_pos) return false;
  if (n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0) return false;
  L.reads(q, K, V, d_pos);
  L.writes(out, partials);
  return L.sent(L.lib.attn_decode_dpos(q, K, V, out, n_q_heads, n_kv_heads, d_pos, kv_max, D,
                                               scale, kv_bf16 ? 1 : 0, partials, partials_bytes));
}
inline bool qkv_rope_append_dpos(void* qkv, void* bq, void* bk, void* bv, void* Kc, void* Vc,
                                 int64_t n_q_heads, int64_t n_kv_heads, int64_t D, void* d_pos,
                                 int64_t kv_max, float base, bool kv_bf16 = false) {
  launch L;
  if (!L.ok || (D != 128 && D != 64) || !d_pos) return false;
  L.reads(qkv);
  if (bq) L.reads(bq);
  if (bk) L.reads(bk);
  if (bv) L.reads(bv);
  L.reads(d_pos);
  L.writes(qkv, Kc, Vc);
  return L.sent(L.lib.qkv_rope_append_dpos(qkv, bq, bk, bv, Kc, Vc, n_q_heads, n_kv_heads, D,
                                                   d_pos, kv_max, base, kv_bf16 ? 1 : 0));
}

// ---- rotary angles formed once per step -------------------------------------------------------
// All layers of a decode step rotate by the same angles: rope_table writes (cos, sin)
// for position pos (or *d_pos) once, qkv_rope_append_tab reads them instead of
// evaluating fp64 pow/cos/sin per layer. Bit-identical to qkv_rope_append.
inline bool rope_table(void* table, int64_t D, int64_t pos, void* d_pos, float base) {
  launch L;
  if (!L.ok || !table) return false;
  if (d_pos) L.reads(d_pos);
  L.writes(table);
  return L.sent(L.lib.rope_table(table, D, pos, d_pos, base));
}
inline bool qkv_rope_append_tab(void* qkv, void* bq, void* bk, void* bv, void* Kc, void* Vc,
                                int64_t n_q_heads, int64_t n_kv_heads, int64_t D, int64_t pos,
                                void* d_pos, int64_t kv_max, void* table, bool kv_bf16 = false) {
  launch L;
  if (!L.ok || (D != 128 && D != 64) || !table) return false;
  if (!d_pos && (pos < 0 || pos >= kv_max)) return false;
  L.reads(qkv);
  if (bq) L.reads(bq);
  if (bk) L.reads(bk);
  if (bv) L.reads(bv);
  if (d_pos) L.reads(d_pos);
  L.reads(table);
  L.writes(qkv, Kc, Vc);
  return L.sent(L.lib.qkv_rope_append_tab(qkv, bq, bk, bv, Kc, Vc, n_q_heads, n_kv_heads, D, pos,
                                                  d_pos, kv_max, table, kv_bf16 ? 1 : 0));
}

// The same for a prompt chunk: rope_table_range writes the angles of positions pos0 .. pos0+T-1
// once per chunk; qkv_rope_fill takes the raw token-major [T, (Hq + 2 Hkv) D] projection, adds the
// biases, rotates q and k, writes q head-major into qh [Hq, T, D] and k, v into cache rows
// pos0 .. pos0+T-1 (one launch for split_heads + 2 x rope + kv_fill; bit-identical to them).
inline bool rope_table_range(void* table, int64_t D, int64_t pos0, int64_t T, float base) {
  launch L;
  if (!L.ok || !table) return false;
  L.writes(table);
  return L.sent(L.lib.rope_table_range(table, D, pos0, T, base));
}
// n_parts > 1: qkv is the projection's K-split parts (gemm_bf16_nt_parts), summed as they are read.
inline bool qkv_rope_fill(void* qkv, void* bq, void* bk, void* bv, void* table, void* qh, void* Kc,
                          void* Vc, int64_t T, int64_t n_q_heads, int64_t n_kv_heads, int64_t D,
                          int64_t pos0, int64_t kv_max, bool kv_bf16 = false, int64_t n_parts = 1) {
  launch L;
  if (!L.ok || !table || (D != 128 && D != 64) || pos0 < 0 || pos0 + T > kv_max || n_parts <= 0) return false;
  L.reads(qkv);
  if (bq) L.reads(bq);
  if (bk) L.reads(bk);
  if (bv) L.reads(bv);
  L.reads(table);
  L.writes(qh, Kc, Vc);
  return L.sent(L.lib.qkv_rope_fill_parts(qkv, n_parts, bq, bk, bv, table, qh, Kc, Vc, T, n_q_heads,
                                                  n_kv_heads, D, pos0, kv_max, kv_bf16 ? 1 : 0));
}
// attn_prefill with the result written token-major, [T, Hq*D] (no merge_heads afterwards).
inline bool attn_prefill_tok(void* q, void* K, void* V, void* out, int64_t n_q_heads, int64_t n_kv_heads,
                             int64_t T, int64_t kv_max, int64_t D, float scale, bool kv_bf16 = false,
                             int64_t pos0 = 0) {
  launch L;
  if (!L.ok || (D != 128 && D != 64)) return false;
  if (n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0) return false;
  if (T <= 0 || T > 65535) return false;
  L.reads(q, K, V);
  L.writes(out);
  return L.sent(L.lib.attn_prefill_tok(q, K, V, out, n_q_heads, n_kv_heads, T, kv_max, D, scale,
                                               kv_bf16 ? 1 : 0, pos0));
}

// Bias + rotation of the raw [q|k|v] projection, the cache append and the attention over
// keys [0, pos] in one launch (plus the split merge). qkv itself is left untouched.
inline bool attn_decode_qkv(void* qkv, void* bq, void* bk, void* bv, void* Kc, void* Vc, void* out,
                            int64_t n_q_heads, int64_t n_kv_heads, int64_t pos, void* d_pos,
                            int64_t kv_max, int64_t D, float scale, void* table, void* partials,
                            int64_t partials_bytes, bool kv_bf16 = false) {
  launch L;
  if (!L.ok || (D != 128 && D != 64) || !table) return false;
  if (n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0) return false;
  if (d_pos ? !partials : (pos < 0 || pos >= kv_max)) return false;
  L.reads(qkv);
  if (bq) L.reads(bq);
  if (bk) L.reads(bk);
  if (bv) L.reads(bv);
  if (d_pos) L.reads(d_pos);
  L.reads(table);
  L.writes(Kc, Vc, out);
  if (partials) L.writes(partials);
  return L.sent(L.lib.attn_decode_qkv(qkv, bq, bk, bv, Kc, Vc, out, n_q_heads, n_kv_heads, pos,
                                              d_pos, kv_max, D, scale, table, kv_bf16 ? 1 : 0, partials,
                                              partials_bytes));
}

// attn_decode_qkv with the split merge left to the o-projection (gemv_*_attn): writes the cache row
// and `partials` (n_parts splits, also when that is 1), no `out`. attn_parts_splits says whether a
// shape is served (0: it is not) for a grid planned for plan_ctx keys.
inline int attn_parts_splits(int64_t n_q_heads, int64_t n_kv_heads, int64_t plan_ctx, int64_t D, bool kv_bf16 = false) {
  auto& c = context::get();
  return c.ready ? c.f.attn_parts_splits(n_q_heads, n_kv_heads, plan_ctx, D, kv_bf16 ? 1 : 0) : 0;
}
inline bool attn_decode_qkv_parts(void* qkv, void* bq, void* bk, void* bv, void* Kc, void* Vc, int64_t n_q_heads,
                                  int64_t n_kv_heads, int64_t pos, void* d_pos, int64_t kv_max, int64_t D,
                                  float scale, void* table, void* partials, int64_t partials_bytes, int* n_parts) {
  launch L;
  if (!L.ok || (D != 128 && D != 64) || !table || !partials || !n_parts) return false;
  if (n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0) return false;
  if (!d_pos && (pos < 0 || pos >= kv_max)) return false;
  L.reads(qkv);
  if (bq) L.reads(bq);
  if (bk) L.reads(bk);
  if (bv) L.reads(bv);
  if (d_pos) L.reads(d_pos);
  L.reads(table);
  L.writes(Kc, Vc, partials);
  return L.sent(L.lib.attn_decode_qkv_parts(qkv, bq, bk, bv, Kc, Vc, n_q_heads, n_kv_heads, pos, d_pos, kv_max, D,
                                            scale, table, partials, partials_bytes, n_parts));
}

// ---- load-time weight conversion on the device ---------------------------------------------
// The file's element types as the converters number them.
enum class elem : int { f32 = 0, f16 = 1, bf16 = 2 };
// dst[i] = narrow(widen(src[i])): file rows [out, in] into bf16 (or f32) rows [N, K].
inline bool convert(void* src, elem st, void* dst, elem dt, int64_t n) {
  launch L;
  if (!L.ok || !src || !dst || n <= 0) return false;
  L.reads(src);
  L.writes(dst);
  return L.sent(L.lib.convert(src, (int)st, dst, (int)dt, n));
}
// file rows [out = rows, in = cols] into the seam's [K, N] layout at columns [col_base, col_base + rows)
inline bool convert_transpose(void* src, elem st, void* dst, elem dt, int64_t rows, int64_t cols,
                              int64_t ld_dst, int64_t col_base) {
  launch L;
  if (!L.ok || !src || !dst) return false;
  L.reads(src);
  L.writes(dst);
  return L.sent(L.lib.convert_transpose(src, (int)st, dst, (int)dt, rows, cols, ld_dst, col_base));
}
// array::to_q4 of the widened rows, written into the packed and scale sections given
inline bool quantize_q4(void* src, elem st, void* packed, void* scales, int64_t rows, int64_t K) {
  launch L;
  if (!L.ok || !src || !packed || !scales) return false;
  L.reads(src);
  L.writes(packed);
  return L.sent(L.lib.quantize_q4(src, (int)st, packed, scales, rows, K, kQ4Group));
}
inline bool embed_gather_f16(void* table, void* d_token, void* out, int64_t hidden, int64_t vocab) {
  launch L;
  if (!L.ok) return false;
  L.reads(table, d_token);
  L.writes(out);
  return L.sent(L.lib.embed_gather_f16(table, d_token, out, hidden, vocab));
}

// ---- device-resident greedy loop -----------------------------------------------------------
// The next token never visits the host: the embedding row of *d_token (a device
// int32, what argmax_async wrote) is gathered on the device, and the step's tail
// appends the token to a device history and advances the position.
inline bool embed_gather_bf16(void* table, void* d_token, void* out, int64_t hidden, int64_t vocab) {
  launch L;
  if (!L.ok) return false;
  L.reads(table, d_token);
  L.writes(out);
  return L.sent(L.lib.embed_gather_bf16(table, d_token, out, hidden, vocab));
}
inline bool argmax_async(void* in, int64_t n, void* d_token) {
  launch L;
  if (!L.ok || !d_token) return false;
  L.reads(in);
  L.writes(d_token);
  return L.sent(L.lib.argmax_async(in, n, d_token));
}
inline bool token_advance(void* d_pos, void* d_token, void* history, int64_t capacity) {
  launch L;
  if (!L.ok || !d_pos || !d_token) return false;
  L.reads(d_pos, d_token);
  L.writes(d_pos);
  if (history) L.writes(history);
  return L.sent(L.lib.token_advance(d_pos, d_token, history, capacity));
}

// GEMVs that evaluate the producer of their activation vector while staging it:
// swiglu(gu) -> GEMV and rmsnorm_res(x, delta) -> GEMV in one launch each. They
// decline (false) on shapes the fused kernel does not take; the caller then
// issues the two separate calls.
inline bool gemv_q4_swiglu(void* gu, void* qw, void* scales, void* y, int64_t N, int64_t K,
                           int64_t group) {
  launch L;
  if (!L.ok || group != 32 || (K % 32) != 0) return false;
  L.reads(gu, qw, scales);
  L.writes(y);
  return L.sent(L.lib.gemv_q4_swiglu(gu, qw, scales, y, N, K, group));
}
inline bool gemv_bf16_row_swiglu(void* gu, void* B, void* y, int64_t n, int64_t k) {
  launch L;
  if (!L.ok || (k % 8) != 0) return false;
  L.reads(gu, B);
  L.writes(y);
  return L.sent(L.lib.gemv_bf16_row_swiglu(gu, B, y, n, k));
}
// y = W . (the decode attention's output merged from the n_parts split partials of attn_decode_qkv_parts)
inline bool gemv_q4_attn(void* parts, int64_t n_parts, int64_t heads, int64_t head_dim, void* qw, void* scales,
                         void* y, int64_t N, int64_t K, int64_t group) {
  launch L;
  if (!L.ok || group != 32 || (K % 32) != 0 || heads * head_dim != K) return false;
  L.reads(parts, qw, scales);
  L.writes(y);
  return L.sent(L.lib.gemv_q4_attn(parts, n_parts, heads, head_dim, qw, scales, y, N, K, group));
}
inline bool gemv_bf16_row_attn(void* parts, int64_t n_parts, int64_t heads, int64_t head_dim, void* B, void* y,
                               int64_t n, int64_t k) {
  launch L;
  if (!L.ok || (k % 8) != 0 || heads * head_dim != k) return false;
  L.reads(parts, B);
  L.writes(y);
  return L.sent(L.lib.gemv_bf16_row_attn(parts, n_parts, heads, head_dim, B, y, n, k));
}
// s = x (+ delta); xout (optional, distinct from x and delta) receives s;
// y = W . rmsnorm(s, norm_w, eps)
inline bool gemv_q4_rmsnorm(void* x, void* delta, void* norm_w, void* xout, void* qw, void* scales,
                            void* y, int64_t N, int64_t K, int64_t group, float eps) {
  launch L;
  if (!L.ok || group != 32 || (K % 32) != 0 || (xout && (xout == x || xout == delta))) return false;
  L.reads(x);
  if (delta) L.reads(delta);
  L.reads(norm_w, qw, scales);
  if (xout) L.writes(xout);
  L.writes(y);
  return L.sent(L.lib.gemv_q4_rmsnorm(x, delta, norm_w, xout, qw, scales, y, N, K, group, eps));
}
inline bool gemv_bf16_row_rmsnorm(void* x, void* delta, void* norm_w, void* xout, void* B, void* y,
                                  int64_t n, int64_t k, float eps) {
  launch L;
  if (!L.ok || (k % 8) != 0 || (xout && (xout == x || xout == delta))) return false;
  L.reads(x);
  if (delta) L.reads(delta);
  L.reads(norm_w, B);
  if (xout) L.writes(xout);
  L.writes(y);
  return L.sent(L.lib.gemv_bf16_row_rmsnorm(x, delta, norm_w, xout, B, y, n, k, eps));
}
// The same with W = [gate rows | up rows] (N2 / 2 each) and the gated activation as the
// epilogue: act[i] = swiglu(gate_i, up_i), i < N2 / 2.
inline bool gemv_q4_rmsnorm_gateup(void* x, void* delta, void* norm_w, void* xout, void* qw, void* scales,
                                   void* act, int64_t N2, int64_t K, int64_t group, float eps) {
  launch L;
  if (!L.ok || group != 32 || (K % 32) != 0 || (N2 % 2) != 0 || (xout && (xout == x || xout == delta)))
    return false;
  L.reads(x);
  if (delta) L.reads(delta);
  L.reads(norm_w, qw, scales);
  if (xout) L.writes(xout);
  L.writes(act);
  return L.sent(L.lib.gemv_q4_rmsnorm_gateup(x, delta, norm_w, xout, qw, scales, act, N2, K, group, eps));
}
inline bool gemv_bf16_row_rmsnorm_gateup(void* x, void* delta, void* norm_w, void* xout, void* B, void* act,
                                         int64_t n2, int64_t k, float eps) {
  launch L;
  if (!L.ok || (k % 8) != 0 || (n2 % 2) != 0 || (xout && (xout == x || xout == delta))) return false;
  L.reads(x);
  if (delta) L.reads(delta);
  L.reads(norm_w, B);
  if (xout) L.writes(xout);
  L.writes(act);
  return L.sent(L.lib.gemv_bf16_row_rmsnorm_gateup(x, delta, norm_w, xout, B, act, n2, k, eps));
}

// ---- events on the library's stream: GPU time between two points of the launch sequence ------
inline void* event_create() {
  auto& c = context::get();
  void* ev = nullptr;
  return c.ready && c.f.event_create(&ev) == 0 ? ev : nullptr;
}
inline bool event_record(void* ev) {
  auto& c = context::get();
  return c.ready && ev && c.f.event_record(ev) == 0;
}
// Waits for `stop`; negative when either event is unusable.
inline float event_elapsed_ms(void* start, void* stop) {
  auto& c = context::get();
  float ms = -1.0f;
  if (!c.ready || !start || !stop || c.f.event_elapsed_ms(start, stop, &ms) != 0) return -1.0f;
  return ms;
}
inline void event_destroy(void* ev) {
  auto& c = context::get();
  if (c.ready && ev) c.f.event_destroy(ev);
}

// ---- graph capture (cuda.h:508-551), hipGraph underneath --------------------------
inline bool graph_available() { return context::get().ready; }
inline bool capture_begin() {
  auto& c = context::get();
  if (!c.ready || c.capturing) return false;
  if (c.pending) flush();
  if (c.f.graph_begin() != 0) return false;
  c.capturing = true;
  c.capture_writes.clear();
  return true;
}
inline void* capture_end() {
  auto& c = context::get();
  if (!c.capturing) return nullptr;
  void* g = nullptr;
  int rc = c.f.graph_end(&g);
  c.capturing = false;
  c.pending = false;  // recorded launches did not run
  c.free_deferred();
  if (rc != 0 || !g) return nullptr;
  std::sort(c.capture_writes.begin(), c.capture_writes.end());
  c.capture_writes.erase(std::unique(c.capture_writes.begin(), c.capture_writes.end()),
                         c.capture_writes.end());
  c.graph_writes[g] = std::move(c.capture_writes);
  c.capture_writes.clear();
  return g;
}
inline bool graph_launch(void* g) {
  auto& c = context::get();
  if (!c.ready || !g) return false;
  if (c.f.graph_launch(g) != 0) return false;
  c.pending = true;
  auto it = c.graph_writes.find(g);
  if (it != c.graph_writes.end())
    for (uintptr_t base : it->second)
      if (extent* e = c.buffers.at_base(base)) {
        c.forget_derived(*e);        // a replay rewrites the bytes an image was made from
        e->live = extent::side::device;
      }
  return true;
}
inline void graph_destroy(void* g) {
  auto& c = context::get();
  if (!c.ready || !g) return;
  c.graph_writes.erase(g);
  c.f.graph_destroy(g);
}

// ---- persistent KV cache (cuda.h:1321-1405) --------------------------------------
struct kv_cache {
  void* K = nullptr;
  void* V = nullptr;
  int64_t n_kv_heads = 0, max_ctx = 0, D = 0, pos = 0;
  bool kv_bf16 = false;

  bool init(int64_t kv_heads, int64_t maxctx, int64_t d, dtype kv_dt = dtype::f32) {
    n_kv_heads = kv_heads;
    max_ctx = maxctx;
    D = d;
    pos = 0;
    kv_bf16 = (kv_dt == dtype::bf16);
    const int64_t w = kv_bf16 ? 2 : 4;
    K = alloc_device(n_kv_heads * max_ctx * D * w);  // the cache never visits the host
    V = alloc_device(n_kv_heads * max_ctx * D * w);
    return K && V;
  }
  bool append(void* k_new, void* v_new) {
    if (pos >= max_ctx) return false;
    if (!kv_append(K, V, k_new, v_new, pos, max_ctx, n_kv_heads, D, kv_bf16)) return false;
    pos++;
    return true;
  }
  // fused epilogue + append of this step's [q|k|v] (see qkv_rope_append)
  bool rope_append(void* qkv, void* bq, void* bk, void* bv, int64_t n_q_heads, float base) {
    if (pos >= max_ctx) return false;
    if (!qkv_rope_append(qkv, bq, bk, bv, K, V, n_q_heads, n_kv_heads, D, pos, max_ctx, base, kv_bf16))
      return false;
    pos++;
    return true;
  }
  bool attn(void* q, void* out, int64_t n_q_heads, float scale) {
    return attn_decode(q, K, V, out, n_q_heads, n_kv_heads, pos, max_ctx, D, scale, kv_bf16);
  }
  // fused epilogue reading this step's rotary table; position on the host or (d_pos) the device
  bool rope_append_tab(void* qkv, void* bq, void* bk, void* bv, int64_t n_q_heads, void* table,
                       void* d_pos = nullptr) {
    if (!d_pos && pos >= max_ctx) return false;
    if (!qkv_rope_append_tab(qkv, bq, bk, bv, K, V, n_q_heads, n_kv_heads, D, pos, d_pos, max_ctx, table,
                             kv_bf16))
      return false;
    if (!d_pos) pos++;
    return true;
  }
  // rope_append_tab + attn in one launch: out = attention of this step's rotated q over the
  // cache plus the step's own row, which is appended on the way.
  bool attn_qkv(void* qkv, void* bq, void* bk, void* bv, void* out, int64_t n_q_heads, float scale,
                void* table, void* d_pos = nullptr, void* partials = nullptr,
                int64_t partials_bytes = 0) {
    if (!d_pos && pos >= max_ctx) return false;
    if (!attn_decode_qkv(qkv, bq, bk, bv, K, V, out, n_q_heads, n_kv_heads, pos, d_pos, max_ctx, D,
                         scale, table, partials, partials_bytes, kv_bf16))
      return false;
    if (!d_pos) pos++;
    return true;
  }
  // attn_qkv with the split merge left to the o-projection's GEMV (gemv_*_attn)
  bool attn_qkv_parts(void* qkv, void* bq, void* bk, void* bv, int64_t n_q_heads, float scale, void* table,
                      void* d_pos, void* partials, int64_t partials_bytes, int* n_parts) {
    if (!d_pos && pos >= max_ctx) return false;
    if (kv_bf16 || !attn_decode_qkv_parts(qkv, bq, bk, bv, K, V, n_q_heads, n_kv_heads, pos, d_pos, max_ctx, D, scale,
                                          table, partials, partials_bytes, n_parts))
      return false;
    if (!d_pos) pos++;
    return true;
  }
  // The same two with the position on the device (the host pos is NOT advanced:
  // a recorded graph replays these; captured_decoder reconciles pos afterwards).
  // Reference forms (cuda.h:1370-1388): the cache owns the split-partials buffer of its
  // device-position attention, sized once for the capacity on the first (warm) call.
  bool append_dpos(void* k_new, void* v_new, void* d_pos) {
    return kv_append_dpos(K, V, k_new, v_new, d_pos, max_ctx, n_kv_heads, D, kv_bf16);
  }
  void* dpos_partials = nullptr;
  int64_t dpos_partials_bytes = 0;
  bool attn_dpos(void* q, void* out, int64_t n_q_heads, void* d_pos, float scale) {
    if (!dpos_partials) {
      dpos_partials_bytes = attn_partials_bytes(n_q_heads, n_kv_heads, max_ctx, D);
      dpos_partials = alloc_device(dpos_partials_bytes);
      if (!dpos_partials) return false;
    }
    return attn_decode_dpos(q, K, V, out, n_q_heads, n_kv_heads, d_pos, max_ctx, D, scale, dpos_partials,
                            dpos_partials_bytes, kv_bf16);
  }
  bool rope_append_dpos(void* qkv, void* bq, void* bk, void* bv, int64_t n_q_heads, float base,
                        void* d_pos) {
    return qkv_rope_append_dpos(qkv, bq, bk, bv, K, V, n_q_heads, n_kv_heads, D, d_pos, max_ctx, base,
                                kv_bf16);
  }
  bool attn_dpos(void* q, void* out, int64_t n_q_heads, float scale, void* d_pos, void* partials,
                 int64_t partials_bytes) {
    return attn_decode_dpos(q, K, V, out, n_q_heads, n_kv_heads, d_pos, max_ctx, D, scale, partials,
                            partials_bytes, kv_bf16);
  }
  bool prefill(void* q, void* k_src, void* v_src, void* out, int64_t T, int64_t n_q_heads,
               float scale) {
    if (T <= 0 || pos + T > max_ctx) return false;
    if (!kv_fill(K, V, k_src, v_src, T, max_ctx, n_kv_heads, D, kv_bf16, pos)) return false;
    const int64_t p0 = pos;
    pos += T;
    return attn_prefill(q, K, V, out, n_q_heads, n_kv_heads, T, max_ctx, D, scale, kv_bf16, p0);
  }
  // The chunk form of attn_qkv: raw token-major projection in, token-major attention out;
  // qh is [n_q_heads, T, D] scratch for the rotated queries.
  // qkv_parts > 1: qkv holds the projection's K-split parts.
  bool prefill_qkv(void* qkv, void* bq, void* bk, void* bv, void* table, void* qh, void* out_tok, int64_t T,
                   int64_t n_q_heads, float scale, int64_t qkv_parts = 1) {
    if (T <= 0 || pos + T > max_ctx) return false;
    if (!qkv_rope_fill(qkv, bq, bk, bv, table, qh, K, V, T, n_q_heads, n_kv_heads, D, pos, max_ctx, kv_bf16,
                       qkv_parts))
      return false;
    const int64_t p0 = pos;
    pos += T;
    return attn_prefill_tok(qh, K, V, out_tok, n_q_heads, n_kv_heads, T, max_ctx, D, scale, kv_bf16, p0);
  }
  void destroy() {
    if (K) release(K, 0, nullptr);
    if (V) release(V, 0, nullptr);
    if (dpos_partials) release(dpos_partials, 0, nullptr);
    K = V = dpos_partials = nullptr;
  }
};

}  // namespace hip
}  // namespace tl
