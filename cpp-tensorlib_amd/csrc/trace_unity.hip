// The library as ONE translation unit with the kernels' phase timestamps switched on
// (TLHIP_MARK in the kernels, g_trace in common.hpp: one file-scope array, hence one unit).
// Built only on request (python cpp-tensorlib_amd/build.py --trace) into
// lib/libtensorlib_hip_trace.so, which exports the whole C ABI plus tlhip_trace_read;
// cpp-tensorlib_amd/trace_phases.py drives it. Not part of the product library.
#define TLHIP_TRACE 1
#include "runtime.hip"
#include "gemv.hip"
#include "elementwise.hip"
#include "modelops.hip"
#include "attn.hip"
#include "attn_prefill_mfma.hip"
#include "attn_prefill_x3.hip"
#include "prefill.hip"
#include "gemm_f16t.hip"
#include "convert.hip"
#include "sgemm.hip"

// Copies the timestamp array to the host (bytes: at most its size) and optionally clears it.
extern "C" int tlhip_trace_read(void* host, size_t bytes, int clear) {
  if (bytes > sizeof(tlhip::g_trace)) bytes = sizeof(tlhip::g_trace);
  hipError_t e = hipMemcpyFromSymbol(host, HIP_SYMBOL(tlhip::g_trace), bytes);
  if (e != hipSuccess) return -1;
  if (clear) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(tlhip::g_trace)) != hipSuccess) return -1;
    if (hipMemset(p, 0, sizeof(tlhip::g_trace)) != hipSuccess) return -1;
  }
  return 0;
}
