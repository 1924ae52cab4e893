// TEST INFRASTRUCTURE. The `gpu.h` a maintainer of the reference would end up with after
// adding the MI355X arm (one more `#elif` that includes tl/hip.h and aliases it), reduced to that arm: the
// reference's own backend headers for the shared `kop` enum and their stubs, then tl::hip,
// then the alias. oracle/Makefile copies it as gpu.h into a directory that precedes the
// reference's include path, so the reference's storage.h / array.h (`#include <gpu.h>`)
// compile, unmodified, on top of this repository's backend header.
#pragma once

#include "cuda.h"
#include "metal.h"
#include "webgpu.h"

#define TL_HIP_USE_METAL_KOP 1
#include "hip.h"

namespace tl {

namespace gpu = hip;

inline bool gpu_available() { return gpu::available(); }

}  // namespace tl
