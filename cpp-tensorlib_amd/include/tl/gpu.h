#pragma once

// The GPU facade of this host layer: tl::gpu is the MI355X backend. In the
// reference, include/gpu.h:28-34 picks webgpu / cuda / metal by macro; the arm
// a maintainer adds there for this backend is
//     #elif defined(TENSORLIB_HIP)
//     namespace gpu = hip;
// and this file is that arm on its own.

#include "hip.h"

namespace tl {
namespace gpu = hip;
inline bool gpu_available() { return gpu::available(); }
}  // namespace tl
