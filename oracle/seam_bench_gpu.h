// TEST INFRASTRUCTURE. gpu.h for building the reference's own CUDA-side programs (its
// bench/cuda checks, benchmarks and decode harness, unmodified) on this repository's backend:
// those programs name their backend `tl::cuda` and include "cuda.h" directly, so here tl::cuda
// is an alias of tl::hip (the rename a maintainer would make in those files) and oracle/Makefile
// places a one-line cuda.h next to this file that includes it. CUgraphExec is the graph handle
// type the harness spells out (bench/cuda/qwen_model.h:793).
#pragma once

#include "metal.h"
#include "webgpu.h"

#define TL_HIP_USE_METAL_KOP 1
#include "hip.h"

namespace tl {

namespace hip {
using CUgraphExec = void*;
}
namespace gpu = hip;
namespace cuda = hip;

inline bool gpu_available() { return gpu::available(); }

}  // namespace tl
