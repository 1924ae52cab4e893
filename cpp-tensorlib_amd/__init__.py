"""MI355X (gfx950) backend for the cpp-tensorlib LLM decode path.

The product is native: HIP kernels and a C ABI (csrc/, include/tensorlib_hip.h)
under a header-only C++17 host layer (include/tl/). This Python package only
builds the library (build.py) and binds its C ABI for tests and benchmarks
(capi.py). Import it with importlib.import_module("cpp-tensorlib_amd").
"""
from . import build as _build  # noqa: F401
from .capi import LIB_PATH, TlHip, TlHipError, load  # noqa: F401
