"""Builds libtensorlib_hip.so (gfx950 code objects + the C ABI) with hipcc.

Usage: python cpp-tensorlib_amd/build.py [--force]
The library is written next to this file under lib/ and is what the backend
header, the tests and bench.py load; nothing is built at import time.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")
LIB = os.path.join(LIBDIR, "libtensorlib_hip.so")
SOURCES = ["runtime.hip", "gemv.hip", "elementwise.hip", "modelops.hip", "attn.hip", "attn_prefill_mfma.hip", "attn_prefill_f16.hip", "prefill.hip", "gemm_f16t.hip", "convert.hip", "sgemm.hip"]
# -packed-fp32-ops off: hipcc must not form v_pk_*_f32 on this pool.
FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-fno-gpu-rdc",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function", "-Wno-unknown-cuda-version"]


def hipcc():
    for p in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if p and (os.path.sep not in p or os.path.exists(p)):
            return p
    return "hipcc"


def _stale(out, deps):
    if not os.path.exists(out):
        return True
    t = os.path.getmtime(out)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=False, verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    headers = [os.path.join(CSRC, "common.hpp"),
               os.path.join(os.path.dirname(HERE), "include", "tensorlib_hip.h")]
    headers += [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    jobs = []
    for s in SOURCES:
        src = os.path.join(CSRC, s)
        obj = os.path.join(OBJDIR, s.replace(".hip", ".o"))
        if force or _stale(obj, [src] + headers):
            jobs.append((src, obj))

    def compile_one(job):
        src, obj = job
        cmd = [hipcc()] + FLAGS + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, r.stderr))
        warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if warn and verbose:
            print(warn)

    with ThreadPoolExecutor(max_workers=min(6, max(1, len(jobs)))) as ex:
        list(ex.map(compile_one, jobs))
    objs = [os.path.join(OBJDIR, s.replace(".hip", ".o")) for s in SOURCES]
    if force or jobs or _stale(LIB, objs):
        cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    build_host(force, verbose)
    return LIB


QWEN_LIB = os.path.join(LIBDIR, "libtl_qwen.so")


def build_host(force=False, verbose=True):
    """libtl_qwen.so: the header-only C++ host layer (include/tl/) behind a C entry
    layer, compiled with plain g++; it reaches the HIP library through dlopen."""
    src = os.path.join(CSRC, "qwen_capi.cpp")
    inc = os.path.join(HERE, "include")
    deps = [src] + [os.path.join(inc, "tl", f) for f in os.listdir(os.path.join(inc, "tl"))]
    if force or _stale(QWEN_LIB, deps):
        cmd = ["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-Wextra", "-I", inc, src,
               "-o", QWEN_LIB, "-ldl"]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return QWEN_LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
