"""CPU: the shared libraries load without a GPU and export every symbol the C header
declares; the backend reports 'unavailable' instead of failing when no device exists."""
import ctypes as C
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(headers=("tensorlib_hip.h", "tensorlib_hip_bench.h")):
    """Entry points declared by the boundary header and by the benchmark / tuning header."""
    names = set()
    for h in headers:
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(tlhip_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_every_declared_symbol_is_exported(pkg):
    lib = C.CDLL(pkg.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 45
    for n in names:
        assert hasattr(lib, n), "%s declared in tensorlib_hip.h but not exported" % n


def test_boundary_header_holds_no_benchmark_or_tuning_hooks():
    """What a backend binds and what benchmarks use are declared apart."""
    boundary = declared_symbols(("tensorlib_hip.h",))
    assert not [n for n in boundary if n.startswith("tlhip_bench_")]
    assert [n for n in boundary if n.startswith("tlhip_tune_")] == ["tlhip_tune_gemv_cols"]   # the reference's set_no_splitk


def test_python_binding_matches_header(pkg):
    from importlib import import_module
    capi = import_module("cpp-tensorlib_amd.capi")
    assert set(capi.SIGNATURES) == set(declared_symbols())


def test_abi_version_and_error_path_without_gpu(pkg):
    lib = pkg.TlHip(init=False)
    assert lib.c.tlhip_abi_version() == 1
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    assert lib.c.tlhip_init(0) == -1                 # TLHIP_ENODEVICE, no abort
    assert b"device" in lib.c.tlhip_last_error().lower()
    out = C.c_void_p()
    assert lib.c.tlhip_malloc(C.byref(out), 64) == -1 and not out.value
    assert lib.c.tlhip_gemv_q4(None, None, None, None, 8, 32, 32) == -1      # ops fail loudly, no fallback


def test_product_does_not_touch_the_oracle():
    """Nothing shipped may include, link or import anything under oracle/."""
    bad = []
    for base in ("cpp-tensorlib_amd", "include"):
        for d, _, files in os.walk(os.path.join(ROOT, base)):
            if os.sep + "build" in d or d.endswith("__pycache__"):
                continue
            for f in files:
                if f.endswith((".so", ".o", ".pyc")):
                    continue
                t = open(os.path.join(d, f), errors="ignore").read()
                if re.search(r"oraclelib|liboracle|oracle\.h|orc_[a-z]+\(|tlref_", t):
                    bad.append(os.path.join(d, f))
    assert not bad, bad
    for so in ("libtensorlib_hip.so", "libtl_qwen.so"):
        p = os.path.join(ROOT, "cpp-tensorlib_amd", "lib", so)
        deps = subprocess.run(["ldd", p], capture_output=True, text=True).stdout
        assert "oracle" not in deps and "tlref" not in deps


def test_host_layer_declines_without_backend(pkg):
    """tl::hip with no reachable GPU: available() is false and the harness refuses to
    construct (no silent CPU path)."""
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    from importlib import import_module
    qwen = import_module("cpp-tensorlib_amd.qwen")
    with pytest.raises(RuntimeError) as e:
        qwen.QwenGPU(dict(qwen.QWEN_05B))
    assert "unavailable" in str(e.value)
