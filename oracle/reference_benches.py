#!/usr/bin/env python3
"""The reference's own benchmark programs on this backend (test infrastructure, not the bench line).

  python oracle/reference_benches.py
"""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests"))


def main():
    """Runs the REFERENCE's own benchmark programs (bench/cuda/speed/*.cpp,
    compiled unmodified against this backend by `make -C oracle refprogs` where the reference tree
    exists; the binaries travel, the sources do not) and prints what they print. The three that
    load a model get a synthetic Qwen2.5-0.5B-shaped F16 GGUF (tests/ggufwriter.py): the shape the
    reference's published RTX 3090 figures are quoted on (README.md:310-313)."""
    import subprocess
    import tempfile
    import ggufwriter
    progs = os.path.join(ROOT, "oracle", "_ref", "refprogs")
    if not os.path.isdir(progs):
        print("reference_benches.py: oracle/_ref/refprogs is not built (make -C oracle refprogs, needs the reference tree)", file=sys.stderr)
        sys.exit(2)
    env = dict(os.environ, TENSORLIB_HIP_LIB=os.path.join(ROOT, "cpp-tensorlib_amd", "lib", "libtensorlib_hip.so"))
    out = {}

    def run(name, *args, limit=280):
        print("== %s %s" % (name, " ".join(args[1:])), flush=True)
        r = subprocess.run([os.path.join(progs, name)] + list(args), env=env, stdout=subprocess.PIPE,
                           stderr=subprocess.STDOUT, timeout=limit)
        text = r.stdout.decode(errors="replace")
        print(text, flush=True)
        out[" ".join([name] + [os.path.basename(a) for a in args])] = {"rc": r.returncode, "output": text}
    for name in ("bench_q4_gemv", "bench_bf16_gemv", "bench_qwen_gemv", "bench_attn_decode", "bench_llm"):
        run(name)
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "qwen05b_synthetic_f16.gguf")
        ggufwriter.qwen05b_synthetic(path)
        run("bench_qwen_decode", path)
        run("bench_qwen_decode", path, "bf16", "64", "all")
        run("bench_qwen_prefill", path)
        run("bench_qwen_ctx", path)
    print(json.dumps({"reference_benches": out}))


if __name__ == "__main__":
    main()
