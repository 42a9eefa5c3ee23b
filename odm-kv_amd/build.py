"""Builds libodmkv.so (the HIP kernels and their C ABI) for gfx950 with hipcc, and
libodmkv_bench.so: the same object files plus the measurement entry points of csrc/bench_hooks.hip
(include/odmkv_bench.h), which the product library does not export.

    python odm-kv_amd/build.py [--force]

hipcc cross-compiles without a GPU.  Flags that matter:
  -ffp-contract=off   nothing is fused unless the source says fma: the allocator's cost and the
                      quantiser's rotation are bit-exact contracts with their CPU statements;
  packed-fp32-ops off the compiler must not form packed fp32 instructions.
Both libraries are linked with csrc/exports.map: only the C entry points (odmkv_*) are dynamic symbols.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libodmkv.so")
BENCH_LIB = os.path.join(LIBDIR, "libodmkv_bench.so")
SOURCES = ["error.hip", "score.hip", "window.hip", "allocate.hip", "pack.hip", "rows.hip", "decode.hip", "flush.hip", "codebook.hip"]
BENCH_SOURCES = ["bench_hooks.hip"]
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def _newest(paths):
    return max(os.path.getmtime(p) for p in paths)


def build(force: bool = False, verbose: bool = True) -> str:
    srcs = [os.path.join(CSRC, s) for s in SOURCES + BENCH_SOURCES]
    deps = srcs + [os.path.join(CSRC, h) for h in ("common.h", "quant.h", "decode.h", "exports.map")] + [
        os.path.join(HERE, "..", "include", "odmkv.h"), os.path.join(HERE, "..", "include", "odmkv_bench.h"), __file__]
    if (not force and os.path.exists(LIB) and os.path.exists(BENCH_LIB)
            and min(os.path.getmtime(LIB), os.path.getmtime(BENCH_LIB)) >= _newest(deps)):
        return LIB
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(objdir, os.path.basename(src) + ".o")
        cmd = ["hipcc", *FLAGS, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
        warn = [ln for ln in r.stderr.splitlines() if "packed-fp32-ops" not in ln and ln.strip()]
        if warn and verbose:
            print("\n".join(warn))
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(compile_one, srcs))
    product = objs[:len(SOURCES)]
    for lib, parts in ((LIB, product), (BENCH_LIB, objs)):
        cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", f"-Wl,--version-script={os.path.join(CSRC, 'exports.map')}",
               "-o", lib, *parts]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
