"""Builds libgllm_hip_quant.so in-tree: kernels -> gfx950 code object -> host library.

    python -m gllm_amd.build

Three steps, all plain compiler invocations (no cmake, no JIT cache):
  1. hipcc --genco --offload-arch=gfx950   csrc/kernels_*.hip -> csrc/build/kernels_*.hsaco, side by side
  2. hipcc -c --offload-arch=gfx950        csrc/gllmq_noalloc.hip -> csrc/build/gllmq_noalloc.o (host code plus the
                                           device array behind the entry point that allocates nothing)
  3. hipcc (host only)                     csrc/gllmq_host.cpp, csrc/gguf_reader.cpp + the object of step 2 + the code
                                           objects of step 1 embedded with .incbin -> gllm_amd/libgllm_hip_quant.so
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
BUILD = os.path.join(CSRC, "build")
KERNEL_UNITS = ["codec", "mm8", "mm8s", "mm8s_q8_0", "mm8c", "mm8_q6k_q8_0", "mmf", "mmfs", "moe"]  # csrc/kernels_<unit>.hip, one code object each
LIB = os.path.join(HERE, "libgllm_hip_quant.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

# Packed FP32 instructions are switched off for every kernel of the library.
DEVICE_FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-Werror",  # (a loop the optimizer could not unroll as asked is a warning: none are left standing)
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd: list[str]) -> None:
    print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.stdout.strip():
        print(res.stdout, flush=True)
    if res.returncode != 0:
        raise RuntimeError(f"command failed ({res.returncode}): {' '.join(cmd)}")


def build_kernels(units: list[str] | None = None) -> list[str]:
    """Compiles the given kernel units (all of them by default)."""
    os.makedirs(BUILD, exist_ok=True)
    units = list(units or KERNEL_UNITS)

    def one(unit: str) -> str:
        out = os.path.join(BUILD, f"kernels_{unit}.hsaco")
        _run([HIPCC, "--genco", *DEVICE_FLAGS, "-I", CSRC, "-o", out, os.path.join(CSRC, f"kernels_{unit}.hip")])
        return out
    with ThreadPoolExecutor(max_workers=min(len(units), os.cpu_count() or 1)) as pool:
        return list(pool.map(one, units))


NOALLOC_OBJ = os.path.join(BUILD, "gllmq_noalloc.o")


def build_noalloc() -> str:
    os.makedirs(BUILD, exist_ok=True)
    _run([HIPCC, "-c", "-fPIC", *DEVICE_FLAGS, "-I", os.path.join(ROOT, "include"), "-I", CSRC,
          os.path.join(CSRC, "gllmq_noalloc.hip"), "-o", NOALLOC_OBJ])
    return NOALLOC_OBJ


def build_host() -> str:
    _run([HIPCC, NOALLOC_OBJ, "-x", "c++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra",
          "-D__HIP_PLATFORM_AMD__=1", f'-DGLLMQ_HSACO_DIR="{BUILD}"',
          "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROCM, "include"),
          "-I", CSRC, os.path.join(CSRC, "gllmq_host.cpp"), os.path.join(CSRC, "gguf_reader.cpp"), "-o", LIB,
          "-L", os.path.join(ROCM, "lib"), "-lamdhip64", f"-Wl,-rpath,{os.path.join(ROCM, 'lib')}"])
    return LIB


def build() -> str:
    build_kernels()
    build_noalloc()
    return build_host()


def stale_units() -> list[str]:
    """Kernel units whose code object is missing or older than a source it is built from (its own
    includes, directly or through another include, and the shared headers)."""
    import re

    def sources(path: str, seen: set[str]) -> set[str]:
        if path in seen or not os.path.exists(path):
            return seen
        seen.add(path)
        for inc in re.findall(r'^\s*#include\s+"([^"]+)"', open(path).read(), flags=re.M):
            sources(os.path.join(CSRC, inc), seen)
        return seen
    out = []
    for unit in KERNEL_UNITS:
        obj = os.path.join(BUILD, f"kernels_{unit}.hsaco")
        deps = sources(os.path.join(CSRC, f"kernels_{unit}.hip"), set())
        if not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(d) for d in deps):
            out.append(unit)
    return out


if __name__ == "__main__":
    # `python -m gllm_amd.build [unit ...]`: with unit names, only those kernel units are recompiled,
    # together with every other unit that is older than one of its sources (a change to a shared
    # header reaches all of them: host and kernels must agree on the parameter blocks), and the
    # host library is linked again
    if len(sys.argv) > 1:
        build_kernels(sorted(set(sys.argv[1:]) | set(stale_units())))
        if not os.path.exists(NOALLOC_OBJ):
            build_noalloc()
        build_host()
    else:
        build()
    print(LIB)
    sys.exit(0)
