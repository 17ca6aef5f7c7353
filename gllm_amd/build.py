"""Builds libgllm_hip_quant.so in-tree: kernels -> gfx950 code object -> host library.

    python -m gllm_amd.build

Three steps, all plain compiler invocations (no cmake, no JIT cache):
  1. hipcc --genco --offload-arch=gfx950   csrc/gllmq_kernels.hip -> csrc/build/gllmq_kernels.hsaco
  2. hipcc -c --offload-arch=gfx950        csrc/gllmq_noalloc.hip -> csrc/build/gllmq_noalloc.o (host code plus the
                                           device array behind the entry point that allocates nothing)
  3. hipcc (host only)                     csrc/gllmq_host.cpp, csrc/gguf_reader.cpp + the object of step 2 + the code
                                           object of step 1 embedded with .incbin -> gllm_amd/libgllm_hip_quant.so
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
BUILD = os.path.join(CSRC, "build")
HSACO = os.path.join(BUILD, "gllmq_kernels.hsaco")
LIB = os.path.join(HERE, "libgllm_hip_quant.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

# Packed FP32 instructions are switched off for every kernel of the library.
DEVICE_FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd: list[str]) -> None:
    print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.stdout.strip():
        print(res.stdout, flush=True)
    if res.returncode != 0:
        raise RuntimeError(f"command failed ({res.returncode}): {' '.join(cmd)}")


def build_kernels() -> str:
    os.makedirs(BUILD, exist_ok=True)
    _run([HIPCC, "--genco", *DEVICE_FLAGS, "-I", CSRC, "-o", HSACO, os.path.join(CSRC, "gllmq_kernels.hip")])
    return HSACO


NOALLOC_OBJ = os.path.join(BUILD, "gllmq_noalloc.o")


def build_noalloc() -> str:
    os.makedirs(BUILD, exist_ok=True)
    _run([HIPCC, "-c", "-fPIC", *DEVICE_FLAGS, "-I", os.path.join(ROOT, "include"), "-I", CSRC,
          os.path.join(CSRC, "gllmq_noalloc.hip"), "-o", NOALLOC_OBJ])
    return NOALLOC_OBJ


def build_host() -> str:
    _run([HIPCC, NOALLOC_OBJ, "-x", "c++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra",
          "-D__HIP_PLATFORM_AMD__=1", f'-DGLLMQ_HSACO_PATH="{HSACO}"',
          "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROCM, "include"),
          "-I", CSRC, os.path.join(CSRC, "gllmq_host.cpp"), os.path.join(CSRC, "gguf_reader.cpp"), "-o", LIB,
          "-L", os.path.join(ROCM, "lib"), "-lamdhip64", f"-Wl,-rpath,{os.path.join(ROCM, 'lib')}"])
    return LIB


def build() -> str:
    build_kernels()
    build_noalloc()
    return build_host()


if __name__ == "__main__":
    build()
    print(LIB)
    sys.exit(0)
