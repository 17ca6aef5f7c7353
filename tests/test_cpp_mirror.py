"""The C++ host mirror (include/gllm_hip_quant.hpp): its parity program is built by
__graft_entry__.build() (tests/cpp/Makefile) and run here on the GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROG = os.path.join(ROOT, "tests", "cpp", "test_backend")


def test_cpp_mirror_compiles_against_the_header():
    # syntax/type check of the header-only mirror on the CPU (no GPU call)
    src = '#include "gllm_hip_quant.hpp"\nint main() { return sizeof(gllm::HipBackend) ? 0 : 1; }\n'
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Wextra", "-Werror", "-I",
                        os.path.join(ROOT, "include"), "-x", "c++", "-"], input=src.encode(), capture_output=True)
    assert r.returncode == 0, r.stderr.decode()


@pytest.mark.gpu
def test_cpp_mirror_parity_program():
    if not os.path.exists(PROG):
        pytest.fail("tests/cpp/test_backend is not built; run __graft_entry__.build() first")
    print("running tests/cpp/test_backend", flush=True)
    r = subprocess.run([PROG], capture_output=True, timeout=100)
    out = r.stdout.decode() + r.stderr.decode()
    print(out)
    assert r.returncode == 0, out
