"""GPU parity of the streamed form of the f16 matrix-core GEMM (Q4_K and Q5_K, 9 rows and more,
from 8 weight rows per CU up: a workgroup takes a range of weight rows and four blocks of K, its
four arithmetic waves keep one block's activations in registers each while loader waves stream the
weight items through an LDS ring; the slices of K meet inside the launch) against the oracle,
through the C ABI.  Same bar as the other matmul tests: rel-L2 <= 1e-4 and
|err| <= 1e-3 * max|y| against float64 accumulation."""
import numpy as np
import pytest

from gllm_amd.synth import random_activations, random_weight
from tests.test_gpu_parity import check_close, gpu_matmul

pytestmark = pytest.mark.gpu

Q4_K, Q5_K = 12, 13


@pytest.fixture(scope="module")
def hip():
    # "mmfs_all": the streamed form wherever the shape fits, not only where it was timed fastest
    from gllm_amd.backend import HipBackend
    # ("mmfr" = 0: not its successor, which prepares its own activations and would take these shapes)
    return HipBackend(0, options={"mmfs_all": 1, "mmfr": 0})


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def cus(torch):
    return torch.cuda.get_device_properties(0).multi_processor_count


@pytest.mark.parametrize("dtype", [Q4_K, Q5_K])
def test_streamed_gemm_shapes_against_the_oracle(hip, torch, oracle, dtype):
    """One to sixteen slices of K (a last slice with fewer than four blocks, a partial last block),
    one to many tiles per workgroup with a reused ring, a ragged last workgroup, tiles lower than 32
    rows, 9 to 70 activation rows (one to three launches of 32)."""
    c = cus(torch)
    cases = [(16, 16 * c, 1024), (9, 24 * c + 7, 2048), (32, 56 * c, 4096), (17, 56 * c + 17, 1024 - 32), (33, 100 * c, 512),
             (12, 128 * c + 3, 768), (64, 200 * c, 256), (20, 300 * c + 11, 512), (70, 40 * c, 1280), (16, 8 * c, 14336),
             (32, 600 * c + 5, 256)]
    for m, n, k in cases:
        print(f"streamed gemm dtype={dtype} m={m} n={n} k={k}", flush=True)
        w, x = random_weight(dtype, n, k, seed=m + n), random_activations(m, k, seed=k + m)
        want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=16)
        got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        assert hip.last_kernel_name().startswith("gq_mmfs_"), hip.last_kernel_name()
        check_close(got, want, f"streamed gemm dtype={dtype} m={m} n={n} k={k}")


def test_streamed_gemm_bf16_mode_and_repeats(hip, torch, oracle):
    """Activations rounded to bf16 first (no lo plane), and the same launch twice with different
    inputs: the counters in LDS start from zero every launch."""
    from gllm_amd.backend import ACT_BF16
    from oracle import npref
    c = cus(torch)
    m, n, k = 24, 56 * c + 9, 2048
    w = random_weight(Q4_K, n, k, seed=3)
    for seed in (1, 2):
        print(f"streamed gemm bf16 seed={seed}", flush=True)
        x = random_activations(m, k, seed=seed)
        want = oracle.quantized_matmul(w, npref.bf16_rne(x), Q4_K, m, n, k, acc=oracle.ACC_F64, threads=16)
        got = gpu_matmul(hip, torch, w, x, Q4_K, m, n, k, act_mode=ACT_BF16)
        assert hip.last_kernel_name().startswith("gq_mmfs_") and hip.last_kernel_name().endswith("_bf16")
        check_close(got, want, f"bf16 seed={seed}")


def test_streamed_gemm_against_the_three_launch_form(hip, torch):
    """Also the default choice between the two: the streamed form up to 40 M weights."""
    from gllm_amd.backend import HipBackend
    plain, default = HipBackend(0, options={"mmfs": 0, "mmfr": 0}), HipBackend(0, options={"mmfr": 0})
    c = cus(torch)
    x, w = random_activations(16, 1024, seed=1), random_weight(Q4_K, 16 * c, 1024, seed=2)
    gpu_matmul(default, torch, w, x, Q4_K, 16, 16 * c, 1024)
    assert default.last_kernel_name().startswith("gq_mmfs_")
    w = random_weight(Q4_K, 56 * c, 4096, seed=2)
    gpu_matmul(default, torch, w, random_activations(16, 4096, seed=1), Q4_K, 16, 56 * c, 4096)
    assert not default.last_kernel_name().startswith("gq_mmfs_")
    c = cus(torch)
    for dtype, m, n, k in ((Q4_K, 32, 56 * c, 4096), (Q5_K, 48, 56 * c, 2048)):
        print(f"streamed gemm vs three launches dtype={dtype} m={m}", flush=True)
        w, x = random_weight(dtype, n, k, seed=5), random_activations(m, k, seed=6)
        a = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        assert hip.last_kernel_name().startswith("gq_mmfs_")
        b = gpu_matmul(plain, torch, w, x, dtype, m, n, k)
        assert not plain.last_kernel_name().startswith("gq_mmfs_")
        check_close(a, b, f"dtype={dtype} m={m}")
