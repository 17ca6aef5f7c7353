"""GPU parity of the f16 matrix-core GEMM whose arithmetic waves prepare their own activations
(mmfr.hip.inc: Q4_K and Q5_K, 9 to 16 rows of f32 activations, from 8 weight rows per CU up;
eight arithmetic waves with sixteen activation rows of one block of K in registers each, loader
waves streaming the weight items through an LDS ring, the slices of K meeting inside the one
launch) against the oracle, through the C ABI.  Reference: Backend::quantized_matmul with m > 1
(src/compat/cpu_backend.rs:991-1049; Op::QuantGemm, build_graph.inc.rs:108-123).  Same bar as the
other matmul tests: rel-L2 <= 1e-4 and |err| <= 1e-3 * max|y| against float64 accumulation."""
import numpy as np
import pytest

from gllm_amd.synth import random_activations, random_weight
from tests.test_gpu_parity import check_close, gpu_matmul

pytestmark = pytest.mark.gpu

Q4_K, Q5_K = 12, 13


@pytest.fixture(scope="module")
def hip():
    from gllm_amd.backend import HipBackend
    return HipBackend(0)


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def cus(torch):
    return torch.cuda.get_device_properties(0).multi_processor_count


@pytest.mark.parametrize("dtype", [Q4_K, Q5_K])
def test_shapes_against_the_oracle(hip, torch, oracle, dtype):
    """One to many slices of K of eight blocks (last slices with fewer blocks than waves; a partial
    last block), one to many tiles per workgroup with a reused ring, a ragged last workgroup, tiles
    lower than 32 and lower than 16 rows, 9 to 16 activation rows, K below one slice (no meeting at
    all)."""
    c = cus(torch)
    cases = [(16, 16 * c, 1024), (9, 24 * c + 7, 2048), (16, 56 * c, 4096), (13, 56 * c + 17, 1024 - 32), (11, 100 * c, 512),
             (12, 128 * c + 3, 768), (16, 200 * c, 256), (10, 300 * c + 11, 512), (15, 40 * c, 1280), (16, 8 * c, 14336),
             (16, 600 * c + 5, 256), (14, 9 * c + 1, 2304), (10, 12 * c, 2048 + 256), (9, 8 * c, 1536), (16, 8 * c, 4096 + 2048)]
    for m, n, k in cases:
        print(f"gemm rows dtype={dtype} m={m} n={n} k={k}", flush=True)
        w, x = random_weight(dtype, n, k, seed=m + n), random_activations(m, k, seed=k + m)
        want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=16)
        got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        assert hip.last_kernel_name().startswith("gq_mmfr_"), hip.last_kernel_name()
        check_close(got, want, f"gemm rows dtype={dtype} m={m} n={n} k={k}")


def test_repeats_rows_of_zeros_and_non_finite_rows(hip, torch, oracle):
    """The same launch twice with different inputs (the counters in LDS and the arrival counters in
    memory start from zero every launch); an all-zero activation row gives zeros; a row with an
    infinity or a NaN gives NaN in its own outputs and leaves the other rows alone."""
    c = cus(torch)
    m, n, k = 14, 56 * c + 9, 2048 + 512
    w = random_weight(Q4_K, n, k, seed=3)
    for seed in (1, 2):
        print(f"gemm rows repeat seed={seed}", flush=True)
        x = random_activations(m, k, seed=seed)
        x[3] = 0.0
        x[7, 100] = np.inf
        x[12, 2047] = np.nan
        clean = x.copy()
        clean[7] = 0.0
        clean[12] = 0.0
        want = oracle.quantized_matmul(w, clean, Q4_K, m, n, k, acc=oracle.ACC_F64, threads=16)
        got = gpu_matmul(hip, torch, w, x, Q4_K, m, n, k)
        assert hip.last_kernel_name().startswith("gq_mmfr_")
        assert np.isnan(got[7]).all() and np.isnan(got[12]).all()
        assert np.all(got[3] == 0.0)
        keep = [r for r in range(m) if r not in (7, 12)]
        check_close(got[keep], want[keep], f"seed={seed}")


def test_against_the_three_launch_form_and_what_it_leaves(hip, torch):
    """Equal to the three-launch GEMM within the matmul bar (another order of sums); bf16-rounded
    activations, few weight rows per CU and more than 16 rows stay with the other kernels."""
    from gllm_amd.backend import ACT_BF16, HipBackend
    plain = HipBackend(0, options={"mmfs": 0, "mmfr": 0})
    c = cus(torch)
    for dtype, m, n, k in ((Q4_K, 12, 56 * c, 4096), (Q5_K, 16, 56 * c, 2048), (Q4_K, 16, 56 * c, 4096)):
        print(f"gemm rows vs three launches dtype={dtype} m={m}", flush=True)
        w, x = random_weight(dtype, n, k, seed=5), random_activations(m, k, seed=6)
        a = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        assert hip.last_kernel_name().startswith("gq_mmfr_")
        b = gpu_matmul(plain, torch, w, x, dtype, m, n, k)
        assert not plain.last_kernel_name().startswith("gq_mmfr_")
        check_close(a, b, f"dtype={dtype} m={m}")
    w, x = random_weight(Q4_K, 16 * c, 1024, seed=2), random_activations(16, 1024, seed=1)
    gpu_matmul(hip, torch, w, x, Q4_K, 16, 16 * c, 1024, act_mode=ACT_BF16)
    assert not hip.last_kernel_name().startswith("gq_mmfr_")
    w = random_weight(Q4_K, 4 * c, 1024, seed=2)
    gpu_matmul(hip, torch, w, x, Q4_K, 16, 4 * c, 1024)
    assert not hip.last_kernel_name().startswith("gq_mmfr_")
    # 17 rows and more as well
    w = random_weight(Q4_K, 16 * c, 1024, seed=2)
    gpu_matmul(hip, torch, w, random_activations(17, 1024, seed=1), Q4_K, 17, 16 * c, 1024)
    assert not hip.last_kernel_name().startswith("gq_mmfr_")
