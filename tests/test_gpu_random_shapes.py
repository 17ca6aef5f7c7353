"""GPU parity on shapes drawn from a seeded generator: formats, one to twelve activation rows,
weight rows from a few to a few dozen per CU and rows of one to sixty blocks with ragged ends, so
that every kernel family the dispatch can pick (integer-dot GEMV, fetch-and-compute, streamed with
and without pairs of blocks or slices of K, the small GEMMs) meets sizes nobody chose by hand.
Same bar as the other matmul tests, against the oracle's float64 accumulation; guard regions
behind the inputs and the output catch reads and writes past the end."""
import numpy as np
import pytest

from gllm_amd.synth import random_activations, random_weight
from tests.test_gpu_parity import check_close, gpu_matmul

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_shapes_from_a_seeded_generator(torch, oracle, seed):
    from gllm_amd.backend import HipBackend
    hip = HipBackend(0)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    rng = np.random.default_rng(seed)
    seen = set()
    for i in range(36):
        dtype = int(rng.choice([Q8_0, Q4_K, Q5_K, Q6_K]))
        m = int(rng.choice([1, 1, 1, 2, 3, 4, 5, 8, 9, 12]))
        rows_per_cu = float(rng.choice([0.3, 1, 4, 8, 16, 24, 33, 56]))
        n = max(1, int(rows_per_cu * cus) + int(rng.integers(-7, 8)))
        blocks = int(rng.choice([1, 2, 3, 6, 8, 9, 16, 17, 24, 35, 56, 60]))
        # Q8_0 rows are whole 32-element blocks, the others end anywhere a multiple of 8 allows
        k = blocks * 256 - int(rng.choice([0, 0, 32, 64, 96])) if blocks > 1 else 256
        if m * n * k > 48e6 * 12:  # keep the oracle's share of the run to seconds
            n = max(1, n // 4)
        print(f"seeded shape {seed}/{i}: dtype={dtype} m={m} n={n} k={k}", flush=True)
        w, x = random_weight(dtype, n, k, seed=seed * 1000 + i), random_activations(m, k, seed=seed * 2000 + i)
        want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=16)
        got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        check_close(got, want, f"dtype={dtype} m={m} n={n} k={k} kernel={hip.last_kernel_name()}")
        seen.add(hip.last_kernel_name().split("_")[1])
    print("kernel families met:", sorted(seen), flush=True)
    assert len(seen) >= 3, seen
