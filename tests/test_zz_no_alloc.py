"""The quantized matmul through the entry point that allocates nothing
(gllmq_quantized_matmul_noalloc, scratch in a fixed device array) against
gllmq_quantized_matmul on the same inputs, through the C ABI: same kernels and launch shapes, so
the outputs must be equal bit for bit.  Pairs of calls in a row, the second with a smaller input,
over the kernels that use scratch: the GEMM with its K split (activation images, partial sums)
and the 8-row kernels' K split (slice sums, arrival counters)."""
import numpy as np
import pytest

from gllm_amd.ggml import row_bytes
from gllm_amd.synth import random_activations, random_weight

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14


@pytest.fixture(scope="module")
def hip():
    from gllm_amd.backend import HipBackend
    return HipBackend(0)


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def both(hip, torch, dtype, m, n, k, seed):
    w = torch.from_numpy(random_weight(dtype, n, k, seed=seed)).cuda()
    x = torch.from_numpy(random_activations(m, k, seed=seed + 1)).cuda()
    want = torch.full((m, n), float("nan"), device="cuda")
    got = torch.full((m, n), float("nan"), device="cuda")
    hip.quantized_matmul(w, x, want, dtype, m, n, k)
    hip.quantized_matmul_noalloc(w, x, got, dtype, m, n, k)
    torch.cuda.synchronize()
    assert not bool(torch.isnan(want).any())
    assert torch.equal(got.view(torch.int32), want.view(torch.int32)), f"dtype={dtype} m={m} n={n} k={k}"


@pytest.mark.parametrize("dtype", [Q4_K, Q5_K, Q6_K, Q8_0])
def test_two_calls_in_a_row_second_smaller(hip, torch, dtype):
    # GEMM with a K split: 8 row tiles share the device, partial sums meet in the scratch
    for m, n, k in ((32, 2048, 4096), (16, 520, 2048)):
        print(f"noalloc GEMM dtype={dtype} m={m} n={n} k={k}", flush=True)
        both(hip, torch, dtype, m, n, k, seed=3 * m)
    # few weight rows of long rows on the 8-row kernels: K split with slice sums and arrival
    # counters in the scratch; then smaller; then the same shape again (counters back at zero)
    for m, n, k in ((4, 1024, 8192), (2, 256, 4096), (4, 1024, 8192)):
        print(f"noalloc K split dtype={dtype} m={m} n={n} k={k}", flush=True)
        both(hip, torch, dtype, m, n, k, seed=5 * m)
    # the streamed kernels' slices of K (sums and counters in the scratch as well): 32-row tiles
    # for half of the CUs, long rows; then smaller; then again
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    for m, n, k in ((2, 16 * cus, 8192 + 512), (3, 16 * cus - 40, 8192), (2, 16 * cus, 8192 + 512)):
        print(f"noalloc streamed K split dtype={dtype} m={m} n={n} k={k}", flush=True)
        both(hip, torch, dtype, m, n, k, seed=7 * m)
        if dtype != Q6_K or m == 2:
            assert hip.last_kernel_name().endswith("_s"), hip.last_kernel_name()
    # shapes without scratch go through the same entry point (also one row in pairs of blocks)
    both(hip, torch, dtype, 1, 777, 1024, seed=9)
    both(hip, torch, dtype, 1, 12 * cus, 4096, seed=10)


def test_baseline_shapes_fit(hip, torch):
    for m in (16, 64):
        print(f"noalloc baseline GEMM m={m}", flush=True)
        both(hip, torch, Q4_K, m, 14336, 4096, seed=m)
    both(hip, torch, Q6_K, 32, 4096, 14336, seed=7)


def test_too_large_a_shape_is_refused_and_nothing_runs(hip, torch):
    from gllm_amd.backend import OtherError
    m, n, k = 64, 16384, 65536
    print("noalloc: refusal", flush=True)
    w = torch.empty(n * row_bytes(Q4_K, k), dtype=torch.uint8, device="cuda")
    x = torch.zeros(m, k, device="cuda")
    y = torch.full((m, n), 5.0, device="cuda")
    with pytest.raises(OtherError, match="scratch"):
        hip.quantized_matmul_noalloc(w, x, y, Q4_K, m, n, k)
    torch.cuda.synchronize()
    assert bool((y == 5.0).all())
    # and the entry point still works afterwards
    both(hip, torch, Q4_K, 16, 520, 2048, seed=11)


def test_first_call_of_a_fresh_context_under_capture_allocates_nothing(torch):
    """A new context whose very first call is the no-alloc entry point, made while its stream is
    being captured: the scratch array was placed at init, so the call records kernels only; the
    replays (with a smaller shape in the same graph) give the bits of the allocating entry point.
    (The capture runs in torch's default mode, in which an allocation by the capturing thread is an
    error.)  And the very first, eager, call of another new context leaves the device's free memory
    where it was: nothing is placed on the device by the call itself."""
    from gllm_amd.backend import HipBackend
    fresh = HipBackend(0)
    ref = HipBackend(0)
    shapes = ((32, 2048, 4096), (4, 1024, 8192), (16, 520, 2048))  # GEMM with K split, 8-row K split, smaller GEMM
    ws = [torch.from_numpy(random_weight(Q4_K, n, k, seed=21 + i)).cuda() for i, (m, n, k) in enumerate(shapes)]
    xs = [torch.empty(m, k, device="cuda") for m, n, k in shapes]
    got = [torch.full((m, n), float("nan"), device="cuda") for m, n, k in shapes]
    want = [torch.full((m, n), float("nan"), device="cuda") for m, n, k in shapes]
    eager_first = HipBackend(0)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    print("noalloc: first call of a fresh context, eager", flush=True)
    for (m, n, k), w, x, y in zip(shapes, ws, xs, got):
        x.fill_(1.0)
        eager_first.quantized_matmul_noalloc(w, x, y, Q4_K, m, n, k)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the first calls of a new context changed the device's free memory"
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    print("noalloc: first call of a fresh context under capture", flush=True)
    with torch.cuda.stream(side):
        graph.capture_begin()
        for (m, n, k), w, x, y in zip(shapes, ws, xs, got):
            fresh.quantized_matmul_noalloc(w, x, y, Q4_K, m, n, k)
        graph.capture_end()
    torch.cuda.synchronize()
    for rep in range(3):
        for i, ((m, n, k), x) in enumerate(zip(shapes, xs)):
            x.copy_(torch.from_numpy(random_activations(m, k, seed=100 * rep + i)).cuda())
        for y in got:
            y.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for (m, n, k), w, x, y, z in zip(shapes, ws, xs, got, want):
            ref.quantized_matmul(w, x, z, Q4_K, m, n, k)
        torch.cuda.synchronize()
        for (m, n, k), y, z in zip(shapes, got, want):
            assert not bool(torch.isnan(z).any())
            assert torch.equal(y.view(torch.int32), z.view(torch.int32)), f"replay {rep} m={m} n={n} k={k}"
    # eager calls afterwards: still nothing allocated by the entry point
    free_mid = torch.cuda.mem_get_info()[0]
    for (m, n, k), w, x, y in zip(shapes, ws, xs, got):
        fresh.quantized_matmul_noalloc(w, x, y, Q4_K, m, n, k)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_mid
