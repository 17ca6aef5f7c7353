"""Behaviour of the drop-in boundary that a host runtime relies on and the reference states for its
own backends: one context shared by host threads that each drive their own stream
(`HipBackend: Send + Sync`, src/compat/hip_backend.rs), stream capture of a decode step
(the reference's mega-kernel is launched once per step, hip_backend.rs:224-236: a captured graph
plays that role here), and weights that stay resident between calls of the host-slice form
(Backend::quantized_matmul takes `&[u8]` every call, src/compat/cpu_backend.rs:991-1049).
Results are held to the bars of the other GPU tests: equal bit for bit to the same call made
alone, which itself is checked against the oracle."""
import threading

import numpy as np
import pytest

from gllm_amd.synth import random_activations, random_weight
from tests.test_gpu_parity import check_close

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def dev(torch, a):
    return torch.from_numpy(np.asarray(a).view(np.uint8).reshape(-1)).cuda()


# shapes whose kernels use the context's scratch: a K split across workgroups (partial sums and
# arrival counters), a 16-row GEMM (activation images, partial sums, a reduce launch), and the
# feed-forward block (its hidden state); plus a plain one-row matmul
SHAPES = [(Q4_K, 2, 256, 8192), (Q5_K, 16, 512, 1024), (Q6_K, 1, 96, 14336), (Q4_K, 1, 3072, 1024)]


def test_two_threads_two_streams_one_context(torch, oracle):
    from gllm_amd.backend import HipBackend
    hip = HipBackend(0)
    hidden, ffn = 1024, 1536
    weights = [dev(torch, random_weight(dt, n, k, seed=i)) for i, (dt, m, n, k) in enumerate(SHAPES)]
    wg, wu = dev(torch, random_weight(Q4_K, ffn, hidden, seed=20)), dev(torch, random_weight(Q4_K, ffn, hidden, seed=21))
    wd = dev(torch, random_weight(Q6_K, hidden, ffn, seed=22))
    rounds, workers = 40, 2

    def inputs(worker, r):
        xs = [torch.from_numpy(random_activations(m, k, seed=1000 * worker + 10 * r + i)).cuda()
              for i, (dt, m, n, k) in enumerate(SHAPES)]
        return xs, torch.from_numpy(random_activations(1, hidden, seed=5000 + 100 * worker + r)).cuda()

    def run(xs, xf):
        outs = []
        for (dt, m, n, k), w, x in zip(SHAPES, weights, xs):
            y = torch.full((m, n), float("nan"), device="cuda")
            hip.quantized_matmul(w, x, y, dt, m, n, k)
            outs.append(y)
        h = torch.full((1, hidden), float("nan"), device="cuda")
        hip.ffn_swiglu(wg, wu, Q4_K, wd, Q6_K, xf, h, 1, hidden, ffn)
        outs.append(h)
        return outs

    # what every call gives when nothing else runs; the first round of each worker also against the oracle
    print("boundary: single-threaded expectations", flush=True)
    data = {(wk, r): inputs(wk, r) for wk in range(workers) for r in range(rounds)}
    want = {key: [o.clone() for o in run(*val)] for key, val in data.items()}
    torch.cuda.synchronize()
    for wk in range(workers):
        xs, _ = data[(wk, 0)]
        for (dt, m, n, k), x, y, i in zip(SHAPES, xs, want[(wk, 0)], range(len(SHAPES))):
            ref = oracle.quantized_matmul(random_weight(dt, n, k, seed=i), x.cpu().numpy(), dt, m, n, k, acc=oracle.ACC_F64, threads=8)
            check_close(y.cpu().numpy(), ref, f"worker {wk} shape {i}")

    failures = []
    go = threading.Barrier(workers)

    def worker(wk):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                go.wait()
                for r in range(rounds):
                    got = run(*data[(wk, r)])
                    stream.synchronize()
                    for i, (g, w_) in enumerate(zip(got, want[(wk, r)])):
                        if not torch.equal(g, w_):
                            failures.append(f"worker {wk} round {r} output {i} differs from the call made alone")
        except Exception as e:  # noqa: BLE001 - reported below, in the main thread
            failures.append(f"worker {wk}: {type(e).__name__}: {e}")

    print("boundary: two threads, two streams", flush=True)
    threads = [threading.Thread(target=worker, args=(wk,)) for wk in range(workers)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert not any(t.is_alive() for t in threads), "a worker did not finish"
    assert not failures, failures[:5]


def test_capture_needs_reserved_scratch(torch):
    """A stream the context has not worked on owns no scratch, and none can be allocated while the
    stream is being captured: the call fails with a message that names the remedy, records nothing
    and leaves the capture usable.  After gllmq_reserve_* on that stream the same capture works,
    and its replays give the eager results."""
    from gllm_amd.backend import BackendError, HipBackend
    hip = HipBackend(0)
    dt, m, n, k = Q5_K, 16, 512, 1024  # a GEMM: activation images and partial sums live in scratch
    w = dev(torch, random_weight(dt, n, k, seed=1))
    x = torch.from_numpy(random_activations(m, k, seed=2)).cuda()
    y = torch.full((m, n), float("nan"), device="cuda")
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    print("boundary: capture without scratch", flush=True)
    graph = torch.cuda.CUDAGraph()
    refused = None
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            try:
                hip.quantized_matmul(w, x, y, dt, m, n, k)
            except BackendError as e:
                refused = str(e)
    torch.cuda.synchronize()
    assert refused is not None and "reserve" in refused, refused

    print("boundary: reserve, then capture", flush=True)
    with torch.cuda.stream(side):
        hip.reserve_matmul(dt, m, n, k)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            hip.quantized_matmul(w, x, y, dt, m, n, k)
    torch.cuda.synchronize()
    eager = torch.empty_like(y)
    for seed in (3, 4, 5):
        x.copy_(torch.from_numpy(random_activations(m, k, seed=seed)))
        hip.quantized_matmul(w, x, eager, dt, m, n, k)
        torch.cuda.synchronize()
        y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), f"replay with inputs {seed} differs from the eager call"


def test_capture_of_16_bit_elements_through_the_conversion_launches(torch):
    """A 16-bit call whose kernel reads f32 only (few weight rows: the K-split form) needs room for
    the widened copies: refused under capture on a fresh stream, fine after reserve_matmul with the
    element type; replays equal the eager call."""
    from gllm_amd.backend import BackendError, ELEM_BF16, HipBackend
    hip = HipBackend(0)
    dt, m, n, k = Q4_K, 2, 256, 8192
    w = dev(torch, random_weight(dt, n, k, seed=1))
    x = torch.from_numpy(random_activations(m, k, seed=2)).cuda().to(torch.bfloat16)
    y = torch.zeros(m, n, device="cuda", dtype=torch.bfloat16)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    print("boundary: 16-bit capture without scratch", flush=True)
    graph = torch.cuda.CUDAGraph()
    refused = None
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            try:
                hip.quantized_matmul(w, x, y, dt, m, n, k)
            except BackendError as e:
                refused = str(e)
    torch.cuda.synchronize()
    assert refused is not None and "reserve" in refused, refused
    print("boundary: 16-bit reserve, then capture", flush=True)
    with torch.cuda.stream(side):
        hip.reserve_matmul(dt, m, n, k, elem=ELEM_BF16)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            hip.quantized_matmul(w, x, y, dt, m, n, k)
    torch.cuda.synchronize()
    eager = torch.empty_like(y)
    for seed in (3, 4):
        x.copy_(torch.from_numpy(random_activations(m, k, seed=seed)).to(torch.bfloat16))
        hip.quantized_matmul(w, x, eager, dt, m, n, k)
        torch.cuda.synchronize()
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), eager.view(torch.int16)), f"replay with inputs {seed} differs from the eager call"


def test_host_slices_are_uploaded_once(torch, oracle):
    """The reference's signature hands over host slices on every call; the same weight slice is
    copied to the device on its first use only, until the caller says it has changed."""
    from gllm_amd.backend import HipBackend
    hip = HipBackend(0)
    dt, n, k = Q4_K, 700, 2048
    w = random_weight(dt, n, k, seed=8)
    before = hip.weight_uploads()
    outs = []
    for seed in (1, 2, 3):
        print(f"boundary: host-slice call {seed}", flush=True)
        x = random_activations(1, k, seed=seed)
        y = np.empty((1, n), np.float32)
        hip.quantized_matmul(w, x, y, dt, 1, n, k)
        check_close(y, oracle.quantized_matmul(w, x, dt, 1, n, k, acc=oracle.ACC_F64, threads=4), f"host call {seed}")
        outs.append(y)
    assert hip.weight_uploads() == before + 1
    # the caller rewrites the buffer in place and says so: the next call uploads again and sees the new bytes
    w2 = random_weight(dt, n, k, seed=9)
    np.asarray(w).view(np.uint8).reshape(-1)[:] = np.asarray(w2).view(np.uint8).reshape(-1)
    hip.weights_forget(w)
    x = random_activations(1, k, seed=1)
    y = np.empty((1, n), np.float32)
    hip.quantized_matmul(w, x, y, dt, 1, n, k)
    assert hip.weight_uploads() == before + 2
    check_close(y, oracle.quantized_matmul(w2, x, dt, 1, n, k, acc=oracle.ACC_F64, threads=4), "after weights_forget")
    assert not np.array_equal(y, outs[0])
