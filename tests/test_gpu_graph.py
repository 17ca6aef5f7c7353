"""The library's launches inside a HIP graph: once a context's scratch buffers exist (one eager
call of each shape), its entry points enqueue kernels only, so a stream capture records them and
replays give the eager results.  Every replay is checked, with eager work and synchronisations
between the replays."""
import numpy as np
import pytest

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


def test_graph_replays_match_eager(hip, torch):
    hidden, ffn, vocab = 1024, 1536, 3000
    dev = lambda a: torch.from_numpy(np.asarray(a).view(np.uint8).reshape(-1)).cuda()
    wq = dev(random_weight(Q4_K, 3 * hidden, hidden, seed=1))   # a QKV-like projection, one row
    wg, wu = dev(random_weight(Q4_K, ffn, hidden, seed=2)), dev(random_weight(Q4_K, ffn, hidden, seed=3))
    wd = dev(random_weight(Q6_K, hidden, ffn, seed=4))
    wo = dev(random_weight(Q6_K, vocab, hidden, seed=5))          # lm_head
    wb = dev(random_weight(Q5_K, 512, hidden, seed=6))            # a 16-row GEMM (prepare, GEMM, reduce)
    ws = dev(random_weight(Q4_K, 256, 8 * hidden, seed=7))        # few rows of long rows: K split across workgroups
    xs = torch.empty(2, 8 * hidden, device="cuda")
    ys = torch.empty(2, 256, device="cuda")
    x = torch.empty(1, hidden, device="cuda")
    xb = torch.empty(16, hidden, device="cuda")
    qkv = torch.empty(1, 3 * hidden, device="cuda")
    h = torch.empty(1, hidden, device="cuda")
    logits = torch.empty(1, vocab, device="cuda")
    yb = torch.empty(16, 512, device="cuda")
    tok = torch.zeros(1, dtype=torch.int32, device="cuda")
    tok2 = torch.zeros(1, dtype=torch.int32, device="cuda")      # lm_head and token as one launch (a ticket counter in scratch)
    xh = torch.empty(1, hidden, device="cuda", dtype=torch.bfloat16)
    yh = torch.empty(1, 3 * hidden, device="cuda", dtype=torch.bfloat16)  # bf16 activations and outputs
    wg6, wu6 = dev(random_weight(Q6_K, ffn, hidden, seed=8)), dev(random_weight(Q6_K, ffn, hidden, seed=9))
    h6 = torch.empty(1, hidden, device="cuda")                    # gate applied in the down projection's loads
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    wf = dev(random_weight(Q5_K, 12 * cus, 4 * hidden, seed=10))  # one row over low tiles: pairs of blocks
    xf, yf = torch.empty(1, 4 * hidden, device="cuda"), torch.empty(1, 12 * cus, device="cuda")
    wk = dev(random_weight(Q4_K, 16 * cus, 8 * hidden + 256, seed=11))  # three long rows over few weight rows: streamed slices of K
    xk, yk = torch.empty(3, 8 * hidden + 256, device="cuda"), torch.empty(3, 16 * cus, device="cuda")

    def step():
        hip.quantized_matmul(wq, x, qkv, Q4_K, 1, 3 * hidden, hidden)
        hip.ffn_swiglu(wg, wu, Q4_K, wd, Q6_K, x, h, 1, hidden, ffn)
        hip.quantized_matmul(wo, h, logits, Q6_K, 1, vocab, hidden)
        hip.argmax(logits, tok)
        hip.lm_head_argmax(wo, h, Q6_K, vocab, hidden, tok2)
        hip.quantized_matmul(wq, xh, yh, Q4_K, 1, 3 * hidden, hidden)
        hip.ffn_swiglu(wg6, wu6, Q6_K, wd, Q6_K, x, h6, 1, hidden, ffn)
        hip.quantized_matmul(wb, xb, yb, Q5_K, 16, 512, hidden)
        hip.quantized_matmul(ws, xs, ys, Q4_K, 2, 256, 8 * hidden)
        hip.quantized_matmul(wf, xf, yf, Q5_K, 1, 12 * cus, 4 * hidden)
        assert hip.last_kernel_name().endswith("_f"), hip.last_kernel_name()
        hip.quantized_matmul(wk, xk, yk, Q4_K, 3, 16 * cus, 8 * hidden + 256)
        assert hip.last_kernel_name().endswith("_s"), hip.last_kernel_name()

    def fill(seed):
        x.copy_(torch.from_numpy(random_activations(1, hidden, seed=seed)))
        xb.copy_(torch.from_numpy(random_activations(16, hidden, seed=seed + 50)))
        xs.copy_(torch.from_numpy(random_activations(2, 8 * hidden, seed=seed + 90)))
        xh.copy_(x.to(torch.bfloat16))
        xf.copy_(torch.from_numpy(random_activations(1, 4 * hidden, seed=seed + 120)))
        xk.copy_(torch.from_numpy(random_activations(3, 8 * hidden + 256, seed=seed + 150)))

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        fill(0)
        step()  # eager once: scratch buffers are allocated here, not under capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.synchronize()
    for seed in (1, 2, 3, 4):
        print(f"graph replay with inputs {seed}", flush=True)
        fill(seed)
        step()
        torch.cuda.synchronize()
        outs = (qkv, h, logits, yb, ys, tok, tok2, yh, h6, yf, yk)
        want = [t.clone() for t in outs]
        assert int(tok2[0]) == int(tok[0])
        for t in (qkv, h, logits, yb, ys, yh, h6, yf, yk):
            t.fill_(float("nan"))
        tok.fill_(-7)
        tok2.fill_(-7)
        # eager work of the program's own between the replays
        hip.quantized_matmul(wq, x, torch.empty(1, 3 * hidden, device="cuda"), Q4_K, 1, 3 * hidden, hidden)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, exp in zip(outs, want):
            assert torch.equal(got, exp), f"replay {seed} differs from the eager run"
