"""Committed fixtures (tests/golden/kquant_golden.npz, written by tests/golden/make_golden.py
from the per-element numpy decoders) against the C oracle on the CPU and against the HIP
library on the GPU."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kquant_golden.npz")
FORMATS = [(8, "q8_0"), (12, "q4_k"), (13, "q5_k"), (14, "q6_k")]


@pytest.fixture(scope="module")
def golden():
    with np.load(GOLDEN, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


@pytest.mark.parametrize("dtype,tag", FORMATS)
def test_oracle_matches_golden(oracle, golden, dtype, tag):
    m, n, k = (int(v) for v in golden[f"{tag}_shape_mnk"])
    w, x = golden[f"{tag}_blocks"], golden[f"{tag}_x"]
    deq = oracle.dequantize(w, dtype)
    assert np.array_equal(deq.view(np.uint32).reshape(n, k), golden[f"{tag}_dequant_bits"])
    for acc in (oracle.ACC_F64, oracle.ACC_F32):
        y = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=acc)
        want = golden[f"{tag}_y_f64"]
        assert np.linalg.norm(y - want) / np.linalg.norm(want) < 2e-6


def test_oracle_routing_matches_golden(oracle, golden):
    logits = golden["route_logits"]
    for t in range(logits.shape[0]):
        idx, w = oracle.topk_with_weights(logits[t], 3)
        assert np.array_equal(idx, golden["route_topk_idx"][t])
        assert np.allclose(w, golden["route_topk_weight"][t], rtol=2e-6, atol=0)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tag", FORMATS)
def test_hip_matches_golden(golden, dtype, tag):
    import torch

    from gllm_amd.backend import HipBackend
    hip = HipBackend(0)
    m, n, k = (int(v) for v in golden[f"{tag}_shape_mnk"])
    w, x = golden[f"{tag}_blocks"], golden[f"{tag}_x"]
    print(f"golden dtype={dtype}", flush=True)
    wd = hip.upload_weights(w)
    od = torch.zeros(n * k, dtype=torch.float32, device="cuda")
    hip.dequantize(wd, od, dtype)
    assert np.array_equal(od.cpu().numpy().view(np.uint32).reshape(n, k), golden[f"{tag}_dequant_bits"])
    xd = torch.from_numpy(x).cuda()
    yd = torch.zeros(m, n, dtype=torch.float32, device="cuda")
    hip.quantized_matmul(wd, xd, yd, dtype, m, n, k)
    torch.cuda.synchronize()
    got, want = yd.cpu().numpy().astype(np.float64), golden[f"{tag}_y_f64"]
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-4
    assert np.abs(got - want).max() <= 1e-3 * np.abs(want).max()
