"""Writes tests/golden/kquant_golden.npz: small fixed inputs and expected outputs for the
four block formats, the matmul and the routing rule.

The expected values come from the per-element numpy decoders in oracle/npref.py (the
formulas of docs/domain-knowledge/quant-kquant-iq-proprietary.md:40-64,123-154 and
gguf-classic-quant-layout.md:33-64 of the reference, evaluated element by element), NOT
from the C restatement or the GPU code that the tests then compare against them.  No
reference code is run: its implementation of this path (crate gllm-kernels 0.1.0) is not
part of the reference tree.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from gllm_amd.synth import random_activations, random_gate_logits, random_weight  # noqa: E402
from oracle import npref  # noqa: E402

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
DEQ = {Q8_0: npref.dequant_q8_0, Q4_K: npref.dequant_q4_k, Q5_K: npref.dequant_q5_k, Q6_K: npref.dequant_q6_k}
TAG = {Q8_0: "q8_0", Q4_K: "q4_k", Q5_K: "q5_k", Q6_K: "q6_k"}


def main():
    out = {}
    for dtype in (Q8_0, Q4_K, Q5_K, Q6_K):
        n, k, m = 6, 512, 3
        w = random_weight(dtype, n, k, seed=1000 + dtype)
        x = random_activations(m, k, seed=2000 + dtype)
        deq = DEQ[dtype](w).reshape(n, k)
        y = x.astype(np.float64) @ deq.astype(np.float64).T
        t = TAG[dtype]
        out[f"{t}_blocks"] = w
        out[f"{t}_dequant_bits"] = deq.view(np.uint32)
        out[f"{t}_x"] = x
        out[f"{t}_y_f64"] = y
        out[f"{t}_shape_mnk"] = np.array([m, n, k], np.int64)
    # routing: softmax -> stable descending sort -> top-k -> renormalise (src/moe/routing.rs:263-302)
    logits = random_gate_logits(5, 12, seed=7)
    idx = np.zeros((5, 3), np.uint32)
    wts = np.zeros((5, 3), np.float32)
    for t in range(5):
        i, w_ = npref.topk_with_weights(logits[t], 3)
        idx[t], wts[t] = i, w_
    out["route_logits"] = logits
    out["route_topk_idx"] = idx
    out["route_topk_weight"] = wts
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kquant_golden.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
