"""Oracle pin for the dense feed-forward block: the C restatement against a float64 numpy
evaluation of the reference's formula down(silu(gate x) * (up x)) (SPEC 04-OPERATORS.md:114)
on the numpy twin's dequantized weights, and against closed forms."""
import numpy as np
import pytest

from gllm_amd.synth import random_activations, random_weight
from oracle import npref

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14


def numpy_ffn(gate, up, t_gu, down, t_dn, x, hidden, ffn, relu=False):
    wg = npref.dequantize(gate, t_gu).reshape(ffn, -1)[:, :hidden].astype(np.float64)
    wu = npref.dequantize(up, t_gu).reshape(ffn, -1)[:, :hidden].astype(np.float64)
    wd = npref.dequantize(down, t_dn).reshape(hidden, -1)[:, :ffn].astype(np.float64)
    g = x.astype(np.float64) @ wg.T
    if relu:
        g = np.maximum(g, 0.0)
    with np.errstate(over="ignore"):  # exp(-g) overflows to inf for very negative gates: silu is -0 there
        h = g / (1.0 + np.exp(-g)) * (x.astype(np.float64) @ wu.T)
    return h @ wd.T


@pytest.mark.parametrize("t_gu,t_dn", [(Q4_K, Q6_K), (Q5_K, Q4_K), (Q6_K, Q8_0), (Q8_0, Q5_K)])
@pytest.mark.parametrize("relu", [False, True])
def test_matches_float64_formula(oracle, t_gu, t_dn, relu):
    m, hidden, ffn = 3, 512, 768
    gate, up = random_weight(t_gu, ffn, hidden, seed=1), random_weight(t_gu, ffn, hidden, seed=2)
    down = random_weight(t_dn, hidden, ffn, seed=3)
    x = random_activations(m, hidden, seed=4)
    want = numpy_ffn(gate, up, t_gu, down, t_dn, x, hidden, ffn, relu)
    got = oracle.ffn_swiglu(gate, up, t_gu, down, t_dn, x, m, hidden, ffn, relu_gate=relu, acc=oracle.ACC_F64)
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert rel < 2e-6, rel


def test_zero_gate_gives_zero_and_relu_kills_negative_gates(oracle):
    """silu(0) = 0: a gate matrix that decodes to zeros silences the block whatever up and down
    hold; with the ReLU flag a gate that is negative everywhere does the same."""
    m, hidden, ffn = 2, 256, 256
    up, down = random_weight(Q8_0, ffn, hidden, seed=5), random_weight(Q8_0, hidden, ffn, seed=6)
    x = np.abs(random_activations(m, hidden, seed=7))  # positive activations
    gate0 = np.zeros((ffn, hidden // 32, 34), np.uint8)  # d = 0, q = 0
    out = oracle.ffn_swiglu(gate0, up, Q8_0, down, Q8_0, x, m, hidden, ffn)
    assert np.all(out == 0.0)
    gneg = np.zeros((ffn, hidden // 32, 34), np.uint8)
    gneg[:, :, 0:2] = np.array([2.0 ** -8], np.float16).view(np.uint8)  # gate . x of about -0.8
    gneg[:, :, 2:] = np.uint8(0xFF)  # q = -1 everywhere: gate . x < 0 for positive x
    out = oracle.ffn_swiglu(gneg, up, Q8_0, down, Q8_0, x, m, hidden, ffn, relu_gate=True)
    assert np.all(out == 0.0)
    assert np.any(oracle.ffn_swiglu(gneg, up, Q8_0, down, Q8_0, x, m, hidden, ffn, relu_gate=False) != 0.0)
