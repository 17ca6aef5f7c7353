"""GPU parity over the dynamic range of the activations, for every kernel family behind
Backend::quantized_matmul (src/compat/cpu_backend.rs:991-1049), the feed-forward block and the
expert matvec, against the oracle's float64 accumulation.

The kernels do not multiply f32 by f32 as the reference does: the int8 families turn every
256-element block (64-element part in the integer-dot GEMV) of an activation row into 23-bit
integers under one power-of-two scale, the f16 family into a hi and a lo f16 plane under one scale.
What that costs is bounded here, per output element, by

    |y - y64| <= 2^-22 * sum_b max_b|x| * sum_{j in b} W+_j          (block fixed point)
               + c * 2^-24 * sum_j W+_j |x_j|                        (f32 finishing and sums)
               + 2^-147 * sum_j W+_j                                 (subnormal floor)

with W+ the magnitudes of the terms a kernel forms apart (oracle.npref.term_magnitudes) and c the
number of f32 roundings on the way of one output (32 + k/2048 for the int8 families, 64 + k/256
for the f16 matrix-core GEMM, 160 for the f32 multiply-add GEMV).  The bound is asserted for every
case; the matmul bar (rel-L2 <= 1e-4, |err| <= 1e-3 max|y|) is asserted for every case except
the row built to cancel (+2^20 and -2^20 on two elements whose weights are equal, unit-size values
elsewhere): there y is the size of the small terms while every partial sum that holds one of the
pair is 2^20 times larger, and a bar relative to y is beyond f32 arithmetic in general: the
oracle's f32 reference-style accumulation misses it on the same input (rel-L2 3e-4 to 6e-4).
"""
import numpy as np
import pytest

from gllm_amd.synth import random_weight
from tests.test_gpu_parity import check_close, gpu_matmul

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
ALL = [Q8_0, Q4_K, Q5_K, Q6_K]


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def activations(kind, m, k, seed):
    """m x k float32 activations of one of the patterns; returns (x, meets the matmul bar)."""
    rng = np.random.default_rng(seed)
    base = rng.standard_normal((m, k))
    nb = (k + 255) // 256
    block_of = np.arange(k) // 256
    if kind == "heavy_tailed":  # Cauchy, clipped: a few values per block thousands of times the rest
        return np.clip(rng.standard_cauchy((m, k)), -1e4, 1e4).astype(np.float32), True
    if kind == "outlier_per_block":  # one +-2^20 in every block of unit-size values
        x = base.copy()
        for r in range(m):
            pos = rng.integers(0, 256, nb) + 256 * np.arange(nb)
            pos = pos[pos < k]
            x[r, pos] = (2.0 ** 20) * rng.choice([-1.0, 1.0], pos.size)
        return x.astype(np.float32), True
    if kind == "subnormal_blocks":  # every third block holds only subnormal values
        x = base.copy()
        x[:, block_of % 3 == 1] *= 1e-41
        return x.astype(np.float32), True
    if kind == "all_subnormal":  # nothing but subnormal values (about 2^-133 .. 2^-128)
        return (base * 1e-40).astype(np.float32), True
    if kind == "zero_blocks":  # every other block zero, and (with several rows) one row all zero
        x = base.copy()
        x[:, block_of % 2 == 0] = 0.0
        if m > 1:
            x[m - 1] = 0.0
        return x.astype(np.float32), True
    if kind == "cancelling":  # +2^20 and -2^20 in the middle of the row, on two elements whose weights are made equal
        x = base.copy()
        p = cancel_position(k)
        x[:, p], x[:, p + 1] = 2.0 ** 20, -(2.0 ** 20)
        return x.astype(np.float32), False
    if kind == "scale_1e-30":
        return (base * 1e-30).astype(np.float32), True
    if kind == "scale_1e+30":
        return (base * 1e30).astype(np.float32), True
    raise KeyError(kind)


def cancel_position(k):
    """An even element in the middle of the row whose right neighbour shares its sub-block in every format."""
    return 256 * ((k // 256) // 2) + 70


def with_equal_pair(npref, w, dtype, n, k, p):
    """`w` with element p + 1 of every row made a copy of element p (quant bits copied; p and p + 1
    share their scales), so that equal and opposite activations on the two cancel exactly."""
    bb, bs = npref.BLOCK_BYTES[dtype], npref.BLOCK_SIZE[dtype]
    a = np.array(w, copy=True).view(np.uint8).reshape(n, -(-k // bs), bb)
    b, i = a[:, p // bs, :], p % bs

    def copy_bits(src, dst, mask):
        b[:, dst] = (b[:, dst] & np.uint8(~mask & 0xFF)) | (b[:, src] & np.uint8(mask))

    if dtype in (Q4_K, Q5_K):
        sub, l = i // 32, i % 32
        byte = (16 if dtype == Q4_K else 48) + 32 * (sub // 2) + l
        copy_bits(byte, byte + 1, 0x0F if sub % 2 == 0 else 0xF0)
        if dtype == Q5_K:
            copy_bits(16 + l, 16 + l + 1, 1 << sub)
    elif dtype == Q6_K:
        half, quarter, l = i // 128, (i % 128) // 32, i % 32
        byte = 64 * half + l + 32 * (quarter % 2)
        copy_bits(byte, byte + 1, 0xF0 if quarter >= 2 else 0x0F)
        copy_bits(128 + 32 * half + l, 128 + 32 * half + l + 1, 3 << (2 * quarter))
    else:
        copy_bits(2 + i, 2 + i + 1, 0xFF)
    out = a.reshape(-1)
    wf = npref.dequantize(out, dtype).reshape(n, -1)
    assert np.array_equal(wf[:, p], wf[:, p + 1])
    return out


KINDS = ["heavy_tailed", "outlier_per_block", "subnormal_blocks", "all_subnormal", "zero_blocks", "cancelling",
         "scale_1e-30", "scale_1e+30"]


def error_bound(npref, w, x, dtype, n, k, roundings):
    bs = npref.BLOCK_SIZE[dtype]
    kp = -(-k // bs) * bs
    wp = npref.term_magnitudes(w, dtype).reshape(n, kp)[:, :k]
    ax = np.abs(np.asarray(x, np.float64))
    nb = (k + 255) // 256
    pad = nb * 256 - k
    axp = np.pad(ax, ((0, 0), (0, pad)))
    wpp = np.pad(wp, ((0, 0), (0, pad)))
    block_max = axp.reshape(-1, nb, 256).max(axis=2)          # m x nb
    block_w = wpp.reshape(n, nb, 256).sum(axis=2)             # n x nb
    return (2.0 ** -22) * (block_max @ block_w.T) + roundings * (2.0 ** -24) * (ax @ wp.T) + (2.0 ** -147) * wp.sum(axis=1)[None, :]


# (name, options, activation rows, weight rows as a function of the CU count, k, formats, roundings(k), kernel-name prefix)
FAMILIES = [
    ("streamed int8", {"mm8s_all": 1}, 1, lambda c: 8 * c + 5, 4096, [Q4_K, Q5_K, Q6_K], lambda k: 32 + k / 2048, "gq_mm8s_"),
    ("streamed int8 long rows", {"mm8s_all": 1}, 2, lambda c: 8 * c, 14336, [Q4_K, Q6_K], lambda k: 32 + k / 2048, "gq_mm8s_"),
    ("int8 matrix cores", {"mm8s": 0, "mm8_q5k_min_m": 1, "mm8_q6k_min_m": 1, "mm8_q8_0_min_m": 1}, 4, lambda c: 300, 2048 + 256, ALL,
     lambda k: 32 + k / 2048, "gq_mm8_"),
    ("int8 matrix cores, K split", {"mm8s": 0, "mm8_q5k_min_m": 1, "mm8_q6k_min_m": 1, "mm8_small_to_gemv": 0}, 1, lambda c: 96, 14336, [Q4_K, Q5_K, Q6_K],
     lambda k: 40 + k / 2048, "gq_mm8_"),
    ("integer-dot GEMV", {"mm8": 0, "mmf": 0}, 2, lambda c: 257, 4096 - 64, ALL, lambda k: 32 + k / 2048, "gq_gemv_i8_"),
    ("f32 multiply-add GEMV", {"gemv_f32": 1, "mm8": 0, "mmf": 0}, 1, lambda c: 130, 2048, ALL, lambda k: 160, "gq_gemv_"),
    ("f16 matrix-core GEMM", {}, 24, lambda c: 520, 4096, ALL, lambda k: 64 + k / 256, "gq_mmf_"),
    ("f16 matrix-core GEMM, two row tiles", {}, 40, lambda c: 300, 1024 + 32, [Q4_K, Q6_K], lambda k: 64 + k / 256, "gq_mmf_"),
]


@pytest.mark.parametrize("family", FAMILIES, ids=[f[0] for f in FAMILIES])
def test_matmul_families_over_the_dynamic_range(torch, oracle, family):
    from gllm_amd.backend import HipBackend
    from oracle import npref
    name, options, m, rows, k, formats, roundings, prefix = family
    hip = HipBackend(0, options=options)
    n = rows(torch.cuda.get_device_properties(0).multi_processor_count)
    for dtype in formats:
        w = with_equal_pair(npref, random_weight(dtype, n, k, seed=dtype), dtype, n, k, cancel_position(k))
        for kind in KINDS:
            print(f"dynamic range: {name} dtype={dtype} m={m} n={n} k={k} {kind}", flush=True)
            x, meets_bar = activations(kind, m, k, seed=len(kind) + dtype)
            want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=16)
            got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
            assert hip.last_kernel_name().startswith(prefix), hip.last_kernel_name()
            assert np.isfinite(got).all(), f"{name} dtype={dtype} {kind}: non-finite output"
            err = np.abs(got.astype(np.float64) - want.astype(np.float64))
            bound = error_bound(npref, w, x, dtype, n, k, roundings(k))
            worst = float((err / np.maximum(bound, 1e-300)).max())
            assert worst <= 1.0, f"{name} dtype={dtype} {kind}: error is {worst:.2f} times the bound"
            if meets_bar:
                check_close(got, want, f"{name} dtype={dtype} {kind}")


BENIGN = ["heavy_tailed", "outlier_per_block", "subnormal_blocks", "zero_blocks"]


@pytest.mark.parametrize("m", [1, 4, 12])
def test_ffn_over_the_dynamic_range(torch, oracle, m):
    """The feed-forward block (fused gate/up + activation, then down) on the patterns whose
    outputs the bar applies to; the hidden state between the two matmuls goes through the same
    block fixed point as the input."""
    from gllm_amd.backend import HipBackend
    from tests.test_gpu_ffn import check, run_ffn
    hip = HipBackend(0)
    hidden, ffn = 2048, 1536
    gate, up = random_weight(Q4_K, ffn, hidden, seed=1), random_weight(Q4_K, ffn, hidden, seed=2)
    down = random_weight(Q6_K, hidden, ffn, seed=3)
    for kind in BENIGN + ["scale_1e-30"]:
        print(f"dynamic range: ffn m={m} {kind}", flush=True)
        x, _ = activations(kind, m, hidden, seed=7)
        if kind == "outlier_per_block":
            x = np.where(np.abs(x) > 1e3, np.sign(x) * 64.0, x).astype(np.float32)  # keeps gate * up inside f32
        if kind == "heavy_tailed":
            x = np.clip(x, -100.0, 100.0)
        want = oracle.ffn_swiglu(gate, up, Q4_K, down, Q6_K, x, m, hidden, ffn, acc=oracle.ACC_F64, threads=8)
        got = run_ffn(hip, torch, gate, up, Q4_K, down, Q6_K, x, m, hidden, ffn)
        assert np.isfinite(got).all()
        check(got, want, f"ffn m={m} {kind}")


def test_moe_over_the_dynamic_range(torch, oracle):
    from gllm_amd.backend import HipBackend
    from tests.test_gpu_moe import check_close as check_moe, expert_weights, route_gpu, run_gpu
    from gllm_amd.synth import random_gate_logits
    hip = HipBackend(0)
    experts, hidden, ffn, tokens, top_k = 8, 1024, 768, 12, 2
    gu, dn = expert_weights(Q4_K, Q6_K, experts, hidden, ffn, seed=5)
    _, r = route_gpu(hip, torch, oracle, random_gate_logits(tokens, experts, seed=2), top_k, capacity_factor=float(experts))
    for kind in BENIGN + ["scale_1e-30"]:
        print(f"dynamic range: moe {kind}", flush=True)
        x, _ = activations(kind, tokens, hidden, seed=11)
        if kind == "outlier_per_block":
            x = np.where(np.abs(x) > 1e3, np.sign(x) * 64.0, x).astype(np.float32)
        if kind == "heavy_tailed":
            x = np.clip(x, -100.0, 100.0)
        want = oracle.moe_ffn(gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, r["expert"], r["weight"], r["len"], threads=8)
        got = run_gpu(hip, torch, gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, r["expert"], r["weight"], r["len"])
        assert np.isfinite(got).all()
        check_moe(got, want, f"moe {kind}")
