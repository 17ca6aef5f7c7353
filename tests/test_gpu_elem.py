"""Backend<E>::quantized_matmul for E = f16 and bf16 (the reference's backend trait is generic over
the element type of activations and outputs, src/compat/mod.rs:376-378, 233-246) through
gllmq_quantized_matmul_elem.  The contract: 16-bit activations widen exactly, the arithmetic is the
f32 call's, and every result is rounded to the nearest element, ties to even (E::from_f32).  So the
output must equal, bit for bit, the oracle's rounding of what the f32 call gives on the widened
activations (the f32 call itself is held to the usual bars against the oracle), whichever kernel
does the conversion: the int8 and integer-dot kernels in their own loads and stores, or a widening
and a rounding launch around the f32 kernels."""
import numpy as np
import pytest

from gllm_amd.synth import random_activations, random_weight
from oracle import npref
from tests.test_gpu_parity import check_close

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
F16, BF16 = npref.ELEM_F16, npref.ELEM_BF16

# (dtype, m, n, k): the streamed one-pass kernels, the fetch-and-compute kernels with and without a K
# split, the GEMV (rows of whole and of ragged 64-element parts), rows in several passes, and
# shapes that take the conversion launches (GEMM, K beyond one GEMV launch)
SHAPES = [(Q4_K, 1, 4096, 2048), (Q5_K, 4, 3072, 1024), (Q6_K, 2, 4096, 4096), (Q4_K, 8, 2048, 1024),
          (Q4_K, 3, 300, 512), (Q4_K, 2, 256, 8192), (Q6_K, 1, 96, 14336), (Q5_K, 1, 128, 11008),
          (Q8_0, 1, 500, 1024), (Q8_0, 2, 333, 1056), (Q6_K, 2, 1000, 768), (Q8_0, 5, 300, 2048), (Q6_K, 7, 64, 12288),
          (Q4_K, 16, 512, 1024), (Q4_K, 32, 4096, 4096), (Q6_K, 1, 64, 16640), (Q8_0, 40, 100, 512),
          # one row over low tiles (pairs of blocks), registers and LDS operands; slices of K fall back to conversions
          (Q4_K, 1, 4096, 4096), (Q5_K, 1, 3000, 8192), (Q6_K, 1, 4096, 14336), (Q4_K, 1, 2048, 11008), (Q4_K, 3, 4096, 9216)]


@pytest.fixture(scope="module")
def hip():
    from gllm_amd.backend import HipBackend
    return HipBackend(0)


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def elem_inputs(x32, elem):
    """Activations that are exactly representable in the element type, as bits and as f32."""
    bits = npref.f32_to_elem_bits(x32, elem)
    return bits, npref.elem_bits_to_f32(bits, elem)


def run_elem(hip, torch, w, bits, elem, dt, m, n, k, offset=0):
    tt = torch.float16 if elem == F16 else torch.bfloat16
    wd = torch.from_numpy(np.asarray(w).view(np.uint8).reshape(-1)).cuda()
    xbuf = torch.full((m * k + offset + 64,), float("nan"), dtype=tt, device="cuda")
    xbuf[offset:offset + m * k] = torch.from_numpy(bits.view(np.int16).reshape(-1)).cuda().view(tt)
    ybuf = torch.full((m * n + offset + 64,), float("nan"), dtype=tt, device="cuda")
    ybuf[offset + m * n:] = 7.0
    y = ybuf[offset:offset + m * n]
    hip.quantized_matmul(wd, xbuf[offset:offset + m * k], y, dt, m, n, k)
    torch.cuda.synchronize()
    assert bool(torch.all(ybuf[offset + m * n:] == 7.0)), "write past the output"
    assert bool(torch.all(torch.isnan(ybuf[:offset]))), "write ahead of the output"
    return y.view(torch.int16).cpu().numpy().view(np.uint16).reshape(m, n)


def run_f32(hip, torch, w, x32, dt, m, n, k, offset=0):
    wd = torch.from_numpy(np.asarray(w).view(np.uint8).reshape(-1)).cuda()
    xbuf = torch.zeros(m * k + offset, device="cuda")
    xbuf[offset:] = torch.from_numpy(x32.reshape(-1)).cuda()
    y = torch.empty(m, n, device="cuda")
    hip.quantized_matmul(wd, xbuf[offset:], y, dt, m, n, k)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def same_bits(got, want32, elem, what):
    want = npref.f32_to_elem_bits(want32, elem)
    nan = np.isnan(want32)
    assert np.array_equal(np.isnan(npref.elem_bits_to_f32(got, elem)), nan), f"{what}: NaN pattern"
    bad = (got != want) & ~nan
    assert not bad.any(), f"{what}: {int(bad.sum())} of {got.size} elements differ from the rounded f32 result"


@pytest.mark.parametrize("elem", [F16, BF16])
@pytest.mark.parametrize("dt,m,n,k", SHAPES)
def test_rounded_f32_result_bit_for_bit(hip, torch, oracle, elem, dt, m, n, k):
    print(f"elem={elem} dtype={dt} m={m} n={n} k={k}", flush=True)
    w = random_weight(dt, n, k, seed=n + k)
    bits, x32 = elem_inputs(random_activations(m, k, seed=m + k), elem)
    y32 = run_f32(hip, torch, w, x32, dt, m, n, k)
    got = run_elem(hip, torch, w, bits, elem, dt, m, n, k)
    same_bits(got, y32, elem, "in-kernel or default path")
    # the f32 call these are rounded from, against the oracle on the same (widened) activations
    want = oracle.quantized_matmul(w, x32, dt, m, n, k, acc=oracle.ACC_F64, threads=8)
    check_close(y32, want, "f32 call on widened activations")
    # and the element-typed result itself: the oracle's result rounded the same way, up to the one
    # step of the element type that the f32 result's own error can flip
    back, ref = npref.elem_bits_to_f32(got, elem).astype(np.float64), npref.elem_bits_to_f32(
        npref.f32_to_elem_bits(want.astype(np.float32), elem), elem).astype(np.float64)
    step = 2.0 ** (-10 if elem == F16 else -7)
    assert np.all(np.abs(back - ref) <= step * np.maximum(np.abs(ref), 2.0 ** -14) + 1e-3 * np.abs(want).max())
    frac = np.mean(back != ref)
    assert frac < 0.02, f"{frac:.3%} of the elements round differently from the oracle's"


@pytest.mark.parametrize("elem", [F16, BF16])
def test_conversion_launches_give_the_same_bits(torch, oracle, elem):
    """With the in-kernel conversion switched off every shape takes the widening and rounding
    launches: same bits."""
    from gllm_amd.backend import HipBackend
    side = HipBackend(0)
    side.set_option("elem_fused", 0)
    for dt, m, n, k in SHAPES[:9]:
        print(f"conversion launches elem={elem} dtype={dt} m={m} n={n} k={k}", flush=True)
        w = random_weight(dt, n, k, seed=n + k)
        bits, x32 = elem_inputs(random_activations(m, k, seed=m + k), elem)
        same_bits(run_elem(side, torch, w, bits, elem, dt, m, n, k), run_f32(side, torch, w, x32, dt, m, n, k), elem,
                  f"conversion launches {dt} {m}x{n}x{k}")


@pytest.mark.parametrize("elem", [F16, BF16])
def test_unaligned_rows_special_values_and_overflow(hip, torch, oracle, elem):
    """Activations that start 4 bytes past a 16-byte boundary (the vector loads do not apply), a
    NaN and an infinity among them, and f16 results beyond 65504 (infinity, as from_f32 gives)."""
    print(f"elem={elem} unaligned, NaN, Inf, overflow", flush=True)
    dt, m, n, k = Q4_K, 2, 700, 1024
    w = random_weight(dt, n, k, seed=1)
    x = random_activations(m, k, seed=2)
    bits, x32 = elem_inputs(x, elem)
    same_bits(run_elem(hip, torch, w, bits, elem, dt, m, n, k, offset=2), run_f32(hip, torch, w, x32, dt, m, n, k, offset=1),
              elem, "unaligned")
    x[0, 5], x[1, 700] = np.nan, np.inf
    bits, x32 = elem_inputs(x, elem)
    got = run_elem(hip, torch, w, bits, elem, dt, m, n, k)
    same_bits(got, run_f32(hip, torch, w, x32, dt, m, n, k), elem, "NaN and Inf")
    assert np.all(np.isnan(npref.elem_bits_to_f32(got[0], elem)))
    big = random_activations(m, k, seed=3) * np.float32(300.0)  # representable in f16, results beyond it
    bits, x32 = elem_inputs(big, elem)
    y32 = run_f32(hip, torch, w, x32, dt, m, n, k)
    got = run_elem(hip, torch, w, bits, elem, dt, m, n, k)
    same_bits(got, y32, elem, "large results")
    if elem == F16:
        assert np.isinf(npref.elem_bits_to_f32(got, elem)).any() and np.isfinite(y32).all()


def test_batch_entries_of_mixed_element_types(hip, torch):
    """A batch whose entries hold f32, bf16 and f16 activations: each entry's result equals the
    single call's, bit for bit (16-bit entries are launches of their own between chained f32 ones)."""
    print("elem in a batch", flush=True)
    dt, n, k = Q4_K, 4096, 2048
    ws = [torch.from_numpy(np.asarray(random_weight(dt, n, k, seed=s)).view(np.uint8).reshape(-1)).cuda() for s in range(6)]
    kinds = [torch.float32, torch.float32, torch.bfloat16, torch.float16, torch.float32, torch.bfloat16]
    xs = [torch.from_numpy(random_activations(1, k, seed=10 + i)).cuda().to(t) for i, t in enumerate(kinds)]
    ys = [torch.full((1, n), float("nan"), device="cuda", dtype=t) for t in kinds]
    hip.run_batch(hip.make_batch([(w, x, y, dt, 1, n, k) for w, x, y in zip(ws, xs, ys)]))
    torch.cuda.synchronize()
    for i, (w, x, y) in enumerate(zip(ws, xs, ys)):
        alone = torch.empty_like(y)
        hip.quantized_matmul(w, x, alone, dt, 1, n, k)
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16) if y.dtype != torch.float32 else y,
                           alone.view(torch.int16) if y.dtype != torch.float32 else alone), f"entry {i}"


def test_argument_errors(hip, torch):
    from gllm_amd.backend import BackendError
    print("elem errors", flush=True)
    w = torch.zeros(144 * 8, dtype=torch.uint8, device="cuda")
    x = torch.zeros(256, dtype=torch.float16, device="cuda")
    with pytest.raises(BackendError):  # one element type for both
        hip.quantized_matmul(w, x, torch.zeros(8, dtype=torch.bfloat16, device="cuda"), Q4_K, 1, 8, 256)
    with pytest.raises(BackendError):
        hip.quantized_matmul(w, x.to(torch.float64), torch.zeros(8, dtype=torch.float64, device="cuda"), Q4_K, 1, 8, 256)
    with pytest.raises(BackendError):  # the bf16 activation mode belongs to f32 tensors
        hip.quantized_matmul(w, x, torch.zeros(8, dtype=torch.float16, device="cuda"), Q4_K, 1, 8, 256, act_mode=1)
