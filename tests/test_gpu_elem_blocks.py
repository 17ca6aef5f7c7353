"""The ops around the matmul for E = f16 and bf16, and added to their output instead of replacing
it: gllmq_ffn_swiglu_elem, gllmq_moe_matvec_elem, gllmq_quant_gather_elem (the reference's backend
trait is generic over the element type, src/compat/mod.rs:376-378; the shared expert's block is
Op::Add-ed to the routed experts' sum and the residual behind it, build_graph.inc.rs:2132-2170).
The contract, as for gllmq_quantized_matmul_elem: 16-bit activations widen exactly, the op runs in
f32, the result (plus what the output held, when adding) is rounded once to the nearest element,
ties to even.  So the output must equal, bit for bit, the oracle's rounding of "what the f32 entry
point gives on the widened activations, plus the widened old output"; the f32 entry point itself is
held to the matmul bar against the oracle, here and in its own tests."""
import numpy as np
import pytest

from gllm_amd.synth import random_activations, random_gate_logits, random_weight
from oracle import npref
from tests.test_gpu_parity import check_close

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
F16, BF16 = npref.ELEM_F16, npref.ELEM_BF16


@pytest.fixture(scope="module")
def hip():
    from gllm_amd.backend import HipBackend
    return HipBackend(0)


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def dev_bytes(torch, host):
    return torch.from_numpy(np.asarray(host).view(np.uint8).reshape(-1)).cuda()


def torch_type(torch, elem):
    return {None: torch.float32, F16: torch.float16, BF16: torch.bfloat16}[elem]


def to_dev(torch, values32, elem):
    """f32 values (exactly representable in the element type) as a device tensor of that type."""
    t = torch.from_numpy(np.ascontiguousarray(values32, np.float32)).cuda()
    return t if elem is None else t.to(torch_type(torch, elem))


def representable(values32, elem):
    if elem is None:
        return np.ascontiguousarray(values32, np.float32)
    return npref.elem_bits_to_f32(npref.f32_to_elem_bits(values32, elem), elem)


def expected(result32, old32, elem, accumulate):
    total = (old32 + result32).astype(np.float32) if accumulate else result32
    return total if elem is None else npref.elem_bits_to_f32(npref.f32_to_elem_bits(total, elem), elem)


def as_f32(torch, t):
    return t.to(torch.float32).cpu().numpy()


@pytest.mark.parametrize("elem", [None, F16, BF16])
@pytest.mark.parametrize("accumulate", [False, True])
def test_feed_forward_block(hip, torch, oracle, elem, accumulate):
    """One row through the gated epilogue, four rows, and 12 rows through the GEMM; ragged ffn."""
    if elem is None and not accumulate:
        pytest.skip("the plain f32 form has its own tests")
    for (t_gu, t_dn, m, hidden, ffn) in ((Q4_K, Q6_K, 1, 1024, 2048), (Q5_K, Q4_K, 4, 512, 1536), (Q4_K, Q4_K, 12, 1024, 1024),
                                         (Q8_0, Q6_K, 2, 256, 768)):
        print(f"ffn elem={elem} accumulate={accumulate} {t_gu}/{t_dn} m={m}", flush=True)
        gate, up = random_weight(t_gu, ffn, hidden, seed=1), random_weight(t_gu, ffn, hidden, seed=2)
        down = random_weight(t_dn, hidden, ffn, seed=3)
        x32 = representable(random_activations(m, hidden, seed=4) * 0.25, elem)
        old32 = representable(random_activations(m, hidden, seed=5) * 30.0, elem)
        gd, ud, dd = dev_bytes(torch, gate), dev_bytes(torch, up), dev_bytes(torch, down)
        # the f32 entry point on the widened activations
        xf, rf = to_dev(torch, x32, None), torch.full((m, hidden), float("nan"), device="cuda")
        hip.ffn_swiglu(gd, ud, t_gu, dd, t_dn, xf, rf, m, hidden, ffn)
        torch.cuda.synchronize()
        result32 = rf.cpu().numpy()
        check_close(result32, oracle.ffn_swiglu(gate, up, t_gu, down, t_dn, x32, m, hidden, ffn), "the f32 block")
        # the form under test
        xe, oe = to_dev(torch, x32, elem), to_dev(torch, old32, elem)
        hip.ffn_swiglu(gd, ud, t_gu, dd, t_dn, xe, oe, m, hidden, ffn, accumulate=accumulate)
        torch.cuda.synchronize()
        got, want = as_f32(torch, oe), expected(result32, old32, elem, accumulate)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"{t_gu}/{t_dn} m={m}"


@pytest.mark.parametrize("elem", [None, F16, BF16])
@pytest.mark.parametrize("accumulate", [False, True])
def test_expert_matvec(hip, torch, oracle, elem, accumulate):
    if elem is None and not accumulate:
        pytest.skip("the plain f32 form has its own tests")
    experts, tokens, top_k, hidden, ffn = 8, 7, 2, 512, 256
    print(f"moe elem={elem} accumulate={accumulate}", flush=True)
    gu = np.concatenate([np.asarray(random_weight(Q4_K, 2 * ffn, hidden, seed=40 + e)).view(np.uint8).reshape(-1) for e in range(experts)])
    dn = np.concatenate([np.asarray(random_weight(Q6_K, hidden, ffn, seed=60 + e)).view(np.uint8).reshape(-1) for e in range(experts)])
    gud, dnd = dev_bytes(torch, gu), dev_bytes(torch, dn)
    x32 = representable(random_activations(tokens, hidden, seed=41) * 0.25, elem)
    old32 = representable(random_activations(tokens, hidden, seed=43) * 10.0, elem)
    logits = torch.from_numpy(random_gate_logits(tokens, experts, seed=42)).cuda()
    re_ = torch.empty(tokens, top_k, dtype=torch.int32, device="cuda")
    rw = torch.empty(tokens, top_k, device="cuda")
    rl = torch.empty(tokens, dtype=torch.int32, device="cuda")
    hip.moe_route(logits, top_k, re_, rw, rl, capacity_factor=float(experts))
    xf, rf = to_dev(torch, x32, None), torch.full((tokens, hidden), float("nan"), device="cuda")
    hip.moe_matvec(gud, Q4_K, dnd, Q6_K, xf, rf, hidden, ffn, experts, re_, rw, rl)
    torch.cuda.synchronize()
    result32 = rf.cpu().numpy()
    want64 = oracle.moe_ffn(gu, Q4_K, dn, Q6_K, x32, hidden, ffn, experts, re_.cpu().numpy().astype(np.uint32), rw.cpu().numpy(),
                            rl.cpu().numpy().astype(np.uint32))
    check_close(result32, want64, "the f32 expert matvec")
    xe, oe = to_dev(torch, x32, elem), to_dev(torch, old32, elem)
    hip.moe_matvec(gud, Q4_K, dnd, Q6_K, xe, oe, hidden, ffn, experts, re_, rw, rl, accumulate=accumulate)
    torch.cuda.synchronize()
    got, want = as_f32(torch, oe), expected(result32, old32, elem, accumulate)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_shared_expert_on_top_of_routed_experts_and_residual(hip, torch, oracle):
    """The layer's sequence (build_graph.inc.rs:2076-2170): routed experts into the accumulator, the
    shared expert's block added to it, the sum added to the residual stream; against numpy adds of
    the oracle's two blocks."""
    experts, tokens, top_k, hidden, ffn = 4, 5, 2, 256, 512
    gu = np.concatenate([np.asarray(random_weight(Q4_K, 2 * ffn, hidden, seed=10 + e)).view(np.uint8).reshape(-1) for e in range(experts)])
    dn = np.concatenate([np.asarray(random_weight(Q6_K, hidden, ffn, seed=20 + e)).view(np.uint8).reshape(-1) for e in range(experts)])
    sg, su, sd = random_weight(Q4_K, ffn, hidden, seed=30), random_weight(Q4_K, ffn, hidden, seed=31), random_weight(Q6_K, hidden, ffn, seed=32)
    x = random_activations(tokens, hidden, seed=33) * 0.25
    residual = random_activations(tokens, hidden, seed=34)
    logits = torch.from_numpy(random_gate_logits(tokens, experts, seed=35)).cuda()
    re_ = torch.empty(tokens, top_k, dtype=torch.int32, device="cuda")
    rw = torch.empty(tokens, top_k, device="cuda")
    rl = torch.empty(tokens, dtype=torch.int32, device="cuda")
    hip.moe_route(logits, top_k, re_, rw, rl, capacity_factor=float(experts))
    xd = torch.from_numpy(x).cuda()
    acc = torch.full((tokens, hidden), float("nan"), device="cuda")
    stream = torch.from_numpy(residual).cuda()
    print("shared expert and residual", flush=True)
    hip.moe_matvec(dev_bytes(torch, gu), Q4_K, dev_bytes(torch, dn), Q6_K, xd, acc, hidden, ffn, experts, re_, rw, rl)
    hip.ffn_swiglu(dev_bytes(torch, sg), dev_bytes(torch, su), Q4_K, dev_bytes(torch, sd), Q6_K, xd, acc, tokens, hidden, ffn, accumulate=True)
    torch.cuda.synchronize()
    routed = oracle.moe_ffn(gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, re_.cpu().numpy().astype(np.uint32), rw.cpu().numpy(),
                            rl.cpu().numpy().astype(np.uint32)).astype(np.float64)
    shared = oracle.ffn_swiglu(sg, su, Q4_K, sd, Q6_K, x, tokens, hidden, ffn).astype(np.float64)
    check_close(acc.cpu().numpy(), routed + shared, "routed + shared")
    # ... and the sum into the residual stream: residual += routed + shared, as two adding calls would leave it
    stream2 = torch.from_numpy(residual).cuda()
    hip.moe_matvec(dev_bytes(torch, gu), Q4_K, dev_bytes(torch, dn), Q6_K, xd, stream2, hidden, ffn, experts, re_, rw, rl, accumulate=True)
    hip.ffn_swiglu(dev_bytes(torch, sg), dev_bytes(torch, su), Q4_K, dev_bytes(torch, sd), Q6_K, xd, stream2, tokens, hidden, ffn, accumulate=True)
    torch.cuda.synchronize()
    check_close(stream2.cpu().numpy(), residual.astype(np.float64) + routed + shared, "residual + routed + shared")


@pytest.mark.parametrize("elem", [F16, BF16])
@pytest.mark.parametrize("dtype", [Q8_0, Q4_K, Q5_K, Q6_K])
def test_embedding_lookup(hip, torch, oracle, elem, dtype):
    """Rows of a 16-bit element type: the oracle's lookup (bit-exact decoders, the scale applied in
    f32) rounded to the element; aligned rows (8-byte stores) and an odd start, an id outside the
    table (a row of NaN)."""
    vocab, hidden, count = 97, 768, 13
    table = random_weight(dtype, vocab, hidden, seed=dtype)
    ids = np.random.default_rng(elem).integers(0, vocab, count).astype(np.uint32)
    td, idd = dev_bytes(torch, table), torch.from_numpy(ids.astype(np.int32)).cuda()
    tt = torch_type(torch, elem)
    for scale, offset in ((None, 0), (float(np.sqrt(hidden)), 1)):
        print(f"gather elem={elem} dtype={dtype} scale={scale} offset={offset}", flush=True)
        buf = torch.full((count * hidden + offset + 64,), 7.0, dtype=tt, device="cuda")
        out = buf[offset:offset + count * hidden]
        hip.quant_gather(td, dtype, vocab, hidden, idd, out, scale=scale)
        torch.cuda.synchronize()
        assert bool(torch.all(buf[offset + count * hidden:] == 7.0)) and bool(torch.all(buf[:offset] == 7.0))
        want32 = oracle.quant_gather(table, dtype, vocab, hidden, ids, scale=scale)
        want = npref.f32_to_elem_bits(want32, elem).reshape(-1)
        got = out.view(torch.int16).cpu().numpy().view(np.uint16)
        assert np.array_equal(got, want)
    bad = torch.tensor([3, vocab, 5], dtype=torch.int32, device="cuda")
    out = torch.zeros(3 * hidden, dtype=tt, device="cuda")
    hip.quant_gather(td, dtype, vocab, hidden, bad, out)
    torch.cuda.synchronize()
    rows = out.to(torch.float32).cpu().numpy().reshape(3, hidden)
    assert np.isnan(rows[1]).all() and np.isfinite(rows[0]).all() and np.isfinite(rows[2]).all()
