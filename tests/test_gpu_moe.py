"""GPU parity of the MoE path (through the C ABI): gate logits go to the library's router
(gllmq_moe_route), its route table goes to the expert matvec (gllmq_moe_matvec); the oracle
routes the same logits on the CPU and evaluates route by route, which is the dense "run the
expert, weight, add" rule of src/moe/routing.rs:307-327 restricted to the routed pairs.  The
oracle only checks: the route tables must agree (experts and lengths exactly, weights to a few
ulp) and the outputs must meet the bar.

Bar: rel-L2 <= 1e-4 and per-element |err| <= 1e-3 * max|out| against float64 accumulation.
"""
import numpy as np
import pytest

from gllm_amd.ggml import row_bytes
from gllm_amd.synth import random_activations, random_gate_logits, random_weight

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
REL_L2_TOL = 1e-4
ELEM_TOL = 1e-3


@pytest.fixture(scope="module")
def hip():
    from gllm_amd.backend import HipBackend
    return HipBackend(0)


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def check_close(got, want, what=""):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    rel = np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-300)
    worst = np.abs(got - want).max() / max(np.abs(want).max(), 1e-300)
    assert rel <= REL_L2_TOL and worst <= ELEM_TOL, f"{what}: rel_l2={rel:.3e} max_err/max|y|={worst:.3e}"
    return rel


def expert_weights(dt_gu, dt_dn, experts, hidden, ffn, seed):
    gu = random_weight(dt_gu, experts * 2 * ffn, hidden, seed=seed)
    dn = random_weight(dt_dn, experts * hidden, ffn, seed=seed + 1)
    return gu, dn


def route_gpu(hip, torch, oracle, logits, top_k, capacity_factor=1.25):
    """Routes `logits` with the library's router, checks the table against the oracle's and
    returns (device table, oracle table)."""
    tokens, experts = logits.shape
    lg = torch.from_numpy(np.ascontiguousarray(logits, np.float32)).cuda()
    red = torch.full((tokens, top_k), -1, dtype=torch.int32, device="cuda")
    rwd = torch.full((tokens, top_k), float("nan"), dtype=torch.float32, device="cuda")
    rld = torch.full((tokens,), -1, dtype=torch.int32, device="cuda")
    hip.moe_route(lg, top_k, red, rwd, rld, capacity_factor=capacity_factor)
    torch.cuda.synchronize()
    r = oracle.route(logits, top_k, capacity_factor=capacity_factor)
    got_e, got_w, got_l = red.cpu().numpy().view(np.uint32), rwd.cpu().numpy(), rld.cpu().numpy().view(np.uint32)
    assert np.array_equal(got_l, r["len"]), "route lengths differ from the oracle's"
    assert np.array_equal(got_e, r["expert"]), "routed experts differ from the oracle's"
    np.testing.assert_allclose(got_w, r["weight"], rtol=4 * top_k * 2.0 ** -24, atol=0)
    return (red, rwd, rld), r


def run_gpu(hip, torch, gu, dt_gu, dn, dt_dn, x, hidden, ffn, experts, re, rw, rl, relu_gate=False, split=False):
    """re, rw, rl: the route table as numpy arrays or as device tensors.  split: gate rows and up
    rows as a tensor each ([experts, ffn, hidden]: GGUF's layout) instead of one stacked tensor."""
    tokens = x.shape[0]
    # poison behind every input: a read past the end turns the result into NaN
    def guarded(host, fill):
        flat = torch.from_numpy(np.ascontiguousarray(host).reshape(-1))
        buf = torch.full((flat.numel() + 4096,), fill, dtype=flat.dtype, device="cuda")
        buf[:flat.numel()] = flat.cuda()
        return buf[:flat.numel()]
    gud, dnd = guarded(np.asarray(gu).view(np.uint8), 0xFF), guarded(np.asarray(dn).view(np.uint8), 0xFF)
    xd = guarded(np.ascontiguousarray(x, np.float32), float("nan")).view(tokens, -1)
    out = torch.full((tokens, hidden), float("nan"), dtype=torch.float32, device="cuda")
    if isinstance(re, np.ndarray):
        red = torch.from_numpy(np.ascontiguousarray(re, np.uint32).view(np.int32)).cuda()
        rwd = torch.from_numpy(np.ascontiguousarray(rw, np.float32)).cuda()
        rld = torch.from_numpy(np.ascontiguousarray(rl, np.uint32).view(np.int32)).cuda()
    else:
        red, rwd, rld = re, rw, rl
    if split:
        each = ffn * row_bytes(dt_gu, hidden)
        both = np.asarray(gu).view(np.uint8).reshape(experts, 2, each)
        gate_d, up_d = guarded(both[:, 0], 0xFF), guarded(both[:, 1], 0xFF)
        hip.moe_matvec(gate_d, dt_gu, dnd, dt_dn, xd, out, hidden, ffn, experts, red, rwd, rld, relu_gate=relu_gate, up=up_d)
    else:
        hip.moe_matvec(gud, dt_gu, dnd, dt_dn, xd, out, hidden, ffn, experts, red, rwd, rld, relu_gate=relu_gate)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("dt_gu,dt_dn", [(Q4_K, Q6_K), (Q5_K, Q8_0), (Q6_K, Q4_K), (Q8_0, Q5_K)])
def test_moe_small_routed(hip, torch, oracle, dt_gu, dt_dn):
    print(f"moe small gu={dt_gu} dn={dt_dn}", flush=True)
    experts, tokens, top_k, hidden, ffn = 8, 7, 2, 512, 256
    gu, dn = expert_weights(dt_gu, dt_dn, experts, hidden, ffn, seed=40)
    x = random_activations(tokens, hidden, seed=41)
    dev, r = route_gpu(hip, torch, oracle, random_gate_logits(tokens, experts, seed=42), top_k, float(experts))
    want = oracle.moe_ffn(gu, dt_gu, dn, dt_dn, x, hidden, ffn, experts, r["expert"], r["weight"], r["len"])
    got = run_gpu(hip, torch, gu, dt_gu, dn, dt_dn, x, hidden, ffn, experts, *dev)
    check_close(got, want, "moe small")
    got = run_gpu(hip, torch, gu, dt_gu, dn, dt_dn, x, hidden, ffn, experts, *dev, split=True)
    check_close(got, want, "moe small, gate and up as separate tensors")


def test_moe_ragged_routes_repeats_and_empty_tokens(hip, torch, oracle):
    """Hand-made table: a token with no route (zeros), an expert hit by 1, 2, 3 and 5 tokens,
    one token naming the same expert twice, an expert nobody uses, relu_gate on."""
    print("moe ragged", flush=True)
    experts, tokens, top_k, hidden, ffn = 6, 9, 3, 256, 512
    gu, dn = expert_weights(Q4_K, Q6_K, experts, hidden, ffn, seed=50)
    x = random_activations(tokens, hidden, seed=51)
    re = np.zeros((tokens, top_k), np.uint32)
    rw = np.zeros((tokens, top_k), np.float32)
    rl = np.zeros(tokens, np.uint32)
    table = {
        0: [(0, 0.5), (1, 0.3), (2, 0.2)],
        1: [],
        2: [(1, 1.0)],
        3: [(2, 0.6), (2, 0.4)],
        4: [(1, 0.7), (4, 0.3)],
        5: [(4, 0.25), (2, 0.5), (1, 0.25)],
        6: [(2, 1.0)],
        7: [(4, 0.9), (1, 0.1)],
        8: [(2, 0.5), (4, 0.5)],
    }
    for t, routes in table.items():
        rl[t] = len(routes)
        for i, (e, w) in enumerate(routes):
            re[t, i], rw[t, i] = e, w
    # slots past route_len hold junk that must be ignored
    re[1, :] = 5
    rw[1, :] = 123.0
    re[2, 1:] = 3
    rw[2, 1:] = -7.0
    for relu in (False, True):
        want = oracle.moe_ffn(gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, re, rw, rl, relu_gate=relu)
        got = run_gpu(hip, torch, gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, re, rw, rl, relu_gate=relu)
        assert np.array_equal(got[1], np.zeros(hidden, np.float32))
        check_close(got, want, f"moe ragged relu={relu}")


def test_moe_matches_dense_masked_evaluation(hip, torch, oracle):
    """Brute force on 4 experts x 3 tokens: every expert on every token, masked by the
    routing weights (what the reference graph does, build_graph.inc.rs:2119-2123)."""
    print("moe dense-masked", flush=True)
    experts, tokens, top_k, hidden, ffn = 4, 3, 2, 256, 256
    gu, dn = expert_weights(Q4_K, Q6_K, experts, hidden, ffn, seed=60)
    x = random_activations(tokens, hidden, seed=61)
    dev, r = route_gpu(hip, torch, oracle, random_gate_logits(tokens, experts, seed=62), top_k, float(experts))
    gu_f = oracle.dequantize(gu, Q4_K).reshape(experts, 2 * ffn, hidden).astype(np.float64)
    dn_f = oracle.dequantize(dn, Q6_K).reshape(experts, hidden, ffn).astype(np.float64)
    dense = np.zeros((tokens, hidden))
    for t in range(tokens):
        mask = np.zeros(experts)
        for i in range(int(r["len"][t])):
            mask[r["expert"][t, i]] += float(r["weight"][t, i])
        for e in range(experts):
            g = gu_f[e, :ffn] @ x[t].astype(np.float64)
            u = gu_f[e, ffn:] @ x[t].astype(np.float64)
            dense[t] += mask[e] * (dn_f[e] @ (g / (1.0 + np.exp(-g)) * u))
    got = run_gpu(hip, torch, gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, *dev)
    check_close(got, dense, "moe dense")


def test_moe_baseline_shape_full_size(hip, torch, oracle):
    """The baseline MoE configuration at its full size: 128 experts, 16 tokens, top-8, gate/up
    Q4_K 3072x4096 and down Q6_K 4096x1536 per expert (1.5 GB of expert weights, generated on the
    host with the seeded generator), gate logits routed by the library.  The oracle evaluates the
    128 routed pairs (about a fifth of a second per pair and thread)."""
    print("moe baseline shape, 128 experts", flush=True)
    experts, tokens, top_k, hidden, ffn = 128, 16, 8, 4096, 1536
    gu, dn = expert_weights(Q4_K, Q6_K, experts, hidden, ffn, seed=70)
    assert gu.size == experts * 2 * ffn * row_bytes(Q4_K, hidden)
    x = random_activations(tokens, hidden, seed=71)
    logits = random_gate_logits(tokens, experts, seed=72)
    dev, r = route_gpu(hip, torch, oracle, logits, top_k, float(experts))
    assert int(r["len"].sum()) == tokens * top_k
    want = oracle.moe_ffn(gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, r["expert"], r["weight"], r["len"], threads=16)
    got = run_gpu(hip, torch, gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, *dev)
    check_close(got, want, "moe baseline shape")
    # the reference's default capacity factor 1.25: capacity 1 at 16 tokens over 128 experts, so
    # most choices overflow and some tokens fall back to the least loaded expert
    dev2, r2 = route_gpu(hip, torch, oracle, logits, top_k, 1.25)
    assert r2["overflow"] > 0 and int(r2["counts"].max()) == 1
    want2 = oracle.moe_ffn(gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, r2["expert"], r2["weight"], r2["len"], threads=16)
    got2 = run_gpu(hip, torch, gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, *dev2)
    check_close(got2, want2, "moe baseline shape, default capacity")


@pytest.mark.parametrize("hidden,ffn", [(256, 768), (512, 2304), (4352, 256)])
def test_moe_more_than_eight_tokens_per_expert(hip, torch, oracle, hidden, ffn):
    """Experts with around twenty tokens each: jobs of eight tokens plus a remainder.  ffn = 768
    takes the wave-per-tile Q6_K kernel, ffn = 2304 (9 blocks per row) the tile-split one with two
    passes per tile, hidden = 4352 (17 blocks) leaves the matrix-core kernels for the GEMV."""
    print(f"moe >8 tokens per expert hidden={hidden} ffn={ffn}", flush=True)
    experts, tokens, top_k = 4, 40, 2
    gu, dn = expert_weights(Q4_K, Q6_K, experts, hidden, ffn, seed=90)
    x = random_activations(tokens, hidden, seed=91)
    dev, r = route_gpu(hip, torch, oracle, random_gate_logits(tokens, experts, seed=92), top_k, float(experts))
    counts = np.bincount(r["expert"][:, :top_k].reshape(-1), minlength=experts)
    assert counts.max() > 8
    want = oracle.moe_ffn(gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, r["expert"], r["weight"], r["len"], threads=8)
    got = run_gpu(hip, torch, gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, *dev)
    check_close(got, want, f"moe hidden={hidden} ffn={ffn}")
    # the streamed grouped kernels (by default for experts with few tokens each): jobs of four tokens
    from gllm_amd.backend import HipBackend
    got = run_gpu(HipBackend(0, options={"moe_streamed": 2}), torch, gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, *dev)
    check_close(got, want, f"moe streamed hidden={hidden} ffn={ffn}")


def test_moe_grouped_kernel_alternatives(hip, torch, oracle):
    """The grouped kernels the default dispatch does not pick for this shape: the matrix-core
    kernels whose waves fetch and multiply (a wave per tile and tile-split for the Q6_K down rows),
    the integer-dot GEMV, gate/up results through memory with the activation as a kernel of its own."""
    from gllm_amd.backend import HipBackend
    experts, tokens, top_k, hidden, ffn = 6, 20, 3, 512, 1024
    gu, dn = expert_weights(Q4_K, Q6_K, experts, hidden, ffn, seed=95)
    x = random_activations(tokens, hidden, seed=96)
    dev, r = route_gpu(hip, torch, oracle, random_gate_logits(tokens, experts, seed=97), top_k, float(experts))
    want = oracle.moe_ffn(gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, r["expert"], r["weight"], r["len"], threads=8)
    for options in ({"moe_streamed": 0}, {"moe_streamed": 0, "moe_mm8_rows": 0}, {"moe_mm8_rows": 0}, {"moe_mm8_q6k": 0}, {"moe_mm8": 0},
                    {"moe_glu": 0}, {"moe_streamed": 0, "moe_glu": 0}):
        hip2 = HipBackend(0, options=options)
        for split in (False, True):
            print(f"moe alternatives {options} split={split}", flush=True)
            got = run_gpu(hip2, torch, gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, *dev, split=split)
            check_close(got, want, f"moe {options} split={split}")


def test_moe_random_shapes_sweep(hip, torch, oracle):
    """Sixteen seeded MoE shapes: formats in every role, expert counts from 2 to 40, top-k from 1
    to 6, ragged hidden/ffn sizes on both sides of the matrix-core kernels' limits."""
    from gllm_amd.backend import HipBackend
    streamed = HipBackend(0, options={"moe_streamed": 2})  # also where experts see many tokens each
    rng = np.random.default_rng(77)
    fmts = [Q4_K, Q5_K, Q6_K, Q8_0]
    for case in range(16):
        dt_gu, dt_dn = fmts[case % 4], fmts[(case // 4 + case) % 4]
        experts = int(rng.integers(2, 41))
        top_k = int(rng.integers(1, min(6, experts) + 1))
        tokens = int(rng.integers(1, 30))
        hidden = int(rng.integers(1, 9)) * 256
        ffn = int(rng.integers(1, 10)) * 256
        print(f"moe sweep case {case}: gu={dt_gu} dn={dt_dn} E={experts} k={top_k} T={tokens} H={hidden} F={ffn}", flush=True)
        gu, dn = expert_weights(dt_gu, dt_dn, experts, hidden, ffn, seed=300 + case)
        x = random_activations(tokens, hidden, seed=400 + case)
        factor = float(experts) if case % 3 else 1.25  # a third of the cases with the default capacity: drops and fallbacks
        dev, r = route_gpu(hip, torch, oracle, random_gate_logits(tokens, experts, seed=500 + case), top_k, factor)
        want = oracle.moe_ffn(gu, dt_gu, dn, dt_dn, x, hidden, ffn, experts, r["expert"], r["weight"], r["len"], threads=8)
        got = run_gpu(hip, torch, gu, dt_gu, dn, dt_dn, x, hidden, ffn, experts, *dev, split=bool(case & 1))
        check_close(got, want, f"moe sweep case {case}")
        got = run_gpu(streamed, torch, gu, dt_gu, dn, dt_dn, x, hidden, ffn, experts, *dev, split=bool(case & 1))
        check_close(got, want, f"moe sweep case {case}, streamed grouped kernels")


def test_moe_many_pairs(hip, torch, oracle):
    """More (token, expert) pairs than the plan kernel's per-pair placement takes (4096): the
    per-expert walk is used; experts get hundreds of tokens each."""
    print("moe many pairs", flush=True)
    experts, tokens, top_k, hidden, ffn = 16, 640, 8, 256, 256
    gu, dn = expert_weights(Q4_K, Q6_K, experts, hidden, ffn, seed=80)
    x = random_activations(tokens, hidden, seed=81)
    dev, r = route_gpu(hip, torch, oracle, random_gate_logits(tokens, experts, seed=82), top_k, float(experts))
    assert int(r["len"].sum()) == tokens * top_k > 4096
    want = oracle.moe_ffn(gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, r["expert"], r["weight"], r["len"], threads=16)
    got = run_gpu(hip, torch, gu, Q4_K, dn, Q6_K, x, hidden, ffn, experts, *dev)
    check_close(got, want, "moe many pairs")


def test_moe_error_behaviour(hip, torch):
    from gllm_amd.backend import Unimplemented
    print("moe errors", flush=True)
    z = torch.zeros(1024, dtype=torch.float32, device="cuda")
    zi = torch.zeros(8, dtype=torch.int32, device="cuda").reshape(4, 2)
    zl = torch.zeros(4, dtype=torch.int32, device="cuda")
    zw = torch.zeros(8, dtype=torch.float32, device="cuda").reshape(4, 2)
    with pytest.raises(Unimplemented):
        hip.moe_matvec(z, 2, z, Q6_K, z, z, 256, 256, 4, zi, zw, zl)  # Q4_0 gate/up: not covered


@pytest.mark.parametrize("seed", [11, 12])
def test_moe_shapes_from_a_seeded_generator(hip, torch, oracle, seed):
    """Experts, tokens, routes per token, capacity, widths and formats drawn from a seeded
    generator: jobs of one to many tokens, experts nobody is routed to, dropped routes, rows of
    one to eight blocks, expert matrices too low for the grouped matrix-core kernels."""
    rng = np.random.default_rng(seed)
    for i in range(12):
        experts = int(rng.choice([2, 4, 8, 16, 24, 40]))
        tokens = int(rng.choice([1, 2, 5, 9, 16, 33]))
        top_k = int(rng.integers(1, min(4, experts) + 1))
        hidden = 256 * int(rng.choice([1, 2, 3, 4, 8]))
        ffn = 256 * int(rng.choice([1, 2, 3, 6]))
        dt_gu, dt_dn = int(rng.choice([Q4_K, Q5_K, Q6_K, Q8_0])), int(rng.choice([Q4_K, Q5_K, Q6_K, Q8_0]))
        capacity = float(rng.choice([0.5, 1.25, float(experts)]))
        relu = bool(rng.integers(0, 2))
        print(f"moe seeded {seed}/{i}: experts={experts} tokens={tokens} top_k={top_k} hidden={hidden} ffn={ffn} "
              f"gu={dt_gu} dn={dt_dn} capacity={capacity} relu={relu}", flush=True)
        gu, dn = expert_weights(dt_gu, dt_dn, experts, hidden, ffn, seed=seed * 100 + i)
        x = random_activations(tokens, hidden, seed=seed * 300 + i)
        dev, r = route_gpu(hip, torch, oracle, random_gate_logits(tokens, experts, seed=seed * 500 + i), top_k, capacity)
        want = oracle.moe_ffn(gu, dt_gu, dn, dt_dn, x, hidden, ffn, experts, r["expert"], r["weight"], r["len"], relu_gate=relu)
        got = run_gpu(hip, torch, gu, dt_gu, dn, dt_dn, x, hidden, ffn, experts, *dev, relu_gate=relu, split=bool(i & 1))
        check_close(got, want, f"moe seeded {seed}/{i}")
