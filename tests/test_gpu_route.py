"""GPU parity of the MoE router (gllmq_moe_route through the C ABI) against the oracle's
restatement of ExpertRouteTable::from_gate_logits (src/moe/routing.rs:100-160) and
topk_with_weights / softmax (src/moe/routing.rs:263-302).

Bar: routed experts, route lengths, positions, per-expert counts and the overflow count equal to
the oracle's; weights within 4 * top_k ulp (the device's exp() and the host's libm differ in the
last bit, and a weight is a quotient of sums of such values).
"""
import numpy as np
import pytest

from gllm_amd.synth import random_gate_logits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from gllm_amd.backend import HipBackend
    return HipBackend(0)


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def route(hip, torch, logits, top_k, capacity_factor=1.25):
    logits = np.ascontiguousarray(logits, np.float32)
    tokens, experts = logits.shape
    lg = torch.from_numpy(logits).cuda()
    # markers behind every output: a write past the end shows
    re = torch.full((tokens * top_k + 16,), -7, dtype=torch.int32, device="cuda")
    rw = torch.full((tokens * top_k + 16,), 777.0, dtype=torch.float32, device="cuda")
    rl = torch.full((tokens + 16,), -7, dtype=torch.int32, device="cuda")
    rp = torch.full((tokens * top_k + 16,), -7, dtype=torch.int32, device="cuda")
    ec = torch.full((experts + 16,), -7, dtype=torch.int32, device="cuda")
    ov = torch.full((1 + 16,), -7, dtype=torch.int32, device="cuda")
    hip.moe_route(lg, top_k, re, rw, rl, capacity_factor=capacity_factor, route_pos=rp, expert_counts=ec, overflow=ov)
    torch.cuda.synchronize()
    for t, n in ((re, tokens * top_k), (rl, tokens), (rp, tokens * top_k), (ec, experts), (ov, 1)):
        assert bool((t[n:] == -7).all()), "a marker behind an output changed"
    assert bool((rw[tokens * top_k:] == 777.0).all())
    return dict(expert=re[:tokens * top_k].cpu().numpy().view(np.uint32).reshape(tokens, top_k),
                weight=rw[:tokens * top_k].cpu().numpy().reshape(tokens, top_k),
                len=rl[:tokens].cpu().numpy().view(np.uint32),
                pos=rp[:tokens * top_k].cpu().numpy().view(np.uint32).reshape(tokens, top_k),
                counts=ec[:experts].cpu().numpy().view(np.uint32), overflow=int(ov[0].item()))


def check_against_oracle(oracle, got, logits, top_k, capacity_factor, what):
    want = oracle.route(logits, top_k, capacity_factor=capacity_factor)
    assert np.array_equal(got["len"], want["len"]), f"{what}: lengths"
    assert np.array_equal(got["expert"], want["expert"]), f"{what}: experts"
    assert np.array_equal(got["pos"], want["pos"]), f"{what}: positions"
    assert np.array_equal(got["counts"], want["counts"]), f"{what}: per-expert counts"
    assert got["overflow"] == want["overflow"], f"{what}: overflow"
    np.testing.assert_allclose(got["weight"], want["weight"], rtol=4 * top_k * 2.0 ** -24, atol=0, err_msg=what)
    return want


def test_reference_unit_test_vectors(hip, torch, oracle):
    print("route: reference vectors", flush=True)
    # src/moe/routing.rs:462-466: topk_indices([.1,.5,.3,.9,.2], 2) == [3, 1] (softmax keeps the order)
    r = route(hip, torch, [[0.1, 0.5, 0.3, 0.9, 0.2]], 2, capacity_factor=5.0)
    assert r["expert"][0].tolist() == [3, 1] and r["len"][0] == 2
    # src/moe/routing.rs:469-478: weights renormalise to 1, best expert first
    r = route(hip, torch, [[1.0, 2.0, 3.0, 4.0]], 2, capacity_factor=4.0)
    assert r["expert"][0].tolist() == [3, 2]
    assert abs(float(r["weight"][0].sum()) - 1.0) < 1e-6 and r["weight"][0, 0] > r["weight"][0, 1]
    # src/moe/routing.rs:1620-1640: equal logits give 0.5 / 0.5, lower index first
    r = route(hip, torch, [[0.0, 0.0]], 2, capacity_factor=2.0)
    assert r["expert"][0].tolist() == [0, 1] and r["weight"][0].tolist() == [0.5, 0.5]
    # src/moe/routing.rs:516-540: four tokens all prefer expert 0, capacity 1: one keeps it, the
    # others fall back to the least loaded expert with weight 1
    lg = np.array([[10.0, 0.0]] * 4, np.float32)
    r = route(hip, torch, lg, 1, capacity_factor=0.5)
    check_against_oracle(oracle, r, lg, 1, 0.5, "capacity 1")
    assert r["expert"][:, 0].tolist() == [0, 1, 0, 1] and r["weight"][1:, 0].tolist() == [1.0, 1.0, 1.0]
    # src/moe/routing.rs:543-547: expert_capacity(128) = 20 for 8 experts at the default factor
    lg = random_gate_logits(128, 8, seed=3)
    r = route(hip, torch, lg, 2)
    w = check_against_oracle(oracle, r, lg, 2, 1.25, "128 tokens, 8 experts")
    # a kept choice sits below the capacity; only the weight-1 fallbacks go beyond it
    kept = np.arange(2)[None, :] < r["len"][:, None]
    assert bool(((r["pos"] < 20) | (r["weight"] == 1.0))[kept].all()) and w["overflow"] > 0


def test_baseline_shape_default_and_open_capacity(hip, torch, oracle):
    """16 tokens over 128 experts, top-8: with capacity_factor = experts nothing is dropped; with
    the reference's default 1.25 the capacity is 1 and most choices overflow."""
    for seed in range(6):
        lg = random_gate_logits(16, 128, seed=seed)
        print(f"route: 16 x 128 top-8 seed={seed}", flush=True)
        r = route(hip, torch, lg, 8, capacity_factor=128.0)
        w = check_against_oracle(oracle, r, lg, 8, 128.0, f"seed {seed} open")
        assert int(w["len"].sum()) == 128 and w["overflow"] == 0
        r = route(hip, torch, lg, 8)
        w = check_against_oracle(oracle, r, lg, 8, 1.25, f"seed {seed} default")
        assert int(w["counts"].max()) == 1 and w["overflow"] > 0


def test_random_shapes_both_launch_forms(hip, torch, oracle):
    """Seeded shapes on both sides of the one-launch limit (64 tokens), top_k from 1 up to more
    than the experts, capacity factors that drop nothing, some, and nearly everything."""
    rng = np.random.default_rng(11)
    for case in range(40):
        tokens = int(rng.integers(1, 65)) if case % 2 == 0 else int(rng.integers(65, 700))
        experts = int(rng.integers(1, 200))
        top_k = int(rng.integers(1, min(experts + 2, 12)))
        factor = [float(experts), 1.25, 0.3, 2.0, 0.0][case % 5]
        lg = rng.standard_normal((tokens, experts)).astype(np.float32) * float(rng.choice([0.1, 1.0, 8.0]))
        print(f"route case {case}: T={tokens} E={experts} k={top_k} cf={factor}", flush=True)
        r = route(hip, torch, lg, top_k, capacity_factor=factor)
        check_against_oracle(oracle, r, lg, top_k, factor, f"case {case}")


def test_ties_nan_and_infinite_logits(hip, torch, oracle):
    print("route: ties, NaN, infinities", flush=True)
    # equal logits: the stable order keeps the lower index first
    lg = np.zeros((3, 10), np.float32)
    lg[1, 4] = lg[1, 7] = 2.0
    r = route(hip, torch, lg, 4, capacity_factor=10.0)
    check_against_oracle(oracle, r, lg, 4, 10.0, "ties")
    assert r["expert"][0].tolist() == [0, 1, 2, 3] and r["expert"][1].tolist() == [4, 7, 0, 1]
    # a NaN or +inf logit makes the softmax sum NaN: every probability becomes 1 / experts;
    # a row of -inf does the same; a single -inf entry just gets probability 0
    lg = np.array([[0.5, np.nan, 1.0, 2.0], [np.inf, 0.0, 1.0, 2.0], [-np.inf] * 4, [0.0, -np.inf, 1.0, -1.0]], np.float32)
    r = route(hip, torch, lg, 2, capacity_factor=4.0)
    check_against_oracle(oracle, r, lg, 2, 4.0, "non-finite")
    assert r["expert"][0].tolist() == [0, 1] and r["weight"][0].tolist() == [0.5, 0.5]
    assert r["expert"][2].tolist() == [0, 1] and r["expert"][3].tolist() == [2, 0]
    # very large and very small logits: exp underflows to 0 for all but the maximum
    lg = np.array([[1000.0, -1000.0, 999.0, 0.0, 1.0e30, -1.0e30]], np.float32)
    r = route(hip, torch, lg, 3, capacity_factor=6.0)
    check_against_oracle(oracle, r, lg, 3, 6.0, "huge")


def test_route_error_behaviour(hip, torch):
    from gllm_amd.backend import OtherError, Unimplemented
    print("route: errors", flush=True)
    lg = torch.zeros(2, 5000, device="cuda")
    re = torch.zeros(2, 2, dtype=torch.int32, device="cuda")
    rw = torch.zeros(2, 2, device="cuda")
    rl = torch.zeros(2, dtype=torch.int32, device="cuda")
    with pytest.raises(Unimplemented):
        hip.moe_route(lg, 2, re, rw, rl)  # more experts than this build routes
    with pytest.raises(OtherError):
        hip.moe_route(lg[:, :8].contiguous(), 2, re[:1], rw, rl)  # outputs too short
