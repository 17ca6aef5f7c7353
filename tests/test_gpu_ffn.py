"""GPU parity of the dense feed-forward block (gllmq_ffn_swiglu through the C ABI) against the
oracle's float64-accumulated evaluation: rel-L2 <= 1e-4 and |err| <= 1e-3 max|y|, the matmul bar."""
import numpy as np
import pytest

from gllm_amd.synth import random_activations, random_weight

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
ALL = [Q8_0, Q4_K, Q5_K, Q6_K]
GUARD = 4096


@pytest.fixture(scope="module")
def hip():
    from gllm_amd.backend import HipBackend
    return HipBackend(0)


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def dev_bytes(torch, host):
    flat = torch.from_numpy(np.asarray(host).view(np.uint8).reshape(-1))
    buf = torch.full((flat.numel() + GUARD,), 0xFF, dtype=torch.uint8, device="cuda")
    buf[:flat.numel()] = flat.cuda()
    return buf[:flat.numel()]


def run_ffn(hip, torch, gate, up, t_gu, down, t_dn, x, m, hidden, ffn, relu=False, stacked=False):
    if stacked:  # up rows right behind the gate rows, as one [2 ffn x hidden] tensor
        both = dev_bytes(torch, np.concatenate([np.asarray(gate).view(np.uint8).reshape(-1),
                                                np.asarray(up).view(np.uint8).reshape(-1)]))
        half = both.numel() // 2
        gd, ud = both[:half], both[half:]
    else:
        gd, ud = dev_bytes(torch, gate), dev_bytes(torch, up)
    dd = dev_bytes(torch, down)
    xbuf = torch.full((m * hidden + GUARD,), float("nan"), dtype=torch.float32, device="cuda")
    xbuf[:m * hidden] = torch.from_numpy(np.ascontiguousarray(x, np.float32).reshape(-1)).cuda()
    obuf = torch.full((m * hidden + GUARD,), float("nan"), dtype=torch.float32, device="cuda")
    obuf[m * hidden:] = 7.0
    hip.ffn_swiglu(gd, ud, t_gu, dd, t_dn, xbuf[:m * hidden], obuf[:m * hidden], m, hidden, ffn, relu_gate=relu)
    torch.cuda.synchronize()
    assert bool(torch.all(obuf[m * hidden:] == 7.0)), "write past the end of the output"
    return obuf[:m * hidden].cpu().numpy().reshape(m, hidden)


def check(got, want, what):
    got, want = got.astype(np.float64), want.astype(np.float64)
    rel = np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-300)
    worst = np.abs(got - want).max() / max(np.abs(want).max(), 1e-300)
    assert rel <= 1e-4 and worst <= 1e-3, f"{what}: rel_l2={rel:.3e} max_err/max|y|={worst:.3e}"


@pytest.mark.parametrize("t_gu", ALL)
@pytest.mark.parametrize("t_dn", [Q6_K, Q4_K, Q8_0])
def test_ffn_all_format_pairs(hip, torch, oracle, t_gu, t_dn):
    hidden, ffn = 1024, 1536
    gate, up = random_weight(t_gu, ffn, hidden, seed=1), random_weight(t_gu, ffn, hidden, seed=2)
    down = random_weight(t_dn, hidden, ffn, seed=3)
    for m in (1, 2, 5, 8, 9, 33):
        print(f"ffn gate/up={t_gu} down={t_dn} m={m}", flush=True)
        x = random_activations(m, hidden, seed=10 + m)
        want = oracle.ffn_swiglu(gate, up, t_gu, down, t_dn, x, m, hidden, ffn, acc=oracle.ACC_F64, threads=4)
        got = run_ffn(hip, torch, gate, up, t_gu, down, t_dn, x, m, hidden, ffn, stacked=(m % 2 == 1))
        check(got, want, f"gu={t_gu} dn={t_dn} m={m}")


@pytest.mark.parametrize("t_gu", [Q4_K, Q5_K])
def test_ffn_ragged_shapes_and_relu_gate(hip, torch, oracle, t_gu):
    # ffn not a multiple of 32 (a partial last tile in both halves), hidden with 2 and 3 passes per tile
    for hidden, ffn, m, relu in [(2560, 1000, 1, False), (4096, 776, 2, True), (6144, 520, 4, False), (512, 33, 7, True),
                                 (6144, 2100, 1, True), (8192, 2048, 1, False), (1024, 2304, 3, False)]:
        print(f"ffn ragged gate/up={t_gu} hidden={hidden} ffn={ffn} m={m} relu={relu}", flush=True)
        gate, up = random_weight(t_gu, ffn, hidden, seed=ffn), random_weight(t_gu, ffn, hidden, seed=ffn + 1)
        down = random_weight(Q8_0, hidden, ffn, seed=ffn + 2)
        x = random_activations(m, hidden, seed=m)
        want = oracle.ffn_swiglu(gate, up, t_gu, down, Q8_0, x, m, hidden, ffn, relu_gate=relu, acc=oracle.ACC_F64, threads=4)
        got = run_ffn(hip, torch, gate, up, t_gu, down, Q8_0, x, m, hidden, ffn, relu=relu)
        check(got, want, f"gu={t_gu} hidden={hidden} ffn={ffn} m={m}")


def test_ffn_layer_shape(hip, torch, oracle):
    """The decode shape of the layer mix: Q4_K gate/up 4096 -> 14336, Q6_K down 14336 -> 4096."""
    hidden, ffn = 4096, 14336
    print("ffn 4096/14336", flush=True)
    gate, up = random_weight(Q4_K, ffn, hidden, seed=21), random_weight(Q4_K, ffn, hidden, seed=22)
    down = random_weight(Q6_K, hidden, ffn, seed=23)
    for m in (1, 2, 4, 16):  # (two to four rows: the down projection's workgroups share slices of K)
        x = random_activations(m, hidden, seed=24 + m)
        want = oracle.ffn_swiglu(gate, up, Q4_K, down, Q6_K, x, m, hidden, ffn, acc=oracle.ACC_F64, threads=16)
        got = run_ffn(hip, torch, gate, up, Q4_K, down, Q6_K, x, m, hidden, ffn, stacked=True)
        check(got, want, f"layer shape m={m}")


def test_ffn_three_step_form(torch, oracle):
    """Option ffn_fused = 0: the two products, the activation kernel, the down projection."""
    from gllm_amd.backend import HipBackend
    hip2 = HipBackend(0, options={"ffn_fused": 0})
    hidden, ffn = 1024, 800
    gate, up = random_weight(Q4_K, ffn, hidden, seed=1), random_weight(Q4_K, ffn, hidden, seed=2)
    down = random_weight(Q6_K, hidden, ffn, seed=3)
    for m, stacked in [(1, True), (1, False), (4, True), (70, False)]:
        print(f"ffn three steps m={m} stacked={stacked}", flush=True)
        x = random_activations(m, hidden, seed=m)
        want = oracle.ffn_swiglu(gate, up, Q4_K, down, Q6_K, x, m, hidden, ffn, acc=oracle.ACC_F64, threads=4)
        got = run_ffn(hip2, torch, gate, up, Q4_K, down, Q6_K, x, m, hidden, ffn, stacked=stacked)
        check(got, want, f"three steps m={m}")


@pytest.mark.parametrize("t_gu,t_dn,hidden,ffn,ms", [
    (Q6_K, Q6_K, 2048, 4352, (1, 2, 4, 8)),    # GEMV gate/up; streamed down projection that reads the gated product
    (Q8_0, Q4_K, 2048, 4608, (1, 3)),          # Q8_0 gate/up, streamed Q4_K down
    (Q6_K, Q6_K, 2048, 8192, (2, 4)),          # the down projection's workgroups share slices of K and read the gated product
    (Q8_0, Q5_K, 1024, 8448, (3,)),
    (Q6_K, Q8_0, 1024, 1536, (1, 2, 5)),       # GEMV down projection (two rows at a time)
    (Q4_K, Q5_K, 2048, 5120, (16, 40)),        # GEMM: the preparation launch of the down projection applies the gate
    (Q6_K, Q6_K, 512, 776, (1, 9)),            # ragged ffn
    (Q8_0, Q8_0, 256, 200, (1, 2, 70)),        # ffn not a multiple of 64: the GEMV's scalar loads
    (Q6_K, Q6_K, 2048, 4096, (5, 8)),          # five to eight rows: kernels of four row pairs that read the gated product
    (Q4_K, Q8_0, 2048, 4352, (6, 7)),
    (Q5_K, Q4_K, 4096, 3072, (5, 8)),
    (Q4_K, Q5_K, 1024, 2560, (7,)),
    (Q4_K, Q6_K, 4096, 14336, (6,)),           # rows of 14336 elements: a K split, or passes of fewer rows than the call has
])
def test_down_projection_reads_the_gated_product(torch, oracle, t_gu, t_dn, hidden, ffn, ms):
    """Where the gate/up products are not gated in their kernel's epilogue, the down projection's
    activation loads apply act(gate) * up themselves (no launch and no buffer for it): the same bits
    as with the activation as a launch of its own (option ffn_glu_load = 0), for stacked and
    separate gate/up tensors and the ReLU gate; and the oracle's bars."""
    from gllm_amd.backend import HipBackend
    # 9 to 16 rows without gated loads would take the kernel that prepares its own operands: another
    # order of sums; the comparison here is the same kernel with and without the gated loads
    fused = HipBackend(0, options={"ffn_fused": 0, "mmfr": 0})
    plain = HipBackend(0, options={"ffn_fused": 0, "ffn_glu_load": 0, "mmfr": 0})
    gate, up = random_weight(t_gu, ffn, hidden, seed=1), random_weight(t_gu, ffn, hidden, seed=2)
    down = random_weight(t_dn, hidden, ffn, seed=3)
    for m in ms:
        for stacked, relu in ((True, False), (False, True)):
            print(f"gated loads gate/up={t_gu} down={t_dn} hidden={hidden} ffn={ffn} m={m} stacked={stacked} relu={relu}", flush=True)
            x = random_activations(m, hidden, seed=m)
            got = run_ffn(fused, torch, gate, up, t_gu, down, t_dn, x, m, hidden, ffn, relu=relu, stacked=stacked)
            ref = run_ffn(plain, torch, gate, up, t_gu, down, t_dn, x, m, hidden, ffn, relu=relu, stacked=stacked)
            if 5 <= m <= 8:  # (the streamed kernel of four row pairs, or the fetch-and-compute one, with gated loads)
                assert fused.last_kernel_name().endswith("_p4_e4_g"), fused.last_kernel_name()
            assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), "differs from the activation as its own launch"
            want = oracle.ffn_swiglu(gate, up, t_gu, down, t_dn, x, m, hidden, ffn, relu_gate=relu, acc=oracle.ACC_F64, threads=8)
            check(got, want, f"gated loads m={m}")


def test_ffn_argument_errors(hip, torch):
    from gllm_amd.backend import BackendError, Unimplemented
    print("ffn errors", flush=True)
    w = torch.zeros(144 * 64, dtype=torch.uint8, device="cuda")
    x = torch.zeros(256, device="cuda")
    out = torch.full((256,), 7.0, device="cuda")
    with pytest.raises(Unimplemented):
        hip.ffn_swiglu(w, w, 2, w, Q4_K, x, out, 1, 256, 256)      # Q4_0 gate/up
    with pytest.raises(BackendError):
        hip.ffn_swiglu(w[:100], w, Q4_K, w, Q4_K, x, out, 1, 256, 64)  # gate shorter than 64 rows
    hip.ffn_swiglu(w, w, Q4_K, w, Q4_K, x, out, 0, 256, 64)       # no rows: nothing written
    torch.cuda.synchronize()
    assert bool(torch.all(out == 7.0))


@pytest.mark.parametrize("seed", [21, 22])
def test_ffn_shapes_from_a_seeded_generator(hip, torch, oracle, seed):
    """Rows, widths, formats, the ReLU gate and stacked or separate gate/up tensors drawn from a
    seeded generator: every path of the block (gated kernels, gated activation loads of the down
    projection for one to eight rows, the activation launch, the GEMMs) at sizes nobody chose."""
    rng = np.random.default_rng(seed)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    seen = set()
    for i in range(14):
        t_gu, t_dn = int(rng.choice(ALL)), int(rng.choice(ALL))
        m = int(rng.choice([1, 1, 2, 3, 4, 6, 8, 9, 16, 20]))
        hidden = 256 * int(rng.choice([2, 4, 8, 16]))
        ffn = 256 * int(rng.choice([1, 3, 6, 11, 14])) if rng.integers(0, 2) else int(rng.choice([8, 16, 33])) * cus
        ffn = max(256, (ffn // 256) * 256)  # the down projection's rows are whole blocks here
        relu = bool(rng.integers(0, 2))
        print(f"ffn seeded {seed}/{i}: gu={t_gu} dn={t_dn} m={m} hidden={hidden} ffn={ffn} relu={relu}", flush=True)
        gate, up = random_weight(t_gu, ffn, hidden, seed=seed * 10 + i), random_weight(t_gu, ffn, hidden, seed=seed * 20 + i)
        down = random_weight(t_dn, hidden, ffn, seed=seed * 30 + i)
        x = random_activations(m, hidden, seed=seed * 40 + i)
        want = oracle.ffn_swiglu(gate, up, t_gu, down, t_dn, x, m, hidden, ffn, relu_gate=relu, acc=oracle.ACC_F64, threads=16)
        got = run_ffn(hip, torch, gate, up, t_gu, down, t_dn, x, m, hidden, ffn, relu=relu, stacked=bool(i & 1))
        check(got, want, f"ffn seeded {seed}/{i} kernel={hip.last_kernel_name()}")
        seen.add(hip.last_kernel_name())
    print("last kernels met:", sorted(seen), flush=True)
