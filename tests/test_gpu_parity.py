"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same inputs.

Bars: dequantized weights bit-exact; matmul outputs rel-L2 <= 1e-4 and per-element
|err| <= 1e-3 * max|y| against the oracle's float64 accumulation.
"""
import numpy as np
import pytest

from gllm_amd.synth import random_activations, random_blocks, random_weight

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
ALL = [Q8_0, Q4_K, Q5_K, Q6_K]
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


GUARD = 4096  # elements of poison behind every device input: a read past the end shows up as NaN


def guarded(torch, host, fill):
    """`host` on the device at the start of a buffer whose tail is `fill` (NaN for floats, 0xFF
    bytes for blocks: an f16 scale of 0xFFFF is a NaN)."""
    flat = torch.from_numpy(np.ascontiguousarray(host).reshape(-1))
    buf = torch.full((flat.numel() + GUARD,), fill, dtype=flat.dtype, device="cuda")
    buf[:flat.numel()] = flat.cuda()
    return buf[:flat.numel()]


def gpu_matmul(hip, torch, w, x, dtype, m, n, k, act_mode=0):
    wd = guarded(torch, np.asarray(w).view(np.uint8), 0xFF)
    xd = guarded(torch, np.ascontiguousarray(x, np.float32), float("nan")).view(m, k)
    # outputs start as NaN (an element nobody writes stays visible); a marker behind them must survive
    ybuf = torch.full((m * n + GUARD,), float("nan"), dtype=torch.float32, device="cuda")
    ybuf[m * n:] = 7.0
    yd = ybuf[:m * n].view(m, n)
    hip.quantized_matmul(wd, xd, yd, dtype, m, n, k, act_mode=act_mode)
    torch.cuda.synchronize()
    assert bool(torch.all(ybuf[m * n:] == 7.0)), "write past the end of the output"
    return yd.cpu().numpy()


# ---------------------------------------------------------------- dequantize
@pytest.mark.parametrize("dtype", ALL)
def test_dequantize_bit_exact(hip, torch, oracle, dtype):
    print(f"dequantize dtype={dtype}", flush=True)
    nb = 1031
    raw = random_blocks(dtype, nb, seed=100 + dtype)
    blocks = raw.reshape(nb, -1)
    off = {Q8_0: 0, Q4_K: 0, Q5_K: 0, Q6_K: 208}[dtype]
    for i, pat in enumerate([0x0001, 0x03FF, 0x0000, 0x8000, 0xBC00, 0x7BFF, 0x0400, 0x8001]):
        blocks[i, off:off + 2] = np.array([pat], np.uint16).view(np.uint8)
    want = oracle.dequantize(raw, dtype)
    bd = torch.from_numpy(raw).cuda()
    od = torch.zeros(want.size, dtype=torch.float32, device="cuda")
    hip.dequantize(bd, od, dtype)
    torch.cuda.synchronize()
    got = od.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # host-slice form of the same call (the reference's signature)
    out = np.zeros(want.size, np.float32)
    hip.dequantize(raw, out, dtype)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("dtype", ALL)
def test_dequantize_partial_chunks_and_odd_alignment(hip, torch, oracle, dtype):
    print(f"dequantize partial dtype={dtype}", flush=True)
    bb, bs = oracle.block_bytes(dtype), oracle.block_size(dtype)
    raw = random_blocks(dtype, 5, seed=7)
    want = oracle.dequantize(raw, dtype)
    # input one byte short of 5 blocks, output with room for 5: four blocks decoded
    bd = torch.from_numpy(raw[: 5 * bb - 1].copy()).cuda()
    od = torch.full((5 * bs,), -1.0, dtype=torch.float32, device="cuda")
    hip.dequantize(bd, od, dtype)
    got = od.cpu().numpy()
    assert np.array_equal(got[: 4 * bs], want[: 4 * bs]) and np.all(got[4 * bs:] == -1.0)
    # output short: three whole blocks fit; output pointer only 4-byte aligned; input at an odd address
    shifted = torch.zeros(5 * bb + 1, dtype=torch.uint8, device="cuda")
    shifted[1:] = torch.from_numpy(raw).cuda()
    buf = torch.full((3 * bs + 9,), -1.0, dtype=torch.float32, device="cuda")
    hip.dequantize(shifted[1:], buf[1:], dtype)
    got = buf.cpu().numpy()
    assert got[0] == -1.0 and np.array_equal(got[1: 1 + 3 * bs], want[: 3 * bs]) and np.all(got[1 + 3 * bs:] == -1.0)
    # empty input is a no-op
    hip.dequantize(bd[:0], od, dtype)


# -------------------------------------------------------------------- GEMV
SHAPES = [  # (n, k)
    (33, 256), (7, 512), (64, 1536), (100, 4096), (40, 14336), (19, 8192), (5, 20480), (3, 11008),
]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("n,k", SHAPES)
def test_gemv_m1_matches_oracle(hip, torch, oracle, dtype, n, k):
    print(f"gemv dtype={dtype} n={n} k={k}", flush=True)
    w, x = random_weight(dtype, n, k, seed=n + k), random_activations(1, k, seed=k)
    want = oracle.quantized_matmul(w, x, dtype, 1, n, k, acc=oracle.ACC_F64, threads=4)
    got = gpu_matmul(hip, torch, w, x, dtype, 1, n, k)
    check_close(got, want, f"dtype={dtype} n={n} k={k}")


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("m", [2, 3, 5, 8])
def test_small_m_matches_oracle(hip, torch, oracle, dtype, m):
    n, k = 77, 4096
    print(f"small-m dtype={dtype} m={m}", flush=True)
    w, x = random_weight(dtype, n, k, seed=m), random_activations(m, k, seed=m)
    want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
    got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
    check_close(got, want, f"dtype={dtype} m={m}")


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("m", [3, 8])
def test_small_m_down_projection_shape(hip, torch, oracle, dtype, m):
    # K = 14336: the prepared activations of all rows do not fit the LDS of one pass of the
    # 8-row kernels, so these few rows take the GEMM kernels
    n, k = 70, 14336
    print(f"small-m long rows dtype={dtype} m={m}", flush=True)
    w, x = random_weight(dtype, n, k, seed=40 + m), random_activations(m, k, seed=41)
    want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
    got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
    check_close(got, want, f"dtype={dtype} m={m} k={k}")


@pytest.mark.parametrize("dtype,k", [(Q4_K, 300), (Q5_K, 511), (Q6_K, 257), (Q8_0, 40), (Q8_0, 4000), (Q4_K, 4100)])
def test_row_padding(hip, torch, oracle, dtype, k):
    print(f"padding dtype={dtype} k={k}", flush=True)
    n = 21
    w, x = random_weight(dtype, n, k, seed=3), random_activations(2, k, seed=3)
    want = oracle.quantized_matmul(w, x, dtype, 2, n, k, acc=oracle.ACC_F64)
    got = gpu_matmul(hip, torch, w, x, dtype, 2, n, k)
    check_close(got, want, f"dtype={dtype} k={k}")
    got1 = gpu_matmul(hip, torch, w, x[:1], dtype, 1, n, k)
    check_close(got1, want[:1], f"dtype={dtype} k={k} m=1")


@pytest.mark.parametrize("dtype", ALL)
def test_unit_vector_returns_weight_column_bit_exactly(hip, torch, oracle, dtype):
    print(f"unit vector dtype={dtype}", flush=True)
    n, k = 50, 1024
    w = random_weight(dtype, n, k, seed=12)
    deq = oracle.dequantize(w, dtype).reshape(n, k)
    for col in (0, 31, 32, 63, 64, 255, 256, 700, 1023):
        x = np.zeros((1, k), np.float32)
        x[0, col] = 1.0
        got = gpu_matmul(hip, torch, w, x, dtype, 1, n, k)
        # value equality: a sum of zeros is +0 where the decoder's d*sc*0 may be -0
        assert np.array_equal(got[0], deq[:, col]), f"col {col}"


def test_linearity_at_full_size(hip, torch):
    # size-independent property at the headline shape: Q4_K 4096 -> 14336
    n, k = 14336, 4096
    print("linearity 14336x4096", flush=True)
    w = random_weight(Q4_K, n, k, seed=0)
    x1, x2 = random_activations(1, k, seed=1), random_activations(1, k, seed=2)
    y1 = gpu_matmul(hip, torch, w, x1, Q4_K, 1, n, k).astype(np.float64)
    y2 = gpu_matmul(hip, torch, w, x2, Q4_K, 1, n, k).astype(np.float64)
    y12 = gpu_matmul(hip, torch, w, 3.0 * x1 - 2.0 * x2, Q4_K, 1, n, k)
    check_close(y12, 3.0 * y1 - 2.0 * y2, "linearity")


@pytest.mark.parametrize("dtype,n,k", [(Q4_K, 4096, 4096), (Q4_K, 14336, 4096), (Q6_K, 14336, 4096),
                                       (Q6_K, 4096, 14336), (Q4_K, 6144, 4096)])
def test_baseline_shapes_match_oracle(hip, torch, oracle, dtype, n, k):
    print(f"baseline shape dtype={dtype} n={n} k={k}", flush=True)
    w, x = random_weight(dtype, n, k, seed=0), random_activations(1, k, seed=0)
    want = oracle.quantized_matmul(w, x, dtype, 1, n, k, acc=oracle.ACC_F64, threads=8)
    got = gpu_matmul(hip, torch, w, x, dtype, 1, n, k)
    rel = check_close(got, want, f"dtype={dtype} n={n} k={k}")
    print(f"  rel_l2={rel:.3e}", flush=True)
    # host-slice form of the call on the smallest of them
    if n == 4096 and k == 4096:
        out = np.zeros((1, n), np.float32)
        hip.quantized_matmul(w, x, out, dtype, 1, n, k)
        assert np.array_equal(out, got)


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("m", [9, 16, 17, 33, 70])
def test_batched_m_matches_oracle(hip, torch, oracle, dtype, m):
    n, k = 203, 2048
    print(f"batched-m dtype={dtype} m={m}", flush=True)
    w, x = random_weight(dtype, n, k, seed=m), random_activations(m, k, seed=m + 1)
    want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
    got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
    check_close(got, want, f"dtype={dtype} m={m}")


@pytest.mark.parametrize("m", [16, 32, 64])
def test_batched_decode_baseline_shape(hip, torch, oracle, m):
    # Q4_K, K=4096, N=14336, M in {16, 32, 64}
    n, k = 14336, 4096
    print(f"batched decode m={m}", flush=True)
    w, x = random_weight(Q4_K, n, k, seed=0), random_activations(m, k, seed=5)
    want = oracle.quantized_matmul(w, x, Q4_K, m, n, k, acc=oracle.ACC_F64, threads=16)
    got = gpu_matmul(hip, torch, w, x, Q4_K, m, n, k)
    rel = check_close(got, want, f"m={m}")
    print(f"  rel_l2={rel:.3e}", flush=True)


def test_decode_layer_mix_batch(hip, torch, oracle):
    """QKV 4096->6144 (Q4_K), O 4096->4096 (Q4_K), gate+up 4096->2x14336 (Q4_K), down 14336->4096
    (Q6_K) enqueued by one batch call, each fed a fresh N(0,1) vector."""
    print("layer mix", flush=True)
    ops = [(Q4_K, 6144, 4096), (Q4_K, 4096, 4096), (Q4_K, 2 * 14336, 4096), (Q6_K, 4096, 14336)]
    descs, wants, outs = [], [], []
    for i, (dtype, n, k) in enumerate(ops):
        w, x = random_weight(dtype, n, k, seed=20 + i), random_activations(1, k, seed=30 + i)
        wants.append(oracle.quantized_matmul(w, x, dtype, 1, n, k, acc=oracle.ACC_F64, threads=16))
        wd = hip.upload_weights(w)
        xd = torch.from_numpy(x).cuda()
        yd = torch.full((1, n), float("nan"), dtype=torch.float32, device="cuda")
        descs.append((wd, xd, yd, dtype, 1, n, k))
        outs.append(yd)
    hip.quantized_matmul_batch(descs)
    torch.cuda.synchronize()
    for (dtype, n, k), yd, want in zip(ops, outs, wants):
        check_close(yd.cpu().numpy(), want, f"layer mix dtype={dtype} n={n} k={k}")


def test_batch_overlap_keeps_results_and_order(hip, torch, oracle):
    """The kernels of a batch of independent matmuls may overlap on the device.  A batch with
    several users of the stream's scratch (two K-split launches, two GEMMs, which must not overlap
    with each other), a chain of entries that depend on each other (each reads what the one before
    it wrote, marked GLLMQ_DESC_AFTER_PREVIOUS) and plain one-row entries, repeated several times
    with work of the caller's own behind it on the same stream: every result equals, bit for bit,
    what the same entries give one call at a time."""
    from gllm_amd.backend import HipBackend
    print("batch overlap", flush=True)
    serial = HipBackend(0, options={"batch_overlap": 0})
    shapes = [(Q4_K, 1, 8192, 4096), (Q6_K, 1, 2048, 11008), (Q4_K, 16, 1024, 2048), (Q5_K, 2, 1024, 12288),
              (Q8_0, 12, 512, 1024), (Q4_K, 1, 4096, 4096), (Q6_K, 3, 4096, 4096)]
    base = []
    for i, (dtype, m, n, k) in enumerate(shapes):
        w = hip.upload_weights(random_weight(dtype, n, k, seed=50 + i))
        x = torch.from_numpy(random_activations(m, k, seed=60 + i)).cuda()
        base.append((w, x, dtype, m, n, k))
    # a dependent chain: 4096 -> 4096 -> 4096, each entry reading the previous entry's output
    chain_w = [hip.upload_weights(random_weight(Q4_K, 4096, 4096, seed=70 + i)) for i in range(3)]
    chain_x0 = torch.from_numpy(random_activations(1, 4096, seed=77)).cuda()

    def build(backend):
        outs, descs, dep = [], [], []
        for w, x, dtype, m, n, k in base:
            y = torch.full((m, n), float("nan"), device="cuda")
            descs.append((w, x, y, dtype, m, n, k))
            dep.append(False)
            outs.append(y)
        cur = chain_x0
        for i, w in enumerate(chain_w):
            y = torch.full((1, 4096), float("nan"), device="cuda")
            descs.append((w, cur, y, Q4_K, 1, 4096, 4096))
            dep.append(i > 0)
            outs.append(y)
            cur = y
        return backend.make_batch(descs, after_previous=lambda i: dep[i]), descs, outs

    batch_s, descs_s, outs_s = build(serial)
    for w, x, y, dtype, m, n, k in descs_s:  # one call at a time
        serial.quantized_matmul(w, x, y, dtype, m, n, k)
    torch.cuda.synchronize()
    want = [o.clone() for o in outs_s]
    # the chain against the oracle, so that "equal to serial" means "right"
    hx = chain_x0.cpu().numpy()
    for i in range(3):
        hw = chain_w[i].cpu().numpy()
        hx = oracle.quantized_matmul(hw, hx.astype(np.float32), Q4_K, 1, 4096, 4096, acc=oracle.ACC_F64, threads=8)
    check_close(want[-1].cpu().numpy(), hx, "dependent chain")
    batch_o, descs_o, outs_o = build(hip)
    for rep in range(5):
        for o in outs_o:
            o.fill_(float("nan"))
        hip.run_batch(batch_o)
        after = outs_o[-1] * 2.0  # the caller's own work behind the batch sees finished results
        torch.cuda.synchronize()
        for i, (o, wnt) in enumerate(zip(outs_o, want)):
            assert torch.equal(o.view(torch.int32), wnt.view(torch.int32)), f"rep {rep} entry {i}"
        assert torch.equal(after, want[-1] * 2.0)
    with pytest.raises(Exception):
        bad = hip.make_batch(descs_o[:1])
        bad[0].flags = 6
        hip.run_batch(bad)


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("m", [1, 16, 40])
def test_bf16_activation_mode(hip, torch, oracle, dtype, m):
    """GLLMQ_ACT_BF16: exact weights times activations rounded to bf16 (ties to even)."""
    from gllm_amd.backend import ACT_BF16
    from oracle import npref
    n, k = 301, 4096
    print(f"bf16 activations dtype={dtype} m={m}", flush=True)
    w, x = random_weight(dtype, n, k, seed=9), random_activations(m, k, seed=10)
    assert npref.bf16_rne(np.array([1.0, -1.0], np.float32)).view(np.uint32).tolist() == [0x3F800000, 0xBF800000]
    xb = npref.bf16_rne(x)
    want = oracle.quantized_matmul(w, xb, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
    got = gpu_matmul(hip, torch, w, x, dtype, m, n, k, act_mode=ACT_BF16)
    check_close(got, want, f"bf16 dtype={dtype} m={m}")
    # and it is a different computation from the f32 one: the rounding shows
    full = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
    rel = np.linalg.norm(got - full) / np.linalg.norm(full)
    assert rel > 3e-4, rel


@pytest.mark.parametrize("env", [{"mm8": 0, "mmf": 0}, {"mmf": 0},
                                 {"gemv_f32": 1, "mm8": 0, "mmf": 0},
                                 {"mm8_q6k_min_m": 1, "mm8_q5k_min_m": 1, "mm8_q8_0_min_m": 1},
                                 {"mm8_q6k_min_m": 0, "mm8_q5k_min_m": 0, "mm8_q8_0_min_m": 0},
                                 {"mmf_small_min_m": 0}, {"mm8_ksplit": 0},
                                 {"mm8_ksplit": 2, "mmf_small_min_m": 0}])
def test_alternative_kernel_paths(torch, oracle, env):
    """The kernels the default dispatch does not pick: integer-dot GEMV for Q4_K, 8-row passes
    for more than 8 rows, the f32 multiply-add flavour, Q5_K and Q6_K on the matrix cores from one
    row up and on the GEMV kernels throughout (Q8_0 too), no GEMM for few rows; selected per context at init."""
    from gllm_amd.backend import HipBackend
    hip2 = HipBackend(0, options=env)
    print(f"alternative paths {env}", flush=True)
    for dtype in ALL:
        for m in (1, 2, 5, 11):
            n, k = 130, 2048
            w, x = random_weight(dtype, n, k, seed=dtype + m), random_activations(m, k, seed=m)
            want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
            got = gpu_matmul(hip2, torch, w, x, dtype, m, n, k)
            check_close(got, want, f"env={env} dtype={dtype} m={m}")
    if "mmf_small_min_m" in env:
        # long rows on the 8-row kernels: several passes over the weights, seven blocks per wave and tile
        for dtype in ALL:
            for m in (3, 8):
                n, k = 70, 14336
                w, x = random_weight(dtype, n, k, seed=40 + m), random_activations(m, k, seed=41)
                want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
                got = gpu_matmul(hip2, torch, w, x, dtype, m, n, k)
                check_close(got, want, f"env={env} dtype={dtype} m={m} k={k}")


def test_random_shapes_sweep(hip, torch, oracle):
    """Sixty seeded shapes across the formats, row counts on both sides of every kernel boundary
    (1, 2, 3, 8, 9, 32, 33, 64, 65 and random ones), ragged n, k with and without a partial block."""
    rng = np.random.default_rng(2024)
    edge_m = [1, 2, 3, 8, 9, 32, 33, 64, 65]
    for case in range(60):
        dtype = ALL[case % len(ALL)]
        m = edge_m[case % len(edge_m)] if case < 36 else int(rng.integers(1, 71))
        n = int(rng.integers(1, 300))
        step = 32 if dtype == Q8_0 else 256
        k = int(rng.integers(1, 12)) * step
        if case % 5 == 4:
            k -= int(rng.integers(1, step // 4)) * 4  # a partial last block (k stays a multiple of 4)
        print(f"sweep case {case}: dtype={dtype} m={m} n={n} k={k}", flush=True)
        w, x = random_weight(dtype, n, k, seed=1000 + case), random_activations(m, k, seed=2000 + case)
        want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
        got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        check_close(got, want, f"case {case} dtype={dtype} m={m} n={n} k={k}")


def test_k_split_of_the_8_row_kernels(torch, oracle):
    """Few weight rows (tiles for at most half of the CUs) and at least two passes per tile: several
    workgroups share a tile, each takes a slice of K, the last one to finish adds the slices up.
    Every format from one row up, 2 to 8 slices, slices of unequal length, a partial last block,
    ragged n, a repeat of every call (the arrival counters must be back at zero; the sum order is
    fixed, so the repeat is bit-identical) with an unsplit call in between."""
    from gllm_amd.backend import HipBackend
    hip2 = HipBackend(0, options={"mm8_q6k_min_m": 1, "mm8_q5k_min_m": 1, "mm8_q8_0_min_m": 1, "mmf_small_min_m": 0})
    cases = [(1, 4096, 4096), (2, 1024, 4096), (1, 100, 14336), (4, 512, 8192), (8, 33, 6144), (3, 2048, 2048 + 1024),
             (5, 64, 16384), (1, 4000, 4096 + 2048), (2, 31, 4096 + 256 * 5 - 8), (8, 4096, 4096), (6, 300, 11008)]
    for dtype in ALL:
        for m, n, k in cases:
            print(f"k split dtype={dtype} m={m} n={n} k={k}", flush=True)
            w, x = random_weight(dtype, n, k, seed=m * 100 + n), random_activations(m, k, seed=k % 997)
            want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
            got = gpu_matmul(hip2, torch, w, x, dtype, m, n, k)
            check_close(got, want, f"k split dtype={dtype} m={m} n={n} k={k}")
            w2, x2 = random_weight(dtype, 8200, 256, seed=5), random_activations(1, 256, seed=6)
            gpu_matmul(hip2, torch, w2, x2, dtype, 1, 8200, 256)
            again = gpu_matmul(hip2, torch, w, x, dtype, m, n, k)
            assert np.array_equal(got.view(np.uint32), again.view(np.uint32)), f"repeat differs: dtype={dtype} m={m} n={n} k={k}"


def test_q8_0_matrix_core_shapes(hip, torch, oracle):
    """Q8_0 with three rows and more runs on the matrix cores in groups of 8 blocks (int8 up to 8
    rows, the f16 GEMM beyond): rows of whole groups, rows whose last group has 1..7 blocks (its window ends with the row), one group
    only, long rows (several passes per tile, fewer rows per pass), ragged n."""
    cases = [(3, 70, 256), (4, 33, 288), (8, 129, 480), (5, 64, 512), (7, 31, 544), (3, 257, 4096),
             (8, 100, 4128), (6, 40, 14336), (9, 65, 1056), (20, 50, 2272), (3, 1, 256 + 224),
             (40, 300, 4096), (64, 257, 480), (33, 64, 256), (17, 513, 14336 + 96), (12, 20, 272)]
    for m, n, k in cases:
        print(f"q8_0 matrix cores m={m} n={n} k={k}", flush=True)
        w, x = random_weight(Q8_0, n, k, seed=m * 1000 + n), random_activations(m, k, seed=k)
        want = oracle.quantized_matmul(w, x, Q8_0, m, n, k, acc=oracle.ACC_F64, threads=4)
        got = gpu_matmul(hip, torch, w, x, Q8_0, m, n, k)
        check_close(got, want, f"q8_0 m={m} n={n} k={k}")


@pytest.mark.parametrize("dtype", ALL)
def test_long_rows_one_and_two_activation_rows(hip, torch, oracle, dtype):
    """Long rows with one and two activation rows (the waves of a GEMV workgroup share a row, rows
    past 16384 elements take several launches; two rows past 9728 elements take the 8-row kernel,
    and so does one Q5_K or Q6_K row of 40 blocks and more over few weight rows, K split across
    workgroups): whole groups, a partial last group, ragged n, up to 65536 elements, two down
    projection shapes."""
    step = 32 if dtype == Q8_0 else 256
    for n, k in [(257, 8192), (70, 14336), (33, 11008), (5, 8448 + step), (129, 16384 + 4 * step - 8), (64, 65536),
                 (4096, 11008), (2000, 10240)]:
        for m in (1, 2):
            print(f"long rows dtype={dtype} n={n} k={k} m={m}", flush=True)
            w, x = random_weight(dtype, n, k, seed=n + m), random_activations(m, k, seed=k % 1000)
            want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
            got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
            check_close(got, want, f"dtype={dtype} n={n} k={k} m={m}")


def test_empty_shapes_are_no_ops(hip, torch):
    print("empty shapes", flush=True)
    w = torch.zeros(144 * 16, dtype=torch.uint8, device="cuda")
    x = torch.zeros(4096, dtype=torch.float32, device="cuda")
    y = torch.full((8,), 7.0, dtype=torch.float32, device="cuda")
    hip.quantized_matmul(w, x, y, Q4_K, 0, 1, 4096)  # m = 0
    hip.quantized_matmul(w, x, y, Q4_K, 1, 0, 4096)  # n = 0
    out = torch.full((8,), 7.0, dtype=torch.float32, device="cuda")
    hip.dequantize(w[:100], out, Q4_K)               # less than one block in
    hip.dequantize(w, out[:100], Q4_K)               # room for less than one block out
    torch.cuda.synchronize()
    assert torch.all(y == 7.0) and torch.all(out == 7.0)


@pytest.mark.parametrize("dtype", ALL)
def test_rows_longer_than_one_launch_covers(hip, torch, oracle, dtype):
    # K = 20480: the GEMV kernels take 16384 elements per launch and accumulate the rest
    n, k = 67, 20480
    print(f"long rows dtype={dtype}", flush=True)
    for m in (1, 2, 3):
        w, x = random_weight(dtype, n, k, seed=77 + m), random_activations(m, k, seed=78)
        want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
        got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        check_close(got, want, f"dtype={dtype} m={m} k={k}")


def test_vocabulary_sized_output(hip, torch, oracle):
    # lm_head shape: Q6_K, 151936 rows over 4096 (the largest matvec of a decode step)
    n, k = 151936, 4096
    print("lm_head 151936x4096 Q6_K", flush=True)
    w, x = random_weight(Q6_K, n, k, seed=5), random_activations(1, k, seed=6)
    want = oracle.quantized_matmul(w, x, Q6_K, 1, n, k, acc=oracle.ACC_F64, threads=16)
    got = gpu_matmul(hip, torch, w, x, Q6_K, 1, n, k)
    check_close(got, want, "lm_head")


@pytest.mark.parametrize("dtype", ALL)
def test_activations_that_are_only_4_byte_aligned(hip, torch, oracle, dtype):
    n, k, m = 45, 1024, 2
    print(f"unaligned activations dtype={dtype}", flush=True)
    w, x = random_weight(dtype, n, k, seed=31), random_activations(m, k, seed=32)
    want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64)
    wd = hip.upload_weights(w)
    buf = torch.zeros(m * k + 1, dtype=torch.float32, device="cuda")
    buf[1:] = torch.from_numpy(x.reshape(-1)).cuda()
    yd = torch.zeros(m * n + 1, dtype=torch.float32, device="cuda")
    hip.quantized_matmul(wd, buf[1:], yd[1:], dtype, m, n, k)
    torch.cuda.synchronize()
    check_close(yd[1:].cpu().numpy().reshape(m, n), want, f"unaligned dtype={dtype}")


@pytest.mark.parametrize("dtype", ALL)
def test_non_finite_activations_give_non_finite_outputs(hip, torch, oracle, dtype):
    """An Inf or NaN activation makes every output that depends on it non-finite (the exact
    non-finite value is not pinned: the oracle may say Inf where the GPU says NaN)."""
    n, k = 40, 1024
    print(f"non-finite dtype={dtype}", flush=True)
    w = random_weight(dtype, n, k, seed=41)
    for bad in (np.inf, -np.inf, np.nan):
        x = random_activations(1, k, seed=42)
        x[0, 300] = bad
        want = oracle.quantized_matmul(w, x, dtype, 1, n, k, acc=oracle.ACC_F64)
        got = gpu_matmul(hip, torch, w, x, dtype, 1, n, k)
        assert not np.isfinite(got[~np.isfinite(want)]).any()


# ------------------------------------------------------------------- errors
def test_unsupported_formats_are_errors(hip, torch):
    from gllm_amd.backend import OtherError, Unimplemented
    w = torch.zeros(18 * 4, dtype=torch.uint8, device="cuda")
    x = torch.zeros(32, dtype=torch.float32, device="cuda")
    y = torch.zeros(4, dtype=torch.float32, device="cuda")
    for dt in (0, 1, 2, 3, 6, 7, 10, 11, 15, 30, 39):  # F32, F16, Q4_0 ... Q8_K, BF16, MXFP4
        with pytest.raises(Unimplemented):
            hip.quantized_matmul(w, x, y, dt, 1, 4, 32)
        with pytest.raises(Unimplemented):
            hip.dequantize(w, y, dt)
    with pytest.raises(OtherError):  # weight buffer shorter than n rows
        hip.quantized_matmul(w, x, y, Q8_0, 1, 4, 64)
    hip.quantized_matmul(w, x, y, Q8_0, 0, 4, 32)  # m = 0: nothing to do


def test_weight_matrix_larger_than_4_gib(hip, torch, oracle):
    """A Q8_0 matrix of 4.6 GB: rows that start past byte offset 2^32 must be addressed with
    64-bit arithmetic on every kernel path (1, 2, 5 and 16 activation rows; the GEMM addresses rows
    with 32-bit offsets from the start of the matrix and must leave such a matrix to the other
    kernels).  Weights are made on the device; sampled rows on both sides of the 4 GiB line are
    checked against the oracle."""
    dtype, n, k = Q8_0, 132000, 32768
    rb = (k // 32) * 34
    assert n * rb > 2**32
    g = torch.Generator(device="cuda")
    g.manual_seed(77)
    wd = torch.randint(0, 256, (n * rb,), dtype=torch.uint8, device="cuda", generator=g)
    blocks = wd.view(-1, 34)
    d = (torch.rand(blocks.shape[0], 1, device="cuda", generator=g) * 0.049 + 0.001).to(torch.float16)
    blocks[:, 0:2] = d.view(torch.uint8)
    del d
    first_past = 2**32 // rb + 1
    rows = [0, 1, 31, 4097, first_past - 2, first_past - 1, first_past, first_past + 1, first_past + 300, n - 33, n - 2, n - 1]
    w_rows = torch.stack([wd[r * rb:(r + 1) * rb] for r in rows]).cpu().numpy()
    for m in (1, 2, 5, 16):
        print(f"4 GiB matrix m={m}", flush=True)
        x = random_activations(m, k, seed=m)
        xd = torch.from_numpy(x).cuda()
        yd = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
        hip.quantized_matmul(wd, xd, yd, dtype, m, n, k)
        torch.cuda.synchronize()
        got = yd[:, rows].cpu().numpy()
        want = oracle.quantized_matmul(w_rows, x, dtype, m, len(rows), k, acc=oracle.ACC_F64, threads=4)
        check_close(got, want, f"4 GiB matrix m={m}")
        assert not bool(torch.isnan(yd).any())


@pytest.mark.parametrize("dtype", ALL)
def test_k_split_with_a_shorter_last_slice(hip, torch, oracle, dtype):
    """K slices of two passes and a last slice of one (an odd number of 8-block passes per tile),
    several tiles per workgroup: the variants that keep a wave's activation operands in registers
    are compiled for one number of passes per tile and must not run such a launch (they gave wrong
    sums for every tile after a workgroup's first)."""
    for m, n, k in [(4, 4096, 13824), (4, 4096, 14336 - 256), (3, 2048, 9728), (4, 1024, 5632), (4, 3000, 13824), (2, 4096, 13824)]:
        print(f"uneven k slices dtype={dtype} m={m} n={n} k={k}", flush=True)
        w, x = random_weight(dtype, n, k, seed=276), random_activations(m, k, seed=277)
        want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
        got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        check_close(got, want, f"uneven k slices dtype={dtype} m={m} n={n} k={k}")


def test_few_weight_rows_long_rows_sweep(hip, torch, oracle):
    """A hundred seeded shapes where the K split of the 8-row kernels and the long-row dispatch
    decide: up to 5000 weight rows (among them 2048 and 4096 exactly: whole rounds of workgroups),
    rows of 8 to 71 blocks with and without a partial last one, 1 to 33 activation rows; every
    call twice, the repeat bit-identical (sums meet in a fixed order, counters return to zero)."""
    rng = np.random.default_rng(23)
    for case in range(100):
        dtype = ALL[case % len(ALL)]
        m = int(rng.choice([1, 1, 1, 2, 2, 3, 4, 5, 7, 8, 9, 16, 33]))
        n = int(rng.choice([rng.integers(1, 64), rng.integers(64, 1024), rng.integers(1024, 5000), 4096, 2048]))
        k = int(rng.integers(8, 72)) * 256
        if rng.random() < 0.3:
            k -= int(rng.integers(1, 8)) * (4 if dtype != Q8_0 else 32)
        print(f"few rows sweep case {case}: dtype={dtype} m={m} n={n} k={k}", flush=True)
        w, x = random_weight(dtype, n, k, seed=case), random_activations(m, k, seed=case + 1)
        want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=4)
        got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        check_close(got, want, f"few rows sweep case {case} dtype={dtype} m={m} n={n} k={k}")
        again = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        assert np.array_equal(got.view(np.uint32), again.view(np.uint32)), f"repeat differs: case {case}"
