"""GPU parity of the streamed form of the int8 matrix-core kernels (loader waves bring the weights
into an LDS ring, arithmetic waves take them out; Q4_K, Q5_K and Q6_K, up to 8 activation rows, at
least 8 weight rows per CU) against the oracle, through the C ABI.  Same bar as the other matmul
tests: rel-L2 <= 1e-4 and |err| <= 1e-3 * max|y| against float64 accumulation; against the
fetch-and-compute kernels (option "mm8s" = 0) the results are equal bit for bit whenever the two
forms add a row's blocks in the same order, which they do (wave order, block order)."""
import numpy as np
import pytest

from gllm_amd.synth import random_activations, random_weight
from tests.test_gpu_parity import check_close, gpu_matmul

pytestmark = pytest.mark.gpu

Q4_K, Q5_K, Q6_K = 12, 13, 14


@pytest.fixture(scope="module")
def hip():
    # "mm8s_all": the streamed form wherever the shape fits, not only where it was timed fastest
    from gllm_amd.backend import HipBackend
    # ("mm8s_split" = 0: whole rows of K per workgroup also where slices of K would be shared; that
    # form has its own test below)
    return HipBackend(0, options={"mm8s_all": 1, "mm8s_split": 0})


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def cus(torch):
    return torch.cuda.get_device_properties(0).multi_processor_count


@pytest.mark.parametrize("dtype", [Q4_K, Q5_K, Q6_K])
def test_streamed_shapes_against_the_oracle(hip, torch, oracle, dtype):
    """Rows per workgroup that are and are not whole tiles, a ragged last workgroup, a partial last
    block of K, one to eight activation rows, rows whose operands stay in registers (K <= 4096) and
    rows that read them from LDS, and a ring that is reused many times (K = 14336)."""
    c = cus(torch)
    # (rows, weight rows, k, streamed?): eight rows of 4096 elements leave no room for the ring
    # beside their digit planes (99 KB of the 160 KB of LDS) and stay on the other form
    cases = [(1, 32 * c, 4096, True), (1, 56 * c, 4096, True), (2, 56 * c + 17, 4096, True), (1, 33 * c, 2048, True),
             (3, 40 * c, 1024, True), (4, 56 * c, 4096 - 8, True), (5, 32 * c + 5, 1536, True), (8, 35 * c, 4096, False),
             (1, 32 * c, 14336, True), (2, 33 * c + 1, 8192 + 256 * 3 - 64, True), (6, 32 * c, 2048, True),
             (1, 64 * c + 3, 256, True), (7, 96 * c, 512, True), (8, 32 * c, 1024, True)]
    for m, n, k, streamed in cases:
        print(f"streamed dtype={dtype} m={m} n={n} k={k}", flush=True)
        w, x = random_weight(dtype, n, k, seed=m + n), random_activations(m, k, seed=k + m)
        want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=16)
        got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        check_close(got, want, f"streamed dtype={dtype} m={m} n={n} k={k}")
        # (a Q6_K item is half as large again as a Q4_K one, so fewer of the shapes with many
        # activation rows leave room for its ring, and three and more rows of long Q6_K rows never
        # take this form: only the shapes of up to 2 rows are checked there)
        if dtype != Q6_K or (m <= 2 and k <= 8192):
            assert hip.last_kernel_name().startswith("gq_mm8s_") == streamed, hip.last_kernel_name()


def test_streamed_equals_the_fetch_and_compute_form_bitwise(hip, torch):
    from gllm_amd.backend import HipBackend
    plain = HipBackend(0, options={"mm8s": 0, "mm8_q6k_min_m": 1, "mm8_ksplit": 0})  # no K split there: the same order of sums
    c = cus(torch)
    for dtype, m, n, k in ((Q4_K, 1, 56 * c, 4096), (Q4_K, 4, 40 * c + 9, 2048), (Q5_K, 2, 56 * c, 4096), (Q4_K, 8, 32 * c, 1024),
                           (Q6_K, 1, 56 * c, 4096), (Q6_K, 2, 16 * c, 14336), (Q6_K, 1, 8 * c + 3, 512)):
        print(f"streamed vs plain dtype={dtype} m={m} n={n} k={k}", flush=True)
        w, x = random_weight(dtype, n, k, seed=3), random_activations(m, k, seed=4)
        a = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        assert hip.last_kernel_name().startswith("gq_mm8s_")
        b = gpu_matmul(plain, torch, w, x, dtype, m, n, k)
        assert not plain.last_kernel_name().startswith("gq_mm8s_")
        if plain.last_kernel_name().startswith("gq_mm8_"):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        else:  # one or two rows of Q6_K take the integer-dot GEMV there: another order of sums
            check_close(a, b, f"streamed vs GEMV dtype={dtype} m={m}")


@pytest.mark.parametrize("dtype", [Q4_K, Q5_K, Q6_K])
def test_pairs_of_blocks_over_low_tiles(hip, torch, oracle, dtype):
    """One activation row over at most 16 weight rows per workgroup: an item is a pair of blocks of
    the tile (blocks i and i + 8 of every 16).  Rows of whole sixteens of blocks and rows that end
    in pairs without a second block (9, 10, 12, 15, 20, 24, 33 and 56 blocks), a partial last
    block, a ragged last workgroup, operands in registers (up to 32 blocks) and in LDS, a reused
    ring, and tiles of 16 down to 4 rows."""
    c = cus(torch)
    cases = [(16 * c, 4096), (16 * c, 14336), (9 * c + 5, 2304), (13 * c - 2, 2560), (8 * c, 8192), (16 * c - 7, 4096 - 8),
             (5 * c + 1, 3072), (12 * c, 8192 + 256), (4 * c + 3, 6144), (16 * c, 5120), (7 * c, 3840 - 16)]
    for n, k in cases:
        print(f"pairs dtype={dtype} n={n} k={k}", flush=True)
        w, x = random_weight(dtype, n, k, seed=n % 97), random_activations(1, k, seed=k % 89)
        want = oracle.quantized_matmul(w, x, dtype, 1, n, k, acc=oracle.ACC_F64, threads=16)
        got = gpu_matmul(hip, torch, w, x, dtype, 1, n, k)
        name = hip.last_kernel_name()
        assert name.startswith("gq_mm8s_") and name.endswith("_f"), name
        check_close(got, want, f"pairs dtype={dtype} n={n} k={k}")


def test_pairs_of_blocks_equal_single_blocks_within_the_bar(hip, torch):
    """The same launches block by block (option "mm8s_fold" = 0): another order of sums, the same
    bar; and twice in a row, the counters in LDS starting from zero."""
    from gllm_amd.backend import HipBackend
    single = HipBackend(0, options={"mm8s_all": 1, "mm8s_fold": 0})
    c = cus(torch)
    for dtype, n, k in ((Q4_K, 16 * c, 14336), (Q5_K, 11 * c, 4096), (Q6_K, 16 * c, 11008 + 256 - 11008 % 256)):
        print(f"pairs vs single dtype={dtype} n={n} k={k}", flush=True)
        w, x = random_weight(dtype, n, k, seed=21), random_activations(1, k, seed=22)
        a = gpu_matmul(hip, torch, w, x, dtype, 1, n, k)
        assert hip.last_kernel_name().endswith("_f"), hip.last_kernel_name()
        b = gpu_matmul(single, torch, w, x, dtype, 1, n, k)
        assert single.last_kernel_name().startswith("gq_mm8s_") and not single.last_kernel_name().endswith("_f")
        check_close(a, b, f"pairs vs single dtype={dtype}")
        again = gpu_matmul(hip, torch, w, x, dtype, 1, n, k)
        assert np.array_equal(a.view(np.uint32), again.view(np.uint32))


@pytest.mark.parametrize("dtype", [Q4_K, Q5_K, Q6_K])
def test_slices_of_k_shared_among_workgroups(torch, oracle, dtype):
    """Two to four rows of long activations over few weight rows (a down projection of a small
    batch): the workgroups of a 32-row tile take a slice of K each and the one that finishes last
    adds the slices up.  Two to four slices, a last slice that is shorter, a ragged last tile, a
    partial last block; twice in a row (the arrival counters are left at zero)."""
    from gllm_amd.backend import HipBackend
    hip = HipBackend(0, options={"mm8s_all": 1})  # (by default three and four rows of Q6_K stay on the other form)
    c = cus(torch)
    cases = [(2, 16 * c, 14336), (4, 16 * c, 11008 + 256 - 11008 % 256), (3, 16 * c - 9, 11008 + 256 - 11008 % 256), (4, 8 * c + 5, 8192 + 512 - 8),
             (2, 4 * c, 14336), (3, 10 * c, 9216)]
    for m, n, k in cases:
        print(f"k split dtype={dtype} m={m} n={n} k={k}", flush=True)
        w, x = random_weight(dtype, n, k, seed=n % 89 + m), random_activations(m, k, seed=k % 83 + m)
        want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=16)
        got = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        name = hip.last_kernel_name()
        assert name.startswith("gq_mm8s_") and name.endswith("_s"), name
        check_close(got, want, f"k split dtype={dtype} m={m} n={n} k={k}")
        again = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        assert np.array_equal(got.view(np.uint32), again.view(np.uint32))


def test_q8_0_in_groups_of_eight_blocks(torch, oracle):
    """Q8_0 rows of whole 256-element groups take the streamed form too (an item is a group of 8
    blocks of a tile, 272 bytes per row): one to eight rows, registers and LDS operands, pairs of
    groups over low tiles, slices of K; rows with a partial group stay on the other kernels."""
    from gllm_amd.backend import HipBackend
    Q8_0 = 8
    hip = HipBackend(0, options={"mm8s_all": 1})
    c = cus(torch)
    cases = [(1, 56 * c, 4096, ""), (1, 16 * c, 14336, "_f"), (2, 33 * c + 5, 2048, ""), (1, 9 * c + 3, 2304, "_f"),
             (3, 40 * c, 1024, ""), (4, 16 * c - 7, 8192 + 256, "_s"), (1, 64 * c + 3, 256, ""), (8, 32 * c, 1024, ""),
             (1, 12 * c, 4096, "_f"), (2, 56 * c, 4096, ""), (5, 32 * c + 5, 1536, ""), (1, 32 * c, 4096 + 32, None),
             (2, 40 * c, 1000, None)]
    for m, n, k, suffix in cases:
        print(f"streamed Q8_0 m={m} n={n} k={k}", flush=True)
        w, x = random_weight(Q8_0, n, k, seed=m + n), random_activations(m, k, seed=k + m)
        want = oracle.quantized_matmul(w, x, Q8_0, m, n, k, acc=oracle.ACC_F64, threads=16)
        got = gpu_matmul(hip, torch, w, x, Q8_0, m, n, k)
        name = hip.last_kernel_name()
        if suffix is None:
            assert not name.startswith("gq_mm8s_"), name
        else:
            assert name.startswith("gq_mm8s_q8_0_") and (name.endswith(suffix) if suffix else name[-2:] not in ("_f", "_s")), name
        check_close(got, want, f"streamed Q8_0 m={m} n={n} k={k}")


def test_streamed_large_vocabulary_and_repeats(hip, torch, oracle):
    """A Llama-3 vocabulary of Q4_K rows (501 rows per workgroup, 16 tiles, the ring reused eight
    times), twice in a row with different inputs: the counters in LDS start from zero every launch."""
    n, k = 128256, 4096
    w = random_weight(Q4_K, n, k, seed=9)
    for seed in (1, 2):
        print(f"streamed vocabulary seed={seed}", flush=True)
        x = random_activations(1, k, seed=seed)
        want = oracle.quantized_matmul(w, x, Q4_K, 1, n, k, acc=oracle.ACC_F64, threads=16)
        got = gpu_matmul(hip, torch, w, x, Q4_K, 1, n, k)
        check_close(got, want, f"vocabulary seed={seed}")
    assert hip.last_kernel_name().startswith("gq_mm8s_")


def test_default_choice_of_form(torch):
    """Without "mm8s_all" the streamed form runs where it was timed fastest: single rows of Q4_K
    and Q5_K from 4 weight rows per CU (short rows over exactly 4 excepted), Q6_K for one row of
    20 blocks and more over at most 16 weight rows per CU, of 40 and more over any number, or two
    short ones; two to four rows of 32 blocks and more over 32-row tiles for at most half of the
    CUs (slices of K shared among workgroups); the results stay those of the oracle's bar either
    way (checked against the other form here)."""
    from gllm_amd.backend import HipBackend
    default, plain = HipBackend(0), HipBackend(0, options={"mm8s": 0})
    c = cus(torch)
    for dtype, m, n, k, streamed in ((Q4_K, 1, 56 * c, 4096, True), (Q4_K, 2, 16 * c, 14336, True), (Q6_K, 1, 16 * c, 14336, True),
                                     (Q4_K, 1, 16 * c, 8192, True), (Q4_K, 1, 12 * c, 8192, True), (Q5_K, 1, 8 * c, 8192, True),
                                     (Q4_K, 1, 4 * c, 4096, False), (Q4_K, 1, 4 * c, 8192, True), (Q5_K, 1, 8 * c, 4096, True),
                                     (Q6_K, 1, 16 * c, 4096, False), (Q6_K, 1, 16 * c, 5120, True), (Q6_K, 1, 24 * c, 5120, False),
                                     (Q6_K, 1, 56 * c, 4096, False), (Q6_K, 2, 56 * c, 4096, True), (Q6_K, 2, 16 * c, 14336, True),
                                     (Q4_K, 2, 40 * c, 14336, False), (Q6_K, 4, 16 * c, 14336, False), (Q5_K, 4, 16 * c, 14336, True),
                                     (Q4_K, 5, 16 * c, 14336, False)):
        print(f"default form dtype={dtype} m={m} n={n} k={k}", flush=True)
        w, x = random_weight(dtype, n, k, seed=5), random_activations(m, k, seed=6)
        a = gpu_matmul(default, torch, w, x, dtype, m, n, k)
        assert default.last_kernel_name().startswith("gq_mm8s_") == streamed, default.last_kernel_name()
        check_close(a, gpu_matmul(plain, torch, w, x, dtype, m, n, k), f"default form dtype={dtype} m={m} n={n} k={k}")


@pytest.mark.parametrize("dtype", [Q4_K, Q5_K, Q6_K])
def test_more_open_requests_per_loader_change_no_bit(hip, torch, dtype):
    """A loader wave keeps one or two items open by default (two for pairs of Q4_K / Q5_K blocks of
    a long row).  With up to four, on long rows whose ring is short beside them, a loader stands
    before taken slots most of the time and counts its open requests in there: every item must
    still be seen by its arithmetic wave, complete, whatever the depth."""
    from gllm_amd.backend import HipBackend
    c = cus(torch)
    for m, n, k in ((1, 16 * c, 14336), (1, 16 * c + 5, 8192 + 256), (2, 32 * c, 8192), (1, 56 * c, 4096), (4, 40 * c, 2048)):
        if dtype == Q6_K and m > 2:
            continue
        w, x = random_weight(dtype, n, k, seed=n + k), random_activations(m, k, seed=m)
        base = gpu_matmul(hip, torch, w, x, dtype, m, n, k)
        name = hip.last_kernel_name()
        assert name.startswith("gq_mm8s_"), name
        for depth in (1, 2, 3, 4):
            print(f"open requests dtype={dtype} m={m} n={n} k={k} depth={depth}", flush=True)
            deep = HipBackend(0, options={"mm8s_all": 1, "mm8s_split": 0, "mm8s_depth": depth})
            got = gpu_matmul(deep, torch, w, x, dtype, m, n, k)
            assert deep.last_kernel_name() == name
            assert np.array_equal(got.view(np.uint32), base.view(np.uint32)), (dtype, m, n, k, depth)
