"""GPU parity of the quantized embedding lookup (gllmq_quant_gather through the C ABI) against
the CPU oracle: bit-exact, as for the dequantized weights."""
import numpy as np
import pytest

from gllm_amd.synth import random_weight

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


def gpu_gather(hip, torch, table, dtype, vocab, hidden, ids, scale=None, offset=0):
    """Runs the lookup with 0xFF bytes behind the table, a marker behind the output and the
    output `offset` floats into its allocation (1: rows are not 16-byte aligned)."""
    flat = torch.from_numpy(np.asarray(table).view(np.uint8).reshape(-1))
    tbuf = torch.full((flat.numel() + GUARD,), 0xFF, dtype=torch.uint8, device="cuda")
    tbuf[:flat.numel()] = flat.cuda()
    idd = torch.from_numpy(np.ascontiguousarray(ids, np.uint32).view(np.int32)).cuda()
    n = len(ids) * hidden
    obuf = torch.full((offset + n + GUARD,), float("nan"), dtype=torch.float32, device="cuda")
    obuf[offset + n:] = 7.0
    hip.quant_gather(tbuf[:flat.numel()], dtype, vocab, hidden, idd, obuf[offset:offset + n], scale=scale)
    torch.cuda.synchronize()
    assert bool(torch.all(obuf[offset + n:] == 7.0)), "write past the end of the output"
    assert offset == 0 or bool(torch.isnan(obuf[:offset]).all()), "write ahead of the output"
    return obuf[offset:offset + n].cpu().numpy().reshape(len(ids), hidden)


@pytest.mark.parametrize("dtype", ALL)
def test_gather_bit_exact(hip, torch, oracle, dtype):
    rng = np.random.default_rng(dtype)
    for vocab, hidden, count in [(1000, 4096, 1), (333, 2048, 7), (64, 1024, 300), (50, 256, 33)]:
        print(f"gather dtype={dtype} vocab={vocab} hidden={hidden} count={count}", flush=True)
        table = random_weight(dtype, vocab, hidden, seed=vocab + dtype)
        ids = rng.integers(0, vocab, count).astype(np.uint32)
        ids[0], ids[-1] = vocab - 1, 0
        want = oracle.quant_gather(table, dtype, vocab, hidden, ids)
        for offset in (0, 1):
            got = gpu_gather(hip, torch, table, dtype, vocab, hidden, ids, offset=offset)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (dtype, vocab, hidden, count, offset)


@pytest.mark.parametrize("dtype", ALL)
def test_gather_with_embedding_scale(hip, torch, oracle, dtype):
    vocab, hidden = 128, 2560
    print(f"gather scale dtype={dtype}", flush=True)
    table = random_weight(dtype, vocab, hidden, seed=11)
    ids = np.array([5, 127, 0, 5, 64], np.uint32)
    scale = float(np.sqrt(np.float32(hidden)))  # the reference's embedding scale, sqrt(hidden)
    want = oracle.quant_gather(table, dtype, vocab, hidden, ids, scale=scale)
    got = gpu_gather(hip, torch, table, dtype, vocab, hidden, ids, scale=scale)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("dtype,hidden", [(Q4_K, 300), (Q5_K, 516), (Q6_K, 260), (Q8_0, 300), (Q8_0, 36)])
def test_gather_padded_rows(hip, torch, oracle, dtype, hidden):
    """hidden not a multiple of the block: table rows are padded to whole blocks, outputs are not."""
    vocab = 23
    print(f"gather padded dtype={dtype} hidden={hidden}", flush=True)
    table = random_weight(dtype, vocab, hidden, seed=hidden)
    ids = np.arange(vocab - 1, -1, -1).astype(np.uint32)
    want = oracle.quant_gather(table, dtype, vocab, hidden, ids)
    got = gpu_gather(hip, torch, table, dtype, vocab, hidden, ids)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_gather_more_rows_than_one_grid_covers(hip, torch, oracle):
    # 70000 looked-up rows: the grid's second dimension ends at 65535 and walks the rest
    vocab, hidden, count = 500, 32, 70000
    print("gather 70000 rows", flush=True)
    table = random_weight(Q8_0, vocab, hidden, seed=9)
    ids = np.random.default_rng(1).integers(0, vocab, count).astype(np.uint32)
    want = oracle.quant_gather(table, Q8_0, vocab, hidden, ids)
    got = gpu_gather(hip, torch, table, Q8_0, vocab, hidden, ids)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_gather_id_outside_the_table_gives_nan_row(hip, torch, oracle):
    vocab, hidden = 10, 512
    print("gather bad id", flush=True)
    table = random_weight(Q6_K, vocab, hidden, seed=2)
    ids = np.array([1, 10, 2, 0xFFFFFFFF], np.uint32)
    got = gpu_gather(hip, torch, table, Q6_K, vocab, hidden, ids)
    want = oracle.quant_gather(table, Q6_K, vocab, hidden, ids[[0, 2]])
    assert np.array_equal(got[[0, 2]].view(np.uint32), want.view(np.uint32))
    assert np.isnan(got[1]).all() and np.isnan(got[3]).all()


def test_gather_argument_errors(hip, torch):
    from gllm_amd.backend import BackendError, Unimplemented
    print("gather errors", flush=True)
    table = torch.zeros(144 * 8, dtype=torch.uint8, device="cuda")
    ids = torch.zeros(2, dtype=torch.int32, device="cuda")
    out = torch.full((2 * 256,), 7.0, dtype=torch.float32, device="cuda")
    with pytest.raises(Unimplemented):
        hip.quant_gather(table, 2, 8, 256, ids, out)          # Q4_0
    with pytest.raises(BackendError):
        hip.quant_gather(table, Q4_K, 9, 256, ids, out)       # table shorter than 9 rows
    with pytest.raises(BackendError):
        hip.quant_gather(table, Q8_0, 8, 30, ids, out)        # hidden not a multiple of 4
    hip.quant_gather(table, Q4_K, 8, 256, ids[:0], out)       # nothing to look up
    torch.cuda.synchronize()
    assert bool(torch.all(out == 7.0))
