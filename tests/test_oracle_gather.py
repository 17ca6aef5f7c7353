"""Oracle pins for the quantized embedding lookup (Op::QuantGather,
src/arch/auto_graph_fragments/build_graph.inc.rs:203-211): the C restatement against closed
forms that fix the row stride and the id -> row mapping, against a row gather of the pinned
block decoders, and against the numpy twin."""
import numpy as np
import pytest

from gllm_amd.synth import random_weight
from oracle import npref

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
ALL = [Q8_0, Q4_K, Q5_K, Q6_K]


def test_row_identity_table(oracle):
    """Q8_0 table whose row r decodes to the constant r (d = 1, every quant r): the lookup must
    return the ids themselves, whatever the decoder does inside a block."""
    vocab, hidden = 100, 96
    table = np.zeros((vocab, hidden // 32, 34), np.uint8)
    table[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    table[:, :, 2:] = np.arange(vocab, dtype=np.uint8)[:, None, None]
    ids = np.array([0, 99, 5, 5, 42, 1], np.uint32)
    out = oracle.quant_gather(table, Q8_0, vocab, hidden, ids)
    assert out.shape == (6, hidden)
    assert np.array_equal(out, np.repeat(ids.astype(np.float32)[:, None], hidden, axis=1))


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("hidden", [256, 1024, 300])
def test_gather_is_rows_of_dequantize(oracle, dtype, hidden):
    """hidden = 300 is not a multiple of any block size (256 or 32): rows are padded to whole
    blocks (src/compat/weight_helpers.rs:42-71) and the padding is dropped."""
    vocab = 37
    table = random_weight(dtype, vocab, hidden, seed=dtype * 7 + hidden)
    rng = np.random.default_rng(hidden)
    ids = rng.integers(0, vocab, 50).astype(np.uint32)
    bs = oracle.block_size(dtype)
    padded = -(-hidden // bs) * bs
    full = oracle.dequantize(table, dtype).reshape(vocab, padded)
    want = full[ids, :hidden]
    got = oracle.quant_gather(table, dtype, vocab, hidden, ids)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    twin = npref.dequantize(table, dtype).reshape(vocab, padded)[ids, :hidden]
    assert np.array_equal(got.view(np.uint32), twin.astype(np.float32).view(np.uint32))


@pytest.mark.parametrize("dtype", ALL)
def test_scaled_gather_is_one_f32_multiply(oracle, dtype):
    vocab, hidden = 20, 512
    table = random_weight(dtype, vocab, hidden, seed=3)
    ids = np.array([3, 19, 0], np.uint32)
    scale = float(np.sqrt(np.float32(hidden)))
    plain = oracle.quant_gather(table, dtype, vocab, hidden, ids)
    got = oracle.quant_gather(table, dtype, vocab, hidden, ids, scale=scale)
    assert np.array_equal(got.view(np.uint32), (plain * np.float32(scale)).view(np.uint32))
    # a scale of exactly one changes no bit
    one = oracle.quant_gather(table, dtype, vocab, hidden, ids, scale=1.0)
    assert np.array_equal(one.view(np.uint32), plain.view(np.uint32))


def test_gather_errors(oracle):
    table = random_weight(Q4_K, 4, 256, seed=1)
    with pytest.raises(ValueError):
        oracle.quant_gather(table, Q4_K, 4, 256, np.array([4], np.uint32))  # id == vocab
    with pytest.raises(NotImplementedError):
        oracle.quant_gather(table, 2, 4, 256, np.array([0], np.uint32))     # Q4_0 is not covered
    assert oracle.quant_gather(table, Q4_K, 4, 256, np.zeros(0, np.uint32)).shape == (0, 256)
