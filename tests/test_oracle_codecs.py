"""Pins for the CPU oracle's codecs (no GPU).

The reference holds no test that feeds K-quant bytes through dequantize/quantized_matmul, so
the oracle is pinned by: the reference's format constants, encoders written from the
quantizer side, closed forms and special cases, bit walks over every packed plane, the
known answers its bug log documents, an exhaustive f16 table, and bitwise agreement of two
structurally different restatements (C loop form, numpy element form).
"""
import numpy as np
import pytest

from oracle import npref
from tests.packing import (f16_bytes, pack_q4_k, pack_q5_k, pack_q6_k, pack_q8_0,
                           pack_scales_k4)

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
ALL = [Q8_0, Q4_K, Q5_K, Q6_K]


# ---------------------------------------------------------------- constants
def test_block_constants_match_reference_unit_tests(oracle):
    # src/loader/gguf/types.rs:594,601,627,629,998-999,1832-1833
    assert [oracle.block_size(t) for t in ALL] == [32, 256, 256, 256]
    assert [oracle.block_bytes(t) for t in ALL] == [34, 144, 176, 210]
    assert oracle.block_size(2) == 0 and oracle.block_bytes(15) == 0


def test_row_bytes_matches_tensor_nbytes_vectors(oracle):
    # src/loader/gguf/types.rs:1548,1734,1941-1942,1947-1948,1971-1972
    assert oracle.row_bytes(Q8_0, 1) == 34
    assert oracle.row_bytes(Q8_0, 33) == 68
    assert oracle.row_bytes(Q4_K, 256) * 4 == 576
    assert oracle.row_bytes(Q5_K, 256) == 176 and oracle.row_bytes(Q5_K, 512) == 352
    assert oracle.row_bytes(Q6_K, 256) == 210 and oracle.row_bytes(Q6_K, 256) * 4 == 840
    for t in ALL:
        for k in (1, 31, 32, 255, 256, 257, 4096, 14336):
            assert oracle.row_bytes(t, k) == npref.row_bytes(t, k)


# ------------------------------------------------------------ scalar helpers
def test_f16_to_f32_exhaustive(oracle):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32).view(np.uint32)
    got = np.array([oracle.f16_to_f32(int(v)) for v in h], np.float32).view(np.uint32)
    nan = np.isnan(h.view(np.float16))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(got.view(np.float32)[nan]))


def test_bf16_rounding_known_answers_and_torch(oracle):
    import torch
    # src/compat/weight_helpers.rs:1202-1215
    assert oracle.f32_to_bf16(1.0) == 0x3F80
    assert oracle.f32_to_bf16(-1.0) == 0xBF80
    rng = np.random.default_rng(1)
    v = np.concatenate([rng.standard_normal(2000).astype(np.float32),
                        np.array([0.0, -0.0, 1.00390625, 1.01171875, 3.3895314e38, 1e-40], np.float32)])
    want = torch.from_numpy(v).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([oracle.f32_to_bf16(float(x)) for x in v], np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(npref.bf16_rne(v).view(np.uint32) >> 16, want.astype(np.uint32))


def test_element_type_conversions_against_torch_and_known_answers():
    """The 16-bit element types at the boundary: widening is exact, narrowing is nearest-even,
    checked against torch's conversions (an independent implementation), the reference's known
    answers and hand-built ties."""
    import torch
    rng = np.random.default_rng(3)
    v = np.concatenate([rng.standard_normal(4000).astype(np.float32) * np.float32(100.0),
                        np.array([0.0, -0.0, 1.0, -1.0, 65504.0, 65519.9, 65520.0, 1e-8, 6e-8, 2.98e-8, 2.9802325e-8,
                                  1.00048828125, 1.00146484375, 1.00390625, 1.01171875, 3.3895314e38, 3.4e38, 1e-40,
                                  np.inf, -np.inf], np.float32)])
    t = torch.from_numpy(v)
    for elem, tt in ((npref.ELEM_F16, torch.float16), (npref.ELEM_BF16, torch.bfloat16)):
        bits = npref.f32_to_elem_bits(v, elem)
        assert np.array_equal(bits, t.to(tt).view(torch.int16).numpy().view(np.uint16)), elem
        back = npref.elem_bits_to_f32(bits, elem)
        assert np.array_equal(back.view(np.uint32), t.to(tt).to(torch.float32).numpy().view(np.uint32)), elem
    bf = npref.f32_to_elem_bits(np.array([1.0, -1.0, 1.00390625, 1.01171875], np.float32), npref.ELEM_BF16)
    assert bf.tolist() == [0x3F80, 0xBF80, 0x3F80, 0x3F82]  # the two ties go to the even neighbour
    hf = npref.f32_to_elem_bits(np.array([1.0, 1.00048828125, 1.00146484375, 65520.0, 2.9802322e-8], np.float32), npref.ELEM_F16)
    assert hf.tolist() == [0x3C00, 0x3C00, 0x3C02, 0x7C00, 0x0000]
    assert np.all(np.isnan(npref.elem_bits_to_f32(npref.f32_to_elem_bits(np.array([np.nan], np.float32), npref.ELEM_BF16),
                                                   npref.ELEM_BF16)))


def test_scale_min_k4_inverts_the_quantizer_packing(oracle):
    rng = np.random.default_rng(7)
    for _ in range(200):
        sc, mn = rng.integers(0, 64, 8), rng.integers(0, 64, 8)
        q = pack_scales_k4(sc, mn)
        got = [oracle.scale_min_k4(j, q) for j in range(8)]
        assert [g[0] for g in got] == list(sc)
        assert [g[1] for g in got] == list(mn)
        s2, m2 = npref.scale_min_k4(q[None, :])
        assert list(s2[0]) == list(sc) and list(m2[0]) == list(mn)


def test_scale_min_k4_single_field_walk(oracle):
    # one six-bit field at a time set to all ones: exactly that field decodes to 63
    for which in range(16):
        sc, mn = np.zeros(8, int), np.zeros(8, int)
        (sc if which < 8 else mn)[which % 8] = 63
        q = pack_scales_k4(sc, mn)
        for j in range(8):
            assert oracle.scale_min_k4(j, q) == (sc[j], mn[j])


# ------------------------------------------------------------------- Q4_K
def test_q4k_zero_quants_give_minus_dmin_m(oracle):
    mn = np.arange(8) * 7 + 3
    b = pack_q4_k(0.5, 0.25, np.full(8, 9), mn, np.zeros(256, int))
    y = oracle.dequantize(b, Q4_K)
    assert np.array_equal(y, np.repeat(-(0.25 * mn).astype(np.float32), 32))


def test_q4k_unit_scale_reduces_to_d_times_q(oracle):
    rng = np.random.default_rng(3)
    q = rng.integers(0, 16, 256)
    b = pack_q4_k(0.125, 0.75, np.ones(8, int), np.zeros(8, int), q)
    assert np.array_equal(oracle.dequantize(b, Q4_K), (0.125 * q).astype(np.float32))


def test_q4k_nibble_placement_is_split_per_64(oracle):
    # a single nibble set: low nibble of qs[32g+l] is element 64g+l, high nibble 64g+32+l
    for byte in (0, 5, 31, 32, 77, 127):
        for hi in (0, 1):
            blk = np.zeros(144, np.uint8)
            blk[0:2], blk[2:4] = f16_bytes(1.0), f16_bytes(0.0)
            blk[4:16] = pack_scales_k4(np.ones(8, int), np.zeros(8, int))
            blk[16 + byte] = 0x0F << (4 * hi)
            y = oracle.dequantize(blk, Q4_K)
            want = np.zeros(256, np.float32)
            want[64 * (byte // 32) + 32 * hi + byte % 32] = 15.0
            assert np.array_equal(y, want)


def test_q4k_per_subblock_scales_and_subtracted_min(oracle):
    sc = np.array([1, 2, 3, 4, 33, 47, 58, 63])
    mn = np.array([63, 50, 40, 30, 20, 10, 5, 0])
    q = (np.arange(256) * 5) % 16
    b = pack_q4_k(0.01, 0.02, sc, mn, q)
    d, dm = np.float32(np.float16(0.01)), np.float32(np.float16(0.02))
    want = (d * np.repeat(sc, 32).astype(np.float32)) * q.astype(np.float32) \
        - dm * np.repeat(mn, 32).astype(np.float32)
    assert np.array_equal(oracle.dequantize(b, Q4_K), want.astype(np.float32))


# ------------------------------------------------------------------- Q5_K
def test_q5k_high_bit_plane_is_transposed(oracle):
    # bit `sub` of qh[l] is the fifth bit of element 32*sub + l
    for l in (0, 1, 17, 31):
        for sub in range(8):
            blk = np.zeros(176, np.uint8)
            blk[0:2], blk[2:4] = f16_bytes(1.0), f16_bytes(0.0)
            blk[4:16] = pack_scales_k4(np.ones(8, int), np.zeros(8, int))
            blk[16 + l] = 1 << sub
            want = np.zeros(256, np.float32)
            want[32 * sub + l] = 16.0
            assert np.array_equal(oracle.dequantize(blk, Q5_K), want)


def test_q5k_round_trip_through_quantizer_packing(oracle):
    rng = np.random.default_rng(11)
    for _ in range(20):
        sc, mn, q = rng.integers(0, 64, 8), rng.integers(0, 64, 8), rng.integers(0, 32, 256)
        b = pack_q5_k(0.03, 0.007, sc, mn, q)
        d, dm = np.float32(np.float16(0.03)), np.float32(np.float16(0.007))
        want = (d * np.repeat(sc, 32).astype(np.float32)) * q.astype(np.float32) \
            - dm * np.repeat(mn, 32).astype(np.float32)
        assert np.array_equal(oracle.dequantize(b, Q5_K), want.astype(np.float32))


def test_q5k_zero_quants(oracle):
    mn = np.array([1, 2, 3, 4, 60, 61, 62, 63])
    b = pack_q5_k(1.0, 2.0, np.full(8, 63), mn, np.zeros(256, int))
    assert np.array_equal(oracle.dequantize(b, Q5_K), np.repeat(-2.0 * mn, 32).astype(np.float32))


# ------------------------------------------------------------------- Q6_K
def test_q6k_documented_known_answer(oracle):
    # BUG-KNOWLEDGE.md:4046: q1=1,q2=2,q3=3,q4=4 (one element per quarter), d=1, scales 1,
    # unit activations -> row 0 sums to 10; an all-"zero" row (every q = 0) sums to 0.
    q = np.zeros(256, int)
    q[[0, 32, 64, 96]] = [1, 2, 3, 4]
    row0 = pack_q6_k(1.0, np.ones(16, int), q)
    row1 = pack_q6_k(1.0, np.ones(16, int), np.zeros(256, int))
    w = np.concatenate([row0, row1])
    y = oracle.quantized_matmul(w, np.ones((1, 256), np.float32), Q6_K, 1, 2, 256, acc=oracle.ACC_F32)
    assert y.tolist() == [[10.0, 0.0]]
    deq = oracle.dequantize(row0, Q6_K)
    assert deq[[0, 32, 64, 96]].tolist() == [1.0, 2.0, 3.0, 4.0] and np.count_nonzero(deq) == 4


def test_q6k_zero_bytes_give_minus_32_d_sc(oracle):
    blk = np.zeros(210, np.uint8)
    sc = np.arange(-8, 8)
    blk[192:208] = sc.astype(np.int8).view(np.uint8)
    blk[208:210] = f16_bytes(0.5)
    y = oracle.dequantize(blk, Q6_K).reshape(2, 4, 2, 16)  # [half][quarter][l/16][l%16]
    for h in range(2):
        for qt in range(4):
            for lh in range(2):
                assert np.all(y[h, qt, lh] == -32.0 * 0.5 * sc[8 * h + 2 * qt + lh])


def test_q6k_bit_walks(oracle):
    base = np.zeros(210, np.uint8)
    base[192:208] = 1
    base[208:210] = f16_bytes(1.0)
    zero = oracle.dequantize(base, Q6_K)
    assert np.all(zero == -32.0)
    # ql nibble walk: byte 64h + 32p + l, low -> quarter p, high -> quarter p + 2
    for byte in (0, 9, 31, 32, 63, 64, 100, 127):
        for hi in (0, 1):
            blk = base.copy()
            blk[byte] = 0x0F << (4 * hi)
            h, p, l = byte // 64, (byte % 64) // 32, byte % 32
            diff = oracle.dequantize(blk, Q6_K) - zero
            want = np.zeros(256, np.float32)
            want[128 * h + 32 * (p + 2 * hi) + l] = 15.0
            assert np.array_equal(diff, want)
    # qh two-bit walk: bits 2q..2q+1 of qh[32h + l] are element 128h + 32q + l
    for byte in (0, 15, 31, 32, 50, 63):
        for qt in range(4):
            blk = base.copy()
            blk[128 + byte] = 3 << (2 * qt)
            h, l = byte // 32, byte % 32
            diff = oracle.dequantize(blk, Q6_K) - zero
            want = np.zeros(256, np.float32)
            want[128 * h + 32 * qt + l] = 48.0
            assert np.array_equal(diff, want)


def test_q6k_round_trip_and_exact_representability(oracle):
    rng = np.random.default_rng(5)
    for _ in range(20):
        sc, q = rng.integers(-128, 128, 16), rng.integers(-32, 32, 256)
        d = float(np.float16(rng.uniform(0.001, 0.02)))
        b = pack_q6_k(d, sc, q)
        exact = np.float64(d) * sc.reshape(2, 4, 2, 1).astype(np.float64) \
            * q.reshape(2, 4, 2, 16).astype(np.float64)  # scale index 8*half + 2*quarter + l/16
        got = oracle.dequantize(b, Q6_K)
        assert np.array_equal(got.astype(np.float64), exact.reshape(-1))  # no rounding at all


# ------------------------------------------------------------------- Q8_0
def test_q8_0_closed_form(oracle):
    q = np.arange(-16, 16) * 7
    q = np.clip(q, -128, 127)
    b = pack_q8_0(0.0625, q)
    assert np.array_equal(oracle.dequantize(b, Q8_0), (0.0625 * q).astype(np.float32))


# --------------------------------------------------- two restatements agree
@pytest.mark.parametrize("dtype", ALL)
def test_c_and_numpy_restatements_agree_bitwise(oracle, dtype):
    from gllm_amd.synth import random_blocks
    raw = random_blocks(dtype, 300, seed=dtype)
    # sprinkle f16 corner cases into the scale fields: subnormal, zero, negative, large
    blocks = raw.reshape(300, -1)
    off = {Q8_0: 0, Q4_K: 0, Q5_K: 0, Q6_K: 208}[dtype]
    for i, pattern in enumerate([0x0001, 0x03FF, 0x0000, 0x8000, 0xBC00, 0x7BFF, 0x0400]):
        blocks[i, off:off + 2] = np.array([pattern], np.uint16).view(np.uint8)
    a = oracle.dequantize(raw, dtype)
    b = npref.dequantize(raw, dtype)
    assert a.shape == b.shape
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("dtype", ALL)
def test_dequantize_ignores_trailing_partial_chunks(oracle, dtype):
    # chunks_exact on both sides, src/compat/cpu_backend.rs:1066-1075
    from gllm_amd.synth import random_blocks
    bb, bs = oracle.block_bytes(dtype), oracle.block_size(dtype)
    raw = random_blocks(dtype, 3, seed=1)
    full = oracle.dequantize(raw, dtype)
    short_in = oracle.dequantize(raw[: 2 * bb + 5], dtype, n_out=3 * bs)
    assert np.array_equal(short_in[: 2 * bs], full[: 2 * bs]) and np.all(short_in[2 * bs:] == 0)
    short_out = oracle.dequantize(raw, dtype, n_out=2 * bs + 7)
    assert np.array_equal(short_out[: 2 * bs], full[: 2 * bs]) and np.all(short_out[2 * bs:] == 0)
    assert oracle.dequantize(raw[:0], dtype).size == 0


def test_unsupported_dtype_is_an_error_not_a_fallback(oracle):
    with pytest.raises(NotImplementedError):
        oracle.dequantize(np.zeros(18, np.uint8), 2)
    with pytest.raises(NotImplementedError):
        oracle.quantized_matmul(np.zeros(18, np.uint8), np.zeros((1, 32), np.float32), 2, 1, 1, 32)
