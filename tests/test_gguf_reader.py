"""The GGUF reader against what the reference's reader accepts, rejects and hands out
(src/loader/gguf/reader.rs:38-187 and its unit tests; src/loader/gguf/types.rs:443-472).
Host only: no GPU."""
import os

import numpy as np
import pytest

from gllm_amd.gguf import GgufError, GgufFile
from gllm_amd.synth import random_weight
from tests import gguf_writer as W

Q8_0, Q4_K, Q6_K = 8, 12, 14


def simple(**kw):
    meta = [("general.architecture", W.STR, "llama"), ("llama.block_count", W.U32, 2)]
    a = np.arange(32, dtype=np.float32).reshape(4, 8)
    return W.build(kw.pop("metadata", meta), kw.pop("tensors", [W.f32_tensor("a.weight", a)]), **kw)


def test_header_counts_and_default_alignment():
    g = GgufFile(image=simple())
    assert (g.version, g.tensor_count, g.kv_count, g.alignment) == (3, 1, 2, 32)  # default alignment 32 (reader.rs:102-107)
    assert g.data_offset % 32 == 0
    assert g.meta("general.architecture") == "llama" and g.meta("llama.block_count") == 2
    assert g.meta("no.such.key") is None


def test_shapes_are_reversed_to_outermost_first():
    """reader.rs tests iter_tensors_yields_reversed_shapes ([8,4] -> [4,8]), the 3-D case
    ([8,4,2] -> [2,4,8]) and tensor_provider_1d_shape_not_reversed."""
    t2 = ("m", [8, 4], 0, np.zeros(32, np.float32).tobytes())
    t3 = ("c", [8, 4, 2], 0, np.zeros(64, np.float32).tobytes())
    t1 = ("v", [8], 0, np.zeros(8, np.float32).tobytes())
    g = GgufFile(image=simple(tensors=[t2, t3, t1]))
    assert g.tensor("m").shape == (4, 8) and g.tensor("m").ne == (8, 4)
    assert g.tensor("c").shape == (2, 4, 8)
    assert g.tensor("v").shape == (8,)
    assert [t.name for t in g.tensors()] == ["m", "c", "v"]


def test_tensor_bytes_pad_rows_to_whole_blocks():
    # types.rs:443-472; the documented example: Q4_0 [33, 2] is 2 blocks x 18 bytes x 2 rows = 72
    cases = [(2, [33, 2], 72), (2, [33], 36), (Q8_0, [33], 68), (Q4_K, [256, 4], 576), (Q6_K, [256, 4], 840),
             (Q4_K, [300, 3], 2 * 144 * 3), (0, [5, 7], 140), (30, [6], 12), (15, [256], 292), (39, [64], 34)]
    tensors = [(f"t{i}", ne, dt, bytes(n)) for i, (dt, ne, n) in enumerate(cases)]
    g = GgufFile(image=simple(tensors=tensors))
    for i, (dt, ne, n) in enumerate(cases):
        assert g.tensor(f"t{i}").nbytes == n, (dt, ne)
    # every tensor starts on a multiple of the alignment behind the data offset
    assert all((t.offset - g.data_offset) % 32 == 0 for t in g.tensors())


def test_tensor_data_is_what_was_written_and_alignment_key_is_honoured():
    w = random_weight(Q4_K, 5, 512, seed=1)
    a = np.arange(12, dtype=np.float32)
    meta = [("general.alignment", W.U32, 64), ("x", W.F32, 1.5)]
    g = GgufFile(image=simple(metadata=meta, tensors=[("w", [512, 5], Q4_K, np.asarray(w).tobytes()), W.f32_tensor("a", a)]))
    assert g.alignment == 64 and g.data_offset % 64 == 0
    assert g.tensor_bytes("w") == np.asarray(w).tobytes()
    assert np.array_equal(np.frombuffer(g.tensor_bytes("a"), np.float32), a)
    assert g.tensor("w").shape == (5, 512) and g.tensor("w").ggml_dtype == Q4_K
    assert g.tensor("a").offset % 64 == 0


def test_metadata_value_types():
    meta = [("u8", W.U8, 42), ("i8n", W.I8, -1), ("i8p", W.I8, 100), ("u16", W.U16, 0x1234), ("i16n", W.I16, -32768),
            ("u32", W.U32, 7), ("i32", W.I32, -5), ("f32", W.F32, 0.25), ("yes", W.BOOL, 1), ("no", W.BOOL, 0),
            ("s", W.STR, "中文测试"), ("empty", W.STR, ""), ("u64", W.U64, 2 ** 63 + 5), ("i64", W.I64, -2 ** 62),
            ("f64", W.F64, 1e100), ("toks", W.ARR, (W.STR, ["<s>", "</s>", "hello"])), ("nums", W.ARR, (W.I32, [1, 2, 3])),
            ("nest", W.ARR, (W.ARR, [(W.U8, [1, 2]), (W.U8, [])]))]
    g = GgufFile(image=simple(metadata=meta))
    assert g.kv_count == len(meta)
    # GgufValue::as_u64 (reader.rs tests parse_value_uint8 / _int8 / _int8_positive / _uint16 / _int16_negative)
    assert g.meta_u64("u8") == 42 and g.meta_u64("i8n") is None and g.meta_u64("i8p") == 100
    assert g.meta_u64("u16") == 0x1234 and g.meta_u64("i16n") is None and g.meta_u64("s") is None
    assert g.meta("i8n") == -1 and g.meta("i16n") == -32768 and g.meta("i32") == -5 and g.meta("i64") == -2 ** 62
    assert g.meta("u64") == 2 ** 63 + 5 and g.meta("f32") == 0.25 and g.meta("f64") == 1e100
    assert g.meta("yes") is True and g.meta("no") is False
    assert g.meta("s") == "中文测试" and g.meta("empty") == ""   # read_string_utf8_cjk, read_string_empty
    assert g.meta("toks") == ["<s>", "</s>", "hello"] and g.meta("nums") == (W.I32, 3) and g.meta("nest") == (W.ARR, 2)


def test_rejections():
    def kind(image):
        with pytest.raises(GgufError) as e:
            GgufFile(image=image)
        return e.value.kind
    assert kind(simple(magic=0x46554746)) == "InvalidMagic"
    assert kind(simple(version=2)) == "UnsupportedVersion" and kind(simple(version=4)) == "UnsupportedVersion"
    assert kind(simple(metadata=[("general.alignment", W.U32, 0)], alignment=32)) == "InvalidMetadata"
    assert kind(b"GGUF") == "ParseError" and kind(b"") == "ParseError"
    whole = simple()
    for cut in (10, 24, 40, len(whole) - 130):       # inside the header, a key, a value, the tensor infos
        assert kind(whole[:cut]) == "ParseError", cut
    assert kind(whole[:-1]) == "TensorOutOfBounds"    # the last tensor loses a byte
    assert kind(simple(offsets=[1 << 40])) == "TensorOutOfBounds"
    # a count that claims one more tensor info than the file holds reads padding as an info: rejected one way or the other
    assert kind(simple(tensor_count=2)) in ("ParseError", "TensorOutOfBounds", "UnknownDType")
    two = [W.f32_tensor("same", np.zeros(4)), W.f32_tensor("same", np.ones(4))]
    assert kind(simple(tensors=two)) == "ParseError"  # duplicate tensor name
    assert kind(simple(tensors=[("t", [4], 4, bytes(16))])) == "UnknownDType"   # id 4 is a hole in the table
    assert kind(simple(tensors=[("t", [1 << 62, 1 << 62], 0, b"")])) == "ParseError"  # byte size overflow
    assert kind(simple(metadata=[("k", 13, 0)])) == "ParseError"               # value type outside 0..12
    assert kind(simple(metadata=[("s", W.STR, b"ab\xff")])) == "Utf8"            # str::from_utf8 of the reference
    assert kind(simple(metadata=[("s", W.STR, b"\xed\xa0\x80")])) == "Utf8"     # a surrogate
    assert kind(simple(metadata=[("s", W.STR, b"\xc0\x80")])) == "Utf8"         # an overlong form
    assert kind(simple(tensors=[(b"t\xfe", [4], 0, bytes(16))])) == "Utf8"
    # an array that claims 2^40 items in a file of a few hundred bytes
    img = bytearray(simple(metadata=[("a", W.ARR, (W.U32, [1, 2]))]))
    at = img.index(b"a" + (W.ARR).to_bytes(4, "little") + (W.U32).to_bytes(4, "little")) + 9
    img[at:at + 8] = (1 << 40).to_bytes(8, "little")
    assert kind(bytes(img)) == "ParseError"


def test_a_key_that_repeats_keeps_the_later_value_and_odd_alignment_types_fall_back():
    g = GgufFile(image=simple(metadata=[("k", W.U32, 1), ("k", W.U32, 2)]))
    assert g.meta("k") == 2 and g.kv_count == 2
    # a general.alignment that is not an unsigned number reads as absent: the default 32
    g = GgufFile(image=simple(metadata=[("general.alignment", W.STR, "64")], alignment=32))
    assert g.alignment == 32


def test_open_from_a_file(tmp_path):
    path = os.path.join(tmp_path, "m.gguf")
    w = random_weight(Q6_K, 3, 256, seed=2)
    with open(path, "wb") as f:
        f.write(simple(tensors=[("blk.0.ffn_down.weight", [256, 3], Q6_K, np.asarray(w).tobytes())]))
    g = GgufFile(path)
    assert g.tensor("blk.0.ffn_down.weight").shape == (3, 256)
    assert g.tensor_bytes(0) == np.asarray(w).tobytes()
    with pytest.raises(KeyError):
        g.tensor("blk.1.ffn_down.weight")
    g.close()
    with pytest.raises(GgufError) as e:
        GgufFile(os.path.join(tmp_path, "missing.gguf"))
    assert e.value.kind == "Io"


def test_mutated_files_never_crash_the_reader():
    """Two thousand seeded mutations (byte flips, truncations, length fields blown up) of a valid
    file: each either opens or raises GgufError; tensor views stay inside the image."""
    meta = [("general.architecture", W.STR, "llama"), ("toks", W.ARR, (W.STR, ["a", "bc"])), ("n", W.U64, 5),
            ("nest", W.ARR, (W.ARR, [(W.U8, [1, 2]), (W.U8, [3])]))]
    base = W.build(meta, [W.f32_tensor("a", np.arange(16).reshape(2, 8)), ("q", [64, 2], Q8_0, bytes(136))])
    rng = np.random.default_rng(0)
    opened = 0
    for i in range(2000):
        img = bytearray(base)
        how = i % 4
        if how == 0:
            for _ in range(int(rng.integers(1, 4))):
                img[int(rng.integers(0, len(img)))] = int(rng.integers(0, 256))
        elif how == 1:
            img = img[:int(rng.integers(0, len(img)))]
        elif how == 2:
            at = int(rng.integers(0, max(1, len(img) - 8)))
            img[at:at + 8] = int(rng.integers(0, 1 << 63)).to_bytes(8, "little")
        else:
            at = int(rng.integers(0, max(1, len(img) - 4)))
            img[at:at + 4] = b"\xff\xff\xff\xff"
        try:
            g = GgufFile(image=bytes(img))
        except GgufError:
            continue
        opened += 1
        for t in g.tensors():
            assert t.offset + t.nbytes <= len(img)
            assert len(g.tensor_bytes(t.index)) == t.nbytes
        for key in ("general.architecture", "toks", "n", "nest"):
            g.meta(key)
    assert opened > 0


def k_m_style_file(layers=4, hidden=256, ffn=512, down_q6k=(0, 3)):
    """Per-layer weights as a Q4_K_M file lays them out: ffn_down is Q6_K in some layers, Q4_K in the rest."""
    tensors, host = [], {}
    for layer in range(layers):
        for proj, (n, k) in (("ffn_gate", (ffn, hidden)), ("ffn_up", (ffn, hidden)), ("ffn_down", (hidden, ffn))):
            dt = Q6_K if (proj == "ffn_down" and layer in down_q6k) else Q4_K
            w = random_weight(dt, n, k, seed=100 * layer + len(proj))
            name = f"blk.{layer}.{proj}.weight"
            tensors.append((name, [k, n], dt, np.asarray(w).tobytes()))
            host[name] = (dt, n, k, w)
    tensors.append(W.f32_tensor("output_norm.weight", np.ones(hidden)))
    meta = [("general.architecture", W.STR, "llama"), ("llama.block_count", W.U32, layers)]
    return W.build(meta, tensors), host


def test_layer_table_and_mixed_quant_groups():
    image, host = k_m_style_file()
    g = GgufFile(image=image)
    table = g.layer_table()
    assert list(table) == [0, 1, 2, 3] and sorted(table[2]) == ["ffn_down", "ffn_gate", "ffn_up"]
    assert [table[i]["ffn_down"].ggml_dtype for i in range(4)] == [Q6_K, Q4_K, Q4_K, Q6_K]
    assert all(table[i]["ffn_gate"].ggml_dtype == Q4_K and table[i]["ffn_gate"].shape == (512, 256) for i in range(4))
    groups = g.mixed_quant_groups()
    assert [layers for _, layers in groups] == [[1, 2], [0, 3]]          # by signature (dtype 12 before 14), then first layer
    assert dict(groups[1][0])["ffn_down"] == Q6_K
    uniform, _ = k_m_style_file(down_q6k=())
    assert GgufFile(image=uniform).mixed_quant_groups() is None          # the reference's plan is None for uniform models
    # look-ups through the C ABI: a weight by (layer, projection), absent ones, names that are not per-layer weights
    assert g.layer_tensor(3, "ffn_down").name == "blk.3.ffn_down.weight" and g.layer_tensor(3, "ffn_down").ggml_dtype == Q6_K
    assert g.layer_tensor(4, "ffn_down") is None and g.layer_tensor(0, "attn_q") is None
    assert all("output_norm" not in projs for projs in table.values())


def test_layer_table_with_gaps_and_other_names():
    """Layer indices without weights get no group; names with another shape than
    blk.{layer}.{projection}.weight (biases, nested names, non-numeric layers) stay out of the table."""
    w = lambda name, dt: (name, [256, 4], dt, np.asarray(random_weight(dt, 4, 256, seed=1)).tobytes())
    tensors = [w("blk.0.ffn_down.weight", Q4_K), w("blk.2.ffn_down.weight", Q6_K), w("blk.5.ffn_down.weight", Q4_K),
               w("blk.5.ffn_up.weight", Q4_K), w("blk.1.ffn_down.bias", Q4_K), w("blk.x.ffn_down.weight", Q4_K),
               w("blk.3.attn.q.weight", Q4_K), w("enc.blk.0.ffn_down.weight", Q4_K)]
    g = GgufFile(image=W.build([("general.architecture", W.STR, "llama")], tensors))
    table = g.layer_table()
    assert list(table) == [0, 2, 5] and sorted(table[5]) == ["ffn_down", "ffn_up"]
    groups = g.mixed_quant_groups()
    # signatures in order: (ffn_down Q4_K), (ffn_down Q4_K, ffn_up Q4_K), (ffn_down Q6_K)
    assert [layers for _, layers in groups] == [[0], [5], [2]]


def test_stray_layer_indices_cost_nothing():
    """Layer numbers come from tensor names: a file with a tensor named blk.99999999999999.x.weight
    must not make the table (or anything sized by the layer count) that large.  Layers at or beyond
    the declared `{architecture}.block_count` are ignored, as the reference ignores layers beyond
    num_layers (build_graph.inc.rs:416-428); without the key nothing beyond the tensor count is."""
    w = lambda name, dt: (name, [256, 4], dt, np.asarray(random_weight(dt, 4, 256, seed=1)).tobytes())
    tensors = [w("blk.0.ffn_down.weight", Q4_K), w("blk.1.ffn_down.weight", Q6_K), w("blk.99999999999999.ffn_down.weight", Q4_K),
               w("blk.7.ffn_down.weight", Q4_K)]
    declared = GgufFile(image=W.build([("general.architecture", W.STR, "llama"), ("llama.block_count", W.U32, 2)], tensors))
    assert declared.layer_count() == 2 and list(declared.layer_table()) == [0, 1]
    assert declared.layer_tensor(7, "ffn_down") is None and declared.layer_tensor(99999999999999, "ffn_down") is None
    assert [layers for _, layers in declared.mixed_quant_groups()] == [[0], [1]]
    undeclared = GgufFile(image=W.build([("general.architecture", W.STR, "llama")], tensors))
    assert undeclared.layer_count() == 2 and list(undeclared.layer_table()) == [0, 1]  # four tensors: layers 0..3 at most
    signed = GgufFile(image=W.build([("general.architecture", W.STR, "llama"), ("llama.block_count", W.I32, -1)], tensors))
    assert signed.layer_count() == 2  # a negative count reads as absent
    assert declared.tensor("blk.7.ffn_down.weight").ggml_dtype == Q4_K  # still a tensor of the file
