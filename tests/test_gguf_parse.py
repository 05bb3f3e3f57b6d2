"""GGUF v3 parsing through the C ABI (host only, no GPU): the cases the reference's own tests hold
(crates/xabe-gguf/src/file.rs:584-752, crates/xabe-gguf/src/types.rs:139-181) on files written by an
independent byte-level writer, plus every other error variant of crates/xabe-gguf/src/error.rs and a
truncation sweep (every proper prefix of a valid file is an error status, never a crash)."""
import struct

import numpy as np
import pytest

import gguf_build as G
from gguf_build import GgufWriter


@pytest.fixture(scope="module")
def X():
    import llmxabe_amd as X
    return X


def _sample():
    return (GgufWriter()
            .kv("general.alignment", G.T_U32, 32)
            .kv("general.architecture", G.T_STRING, "qwen35moe")
            .kv("qwen35moe.block_count", G.T_U32, 40)
            .kv("qwen35moe.attention.layer_norm_rms_epsilon", G.T_F32, 1e-6)
            .kv_array("tokenizer.ggml.tokens", G.T_STRING, ["<pad>", "hello", "wörld"])
            .kv_array("qwen35moe.rope.dimension_sections", G.T_U32, [11, 11, 10, 0])
            .tensor("token_embd.weight", [2048], G.F32, np.arange(2048, dtype=np.float32).tobytes())
            .tensor("blk.0.ffn_gate_exps.weight", [2048, 512, 4], G.Q6K, bytes(range(210)) * (2048 * 512 * 4 // 256)))


def test_types_table(X):
    # types.rs:143-161, :164-168, :171-180
    T = X.GgmlType
    want = {T.F32: (1, 4), T.F16: (1, 2), T.Bf16: (1, 2), T.Q4_0: (32, 18), T.Q8_0: (32, 34), T.Q4K: (256, 144),
            T.Q5K: (256, 176), T.Q6K: (256, 210)}
    for t, (b, s) in want.items():
        assert (t.block_size(), t.type_size()) == (b, s), t
    assert [t.type_name() for t in (T.F32, T.F16, T.Q4_0, T.Q8_0, T.Q4K, T.Q5K, T.Q6K, T.Bf16)] == \
        ["f32", "f16", "q4_0", "q8_0", "q4_K", "q5_K", "q6_K", "bf16"]
    with pytest.raises(X.gguf.UnalignedElementCount):
        T.Q6K.bytes_for_elements(255)
    assert T.Q6K.bytes_for_elements(256) == 210 and T.Q6K.bytes_for_elements(512) == 420
    for i, t in ((0, T.F32), (1, T.F16), (2, T.Q4_0), (8, T.Q8_0), (12, T.Q4K), (13, T.Q5K), (14, T.Q6K), (30, T.Bf16)):
        assert T.try_from(i) == t
    with pytest.raises(X.gguf.UnsupportedGgmlType):
        T.try_from(99)


def test_round_trips_header_metadata_and_tensors(X):
    # file.rs:584-643
    data = _sample().build()
    f = X.GgufFile.from_bytes(data)
    assert (f.version(), f.alignment(), f.n_kv(), f.n_tensors()) == (3, 32, 6, 2)
    assert f.get_u32("general.alignment") == 32
    assert f.get_str("general.architecture") == "qwen35moe"
    assert f.get_u32("qwen35moe.block_count") == 40
    assert abs(f.get_f32("qwen35moe.attention.layer_norm_rms_epsilon") - 1e-6) < 1e-12
    assert f.get_string_array("tokenizer.ggml.tokens") == ["<pad>", "hello", "wörld"]
    assert f.get_u32_array("qwen35moe.rope.dimension_sections") == [11, 11, 10, 0]
    # no coercion between types, absent keys are None
    assert f.get_u64("general.alignment") is None and f.get_str("nonexistent.key") is None
    assert f.get_i32_array("qwen35moe.rope.dimension_sections") is None
    assert f.metadata_keys()[:2] == ["general.alignment", "general.architecture"]
    t0, t1 = f.tensors()
    assert (t0.name, t0.dims, t0.ggml_type, t0.n_bytes, t0.offset) == ("token_embd.weight", (2048,), X.GgmlType.F32, 8192, 0)
    assert t1.n_elements == 2048 * 512 * 4 and t1.n_bytes == 2048 * 512 * 4 // 256 * 210 and t1.offset == 8192
    assert f.tensor("blk.0.ffn_gate_exps.weight") == t1
    assert f.data_offset() % 32 == 0
    assert bytes(f.tensor_bytes("token_embd.weight")) == np.arange(2048, dtype=np.float32).tobytes()
    b1 = f.tensor_bytes("blk.0.ffn_gate_exps.weight")
    assert len(b1) == t1.n_bytes and bytes(b1[:210]) == bytes(range(210)) and bytes(b1[-210:]) == bytes(range(210))
    # the bytes sit where the layout says: data section + offset
    start = f.data_offset() + t1.offset
    assert data[start:start + 420] == bytes(b1[:420])
    assert f.tensor("does.not.exist") is None and f.tensor_bytes("does.not.exist") is None


def test_open_maps_a_file(X, tmp_path):
    data = _sample().build()
    p = tmp_path / "sample.gguf"
    p.write_bytes(data)
    f = X.GgufFile.open(p)
    assert f.n_tensors() == 2 and bytes(f.tensor_bytes("token_embd.weight")) == np.arange(2048, dtype=np.float32).tobytes()
    f.close()
    with pytest.raises(X.gguf.Io):
        X.GgufFile.open(tmp_path / "absent.gguf")
    (tmp_path / "empty.gguf").write_bytes(b"")
    with pytest.raises(X.gguf.UnexpectedEof):
        X.GgufFile.open(tmp_path / "empty.gguf")


def test_every_scalar_and_array_type(X):
    w = GgufWriter()
    scalars = [(G.T_U8, 200), (G.T_I8, -5), (G.T_U16, 60000), (G.T_I16, -300), (G.T_U32, 4000000000), (G.T_I32, -7),
               (G.T_F32, 0.5), (G.T_BOOL, 1), (G.T_U64, 2 ** 63 + 1), (G.T_I64, -2 ** 40), (G.T_F64, 0.25)]
    for tag, v in scalars:
        w.kv(f"k{tag}", tag, v)
    w.kv_array("a.i32", G.T_I32, [-1, 2, -3]).kv_array("a.bool", G.T_BOOL, [1, 0, 7]).kv_array("a.f32", G.T_F32, [1.5, -2.0])
    w.kv_array("a.empty", G.T_U32, []).kv_array("a.strs", G.T_STRING, [])
    f = X.GgufFile.from_bytes(w.build())
    assert f.n_kv() == len(scalars) + 5
    for tag, _ in scalars:
        assert f.value_type(f"k{tag}")[0] == tag
    assert f.get_u32("k4") == 4000000000 and f.get_u64("k10") == 2 ** 63 + 1 and f.get_f32("k6") == 0.5
    assert f.get_u32("k5") is None            # an i32 is not a u32
    assert f.get_i32_array("a.i32") == [-1, 2, -3]
    assert f.get_bool_array("a.bool") == [True, False, True]
    assert f.get_f32_array("a.f32") == [1.5, -2.0]
    assert f.get_u32_array("a.empty") == [] and f.get_string_array("a.strs") == []
    assert f.value_type("a.i32") == (G.T_ARRAY, G.T_I32, 3)


def _err(X, data, exc):
    with pytest.raises(exc):
        X.GgufFile.from_bytes(data)


def test_rejects_malformed_headers(X):
    E = X.gguf
    _err(X, GgufWriter(magic=b"GGML").build(), E.BadMagic)                       # file.rs:655-659
    _err(X, GgufWriter(version=2).build(), E.UnsupportedVersion)                 # file.rs:662-669
    _err(X, b"GG", E.UnexpectedEof)                                              # file.rs:686-690
    _err(X, GgufWriter().build(n_tensors=-1), E.NegativeCount)
    _err(X, GgufWriter().build(n_kv=-3), E.NegativeCount)
    _err(X, GgufWriter().build(n_kv=2), E.UnexpectedEof)                         # counts promise more than the file has
    _err(X, GgufWriter().build(n_tensors=2 ** 62), E.UnexpectedEof)


def test_rejects_malformed_metadata(X):
    E = X.gguf
    _err(X, GgufWriter().kv("a", G.T_U32, 1).kv("a", G.T_U32, 2).build(), E.DuplicateKey)        # file.rs:734-737
    _err(X, GgufWriter().kv("general.alignment", G.T_U32, 3).build(), E.BadAlignment)           # file.rs:740-743
    _err(X, GgufWriter().kv("general.alignment", G.T_U32, 0).build(), E.BadAlignment)
    _err(X, GgufWriter().kv("general.alignment", G.T_U64, 32).build(), E.BadAlignmentType)
    _err(X, GgufWriter().kv_raw(G.gstring("k") + struct.pack("<i", 13)).build(), E.UnknownValueType)
    _err(X, GgufWriter().kv_raw(G.gstring("k") + struct.pack("<iiQ", G.T_ARRAY, 42, 1) + b"\0").build(), E.UnknownValueType)
    _err(X, GgufWriter().kv_raw(G.gstring("k") + struct.pack("<iiQ", G.T_ARRAY, G.T_ARRAY, 0)).build(), E.NestedArray)
    _err(X, GgufWriter().kv_raw(G.gstring(b"\xff\xfe") + struct.pack("<iI", G.T_U32, 1)).build(), E.InvalidUtf8)
    _err(X, GgufWriter().kv("k", G.T_STRING, b"\xc0\xaf").build(), E.InvalidUtf8)                # overlong form
    _err(X, GgufWriter().kv("k", G.T_STRING, b"\xed\xa0\x80").build(), E.InvalidUtf8)            # surrogate
    _err(X, GgufWriter().kv("k", G.T_STRING, b"\xe2\x82").build(), E.InvalidUtf8)                # cut sequence
    # an array that claims more elements than the file holds, and one whose byte size overflows
    _err(X, GgufWriter().kv_raw(G.gstring("k") + struct.pack("<iiQ", G.T_ARRAY, G.T_U32, 10) + b"\0" * 8).build(), E.UnexpectedEof)
    _err(X, GgufWriter().kv_raw(G.gstring("k") + struct.pack("<iiQ", G.T_ARRAY, G.T_U64, 2 ** 62)).build(), E.UnexpectedEof)
    _err(X, GgufWriter().kv_raw(struct.pack("<Q", 2 ** 63) + b"abc").build(), E.UnexpectedEof)   # absurd string length
    f = X.GgufFile.from_bytes(GgufWriter().kv("k", G.T_STRING, "ok é 中 \U0001f600").build())
    assert f.get_str("k") == "ok é 中 \U0001f600"


def test_rejects_malformed_tensor_records(X):
    E = X.gguf
    _err(X, GgufWriter().tensor("t", [255], G.Q6K, b"").build(), E.UnalignedElementCount)       # file.rs:707-714
    _err(X, GgufWriter().tensor("t", [4, 0], G.F32, b"").build(), E.ZeroDimension)              # file.rs:717-722
    _err(X, GgufWriter().tensor("t", [4, -2], G.F32, b"").build(), E.ZeroDimension)
    _err(X, GgufWriter().tensor("t", [4], G.F32).tensor("t", [4], G.F32).build(), E.DuplicateTensor)  # file.rs:725-731
    _err(X, GgufWriter().tensor("t", [2, 2, 2, 2, 2], G.F32).build(), E.TooManyDimensions)
    _err(X, GgufWriter().tensor("t", [4], 99, b"").build(), E.UnsupportedGgmlType)
    _err(X, GgufWriter().tensor("t", [4], G.F32, offset=2 ** 64 - 8).build(pad_data=False), E.OffsetOverflow)
    _err(X, GgufWriter().tensor("t", [2 ** 40, 2 ** 40], G.F32, b"").build(), E.OffsetOverflow)
    _err(X, GgufWriter().tensor("t", [1024], G.F32).build(pad_data=False), E.TensorOutOfBounds)  # file.rs:693-704
    good = GgufWriter().tensor("t", [1024], G.F32).build()
    _err(X, good[:-1], E.TensorOutOfBounds)                                                      # file.rs:672-683
    # a rank-0 tensor is one element (empty product)
    f = X.GgufFile.from_bytes(GgufWriter().tensor("s", [], G.F32, struct.pack("<f", 2.5)).build())
    assert f.tensor("s").n_elements == 1 and bytes(f.tensor_bytes("s")) == struct.pack("<f", 2.5)


def test_alignment(X):
    # file.rs:746-751: 32 when the key is absent; a declared alignment moves the data section
    f = X.GgufFile.from_bytes(GgufWriter().tensor("t", [8], G.F32, bytes(range(32))).build())
    assert f.alignment() == 32 and f.data_offset() % 32 == 0
    w = GgufWriter().kv("general.alignment", G.T_U32, 4096).tensor("t", [8], G.F32, bytes(range(32)))
    w.tensor("u", [8], G.F32, bytes(range(32, 64)))
    f = X.GgufFile.from_bytes(w.build())
    assert f.alignment() == 4096 and f.data_offset() == 4096 and f.tensor("u").offset == 4096
    assert bytes(f.tensor_bytes("t")) == bytes(range(32)) and bytes(f.tensor_bytes("u")) == bytes(range(32, 64))


def test_every_prefix_of_a_valid_file_is_an_error(X):
    w = (GgufWriter().kv("general.architecture", G.T_STRING, "qwen35moe").kv_array("a", G.T_STRING, ["x", "yz"])
         .kv_array("b", G.T_U16, [1, 2, 3]).tensor("blk.0.ffn_gate_inp.weight", [32, 4], G.BF16).tensor("n", [32], G.F32))
    data = w.build()
    X.GgufFile.from_bytes(data)
    kinds = set()
    for n in range(len(data)):
        with pytest.raises(X.gguf.GgufError) as e:
            X.GgufFile.from_bytes(data[:n])
        kinds.add(type(e.value).__name__)
    assert kinds == {"UnexpectedEof", "TensorOutOfBounds"}
