"""The GGUF reader behind include/wick_gguf.h against byte images built here, on the cases the
reference's own tests hold (wick/src/gguf.rs:828-1052: minimal header, tiny buffer, bad magic,
tensor_data_size incl. overflow and ragged blocks, unsupported-type tensors listed but not
readable) and the limits of its parser (wick/src/gguf.rs:216-248, 404-545).  Runs without a GPU."""
import os
import struct

import numpy as np
import pytest

import gguf_writer as GW
from wick_amd import gguf as G

F32, F16, Q4_0, Q8_0, Q4_K, Q6_K, I32, BF16 = 0, 1, 2, 8, 12, 14, 26, 30


def minimal():
    return b"GGUF" + struct.pack("<IQQ", 3, 0, 0)


def test_minimal_header():
    with G.GgufFile.from_bytes(minimal()) as g:
        assert g.keys() == [] and g.tensor_names() == []
        assert g.size == 24
        assert g.data_offset == 32 and g.alignment == 32  # header end rounded up to the default alignment


def test_too_small_and_bad_magic_and_version():
    with pytest.raises(G.GgufError, match="too small"):
        G.GgufFile.from_bytes(bytes(10))
    with pytest.raises(G.GgufError, match="not a GGUF file"):
        G.GgufFile.from_bytes(b"ABCD" + minimal()[4:])
    with pytest.raises(G.GgufError, match="unsupported GGUF version 2"):
        G.GgufFile.from_bytes(b"GGUF" + struct.pack("<IQQ", 2, 0, 0))


def test_tensor_data_size_table():
    assert G.tensor_data_size(F32, 10 * 20) == 10 * 20 * 4
    assert G.tensor_data_size(F16, 10 * 20) == 10 * 20 * 2
    assert G.tensor_data_size(BF16, 7) == 14
    assert G.tensor_data_size(I32, 3) == 12
    assert G.tensor_data_size(Q8_0, 256) == 8 * 34
    assert G.tensor_data_size(Q4_0, 256) == 8 * 18
    assert G.tensor_data_size(Q4_K, 512) == 2 * 144
    assert G.tensor_data_size(Q6_K, 512) == 2 * 210
    with pytest.raises(G.GgufError, match="not divisible by block size 32"):
        G.tensor_data_size(Q8_0, 100)
    with pytest.raises(G.GgufError, match="overflow"):
        G.tensor_data_size(F32, 2**63)
    with pytest.raises(G.GgufError) as e:
        G.tensor_data_size(3, 32)  # Q4_1: parseable id, no block size here
    assert e.value.status == -5
    assert [G.type_name(t) for t in (0, 1, 2, 3, 8, 12, 14, 26, 30, 99)] == ["F32", "F16", "Q4_0", "Q4_1", "Q8_0", "Q4_K", "Q6_K",
                                                                              "I32", "BF16", "???"]


METADATA = [
    ("general.architecture", GW.T_STRING, "lfm2"),
    ("lfm2.block_count", GW.T_U32, 16),
    ("lfm2.attention.layer_norm_rms_epsilon", GW.T_F32, 1e-5),
    ("tokenizer.ggml.add_bos_token", GW.T_BOOL, 1),
    ("some.u8", GW.T_U8, 200), ("some.i8", GW.T_I8, -3), ("some.u16", GW.T_U16, 65535), ("some.i16", GW.T_I16, -300),
    ("some.i32", GW.T_I32, -70000), ("some.u64", GW.T_U64, 2**40 + 5), ("some.i64", GW.T_I64, -(2**40)), ("some.f64", GW.T_F64, 0.25),
    ("lfm2.attention.head_count_kv", GW.T_ARRAY, (GW.T_I32, [0, 0, 8, 0, 8])),
    ("tokenizer.ggml.tokens", GW.T_ARRAY, (GW.T_STRING, ["<pad>", "hello", "", "wörld"])),
    ("tokenizer.ggml.scores", GW.T_ARRAY, (GW.T_F32, [0.0, -1.5, 2.25])),
    ("nested", GW.T_ARRAY, (GW.T_ARRAY, [(GW.T_U8, [1, 2]), (GW.T_U8, [])])),
    ("empty", GW.T_ARRAY, (GW.T_U32, [])),
]


def test_metadata_getters_match_exact_types_only():
    img, _ = GW.build(METADATA)
    with G.GgufFile.from_bytes(img) as g:
        assert g.keys() == [k for k, _, _ in METADATA]
        assert g.architecture() == "lfm2"
        assert g.get_u32("lfm2.block_count") == 16
        assert g.get_f32("lfm2.attention.layer_norm_rms_epsilon") == np.float32(1e-5)
        assert g.get_bool("tokenizer.ggml.add_bos_token") is True
        # the reference's typed getters return None on another stored type (wick/src/gguf.rs:553-575)
        assert g.get_u32("some.i32") is None and g.get_f32("some.f64") is None and g.get_str("lfm2.block_count") is None
        assert g.get_u32("missing") is None and g.get_bool("lfm2.block_count") is None
        assert [g.get_int(k) for k in ("some.u8", "some.i8", "some.u16", "some.i16", "some.i32", "some.u64", "some.i64")] == [
            200, -3, 65535, -300, -70000, 2**40 + 5, -(2**40)]
        assert g.get_int("general.architecture") is None
        assert g.get_array("lfm2.attention.head_count_kv", GW.T_I32).tolist() == [0, 0, 8, 0, 8]
        assert g.get_array("lfm2.attention.head_count_kv", GW.T_U32) is None
        assert g.get_array("tokenizer.ggml.scores", GW.T_F32).tolist() == [0.0, -1.5, 2.25]
        assert g.get_array("empty", GW.T_U32).size == 0
        assert g.get_string_array("tokenizer.ggml.tokens") == ["<pad>", "hello", "", "wörld"]
        assert g.get_string_array("tokenizer.ggml.scores") is None
        assert g.value_type("nested") == (GW.T_ARRAY, GW.T_ARRAY, 2)
        assert g.value_type("tokenizer.ggml.tokens") == (GW.T_ARRAY, GW.T_STRING, 4)


def rng_bytes(n, seed):
    return np.random.default_rng(seed).integers(0, 256, n, dtype=np.uint8)


TENSORS = [
    ("blk.0.attn_q.weight", [1024, 96], Q4_0, rng_bytes(96 * 32 * 18, 1)),
    ("blk.0.ffn_down.weight", [512, 40], Q8_0, rng_bytes(40 * 16 * 34, 2)),
    ("token_embd.weight", [256, 9], Q6_K, rng_bytes(9 * 210, 3)),
    ("blk.0.attn_norm.weight", [1024], F32, np.arange(1024, dtype=np.float32)),
    ("conv", [3, 5, 2], F16, np.arange(30, dtype=np.float16)),
    ("odd.type", [64], 3, b""),  # Q4_1: listed with size 0, data refused
]


@pytest.mark.parametrize("alignment", [None, 64, 4096, 1])
def test_tensor_infos_and_bytes(alignment):
    img, where = GW.build(METADATA[:3], TENSORS, alignment=alignment)
    with G.GgufFile.from_bytes(img) as g:
        assert g.alignment == (alignment or 32) and g.data_offset % g.alignment == 0
        assert g.tensor_names() == [t[0] for t in TENSORS]
        for name, dims, gt, data in TENSORS[:-1]:
            info = g.tensor_info(name)
            raw = GW.as_bytes(data) if isinstance(data, np.ndarray) else data
            assert info == {"name": name, "ggml_type": gt, "shape": dims, "offset": where[name], "size_bytes": len(raw)}
            assert g.tensor_data(name).tobytes() == raw
            assert img[info["offset"]: info["offset"] + info["size_bytes"]] == raw
        # rows = ne1, cols = ne0; rank 1 -> one row (wick/src/gguf.rs:678-693)
        assert g.tensor_meta("blk.0.attn_q.weight") == (where["blk.0.attn_q.weight"], 96, 1024, Q4_0)
        assert g.tensor_meta("blk.0.attn_norm.weight") == (where["blk.0.attn_norm.weight"], 1, 1024, F32)
        with pytest.raises(G.GgufError, match="unexpected rank"):
            g.tensor_meta("conv")
        assert g.tensor_info("odd.type")["size_bytes"] == 0
        with pytest.raises(G.GgufError, match=r"unsupported GGML type 3 \(Q4_1\)") as e:
            g.tensor_data("odd.type")
        assert e.value.status == -5
        with pytest.raises(G.GgufError, match="tensor not found: nope") as e:
            g.tensor_data("nope")
        assert e.value.status == -4


def test_open_maps_a_file(tmp_path):
    img, where = GW.build(METADATA, TENSORS)
    p = tmp_path / "model.gguf"
    p.write_bytes(img)
    with G.GgufFile.open(str(p)) as g:
        assert g.size == len(img)
        assert g.tensor_data("token_embd.weight").tobytes() == TENSORS[2][3].tobytes()
        assert g.architecture() == "lfm2"
    with pytest.raises(G.GgufError) as e:
        G.GgufFile.open(str(tmp_path / "missing.gguf"))
    assert e.value.status == -2
    (tmp_path / "tiny.gguf").write_bytes(b"GGUF")
    with pytest.raises(G.GgufError, match="too small"):
        G.GgufFile.open(str(tmp_path / "tiny.gguf"))


def test_malformed_images_are_rejected():
    good, _ = GW.build(METADATA[:2], TENSORS[:2])
    # truncated anywhere inside the header: a clean error, never a read past the end
    with G.GgufFile.from_bytes(good) as g:
        header_end = g.data_offset
    for cut in list(range(24, header_end - 32, 7)):
        with pytest.raises(G.GgufError):
            G.GgufFile.from_bytes(good[:cut])
    # data section cut short
    with pytest.raises(G.GgufError, match="extends beyond file"):
        G.GgufFile.from_bytes(good[:-40])
    # limits of the parser (wick/src/gguf.rs:219, 243, 454-457, 495-498)
    with pytest.raises(G.GgufError, match="string too long"):
        G.GgufFile.from_bytes(b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + struct.pack("<Q", 1_000_000) + bytes(64))
    with pytest.raises(G.GgufError, match="array too long"):
        G.GgufFile.from_bytes(b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + GW.gstr("k") + struct.pack("<IIQ", GW.T_ARRAY, GW.T_U8, 10_000_000) + bytes(64))
    with pytest.raises(G.GgufError, match="unknown GGUF value type"):
        G.GgufFile.from_bytes(b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + GW.gstr("k") + struct.pack("<I", 13) + bytes(64))
    with pytest.raises(G.GgufError, match="too many dimensions: 9"):
        G.GgufFile.from_bytes(b"GGUF" + struct.pack("<IQQ", 3, 1, 0) + GW.gstr("t") + struct.pack("<I", 9) + bytes(128))
    for bad in (0, 2 * 1024 * 1024):
        with pytest.raises(G.GgufError, match="invalid GGUF alignment"):
            G.GgufFile.from_bytes(b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + GW.gstr("general.alignment") + struct.pack("<II", GW.T_U32, bad))
    with pytest.raises(G.GgufError, match="not divisible by block size"):
        G.GgufFile.from_bytes(GW.build([], [("w", [100], Q8_0, bytes(200))])[0])
    with pytest.raises(G.GgufError, match="overflow"):
        G.GgufFile.from_bytes(GW.build([], [("w", [2**40, 2**40], F32, b"")])[0])
    with pytest.raises(G.GgufError, match="invalid UTF-8"):
        G.GgufFile.from_bytes(b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + GW.gstr(b"k\xff") + struct.pack("<II", GW.T_U32, 1))
    for bad in (b"\xc0\x80", b"\xed\xa0\x80", b"\xf4\x90\x80\x80", b"\xe2\x82"):  # overlong, surrogate, > U+10FFFF, cut short
        with pytest.raises(G.GgufError, match="invalid UTF-8"):
            G.GgufFile.from_bytes(GW.build([("k", GW.T_STRING, bad)])[0])
    with pytest.raises(G.GgufError, match="counts exceed the file"):
        G.GgufFile.from_bytes(b"GGUF" + struct.pack("<IQQ", 3, 2**60, 0))


def test_alignment_counts_only_as_u32():
    """general.alignment stored with another type is ignored (wick/src/gguf.rs:487-490)."""
    img, _ = GW.build([("general.alignment", GW.T_U64, 4096)], TENSORS[:1])
    with G.GgufFile.from_bytes(img) as g:
        assert g.alignment == 32


def test_repeated_key_keeps_the_last_value():
    img, _ = GW.build([("a", GW.T_U32, 1), ("a", GW.T_U32, 2)])
    with G.GgufFile.from_bytes(img) as g:
        assert g.get_u32("a") == 2 and g.keys() == ["a"]


def test_mutated_images_never_crash_the_parser():
    """Byte flips, truncations and length-field blow-ups of a valid image either parse or raise."""
    small = [("a", [32, 2], Q4_0, rng_bytes(36, 1)), ("b", [4], F32, rng_bytes(16, 2)), ("c", [256], Q6_K, rng_bytes(210, 3))]
    good, _ = GW.build(METADATA, small)
    with G.GgufFile.from_bytes(good) as g:
        header_end = g.data_offset
    rng = np.random.default_rng(5)
    outcomes = {"ok": 0, "err": 0}
    for it in range(1500):
        img = bytearray(good)
        for _ in range(int(rng.integers(1, 4))):
            pos = int(rng.integers(4, header_end))
            img[pos] = int(rng.integers(0, 256)) if it % 3 else 0xFF
        if it % 5 == 0:
            img = img[: int(rng.integers(24, len(img)))]
        try:
            with G.GgufFile.from_bytes(bytes(img)) as g:
                for name in g.tensor_names():
                    info = g.tensor_info(name)
                    if info["size_bytes"]:
                        assert info["offset"] + info["size_bytes"] <= len(img)
                for k in g.keys():
                    g.value_type(k)
            outcomes["ok"] += 1
        except G.GgufError:
            outcomes["err"] += 1
    assert outcomes["err"] > 100 and outcomes["ok"] > 100  # both the error paths and mutated-but-valid images are reached
