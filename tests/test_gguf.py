"""The GGUF v3 container reader against files written here byte by byte, with the
reference's own unit-test statements (src/gguf/mod.rs:219-231, reader.rs:92-129,
value.rs:107-141, tensor_info.rs:69-100, types.rs:140-150) restated on the C ABI, the
error paths of src/gguf/error.rs, and the load path: container -> repacked slab equals the
oracle's repack of the same tensor bytes."""
import struct

import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import gguf, quant
from oracle import orc
from helpers import (GGUF_ARRAY, GGUF_BOOL, GGUF_F32, GGUF_F64, GGUF_I8, GGUF_I16, GGUF_I32, GGUF_I64, GGUF_STRING,
                     GGUF_U8, GGUF_U16, GGUF_U32, GGUF_U64, gguf_string, random_raw_weights, write_gguf)


def parse_error(data):
    with pytest.raises(rein.ReinError) as e:
        gguf.GgufFile.from_bytes(data)
    assert e.value.code == -7
    return str(e.value)


def test_align_up_cases_of_the_reference():             # mod.rs:223-230
    assert gguf.align_up(0, 32) == 0
    assert gguf.align_up(1, 32) == 32
    assert gguf.align_up(32, 32) == 32
    assert gguf.align_up(33, 32) == 64
    assert gguf.align_up(100, 1) == 100
    assert gguf.align_up(100, 0) == 100


def test_empty_container_and_header():
    data, _ = write_gguf([], [])
    with gguf.GgufFile.from_bytes(data) as g:
        assert g.header == {"version": 3, "tensor_count": 0, "metadata_kv_count": 0}
        assert g.alignment == 32 and g.data_section_offset == 32      # 24 header bytes aligned up
        assert g.tensors == [] and g.tensor("x") is None and g.tensor_data("x") is None
        assert g.metadata_get("x") is None


def test_primitives_round_trip():                        # reader.rs:96-109
    meta = [("a.u32", GGUF_U32, 0xDEADBEEF), ("a.i64", GGUF_I64, -1), ("a.f32", GGUF_F32, 3.5), ("a.bool", GGUF_BOOL, 1),
            ("a.u8", GGUF_U8, 200), ("a.i8", GGUF_I8, -100), ("a.u16", GGUF_U16, 65535), ("a.i16", GGUF_I16, -32768),
            ("a.i32", GGUF_I32, -7), ("a.u64", GGUF_U64, 2 ** 63 + 5), ("a.f64", GGUF_F64, 1.0 / 3.0)]
    data, _ = write_gguf(meta, [])
    with gguf.GgufFile.from_bytes(data) as g:
        assert [k for k, _ in g.metadata_keys()] == [k for k, _, _ in meta]
        assert [t for _, t in g.metadata_keys()] == [t for _, t, _ in meta]
        assert g.metadata_get("a.u32") == 0xDEADBEEF
        assert g.metadata_get("a.i64") == -1
        assert g.metadata_get("a.f32") == 3.5
        assert g.metadata_get("a.bool") is True
        assert g.metadata_get("a.u8") == 200 and g.metadata_get("a.i8") == -100
        assert g.metadata_get("a.u16") == 65535 and g.metadata_get("a.i16") == -32768
        assert g.metadata_get("a.i32") == -7 and g.metadata_get("a.u64") == 2 ** 63 + 5
        assert g.metadata_get("a.f64") == 1.0 / 3.0
        # MetaValue::as_u64 / as_f32 coercions (value.rs:69-94)
        assert g.as_u64("a.u8") == 200 and g.as_u64("a.u64") == 2 ** 63 + 5
        assert g.as_u64("a.i64") is None and g.as_u64("a.i8") is None      # negative
        assert g.as_u64("a.f32") is None and g.as_u64("a.bool") is None and g.as_u64("missing") is None
        assert g.as_f32("a.f32") == 3.5 and g.as_f32("a.f64") == np.float32(1.0 / 3.0)
        assert g.as_f32("a.u32") is None


def test_signed_integers_that_fit_coerce_to_u64():       # value.rs:74-78
    data, _ = write_gguf([("s8", GGUF_I8, 5), ("s16", GGUF_I16, 300), ("s32", GGUF_I32, 70000), ("s64", GGUF_I64, 2 ** 40)], [])
    with gguf.GgufFile.from_bytes(data) as g:
        assert [g.as_u64(k) for k in ("s8", "s16", "s32", "s64")] == [5, 300, 70000, 2 ** 40]


def test_string_values_decode_utf8():                    # reader.rs:111-119, value.rs:111-119
    data, _ = write_gguf([("general.architecture", GGUF_STRING, "qwen3"), ("greeting", GGUF_STRING, "héllo"),
                          ("empty", GGUF_STRING, "")], [])
    with gguf.GgufFile.from_bytes(data) as g:
        assert g.metadata_get("general.architecture") == "qwen3"
        assert g.metadata_get("greeting") == "héllo"
        assert g.metadata_get("empty") == ""
        assert g.as_u64("greeting") is None


def test_typed_arrays():                                 # value.rs:121-140
    meta = [("arr.u32", GGUF_ARRAY, (GGUF_U32, [10, 20, 30])),
            ("arr.f32", GGUF_ARRAY, (GGUF_F32, [0.5, -1.5])),
            ("arr.empty_u32", GGUF_ARRAY, (GGUF_U32, [])),
            ("arr.empty_str", GGUF_ARRAY, (GGUF_STRING, [])),
            ("tokenizer.ggml.tokens", GGUF_ARRAY, (GGUF_STRING, ["<pad>", "a", "", "ĠThe", "日本"])),
            ("arr.bool", GGUF_ARRAY, (GGUF_BOOL, [1, 0, 1])),
            ("arr.nested", GGUF_ARRAY, (GGUF_ARRAY, [(GGUF_U8, [1, 2]), (GGUF_U8, [3])])),
            ("after", GGUF_U32, 77)]
    data, _ = write_gguf(meta, [])
    with gguf.GgufFile.from_bytes(data) as g:
        a = g.metadata_get("arr.u32")
        assert a.dtype == np.uint32 and a.tolist() == [10, 20, 30] and a[1] == 20
        assert g.metadata_get("arr.f32").tolist() == [0.5, -1.5]
        # an empty array keeps its element type (value.rs:7-8)
        assert g.metadata_get("arr.empty_u32").dtype == np.uint32 and g.metadata_get("arr.empty_u32").size == 0
        assert g.metadata_get("arr.empty_str") == []
        assert g.metadata_get("tokenizer.ggml.tokens") == ["<pad>", "a", "", "ĠThe", "日本"]
        assert g.metadata_get("arr.bool").tolist() == [True, False, True]
        with pytest.raises(rein.ReinError):
            g.metadata_get("arr.nested")                  # walked and bounds-checked at open, not decoded
        assert g.metadata_get("after") == 77              # the walk over every array above ended where it should
        assert g.as_u64("arr.u32") is None


def test_repeated_key_resolves_to_the_last_entry():      # HashMap::insert in mod.rs:137
    data, _ = write_gguf([("k", GGUF_U32, 1), ("k", GGUF_U32, 2)], [])
    with gguf.GgufFile.from_bytes(data) as g:
        assert g.header["metadata_kv_count"] == 2 and g.metadata_get("k") == 2


def test_truncation_is_reported():                       # reader.rs:121-128
    assert "truncated read: needed 4 bytes at offset 0, only 3 available" in parse_error(b"GGU")
    assert "truncated read" in parse_error(b"")
    data, _ = write_gguf([("a", GGUF_STRING, "hello")], [])
    for cut in range(4, 24 + 8 + 1 + 4 + 8 + 5):
        assert "truncated read" in parse_error(data[:cut]), cut
    # a string length beyond the file, an array count beyond the file
    bad = b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + struct.pack("<Q", 2 ** 62) + b"ab"
    assert "truncated read" in parse_error(bad)
    bad = b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + gguf_string("k") + struct.pack("<IIQ", GGUF_ARRAY, GGUF_U64, 2 ** 61)
    assert "truncated read" in parse_error(bad)
    bad = b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + gguf_string("k") + struct.pack("<IIQ", GGUF_ARRAY, GGUF_STRING, 2 ** 61)
    assert "truncated read" in parse_error(bad)
    # more tensors / entries announced than present
    assert "truncated read" in parse_error(b"GGUF" + struct.pack("<IQQ", 3, 2 ** 60, 0))
    assert "truncated read" in parse_error(b"GGUF" + struct.pack("<IQQ", 3, 0, 2 ** 60))


def test_bad_magic_version_and_types():                  # error.rs:8-24
    data, _ = write_gguf([], [], magic=b"GGML")
    assert "bad magic: got 0x4c4d4747" in parse_error(data)
    for v in (1, 2, 4):
        data, _ = write_gguf([], [], version=v)
        assert f"unsupported GGUF version: {v} (only v3 is supported)" in parse_error(data)
    bad = b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + gguf_string("k") + struct.pack("<I", 13) + b"\0" * 16
    assert "unknown GGUF metadata value type: 13" in parse_error(bad)
    bad = b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + gguf_string("k") + struct.pack("<IIQ", GGUF_ARRAY, 99, 0)
    assert "unknown GGUF metadata value type: 99" in parse_error(bad)
    for ty in (4, 5, 16, 22, 24, 31, 1000):               # ids the reference's table skips (types.rs:39-58)
        data, _ = write_gguf([], [("t", [32], ty, b"\0" * 64)])
        assert f"unknown ggml tensor type: {ty}" in parse_error(data)


def test_invalid_utf8_is_rejected():                     # reader.rs:76-79
    for raw in (b"\xff", b"\xc3", b"\xc0\x80", b"\xed\xa0\x80", b"\xf4\x90\x80\x80", b"a\x80"):
        bad = b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + gguf_string(raw) + struct.pack("<II", GGUF_U32, 1)
        assert "invalid UTF-8 in GGUF string at offset 24" in parse_error(bad), raw
    # names cross the C ABI NUL-terminated, so a NUL inside one is refused; values may hold one
    bad = b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + gguf_string(b"a\0b") + struct.pack("<II", GGUF_U32, 1)
    assert "NUL byte" in parse_error(bad)
    data, _ = write_gguf([("k", GGUF_STRING, "a\0b")], [])
    with gguf.GgufFile.from_bytes(data) as g:
        assert g.metadata_get("k") == "a\0b"
    data, _ = write_gguf([("k", GGUF_STRING, "é€\U0001F600")], [])
    with gguf.GgufFile.from_bytes(data) as g:
        assert g.metadata_get("k") == "é€\U0001F600"


def test_tensor_directory_and_byte_sizes():              # tensor_info.rs:69-82, types.rs:140-150
    payloads = {"q4k": (12, [256, 4], 576), "q5k": (13, [256, 2], 352), "q6k": (14, [512], 420), "q8_0": (8, [64, 3], 204),
                "q8k": (15, [256], 292), "f32": (0, [3, 5, 2], 120), "f16": (1, [7], 14), "bf16": (30, [4, 4, 2, 2], 128),
                "q4_0": (2, [32, 2], 36), "q3k": (11, [256], 110), "iq4xs": (23, [256], 136), "iq4nl": (20, [32], 18),
                "q5_1": (7, [32], 24), "iq3s": (21, [256], 110), "q2k": (10, [256], 84), "q4_1": (3, [32], 20),
                "q5_0": (6, [32], 22), "q8_1": (9, [32], 36)}
    rng = np.random.default_rng(0)
    tensors = [(n, dims, ty, rng.integers(0, 256, size, dtype=np.uint8).tobytes()) for n, (ty, dims, size) in payloads.items()]
    data, offs = write_gguf([("general.architecture", GGUF_STRING, "test")], tensors)
    with gguf.GgufFile.from_bytes(data) as g:
        assert g.header["tensor_count"] == len(tensors) and g.data_section_offset % 32 == 0
        assert [t.name for t in g.tensors] == list(payloads)
        for name, dims, ty, payload in tensors:
            t = g.tensor(name)
            assert t.ggml_type == ty and t.shape == tuple(dims) and t.offset == offs[name]
            assert t.byte_size == payloads[name][2] == len(payload)
            assert t.n_elements == int(np.prod(dims))
            assert g.tensor_data(name).tobytes() == payload
            assert t.offset % 32 == 0
        assert g.tensor("q4k").byte_size == 576            # the reference's own example


def test_bad_shapes_and_bounds():                        # tensor_info.rs:84-99, mod.rs:160-172
    data, _ = write_gguf([], [("bad", [100], 12, b"\0" * 144)])
    assert "tensor `bad` element count 100 is not a multiple of block size 256" in parse_error(data)
    for dims in ([], [1, 1, 1, 1, 1]):
        data, _ = write_gguf([], [("t", dims, 0, b"\0" * 4)])
        assert f"tensor `t` has invalid shape (n_dims={len(dims)}, max 4 supported)" in parse_error(data)
    data, _ = write_gguf([], [("t", [256, 4], 12, b"\0" * 576)])
    with gguf.GgufFile.from_bytes(data):
        pass
    assert "tensor `t` data extends past file end" in parse_error(data[:-1])
    msg = parse_error(data[:-1])
    assert "size=576" in msg and f"file_len={len(data) - 1}" in msg
    # an offset near 2^64 must not wrap round to "in bounds"
    raw = bytearray(data)
    at = raw.index(struct.pack("<IQ", 12, 0))
    raw[at + 4:at + 12] = struct.pack("<Q", 2 ** 64 - 64)
    assert "extends past file end" in parse_error(bytes(raw))
    data, _ = write_gguf([], [("t", [2 ** 33, 2 ** 33], 0, b"")])
    assert "overflows" in parse_error(data)
    # zero-sized tensors are legal
    data, _ = write_gguf([], [("z", [0, 4], 12, b""), ("y", [256], 12, b"\x01" * 144)])
    with gguf.GgufFile.from_bytes(data) as g:
        assert g.tensor("z").byte_size == 0 and g.tensor_data("z").size == 0
        assert g.tensor_data("y").tobytes() == b"\x01" * 144


@pytest.mark.parametrize("align", [None, 1, 0, 8, 64, 4096])
def test_general_alignment_places_the_data_section(align):   # mod.rs:152-156
    meta = [("pad", GGUF_STRING, "x" * 5)]
    if align is not None:
        meta.append(("general.alignment", GGUF_U32, align))
    payload = bytes(range(144))
    data, _ = write_gguf(meta, [("t", [256], 12, payload), ("u", [32], 8, b"\x07" * 34)])
    with gguf.GgufFile.from_bytes(data) as g:
        a = 32 if align is None else align
        assert g.alignment == a
        if a > 1:
            assert g.data_section_offset % a == 0
        assert g.tensor_data("t").tobytes() == payload and g.tensor_data("u").tobytes() == b"\x07" * 34
    # a signed alignment is accepted (as_u64), a string one falls back to 32
    data, _ = write_gguf([("general.alignment", GGUF_I32, 64)], [("t", [256], 12, payload)])
    with gguf.GgufFile.from_bytes(data) as g:
        assert g.alignment == 64 and g.tensor_data("t").tobytes() == payload
    data, _ = write_gguf([("general.alignment", GGUF_STRING, "64")], [("t", [256], 12, payload)])
    with gguf.GgufFile.from_bytes(data) as g:
        assert g.alignment == 32 and g.tensor_data("t").tobytes() == payload


def test_open_maps_a_file(tmp_path):
    raw = random_raw_weights(rein.Q4_K, 512, 6, seed=1)
    data, _ = write_gguf([("general.architecture", GGUF_STRING, "qwen35")], [("blk.0.ffn_up.weight", [512, 6], 12, raw.tobytes())])
    p = tmp_path / "m.gguf"
    p.write_bytes(data)
    with gguf.GgufFile.open(p) as g:
        assert g.metadata_get("general.architecture") == "qwen35"
        assert np.array_equal(g.tensor_data("blk.0.ffn_up.weight"), raw)
    with pytest.raises(rein.ReinError) as e:
        gguf.GgufFile.open(tmp_path / "absent.gguf")
    assert e.value.code == -7 and "io error" in str(e.value)
    (tmp_path / "empty.gguf").write_bytes(b"")
    with pytest.raises(rein.ReinError) as e:
        gguf.GgufFile.open(tmp_path / "empty.gguf")
    assert "truncated read" in str(e.value)


@pytest.mark.parametrize("fmt", [rein.Q4_0, rein.Q8_0, rein.Q4_K, rein.Q5_K, rein.Q6_K, rein.IQ4_XS])
def test_load_for_matvec_is_the_oracle_repack_of_the_tensor_bytes(fmt):     # qwen35.rs:235-245
    in_dim, out_dim = 768, 40
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=fmt)
    other = random_raw_weights(rein.Q8_0, 64, 2, seed=9)
    data, _ = write_gguf([], [("first", [64, 2], 8, other.tobytes()), ("w", [in_dim, out_dim], fmt, raw.tobytes())])
    with gguf.GgufFile.from_bytes(data) as g:
        slab, label, dims = g.load_for_matvec("w")
    assert label == fmt and dims == {"in_dim": in_dim, "out_dim": out_dim, "n_expert": 1,
                                     "bytes_per_expert": quant.repacked_len(fmt, in_dim, out_dim)}
    assert np.array_equal(slab, orc.repack_for_matvec(fmt, raw, in_dim, out_dim))


@pytest.mark.parametrize("fmt", [rein.Q4_K, rein.Q5_K, rein.Q6_K, rein.Q8_0])
def test_load_expert_tensor_repacks_per_expert(fmt):     # qwen35.rs:397-431
    in_dim, out_dim, n_expert = 512, 24, 5
    raws = [random_raw_weights(fmt, in_dim, out_dim, seed=fmt * 10 + e) for e in range(n_expert)]
    data, _ = write_gguf([], [("blk.3.ffn_gate_exps.weight", [in_dim, out_dim, n_expert], fmt, b"".join(r.tobytes() for r in raws))])
    with gguf.GgufFile.from_bytes(data) as g:
        slab, label, dims = g.load_for_matvec("blk.3.ffn_gate_exps.weight")
    per = quant.repacked_len(fmt, in_dim, out_dim)
    assert label == fmt and dims["n_expert"] == n_expert and dims["bytes_per_expert"] == per and slab.size == per * n_expert
    for e in range(n_expert):
        assert np.array_equal(slab[e * per:(e + 1) * per], orc.repack_for_matvec(fmt, raws[e], in_dim, out_dim)), e


def test_load_relabelled_types_and_errors():
    rng = np.random.default_rng(4)
    bf = (rng.standard_normal(64 * 8).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    data, _ = write_gguf([], [("bf", [64, 8], 30, bf.tobytes()),
                              ("f32", [64, 8], 0, b"\0" * 2048),
                              ("vec", [256], 12, b"\0" * 144),
                              ("odd", [256, 3, 2], 12, b"\0" * 144 * 6),
                              ("q5_1", [32, 4], 7, b"\0" * 96)])
    with gguf.GgufFile.from_bytes(data) as g:
        slab, label, dims = g.load_for_matvec("bf")
        want, want_label = quant.ingest_for_matvec(quant.GGML_BF16, bf.view(np.uint8), 64, 8)
        assert label == want_label == rein.Q8_0 and np.array_equal(slab, want)
        for name, code in (("f32", -2), ("q5_1", -2), ("vec", -3), ("odd", -3), ("absent", -8)):
            with pytest.raises(rein.ReinError) as e:
                g.load_for_matvec(name)
            assert e.value.code == code, name


def test_mutated_directories_never_escape_the_mapping():
    """Seeded byte / length mutations of a valid directory: every parse either fails with a
    container error or yields tensors and values that lie inside the buffer."""
    import random
    rng = random.Random(7)
    meta = [("general.architecture", GGUF_STRING, "qwen35"), ("a", GGUF_U32, 7), ("general.alignment", GGUF_U32, 32),
            ("arr", GGUF_ARRAY, (GGUF_U32, [1, 2, 3])), ("toks", GGUF_ARRAY, (GGUF_STRING, ["a", "bc", "日本"])),
            ("nest", GGUF_ARRAY, (GGUF_ARRAY, [(GGUF_U8, [1, 2]), (GGUF_STRING, ["x"])]))]
    tens = [("w", [256, 4], 12, bytes(576)), ("e", [256, 8, 2], 14, bytes(210 * 16))]
    base, _ = write_gguf(meta, tens)
    directory = len(base) - 576 - 210 * 16 - 32
    n_ok = 0
    for _ in range(1500):
        b = bytearray(base)
        for _ in range(rng.randint(1, 3)):
            pos = rng.randrange(directory)
            if rng.random() < 0.5:
                b[pos] = rng.choice([0, 1, 8, 9, 12, 0x7F, 0x80, 0xFF, rng.randrange(256)])
            else:
                b[pos:pos + 8] = struct.pack("<Q", rng.choice([0, 1, 2 ** 64 - 1, 2 ** 63, 2 ** 32, len(b), 2 ** 61]))
        try:
            g = gguf.GgufFile.from_bytes(bytes(b))
        except rein.ReinError as e:
            assert e.code == -7
            continue
        n_ok += 1
        for t in g.tensors:
            assert g.data_section_offset + t.offset + t.byte_size <= len(b)
            if [u.name for u in g.tensors].count(t.name) == 1:      # a repeated name resolves to its last entry
                assert g.tensor_data(t.name).size == t.byte_size
        for k, vt in g.metadata_keys():
            if vt != GGUF_ARRAY or k != "nest":
                try:
                    g.metadata_get(k)
                except rein.ReinError as e:
                    assert e.code == -2                   # a mutation made another array nested
        g.close()
    assert n_ok > 20
