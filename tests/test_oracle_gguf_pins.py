"""Pins of the GGUF reader oracle (oracle/gguf_oracle.py): the reference's own test cases
(crates/runtime/src/gguf.rs:1118-1480) rebuilt by an independent writer (tests/gguf_builder.py)."""
import struct

import pytest

from gguf_builder import build, entry, gguf_string, raw_entry
from oracle import gguf_oracle as go

QV = [entry("general.quantization_version", "u32", 2)]


def tensor(name="weight", dimensions=(256,), format=10, offset=0, nbytes=84):
    return dict(name=name, dimensions=list(dimensions), format=format, offset=offset, bytes=nbytes)


def test_parses_f32_and_every_supported_k_quant_shape():  # gguf.rs:1118-1176
    tensors = [tensor("dense", (3, 2), 0, 0, 24), tensor("q2", (256, 2), 10, 32, 168),
               tensor("q3", (256, 2), 11, 224, 220), tensor("q4", (512, 2), 12, 448, 576),
               tensor("q5", (256, 2), 13, 1024, 352), tensor("q6", (256, 2), 14, 1376, 420)]
    data, start = build(QV, tensors)
    parsed = go.parse(data)
    assert parsed["architecture"] == "test"
    shapes = [t["physical_shape"] for t in parsed["tensors"]]
    assert parsed["tensors"][0]["logical_shape"] == (2, 3)
    assert shapes == [(2, 3), (2, 84), (2, 110), (2, 288), (2, 176), (2, 210)]
    assert [t["data_offset"] for t in parsed["tensors"]] == [start + t["offset"] for t in tensors]
    assert [t["byte_len"] for t in parsed["tensors"]] == [t["bytes"] for t in tensors]


def test_parses_every_metadata_scalar_and_homogeneous_array_type():  # gguf.rs:1178-1226
    entries = [entry("u8", "u8", 7), entry("i8", "i8", -7), entry("u16", "u16", 17), entry("i16", "i16", -17),
               entry("u32", "u32", 27), entry("i32", "i32", -27), entry("f32", "f32", 1.5), entry("bool", "bool", 1),
               entry("string", "string", "value"), entry("u64", "u64", 37), entry("i64", "i64", -37),
               entry("f64", "f64", 2.5), entry("a_u8", "u8", [1, 2], True), entry("a_i8", "i8", [-1, 2], True),
               entry("a_u16", "u16", [3], True), entry("a_i16", "i16", [-3], True), entry("a_u32", "u32", [4], True),
               entry("a_i32", "i32", [-4], True), entry("a_f32", "f32", [3.5], True),
               entry("a_bool", "bool", [0, 1], True), entry("a_string", "string", ["a", "b"], True),
               entry("a_u64", "u64", [5], True), entry("a_i64", "i64", [-5], True), entry("a_f64", "f64", [4.5], True)]
    parsed = go.parse(build(entries, [tensor("dense", (1,), 0, 0, 4)])[0])
    assert len(parsed["metadata"]) == len(entries) + 2
    assert parsed["metadata"][-1] == ("a_f64", "f64", True, [4.5])
    values = {key: (kind, is_array, value) for key, kind, is_array, value in parsed["metadata"]}
    assert values["i8"] == ("i8", False, -7) and values["bool"] == ("bool", False, True)
    assert values["a_i8"] == ("i8", True, [-1, 2]) and values["a_string"] == ("string", True, ["a", "b"])
    assert values["a_bool"] == ("bool", True, [False, True]) and values["f32"] == ("f32", False, 1.5)


def rejected(data, fragment=None):
    with pytest.raises(go.GgufInvalid) as info:
        go.parse(data)
    assert str(info.value).startswith("gguf: ")
    if fragment:
        assert fragment in str(info.value), str(info.value)


def test_rejects_malformed_headers_catalogs_ranges_and_metadata():  # gguf.rs:1228-1302
    valid, _ = build(QV, [tensor()])
    go.parse(valid)
    rejected(b"X" + valid[1:], "invalid magic")
    rejected(valid[:4] + struct.pack("<I", 2) + valid[8:], "unsupported version 2; expected version 3")
    rejected(build([entry("general.architecture", "string", "other")], [tensor()])[0],
             'duplicate metadata key "general.architecture"')
    rejected(build([entry("unsafe", "u64", 2**64 - 1)], [tensor()])[0], "outside the JavaScript safe integer range")
    rejected(build(QV, [tensor()], 3)[0], "general.alignment must be a positive power of two, got 3")
    rejected(build(QV, [tensor(), tensor()])[0], 'duplicate tensor name "weight"')
    rejected(build(QV, [tensor(), tensor("other", offset=32)])[0], 'tensor ranges for "weight" and "other" overlap')
    rejected(build(QV, [tensor(dimensions=(255,))])[0], "least-major dimension 255 is not divisible by 256 for Q2_K")
    rejected(build(QV, [tensor(format=1)])[0], "unsupported GGML tensor type code 1")
    rejected(build(QV, [tensor(dimensions=(0,))])[0], 'tensor "weight" has invalid dimension 0')
    rejected(valid[:-1], "exceeds file size")


def test_requires_quantization_version_two_for_k_quants():  # gguf.rs:1304-1349
    rejected(build([], [tensor()])[0], "missing general.quantization_version")
    rejected(build([entry("general.quantization_version", "u64", 2)], [tensor()])[0], "must be u32")
    rejected(build([entry("general.quantization_version", "u32", 1)], [tensor()])[0], "expected 2")
    go.parse(build(QV, [tensor()])[0])
    go.parse(build([], [tensor("weight", (1,), 0, 0, 4)])[0])  # allows_f32_without_quantization_version


def test_rejects_counts_and_lengths_over_resource_limits_before_allocation():  # gguf.rs:1363-1388
    head = b"GGUF" + struct.pack("<I", 3)
    rejected(head + struct.pack("<QQ", 0, go.MAX_METADATA_COUNT + 1), "resource limit")
    rejected(head + struct.pack("<QQQ", 0, 1, go.MAX_METADATA_KEY_BYTES + 1) + bytes(13), "resource limit")
    rejected(head + struct.pack("<QQ", 0, 3), "metadata count 3 exceeds the remaining file")


def test_validates_sparse_large_file_ranges_without_reading_payloads():  # gguf.rs:1411-1452
    header, start = build([], [tensor("sparse", (1,), 0, 1 << 32, 4)], with_body=False)
    parsed = go.parse(header, file_len=start + (1 << 32) + 4)
    assert parsed["tensors"][0]["data_offset"] == start + (1 << 32)
    rejected(header, "exceeds file size")


def test_other_rules_of_the_parser():
    rejected(build([], [tensor("t", (1,), 0, 0, 4)], architecture=None)[0], "missing general.architecture metadata")
    rejected(build([], [tensor("t", (1,), 0, 0, 4)], architecture="")[0], "must not be empty")
    rejected(build([raw_entry("general.architecture", 4, struct.pack("<I", 1))], [], architecture=None)[0],
             "general.architecture metadata must be a string")
    rejected(build([raw_entry("nested", 9, struct.pack("<IQ", 9, 0))], [])[0], "nested metadata arrays")
    rejected(build([raw_entry("odd", 13, b"")], [])[0], "unsupported metadata value type 13")
    rejected(build([raw_entry("flag", 7, b"\x02")], [])[0], "invalid boolean metadata byte 2")
    rejected(build([raw_entry("text", 8, gguf_string(b"\xff\xfe"))], [])[0], "metadata string is not valid UTF-8")
    rejected(build([], [tensor("t", (1, 1, 1, 1, 1), 0, 0, 4)])[0], "rank must be in 1..=4, got 5")
    rejected(build([], [tensor("t", (1,), 0, 16, 4)])[0], 'tensor "t" offset 16 is not aligned to 32')
    rejected(build([], [tensor("x" * 65, (1,), 0, 0, 4)])[0], "tensor name count 65 exceeds the resource limit 64")
    # the default alignment is 32 when the key is absent
    data, start = build([], [tensor("t", (1,), 0, 32, 4)], write_alignment=False)
    assert go.parse(data)["tensors"][0]["data_offset"] == start + 32


def test_legacy_block_formats_are_accepted():
    # this build's extension (type codes 2 and 8); the reference rejects them
    data, _ = build(QV, [tensor("a", (64, 3), 2, 0, 3 * 2 * 18), tensor("b", (32, 5), 8, 128, 5 * 34)])
    shapes = [t["physical_shape"] for t in go.parse(data)["tensors"]]
    assert shapes == [(3, 36), (5, 34)]
    rejected(build(QV, [tensor("a", (48,), 2, 0, 27)])[0], "least-major dimension 48 is not divisible by 32 for Q4_0")
