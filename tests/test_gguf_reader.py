"""The GGUF reader of the library (C ABI, host code) against the reference's test cases and against
the Python oracle on built, random and mutated files. No GPU needed."""
import os
import struct

import numpy as np
import pytest

from gguf_builder import build, entry, gguf_string, raw_entry
from oracle import gguf_oracle as go

QV = [entry("general.quantization_version", "u32", 2)]


def tensor(name="weight", dimensions=(256,), format=10, offset=0, nbytes=84):
    return dict(name=name, dimensions=list(dimensions), format=format, offset=offset, bytes=nbytes)


@pytest.fixture
def write(tmp_path):
    counter = [0]

    def _write(data: bytes, length=None) -> str:
        counter[0] += 1
        path = tmp_path / f"case{counter[0]}.gguf"
        with open(path, "wb") as handle:
            handle.write(data)
            if length is not None:
                handle.truncate(length)  # sparse
        return str(path)
    return _write


def as_oracle(parsed):
    """The library's view of a file in the shape oracle.parse returns."""
    return dict(architecture=parsed.architecture,
                metadata=[(key, v.kind, v.is_array, v.value) for key, v in parsed.metadata],
                tensors=[dict(name=t.name, format=t.format, logical_shape=t.logical_shape,
                              physical_shape=t.physical_shape, data_offset=t.data_offset, byte_len=t.byte_len)
                         for t in parsed.tensors])


def same_outcome(et, write, data, length=None):
    """Both accept and agree on everything, or both reject with the same message."""
    path = write(data, length)
    try:
        want = go.parse(data, file_len=length)
    except go.GgufInvalid as error:
        with pytest.raises(et.GgufParseError) as info:
            et.GgufFile.open(path)
        assert str(info.value) == str(error)
        return None
    with et.GgufFile.open(path) as parsed:
        assert as_oracle(parsed) == want
    return want


def test_reference_cases(et, write):
    # gguf.rs:1118-1176: f32 and every K-quant
    tensors = [tensor("dense", (3, 2), 0, 0, 24), tensor("q2", (256, 2), 10, 32, 168),
               tensor("q3", (256, 2), 11, 224, 220), tensor("q4", (512, 2), 12, 448, 576),
               tensor("q5", (256, 2), 13, 1024, 352), tensor("q6", (256, 2), 14, 1376, 420)]
    data, _ = build(QV, tensors)
    with et.GgufFile.open(write(data)) as parsed:
        assert parsed.architecture == "test"
        assert parsed.tensors[0].logical_shape == (2, 3)
        assert [t.physical_shape for t in parsed.tensors] == [(2, 3), (2, 84), (2, 110), (2, 288), (2, 176), (2, 210)]
        assert [t.format_name for t in parsed.tensors] == ["F32", "Q2_K", "Q3_K", "Q4_K", "Q5_K", "Q6_K"]
    same_outcome(et, write, data)
    # gguf.rs:1178-1226: every metadata type
    entries = [entry("u8", "u8", 7), entry("i8", "i8", -7), entry("u16", "u16", 17), entry("i16", "i16", -17),
               entry("u32", "u32", 27), entry("i32", "i32", -27), entry("f32", "f32", 1.5), entry("bool", "bool", 1),
               entry("string", "string", "value"), entry("u64", "u64", 37), entry("i64", "i64", -37),
               entry("f64", "f64", 2.5), entry("a_u8", "u8", [1, 2], True), entry("a_i8", "i8", [-1, 2], True),
               entry("a_u16", "u16", [3], True), entry("a_i16", "i16", [-3], True), entry("a_u32", "u32", [4], True),
               entry("a_i32", "i32", [-4], True), entry("a_f32", "f32", [3.5], True),
               entry("a_bool", "bool", [0, 1], True), entry("a_string", "string", ["a", "b"], True),
               entry("a_u64", "u64", [5], True), entry("a_i64", "i64", [-5], True), entry("a_f64", "f64", [4.5], True)]
    data, _ = build(entries, [tensor("dense", (1,), 0, 0, 4)])
    with et.GgufFile.open(write(data)) as parsed:
        assert len(parsed.metadata) == len(entries) + 2
        assert parsed.metadata[-1][0] == "a_f64" and parsed.metadata[-1][1].value == [4.5]
        assert parsed.get("a_string").value == ["a", "b"] and parsed.get("i64").value == -37
    same_outcome(et, write, data)


def test_reference_rejections(et, write):
    # gguf.rs:1228-1388
    valid, _ = build(QV, [tensor()])
    cases = [b"X" + valid[1:], valid[:4] + struct.pack("<I", 2) + valid[8:],
             build([entry("general.architecture", "string", "other")], [tensor()])[0],
             build([entry("unsafe", "u64", 2**64 - 1)], [tensor()])[0], build(QV, [tensor()], 3)[0],
             build(QV, [tensor(), tensor()])[0], build(QV, [tensor(), tensor("other", offset=32)])[0],
             build(QV, [tensor(dimensions=(255,))])[0], build(QV, [tensor(format=1)])[0],
             build(QV, [tensor(dimensions=(0,))])[0], valid[:-1],
             build([], [tensor()])[0], build([entry("general.quantization_version", "u64", 2)], [tensor()])[0],
             build([entry("general.quantization_version", "u32", 1)], [tensor()])[0],
             b"GGUF" + struct.pack("<IQQ", 3, 0, go.MAX_METADATA_COUNT + 1),
             b"GGUF" + struct.pack("<IQQQ", 3, 0, 1, go.MAX_METADATA_KEY_BYTES + 1) + bytes(13),
             build([], [tensor("t", (1,), 0, 0, 4)], architecture=None)[0],
             build([raw_entry("nested", 9, struct.pack("<IQ", 9, 0))], [])[0],
             build([raw_entry("odd", 13, b"")], [])[0], build([raw_entry("flag", 7, b"\x02")], [])[0],
             build([raw_entry("text", 8, gguf_string(b"\xff\xfe"))], [])[0],
             build([raw_entry("text", 8, gguf_string(b"\xed\xa0\x80"))], [])[0],  # a UTF-16 surrogate
             build([], [tensor("t", (1, 1, 1, 1, 1), 0, 0, 4)])[0], build([], [tensor("t", (1,), 0, 16, 4)])[0],
             build([], [tensor("x" * 65, (1,), 0, 0, 4)])[0], build([entry("i", "i64", -(2**60))], [])[0],
             build(QV, [tensor("a", (48,), 2, 0, 27)])[0], b"", b"GGUF", valid[:40],
             build(QV, [tensor("a\0b\x01\x7f\u0085\"\\", (256,), 10, 0, 84)] * 2)[0]]
    for data in cases:
        assert same_outcome(et, write, data) is None
    for data in (valid, build([], [tensor("weight", (1,), 0, 0, 4)])[0],
                 build(QV, [tensor("a", (64, 3), 2, 0, 108), tensor("b", (32, 5), 8, 128, 170)])[0],
                 build(QV + [entry("k\0ey", "string", "v\0alue")], [tensor("a\0b", (256,), 10, 0, 84)])[0]):
        assert same_outcome(et, write, data) is not None


def test_sparse_file_and_cancellation(et, write):
    # gguf.rs:1411-1452: ranges are validated against the file size without reading payloads
    header, start = build([], [tensor("sparse", (1,), 0, 1 << 32, 4)], with_body=False)
    want = same_outcome(et, write, header, length=start + (1 << 32) + 4)
    assert want["tensors"][0]["data_offset"] == start + (1 << 32)
    # gguf.rs:1390-1409: a cancelled parse stops before any header I/O
    flag = et.CancellationFlag()
    flag.cancel()
    with pytest.raises(et.Cancelled) as info:
        et.GgufFile.open(write(b"not a gguf"), flag)
    assert str(info.value) == "gguf: operation aborted"
    with pytest.raises(et.GgufParseError, match="gguf: I/O failed: No such file or directory"):
        et.GgufFile.open(os.path.join(os.path.dirname(write(b"")), "missing.gguf"))


def test_fills_a_caller_owned_tensor_destination_exactly(et, write):
    # gguf.rs:1454-1479
    payload = struct.pack("<ff", 1.5, -2.25)
    data, _ = build([], [tensor("dense", (2,), 0, 0, 8)], payloads={"dense": payload})
    with et.GgufFile.open(write(data)) as parsed:
        assert parsed.read_tensor("dense").tobytes() == payload
        with pytest.raises(et.GgufParseError, match='gguf: tensor "dense" requires 8 destination bytes, got 7'):
            parsed.read_tensor("dense", np.zeros(7, np.uint8))
        flag = et.CancellationFlag()
        flag.cancel()
        with pytest.raises(et.Cancelled):
            parsed.read_tensor("dense", cancelled=flag)


def random_file(rng):
    kinds = ["u8", "i8", "u16", "i16", "u32", "i32", "f32", "bool", "string", "u64", "i64", "f64"]

    def value(kind):
        if kind == "string":
            return "".join(rng.choice(list("abcé漢 _.")) for _ in range(rng.integers(0, 9)))
        if kind == "bool":
            return int(rng.integers(0, 2))
        if kind in ("f32", "f64"):
            return float(np.float32(rng.standard_normal()))
        bits = int(kind[1:])
        if kind == "u64":
            return int(rng.integers(0, 2**53))
        if kind == "i64":
            return int(rng.integers(-2**53 + 1, 2**53))
        return int(rng.integers(0, 2**bits)) if kind[0] == "u" else int(rng.integers(-2**(bits - 1), 2**(bits - 1)))

    entries = [entry("general.quantization_version", "u32", 2)]
    for i in range(rng.integers(0, 12)):
        kind = kinds[rng.integers(0, len(kinds))]
        if rng.integers(0, 3) == 0:
            entries.append(entry(f"key.{i}", kind, [value(kind) for _ in range(rng.integers(0, 6))], True))
        else:
            entries.append(entry(f"key.{i}", kind, value(kind)))
    alignment = int(2 ** rng.integers(0, 8))
    tensors, payloads, cursor = [], {}, 0
    for i in range(rng.integers(0, 9)):
        code = int(rng.choice([0, 2, 8, 10, 11, 12, 13, 14]))
        _, block_values, block_bytes = go.FORMATS[code]
        rank = int(rng.integers(1, 5))
        dims = [int(rng.integers(1, 4)) for _ in range(rank)]
        if block_bytes:
            dims[0] = block_values * int(rng.integers(1, 4))
            nbytes = dims[0] // block_values * block_bytes * int(np.prod(dims[1:], dtype=np.int64))
        else:
            nbytes = 4 * int(np.prod(dims, dtype=np.int64))
        cursor = -(-cursor // alignment) * alignment + alignment * int(rng.integers(0, 3))
        tensors.append(dict(name=f"t{i}", dimensions=dims, format=code, offset=cursor, bytes=nbytes))
        payloads[f"t{i}"] = rng.integers(0, 256, nbytes, dtype=np.uint8).tobytes()
        cursor += nbytes
    order = rng.permutation(len(tensors))
    return build(entries, [tensors[i] for i in order], alignment, payloads=payloads)[0], payloads


def test_random_files_and_their_mutations(et, write):
    rng = np.random.default_rng(2024)
    accepted = rejected = 0
    for _ in range(60):
        data, payloads = random_file(rng)
        want = same_outcome(et, write, data)
        assert want is not None
        with et.GgufFile.open(write(data)) as parsed:
            for name, payload in payloads.items():
                assert parsed.read_tensor(name).tobytes() == payload
        # single-byte mutations of the header and truncations: the same verdict and message
        header_end = min((t["data_offset"] for t in want["tensors"]), default=len(data))
        for _ in range(12):
            mutated = bytearray(data)
            mutated[int(rng.integers(0, max(header_end, 1)))] = int(rng.integers(0, 256))
            outcome = same_outcome(et, write, bytes(mutated))
            accepted += outcome is not None
            rejected += outcome is None
        same_outcome(et, write, data[:int(rng.integers(0, len(data) + 1))])
    assert accepted > 50 and rejected > 100  # both verdicts were exercised
