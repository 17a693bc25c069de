"""CPU oracle for the GGUF v3 header reader: a plain-Python restatement of ``parse_gguf``
(crates/runtime/src/gguf.rs:682-957) over a bytes object. TEST INFRASTRUCTURE ONLY.

Pin status (tests/test_oracle_gguf_pins.py): the reference's own test cases (gguf.rs:1118-1480) rebuilt
byte for byte by an independent writer - the six tensor formats' physical shapes, every metadata
scalar and array type, each malformed file of ``rejects_malformed_headers_catalogs_ranges_and_metadata``,
the quantization-version rules and their message fragments, the resource limits, the sparse
large-offset file. GGML type codes 2 (Q4_0) and 8 (Q8_0) are this build's extension: PARITY UNPINNED
by the reference (it rejects them); they follow the public ggml block sizes (18 and 34 bytes per 32).
"""
from __future__ import annotations

import struct

VERSION = 3
QUANTIZATION_VERSION = 2
DEFAULT_ALIGNMENT = 32
SAFE_INTEGER = 9_007_199_254_740_991
MAX_HEADER_BYTES = 64 * 1024 * 1024
MAX_METADATA_COUNT = 4096
MAX_TENSOR_COUNT = 65536
MAX_METADATA_KEY_BYTES = 65535
MAX_TENSOR_NAME_BYTES = 64
MAX_METADATA_STRING_BYTES = 16 * 1024 * 1024
MAX_METADATA_ARRAY_ELEMENTS = 1048576

KINDS = ("u8", "i8", "u16", "i16", "u32", "i32", "f32", "bool", "string", "array", "u64", "i64", "f64")
FORMATS = {0: ("F32", 0, 0), 2: ("Q4_0", 32, 18), 8: ("Q8_0", 32, 34), 10: ("Q2_K", 256, 84),
           11: ("Q3_K", 256, 110), 12: ("Q4_K", 256, 144), 13: ("Q5_K", 256, 176), 14: ("Q6_K", 256, 210)}


class GgufInvalid(ValueError):
    """GgufParseError::Invalid; str() carries the reference's "gguf: " prefix."""

    def __init__(self, message):
        super().__init__("gguf: " + message)


def _quoted(text: str) -> str:
    """Rust's {:?} of a str: quotes and backslashes escaped, NUL, tab, CR and LF by name, the other
    control characters (C0, DEL, C1) as a braced hexadecimal escape."""
    out = []
    for ch in text:
        code = ord(ch)
        if ch == '"' or ch == "\\":
            out.append("\\" + ch)
        elif code == 0:
            out.append("\\0")
        elif ch == "\n":
            out.append("\\n")
        elif ch == "\t":
            out.append("\\t")
        elif ch == "\r":
            out.append("\\r")
        elif code < 0x20 or 0x7f <= code < 0xa0:
            out.append("\\u{%x}" % code)
        else:
            out.append(ch)
    return '"' + "".join(out) + '"'


class _Reader:  # HeaderReader, gguf.rs:356-507
    def __init__(self, data: bytes, file_len=None):
        self.data, self.position = data, 0
        self.file_len = len(data) if file_len is None else file_len

    def take(self, length: int) -> bytes:
        end = self.position + length
        if end > self.file_len:
            raise GgufInvalid("unexpected end of file in header")
        if end > MAX_HEADER_BYTES:
            raise GgufInvalid(f"header exceeds the {MAX_HEADER_BYTES}-byte resource limit")
        out = self.data[self.position:end]
        self.position = end
        return out

    def number(self, code: str):
        return struct.unpack("<" + code, self.take(struct.calcsize(code)))[0]

    def boolean(self) -> bool:
        value = self.number("B")
        if value > 1:
            raise GgufInvalid(f"invalid boolean metadata byte {value}")
        return value == 1

    def count(self, value: int, what: str, minimum_bytes: int, maximum: int) -> int:
        if value > maximum:
            raise GgufInvalid(f"{what} count {value} exceeds the resource limit {maximum}")
        remaining = max(min(self.file_len, MAX_HEADER_BYTES) - self.position, 0)
        if minimum_bytes > 0 and value > remaining // minimum_bytes:
            raise GgufInvalid(f"{what} count {value} exceeds the remaining file")
        return value

    def string(self, what: str, maximum: int) -> str:
        length = self.count(self.number("Q"), what, 1, maximum)
        try:
            return self.take(length).decode("utf-8")
        except UnicodeDecodeError:
            raise GgufInvalid(f"{what} is not valid UTF-8") from None


def _safe_u64(value, what):
    if value > SAFE_INTEGER:
        raise GgufInvalid(f"{what} value {value} is outside the JavaScript safe integer range")
    return value


def _safe_i64(value, what):
    if value < -SAFE_INTEGER or value > SAFE_INTEGER:
        raise GgufInvalid(f"{what} value {value} is outside the JavaScript safe integer range")
    return value


def _scalar(reader, kind, what_u64, what_i64, what_string):
    if kind == 7:
        return reader.boolean()
    if kind == 8:
        return reader.string(what_string, MAX_METADATA_STRING_BYTES)
    if kind == 10:
        return _safe_u64(reader.number("Q"), what_u64)
    if kind == 11:
        return _safe_i64(reader.number("q"), what_i64)
    return reader.number({0: "B", 1: "b", 2: "H", 3: "h", 4: "I", 5: "i", 6: "f", 12: "d"}[kind])


def _value(reader, kind):
    """-> (kind name of the value or of its elements, is_array, python value)"""
    if kind == 9:  # read_array, gguf.rs:537-615
        element = reader.number("I")
        if element == 9:
            raise GgufInvalid("nested metadata arrays are not supported by this parser")
        raw_count = reader.number("Q")
        minimum = {0: 1, 1: 1, 7: 1, 2: 2, 3: 2, 4: 4, 5: 4, 6: 4, 8: 8, 10: 8, 11: 8, 12: 8}.get(element)
        if minimum is None:
            raise GgufInvalid(f"unsupported metadata array element type {element}")
        count = reader.count(raw_count, "metadata array", minimum, MAX_METADATA_ARRAY_ELEMENTS)
        return KINDS[element], True, [_scalar(reader, element, "metadata u64 array", "metadata i64 array",
                                              "metadata array string") for _ in range(count)]
    if kind > 12:
        raise GgufInvalid(f"unsupported metadata value type {kind}")
    return KINDS[kind], False, _scalar(reader, kind, "metadata u64", "metadata i64", "metadata string")


def parse(data: bytes, file_len=None) -> dict:
    """{'architecture', 'metadata': [(key, kind, is_array, value)], 'tensors': [dict]}; raises GgufInvalid.
    ``file_len`` lets a header stand for a larger (sparse) file."""
    reader = _Reader(data, file_len)
    if reader.take(4) != b"GGUF":
        raise GgufInvalid("invalid magic")
    version = reader.number("I")
    if version != VERSION:
        raise GgufInvalid(f"unsupported version {version}; expected version {VERSION}")
    raw_tensors, raw_metadata = reader.number("Q"), reader.number("Q")
    metadata_count = reader.count(raw_metadata, "metadata", 13, MAX_METADATA_COUNT)
    tensor_count = reader.count(raw_tensors, "tensor", 32, MAX_TENSOR_COUNT)

    metadata, seen = [], set()
    for _ in range(metadata_count):
        key = reader.string("metadata key", MAX_METADATA_KEY_BYTES)
        if key == "":
            raise GgufInvalid("metadata key must not be empty")
        if key in seen:
            raise GgufInvalid(f"duplicate metadata key {_quoted(key)}")
        seen.add(key)
        metadata.append((key,) + _value(reader, reader.number("I")))

    def find(key):
        return next((entry for entry in metadata if entry[0] == key), None)

    entry = find("general.architecture")
    if entry is None:
        raise GgufInvalid("missing general.architecture metadata")
    if entry[1] != "string" or entry[2]:
        raise GgufInvalid("general.architecture metadata must be a string")
    if entry[3] == "":
        raise GgufInvalid("general.architecture metadata must not be empty")
    architecture = entry[3]

    alignment = DEFAULT_ALIGNMENT
    entry = find("general.alignment")
    if entry is not None:
        if entry[1] != "u32" or entry[2]:
            raise GgufInvalid("general.alignment metadata must be u32")
        alignment = entry[3]
    if alignment == 0 or alignment & (alignment - 1):
        raise GgufInvalid(f"general.alignment must be a positive power of two, got {alignment}")

    raw, names, quantized = [], set(), False
    for _ in range(tensor_count):
        name = reader.string("tensor name", MAX_TENSOR_NAME_BYTES)
        if name == "":
            raise GgufInvalid("tensor name must not be empty")
        if name in names:
            raise GgufInvalid(f"duplicate tensor name {_quoted(name)}")
        names.add(name)
        rank = reader.number("I")
        if not 1 <= rank <= 4:
            raise GgufInvalid(f"tensor {_quoted(name)} rank must be in 1..=4, got {rank}")
        dimensions = []
        for _ in range(rank):
            dimension = reader.number("Q")
            if dimension == 0 or dimension > SAFE_INTEGER:
                raise GgufInvalid(f"tensor {_quoted(name)} has invalid dimension {dimension}")
            dimensions.append(dimension)
        code = reader.number("I")
        if code not in FORMATS:
            raise GgufInvalid(f"unsupported GGML tensor type code {code}")
        quantized |= FORMATS[code][2] != 0
        offset = reader.number("Q")
        if offset % alignment:
            raise GgufInvalid(f"tensor {_quoted(name)} offset {offset} is not aligned to {alignment}")
        raw.append((name, dimensions, code, offset))

    if quantized:
        entry = find("general.quantization_version")
        if entry is None:
            raise GgufInvalid("missing general.quantization_version metadata for quantized tensors")
        if entry[1] != "u32" or entry[2]:
            raise GgufInvalid("general.quantization_version metadata must be u32")
        if entry[3] != QUANTIZATION_VERSION:
            raise GgufInvalid(f"unsupported general.quantization_version {entry[3]}; expected {QUANTIZATION_VERSION}")

    data_start = (reader.position + alignment - 1) & ~(alignment - 1)
    if data_start > reader.file_len:
        raise GgufInvalid("aligned tensor-data section starts beyond the file")

    limit = 1 << 64
    tensors = []
    for name, dimensions, code, offset in raw:
        logical = list(reversed(dimensions))
        label, block_values, block_bytes = FORMATS[code]
        if block_bytes == 0:
            elements = 1
            for d in logical:
                elements *= d
                if elements >= limit:
                    raise GgufInvalid(f"tensor {_quoted(name)} size overflows")
            byte_len = elements * 4
            physical = logical
        else:
            columns = dimensions[0]
            if columns % block_values:
                raise GgufInvalid(f"tensor {_quoted(name)} least-major dimension {columns} is not divisible by "
                                  f"{block_values} for {label}")
            rows = 1
            for d in dimensions[1:]:
                rows *= d
                if rows >= limit:
                    raise GgufInvalid(f"tensor {_quoted(name)} row count size overflows")
            row_bytes = columns // block_values * block_bytes
            byte_len = rows * row_bytes
            physical = [rows, row_bytes]
        if byte_len >= limit:
            raise GgufInvalid(f"tensor {_quoted(name)} byte length overflows")
        data_offset = data_start + offset
        if data_offset >= limit:
            raise GgufInvalid("absolute tensor offset overflows")
        end = data_offset + byte_len
        if end >= limit:
            raise GgufInvalid("tensor range end overflows")
        if end > reader.file_len:
            raise GgufInvalid(f"tensor {_quoted(name)} range [{data_offset}, {end}) exceeds file size {reader.file_len}")
        tensors.append(dict(name=name, format=code, logical_shape=tuple(logical), physical_shape=tuple(physical),
                            data_offset=data_offset, byte_len=byte_len))
    order = sorted(tensors, key=lambda t: t["data_offset"])
    for before, after in zip(order, order[1:]):
        if after["data_offset"] < before["data_offset"] + before["byte_len"]:
            raise GgufInvalid(f"tensor ranges for {_quoted(before['name'])} and {_quoted(after['name'])} overlap")
    return dict(architecture=architecture, metadata=metadata, tensors=tensors)
