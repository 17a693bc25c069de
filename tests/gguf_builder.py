"""Writes GGUF v3 files for the tests, following the public GGUF layout: magic, version, tensor
count, metadata count, metadata entries (key, type, value), tensor infos (name, rank, dimensions
least-major first, ggml type, offset relative to the aligned data section), padding, payloads."""
import struct

CODES = {"u8": (0, "B"), "i8": (1, "b"), "u16": (2, "H"), "i16": (3, "h"), "u32": (4, "I"), "i32": (5, "i"),
         "f32": (6, "f"), "bool": (7, "B"), "u64": (10, "Q"), "i64": (11, "q"), "f64": (12, "d")}


def gguf_string(text) -> bytes:
    raw = text if isinstance(text, bytes) else text.encode()
    return struct.pack("<Q", len(raw)) + raw


def scalar(kind: str, value) -> bytes:
    if kind == "string":
        return gguf_string(value)
    return struct.pack("<" + CODES[kind][1], value)


def entry(key, kind: str, value, array=False) -> bytes:
    """One metadata entry; ``array=True`` makes ``value`` a list of ``kind`` elements."""
    code = 8 if kind == "string" else CODES[kind][0]
    if array:
        body = struct.pack("<IQ", code, len(value)) + b"".join(scalar(kind, v) for v in value)
        return gguf_string(key) + struct.pack("<I", 9) + body
    return gguf_string(key) + struct.pack("<I", code) + scalar(kind, value)


def raw_entry(key, code: int, payload: bytes) -> bytes:
    return gguf_string(key) + struct.pack("<I", code) + payload


def build(entries, tensors, alignment=32, *, architecture="test", payloads=None, write_alignment=True,
          version=3, magic=b"GGUF", with_body=True):
    """``entries``: encoded metadata entries (after general.architecture and general.alignment);
    ``tensors``: dicts name / dimensions (least-major first) / format / offset / bytes;
    ``payloads``: optional {name: bytes} placed at the tensors' offsets. Returns (bytes, start of the data
    section); ``with_body=False`` returns the header alone (for sparse files)."""
    head = []
    if architecture is not None:
        head.append(entry("general.architecture", "string", architecture))
    if write_alignment:
        head.append(entry("general.alignment", "u32", alignment))
    out = magic + struct.pack("<IQQ", version, len(tensors), len(head) + len(entries)) + b"".join(head) + b"".join(entries)
    for t in tensors:
        out += gguf_string(t["name"]) + struct.pack("<I", len(t["dimensions"]))
        out += b"".join(struct.pack("<Q", d) for d in t["dimensions"])
        out += struct.pack("<IQ", t["format"], t["offset"])
    step = max(alignment, 1)
    out += b"\0" * (-len(out) % step)
    start = len(out)
    if not with_body:
        return out, start
    length = max((t["offset"] + t["bytes"] for t in tensors), default=0)
    body = bytearray(length)
    for t in tensors:
        if payloads and t["name"] in payloads:
            data = payloads[t["name"]]
            assert len(data) == t["bytes"]
            body[t["offset"]:t["offset"] + len(data)] = data
    return out + bytes(body), start
