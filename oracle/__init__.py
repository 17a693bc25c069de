"""ctypes binding of the CPU oracle (``libet_oracle.so``).

TEST INFRASTRUCTURE ONLY. Importable from ``tests/``, from the smoke check and
from the benchmark's CPU-baseline leg; never from the product package.
The oracle restates crates/runtime-cpu/src/quantized.rs of the reference in
plain C (see ``et_oracle.h`` for the per-function citations and pin status).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libet_oracle.so")

Q4_0, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 2, 8, 10, 11, 12, 13, 14
K_QUANTS = (Q2_K, Q3_K, Q4_K, Q5_K, Q6_K)
ALL_CODECS = (Q4_0, Q8_0) + K_QUANTS


class OracleError(RuntimeError):
    """An ``Err(String)`` of the restated reference routine."""


class _Layout(ctypes.Structure):
    _fields_ = [
        ("rank", ctypes.c_int),
        ("shape", ctypes.POINTER(ctypes.c_size_t)),
        ("strides", ctypes.POINTER(ctypes.c_size_t)),
        ("offset", ctypes.c_size_t),
    ]


def build() -> str:
    """Compiles the oracle with gcc (always; it takes about a second)."""
    subprocess.run(["make", "-C", _HERE, "-B", "libet_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        sz, vp, ci = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int
        L.et_oracle_codec_name.restype = ctypes.c_char_p
        L.et_oracle_codec_name.argtypes = [ci]
        for name in ("et_oracle_block_values", "et_oracle_block_bytes"):
            getattr(L, name).restype = sz
            getattr(L, name).argtypes = [ci]
        L.et_oracle_encoded_row_bytes.restype = sz
        L.et_oracle_encoded_row_bytes.argtypes = [ci, sz]
        L.et_oracle_fp16_to_f32.restype = ctypes.c_float
        L.et_oracle_fp16_to_f32.argtypes = [ctypes.c_uint16]
        L.et_oracle_scale_min_k4.restype = None
        L.et_oracle_scale_min_k4.argtypes = [sz, vp, vp, vp]
        L.et_oracle_decode_block.restype = ci
        L.et_oracle_decode_block.argtypes = [ci, vp, sz, vp, ctypes.c_char_p, sz]
        L.et_oracle_source_index.restype = sz
        L.et_oracle_source_index.argtypes = [ctypes.POINTER(_Layout), sz]
        L.et_oracle_linear_into.restype = ci
        L.et_oracle_linear_into.argtypes = [ci, sz, sz, vp, ctypes.POINTER(_Layout), vp, sz, vp,
                                            ctypes.POINTER(_Layout), vp, vp, ctypes.c_char_p, sz]
        L.et_oracle_linear_rows.restype = ci
        L.et_oracle_linear_rows.argtypes = [ci, sz, sz, sz, vp, vp, vp, vp, sz, sz]
        L.et_oracle_embedding_into.restype = ci
        L.et_oracle_embedding_into.argtypes = [ci, sz, sz, vp, ci, ctypes.POINTER(_Layout), sz, vp,
                                               sz, vp, vp, ctypes.c_char_p, sz]
        L.et_oracle_quantize_q8.restype = None
        L.et_oracle_quantize_q8.argtypes = [sz, sz, vp, vp, vp, vp]
        L.et_oracle_linear_q8_rows.restype = ci
        L.et_oracle_linear_q8_rows.argtypes = [ci, sz, sz, sz, vp, vp, vp, vp, vp, vp, sz, sz]
        L.et_oracle_rms_norm.restype = None
        L.et_oracle_rms_norm.argtypes = [vp, vp, ctypes.c_double, vp, sz, sz]
        L.et_oracle_rotary.restype = ci
        L.et_oracle_rotary.argtypes = [vp, vp, sz, ctypes.c_double, ctypes.c_double, ci, vp, sz, sz, sz, sz,
                                       ctypes.c_char_p, sz]
        L.et_oracle_silu_mul.restype = None
        L.et_oracle_silu_mul.argtypes = [vp, vp, vp, sz]
        L.et_oracle_add.restype = None
        L.et_oracle_add.argtypes = [vp, vp, vp, sz]
        L.et_oracle_argmax.restype = ci
        L.et_oracle_argmax.argtypes = [vp, sz, sz, vp, ctypes.c_char_p, sz]
        L.et_oracle_gather_rows.restype = ci
        L.et_oracle_gather_rows.argtypes = [vp, sz, sz, vp, sz, vp, ctypes.c_char_p, sz]
        L.et_oracle_f32_to_fp16.restype = ctypes.c_uint16
        L.et_oracle_f32_to_fp16.argtypes = [ctypes.c_float]
        L.et_oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.et_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.et_oracle_kv_attention_scaled.restype = ci
        L.et_oracle_kv_attention_scaled.argtypes = [ci, vp, vp, vp, vp, sz, sz, sz, sz, vp, sz, vp, vp, sz, sz, sz, sz,
                                                    vp, vp, vp, ctypes.c_double, sz, sz, vp, ctypes.c_char_p, sz]
        _lib = L
    return _lib


def _ptr(array):
    return None if array is None else array.ctypes.data_as(ctypes.c_void_p)


def _layout(shape, strides=None, offset=0):
    rank = len(shape)
    shape_arr = (ctypes.c_size_t * max(rank, 1))(*shape)
    strides_arr = None
    if strides is not None:
        strides_arr = (ctypes.c_size_t * max(rank, 1))(*strides)
    layout = _Layout(rank, shape_arr, strides_arr, offset)
    layout._keep = (shape_arr, strides_arr)
    return layout


def codec_name(codec: int) -> str:
    return lib().et_oracle_codec_name(codec).decode()


def block_values(codec: int) -> int:
    return lib().et_oracle_block_values(codec)


def block_bytes(codec: int) -> int:
    return lib().et_oracle_block_bytes(codec)


def encoded_row_bytes(codec: int, columns: int):
    """``None`` when ``columns`` is not a whole number of blocks (gguf.rs:245-250)."""
    value = lib().et_oracle_encoded_row_bytes(codec, columns)
    return None if value == 0 and columns != 0 else value


def fp16_to_f32_bits(bits: int) -> int:
    value = np.float32(lib().et_oracle_fp16_to_f32(bits))
    return int(value.view(np.uint32))


def scale_min_k4(index: int, scales12: bytes):
    buf = np.frombuffer(bytes(scales12), dtype=np.uint8).copy()
    sc = ctypes.c_uint8()
    mn = ctypes.c_uint8()
    lib().et_oracle_scale_min_k4(index, _ptr(buf), ctypes.byref(sc), ctypes.byref(mn))
    return sc.value, mn.value


def decode_block(codec: int, block: bytes) -> np.ndarray:
    buf = np.frombuffer(bytes(block), dtype=np.uint8).copy()
    out = np.zeros(max(block_values(codec), 1), dtype=np.float32)
    err = ctypes.create_string_buffer(256)
    if lib().et_oracle_decode_block(codec, _ptr(buf), buf.size, _ptr(out), err, 256) != 0:
        raise OracleError(err.value.decode())
    return out


def decode_rows(codec: int, weight: np.ndarray, columns: int) -> np.ndarray:
    """Decodes a packed ``[rows, row_bytes]`` u8 matrix to ``[rows, columns]`` f32."""
    weight = np.ascontiguousarray(weight, dtype=np.uint8)
    rows = weight.shape[0]
    indexes = np.arange(rows, dtype=np.uint32)
    return embedding_into(codec, rows, columns, indexes, weight)


def linear_into(codec, rows, columns, x, weight, bias=None, *, x_shape=None, x_strides=None,
                x_offset=0, bias_strides=None, bias_offset=0, cancel=None) -> np.ndarray:
    """``linear_into`` of the reference (quantized.rs:419-499).

    ``x`` is the storage buffer; ``x_shape``/``x_strides``/``x_offset`` describe
    the logical view (default: ``x`` itself, dense). Returns ``[.., rows]`` f32.
    """
    x = np.ascontiguousarray(x, dtype=np.float32) if x_shape is None else x
    assert x.dtype == np.float32
    shape = tuple(x.shape) if x_shape is None else tuple(x_shape)
    weight = np.ascontiguousarray(weight, dtype=np.uint8)
    vectors = int(np.prod(shape[:-1])) if len(shape) >= 1 else 0
    # Sizes that cannot be allocated never get that far: validation rejects them first.
    total = vectors * rows
    y = np.zeros(total if total < (1 << 34) else 1, dtype=np.float32)
    xl = _layout(shape, x_strides, x_offset)
    bl = _layout((rows,), bias_strides, bias_offset)
    if bias is not None:
        assert bias.dtype == np.float32
    flag = None
    if cancel is not None:
        flag = np.array([1 if cancel else 0], dtype=np.int32)
    err = ctypes.create_string_buffer(256)
    rc = lib().et_oracle_linear_into(codec, rows, columns, _ptr(x), ctypes.byref(xl), _ptr(weight),
                                     weight.size, _ptr(bias), ctypes.byref(bl), _ptr(y), _ptr(flag),
                                     err, 256)
    if rc != 0:
        raise OracleError(err.value.decode())
    return y.reshape(shape[:-1] + (rows,))


def linear_rows(codec, rows, columns, x, weight, bias=None, row_begin=0, row_end=None,
                out=None) -> np.ndarray:
    """Dense-input variant restricted to rows ``[row_begin, row_end)``; other rows stay 0."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, columns)
    weight = np.ascontiguousarray(weight, dtype=np.uint8)
    vectors = x.shape[0]
    row_end = rows if row_end is None else row_end
    y = np.zeros((vectors, rows), dtype=np.float32) if out is None else out
    rc = lib().et_oracle_linear_rows(codec, rows, columns, vectors, _ptr(x), _ptr(weight),
                                     _ptr(bias), _ptr(y), row_begin, row_end)
    if rc != 0:
        raise OracleError("et_oracle_linear_rows: invalid geometry")
    return y


def embedding_into(codec, rows, columns, indexes, weight, *, index_shape=None, index_strides=None,
                   index_offset=0, cancel=None) -> np.ndarray:
    """``embedding_into`` of the reference (quantized.rs:546-616)."""
    assert indexes.dtype in (np.uint32, np.int64)
    weight = np.ascontiguousarray(weight, dtype=np.uint8)
    shape = tuple(indexes.shape) if index_shape is None else tuple(index_shape)
    count = int(np.prod(shape)) if len(shape) else 1
    out = np.zeros(count * columns, dtype=np.float32)
    il = _layout(shape, index_strides, index_offset)
    flag = None
    if cancel is not None:
        flag = np.array([1 if cancel else 0], dtype=np.int32)
    err = ctypes.create_string_buffer(256)
    rc = lib().et_oracle_embedding_into(codec, rows, columns, _ptr(indexes),
                                        1 if indexes.dtype == np.int64 else 0, ctypes.byref(il),
                                        count, _ptr(weight), weight.size, _ptr(out), _ptr(flag),
                                        err, 256)
    if rc != 0:
        raise OracleError(err.value.decode())
    return out.reshape(shape + (columns,))


def quantize_q8(x: np.ndarray):
    """int8 activation quantizer per 32 columns -> (q int8, scale f32, sum i32)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    columns = x.shape[-1]
    x2 = x.reshape(-1, columns)
    vectors = x2.shape[0]
    q = np.zeros((vectors, columns), dtype=np.int8)
    scale = np.zeros((vectors, columns // 32), dtype=np.float32)
    total = np.zeros((vectors, columns // 32), dtype=np.int32)
    lib().et_oracle_quantize_q8(vectors, columns, _ptr(x2), _ptr(q), _ptr(scale), _ptr(total))
    return q, scale, total


def linear_q8_rows(codec, rows, columns, q, scale, total, weight, bias=None, row_begin=0,
                   row_end=None) -> np.ndarray:
    weight = np.ascontiguousarray(weight, dtype=np.uint8)
    vectors = q.shape[0]
    row_end = rows if row_end is None else row_end
    y = np.zeros((vectors, rows), dtype=np.float32)
    rc = lib().et_oracle_linear_q8_rows(codec, rows, columns, vectors, _ptr(q), _ptr(scale),
                                        _ptr(total), _ptr(weight), _ptr(bias), _ptr(y), row_begin,
                                        row_end)
    if rc != 0:
        raise OracleError("et_oracle_linear_q8_rows: invalid geometry or codec")
    return y


def f32_to_fp16_bits(value) -> int:
    """binary32 -> binary16 bits, round to nearest even (et_oracle_f32_to_fp16)."""
    return int(lib().et_oracle_f32_to_fp16(ctypes.c_float(float(np.float32(value)))))


def f32_to_bf16_bits(value) -> int:
    """binary32 -> bfloat16 bits, round to nearest even (et_oracle_f32_to_bf16)."""
    return int(lib().et_oracle_f32_to_bf16(ctypes.c_float(float(np.float32(value)))))


def kv_attention(k_slab: np.ndarray, v_slab: np.ndarray, block_size: int, block_table: np.ndarray,
                 cursors, advances, q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float,
                 window: int = 0, active_batch=None, context_window: int = 0, k_scales=None,
                 v_scales=None) -> np.ndarray:
    """Paged KV attention (et_oracle_kv_attention_scaled): writes the new rows of ``k`` / ``v`` into
    the slabs IN PLACE, then attends. Slabs are ``[max_tokens, kv_heads, width]`` in float32, float16,
    uint16 (bfloat16 bits) or uint8 (the int8-quantized tier, with float32 ``k_scales`` / ``v_scales``
    ``[max_tokens, kv_heads]``, written in place too). ``q`` is ``[batch, query_heads, tokens, width]``;
    returns the output of the same shape."""
    codes = {np.dtype(np.float32): 0, np.dtype(np.float16): 2, np.dtype(np.uint16): 3, np.dtype(np.uint8): 4}
    assert k_slab.dtype == v_slab.dtype and k_slab.dtype in codes
    code = codes[k_slab.dtype]
    if code == 4:
        for scales in (k_scales, v_scales):
            assert scales is not None and scales.dtype == np.float32 and scales.flags.c_contiguous
            assert scales.shape == k_slab.shape[:2]
    assert k_slab.flags.c_contiguous and v_slab.flags.c_contiguous and k_slab.shape == v_slab.shape
    max_tokens, kv_heads, width = k_slab.shape
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    batch, query_heads, tokens, _ = q.shape
    assert k.shape == (batch, kv_heads, tokens, width) and v.shape == k.shape
    table = np.ascontiguousarray(block_table, dtype=np.uint32).reshape(batch, -1)
    cursors = np.ascontiguousarray(cursors, dtype=np.uint32)
    advances = np.ascontiguousarray(advances, dtype=np.uint32)
    out = np.zeros_like(q)
    err = ctypes.create_string_buffer(256)
    rc = lib().et_oracle_kv_attention_scaled(code, _ptr(k_slab), _ptr(v_slab),
                                             _ptr(k_scales) if code == 4 else None,
                                             _ptr(v_scales) if code == 4 else None,
                                             max_tokens, kv_heads, width, block_size, _ptr(table), table.shape[1],
                                             _ptr(cursors), _ptr(advances), batch,
                                             batch if active_batch is None else active_batch, query_heads, tokens,
                                             _ptr(q), _ptr(k), _ptr(v), float(scale), context_window, window,
                                             _ptr(out), err, 256)
    if rc != 0:
        raise OracleError(err.value.decode())
    return out


def rms_norm(x: np.ndarray, weight, eps: float) -> np.ndarray:
    """et_oracle_rms_norm over the last dimension of a float32 array."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = None if weight is None else np.ascontiguousarray(weight, dtype=np.float32)
    out = np.empty_like(x)
    lib().et_oracle_rms_norm(_ptr(x), None if w is None else _ptr(w), float(eps), _ptr(out),
                             x.size // x.shape[-1], x.shape[-1])
    return out


def rotary(x: np.ndarray, offsets, theta: float, sign: float = 1.0, interleaved: bool = False) -> np.ndarray:
    """et_oracle_rotary for ``[..., steps, head_dim]``; the batch is the first dimension (1 for rank 2)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    offsets = np.ascontiguousarray(offsets, dtype=np.uint32)
    batch = 1 if x.ndim == 2 else x.shape[0]
    steps, head_dim = x.shape[-2], x.shape[-1]
    rows = x.size // (steps * head_dim) if steps * head_dim else 0
    out = np.empty_like(x)
    err = ctypes.create_string_buffer(256)
    rc = lib().et_oracle_rotary(_ptr(x), _ptr(offsets), offsets.size, float(theta), float(sign),
                                1 if interleaved else 0, _ptr(out), batch, rows, steps, head_dim, err, 256)
    if rc != 0:
        raise OracleError(err.value.decode())
    return out


def silu_mul(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    gate = np.ascontiguousarray(gate, dtype=np.float32)
    up = np.ascontiguousarray(up, dtype=np.float32)
    assert gate.shape == up.shape
    out = np.empty_like(gate)
    lib().et_oracle_silu_mul(_ptr(gate), _ptr(up), _ptr(out), gate.size)
    return out


def argmax_rows(logits: np.ndarray) -> np.ndarray:
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    rows = logits.size // logits.shape[-1] if logits.shape[-1] else 0
    out = np.empty(rows, dtype=np.uint32)
    err = ctypes.create_string_buffer(256)
    if lib().et_oracle_argmax(_ptr(logits), rows, logits.shape[-1], _ptr(out), err, 256) != 0:
        raise OracleError(err.value.decode())
    return out.reshape(logits.shape[:-1])


def gather_rows(table: np.ndarray, indexes) -> np.ndarray:
    table = np.ascontiguousarray(table)
    indexes = np.ascontiguousarray(indexes, dtype=np.int64)
    out = np.empty(indexes.shape + table.shape[1:], dtype=table.dtype)
    err = ctypes.create_string_buffer(256)
    row_bytes = table.dtype.itemsize * int(np.prod(table.shape[1:], dtype=np.int64))
    if lib().et_oracle_gather_rows(_ptr(table), table.shape[0], row_bytes, _ptr(indexes), indexes.size,
                                   _ptr(out), err, 256) != 0:
        raise OracleError(err.value.decode())
    return out


def add(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    assert a.shape == b.shape
    out = np.empty_like(a)
    lib().et_oracle_add(_ptr(a), _ptr(b), _ptr(out), a.size)
    return out
