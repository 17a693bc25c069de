"""Host mirror of the reference's GGUF v3 reader (crates/runtime/src/gguf.rs) over the C ABI.

``GgufFile.open(path)`` = ``parse_gguf`` (:682-957): the metadata table and the tensor catalog, with the
reference's validation, limits and messages. ``read_tensor`` = ``read_gguf_tensor_into`` (:959-994);
``upload_tensor`` puts the same bytes into device memory, where a quantized tensor is the
``[rows, encoded_row_bytes]`` u8 matrix the contraction takes.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple, Union

import numpy as np
import torch

from . import _native as N
from .quantized import CancellationFlag, Cancelled, QuantizedError, _stream_handle

VALUE_TYPES = ("u8", "i8", "u16", "i16", "u32", "i32", "f32", "bool", "string", "array", "u64", "i64", "f64")
FORMAT_NAMES = {0: "F32", 2: "Q4_0", 8: "Q8_0", 10: "Q2_K", 11: "Q3_K", 12: "Q4_K", 13: "Q5_K", 14: "Q6_K"}


class GgufParseError(QuantizedError):
    """``GgufParseError`` (gguf.rs:80-107): ``Invalid``, ``Io`` or - as :class:`Cancelled` - cancelled."""


def _check(status: int) -> None:
    if status == N.OK:
        return
    message = N.last_error()
    if status == N.ERR_CANCELLED:
        raise Cancelled(status, message)
    raise GgufParseError(status, message)


@dataclass(frozen=True)
class GgufMetadataValue:
    """A typed metadata value: ``kind`` is the element type name (arrays report their elements', as
    ``GgufMetadataValue::kind`` does), ``is_array`` tells the two apart."""
    kind: str
    is_array: bool
    value: Union[int, float, bool, str, list]


@dataclass(frozen=True)
class GgufTensorDescriptor:
    name: str
    format: int               # GGML type code
    logical_shape: Tuple[int, ...]
    physical_shape: Tuple[int, ...]
    data_offset: int
    byte_len: int

    @property
    def format_name(self) -> str:
        return FORMAT_NAMES[self.format]


class GgufFile:
    def __init__(self, handle: int):
        self._handle = handle
        lib = N.lib()
        self.metadata: List[Tuple[str, GgufMetadataValue]] = []
        for index in range(lib.et_hip_gguf_metadata_count(handle)):
            key = ctypes.string_at(lib.et_hip_gguf_metadata_key(handle, index),
                                   lib.et_hip_gguf_metadata_key_length(handle, index)).decode()
            self.metadata.append((key, self._value(index)))
        self.architecture = self.get("general.architecture").value
        self.tensors: List[GgufTensorDescriptor] = []
        raw = N.EtGgufTensor()
        for index in range(lib.et_hip_gguf_tensor_count(handle)):
            _check(lib.et_hip_gguf_tensor_at(handle, index, ctypes.byref(raw)))
            self.tensors.append(GgufTensorDescriptor(
                ctypes.string_at(raw.name, raw.name_length).decode(), raw.format, tuple(raw.logical_shape[:raw.logical_rank]),
                tuple(raw.physical_shape[:raw.physical_rank]), raw.data_offset, raw.byte_len))
        self._index: Dict[str, int] = {t.name: i for i, t in enumerate(self.tensors)}

    @classmethod
    def open(cls, path: str, cancelled: Optional[CancellationFlag] = None) -> "GgufFile":
        out = ctypes.c_void_p()
        _check(N.lib().et_hip_gguf_open(str(path).encode(), cancelled.ptr if cancelled is not None else None,
                                        ctypes.byref(out)))
        return cls(out.value)

    def close(self) -> None:
        if self._handle:
            N.lib().et_hip_gguf_close(self._handle)
            self._handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:  # noqa: BLE001 - interpreter shutdown
            pass

    def _value(self, index: int) -> GgufMetadataValue:
        lib, handle = N.lib(), self._handle
        kind = lib.et_hip_gguf_metadata_type(handle, index)
        element = lib.et_hip_gguf_metadata_element_type(handle, index)
        length = lib.et_hip_gguf_metadata_length(handle, index)
        name = VALUE_TYPES[element]

        def one(i):
            if name in ("u8", "u16", "u32", "u64", "bool"):
                out = ctypes.c_uint64()
                assert lib.et_hip_gguf_metadata_unsigned(handle, index, i, ctypes.byref(out)) == 0
                return bool(out.value) if name == "bool" else out.value
            if name in ("i8", "i16", "i32", "i64"):
                out = ctypes.c_int64()
                assert lib.et_hip_gguf_metadata_signed(handle, index, i, ctypes.byref(out)) == 0
                return out.value
            if name in ("f32", "f64"):
                out = ctypes.c_double()
                assert lib.et_hip_gguf_metadata_real(handle, index, i, ctypes.byref(out)) == 0
                return out.value
            size = ctypes.c_uint64()
            pointer = lib.et_hip_gguf_metadata_string(handle, index, i, ctypes.byref(size))
            return ctypes.string_at(pointer, size.value).decode()

        if kind == 9:
            return GgufMetadataValue(name, True, [one(i) for i in range(length)])
        return GgufMetadataValue(name, False, one(0))

    def get(self, key: str) -> Optional[GgufMetadataValue]:
        for name, value in self.metadata:
            if name == key:
                return value
        return None

    def tensor(self, name: str) -> GgufTensorDescriptor:
        return self.tensors[self._index[name]]

    def read_tensor(self, name: str, destination: Optional[np.ndarray] = None,
                    cancelled: Optional[CancellationFlag] = None) -> np.ndarray:
        """The tensor's payload bytes (``read_gguf_tensor_into``); ``destination``: a uint8 array of exactly
        ``byte_len`` bytes, allocated when omitted."""
        descriptor = self.tensor(name)
        if destination is None:
            destination = np.empty(descriptor.byte_len, dtype=np.uint8)
        assert destination.dtype == np.uint8 and destination.flags.c_contiguous
        _check(N.lib().et_hip_gguf_read_tensor_into(self._handle, self._index[name], destination.ctypes.data,
                                                    destination.size, cancelled.ptr if cancelled is not None else None))
        return destination

    def upload_tensor(self, name: str, device, destination: Optional[torch.Tensor] = None, stream=None,
                      cancelled: Optional[CancellationFlag] = None) -> torch.Tensor:
        """The payload in device memory: a u8 tensor of the physical shape for quantized formats, an f32
        tensor of the logical shape for F32."""
        descriptor = self.tensor(name)
        if destination is None:
            if descriptor.format == 0:
                destination = torch.empty(descriptor.logical_shape, dtype=torch.float32, device=device)
            else:
                destination = torch.empty(descriptor.physical_shape, dtype=torch.uint8, device=device)
        assert destination.is_contiguous()
        _check(N.lib().et_hip_gguf_upload_tensor(self._handle, self._index[name], destination.data_ptr(),
                                                 destination.numel() * destination.element_size(),
                                                 _stream_handle(stream),
                                                 cancelled.ptr if cancelled is not None else None))
        return destination
