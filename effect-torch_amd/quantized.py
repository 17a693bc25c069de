"""Host-side mirror of the reference's quantized operator pair, over torch device tensors.

Same names, argument meaning and error text as the backend crates of the
reference (crates/runtime-cpu/src/quantized.rs): ``linear_requirements``
(:297-336) plans and validates, ``linear_into`` (:419-499) executes into a
caller-provided destination; ``embedding_requirements`` (:340-365) and
``embedding_into`` (:546-616) likewise. Errors the reference returns as
``Err(String)`` are raised as :class:`QuantizedError` carrying the same text.

torch is used for device memory and streams only; all arithmetic happens in
``libet_hip.so`` behind the C ABI of ``include/et_hip.h``.
"""
from __future__ import annotations

import ctypes
import enum
from typing import Optional, Sequence

import torch

from . import _native as N


class GgmlQuant(enum.IntEnum):
    """GGML tensor type codes; Q2_K..Q6_K are the reference's ``GgmlKQuant``
    (crates/runtime/src/gguf.rs:199-205)."""

    Q4_0 = 2
    Q8_0 = 8
    Q2_K = 10
    Q3_K = 11
    Q4_K = 12
    Q5_K = 13
    Q6_K = 14

    @property
    def ggml_name(self) -> str:  # GgmlKQuant::name, gguf.rs:208-217
        return N.lib().et_hip_codec_name(int(self)).decode()

    @classmethod
    def from_name(cls, name: str) -> Optional["GgmlQuant"]:  # gguf.rs:220-230
        for member in cls:
            if member.ggml_name == name:
                return member
        return None

    @property
    def block_values(self) -> int:
        return N.lib().et_hip_block_values(int(self))

    @property
    def block_bytes(self) -> int:  # quantized.rs:60-68
        return N.lib().et_hip_block_bytes(int(self))

    def encoded_row_bytes(self, columns: int) -> Optional[int]:  # gguf.rs:245-250
        value = N.lib().et_hip_encoded_row_bytes(int(self), columns)
        return None if value == 0 and columns != 0 else value


class ActivationMode(enum.IntEnum):
    F32 = N.ACT_F32
    INT8 = N.ACT_INT8


class QuantizedError(RuntimeError):
    """An ``Err(String)`` of the reference operator; ``status`` is the et_status."""

    def __init__(self, status: int, message: str):
        super().__init__(message)
        self.status = status


class Cancelled(QuantizedError):
    """``"operation aborted"`` (crates/runtime-cpu/src/quantized.rs:451-453)."""


_DTYPES = {
    torch.float32: N.DTYPE_F32,
    torch.float64: N.DTYPE_F64,
    torch.float16: N.DTYPE_F16,
    torch.bfloat16: N.DTYPE_BF16,
    torch.uint8: N.DTYPE_U8,
    torch.uint32: N.DTYPE_U32,
    torch.int64: N.DTYPE_I64,
}


def _check(status: int) -> None:
    if status == N.OK:
        return
    message = N.last_error()
    if status == N.ERR_CANCELLED:
        raise Cancelled(status, message)
    raise QuantizedError(status, message)


def _check_calibration(status: int) -> None:
    """:func:`_check` for the measurement library, which keeps its own error message."""
    if status != N.OK:
        raise QuantizedError(status, (N.calibrate_lib().et_hip_calibration_last_error() or b"").decode())


class _Desc:
    """Keeps the ctypes arrays of an ``et_tensor`` alive."""

    def __init__(self, tensor: torch.Tensor):
        if tensor.dtype not in _DTYPES:
            raise QuantizedError(N.ERR_UNSUPPORTED, f"unsupported dtype {tensor.dtype}")
        rank = tensor.dim()
        self.shape = (ctypes.c_uint64 * max(rank, 1))(*tensor.shape)
        self.strides = (ctypes.c_uint64 * max(rank, 1))(*tensor.stride())
        storage_ptr = tensor.untyped_storage().data_ptr() if tensor.numel() or tensor.device.type != "meta" else 0
        self.struct = N.EtTensor(storage_ptr, _DTYPES[tensor.dtype], rank, self.shape, self.strides,
                                 tensor.storage_offset())

    @property
    def ref(self):
        return ctypes.byref(self.struct)


def _desc(tensor: Optional[torch.Tensor]):
    return None if tensor is None else _Desc(tensor)


def _ref(desc: Optional[_Desc]):
    return None if desc is None else desc.ref


def _stream_handle(stream) -> int:
    if stream is None:
        stream = torch.cuda.current_stream()
    return stream.cuda_stream if hasattr(stream, "cuda_stream") else int(stream)


class CancellationFlag:
    """Host flag polled before work is enqueued (crates/runtime/src/cancellation.rs:18-35)."""

    def __init__(self):
        self._value = ctypes.c_int32(0)

    def cancel(self) -> None:
        self._value.value = 1

    def is_cancelled(self) -> bool:
        return self._value.value != 0

    @property
    def ptr(self):
        return ctypes.cast(ctypes.byref(self._value), ctypes.c_void_p)


class QuantizedRequirements:
    """Frozen plan of one quantized linear (crates/runtime-cpu/src/quantized.rs:35-42)."""

    def __init__(self, handle: int, codec: GgmlQuant, rows: int, columns: int):
        self._handle = ctypes.c_void_p(handle)
        self.codec, self.rows, self.columns = codec, rows, columns
        lib = N.lib()
        rank = lib.et_hip_linear_plan_output_rank(self._handle)
        shape = (ctypes.c_uint64 * max(rank, 1))()
        lib.et_hip_linear_plan_output_shape(self._handle, shape)
        self.output_shape = tuple(shape[i] for i in range(rank))
        self.vectors = lib.et_hip_linear_plan_vectors(self._handle)
        self.output_bytes = lib.et_hip_linear_plan_output_bytes(self._handle)
        self.workspace_bytes = lib.et_hip_linear_plan_workspace_bytes(self._handle)
        self.kernel = lib.et_hip_linear_plan_kernel(self._handle).decode()
        self.algorithmic_bytes = lib.et_hip_linear_plan_algorithmic_bytes(self._handle)

    def __del__(self):
        handle, self._handle = getattr(self, "_handle", None), None
        if handle:
            try:
                N.lib().et_hip_linear_plan_destroy(handle)
            except Exception:
                pass


class EmbeddingRequirements:
    def __init__(self, handle: int, codec: GgmlQuant, rows: int, columns: int):
        self._handle = ctypes.c_void_p(handle)
        self.codec, self.rows, self.columns = codec, rows, columns
        lib = N.lib()
        rank = lib.et_hip_embedding_plan_output_rank(self._handle)
        shape = (ctypes.c_uint64 * max(rank, 1))()
        lib.et_hip_embedding_plan_output_shape(self._handle, shape)
        self.output_shape = tuple(shape[i] for i in range(rank))
        self.output_bytes = lib.et_hip_embedding_plan_output_bytes(self._handle)

    def __del__(self):
        handle, self._handle = getattr(self, "_handle", None), None
        if handle:
            try:
                N.lib().et_hip_embedding_plan_destroy(handle)
            except Exception:
                pass


def is_available() -> bool:
    """A gfx950 device is visible (cf. isAvailable, native-addon.ts:266)."""
    return bool(N.lib().et_hip_is_available())


def linear_requirements(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                        codec: GgmlQuant, weight_shape: Sequence[int],
                        activation_mode: ActivationMode = ActivationMode.F32) -> QuantizedRequirements:
    """Plan step (crates/runtime-cpu/src/quantized.rs:297-336). Reads metadata only."""
    rows, columns = weight_shape
    descs = (_desc(input), _desc(weight), _desc(bias))
    out = ctypes.c_void_p()
    _check(N.lib().et_hip_linear_requirements(_ref(descs[0]), _ref(descs[1]), _ref(descs[2]),
                                              int(codec), rows, columns, int(activation_mode),
                                              ctypes.byref(out)))
    return QuantizedRequirements(out.value, GgmlQuant(codec), rows, columns)


def linear_into(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                codec: GgmlQuant, destination: torch.Tensor, requirements: QuantizedRequirements,
                cancelled: Optional[CancellationFlag] = None, *,
                workspace: Optional[torch.Tensor] = None, stream=None) -> None:
    """Execute step (crates/runtime-cpu/src/quantized.rs:419-499): enqueues on ``stream``."""
    if int(codec) != int(requirements.codec):
        raise QuantizedError(N.ERR_EXECUTION, "quantized_linear: codec does not match the immutable plan")
    descs = (_desc(input), _desc(weight), _desc(bias), _desc(destination))
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(N.lib().et_hip_linear_into(requirements._handle, _ref(descs[0]), _ref(descs[1]),
                                      _ref(descs[2]), _ref(descs[3]), ws_ptr, ws_bytes,
                                      _stream_handle(stream),
                                      cancelled.ptr if cancelled is not None else None))


def quantized_linear(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                     codec: GgmlQuant, weight_shape: Sequence[int],
                     activation_mode: ActivationMode = ActivationMode.F32) -> torch.Tensor:
    """Plan + allocate + execute, for callers that do not manage buffers themselves."""
    requirements = linear_requirements(input, weight, bias, codec, weight_shape, activation_mode)
    destination = torch.empty(requirements.output_shape, dtype=torch.float32, device=input.device)
    workspace = None
    if requirements.workspace_bytes:
        workspace = torch.empty(requirements.workspace_bytes, dtype=torch.uint8, device=input.device)
    linear_into(input, weight, bias, codec, destination, requirements, workspace=workspace)
    return destination


def embedding_requirements(indexes: torch.Tensor, weight: torch.Tensor, codec: GgmlQuant,
                           weight_shape: Sequence[int]) -> EmbeddingRequirements:
    """Plan step (crates/runtime-cpu/src/quantized.rs:340-365)."""
    rows, columns = weight_shape
    descs = (_desc(indexes), _desc(weight))
    out = ctypes.c_void_p()
    _check(N.lib().et_hip_embedding_requirements(_ref(descs[0]), _ref(descs[1]), int(codec), rows,
                                                 columns, ctypes.byref(out)))
    return EmbeddingRequirements(out.value, GgmlQuant(codec), rows, columns)


def embedding_into(indexes: torch.Tensor, weight: torch.Tensor, codec: GgmlQuant,
                   destination: torch.Tensor, requirements: EmbeddingRequirements,
                   cancelled: Optional[CancellationFlag] = None, *, stream=None,
                   synchronize: bool = True) -> Optional[torch.Tensor]:
    """Execute step (crates/runtime-cpu/src/quantized.rs:546-616).

    The kernel skips out-of-range indexes and records the first one in a device
    status block. With ``synchronize`` (default) the stream is drained and the
    reference's error is raised here; otherwise the status tensor is returned
    for :func:`embedding_status_check` after the caller's own fence.
    """
    if int(codec) != int(requirements.codec):
        raise QuantizedError(N.ERR_EXECUTION, "quantized_embedding: codec does not match the immutable plan")
    status = torch.empty(N.STATUS_BYTES, dtype=torch.uint8, device=destination.device)
    descs = (_desc(indexes), _desc(weight), _desc(destination))
    _check(N.lib().et_hip_embedding_into(requirements._handle, _ref(descs[0]), _ref(descs[1]),
                                         _ref(descs[2]), status.data_ptr(), _stream_handle(stream),
                                         cancelled.ptr if cancelled is not None else None))
    if not synchronize:
        return status
    embedding_status_check(requirements, status)
    return None


def embedding_status_check(requirements: EmbeddingRequirements, status: torch.Tensor) -> None:
    host = status.cpu().numpy().tobytes()  # synchronises with the producing stream
    buf = ctypes.create_string_buffer(host, N.STATUS_BYTES)
    _check(N.lib().et_hip_embedding_status_check(requirements._handle, buf))


def dequantize_rows(weight: torch.Tensor, codec: GgmlQuant, weight_shape: Sequence[int],
                    stream=None) -> torch.Tensor:
    """Bit-exact decode of every row: ``[rows, columns]`` f32."""
    rows, columns = weight_shape
    out = torch.empty((rows, columns), dtype=torch.float32, device=weight.device)
    _check(N.lib().et_hip_dequantize_rows(int(codec), rows, columns, weight.data_ptr(),
                                          out.data_ptr(), _stream_handle(stream)))
    return out


def quantize_activations(x: torch.Tensor, stream=None):
    """int8 activation quantiser: returns (q int8 [M, K], scale f32 [K/32, M], sum i32 [K/32, M]).

    The library writes the two tables with a row stride of M rounded up to 32;
    the returned tensors are views of the first M columns."""
    assert x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1
    vectors, columns = x.shape
    padded = (vectors + 31) // 32 * 32
    q = torch.empty((vectors, columns), dtype=torch.int8, device=x.device)
    scale = torch.zeros((columns // 32, padded), dtype=torch.float32, device=x.device)
    total = torch.zeros((columns // 32, padded), dtype=torch.int32, device=x.device)
    _check(N.lib().et_hip_quantize_activations(x.data_ptr(), x.stride(0), vectors, columns,
                                               q.data_ptr(), scale.data_ptr(), total.data_ptr(),
                                               _stream_handle(stream)))
    return q, scale[:, :vectors], total[:, :vectors]


STATIC_WORKSPACE_BYTES = 16 << 20  # ET_HIP_STATIC_WORKSPACE_BYTES of include/et_hip.h


class RawLinear:
    """Raw-pointer plan/enqueue pair (``et_hip_linear_plan_create`` / ``et_hip_linear_enqueue``)
    for dense ``[vectors, columns]`` inputs; what a timing loop or a graph capture uses."""

    def __init__(self, codec: GgmlQuant, rows: int, columns: int, vectors: int, has_bias: bool = False,
                 activation_mode: ActivationMode = ActivationMode.F32):
        out = ctypes.c_void_p()
        _check(N.lib().et_hip_linear_plan_create(int(codec), rows, columns, vectors, int(has_bias),
                                                 int(activation_mode), ctypes.byref(out)))
        self.requirements = QuantizedRequirements(out.value, GgmlQuant(codec), rows, columns)
        self.rows, self.columns, self.vectors = rows, columns, vectors

    # The C entry points below take raw device pointers and cannot see how large the buffers behind
    # them are; a kernel that reads past one faults the GPU. These checks are what the holder of the
    # tensors can do for them: every operand must hold at least what the plan will touch.
    def _holds(self, what: str, tensor: Optional[torch.Tensor], nbytes: int) -> None:
        if tensor is None:
            return
        have = tensor.numel() * tensor.element_size()
        if not tensor.is_contiguous() and what != "x":
            raise QuantizedError(N.ERR_INVALID, f"quantized_linear: {what} must be contiguous")
        if have < nbytes:
            raise QuantizedError(N.ERR_INVALID, f"quantized_linear: {what} holds {have} bytes, the plan "
                                                f"[{self.vectors} x {self.columns}] -> [{self.vectors} x {self.rows}] "
                                                f"touches {nbytes}")

    def _check_weight(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> None:
        self._holds("weight", weight, self.rows * (self.requirements.codec.encoded_row_bytes(self.columns) or 0))
        self._holds("bias", bias, 4 * self.rows)

    def _check_input(self, x: torch.Tensor) -> None:
        if x.dim() != 2 or x.shape[1] < self.columns or x.shape[0] < self.vectors or x.stride(1) != 1:
            raise QuantizedError(N.ERR_INVALID, f"quantized_linear: activations of shape {tuple(x.shape)} for a plan of "
                                                f"{self.vectors} vectors x {self.columns} columns")

    def _check_output(self, y: torch.Tensor, residual: Optional[torch.Tensor] = None) -> None:
        self._holds("y", y, 4 * self.vectors * self.rows)
        self._holds("residual", residual, 4 * self.vectors * self.rows)

    def enqueue(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                y: torch.Tensor, workspace: Optional[torch.Tensor] = None, stream=None,
                cancelled: Optional[CancellationFlag] = None) -> None:
        self._check_input(x)
        self._check_weight(weight, bias)
        self._check_output(y)
        ws_ptr = workspace.data_ptr() if workspace is not None else None
        ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
        _check(N.lib().et_hip_linear_enqueue(self.requirements._handle, x.data_ptr(), x.stride(0),
                                             weight.data_ptr(),
                                             bias.data_ptr() if bias is not None else None,
                                             y.data_ptr(), ws_ptr, ws_bytes, _stream_handle(stream),
                                             cancelled.ptr if cancelled is not None else None))


    def enqueue_static_workspace(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                                 y: torch.Tensor, stream=None, cancelled: Optional[CancellationFlag] = None) -> None:
        """:meth:`enqueue` with the library's own static device workspace (``et_hip_linear_enqueue_static_workspace``):
        no allocation anywhere; plans that need more than ``STATIC_WORKSPACE_BYTES`` are refused; calls that
        overlap in time on one GPU race on the array."""
        self._check_input(x)
        self._check_weight(weight, bias)
        self._check_output(y)
        _check(N.lib().et_hip_linear_enqueue_static_workspace(
            self.requirements._handle, x.data_ptr(), x.stride(0), weight.data_ptr(),
            bias.data_ptr() if bias is not None else None, y.data_ptr(), _stream_handle(stream),
            cancelled.ptr if cancelled is not None else None))

    @property
    def prepared_input_bytes(self) -> int:
        """Bytes of the shared quantised activations this plan consumes; 0 = it reads x itself."""
        return int(N.lib().et_hip_linear_plan_prepared_input_bytes(self.requirements._handle))

    def prepare_input(self, x: torch.Tensor, prepared: torch.Tensor, stream=None) -> None:
        self._check_input(x)
        _check(N.lib().et_hip_linear_prepare_input(self.requirements._handle, x.data_ptr(), x.stride(0),
                                                   prepared.data_ptr(), prepared.numel() * prepared.element_size(),
                                                   _stream_handle(stream)))

    @property
    def fused_prepare(self) -> bool:
        """Whether :meth:`prepare_input_rms_norm` and :meth:`prepare_input_silu_mul` exist for this plan."""
        return bool(N.lib().et_hip_linear_plan_fused_prepare(self.requirements._handle))

    def _prepare_from(self, kind: int, x: torch.Tensor, second: Optional[torch.Tensor], eps: float,
                      prepared: torch.Tensor, stream) -> None:
        self._check_input(x)
        if second is not None:
            self._holds("second operand", second, second.element_size() * self.columns *
                        (self.vectors if kind == N.PREPARE_SILU_MUL else 1))
        source = N.EtPrepareSource(kind, x.data_ptr(), x.stride(0), second.data_ptr() if second is not None else None,
                                   float(eps), _weight_dtype(second))
        _check(N.lib().et_hip_linear_prepare_input_from(self.requirements._handle, ctypes.byref(source),
                                                        prepared.data_ptr(), prepared.numel() * prepared.element_size(),
                                                        _stream_handle(stream)))

    def prepare_input_rms_norm(self, x: torch.Tensor, weight: Optional[torch.Tensor], eps: float,
                               prepared: torch.Tensor, stream=None) -> None:
        """The prepared input of ``rms_norm(x) * weight`` without the operator's own launch: the same
        bytes as :func:`rms_norm_into` followed by :meth:`prepare_input`."""
        self._prepare_from(N.PREPARE_RMS_NORM, x, weight, eps, prepared, stream)

    def prepare_input_silu_mul(self, gate: torch.Tensor, up: torch.Tensor, prepared: torch.Tensor, stream=None) -> None:
        """The prepared input of ``silu(gate) * up`` (rows of ``up`` laid out like those of ``gate``)."""
        if up.stride(0) != gate.stride(0):
            raise QuantizedError(N.ERR_INVALID, "quantized_linear: gate and up must share their row stride")
        self._prepare_from(N.PREPARE_SILU_MUL, gate, up, 0.0, prepared, stream)

    def enqueue_prepared(self, prepared: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                         y: torch.Tensor, workspace: Optional[torch.Tensor] = None,
                         residual: Optional[torch.Tensor] = None, stream=None,
                         cancelled: Optional[CancellationFlag] = None) -> None:
        """``y = W x (+ bias) (+ residual)`` from activations prepared once by any plan of the same
        columns, vectors and activation mode; ``residual`` may be ``y``."""
        self._holds("prepared input", prepared, self.prepared_input_bytes)
        self._check_weight(weight, bias)
        self._check_output(y, residual)
        ws_ptr = workspace.data_ptr() if workspace is not None else None
        ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
        _check(N.lib().et_hip_linear_enqueue_prepared(
            self.requirements._handle, prepared.data_ptr(), weight.data_ptr(),
            bias.data_ptr() if bias is not None else None, residual.data_ptr() if residual is not None else None,
            y.data_ptr(), ws_ptr, ws_bytes, _stream_handle(stream), cancelled.ptr if cancelled is not None else None))

    def enqueue_prepared_then_norm(self, prepared: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                                   y: torch.Tensor, workspace: Optional[torch.Tensor], following: "RawLinear",
                                   norm_weight: Optional[torch.Tensor], eps: float, next_prepared: torch.Tensor,
                                   residual: Optional[torch.Tensor] = None, stream=None,
                                   cancelled: Optional[CancellationFlag] = None) -> None:
        """:meth:`enqueue_prepared`, then ``next_prepared`` = the prepared input of
        ``rms_norm(y) * norm_weight`` for ``following`` (``et_hip_linear_enqueue_prepared_then_norm``):
        the same bytes as the two calls, one launch less where this plan shares K over workgroups."""
        self._holds("prepared input", prepared, self.prepared_input_bytes)
        self._check_weight(weight, bias)
        self._check_output(y, residual)
        if norm_weight is not None:
            self._holds("norm weight", norm_weight, norm_weight.element_size() * self.rows)
        ws_ptr = workspace.data_ptr() if workspace is not None else None
        ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
        _check(N.lib().et_hip_linear_enqueue_prepared_then_norm(
            self.requirements._handle, prepared.data_ptr(), weight.data_ptr(),
            bias.data_ptr() if bias is not None else None, residual.data_ptr() if residual is not None else None,
            y.data_ptr(), ws_ptr, ws_bytes, following.requirements._handle,
            norm_weight.data_ptr() if norm_weight is not None else None, _weight_dtype(norm_weight), float(eps),
            next_prepared.data_ptr(),
            next_prepared.numel() * next_prepared.element_size(), _stream_handle(stream),
            cancelled.ptr if cancelled is not None else None))


def _weight_dtype(weight: Optional[torch.Tensor]) -> int:
    """``et_dtype`` of a second operand: f32, or f16 for an rms norm weight held as half floats."""
    if weight is None or weight.dtype == torch.float32:
        return N.DTYPE_F32
    if weight.dtype == torch.float16:
        return N.DTYPE_F16
    raise QuantizedError(N.ERR_UNSUPPORTED, f"quantized_linear: second operand of dtype {weight.dtype}")


class LinearGroup:
    """Up to four :class:`RawLinear` plans of the same columns and vectors that run from one prepared
    input in one launch (``et_hip_linear_enqueue_prepared_group``)."""

    def __init__(self, plans: Sequence["RawLinear"]):
        self.plans = list(plans)
        self._handles = (ctypes.c_void_p * len(self.plans))(*[p.requirements._handle for p in self.plans])
        size = ctypes.c_uint64()
        _check(N.lib().et_hip_linear_group_workspace_bytes(self._handles, len(self.plans), ctypes.byref(size)))
        self.workspace_bytes = int(size.value)

    def enqueue_prepared(self, prepared: torch.Tensor, weights: Sequence[torch.Tensor],
                         ys: Sequence[torch.Tensor], workspace: Optional[torch.Tensor] = None,
                         biases: Optional[Sequence[Optional[torch.Tensor]]] = None,
                         residuals: Optional[Sequence[Optional[torch.Tensor]]] = None, stream=None,
                         cancelled: Optional[CancellationFlag] = None) -> None:
        count = len(self.plans)
        self._check_members(prepared, weights, ys, biases, residuals)
        pointers = lambda tensors: (ctypes.c_void_p * count)(  # noqa: E731
            *[t.data_ptr() if t is not None else None for t in tensors])
        _check(N.lib().et_hip_linear_enqueue_prepared_group(
            self._handles, count, prepared.data_ptr(), pointers(weights),
            pointers(biases) if biases is not None else None,
            pointers(residuals) if residuals is not None else None, pointers(ys),
            workspace.data_ptr() if workspace is not None else None,
            workspace.numel() * workspace.element_size() if workspace is not None else 0,
            _stream_handle(stream), cancelled.ptr if cancelled is not None else None))

    def shares_layout(self) -> "N.EtGroupShares":
        """Where :meth:`enqueue_prepared_shares` leaves the K shares (``count`` <= 1: this group does not
        share K over workgroups; ``et_hip_linear_group_shares_layout``)."""
        layout = N.EtGroupShares()
        _check(N.lib().et_hip_linear_group_shares_layout(self._handles, len(self.plans), ctypes.byref(layout)))
        return layout

    def enqueue_prepared_shares(self, prepared: torch.Tensor, weights: Sequence[torch.Tensor], workspace: torch.Tensor,
                                stream=None, cancelled: Optional[CancellationFlag] = None) -> "N.EtGroupShares":
        """The group's launch without the one that sums its K shares: ``workspace`` keeps them for the
        launch that takes the results (``et_hip_linear_enqueue_prepared_group_shares``)."""
        count = len(self.plans)
        if len(weights) != count:
            raise QuantizedError(N.ERR_INVALID, f"quantized_linear: a group of {count} plans takes {count} weights")
        self.plans[0]._holds("prepared input", prepared, self.plans[0].prepared_input_bytes)
        for index, plan in enumerate(self.plans):
            plan._check_weight(weights[index])
        layout = N.EtGroupShares()
        _check(N.lib().et_hip_linear_enqueue_prepared_group_shares(
            self._handles, count, prepared.data_ptr(), (ctypes.c_void_p * count)(*[w.data_ptr() for w in weights]),
            workspace.data_ptr(), workspace.numel() * workspace.element_size(), ctypes.byref(layout),
            _stream_handle(stream), cancelled.ptr if cancelled is not None else None))
        return layout

    def _check_members(self, prepared, weights, ys, biases, residuals) -> None:
        """Every member's operands hold what its plan touches (see RawLinear._holds)."""
        count = len(self.plans)
        if len(weights) != count or len(ys) != count:
            raise QuantizedError(N.ERR_INVALID, f"quantized_linear: a group of {count} plans takes {count} weights and results")
        self.plans[0]._holds("prepared input", prepared, self.plans[0].prepared_input_bytes)
        for index, plan in enumerate(self.plans):
            plan._check_weight(weights[index], biases[index] if biases is not None else None)
            plan._check_output(ys[index], residuals[index] if residuals is not None else None)

    def enqueue_prepared_then_rotary(self, prepared: torch.Tensor, weights: Sequence[torch.Tensor],
                                     ys: Sequence[torch.Tensor], workspace: Optional[torch.Tensor],
                                     rotate: Sequence[int], offsets: torch.Tensor, theta: float, sign: float, layout: int,
                                     head_dim: int, biases=None, residuals=None, stream=None,
                                     cancelled: Optional[CancellationFlag] = None) -> None:
        """:meth:`enqueue_prepared`, then the rotary embedding in place on the results of the members
        listed in ``rotate`` (``[vectors, rows / head_dim, 1, head_dim]`` at ``offsets``), in the launch
        that sums the K shares where there is one (``et_hip_linear_enqueue_prepared_group_then_rotary``)."""
        _group_then_rotary(self, prepared, weights, ys, workspace, rotate, offsets, theta, sign, layout, head_dim,
                           biases, residuals, stream, cancelled)


def _group_then_rotary(group: "LinearGroup", prepared, weights, ys, workspace, rotate, offsets, theta, sign, layout,
                       head_dim, biases, residuals, stream, cancelled) -> None:
    count = len(group.plans)
    group._check_members(prepared, weights, ys, biases, residuals)
    pointers = lambda tensors: (ctypes.c_void_p * count)(  # noqa: E731
        *[t.data_ptr() if t is not None else None for t in tensors])
    if offsets.dtype not in (torch.uint32, torch.int32) or not offsets.is_contiguous():
        raise ValueError("rotary offsets must be a contiguous u32 device tensor")
    if offsets.numel() not in (1, group.plans[0].vectors):
        raise QuantizedError(N.ERR_INVALID, f"rotary embedding: {offsets.numel()} offsets for batch {group.plans[0].vectors}")
    after = N.EtRotaryAfter(sum(1 << i for i in rotate), offsets.data_ptr(), offsets.numel(), float(theta), float(sign),
                            int(layout), int(head_dim))
    _check(N.lib().et_hip_linear_enqueue_prepared_group_then_rotary(
        group._handles, count, prepared.data_ptr(), pointers(weights),
        pointers(biases) if biases is not None else None,
        pointers(residuals) if residuals is not None else None, pointers(ys),
        workspace.data_ptr() if workspace is not None else None,
        workspace.numel() * workspace.element_size() if workspace is not None else 0,
        ctypes.byref(after), _stream_handle(stream), cancelled.ptr if cancelled is not None else None))


HANDOVER_DEFAULT_SPIN_LIMIT = 0xFFFFFFFF


def handover_timeouts() -> int:
    """Waves of this process that have abandoned a bounded wait on another wave in a GEMV kernel on the
    current device (0 on a healthy run). Synchronises with the device."""
    count = ctypes.c_uint64(0)
    _check(N.lib().et_hip_handover_timeouts(ctypes.byref(count)))
    return int(count.value)


def set_handover_spin_limit(limit: int = HANDOVER_DEFAULT_SPIN_LIMIT) -> None:
    """Test hook: polls after which a wave gives up such a wait (0: at once; the default restores the
    library's own limit)."""
    N.lib().et_hip_test_set_handover_spin_limit(ctypes.c_uint32(limit))


def calibration_read(src: torch.Tensor, sink: torch.Tensor, workgroups: int, stream=None) -> None:
    """Plain streaming read of ``src`` (measurement aid, ``et_hip_calibration_read``)."""
    assert sink.numel() >= 4 * workgroups and sink.element_size() == 4
    _check_calibration(N.calibrate_lib().et_hip_calibration_read(src.data_ptr(), src.numel() * src.element_size(),
                                           sink.data_ptr(), workgroups, _stream_handle(stream)))


READ_VARIANTS = {"plain": 0, "deep": 1, "streaming": 2, "lds4": 3, "lds8": 4, "lds8_nt": 5, "lds8_nt_shallow": 6,
                 "lds8_nt_ranges": 7, "lds8_nt_ranges_shallow": 8}


def calibration_read_variant(variant: str, src: torch.Tensor, sink: torch.Tensor, workgroups: int, stream=None) -> None:
    """The streaming read by one of several kernels (measurement aid, ``et_hip_calibration_read_variant``)."""
    assert sink.numel() >= max(4 * workgroups, 1024) and sink.element_size() == 4
    _check_calibration(N.calibrate_lib().et_hip_calibration_read_variant(READ_VARIANTS[variant], src.data_ptr(),
                                                   src.numel() * src.element_size(), sink.data_ptr(), workgroups,
                                                   _stream_handle(stream)))


def calibration_copy(src: torch.Tensor, dst: torch.Tensor, stream=None) -> None:
    """Plain copy ``dst <- src`` (measurement aid, ``et_hip_calibration_copy``)."""
    _check_calibration(N.calibrate_lib().et_hip_calibration_copy(src.data_ptr(), dst.data_ptr(),
                                           src.numel() * src.element_size(), _stream_handle(stream)))


MFMA_KINDS = {"i8": 0, "i8_scaled": 1, "f16": 2, "f16_16x16": 3, "i8_scaled_bf16": 4, "i8_biased": 5,
              "i8_biased_matrix_only": 6, "i8_biased_valu_only": 7}
MFMA_OPERATIONS = {"i8": 65536, "i8_scaled": 65536, "f16": 32768, "f16_16x16": 16384, "i8_scaled_bf16": 65536,
                   "i8_biased": 65536, "i8_biased_matrix_only": 65536, "i8_biased_valu_only": 65536}


CONTRACTION_PROBES = {"whole": 0, "no_arithmetic": 1, "no_copies": 2, "no_weight_copies": 3, "no_activation_copies": 4,
                      "weight_copies_only": 5, "activation_copies_only": 6}


def calibration_contraction(probe: str, plan: "RawLinear", weight: torch.Tensor, prepared: torch.Tensor, y: torch.Tensor,
                            stream=None) -> None:
    """The batched Q4_K contraction of ``plan`` as it is (``whole``) or with a part left out (measurement
    aid, ``et_hip_calibration_contraction``; ``y`` is meaningful for ``whole`` only)."""
    plan._holds("prepared input", prepared, plan.prepared_input_bytes)
    plan._check_weight(weight)
    plan._check_output(y)
    _check_calibration(N.calibrate_lib().et_hip_calibration_contraction(CONTRACTION_PROBES[probe], weight.data_ptr(), prepared.data_ptr(),
                                                  y.data_ptr(), plan.rows, plan.columns, plan.vectors,
                                                  _stream_handle(stream)))


def calibration_mfma(kind: str, iterations: int, sink: torch.Tensor, stream=None) -> None:
    """Rounds of four independent matrix-core instructions per wave, no memory traffic (measurement
    aid, ``et_hip_calibration_mfma``); ``sink`` is f32 with 256 elements per workgroup."""
    if sink.dtype != torch.float32 or sink.numel() % 256 != 0 or sink.numel() == 0:
        raise ValueError("calibration_mfma: sink must be f32 with a multiple of 256 elements")
    _check_calibration(N.calibrate_lib().et_hip_calibration_mfma(MFMA_KINDS[kind], iterations, sink.numel() // 256, sink.data_ptr(),
                                           _stream_handle(stream)))
