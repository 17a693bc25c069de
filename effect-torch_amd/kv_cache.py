"""Host mirror of the reference's paged key/value cache for ONE layer, over torch device tensors.

``KvLayer`` holds what ``KvContext`` + ``PoolInner`` + ``SeqState`` hold for a layer
(crates/runtime-cpu/src/napi/mod.rs:2501-2513, :2623-2634, :2656-2664): the K / V slabs, the
block table, cursors and advances. ``kv_attention_into`` is the operator
(napi/mod.rs:3320-3544). Block allocation and eviction stay with the caller, as they stay on the
host in the reference.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from . import _native as N
from .quantized import CancellationFlag, QuantizedError, _check, _desc, _ref, _stream_handle

_SLAB_DTYPES = {torch.float32: N.DTYPE_F32, torch.float16: N.DTYPE_F16, torch.bfloat16: N.DTYPE_BF16,
                torch.uint8: N.DTYPE_U8}


class KvLayer:
    """Device state of one layer. ``k_slab`` / ``v_slab``: ``[max_tokens, kv_heads, head_dim]`` f32,
    f16, bf16 or uint8 (the int8-quantized tier, with f32 ``k_scales`` / ``v_scales``
    ``[max_tokens, kv_heads]``); ``block_table``: uint32/int32 ``[slots, table_stride]``; ``cursors`` / ``advances``:
    uint32/int32 ``[slots]``. ``max_context`` bounds ``cursor + advance`` (it sizes the launch)."""

    def __init__(self, k_slab: torch.Tensor, v_slab: torch.Tensor, block_size: int, block_table: torch.Tensor,
                 cursors: torch.Tensor, advances: torch.Tensor, max_context: int,
                 active_batch: Optional[int] = None, context_window: int = 0,
                 k_scales: Optional[torch.Tensor] = None, v_scales: Optional[torch.Tensor] = None):
        if k_slab.dtype not in _SLAB_DTYPES or v_slab.dtype != k_slab.dtype:
            raise QuantizedError(N.ERR_UNSUPPORTED, "kv pool: dtype must be f32, f16, bf16 or u8 (int8-quantized)")
        if k_slab.dtype == torch.uint8:
            for scales in (k_scales, v_scales):
                if scales is None or scales.dtype != torch.float32 or not scales.is_contiguous() or \
                        tuple(scales.shape) != tuple(k_slab.shape[:2]):
                    raise QuantizedError(N.ERR_UNSUPPORTED,
                                         "kv attention: the u8 tier needs contiguous f32 scales [tokens, heads]")
        elif k_scales is not None or v_scales is not None:
            raise QuantizedError(N.ERR_UNSUPPORTED, "kv attention: only the u8 tier has scale slabs")
        self.k_scales, self.v_scales = k_scales, v_scales
        if k_slab.dim() != 3 or k_slab.shape != v_slab.shape or not k_slab.is_contiguous() or \
                not v_slab.is_contiguous():
            raise QuantizedError(N.ERR_UNSUPPORTED, "kv attention: slabs must be contiguous [tokens, heads, width]")
        for name, t in (("block_table", block_table), ("cursors", cursors), ("advances", advances)):
            if t.dtype not in (torch.int32, torch.uint32) or not t.is_contiguous():
                raise QuantizedError(N.ERR_UNSUPPORTED, f"kv attention: {name} must be contiguous 32-bit integers")
        slots = cursors.numel()
        if block_table.dim() != 2 or block_table.shape[0] != slots or advances.numel() != slots:
            raise QuantizedError(N.ERR_UNSUPPORTED, "kv attention: block table, cursors and advances disagree")
        self.k_slab, self.v_slab = k_slab, v_slab
        self.block_table, self.cursors, self.advances = block_table, cursors, advances
        self.block_size = int(block_size)
        self.max_context = int(max_context)
        self.active_batch = slots if active_batch is None else int(active_batch)
        self.context_window = int(context_window)

    def struct(self) -> N.EtKvLayer:
        max_tokens, kv_heads, width = self.k_slab.shape
        return N.EtKvLayer(self.k_slab.data_ptr(), self.v_slab.data_ptr(), _SLAB_DTYPES[self.k_slab.dtype],
                           max_tokens, kv_heads, width, self.block_size, self.block_table.data_ptr(),
                           self.block_table.shape[1], self.cursors.data_ptr(), self.advances.data_ptr(),
                           self.cursors.numel(), self.active_batch, self.context_window, self.max_context,
                           self.k_scales.data_ptr() if self.k_scales is not None else None,
                           self.v_scales.data_ptr() if self.v_scales is not None else None)


def kv_attention_workspace_bytes(layer: KvLayer, query_heads: int, tokens: int) -> int:
    return int(N.lib().et_hip_kv_attention_workspace_bytes(ctypes.byref(layer.struct()), query_heads, tokens))


def kv_attention_workspace(layer: KvLayer, query_heads: int, tokens: int, device=None) -> torch.Tensor:
    """A workspace for these sizes; it can serve any number of calls that do not overlap in time."""
    need = kv_attention_workspace_bytes(layer, query_heads, tokens)
    return torch.empty(max(need, 16), dtype=torch.uint8, device=device or layer.k_slab.device)


def kv_attention_kernel(layer: KvLayer, query_heads: int, tokens: int) -> str:
    return N.lib().et_hip_kv_attention_kernel(ctypes.byref(layer.struct()), query_heads, tokens).decode()


def kv_commit(layer: "KvLayer", *, stream=None) -> None:
    """``cursor += advance`` for the layer's active slots, on the device (``et_hip_kv_commit``): the commit
    of a decode step (crates/runtime-cpu/src/napi/mod.rs:4511-4517). Layers sharing one cursor tensor are
    committed by one call."""
    _check(N.lib().et_hip_kv_commit(ctypes.byref(layer.struct()), _stream_handle(stream)))


def kv_attention_status_check(layer: KvLayer, tokens: int, status: torch.Tensor) -> None:
    host = status.cpu().numpy().tobytes()  # synchronises with the producing stream
    buf = ctypes.create_string_buffer(host, len(host))
    _check(N.lib().et_hip_kv_attention_status_check(ctypes.byref(layer.struct()), tokens, buf))


def kv_attention_into(layer: KvLayer, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                      window: Optional[int], destination: torch.Tensor, *,
                      workspace: Optional[torch.Tensor] = None, cancelled: Optional[CancellationFlag] = None,
                      stream=None, synchronize: bool = True, prepared_for=None,
                      prepared: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """kv_attention_into (napi/mod.rs:3320-3544): appends the new rows of ``k`` / ``v`` to the slabs,
    then attends. With ``synchronize`` (default) the stream is drained and a failed per-slot check
    raises the reference's error here; otherwise the device status block is returned for
    :func:`kv_attention_status_check` after the caller's own fence.

    ``prepared_for`` (a :class:`RawLinear` whose activations are the result, one token per slot) and
    ``prepared``: also leaves that plan's prepared input behind (``et_hip_kv_attention_prepared_into``)."""
    struct = layer.struct()
    tokens = q.shape[-2] if q.dim() >= 2 else 0
    heads = q.shape[-3] if q.dim() >= 3 else 0
    if workspace is None:
        need = 0
        if q.dim() >= 4 and heads and tokens:
            need = int(N.lib().et_hip_kv_attention_workspace_bytes(ctypes.byref(struct), heads, tokens))
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=destination.device)
    status = torch.empty(8 * max(layer.cursors.numel(), 1), dtype=torch.uint8, device=destination.device)
    descs = (_desc(q), _desc(k), _desc(v), _desc(destination))
    if prepared_for is not None:
        _check(N.lib().et_hip_kv_attention_prepared_into(
            ctypes.byref(struct), _ref(descs[0]), _ref(descs[1]), _ref(descs[2]), float(scale), int(window or 0),
            _ref(descs[3]), workspace.data_ptr(), workspace.numel(), status.data_ptr(),
            prepared_for.requirements._handle, prepared.data_ptr() if prepared is not None else None,
            prepared.numel() * prepared.element_size() if prepared is not None else 0, _stream_handle(stream),
            cancelled.ptr if cancelled is not None else None))
    else:
        _check(N.lib().et_hip_kv_attention_into(ctypes.byref(struct), _ref(descs[0]), _ref(descs[1]), _ref(descs[2]),
                                                float(scale), int(window or 0), _ref(descs[3]),
                                                workspace.data_ptr(), workspace.numel(), status.data_ptr(),
                                                _stream_handle(stream),
                                                cancelled.ptr if cancelled is not None else None))
    if not synchronize:
        return status
    kv_attention_status_check(layer, tokens, status)
    return None


def kv_attention_projected_into(layer: KvLayer, shares, members: Sequence[int],
                                biases: Sequence[Optional[torch.Tensor]], offsets: torch.Tensor, theta: float,
                                sign: float, layout: int, scale: float, window: Optional[int],
                                destination: torch.Tensor, *, workspace: Optional[torch.Tensor] = None,
                                cancelled: Optional[CancellationFlag] = None, stream=None, synchronize: bool = True,
                                prepared_for=None, prepared: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """:func:`kv_attention_into` for one token per slot whose q, k and v are still the unsummed K
    shares of their projections (``shares``: what ``LinearGroup.enqueue_prepared_shares`` returned;
    ``members``: which plans of that group are q, k and v; ``biases``: theirs, or None): the attention
    launch sums the rows it needs, adds the biases and rotates q and k at ``offsets`` before it attends
    (``et_hip_kv_attention_projected_into``). ``destination``: ``[.., query_heads, 1, head_dim]``."""
    struct = layer.struct()
    heads = destination.shape[-3] if destination.dim() >= 3 else 0
    if offsets.dtype not in (torch.uint32, torch.int32) or not offsets.is_contiguous():
        raise ValueError("rotary offsets must be a contiguous u32 device tensor")
    if workspace is None:
        need = int(N.lib().et_hip_kv_attention_workspace_bytes(ctypes.byref(struct), heads, 1)) if heads else 0
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=destination.device)
    status = torch.empty(8 * max(layer.cursors.numel(), 1), dtype=torch.uint8, device=destination.device)
    pointer = lambda t: t.data_ptr() if t is not None else None  # noqa: E731
    projected = N.EtKvProjected(shares, int(members[0]), int(members[1]), int(members[2]), pointer(biases[0]),
                                pointer(biases[1]), pointer(biases[2]), offsets.data_ptr(), offsets.numel(),
                                float(theta), float(sign), int(layout))
    desc = _desc(destination)
    _check(N.lib().et_hip_kv_attention_projected_into(
        ctypes.byref(struct), ctypes.byref(projected), float(scale), int(window or 0), _ref(desc),
        workspace.data_ptr(), workspace.numel(), status.data_ptr(),
        prepared_for.requirements._handle if prepared_for is not None else None,
        prepared.data_ptr() if prepared is not None else None,
        prepared.numel() * prepared.element_size() if prepared is not None else 0, _stream_handle(stream),
        cancelled.ptr if cancelled is not None else None))
    if not synchronize:
        return status
    kv_attention_status_check(layer, 1, status)
    return None
