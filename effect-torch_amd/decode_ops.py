"""Host mirror of the small operators of a decode step, over torch device tensors.

RMS norm (crates/runtime-cpu/src/composed.rs:1491), rotary embedding (:2735), SiLU(gate) * up
(packages/core/src/Tensor.ts:1537), greedy token selection (crates/runtime/src/sampling.rs:86) and
the dense embedding lookup (crates/runtime-cpu/src/indexing.rs:396). Every function enqueues one
kernel on the current stream and allocates only what it returns.
"""
from __future__ import annotations

import ctypes
import enum
from typing import Optional

import torch

from . import _native as N
from .quantized import QuantizedError, _check, _desc, _ref, _stream_handle


class RotaryLayout(enum.IntEnum):
    HALF_SPLIT = 0
    INTERLEAVED_PAIRS = 1


def rms_norm_into(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, destination: torch.Tensor, *,
                  stream=None) -> None:
    descs = (_desc(x), _desc(weight), _desc(destination))
    _check(N.lib().et_hip_rms_norm_into(_ref(descs[0]), _ref(descs[1]), float(eps), _ref(descs[2]),
                                        _stream_handle(stream)))


def rotary_into(x: torch.Tensor, offsets: torch.Tensor, theta: float, sign: float, layout: RotaryLayout,
                destination: torch.Tensor, *, stream=None) -> None:
    """``offsets``: device tensor of 1 or batch 32-bit integers (in a decode step, the kv cursors)."""
    if offsets.dtype not in (torch.int32, torch.uint32) or not offsets.is_contiguous():
        raise QuantizedError(N.ERR_UNSUPPORTED, "rotary: offsets must be contiguous 32-bit integers")
    descs = (_desc(x), _desc(destination))
    _check(N.lib().et_hip_rotary_into(_ref(descs[0]), offsets.data_ptr(), offsets.numel(), float(theta),
                                      float(sign), int(layout), _ref(descs[1]), _stream_handle(stream)))


def rotary_pair_into(x: torch.Tensor, second: torch.Tensor, offsets: torch.Tensor, theta: float, sign: float,
                     layout: RotaryLayout, destination: torch.Tensor, second_destination: torch.Tensor, *,
                     stream=None) -> None:
    """:func:`rotary_into` for two tensors of one batch, steps and head width (queries and keys) in one launch."""
    if offsets.dtype not in (torch.int32, torch.uint32) or not offsets.is_contiguous():
        raise QuantizedError(N.ERR_UNSUPPORTED, "rotary: offsets must be contiguous 32-bit integers")
    descs = (_desc(x), _desc(second), _desc(destination), _desc(second_destination))
    _check(N.lib().et_hip_rotary_pair_into(_ref(descs[0]), _ref(descs[1]), offsets.data_ptr(), offsets.numel(),
                                           float(theta), float(sign), int(layout), _ref(descs[2]), _ref(descs[3]),
                                           _stream_handle(stream)))


def add_into(a: torch.Tensor, b: torch.Tensor, destination: torch.Tensor, *, stream=None) -> None:
    descs = (_desc(a), _desc(b), _desc(destination))
    _check(N.lib().et_hip_add_into(_ref(descs[0]), _ref(descs[1]), _ref(descs[2]), _stream_handle(stream)))


def silu_mul_into(gate: torch.Tensor, up: torch.Tensor, destination: torch.Tensor, *, stream=None) -> None:
    descs = (_desc(gate), _desc(up), _desc(destination))
    _check(N.lib().et_hip_silu_mul_into(_ref(descs[0]), _ref(descs[1]), _ref(descs[2]), _stream_handle(stream)))


def greedy_status_check(status: torch.Tensor) -> None:
    host = status.cpu().numpy().tobytes()  # synchronises with the producing stream
    _check(N.lib().et_hip_greedy_status_check(len(host) // 4, ctypes.create_string_buffer(host, len(host))))


def greedy_workspace_bytes(rows: int, vocabulary: int) -> int:
    return int(N.lib().et_hip_greedy_workspace_bytes(rows, vocabulary))


def greedy_tokens(logits: torch.Tensor, *, workspace: Optional[torch.Tensor] = None, stream=None,
                  synchronize: bool = True, tokens: Optional[torch.Tensor] = None):
    """Greedy token per row of ``[.., vocabulary]`` logits as an int32 tensor (``tokens``, when given:
    a contiguous int32 tensor of one element per row that receives them). With ``synchronize`` a logit
    that is not finite raises the reference's error here; otherwise ``(tokens, status)``."""
    rows = logits.numel() // logits.shape[-1] if logits.dim() and logits.shape[-1] else 0
    if tokens is None:
        tokens = torch.empty(logits.shape[:-1], dtype=torch.int32, device=logits.device)
    elif tokens.dtype != torch.int32 or tokens.numel() != rows or not tokens.is_contiguous():
        raise QuantizedError(N.ERR_INVALID, "sample: tokens must be a contiguous int32 tensor of one element per row")
    status = torch.empty(4 * max(rows, 1), dtype=torch.uint8, device=logits.device)
    if workspace is None:
        need = greedy_workspace_bytes(rows, logits.shape[-1]) if rows else 0
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=logits.device)
    desc = _desc(logits)
    _check(N.lib().et_hip_greedy_tokens_into(_ref(desc), tokens.data_ptr(), workspace.data_ptr(), workspace.numel(),
                                             status.data_ptr(), _stream_handle(stream)))
    if not synchronize:
        return tokens, status
    greedy_status_check(status[:4 * rows])
    return tokens


def gather_rows_status_check(table_rows: int, status: torch.Tensor) -> None:
    host = status.cpu().numpy().tobytes()
    _check(N.lib().et_hip_gather_rows_status_check(table_rows, len(host) // 8,
                                                   ctypes.create_string_buffer(host, len(host))))


def gather_rows_into(table: torch.Tensor, indexes: torch.Tensor, destination: torch.Tensor, *, stream=None,
                     synchronize: bool = True) -> Optional[torch.Tensor]:
    """``destination[p, :] = table[indexes[p], :]`` for a ``[rows, width]`` table; ``destination`` is
    ``[indexes.numel(), width]`` of the table's dtype."""
    count = indexes.numel()
    status = torch.empty(8 * max(count, 1), dtype=torch.uint8, device=destination.device)
    descs = (_desc(table), _desc(indexes), _desc(destination))
    _check(N.lib().et_hip_gather_rows_into(_ref(descs[0]), _ref(descs[1]), _ref(descs[2]), status.data_ptr(),
                                           _stream_handle(stream)))
    if not synchronize:
        return status
    gather_rows_status_check(table.shape[0], status[:8 * count])
    return None
