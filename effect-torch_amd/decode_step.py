"""One batched decode step of a Llama-shaped model over the operators of this package, and the
loop around it.

The reference runs batched decode as a fixed-shape program ``[decodeBatch, 1]`` over per-sequence
key/value state (packages/core/src/Model.ts:1906-1975): every step embeds one token per sequence,
runs the layers against the paged cache at the sequences' cursors, takes the last (only) row of
logits per sequence, samples it (greedy: crates/runtime/src/sampling.rs:86-103), commits
``cursor += advance`` (crates/runtime-cpu/src/napi/mod.rs:4511-4517) and feeds the sampled token to
the next step. :class:`LlamaDecoder` is that step with all of its state on the device - the token
buffer is both the step's input and where greedy selection leaves the next input, the cursors are
advanced by a kernel - so that one captured HIP graph, replayed, IS the decode loop: no host round
trip between steps.

Storage types follow the model files this path serves: linear weights packed (Q4_K ...), embedding
table and norm weights as half floats, widened on use.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import torch

from .decode_ops import (RotaryLayout, add_into, gather_rows_into, greedy_tokens, greedy_workspace_bytes,
                         rms_norm_into, rotary_into, rotary_pair_into, silu_mul_into)
from .kv_cache import (KvLayer, kv_attention_into, kv_attention_kernel, kv_attention_projected_into,
                       kv_attention_workspace, kv_commit)
from .quantized import ActivationMode, GgmlQuant, LinearGroup, RawLinear

LINEARS = ("wq", "wk", "wv", "wo", "gate", "up", "down")


@dataclass
class LlamaShape:
    hidden: int = 4096
    heads: int = 32
    kv_heads: int = 8
    head_dim: int = 128
    ffn: int = 14336
    vocab: int = 128256
    layers: int = 32
    rope_theta: float = 500000.0
    eps: float = 1e-5

    def linear_shapes(self) -> Dict[str, tuple]:
        kv = self.kv_heads * self.head_dim
        return {"wq": (self.hidden, self.hidden), "wk": (kv, self.hidden), "wv": (kv, self.hidden),
                "wo": (self.hidden, self.hidden), "gate": (self.ffn, self.hidden), "up": (self.ffn, self.hidden),
                "down": (self.hidden, self.ffn), "head": (self.vocab, self.hidden)}


class LlamaDecoder:
    """Device state and launch sequence of one decode step for ``slots`` sequences.

    ``weights[layer][name]``: packed ``[rows, row_bytes]`` u8 for the seven linears of a layer;
    ``head``: the packed output projection; ``norms[layer]``: ``[2, hidden]`` (attention norm, ffn
    norm) and ``final_norm`` ``[hidden]``, f16 or f32; ``embedding``: ``[vocab, hidden]`` f16 or f32;
    ``kv[layer]``: the layer's :class:`KvLayer` (all layers share ``cursors`` / ``advances``);
    ``tokens``: int32 ``[slots]``, the step's input and, after the step, the next one's.

    ``fused``: one quantisation per distinct input, residual sums in the contraction epilogues,
    norms / SiLU * up / rotary computed inside the launches next to them where the plans can
    (``on_the_fly``); otherwise one launch sequence per operator, as the reference's executor runs
    them. The results agree within the f32 bars either way.
    """

    def __init__(self, shape: LlamaShape, codec: GgmlQuant, slots: int, weights: Sequence[Dict[str, torch.Tensor]],
                 head: torch.Tensor, norms: Sequence[torch.Tensor], final_norm: torch.Tensor,
                 embedding: torch.Tensor, kv: Sequence[KvLayer], tokens: torch.Tensor, *,
                 mode: ActivationMode = ActivationMode.F32, fused: bool = True):
        self.shape, self.slots, self.weights, self.head = shape, slots, weights, head
        self.norms, self.final_norm, self.embedding, self.kv, self.tokens = norms, final_norm, embedding, kv, tokens
        self.layers = len(weights)
        assert len(norms) == self.layers and len(kv) == self.layers
        device = head.device
        self.device = device
        shapes = shape.linear_shapes()
        self.plans = {name: RawLinear(codec, rows, columns, slots, False, mode) for name, (rows, columns) in shapes.items()}
        plans = self.plans
        u8 = lambda n: torch.empty(max(n, 16), dtype=torch.uint8, device=device)  # noqa: E731
        f32 = lambda *dims: torch.empty(dims, device=device)  # noqa: E731
        self.linear_ws = u8(max(p.requirements.workspace_bytes for p in plans.values()))
        self.fused = fused
        self.shared_hidden = u8(plans["wq"].prepared_input_bytes)
        self.shared_ffn = u8(plans["down"].prepared_input_bytes)
        self.shared_attended = u8(plans["wo"].prepared_input_bytes)
        self.on_the_fly = fused and all(plans[name].fused_prepare for name in ("wq", "gate", "down", "head"))
        if self.on_the_fly:
            self.qkv_group = LinearGroup([plans["wq"], plans["wk"], plans["wv"]])
            self.ffn_group = LinearGroup([plans["gate"], plans["up"]])
            self.group_ws = u8(max(self.qkv_group.workspace_bytes, self.ffn_group.workspace_bytes))
        self.kv_ws = kv_attention_workspace(kv[0], shape.heads, 1)
        # q / k / v can stay the K shares of their group launch when the attention kernel is the one that sums them
        self.project_in_attention = (self.on_the_fly and self.qkv_group.shares_layout().count > 1 and
                                     kv_attention_kernel(kv[0], shape.heads, 1).split("+")[0] == "kv_attend")
        self.greedy_ws = u8(greedy_workspace_bytes(slots, shape.vocab))
        kv_width = shape.kv_heads * shape.head_dim
        self.x, self.h = f32(slots, shape.hidden), f32(slots, shape.hidden)
        self.q, self.k, self.v = f32(slots, shape.hidden), f32(slots, kv_width), f32(slots, kv_width)
        self.attended, self.projected = f32(slots, shape.hidden), f32(slots, shape.hidden)
        self.gate, self.up, self.down = f32(slots, shape.ffn), f32(slots, shape.ffn), f32(slots, shape.hidden)
        self.logits = f32(slots, shape.vocab)
        self.scale = 1.0 / float(shape.head_dim) ** 0.5
        self.status: List[torch.Tensor] = []  # device status blocks of the step's calls, for checks after a fence
        self.cursors = kv[0].cursors

    # ------------------------------------------------------------------ pieces of a step
    def embed(self) -> None:
        """x = embedding[tokens], widened to f32."""
        self.status.append(gather_rows_into(self.embedding, self.tokens.view(torch.uint32), self.x, synchronize=False))

    def _after_down(self, index: int):
        if index + 1 < self.layers:
            return self.plans["wq"], self.norms[index + 1][0]
        return self.plans["head"], self.final_norm

    def layer_step(self, index: int, prepared_by_previous: bool = False) -> None:
        """Layer ``index`` on the residual stream ``x`` (in place). ``prepared_by_previous``: the call
        before (the previous layer, on the fly) has already left this layer's normed input behind."""
        s, plans, w, kvl = self.shape, self.plans, self.weights[index], self.kv[index]
        slots, width = self.slots, s.head_dim
        x, h, q, k, v = self.x, self.h, self.q, self.k, self.v
        theta, eps, half_split = s.rope_theta, s.eps, RotaryLayout.HALF_SPLIT
        q4 = q.view(slots, s.heads, 1, width)
        k4, v4 = k.view(slots, s.kv_heads, 1, width), v.view(slots, s.kv_heads, 1, width)
        attended4 = self.attended.view(slots, s.heads, 1, width)
        if self.on_the_fly:
            if not prepared_by_previous:
                plans["wq"].prepare_input_rms_norm(x, self.norms[index][0], eps, self.shared_hidden)
            if self.project_in_attention:
                # the attention kernel sums the group's K shares, rotates q and k at the slots' cursors,
                # appends, attends and quantises its result for Wo
                shares = self.qkv_group.enqueue_prepared_shares(self.shared_hidden, [w["wq"], w["wk"], w["wv"]],
                                                                self.group_ws)
                self.status.append(kv_attention_projected_into(
                    kvl, shares, (0, 1, 2), (None, None, None), self.cursors, theta, 1.0, half_split, self.scale, None,
                    attended4, workspace=self.kv_ws, synchronize=False, prepared_for=plans["wo"],
                    prepared=self.shared_attended))
            else:
                # q and k rotated at the slots' cursors in the launch that sums the group's K shares
                self.qkv_group.enqueue_prepared_then_rotary(self.shared_hidden, [w["wq"], w["wk"], w["wv"]], [q, k, v],
                                                            self.group_ws, (0, 1), self.cursors, theta, 1.0, half_split,
                                                            width)
                # the attention kernel quantises its result for Wo in its epilogue
                self.status.append(kv_attention_into(kvl, q4, k4, v4, self.scale, None, attended4, workspace=self.kv_ws,
                                                     synchronize=False, prepared_for=plans["wo"],
                                                     prepared=self.shared_attended))
            # x += attended Wo, then the ffn norm inside the quantiser, in the launch that sums Wo's K shares
            plans["wo"].enqueue_prepared_then_norm(self.shared_attended, w["wo"], None, x, self.linear_ws, plans["gate"],
                                                   self.norms[index][1], eps, self.shared_hidden, residual=x)
            self.ffn_group.enqueue_prepared(self.shared_hidden, [w["gate"], w["up"]], [self.gate, self.up], self.group_ws)
            plans["down"].prepare_input_silu_mul(self.gate, self.up, self.shared_ffn)
            following, norm_weight = self._after_down(index)
            plans["down"].enqueue_prepared_then_norm(self.shared_ffn, w["down"], None, x, self.linear_ws, following,
                                                     norm_weight, eps, self.shared_hidden, residual=x)
            return
        rms_norm_into(x, self.norms[index][0], eps, h)
        if self.fused:
            plans["wq"].prepare_input(h, self.shared_hidden)
            for name, out in (("wq", q), ("wk", k), ("wv", v)):
                plans[name].enqueue_prepared(self.shared_hidden, w[name], None, out, self.linear_ws)
            rotary_pair_into(q4, k4, self.cursors, theta, 1.0, half_split, q4, k4)
        else:
            for name, out in (("wq", q), ("wk", k), ("wv", v)):
                plans[name].enqueue(h, w[name], None, out, self.linear_ws)
            rotary_into(q4, self.cursors, theta, 1.0, half_split, q4)
            rotary_into(k4, self.cursors, theta, 1.0, half_split, k4)
        self.status.append(kv_attention_into(kvl, q4, k4, v4, self.scale, None, attended4, workspace=self.kv_ws,
                                             synchronize=False))
        if self.fused:
            plans["wo"].prepare_input(self.attended, self.shared_hidden)
            plans["wo"].enqueue_prepared(self.shared_hidden, w["wo"], None, x, self.linear_ws, residual=x)
        else:
            plans["wo"].enqueue(self.attended, w["wo"], None, self.projected, self.linear_ws)
            add_into(x, self.projected, x)
        rms_norm_into(x, self.norms[index][1], eps, h)
        if self.fused:
            plans["gate"].prepare_input(h, self.shared_hidden)
            plans["gate"].enqueue_prepared(self.shared_hidden, w["gate"], None, self.gate, self.linear_ws)
            plans["up"].enqueue_prepared(self.shared_hidden, w["up"], None, self.up, self.linear_ws)
        else:
            plans["gate"].enqueue(h, w["gate"], None, self.gate, self.linear_ws)
            plans["up"].enqueue(h, w["up"], None, self.up, self.linear_ws)
        silu_mul_into(self.gate, self.up, self.gate)
        if self.fused:
            plans["down"].prepare_input(self.gate, self.shared_ffn)
            plans["down"].enqueue_prepared(self.shared_ffn, w["down"], None, x, self.linear_ws, residual=x)
        else:
            plans["down"].enqueue(self.gate, w["down"], None, self.down, self.linear_ws)
            add_into(x, self.down, x)

    def project(self) -> None:
        """logits = head(final_norm(x))."""
        if self.on_the_fly:  # the last layer has left the normed, prepared x behind
            self.plans["head"].enqueue_prepared(self.shared_hidden, self.head, None, self.logits, self.linear_ws)
        else:
            rms_norm_into(self.x, self.final_norm, self.shape.eps, self.h)
            self.plans["head"].enqueue(self.h, self.head, None, self.logits, self.linear_ws)

    def select_and_commit(self) -> None:
        """tokens = greedy(logits): the next step's input; cursors += advances."""
        self.status.append(greedy_tokens(self.logits, workspace=self.greedy_ws, synchronize=False,
                                         tokens=self.tokens)[1])
        kv_commit(self.kv[0])

    def step(self) -> None:
        """Enqueues one whole decode step; every piece of state it leaves is what the next step reads."""
        self.status.clear()
        self.embed()
        for index in range(self.layers):
            self.layer_step(index, prepared_by_previous=self.on_the_fly and index > 0)
        self.project()
        self.select_and_commit()


def algorithmic_bytes_per_step(shape: LlamaShape, codec: GgmlQuant, slots: int, layers: int, context: int,
                               kv_row_bytes: int) -> Dict[str, int]:
    """Bytes one step must move: every packed weight once, every cached key / value row once, the
    logits written and read once."""
    shapes = shape.linear_shapes()
    per_layer = sum(rows * codec.encoded_row_bytes(columns) for name, (rows, columns) in shapes.items() if name != "head")
    head = shapes["head"][0] * codec.encoded_row_bytes(shapes["head"][1])
    weights = layers * per_layer + head
    kv = layers * 2 * slots * context * shape.kv_heads * kv_row_bytes
    return {"weights": weights, "kv": kv, "logits": slots * shape.vocab * 4 * 2}
