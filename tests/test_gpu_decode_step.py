"""Batched decode, chained: several consecutive steps of a two-layer Llama-3-8B-shaped model on the
GPU against the CPU oracle's operators chained the same way.

The model has the end-to-end configuration's shapes (hidden 4096, 32 query heads over 8 kv heads of
width 128, ffn 14336, vocabulary 128256, RoPE theta 500000, Q4_K linears including the output
projection, half-float embedding table and norm weights widened on use, half-float paged key/value
slabs in blocks of 16) with two layers and short ragged contexts, so that the oracle - a scalar loop
on one core - follows in seconds. 32 slots decode on the GPU; four of them are followed by the oracle.

The loop is the reference's (packages/core/src/Model.ts:1906-1975, crates/runtime/src/sampling.rs:86-103,
crates/runtime-cpu/src/napi/mod.rs:4511-4517): embed the slot's token, run the layers against the
cache at the slot's cursor, take greedy tokens from the logits, advance the cursors, feed the tokens back.

Bars: embedding rows exact; residual stream after every layer and the full logits rows within
``1e-3 * max(|want|, 1)`` plus the oracle's own summation noise (``close`` of test_gpu_parity); greedy
tokens equal to the oracle chain's; cursors exact; appended slab rows within one half-float step of
the element plus the f32 bar at the row's scale.
"""
import numpy as np
import pytest
import torch

import oracle
from effect_torch_amd import synth
from test_gpu_parity import close

pytestmark = pytest.mark.gpu

def followed_slots(slots):
    """The slots the oracle follows: the first, the last and two in between."""
    return sorted({0, 9 % slots, 20 % slots, slots - 1})


STEPS = 3


def tiled_rows(base, rows):
    """`rows` rows: the base block over and over, each repeat rolled by one more row."""
    repeats = -(-rows // base.shape[0])
    return np.concatenate([np.roll(base, r, axis=0) for r in range(repeats)])[:rows]


class Model:
    def __init__(self, et, device, layers, slots, fused, contexts=(40, 200)):
        rng = np.random.default_rng(0x11A3A + layers)
        self.shape = shape = et.LlamaShape(layers=layers)
        self.shapes = shapes = shape.linear_shapes()
        self.slots, self.layers = slots, layers
        self.followed = followed_slots(slots)
        Q4K = synth.Q4_K
        # every matrix at its full height; only the output projection is a block of 8192 rows tiled
        base = {name: synth.random_weight(Q4K, 8192 if name == "head" else rows, columns, rng)
                for name, (rows, columns) in shapes.items()}
        self.host_weights = [{name: (np.roll(base[name], layer, axis=0) if layer else base[name])
                              for name in shapes if name != "head"} for layer in range(layers)]
        self.host_head = tiled_rows(base["head"], shape.vocab)
        for layer in self.host_weights:  # what the plans will read is what the buffers hold
            for name, weight in layer.items():
                assert weight.shape == (shapes[name][0], synth.row_bytes(Q4K, shapes[name][1])), name
        assert self.host_head.shape == (shape.vocab, synth.row_bytes(Q4K, shape.hidden))
        self.norms_host = [(1.0 + 0.1 * rng.standard_normal((2, shape.hidden))).astype(np.float16) for _ in range(layers)]
        self.final_norm_host = (1.0 + 0.1 * rng.standard_normal(shape.hidden)).astype(np.float16)
        self.embedding_base = rng.standard_normal((4096, shape.hidden)).astype(np.float16)  # row t = base[t % 4096]
        block = 16
        self.block = block
        self.contexts = rng.integers(contexts[0], contexts[1], slots).astype(np.uint32)
        self.max_context = int(self.contexts.max()) + STEPS
        blocks_per_slot = -(-self.max_context // block)
        total_blocks = slots * blocks_per_slot + 5
        self.table_host = rng.permutation(total_blocks)[: slots * blocks_per_slot].reshape(slots, blocks_per_slot).astype(np.uint32)
        self.slabs_host = [[rng.standard_normal((total_blocks * block, shape.kv_heads, shape.head_dim)).astype(np.float16)
                            for _ in range(2)] for _ in range(layers)]
        self.tokens_host = rng.integers(0, shape.vocab, slots).astype(np.int32)

        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
        weights = [{name: dev(w) for name, w in layer.items()} for layer in self.host_weights]
        embedding = dev(self.embedding_base).repeat(-(-shape.vocab // 4096), 1)[: shape.vocab].contiguous()
        table = dev(self.table_host.view(np.int32))
        self.cursors = dev(self.contexts.view(np.int32))
        advances = torch.ones(slots, dtype=torch.int32, device=device)
        kv = [et.KvLayer(dev(k), dev(v), block, table, self.cursors, advances, self.max_context)
              for k, v in self.slabs_host]
        self.tokens = dev(self.tokens_host)
        self.decoder = et.LlamaDecoder(shape, et.GgmlQuant.Q4_K, slots, weights, dev(self.host_head),
                                       [dev(n) for n in self.norms_host], dev(self.final_norm_host), embedding, kv,
                                       self.tokens, fused=fused)

    # ---- the oracle's operators, chained like the decoder's, for the followed slots
    def linear(self, name, layer, x):
        rows, columns = self.shapes[name]
        weight = self.host_head if name == "head" else self.host_weights[layer][name]
        return oracle.linear_into(synth.Q4_K, rows, columns, x, weight)

    def oracle_layer(self, layer, x, cursors):
        s, n = self.shape, len(self.followed)
        norms = self.norms_host[layer].astype(np.float32)  # widened on use
        h = oracle.rms_norm(x, norms[0], s.eps)
        q = oracle.rotary(self.linear("wq", layer, h).reshape(n, s.heads, 1, s.head_dim), cursors, s.rope_theta)
        k = oracle.rotary(self.linear("wk", layer, h).reshape(n, s.kv_heads, 1, s.head_dim), cursors, s.rope_theta)
        v = self.linear("wv", layer, h).reshape(n, s.kv_heads, 1, s.head_dim)
        k_slab, v_slab = self.slabs_host[layer]
        attended = oracle.kv_attention(k_slab, v_slab, self.block, self.table_host[self.followed], cursors,
                                       np.ones(n, np.uint32), q, k, v, 1.0 / np.sqrt(s.head_dim))
        x = oracle.add(x, self.linear("wo", layer, attended.reshape(n, s.hidden)))
        h = oracle.rms_norm(x, norms[1], s.eps)
        return oracle.add(x, self.linear("down", layer, oracle.silu_mul(self.linear("gate", layer, h),
                                                                         self.linear("up", layer, h))))


@pytest.mark.parametrize("fused,slots,contexts", [(True, 32, (40, 200)), (False, 32, (40, 200)), (True, 12, (40, 200)),
                                                  (True, 32, (2030, 2060))],
                         ids=["fused", "one_operator_per_launch", "fused_12_slots", "fused_context_2048"])
def test_decode_steps_follow_the_oracle_chain(et, device, fused, slots, contexts):
    # 12 slots: the contractions' narrow tile, attention workgroups of four waves with the context split;
    # contexts around 2048: the end-to-end configuration's cache length (130 blocks of 16 per slot)
    layers = 2
    model = Model(et, device, layers, slots, fused, contexts)
    dec, shape = model.decoder, model.shape
    if fused:
        assert dec.on_the_fly, "the Q4_K plans of these shapes take their inputs on the fly"
    tokens_ref = model.tokens_host[model.followed].copy()
    cursors_ref = model.contexts[model.followed].copy()
    for step in range(STEPS):
        dec.status.clear()
        dec.embed()
        torch.cuda.synchronize()
        et.gather_rows_status_check(shape.vocab, dec.status[-1])
        assert np.array_equal(dec.tokens.cpu().numpy()[model.followed], tokens_ref), f"step {step}: input tokens differ"
        x_ref = model.embedding_base[tokens_ref % 4096].astype(np.float32)
        assert np.array_equal(dec.x.cpu().numpy()[model.followed].view(np.uint32), x_ref.view(np.uint32))
        for layer in range(layers):
            dec.layer_step(layer, prepared_by_previous=dec.on_the_fly and layer > 0)
            torch.cuda.synchronize()
            et.kv_attention_status_check(dec.kv[layer], 1, dec.status[-1])
            x_ref = model.oracle_layer(layer, x_ref, cursors_ref)
            close(dec.x.cpu().numpy()[model.followed], x_ref)
        dec.project()
        torch.cuda.synchronize()
        logits = dec.logits.cpu().numpy()
        logits_ref = model.linear("head", None, oracle.rms_norm(x_ref, model.final_norm_host.astype(np.float32), shape.eps))
        close(logits[model.followed], logits_ref)
        dec.select_and_commit()
        torch.cuda.synchronize()
        et.greedy_status_check(dec.status[-1])
        chosen = dec.tokens.cpu().numpy()
        assert np.array_equal(chosen, np.argmax(logits, axis=1).astype(np.int32)), "greedy tokens are not the argmax"
        want = oracle.argmax_rows(logits_ref).astype(np.int32)
        for i, slot in enumerate(model.followed):
            if chosen[slot] != want[i]:  # only a tie within the f32 bar may be decided differently
                gap = logits_ref[i, want[i]] - logits_ref[i, chosen[slot]]
                assert gap <= 1e-3 * max(abs(float(logits_ref[i, want[i]])), 1.0), (step, slot, chosen[slot], want[i], gap)
        tokens_ref = chosen[model.followed].copy()
        cursors_ref = cursors_ref + 1
        assert np.array_equal(dec.cursors.cpu().numpy().view(np.uint32), model.contexts + step + 1)
    # the rows the steps appended for the followed slots: the oracle's, within one half-float step
    for layer in range(layers):
        for which in range(2):
            slab = (dec.kv[layer].k_slab, dec.kv[layer].v_slab)[which].cpu().numpy()
            ref = model.slabs_host[layer][which]
            for i, slot in enumerate(model.followed):
                for position in range(int(model.contexts[slot]), int(model.contexts[slot]) + STEPS):
                    row = int(model.table_host[slot, position // model.block]) * model.block + position % model.block
                    # The two chains round f32 rows that agree within the f32 bar, and that bar follows the
                    # scale of the ROW (a contraction's error does not shrink with the element): one
                    # half-float step of the element plus 2e-4 of the row's largest value (+ 1e-3 at |row| <= 1).
                    mine, theirs = slab[row].astype(np.float64), ref[row].astype(np.float64)
                    scale = np.abs(theirs).max(axis=-1, keepdims=True)
                    assert np.all(np.abs(mine - theirs) <= 2.0 ** -10 * np.abs(theirs) + 2e-4 * scale + 1e-3), \
                        (layer, which, slot, position, float(np.abs(mine - theirs).max()), float(scale.max()))


def test_decode_loop_as_a_replayed_graph_matches_step_by_step_launches(et, device):
    # The benchmark's loop: ONE captured graph of a whole step, replayed; tokens, cursors and slabs
    # carry the state from replay to replay. The replays must leave what the same steps enqueued one
    # by one leave: the same tokens after every step, the same cursors, the same slabs.
    layers, slots, steps = 2, 32, 4
    eager = Model(et, device, layers, slots, True)
    graphed = Model(et, device, layers, slots, True)
    history = []
    for _ in range(steps):
        eager.decoder.step()
        torch.cuda.synchronize()
        history.append(eager.decoder.tokens.cpu().numpy().copy())
    dec = graphed.decoder
    # warm up outside the capture on a copy of the state, then restore it
    saved = (dec.tokens.clone(), dec.cursors.clone(), [(l.k_slab.clone(), l.v_slab.clone()) for l in dec.kv])
    dec.step()
    torch.cuda.synchronize()
    dec.tokens.copy_(saved[0])
    dec.cursors.copy_(saved[1])
    for layer, (k, v) in zip(dec.kv, saved[2]):
        layer.k_slab.copy_(k)
        layer.v_slab.copy_(v)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        dec.step()
    # capturing enqueues nothing: restore nothing, replay from the initial state
    for step in range(steps):
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(dec.tokens.cpu().numpy(), history[step]), f"replay {step}: tokens differ"
    assert np.array_equal(dec.cursors.cpu().numpy(), eager.decoder.cursors.cpu().numpy())
    assert np.array_equal(dec.cursors.cpu().numpy().view(np.uint32), graphed.contexts + steps)
    for a, b in zip(dec.kv, eager.decoder.kv):
        assert torch.equal(a.k_slab, b.k_slab) and torch.equal(a.v_slab, b.v_slab)
