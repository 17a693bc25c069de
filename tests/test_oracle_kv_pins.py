"""Pins of the paged KV attention oracle (CPU only; see oracle/et_oracle_kv.h for the list)."""
import numpy as np
import pytest

import oracle


def dense_attention(q, keys, values, scale, begin_of, end_of):
    """Independent statement: softmax(q K^T * scale) V in float64, one (head, query) at a time."""
    batch, heads, tokens, width = q.shape
    out = np.zeros(q.shape, np.float64)
    group = heads // keys.shape[1]
    for b in range(batch):
        for h in range(heads):
            for t in range(tokens):
                lo, hi = begin_of(b, t), end_of(b, t)
                kk = keys[b, h // group, lo:hi].astype(np.float64)
                vv = values[b, h // group, lo:hi].astype(np.float64)
                s = kk @ q[b, h, t].astype(np.float64) * scale
                w = np.exp(s - s.max())
                out[b, h, t] = (w / w.sum()) @ vv
    return out


def test_f32_to_fp16_matches_numpy_rounding():
    rng = np.random.default_rng(0)
    bits = rng.integers(0, 2**32, 1 << 20, dtype=np.uint64).astype(np.uint32)
    edge = np.array([0, 0x80000000, 0x7f800000, 0xff800000, 0x7fc00000, 0x7f800001, 0x33000000, 0x33000001,
                     0x33800000, 0x387fe000, 0x387ff000, 0x38800000, 0x477fe000, 0x477fefff, 0x477ff000,
                     0x47800000, 0x3f801000, 0x3f803000, 0x3f801001, 0x00000001, 0x007fffff], np.uint32)
    bits = np.concatenate([bits, edge])
    values = bits.view(np.float32)
    with np.errstate(over="ignore"):
        want = values.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_fp16_bits(x) for x in values[:20000]] +
                   [oracle.f32_to_fp16_bits(x) for x in values[-len(edge):]], np.uint16)
    want = np.concatenate([want[:20000], want[-len(edge):]])
    nan = np.isnan(np.concatenate([values[:20000], values[-len(edge):]]))
    assert np.array_equal(got[~nan], want[~nan])
    # NaNs stay NaNs with their sign
    assert np.all((got[nan] & 0x7c00) == 0x7c00) and np.all((got[nan] & 0x03ff) != 0)
    assert np.array_equal(got[nan] & 0x8000, want[nan] & 0x8000)


def test_reference_test_case_against_causal_attention():
    # napi/mod.rs:4963-5051: one slot, cursor 0, advance 3; q [1,4,3,4] = 0..47, k = 0.24.., v = 0.48..
    q = np.arange(48, dtype=np.float32).reshape(1, 4, 3, 4)
    k = (np.arange(24, 48).astype(np.float32) * np.float32(0.01)).reshape(1, 2, 3, 4)
    v = (np.arange(48, 72).astype(np.float32) * np.float32(0.01)).reshape(1, 2, 3, 4)
    k_slab = np.zeros((8, 2, 4), np.float32)
    v_slab = np.zeros((8, 2, 4), np.float32)
    got = oracle.kv_attention(k_slab, v_slab, 4, np.array([[1, 0]]), [0], [3], q, k, v, 0.5)
    want = dense_attention(q, k, v, 0.5, lambda b, t: 0, lambda b, t: t + 1)
    assert np.allclose(got, want, rtol=0, atol=1e-6)  # the reference's assert_close(.., 1e-6)
    # the rows went to physical block 1: rows 4..6
    assert np.array_equal(k_slab[4:7], k[0].transpose(1, 0, 2)) and np.all(k_slab[:4] == 0)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_closed_forms_and_paging(dtype):
    rng = np.random.default_rng(5)
    batch, hq, hkv, width, bs = 3, 4, 2, 8, 4
    context = np.array([9, 4, 0])            # tokens already cached
    tokens = 2
    advances = np.array([2, 1, 2])
    blocks = 4
    max_tokens = batch * blocks * bs
    # fill the caches through the oracle itself, one call per prefix length, with shuffled block tables
    table = rng.permutation(batch * blocks).reshape(batch, blocks).astype(np.uint32)
    k_all = rng.standard_normal((batch, hkv, 16, width)).astype(np.float32)
    v_all = rng.standard_normal((batch, hkv, 16, width)).astype(np.float32)
    k_slab = np.zeros((max_tokens, hkv, width), dtype)
    v_slab = np.zeros((max_tokens, hkv, width), dtype)
    for b in range(batch):
        for p in range(context[b]):
            row = table[b, p // bs] * bs + p % bs
            k_slab[row] = k_all[b, :, p]
            v_slab[row] = v_all[b, :, p]
    q = rng.standard_normal((batch, hq, tokens, width)).astype(np.float32)
    k_new = np.stack([k_all[b, :, context[b]:context[b] + tokens] for b in range(batch)])
    v_new = np.stack([v_all[b, :, context[b]:context[b] + tokens] for b in range(batch)])
    got = oracle.kv_attention(k_slab, v_slab, bs, table, context, advances, q, k_new, v_new, 0.35)
    # dense statement over the (rounded) full sequences
    k_seen = k_all.astype(dtype).astype(np.float32)
    v_seen = v_all.astype(dtype).astype(np.float32)
    needed = context + advances
    want = dense_attention(q, k_seen, v_seen, 0.35, lambda b, t: 0,
                           lambda b, t: min(context[b] + t + 1, needed[b]))
    assert np.allclose(got, want, rtol=0, atol=2e-6)
    # a different paging of the same logical content gives the same output
    table2 = np.roll(table.reshape(-1), 5).reshape(batch, blocks)
    k2 = np.zeros_like(k_slab); v2 = np.zeros_like(v_slab)
    for b in range(batch):
        for p in range(context[b]):
            row = table2[b, p // bs] * bs + p % bs
            k2[row] = k_all[b, :, p]; v2[row] = v_all[b, :, p]
    again = oracle.kv_attention(k2, v2, bs, table2, context, advances, q, k_new, v_new, 0.35)
    assert np.array_equal(got, again)
    # windowed: the last 5 positions only
    for context_window, window in ((0, 5), (5, 0), (6, 3), (3, 6)):
        windowed = oracle.kv_attention(k2.copy(), v2.copy(), bs, table2, context, advances, q, k_new, v_new,
                                       0.35, window=window, context_window=context_window)
        start = np.maximum(needed - context_window, 0) if context_window else np.zeros_like(needed)
        end = lambda b, t: min(context[b] + t + 1, needed[b])
        begin = lambda b, t: max(end(b, t) - window, start[b], 0) if window else start[b]
        want_w = dense_attention(q, k_seen, v_seen, 0.35, begin, end)
        assert np.allclose(windowed, want_w, rtol=0, atol=2e-6)
    # inactive slots stay zero
    part = oracle.kv_attention(k2.copy(), v2.copy(), bs, table2, context, advances, q, k_new, v_new, 0.35,
                               active_batch=1)
    assert np.array_equal(part[0], got[0]) and np.all(part[1:] == 0)


def test_equal_scores_give_the_mean_and_single_position_gives_the_row():
    rng = np.random.default_rng(9)
    width, bs, ctx = 16, 4, 11
    v_rows = rng.standard_normal((ctx + 1, 1, width)).astype(np.float32)
    k_slab = np.zeros((16, 1, width), np.float32)
    v_slab = np.zeros((16, 1, width), np.float32)
    v_slab[:ctx] = v_rows[:ctx]
    table = np.array([[0, 1, 2, 3]])
    q = rng.standard_normal((1, 2, 1, width)).astype(np.float32)
    # all keys zero -> every score 0 -> plain mean of the ctx + 1 value rows
    got = oracle.kv_attention(k_slab, v_slab, bs, table, [ctx], [1], q, np.zeros((1, 1, 1, width), np.float32),
                              v_rows[ctx:ctx + 1].reshape(1, 1, 1, width), 1.0)
    assert np.allclose(got[0, :, 0], v_rows[:, 0].astype(np.float64).mean(axis=0), atol=1e-6)
    # empty cache, one new token: the output is that token's value row
    got = oracle.kv_attention(np.zeros_like(k_slab), np.zeros_like(v_slab), bs, table, [0], [1], q,
                              rng.standard_normal((1, 1, 1, width)).astype(np.float32),
                              v_rows[:1].reshape(1, 1, 1, width), 3.0)
    assert np.array_equal(got[0, 0, 0], v_rows[0, 0]) and np.array_equal(got[0, 1, 0], v_rows[0, 0])


def test_errors():
    z = np.zeros((8, 1, 4), np.float32)
    q = np.zeros((1, 1, 2, 4), np.float32)
    kv = np.zeros((1, 1, 2, 4), np.float32)
    with pytest.raises(oracle.OracleError, match="advance 3 out of range for chunk length 2"):
        oracle.kv_attention(z.copy(), z.copy(), 4, [[0, 1]], [0], [3], q, kv, kv, 1.0)
    with pytest.raises(oracle.OracleError, match="advance 0 out of range"):
        oracle.kv_attention(z.copy(), z.copy(), 4, [[0, 1]], [0], [0], q, kv, kv, 1.0)


def test_adding_one_vector_to_every_key_changes_nothing():
    # q.(k + c) = q.k + q.c: every score of a query moves by the same amount, softmax is unchanged
    rng = np.random.default_rng(21)
    width, bs, ctx = 8, 4, 7
    table = np.array([[2, 0, 1]])
    k_rows = rng.standard_normal((ctx + 1, 2, width))
    v_rows = rng.standard_normal((ctx + 1, 2, width)).astype(np.float32)
    shift = rng.standard_normal(width)
    q = rng.standard_normal((1, 4, 1, width)).astype(np.float32)
    outs = []
    for keys in (k_rows, k_rows + shift):
        keys = keys.astype(np.float32)
        k_slab = np.zeros((12, 2, width), np.float32)
        v_slab = np.zeros((12, 2, width), np.float32)
        for p in range(ctx):
            k_slab[table[0, p // bs] * bs + p % bs] = keys[p]
            v_slab[table[0, p // bs] * bs + p % bs] = v_rows[p]
        outs.append(oracle.kv_attention(k_slab, v_slab, bs, table, [ctx], [1], q,
                                        keys[ctx].reshape(1, 2, 1, width),
                                        v_rows[ctx].reshape(1, 2, 1, width), 0.7))
    assert np.allclose(outs[0], outs[1], rtol=0, atol=2e-6)
    assert not np.array_equal(outs[0], np.zeros_like(outs[0]))


def test_f32_to_bf16_matches_torch_rounding():
    import torch
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2**32, 30000, dtype=np.uint64).astype(np.uint32)
    edge = np.array([0, 0x80000000, 0x7f800000, 0xff800000, 0x7fc00000, 0x7f800001, 0x3f808000, 0x3f818000,
                     0x3f808001, 0x3f807fff, 0x7f7fffff, 0x7f7f8000, 0x00008000, 0x00018000, 0x00000001], np.uint32)
    bits = np.concatenate([bits, edge])
    values = bits.view(np.float32)
    want = torch.from_numpy(values.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([oracle.f32_to_bf16_bits(x) for x in values], np.uint16)
    nan = np.isnan(values)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all((got[nan] & 0x7f80) == 0x7f80) and np.all((got[nan] & 0x007f) != 0)
    assert np.array_equal(got[nan] & 0x8000, (bits[nan] >> 16).astype(np.uint16) & 0x8000)


def _pool_case(rng, dtype):
    """One slot with 9 cached positions and 2 arriving ones, 2 kv heads of width 8, blocks of 4."""
    heads, kv_heads, width, block, cached, new = 4, 2, 8, 4, 9, 2
    q = rng.standard_normal((1, heads, new, width)).astype(np.float32)
    k = rng.standard_normal((1, kv_heads, cached + new, width)).astype(np.float32)
    v = rng.standard_normal((1, kv_heads, cached + new, width)).astype(np.float32)
    table = np.array([[2, 0, 1]])
    slabs = [np.zeros((12, kv_heads, width), dtype) for _ in range(2)]
    scales = [np.zeros((12, kv_heads), np.float32) for _ in range(2)] if dtype == np.uint8 else [None, None]
    # fill the cache through the oracle itself: one call that appends the first nine positions
    oracle.kv_attention(slabs[0], slabs[1], block, table, [0], [cached], np.zeros((1, heads, cached, width), np.float32),
                        k[:, :, :cached], v[:, :, :cached], 1.0, k_scales=scales[0], v_scales=scales[1])
    out = oracle.kv_attention(slabs[0], slabs[1], block, table, [cached], [new], q, k[:, :, cached:], v[:, :, cached:],
                              0.35, k_scales=scales[0], v_scales=scales[1])
    return q, k, v, slabs, scales, out, table


def test_reduced_precision_pools_track_the_f32_pool():
    # the reference tests these tiers through a whole model (Inference.test.ts:509-550); here the
    # attention over a bf16 / u8 pool is held against the f32 pool on the same inputs
    outputs = {}
    for dtype in (np.float32, np.float16, np.uint16, np.uint8):
        outputs[np.dtype(dtype).name] = _pool_case(np.random.default_rng(5), dtype)[5]
    assert np.abs(outputs["float16"] - outputs["float32"]).max() < 2e-3
    assert np.abs(outputs["uint16"] - outputs["float32"]).max() < 2e-2   # bf16: 8 bits of mantissa
    assert np.abs(outputs["uint8"] - outputs["float32"]).max() < 3e-2    # 127 steps per row
    assert np.abs(outputs["uint8"] - outputs["float32"]).max() > 1e-5    # and it is not the f32 path


def test_u8_tier_rows_scales_and_rounding():
    rng = np.random.default_rng(6)
    q, k, v, slabs, scales, out, table = _pool_case(rng, np.uint8)
    block = 4
    for slab, scale, source in ((slabs[0], scales[0], k), (slabs[1], scales[1], v)):
        for position in range(11):
            row = table[0, position // block] * block + position % block
            for head in range(2):
                x = source[0, head, position]
                want_scale = np.float32(np.abs(x).max()) / np.float32(127.0) + np.float32(1e-12)
                assert scale[row, head] == want_scale
                ratio = (x / want_scale).astype(np.float32)
                rounded = np.where(ratio >= 0, np.floor(ratio + np.float32(0.5)), np.ceil(ratio - np.float32(0.5)))
                assert np.array_equal(slab[row, head], (np.clip(rounded, -127, 127) + 128).astype(np.uint8))
                # dequantised values are within half a step of the input
                back = (slab[row, head].astype(np.float32) - 128) * scale[row, head]
                assert np.abs(back - x).max() <= 0.5 * scale[row, head] * (1 + 1e-6)
    # a row of equal magnitudes stores +-127; halves round away from zero
    slab = [np.zeros((4, 1, 4), np.uint8) for _ in range(2)]
    scale = [np.zeros((4, 1), np.float32) for _ in range(2)]
    row = np.array([[[[3.0, -3.0, 3.0, -3.0]]]], np.float32)
    half = np.array([[[[127.0, 0.5, -0.5, 1.5]]]], np.float32)  # scale 1 + 1e-12 rounds to 1
    oracle.kv_attention(slab[0], slab[1], 4, np.array([[0]]), [0], [1], np.zeros((1, 1, 1, 4), np.float32), row, half, 1.0,
                        k_scales=scale[0], v_scales=scale[1])
    assert slab[0][0, 0].tolist() == [255, 1, 255, 1] and scale[0][0, 0] == np.float32(3.0) / np.float32(127.0) + np.float32(1e-12)
    assert slab[1][0, 0].tolist() == [255, 129, 127, 130]
    # the attention output over one position is that dequantised value row
    got = oracle.kv_attention(slab[0], slab[1], 4, np.array([[0]]), [1], [1], np.ones((1, 1, 1, 4), np.float32),
                              row, half, 1.0, k_scales=scale[0], v_scales=scale[1], window=1)
    assert np.allclose(got[0, 0, 0], (slab[1][1, 0].astype(np.float32) - 128) * scale[1][1, 0], rtol=1e-6)
