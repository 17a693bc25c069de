"""The small operators of a decode step on the GPU against the CPU oracle (oracle/et_oracle_ops.c).

Bars: RMS norm and rotary compute in f64 and round once, like the reference: at most one f32 unit in
the last place from the oracle (different f64 summation order / library pow, sin, cos). SiLU * up:
1e-6 relative (+ an absolute term where tanh(x / 2) / 2 + 1 / 2 cancels), the f32 tanh differs between
libraries. Greedy tokens and gathered rows: exact.
"""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def ulps(got, want):
    spacing = np.spacing(np.maximum(np.abs(want), np.float32(1e-30)).astype(np.float32))
    return np.abs(got.astype(np.float64) - want.astype(np.float64)) / spacing


@pytest.mark.parametrize("shape", [(1, 4096), (32, 4096), (2, 3, 1000), (5, 1), (3, 8192), (4, 33)])
@pytest.mark.parametrize("weighted", [False, True])
def test_rms_norm(et, device, shape, weighted):
    rng = np.random.default_rng(sum(shape))
    x = (rng.standard_normal(shape) * 5).astype(np.float32)
    w = rng.standard_normal(shape[-1]).astype(np.float32) if weighted else None
    xd = torch.from_numpy(x).to(device)
    out = torch.empty_like(xd)
    et.rms_norm_into(xd, None if w is None else torch.from_numpy(w).to(device), 1e-5, out)
    want = oracle.rms_norm(x, w, 1e-5)
    assert ulps(out.cpu().numpy(), want).max() <= 1.0


def test_rms_norm_reference_vectors(et, device):
    # packages/core/test/Tensor.test.ts:462-481
    x = np.array([-2, -1, 0, 1, 1, 2, 3, 4, 4, 3, 2, 1, -1, -2, -3, -4], np.float32).reshape(2, 2, 4)
    w = np.array([0.5, 1, 1.5, 2], np.float32)
    xd = torch.from_numpy(x).to(device)
    out = torch.empty_like(xd)
    et.rms_norm_into(xd, torch.from_numpy(w).to(device), 1e-5, out)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 * x64).mean(-1, keepdims=True) + 1e-5) * w
    assert np.array_equal(out.cpu().numpy(), want.astype(np.float32))


@pytest.mark.parametrize("layout", ["HALF_SPLIT", "INTERLEAVED_PAIRS"])
@pytest.mark.parametrize("shape,offsets", [((32, 32, 1, 128), None), ((2, 8, 7, 64), [5]), ((3, 4, 5, 16), None),
                                           ((6, 8), [0]), ((1, 1, 4), [1])])
def test_rotary(et, device, layout, shape, offsets):
    rng = np.random.default_rng(len(shape) * 100 + shape[-1])
    x = rng.standard_normal(shape).astype(np.float32)
    batch = 1 if len(shape) == 2 else shape[0]
    if offsets is None:
        offsets = rng.integers(0, 100000, batch)
    xd = torch.from_numpy(x).to(device)
    out = torch.empty_like(xd)
    od = torch.tensor(np.asarray(offsets), dtype=torch.int32, device=device)
    et.rotary_into(xd, od, 500000.0, 1.0, et.RotaryLayout[layout], out)
    want = oracle.rotary(x, offsets, 500000.0, 1.0, interleaved=layout == "INTERLEAVED_PAIRS")
    got = out.cpu().numpy()
    # one rounding of a f64 result whose sin / cos / pow may differ in their last f64 bit
    assert np.abs(got - want).max() <= 2.4e-7 * max(1.0, np.abs(want).max())
    back = torch.empty_like(xd)
    et.rotary_into(out, od, 500000.0, -1.0, et.RotaryLayout[layout], back)
    assert np.abs(back.cpu().numpy() - x).max() <= 2e-6  # the reference's own round-trip bar


@pytest.mark.parametrize("layout", ["HALF_SPLIT", "INTERLEAVED_PAIRS"])
def test_rotary_pair_is_two_rotaries(et, device, layout):
    # queries and keys of a step in one launch: the bits of the two separate launches, in place too
    rng = np.random.default_rng(17)
    for q_shape, k_shape in (((32, 32, 1, 128), (32, 8, 1, 128)), ((3, 5, 4, 16), (3, 1, 4, 16))):
        q = torch.from_numpy(rng.standard_normal(q_shape).astype(np.float32)).to(device)
        k = torch.from_numpy(rng.standard_normal(k_shape).astype(np.float32)).to(device)
        offsets = torch.tensor(rng.integers(0, 9000, q_shape[0]), dtype=torch.int32, device=device)
        q_alone, k_alone = torch.empty_like(q), torch.empty_like(k)
        et.rotary_into(q, offsets, 500000.0, 1.0, et.RotaryLayout[layout], q_alone)
        et.rotary_into(k, offsets, 500000.0, 1.0, et.RotaryLayout[layout], k_alone)
        q_pair, k_pair = q.clone(), k.clone()
        et.rotary_pair_into(q_pair, k_pair, offsets, 500000.0, 1.0, et.RotaryLayout[layout], q_pair, k_pair)
        assert torch.equal(q_pair, q_alone) and torch.equal(k_pair, k_alone)
    with pytest.raises(et.QuantizedError, match="share batch, steps and head dimension"):
        shorter = k[:, :, :2].contiguous()  # other steps
        et.rotary_pair_into(q, shorter, offsets, 500000.0, 1.0, et.RotaryLayout[layout], q, shorter)


def test_silu_mul(et, device):
    rng = np.random.default_rng(5)
    for count in (32 * 14336, 1001, 3):
        gate = (rng.standard_normal(count) * 4).astype(np.float32)
        up = rng.standard_normal(count).astype(np.float32)
        gate[:3] = [0.0, 40.0, -40.0]
        gd, ud = torch.from_numpy(gate).to(device), torch.from_numpy(up).to(device)
        out = torch.empty_like(gd)
        et.silu_mul_into(gd, ud, out)
        want = oracle.silu_mul(gate, up)
        got = out.cpu().numpy()
        assert np.all(np.abs(got - want) <= 1e-6 * np.abs(want) + 1.5e-7 * np.abs(gate * up))
        g64 = gate.astype(np.float64)
        exact = g64 / (1.0 + np.exp(-g64)) * up
        assert np.all(np.abs(got - exact) <= 1e-6 * np.abs(exact) + 1.5e-7 * np.abs(gate * up))


def test_greedy_tokens(et, device):
    rng = np.random.default_rng(6)
    logits = rng.standard_normal((32, 128256)).astype(np.float32)
    logits[3, 100] = logits[3, 90000] = 9.0       # equal maxima: the lower token wins
    logits[4, 128255] = 10.0
    logits[5, 0] = 10.0
    got = et.greedy_tokens(torch.from_numpy(logits).to(device)).cpu().numpy()
    want = oracle.argmax_rows(logits)
    assert np.array_equal(got, want) and got[3] == 100 and got[4] == 128255 and got[5] == 0
    tie = torch.tensor([[1.0, 4.0, 4.0, 2.0]], device=device)  # sampling.rs:223-238
    assert int(et.greedy_tokens(tie)[0]) == 1
    small = rng.standard_normal((2, 3, 7)).astype(np.float32)
    assert np.array_equal(et.greedy_tokens(torch.from_numpy(small).to(device)).cpu().numpy(),
                          oracle.argmax_rows(small))
    logits[7, 4000] = np.inf
    logits[9, 17] = np.nan
    with pytest.raises(et.QuantizedError, match="sample: logit 4000 is not finite"):
        et.greedy_tokens(torch.from_numpy(logits).to(device))


@pytest.mark.parametrize("dtype,width", [(np.float16, 4096), (np.float32, 100), (np.float16, 3), (np.uint8, 5)])
@pytest.mark.parametrize("wide_index", [False, True])
def test_gather_rows(et, device, dtype, width, wide_index):
    rng = np.random.default_rng(width)
    table = (rng.standard_normal((1000, width)) * 3).astype(dtype)
    indexes = rng.integers(0, 1000, (4, 9))
    td = torch.from_numpy(table).to(device)
    as_index = lambda a: (torch.from_numpy(a.astype(np.int64)).to(device) if wide_index else
                          torch.from_numpy(a.astype(np.int32)).to(device).view(torch.uint32))
    idx = as_index(indexes)
    out = torch.zeros((36, width), dtype=td.dtype, device=device)
    et.gather_rows_into(td, idx, out)
    want = oracle.gather_rows(table, indexes.reshape(-1))
    assert np.array_equal(out.cpu().numpy().view(np.uint8), want.view(np.uint8))
    bad = indexes.copy()
    bad[2, 3] = 1000
    idx = as_index(bad)
    with pytest.raises(et.QuantizedError, match="index_select: index 1000 is out of bounds for extent 1000"):
        et.gather_rows_into(td, idx, out)
    if wide_index:
        bad[0, 0] = -2
        idx = torch.from_numpy(bad.astype(np.int64)).to(device)
        with pytest.raises(et.QuantizedError, match="index_select: index -2 is out of bounds for extent 1000"):
            et.gather_rows_into(td, idx, out)


def test_add(et, device):
    rng = np.random.default_rng(8)
    for count in (32 * 4096, 1001):
        a = (rng.standard_normal(count) * 100).astype(np.float32)
        b = rng.standard_normal(count).astype(np.float32)
        ad, bd = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
        out = torch.empty_like(ad)
        et.add_into(ad, bd, out)
        assert np.array_equal(out.cpu().numpy(), oracle.add(a, b))
        et.add_into(ad, bd, ad)  # in place, as the residual stream is updated
        assert np.array_equal(ad.cpu().numpy(), oracle.add(a, b))


@pytest.mark.parametrize("shape", [(32, 4096), (3, 1000), (2, 33)])
def test_rms_norm_with_a_half_float_weight_is_the_widened_weight(et, device, shape):
    # a weight stored as half floats is widened on use: the bits of the same call with the f32 copy
    rng = np.random.default_rng(7 + shape[-1])
    x = torch.from_numpy((rng.standard_normal(shape) * 3).astype(np.float32)).to(device)
    half = torch.from_numpy((1.0 + 0.2 * rng.standard_normal(shape[-1])).astype(np.float16)).to(device)
    wide, narrow = torch.empty_like(x), torch.empty_like(x)
    et.rms_norm_into(x, half.float(), 1e-5, wide)
    et.rms_norm_into(x, half, 1e-5, narrow)
    assert torch.equal(wide, narrow)
    want = oracle.rms_norm(x.cpu().numpy(), half.float().cpu().numpy(), 1e-5)
    assert ulps(narrow.cpu().numpy(), want).max() <= 1.0
    with pytest.raises(et.QuantizedError, match="weight must match the last dimension and dtype"):
        et.rms_norm_into(x, half.to(torch.bfloat16), 1e-5, narrow)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("width", [4096, 100, 7])
def test_gather_rows_widens_half_float_tables(et, device, dtype, width):
    rng = np.random.default_rng(width)
    table = torch.from_numpy(rng.standard_normal((300, width)).astype(np.float32)).to(device).to(dtype)
    ids = torch.from_numpy(rng.integers(0, 300, 40).astype(np.int64)).to(device)
    out = torch.full((40, width), float("nan"), device=device)
    et.gather_rows_into(table, ids, out)
    assert torch.equal(out, table[ids].float())  # index_select, then the exact cast
    bad = ids.clone()
    bad[3] = 300
    with pytest.raises(et.QuantizedError, match="index_select: index 300 is out of bounds for extent 300"):
        et.gather_rows_into(table, bad, out)
    with pytest.raises(et.QuantizedError, match="index_select"):
        et.gather_rows_into(table, ids, torch.empty((40, width), dtype=torch.float64, device=device))


def test_kv_commit_advances_the_active_cursors(et, device):
    # cursor += advance for the active slots (crates/runtime-cpu/src/napi/mod.rs:4511-4517)
    slab = torch.zeros((64, 2, 128), dtype=torch.float16, device=device)
    table = torch.arange(12, dtype=torch.int32, device=device).reshape(3, 4) % 4
    cursors = torch.tensor([5, 0, 17], dtype=torch.int32, device=device)
    advances = torch.tensor([1, 3, 2], dtype=torch.int32, device=device)
    layer = et.KvLayer(slab, slab.clone(), 16, table, cursors, advances, 32, active_batch=2)
    et.kv_commit(layer)
    et.kv_commit(layer)
    torch.cuda.synchronize()
    assert cursors.tolist() == [7, 6, 17]  # the slot beyond the active batch stays
