"""Paged key/value-cache attention on the GPU against the CPU oracle (oracle/et_oracle_kv.c).

Bars: slabs after the call are bit-identical to the oracle's (f32 copies, f16 / bf16
round-to-nearest-even, the u8 tier's bytes and scales); outputs agree to 1e-4 (f32 online softmax
against the oracle's f64 three passes over the same stored values).
"""
import numpy as np
import pytest
import torch

import oracle
from effect_torch_amd import synth

pytestmark = pytest.mark.gpu

OUT_TOL = 1e-4
ALL_DTYPES = [np.float32, np.float16, "bf16", "u8"]


def dims_per_piece(dtype):
    """Elements of a slab row one lane of the streaming kernel takes."""
    return {np.float32: 4, np.float16: 8, "bf16": 8, "u8": 8}[dtype]


def random_slab(rng, shape, dtype):
    values = rng.standard_normal(shape).astype(np.float32)
    if dtype == "bf16":  # bfloat16 bits
        return torch.from_numpy(values).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16), None
    if dtype == "u8":    # bytes 1..255 and positive scales, as the write produces them
        scales = (np.abs(values).max(-1) / np.float32(127.0) + np.float32(1e-12)).astype(np.float32)
        return rng.integers(1, 256, shape).astype(np.uint8), scales
    return values.astype(dtype), None


def make_case(rng, *, slots, query_heads, kv_heads, width, block_size, contexts, tokens, advances, dtype,
              spare_blocks=3):
    """Random slabs with `contexts[b]` cached positions per slot behind a shuffled block table."""
    contexts = np.asarray(contexts, dtype=np.int64)
    advances = np.asarray(advances, dtype=np.int64)
    blocks_per_slot = int(max(1, -(-int((contexts + tokens).max()) // block_size)))
    total_blocks = slots * blocks_per_slot + spare_blocks
    max_tokens = total_blocks * block_size
    table = rng.permutation(total_blocks)[: slots * blocks_per_slot].reshape(slots, blocks_per_slot).astype(np.uint32)
    k_slab, k_scales = random_slab(rng, (max_tokens, kv_heads, width), dtype)
    v_slab, v_scales = random_slab(rng, (max_tokens, kv_heads, width), dtype)
    q = rng.standard_normal((slots, query_heads, tokens, width)).astype(np.float32)
    k = rng.standard_normal((slots, kv_heads, tokens, width)).astype(np.float32)
    v = rng.standard_normal((slots, kv_heads, tokens, width)).astype(np.float32)
    return dict(k_slab=k_slab, v_slab=v_slab, k_scales=k_scales, v_scales=v_scales, table=table,
                cursors=contexts.astype(np.uint32),
                advances=advances.astype(np.uint32), q=q, k=k, v=v, block_size=block_size,
                max_context=int((contexts + advances).max()))


def run_gpu(et, device, case, scale, *, window=0, context_window=0, active_batch=None, max_context=None,
            workspace=None):
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    bf16 = case["k_slab"].dtype == np.uint16

    def slab(array):
        return dev(array.view(np.int16)).view(torch.bfloat16) if bf16 else dev(array)

    def back(tensor):
        return tensor.view(torch.int16).cpu().numpy().view(np.uint16) if bf16 else tensor.cpu().numpy()

    k_slab, v_slab = slab(case["k_slab"]), slab(case["v_slab"])
    scales = [dev(case[name]) if case.get(name) is not None else None for name in ("k_scales", "v_scales")]
    layer = et.KvLayer(k_slab, v_slab, case["block_size"], dev(case["table"].view(np.int32)),
                       dev(case["cursors"].view(np.int32)), dev(case["advances"].view(np.int32)),
                       case["max_context"] if max_context is None else max_context,
                       active_batch=active_batch, context_window=context_window, k_scales=scales[0],
                       v_scales=scales[1])
    q = dev(case["q"])
    out = torch.full_like(q, float("nan"))
    et.kv_attention_into(layer, q, dev(case["k"]), dev(case["v"]), scale, window, out, workspace=workspace)
    got_scales = [t.cpu().numpy() if t is not None else None for t in scales]
    return out.cpu().numpy(), back(k_slab), back(v_slab), layer, got_scales


def run_oracle(case, scale, *, window=0, context_window=0, active_batch=None):
    k_slab, v_slab = case["k_slab"].copy(), case["v_slab"].copy()
    scales = [case[name].copy() if case.get(name) is not None else None for name in ("k_scales", "v_scales")]
    out = oracle.kv_attention(k_slab, v_slab, case["block_size"], case["table"], case["cursors"], case["advances"],
                              case["q"], case["k"], case["v"], scale, window=window,
                              context_window=context_window, active_batch=active_batch, k_scales=scales[0],
                              v_scales=scales[1])
    return out, k_slab, v_slab, scales


def compare(got, want):
    out, k_slab, v_slab = got[:3]
    ref_out, ref_k, ref_v = want[:3]
    assert np.array_equal(k_slab.view(np.uint8), ref_k.view(np.uint8)), "K slab differs"
    assert np.array_equal(v_slab.view(np.uint8), ref_v.view(np.uint8)), "V slab differs"
    if len(got) > 4 and got[4][0] is not None:
        for mine, theirs in zip(got[4], want[3]):
            assert np.array_equal(mine.view(np.uint32), theirs.view(np.uint32)), "scale slab differs"
    assert np.isfinite(out).all()
    error = np.abs(out - ref_out).max()
    assert error <= OUT_TOL, f"max |out - oracle| = {error}"


def test_the_reference_test_case(et, device):
    # napi/mod.rs:4963-5051
    q = np.arange(48, dtype=np.float32).reshape(1, 4, 3, 4)
    k = (np.arange(24, 48).astype(np.float32) * np.float32(0.01)).reshape(1, 2, 3, 4)
    v = (np.arange(48, 72).astype(np.float32) * np.float32(0.01)).reshape(1, 2, 3, 4)
    case = dict(k_slab=np.zeros((8, 2, 4), np.float32), v_slab=np.zeros((8, 2, 4), np.float32),
                table=np.array([[1, 0]], np.uint32), cursors=np.array([0], np.uint32),
                advances=np.array([3], np.uint32), q=q, k=k, v=v, block_size=4, max_context=3)
    got = run_gpu(et, device, case, 0.5)
    assert et.kv_attention_kernel(got[3], 4, 3).startswith("kv_attend_any")
    compare(got, run_oracle(case, 0.5))


@pytest.mark.parametrize("dtype", ALL_DTYPES)
@pytest.mark.parametrize("lanes", [8, 16, 32])
@pytest.mark.parametrize("group,kv_heads", [(1, 3), (2, 2), (4, 2), (8, 1), (3, 2), (12, 1)])
def test_streaming_kernel_shapes(et, device, dtype, lanes, group, kv_heads):
    width = lanes * dims_per_piece(dtype)
    rng = np.random.default_rng(1000 * lanes + 10 * group + kv_heads)
    case = make_case(rng, slots=3, query_heads=group * kv_heads, kv_heads=kv_heads, width=width, block_size=16,
                     contexts=[0, 37, 200], tokens=1, advances=[1, 1, 1], dtype=dtype)
    scale = 1.0 / np.sqrt(width)
    got = run_gpu(et, device, case, scale)
    assert et.kv_attention_kernel(got[3], group * kv_heads, 1) in ("kv_attend", "kv_attend+kv_merge")
    compare(got, run_oracle(case, scale))


@pytest.mark.parametrize("dtype", ALL_DTYPES)
@pytest.mark.parametrize("lanes", [8, 16, 32])
@pytest.mark.parametrize("group", [1, 4, 8])
def test_eight_wave_workgroups_without_context_splits(et, device, dtype, lanes, group):
    # 256 rows of queries: one eight-wave workgroup per (slot, kv head), no partial records
    width = lanes * dims_per_piece(dtype)
    rng = np.random.default_rng(7000 + 100 * lanes + group)
    slots, kv_heads = 32, 8
    contexts = rng.integers(0, 150, slots)
    contexts[:2] = [0, 600]
    case = make_case(rng, slots=slots, query_heads=group * kv_heads, kv_heads=kv_heads, width=width, block_size=16,
                     contexts=contexts, tokens=1, advances=[1] * slots, dtype=dtype)
    scale = 1.0 / np.sqrt(width)
    got = run_gpu(et, device, case, scale)
    assert et.kv_attention_kernel(got[3], group * kv_heads, 1) == "kv_attend"
    assert et.kv_attention_workspace_bytes(got[3], group * kv_heads, 1) == 0
    compare(got, run_oracle(case, scale))


@pytest.mark.parametrize("dtype", ALL_DTYPES)
@pytest.mark.parametrize("block_size", [1, 5, 16, 64])
@pytest.mark.parametrize("tokens,advances", [(1, [1, 1, 1, 1]), (4, [4, 1, 3, 2])])
def test_paging_chunks_and_ragged_advances(et, device, dtype, block_size, tokens, advances):
    rng = np.random.default_rng(block_size * 7 + tokens)
    case = make_case(rng, slots=4, query_heads=8, kv_heads=2, width=128, block_size=block_size,
                     contexts=[0, 1, 63, 129], tokens=tokens, advances=advances, dtype=dtype)
    got = run_gpu(et, device, case, 0.09)
    compare(got, run_oracle(case, 0.09))


@pytest.mark.parametrize("width,dtype", [(4, np.float16), (20, np.float32), (96, np.float16), (200, np.float32),
                                         (40, "bf16"), (24, "u8"), (100, "u8")])
def test_any_width_kernel(et, device, width, dtype):
    rng = np.random.default_rng(width)
    case = make_case(rng, slots=2, query_heads=6, kv_heads=3, width=width, block_size=8,
                     contexts=[5, 300], tokens=2, advances=[2, 1], dtype=dtype)
    got = run_gpu(et, device, case, 0.2)
    assert "kv_attend_any" in et.kv_attention_kernel(got[3], 6, 2)
    compare(got, run_oracle(case, 0.2))


@pytest.mark.parametrize("context_window,window", [(0, 50), (70, 0), (100, 33), (40, 90), (0, 1)])
@pytest.mark.parametrize("width", [128, 24])
def test_sliding_windows(et, device, context_window, window, width):
    rng = np.random.default_rng(context_window + window + width)
    case = make_case(rng, slots=3, query_heads=4, kv_heads=2, width=width, block_size=16,
                     contexts=[3, 64, 250], tokens=2, advances=[2, 2, 1], dtype=np.float16)
    got = run_gpu(et, device, case, 0.1, window=window, context_window=context_window)
    compare(got, run_oracle(case, 0.1, window=window, context_window=context_window))


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_long_context_is_split(et, device, dtype):
    rng = np.random.default_rng(77)
    case = make_case(rng, slots=2, query_heads=8, kv_heads=2, width=128, block_size=16,
                     contexts=[5000, 777], tokens=1, advances=[1, 1], dtype=dtype)
    scale = 1.0 / np.sqrt(128)
    got = run_gpu(et, device, case, scale)
    assert et.kv_attention_kernel(got[3], 8, 1).endswith("+kv_merge")
    assert et.kv_attention_workspace_bytes(got[3], 8, 1) > 0
    compare(got, run_oracle(case, scale))
    # a generous bound changes the launch, not the result
    again = run_gpu(et, device, case, scale, max_context=100000)
    compare(again, run_oracle(case, scale))


def test_one_workspace_serves_calls_of_any_geometry(et, device):
    workspace = torch.full((64 << 20,), 255, dtype=torch.uint8, device=device)
    rng = np.random.default_rng(11)
    for slots, heads, kv_heads, width, contexts, dtype in (
            (2, 8, 2, 128, [5000, 777], np.float16), (5, 4, 4, 64, [900, 30, 2000, 1, 64], np.float32),
            (1, 6, 3, 20, [700], np.float16), (2, 8, 2, 128, [4000, 4100], np.float16),
            (3, 16, 2, 128, [300, 1200, 40], np.float16)):
        case = make_case(rng, slots=slots, query_heads=heads, kv_heads=kv_heads, width=width, block_size=16,
                         contexts=contexts, tokens=1, advances=[1] * slots, dtype=dtype)
        for _ in range(2):
            compare(run_gpu(et, device, case, 0.1, workspace=workspace), run_oracle(case, 0.1))


def test_inactive_slots_are_zero_and_untouched(et, device):
    rng = np.random.default_rng(3)
    case = make_case(rng, slots=4, query_heads=8, kv_heads=2, width=128, block_size=16,
                     contexts=[10, 20, 30, 40], tokens=1, advances=[1, 1, 1, 1], dtype=np.float16)
    got = run_gpu(et, device, case, 0.1, active_batch=2)
    assert np.all(got[0][2:] == 0)
    compare(got, run_oracle(case, 0.1, active_batch=2))


def test_decode_steps_advance_the_cache(et, device):
    # three decode steps through one layer object: what a step writes, the next reads
    rng = np.random.default_rng(8)
    case = make_case(rng, slots=2, query_heads=8, kv_heads=2, width=128, block_size=16,
                     contexts=[14, 28], tokens=1, advances=[1, 1], dtype=np.float16, spare_blocks=0)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    k_slab, v_slab = dev(case["k_slab"]), dev(case["v_slab"])
    cursors = dev(case["cursors"].view(np.int32))
    layer = et.KvLayer(k_slab, v_slab, 16, dev(case["table"].view(np.int32)), cursors,
                       dev(case["advances"].view(np.int32)), 40)
    ref_k, ref_v = case["k_slab"].copy(), case["v_slab"].copy()
    ref_cursors = case["cursors"].copy()
    for step in range(3):
        q = rng.standard_normal((2, 8, 1, 128)).astype(np.float32)
        k = rng.standard_normal((2, 2, 1, 128)).astype(np.float32)
        v = rng.standard_normal((2, 2, 1, 128)).astype(np.float32)
        out = torch.empty(2, 8, 1, 128, device=device)
        et.kv_attention_into(layer, dev(q), dev(k), dev(v), 0.1, None, out)
        want = oracle.kv_attention(ref_k, ref_v, 16, case["table"], ref_cursors, case["advances"], q, k, v, 0.1)
        assert np.abs(out.cpu().numpy() - want).max() <= OUT_TOL
        cursors += 1
        ref_cursors += 1
    assert np.array_equal(k_slab.cpu().numpy().view(np.uint8), ref_k.view(np.uint8))


def test_device_side_checks_report_the_reference_errors(et, device):
    rng = np.random.default_rng(4)
    base = dict(slots=2, query_heads=4, kv_heads=2, width=128, block_size=16, contexts=[10, 20], tokens=2,
                dtype=np.float16)
    case = make_case(rng, advances=[2, 3], **base)
    with pytest.raises(et.QuantizedError, match="kv attention: advance 3 out of range for chunk length 2"):
        run_gpu(et, device, case, 0.1, max_context=64)
    case = make_case(rng, advances=[0, 3], **base)
    with pytest.raises(et.QuantizedError, match="kv attention: advance 0 out of range for chunk length 2"):
        run_gpu(et, device, case, 0.1, max_context=64)
    case = make_case(rng, advances=[1, 1], **base)
    case["cursors"][1] = 40  # the table covers 2 blocks = 32 positions
    with pytest.raises(et.QuantizedError, match="block table of slot 1 does not cover 41 tokens"):
        run_gpu(et, device, case, 0.1, max_context=64)
    case = make_case(rng, advances=[1, 1], **base)
    with pytest.raises(et.QuantizedError, match="above the declared max_context 5"):
        run_gpu(et, device, case, 0.1, max_context=5)
    case = make_case(rng, advances=[1, 1], **base)
    case["table"][0, 0] = 1000
    with pytest.raises(et.QuantizedError, match="outside the pool"):
        run_gpu(et, device, case, 0.1)


@pytest.mark.parametrize("width", [128, 20])
def test_a_cursor_at_the_top_of_32_bits_fails_a_check_instead_of_wrapping(et, device, width):
    # cursor + advance is a usize sum in the reference (napi/mod.rs:3595) and cannot wrap; an idle
    # slot's -1 inside the active batch must be reported, and no block-table entry may be read for it
    rng = np.random.default_rng(5)
    base = dict(slots=2, query_heads=4, kv_heads=2, width=width, block_size=16, contexts=[10, 20], tokens=1,
                dtype=np.float16)
    case = make_case(rng, advances=[1, 1], **base)
    case["cursors"][1] = 0xFFFFFFFF
    with pytest.raises(et.QuantizedError, match="live context 4294967296 exceeds pool capacity"):
        run_gpu(et, device, case, 0.1, max_context=64)
    with pytest.raises(et.QuantizedError, match="block table of slot 1 does not cover 4294967296 tokens"):
        run_gpu(et, device, case, 0.1, max_context=64, context_window=8)
    case["cursors"][1] = 0xFFFFFFF0
    case["advances"][1] = 1
    with pytest.raises(et.QuantizedError, match="live context 4294967281 exceeds pool capacity"):
        run_gpu(et, device, case, 0.1, max_context=64)


@pytest.mark.parametrize("dtype", [np.float16, "u8"])
def test_decode_batch_at_full_size(et, device, dtype):
    # 32 slots x 32 query heads over 8 kv heads of width 128, contexts around 2048, block size 16
    rng = np.random.default_rng(2048)
    contexts = rng.integers(1900, 2048, 32)
    case = make_case(rng, slots=32, query_heads=32, kv_heads=8, width=128, block_size=16, contexts=contexts,
                     tokens=1, advances=[1] * 32, dtype=dtype, spare_blocks=7)
    scale = 1.0 / np.sqrt(128)
    got = run_gpu(et, device, case, scale)
    compare(got, run_oracle(case, scale))
    # size-independent property: with every key zero all scores are equal, the output is the mean of V
    case["k_slab"][:] = 128 if dtype == "u8" else 0
    case["k"][:] = 0
    out, _, v_after, _, scales_after = run_gpu(et, device, case, scale)
    for b in (0, 31):
        rows = [case["table"][b, p // 16] * 16 + p % 16 for p in range(contexts[b] + 1)]  # with the new row
        if dtype == "u8":
            values = (v_after[rows].astype(np.float64) - 128) * scales_after[1][rows][..., None].astype(np.float64)
        else:
            values = v_after[rows].astype(np.float64)
        mean = values.mean(axis=0)  # [kv_heads, width]
        assert np.abs(out[b, :, 0] - np.repeat(mean, 4, axis=0)).max() <= OUT_TOL


@pytest.mark.parametrize("dtype", [np.float16, np.float32, "u8"])
@pytest.mark.parametrize("slots,kv_heads,group,width,contexts_top", [
    (32, 8, 4, 128, 150),    # eight-wave workgroups, four heads = two stages each: quantised in the epilogue
    (33, 8, 8, 64, 150),     # eight heads of 64 = two stages; a ragged last tile of vectors
    (32, 8, 1, 128, 150),    # one head = half a stage: the quantiser launch follows
    (8, 2, 4, 128, 3000),    # few rows: context splits + merge, then the quantiser launch
])
def test_prepared_input_of_the_next_contraction_from_the_attention_launch(et, device, dtype, slots, kv_heads, group,
                                                                          width, contexts_top):
    # the result as the activations of the output projection: the same bytes as kv_attention_into
    # followed by prepare_input, for the destination, the slabs and the prepared tiles
    rng = np.random.default_rng(9100 + slots + group)
    heads = group * kv_heads
    contexts = rng.integers(0, contexts_top, slots)
    case = make_case(rng, slots=slots, query_heads=heads, kv_heads=kv_heads, width=width, block_size=16,
                     contexts=contexts, tokens=1, advances=[1] * slots, dtype=dtype)
    scale = 1.0 / np.sqrt(width)
    plan = et.RawLinear(et.GgmlQuant.Q4_K, 64, heads * width, slots)
    assert plan.fused_prepare
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    results = []
    for fused in (False, True):
        k_slab, v_slab = dev(case["k_slab"]), dev(case["v_slab"])
        scales = [dev(case[name]) if case.get(name) is not None else None for name in ("k_scales", "v_scales")]
        layer = et.KvLayer(k_slab, v_slab, case["block_size"], dev(case["table"].view(np.int32)),
                           dev(case["cursors"].view(np.int32)), dev(case["advances"].view(np.int32)),
                           case["max_context"], k_scales=scales[0], v_scales=scales[1])
        q = dev(case["q"])
        out = torch.full_like(q, float("nan"))
        prepared = torch.zeros(plan.prepared_input_bytes, dtype=torch.uint8, device=device)
        if fused:
            et.kv_attention_into(layer, q, dev(case["k"]), dev(case["v"]), scale, 0, out, prepared_for=plan,
                                 prepared=prepared)
        else:
            et.kv_attention_into(layer, q, dev(case["k"]), dev(case["v"]), scale, 0, out)
            plan.prepare_input(out.view(slots, heads * width), prepared)
        results.append((out, k_slab, v_slab, prepared))
    for two, one in zip(*results):
        assert torch.equal(two, one)
    # more than one token per slot has no such rows
    case = make_case(rng, slots=4, query_heads=heads, kv_heads=kv_heads, width=width, block_size=16,
                     contexts=[5, 6, 7, 8], tokens=2, advances=[2] * 4, dtype=dtype)
    layer = et.KvLayer(dev(case["k_slab"]), dev(case["v_slab"]), 16, dev(case["table"].view(np.int32)),
                       dev(case["cursors"].view(np.int32)), dev(case["advances"].view(np.int32)), case["max_context"],
                       k_scales=dev(case["k_scales"]) if case["k_scales"] is not None else None,
                       v_scales=dev(case["v_scales"]) if case["v_scales"] is not None else None)
    q = dev(case["q"])
    with pytest.raises(et.QuantizedError, match="one token per slot"):
        et.kv_attention_into(layer, q, dev(case["k"]), dev(case["v"]), scale, 0, torch.empty_like(q),
                             prepared_for=et.RawLinear(et.GgmlQuant.Q4_K, 64, heads * width, 4),
                             prepared=torch.zeros(1 << 20, dtype=torch.uint8, device=device))


@pytest.mark.parametrize("dtype", [np.float16, np.float32, "bf16", "u8"])
@pytest.mark.parametrize("slots,kv_heads,group,width,contexts_top,with_bias", [
    (32, 8, 4, 128, 150, False),   # a decode step's geometry: eight-wave workgroups, no context splits
    (32, 8, 4, 128, 150, True),
    (12, 2, 8, 64, 400, True),     # eight heads per workgroup, narrow tile of the contraction, context splits + merge
    (7, 4, 1, 128, 90, False),     # one head per workgroup
])
def test_attention_sums_and_rotates_the_k_shares_of_the_projections(et, device, dtype, slots, kv_heads, group, width,
                                                                    contexts_top, with_bias):
    # q, k, v of a decode step left as the K shares of their group launch: the attention launch sums them,
    # adds the biases, rotates q and k at the cursors, appends and attends - the bytes of the group launch
    # that rotates in its reduction followed by the attention launch, for the result, the slabs, the scales
    # and the prepared input of the next contraction
    rng = np.random.default_rng(9300 + slots + group + int(with_bias))
    heads, columns = group * kv_heads, 1024
    contexts = rng.integers(0, contexts_top, slots)
    case = make_case(rng, slots=slots, query_heads=heads, kv_heads=kv_heads, width=width, block_size=16,
                     contexts=contexts, tokens=1, advances=[1] * slots, dtype=dtype)
    scale = 1.0 / np.sqrt(width)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    sizes = (heads * width, kv_heads * width, kv_heads * width)
    plans = [et.RawLinear(et.GgmlQuant.Q4_K, rows, columns, slots, with_bias) for rows in sizes]
    group_launch = et.LinearGroup(plans)
    assert group_launch.shares_layout().count > 1
    weights = [dev(synth.random_weight(oracle.Q4_K, rows, columns, rng)) for rows in sizes]
    biases = [dev(rng.standard_normal(rows).astype(np.float32)) if with_bias else None for rows in sizes]
    x = dev(synth.random_activations(slots, columns, rng))
    hidden = torch.empty(plans[0].prepared_input_bytes, dtype=torch.uint8, device=device)
    plans[0].prepare_input(x, hidden)
    consumer = et.RawLinear(et.GgmlQuant.Q4_K, 64, heads * width, slots)
    workspace = torch.empty(group_launch.workspace_bytes, dtype=torch.uint8, device=device)
    for layout in (et.RotaryLayout.HALF_SPLIT, et.RotaryLayout.INTERLEAVED_PAIRS):
        results = []
        for in_attention in (False, True):
            slab = lambda a: dev(a.view(np.int16)).view(torch.bfloat16) if dtype == "bf16" else dev(a)  # noqa: E731
            k_slab, v_slab = slab(case["k_slab"]), slab(case["v_slab"])
            scales = [dev(case[name]) if case.get(name) is not None else None for name in ("k_scales", "v_scales")]
            cursors = dev(case["cursors"].view(np.int32))
            layer = et.KvLayer(k_slab, v_slab, case["block_size"], dev(case["table"].view(np.int32)), cursors,
                               dev(case["advances"].view(np.int32)), case["max_context"], k_scales=scales[0],
                               v_scales=scales[1])
            assert et.kv_attention_kernel(layer, heads, 1).split("+")[0] == "kv_attend"
            out = torch.full((slots, heads, 1, width), float("nan"), device=device)
            prepared = torch.zeros(consumer.prepared_input_bytes, dtype=torch.uint8, device=device)
            if in_attention:
                shares = group_launch.enqueue_prepared_shares(hidden, weights, workspace)
                et.kv_attention_projected_into(layer, shares, (0, 1, 2), biases, cursors, 500000.0, 1.0, layout, scale, 0,
                                               out, prepared_for=consumer, prepared=prepared)
            else:
                ys = [torch.empty((slots, rows), device=device) for rows in sizes]
                group_launch.enqueue_prepared_then_rotary(hidden, weights, ys, workspace, (0, 1), cursors, 500000.0, 1.0,
                                                          layout, width, biases=biases if with_bias else None)
                et.kv_attention_into(layer, ys[0].view(slots, heads, 1, width), ys[1].view(slots, kv_heads, 1, width),
                                     ys[2].view(slots, kv_heads, 1, width), scale, 0, out, prepared_for=consumer,
                                     prepared=prepared)
            results.append([out, k_slab, v_slab, prepared] + [s for s in scales if s is not None])
        assert torch.isfinite(results[0][0]).all()
        for two, one in zip(*results):
            assert torch.equal(two.view(torch.uint8), one.view(torch.uint8))


def test_attention_from_k_shares_is_refused_where_the_kernel_takes_tensors(et, device):
    # head width 20: the any-width kernel; the caller sums and rotates first
    rng = np.random.default_rng(9400)
    slots, kv_heads, group, width, columns = 4, 2, 2, 20, 1024
    heads = group * kv_heads
    case = make_case(rng, slots=slots, query_heads=heads, kv_heads=kv_heads, width=width, block_size=16,
                     contexts=[3, 0, 40, 9], tokens=1, advances=[1] * slots, dtype=np.float32)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    sizes = (heads * width, kv_heads * width, kv_heads * width)
    plans = [et.RawLinear(et.GgmlQuant.Q4_K, rows, columns, 8) for rows in sizes]
    group_launch = et.LinearGroup(plans)
    cursors = dev(case["cursors"].view(np.int32))
    layer = et.KvLayer(dev(case["k_slab"]), dev(case["v_slab"]), 16, dev(case["table"].view(np.int32)), cursors,
                       dev(case["advances"].view(np.int32)), case["max_context"])
    assert et.kv_attention_kernel(layer, heads, 1).startswith("kv_attend_any")
    shares = group_launch.shares_layout()
    shares.shares = cursors.data_ptr()  # never read
    shares.vectors = slots
    out = torch.empty((slots, heads, 1, width), device=device)
    with pytest.raises(et.QuantizedError, match="takes q, k and v as tensors"):
        et.kv_attention_projected_into(layer, shares, (0, 1, 2), (None, None, None), cursors, 10000.0, 1.0,
                                       et.RotaryLayout.HALF_SPLIT, 1.0, 0, out)


@pytest.mark.parametrize("active_batch,context_window,window", [(5, 0, 0), (None, 60, 0), (None, 0, 33), (6, 80, 50)])
def test_attention_from_k_shares_with_inactive_slots_and_sliding_windows(et, device, active_batch, context_window, window):
    # the same bytes as the two launches it replaces, also where slots beyond the active batch get zeros and
    # where the context's or the operator's window cuts the cached rows
    rng = np.random.default_rng(9500 + (active_batch or 0) + context_window + window)
    slots, kv_heads, group, width, columns = 8, 2, 4, 128, 1024
    heads = group * kv_heads
    case = make_case(rng, slots=slots, query_heads=heads, kv_heads=kv_heads, width=width, block_size=16,
                     contexts=rng.integers(0, 150, slots), tokens=1, advances=[1] * slots, dtype=np.float16)
    scale = 1.0 / np.sqrt(width)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    sizes = (heads * width, kv_heads * width, kv_heads * width)
    plans = [et.RawLinear(et.GgmlQuant.Q4_K, rows, columns, slots) for rows in sizes]
    group_launch = et.LinearGroup(plans)
    weights = [dev(synth.random_weight(oracle.Q4_K, rows, columns, rng)) for rows in sizes]
    hidden = torch.empty(plans[0].prepared_input_bytes, dtype=torch.uint8, device=device)
    plans[0].prepare_input(dev(synth.random_activations(slots, columns, rng)), hidden)
    workspace = torch.empty(group_launch.workspace_bytes, dtype=torch.uint8, device=device)
    results = []
    for in_attention in (False, True):
        k_slab, v_slab = dev(case["k_slab"]), dev(case["v_slab"])
        cursors = dev(case["cursors"].view(np.int32))
        layer = et.KvLayer(k_slab, v_slab, case["block_size"], dev(case["table"].view(np.int32)), cursors,
                           dev(case["advances"].view(np.int32)), case["max_context"], active_batch=active_batch,
                           context_window=context_window)
        out = torch.full((slots, heads, 1, width), float("nan"), device=device)
        if in_attention:
            shares = group_launch.enqueue_prepared_shares(hidden, weights, workspace)
            et.kv_attention_projected_into(layer, shares, (0, 1, 2), (None, None, None), cursors, 10000.0, 1.0,
                                           et.RotaryLayout.INTERLEAVED_PAIRS, scale, window, out)
        else:
            ys = [torch.empty((slots, rows), device=device) for rows in sizes]
            group_launch.enqueue_prepared_then_rotary(hidden, weights, ys, workspace, (0, 1), cursors, 10000.0, 1.0,
                                                      et.RotaryLayout.INTERLEAVED_PAIRS, width)
            et.kv_attention_into(layer, ys[0].view(slots, heads, 1, width), ys[1].view(slots, kv_heads, 1, width),
                                 ys[2].view(slots, kv_heads, 1, width), scale, window, out)
        results.append([out, k_slab, v_slab])
    assert torch.isfinite(results[0][0]).all()
    if active_batch is not None:
        assert torch.all(results[1][0][active_batch:] == 0)
    for two, one in zip(*results):
        assert torch.equal(two.view(torch.uint8), one.view(torch.uint8))
