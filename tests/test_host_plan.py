"""Host logic of the C ABI, without a GPU: the library loads, exports every
symbol the header declares, and the plan step validates like the reference's
linear_requirements / embedding_requirements (crates/runtime-cpu/src/quantized.rs:297-365;
test cases of :923-978 and crates/graph/src/lib.rs:3523-3579).

Plans read metadata only, so tensors here live on the CPU or are zero-sized;
nothing is ever launched.
"""
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(et):
    # the operator boundary <-> libet_hip.so, the measurement aids <-> libet_hip_calibrate.so: each library
    # exports what its header declares, and the operators' library carries none of the aids
    from effect_torch_amd import _native
    boundary = open(os.path.join(ROOT, "include", "et_hip.h")).read()
    assert "calibration" not in boundary, "measurement aids belong in et_hip_calibrate.h"
    for name, lib, signatures in (("et_hip.h", _native.lib(), _native.SIGNATURES),
                                  ("et_hip_calibrate.h", _native.calibrate_lib(), _native.CALIBRATE_SIGNATURES)):
        header = open(os.path.join(ROOT, "include", name)).read()
        declared = set(re.findall(r"\b(et_hip_[a-z0-9_]+)\s*\(", header))
        assert declared, f"no declarations found in {name}"
        for symbol in sorted(declared):
            assert hasattr(lib, symbol), f"{symbol} is declared in include/{name} but not exported"
        assert declared == set(signatures), declared ^ set(signatures)
    for symbol in _native.CALIBRATE_SIGNATURES:
        assert not hasattr(_native.lib(), symbol), f"{symbol} belongs in the measurement library"


def test_codec_tables(et):
    Q = et.GgmlQuant
    assert [(q.ggml_name, q.block_bytes) for q in (Q.Q2_K, Q.Q3_K, Q.Q4_K, Q.Q5_K, Q.Q6_K)] == [
        ("Q2_K", 84), ("Q3_K", 110), ("Q4_K", 144), ("Q5_K", 176), ("Q6_K", 210)]
    assert (Q.Q8_0.block_bytes, Q.Q4_0.block_bytes) == (34, 18)
    assert Q.Q4_K.encoded_row_bytes(512) == 288      # gguf.rs:1117-1181
    assert Q.Q4_K.encoded_row_bytes(255) is None
    assert Q.Q4_K.encoded_row_bytes(14336) == 8064
    assert Q.from_name("Q5_K") is Q.Q5_K and Q.from_name("Q9_K") is None


def _w(rows, row_bytes):
    return torch.zeros((rows, row_bytes), dtype=torch.uint8)


def test_linear_plan_shapes(et):
    # crates/graph/src/lib.rs:3523-3579: x [2,256], W [3,144] u8, Q4_K -> [2,3] f32
    plan = et.linear_requirements(torch.zeros(2, 256), _w(3, 144), None, et.GgmlQuant.Q4_K, (3, 256))
    assert plan.output_shape == (2, 3) and plan.vectors == 2
    assert plan.output_bytes == 24  # crates/runtime-metal/src/quantized.rs:1393-1449
    plan = et.linear_requirements(torch.zeros(2, 5, 512), _w(7, 288), torch.zeros(7), et.GgmlQuant.Q4_K, (7, 512))
    assert plan.output_shape == (2, 5, 7) and plan.vectors == 10
    # ten vectors: fixed-point activations on the matrix cores, with its workspace planned
    assert plan.kernel in ("quantize_halves+gemm_h16", "quantize_halves+gemm_h16+reduce") and plan.workspace_bytes > 4 * 10 * 512
    plan5 = et.linear_requirements(torch.zeros(10, 512), _w(7, 352), None, et.GgmlQuant.Q5_K, (7, 512))
    assert plan5.kernel in ("quantize_halves+gemm_h16", "quantize_halves+gemm_h16+reduce")
    plan6 = et.linear_requirements(torch.zeros(10, 512), _w(7, 420), None, et.GgmlQuant.Q6_K, (7, 512))
    assert plan6.kernel in ("quantize_halves+gemm_h16", "quantize_halves+gemm_h16+reduce")
    for codec, row_bytes in ((et.GgmlQuant.Q3_K, 220), (et.GgmlQuant.Q2_K, 168)):
        batch = et.linear_requirements(torch.zeros(10, 512), _w(7, row_bytes), None, codec, (7, 512))
        assert batch.kernel in ("quantize_halves+gemm_h16", "quantize_halves+gemm_h16+reduce")
    plan8 = et.linear_requirements(torch.zeros(10, 512), _w(7, 544), None, et.GgmlQuant.Q8_0, (7, 512))
    assert plan8.kernel in ("quantize_limbs+gemm_i8", "quantize_limbs+gemm_i8+reduce")
    # the name says what the launches of one call are: three vectors per launch, the rest in one more
    for few, name in ((3, "gemv_limb"), (6, "gemv_limb x2"), (4, "gemv_limb+gemv_limb"), (5, "gemv_limb+gemv_limb")):
        plan3 = et.linear_requirements(torch.zeros(few, 512), _w(7, 288), None, et.GgmlQuant.Q4_K, (7, 512))
        assert plan3.kernel == name
    # a trailing launch of one vector takes its weights through LDS copies where a single vector would
    tall = et.linear_requirements(torch.zeros(4, 8192), _w(14336, 4608), None, et.GgmlQuant.Q4_K, (14336, 8192))
    assert tall.kernel == "gemv_limb+gemv_limb", tall.kernel
    three = et.linear_requirements(torch.zeros(3, 4096), _w(14336, 1344), None, et.GgmlQuant.Q2_K, (14336, 4096))
    assert three.kernel == "gemv_limb+gemv_limb_dma", three.kernel
    four = et.linear_requirements(torch.zeros(4, 4096), _w(1024 * 9, 2304), None, et.GgmlQuant.Q4_K, (1024 * 9, 4096))
    assert four.kernel == "gemv_mma"
    assert plan.algorithmic_bytes == 7 * 288 + 4 * 10 * 512 + 4 * 10 * 7 + 4 * 7
    plan = et.linear_requirements(torch.zeros(1, 256), _w(2, 210), None, et.GgmlQuant.Q6_K, (2, 256))
    assert plan.kernel == "gemv_limb"
    plan = et.linear_requirements(torch.zeros(1, 256), _w(2, 176), None, et.GgmlQuant.Q5_K, (2, 256))
    assert plan.kernel == "gemv_limb"
    plan = et.linear_requirements(torch.zeros(1, 256), _w(2, 110), None, et.GgmlQuant.Q3_K, (2, 256))
    assert plan.kernel == "gemv_limb"
    plan = et.linear_requirements(torch.zeros(2, 512), _w(2, 168), None, et.GgmlQuant.Q2_K, (2, 512))
    assert plan.kernel == "gemv_limb"
    plan = et.linear_requirements(torch.zeros(64, 256), _w(2, 144), None, et.GgmlQuant.Q4_K, (2, 256),
                                  et.ActivationMode.INT8)
    assert plan.kernel == "quantize_act+gemm_i8" and plan.workspace_bytes > 64 * 256
    # few 64-row tiles: K is shared over workgroups and a second kernel sums the shares
    few = et.linear_requirements(torch.zeros(32, 4096), _w(1024, 2304), None, et.GgmlQuant.Q4_K, (1024, 4096))
    many = et.linear_requirements(torch.zeros(32, 4096), _w(14336, 2304), None, et.GgmlQuant.Q4_K, (14336, 4096))
    assert few.kernel == "quantize_halves+gemm_h16+reduce" and many.kernel == "quantize_halves+gemm_h16"
    assert few.workspace_bytes >= 16 * 32 * 1024 * 4  # 16 tiles x 16 stages: one stage per share
    # empty output: nothing to dispatch
    plan = et.linear_requirements(torch.zeros(0, 256), _w(2, 144), None, et.GgmlQuant.Q4_K, (2, 256))
    assert plan.output_shape == (0, 2) and plan.kernel == "none"


def test_linear_plan_rejects_malformed_geometry(et):
    Q4 = et.GgmlQuant.Q4_K
    x = torch.zeros(1, 256)
    with pytest.raises(et.QuantizedError, match="input must be rank >= 2 f32"):
        et.linear_requirements(torch.zeros(256), _w(1, 144), None, Q4, (1, 256))
    with pytest.raises(et.QuantizedError, match="input must be rank >= 2 f32"):
        et.linear_requirements(torch.zeros(1, 256, dtype=torch.float16), _w(1, 144), None, Q4, (1, 256))
    with pytest.raises(et.QuantizedError, match=r"expected input trailing width 256, got \[1, 512\]"):
        et.linear_requirements(torch.zeros(1, 512), _w(1, 144), None, Q4, (1, 256))
    # wrong rank / width-1 / offset view -> "exact contiguous" (quantized.rs:923-960)
    with pytest.raises(et.QuantizedError, match="exact contiguous"):
        et.linear_requirements(x, torch.zeros(144, dtype=torch.uint8), None, Q4, (1, 256))
    with pytest.raises(et.QuantizedError, match="exact contiguous"):
        et.linear_requirements(x, _w(1, 143), None, Q4, (1, 256))
    offset_view = torch.zeros(145, dtype=torch.uint8)[1:].reshape(1, 144)
    with pytest.raises(et.QuantizedError, match=r"expected exact contiguous packed Q4_K weight \[1, 144\] u8"):
        et.linear_requirements(x, offset_view, None, Q4, (1, 256))
    with pytest.raises(et.QuantizedError, match="exact contiguous"):
        et.linear_requirements(x, torch.zeros((1, 288), dtype=torch.uint8)[:, ::2], None, Q4, (1, 256))
    with pytest.raises(et.QuantizedError, match="exact contiguous"):
        et.linear_requirements(x, torch.zeros((1, 144), dtype=torch.float16), None, Q4, (1, 256))
    # wrong codec for the bytes: graph/lib.rs:3570-3579
    with pytest.raises(et.QuantizedError, match=r"expected exact contiguous packed Q5_K weight \[3, 176\] u8"):
        et.linear_requirements(torch.zeros(2, 256), _w(3, 144), None, et.GgmlQuant.Q5_K, (3, 256))
    with pytest.raises(et.QuantizedError, match="logical row width 255 is invalid for Q4_K"):
        et.linear_requirements(torch.zeros(1, 255), _w(1, 0), None, Q4, (1, 255))
    with pytest.raises(et.QuantizedError, match="byte size overflow"):
        et.linear_requirements(x, torch.zeros(144, dtype=torch.uint8), None, Q4, (2**64 - 1, 256))
    with pytest.raises(et.QuantizedError, match=r"bias must be \[1\] f32, got \[2\] f32"):
        et.linear_requirements(x, _w(1, 144), torch.zeros(2), Q4, (1, 256))
    with pytest.raises(et.QuantizedError, match=r"bias must be \[1\] f32, got \[1\] f64"):
        et.linear_requirements(x, _w(1, 144), torch.zeros(1, dtype=torch.float64), Q4, (1, 256))
    with pytest.raises(et.QuantizedError, match="int8 activation mode is not available for Q6_K"):
        et.linear_requirements(x, _w(1, 210), None, et.GgmlQuant.Q6_K, (1, 256), et.ActivationMode.INT8)


def test_workspace_sizes_are_checked_products(et):
    # rows, columns and vectors each fit 32 bits; vectors * columns * 4 does not fit 64: refused, not wrapped
    with pytest.raises(et.QuantizedError, match="workspace byte size overflow"):
        et.RawLinear(et.GgmlQuant.Q4_K, 1, 2**32 - 256, 2**32 - 1)
    with pytest.raises(et.QuantizedError, match="workspace byte size overflow"):
        et.RawLinear(et.GgmlQuant.Q8_0, 64, 2**32 - 256, 2**32 - 1, False, et.ActivationMode.INT8)
    # the largest sizes that do fit plan as before
    plan = et.RawLinear(et.GgmlQuant.Q4_K, 14336, 4096, 512)
    assert plan.requirements.workspace_bytes >= 512 * 4096 * 4


def test_embedding_plan(et):
    Q5 = et.GgmlQuant.Q5_K
    plan = et.embedding_requirements(torch.zeros((2, 3), dtype=torch.int64), _w(3, 176), Q5, (3, 256))
    assert plan.output_shape == (2, 3, 256) and plan.output_bytes == 2 * 3 * 256 * 4
    plan = et.embedding_requirements(torch.zeros(2, dtype=torch.uint32), _w(3, 176), Q5, (3, 256))
    assert plan.output_shape == (2, 256)
    with pytest.raises(et.QuantizedError, match="indexes must be u32 or i64, got f32"):
        et.embedding_requirements(torch.zeros(2), _w(3, 176), Q5, (3, 256))
    with pytest.raises(et.QuantizedError, match="quantized_embedding: expected exact contiguous"):
        et.embedding_requirements(torch.zeros(2, dtype=torch.int64), _w(3, 175), Q5, (3, 256))
    with pytest.raises(et.QuantizedError, match="quantized_embedding: logical row width 100"):
        et.embedding_requirements(torch.zeros(2, dtype=torch.int64), _w(3, 0), Q5, (3, 100))


def test_execute_revalidates_against_the_plan_and_observes_cancellation(et):
    # validate_linear_execution (quantized.rs:367-415) runs before anything is
    # enqueued, so these never reach a device.
    Q4 = et.GgmlQuant.Q4_K
    plan = et.linear_requirements(torch.zeros(2, 256), _w(3, 144), None, Q4, (3, 256))
    dst = torch.zeros(2, 3)
    with pytest.raises(et.QuantizedError, match="input does not match the immutable plan"):
        et.linear_into(torch.zeros(2, 512), _w(3, 144), None, Q4, dst, plan, stream=0)
    with pytest.raises(et.QuantizedError, match="exact contiguous"):
        et.linear_into(torch.zeros(2, 256), _w(3, 143), None, Q4, dst, plan, stream=0)
    with pytest.raises(et.QuantizedError, match="bias does not match the immutable plan"):
        et.linear_into(torch.zeros(2, 256), _w(3, 144), torch.zeros(3), Q4, dst, plan, stream=0)
    with pytest.raises(et.QuantizedError, match="destination does not match the logical node shape"):
        et.linear_into(torch.zeros(2, 256), _w(3, 144), None, Q4, torch.zeros(2, 4), plan, stream=0)
    flag = et.CancellationFlag()
    flag.cancel()
    with pytest.raises(et.Cancelled) as info:
        et.linear_into(torch.zeros(2, 256), _w(3, 144), None, Q4, dst, plan, flag, stream=0)
    assert str(info.value) == "operation aborted"  # quantized.rs:980-1000
    eplan = et.embedding_requirements(torch.zeros(1, dtype=torch.uint32), _w(1, 210), et.GgmlQuant.Q6_K, (1, 256))
    from effect_torch_amd import _native as N
    import ctypes
    from effect_torch_amd.quantized import _Desc
    descs = (_Desc(torch.zeros(1, dtype=torch.uint32)), _Desc(_w(1, 210)), _Desc(torch.zeros(1, 256)))
    status = N.lib().et_hip_embedding_into(eplan._handle, descs[0].ref, descs[1].ref, descs[2].ref,
                                           None, None, flag.ptr)
    assert status == N.ERR_CANCELLED and N.last_error() == "operation aborted"


def test_embedding_status_wording(et):
    # quantized.rs:899-921: "... index {i} is outside 0..{rows}"
    import ctypes
    import struct
    from effect_torch_amd import _native as N
    plan = et.embedding_requirements(torch.zeros(1, dtype=torch.int64), _w(1, 84), et.GgmlQuant.Q2_K, (1, 256))
    ok = ctypes.create_string_buffer(struct.pack("<Qq", 2**64 - 1, 0), 16)
    assert N.lib().et_hip_embedding_status_check(plan._handle, ok) == N.OK
    for value in (-1, 1):
        bad = ctypes.create_string_buffer(struct.pack("<Qq", 0, value), 16)
        assert N.lib().et_hip_embedding_status_check(plan._handle, bad) == N.ERR_EXECUTION
        assert N.last_error() == f"quantized_embedding: index {value} is outside 0..1"


def _kv_layer(et, torch, *, slots=2, kv_heads=2, width=8, max_tokens=32, block_size=4, dtype=None, **kw):
    dtype = dtype or torch.float32
    slab = torch.zeros(max_tokens, kv_heads, width, dtype=dtype)
    table = torch.zeros(slots, 4, dtype=torch.int32)
    zeros = torch.zeros(slots, dtype=torch.int32)
    return et.KvLayer(slab, slab.clone(), block_size, table, zeros, zeros.clone(), kw.pop("max_context", 16), **kw)


def test_kv_attention_validation_follows_the_reference(et):
    import torch
    layer = _kv_layer(et, torch)
    q = torch.zeros(2, 4, 3, 8)
    kv = torch.zeros(2, 2, 3, 8)
    out = torch.zeros_like(q)

    def fails(message, *args):
        with pytest.raises(et.QuantizedError, match=message):
            et.kv_attention_into(layer, *args, stream=0)

    fails("expected matching rank-4-or-higher f32 tensors", q[0], kv[0], kv[0], 1.0, None, out[0])
    fails("expected matching rank-4-or-higher f32 tensors", q.double(), kv, kv, 1.0, None, out)
    fails("expected matching rank-4-or-higher f32 tensors", q, kv, kv, 1.0, None, out[:, :2])
    fails("incompatible grouped-query q/k/v shapes", q, kv[:, :, :2], kv, 1.0, None, out)
    fails("incompatible grouped-query q/k/v shapes", q, torch.zeros(2, 3, 3, 8), torch.zeros(2, 3, 3, 8), 1.0, None, out)
    fails("incompatible grouped-query q/k/v shapes", q[:1], kv, kv, 1.0, None, out[:1])
    fails("batch 3 does not match 2 kv slots", torch.zeros(3, 4, 3, 8), torch.zeros(3, 2, 3, 8),
          torch.zeros(3, 2, 3, 8), 1.0, None, torch.zeros(3, 4, 3, 8))
    fails(r"layer shape \[1, 8\] does not match pool geometry \[2, 8\]", q, kv[:, :1], kv[:, :1], 1.0, None, out)
    fails("must be contiguous", q.transpose(0, 1).contiguous().transpose(0, 1), kv, kv, 1.0, None, out)
    flag = et.CancellationFlag()
    flag.cancel()
    with pytest.raises(et.Cancelled, match="operation aborted"):
        et.kv_attention_into(layer, q, kv, kv, 1.0, None, out, cancelled=flag, stream=0)
    with pytest.raises(et.QuantizedError, match=r"kv pool: dtype must be f32, f16, bf16 or u8 \(int8-quantized\)"):
        _kv_layer(et, torch, dtype=torch.float64)
    with pytest.raises(et.QuantizedError, match="the u8 tier needs contiguous f32 scales"):
        _kv_layer(et, torch, dtype=torch.uint8)


def test_kv_attention_launch_shapes_and_status_wording(et):
    import ctypes
    import struct
    import torch
    from effect_torch_amd import _native
    decode = _kv_layer(et, torch, slots=32, kv_heads=8, width=128, max_tokens=32 * 2048, block_size=16,
                       dtype=torch.float16, max_context=2048)
    # 256 rows of queries: one eight-wave workgroup per compute unit, the context is not split
    assert et.kv_attention_kernel(decode, 32, 1) == "kv_attend"
    assert et.kv_attention_workspace_bytes(decode, 32, 1) == 0
    few = _kv_layer(et, torch, slots=4, kv_heads=8, width=128, max_tokens=4 * 2048, block_size=16,
                    dtype=torch.float16, max_context=2048)
    assert et.kv_attention_kernel(few, 32, 1) == "kv_attend+kv_merge"
    assert et.kv_attention_workspace_bytes(few, 32, 1) % (4 * 32 * 130 * 4) == 0
    short = _kv_layer(et, torch, slots=512, kv_heads=8, width=128, max_tokens=4096, block_size=16,
                      dtype=torch.float16, max_context=8)
    assert et.kv_attention_kernel(short, 32, 1) == "kv_attend"
    assert et.kv_attention_workspace_bytes(short, 32, 1) == 0
    odd = _kv_layer(et, torch, width=12)
    assert et.kv_attention_kernel(odd, 4, 1).startswith("kv_attend_any")
    assert et.kv_attention_kernel(odd, 3, 1) == ""  # 3 query heads over 2 kv heads

    def message(word, slot=0):
        layer = decode.struct()
        words = [0] * 32
        words[slot] = word
        words[-1] = (3 << 56) | 5  # a later slot's failure is not the one reported
        buf = ctypes.create_string_buffer(struct.pack("<32Q", *words), 256)
        status = _native.lib().et_hip_kv_attention_status_check(ctypes.byref(layer), 7, buf)
        return status, _native.last_error()

    layer = decode.struct()
    clean = ctypes.create_string_buffer(256)
    assert _native.lib().et_hip_kv_attention_status_check(ctypes.byref(layer), 7, clean) == 0
    assert message((1 << 56) | 9, slot=3) == (2, "kv attention: advance 9 out of range for chunk length 7")
    assert message((1 << 56) | 0) == (2, "kv attention: advance 0 out of range for chunk length 7")
    assert message((2 << 56) | 70000) == (2, "kv attention: live context 70000 exceeds pool capacity 65536")
    # cursor + advance is a 33-bit sum: the value field is 56 bits wide
    assert message((2 << 56) | (1 << 32)) == (2, "kv attention: live context 4294967296 exceeds pool capacity 65536")
    assert message((3 << 56) | 41, slot=30) == (2, "kv attention: block table of slot 30 does not cover 41 tokens")


def test_decode_operator_validation(et):
    import torch
    x = torch.zeros(2, 8)
    with pytest.raises(et.QuantizedError, match="rms_norm: input must have rank at least 1"):
        et.rms_norm_into(torch.zeros(()), None, 1e-5, torch.zeros(()), stream=0)
    with pytest.raises(et.QuantizedError, match="rms_norm: weight must match the last dimension and dtype"):
        et.rms_norm_into(x, torch.zeros(2, 4), 1e-5, torch.zeros(2, 8), stream=0)
    with pytest.raises(et.QuantizedError, match="rms_norm: zero-sized dimensions are unsupported"):
        et.rms_norm_into(torch.zeros(2, 0), None, 1e-5, torch.zeros(2, 0), stream=0)
    offsets = torch.zeros(3, dtype=torch.int32)
    with pytest.raises(et.QuantizedError, match="rotary: expected a float rank >= 2 tensor with even head dimension"):
        et.rotary_into(torch.zeros(2, 7), offsets[:1], 1e4, 1.0, et.RotaryLayout.HALF_SPLIT, torch.zeros(2, 7), stream=0)
    with pytest.raises(et.QuantizedError, match="rotary embedding: 3 offsets for batch 2"):
        et.rotary_into(torch.zeros(2, 4, 1, 8), offsets, 1e4, 1.0, et.RotaryLayout.HALF_SPLIT,
                       torch.zeros(2, 4, 1, 8), stream=0)
    with pytest.raises(et.QuantizedError, match="silu_mul: gate, up and the destination must have one shape"):
        et.silu_mul_into(x, torch.zeros(2, 4), torch.zeros(2, 8), stream=0)
    with pytest.raises(et.QuantizedError, match="sample: logits must be non-empty"):
        et.greedy_tokens(torch.zeros(2, 0), stream=0)
    with pytest.raises(et.QuantizedError, match="sample: vocabulary 1048577 exceeds limit 1048576"):
        et.greedy_tokens(torch.zeros(1, 1048577), stream=0)
    table = torch.zeros(10, 4, dtype=torch.float16)
    with pytest.raises(et.QuantizedError, match="index_select destination shape mismatch at dimension 0: expected 3, got 2"):
        et.gather_rows_into(table, torch.zeros(3, dtype=torch.int64), torch.zeros(2, 4, dtype=torch.float16), stream=0)
    with pytest.raises(et.QuantizedError, match="index_select: indexes must be u32 or i64"):
        et.gather_rows_into(table, torch.zeros(3, dtype=torch.float32), torch.zeros(3, 4, dtype=torch.float16), stream=0)


def test_raw_pointer_wrappers_refuse_operands_smaller_than_the_plan(et):
    # The C entry points take raw device pointers; a buffer smaller than what the plan touches would make a
    # kernel read or write past it. The host mirror checks sizes first and raises before anything is enqueued.
    import torch
    plan = et.RawLinear(et.GgmlQuant.Q4_K, 14336, 4096, 32)
    x = torch.zeros(32, 4096)
    y = torch.zeros(32, 14336)
    full = torch.zeros((14336, 2304), dtype=torch.uint8)
    with pytest.raises(et.QuantizedError, match="weight holds 18874368 bytes, the plan .* touches 33030144"):
        plan.enqueue(x, full[:8192], None, y)
    with pytest.raises(et.QuantizedError, match="y holds"):
        plan.enqueue(x, full, None, y[:, :4096].contiguous())
    with pytest.raises(et.QuantizedError, match="activations of shape"):
        plan.enqueue(x[:16], full, None, y)
    prepared = torch.zeros(max(plan.prepared_input_bytes, 16), dtype=torch.uint8)
    with pytest.raises(et.QuantizedError, match="prepared input holds"):
        plan.enqueue_prepared(prepared[:100], full, None, y)
    with pytest.raises(et.QuantizedError, match="residual holds"):
        plan.enqueue_prepared(prepared, full, None, y, residual=torch.zeros(8))
    group = et.LinearGroup([plan, plan])
    with pytest.raises(et.QuantizedError, match="weight holds"):
        group.enqueue_prepared(prepared, [full, full[:100]], [y, y])


def test_projections_left_as_k_shares_layout_and_validation(et):
    import torch
    q4k = et.GgmlQuant.Q4_K
    plans = [et.RawLinear(q4k, rows, 4096, 32) for rows in (4096, 1024, 1000)]
    group = et.LinearGroup(plans)
    layout = group.shares_layout()
    # 64-row tiles, two K shares; the ragged last member is rounded up to whole tiles
    assert (layout.count, layout.vectors, layout.launch_rows) == (2, 32, 4096 + 1024 + 1024)
    assert list(layout.first_row)[:3] == [0, 4096, 5120]
    assert group.workspace_bytes == layout.count * 32 * layout.launch_rows * 4
    big = et.LinearGroup([et.RawLinear(q4k, 14336, 4096, 32) for _ in range(2)])
    assert big.shares_layout().count == 1  # 128-row tiles fill the device: no shares to leave
    prepared = torch.zeros(plans[0].prepared_input_bytes, dtype=torch.uint8)
    heavy = torch.zeros(14336 * 2304, dtype=torch.uint8)
    with pytest.raises(et.QuantizedError, match="this group does not share K over workgroups"):
        big.enqueue_prepared_shares(prepared, [heavy, heavy], torch.zeros(16, dtype=torch.uint8), stream=0)
    weights = [torch.zeros(rows * 2304, dtype=torch.uint8) for rows in (4096, 1024, 1000)]
    with pytest.raises(et.QuantizedError, match="workspace of 16 bytes is smaller than the"):
        group.enqueue_prepared_shares(prepared, weights, torch.zeros(16, dtype=torch.uint8), stream=0)

    decode = _kv_layer(et, torch, slots=32, kv_heads=8, width=128, max_tokens=32 * 64, block_size=16,
                       dtype=torch.float16, max_context=40)
    cursors = torch.zeros(32, dtype=torch.int32)
    out = torch.zeros(32, 32, 1, 128)
    layout.shares = prepared.data_ptr()  # validation never reads it

    def fails(message, layer=decode, shares=layout, offsets=cursors, rotary=et.RotaryLayout.HALF_SPLIT, destination=out):
        with pytest.raises(et.QuantizedError, match=message):
            et.kv_attention_projected_into(layer, shares, (0, 1, 2), (None, None, None), offsets, 500000.0, 1.0, rotary,
                                           1.0, None, destination, stream=0)

    fails("rotary embedding: 5 offsets for batch 32", offsets=cursors[:5].contiguous())
    fails("rotary: unknown layout 7", rotary=7)
    fails("projections as K shares take one token per slot", destination=torch.zeros(32, 32, 3, 128))
    fails("expected matching rank-4-or-higher f32 tensors", destination=torch.zeros(32, 1, 128))
    fewer = et.LinearGroup([et.RawLinear(q4k, rows, 4096, 32) for rows in (2048, 1024, 1024)]).shares_layout()
    fewer.shares = prepared.data_ptr()
    fails("the projections do not fit the rows of the shares", shares=fewer)
    other = et.LinearGroup([et.RawLinear(q4k, rows, 4096, 16) for rows in (4096, 1024, 1024)]).shares_layout()
    other.shares = prepared.data_ptr()
    fails(r"the K shares do not describe \[32\] projected vectors", shares=other)
    odd = _kv_layer(et, torch, slots=32, kv_heads=8, width=12, max_tokens=32 * 64, block_size=16, max_context=40)
    narrow = et.LinearGroup([et.RawLinear(q4k, rows, 4096, 32) for rows in (32 * 12, 8 * 12, 8 * 12)]).shares_layout()
    narrow.shares = prepared.data_ptr()
    fails("this geometry's kernel takes q, k and v as tensors", layer=odd, shares=narrow,
          destination=torch.zeros(32, 32, 1, 12))
