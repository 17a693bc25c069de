"""GPU parity: the HIP path behind the C ABI against the CPU oracle on the same seeded inputs.

Bars: decoded weights bit-exact; f32-activation outputs within
``|a-b| <= 1e-3 * max(|b|, 1)`` (the reference's own form,
crates/runtime-metal/src/executable.rs:8372-8381, at the tolerance the workload
states); the int8-activation path equals its own CPU restatement within the
same 1e-3 bar (integer dots are exact, only the f32 summation order differs)
and stays within ``2e-2 * max(|b|, rms(b))`` of the f32 reference.
"""
import numpy as np
import pytest
import torch

import oracle
import packers
import ref_fixtures as rf
from effect_torch_amd import synth

pytestmark = pytest.mark.gpu

ALL = oracle.ALL_CODECS
K_QUANTS = oracle.K_QUANTS


def close(got, want, tol=1e-3, oracle_noise=4e-5):
    """|got - want| <= tol * max(|want|, 1) [+ oracle_noise * rms(want row)].

    The second term allows for the rounding noise of the ORACLE's own strictly
    sequential f32 sum (about eps * sqrt(K / 6) * rms for K terms, 4 sigma),
    which at K ~ 10^4 and |y| >> 1 exceeds 1e-3 * 1 for outputs that happen to
    land near zero. Pass ``oracle_noise=0`` when ``want`` is exact (f64)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    rms = np.sqrt(np.mean(want.reshape(-1, want.shape[-1]) ** 2, axis=-1)).reshape(want.shape[:-1] + (1,))
    bound = tol * np.maximum(np.abs(want), 1.0) + oracle_noise * rms
    bad = np.abs(got - want) > bound
    assert not bad.any(), (f"{bad.sum()} of {bad.size} outside {tol}: max |err| "
                           f"{np.abs(got - want).max():.4g} at {np.unravel_index(np.argmax(np.abs(got - want)), got.shape)}")


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def to_dev(array, device):
    return torch.from_numpy(np.ascontiguousarray(array)).to(device)


def finite_random_weight(codec, rows, columns, rng):
    """Uniform random bytes everywhere; fp16 fields forced finite (any sign, subnormals included)."""
    w = rng.integers(0, 256, (rows * columns // synth.BLOCK_VALUES[codec], synth.BLOCK_BYTES[codec]),
                     dtype=np.uint8)
    for off in synth._FP16_FIELDS[codec]:
        hi = w[:, off + 1]
        hi[(hi & 0x7C) == 0x7C] &= 0xBF  # exponent 31 (inf/nan) -> exponent 15 or 23
    return w.reshape(rows, -1)


# --------------------------------------------------------------------------- dequant

@pytest.mark.parametrize("codec", K_QUANTS)
def test_dequant_reference_fixtures(et, device, codec):
    block = rf.FIXTURES[codec]["bytes"]
    w = np.tile(block, 6).reshape(3, -1)
    out = et.dequantize_rows(to_dev(w, device), et.GgmlQuant(codec), (3, 512)).cpu().numpy()
    want = np.tile(rf.expected_values(codec), 6).reshape(3, 512)
    assert np.array_equal(bits(out), bits(want))


@pytest.mark.parametrize("codec", ALL)
def test_dequant_bit_exact_on_packed_random_fields(et, device, codec):
    rng = np.random.default_rng(500 + codec)
    values = oracle.block_values(codec)
    per_row = 512 // values
    blocks = [packers.random_block(codec, rng) for _ in range(64 * per_row)]
    w = np.concatenate([b for b, _ in blocks]).reshape(64, -1)
    want = np.concatenate([v for _, v in blocks]).reshape(64, 512)
    out = et.dequantize_rows(to_dev(w, device), et.GgmlQuant(codec), (64, 512)).cpu().numpy()
    assert np.array_equal(bits(out), bits(want))
    assert np.array_equal(bits(out), bits(oracle.decode_rows(codec, w, 512)))


@pytest.mark.parametrize("codec", ALL)
def test_dequant_bit_exact_on_random_bytes(et, device, codec):
    rng = np.random.default_rng(600 + codec)
    rows, columns = 257, 2048
    w = finite_random_weight(codec, rows, columns, rng)
    out = et.dequantize_rows(to_dev(w, device), et.GgmlQuant(codec), (rows, columns)).cpu().numpy()
    assert np.array_equal(bits(out), bits(oracle.decode_rows(codec, w, columns)))


def test_dequant_full_size_q4k_matches_oracle_checksum(et, device):
    rng = np.random.default_rng(0xE77C0DE2)
    rows, columns = 14336, 4096
    w = synth.random_weight(synth.Q4_K, rows, columns, rng)
    out = et.dequantize_rows(to_dev(w, device), et.GgmlQuant.Q4_K, (rows, columns))
    got = out.cpu().numpy()
    want = oracle.decode_rows(oracle.Q4_K, w, columns)
    assert np.array_equal(bits(got), bits(want))


# --------------------------------------------------------------------------- embedding

@pytest.mark.parametrize("index_dtype", [torch.uint32, torch.int64])
def test_embedding_kat(et, device, index_dtype):
    # quantized.rs:867-897
    table = np.zeros((3, 176), np.uint8)
    table[1] = rf.FIXTURES[rf.Q5_K]["bytes"]
    indexes = torch.tensor([1, 1], dtype=index_dtype).to(device)
    w = to_dev(table, device)
    plan = et.embedding_requirements(indexes, w, et.GgmlQuant.Q5_K, (3, 256))
    out = torch.full(plan.output_shape, float("nan"), dtype=torch.float32, device=device)
    et.embedding_into(indexes, w, et.GgmlQuant.Q5_K, out, plan)
    want = rf.expected_values(rf.Q5_K)
    got = out.cpu().numpy()
    assert np.array_equal(got[0], want) and np.array_equal(got[1], want)


@pytest.mark.parametrize("codec", ALL)
def test_embedding_strided_indexes_all_codecs(et, device, codec):
    rng = np.random.default_rng(700 + codec)
    rows, columns = 50, 1024
    table = finite_random_weight(codec, rows, columns, rng)
    storage = rng.integers(0, rows, 64).astype(np.int64)
    view = torch.from_numpy(storage).to(device)[4:].reshape(10, 6)[::2, 1:5]  # [5, 4], strided
    w = to_dev(table, device)
    plan = et.embedding_requirements(view, w, et.GgmlQuant(codec), (rows, columns))
    assert plan.output_shape == (5, 4, columns)
    out = torch.empty(plan.output_shape, dtype=torch.float32, device=device)
    et.embedding_into(view, w, et.GgmlQuant(codec), out, plan)
    want = oracle.embedding_into(codec, rows, columns, np.ascontiguousarray(view.cpu().numpy()), table)
    assert np.array_equal(bits(out.cpu().numpy()), bits(want))


@pytest.mark.parametrize("bad", [-1, 1, 2**40])
def test_embedding_reports_out_of_range_indexes(et, device, bad):
    # quantized.rs:899-921
    table = to_dev(rf.FIXTURES[rf.Q2_K]["bytes"].reshape(1, 84), device)
    indexes = torch.tensor([0, bad, 0, 7], dtype=torch.int64, device=device)
    plan = et.embedding_requirements(indexes, table, et.GgmlQuant.Q2_K, (1, 256))
    out = torch.zeros(plan.output_shape, dtype=torch.float32, device=device)
    with pytest.raises(et.QuantizedError) as info:
        et.embedding_into(indexes, table, et.GgmlQuant.Q2_K, out, plan)
    assert str(info.value) == f"quantized_embedding: index {bad} is outside 0..1"
    # valid rows were still decoded, the bad ones skipped
    got = out.cpu().numpy()
    assert np.array_equal(got[0], rf.expected_values(rf.Q2_K)) and not got[1].any()
    u32 = torch.tensor([0, 5], dtype=torch.uint32).to(device)
    plan = et.embedding_requirements(u32, table, et.GgmlQuant.Q2_K, (1, 256))
    with pytest.raises(et.QuantizedError, match="index 5 is outside 0..1"):
        et.embedding_into(u32, table, et.GgmlQuant.Q2_K, torch.zeros((2, 256), device=device), plan)


# --------------------------------------------------------------------------- f32-activation linear

def run_linear(et, device, codec, rows, columns, x, weight, bias=None, mode=None):
    mode = et.ActivationMode.F32 if mode is None else mode
    xt = x if isinstance(x, torch.Tensor) else to_dev(x, device)
    bt = None if bias is None else to_dev(bias, device)
    y = et.quantized_linear(xt, to_dev(weight, device), bt, et.GgmlQuant(codec), (rows, columns), mode)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def test_linear_kats(et, device):
    # quantized.rs:827-865 and executable.rs:4881-4918
    x = np.zeros(1024, np.float32)
    x[:576] = 1.0
    weight = np.tile(rf.FIXTURES[rf.Q4_K]["bytes"], 4).reshape(2, 288)
    y = run_linear(et, device, oracle.Q4_K, 2, 512, x.reshape(2, 512), weight, np.array([0.5, -0.5], np.float32))
    assert y.tolist() == [[4096.5, 4095.5], [512.5, 511.5]]
    weight = np.tile(rf.FIXTURES[rf.Q4_K]["bytes"], 3).reshape(3, 144)
    y = run_linear(et, device, oracle.Q4_K, 3, 256, np.ones((1, 256), np.float32), weight)
    assert y.tolist() == [[2048.0, 2048.0, 2048.0]]


@pytest.mark.parametrize("codec", K_QUANTS)
@pytest.mark.parametrize("vectors", [1, 3, 4, 5, 16, 17])
def test_linear_cross_backend_protocol(et, device, codec, vectors):
    # crates/runtime-metal/src/executable.rs:8458-8505, at the reference's own 1e-4
    columns = 512
    i = np.arange(vectors * columns)
    x = (((i * 7 + i // columns * 3) % 17).astype(np.float32) * np.float32(0.125) - np.float32(1.0))
    x = x.reshape(vectors, columns)
    weight = np.tile(rf.FIXTURES[codec]["bytes"], 4).reshape(2, -1)
    bias = np.array([0.25, -0.5], np.float32) if vectors == 1 else None
    got = run_linear(et, device, codec, 2, columns, x, weight, bias)
    want = oracle.linear_into(codec, 2, columns, x, weight, bias)
    close(got, want, 1e-4)


@pytest.mark.parametrize("codec", ALL)
@pytest.mark.parametrize("rows,columns", [(1, 256), (37, 512), (130, 4096), (64, 14336), (9, 1280)])
@pytest.mark.parametrize("vectors", [1, 2, 3, 4, 7])
def test_linear_matches_oracle(et, device, codec, rows, columns, vectors):
    rng = np.random.default_rng(rows * 131 + columns + vectors + codec)
    weight = synth.random_weight(codec, rows, columns, rng)
    x = synth.random_activations(vectors, columns, rng)
    bias = rng.standard_normal(rows).astype(np.float32) if (rows + vectors) % 2 else None
    got = run_linear(et, device, codec, rows, columns, x, weight, bias)
    want = oracle.linear_into(codec, rows, columns, x, weight, bias)
    assert got.shape == (vectors, rows)
    close(got, want)
    # against the exact value of the same contraction (bit-exact decode, f64 sum): no allowance
    exact = x.astype(np.float64) @ oracle.decode_rows(codec, weight, columns).astype(np.float64).T
    if bias is not None:
        exact = exact + bias.astype(np.float64)
    close(got, exact, oracle_noise=0)


@pytest.mark.parametrize("codec", [oracle.Q2_K, oracle.Q3_K, oracle.Q4_K, oracle.Q5_K, oracle.Q6_K, oracle.Q8_0, oracle.Q4_0])
@pytest.mark.parametrize("vectors,rows,columns", [(7, 129, 256), (12, 64, 2304), (33, 1, 512), (65, 300, 1024),
                                                  (100, 130, 4096), (130, 257, 768), (200, 63, 256)])
def test_linear_many_vectors_f32_matrix_core_tiles(et, device, codec, vectors, rows, columns):
    # seven or more vectors: fixed-point activations on the matrix cores (two 12-bit halves as half
    # floats for the K-quants, three byte limbs for the 32-wide codecs); ragged tiles on both sides, one and
    # several stages of 256 columns, ring turns with padding stages
    rng = np.random.default_rng(codec * 11 + vectors + rows + columns)
    weight = synth.random_weight(codec, rows, columns, rng)
    x = synth.random_activations(vectors, columns, rng)
    x[vectors // 2, :64] = 0.0  # all-zero blocks: unit 0
    bias = rng.standard_normal(rows).astype(np.float32) if rows % 2 else None
    plan = et.linear_requirements(torch.zeros(vectors, columns), torch.zeros((rows, weight.shape[1]), dtype=torch.uint8),
                                  None, et.GgmlQuant(codec), (rows, columns))
    k_quants = (oracle.Q2_K, oracle.Q3_K, oracle.Q4_K, oracle.Q5_K, oracle.Q6_K)
    family = "quantize_halves+gemm_h16" if codec in k_quants else "quantize_limbs+gemm_i8"
    assert plan.kernel in (family, family + "+reduce")
    got = run_linear(et, device, codec, rows, columns, x, weight, bias)
    if codec not in k_quants:
        # a width that is not a whole number of 256-column stages stays on the GEMV kernels
        odd = columns + 32
        weight_odd = synth.random_weight(codec, rows, odd, rng)
        x_odd = synth.random_activations(vectors, odd, rng)
        plan = et.linear_requirements(torch.zeros(vectors, odd), torch.zeros((rows, weight_odd.shape[1]), dtype=torch.uint8),
                                      None, et.GgmlQuant(codec), (rows, odd))
        assert plan.kernel.startswith("gemv")
        close(run_linear(et, device, codec, rows, odd, x_odd, weight_odd, bias),
              oracle.linear_into(codec, rows, odd, x_odd, weight_odd, bias))
    close(got, oracle.linear_into(codec, rows, columns, x, weight, bias))
    exact = x.astype(np.float64) @ oracle.decode_rows(codec, weight, columns).astype(np.float64).T
    if bias is not None:
        exact = exact + bias.astype(np.float64)
    close(got, exact, oracle_noise=0)


@pytest.mark.parametrize("mode", ["F32", "INT8"])
@pytest.mark.parametrize("codec,vectors,rows,columns", [(oracle.Q4_K, 32, 1024, 4096), (oracle.Q4_K, 32, 4096, 4096),
                                                        (oracle.Q4_K, 32, 4096, 14336), (oracle.Q5_K, 32, 4096, 4096),
                                                        (oracle.Q5_K, 64, 14336, 4096), (oracle.Q6_K, 32, 1024, 4096),
                                                        (oracle.Q6_K, 32, 4096, 14336), (oracle.Q3_K, 32, 4096, 4096),
                                                        (oracle.Q2_K, 64, 14336, 4096), (oracle.Q2_K, 32, 1024, 4096),
                                                        (oracle.Q8_0, 40, 700, 2304),
                                                        (oracle.Q4_0, 9, 65, 1280)])
def test_linear_few_tiles_share_k_over_workgroups(et, device, mode, codec, vectors, rows, columns):
    # decode-batch shapes: far fewer 64-row tiles than compute units, so the stages of K are shared
    # out over several workgroups per tile and summed by a second kernel, in a fixed order
    if codec in (oracle.Q2_K, oracle.Q3_K, oracle.Q5_K, oracle.Q6_K) and mode == "INT8":
        # the documented refusal (include/et_hip.h, et_activation_mode): these codecs' batches run in f32 mode
        with pytest.raises(et.QuantizedError, match="int8 activation mode is not available for"):
            et.RawLinear(et.GgmlQuant(codec), rows, columns, vectors, True, et.ActivationMode.INT8)
        return
    rng = np.random.default_rng(rows + columns + vectors)
    weight = synth.random_weight(codec, rows, columns, rng)
    x = synth.random_activations(vectors, columns, rng)
    bias = rng.standard_normal(rows).astype(np.float32)
    act = et.ActivationMode[mode]
    plan = et.linear_requirements(torch.zeros(vectors, columns), torch.zeros((rows, weight.shape[1]), dtype=torch.uint8),
                                  torch.zeros(rows), et.GgmlQuant(codec), (rows, columns), act)
    if rows == 14336:
        assert plan.kernel == "quantize_halves+gemm_h16"  # 128-row tiles fill the device: no K shares
    else:
        assert plan.kernel.endswith("+gemm_i8+reduce" if mode == "INT8" or codec in (oracle.Q8_0, oracle.Q4_0)
                                    else "+gemm_h16+reduce")
    got = run_linear(et, device, codec, rows, columns, x, weight, bias, act)
    again = run_linear(et, device, codec, rows, columns, x, weight, bias, act)
    assert np.array_equal(got, again)  # the same bits on every run
    check_rows = min(rows, 192)
    if mode == "F32":
        want = oracle.linear_rows(codec, rows, columns, x, weight, bias, 0, check_rows)[:, :check_rows]
        close(got[:, :check_rows], want)
    else:
        q, scale, total = oracle.quantize_q8(x)
        want = oracle.linear_q8_rows(codec, rows, columns, q, scale, total, weight, bias, 0, check_rows)[:, :check_rows]
        close(got[:, :check_rows], want)


@pytest.mark.parametrize("codec,vectors,rows,columns", [(oracle.Q4_K, 7, 100, 8192), (oracle.Q4_K, 16, 1000, 4096),
                                                        (oracle.Q4_K, 17, 33, 9216), (oracle.Q5_K, 16, 520, 8448),
                                                        (oracle.Q5_K, 12, 64, 14336), (oracle.Q6_K, 9, 300, 4096),
                                                        (oracle.Q3_K, 16, 130, 2048), (oracle.Q2_K, 8, 14336, 4096),
                                                        (oracle.Q4_K, 13, 28672, 4096)])
def test_linear_up_to_sixteen_vectors_contract_both_planes_in_one_instruction(et, device, codec, vectors, rows, columns):
    # batches of 7 ... 16 vectors: rows 0-15 of the matrix instruction's activation operand are the
    # high plane of the vectors and rows 16-31 their low plane, added once per stage - every K-quant,
    # 64- and 128-row tiles, with and without K shares, rows that end inside a tile (17 vectors: the
    # ordinary tile beside them)
    rng = np.random.default_rng(7 * rows + columns + vectors)
    weight = synth.random_weight(codec, rows, columns, rng)
    x = synth.random_activations(vectors, columns, rng)
    bias = rng.standard_normal(rows).astype(np.float32)
    plan = et.linear_requirements(torch.zeros(vectors, columns), torch.zeros((rows, weight.shape[1]), dtype=torch.uint8),
                                  torch.zeros(rows), et.GgmlQuant(codec), (rows, columns), et.ActivationMode.F32)
    assert plan.kernel.startswith("quantize_halves+gemm_h16")
    got = run_linear(et, device, codec, rows, columns, x, weight, bias, et.ActivationMode.F32)
    again = run_linear(et, device, codec, rows, columns, x, weight, bias, et.ActivationMode.F32)
    assert np.array_equal(got, again)
    begin = max(0, rows - 200)  # the last rows (a ragged tile where there is one) against the oracle
    want = oracle.linear_rows(codec, rows, columns, x, weight, bias, begin, rows)[:, begin:]
    close(got[:, begin:], want)
    start = rows - min(rows, 40)  # and against exact arithmetic
    exact = x.astype(np.float64) @ oracle.decode_rows(codec, weight[start:], columns).astype(np.float64).T + bias[start:]
    close(got[:, start:], exact, oracle_noise=0)


def test_group_launch_of_fewer_than_seventeen_vectors(et, device):
    # two matrices behind one prepared input of 12 vectors (the narrow tile) with 8192 columns: tiles of
    # both members in one launch, the first member ending inside a tile; bias and residual ride on the
    # launch that sums the K shares
    rng = np.random.default_rng(4242)
    columns, vectors, sizes = 8192, 12, (100, 64)
    x_host = synth.random_activations(vectors, columns, rng)
    plans = [et.RawLinear(et.GgmlQuant.Q4_K, rows, columns, vectors, rows == 64) for rows in sizes]
    group = et.LinearGroup(plans)
    assert group.workspace_bytes > 0  # K shares
    prepared = torch.empty(plans[0].prepared_input_bytes, dtype=torch.uint8, device=device)
    plans[0].prepare_input(to_dev(x_host, device), prepared)
    host_weights = [synth.random_weight(oracle.Q4_K, rows, columns, rng) for rows in sizes]
    weights = [to_dev(w, device) for w in host_weights]
    bias_host = rng.standard_normal(64).astype(np.float32)
    residual_host = rng.standard_normal((vectors, 100)).astype(np.float32)
    workspace = torch.empty(group.workspace_bytes, dtype=torch.uint8, device=device)
    ys = [torch.full((vectors, rows), float("nan"), device=device) for rows in sizes]
    group.enqueue_prepared(prepared, weights, ys, workspace, biases=[None, to_dev(bias_host, device)],
                           residuals=[to_dev(residual_host, device), None])
    for index, rows in enumerate(sizes):
        want = oracle.linear_rows(oracle.Q4_K, rows, columns, x_host, host_weights[index],
                                  bias_host if index == 1 else None)
        got = ys[index].cpu().numpy()
        close(got - residual_host if index == 0 else got, want)


@pytest.mark.parametrize("codec", [oracle.Q4_K, oracle.Q8_0, oracle.Q4_0, oracle.Q6_K])
def test_linear_unit_vectors_select_decoded_weights(et, device, codec):
    rng = np.random.default_rng(800 + codec)
    rows, columns = 33, 4096
    weight = synth.random_weight(codec, rows, columns, rng)
    dense = oracle.decode_rows(codec, weight, columns)
    picks = rng.choice(columns, 4, replace=False)
    x = np.zeros((4, columns), np.float32)
    x[np.arange(4), picks] = 1.0
    got = run_linear(et, device, codec, rows, columns, x, weight)
    # factored forms may differ from the decoded value by a rounding or two, never more
    assert np.allclose(got, dense[:, picks].T, rtol=4e-6, atol=1e-6)


def test_linear_strided_and_high_rank_inputs(et, device):
    rng = np.random.default_rng(900)
    rows, columns = 40, 1024
    weight = synth.random_weight(synth.Q4_K, rows, columns, rng)
    w = to_dev(weight, device)
    Q4 = et.GgmlQuant.Q4_K
    # every second row of a [10, K] buffer, at a storage offset that breaks 16-byte alignment
    storage = torch.from_numpy(rng.standard_normal(3 + 10 * columns).astype(np.float32)).to(device)
    view = storage[3:].reshape(10, columns)[::2]
    got = et.quantized_linear(view, w, None, Q4, (rows, columns)).cpu().numpy()
    close(got, oracle.linear_into(oracle.Q4_K, rows, columns, view.cpu().numpy(), weight))
    # transposed (non unit trailing stride) view
    base = torch.from_numpy(rng.standard_normal((columns, 3)).astype(np.float32)).to(device)
    got = et.quantized_linear(base.T, w, None, Q4, (rows, columns)).cpu().numpy()
    close(got, oracle.linear_into(oracle.Q4_K, rows, columns, np.ascontiguousarray(base.T.cpu().numpy()), weight))
    # rank 3, with a strided bias
    x3 = torch.from_numpy(rng.standard_normal((2, 3, columns)).astype(np.float32)).to(device)
    bias2 = torch.from_numpy(rng.standard_normal(2 * rows).astype(np.float32)).to(device)
    got = et.quantized_linear(x3, w, bias2[::2], Q4, (rows, columns)).cpu().numpy()
    assert got.shape == (2, 3, rows)
    want = oracle.linear_into(oracle.Q4_K, rows, columns, x3.cpu().numpy(), weight, bias2[::2].cpu().numpy().copy())
    close(got, want)
    # empty batch: nothing is dispatched
    empty = et.quantized_linear(torch.zeros((0, columns), device=device), w, None, Q4, (rows, columns))
    assert empty.shape == (0, rows)


FULL = [("q8_0_gemv_4096x4096", 1), ("q4_0_gemv_11008x4096", 1), ("q4_0_gemv_11008x4096", 4),
        ("q4_0_gemv_11008x4096", 8), ("q4_k_gemv_14336x4096", 1)]


@pytest.mark.parametrize("name,vectors", FULL)
def test_linear_full_size_configs(et, device, name, vectors):
    cfg = synth.CONFIGS[name]
    rng = np.random.default_rng(cfg["seed"])
    weight = synth.random_weight(cfg["codec"], cfg["rows"], cfg["columns"], rng)
    x = synth.random_activations(vectors, cfg["columns"], rng, cfg["x_scale"])
    got = run_linear(et, device, cfg["codec"], cfg["rows"], cfg["columns"], x, weight)
    want = oracle.linear_into(cfg["codec"], cfg["rows"], cfg["columns"], x, weight)
    close(got, want)
    exact = x.astype(np.float64) @ oracle.decode_rows(cfg["codec"], weight, cfg["columns"]).astype(np.float64).T
    close(got, exact, oracle_noise=0)


@pytest.mark.parametrize("vectors", [16, 64])
def test_linear_full_size_q4k_batched_row_ranges(et, device, vectors):
    cfg = synth.CONFIGS["q4_k_gemv_14336x4096"]
    rng = np.random.default_rng(cfg["seed"] + vectors)
    weight = synth.random_weight(cfg["codec"], cfg["rows"], cfg["columns"], rng)
    x = synth.random_activations(vectors, cfg["columns"], rng)
    got = run_linear(et, device, cfg["codec"], cfg["rows"], cfg["columns"], x, weight)
    for begin in (0, 7000, cfg["rows"] - 96):
        want = oracle.linear_rows(cfg["codec"], cfg["rows"], cfg["columns"], x, weight, None, begin, begin + 96)
        close(got[:, begin:begin + 96], want[:, begin:begin + 96])
    # linearity in the activations, over all rows: y(a) + y(b) ~ y(a + b)
    x2 = synth.random_activations(vectors, cfg["columns"], rng)
    y2 = run_linear(et, device, cfg["codec"], cfg["rows"], cfg["columns"], x2, weight)
    y12 = run_linear(et, device, cfg["codec"], cfg["rows"], cfg["columns"], x + x2, weight)
    close(y12, got.astype(np.float64) + y2, 2e-3)


@pytest.mark.parametrize("vectors", [16, 64])
def test_linear_full_size_q4k_batched_whole_matrix(et, device, vectors):
    # config 2 at M = 16 and 64, every output: against the oracle (the reference's scalar loop: a few seconds of
    # one host core) and, with no allowance, against the f64-exact value of the same contraction
    cfg = synth.CONFIGS["q4_k_gemv_14336x4096"]
    rng = np.random.default_rng(cfg["seed"] + 2000 + vectors)
    weight = synth.random_weight(cfg["codec"], cfg["rows"], cfg["columns"], rng)
    x = synth.random_activations(vectors, cfg["columns"], rng)
    got = run_linear(et, device, cfg["codec"], cfg["rows"], cfg["columns"], x, weight)
    close(got, oracle.linear_into(cfg["codec"], cfg["rows"], cfg["columns"], x, weight))
    exact = x.astype(np.float64) @ oracle.decode_rows(cfg["codec"], weight, cfg["columns"]).astype(np.float64).T
    close(got, exact, oracle_noise=0)


@pytest.mark.parametrize("codec", [oracle.Q4_K, oracle.Q5_K, oracle.Q8_0, oracle.Q4_0, oracle.Q2_K])
@pytest.mark.parametrize("vectors,rows,columns", [(1, 2048, 4096), (2, 2100, 4096), (1, 4099, 1024), (2, 5003, 256),
                                                  (3, 3000, 2048), (1, 30000, 512), (1, 1793, 4096), (1, 8193, 4096),
                                                  (1, 9000, 1024), (1, 12000, 2048), (1, 14336, 4096), (1, 20000, 768)])
def test_gemv_with_weights_copied_through_lds(et, device, codec, vectors, rows, columns):
    if columns % 256 and codec not in (oracle.Q8_0, oracle.Q4_0):
        pytest.skip("the K-quants take whole 256-column blocks")
    # One vector, one slice of columns, 32 or more rows per compute unit whose packed bytes fit LDS, rows of
    # whole 16-byte pieces: the loader waves copy the workgroup's share of W into LDS and the consumer waves
    # fold it as it lands (gemv_limb_dma). Ragged last shares (8193 rows: a last share of one row), shares
    # that end inside a 1 KiB copy, narrow rows, bias. The other shapes - fewer rows, more vectors, rows that
    # are not whole 16-byte pieces (a loader lane copies 16 bytes and must not read past the matrix) - run on
    # another GEMV kernel and must agree just the same.
    share = -(-rows // 256)
    row_bytes = columns // synth.BLOCK_VALUES[codec] * synth.BLOCK_BYTES[codec]
    # eight ranges of whole KiB below the activation stage (13056 bytes) and the control block (1 KiB)
    fits = -(-(-(-share // 8) * row_bytes) // 1024) * 1024 * 8 <= 160 * 1024 - 1024 - 13056
    copied = vectors == 1 and share >= 32 and row_bytes % 16 == 0 and fits
    plan = et.RawLinear(et.GgmlQuant(codec), rows, columns, vectors, bool(rows % 2))
    if copied:
        assert plan.requirements.kernel == "gemv_limb_dma"
    else:
        assert plan.requirements.kernel != "gemv_limb_dma"
    rng = np.random.default_rng(codec * 17 + vectors + rows + columns)
    weight = synth.random_weight(codec, rows, columns, rng)
    x = synth.random_activations(vectors, columns, rng)
    bias = rng.standard_normal(rows).astype(np.float32) if rows % 2 else None
    got = run_linear(et, device, codec, rows, columns, x, weight, bias)
    again = run_linear(et, device, codec, rows, columns, x, weight, bias)
    assert np.array_equal(got, again)  # arrival order of the copies does not reach the sums
    close(got, oracle.linear_into(codec, rows, columns, x, weight, bias))
    exact = x.astype(np.float64) @ oracle.decode_rows(codec, weight, columns).astype(np.float64).T
    if bias is not None:
        exact = exact + bias.astype(np.float64)
    close(got, exact, oracle_noise=0)


@pytest.mark.parametrize("vectors", [16, 64])
def test_linear_full_size_q4k_batched_random_rows(et, device, vectors):
    # the batched Q4_K 14336 x 4096 contraction on 1024 rows drawn at random from the whole matrix
    cfg = synth.CONFIGS["q4_k_gemv_14336x4096"]
    rng = np.random.default_rng(cfg["seed"] + 1000 + vectors)
    weight = synth.random_weight(cfg["codec"], cfg["rows"], cfg["columns"], rng)
    x = synth.random_activations(vectors, cfg["columns"], rng)
    got = run_linear(et, device, cfg["codec"], cfg["rows"], cfg["columns"], x, weight)
    picks = np.sort(rng.choice(cfg["rows"], 1024, replace=False))
    want = oracle.linear_into(cfg["codec"], len(picks), cfg["columns"], x, np.ascontiguousarray(weight[picks]))
    close(got[:, picks], want)


def test_output_head_at_decode_batch(et, device):
    # Q4_K 128256 x 4096 with 32 vectors (the output projection of a batched decode step) on row ranges
    # at the start, in the middle and over the last two row tiles of the matrix
    rows, columns, vectors = 128256, 4096, 32
    rng = np.random.default_rng(128256)
    base = synth.random_weight(oracle.Q4_K, 8192, columns, rng)
    weight = np.concatenate([np.roll(base, r, axis=0) for r in range(-(-rows // 8192))])[:rows]
    x = synth.random_activations(vectors, columns, rng)
    got = run_linear(et, device, oracle.Q4_K, rows, columns, x, weight)
    assert got.shape == (vectors, rows)
    for begin, end in ((0, 160), (70000, 70130), (rows - 256, rows)):
        want = oracle.linear_into(oracle.Q4_K, end - begin, columns, x, np.ascontiguousarray(weight[begin:end]))
        close(got[:, begin:end], want)


# --------------------------------------------------------------------------- int8-activation path

def int8_close_to_f32_reference(got, ref, tol=2e-2):
    """The 2e-2 bar of the int8-activation path against the f32-activation reference.

    int8 rounding noise is proportional to |w|.|x|, not to the individual output,
    and its maximum over N*M outputs grows with their count, so the bar is stated
    per vector: relative L2 error <= tol, and every element within
    tol * max(|ref|, max|ref row|)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    l2 = np.linalg.norm(got - ref, axis=1) / np.maximum(np.linalg.norm(ref, axis=1), 1e-30)
    assert np.all(l2 <= tol), l2.max()
    peak = np.abs(ref).max(axis=1, keepdims=True)
    assert np.all(np.abs(got - ref) <= tol * np.maximum(np.abs(ref), peak))


@pytest.mark.parametrize("vectors,columns", [(1, 32), (5, 4096), (33, 14336), (512, 256)])
def test_activation_quantiser_is_bit_exact(et, device, vectors, columns):
    rng = np.random.default_rng(vectors + columns)
    x = synth.random_activations(vectors, columns, rng, 0.5)
    x[0, :32] = 0.0
    q, scale, total = et.quantize_activations(to_dev(x, device))
    wq, wscale, wtotal = oracle.quantize_q8(x)
    assert np.array_equal(q.cpu().numpy(), wq)
    assert np.array_equal(bits(scale.cpu().numpy().T), bits(wscale))
    assert np.array_equal(total.cpu().numpy().T, wtotal)


@pytest.mark.parametrize("codec", [oracle.Q8_0, oracle.Q4_0, oracle.Q4_K])
@pytest.mark.parametrize("vectors,rows,columns", [(16, 128, 512), (64, 200, 4096), (33, 37, 1024),
                                                  (512, 96, 2048), (1, 5, 256), (97, 129, 768),
                                                  (130, 300, 2304)])
def test_int8_path_matches_its_oracle(et, device, codec, vectors, rows, columns):
    rng = np.random.default_rng(codec * 7 + vectors + rows)
    weight = synth.random_weight(codec, rows, columns, rng)
    x = synth.random_activations(vectors, columns, rng, 0.5)
    bias = rng.standard_normal(rows).astype(np.float32) if rows % 2 else None
    got = run_linear(et, device, codec, rows, columns, x, weight, bias, et.ActivationMode.INT8)
    q, scale, total = oracle.quantize_q8(x)
    want = oracle.linear_q8_rows(codec, rows, columns, q, scale, total, weight, bias)
    close(got, want)
    int8_close_to_f32_reference(got, oracle.linear_into(codec, rows, columns, x, weight, bias))


def test_int8_full_size_prefill_row_ranges(et, device):
    cfg = synth.CONFIGS["q8_0_gemm_i8_512x14336x4096"]
    rng = np.random.default_rng(cfg["seed"])
    weight = synth.random_weight(cfg["codec"], cfg["rows"], cfg["columns"], rng)
    x = synth.random_activations(512, cfg["columns"], rng, cfg["x_scale"])
    got = run_linear(et, device, cfg["codec"], cfg["rows"], cfg["columns"], x, weight, None,
                     et.ActivationMode.INT8)
    q, scale, total = oracle.quantize_q8(x)
    for begin in (0, 2048, cfg["rows"] - 16):
        want = oracle.linear_q8_rows(cfg["codec"], cfg["rows"], cfg["columns"], q, scale, total, weight,
                                     None, begin, begin + 16)
        close(got[:, begin:begin + 16], want[:, begin:begin + 16])


def test_int8_full_size_prefill_whole_matrix(et, device):
    # config 3, every one of the 512 x 4096 outputs against the oracle's int8 path (15 s of one host core)
    cfg = synth.CONFIGS["q8_0_gemm_i8_512x14336x4096"]
    rng = np.random.default_rng(cfg["seed"] + 1)
    weight = synth.random_weight(cfg["codec"], cfg["rows"], cfg["columns"], rng)
    x = synth.random_activations(512, cfg["columns"], rng, cfg["x_scale"])
    got = run_linear(et, device, cfg["codec"], cfg["rows"], cfg["columns"], x, weight, None, et.ActivationMode.INT8)
    q, scale, total = oracle.quantize_q8(x)
    want = oracle.linear_q8_rows(cfg["codec"], cfg["rows"], cfg["columns"], q, scale, total, weight, None, 0, cfg["rows"])
    close(got, want)


def test_int8_full_size_prefill_against_the_f32_reference(et, device, capsys):
    # config 3 (Q8_0 4096 x 14336, 512 vectors, int8 activations) against the f32-ACTIVATION reference
    # on row ranges. Asserted: the per-vector bar (relative L2 <= 2e-2, elements within 2e-2 of the
    # larger of |ref| and the row's peak). Reported, not asserted: the literal elementwise bar
    # |a - b| <= 2e-2 * max(|b|, 1) - int8 rounding noise is proportional to |w|.|x| whatever the
    # output's own size, so outputs that land near zero can miss it.
    cfg = synth.CONFIGS["q8_0_gemm_i8_512x14336x4096"]
    rng = np.random.default_rng(cfg["seed"])
    weight = synth.random_weight(cfg["codec"], cfg["rows"], cfg["columns"], rng)
    x = synth.random_activations(512, cfg["columns"], rng, cfg["x_scale"])
    got = run_linear(et, device, cfg["codec"], cfg["rows"], cfg["columns"], x, weight, None, et.ActivationMode.INT8)
    outside, worst, count = 0, 0.0, 0
    for begin in (0, 1000, 2048, cfg["rows"] - 64):
        ref = oracle.linear_into(cfg["codec"], 64, cfg["columns"], x, np.ascontiguousarray(weight[begin:begin + 64]))
        mine = got[:, begin:begin + 64]
        int8_close_to_f32_reference(mine, ref)
        ratio = np.abs(mine.astype(np.float64) - ref) / (2e-2 * np.maximum(np.abs(ref), 1.0))
        outside += int((ratio > 1.0).sum())
        worst = max(worst, float(ratio.max()))
        count += ratio.size
    with capsys.disabled():
        print(f"\n  literal bar |a-b| <= 2e-2*max(|b|,1): {outside} of {count} outputs outside "
              f"({100.0 * outside / count:.3f} %), worst ratio {worst:.2f}")


def test_gguf_file_to_contraction(et, device, tmp_path):
    # a GGUF file with Q4_K, Q8_0 and F32 tensors: parse, upload, contract - the file's bytes are the weights
    import struct
    from gguf_builder import build, entry
    rng = np.random.default_rng(77)
    rows, columns = 300, 1024
    w4 = synth.random_weight(oracle.Q4_K, rows, columns, rng)
    w8 = synth.random_weight(oracle.Q8_0, 70, 512, rng)
    dense = rng.standard_normal((5, 33)).astype(np.float32)
    big = rng.integers(0, 256, (20 << 20) + 144, dtype=np.uint8)  # more than two staging buffers
    big = big[: big.size // 144 * 144]
    tensors, payloads, cursor = [], {}, 0
    for name, dims, code, data in (("blk.0.ffn_up.weight", (columns, rows), 12, w4.tobytes()),
                                   ("blk.0.attn_q.weight", (512, 70), 8, w8.tobytes()),
                                   ("norm.weight", (33, 5), 0, dense.tobytes()),
                                   ("big.weight", (256, big.size // 144), 12, big.tobytes())):
        cursor = -(-cursor // 32) * 32
        tensors.append(dict(name=name, dimensions=list(dims), format=code, offset=cursor, bytes=len(data)))
        payloads[name] = data
        cursor += len(data)
    data, _ = build([entry("general.quantization_version", "u32", 2), entry("llama.block_count", "u32", 1)],
                    tensors, architecture="llama", payloads=payloads)
    path = tmp_path / "model.gguf"
    path.write_bytes(data)
    with et.GgufFile.open(str(path)) as model:
        assert model.architecture == "llama" and model.get("llama.block_count").value == 1
        up = model.tensor("blk.0.ffn_up.weight")
        assert up.format_name == "Q4_K" and up.logical_shape == (rows, columns) and up.physical_shape == (rows, 576)
        weight = model.upload_tensor("blk.0.ffn_up.weight", device)
        assert np.array_equal(weight.cpu().numpy(), w4)
        x = synth.random_activations(9, columns, rng)
        y = et.quantized_linear(to_dev(x, device), weight, None, et.GgmlQuant(up.format), up.logical_shape)
        close(y.cpu().numpy(), oracle.linear_into(oracle.Q4_K, rows, columns, x, w4, None))
        q = model.upload_tensor("blk.0.attn_q.weight", device)
        x = synth.random_activations(2, 512, rng)
        y = et.quantized_linear(to_dev(x, device), q, None, et.GgmlQuant.Q8_0, (70, 512))
        close(y.cpu().numpy(), oracle.linear_into(oracle.Q8_0, 70, 512, x, w8, None))
        assert np.array_equal(model.upload_tensor("norm.weight", device).cpu().numpy(), dense)
        assert np.array_equal(model.upload_tensor("big.weight", device).cpu().numpy().reshape(-1), big)
        with pytest.raises(et.GgufParseError, match="requires 38080 destination bytes, got 300"):
            model.upload_tensor("blk.0.attn_q.weight", device, torch.empty(300, dtype=torch.uint8, device=device))


@pytest.mark.parametrize("codec", [oracle.Q4_K, oracle.Q6_K])
def test_embedding_at_vocabulary_scale(et, device, codec):
    # a [128256, 4096] table, 8192 ids (repeats, the first and the last row): sampled rows against the
    # oracle bit for bit; every output row equals the first output row of the same id; a table row
    # gathered is that row of the whole-table decode
    rng = np.random.default_rng(1200 + codec)
    rows, columns, base = 128256, 4096, 2048
    block = synth.random_weight(codec, base, columns, rng)
    table = np.concatenate([np.roll(block, r, axis=0) for r in range(-(-rows // base))])[:rows]
    ids = rng.integers(0, rows, 8192).astype(np.int64)
    ids[:4] = [0, rows - 1, 0, rows - 1]
    w, index = to_dev(table, device), torch.from_numpy(ids).to(device)
    plan = et.embedding_requirements(index, w, et.GgmlQuant(codec), (rows, columns))
    out = torch.full(plan.output_shape, float("nan"), dtype=torch.float32, device=device)
    et.embedding_into(index, w, et.GgmlQuant(codec), out, plan)
    got = out.cpu().numpy()
    picks = np.concatenate([np.arange(4), rng.integers(0, ids.size, 60)])
    want = oracle.embedding_into(codec, rows, columns, ids[picks], table)
    assert np.array_equal(bits(got[picks]), bits(want))
    order = np.argsort(ids, kind="stable")
    first_of = order[np.searchsorted(ids[order], ids)]  # first position holding the same id
    assert np.array_equal(bits(got), bits(got[first_of]))
    # ids of rows that repeat `block` decode to the same values as the block's rows
    whole = et.dequantize_rows(to_dev(block, device), et.GgmlQuant(codec), (base, columns)).cpu().numpy()
    source = (ids % base - ids // base) % base  # table row r holds block row (r % base - r // base) mod base
    assert np.array_equal(bits(got), bits(whole[source]))
    bad = index.clone()
    bad[4097] = rows
    with pytest.raises(et.QuantizedError, match=f"outside 0..{rows}"):
        et.embedding_into(bad, w, et.GgmlQuant(codec), out, plan)


@pytest.mark.parametrize("codec", [oracle.Q2_K, oracle.Q3_K, oracle.Q5_K, oracle.Q6_K])
@pytest.mark.parametrize("vectors", [1, 2, 5])
def test_k_quant_gemv_at_full_size(et, device, codec, vectors):
    # the integer-dot GEMV for the other K-quants at 14336 x 4096: a row range against the oracle,
    # and linearity in x over all rows
    rng = np.random.default_rng(900 + codec + vectors)
    rows, columns = 14336, 4096
    weight = synth.random_weight(codec, rows, columns, rng)
    x = synth.random_activations(vectors, columns, rng)
    plan = et.linear_requirements(torch.zeros(vectors, columns), torch.zeros((rows, weight.shape[1]), dtype=torch.uint8),
                                  None, et.GgmlQuant(codec), (rows, columns))
    single = "gemv_limb_dma" if codec == oracle.Q2_K else "gemv_limb"  # one vector of Q2_K: shares of 56 rows that fit LDS
    if vectors > 1 and codec == oracle.Q5_K:
        expected = "gemv_mma"  # 2..8 vectors of Q5_K: the small-batch kernel
    else:  # at most two vectors per launch (Q5_K: one vector here), the name lists the launches of a call
        expected = {1: single, 2: "gemv_limb", 5: "gemv_limb x2+" + single}[vectors]
    assert plan.kernel == expected
    got = run_linear(et, device, codec, rows, columns, x, weight)
    for start in (0, rows - 128):
        want = oracle.linear_rows(codec, rows, columns, x, weight, None, start, start + 128)[:, start:start + 128]
        close(got[:, start:start + 128], want)
    doubled = run_linear(et, device, codec, rows, columns, 2.0 * x, weight)
    assert np.array_equal(doubled, 2.0 * got)  # scaling by two is exact in every step


@pytest.mark.parametrize("mode", ["F32", "INT8"])
def test_shared_prepared_input_and_residual_epilogue(et, device, mode):
    # q / k / v style: one quantisation of the activations feeds plans of different row counts; the
    # residual rides in the epilogue. Every result has the bits of the unfused sequence.
    rng = np.random.default_rng(61)
    columns, vectors = 4096, 32
    act = et.ActivationMode[mode]
    x = to_dev(synth.random_activations(vectors, columns, rng), device)
    plans, prepared = {}, None
    for rows in (4096, 1024, 14336):  # K shares of 4, 16 and none
        plans[rows] = et.RawLinear(et.GgmlQuant.Q4_K, rows, columns, vectors, rows == 1024, act)
    sizes = {p.prepared_input_bytes for p in plans.values()}
    assert len(sizes) == 1 and sizes.pop() > 0
    prepared = torch.empty(plans[4096].prepared_input_bytes, dtype=torch.uint8, device=device)
    plans[1024].prepare_input(x, prepared)  # any of the plans may prepare it
    for rows, plan in plans.items():
        weight = to_dev(synth.random_weight(oracle.Q4_K, rows, columns, rng), device)
        bias = to_dev(rng.standard_normal(rows).astype(np.float32), device) if rows == 1024 else None
        workspace = torch.empty(max(plan.requirements.workspace_bytes, 16), dtype=torch.uint8, device=device)
        plain = torch.empty(vectors, rows, device=device)
        plan.enqueue(x, weight, bias, plain, workspace)
        shared = torch.empty_like(plain)
        plan.enqueue_prepared(prepared, weight, bias, shared, workspace)
        assert torch.equal(plain, shared)
        residual = torch.randn(vectors, rows, device=device)
        fused = torch.empty_like(plain)
        plan.enqueue_prepared(prepared, weight, bias, fused, workspace, residual=residual)
        assert torch.equal(fused, plain + residual)
        stream = residual.clone()  # in place, as a residual stream is updated
        plan.enqueue_prepared(prepared, weight, bias, stream, workspace, residual=stream)
        assert torch.equal(stream, plain + residual)
    small = et.RawLinear(et.GgmlQuant.Q4_K, 64, columns, 2, False, et.ActivationMode.F32)
    assert small.prepared_input_bytes == 0
    with pytest.raises(et.QuantizedError, match="takes the activations as they are"):
        small.prepare_input(x[:2], prepared)


@pytest.mark.parametrize("mode,blob_bytes,limbs", [("INT8", 12288, 1), ("F32", 28672, 3)])
def test_large_inputs_prepare_blob_by_blob_with_the_same_bytes(et, device, mode, blob_bytes, limbs):
    # Inputs of 512 and more blobs (256-column stages x 32-vector tiles) are quantised by a kernel that
    # assembles each blob in LDS; smaller ones by the kernel that stores every dword where it belongs.
    # The same rows prepared 32 at a time (few blobs per call) must give the same bytes, blob by blob -
    # what lies behind the last valid vector of a ragged tile is not compared.
    rng = np.random.default_rng(4242 + limbs)
    columns, vectors = 14336, 500  # 56 stages x 16 tiles = 896 blobs; the last tile holds 20 vectors
    act = et.ActivationMode[mode]
    x = to_dev(synth.random_activations(vectors, columns, rng), device)
    x[3, 512:768] = 0.0  # a stage of zeros: unit 0
    big = et.RawLinear(et.GgmlQuant.Q8_0, 64, columns, vectors, False, act)
    stages, tiles = columns // 256, -(-vectors // 32)
    assert big.prepared_input_bytes == stages * tiles * blob_bytes
    prepared = torch.zeros(big.prepared_input_bytes, dtype=torch.uint8, device=device)
    big.prepare_input(x, prepared)
    whole = prepared.cpu().numpy().reshape(stages, tiles, blob_bytes)
    for tile in range(tiles):
        count = min(32, vectors - 32 * tile)
        small = et.RawLinear(et.GgmlQuant.Q8_0, 64, columns, count, False, act)
        part = torch.zeros(small.prepared_input_bytes, dtype=torch.uint8, device=device)
        small.prepare_input(x[32 * tile:32 * tile + count], part)
        want = part.cpu().numpy().reshape(stages, blob_bytes)
        got = whole[:, tile]
        planes = lambda a: a[:, :limbs * 8192].reshape(stages, limbs, 16, 32, 16)[:, :, :, :count]  # noqa: E731
        assert np.array_equal(planes(got), planes(want)), tile
        tables = lambda a: a[:, limbs * 8192:limbs * 8192 + 2048].reshape(stages, 2, 8, 32, 4)[:, :, :, :count]  # noqa: E731
        assert np.array_equal(tables(got), tables(want)), tile
        pieces = lambda a: a[:, limbs * 8192 + 2048:limbs * 8192 + 4096].reshape(stages, 8, 32, 8)[:, :, :count]  # noqa: E731
        assert np.array_equal(pieces(got), pieces(want)), tile


def test_prepared_input_of_an_operator_on_the_fly(et, device):
    # rms_norm(x) * w and silu(gate) * up applied while the activations are quantised: the prepared
    # bytes, and so every contraction from them, are those of the operator followed by prepare_input
    rng = np.random.default_rng(77)
    vectors = 33
    for columns in (4096, 5632):  # 16 stages: all in registers; 22: the tail loop of the norm
        plan = et.RawLinear(et.GgmlQuant.Q4_K, 64, columns, vectors)
        assert plan.fused_prepare and plan.prepared_input_bytes > 0
        x = to_dev(synth.random_activations(vectors, columns, rng, 3.0), device)
        x[5, 256:512] = 0.0
        weight = to_dev(rng.standard_normal(columns).astype(np.float32), device)
        plain, fused = (torch.zeros(plan.prepared_input_bytes, dtype=torch.uint8, device=device) for _ in range(2))
        for w in (weight, None):
            normed = torch.empty_like(x)
            et.rms_norm_into(x, w, 1e-5, normed)
            plan.prepare_input(normed, plain)
            plan.prepare_input_rms_norm(x, w, 1e-5, fused)
            assert torch.equal(plain, fused)
            if w is not None:  # a weight held as half floats is widened on use: the bytes of its f32 copy
                half = w.to(torch.float16)
                plan.prepare_input_rms_norm(x, half.float(), 1e-5, plain)
                plan.prepare_input_rms_norm(x, half, 1e-5, fused)
                assert torch.equal(plain, fused)
        gate, up = x * 2.0, to_dev(synth.random_activations(vectors, columns, rng), device)
        product = torch.empty_like(gate)
        et.silu_mul_into(gate, up, product)
        plan.prepare_input(product, plain)
        plan.prepare_input_silu_mul(gate, up, fused)
        assert torch.equal(plain, fused)
    # plans without such a quantiser say so
    small = et.RawLinear(et.GgmlQuant.Q4_K, 64, 4096, 2)
    int8 = et.RawLinear(et.GgmlQuant.Q4_K, 64, 4096, vectors, False, et.ActivationMode.INT8)
    assert not small.fused_prepare and not int8.fused_prepare
    buffer = torch.zeros(max(int8.prepared_input_bytes, 16), dtype=torch.uint8, device=device)
    with pytest.raises(et.QuantizedError, match="on the fly"):
        int8.prepare_input_rms_norm(x[:, :4096].contiguous(), None, 1e-5, buffer)


def test_group_launch_of_contractions_sharing_their_input(et, device):
    # q / k / v style: three matrices, one prepared input, one launch over the row tiles of all
    rng = np.random.default_rng(88)
    columns, vectors = 4096, 32
    x_host = synth.random_activations(vectors, columns, rng)
    x = to_dev(x_host, device)
    sizes = (4096, 1024, 1000)  # the last one ends in a ragged tile
    plans = [et.RawLinear(et.GgmlQuant.Q4_K, rows, columns, vectors, rows == 1024) for rows in sizes]
    group = et.LinearGroup(plans)
    assert group.workspace_bytes >= 2 * vectors * sum(-(-rows // 64) * 64 for rows in sizes) * 4  # two K shares
    prepared = torch.empty(plans[0].prepared_input_bytes, dtype=torch.uint8, device=device)
    plans[0].prepare_input(x, prepared)
    host_weights = [synth.random_weight(oracle.Q4_K, rows, columns, rng) for rows in sizes]
    weights = [to_dev(w, device) for w in host_weights]
    bias_host = rng.standard_normal(1024).astype(np.float32)
    biases = [None, to_dev(bias_host, device), None]
    residual = to_dev(rng.standard_normal((vectors, 4096)).astype(np.float32), device)
    workspace = torch.empty(group.workspace_bytes, dtype=torch.uint8, device=device)
    runs = []
    for _ in range(2):
        ys = [torch.full((vectors, rows), float("nan"), device=device) for rows in sizes]
        group.enqueue_prepared(prepared, weights, ys, workspace, biases=biases, residuals=[residual, None, None])
        runs.append([y.cpu().numpy() for y in ys])
    for first, second in zip(*runs):
        assert np.array_equal(first, second)  # the same bits on every run
    for index, rows in enumerate(sizes):
        want = oracle.linear_rows(oracle.Q4_K, rows, columns, x_host, host_weights[index],
                                  bias_host if index == 1 else None, 0, min(rows, 192))[:, :min(rows, 192)]
        got = runs[0][index][:, :min(rows, 192)]
        if index == 0:
            got = got - residual.cpu().numpy()[:, :192]
        close(got, want)
        # all rows against the member's own launch (another order of the K shares: not the same bits)
        alone = torch.empty((vectors, rows), device=device)
        single_ws = torch.empty(max(plans[index].requirements.workspace_bytes, 16), dtype=torch.uint8, device=device)
        plans[index].enqueue_prepared(prepared, weights[index], biases[index], alone, single_ws,
                                      residual=residual if index == 0 else None)
        close(runs[0][index], alone.cpu().numpy())
    # two large members (gate / up): enough 128-row tiles for every compute unit, no K shares
    big = [et.RawLinear(et.GgmlQuant.Q4_K, 14336, columns, vectors) for _ in range(2)]
    pair = et.LinearGroup(big)
    assert pair.workspace_bytes == 0
    big_host = [synth.random_weight(oracle.Q4_K, 14336, columns, rng) for _ in range(2)]
    big_weights = [to_dev(w, device) for w in big_host]
    together = [torch.empty((vectors, 14336), device=device) for _ in range(2)]
    pair.enqueue_prepared(prepared, big_weights, together)
    again = [torch.empty((vectors, 14336), device=device) for _ in range(2)]
    pair.enqueue_prepared(prepared, big_weights, again)
    for index in range(2):
        assert torch.equal(together[index], again[index])
        alone = torch.empty((vectors, 14336), device=device)
        big_ws = torch.empty(max(big[index].requirements.workspace_bytes, 16), dtype=torch.uint8, device=device)
        big[index].enqueue_prepared(prepared, big_weights[index], None, alone, big_ws)
        close(together[index].cpu().numpy(), alone.cpu().numpy())
        for start in (0, 14336 - 128):
            want = oracle.linear_rows(oracle.Q4_K, 14336, columns, x_host, big_host[index], None, start, start + 128)
            close(together[index].cpu().numpy()[:, start:start + 128], want[:, start:start + 128])
    # members must share the prepared input, and run on the kernel that has the group launch
    with pytest.raises(et.QuantizedError, match="share columns and vectors"):
        et.LinearGroup([plans[0], et.RawLinear(et.GgmlQuant.Q4_K, 64, 512, vectors)])
    with pytest.raises(et.QuantizedError, match="no group launch"):
        et.LinearGroup([et.RawLinear(et.GgmlQuant.Q4_K, 64, columns, 2)])


def test_contraction_then_norm_prepared_input_in_the_reduction_launch(et, device):
    # y = W x + residual, then the next block's norm inside the quantiser: where the contraction shares
    # K over workgroups the launch that sums the shares also writes y, norms and quantises - the same
    # bytes as the two calls, for y and for the prepared input
    rng = np.random.default_rng(91)
    vectors = 33
    # (rows, columns, bias, K shares?) - 14336 rows fill the device without shares: the two steps in turn
    for rows, columns, with_bias, shares in ((4096, 4096, False, True), (4096, 14336, True, True),
                                            (2560, 1024, False, True), (14336, 4096, False, False)):
        plan = et.RawLinear(et.GgmlQuant.Q4_K, rows, columns, vectors, with_bias)
        following = et.RawLinear(et.GgmlQuant.Q4_K, 64, rows, vectors)
        assert ("reduce" in plan.requirements.kernel) == shares
        weight = to_dev(synth.random_weight(oracle.Q4_K, rows, columns, rng), device)
        x = to_dev(synth.random_activations(vectors, columns, rng), device)
        bias = to_dev(rng.standard_normal(rows).astype(np.float32), device) if with_bias else None
        norm_weight = to_dev(rng.standard_normal(rows).astype(np.float32), device)
        stream_in = to_dev(rng.standard_normal((vectors, rows)).astype(np.float32), device)
        prepared = torch.empty(plan.prepared_input_bytes, dtype=torch.uint8, device=device)
        plan.prepare_input(x, prepared)
        workspace = torch.empty(max(plan.requirements.workspace_bytes, 16), dtype=torch.uint8, device=device)
        for w in (norm_weight, None, norm_weight.to(torch.float16)):  # the last: half floats, widened on use
            # in place, as a residual stream is updated
            y_two, y_one = stream_in.clone(), stream_in.clone()
            next_two, next_one = (torch.zeros(following.prepared_input_bytes, dtype=torch.uint8, device=device)
                                  for _ in range(2))
            plan.enqueue_prepared(prepared, weight, bias, y_two, workspace, residual=y_two)
            following.prepare_input_rms_norm(y_two, w, 1e-5, next_two)
            plan.enqueue_prepared_then_norm(prepared, weight, bias, y_one, workspace, following, w, 1e-5, next_one,
                                            residual=y_one)
            assert torch.equal(y_two, y_one)
            assert torch.equal(next_two, next_one)
        # without a residual, into a fresh y
        y_two, y_one = torch.empty((vectors, rows), device=device), torch.full((vectors, rows), float("nan"), device=device)
        plan.enqueue_prepared(prepared, weight, bias, y_two, workspace)
        following.prepare_input_rms_norm(y_two, norm_weight, 1e-5, next_two)
        plan.enqueue_prepared_then_norm(prepared, weight, bias, y_one, workspace, following, norm_weight, 1e-5, next_one)
        assert torch.equal(y_two, y_one) and torch.equal(next_two, next_one)
    # the next contraction must take this one's result, and be able to prepare from an operator
    plan = et.RawLinear(et.GgmlQuant.Q4_K, 4096, 4096, vectors)
    with pytest.raises(et.QuantizedError, match="must take this one's result"):
        plan.enqueue_prepared_then_norm(prepared, weight, None, y_one, workspace, et.RawLinear(et.GgmlQuant.Q4_K, 64, 512, vectors),
                                        None, 1e-5, next_one)


def test_group_launch_then_rotary_in_the_reduction_launch(et, device):
    # q / k / v of a decode step: the launch that sums the group's K shares also rotates q and k at the
    # slots' cursors - the bytes of the group launch followed by the rotary launch
    rng = np.random.default_rng(92)
    vectors, columns, head_dim = 32, 4096, 128
    sizes = (4096, 1024, 1024)
    plans = [et.RawLinear(et.GgmlQuant.Q4_K, rows, columns, vectors) for rows in sizes]
    group = et.LinearGroup(plans)
    assert group.workspace_bytes > 0  # K shares
    weights = [to_dev(synth.random_weight(oracle.Q4_K, rows, columns, rng), device) for rows in sizes]
    x = to_dev(synth.random_activations(vectors, columns, rng), device)
    prepared = torch.empty(plans[0].prepared_input_bytes, dtype=torch.uint8, device=device)
    plans[0].prepare_input(x, prepared)
    workspace = torch.empty(group.workspace_bytes, dtype=torch.uint8, device=device)
    cursors = to_dev(rng.integers(0, 4000, vectors).astype(np.uint32), device)
    for layout in (et.RotaryLayout.HALF_SPLIT, et.RotaryLayout.INTERLEAVED_PAIRS):
        for offsets in (cursors, cursors[:1].contiguous()):
            two = [torch.empty((vectors, rows), device=device) for rows in sizes]
            one = [torch.full((vectors, rows), float("nan"), device=device) for rows in sizes]
            group.enqueue_prepared(prepared, weights, two, workspace)
            q4, k4 = two[0].view(vectors, 32, 1, head_dim), two[1].view(vectors, 8, 1, head_dim)
            et.rotary_pair_into(q4, k4, offsets, 500000.0, 1.0, layout, q4, k4)
            group.enqueue_prepared_then_rotary(prepared, weights, one, workspace, (0, 1), offsets, 500000.0, 1.0, layout,
                                               head_dim)
            for a, b in zip(two, one):
                assert torch.equal(a, b)
    # a group without K shares runs the two steps in turn: the same bytes
    big = [et.RawLinear(et.GgmlQuant.Q4_K, 14336, columns, vectors) for _ in range(2)]
    pair = et.LinearGroup(big)
    assert pair.workspace_bytes == 0
    big_weights = [to_dev(synth.random_weight(oracle.Q4_K, 14336, columns, rng), device) for _ in range(2)]
    two = [torch.empty((vectors, 14336), device=device) for _ in range(2)]
    one = [torch.empty((vectors, 14336), device=device) for _ in range(2)]
    pair.enqueue_prepared(prepared, big_weights, two)
    first = two[0].view(vectors, 112, 1, head_dim)
    et.rotary_into(first, cursors, 10000.0, -1.0, et.RotaryLayout.HALF_SPLIT, first)
    pair.enqueue_prepared_then_rotary(prepared, big_weights, one, None, (0,), cursors, 10000.0, -1.0,
                                      et.RotaryLayout.HALF_SPLIT, head_dim)
    assert torch.equal(two[0], one[0]) and torch.equal(two[1], one[1])
    three = [torch.empty((vectors, plan.rows), device=device) for plan in group.plans]
    with pytest.raises(et.QuantizedError, match="not whole heads"):
        group.enqueue_prepared_then_rotary(prepared, weights, three, workspace, (0,), cursors, 500000.0, 1.0,
                                           et.RotaryLayout.HALF_SPLIT, 96)
    with pytest.raises(et.QuantizedError, match="offsets for batch"):
        group.enqueue_prepared_then_rotary(prepared, weights, three, workspace, (0,), cursors[:5].contiguous(), 500000.0, 1.0,
                                           et.RotaryLayout.HALF_SPLIT, head_dim)
    with pytest.raises(et.QuantizedError, match="a group of 3 plans takes 3 weights and results"):
        group.enqueue_prepared(prepared, weights, one, workspace)


# --------------------------------------------------------------------------- measurement aids

@pytest.mark.parametrize("kind,per_round,elements", [("i8", 32.0, 64), ("i8_scaled", 16.0, 64), ("i8_scaled_bf16", 16.0, 64), ("f16", 16.0, 64),
                                                      ("f16_16x16", 32.0, 16)])
def test_matrix_core_calibration_loops_sum_what_they_should(et, device, kind, per_round, elements):
    """All operands are ones, so every accumulator element ends at a known integer: K ones per round
    (times the scale product 0.5 for the scaled kind); a thread reports the sum of its elements."""
    rounds, workgroups = 37, 3
    sink = torch.full((256 * workgroups,), float("nan"), device=device)
    et.calibration_mfma(kind, rounds, sink)
    assert torch.all(sink == per_round * rounds * elements), (float(sink[0]), per_round * rounds * elements)
    with pytest.raises(et.QuantizedError, match="calibration_mfma"):
        et.calibration_mfma(kind, 0, sink)


@pytest.mark.parametrize("vectors", [12, 32])
def test_contraction_probe_runs_the_operator_paths_kernel(et, device, vectors):
    """The measurement aid that takes the batched Q4_K kernel apart launches, as `whole`, the kernel of
    the operator path (the same bits); the partial kernels run to completion; other shapes are refused."""
    rng = np.random.default_rng(515 + vectors)
    rows, columns = 14336, 1024
    weight = to_dev(synth.random_weight(oracle.Q4_K, rows, columns, rng), device)
    x = to_dev(synth.random_activations(vectors, columns, rng), device)
    plan = et.RawLinear(et.GgmlQuant.Q4_K, rows, columns, vectors)
    assert plan.requirements.kernel == "quantize_halves+gemm_h16"  # 64-row tiles, no K shares
    prepared = torch.empty(plan.prepared_input_bytes, dtype=torch.uint8, device=device)
    plan.prepare_input(x, prepared)
    want = torch.empty((vectors, rows), device=device)
    plan.enqueue_prepared(prepared, weight, None, want, torch.empty(16, dtype=torch.uint8, device=device))
    got = torch.full_like(want, float("nan"))
    et.calibration_contraction("whole", plan, weight, prepared, got)
    assert torch.equal(got, want)
    for probe in ("no_arithmetic", "no_copies", "no_weight_copies", "no_activation_copies", "weight_copies_only",
                  "activation_copies_only"):
        et.calibration_contraction(probe, plan, weight, prepared, got)
    torch.cuda.synchronize()
    shared = et.RawLinear(et.GgmlQuant.Q4_K, 4096, columns, vectors)  # K shared over workgroups
    with pytest.raises(et.QuantizedError, match="64-row tiles without K shares"):
        et.calibration_contraction("whole", shared, weight, prepared, got)
