"""Pins the CPU oracle before anything is compared with it (no GPU needed).

Sources of truth used here, none of which is the oracle's own formula retyped:
  * the reference's test fixtures and known answers (tests/ref_fixtures.py and
    the KATs of crates/runtime-cpu/src/quantized.rs:827-1000),
  * numpy's float16 -> float32 widening for all 65536 codes,
  * packers written from the documented block layouts (tests/packers.py) with
    closed forms evaluated in numpy float32,
  * structural identities: x = e_k selects one decoded weight, x = ones gives the
    sequential row sum, a strided view equals its dense copy, an int64
    brute-force dot for the int8 path.
"""
import numpy as np
import pytest

import oracle
import packers
import ref_fixtures as rf

K_QUANTS = oracle.K_QUANTS
ALL = oracle.ALL_CODECS


def test_codec_tables_match_reference_row_bytes():
    # crates/runtime/src/gguf.rs:1117-1181: [2,84] [2,110] [2,288 (K=512)] [2,176] [2,210]
    assert oracle.encoded_row_bytes(oracle.Q2_K, 256) == 84
    assert oracle.encoded_row_bytes(oracle.Q3_K, 256) == 110
    assert oracle.encoded_row_bytes(oracle.Q4_K, 512) == 288
    assert oracle.encoded_row_bytes(oracle.Q5_K, 256) == 176
    assert oracle.encoded_row_bytes(oracle.Q6_K, 256) == 210
    assert oracle.encoded_row_bytes(oracle.Q4_K, 255) is None
    assert oracle.encoded_row_bytes(oracle.Q4_K, 4096) == 2304
    assert oracle.encoded_row_bytes(oracle.Q4_K, 14336) == 8064
    assert [oracle.codec_name(c) for c in K_QUANTS] == ["Q2_K", "Q3_K", "Q4_K", "Q5_K", "Q6_K"]
    # legacy ggml blocks (not in the reference)
    assert oracle.encoded_row_bytes(oracle.Q8_0, 4096) == 128 * 34
    assert oracle.encoded_row_bytes(oracle.Q4_0, 4096) == 128 * 18
    assert oracle.encoded_row_bytes(oracle.Q8_0, 48) is None


def test_fp16_widening_all_codes_against_numpy():
    codes = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = codes.view(np.float16).astype(np.float32).view(np.uint32)
    got = np.array([oracle.fp16_to_f32_bits(int(c)) for c in codes], dtype=np.uint32)
    exp = (codes >> 10) & 0x1F
    man = codes & 0x3FF
    nan = (exp == 0x1F) & (man != 0)
    assert np.array_equal(got[~nan], want[~nan])
    # NaNs: quiet bit set, payload shifted by 13 (half 2.7.1 / IEEE convertFormat)
    assert np.all((got[nan] & 0x7FC00000) == 0x7FC00000)
    assert np.array_equal(got[nan] & 0x003FE000, (man[nan].astype(np.uint32) << 13) & 0x003FE000)
    # the fixture constants of crates/runtime-cpu/src/quantized.rs:641-644
    assert oracle.fp16_to_f32_bits(0x3C00) == np.float32(1.0).view(np.uint32)
    assert oracle.fp16_to_f32_bits(0x3800) == np.float32(0.5).view(np.uint32)


def test_scale_min_k4_inverts_the_packer_for_every_pair_and_position():
    for position in range(8):
        for scale in range(64):
            sc = [(7 * i + 3) % 64 for i in range(8)]
            mn = [(11 * i + 5) % 64 for i in range(8)]
            for minimum in (0, 1, 31, 32, 47, 63, (scale * 5 + 1) % 64):
                sc[position], mn[position] = scale, minimum
                packed = packers.pack_scales_k4(sc, mn).tobytes()
                for j in range(8):
                    assert oracle.scale_min_k4(j, packed) == (sc[j], mn[j])
    rng = np.random.default_rng(5)
    for _ in range(2000):
        sc, mn = rng.integers(0, 64, 8), rng.integers(0, 64, 8)
        packed = packers.pack_scales_k4(sc, mn).tobytes()
        assert [oracle.scale_min_k4(j, packed) for j in range(8)] == list(zip(sc.tolist(), mn.tolist()))


@pytest.mark.parametrize("codec", K_QUANTS)
def test_reference_fixtures_decode_exactly(codec):
    # canonical_k_quant_fixtures_decode_exactly, quantized.rs:804-811
    got = oracle.decode_block(codec, rf.FIXTURES[codec]["bytes"].tobytes())
    assert np.array_equal(got.view(np.uint32), rf.expected_values(codec).view(np.uint32))


@pytest.mark.parametrize("codec", K_QUANTS)
def test_decoder_rejects_noncanonical_block_lengths(codec):
    # quantized.rs:813-825
    with pytest.raises(oracle.OracleError, match="expected"):
        oracle.decode_block(codec, rf.FIXTURES[codec]["bytes"].tobytes()[:-1])


@pytest.mark.parametrize("codec", ALL)
def test_pack_then_decode_matches_closed_form(codec):
    rng = np.random.default_rng(100 + codec)
    for _ in range(300):
        block, want = packers.random_block(codec, rng)
        got = oracle.decode_block(codec, block.tobytes())
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_linear_kat_prefill():
    # linear_decodes_blocks_during_prefill, quantized.rs:827-865
    x = np.zeros(1024, np.float32)
    x[:576] = 1.0
    weight = np.tile(rf.FIXTURES[rf.Q4_K]["bytes"], 4).reshape(2, 288)
    bias = np.array([0.5, -0.5], np.float32)
    y = oracle.linear_into(oracle.Q4_K, 2, 512, x.reshape(2, 512), weight, bias)
    assert y.tolist() == [[4096.5, 4095.5], [512.5, 511.5]]


def test_linear_kat_executable_level():
    # crates/runtime-cpu/src/executable.rs:4881-4918: ones [1,256] x 3 fixture rows -> 2048 each
    weight = np.tile(rf.FIXTURES[rf.Q4_K]["bytes"], 3).reshape(3, 144)
    y = oracle.linear_into(oracle.Q4_K, 3, 256, np.ones((1, 256), np.float32), weight)
    assert y.tolist() == [[2048.0, 2048.0, 2048.0]]


@pytest.mark.parametrize("codec", K_QUANTS)
@pytest.mark.parametrize("vectors", [1, 3, 4, 5, 16, 17])
def test_linear_cross_backend_protocol(codec, vectors):
    # The reference's own second-backend protocol
    # (crates/runtime-metal/src/executable.rs:8458-8505): fixture rows cycled,
    # inputs ((i*7 + (i/columns)*3) % 17) * 0.125 - 1, expected = sequential fold.
    columns = 512
    decoded = np.tile(rf.expected_values(codec), 2)
    i = np.arange(vectors * columns)
    x = (((i * 7 + i // columns * 3) % 17).astype(np.float32) * np.float32(0.125) - np.float32(1.0))
    x = x.astype(np.float32).reshape(vectors, columns)
    weight = np.tile(rf.FIXTURES[codec]["bytes"], 4).reshape(2, -1)
    bias = np.array([0.25, -0.5], np.float32) if vectors == 1 else None
    got = oracle.linear_into(codec, 2, columns, x, weight, bias)
    for v in range(vectors):
        dot = np.float32(0)
        for k in range(columns):
            dot = np.float32(dot + np.float32(x[v, k] * decoded[k]))
        want = [dot + np.float32(0.25), dot - np.float32(0.5)] if vectors == 1 else [dot, dot]
        assert got[v].tolist() == [float(w) for w in want]


@pytest.mark.parametrize("codec", ALL)
def test_linear_unit_vectors_select_single_weights(codec):
    rng = np.random.default_rng(7 + codec)
    values = oracle.block_values(codec)
    columns, rows = 2 * max(values, 256), 3
    blocks = [packers.random_block(codec, rng, d_bits=0x2E66, dmin_bits=0x211F)
              for _ in range(rows * columns // values)]
    weight = np.concatenate([b for b, _ in blocks]).reshape(rows, -1)
    dense = np.concatenate([v for _, v in blocks]).reshape(rows, columns)
    picks = rng.choice(columns, 16, replace=False)
    x = np.zeros((16, columns), np.float32)
    x[np.arange(16), picks] = 1.0
    y = oracle.linear_into(codec, rows, columns, x, weight)
    # 0 + 1*w plus exact zeros: bit-exact selection (up to the sign of zero)
    assert np.array_equal(y, dense[:, picks].T)
    # x = ones: the sequential left-to-right f32 row sum
    y1 = oracle.linear_into(codec, rows, columns, np.ones((1, columns), np.float32), weight)
    for r in range(rows):
        acc = np.float32(0)
        for k in range(columns):
            acc = np.float32(acc + dense[r, k])
        assert y1[0, r] == acc


def test_linear_strided_views_equal_dense_copies():
    rng = np.random.default_rng(11)
    columns, rows = 512, 4
    weight = rng.integers(0, 256, (rows, 288), dtype=np.uint8)
    weight[:, 0:4] = [0x66, 0x2E, 0x1F, 0x21]
    weight[:, 144:148] = [0x66, 0x2E, 0x1F, 0x21]
    storage = rng.standard_normal(3 + 5 * 2 * columns).astype(np.float32)
    # view [5, 512] taking every second row of a [10, 512] buffer at offset 3
    view = storage[3:].reshape(10, columns)[::2]
    want = oracle.linear_into(oracle.Q4_K, rows, columns, np.ascontiguousarray(view), weight)
    got = oracle.linear_into(oracle.Q4_K, rows, columns, storage, weight, x_shape=(5, columns),
                             x_strides=(2 * columns, 1), x_offset=3)
    assert np.array_equal(got, want)
    # transposed view [512 rows of storage] -> logical [4, 512] with strides (1, 4)
    storage2 = rng.standard_normal(columns * 4).astype(np.float32)
    view2 = storage2.reshape(columns, 4).T
    want2 = oracle.linear_into(oracle.Q4_K, rows, columns, np.ascontiguousarray(view2), weight)
    got2 = oracle.linear_into(oracle.Q4_K, rows, columns, storage2, weight, x_shape=(4, columns),
                              x_strides=(1, 4))
    assert np.array_equal(got2, want2)
    # rank-3 input [2, 3, 512]
    x3 = rng.standard_normal((2, 3, columns)).astype(np.float32)
    y3 = oracle.linear_into(oracle.Q4_K, rows, columns, x3, weight)
    assert y3.shape == (2, 3, rows)
    assert np.array_equal(y3.reshape(6, rows),
                          oracle.linear_into(oracle.Q4_K, rows, columns, x3.reshape(6, columns), weight))


def test_linear_rows_subset_equals_full():
    rng = np.random.default_rng(12)
    weight = rng.integers(0, 256, (8, 288), dtype=np.uint8)
    weight[:, 0:4] = weight[:, 144:148] = [0x66, 0x2E, 0x1F, 0x21]
    x = rng.standard_normal((3, 512)).astype(np.float32)
    bias = rng.standard_normal(8).astype(np.float32)
    full = oracle.linear_into(oracle.Q4_K, 8, 512, x, weight, bias)
    part = oracle.linear_rows(oracle.Q4_K, 8, 512, x, weight, bias, 2, 6)
    assert np.array_equal(part[:, 2:6], full[:, 2:6])
    assert not part[:, :2].any() and not part[:, 6:].any()


def test_linear_validation_messages():
    # malformed_packed_rows_and_layouts_are_rejected, quantized.rs:923-978
    x = np.zeros((1, 256), np.float32)
    with pytest.raises(oracle.OracleError, match="exact contiguous"):
        oracle.linear_into(oracle.Q4_K, 1, 256, x, np.zeros(143, np.uint8))
    with pytest.raises(oracle.OracleError, match="logical row width"):
        oracle.linear_into(oracle.Q4_K, 1, 255, np.zeros((1, 255), np.float32), np.zeros(0, np.uint8))
    with pytest.raises(oracle.OracleError, match="byte size overflow"):
        oracle.linear_into(oracle.Q4_K, 2**64 - 1, 256, x, np.zeros(144, np.uint8))


@pytest.mark.parametrize("index_dtype", [np.uint32, np.int64])
def test_embedding_kat_selected_rows(index_dtype):
    # embedding_decodes_only_selected_rows_for_both_index_types, quantized.rs:867-897
    table = np.zeros((3, 176), np.uint8)
    table[1] = rf.FIXTURES[rf.Q5_K]["bytes"]
    out = oracle.embedding_into(oracle.Q5_K, 3, 256, np.array([1, 1], index_dtype), table)
    want = rf.expected_values(rf.Q5_K)
    assert out.shape == (2, 256)
    assert np.array_equal(out[0], want) and np.array_equal(out[1], want)


@pytest.mark.parametrize("index", [-1, 1])
def test_embedding_rejects_negative_and_out_of_range(index):
    # quantized.rs:899-921
    table = rf.FIXTURES[rf.Q2_K]["bytes"].reshape(1, 84)
    with pytest.raises(oracle.OracleError, match="outside 0..1"):
        oracle.embedding_into(oracle.Q2_K, 1, 256, np.array([index], np.int64), table)


def test_embedding_strided_indexes_and_shapes():
    rng = np.random.default_rng(3)
    table = rng.integers(0, 256, (6, 210), dtype=np.uint8)
    table[:, 208:210] = [0x66, 0x2E]
    storage = np.array([5, 9, 0, 9, 3, 9, 1, 9], np.uint32)
    got = oracle.embedding_into(oracle.Q6_K, 6, 256, storage, table, index_shape=(2, 2),
                                index_strides=(4, 2))
    want = oracle.embedding_into(oracle.Q6_K, 6, 256, np.array([[5, 0], [3, 1]], np.uint32), table)
    assert got.shape == (2, 2, 256) and np.array_equal(got, want)


def test_cancellation_is_observed():
    # quantized_execution_observes_cancellation, quantized.rs:980-1000
    table = rf.FIXTURES[rf.Q6_K]["bytes"].reshape(1, 210)
    with pytest.raises(oracle.OracleError) as info:
        oracle.embedding_into(oracle.Q6_K, 1, 256, np.array([0], np.uint32), table, cancel=True)
    assert str(info.value) == "operation aborted"
    with pytest.raises(oracle.OracleError) as info:
        oracle.linear_into(oracle.Q6_K, 1, 256, np.zeros((1, 256), np.float32), table, cancel=True)
    assert str(info.value) == "operation aborted"


# ---- int8-activation path: builder-defined semantics, pinned by brute force ----

def test_quantize_q8_properties_and_brute_force():
    rng = np.random.default_rng(21)
    x = rng.standard_normal((3, 96)).astype(np.float32) * np.float32(3)
    x[0, :32] = 0  # an all-zero block
    x[1, 40] = 1e-30
    q, scale, total = oracle.quantize_q8(x)
    blocks = x.reshape(3, 3, 32)
    amax = np.abs(blocks).max(axis=2)
    assert np.array_equal(scale, (amax / np.float32(127)).astype(np.float32))
    assert not q[0, :32].any() and scale[0, 0] == 0
    assert np.array_equal(total, q.reshape(3, 3, 32).sum(axis=2, dtype=np.int32))
    assert np.abs(q.astype(np.int32)).max() <= 127
    # every block with a non-zero value reaches +-127 at its absmax element
    for v in range(3):
        for b in range(3):
            if amax[v, b] > 0:
                assert np.abs(q[v, 32 * b:32 * b + 32].astype(np.int32)).max() == 127
    with np.errstate(divide="ignore", invalid="ignore"):
        inv = np.where(amax > 0, np.float32(127) / amax, np.float32(0)).astype(np.float32)
    want = np.clip(np.rint((blocks * inv[:, :, None]).astype(np.float32)), -127, 127).astype(np.int8)
    assert np.array_equal(q.reshape(3, 3, 32), want)
    # dequantised activations are within half a step of the originals
    deq = q.reshape(3, 3, 32).astype(np.float32) * scale[:, :, None]
    assert np.all(np.abs(deq - blocks) <= scale[:, :, None] * 0.5 * (1 + 1e-6) + 1e-37)


@pytest.mark.parametrize("codec", [oracle.Q8_0, oracle.Q4_0, oracle.Q4_K])
def test_linear_q8_against_integer_brute_force_and_f32_reference(codec):
    rng = np.random.default_rng(30 + codec)
    rows, columns, vectors = 5, 512, 3
    values = oracle.block_values(codec)
    blocks = [packers.random_block(codec, rng, d_bits=0x2E66, dmin_bits=0x211F)
              for _ in range(rows * columns // values)]
    weight = np.concatenate([b for b, _ in blocks]).reshape(rows, -1)
    dense = np.concatenate([v for _, v in blocks]).reshape(rows, columns).astype(np.float64)
    x = rng.standard_normal((vectors, columns)).astype(np.float32)
    q, scale, total = oracle.quantize_q8(x)
    got = oracle.linear_q8_rows(codec, rows, columns, q, scale, total, weight)
    # exact value of the int8 model: dequantised activations times decoded weights, in f64
    xq = (q.reshape(vectors, -1, 32).astype(np.float64) * scale[:, :, None].astype(np.float64))
    model = xq.reshape(vectors, columns) @ dense.T
    assert np.allclose(got, model, rtol=0, atol=2e-4 * np.abs(dense).max() * np.sqrt(columns))
    # and it stays within 2e-2 of the f32-activation reference: per vector, in
    # relative L2 and elementwise against the vector's peak output (int8 rounding
    # noise scales with |w|.|x|, not with the possibly tiny individual output)
    ref = oracle.linear_into(codec, rows, columns, x, weight).astype(np.float64)
    l2 = np.linalg.norm(got - ref, axis=1) / np.linalg.norm(ref, axis=1)
    assert np.all(l2 <= 2e-2)
    peak = np.abs(ref).max(axis=1, keepdims=True)
    assert np.all(np.abs(got - ref) <= 2e-2 * np.maximum(np.abs(ref), peak))
