"""Pins of the decode-neighbour operators of the oracle (CPU only; list in oracle/et_oracle_ops.h)."""
import numpy as np
import pytest

import oracle


def test_rms_norm_reference_vectors_and_closed_forms():
    # packages/core/test/Tensor.test.ts:462-481
    values = np.array([-2, -1, 0, 1, 1, 2, 3, 4, 4, 3, 2, 1, -1, -2, -3, -4], np.float32).reshape(2, 2, 4)
    weight = np.array([0.5, 1, 1.5, 2], np.float32)
    eps = 1e-5
    x64 = values.astype(np.float64)
    scale = 1.0 / np.sqrt((x64 * x64).mean(axis=-1, keepdims=True) + eps)
    assert np.array_equal(oracle.rms_norm(values, None, eps), (x64 * scale).astype(np.float32))
    assert np.array_equal(oracle.rms_norm(values, weight, eps), (x64 * scale * weight).astype(np.float32))
    # a constant row: x / sqrt(x^2 + eps)
    row = np.full((1, 64), -3.0, np.float32)
    assert np.allclose(oracle.rms_norm(row, None, 0.25), -3.0 / np.sqrt(9.25), rtol=0, atol=1e-7)
    # random rows against numpy f64 (summation order may differ in the last f64 bits only)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((7, 1000)).astype(np.float32) * 30
    w = rng.standard_normal(1000).astype(np.float32)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 * x64).mean(axis=-1, keepdims=True) + 1e-6) * w
    got = oracle.rms_norm(x, w, 1e-6)
    assert np.abs(got - want).max() <= np.abs(want).max() * 6e-8


def test_rotary_reference_test():
    # composed.rs:6393-6466
    x = np.array([1, 2, 3, 4], np.float32).reshape(1, 1, 4)
    s0, c0 = np.sin(np.float32(1.0)), np.cos(np.float32(1.0))
    s1, c1 = np.sin(np.float32(0.01)), np.cos(np.float32(0.01))
    half = oracle.rotary(x, [1], 10000.0)
    inter = oracle.rotary(x, [1], 10000.0, interleaved=True)
    assert np.allclose(half.ravel(), [1 * c0 - 3 * s0, 2 * c1 - 4 * s1, 3 * c0 + 1 * s0, 4 * c1 + 2 * s1],
                       rtol=0, atol=2e-6)
    assert np.allclose(inter.ravel(), [1 * c0 - 2 * s0, 2 * c0 + 1 * s0, 3 * c1 - 4 * s1, 4 * c1 + 3 * s1],
                       rtol=0, atol=2e-6)
    assert np.allclose(oracle.rotary(half, [1], 10000.0, sign=-1.0), x, rtol=0, atol=2e-6)
    assert np.allclose(oracle.rotary(inter, [1], 10000.0, sign=-1.0, interleaved=True), x, rtol=0, atol=2e-6)
    rank_two = oracle.rotary(np.arange(1, 9, dtype=np.float32).reshape(2, 4), [0], 10000.0, interleaved=True)
    assert np.allclose(rank_two.ravel(), [1, 2, 3, 4, 5 * c0 - 6 * s0, 6 * c0 + 5 * s0, 7 * c1 - 8 * s1,
                                          8 * c1 + 7 * s1], rtol=0, atol=2e-6)


@pytest.mark.parametrize("interleaved", [False, True])
def test_rotary_invariants(interleaved):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 4, 5, 16)).astype(np.float32)
    out = oracle.rotary(x, [7, 0, 123456], 500000.0, interleaved=interleaved)
    pairs = (lambda a: a.reshape(a.shape[:-1] + (8, 2))) if interleaved else \
        (lambda a: np.stack([a[..., :8], a[..., 8:]], axis=-1))
    assert np.allclose((pairs(out) ** 2).sum(-1), (pairs(x) ** 2).sum(-1), rtol=1e-5)
    # per-batch offsets are the same as one call per batch entry
    for b, offset in enumerate([7, 0, 123456]):
        assert np.array_equal(out[b:b + 1], oracle.rotary(x[b:b + 1], [offset], 500000.0, interleaved=interleaved))
    # position 0 is the identity; against the formula in numpy f64
    assert np.array_equal(oracle.rotary(x[:, :, :1], [0], 500000.0, interleaved=interleaved), x[:, :, :1])
    position = 7 + np.arange(5)[:, None]
    angle = position * 500000.0 ** (-2.0 * np.arange(8) / 16.0)
    a, b = pairs(x[0].astype(np.float64))[..., 0], pairs(x[0].astype(np.float64))[..., 1]
    want = np.stack([a * np.cos(angle) - b * np.sin(angle), b * np.cos(angle) + a * np.sin(angle)], axis=-1)
    assert np.abs(pairs(out[0]) - want).max() <= 1e-6
    with pytest.raises(oracle.OracleError, match="rotary embedding: 2 offsets for batch 3"):
        oracle.rotary(x, [1, 2], 10000.0)


def test_silu_mul_against_the_closed_form():
    rng = np.random.default_rng(2)
    gate = np.concatenate([rng.standard_normal(5000) * 4, [0.0, -0.0, 30.0, -30.0, 1e-8, 88.0, -88.0]]).astype(np.float32)
    up = rng.standard_normal(gate.size).astype(np.float32)
    got = oracle.silu_mul(gate, up)
    g64, u64 = gate.astype(np.float64), up.astype(np.float64)
    want = g64 / (1.0 + np.exp(-g64)) * u64
    # tanh(x / 2) / 2 + 1 / 2 loses the sigmoid's relative accuracy for very negative x: absolute bar there
    assert np.all(np.abs(got - want) <= 1e-6 * np.abs(want) + 1e-7 * np.abs(g64 * u64))
    assert got[5000] == 0.0 and got[5002] == np.float32(30.0) * up[5002]


def test_argmax_reference_tie_and_errors():
    assert oracle.argmax_rows(np.array([[1.0, 4.0, 4.0, 2.0]], np.float32))[0] == 1  # sampling.rs:223-238
    rng = np.random.default_rng(3)
    logits = rng.standard_normal((9, 5000)).astype(np.float32)
    logits[4, 77] = logits[4].max()  # a later duplicate of the maximum loses
    assert np.array_equal(oracle.argmax_rows(logits), logits.argmax(axis=-1))
    logits[6, 4000] = np.inf
    with pytest.raises(oracle.OracleError, match="sample: logit 4000 is not finite"):
        oracle.argmax_rows(logits)
    logits[2, 5] = np.nan
    with pytest.raises(oracle.OracleError, match="sample: logit 5 is not finite"):
        oracle.argmax_rows(logits)


def test_gather_rows():
    rng = np.random.default_rng(4)
    table = rng.standard_normal((50, 24)).astype(np.float16)
    indexes = rng.integers(0, 50, (3, 7))
    assert np.array_equal(oracle.gather_rows(table, indexes).view(np.uint16), table[indexes].view(np.uint16))
    with pytest.raises(oracle.OracleError, match="index_select: index 50 is out of bounds for extent 50"):
        oracle.gather_rows(table, [1, 50])


def test_add_is_ieee_addition():
    rng = np.random.default_rng(5)
    a = (rng.standard_normal(10000) * 1e3).astype(np.float32)
    b = (rng.standard_normal(10000) * 1e-3).astype(np.float32)
    assert np.array_equal(oracle.add(a, b), a + b)
