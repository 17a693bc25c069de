"""GPU parity of the one-pass small-batch GEMV (2..8 activation vectors; Q4_K, Q5_K, Q4_0, Q8_0; the regime
crates/runtime-metal/src/quantized.rs:1204-1220 keeps in its GEMV family): the HIP path through the C
ABI against the CPU oracle (linear_into, crates/runtime-cpu/src/quantized.rs:419-499) on the same
seeded inputs. Bar: |a-b| <= 1e-3 * max(|b|, 1), once against the oracle and once, with no allowance,
against the f64-exact value of the same contraction; and the same bits on a second run.
"""
import numpy as np
import pytest
import torch

import oracle
from effect_torch_amd import synth
from test_gpu_parity import close, run_linear, to_dev

pytestmark = pytest.mark.gpu

CODECS = [oracle.Q4_K, oracle.Q4_0, oracle.Q5_K, oracle.Q8_0]


def planned_kernel(et, codec, rows, columns, vectors, bias=False):
    return et.RawLinear(et.GgmlQuant(codec), rows, columns, vectors, bias).requirements.kernel


def check(et, device, codec, rows, columns, vectors, rng, bias=None, x_scale=1.0):
    weight = synth.random_weight(codec, rows, columns, rng)
    x = synth.random_activations(vectors, columns, rng, x_scale)
    assert planned_kernel(et, codec, rows, columns, vectors, bias is not None) == "gemv_mma"
    print(f"gemv_mma codec={codec} rows={rows} columns={columns} vectors={vectors}", flush=True)
    abandoned = et.handover_timeouts()
    got = run_linear(et, device, codec, rows, columns, x, weight, bias)
    again = run_linear(et, device, codec, rows, columns, x, weight, bias)
    assert np.array_equal(got, again)  # neither the arrival order of the copies nor that of the waves reaches the sums
    close(got, oracle.linear_into(codec, rows, columns, x, weight, bias))
    exact = x.astype(np.float64) @ oracle.decode_rows(codec, weight, columns).astype(np.float64).T
    if bias is not None:
        exact = exact + bias.astype(np.float64)
    close(got, exact, oracle_noise=0)
    assert et.handover_timeouts() == abandoned  # no wave gave up a wait
    return got


@pytest.mark.parametrize("codec", CODECS)
@pytest.mark.parametrize("vectors", [2, 3, 4, 5, 6, 7, 8])
def test_every_vector_count(et, device, codec, vectors):
    # 4099 rows: ranges of 17 rows (a whole group of sixteen and a group of one), a ragged last range
    rng = np.random.default_rng(100 * codec + vectors)
    check(et, device, codec, 4099, 4096, vectors, rng, rng.standard_normal(4099).astype(np.float32))


@pytest.mark.parametrize("codec", CODECS)
@pytest.mark.parametrize("vectors,rows,columns", [
    (2, 2048, 4096),     # half a group per range
    (4, 2100, 4096),     # ranges of 9 rows, the last of 6
    (3, 5003, 256),      # one unit per row: seven of the eight consumer waves hold no columns
    (8, 3000, 2048),     # four consumer waves hold columns
    (5, 30000, 512),     # 118 rows per range, images of 36 KiB
    (8, 40000, 4096),    # more rows than 256 images hold: three rounds of 256 ranges of 53 rows
    (6, 9000, 1024),
    (4, 12000, 3072),    # the last consumer waves hold one unit / none
    (7, 2300, 3840),     # fifteen units: the last wave holds one
])
def test_shapes(et, device, codec, vectors, rows, columns):
    rng = np.random.default_rng(7 * codec + vectors + rows + columns)
    bias = rng.standard_normal(rows).astype(np.float32) if rows % 2 else None
    check(et, device, codec, rows, columns, vectors, rng, bias)


@pytest.mark.parametrize("name", ["q4_0_gemv_11008x4096", "q4_k_gemv_14336x4096", "q8_0_gemv_4096x4096"])
@pytest.mark.parametrize("vectors", [2, 3, 4, 5, 6, 7, 8])
def test_full_size(et, device, name, vectors):
    cfg = synth.CONFIGS[name]
    rng = np.random.default_rng(cfg["seed"] + 50 + vectors)
    check(et, device, cfg["codec"], cfg["rows"], cfg["columns"], vectors, rng, None, cfg["x_scale"])


@pytest.mark.parametrize("codec", CODECS)
def test_special_activations(et, device, codec):
    # unit vectors select one decoded weight (every other product is an exact zero; what is left is the
    # rounding of d * (scale * quant) against the decoder's (d * scale) * quant, and for Q4_0 of d * quant - 8 * d: a
    # few 1e-8 of the largest weight); a vector of
    # zeros gives zeros; a vector whose 256-column units differ by 2^20 in size keeps every unit's precision
    rows, columns, vectors = 2304, 4096, 4
    rng = np.random.default_rng(31 + codec)
    weight = synth.random_weight(codec, rows, columns, rng)
    decoded = oracle.decode_rows(codec, weight, columns)
    x = np.zeros((vectors, columns), np.float32)
    picks = [5, 1000, 4095]
    for v, k in enumerate(picks):
        x[v, k] = 1.0
    got = run_linear(et, device, codec, rows, columns, x, weight)
    for v, k in enumerate(picks):
        np.testing.assert_allclose(got[v], decoded[:, k], rtol=5e-7, atol=1e-7 * np.abs(decoded[:, k]).max())
    assert not got[3].any()
    x = synth.random_activations(vectors, columns, rng)
    x[:, :256] *= 2.0 ** 20
    x[:, 256:512] *= 2.0 ** -20
    got = run_linear(et, device, codec, rows, columns, x, weight)
    exact = x.astype(np.float64) @ decoded.astype(np.float64).T
    close(got, exact)  # outputs that cancel to a millionth of the row's size: the allowance of an f32 sum
    small = x.copy()
    small[:, :256] = 0.0  # without the large unit the small one must come out to its own precision
    tail = run_linear(et, device, codec, rows, columns, small, weight)
    exact_tail = x[:, 256:].astype(np.float64) @ decoded[:, 256:].astype(np.float64).T
    close(tail, exact_tail, oracle_noise=0)


def test_strided_activation_rows(et, device):
    # rows of a wider tensor (unit trailing stride, 16-byte aligned): read in place
    rows, columns, vectors = 4096, 4096, 5
    rng = np.random.default_rng(77)
    weight = synth.random_weight(oracle.Q4_K, rows, columns, rng)
    wide = torch.from_numpy(rng.standard_normal((vectors, 2 * columns)).astype(np.float32)).to(device)
    view = wide[:, columns:]
    got = run_linear(et, device, oracle.Q4_K, rows, columns, view, weight)
    close(got, oracle.linear_into(oracle.Q4_K, rows, columns, view.cpu().numpy().copy(), weight))


def test_a_wait_that_is_given_up_ends_the_launch(et, device):
    # Every wait of a consumer wave on another wave is bounded. With the bound at zero polls a wave that
    # finds its rows not landed yet gives up at once: the launch must still end (every wave leaves the
    # kernel), the device word counts the waves, and the next launch with the library's own bound is right.
    codec, rows, columns, vectors = oracle.Q4_K, 14336, 4096, 4
    rng = np.random.default_rng(5)
    weight = synth.random_weight(codec, rows, columns, rng)
    x = synth.random_activations(vectors, columns, rng)
    before = et.handover_timeouts()
    et.set_handover_spin_limit(0)
    try:
        run_linear(et, device, codec, rows, columns, x, weight)  # returns: the launch has ended
        single = run_linear(et, device, codec, rows, columns, x[:1], weight)  # gemv_limb_dma, same bound
    finally:
        et.set_handover_spin_limit()
    assert single.shape == (1, rows)
    assert et.handover_timeouts() > before
    counted = et.handover_timeouts()
    got = run_linear(et, device, codec, rows, columns, x, weight)
    close(got, oracle.linear_into(codec, rows, columns, x, weight))
    one = run_linear(et, device, codec, rows, columns, x[:1], weight)
    close(one, oracle.linear_into(codec, rows, columns, x[:1], weight))
    assert et.handover_timeouts() == counted
