"""Seeded synthetic weights and activations in the packed GGUF block layouts.

Used by the benchmark, the smoke check and the tests to build inputs of the
shapes and distributions the workload definitions name: quants uniform over
their range, per-block fp16 scales ``|N(0,1)| * s``, activations ``N(0,1)``.
Pure numpy; nothing here touches the GPU.
"""
from __future__ import annotations

import numpy as np

Q4_0, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 2, 8, 10, 11, 12, 13, 14

BLOCK_VALUES = {Q4_0: 32, Q8_0: 32, Q2_K: 256, Q3_K: 256, Q4_K: 256, Q5_K: 256, Q6_K: 256}
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34, Q2_K: 84, Q3_K: 110, Q4_K: 144, Q5_K: 176, Q6_K: 210}
# byte offsets of the fp16 fields of a block
_FP16_FIELDS = {Q4_0: (0,), Q8_0: (0,), Q2_K: (80, 82), Q3_K: (108,), Q4_K: (0, 2), Q5_K: (0, 2),
                Q6_K: (208,)}
# Q4_0 / Q8_0 / Q4_K: the scales the workload definitions name. The others are chosen so
# that decoded weights have a comparable magnitude (a few units).
DEFAULT_SCALE = {Q4_0: 0.02, Q8_0: 0.01, Q2_K: 0.1, Q3_K: 0.05, Q4_K: 0.01, Q5_K: 0.005, Q6_K: 0.002}


def row_bytes(codec: int, columns: int) -> int:
    assert columns % BLOCK_VALUES[codec] == 0
    return columns // BLOCK_VALUES[codec] * BLOCK_BYTES[codec]


def random_weight(codec: int, rows: int, columns: int, rng: np.random.Generator,
                  scale: float | None = None) -> np.ndarray:
    """Packed ``[rows, row_bytes]`` u8: every quant / sub-scale bit uniform,
    fp16 block scales ``|N(0,1)| * scale`` (round to nearest even)."""
    scale = DEFAULT_SCALE[codec] if scale is None else scale
    blocks = rows * (columns // BLOCK_VALUES[codec])
    size = BLOCK_BYTES[codec]
    data = rng.integers(0, 256, size=(blocks, size), dtype=np.uint8)
    if codec == Q8_0:
        # int8 quants uniform in [-127, 127] (-128 is never produced by a quantiser)
        data[:, 2:] = rng.integers(-127, 128, size=(blocks, 32), dtype=np.int8).view(np.uint8)
    for offset in _FP16_FIELDS[codec]:
        value = (np.abs(rng.standard_normal(blocks)) * scale).astype(np.float16)
        data[:, offset:offset + 2] = value.view(np.uint8).reshape(blocks, 2)
    return data.reshape(rows, -1)


def random_activations(vectors: int, columns: int, rng: np.random.Generator,
                       scale: float = 1.0) -> np.ndarray:
    return (rng.standard_normal((vectors, columns)) * scale).astype(np.float32)


# The benchmark configurations: (codec, rows, columns, vector counts, activation scale, mode).
CONFIGS = {
    "q8_0_gemv_4096x4096": dict(codec=Q8_0, rows=4096, columns=4096, vectors=(1,), x_scale=1.0, seed=0xE77C0DE0),
    "q4_0_gemv_11008x4096": dict(codec=Q4_0, rows=11008, columns=4096, vectors=(1, 4, 8), x_scale=1.0, seed=0xE77C0DE1),
    "q4_k_gemv_14336x4096": dict(codec=Q4_K, rows=14336, columns=4096, vectors=(1, 16, 64), x_scale=1.0, seed=0xE77C0DE2),
    "q2_k_gemv_14336x4096": dict(codec=Q2_K, rows=14336, columns=4096, vectors=(1, 2), x_scale=1.0, seed=0xE77C0DE2),
    "q3_k_gemv_14336x4096": dict(codec=Q3_K, rows=14336, columns=4096, vectors=(1, 2), x_scale=1.0, seed=0xE77C0DE3),
    "q5_k_gemv_14336x4096": dict(codec=Q5_K, rows=14336, columns=4096, vectors=(1, 2), x_scale=1.0, seed=0xE77C0DE5),
    "q6_k_gemv_14336x4096": dict(codec=Q6_K, rows=14336, columns=4096, vectors=(1, 2), x_scale=1.0, seed=0xE77C0DE6),
    "q8_0_gemm_i8_512x14336x4096": dict(codec=Q8_0, rows=4096, columns=14336, vectors=(512,), x_scale=0.5, seed=0xE77C0DE3),
}
