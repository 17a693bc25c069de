"""The canonical K-quant block fixtures the reference's own tests hold, as data.

Bytes and expected per-group values of the five fixtures declared in
crates/runtime-cpu/src/quantized.rs:629-778 (re-declared for the Metal backend
in crates/runtime-metal/src/executable.rs:8294-8370). Each fixture decodes to
groups of ``group_width`` equal values.
"""
import numpy as np

Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 10, 11, 12, 13, 14


def _q2():
    b = np.zeros(84, np.uint8)
    for i in range(16):
        b[i] = 0x10 | (i % 15 + 1)
    b[16:80] = 0xE4
    b[80:84] = [0x00, 0x3C, 0x00, 0x38]
    return b


def _q3():
    b = np.zeros(110, np.uint8)
    b[0:32] = 0xAA
    b[32:96] = 0xE4
    b[96:104] = 0x11
    b[104:108] = 0xAA
    b[108:110] = [0x00, 0x3C]
    return b


def _scale_min(n, quant_offset, high_offset=None):
    b = np.zeros(n, np.uint8)
    b[0:4] = [0x00, 0x3C, 0x00, 0x38]
    b[4:8] = 1
    b[8:12] = 2
    b[12:16] = 0x21
    if high_offset is not None:
        b[high_offset:high_offset + 32] = 0x99
    b[quant_offset:] = 0xE4
    return b


def _q6():
    b = np.zeros(210, np.uint8)
    b[0:192] = 0xE4
    for i in range(16):
        b[192 + i] = i + 1
    b[208:210] = [0x00, 0x38]
    return b


FIXTURES = {
    Q2_K: dict(bytes=_q2(), group_width=16, expected=[-0.5, -0.5, 2.5, 3.5, 9.5, 11.5, 20.5, 23.5,
                                                      -0.5, -0.5, 10.5, 11.5, 25.5, 27.5, 44.5, 2.5]),
    Q3_K: dict(bytes=_q3(), group_width=16, expected=[-4.0, -4.0, 1.0, 1.0, -2.0, -2.0, 3.0, 3.0,
                                                      -4.0, -4.0, 1.0, 1.0, -2.0, -2.0, 3.0, 3.0]),
    Q4_K: dict(bytes=_scale_min(144, 16), group_width=32,
               expected=[3.0, 13.0, 3.0, 13.0, 3.0, 13.0, 3.0, 13.0]),
    Q5_K: dict(bytes=_scale_min(176, 48, 16), group_width=32,
               expected=[19.0, 13.0, 3.0, 29.0, 19.0, 13.0, 3.0, 29.0]),
    Q6_K: dict(bytes=_q6(), group_width=16, expected=[-14.0, -28.0, -18.0, -24.0, 35.0, 42.0, 105.0,
                                                      120.0, -126.0, -140.0, -66.0, -72.0, 91.0,
                                                      98.0, 225.0, 240.0]),
}


def expected_values(codec):
    f = FIXTURES[codec]
    return np.repeat(np.asarray(f["expected"], np.float32), f["group_width"])
