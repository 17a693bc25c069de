"""Block packers written from the documented ggml layouts, independently of any decoder.

Each ``pack_*`` takes the logical fields of ONE block (fp16 bit patterns, integer
sub-scales, integer quants in logical element order) and lays them out in the
packed byte format; each ``closed_form_*`` gives the f32 values those fields
stand for, evaluated with numpy float32 arithmetic one rounding per operation
(the reference's order: ``d*scale``, ``dmin*min``, then multiply, then subtract).
A decoder that returns ``closed_form(fields)`` for ``pack(fields)`` on random
fields has the right offsets, bit order, element order and rounding sequence.
"""
import numpy as np


def f16_bits_to_f32(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float32)


def _le16(bits):
    return [bits & 0xFF, (bits >> 8) & 0xFF]


def pack_scales_k4(sc, mn):
    """8 six-bit scales + 8 six-bit mins -> 12 bytes (Q4_K / Q5_K)."""
    out = np.zeros(12, np.uint8)
    for j in range(4):
        out[j] = sc[j] | ((sc[j + 4] >> 4) << 6)
        out[j + 4] = mn[j] | ((mn[j + 4] >> 4) << 6)
        out[j + 8] = (sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4)
    return out


def pack_q4_k(d_bits, dmin_bits, sc, mn, q):
    b = np.zeros(144, np.uint8)
    b[0:2] = _le16(d_bits)
    b[2:4] = _le16(dmin_bits)
    b[4:16] = pack_scales_k4(sc, mn)
    q = np.asarray(q, np.uint8)
    for p in range(4):
        b[16 + 32 * p:16 + 32 * p + 32] = q[64 * p:64 * p + 32] | (q[64 * p + 32:64 * p + 64] << 4)
    return b


def closed_form_k4(d_bits, dmin_bits, sc, mn, q):
    d = f16_bits_to_f32(d_bits)
    dmin = f16_bits_to_f32(dmin_bits)
    dl = (d * np.asarray(sc, np.float32)).astype(np.float32)
    ml = (dmin * np.asarray(mn, np.float32)).astype(np.float32)
    q = np.asarray(q, np.float32).reshape(8, 32)
    prod = (dl[:, None] * q).astype(np.float32)
    return (prod - ml[:, None]).astype(np.float32).reshape(256)


def pack_q5_k(d_bits, dmin_bits, sc, mn, q):
    b = np.zeros(176, np.uint8)
    b[0:2] = _le16(d_bits)
    b[2:4] = _le16(dmin_bits)
    b[4:16] = pack_scales_k4(sc, mn)
    q = np.asarray(q, np.uint8)
    for g in range(8):
        hi = (q[32 * g:32 * g + 32] >> 4) & 1
        b[16:48] |= (hi << g).astype(np.uint8)
    low = q & 0xF
    for p in range(4):
        b[48 + 32 * p:48 + 32 * p + 32] = low[64 * p:64 * p + 32] | (low[64 * p + 32:64 * p + 64] << 4)
    return b


def pack_q6_k(d_bits, scales_i8, q):
    """q: 256 values in -32..31; scales_i8: 16 signed bytes (one per 16 values)."""
    b = np.zeros(210, np.uint8)
    u = (np.asarray(q, np.int32) + 32).astype(np.uint8)
    for h in range(2):
        e = 128 * h
        lo, hi = u & 0xF, u >> 4
        b[64 * h:64 * h + 32] = lo[e:e + 32] | (lo[e + 64:e + 96] << 4)
        b[64 * h + 32:64 * h + 64] = lo[e + 32:e + 64] | (lo[e + 96:e + 128] << 4)
        b[128 + 32 * h:128 + 32 * h + 32] = (hi[e:e + 32] | (hi[e + 32:e + 64] << 2) |
                                               (hi[e + 64:e + 96] << 4) | (hi[e + 96:e + 128] << 6))
    b[192:208] = np.asarray(scales_i8, np.int8).view(np.uint8)
    b[208:210] = _le16(d_bits)
    return b


def closed_form_q6_k(d_bits, scales_i8, q):
    d = f16_bits_to_f32(d_bits)
    ds = (d * np.asarray(scales_i8, np.float32)).astype(np.float32)
    return (np.repeat(ds, 16) * np.asarray(q, np.float32)).astype(np.float32)


def _two_bit_positions():
    """byte index (within the 64 quant bytes) and shift of element e, Q2_K / Q3_K."""
    e = np.arange(256)
    return 32 * (e // 128) + (e % 32), 2 * ((e % 128) // 32)


def pack_q2_k(d_bits, dmin_bits, sc4, mn4, q):
    """sc4 / mn4: 16 four-bit values (one per 16 elements); q: 256 values in 0..3."""
    b = np.zeros(84, np.uint8)
    b[0:16] = np.asarray(sc4, np.uint8) | (np.asarray(mn4, np.uint8) << 4)
    byte, shift = _two_bit_positions()
    for e in range(256):
        b[16 + byte[e]] |= int(q[e]) << int(shift[e])
    b[80:82] = _le16(d_bits)
    b[82:84] = _le16(dmin_bits)
    return b


def closed_form_q2_k(d_bits, dmin_bits, sc4, mn4, q):
    d = f16_bits_to_f32(d_bits)
    dmin = f16_bits_to_f32(dmin_bits)
    dl = np.repeat((d * np.asarray(sc4, np.float32)).astype(np.float32), 16)
    ml = np.repeat((dmin * np.asarray(mn4, np.float32)).astype(np.float32), 16)
    return ((dl * np.asarray(q, np.float32)).astype(np.float32) - ml).astype(np.float32)


def pack_q3_k(d_bits, sc6, q):
    """sc6: 16 six-bit scale codes (value = code - 32); q: 256 values in -4..3."""
    b = np.zeros(110, np.uint8)
    u = np.asarray(q, np.int32) + 4  # 0..7
    byte, shift = _two_bit_positions()
    for e in range(256):
        b[32 + byte[e]] |= int(u[e] & 3) << int(shift[e])
        if u[e] >> 2:
            b[e % 32] |= 1 << (e // 32)
    for g in range(16):
        low, high = sc6[g] & 0xF, sc6[g] >> 4
        if g < 8:
            b[96 + g] |= low
        else:
            b[96 + g - 8] |= low << 4
        b[96 + 8 + g % 4] |= high << (2 * (g // 4))
    b[108:110] = _le16(d_bits)
    return b


def closed_form_q3_k(d_bits, sc6, q):
    d = f16_bits_to_f32(d_bits)
    dl = (d * (np.asarray(sc6, np.float32) - np.float32(32))).astype(np.float32)
    return (np.repeat(dl, 16) * np.asarray(q, np.float32)).astype(np.float32)


def pack_q8_0(d_bits, q):
    b = np.zeros(34, np.uint8)
    b[0:2] = _le16(d_bits)
    b[2:34] = np.asarray(q, np.int8).view(np.uint8)
    return b


def pack_q4_0(d_bits, q):
    """q: 32 values in -8..7."""
    b = np.zeros(18, np.uint8)
    b[0:2] = _le16(d_bits)
    u = (np.asarray(q, np.int32) + 8).astype(np.uint8)
    b[2:18] = u[0:16] | (u[16:32] << 4)
    return b


def closed_form_scaled(d_bits, q):
    return (f16_bits_to_f32(d_bits) * np.asarray(q, np.float32)).astype(np.float32)


INTERESTING_F16 = [0x3C00, 0x3800, 0x0001, 0x03FF, 0x0400, 0x7BFF, 0x1234, 0x2E66, 0xBC00, 0x8001,
                   0x0000, 0x211F]


def random_block(codec, rng, d_bits=None, dmin_bits=None):
    """(packed bytes, closed-form f32 values) of one random block of ``codec``."""
    d_bits = int(rng.choice(INTERESTING_F16)) if d_bits is None else d_bits
    dmin_bits = int(rng.choice(INTERESTING_F16)) if dmin_bits is None else dmin_bits
    if codec == 12:
        sc, mn, q = rng.integers(0, 64, 8), rng.integers(0, 64, 8), rng.integers(0, 16, 256)
        return pack_q4_k(d_bits, dmin_bits, sc, mn, q), closed_form_k4(d_bits, dmin_bits, sc, mn, q)
    if codec == 13:
        sc, mn, q = rng.integers(0, 64, 8), rng.integers(0, 64, 8), rng.integers(0, 32, 256)
        return pack_q5_k(d_bits, dmin_bits, sc, mn, q), closed_form_k4(d_bits, dmin_bits, sc, mn, q)
    if codec == 14:
        sc, q = rng.integers(-128, 128, 16), rng.integers(-32, 32, 256)
        return pack_q6_k(d_bits, sc, q), closed_form_q6_k(d_bits, sc, q)
    if codec == 10:
        sc, mn, q = rng.integers(0, 16, 16), rng.integers(0, 16, 16), rng.integers(0, 4, 256)
        return pack_q2_k(d_bits, dmin_bits, sc, mn, q), closed_form_q2_k(d_bits, dmin_bits, sc, mn, q)
    if codec == 11:
        sc, q = rng.integers(0, 64, 16), rng.integers(-4, 4, 256)
        return pack_q3_k(d_bits, sc, q), closed_form_q3_k(d_bits, sc, q)
    if codec == 8:
        q = rng.integers(-128, 128, 32)
        return pack_q8_0(d_bits, q), closed_form_scaled(d_bits, q)
    if codec == 2:
        q = rng.integers(-8, 8, 32)
        return pack_q4_0(d_bits, q), closed_form_scaled(d_bits, q)
    raise ValueError(codec)
