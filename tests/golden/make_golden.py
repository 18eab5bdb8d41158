#!/usr/bin/env python3
"""Writes tests/golden/blocks.npz: known-answer vectors for the block formats on the stage path.

The reference (mesh-llm) ships no vectors for this arithmetic -- it lives in un-vendored llama.cpp
(third_party/llama.cpp/upstream.txt:1) -- so the expected outputs here are derived independently of
both the C oracle and the HIP kernels: every block is packed from its "natural domain" description
(integer quants, integer sub-scales, fp16 super-scales) by the packers below, and every expected
value is computed in exact rational arithmetic (fractions.Fraction) with an explicit
round-to-nearest-even step wherever the format's definition rounds to binary32 / binary16.

Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import struct
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


# ---------------------------------------------------------------- exact IEEE rounding on rationals
def _round_rne(fr, mant_bits, emin):
    """Nearest (ties-to-even) value with `mant_bits` explicit mantissa bits and minimum normal exponent emin."""
    if fr == 0:
        return Fraction(0)
    s = -1 if fr < 0 else 1
    a = abs(fr)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    while Fraction(2) ** e > a:
        e -= 1
    while Fraction(2) ** (e + 1) <= a:
        e += 1
    e = max(e, emin)
    ulp = Fraction(2) ** (e - mant_bits)
    n = a / ulp
    q = n.numerator // n.denominator
    r = n - q
    if r > Fraction(1, 2) or (r == Fraction(1, 2) and q % 2 == 1):
        q += 1
    return s * q * ulp


def fl32(fr):
    return _round_rne(Fraction(fr), 23, -126)


def fl16(fr):
    v = _round_rne(Fraction(fr), 10, -14)
    return v  # caller checks overflow


def f32_exact(x):
    """Fraction of a python/numpy float that is already a binary32 value."""
    return Fraction(float(np.float32(x)))


def half_bits(fr):
    """binary16 bit pattern of an exactly representable rational (|fr| <= 65504)."""
    if fr == 0:
        return 0
    sign = 0x8000 if fr < 0 else 0
    a = abs(fr)
    if a < Fraction(2) ** -14:
        m = a / Fraction(2) ** -24
        assert m.denominator == 1
        return sign | int(m)
    e = 0
    while Fraction(2) ** (e + 1) <= a:
        e += 1
    while Fraction(2) ** e > a:
        e -= 1
    m = (a / Fraction(2) ** e - 1) * 1024
    assert m.denominator == 1, fr
    return sign | ((e + 15) << 10) | int(m)


def half_value(bits):
    s = -1 if bits & 0x8000 else 1
    e = (bits >> 10) & 0x1F
    m = bits & 0x3FF
    assert e != 0x1F
    if e == 0:
        return s * Fraction(m) * Fraction(2) ** -24
    return s * (1 + Fraction(m, 1024)) * Fraction(2) ** (e - 15)


def f32_to_half_bits(x):
    """binary32 -> binary16 bits, RNE, overflow to inf (finite input)."""
    fr = f32_exact(x)
    r = fl16(fr)
    if abs(r) > 65504:
        return (0x8000 if fr < 0 else 0) | 0x7C00
    b = half_bits(r)
    if fr < 0 or (fr == 0 and np.signbit(np.float32(x))):
        b |= 0x8000
    return b


class SF:
    """A rational with IEEE signed-zero bookkeeping: (value, sign bit)."""

    def __init__(self, v, neg=None):
        self.v = Fraction(v)
        self.neg = (self.v < 0) if neg is None or self.v != 0 else bool(neg)

    def mul32(self, o):
        return SF(fl32(self.v * o.v), self.neg != o.neg)

    def sub32(self, o):
        r = fl32(self.v - o.v)
        # x - y == 0: -0 only for (-0) - (+0); RNE gives +0 for exact cancellation
        return SF(r, self.neg and not o.neg) if r == 0 else SF(r)

    def f32(self):
        x = np.float32(float(self.v))
        return np.float32(-0.0) if (self.v == 0 and self.neg) else x


def round_half_away(fr):
    a = abs(fr)
    q = (a + Fraction(1, 2)).numerator // (a + Fraction(1, 2)).denominator
    return -q if fr < 0 else q


# ---------------------------------------------------------------- q8_0
def q8_0_expected(x):
    """x: 32 binary32 values -> 34 bytes, from the definition of quantize_row_q8_0_ref."""
    xs = [f32_exact(v) for v in x]
    amax = max(abs(v) for v in xs)
    d = fl32(amax / 127)
    inv = fl32(1 / d) if d != 0 else Fraction(0)
    out = bytearray(struct.pack("<H", f32_to_half_bits(float(d))))
    for v in xs:
        q = round_half_away(fl32(v * inv))
        assert -128 <= q <= 127
        out += struct.pack("<b", q)
    return bytes(out)


def q8_0_cases():
    rng = np.random.Generator(np.random.PCG64(2024))
    cases = []
    # (a) amax = 127 -> d = 1, id = 1: pure rounding-mode test (half away from zero, not half-even)
    a = np.zeros(32, np.float32)
    a[:16] = [127, -127, 63.5, 0.5, -0.5, 1.5, 2.5, -2.5, 3.5, -3.5, 126.5, -126.5, 0.49999997, -0.49999997, 1e-3, 0]
    a[16:] = np.arange(16, dtype=np.float32) * 4.5 - 30.25
    cases.append(a)
    cases.append(np.zeros(32, np.float32))                       # (b) all-zero block -> d = 0, q = 0
    cases.append((rng.standard_normal(32) * 1e-6).astype(np.float32))   # (c) tiny: fp16(d) is subnormal
    cases.append((rng.standard_normal(32) * 3e4).astype(np.float32))    # (d) large
    o = rng.standard_normal(32).astype(np.float32)               # (e) outlier channel x50
    o[7] *= 50
    cases.append(o)
    # (f) blocks where id = 1/d (unrounded f32 d) and 1/fp16(d) quantise some element differently
    found = 0
    while found < 3:
        v = rng.standard_normal(32).astype(np.float32)
        xs = [f32_exact(t) for t in v]
        amax = max(abs(t) for t in xs)
        d = fl32(amax / 127)
        inv = fl32(1 / d)
        dh = half_value(f32_to_half_bits(float(d)))
        inv_h = fl32(1 / dh)
        if any(round_half_away(fl32(t * inv)) != round_half_away(fl32(t * inv_h)) for t in xs):
            cases.append(v)
            found += 1
    for _ in range(6):                                            # (g) plain N(0,1)
        cases.append(rng.standard_normal(32).astype(np.float32))
    x = np.stack(cases)
    y = np.frombuffer(b"".join(q8_0_expected(r) for r in x), dtype=np.uint8).reshape(len(cases), 34)
    return x, y


# ---------------------------------------------------------------- fp16
def f16_cases():
    rng = np.random.Generator(np.random.PCG64(77))
    vals = [0.0, -0.0, 1.0, -1.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e6, -1e6, 2.0 ** -14, 2.0 ** -24,
            2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -26, 1.5 * 2.0 ** -24,
            2.5 * 2.0 ** -24, 6.1e-5, 6.0e-5, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11,
            np.nextafter(np.float32(1.0 + 2.0 ** -11), np.float32(2)), 0.1, -0.3333333, 1.11e-4, 1.38e-5,
            3.1415927, 1e-8, 2047.5, 2048.5, 2049.0]
    # every tie between neighbouring halves in a few binades, and the f32 values either side of it
    for e in (-16, -15, -14, -1, 0, 10, 15):
        for m in (0, 1, 2, 511, 1022, 1023):
            lo = (1 + m / 1024.0) * 2.0 ** e if e >= -14 else None
            if lo is None:
                continue
            step = 2.0 ** (e - 10)
            tie = np.float32(lo + step / 2)
            vals += [tie, np.nextafter(tie, np.float32(0)), np.nextafter(tie, np.float32(1e9))]
    vals += list((rng.standard_normal(64) * 10.0 ** rng.integers(-8, 5, 64)).astype(np.float32))
    x = np.array(vals, dtype=np.float32)
    y = np.array([f32_to_half_bits(v) for v in x], dtype=np.uint16)
    return x, y


# ---------------------------------------------------------------- K-quant packers (natural domain -> bytes)
def pack_scales_k4(sc, m):
    """8 six-bit scales + 8 six-bit mins -> 12 bytes (inverse of get_scale_min_k4)."""
    q = [0] * 12
    for j in range(8):
        if j < 4:
            q[j] |= sc[j]
            q[j + 4] |= m[j]
        else:
            q[j + 4] |= (sc[j] & 0xF) | ((m[j] & 0xF) << 4)
            q[j - 4] |= (sc[j] >> 4) << 6
            q[j] |= (m[j] >> 4) << 6
    return bytes(q)


def pack_q4_K(d_bits, dmin_bits, sc, m, L):
    """L: 256 ints in [0,15]; element 64c+l -> low nibble of qs[32c+l], element 64c+32+l -> high nibble."""
    qs = bytearray(128)
    for c in range(4):
        for l in range(32):
            qs[32 * c + l] = L[64 * c + l] | (L[64 * c + 32 + l] << 4)
    return struct.pack("<HH", d_bits, dmin_bits) + pack_scales_k4(sc, m) + bytes(qs)


def expect_q4_K(d_bits, dmin_bits, sc, m, L):
    d, dmin = SF(half_value(d_bits), d_bits >> 15), SF(half_value(dmin_bits), dmin_bits >> 15)
    out = []
    for i in range(256):
        s = i // 32
        d1 = d.mul32(SF(sc[s]))
        m1 = dmin.mul32(SF(m[s]))
        out.append(d1.mul32(SF(L[i])).sub32(m1).f32())
    return np.array(out, dtype=np.float32)


def pack_q6_K(d_bits, sc, L):
    """L: 256 ints in [0,63] (value = L-32); 16 signed sub-scales, one per 16 elements."""
    ql = bytearray(128)
    qh = bytearray(64)
    for n in range(2):
        for l in range(32):
            a, b, c, e = (L[128 * n + l + 32 * t] for t in range(4))
            ql[64 * n + l] = (a & 0xF) | ((c & 0xF) << 4)
            ql[64 * n + l + 32] = (b & 0xF) | ((e & 0xF) << 4)
            qh[32 * n + l] = (a >> 4) | ((b >> 4) << 2) | ((c >> 4) << 4) | ((e >> 4) << 6)
    return bytes(ql) + bytes(qh) + struct.pack("<16b", *sc) + struct.pack("<H", d_bits)


def expect_q6_K(d_bits, sc, L):
    d = SF(half_value(d_bits), d_bits >> 15)
    return np.array([d.mul32(SF(sc[i // 16])).mul32(SF(L[i] - 32)).f32() for i in range(256)], dtype=np.float32)


def pack_q5_0(d_bits, L):
    """L: 32 ints in [0,31] (value = L-16)."""
    qs = bytearray(16)
    qh = 0
    for j in range(16):
        qs[j] = (L[j] & 0xF) | ((L[j + 16] & 0xF) << 4)
        qh |= ((L[j] >> 4) & 1) << j
        qh |= ((L[j + 16] >> 4) & 1) << (j + 16)
    return struct.pack("<H", d_bits) + struct.pack("<I", qh) + bytes(qs)


def expect_q5_0(d_bits, L):
    d = SF(half_value(d_bits), d_bits >> 15)
    return np.array([SF(L[j] - 16).mul32(d).f32() for j in range(32)], dtype=np.float32)


def kquant_cases():
    rng = np.random.Generator(np.random.PCG64(99))
    h = lambda v: int(np.float16(v).view(np.uint16))
    q4_blocks, q4_exp = [], []
    q4_specs = [
        # all sub-scales equal, no mins: plain 4-bit affine y = d*7*q
        (h(0.5), h(0.0), [7] * 8, [0] * 8, [i % 16 for i in range(256)]),
        # sc_j = j+1, m_j = 60-j: both 6-bit paths (j<4 and j>=4, values >= 32 use the spilled high bits)
        (h(1.11e-4), h(8.3e-4), [j + 1 for j in range(8)], [60 - j for j in range(8)],
         [(i * 7 + i // 32) % 16 for i in range(256)]),
        (h(3.0e-3), h(1.7e-2), [63, 0, 32, 31, 48, 15, 16, 47], [0, 63, 31, 32, 15, 48, 47, 16],
         [(15 - i) % 16 for i in range(256)]),
        # subnormal fp16 super-scales
        (0x0123, 0x0045, list(rng.integers(0, 64, 8)), list(rng.integers(0, 64, 8)), list(rng.integers(0, 16, 256))),
        (h(-2.5e-4), h(9.9e-4), list(rng.integers(0, 64, 8)), list(rng.integers(0, 64, 8)), list(rng.integers(0, 16, 256))),
    ]
    for spec in q4_specs:
        spec = (spec[0], spec[1], [int(v) for v in spec[2]], [int(v) for v in spec[3]], [int(v) for v in spec[4]])
        q4_blocks.append(np.frombuffer(pack_q4_K(*spec), dtype=np.uint8))
        q4_exp.append(expect_q4_K(*spec))
    q6_blocks, q6_exp = [], []
    q6_specs = [
        (h(0.25), [1] * 16, [i % 64 for i in range(256)]),
        (h(1.5e-3), [(-1) ** i * (i * 8 + 1) for i in range(16)], [(i * 5 + i // 16) % 64 for i in range(256)]),
        (0x00E7, [int(v) for v in rng.integers(-128, 128, 16)], [int(v) for v in rng.integers(0, 64, 256)]),  # subnormal d
        (h(-7.0e-4), [int(v) for v in rng.integers(-128, 128, 16)], [int(v) for v in rng.integers(0, 64, 256)]),
    ]
    for spec in q6_specs:
        q6_blocks.append(np.frombuffer(pack_q6_K(*spec), dtype=np.uint8))
        q6_exp.append(expect_q6_K(*spec))
    q5_blocks, q5_exp = [], []
    for spec in [(h(0.125), list(range(32))), (h(3.3e-3), [int(v) for v in rng.integers(0, 32, 32)]),
                 (0x0201, [31 - i for i in range(32)])]:
        q5_blocks.append(np.frombuffer(pack_q5_0(*spec), dtype=np.uint8))
        q5_exp.append(expect_q5_0(*spec))
    return (np.stack(q4_blocks), np.stack(q4_exp), np.stack(q6_blocks), np.stack(q6_exp),
            np.stack(q5_blocks), np.stack(q5_exp))


def main():
    q8_x, q8_y = q8_0_cases()
    f16_x, f16_y = f16_cases()
    q4b, q4e, q6b, q6e, q5b, q5e = kquant_cases()
    out = os.path.join(HERE, "blocks.npz")
    np.savez_compressed(out, q8_0_x=q8_x, q8_0_blocks=q8_y, f16_x=f16_x, f16_bits=f16_y,
                        q4_K_blocks=q4b, q4_K_y=q4e, q6_K_blocks=q6b, q6_K_y=q6e,
                        q5_0_blocks=q5b, q5_0_y=q5e)
    print("wrote", out, {k: v.shape for k, v in np.load(out).items()})


if __name__ == "__main__":
    main()
