"""Pins oracle/mesh_oracle.c's block formats by means independent of it: numpy's IEEE binary16,
the exact-rational golden vectors of tests/golden/make_golden.py, natural-domain closed forms and
invariants.  (ggml itself is not reachable offline, so this is what "parity" rests on.)"""
import numpy as np
import pytest

import oracle


def test_fp16_decode_exhaustive_vs_numpy():
    h = np.arange(65536, dtype=np.uint16)
    got = oracle.fp16_to_fp32(h)
    ref = h.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), ref[~nan].view(np.uint32))


def test_fp16_encode_vs_numpy_random_bits():
    rng = np.random.Generator(np.random.PCG64(5))
    bits = rng.integers(0, 2**32, size=4_000_000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.fp32_to_fp16(x), ref)


def test_fp16_encode_all_ties_and_neighbours():
    # every midpoint between adjacent finite halves, and the binary32 values just below/above it
    h = np.arange(0, 0x7C00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    hi[-1] = 65536.0  # the value "after" 65504 for rounding purposes
    mid = ((lo + hi) / 2).astype(np.float32)  # exactly representable in binary32
    for x in (mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9)), -mid):
        with np.errstate(over="ignore"):
            ref = x.astype(np.float16).view(np.uint16)
        assert np.array_equal(oracle.fp32_to_fp16(x), ref)


def test_fp16_encode_nan_inf():
    x = np.array([np.inf, -np.inf, np.nan, -np.nan], dtype=np.float32)
    got = oracle.fp32_to_fp16(x)
    assert got[0] == 0x7C00 and got[1] == 0xFC00
    assert got[2] & 0x7FFF == 0x7E00 and got[3] & 0x7FFF == 0x7E00


def test_fp16_golden(golden):
    assert np.array_equal(oracle.fp32_to_fp16(golden["f16_x"]), golden["f16_bits"])


def test_q8_0_golden(golden):
    x, y = golden["q8_0_x"], golden["q8_0_blocks"]
    got = oracle.quantize_q8_0(x.reshape(-1)).reshape(-1, 34)
    assert np.array_equal(got, y)
    # rounding mode spelled out: block 0 has d = 1
    q = got[0, 2:].view(np.int8)
    assert list(q[:14]) == [127, -127, 64, 1, -1, 2, 3, -3, 4, -4, 127, -127, 0, 0]


def _c2_like(T, h=4096, seed=None):
    rng = np.random.Generator(np.random.PCG64(1234 + T if seed is None else seed))
    x = rng.standard_normal((T, h)).astype(np.float32)
    ch = np.random.Generator(np.random.PCG64(1234)).choice(h, size=5, replace=False)
    x[:, ch] *= 50
    return x


def test_q8_0_invariants():
    x = _c2_like(16)
    blk = oracle.quantize_q8_0(x.reshape(-1)).reshape(-1, 34)
    q = blk[:, 2:].view(np.int8).astype(np.int32)
    d = blk[:, :2].copy().view(np.float16).astype(np.float32).reshape(-1)
    xb = x.reshape(-1, 32)
    am = np.argmax(np.abs(xb), axis=1)
    rows = np.arange(xb.shape[0])
    assert np.array_equal(q[rows, am], np.where(xb[rows, am] > 0, 127, -127))
    assert np.abs(q).max() <= 127
    # reconstruction bound: half a step plus the fp16 rounding of the scale
    err = np.abs(xb - q * d[:, None])
    dtrue = np.abs(xb).max(axis=1) / 127
    assert np.all(err <= dtrue[:, None] * 0.5 * 1.0001 + np.abs(xb) * 2.0**-10)
    # dequantize is q * fp16(d)
    deq = oracle.dequantize(oracle.Q8_0, blk.reshape(-1), x.size).reshape(-1, 32)
    assert np.array_equal(deq, (q * d[:, None]).astype(np.float32))


def test_q8_0_matches_float32_numpy_restatement():
    # same definition evaluated by numpy's IEEE float32 ops (vectorised), half-away rounding done in float64
    x = _c2_like(64, seed=9).reshape(-1, 32)
    amax = np.abs(x).max(axis=1)
    d = (amax / np.float32(127)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1) / d, np.float32(0)).astype(np.float32)
    v = (x * inv[:, None]).astype(np.float32).astype(np.float64)
    q = (np.sign(v) * np.floor(np.abs(v) + 0.5)).astype(np.int8)
    blk = oracle.quantize_q8_0(x.reshape(-1)).reshape(-1, 34)
    assert np.array_equal(blk[:, 2:].view(np.int8), q)
    assert np.array_equal(blk[:, :2].copy().view(np.uint16).reshape(-1), d.astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("name,type_,k", [("q4_K", oracle.Q4_K, 256), ("q6_K", oracle.Q6_K, 256), ("q5_0", oracle.Q5_0, 32)])
def test_kquant_golden(golden, name, type_, k):
    blocks, y = golden[name + "_blocks"], golden[name + "_y"]
    got = oracle.dequantize(type_, blocks.reshape(-1), k * blocks.shape[0]).reshape(-1, k)
    assert np.array_equal(got.view(np.uint32), y.view(np.uint32))


def test_q4_K_plain_affine_special_case():
    # all sub-scales equal and dmin = 0 reduces to y = (d*s) * nibble, nibble l of byte b at 64c+l / 64c+32+l
    rng = np.random.Generator(np.random.PCG64(3))
    qs = rng.integers(0, 256, 128, dtype=np.uint8)
    s = 21
    scales = bytes([s] * 4 + [0] * 4 + [s & 0xF] * 4)  # j<4: sc=s,m=0 ; j>=4: low nibble sc, high bits from q[j-4]>>6 = 0
    d = np.float16(0.0123)
    blk = np.frombuffer(d.tobytes() + np.float16(0).tobytes() + scales + qs.tobytes(), dtype=np.uint8)
    y = oracle.dequantize(oracle.Q4_K, blk, 256)
    ds_lo = np.float32(d) * np.float32(s)
    ds_hi = np.float32(d) * np.float32(s & 0xF)
    for c in range(4):
        ds = ds_lo if c < 2 else ds_hi
        assert np.array_equal(y[64 * c:64 * c + 32], ds * (qs[32 * c:32 * c + 32] & 0xF).astype(np.float32) - np.float32(0))
        assert np.array_equal(y[64 * c + 32:64 * c + 64], ds * (qs[32 * c:32 * c + 32] >> 4).astype(np.float32))


def test_row_bytes():
    assert oracle.row_bytes(oracle.Q4_K, 4096) == 16 * 144
    assert oracle.row_bytes(oracle.Q6_K, 14336) == 56 * 210
    assert oracle.row_bytes(oracle.Q8_0, 896) == 28 * 34
    assert oracle.row_bytes(oracle.Q5_0, 896) == 28 * 22
    assert oracle.row_bytes(oracle.Q4_K, 896) == -1
    assert oracle.row_bytes(oracle.F16, 7) == 14 and oracle.row_bytes(oracle.F32, 7) == 28


def test_add_and_truncate_equals_round_half_away():
    """The q8_0 pack kernel rounds x*id with trunc(x + copysign(nextbelow(0.5), x)) instead of roundf; the two agree
    for every float of magnitude below 2^23.  Checked here on every tie k + 0.5, its two float neighbours, and a dense
    stride through all floats in [0, 256) (the quantiser's products stay within +-127.5)."""
    c = np.nextafter(np.float32(0.5), np.float32(0))
    assert c == np.float32(0.49999997)
    ties = np.arange(0, 4096, dtype=np.float32) + np.float32(0.5)
    cand = np.concatenate([ties, np.nextafter(ties, np.float32(0)), np.nextafter(ties, np.float32(1e9)),
                           np.arange(0, 0x43800000, 37, dtype=np.uint32).view(np.float32)])
    for x in (cand, -cand):
        fast = np.trunc(x + np.copysign(c, x))                                   # float32 add, round to nearest even
        exact = np.copysign(np.floor(np.abs(x).astype(np.float64) + 0.5), x)     # roundf
        assert np.array_equal(fast.astype(np.float64), exact)


def test_q4_0_known_answer_block():
    """Hand-packed block: d = 0.5, byte j = (j) | ((15 - j) << 4): element j is (j - 8) / 2, element j + 16 is
    (7 - j) / 2.  A swap of the nibbles, of the halves, or a missing -8 fails this."""
    blk = np.zeros(18, np.uint8)
    blk[:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    j = np.arange(16)
    blk[2:] = j | ((15 - j) << 4)
    y = oracle.dequantize(oracle.Q4_0, blk, 32)
    assert np.array_equal(y[:16], (j - 8) * 0.5)
    assert np.array_equal(y[16:], (7 - j) * 0.5)
    assert oracle.row_bytes(oracle.Q4_0, 128) == 72


def test_q4_0_quantise_invariants_and_numpy_restatement():
    rng = np.random.default_rng(404)
    x = rng.standard_normal((4000, 32)).astype(np.float32)
    x[0] = 0.0                                   # all-zero block: d = 0 / -8 = -0.0, every nibble 8
    x[1, 3], x[1, 20] = 5.0, -5.0                # tie in magnitude: the first element (positive) decides the sign of d
    x[1, [i for i in range(32) if i not in (3, 20)]] *= 0.1
    x[2, 7], x[2, 2] = -6.0, 6.0                 # tie the other way round: index 2 (positive) comes first
    x[2, [i for i in range(32) if i not in (2, 7)]] *= 0.1
    x[3] *= 1e-6                                 # small values: d is an fp16 subnormal
    packed = oracle.quantize_q4_0(x).reshape(-1, 18)
    # independent float32 restatement in numpy
    idx = np.argmax(np.abs(x), axis=1)           # argmax returns the first maximum
    mx = x[np.arange(len(x)), idx]
    d = (mx / np.float32(-8.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        idv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
    q = np.minimum(15, np.trunc((x * idv[:, None]).astype(np.float32) + np.float32(8.5)).astype(np.int32))
    want = (q[:, :16] | (q[:, 16:] << 4)).astype(np.uint8)
    assert np.array_equal(packed[:, 2:], want)
    assert np.array_equal(packed[:, :2].copy().view(np.float16)[:, 0], d.astype(np.float16))
    assert np.all(packed[0] == np.r_[np.array([0x00, 0x80], np.uint8), np.full(16, 0x88, np.uint8)])
    assert d[1] < 0 and d[2] < 0                 # the first of the tied elements is the positive one in both rows
    # the element of largest magnitude is reproduced as -8 * d; everything else within one step
    y = oracle.dequantize(oracle.Q4_0, packed.reshape(-1), x.size).reshape(x.shape)
    dh = d.astype(np.float16).astype(np.float32)
    assert np.array_equal(y[np.arange(len(x)), idx], np.float32(-8) * dh)
    assert np.all(np.abs(y - x) <= np.abs(dh)[:, None] * 1.001 + np.abs(x) * 2.0 ** -10)


def test_kv_round_is_quantise_then_dequantise():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, 2, 64)).astype(np.float32)
    assert np.array_equal(oracle.kv_round(oracle.F16, x), x.astype(np.float16).astype(np.float32))
    r8 = oracle.kv_round(oracle.Q8_0, x)
    assert r8.shape == x.shape and np.array_equal(r8.reshape(-1), oracle.dequantize(oracle.Q8_0, oracle.quantize_q8_0(x), x.size))
    r4 = oracle.kv_round(oracle.Q4_0, x)
    assert np.abs(r4 - x).max() < 0.5 and np.abs(r8 - x).max() < 0.03
