"""Pins the oracle's data-type conversions (oracle/oracle_dtypes.h) and the
product's numpy helpers (onednn_amd/dtypes.py).

Sources of truth, none of which is this repository's conversion code:
  * the reference's own known-answer tests, restated:
      tests/gtests/internals/test_float8.cpp:34-90   all 256 f8 codes survive
                                                     f8 -> f32 -> f8 (sNaN gets
                                                     its quiet bit)
      tests/gtests/internals/test_float8.cpp:152-180 f32 -> e4m3 equals
                                                     f32 -> f16 -> e4m3
      tests/gtests/internals/test_nibble.cpp:36-88   4-bit limits, low nibble =
                                                     even index, byte round trip
  * the OCP formats themselves: value of a code computed from its fields with
    exact rationals, and "nearest code, ties to the even code" found by brute
    force over the whole code table;
  * numpy's IEEE float16 as an independent f32 -> f16 rounding.
"""
from fractions import Fraction

import numpy as np
import pytest

from onednn_amd import cabi
from onednn_amd import dtypes as dtp


def e4m3_value(code):
    s, e, m = code >> 7, (code >> 3) & 0xF, code & 7
    if e == 0xF and m == 7:
        return None  # NaN
    v = Fraction(m, 8) * Fraction(2) ** (1 - 7) if e == 0 else (1 + Fraction(m, 8)) * Fraction(2) ** (e - 7)
    return -v if s else v


def e5m2_value(code):
    s, e, m = code >> 7, (code >> 2) & 0x1F, code & 3
    if e == 0x1F:
        return None  # inf / NaN
    v = Fraction(m, 4) * Fraction(2) ** (1 - 15) if e == 0 else (1 + Fraction(m, 4)) * Fraction(2) ** (e - 15)
    return -v if s else v


def f16_value(h):
    s, e, m = h >> 15, (h >> 10) & 0x1F, h & 0x3FF
    if e == 0x1F:
        return None
    v = Fraction(m, 1024) * Fraction(2) ** (-14) if e == 0 else (1 + Fraction(m, 1024)) * Fraction(2) ** (e - 15)
    return -v if s else v


def nearest_code(x, table):
    """table: list of (code, Fraction) for non-negative finite codes, sorted by
    value.  Ties go to the even code."""
    best, bestd = None, None
    for code, v in table:
        d = abs(v - x)
        if bestd is None or d < bestd or (d == bestd and code % 2 == 0):
            best, bestd = code, d
    return best


def test_e4m3_decode_matches_ocp_fields(oracle):
    codes = np.arange(256, dtype=np.uint8)
    got = oracle.e4m3_to_f32(codes)
    for c in range(256):
        v = e4m3_value(c)
        if v is None:
            assert np.isnan(got[c])
        else:
            assert Fraction(float(got[c])) == v, c
    # numpy helper agrees bit for bit (NaN payload aside)
    mine = dtp.e4m3_to_f32(codes)
    ok = (mine.view(np.uint32) == got.view(np.uint32)) | (np.isnan(mine) & np.isnan(got))
    assert ok.all()


def test_e4m3_all_codes_round_trip(oracle):
    # test_float8.cpp:57-90
    codes = np.arange(256, dtype=np.uint8)
    back = oracle.f32_to_e4m3(oracle.e4m3_to_f32(codes))
    assert np.array_equal(back, codes)


def test_e5m2_all_codes_round_trip_with_quieted_snan(oracle):
    # test_float8.cpp:34-55: 0x7d -> 0x7f and 0xfd -> 0xff, everything else exact
    codes = np.arange(256, dtype=np.uint8)
    back = oracle.f32_to_e5m2(oracle.e5m2_to_f32(codes))
    expect = codes.copy()
    expect[0x7D] = 0x7F
    expect[0xFD] = 0xFF
    assert np.array_equal(back, expect)


def test_f16_to_e4m3_is_nearest_even_over_all_f16(oracle):
    table = sorted(((c, e4m3_value(c)) for c in range(0x7F)), key=lambda t: t[1])
    h = np.arange(0x8000, dtype=np.uint16)
    got = oracle.f16_to_e4m3(h)
    mine = dtp.f16_bits_to_e4m3(h)
    assert np.array_equal(got, mine)
    # brute force on every 7th input plus every input near a rounding boundary
    check = set(range(0, 0x8000, 7))
    for c in range(0x7F):
        f = float(e4m3_value(c))
        hb = int(np.float16(f).view(np.uint16))
        check.update(range(max(hb - 70, 0), min(hb + 70, 0x7C00)))
    for hb in sorted(check):
        x = f16_value(hb)
        if x is None or hb > 0x5F40:          # > 464, inf, NaN -> NaN code
            assert got[hb] == 0x7F, hex(hb)
        else:
            assert got[hb] == nearest_code(x, table), hex(hb)
    # sign is carried, -0 stays -0
    neg = oracle.f16_to_e4m3((h | 0x8000).astype(np.uint16))
    assert np.array_equal(neg, got | 0x80)
    # the reference's two explicit cut-offs (float8.cpp:229-238)
    assert got[0x5F40] == 0x7E and got[0x5F41] == 0x7F      # 464 -> 448, above -> NaN
    assert got[0x1400] == 0x00 and got[0x1401] == 0x01      # 2^-10 -> 0, above -> 2^-9


def test_f16_to_e5m2_is_nearest_even_over_all_f16(oracle):
    h = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    got = oracle.f16_to_e5m2(h)
    table = sorted(((c, e5m2_value(c)) for c in range(0x7C)), key=lambda t: t[1])
    for hb in list(range(0, 0x7C00, 13)) + [0x7BFF, 0x7BE0, 0x7BDF, 0x0001, 0x0080, 0x0081]:
        x = f16_value(hb)
        want = nearest_code(x, table)
        # a value that rounds beyond the largest finite code becomes inf (0x7c)
        if x > e5m2_value(0x7B) + (e5m2_value(0x7B) - e5m2_value(0x7A)) / 2 or (
                x == e5m2_value(0x7B) + (e5m2_value(0x7B) - e5m2_value(0x7A)) / 2):
            want = 0x7C
        assert got[hb] == want, hex(hb)
    assert got[0x7C00] == 0x7C and got[0xFC00] == 0xFC           # inf
    assert got[0x7C01] == 0x7E and got[0x7E00] == 0x7E           # NaN -> quiet


def test_f32_to_f16_matches_ieee(oracle):
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 2 ** 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    # all exponents around the f16 range, ties and boundaries
    special = []
    for e in range(90, 146):
        for m in (0, 1, 0xFFF, 0x1000, 0x1001, 0x2FFF, 0x3000, 0x7FFFFF, 0x7FF000, 0x7FEFFF):
            special.append((e << 23) | m)
    bits = np.concatenate([bits, np.array(special, dtype=np.uint32)])
    bits = np.concatenate([bits, bits | np.uint32(0x80000000)])
    x = bits.view(np.float32)
    got = oracle.f32_to_f16(x)
    with np.errstate(over="ignore", invalid="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    # f32 subnormals flush to zero in the reference (float16.hpp:67-70); IEEE gives 0 too
    assert np.array_equal(got[~nan], want[~nan])
    assert ((got[nan] & 0x7C00) == 0x7C00).all() and ((got[nan] & 0x3FF) != 0).all()
    back = oracle.f16_to_f32(np.arange(0x10000, dtype=np.uint32).astype(np.uint16))
    ieee = np.arange(0x10000, dtype=np.uint32).astype(np.uint16).view(np.float16).astype(np.float32)
    fin = ~np.isnan(ieee)
    assert np.array_equal(back[fin].view(np.uint32), ieee[fin].view(np.uint32))


def test_f32_to_e4m3_equals_f32_to_f16_to_e4m3(oracle):
    # test_float8.cpp:152-180, on a sweep of all exponents instead of all 2^32
    rng = np.random.default_rng(11)
    bits = rng.integers(0, 2 ** 32, size=1_000_000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    a = oracle.f32_to_e4m3(x)
    b = oracle.f16_to_e4m3(oracle.f32_to_f16(x))
    assert np.array_equal(a, b)
    assert np.array_equal(dtp.f32_to_e4m3(x), a)


def test_bf16_rne_flush_and_nan(oracle):
    rng = np.random.default_rng(3)
    bits = rng.integers(0, 2 ** 32, size=1_000_000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    got = oracle.f32_to_bf16(x)
    assert np.array_equal(got, dtp.f32_to_bf16(x))
    # independent: pick the nearer of the two neighbouring bf16 values in f64
    lo = (bits & 0xFFFF0000).view(np.float32).astype(np.float64)
    hi_bits = ((bits >> 16) + 1).astype(np.uint32) << 16
    hi = hi_bits.view(np.float32).astype(np.float64)
    xv = x.astype(np.float64)
    expo = (bits >> 23) & 0xFF
    normal = (expo != 0) & (expo != 0xFF) & (((bits >> 16) & 0x7FFF) != 0x7F7F)
    dl, dh = np.abs(xv - lo), np.abs(hi - xv)
    pick_hi = (dh < dl) | ((dh == dl) & (((bits >> 16) & 1) == 1))
    want = np.where(pick_hi, hi_bits >> 16, bits >> 16).astype(np.uint16)
    assert np.array_equal(got[normal], want[normal])
    # subnormal f32 -> signed zero (bfloat16.cpp:29-34); NaN keeps sign, quiet bit set
    sub = np.array([0x00000001, 0x007FFFFF, 0x80000001, 0x807FFFFF], dtype=np.uint32).view(np.float32)
    assert list(oracle.f32_to_bf16(sub)) == [0x0000, 0x0000, 0x8000, 0x8000]
    nan = np.array([0x7F800001, 0xFFC12345], dtype=np.uint32).view(np.float32)
    assert list(oracle.f32_to_bf16(nan)) == [0x7FC0, 0xFFC1]
    inf = np.array([0x7F800000, 0xFF800000], dtype=np.uint32).view(np.float32)
    assert list(oracle.f32_to_bf16(inf)) == [0x7F80, 0xFF80]
    # rounding that carries into the exponent, and overflow to inf
    edge = np.array([0x3F7FFFFF, 0x7F7FFFFF], dtype=np.uint32).view(np.float32)
    assert list(oracle.f32_to_bf16(edge)) == [0x3F80, 0x7F80]


def test_e8m0(oracle):
    # float8.cpp:29-45: store keeps the exponent byte (truncation), 0xff -> NaN,
    # 0x00 -> 2^-127
    v = oracle.e8m0_to_f32(np.arange(256, dtype=np.uint8))
    assert np.isnan(v[255])
    assert v[0] == np.float32(2.0) ** -127
    for b in range(1, 255):
        assert v[b] == np.ldexp(np.float32(1), b - 127)
    x = np.array([1.0, 1.99, 2.0, 0.75, 1e-40, 3.0e38], dtype=np.float32)
    assert list(oracle.f32_to_e8m0(x)) == [127, 127, 128, 126, 0, 254]
    assert np.array_equal(dtp.e8m0_to_f32(np.arange(255, dtype=np.uint8)), v[:255])


def test_e2m1_table_round_trip_and_nearest(oracle):
    table = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]  # float4.cpp:80-82
    packed = np.array([(hi << 4) | lo for hi in range(16) for lo in range(16)], dtype=np.uint8)
    vals = oracle.nibbles_to_f32("oracle_e2m1_to_f32", packed, 512)
    for i in range(256):
        lo, hi = i % 16, i // 16
        assert vals[2 * i] == (-1 if lo & 8 else 1) * table[lo & 7]      # even index = low nibble
        assert vals[2 * i + 1] == (-1 if hi & 8 else 1) * table[hi & 7]
    # exhaustive byte round trip (test_nibble.cpp:52-88)
    assert np.array_equal(oracle.f32_to_e2m1_packed(vals), packed)
    # nearest with ties to the even code; saturation at 6; NaN/Inf -> +-6
    xs = np.concatenate([np.linspace(-8, 8, 6401), np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])])
    xs = xs.astype(np.float32)
    got = dtp.unpack_nibbles(oracle.f32_to_e2m1_packed(xs), xs.size)
    for x, c in zip(xs, got):
        a = min(abs(float(x)), 6.0)
        d = [abs(t - a) for t in table]
        best = min(range(8), key=lambda i: (d[i], i % 2))
        assert (c & 7) == best and (c >> 3) == (1 if np.signbit(x) else 0), (x, c)
    sp = np.array([np.nan, np.inf, -np.inf], dtype=np.float32)
    assert list(dtp.unpack_nibbles(oracle.f32_to_e2m1_packed(sp), 3) & 7) == [7, 7, 7]
    assert np.array_equal(dtp.f32_to_e2m1_codes(xs), got)


def test_int4_limits_and_order(oracle):
    # test_nibble.cpp:36-46: s4 in [-8, 7], u4 in [0, 15]
    packed = np.arange(256, dtype=np.uint8)
    s = oracle.nibbles_to_f32("oracle_s4_to_f32", packed, 512)
    u = oracle.nibbles_to_f32("oracle_u4_to_f32", packed, 512)
    assert s.min() == -8 and s.max() == 7 and u.min() == 0 and u.max() == 15
    for b in (0x00, 0x0F, 0xF0, 0x7A, 0x80):
        lo, hi = b & 0xF, b >> 4
        assert u[2 * b] == lo and u[2 * b + 1] == hi
        assert s[2 * b] == (lo - 16 if lo & 8 else lo) and s[2 * b + 1] == (hi - 16 if hi & 8 else hi)
    assert np.array_equal(dtp.unpack_nibbles(packed, 512).astype(np.float32), u)
    assert np.array_equal(dtp.pack_nibbles(dtp.unpack_nibbles(packed, 512)), packed)


def test_integer_store_saturates_then_rounds_to_even(oracle):
    # simple_q10n.hpp:41-81 and the s32 bound of type_helpers.hpp:232
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, 128.4, -128.5, -129.0, 1e9, -1e9,
                  254.5, 255.5, 300.0, -3.0], dtype=np.float32)
    s8 = oracle.store_float(cabi.DT_S8, x)
    assert list(s8) == [0, 2, 2, 0, -2, -2, 126, 127, 127, -128, -128, 127, -128, 127, 127, 127, -3]
    u8 = oracle.store_float(cabi.DT_U8, x)
    assert list(u8) == [0, 2, 2, 0, 0, 0, 126, 128, 128, 0, 0, 255, 0, 254, 255, 255, 0]
    big = np.array([2147483520.0, 2147483648.0, 4e9, -2147483648.0, -4e9, 16777217.0], dtype=np.float32)
    s32 = oracle.store_float(cabi.DT_S32, big)
    assert list(s32) == [2147483520, 2147483520, 2147483520, -2147483648, -2147483648, 16777216]


@pytest.mark.parametrize("dt", [cabi.DT_F32, cabi.DT_BF16, cabi.DT_F16, cabi.DT_F8_E4M3,
                                cabi.DT_F8_E5M2, cabi.DT_S8, cabi.DT_U8, cabi.DT_S32])
def test_store_then_load_is_idempotent(oracle, dt):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(4096) * 50).astype(np.float32)
    raw = oracle.store_float(dt, x)
    y = oracle.load_float(dt, raw, x.size)
    raw2 = oracle.store_float(dt, y)
    assert np.array_equal(raw.view(np.uint8), raw2.view(np.uint8))
