/*
 * TEST INFRASTRUCTURE -- CPU oracle, not part of the shipped library.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may use
 * anything in this directory.
 *
 * Software low-precision data types: a restatement of the conversion contract
 * of the reference (uxlfoundation/oneDNN v3.14):
 *   bf16      src/common/bfloat16.cpp:22-49   (RNE; f32 subnormals flush to 0;
 *                                              NaN keeps sign, quiet bit set)
 *   f16       src/common/float16.hpp:50-135   (RNE; f32 subnormals -> 0)
 *   f8_e4m3   src/common/float8.cpp:216-274 (from f16), :276-281 (from f32,
 *             i.e. f32 -> f16 -> e4m3: two roundings), :341-374 (to f16)
 *   f8_e5m2   src/common/float8.cpp:47-75 (from f16), :171-189 (to f16)
 *   e8m0      src/common/float8.cpp:29-45   (store = exponent byte, truncation;
 *                                            0xff -> NaN, 0x00 -> 2^-127)
 *   f4_e2m1   src/common/float4.cpp:28-60, :78-84 (nearest of 8 magnitudes,
 *             ties to even code; NaN/Inf -> +-6)
 *   s4 / u4   src/common/int4.hpp:28-70; nibble order src/common/nibble.hpp:33
 *             (element with even logical offset sits in the LOW nibble)
 *
 * Pinning (tests/test_oracle_dtypes.py): exhaustive code round trips restated
 * from tests/gtests/internals/test_float8.cpp:34-150 and test_nibble.cpp:36-88,
 * the f32->f16->e4m3 double-rounding identity of test_float8.cpp:152-180 on a
 * strided sweep of all exponents, and -- independent of this file's formulas --
 * a brute-force "nearest code in the OCP value table, ties to even" search in
 * exact rational arithmetic over every f16 input.
 */
#ifndef ORACLE_DTYPES_H
#define ORACLE_DTYPES_H

#include <math.h>
#include <stdint.h>
#include <string.h>

static inline uint32_t orc_f2u(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float orc_u2f(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* ---- bf16 ---- */
static inline uint16_t orc_f32_to_bf16(float f) {
    uint32_t u = orc_f2u(f);
    uint32_t expo = (u >> 23) & 0xff, man = u & 0x7fffff;
    if (expo == 0) return (uint16_t)((u >> 16) & 0x8000); /* zero, subnormal */
    if (expo == 0xff) {
        if (man == 0) return (uint16_t)(u >> 16);        /* inf */
        return (uint16_t)((u >> 16) | 0x40);             /* quiet NaN */
    }
    uint32_t lsb = (u >> 16) & 1u;
    return (uint16_t)((u + 0x7fffu + lsb) >> 16);
}
static inline float orc_bf16_to_f32(uint16_t b) {
    return orc_u2f((uint32_t)b << 16);
}

/* ---- f16 ---- */
static inline uint16_t orc_f32_to_f16(float f) {
    uint32_t u = orc_f2u(f);
    uint32_t sign = (u >> 16) & 0x8000;
    uint32_t expo = (u >> 23) & 0xff, man = u & 0x7fffff;
    if (expo == 0) return (uint16_t)sign; /* f32 zero / subnormal -> 0 */
    if (expo == 0xff) {
        uint32_t m16 = man >> 13;
        if (man) m16 |= 0x200;
        return (uint16_t)(sign | 0x7c00 | m16);
    }
    int e16 = (int)expo - 127 + 15;
    if (e16 >= 0x1f) return (uint16_t)(sign | 0x7c00); /* overflow -> inf */
    if (e16 > 0) {
        /* normal: round the 23-bit mantissa to 10 bits, nearest even; a carry
         * runs into the exponent field, possibly up to inf */
        uint32_t x = ((uint32_t)e16 << 23) | man;
        uint32_t lsb = (x >> 13) & 1u;
        return (uint16_t)(sign | ((x + 0xfffu + lsb) >> 13));
    }
    /* result is an f16 subnormal (or 0): value / 2^-24 rounded to nearest
     * even integer, computed exactly on the 24-bit significand */
    int shift = 14 - e16; /* >= 14 */
    if (shift > 25) return (uint16_t)sign;
    uint32_t sig = man | 0x800000;
    uint32_t q = sig >> shift;
    uint32_t rem = sig & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}
static inline float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000) << 16;
    uint32_t e = (h >> 10) & 0x1f, m = h & 0x3ff;
    if (e == 0) {
        float v = ldexpf((float)m, -24);
        return sign ? -v : v;
    }
    if (e == 0x1f) {
        uint32_t mm = m << 13;
        if (mm) mm |= 0x400000;
        return orc_u2f(sign | 0x7f800000u | mm);
    }
    return orc_u2f(sign | ((e + 112) << 23) | (m << 13));
}

/* ---- f8_e4m3 (OCP: bias 7, no inf, NaN = S.1111.111, max 448) ---- */
static inline uint8_t orc_f16_to_e4m3(uint16_t h) {
    uint8_t s8 = (uint8_t)((h & 0x8000) >> 8);
    uint32_t a = h & 0x7fff;
    if (a > 0x5f40) return s8 | 0x7f; /* > 464, inf, NaN */
    if (a <= 0x1400) return s8;       /* <= 2^-10 */
    uint32_t e16 = a >> 10, m = a & 0x3ff;
    if (e16 >= 9) {
        /* e4m3-normal range: drop 7 mantissa bits, nearest even */
        uint32_t x = a - (8u << 10);
        uint32_t lsb = (x >> 7) & 1u;
        return s8 | (uint8_t)((x + 0x3fu + lsb) >> 7);
    }
    /* e4m3 subnormal: multiples of 2^-9 */
    uint32_t sig = 1024u + m;
    uint32_t shift = 16u - e16; /* 8..11 */
    uint32_t q = sig >> shift;
    uint32_t rem = sig & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return s8 | (uint8_t)q;
}
static inline uint8_t orc_f32_to_e4m3(float f) {
    return orc_f16_to_e4m3(orc_f32_to_f16(f));
}
static inline float orc_e4m3_to_f32(uint8_t b) {
    uint32_t e = (b >> 3) & 0xf, m = b & 7;
    float v;
    if (e == 0xf && m == 7)
        return orc_u2f(((uint32_t)(b & 0x80) << 24) | 0x7fc00000u);
    if (e == 0)
        v = ldexpf((float)m, -9);
    else
        v = ldexpf((float)(8 + m), (int)e - 10);
    return (b & 0x80) ? -v : v;
}

/* ---- f8_e5m2 (f16 with the low mantissa byte dropped) ---- */
static inline uint8_t orc_f16_to_e5m2(uint16_t h) {
    uint32_t a = h;
    if ((a & 0x7c00) == 0x7c00) {
        if (a & 0x3ff) return (uint8_t)((a >> 8) | 0x02); /* quiet NaN */
        return (uint8_t)(a >> 8);
    }
    uint32_t lsb = (a >> 8) & 1u;
    return (uint8_t)((a + 0x7fu + lsb) >> 8);
}
static inline uint8_t orc_f32_to_e5m2(float f) {
    return orc_f16_to_e5m2(orc_f32_to_f16(f));
}
static inline float orc_e5m2_to_f32(uint8_t b) {
    uint8_t r = ((b & 0x7d) == 0x7d) ? (uint8_t)(b | 0x02) : b; /* sNaN->qNaN */
    return orc_f16_to_f32((uint16_t)((uint16_t)r << 8));
}

/* ---- e8m0 ---- */
static inline uint8_t orc_f32_to_e8m0(float f) {
    return (uint8_t)((orc_f2u(f) >> 23) & 0xff);
}
static inline float orc_e8m0_to_f32(uint8_t b) {
    if (b == 0xff) return orc_u2f(0xffc00000u);
    if (b == 0x00) return orc_u2f(0x00400000u);
    return orc_u2f((uint32_t)b << 23);
}

/* ---- f4_e2m1 ---- */
static const float orc_e2m1_mag[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
static inline uint8_t orc_f32_to_e2m1(float f) {
    uint32_t u = orc_f2u(f);
    uint8_t s = (uint8_t)((u >> 28) & 0x8);
    if ((u & 0x7f800000u) == 0x7f800000u) return s | 0x7;
    float a = orc_u2f(u & 0x7fffffffu);
    if (a > 6.0f) a = 6.0f;
    /* nearest magnitude; a tie goes to the even code */
    uint8_t best = 0;
    float bestd = a; /* |0 - a| */
    for (uint8_t i = 1; i < 8; ++i) {
        float d = fabsf(orc_e2m1_mag[i] - a);
        if (d < bestd || (d == bestd && !(i & 1))) {
            bestd = d;
            best = i;
        }
    }
    return s | best;
}
static inline float orc_e2m1_to_f32(uint8_t b) {
    float v = orc_e2m1_mag[b & 7];
    return (b & 8) ? -v : v;
}

/* ---- 4-bit packing: even logical offset = low nibble ---- */
static inline uint8_t orc_nibble_get(const void *p, int64_t off) {
    uint8_t byte = ((const uint8_t *)p)[off / 2];
    return (off % 2) ? (uint8_t)(byte >> 4) : (uint8_t)(byte & 0xf);
}
static inline void orc_nibble_set(void *p, int64_t off, uint8_t v) {
    uint8_t *b = (uint8_t *)p + off / 2;
    if (off % 2)
        *b = (uint8_t)((*b & 0x0f) | (uint8_t)(v << 4));
    else
        *b = (uint8_t)((*b & 0xf0) | (v & 0xf));
}
static inline int orc_s4_to_int(uint8_t nib) {
    return (nib & 0x8) ? (int)nib - 16 : (int)nib;
}

#endif
