// Low-precision data types of the matmul path, usable from host and device.
//
// Bit-level contract (reference: uxlfoundation/oneDNN v3.14):
//   bf16     src/common/bfloat16.cpp:22-49  RNE, f32 subnormals flush to zero
//   f16      src/common/float16.hpp:50-135  RNE, f32 subnormals flush to zero
//   f8_e4m3  src/common/float8.cpp:216-281, :341-374  f32 -> f16 -> e4m3 (two
//            roundings), > 464 -> NaN (0x7f), <= 2^-10 -> 0
//   f8_e5m2  src/common/float8.cpp:47-75, :171-189    f16 with 8 bits dropped
//   e8m0     src/common/float8.cpp:29-45    0xff -> NaN, 0x00 -> 2^-127
//   f4_e2m1  src/common/float4.cpp:28-84    nearest of 8 magnitudes, ties to
//            the even code, NaN/Inf -> +-6
//   s4/u4    src/common/int4.hpp:28-70; even logical offset = low nibble
//            (src/common/nibble.hpp:33)
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define MI_HD __host__ __device__ __forceinline__
#else
#define MI_HD inline
#endif

namespace mi355 {

MI_HD uint32_t f2u(float f) {
    union { float f; uint32_t u; } x;
    x.f = f;
    return x.u;
}
MI_HD float u2f(uint32_t u) {
    union { float f; uint32_t u; } x;
    x.u = u;
    return x.f;
}

// ---- bf16
MI_HD uint16_t f32_to_bf16(float f) {
    const uint32_t u = f2u(f);
    const uint32_t e = (u >> 23) & 0xffu;
    if (e == 0) return (uint16_t)((u >> 16) & 0x8000u);
    if (e == 0xffu)
        return (u & 0x7fffffu) ? (uint16_t)((u >> 16) | 0x40u) : (uint16_t)(u >> 16);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
MI_HD float bf16_to_f32(uint16_t b) { return u2f((uint32_t)b << 16); }

// ---- f16
MI_HD uint16_t f32_to_f16(float f) {
    const uint32_t u = f2u(f);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const uint32_t e = (u >> 23) & 0xffu, man = u & 0x7fffffu;
    if (e == 0) return (uint16_t)sign;
    if (e == 0xffu) {
        uint32_t m16 = man >> 13;
        if (man) m16 |= 0x200u;
        return (uint16_t)(sign | 0x7c00u | m16);
    }
    const int e16 = (int)e - 112;
    if (e16 >= 0x1f) return (uint16_t)(sign | 0x7c00u);
    if (e16 > 0) {
        const uint32_t x = ((uint32_t)e16 << 23) | man;
        return (uint16_t)(sign | ((x + 0xfffu + ((x >> 13) & 1u)) >> 13));
    }
    const int shift = 14 - e16;
    if (shift > 25) return (uint16_t)sign;
    const uint32_t sig = man | 0x800000u;
    uint32_t q = sig >> shift;
    const uint32_t rem = sig & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}
MI_HD float f16_to_f32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0) {
        // m * 2^-24, exact
        const float v = (float)m * 5.9604644775390625e-08f;
        return u2f(f2u(v) | sign);
    }
    if (e == 0x1fu) {
        uint32_t mm = m << 13;
        if (mm) mm |= 0x400000u;
        return u2f(sign | 0x7f800000u | mm);
    }
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

// ---- f8_e4m3
MI_HD uint8_t f16_to_e4m3(uint16_t h) {
    const uint8_t s8 = (uint8_t)((h & 0x8000u) >> 8);
    const uint32_t a = h & 0x7fffu;
    if (a > 0x5f40u) return s8 | 0x7f;
    if (a <= 0x1400u) return s8;
    const uint32_t e16 = a >> 10;
    if (e16 >= 9) {
        const uint32_t x = a - (8u << 10);
        return s8 | (uint8_t)((x + 0x3fu + ((x >> 7) & 1u)) >> 7);
    }
    const uint32_t sig = 1024u + (a & 0x3ffu);
    const uint32_t shift = 16u - e16;
    uint32_t q = sig >> shift;
    const uint32_t rem = sig & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return s8 | (uint8_t)q;
}
MI_HD uint8_t f32_to_e4m3(float f) { return f16_to_e4m3(f32_to_f16(f)); }
MI_HD float e4m3_to_f32(uint8_t b) {
    const uint32_t sign = ((uint32_t)b & 0x80u) << 24;
    const uint32_t e = (b >> 3) & 0xfu, m = b & 7u;
    if (e == 0xfu && m == 7u) return u2f(sign | 0x7fc00000u);
    if (e == 0) return u2f(f2u((float)m * 0.001953125f) | sign); // m * 2^-9
    return u2f(sign | ((e + 120u) << 23) | (m << 20));
}

// ---- f8_e5m2
MI_HD uint8_t f16_to_e5m2(uint16_t h) {
    const uint32_t a = h;
    if ((a & 0x7c00u) == 0x7c00u)
        return (a & 0x3ffu) ? (uint8_t)((a >> 8) | 0x02u) : (uint8_t)(a >> 8);
    return (uint8_t)((a + 0x7fu + ((a >> 8) & 1u)) >> 8);
}
MI_HD uint8_t f32_to_e5m2(float f) { return f16_to_e5m2(f32_to_f16(f)); }
MI_HD float e5m2_to_f32(uint8_t b) {
    const uint8_t r = ((b & 0x7d) == 0x7d) ? (uint8_t)(b | 0x02) : b;
    return f16_to_f32((uint16_t)((uint16_t)r << 8));
}

// ---- e8m0
MI_HD uint8_t f32_to_e8m0(float f) { return (uint8_t)((f2u(f) >> 23) & 0xffu); }
MI_HD float e8m0_to_f32(uint8_t b) {
    if (b == 0xffu) return u2f(0xffc00000u);
    if (b == 0x00u) return u2f(0x00400000u);
    return u2f((uint32_t)b << 23);
}

// ---- f4_e2m1
MI_HD float e2m1_to_f32(uint8_t nib) {
    // magnitudes 0, .5, 1, 1.5, 2, 3, 4, 6 as f32 bit patterns
    const uint32_t c = nib & 7u;
    uint32_t bits;
    if (c == 0) bits = 0;
    else if (c == 1) bits = 0x3f000000u;
    else bits = ((126u + (c >> 1)) << 23) | ((c & 1u) << 22);
    return u2f(bits | (((uint32_t)nib & 8u) << 28));
}
MI_HD uint8_t f32_to_e2m1(float f) {
    const uint32_t u = f2u(f);
    const uint8_t s = (uint8_t)((u >> 28) & 0x8u);
    if ((u & 0x7f800000u) == 0x7f800000u) return s | 0x7;
    float a = u2f(u & 0x7fffffffu);
    if (a > 6.0f) a = 6.0f;
    // thresholds are the midpoints; a tie goes to the even code
    uint8_t c;
    if (a <= 0.25f) c = 0;
    else if (a < 0.75f) c = 1;
    else if (a <= 1.25f) c = 2;
    else if (a < 1.75f) c = 3;
    else if (a <= 2.5f) c = 4;
    else if (a < 3.5f) c = 5;
    else if (a <= 5.0f) c = 6;
    else c = 7;
    return s | c;
}

// ---- 4-bit packing
MI_HD uint8_t nibble_get(const void *p, int64_t off) {
    const uint8_t byte = ((const uint8_t *)p)[off >> 1];
    return (off & 1) ? (uint8_t)(byte >> 4) : (uint8_t)(byte & 0xf);
}
MI_HD int s4_to_int(uint8_t nib) { return (nib & 8) ? (int)nib - 16 : (int)nib; }

} // namespace mi355
