/* Host check of the fma-corrected division the MFMA epilogue uses for integer dst
 * types (onednn_amd/csrc/tile_epilogue.hpp, div_by_fma): for a given divisor s
 * and every float x the device path admits (|x| < 2^100),
 *     q0 = x*y; r0 = fma(-s,q0,x); q1 = fma(r0,y,q0); r1 = fma(-s,q1,x); q = fma(r1,y,q1)
 * with y = 1/s must equal the IEEE quotient x / s bit for bit when
 * 2^-90 <= |x| < 2^100, and must stay below 2^-60 in magnitude, like the IEEE
 * quotient, for smaller |x| (zero and subnormals included): such a quotient
 * vanishes in the rounding to an integer dst that follows.
 *   usage: div_by_fma_check exhaustive <s as hex bits>   -> all admitted x
 *          div_by_fma_check sample <count s> <count x>   -> random s in [2^-20, 2^20], random x
 * prints the number of mismatches; exit status 0 iff none. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float div_by_fma(float x, float s, float y) {
    const float q0 = x * y;
    const float r0 = fmaf(-s, q0, x);
    const float q1 = fmaf(r0, y, q0);
    const float r1 = fmaf(-s, q1, x);
    return fmaf(r1, y, q1);
}

static inline int admitted(float x) { return (f2u(x) & 0x7fffffffu) < 0x71800000u; /* |x| < 2^100 */ }

/* the property the device relies on */
static inline int agrees(float x, float a, float b) {
    if (fabsf(x) >= 0x1p-90f) return f2u(a) == f2u(b);
    return fabsf(a) < 0x1p-60f && fabsf(b) < 0x1p-60f;
}

static long check_all_x(float s) {
    const float y = 1.f / s;
    long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
    for (int64_t u = 0; u < (1LL << 32); ++u) {
        const float x = u2f((uint32_t)u);
        if (!admitted(x)) continue;
        /* below 2^-90 the claim is a magnitude bound only: every 1021st pattern */
        if (fabsf(x) < 0x1p-90f && u % 1021 != 0) continue;
        const float a = div_by_fma(x, s, y), b = x / s;
        if (!agrees(x, a, b)) ++bad;
    }
    return bad;
}

static uint64_t rng_state = 0x9e3779b97f4a7c15ull;
static uint32_t rng(void) {
    rng_state ^= rng_state << 13; rng_state ^= rng_state >> 7; rng_state ^= rng_state << 17;
    return (uint32_t)(rng_state >> 16);
}

int main(int argc, char **argv) {
    long bad = 0;
    if (argc >= 3 && !strcmp(argv[1], "exhaustive")) {
        const float s = u2f((uint32_t)strtoul(argv[2], NULL, 16));
        bad = check_all_x(s);
    } else if (argc >= 4 && !strcmp(argv[1], "sample")) {
        const long ns = atol(argv[2]), nx = atol(argv[3]);
        for (long i = 0; i < ns; ++i) {
            /* sign, exponent in [127-20, 127+20], random mantissa; every 8th with an extreme mantissa */
            uint32_t m = rng() & 0x7fffffu;
            if (i % 8 == 0) m = 0x7fffffu;
            if (i % 8 == 1) m = 0;
            if (i % 8 == 2) m = 0x7ffffeu;
            if (i % 8 == 3) m = 1;
            const uint32_t e = 127 - 20 + rng() % 41;
            const float s = u2f(((rng() & 1u) << 31) | (e << 23) | m);
            const float y = 1.f / s;
            for (long j = 0; j < nx; ++j) {
                const float x = u2f(rng());
                if (!admitted(x)) continue;
                const float a = div_by_fma(x, s, y), b = x / s;
                if (!agrees(x, a, b)) {
                    if (bad < 5) fprintf(stderr, "x=%a s=%a fma=%a div=%a\n", x, s, a, b);
                    ++bad;
                }
            }
        }
    } else {
        fprintf(stderr, "usage: %s exhaustive <hex s> | sample <ns> <nx>\n", argv[0]);
        return 2;
    }
    printf("%ld\n", bad);
    return bad != 0;
}
