// Calibration tool: the hardware conversions the GEMM tile epilogue uses for an
// fp8 dst (v_cvt_f16_f32, then v_cvt_scalef32_pk_{fp8,bf8}_f16 with scale 1)
// against the software conversions that restate the reference
// (src/common/float8.cpp:47-126, :216-281; float16.hpp), for every f16 bit
// pattern and 4 M f32 bit patterns.  Prints the mismatch counts and, as the
// last line, "nan-only" when every mismatch has a NaN input.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
#include "mi355_dtypes.hpp"
using namespace mi355;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef short s2 __attribute__((ext_vector_type(2)));
__global__ void probe(unsigned *out) {
    const unsigned h = blockIdx.x * 256 + threadIdx.x; // all 65536 f16 patterns
    const uint16_t hb = (uint16_t)h;
    h2 src; src[0] = __builtin_bit_cast(_Float16, hb); src[1] = __builtin_bit_cast(_Float16, hb);
    s2 old = {0, 0};
    s2 r8 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(old, src, 1.0f, false);
    s2 r5 = __builtin_amdgcn_cvt_scalef32_pk_bf8_f16(old, src, 1.0f, false);
    const unsigned hw8 = (unsigned)r8[0] & 0xff, hw5 = (unsigned)r5[0] & 0xff;
    const unsigned sw8 = f16_to_e4m3(hb), sw5 = f16_to_e5m2(hb);
    out[h] = hw8 | (sw8 << 8) | (hw5 << 16) | (sw5 << 24);
}
__global__ void probe32(const float *in, unsigned *out, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float v = in[i];
    const uint16_t hw = __builtin_bit_cast(uint16_t, (_Float16)v);
    out[i] = hw | ((unsigned)f32_to_f16(v) << 16);
}
int main() {
    unsigned *d; hipMalloc(&d, 65536 * 4);
    probe<<<256, 256>>>(d);
    static unsigned h[65536]; hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost);
    int bad8 = 0, bad5 = 0, shown = 0, other = 0;
    for (int i = 0; i < 65536; ++i) {
        unsigned hw8 = h[i] & 0xff, sw8 = (h[i] >> 8) & 0xff, hw5 = (h[i] >> 16) & 0xff, sw5 = h[i] >> 24;
        const bool nan = (i & 0x7c00) == 0x7c00 && (i & 0x3ff);
        if (hw8 != sw8) { bad8++; other += !nan; if (!nan && shown < 12) { printf("e4m3 h=%04x hw=%02x sw=%02x\n", i, hw8, sw8); shown++; } }
        if (hw5 != sw5) { bad5++; other += !nan; if (!nan && shown < 24) { printf("e5m2 h=%04x hw=%02x sw=%02x\n", i, hw5, sw5); shown++; } }
    }
    printf("f16->e4m3 mismatches %d, f16->e5m2 mismatches %d of 65536\n", bad8, bad5);
    // f32 -> f16: random bit patterns plus every exponent with special mantissas
    const int n = 1 << 22; float *in; unsigned *o2; hipMalloc(&in, n * 4); hipMalloc(&o2, n * 4);
    static unsigned bits[1 << 22]; unsigned x = 12345;
    for (int i = 0; i < n; ++i) { x = x * 1664525u + 1013904223u; bits[i] = x; }
    for (int e = 0; e < 256; ++e) for (int s = 0; s < 2; ++s) { unsigned m[8] = {0, 1, 0x1000, 0x0fff, 0x1001, 0x3000, 0x7fffff, 0x400000};
        for (int k = 0; k < 8; ++k) bits[(e * 2 + s) * 8 + k] = ((unsigned)s << 31) | ((unsigned)e << 23) | m[k]; }
    hipMemcpy(in, bits, n * 4, hipMemcpyHostToDevice);
    probe32<<<n / 256, 256>>>(in, o2, n);
    static unsigned r[1 << 22]; hipMemcpy(r, o2, n * 4, hipMemcpyDeviceToHost);
    int bad = 0, badnan = 0; shown = 0;
    for (int i = 0; i < n; ++i) if ((r[i] & 0xffff) != (r[i] >> 16)) {
        const bool nan = ((bits[i] >> 23) & 0xff) == 0xff && (bits[i] & 0x7fffff);
        if (nan) badnan++; else { bad++; if (shown++ < 10) printf("f32 %08x hw=%04x sw=%04x\n", bits[i], r[i] & 0xffff, r[i] >> 16); }
    }
    printf("f32->f16 mismatches: %d non-NaN, %d NaN of %d\n", bad, badnan, n);
    printf("%s\n", other == 0 && bad == 0 ? "nan-only" : "differs");
    return 0;
}
