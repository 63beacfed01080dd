// Calibration tool: what the gfx950 MFMA instructions used by the GEMM kernels
// sustain on this machine when nothing else limits them (operands and
// accumulators stay in registers, 4 wavefronts per SIMD, 16 or 8 independent
// accumulator chains per wavefront).
//
//   mfma_peak            random operand bits (what real data looks like to the
//                        power manager)
//   mfma_peak constant   every operand byte 0x01 (lowest toggle rate)
//
// The difference between the two lines of each instruction is clock throttling
// under power, not issue rate: the kernels' rooflines are priced against the
// published peaks, this tool shows how much of the gap the instruction itself
// accounts for.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <string.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

enum { I8_32, I8_16, F8_32, F8_16, F4_32, F4_16 };

template <int MODE>
__global__ void __launch_bounds__(256) chain(int iters, int *out, const int *bits) {
    const v8i *r8 = (const v8i *)bits;
    const v8i a8 = r8[threadIdx.x * 2], b8 = r8[threadIdx.x * 2 + 1];
    const v4i a = {a8[0], a8[1], a8[2], a8[3]}, b = {b8[0], b8[1], b8[2], b8[3]};
    int result = 0;
    if (MODE == I8_32) {
        v16i c[8] = {};
        for (int i = 0; i < iters; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) c[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c[j], 0, 0, 0);
        for (int j = 0; j < 8; ++j) result += c[j][0];
    } else if (MODE == I8_16) {
        v4i c[16] = {};
        for (int i = 0; i < iters; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) c[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c[j], 0, 0, 0);
        for (int j = 0; j < 16; ++j) result += c[j][0];
    } else if (MODE == F8_32 || MODE == F4_32) {
        constexpr int fmt = MODE == F4_32 ? 4 : 0, sc = MODE == F4_32 ? 127 : 0;
        v16f c[8] = {};
        for (int i = 0; i < iters; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j)
                c[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, c[j], fmt, fmt, 0, sc, 0, sc);
        for (int j = 0; j < 8; ++j) result += (int)c[j][0];
    } else {
        constexpr int fmt = MODE == F4_16 ? 4 : 0, sc = MODE == F4_16 ? 127 : 0;
        v4f c[16] = {};
        for (int i = 0; i < iters; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j)
                c[j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, c[j], fmt, fmt, 0, sc, 0, sc);
        for (int j = 0; j < 16; ++j) result += (int)c[j][0];
    }
    out[blockIdx.x * 256 + threadIdx.x] = result;
}

#define CHECK(x)                                                                         \
    do {                                                                                 \
        hipError_t e_ = (x);                                                             \
        if (e_ != hipSuccess) {                                                          \
            fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                      \
            return 1;                                                                    \
        }                                                                                \
    } while (0)

template <int MODE>
static int run(const char *name, double ops_per_inst, int chains, bool random_bits) {
    const int blocks = 1024, iters = 20000;
    int *out, *bits;
    CHECK(hipMalloc(&out, (size_t)blocks * 256 * 4));
    CHECK(hipMalloc(&bits, 256 * 64));
    unsigned h[4096], x = 12345;
    for (int i = 0; i < 4096; i++) {
        x = x * 1664525u + 1013904223u;
        h[i] = random_bits ? (x ^ (x >> 13)) : 0x01010101u;
        // keep fp8 operands finite and moderate: clear sign and top exponent bit
        if (MODE == F8_32 || MODE == F8_16) h[i] &= 0x3f3f3f3fu;
    }
    CHECK(hipMemcpy(bits, h, sizeof(h), hipMemcpyHostToDevice));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    hipLaunchKernelGGL(chain<MODE>, dim3(blocks), dim3(256), 0, 0, 100, out, bits);
    CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL(chain<MODE>, dim3(blocks), dim3(256), 0, 0, iters, out, bits);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    const double insts = (double)blocks * 4 * iters * chains;
    printf("%-24s %-8s %8.3f ms  %8.1f Tops/s\n", name, random_bits ? "random" : "constant", ms,
            insts * ops_per_inst / ms / 1e9);
    CHECK(hipFree(out));
    CHECK(hipFree(bits));
    return 0;
}

int main(int argc, char **argv) {
    const bool rnd = !(argc > 1 && strcmp(argv[1], "constant") == 0);
    int rc = 0;
    rc |= run<I8_32>("i32_32x32x32_i8", 2.0 * 32 * 32 * 32, 8, rnd);
    rc |= run<I8_16>("i32_16x16x64_i8", 2.0 * 16 * 16 * 64, 16, rnd);
    rc |= run<F8_32>("f32_32x32x64_f8f6f4 fp8", 2.0 * 32 * 32 * 64, 8, rnd);
    rc |= run<F8_16>("f32_16x16x128_f8f6f4 fp8", 2.0 * 16 * 16 * 128, 16, rnd);
    rc |= run<F4_32>("f32_32x32x64_f8f6f4 fp4", 2.0 * 32 * 32 * 64, 8, rnd);
    rc |= run<F4_16>("f32_16x16x128_f8f6f4 fp4", 2.0 * 16 * 16 * 128, 16, rnd);
    return rc;
}
