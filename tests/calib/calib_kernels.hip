// Measurement kernels for bench.py's --calib-* switches: they compute nothing a
// caller of the library needs and are built into a library of their own
// (tests/bin/libmi355_calib.so, by tests/Makefile).  Every entry point returns 0
// on success, 1 on bad arguments and 2 when the launch failed.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mi355_calib.h"

namespace mi355 {
typedef int v4i __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(256) copy16_kernel(v4i *dst, const v4i *src, long n16) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n16;
            i += (long)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

__global__ void __launch_bounds__(256) flush_kernel(v4i *buf, long n16) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n16;
            i += (long)gridDim.x * blockDim.x) {
        v4i v = buf[i];
        v[0] += 1;
        buf[i] = v;
    }
}

// a launch that does nothing: what the dispatch of `blocks` workgroups of
// `threads` lanes costs by itself
__global__ void empty_kernel(unsigned *sink) {
    if (sink == (unsigned *)1) *sink = 0; // never true
}

// The skeleton of the packed decode kernel: 128 KB per workgroup read as by
// read_stream_kernel, every lane's values folded into one number, the 16
// wavefronts' numbers added through LDS and 64 values stored per workgroup.
__global__ void __launch_bounds__(1024) read_reduce_kernel(const uint8_t *src, float *out) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    __shared__ float part[16][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint8_t *p = src + ((long)blockIdx.x * 16 + wave) * 8192 + lane * 16;
    v4u r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = __builtin_nontemporal_load((const v4u *)(p + i * 1024));
    unsigned s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s ^= r[i][0] ^ r[i][1] ^ r[i][2] ^ r[i][3];
    part[wave][lane] = (float)s;
    __syncthreads();
    if (wave == 0) {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < 16; ++w) t += part[w][lane];
        out[blockIdx.x * 64 + lane] = t;
    }
}
} // namespace mi355

using namespace mi355;

static int launched() { return hipGetLastError() == hipSuccess ? 0 : 2; }

extern "C" int mi355_calib_copy(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes % 16 || ((uintptr_t)dst & 15) || ((uintptr_t)src & 15)) return 1;
    if (bytes == 0) return 0;
    const long n16 = (long)(bytes / 16);
    long blocks = (n16 + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(copy16_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
            (v4i *)dst, (const v4i *)src, n16);
    return launched();
}

extern "C" int mi355_calib_flush(void *buf, size_t bytes, void *stream) {
    if (bytes % 16 || ((uintptr_t)buf & 15)) return 1;
    if (bytes == 0) return 0;
    const long n16 = (long)(bytes / 16);
    long blocks = (n16 + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(flush_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (v4i *)buf, n16);
    return launched();
}

extern "C" int mi355_calib_empty(int blocks, int threads, void *stream) {
    if (blocks < 1 || threads < 1 || threads > 1024) return 1;
    hipLaunchKernelGGL(empty_kernel, dim3((unsigned)blocks), dim3((unsigned)threads), 0, (hipStream_t)stream,
            (unsigned *)nullptr);
    return launched();
}

extern "C" int mi355_calib_read_reduce(const void *src, size_t bytes, void *out, void *stream) {
    if (bytes % (128 << 10) || ((uintptr_t)src & 15) || !out) return 1;
    if (bytes == 0) return 0;
    hipLaunchKernelGGL(read_reduce_kernel, dim3((unsigned)(bytes / (128 << 10))), dim3(1024), 0, (hipStream_t)stream,
            (const uint8_t *)src, (float *)out);
    return launched();
}

namespace mi355 {
// Reads 128 KB per workgroup with the access shape of the packed decode kernel
// (16 wavefronts, each eight 1 KB runs, non-temporal, all requested before the
// first is consumed) and keeps nothing: what the weight stream alone costs.
__global__ void __launch_bounds__(1024) read_stream_kernel(const uint8_t *src, unsigned *sink) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint8_t *p = src + ((long)blockIdx.x * 16 + wave) * 8192 + lane * 16;
    v4u r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = __builtin_nontemporal_load((const v4u *)(p + i * 1024));
    unsigned s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s ^= r[i][0] ^ r[i][1] ^ r[i][2] ^ r[i][3];
    // never true for the benchmark's fill patterns; keeps the loads
    if (s == 0x9e3779b9u) sink[blockIdx.x] = s;
}
} // namespace mi355

namespace mi355 {
// Access-shape probe for the row-streaming kernels (the grouped matmul tiles): a workgroup of four wavefronts
// streams a slab of 256 rows x K bytes, every wavefront 64 rows, K-major; one load instruction fetches
// 1024 / RUN rows x RUN contiguous bytes (RUN = 128: the whole lines of 8 rows, the shape of the tiles; RUN = 64:
// half lines of 16 rows, the shape a matrix-instruction operand suggests; RUN = 1024: one row's contiguous KB).
// Every byte is read once, non-temporally, and nothing is kept.
template <int RUN>
__global__ void __launch_bounds__(256) read_pattern_kernel(const uint8_t *src, long K, unsigned *sink) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    constexpr int LPR = RUN / 16, RPI = 64 / LPR; // lanes per row, rows per instruction
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint8_t *slab = src + ((long)blockIdx.x * 256 + wave * 64) * K;
    const int r = lane / LPR, c = lane % LPR;
    v4u acc = {0, 0, 0, 0};
    for (long k = 0; k < K; k += RUN) {
#pragma unroll
        for (int i = 0; i < 64 / RPI; ++i)
            acc ^= __builtin_nontemporal_load((const v4u *)(slab + (long)(i * RPI + r) * K + k + c * 16));
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) sink[threadIdx.x] = acc[0];
}
} // namespace mi355

extern "C" int mi355_calib_read_pattern(const void *src, int64_t slabs, int64_t K, int run, void *sink, void *stream) {
    if (slabs < 0 || K <= 0 || K % 1024 || ((uintptr_t)src & 15) || !sink) {
        return 1;
    }
    if (slabs == 0) return 0;
    const dim3 grid((unsigned)slabs), block(256);
    hipStream_t s = (hipStream_t)stream;
    switch (run) {
        case 64: hipLaunchKernelGGL(read_pattern_kernel<64>, grid, block, 0, s, (const uint8_t *)src, (long)K, (unsigned *)sink); break;
        case 128: hipLaunchKernelGGL(read_pattern_kernel<128>, grid, block, 0, s, (const uint8_t *)src, (long)K, (unsigned *)sink); break;
        case 256: hipLaunchKernelGGL(read_pattern_kernel<256>, grid, block, 0, s, (const uint8_t *)src, (long)K, (unsigned *)sink); break;
        case 1024: hipLaunchKernelGGL(read_pattern_kernel<1024>, grid, block, 0, s, (const uint8_t *)src, (long)K, (unsigned *)sink); break;
        default: return 1;
    }
    return launched();
}

extern "C" int mi355_calib_read_stream(const void *src, size_t bytes, void *sink, void *stream) {
    if (bytes % (128 << 10) || ((uintptr_t)src & 15) || !sink) {
        return 1;
    }
    if (bytes == 0) return 0;
    hipLaunchKernelGGL(read_stream_kernel, dim3((unsigned)(bytes / (128 << 10))), dim3(1024), 0, (hipStream_t)stream,
            (const uint8_t *)src, (unsigned *)sink);
    return launched();
}

namespace mi355 {
// What the MFMA instructions of the GEMM kernels sustain when nothing else
// limits them: operands and accumulators stay in registers, 4 wavefronts per
// SIMD, 8 or 16 independent accumulator chains per wavefront.  The operand bits
// come from memory once, so the caller decides how much they toggle (the clock
// the power manager grants depends on it).
enum { RATE_I8_32, RATE_I8_16, RATE_F8_32, RATE_F8_16, RATE_F4_32, RATE_F4_16, RATE_BF16_32, RATE_BF16_16, RATE_F32_32, RATE_COUNT };

template <int MODE>
__global__ void __launch_bounds__(256) mfma_rate_kernel(int iters, int *out, const int *bits) {
    typedef int v8i __attribute__((ext_vector_type(8)));
    typedef int v16i __attribute__((ext_vector_type(16)));
    typedef float v4f __attribute__((ext_vector_type(4)));
    typedef float v16f __attribute__((ext_vector_type(16)));
    const v8i *r8 = (const v8i *)bits;
    const v8i a8 = r8[threadIdx.x * 2], b8 = r8[threadIdx.x * 2 + 1];
    const v4i a = {a8[0], a8[1], a8[2], a8[3]}, b = {b8[0], b8[1], b8[2], b8[3]};
    int result = 0;
    if (MODE == RATE_I8_32) {
        v16i c[8] = {};
        for (int i = 0; i < iters; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) c[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c[j], 0, 0, 0);
        for (int j = 0; j < 8; ++j) result += c[j][0];
    } else if (MODE == RATE_I8_16) {
        v4i c[16] = {};
        for (int i = 0; i < iters; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) c[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c[j], 0, 0, 0);
        for (int j = 0; j < 16; ++j) result += c[j][0];
    } else if (MODE == RATE_BF16_32) {
        typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
        v16f c[8] = {};
        for (int i = 0; i < iters; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j)
                c[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c[j], 0, 0, 0);
        for (int j = 0; j < 8; ++j) result += (int)c[j][0];
    } else if (MODE == RATE_BF16_16) {
        typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
        v4f c[16] = {};
        for (int i = 0; i < iters; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j)
                c[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c[j], 0, 0, 0);
        for (int j = 0; j < 16; ++j) result += (int)c[j][0];
    } else if (MODE == RATE_F32_32) {
        v16f c[8] = {};
        for (int i = 0; i < iters; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j)
                c[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__int_as_float(a[0]), __int_as_float(b[0]), c[j], 0, 0, 0);
        for (int j = 0; j < 8; ++j) result += (int)c[j][0];
    } else if (MODE == RATE_F8_32 || MODE == RATE_F4_32) {
        constexpr int fmt = MODE == RATE_F4_32 ? 4 : 0, sc = MODE == RATE_F4_32 ? 127 : 0;
        v16f c[8] = {};
        for (int i = 0; i < iters; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j)
                c[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, c[j], fmt, fmt, 0, sc, 0, sc);
        for (int j = 0; j < 8; ++j) result += (int)c[j][0];
    } else {
        constexpr int fmt = MODE == RATE_F4_16 ? 4 : 0, sc = MODE == RATE_F4_16 ? 127 : 0;
        v4f c[16] = {};
        for (int i = 0; i < iters; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j)
                c[j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, c[j], fmt, fmt, 0, sc, 0, sc);
        for (int j = 0; j < 16; ++j) result += (int)c[j][0];
    }
    out[blockIdx.x * 256 + threadIdx.x] = result;
}
} // namespace mi355

extern "C" int mi355_calib_mfma_rate(int instr, int iters, void *out, const void *bits, double *ops_per_launch,
        void *stream) {
    constexpr int blocks = 1024;
    if (instr < 0 || instr >= RATE_COUNT || iters < 1 || !out || !bits) {
        return 1;
    }
    static const double inst_ops[RATE_COUNT] = {2.0 * 32 * 32 * 32, 2.0 * 16 * 16 * 64, 2.0 * 32 * 32 * 64,
            2.0 * 16 * 16 * 128, 2.0 * 32 * 32 * 64, 2.0 * 16 * 16 * 128, 2.0 * 32 * 32 * 16, 2.0 * 16 * 16 * 32,
            2.0 * 32 * 32 * 2};
    static const int chains[RATE_COUNT] = {8, 16, 8, 16, 8, 16, 8, 16, 8};
    if (ops_per_launch) *ops_per_launch = (double)blocks * 4 * iters * chains[instr] * inst_ops[instr];
    hipStream_t s = (hipStream_t)stream;
    int *o = (int *)out;
    const int *bp = (const int *)bits;
    switch (instr) {
        case RATE_I8_32: hipLaunchKernelGGL(mfma_rate_kernel<RATE_I8_32>, dim3(blocks), dim3(256), 0, s, iters, o, bp); break;
        case RATE_I8_16: hipLaunchKernelGGL(mfma_rate_kernel<RATE_I8_16>, dim3(blocks), dim3(256), 0, s, iters, o, bp); break;
        case RATE_F8_32: hipLaunchKernelGGL(mfma_rate_kernel<RATE_F8_32>, dim3(blocks), dim3(256), 0, s, iters, o, bp); break;
        case RATE_F8_16: hipLaunchKernelGGL(mfma_rate_kernel<RATE_F8_16>, dim3(blocks), dim3(256), 0, s, iters, o, bp); break;
        case RATE_F4_32: hipLaunchKernelGGL(mfma_rate_kernel<RATE_F4_32>, dim3(blocks), dim3(256), 0, s, iters, o, bp); break;
        case RATE_BF16_32: hipLaunchKernelGGL(mfma_rate_kernel<RATE_BF16_32>, dim3(blocks), dim3(256), 0, s, iters, o, bp); break;
        case RATE_BF16_16: hipLaunchKernelGGL(mfma_rate_kernel<RATE_BF16_16>, dim3(blocks), dim3(256), 0, s, iters, o, bp); break;
        case RATE_F32_32: hipLaunchKernelGGL(mfma_rate_kernel<RATE_F32_32>, dim3(blocks), dim3(256), 0, s, iters, o, bp); break;
        default: hipLaunchKernelGGL(mfma_rate_kernel<RATE_F4_16>, dim3(blocks), dim3(256), 0, s, iters, o, bp); break;
    }
    return launched();
}

