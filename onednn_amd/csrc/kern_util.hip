// Small utility kernels behind the C ABI: a plain copy with a known byte count
// (calibrates the HBM traffic counters) and a cache-evicting sweep.
#include "kernels.hpp"

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

// in: [R][C] bytes with row pitch ld_in  ->  out: [C][R] bytes, pitch ld_out
__global__ void __launch_bounds__(256) transpose_bytes_kernel(const uint8_t *in, long R, long C,
        long ld_in, long in_bstride, uint8_t *out, long ld_out, long out_bstride) {
    __shared__ uint8_t tile[64][65];
    in += blockIdx.z * in_bstride;
    out += blockIdx.z * out_bstride;
    const long r0 = (long)blockIdx.y * 64, c0 = (long)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4) {
        const long r = r0 + i, c = c0 + tx;
        tile[i][tx] = (r < R && c < C) ? in[r * ld_in + c] : 0;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const long c = c0 + i, r = r0 + tx;
        if (c < C && r < R) out[c * ld_out + r] = tile[tx][i];
    }
}


// The same transposition for whole 64 x 64 tiles and aligned pitches: a thread
// loads a 4 x 4 block as four dwords, transposes it in registers with eight
// byte permutes, parks the four result dwords in LDS; the tile leaves as
// 16-byte stores (8192 x 8192: 32 us against 80 us for the byte-wise kernel).
__global__ void __launch_bounds__(256) transpose_bytes_tiles_kernel(const uint8_t *in, long ld_in, long in_bstride,
        uint8_t *out, long ld_out, long out_bstride) {
    constexpr int PITCH = 17; // dwords per LDS row (16 + 1: spreads the banks)
    __shared__ uint32_t tile[64 * PITCH];
    in += blockIdx.z * in_bstride;
    out += blockIdx.z * out_bstride;
    const long r0 = (long)blockIdx.y * 64, c0 = (long)blockIdx.x * 64;
    const int ci = threadIdx.x & 15, ri = threadIdx.x >> 4; // read: block (4 ri .. +3, 4 ci .. +3)
    const int wc = threadIdx.x >> 2, wq = threadIdx.x & 3;  // write: out row c0 + wc, 16 bytes of r
    const uint8_t *p = in + (r0 + 4 * ri) * ld_in + c0 + 4 * ci;
    const uint32_t q0 = *(const uint32_t *)p, q1 = *(const uint32_t *)(p + ld_in),
                   q2 = *(const uint32_t *)(p + 2 * ld_in), q3 = *(const uint32_t *)(p + 3 * ld_in);
    // byte k of q_i is element (r + i, c + k); the results collect byte k of the four rows
    const uint32_t x0 = __builtin_amdgcn_perm(q1, q0, 0x05010400u), x1 = __builtin_amdgcn_perm(q1, q0, 0x07030602u);
    const uint32_t y0 = __builtin_amdgcn_perm(q3, q2, 0x05010400u), y1 = __builtin_amdgcn_perm(q3, q2, 0x07030602u);
    tile[(4 * ci + 0) * PITCH + ri] = __builtin_amdgcn_perm(y0, x0, 0x05040100u);
    tile[(4 * ci + 1) * PITCH + ri] = __builtin_amdgcn_perm(y0, x0, 0x07060302u);
    tile[(4 * ci + 2) * PITCH + ri] = __builtin_amdgcn_perm(y1, x1, 0x05040100u);
    tile[(4 * ci + 3) * PITCH + ri] = __builtin_amdgcn_perm(y1, x1, 0x07060302u);
    __syncthreads();
    uint4 v;
    v.x = tile[wc * PITCH + 4 * wq]; v.y = tile[wc * PITCH + 4 * wq + 1];
    v.z = tile[wc * PITCH + 4 * wq + 2]; v.w = tile[wc * PITCH + 4 * wq + 3];
    *(uint4 *)(out + (c0 + wc) * ld_out + r0 + 16 * wq) = v;
}

// ... and for whole 128 x 128 tiles with 16-byte aligned rows: a thread loads
// 4 rows x 16 bytes, so every load instruction fetches the whole 128-byte lines
// of eight rows and every store instruction writes those of eight output rows
// (with 64-byte tile rows each input line is fetched by two workgroups, on
// different L2s); dword column c of tile row r sits at (c + 8 (r / 16)) % 32:
// conflict-free stores, aligned 16-byte reads.  Output written once, input read
// once: non-temporal both ways.
__global__ void __launch_bounds__(256) transpose_bytes_tiles128_kernel(const uint8_t *in, long ld_in, long in_bstride,
        uint8_t *out, long ld_out, long out_bstride) {
    typedef uint32_t u4v __attribute__((ext_vector_type(4)));
    __shared__ __attribute__((aligned(16))) uint32_t tile[128 * 32];
    in += blockIdx.z * in_bstride;
    out += blockIdx.z * out_bstride;
    const long r0 = (long)blockIdx.y * 128, c0 = (long)blockIdx.x * 128;
    const int ci = threadIdx.x & 7, rg = threadIdx.x >> 3; // read: rows 4 rg .. +3, bytes 16 ci .. +15
    const int wq = threadIdx.x & 7, wr = threadIdx.x >> 3; // write: output row wr + 32 pass, bytes 16 wq .. +15
    const uint8_t *p = in + (r0 + 4 * rg) * ld_in + c0 + 16 * ci;
    u4v q[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = __builtin_nontemporal_load((const u4v *)(p + i * ld_in));
    const int col = (rg + 8 * (ci & 3)) & 31;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t q0 = q[0][k], q1 = q[1][k], q2 = q[2][k], q3 = q[3][k];
        // byte j of q_i is element (r + i, c + 4 k + j); the results collect byte j of the four rows
        const uint32_t x0 = __builtin_amdgcn_perm(q1, q0, 0x05010400u), x1 = __builtin_amdgcn_perm(q1, q0, 0x07030602u);
        const uint32_t y0 = __builtin_amdgcn_perm(q3, q2, 0x05010400u), y1 = __builtin_amdgcn_perm(q3, q2, 0x07030602u);
        const int row = 16 * ci + 4 * k;
        tile[(row + 0) * 32 + col] = __builtin_amdgcn_perm(y0, x0, 0x05040100u);
        tile[(row + 1) * 32 + col] = __builtin_amdgcn_perm(y0, x0, 0x07060302u);
        tile[(row + 2) * 32 + col] = __builtin_amdgcn_perm(y1, x1, 0x05040100u);
        tile[(row + 3) * 32 + col] = __builtin_amdgcn_perm(y1, x1, 0x07060302u);
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int c = wr + 32 * pass;
        const u4v v = *(const u4v *)&tile[c * 32 + ((4 * wq + 8 * ((c >> 4) & 3)) & 31)];
        __builtin_nontemporal_store(v, (u4v *)(out + (c0 + c) * ld_out + r0 + 16 * wq));
    }
}

void transpose_bytes(const void *in, long R, long C, long ld_in, long in_bstride, void *out,
        long ld_out, long out_bstride, long batches, hipStream_t stream) {
    dim3 grid((unsigned)((C + 63) / 64), (unsigned)((R + 63) / 64), (unsigned)batches);
    const bool whole = R % 64 == 0 && C % 64 == 0 && ld_in % 4 == 0 && in_bstride % 4 == 0 && ld_out % 16 == 0
            && out_bstride % 16 == 0 && (uintptr_t)in % 4 == 0 && (uintptr_t)out % 16 == 0;
    const bool whole128 = whole && R % 128 == 0 && C % 128 == 0 && ld_in % 16 == 0 && in_bstride % 16 == 0
            && (uintptr_t)in % 16 == 0;
    if (whole128)
        hipLaunchKernelGGL(transpose_bytes_tiles128_kernel, dim3((unsigned)(C / 128), (unsigned)(R / 128), (unsigned)batches),
                dim3(256), 0, stream, (const uint8_t *)in, ld_in, in_bstride, (uint8_t *)out, ld_out, out_bstride);
    else if (whole)
        hipLaunchKernelGGL(transpose_bytes_tiles_kernel, grid, dim3(256), 0, stream, (const uint8_t *)in, ld_in,
                in_bstride, (uint8_t *)out, ld_out, out_bstride);
    else
        hipLaunchKernelGGL(transpose_bytes_kernel, grid, dim3(256), 0, stream, (const uint8_t *)in, R, C,
                ld_in, in_bstride, (uint8_t *)out, ld_out, out_bstride);
}
} // namespace mi355

using namespace mi355;

extern "C" int mi355_copy_kernel(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes % 16 || ((uintptr_t)dst & 15) || ((uintptr_t)src & 15)) {
        set_error("copy kernel needs 16-byte aligned pointers and size");
        return MI355_INVALID_ARGUMENTS;
    }
    if (bytes == 0) return MI355_SUCCESS;
    const long n16 = (long)(bytes / 16);
    long blocks = (n16 + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(copy16_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
            (v4i *)dst, (const v4i *)src, n16);
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
}

namespace mi355 {
__global__ void store_scalar_kernel(unsigned char *dst, uint64_t bits, int nbytes) {
    if (threadIdx.x < (unsigned)nbytes) dst[threadIdx.x] = (unsigned char)(bits >> (8 * threadIdx.x));
}
} // namespace mi355

extern "C" int mi355_mem_store_scalar(void *dptr, uint64_t bits, int nbytes, void *stream) {
    if (!dptr || (nbytes != 1 && nbytes != 2 && nbytes != 4 && nbytes != 8)) {
        set_error("store_scalar: 1, 2, 4 or 8 bytes to a device pointer");
        return MI355_INVALID_ARGUMENTS;
    }
    hipLaunchKernelGGL(store_scalar_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, (unsigned char *)dptr, bits,
            nbytes);
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
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

extern "C" int mi355_read_pattern_kernel(const void *src, int64_t slabs, int64_t K, int run, void *sink, void *stream) {
    if (slabs < 0 || K <= 0 || K % 1024 || ((uintptr_t)src & 15) || !sink) {
        set_error("read pattern kernel needs a 16-byte aligned pointer, K a multiple of 1024 and a sink of 1 KiB");
        return MI355_INVALID_ARGUMENTS;
    }
    if (slabs == 0) return MI355_SUCCESS;
    const dim3 grid((unsigned)slabs), block(256);
    hipStream_t s = (hipStream_t)stream;
    switch (run) {
        case 64: hipLaunchKernelGGL(read_pattern_kernel<64>, grid, block, 0, s, (const uint8_t *)src, (long)K, (unsigned *)sink); break;
        case 128: hipLaunchKernelGGL(read_pattern_kernel<128>, grid, block, 0, s, (const uint8_t *)src, (long)K, (unsigned *)sink); break;
        case 256: hipLaunchKernelGGL(read_pattern_kernel<256>, grid, block, 0, s, (const uint8_t *)src, (long)K, (unsigned *)sink); break;
        case 1024: hipLaunchKernelGGL(read_pattern_kernel<1024>, grid, block, 0, s, (const uint8_t *)src, (long)K, (unsigned *)sink); break;
        default: set_error("read pattern kernel: run must be 64, 128, 256 or 1024 bytes"); return MI355_INVALID_ARGUMENTS;
    }
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
}

extern "C" int mi355_read_stream_kernel(const void *src, size_t bytes, void *sink, void *stream) {
    if (bytes % (128 << 10) || ((uintptr_t)src & 15) || !sink) {
        set_error("read stream kernel needs a 16-byte aligned pointer, a multiple of 128 KiB and a sink of 4 bytes per 128 KiB");
        return MI355_INVALID_ARGUMENTS;
    }
    if (bytes == 0) return MI355_SUCCESS;
    hipLaunchKernelGGL(read_stream_kernel, dim3((unsigned)(bytes / (128 << 10))), dim3(1024), 0, (hipStream_t)stream,
            (const uint8_t *)src, (unsigned *)sink);
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
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

extern "C" int mi355_mfma_rate_kernel(int instr, int iters, void *out, const void *bits, double *ops_per_launch,
        void *stream) {
    constexpr int blocks = 1024;
    if (instr < 0 || instr >= RATE_COUNT || iters < 1 || !out || !bits) {
        set_error("mfma rate kernel: instruction 0..8, out of 1 MiB, 16 KiB of operand bits");
        return MI355_INVALID_ARGUMENTS;
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
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
}

extern "C" int mi355_flush_kernel(void *buf, size_t bytes, void *stream) {
    if (bytes % 16 || ((uintptr_t)buf & 15)) {
        set_error("flush kernel needs a 16-byte aligned pointer and size");
        return MI355_INVALID_ARGUMENTS;
    }
    if (bytes == 0) return MI355_SUCCESS;
    const long n16 = (long)(bytes / 16);
    long blocks = (n16 + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(flush_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
            (v4i *)buf, n16);
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
}
