// Small utility kernels of the library: the byte transposition the int8 / fp8
// families run on row-major weights, and the host-scalar store.
#include "kernels.hpp"

namespace mi355 {
typedef int v4i __attribute__((ext_vector_type(4)));

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
// out[c] = sum over r of x[r][c], r = 0, 1, ... in that order in f32 (the order of the reference's bias-gradient loop,
// src/cpu/ref_inner_product.cpp:196-210): a thread per column, consecutive lanes consecutive columns
__global__ void __launch_bounds__(256) colsum_kernel(const void *x, int x_dt, long rows, long cols, long ld, void *out,
        int out_dt) {
    const long c = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= cols) return;
    float acc = 0.f;
    for (long r = 0; r < rows; ++r) acc += load_float(x_dt, x, r * ld + c);
    const uint32_t bits = cvt_store_bits(out_dt, acc);
    if (dt_bits(out_dt) == 32) ((uint32_t *)out)[c] = bits;
    else ((uint16_t *)out)[c] = (uint16_t)bits;
}
} // namespace mi355

extern "C" int mi355_colsum_launch(const void *x, int x_dt, int64_t rows, int64_t cols, int64_t ld, void *out, int out_dt,
        void *stream) {
    auto fp = [](int dt) { return dt == MI355_DT_F32 || dt == MI355_DT_BF16 || dt == MI355_DT_F16; };
    if ((!x && rows > 0) || !out || rows < 0 || cols < 0 || ld < cols || !fp(x_dt) || !fp(out_dt)) {
        set_error("colsum: f32 / bf16 / f16 rows of at least `cols` elements");
        return MI355_INVALID_ARGUMENTS;
    }
    if (cols == 0) return MI355_SUCCESS;
    hipLaunchKernelGGL(colsum_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, x_dt,
            (long)rows, (long)cols, (long)ld, out, out_dt);
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
}
