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


void transpose_bytes(const void *in, long R, long C, long ld_in, long in_bstride, void *out,
        long ld_out, long out_bstride, long batches, hipStream_t stream) {
    dim3 grid((unsigned)((C + 63) / 64), (unsigned)((R + 63) / 64), (unsigned)batches);
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
