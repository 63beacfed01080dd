// The row softmax of scaled dot-product attention: probs = softmax(scores * scale + mask) over the keys, one
// workgroup per (batch, head, query) row.  Operation order of the reference's kernel per element
// (src/gpu/intel/sdpa/ref.cl:46-70): s *= scale (the scale read in its own type, its reciprocal rounded to that
// type when inverted), s += mask, exp, division by the row's sum; causal masks set the scores of keys beyond the
// diagonal to -inf (src/gpu/intel/sdpa/micro.cl:864-878).  Differences, both inside rounding: the exponentials are
// taken relative to the row's largest score (no overflow for large scores), and the row sum is a tree over the
// workgroup instead of the reference's left-to-right loop.
#include "kernels.hpp"

namespace mi355 {
namespace {

struct softmax_dev_t {
    mi355_softmax_desc_t d;
    const float *scores;
    void *probs;
    const void *scale, *mask;
};

__device__ __forceinline__ float block_reduce(float v, bool is_max, float *lds) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float y = __shfl_xor(v, o, 64);
        v = is_max ? fmaxf(v, y) : v + y;
    }
    __syncthreads(); // (the previous reduction's readers are done with lds)
    if (lane == 0) lds[wave] = v;
    __syncthreads();
    float r = lds[0];
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) r = is_max ? fmaxf(r, lds[w]) : r + lds[w];
    return r;
}

__global__ void __launch_bounds__(256) sdpa_softmax_kernel(const softmax_dev_t P) {
    __shared__ float lds[4];
    const mi355_softmax_desc_t &D = P.d;
    const long row = blockIdx.x;
    const long q = row % D.sq, h = (row / D.sq) % D.h, b = row / (D.sq * D.h);
    const float *s = P.scores + row * D.sk;
    float sc = 1.f;
    if (D.scale_dt != MI355_DT_UNDEF) {
        sc = load_float(D.scale_dt, P.scale, 0);
        if (D.invert_scale) {
            // the reciprocal lives in a variable of the scale's type
            const uint32_t bits = cvt_store_bits(D.scale_dt, 1.f / sc);
            sc = D.scale_dt == MI355_DT_F32 ? u2f(bits)
                    : D.scale_dt == MI355_DT_BF16 ? u2f(bits << 16) : (float)__builtin_bit_cast(_Float16, (unsigned short)bits);
        }
    }
    long mbase = 0;
    if (D.mask_type == 1)
        mbase = (b % D.mask_dims[0]) * D.mask_stride[0] + (h % D.mask_dims[1]) * D.mask_stride[1]
                + (q % D.mask_dims[2]) * D.mask_stride[2];
    // keys up to `last` take part (causal masks)
    long last = D.sk - 1;
    if (D.mask_type == 2) last = q;
    if (D.mask_type == 3) last = q + (D.sk - D.sq);
    auto score = [&](long k) -> float {
        if (k > last) return -INFINITY;
        float v = s[k];
        if (D.scale_dt != MI355_DT_UNDEF) v *= sc;
        if (D.mask_type == 1) v += load_float(D.mask_dt, P.mask, mbase + (k % D.mask_dims[3]) * D.mask_stride[3]);
        return v;
    };
    float mx = -INFINITY;
    for (long k = threadIdx.x; k < D.sk; k += blockDim.x) mx = fmaxf(mx, score(k));
    mx = block_reduce(mx, true, lds);
    // a row of -inf only: exp(-inf - -inf) would be NaN where the reference's exp(-inf) is 0
    const float shift = mx == -INFINITY ? 0.f : mx;
    float sum = 0.f;
    for (long k = threadIdx.x; k < D.sk; k += blockDim.x) sum += expf(score(k) - shift);
    sum = block_reduce(sum, false, lds);
    const int bits_out = dt_bits(D.out_dt);
    for (long k = threadIdx.x; k < D.sk; k += blockDim.x) {
        float p = expf(score(k) - shift) / sum; // 0 / 0 = NaN for a fully masked row, as in the reference
        if (D.inf_as_zero && sum == 0.f) p = 0.f;
        const uint32_t bits = cvt_store_bits(D.out_dt, p);
        if (bits_out == 32) ((uint32_t *)P.probs)[row * D.sk + k] = bits;
        else ((uint16_t *)P.probs)[row * D.sk + k] = (uint16_t)bits;
    }
}

} // namespace
} // namespace mi355

using namespace mi355;

extern "C" int mi355_sdpa_softmax_launch(const mi355_softmax_desc_t *d, const void *scores, void *probs,
        const void *scale, const void *mask, void *stream) {
    auto fp = [](int dt) { return dt == MI355_DT_F32 || dt == MI355_DT_BF16 || dt == MI355_DT_F16; };
    if (!d || !scores || !probs) return MI355_INVALID_ARGUMENTS;
    if (d->b < 0 || d->h < 0 || d->sq < 0 || d->sk < 0 || !fp(d->out_dt) || d->mask_type < 0 || d->mask_type > 3) {
        set_error("sdpa softmax: bad descriptor");
        return MI355_INVALID_ARGUMENTS;
    }
    if ((d->scale_dt != MI355_DT_UNDEF && (!fp(d->scale_dt) || !scale)) || (d->mask_type == 1 && (!fp(d->mask_dt) || !mask))) {
        set_error("sdpa softmax: scale / mask of f32, bf16 or f16 in device memory");
        return MI355_INVALID_ARGUMENTS;
    }
    if (d->mask_type == 1)
        for (int i = 0; i < 4; ++i)
            if (d->mask_dims[i] < 1) return MI355_INVALID_ARGUMENTS;
    const long rows = d->b * d->h * d->sq;
    if (rows == 0 || d->sk == 0) return MI355_SUCCESS;
    if (rows >= (1L << 31)) {
        set_error("sdpa softmax: %ld rows exceed the grid", rows);
        return MI355_UNIMPLEMENTED;
    }
    softmax_dev_t P;
    P.d = *d;
    P.scores = (const float *)scores;
    P.probs = probs;
    P.scale = scale;
    P.mask = mask;
    hipLaunchKernelGGL(sdpa_softmax_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, P);
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
}
