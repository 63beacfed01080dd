// "hip:ref_grouped:any" -- grouped (mixture-of-experts) matmul, one thread per
// dst element, in the operation order of the reference's ref_grouped_t
// (src/cpu/matmul/ref_grouped_gemm.cpp:215-440):
//
//   per K group of the finest quantization granularity:
//     integer src:  acc = f32( sum_k (s - zs)(w - zw) )       (s32 sum)
//     fp src, integer weights (decompression):  acc += s * f32(w - zw)
//     fp weights:  acc += s * w
//     acc *= src_scale (per row [and K group]);  result += acc * wei_scale
//     (fp weights: acc *= wei_scale; result += acc)
//   + bias[g][n] -> post-ops (eltwise; multiplication by a per-group, per-row
//   or per-element operand) -> conversion to the dst type.
//
// The groups' boundaries are cumulative s32 offsets in device memory.  A thread
// finds its group by bisection; nothing is assumed about the offsets beyond
// what keeps every access inside the tensors.
#include "kernels.hpp"

namespace mi355 {
namespace {

struct grouped_dev_t {
    mi355_grouped_desc_t d;
    mi355_grouped_args_t a;
};

// smallest g with offsets[g] > r, or G
__device__ __forceinline__ long find_group(const int32_t *offsets, long G, long r) {
    long lo = 0, hi = G;
    while (lo < hi) {
        const long mid = (lo + hi) >> 1;
        if ((long)offsets[mid] > r) hi = mid;
        else lo = mid + 1;
    }
    return lo;
}

__device__ __forceinline__ float grouped_finish(const grouped_dev_t &P, float result, long g, long m, long n,
        long dst_row_base) {
    const mi355_grouped_desc_t &D = P.d;
    if (D.bias_dt != MI355_DT_UNDEF) result += load_float(D.bias_dt, P.a.bias, g * D.N + n);
    for (int i = 0; i < D.n_post_ops; ++i) {
        const mi355_grouped_post_op_t &po = D.post_ops[i];
        if (po.kind == MI355_PO_ELTWISE) {
            result = eltwise_f(po.alg, result, po.alpha, po.beta) * po.scale;
        } else {
            // a grouped operand brings offsets of its own, a dense one follows dst's
            long row_base = dst_row_base;
            if (po.grouped) row_base = g > 0 ? (long)P.a.po_offsets[i][g - 1] : 0;
            const bool per_group = po.bin_m == D.group_count && po.bin_n == 1;
            long em = per_group ? g : row_base + m;
            if (em >= po.bin_m) em = po.bin_m - 1; // (offsets are not trusted)
            if (em < 0) em = 0;
            const long en = po.bin_n > 1 ? n : 0;
            result = binary_f(po.alg, result, load_float(po.dt, P.a.po_arg[i], em * po.bin_n + en));
        }
    }
    return result;
}

__global__ void __launch_bounds__(256) grouped_2dx3d_kernel(const grouped_dev_t P) {
    const mi355_grouped_desc_t &D = P.d;
    const long e = (long)blockIdx.x * 256 + threadIdx.x;
    if (e >= D.total * D.N) return;
    const long r = e / D.N, n = e % D.N; // dst row and column
    const long G = D.group_count;
    const long g = find_group(P.a.dst_offsets, G, r);
    if (g >= G) return;
    const long dst_start = g > 0 ? (long)P.a.dst_offsets[g - 1] : 0;
    const long src_start = g > 0 ? (long)P.a.src_offsets[g - 1] : 0;
    const long src_end = P.a.src_offsets[g];
    const long m = r - dst_start;
    if (m < 0 || src_start < 0 || src_start + m >= src_end || src_start + m >= D.total) return;
    const long srow = src_start + m, K = D.K, N = D.N;

    const bool int_src = D.src_dt == MI355_DT_S8 || D.src_dt == MI355_DT_U8;
    const bool int_wei = D.wei_dt == MI355_DT_S8 || D.wei_dt == MI355_DT_U8 || D.wei_dt == MI355_DT_S4
            || D.wei_dt == MI355_DT_U4;
    const bool woq = !int_src && int_wei && D.fpmath_apply_to_int;
    auto ngroups = [&](int dt, long gk) { return dt != MI355_DT_UNDEF && gk > 1 ? K / gk : 1; };
    const long ss_ng = ngroups(D.src_scale_dt, D.src_scale_gk), ws_ng = ngroups(D.wei_scale_dt, D.wei_scale_gk);
    const long sz_ng = ngroups(D.src_zp_dt, D.src_zp_gk), wz_ng = ngroups(D.wei_zp_dt, D.wei_zp_gk);
    long nkg = ss_ng > ws_ng ? ss_ng : ws_ng;
    nkg = sz_ng > nkg ? sz_ng : nkg;
    nkg = wz_ng > nkg ? wz_ng : nkg;
    const long kgs = K / nkg;
    const long wbase = g * D.wei_stride[0];

    float result = 0.f;
    for (long ig = 0; ig < nkg; ++ig) {
        float acc = 0.f;
        if (int_src || woq) {
            int zs = 0, zw = 0;
            float wsc = 1.f;
            if (D.src_zp_dt != MI355_DT_UNDEF) zs = load_int(D.src_zp_dt, P.a.src_zp, srow * sz_ng + ig * sz_ng / nkg);
            if (D.wei_scale_dt != MI355_DT_UNDEF)
                wsc = load_float(D.wei_scale_dt, P.a.wei_scale, g * ws_ng * N + (ig * ws_ng / nkg) * N + n);
            if (D.wei_zp_dt != MI355_DT_UNDEF)
                zw = load_int(D.wei_zp_dt, P.a.wei_zp, g * wz_ng * N + (ig * wz_ng / nkg) * N + n);
            if (int_src) {
                int acc_int = 0;
                for (long k = ig * kgs; k < (ig + 1) * kgs; ++k)
                    acc_int += (load_int(D.src_dt, P.a.src, srow * K + k) - zs)
                            * (load_int(D.wei_dt, P.a.wei, wbase + k * D.wei_stride[1] + n * D.wei_stride[2]) - zw);
                acc = (float)acc_int;
            } else {
                for (long k = ig * kgs; k < (ig + 1) * kgs; ++k)
                    acc += load_float(D.src_dt, P.a.src, srow * K + k)
                            * (float)(load_int(D.wei_dt, P.a.wei, wbase + k * D.wei_stride[1] + n * D.wei_stride[2]) - zw);
            }
            if (D.src_scale_dt != MI355_DT_UNDEF)
                acc *= load_float(D.src_scale_dt, P.a.src_scale, srow * ss_ng + ig * ss_ng / nkg);
            result += acc * wsc;
        } else {
            for (long k = ig * kgs; k < (ig + 1) * kgs; ++k)
                acc += load_float(D.src_dt, P.a.src, srow * K + k)
                        * load_float(D.wei_dt, P.a.wei, wbase + k * D.wei_stride[1] + n * D.wei_stride[2]);
            if (D.src_scale_dt != MI355_DT_UNDEF)
                acc *= load_float(D.src_scale_dt, P.a.src_scale, srow * ss_ng + ig * ss_ng / nkg);
            if (D.wei_scale_dt != MI355_DT_UNDEF)
                acc *= load_float(D.wei_scale_dt, P.a.wei_scale, g * ws_ng * N + (ig * ws_ng / nkg) * N + n);
            result += acc;
        }
    }
    result = grouped_finish(P, result, g, m, n, dst_start);
    store_float(D.dst_dt, result, P.a.dst, r * N + n);
}

// dst[g][m][n] = sum over the group's K range; an empty range writes zeros
__global__ void __launch_bounds__(256) grouped_2dx2d_kernel(const grouped_dev_t P) {
    const mi355_grouped_desc_t &D = P.d;
    const long e = (long)blockIdx.x * 256 + threadIdx.x;
    const long G = D.group_count, M = D.M, N = D.N;
    if (e >= G * M * N) return;
    const long g = e / (M * N), m = (e / N) % M, n = e % N;
    long k0 = g > 0 ? (long)P.a.src_offsets[g - 1] : 0, k1 = P.a.src_offsets[g];
    if (k0 < 0) k0 = 0;
    if (k1 > D.total) k1 = D.total;
    float acc = 0.f;
    for (long k = k0; k < k1; ++k)
        acc += load_float(D.src_dt, P.a.src, m + k * M) * load_float(D.wei_dt, P.a.wei, k * N + n);
    store_float(D.dst_dt, acc, P.a.dst, g * D.dst_stride[0] + m * D.dst_stride[1] + n * D.dst_stride[2]);
}

bool fp_plain(int dt) { return dt == MI355_DT_F32 || dt == MI355_DT_BF16 || dt == MI355_DT_F16; }
bool fp_any(int dt) {
    return fp_plain(dt) || dt == MI355_DT_F8_E4M3 || dt == MI355_DT_F8_E5M2 || dt == MI355_DT_F4_E2M1;
}

} // namespace
} // namespace mi355

using namespace mi355;

extern "C" int mi355_grouped_matmul_query(const mi355_grouped_desc_t *d) {
    if (!d) return MI355_INVALID_ARGUMENTS;
    if (d->group_count < 1 || d->total < 1 || d->N < 1) return MI355_INVALID_ARGUMENTS;
    if (d->n_post_ops < 0 || d->n_post_ops > MI355_MAX_POST_OPS) return MI355_INVALID_ARGUMENTS;
    if (d->total >= (1L << 31) || d->group_count >= (1L << 31)) return MI355_UNIMPLEMENTED; // s32 offsets
    if (!fp_plain(d->dst_dt)) return MI355_UNIMPLEMENTED;
    if (d->pattern == MI355_GROUPED_2DX2D) {
        if (d->M < 1) return MI355_INVALID_ARGUMENTS;
        if (d->src_dt != d->wei_dt || d->src_dt != d->dst_dt) return MI355_UNIMPLEMENTED;
        if (d->bias_dt != MI355_DT_UNDEF || d->n_post_ops != 0 || d->src_scale_dt || d->wei_scale_dt || d->src_zp_dt
                || d->wei_zp_dt)
            return MI355_UNIMPLEMENTED;
        return MI355_SUCCESS;
    }
    if (d->pattern != MI355_GROUPED_2DX3D) return MI355_INVALID_ARGUMENTS;
    if (d->K < 1) return MI355_INVALID_ARGUMENTS;
    const bool int_src = is_int8_dt(d->src_dt), int_wei = is_int8_dt(d->wei_dt) || is_int4_dt(d->wei_dt);
    if (!int_src && !fp_any(d->src_dt)) return MI355_UNIMPLEMENTED;
    if (!int_wei && !fp_any(d->wei_dt)) return MI355_UNIMPLEMENTED;
    if (int_src && !int_wei) return MI355_UNIMPLEMENTED;
    // decompression needs weights scales and the apply_to_int switch
    if (!int_src && int_wei && (d->wei_scale_dt == MI355_DT_UNDEF || !d->fpmath_apply_to_int)) return MI355_UNIMPLEMENTED;
    if (d->src_zp_dt != MI355_DT_UNDEF && !int_src) return MI355_UNIMPLEMENTED;
    if (d->wei_zp_dt != MI355_DT_UNDEF && !int_wei) return MI355_UNIMPLEMENTED;
    const int64_t gks[4] = {d->src_scale_dt ? d->src_scale_gk : 0, d->wei_scale_dt ? d->wei_scale_gk : 0,
            d->src_zp_dt ? d->src_zp_gk : 0, d->wei_zp_dt ? d->wei_zp_gk : 0};
    int64_t finest = d->K;
    for (int64_t gk : gks) {
        if (gk < 0 || (gk > 1 && d->K % gk != 0)) return MI355_UNIMPLEMENTED;
        if (gk > 1 && gk < finest) finest = gk;
    }
    // every K grouping is a multiple of the finest one
    for (int64_t gk : gks)
        if (gk > 1 && gk % finest != 0) return MI355_UNIMPLEMENTED;
    for (int i = 0; i < d->n_post_ops; ++i) {
        const mi355_grouped_post_op_t &po = d->post_ops[i];
        if (po.kind == MI355_PO_ELTWISE) continue;
        if (po.kind != MI355_PO_BINARY || po.alg != MI355_BINARY_MUL) return MI355_UNIMPLEMENTED;
        if (po.bin_m < 1 || (po.bin_n != 1 && po.bin_n != d->N)) return MI355_UNIMPLEMENTED;
        const bool per_group = po.bin_m == d->group_count && po.bin_n == 1;
        if (!per_group && po.bin_m != d->total) return MI355_UNIMPLEMENTED;
    }
    return MI355_SUCCESS;
}

extern "C" int mi355_grouped_matmul_launch(const mi355_grouped_desc_t *d, const mi355_grouped_args_t *a, void *stream) {
    if (!d || !a) return MI355_INVALID_ARGUMENTS;
    if (const int st = mi355_grouped_matmul_query(d)) {
        set_error("grouped matmul: problem not supported (status %d)", st);
        return st;
    }
    const bool x3 = d->pattern == MI355_GROUPED_2DX3D;
    if (!a->src || !a->wei || !a->dst || !a->src_offsets || (x3 ? !a->dst_offsets : !a->wei_offsets)
            || (d->bias_dt != MI355_DT_UNDEF && !a->bias) || (d->src_scale_dt && !a->src_scale)
            || (d->wei_scale_dt && !a->wei_scale) || (d->src_zp_dt && !a->src_zp) || (d->wei_zp_dt && !a->wei_zp)) {
        set_error("grouped matmul: a required buffer is NULL");
        return MI355_INVALID_ARGUMENTS;
    }
    for (int i = 0; i < d->n_post_ops; ++i)
        if (d->post_ops[i].kind == MI355_PO_BINARY && (!a->po_arg[i] || (d->post_ops[i].grouped && !a->po_offsets[i]))) {
            set_error("grouped matmul: the operand of post-op %d is NULL", i);
            return MI355_INVALID_ARGUMENTS;
        }
    grouped_dev_t P;
    P.d = *d;
    P.a = *a;
    const long elems = x3 ? d->total * d->N : d->group_count * d->M * d->N;
    const long blocks = (elems + 255) / 256;
    if (blocks >= (1L << 31)) {
        set_error("grouped matmul: %ld dst elements exceed the grid", elems);
        return MI355_UNIMPLEMENTED;
    }
    if (x3)
        hipLaunchKernelGGL(grouped_2dx3d_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, P);
    else
        hipLaunchKernelGGL(grouped_2dx2d_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, P);
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
}
