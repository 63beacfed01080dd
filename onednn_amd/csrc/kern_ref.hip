// "hip:ref:any" -- one thread per dst element, every data type and attribute
// combination the path admits.  It is the GPU-side counterpart of the
// reference's naive implementations and computes in exactly their order:
//   integer src:  ref_matmul_int8_t::execute_ref  src/cpu/matmul/ref_matmul_int8.cpp:174-306
//   other src:    ref_matmul_t::execute_ref       src/cpu/matmul/ref_matmul.cpp:168-331
// so its f32 results agree bit for bit with them wherever no libm function is
// involved.  The tuned kernel families fall back to it for shapes and
// attribute mixes they do not cover.
#include "mi355_device.hpp"
#include "kernels.hpp"

namespace mi355 {

template <class Q>
__device__ __forceinline__ long ngroups_k(const Q &q, int kdim, long K) {
    if (q.dt == MI355_DT_UNDEF) return 1;
    const long g = kdim ? q.g1 : q.g0;
    return g > 1 ? K / g : 1;
}

// element offset of weights (b, k, n): strided, or the nibble offset of the
// 64-column decode packing (MI355_WEI_PACK_WOQ64)
template <class PT>
__device__ __forceinline__ long wei_off(const PT &P, long bw, long k, long n) {
    if (P.wei_packing == MI355_WEI_PACK_WOQ64)
        return (n / 64) * (P.K * 64) + (k / 8) * 512 + (n % 16) * 32 + ((n % 64) / 16) * 8 + (k % 2) * 4
                + (k % 8) / 2;
    return bw * P.ws[0] + k * P.ws[1] + n * P.ws[2];
}

template <class PT>
__device__ float ref_int_dot(const PT &P, long b, long m, long n) {
    const long K = P.K, M = P.M, N = P.N;
    const long bs = P.ss[0] ? b : 0, bw = P.ws[0] ? b : 0;
    const bool src_zp = P.src_zp.dt != MI355_DT_UNDEF;
    const bool wei_zp = P.wei_zp.dt != MI355_DT_UNDEF;
    const bool src_pr = P.src_pr.dt != MI355_DT_UNDEF;
    long ng = 1, t;
    if ((t = ngroups_k(P.src_zp, 1, K)) > ng) ng = t;
    if ((t = ngroups_k(P.wei_zp, 0, K)) > ng) ng = t;
    if ((t = ngroups_k(P.src_scale, 1, K)) > ng) ng = t;
    if ((t = ngroups_k(P.wei_scale, 0, K)) > ng) ng = t;
    if ((t = ngroups_k(P.src_pr, 1, K)) > ng) ng = t;
    const long gk = K / ng;
    float res = 0.f;
    for (long g = 0; g < ng; ++g) {
        int acc = 0;
        long k = g * gk;
        for (long kk = 0; kk < gk; ++kk) {
            k = g * gk + kk;
            int s = load_int(P.src_dt, P.src, bs * P.ss[0] + m * P.ss[1] + k * P.ss[2]);
            int w = load_int(P.wei_dt, P.wei, wei_off(P, bw, k, n));
            if (src_zp) s -= load_int(P.src_zp.dt, P.src_zp.p, quant_off(P.src_zp, bs, m, k, M, K));
            if (wei_zp && !src_pr)
                w -= load_int(P.wei_zp.dt, P.wei_zp.p, quant_off(P.wei_zp, bw, k, n, K, N));
            acc += s * w;
        }
        if (src_pr) {
            const int pr = load_int(P.src_pr.dt, P.src_pr.p, quant_off(P.src_pr, bs, m, k, M, K));
            const int wzp = load_int(P.wei_zp.dt, P.wei_zp.p, quant_off(P.wei_zp, bw, k, n, K, N));
            acc -= pr * wzp;
            if (src_zp) {
                const int szp = load_int(P.src_zp.dt, P.src_zp.p, quant_off(P.src_zp, bs, m, k, M, K));
                acc += (int)(gk * wzp * szp);
            }
        }
        float f = (float)acc;
        if (P.src_scale.dt != MI355_DT_UNDEF)
            f *= load_float(P.src_scale.dt, P.src_scale.p, quant_off(P.src_scale, bs, m, k, M, K));
        if (P.wei_scale.dt != MI355_DT_UNDEF)
            f *= load_float(P.wei_scale.dt, P.wei_scale.p, quant_off(P.wei_scale, bw, k, n, K, N));
        res += f;
    }
    return res;
}

template <class PT>
__device__ float ref_fp_dot(const PT &P, long b, long m, long n) {
    const long K = P.K, M = P.M, N = P.N;
    const long bs = P.ss[0] ? b : 0, bw = P.ws[0] ? b : 0;
    const bool wei_int = P.wei_dt == MI355_DT_S8 || P.wei_dt == MI355_DT_U8
            || P.wei_dt == MI355_DT_S4 || P.wei_dt == MI355_DT_U4;
    const bool decomp = wei_int && P.apply_to_int;
    const bool wei_zp = P.wei_zp.dt != MI355_DT_UNDEF;
    const bool src_sc = P.src_scale.dt != MI355_DT_UNDEF;
    const bool wei_sc = P.wei_scale.dt != MI355_DT_UNDEF;
    const long sgk = src_sc ? P.src_scale.g1 : 1;
    const long wgk = wei_sc ? P.wei_scale.g0 : 1;
    const long ng = K / sgk > K / wgk ? K / sgk : K / wgk;
    const long gk = K / ng;
    float res = 0.f;
    for (long g = 0; g < ng; ++g) {
        float acc = 0.f;
        long k = g * gk;
        for (long kk = 0; kk < gk; ++kk) {
            k = g * gk + kk;
            const float s = load_float(P.src_dt, P.src, bs * P.ss[0] + m * P.ss[1] + k * P.ss[2]);
            float w = load_float(P.wei_dt, P.wei, wei_off(P, bw, k, n));
            if (decomp) {
                if (wei_zp)
                    w -= load_float(P.wei_zp.dt, P.wei_zp.p, quant_off(P.wei_zp, bw, k, n, K, N));
                if (wei_sc)
                    w *= load_float(P.wei_scale.dt, P.wei_scale.p, quant_off(P.wei_scale, bw, k, n, K, N));
            }
            acc += s * w;
        }
        if (src_sc)
            acc *= load_float(P.src_scale.dt, P.src_scale.p, quant_off(P.src_scale, bs, m, k, M, K));
        if (wei_sc && !decomp)
            acc *= load_float(P.wei_scale.dt, P.wei_scale.p, quant_off(P.wei_scale, bw, k, n, K, N));
        res += acc;
    }
    return res;
}

// bias, dropout (ref_matmul.cpp:283-296), then the rest of the epilogue
template <class PT>
__device__ __forceinline__ float ref_epilogue_value(const PT &P, float v, long b, long m, long n) {
    if (!(P.rnd_flags & MI355_RND_DROPOUT)) return epilogue_value(P, v, b, m, n);
    if (P.bias_dt != MI355_DT_UNDEF)
        v += load_float(P.bias_dt, P.bias, b * P.bs[0] + m * P.bs[1] + n * P.bs[2]);
    v = dropout_f(P, v, b * P.ds[0] + m * P.ds[1] + n * P.ds[2]);
    return epilogue_after_bias(P, v, b, m, n);
}

__global__ void __launch_bounds__(256) ref_matmul_kernel(const problem_t P_) {
    const auto &P = MI355_KERNARG_PROBLEM();
    const long total = P.B * P.M * P.N;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
            i += (long)gridDim.x * blockDim.x) {
        const long n = i % P.N, m = (i / P.N) % P.M, b = i / (P.N * P.M);
        const bool int_path = P.src_dt == MI355_DT_S8 || P.src_dt == MI355_DT_U8;
        float v = int_path ? ref_int_dot(P, b, m, n) : ref_fp_dot(P, b, m, n);
        v = ref_epilogue_value(P, v, b, m, n);
        const long off = b * P.ds[0] + m * P.ds[1] + n * P.ds[2];
        // the offset and the seed truncated to 32 bits, ref_matmul.cpp:322-331
        if (P.rnd_flags & MI355_RND_DST_STOCHASTIC)
            v = stochastic_round_f(v, (uint32_t)off, (uint32_t)dropout_seed(P), P.dst_dt);
        store_float(P.dst_dt, v, P.dst, off);
    }
}

// 4-bit dst (f4_e2m1, s4, u4) with static scales: two consecutive n share a
// byte (low nibble first), so one thread computes both and writes the byte.
// The host has checked: N even, unit n stride, even m / batch strides.

__global__ void __launch_bounds__(256) ref_matmul_nibble_dst_kernel(const problem_t P_) {
    const auto &P = MI355_KERNARG_PROBLEM();
    const long half = P.N / 2, total = P.B * P.M * half;
    const bool int_path = P.src_dt == MI355_DT_S8 || P.src_dt == MI355_DT_U8;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const long n = (i % half) * 2, m = (i / half) % P.M, b = i / (half * P.M);
        uint32_t byte = 0;
#pragma unroll 1
        for (int e = 0; e < 2; ++e) {
            const float v = int_path ? ref_int_dot(P, b, m, n + e) : ref_fp_dot(P, b, m, n + e);
            byte |= nibble_code(P.dst_dt, ref_epilogue_value(P, v, b, m, n + e)) << (4 * e);
        }
        ((uint8_t *)P.dst)[(b * P.ds[0] + m * P.ds[1] + n) >> 1] = (uint8_t)byte;
    }
}

// Dynamic (MX) quantization of dst, ref_matmul.cpp:268-423: one thread per
// group of 32 consecutive n of a dst row.  The values of the group are
// computed exactly as above, their largest magnitude gives the group's e8m0
// scale, which is written to the scales tensor and applied by a multiplication
// with its (exact, power of two) inverse.
//
// G == 16: the dynamic_fp (NVFP4) flavour, ref_matmul.cpp:352-365: the scale
// is amax / max(dst type), clamped to [epsilon, max] of f8_e4m3 and rounded to
// it.  A 4-bit dst is written a byte (two consecutive n) at a time.
template <int G>
__global__ void __launch_bounds__(64) ref_matmul_dynamic_kernel(const problem_t P_) {
    const auto &P = MI355_KERNARG_PROBLEM();
    const long groups_n = P.N / G;
    const long total = P.B * P.M * groups_n;
    const float dt_max = P.dst_dt == MI355_DT_F8_E4M3 ? 448.f : P.dst_dt == MI355_DT_F4_E2M1 ? 6.f : 57344.f;
    const bool int_path = P.src_dt == MI355_DT_S8 || P.src_dt == MI355_DT_U8;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const long ng = i % groups_n, m = (i / groups_n) % P.M, b = i / (groups_n * P.M);
        float d[G];
        float amax = 0.f;
#pragma unroll 1
        for (int e = 0; e < G; ++e) {
            const long n = ng * G + e;
            const float v = int_path ? ref_int_dot(P, b, m, n) : ref_fp_dot(P, b, m, n);
            d[e] = ref_epilogue_value(P, v, b, m, n);
        }
#pragma unroll
        for (int e = 0; e < G; ++e) amax = fmaxf(amax, fabsf(d[e]));
        uint8_t sbyte;
        float inv;
        if (G == 32) {
            // e8m0(x): the exponent byte of x
            const float r = e8m0_to_f32(f32_to_e8m0(amax)) / e8m0_to_f32(f32_to_e8m0(dt_max));
            sbyte = f32_to_e8m0(r);
            inv = 1.f / e8m0_to_f32(sbyte);
        } else {
            float r = amax / dt_max;
            r = fmaxf(fminf(r, 448.f), 0.125f);
            sbyte = f32_to_e4m3(r);
            inv = 1.f / e4m3_to_f32(sbyte);
        }
        ((uint8_t *)P.dst_scale.p)[quant_off(P.dst_scale, b, m, ng * G, P.M, P.N)] = sbyte;
        const long off0 = b * P.ds[0] + m * P.ds[1] + ng * G * P.ds[2];
        if (P.dst_dt == MI355_DT_F4_E2M1) {
            // unit n stride, even row offsets (checked by the host): the group is G / 2 whole bytes
#pragma unroll
            for (int e = 0; e < G; e += 2) {
                const float lo = fminf(fmaxf(d[e] * inv, -dt_max), dt_max), hi = fminf(fmaxf(d[e + 1] * inv, -dt_max), dt_max);
                ((uint8_t *)P.dst)[(off0 + e) >> 1] = (uint8_t)(f32_to_e2m1(lo) | (f32_to_e2m1(hi) << 4));
            }
            continue;
        }
#pragma unroll
        for (int e = 0; e < G; ++e) {
            float v = d[e] * inv;
            v = fminf(fmaxf(v, -dt_max), dt_max);
            store_float(P.dst_dt, v, P.dst, off0 + e * P.ds[2]);
        }
    }
}

int ref_supported(const mi355_matmul_desc_t &d) {
    // 4-bit dst: two elements share a byte, and one thread owns both (a thread
    // per byte, or per group under dynamic scales): whole bytes per row needed
    if (dt_bits(d.dst_dt) < 8) {
        if (d.dst_scale_dynamic != MI355_DST_DYNAMIC_NONE && d.dst_dt != MI355_DT_F4_E2M1) return MI355_UNIMPLEMENTED;
        if ((d.N & 1) || d.dst_stride[2] != 1 || (d.dst_stride[1] & 1) || (d.dst_stride[0] & 1)) return MI355_UNIMPLEMENTED;
    }
    if (d.wei_packing != MI355_WEI_PACK_NONE && !woq64_layout_ok(d)) return MI355_UNIMPLEMENTED;
    if (d.rnd_flags != 0) {
        // ref_matmul_t only (floating-point src); the element's offset in dst seeds its random
        // number, which the reference defines for the plain row-major layout (ref_matmul.hpp:131-149)
        if (is_int8_dt(d.src_dt)) return MI355_UNIMPLEMENTED;
        if (d.dst_stride[2] != 1 || d.dst_stride[1] != d.N || (d.batch > 1 && d.dst_stride[0] != d.M * d.N))
            return MI355_UNIMPLEMENTED;
        if (d.rnd_flags & MI355_RND_DST_STOCHASTIC) {
            const bool fp_dst = d.dst_dt == MI355_DT_F32 || d.dst_dt == MI355_DT_BF16 || d.dst_dt == MI355_DT_F16
                    || is_f8_dt(d.dst_dt);
            if (!fp_dst || d.dst_scale_dynamic != MI355_DST_DYNAMIC_NONE) return MI355_UNIMPLEMENTED;
        }
        if ((d.rnd_flags & ~MI355_RND_DST_STOCHASTIC) && !(d.rnd_flags & MI355_RND_DROPOUT)) return MI355_INVALID_ARGUMENTS;
    }
    // dynamic dst quantization exists in ref_matmul_t only, not in the integer implementation
    if (d.dst_scale_dynamic != MI355_DST_DYNAMIC_NONE && is_int8_dt(d.src_dt)) return MI355_UNIMPLEMENTED;
    return MI355_SUCCESS;
}

int ref_launch(const problem_t &P, hipStream_t stream) {
    const long total = P.B * P.M * P.N;
    if (total == 0) return MI355_SUCCESS;
    if (P.dst_dynamic) {
        const int G = P.dst_dynamic == MI355_DST_DYNAMIC_MX ? 32 : 16;
        long groups = total / G, gblocks = (groups + 63) / 64;
        if (gblocks > 1048576) gblocks = 1048576;
        if (G == 32)
            hipLaunchKernelGGL(ref_matmul_dynamic_kernel<32>, dim3((unsigned)gblocks), dim3(64), 0, stream, P);
        else
            hipLaunchKernelGGL(ref_matmul_dynamic_kernel<16>, dim3((unsigned)gblocks), dim3(64), 0, stream, P);
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
    }
    if (dt_bits(P.dst_dt) < 8) {
        long nblocks = (total / 2 + 255) / 256;
        if (nblocks > 1048576) nblocks = 1048576;
        hipLaunchKernelGGL(ref_matmul_nibble_dst_kernel, dim3((unsigned)nblocks), dim3(256), 0, stream, P);
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
    }
    long blocks = (total + 255) / 256;
    if (blocks > 1048576) blocks = 1048576;
    hipLaunchKernelGGL(ref_matmul_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, P);
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
}

} // namespace mi355
