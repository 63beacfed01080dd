// Device-side problem description and the fused epilogue shared by every
// kernel family.  The order of operations is the reference's
// (src/cpu/matmul/ref_matmul_int8.cpp:275-306, src/cpu/matmul/ref_matmul.cpp:283-331,
// JIT: src/cpu/x64/brgemm/jit_brgemm_kernel.cpp:1839-2010):
//   (+ bias) -> post-ops in attr order -> dst scale -> dst zero point ->
//   saturate -> round-to-nearest-even store.
// All device code is compiled with -ffp-contract=off: each written multiply
// and add rounds once, as in the reference's scalar code.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mi355_matmul.h"
#include "mi355_dtypes.hpp"

namespace mi355 {

struct quant_dev_t {
    int dt, mask;
    long g0, g1;
    const void *p;
};

struct po_dev_t {
    int kind, alg;
    float alpha, beta, scale;
    int zp, dt, pad;
    long s0, s1, s2;
    const void *p;
};

struct problem_t {
    long B, M, N, K;
    int src_dt, wei_dt, dst_dt, bias_dt;
    long ss[3], ws[3], ds[3], bs[3];
    quant_dev_t src_scale, wei_scale, dst_scale, src_zp, wei_zp, dst_zp, src_pr;
    int apply_to_int, dst_scale_mode, n_po, sum_dt;
    int wei_packing, dst_dynamic;
    const void *src, *wei, *bias;
    void *dst;
    po_dev_t po[MI355_MAX_POST_OPS];
    // dropout and stochastic rounding (generic kernel only)
    int rnd_flags; // MI355_RND_*
    const void *drop_p, *drop_seed, *drop_offset;
    void *drop_mask;
};

// The problem description is the first kernel argument of every kernel.  It is
// read in place from the kernarg segment (constant address space): indexing
// the post-op list with a loop counter then compiles to scalar loads instead
// of a private-memory copy of the whole structure.
typedef const __attribute__((address_space(4))) problem_t kernarg_problem_t;
#define MI355_KERNARG_PROBLEM() \
    (*(kernarg_problem_t *)__builtin_amdgcn_kernarg_segment_ptr())

__device__ __forceinline__ int load_int(int dt, const void *p, long off) {
    switch (dt) {
        case MI355_DT_S32: return ((const int *)p)[off];
        case MI355_DT_S8: return ((const int8_t *)p)[off];
        case MI355_DT_U8: return ((const uint8_t *)p)[off];
        case MI355_DT_S4: return s4_to_int(nibble_get(p, off));
        case MI355_DT_U4: return (int)nibble_get(p, off);
        default: return 0x7fffffff;
    }
}

__device__ __forceinline__ float load_float(int dt, const void *p, long off) {
    switch (dt) {
        case MI355_DT_F32: return ((const float *)p)[off];
        case MI355_DT_BF16: return bf16_to_f32(((const uint16_t *)p)[off]);
        case MI355_DT_F16: return f16_to_f32(((const uint16_t *)p)[off]);
        case MI355_DT_F8_E4M3: return e4m3_to_f32(((const uint8_t *)p)[off]);
        case MI355_DT_F8_E5M2: return e5m2_to_f32(((const uint8_t *)p)[off]);
        case MI355_DT_E8M0: return e8m0_to_f32(((const uint8_t *)p)[off]);
        case MI355_DT_F4_E2M1: return e2m1_to_f32(nibble_get(p, off));
        case MI355_DT_S32: return (float)((const int *)p)[off];
        case MI355_DT_S8: return (float)((const int8_t *)p)[off];
        case MI355_DT_U8: return (float)((const uint8_t *)p)[off];
        case MI355_DT_S4: return (float)s4_to_int(nibble_get(p, off));
        case MI355_DT_U4: return (float)nibble_get(p, off);
        default: return __builtin_nanf("");
    }
}

__device__ __forceinline__ float sat(float v, float lo, float hi) {
    // same comparison order as q10n::saturate (src/cpu/simple_q10n.hpp:41-52):
    // NaN falls through both tests
    if (v < lo) v = lo;
    if (v > hi) v = hi;
    return v;
}

// Convert to the (byte-or-wider) dst type and return the raw bits.
__device__ __forceinline__ uint32_t cvt_store_bits(int dt, float v) {
    switch (dt) {
        case MI355_DT_F32: return f2u(v);
        case MI355_DT_BF16: return f32_to_bf16(v);
        case MI355_DT_F16: return f32_to_f16(v);
        case MI355_DT_F8_E4M3: return f32_to_e4m3(v);
        case MI355_DT_F8_E5M2: return f32_to_e5m2(v);
        case MI355_DT_E8M0: return f32_to_e8m0(v);
        case MI355_DT_S32:
            return (uint32_t)(int)__builtin_rintf(sat(v, -2147483648.f, 2147483520.f));
        case MI355_DT_S8:
            return (uint32_t)(int)__builtin_rintf(sat(v, -128.f, 127.f)) & 0xffu;
        case MI355_DT_U8:
            return (uint32_t)(int)__builtin_rintf(sat(v, 0.f, 255.f)) & 0xffu;
        default: return 0;
    }
}

// the four bits of a 4-bit dst value (f4_e2m1, s4, u4): saturated, rounded to nearest even
__device__ __forceinline__ uint32_t nibble_code(int dt, float v) {
    switch (dt) {
        case MI355_DT_F4_E2M1: return f32_to_e2m1(v);
        case MI355_DT_S4: return (uint32_t)(int)__builtin_rintf(sat(v, -8.f, 7.f)) & 0xfu;
        default: return (uint32_t)(int)__builtin_rintf(sat(v, 0.f, 15.f)) & 0xfu;
    }
}

__device__ __forceinline__ void store_float(int dt, float v, void *p, long off) {
    const uint32_t bits = cvt_store_bits(dt, v);
    switch (dt) {
        case MI355_DT_F32:
        case MI355_DT_S32: ((uint32_t *)p)[off] = bits; break;
        case MI355_DT_BF16:
        case MI355_DT_F16: ((uint16_t *)p)[off] = (uint16_t)bits; break;
        default: ((uint8_t *)p)[off] = (uint8_t)bits; break;
    }
}

__host__ __device__ __forceinline__ int dt_bits(int dt) {
    switch (dt) {
        case MI355_DT_F32:
        case MI355_DT_S32: return 32;
        case MI355_DT_BF16:
        case MI355_DT_F16: return 16;
        case MI355_DT_S4:
        case MI355_DT_U4:
        case MI355_DT_F4_E2M1: return 4;
        case MI355_DT_F64: return 64;
        default: return 8;
    }
}

template <class Q>
__device__ __forceinline__ long quant_off(
        const Q &q, long b, long i0, long i1, long D0, long D1) {
    const long q1 = (q.mask & 2) ? D0 / q.g0 : 1;
    const long q2 = (q.mask & 4) ? D1 / q.g1 : 1;
    const long ib = (q.mask & 1) ? b : 0;
    const long j0 = (q.mask & 2) ? i0 / q.g0 : 0;
    const long j1 = (q.mask & 4) ? i1 / q.g1 : 0;
    return (ib * q1 + j0) * q2 + j1;
}

// Eltwise formulas of src/common/math_utils.hpp:120-430.
__device__ __forceinline__ float logistic_f(float s) {
    const float in = -s;
    return in < 88.72283172607421875f ? 1.f / (1.f + expf(in)) : 0.f;
}
__device__ __forceinline__ float soft_relu_f(float s, float alpha) {
    const float in = s * alpha;
    const float v = in < 88.72283172607421875f ? log1pf(expf(in)) : in;
    return v / alpha;
}

__device__ __forceinline__ float eltwise_f(int alg, float s, float alpha, float beta) {
    switch (alg) {
        case MI355_ELTWISE_RELU: return s > 0 ? s : s * alpha;
        case MI355_ELTWISE_TANH: return tanhf(s);
        case MI355_ELTWISE_ELU: return s > 0 ? s : alpha * expm1f(s);
        case MI355_ELTWISE_SQUARE: return s * s;
        case MI355_ELTWISE_ABS: return s > 0 ? s : -s;
        case MI355_ELTWISE_SQRT: return sqrtf(s);
        case MI355_ELTWISE_LINEAR: return alpha * s + beta;
        case MI355_ELTWISE_SOFT_RELU: return soft_relu_f(s, alpha);
        case MI355_ELTWISE_HARDSIGMOID: {
            const float v = alpha * s + beta;
            return v <= 0.f ? 0.f : v >= 1.f ? 1.f : v;
        }
        case MI355_ELTWISE_LOGISTIC: return logistic_f(s);
        case MI355_ELTWISE_EXP: return expf(s);
        case MI355_ELTWISE_GELU_TANH: {
            const float v = tanhf(0.79788458347320556640625f * s * (1 + 0.044715f * s * s));
            // the reference evaluates the outer product in double
            return (float)(0.5 * (double)s * (1. + (double)v));
        }
        case MI355_ELTWISE_SWISH: return s * logistic_f(alpha * s);
        case MI355_ELTWISE_LOG: return logf(s);
        case MI355_ELTWISE_CLIP: {
            s = s > alpha ? s : alpha;
            return s > beta ? beta : s;
        }
        case MI355_ELTWISE_CLIP_V2: {
            s = s > alpha ? s : alpha;
            return s < beta ? s : beta;
        }
        case MI355_ELTWISE_POW: return alpha * powf(s, beta);
        case MI355_ELTWISE_GELU_ERF:
            return 0.5f * s * (1.f + erff(s * 0.707106769084930419921875f));
        case MI355_ELTWISE_ROUND: return __builtin_rintf(s);
        case MI355_ELTWISE_MISH: return s * tanhf(soft_relu_f(s, 1.f));
        case MI355_ELTWISE_HARDSWISH: {
            const float v = alpha * s + beta;
            const float h = v <= 0.f ? 0.f : v >= 1.f ? 1.f : v;
            return s * h;
        }
        default: return __builtin_nanf("");
    }
}

__device__ __forceinline__ float binary_f(int alg, float x, float y) {
    switch (alg) {
        case MI355_BINARY_ADD: return x + y;
        case MI355_BINARY_DIV: return x / y;
        case MI355_BINARY_MAX: return x > y ? x : y;
        case MI355_BINARY_MIN: return x < y ? x : y;
        case MI355_BINARY_MUL: return x * y;
        case MI355_BINARY_SUB: return x - y;
        case MI355_BINARY_GE: return x >= y;
        case MI355_BINARY_GT: return x > y;
        case MI355_BINARY_LE: return x <= y;
        case MI355_BINARY_LT: return x < y;
        case MI355_BINARY_EQ: return x == y;
        case MI355_BINARY_NE: return x != y;
        default: return __builtin_nanf("");
    }
}

// ---- dropout and stochastic rounding of ref_matmul_t (src/cpu/matmul/ref_matmul.cpp:283-331)
// Philox4x32-10 as math::philox4x32 uses it (src/common/math_utils.hpp:458-515)
__device__ __forceinline__ uint32_t philox4x32(uint64_t idx, uint64_t seed, uint64_t offset) {
    const uint64_t x = idx & ~(uint64_t)3;
    uint32_t ctr[4] = {(uint32_t)offset, (uint32_t)(offset >> 32), (uint32_t)x, (uint32_t)(x >> 32)};
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
#pragma unroll
    for (int i = 0; i < 10; ++i) {
        if (i > 0) {
            key[0] += 0x9E3779B9u;
            key[1] += 0xBB67AE85u;
        }
        const uint64_t p0 = (uint64_t)0xD2511F53u * ctr[0], p1 = (uint64_t)0xCD9E8D57u * ctr[2];
        const uint32_t c1 = ctr[1], c3 = ctr[3];
        ctr[0] = (uint32_t)(p1 >> 32) ^ c1 ^ key[0];
        ctr[1] = (uint32_t)p1;
        ctr[2] = (uint32_t)(p0 >> 32) ^ c3 ^ key[1];
        ctr[3] = (uint32_t)p0;
    }
    const int w = (int)(idx & 3);
    return w == 0 ? ctr[0] : w == 1 ? ctr[1] : w == 2 ? ctr[2] : ctr[3];
}

__device__ __forceinline__ uint32_t philox4x32_u32(uint32_t idx, uint32_t seed) {
    const uint64_t x = idx & ~(uint32_t)3;
    return philox4x32(((x + 3) << 32) + (x + 2), ((uint64_t)seed << 32) + seed, ((x + 1) << 32) + x);
}

template <class PT>
__device__ __forceinline__ long dropout_seed(const PT &P) {
    if (!(P.rnd_flags & MI355_RND_DROPOUT)) return 0;
    return (P.rnd_flags & MI355_RND_SEED_S64) ? *(const long *)P.drop_seed : (long)*(const int *)P.drop_seed;
}

// ref_dropout, src/cpu/primitive_attr_postops.cpp:296-310; idx = the element's offset in dst
template <class PT>
__device__ __forceinline__ float dropout_f(const PT &P, float v, long idx) {
    float p = *(const float *)P.drop_p;
    const long seed = dropout_seed(P);
    const long offset = (P.rnd_flags & MI355_RND_DROPOUT_OFFSET) ? *(const long *)P.drop_offset : 0;
    const float inv_q = (p != 1.f) ? 1.f / (1.f - p) : 0.f;
    const uint32_t r = offset ? philox4x32((uint64_t)idx, (uint64_t)seed, (uint64_t)offset)
                              : philox4x32_u32((uint32_t)idx, (uint32_t)seed);
    p = fmaxf(fminf(p, 1.f), 0.f);
    const bool keep = (double)r > 4294967295.0 * (double)p;
    if (P.rnd_flags & MI355_RND_DROPOUT_MASK) ((uint8_t *)P.drop_mask)[idx] = keep;
    return keep ? v * inv_q : 0.f;
}

// math::stochastic_round_fwd, src/common/math_utils.hpp:535-574
__device__ __forceinline__ float stochastic_round_f(float s, uint32_t idx, uint32_t seed, int dst_dt) {
    if (s != s) return s;
    int digits;
    float hi, tiny;
    switch (dst_dt) {
        case MI355_DT_F32: digits = 24; hi = 3.40282347e38f; tiny = 1.17549435e-38f; break;
        case MI355_DT_BF16: digits = 8; hi = 3.38953139e38f; tiny = 1.17549435e-38f; break;
        case MI355_DT_F16: digits = 11; hi = 65504.f; tiny = 6.10351562e-05f; break;
        case MI355_DT_F8_E5M2: digits = 3; hi = 57344.f; tiny = 6.10351562e-05f; break;
        case MI355_DT_F8_E4M3: digits = 4; hi = 448.f; tiny = 0.015625f; break;
        default: return __builtin_nanf("");
    }
    const uint32_t truncation_mask = 0xffffffffu << (24 - digits);
    uint32_t rnd;
    if (dst_dt == MI355_DT_BF16 || dst_dt == MI355_DT_F16)
        rnd = (philox4x32_u32(idx >> 2, seed) >> ((idx & 3) * 8)) & 0xffu;
    else
        rnd = (philox4x32_u32(idx >> 1, seed) >> ((idx & 1) * 16)) & 0xffffu;
    rnd &= ~truncation_mask;
    float r = u2f((f2u(s) + rnd) & truncation_mask);
    r = fminf(fmaxf(r, -hi), hi);
    if (r > 0 && r < tiny) r = 0;
    if (r < 0 && r > -tiny) r = 0;
    return r;
}

// Everything after the K reduction except the store: returns the f32 value
// that store_float() converts.
template <class PT>
__device__ __forceinline__ float epilogue_after_bias(const PT &P, float v, long b, long m, long n);

template <class PT>
__device__ __forceinline__ float epilogue_value(
        const PT &P, float v, long b, long m, long n) {
    if (P.bias_dt != MI355_DT_UNDEF)
        v += load_float(P.bias_dt, P.bias, b * P.bs[0] + m * P.bs[1] + n * P.bs[2]);
    return epilogue_after_bias(P, v, b, m, n);
}

// post-ops, dst scale and dst zero point
template <class PT>
__device__ __forceinline__ float epilogue_after_bias(const PT &P, float v, long b, long m, long n) {
    if (P.n_po > 0) {
        float dst_old = 0.f;
        if (P.sum_dt != MI355_DT_UNDEF)
            dst_old = load_float(P.sum_dt, P.dst, b * P.ds[0] + m * P.ds[1] + n * P.ds[2]);
        for (int i = 0; i < P.n_po; ++i) {
            const auto &po = P.po[i];
            if (po.kind == MI355_PO_ELTWISE) {
                v = eltwise_f(po.alg, v, po.alpha, po.beta) * po.scale;
            } else if (po.kind == MI355_PO_BINARY) {
                const float y = load_float(po.dt, po.p, b * po.s0 + m * po.s1 + n * po.s2);
                if (po.alg == MI355_BINARY_SELECT) {
                    // the next entry holds the condition (checked by the host)
                    const auto &c = P.po[i + 1];
                    v = load_int(c.dt, c.p, b * c.s0 + m * c.s1 + n * c.s2) != 0 ? v : y;
                } else {
                    v = binary_f(po.alg, v, y);
                }
            } else if (po.kind == MI355_PO_SUM) {
                v += po.scale * (dst_old - (float)po.zp);
            } else if (po.kind == MI355_PO_PRELU) {
                if (!(v >= 0)) v = ((const float *)po.p)[b * po.s0 + m * po.s1 + n * po.s2] * v;
            }
        }
    }
    if (P.dst_dynamic) return v; // the group's scale is computed from these values
    if (P.dst_scale.dt != MI355_DT_UNDEF) {
        const float s = load_float(P.dst_scale.dt, P.dst_scale.p, 0);
        if (P.dst_scale_mode == MI355_DST_SCALE_RECIPROCAL) {
            const float r = 1.f / s;
            v *= r;
        } else {
            v /= s;
        }
    }
    if (P.dst_zp.dt != MI355_DT_UNDEF)
        v += (float)((const int *)P.dst_zp.p)[(P.dst_zp.mask & 4) ? n : 0];
    return v;
}

template <class PT>
__device__ __forceinline__ void epilogue_store(
        const PT &P, float v, long b, long m, long n) {
    v = epilogue_value(P, v, b, m, n);
    store_float(P.dst_dt, v, P.dst, b * P.ds[0] + m * P.ds[1] + n * P.ds[2]);
}

} // namespace mi355
