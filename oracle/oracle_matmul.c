/*
 * TEST INFRASTRUCTURE -- CPU oracle, not part of the shipped library.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may use
 * anything in this directory; the product never links or loads it.
 *
 * A plain-C restatement of the two naive matmul implementations of the
 * reference (uxlfoundation/oneDNN v3.14) and of the helpers they call:
 *
 *   orc_int8_dot      ref_matmul_int8_t::execute_ref, the `ker` lambda
 *                     src/cpu/matmul/ref_matmul_int8.cpp:174-261
 *   orc_fp_dot        ref_matmul_t::execute_ref, the `ker` lambda
 *                     src/cpu/matmul/ref_matmul.cpp:168-236
 *   orc_finish        bias + post-ops + dst scale + dst zero point + store
 *                     ref_matmul_int8.cpp:275-306, ref_matmul.cpp:283-331
 *   oracle_dropout / oracle_stochastic_round / oracle_philox4x32
 *                     ref_dropout src/cpu/primitive_attr_postops.cpp:296-310,
 *                     math::stochastic_round_fwd, philox4x32 src/common/math_utils.hpp:458-574
 *   orc_post_ops      ref_post_ops_t::execute src/cpu/primitive_attr_postops.cpp:312-394
 *   orc_eltwise       compute_eltwise_scalar_fwd :49-87 with the formulas of
 *                     src/common/math_utils.hpp:120-430
 *   orc_binary        compute_binary_scalar src/cpu/primitive_attr_postops.cpp:30-47
 *   orc_load_int / orc_load_float / orc_store_float
 *                     io::load_int_value / load_float_value / store_float_value
 *                     src/cpu/ref_io_helper.hpp:34-150 and
 *                     q10n::saturate_and_round src/cpu/simple_q10n.hpp:41-81
 *   oracle_reorder    the generic reorder, simple_reorder_impl_t<..., spec::reference>
 *                     ::execute src/cpu/reorder/simple_reorder.hpp:2579-2661 and
 *                     its 4-bit variants :2168-2288 (f32 -> s4/u4/f4) and
 *                     :2291-2425 (s4/u4/f4 -> f32/bf16/f16)
 *   oracle_inner_product_bwd_data, oracle_inner_product_bwd_weights
 *                     ref_inner_product_bwd_data_t / _bwd_weights_t
 *                     src/cpu/ref_inner_product.cpp:100-217
 *   oracle_sdpa       ref_sdpa, src/gpu/intel/sdpa/ref.cl:21-84 (+ the causal masks of micro.cl:864-878)
 *   oracle_inner_product_fwd
 *                     ref_inner_product_fwd_t::execute_forward src/cpu/ref_inner_product.cpp:33-100
 *                     and ref_inner_product_int8_fwd_t::execute_forward
 *                     src/cpu/ref_inner_product_int8.cpp:34-116
 *   orc_quant_off     quant_entry_t::get_md src/common/primitive_attr_quant.hpp:116-140
 *                     + matmul_helper_t::get_quant_off src/cpu/matmul/matmul_utils.hpp:154-173
 *
 * Implementation choice follows the CPU engine's list
 * (src/cpu/matmul/cpu_matmul_list.cpp:73-109): integer src (s8/u8) takes the
 * s32-accumulating path, every other src the f32 path.
 *
 * Two documented deviations of the reference's JIT path ("brg_matmul") are
 * available as switches because they change bits:
 *   desc->dst_scale_mode == MI355_DST_SCALE_RECIPROCAL:  d *= (1.f/dst_scale)
 *       instead of d /= dst_scale  (src/cpu/x64/matmul/brgemm_matmul.cpp:703-709)
 *   ORC_FLAG_WEI_BF16: decompressed weights are rounded to bf16 before the
 *       multiply (src/cpu/x64/matmul/brgemm_matmul_copy_utils.cpp:2870-2896)
 *
 * Parity status: every function here is pinned by tests/test_oracle_*.py
 * (brute-force int64 loops, closed forms, one-hot decodes, tie vectors, f64
 * restatements with forward error bounds).  The reference cannot be compiled
 * in this environment (its sources need a CMake-generated dnnl_config.h), so
 * no oracle/_ref build exists; see the pinning list in the tests' docstrings.
 * The dynamic (MX) dst quantization (orc_finish_dynamic_group) is pinned by
 * tests/test_dynamic_dst.py: its scale is a pure function of the group's
 * largest magnitude through exponent bytes, restated there with numpy integer
 * arithmetic on the f32 bit patterns and checked on constructed groups
 * (powers of two, just below / above one, zeros, values beyond the dst range).
 * The dynamic_fp branch (f8_e4m3 scales per 16, f4_e2m1 / fp8 dst) is pinned
 * there too: the scale against an exhaustive nearest-value search over the 127
 * positive e4m3 codes on constructed maxima (ties to even, both clamps), the
 * dst codes against a nearest-value search over the type's codes.
 * Dropout and stochastic rounding (oracle_philox4x32*, oracle_dropout,
 * oracle_stochastic_round) are pinned by tests/test_dropout_rounding.py: the
 * Philox core against the known-answer vectors of its authors (Random123) and
 * an independent implementation, the counter / key construction by the block
 * structure it implies, the keep rule where it is decidable by hand, the
 * rounding by representability, neighbourhood, limits and carry probability.
 * The ternary select post-op is pinned by tests/test_oracle_matmul.py (numpy
 * `where` on exact integer sums, three condition types).
 * Precomputed reductions (orc_int8_dot with src_pr, grouped / per-tensor src
 * zero points, true and arbitrary sums), prelu with every weights layout the
 * reference derives, every eltwise and every binary algorithm are pinned by
 * tests/test_oracle_pins.py against closed-form numpy expectations (the
 * formula in f32 with the reference's intermediate roundings; nstl::max / min
 * NaN semantics).
 * The inner product (oracle_inner_product_fwd) is pinned by
 * tests/test_inner_product.py: numpy tensordot over the flattened (ic, spatial)
 * dims on exact data for every ndims and for permuted layouts of src and
 * weights, the scale / bias / dst-scale order on values where a different
 * order changes bits; bias, post-ops and the store are orc_finish.
 * oracle_sdpa is pinned by tests/test_sdpa.py: a float64 numpy softmax(scale * Q K + mask) V for per-head and
 * shared keys / values, broadcast masks, both causal masks (a transposed K, a mask added after the exponential
 * or a diagonal off by one fail it), the inverted scale's rounding on a value where it changes the result.
 * The backward inner products (oracle_inner_product_bwd_data / _bwd_weights)
 * are pinned there too: numpy tensordot on exact data over the other index
 * pair for every ndims and for permuted layouts (a transposed operand or a
 * wrong reduced index changes every element), diff_bias against a column sum
 * and against a hand-ordered f32 sum whose bits depend on the order.
 * Unpinned: none of the functions used by the five benchmark configurations.
 * "Parity unpinned" beyond the textbook formula: the last bits of the
 * libm-dependent eltwise algorithms (tanh, elu, exp, log, pow, gelu_erf,
 * soft_relu, mish, swish, logistic): they agree with float64 evaluations to a
 * few ulp, the reference's own libm bits cannot be pinned without running it.
 */
#include <limits.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "../include/mi355_matmul.h"
#include "oracle_dtypes.h"

#define ORC_FLAG_WEI_BF16 1 /* round decompressed weights to bf16 (JIT flavour) */
#define ORC_FLAG_FOLD_SCALES 2 /* fp path: apply per-tensor scales once after
                                  the K sum (what a GEMM kernel does) */

/* ------------------------------------------------------------------ loads */
static inline int orc_load_int(int dt, const void *p, int64_t off) {
    switch (dt) {
        case MI355_DT_S32: return ((const int32_t *)p)[off];
        case MI355_DT_S8: return ((const int8_t *)p)[off];
        case MI355_DT_U8: return ((const uint8_t *)p)[off];
        case MI355_DT_S4: return orc_s4_to_int(orc_nibble_get(p, off));
        case MI355_DT_U4: return (int)orc_nibble_get(p, off);
        default: return INT_MAX;
    }
}

static inline float orc_load_float(int dt, const void *p, int64_t off) {
    switch (dt) {
        case MI355_DT_F32: return ((const float *)p)[off];
        case MI355_DT_BF16: return orc_bf16_to_f32(((const uint16_t *)p)[off]);
        case MI355_DT_F16: return orc_f16_to_f32(((const uint16_t *)p)[off]);
        case MI355_DT_F8_E4M3: return orc_e4m3_to_f32(((const uint8_t *)p)[off]);
        case MI355_DT_F8_E5M2: return orc_e5m2_to_f32(((const uint8_t *)p)[off]);
        case MI355_DT_E8M0: return orc_e8m0_to_f32(((const uint8_t *)p)[off]);
        case MI355_DT_F4_E2M1: return orc_e2m1_to_f32(orc_nibble_get(p, off));
        case MI355_DT_S32: return (float)((const int32_t *)p)[off];
        case MI355_DT_S8: return (float)((const int8_t *)p)[off];
        case MI355_DT_U8: return (float)((const uint8_t *)p)[off];
        case MI355_DT_S4: return (float)orc_s4_to_int(orc_nibble_get(p, off));
        case MI355_DT_U4: return (float)orc_nibble_get(p, off);
        default: return NAN;
    }
}

static inline float orc_sat(float v, float lo, float hi) {
    if (v < lo) v = lo;
    if (v > hi) v = hi;
    return v;
}

static inline void orc_store_float(int dt, float v, void *p, int64_t off) {
    switch (dt) {
        case MI355_DT_F32: ((float *)p)[off] = v; break;
        case MI355_DT_BF16: ((uint16_t *)p)[off] = orc_f32_to_bf16(v); break;
        case MI355_DT_F16: ((uint16_t *)p)[off] = orc_f32_to_f16(v); break;
        case MI355_DT_F8_E4M3: ((uint8_t *)p)[off] = orc_f32_to_e4m3(v); break;
        case MI355_DT_F8_E5M2: ((uint8_t *)p)[off] = orc_f32_to_e5m2(v); break;
        case MI355_DT_E8M0: ((uint8_t *)p)[off] = orc_f32_to_e8m0(v); break;
        case MI355_DT_F4_E2M1: orc_nibble_set(p, off, orc_f32_to_e2m1(v)); break;
        /* integers: clamp in f32 first, then round to nearest even.  The s32
         * upper bound is the largest float below 2^31
         * (src/common/type_helpers.hpp:232). */
        case MI355_DT_S32:
            ((int32_t *)p)[off]
                    = (int32_t)nearbyintf(orc_sat(v, -2147483648.f, 2147483520.f));
            break;
        case MI355_DT_S8:
            ((int8_t *)p)[off] = (int8_t)nearbyintf(orc_sat(v, -128.f, 127.f));
            break;
        case MI355_DT_U8:
            ((uint8_t *)p)[off] = (uint8_t)nearbyintf(orc_sat(v, 0.f, 255.f));
            break;
        /* int4_t / uint4_t: the same clamp-then-round with the 4-bit limits
         * (src/common/int4.hpp:28-84, type_helpers.hpp max_value/lowest_value) */
        case MI355_DT_S4:
            orc_nibble_set(p, off, (uint8_t)((int)nearbyintf(orc_sat(v, -8.f, 7.f)) & 0xf));
            break;
        case MI355_DT_U4:
            orc_nibble_set(p, off, (uint8_t)((int)nearbyintf(orc_sat(v, 0.f, 15.f)) & 0xf));
            break;
        default: break;
    }
}

/* --------------------------------------------------- quant parameter index */
static inline int64_t orc_quant_off(const mi355_quant_t *q, int64_t b,
        int64_t i0, int64_t i1, int64_t D0, int64_t D1) {
    int64_t q1 = (q->mask & 2) ? D0 / q->group[0] : 1;
    int64_t q2 = (q->mask & 4) ? D1 / q->group[1] : 1;
    int64_t ib = (q->mask & 1) ? b : 0;
    int64_t j0 = (q->mask & 2) ? i0 / q->group[0] : 0;
    int64_t j1 = (q->mask & 4) ? i1 / q->group[1] : 0;
    return (ib * q1 + j0) * q2 + j1;
}

/* number of groups a parameter induces along K; `kdim` = 0/1 is the position
 * of K among the argument's last two dims */
static inline int64_t orc_ngroups_k(const mi355_quant_t *q, int kdim, int64_t K) {
    if (q->dt == MI355_DT_UNDEF) return 1;
    int64_t g = q->group[kdim];
    return g > 1 ? K / g : 1;
}

/* ----------------------------------------------------------------- eltwise */
static float orc_logistic(float s) {
    const float bound = 88.72283172607421875f;
    float in = -s;
    return in < bound ? 1.f / (1.f + expf(in)) : 0.f;
}
static float orc_soft_relu(float s, float alpha) {
    const float bound = 88.72283172607421875f;
    float in = s * alpha;
    float v = in < bound ? log1pf(expf(in)) : in;
    return v / alpha;
}

float orc_eltwise(int alg, float s, float alpha, float beta) {
    switch (alg) {
        case MI355_ELTWISE_RELU: return s > 0 ? s : s * alpha;
        case MI355_ELTWISE_TANH: return tanhf(s);
        case MI355_ELTWISE_ELU: return s > 0 ? s : alpha * expm1f(s);
        case MI355_ELTWISE_SQUARE: return s * s;
        case MI355_ELTWISE_ABS: return s > 0 ? s : -s;
        case MI355_ELTWISE_SQRT: return sqrtf(s);
        case MI355_ELTWISE_LINEAR: return alpha * s + beta;
        case MI355_ELTWISE_SOFT_RELU: return orc_soft_relu(s, alpha);
        case MI355_ELTWISE_HARDSIGMOID: {
            float v = alpha * s + beta;
            return v <= 0.f ? 0.f : v >= 1.f ? 1.f : v;
        }
        case MI355_ELTWISE_LOGISTIC: return orc_logistic(s);
        case MI355_ELTWISE_EXP: return expf(s);
        case MI355_ELTWISE_GELU_TANH: {
            const float sqrt_2_over_pi = 0.79788458347320556640625f;
            const float fit = 0.044715f;
            float v = tanhf(sqrt_2_over_pi * s * (1 + fit * s * s));
            return (float)(0.5 * s * (1. + v)); /* outer product in double */
        }
        case MI355_ELTWISE_SWISH: return s * orc_logistic(alpha * s);
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
        case MI355_ELTWISE_GELU_ERF: {
            const float sqrt_2_over_2 = 0.707106769084930419921875f;
            float v = s * sqrt_2_over_2;
            return 0.5f * s * (1.f + erff(v));
        }
        case MI355_ELTWISE_ROUND: return nearbyintf(s);
        case MI355_ELTWISE_MISH: return s * tanhf(orc_soft_relu(s, 1.f));
        case MI355_ELTWISE_HARDSWISH: {
            float v = alpha * s + beta;
            float h = v <= 0.f ? 0.f : v >= 1.f ? 1.f : v;
            return s * h;
        }
        default: return NAN;
    }
}

float orc_binary(int alg, float x, float y) {
    switch (alg) {
        case MI355_BINARY_ADD: return x + y;
        case MI355_BINARY_DIV: return x / y;
        case MI355_BINARY_MAX: return x > y ? x : y; /* nstl::max: (a > b) ? a : b */
        case MI355_BINARY_MIN: return x < y ? x : y;
        case MI355_BINARY_MUL: return x * y;
        case MI355_BINARY_SUB: return x - y;
        case MI355_BINARY_GE: return x >= y;
        case MI355_BINARY_GT: return x > y;
        case MI355_BINARY_LE: return x <= y;
        case MI355_BINARY_LT: return x < y;
        case MI355_BINARY_EQ: return x == y;
        case MI355_BINARY_NE: return x != y;
        default: return NAN;
    }
}

static float orc_post_ops(const mi355_matmul_desc_t *d,
        const mi355_matmul_args_t *a, float res, float dst_old, int64_t b,
        int64_t m, int64_t n) {
    for (int i = 0; i < d->n_post_ops; ++i) {
        const mi355_post_op_t *po = &d->post_ops[i];
        switch (po->kind) {
            case MI355_PO_SUM:
                res += po->scale * (dst_old - (float)po->zero_point);
                break;
            case MI355_PO_ELTWISE:
                res = orc_eltwise(po->alg, res, po->alpha, po->beta) * po->scale;
                break;
            case MI355_PO_BINARY: {
                int64_t off = b * po->stride[0] + m * po->stride[1]
                        + n * po->stride[2];
                float v = orc_load_float(po->dt, a->po_arg[i], off);
                if (po->alg == MI355_BINARY_SELECT) {
                    /* primitive_attr_postops.cpp:44,345-360: src2 (the entry
                     * that follows) is loaded as an integer; true keeps res */
                    const mi355_post_op_t *c = &d->post_ops[i + 1];
                    int64_t coff = b * c->stride[0] + m * c->stride[1] + n * c->stride[2];
                    res = orc_load_int(c->dt, a->po_arg[i + 1], coff) != 0 ? res : v;
                } else {
                    res = orc_binary(po->alg, res, v);
                }
            } break;
            case MI355_PO_PRELU: {
                if (res >= 0) break;
                int64_t off = b * po->stride[0] + m * po->stride[1]
                        + n * po->stride[2];
                res = ((const float *)a->po_arg[i])[off] * res;
            } break;
            default: break;
        }
    }
    return res;
}

/* ------------------------------------------------------------- int8 path */
static float orc_int8_dot(const mi355_matmul_desc_t *d,
        const mi355_matmul_args_t *a, int64_t b, int64_t m, int64_t n,
        int32_t *last_acc) {
    const int64_t K = d->K, M = d->M, N = d->N;
    const int64_t bs = d->src_stride[0] ? b : 0, bw = d->wei_stride[0] ? b : 0;
    const int with_src_zp = d->src_zp.dt != MI355_DT_UNDEF;
    const int with_wei_zp = d->wei_zp.dt != MI355_DT_UNDEF;
    const int with_src_pr = d->src_pr.dt != MI355_DT_UNDEF;
    const int with_src_sc = d->src_scale.dt != MI355_DT_UNDEF;
    const int with_wei_sc = d->wei_scale.dt != MI355_DT_UNDEF;

    int64_t ng = 1, t;
    if ((t = orc_ngroups_k(&d->src_zp, 1, K)) > ng) ng = t;
    if ((t = orc_ngroups_k(&d->wei_zp, 0, K)) > ng) ng = t;
    if ((t = orc_ngroups_k(&d->src_scale, 1, K)) > ng) ng = t;
    if ((t = orc_ngroups_k(&d->wei_scale, 0, K)) > ng) ng = t;
    if ((t = orc_ngroups_k(&d->src_pr, 1, K)) > ng) ng = t;
    const int64_t gk = K / ng;

    float res = 0.f;
    for (int64_t g = 0; g < ng; ++g) {
        uint32_t acc = 0; /* s32 arithmetic with defined wrap-around */
        int64_t k = g * gk;
        for (int64_t kk = 0; kk < gk; ++kk) {
            k = g * gk + kk;
            int s = orc_load_int(d->src_dt, a->src,
                    bs * d->src_stride[0] + m * d->src_stride[1]
                            + k * d->src_stride[2]);
            int w = orc_load_int(d->wei_dt, a->wei,
                    bw * d->wei_stride[0] + k * d->wei_stride[1]
                            + n * d->wei_stride[2]);
            if (with_src_zp)
                s -= orc_load_int(d->src_zp.dt, a->src_zp,
                        orc_quant_off(&d->src_zp, bs, m, k, M, K));
            if (with_wei_zp && !with_src_pr)
                w -= orc_load_int(d->wei_zp.dt, a->wei_zp,
                        orc_quant_off(&d->wei_zp, bw, k, n, K, N));
            acc += (uint32_t)(s * w);
        }
        if (with_src_pr) {
            /* k is the last index of the group, as in the reference */
            int pr = orc_load_int(d->src_pr.dt, a->src_pr,
                    orc_quant_off(&d->src_pr, bs, m, k, M, K));
            int wzp = orc_load_int(d->wei_zp.dt, a->wei_zp,
                    orc_quant_off(&d->wei_zp, bw, k, n, K, N));
            acc -= (uint32_t)(pr * wzp);
            if (with_src_zp) {
                int szp = orc_load_int(d->src_zp.dt, a->src_zp,
                        orc_quant_off(&d->src_zp, bs, m, k, M, K));
                acc += (uint32_t)(int)(gk * wzp * szp);
            }
        }
        float acc_f = (float)(int32_t)acc;
        if (last_acc) *last_acc = (int32_t)acc;
        if (with_src_sc)
            acc_f *= orc_load_float(d->src_scale.dt, a->src_scale,
                    orc_quant_off(&d->src_scale, bs, m, k, M, K));
        if (with_wei_sc)
            acc_f *= orc_load_float(d->wei_scale.dt, a->wei_scale,
                    orc_quant_off(&d->wei_scale, bw, k, n, K, N));
        res += acc_f;
    }
    return res;
}

/* --------------------------------------------------------------- fp path */
static float orc_fp_dot(const mi355_matmul_desc_t *d,
        const mi355_matmul_args_t *a, int64_t b, int64_t m, int64_t n,
        int flags, double *ideal, double *abs_sum) {
    const int64_t K = d->K, M = d->M, N = d->N;
    const int64_t bs = d->src_stride[0] ? b : 0, bw = d->wei_stride[0] ? b : 0;
    const int wei_is_int = d->wei_dt == MI355_DT_S8 || d->wei_dt == MI355_DT_U8
            || d->wei_dt == MI355_DT_S4 || d->wei_dt == MI355_DT_U4;
    const int decomp = wei_is_int && d->fpmath_apply_to_int;
    const int with_wei_zp = d->wei_zp.dt != MI355_DT_UNDEF;
    const int with_src_sc = d->src_scale.dt != MI355_DT_UNDEF;
    const int with_wei_sc = d->wei_scale.dt != MI355_DT_UNDEF;

    /* get_group() returns 1 when groups are absent, so without groups on
     * both sides every product is its own "group" (ref_matmul.cpp:135-166) */
    int64_t sgk = with_src_sc ? d->src_scale.group[1] : 1;
    int64_t wgk = with_wei_sc ? d->wei_scale.group[0] : 1;
    int64_t ng = K / sgk > K / wgk ? K / sgk : K / wgk;
    int64_t gk = K / ng;
    const int fold = (flags & ORC_FLAG_FOLD_SCALES) && !decomp
            && !(d->src_scale.mask & 4) && !(d->wei_scale.mask & 2);
    if (fold) { ng = 1; gk = K; }

    float res = 0.f;
    double id = 0., as = 0.;
    for (int64_t g = 0; g < ng; ++g) {
        float acc = 0.f;
        double acc_d = 0., acc_a = 0.;
        int64_t k = g * gk;
        for (int64_t kk = 0; kk < gk; ++kk) {
            k = g * gk + kk;
            float s = orc_load_float(d->src_dt, a->src,
                    bs * d->src_stride[0] + m * d->src_stride[1]
                            + k * d->src_stride[2]);
            float w = orc_load_float(d->wei_dt, a->wei,
                    bw * d->wei_stride[0] + k * d->wei_stride[1]
                            + n * d->wei_stride[2]);
            if (decomp) {
                if (with_wei_zp)
                    w -= orc_load_float(d->wei_zp.dt, a->wei_zp,
                            orc_quant_off(&d->wei_zp, bw, k, n, K, N));
                if (with_wei_sc)
                    w *= orc_load_float(d->wei_scale.dt, a->wei_scale,
                            orc_quant_off(&d->wei_scale, bw, k, n, K, N));
                if (flags & ORC_FLAG_WEI_BF16)
                    w = orc_bf16_to_f32(orc_f32_to_bf16(w));
            }
            float p = s * w;
            acc += p;
            acc_d += (double)s * (double)w;
            acc_a += fabs((double)s * (double)w);
        }
        double sc = 1.;
        if (with_src_sc) {
            float v = orc_load_float(d->src_scale.dt, a->src_scale,
                    orc_quant_off(&d->src_scale, bs, m, k, M, K));
            acc *= v;
            sc *= (double)v;
        }
        if (with_wei_sc && !decomp) {
            float v = orc_load_float(d->wei_scale.dt, a->wei_scale,
                    orc_quant_off(&d->wei_scale, bw, k, n, K, N));
            acc *= v;
            sc *= (double)v;
        }
        res += acc;
        id += acc_d * sc;
        as += acc_a * fabs(sc);
    }
    if (ideal) *ideal = id;
    if (abs_sum) *abs_sum = as;
    return res;
}

/* ------------------------------------------- dropout, stochastic rounding */
/* Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3"), the
 * generator of math::philox4x32(idx, seed, offset) src/common/math_utils.hpp:458-506:
 * counter = (offset lo, offset hi, idx & ~3 lo, hi), key = seed; the word idx & 3
 * of the output block is returned. */
void oracle_philox4x32_block(const uint32_t *ctr_in, const uint32_t *key_in, uint32_t *out) {
    uint32_t ctr[4] = {ctr_in[0], ctr_in[1], ctr_in[2], ctr_in[3]};
    uint32_t key[2] = {key_in[0], key_in[1]};
    for (int i = 0; i < 10; ++i) {
        if (i > 0) {
            key[0] += 0x9E3779B9u;
            key[1] += 0xBB67AE85u;
        }
        const uint64_t p0 = (uint64_t)0xD2511F53u * ctr[0], p1 = (uint64_t)0xCD9E8D57u * ctr[2];
        const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
        const uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
        const uint32_t c1 = ctr[1], c3 = ctr[3];
        ctr[0] = hi1 ^ c1 ^ key[0];
        ctr[1] = lo1;
        ctr[2] = hi0 ^ c3 ^ key[1];
        ctr[3] = lo0;
    }
    for (int i = 0; i < 4; ++i) out[i] = ctr[i];
}

uint32_t oracle_philox4x32(uint64_t idx, uint64_t seed, uint64_t offset) {
    const uint64_t x = idx & ~(uint64_t)3;
    const uint32_t ctr[4] = {(uint32_t)offset, (uint32_t)(offset >> 32), (uint32_t)x, (uint32_t)(x >> 32)};
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t out[4];
    oracle_philox4x32_block(ctr, key, out);
    return out[idx & 3];
}

/* the 32-bit flavour, math_utils.hpp:508-515: the counter and the key are
 * built from idx & ~3 and the seed alone (the four indices of a block share
 * one value) */
uint32_t oracle_philox4x32_u32(uint32_t idx, uint32_t seed) {
    const uint64_t x = idx & ~(uint32_t)3;
    const uint64_t idx64 = ((x + 3) << 32) + (x + 2);
    const uint64_t off64 = ((x + 1) << 32) + x;
    const uint64_t seed64 = ((uint64_t)seed << 32) + seed;
    return oracle_philox4x32(idx64, seed64, off64);
}

/* ref_dropout, src/cpu/primitive_attr_postops.cpp:296-310 */
float oracle_dropout(float src, uint8_t *mask, int64_t idx, float p, int64_t seed, int64_t offset) {
    const float inv_q = (p != 1.f) ? 1.f / (1.f - p) : 0.f;
    const uint32_t r = offset ? oracle_philox4x32((uint64_t)idx, (uint64_t)seed, (uint64_t)offset)
                              : oracle_philox4x32_u32((uint32_t)idx, (uint32_t)seed);
    p = fmaxf(fminf(p, 1.f), 0.f);
    const uint8_t m = (double)r > (double)UINT32_MAX * (double)p;
    if (mask) mask[idx] = m;
    return m ? src * inv_q : 0.f;
}

/* math::stochastic_round_fwd, src/common/math_utils.hpp:535-574: `digits` =
 * significand bits of the dst type including the hidden one. */
float oracle_stochastic_round(float s, uint32_t idx, uint32_t seed, int dst_dt) {
    if (s != s) return s;
    int digits;
    float lo, hi, tiny;
    switch (dst_dt) {
        case MI355_DT_F32: digits = 24; hi = 3.40282347e38f; tiny = 1.17549435e-38f; break; /* nothing is truncated */
        case MI355_DT_BF16: digits = 8; hi = 3.38953139e38f; tiny = 1.17549435e-38f; break;
        case MI355_DT_F16: digits = 11; hi = 65504.f; tiny = 6.10351562e-05f; break;
        case MI355_DT_F8_E5M2: digits = 3; hi = 57344.f; tiny = 6.10351562e-05f; break;
        case MI355_DT_F8_E4M3: digits = 4; hi = 448.f; tiny = 0.015625f; break;
        default: return NAN;
    }
    lo = -hi;
    const uint32_t truncation_mask = 0xffffffffu << (24 - digits);
    /* two-byte types take 8 random bits, one-byte types 16 (:560-561) */
    uint32_t rnd;
    if (dst_dt == MI355_DT_BF16 || dst_dt == MI355_DT_F16)
        rnd = (uint8_t)(oracle_philox4x32_u32(idx >> 2, seed) >> ((idx & 3) * 8));
    else
        rnd = (uint16_t)(oracle_philox4x32_u32(idx >> 1, seed) >> ((idx & 1) * 16));
    rnd &= ~truncation_mask;
    uint32_t su;
    memcpy(&su, &s, 4);
    const uint32_t ru = (su + rnd) & truncation_mask;
    float r;
    memcpy(&r, &ru, 4);
    r = fminf(fmaxf(r, lo), hi);
    if (r > 0 && r < tiny) r = 0;
    if (r < 0 && r > -tiny) r = 0;
    return r;
}

static int64_t orc_dropout_seed(const mi355_matmul_desc_t *d, const mi355_matmul_args_t *a) {
    if (!(d->rnd_flags & MI355_RND_DROPOUT)) return 0;
    return (d->rnd_flags & MI355_RND_SEED_S64) ? *(const int64_t *)a->dropout_seed : *(const int32_t *)a->dropout_seed;
}

/* ------------------------------------------------------------- epilogue */
/* bias and post-ops: the value the dst quantization (static or dynamic) sees */
static float orc_pre_quant(const mi355_matmul_desc_t *d,
        const mi355_matmul_args_t *a, float v, int64_t b, int64_t m,
        int64_t n) {
    const int64_t doff
            = b * d->dst_stride[0] + m * d->dst_stride[1] + n * d->dst_stride[2];
    if (d->bias_dt != MI355_DT_UNDEF)
        v += orc_load_float(d->bias_dt, a->bias,
                b * d->bias_stride[0] + m * d->bias_stride[1]
                        + n * d->bias_stride[2]);
    if (d->rnd_flags & MI355_RND_DROPOUT) /* ref_matmul.cpp:293-296 */
        v = oracle_dropout(v, (d->rnd_flags & MI355_RND_DROPOUT_MASK) ? (uint8_t *)a->dropout_mask : NULL, doff,
                *(const float *)a->dropout_p, orc_dropout_seed(d, a),
                (d->rnd_flags & MI355_RND_DROPOUT_OFFSET) ? *(const int64_t *)a->dropout_offset : 0);
    if (d->n_post_ops > 0) {
        float dst_old = 0.f;
        for (int i = 0; i < d->n_post_ops; ++i)
            if (d->post_ops[i].kind == MI355_PO_SUM) {
                int sdt = d->post_ops[i].dt ? d->post_ops[i].dt : d->dst_dt;
                dst_old = orc_load_float(sdt, a->dst, doff);
                break;
            }
        v = orc_post_ops(d, a, v, dst_old, b, m, n);
    }
    return v;
}

static void orc_finish(const mi355_matmul_desc_t *d,
        const mi355_matmul_args_t *a, float v, int64_t b, int64_t m,
        int64_t n) {
    const int64_t doff
            = b * d->dst_stride[0] + m * d->dst_stride[1] + n * d->dst_stride[2];
    v = orc_pre_quant(d, a, v, b, m, n);
    if (d->dst_scale.dt != MI355_DT_UNDEF) {
        float s = orc_load_float(d->dst_scale.dt, a->dst_scale, 0);
        if (d->dst_scale_mode == MI355_DST_SCALE_RECIPROCAL) {
            float r = 1.f / s;
            v *= r;
        } else {
            v /= s;
        }
    }
    if (d->dst_zp.dt != MI355_DT_UNDEF) {
        int z = orc_load_int(MI355_DT_S32, a->dst_zp, (d->dst_zp.mask & 4) ? n : 0);
        v += (float)z;
    }
    if (d->rnd_flags & MI355_RND_DST_STOCHASTIC) /* ref_matmul.cpp:322-331: the offset and the seed truncated to 32 bits */
        v = oracle_stochastic_round(v, (uint32_t)doff, (uint32_t)orc_dropout_seed(d, a), d->dst_dt);
    orc_store_float(d->dst_dt, v, a->dst, doff);
}

/* types::round_to_dt(e8m0, x): through the e8m0 type and back
 * (src/common/type_helpers.hpp:328-350, float8.cpp:29-45) */
static float orc_round_e8m0(float x) {
    return orc_e8m0_to_f32(orc_f32_to_e8m0(x));
}

/* types::max_value<float>(dst type) (type_helpers.hpp:204-221) */
static float orc_dt_max(int dt) {
    switch (dt) {
        case MI355_DT_F8_E4M3: return 448.f;
        case MI355_DT_F8_E5M2: return 57344.f;
        case MI355_DT_F4_E2M1: return 6.f;
        default: return 0.f;
    }
}

/* One group of dynamic (MX or FP) dst quantization, ref_matmul.cpp:268-423: the
 * values `v[0..g)` of columns n0.. of row (b, m), after bias and post-ops. */
static void orc_finish_dynamic_group(const mi355_matmul_desc_t *d,
        const mi355_matmul_args_t *a, const float *v, int g, int64_t b,
        int64_t m, int64_t n0) {
    float max_dst_group = 0.f;
    for (int e = 0; e < g; ++e) max_dst_group = fmaxf(max_dst_group, fabsf(v[e]));
    const float dst_max = orc_dt_max(d->dst_dt);
    float scale;
    if (d->dst_scale_dynamic == MI355_DST_DYNAMIC_FP) {
        /* :352-365: clamped to [epsilon, max] of the scale type f8_e4m3
         * (epsilon = 2^-3, src/common/nstl.hpp:189-191), then rounded to it */
        scale = max_dst_group / dst_max;
        scale = fminf(scale, 448.f);
        scale = fmaxf(scale, 0.125f);
        scale = orc_e4m3_to_f32(orc_f32_to_e4m3(scale));
    } else {
        /* :343-351, the rounding to a power of two happens before the division */
        scale = orc_round_e8m0(max_dst_group) / orc_round_e8m0(dst_max);
        scale = orc_round_e8m0(scale);
    }
    const int64_t soff = orc_quant_off(&d->dst_scale, b, m, n0, d->M, d->N);
    orc_store_float(d->dst_scale.dt, scale, (void *)a->dst_scale, soff); /* :377-378 */
    const float inv = 1.f / scale; /* :381 */
    for (int e = 0; e < g; ++e) {
        float x = v[e] * inv;
        x = fminf(fmaxf(x, -dst_max), dst_max); /* :405-407 */
        orc_store_float(d->dst_dt, x, a->dst,
                b * d->dst_stride[0] + m * d->dst_stride[1] + (n0 + e) * d->dst_stride[2]);
    }
}

static int orc_src_is_int(int dt) {
    return dt == MI355_DT_S8 || dt == MI355_DT_U8;
}

/*
 * Run the matmul described by `d` on host pointers.
 *   flags        ORC_FLAG_*
 *   ideal        optional [batch*M*N] doubles: the pre-bias sum evaluated in
 *                f64 (fp path only)
 *   abs_sum      optional [batch*M*N] doubles: sum of |terms| of that sum, the
 *                scale of its forward rounding error
 */
int oracle_matmul(const mi355_matmul_desc_t *d, const mi355_matmul_args_t *a,
        int flags, double *ideal, double *abs_sum) {
    if (!d || !a) return MI355_INVALID_ARGUMENTS;
    if (d->batch == 0 || d->M == 0 || d->N == 0 || d->K == 0) return MI355_SUCCESS;
    const int int_path = orc_src_is_int(d->src_dt);
    const int64_t B = d->batch, M = d->M, N = d->N;
    if (d->dst_scale_dynamic != MI355_DST_DYNAMIC_NONE) {
        const int g = (int)d->dst_scale.group[1];
        if (g < 1 || g > 64 || N % g) return MI355_INVALID_ARGUMENTS;
#pragma omp parallel for collapse(2) schedule(static)
        for (int64_t b = 0; b < B; ++b)
            for (int64_t m = 0; m < M; ++m)
                for (int64_t n0 = 0; n0 < N; n0 += g) {
                    float v[64];
                    for (int e = 0; e < g; ++e) {
                        const int64_t n = n0 + e;
                        float x;
                        if (int_path) {
                            x = orc_int8_dot(d, a, b, m, n, NULL);
                        } else {
                            int64_t i = (b * M + m) * N + n;
                            x = orc_fp_dot(d, a, b, m, n, flags, ideal ? ideal + i : NULL,
                                    abs_sum ? abs_sum + i : NULL);
                        }
                        v[e] = orc_pre_quant(d, a, x, b, m, n);
                    }
                    orc_finish_dynamic_group(d, a, v, g, b, m, n0);
                }
        return MI355_SUCCESS;
    }
    /* 4-bit dst: two n share a byte, so a thread owns whole rows */
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t b = 0; b < B; ++b)
        for (int64_t m = 0; m < M; ++m)
            for (int64_t n = 0; n < N; ++n) {
                float v;
                if (int_path) {
                    v = orc_int8_dot(d, a, b, m, n, NULL);
                } else {
                    int64_t i = (b * M + m) * N + n;
                    v = orc_fp_dot(d, a, b, m, n, flags, ideal ? ideal + i : NULL,
                            abs_sum ? abs_sum + i : NULL);
                }
                orc_finish(d, a, v, b, m, n);
            }
    return MI355_SUCCESS;
}

/* s32 accumulator only: Sum_k (src - zp_s)(wei - zp_w), for closed-form and
 * brute-force checks of the integer core.  Zero-point and precomputed-
 * reduction groups along K are not meaningful here (one group is reported). */
int oracle_int8_acc(const mi355_matmul_desc_t *d, const mi355_matmul_args_t *a,
        int32_t *acc_out) {
    mi355_matmul_desc_t t = *d;
    t.src_scale.dt = t.wei_scale.dt = MI355_DT_UNDEF;
    t.src_scale.group[0] = t.src_scale.group[1] = 1;
    t.wei_scale.group[0] = t.wei_scale.group[1] = 1;
    if (!orc_src_is_int(d->src_dt)) return MI355_INVALID_ARGUMENTS;
    const int64_t B = d->batch, M = d->M, N = d->N;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t b = 0; b < B; ++b)
        for (int64_t m = 0; m < M; ++m)
            for (int64_t n = 0; n < N; ++n)
                (void)orc_int8_dot(&t, a, b, m, n, &acc_out[(b * M + m) * N + n]);
    return MI355_SUCCESS;
}

/* ------------------------------------------- array conversions for tests */
#define ORC_CVT_LOOP(expr) \
    for (int64_t i = 0; i < n; ++i) { expr; }

void oracle_f32_to_bf16(const float *in, uint16_t *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_f32_to_bf16(in[i]))
}
void oracle_bf16_to_f32(const uint16_t *in, float *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_bf16_to_f32(in[i]))
}
void oracle_f32_to_f16(const float *in, uint16_t *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_f32_to_f16(in[i]))
}
void oracle_f16_to_f32(const uint16_t *in, float *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_f16_to_f32(in[i]))
}
void oracle_f16_to_e4m3(const uint16_t *in, uint8_t *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_f16_to_e4m3(in[i]))
}
void oracle_f32_to_e4m3(const float *in, uint8_t *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_f32_to_e4m3(in[i]))
}
void oracle_e4m3_to_f32(const uint8_t *in, float *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_e4m3_to_f32(in[i]))
}
void oracle_f16_to_e5m2(const uint16_t *in, uint8_t *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_f16_to_e5m2(in[i]))
}
void oracle_f32_to_e5m2(const float *in, uint8_t *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_f32_to_e5m2(in[i]))
}
void oracle_e5m2_to_f32(const uint8_t *in, float *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_e5m2_to_f32(in[i]))
}
void oracle_f32_to_e8m0(const float *in, uint8_t *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_f32_to_e8m0(in[i]))
}
void oracle_e8m0_to_f32(const uint8_t *in, float *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_e8m0_to_f32(in[i]))
}
/* 4-bit arrays: `n` logical elements, packed two per byte, low nibble first */
void oracle_f32_to_e2m1(const float *in, uint8_t *out, int64_t n) {
    ORC_CVT_LOOP(orc_nibble_set(out, i, orc_f32_to_e2m1(in[i])))
}
void oracle_e2m1_to_f32(const uint8_t *in, float *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_e2m1_to_f32(orc_nibble_get(in, i)))
}
void oracle_s4_to_f32(const uint8_t *in, float *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = (float)orc_s4_to_int(orc_nibble_get(in, i)))
}
void oracle_u4_to_f32(const uint8_t *in, float *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = (float)orc_nibble_get(in, i))
}
void oracle_store_float(int dt, const float *in, void *out, int64_t n) {
    ORC_CVT_LOOP(orc_store_float(dt, in[i], out, i))
}
void oracle_load_float(int dt, const void *in, float *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_load_float(dt, in, i))
}
void oracle_eltwise(int alg, float alpha, float beta, const float *in,
        float *out, int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_eltwise(alg, in[i], alpha, beta))
}
void oracle_binary(int alg, const float *x, const float *y, float *out,
        int64_t n) {
    ORC_CVT_LOOP(out[i] = orc_binary(alg, x[i], y[i]))
}

/* ------------------------------------------------------------------ reorder
 * One logical element at a time, in the reference's order of operations:
 *   d = src_scale * (src - src_zp)     (integer sources subtract as integers:
 *                                        `input[i_off] - src_zp_val` with
 *                                        data_t<type_i> promoted to int, :2656;
 *                                        4-bit sources go through float, :2421)
 *   d += beta * dst_old                 (:2657)
 *   d = d / dst_scale + dst_zp          (:2658; skipped when neither is set, as
 *                                        the plain-copy implementations that
 *                                        the reference lists first do)
 *   dst = _qz_a1b0<f32, type_o>()(d)    (:2659) = saturate + nearbyintf for
 *                                        integers, a conversion otherwise
 * e8m0 sources are converted without arithmetic (:2645-2655).
 * Same data type on both sides and no attributes: the value moves unchanged --
 * the reference's copy implementations (spec::direct_copy, :2064-2160, and the
 * JIT reorder that comes first in its list) convert with qz_a1b0_t, which is a
 * plain cast when the source type fits the destination type
 * (simple_q10n.hpp:84-99), where the generic loop would take even an s32 -> s32
 * copy through f32 and lose the low bits of values beyond 2^24.
 * Scale / zero-point offsets: get_quant_off over the logical index with the
 * groups on the last two dims (:2606-2640). */
static int64_t orc_rq_off(const mi355_quant_t *q, const int64_t *idx, int ndims,
        const int64_t *dims) {
    int64_t off = 0, stride = 1;
    for (int d = ndims - 1; d >= 0; --d) {
        int64_t g = 1;
        if (d == ndims - 2) g = q->group[0];
        if (d == ndims - 1) g = q->group[1];
        if (q->mask & (1 << d)) {
            off += (idx[d] / g) * stride;
            stride *= dims[d] / g;
        }
    }
    return off;
}

static int orc_is_int_dt(int dt) {
    return dt == MI355_DT_S32 || dt == MI355_DT_S8 || dt == MI355_DT_U8;
}

int oracle_reorder(const mi355_reorder_desc_t *d, const mi355_reorder_args_t *a) {
    const int nd = d->ndims;
    int64_t total = 1;
    for (int i = 0; i < nd; ++i) total *= d->dims[i];
    const int copy_s32 = d->src_dt == MI355_DT_S32 && d->dst_dt == MI355_DT_S32 && d->beta == 0.f
            && d->src_scale.dt == MI355_DT_UNDEF && d->dst_scale.dt == MI355_DT_UNDEF
            && d->src_zp.dt == MI355_DT_UNDEF && d->dst_zp.dt == MI355_DT_UNDEF;
    for (int64_t l = 0; l < total; ++l) {
        int64_t idx[MI355_REORDER_MAX_DIMS] = {0};
        int64_t rem = l, so = 0, dof = 0;
        for (int i = nd - 1; i >= 0; --i) {
            idx[i] = rem % d->dims[i];
            rem /= d->dims[i];
            so += idx[i] * d->src_stride[i];
            dof += idx[i] * d->dst_stride[i];
        }
        if (copy_s32) { /* (every other type survives the trip through f32 unchanged) */
            ((int32_t *)a->dst)[dof] = ((const int32_t *)a->src)[so];
            continue;
        }
        float x;
        if (d->src_dt == MI355_DT_E8M0) {
            x = orc_load_float(MI355_DT_E8M0, a->src, so);
        } else {
            int zp = 0;
            if (d->src_zp.dt != MI355_DT_UNDEF)
                zp = (int)orc_load_float(d->src_zp.dt, a->src_zp,
                        orc_rq_off(&d->src_zp, idx, nd, d->dims));
            if (orc_is_int_dt(d->src_dt)) x = (float)(orc_load_int(d->src_dt, a->src, so) - zp);
            else x = orc_load_float(d->src_dt, a->src, so) - (float)zp;
            if (d->src_scale.dt != MI355_DT_UNDEF)
                x = orc_load_float(d->src_scale.dt, a->src_scale,
                            orc_rq_off(&d->src_scale, idx, nd, d->dims))
                        * x;
            if (d->beta != 0.f) x += d->beta * orc_load_float(d->dst_dt, a->dst, dof);
            if (d->dst_scale.dt != MI355_DT_UNDEF || d->dst_zp.dt != MI355_DT_UNDEF) {
                float dsc = 1.f;
                int dzp = 0;
                if (d->dst_scale.dt != MI355_DT_UNDEF)
                    dsc = orc_load_float(d->dst_scale.dt, a->dst_scale,
                            orc_rq_off(&d->dst_scale, idx, nd, d->dims));
                if (d->dst_zp.dt != MI355_DT_UNDEF) dzp = orc_load_int(d->dst_zp.dt, a->dst_zp, 0);
                x = x / dsc + (float)dzp;
            }
        }
        orc_store_float(d->dst_dt, x, a->dst, dof);
    }
    return 0;
}

/* Inner product, forward: dst[mb, oc] = sum over (ic, spatial) of
 * src[mb, ic, ...] * weights[oc, ic, ...], both tensors addressed through their
 * own strides (ref_ip_utils::get_data_off / get_weights_off,
 * src/cpu/ref_inner_product_utils.hpp).  `dims` are the src dims
 * (mb, ic, then the spatial dims in the order given), the weights have oc in
 * place of mb.  The loop over the reduced dims runs in the logical row-major
 * order, which is the reference's ic, kd, kh, kw nest.
 *   integer src (ref_inner_product_int8.cpp:64-106): s32 sum; d = (float)acc;
 *     d *= src_scale[0]; d *= wei_scale[mask > 0 ? oc : 0]; bias; post-ops;
 *     d /= dst_scale[0]; store
 *   any other src (ref_inner_product.cpp:52-98): f32 sum of f32 products in
 *     loop order; bias; post-ops; store
 * `e` describes everything after the sum in matmul terms (M = mb, N = oc,
 * batch 1): data types, bias, scales, post-ops, dst strides. */
int oracle_inner_product_fwd(int ndims, const int64_t *dims, int64_t OC, const int64_t *src_stride,
        const int64_t *wei_stride, const mi355_matmul_desc_t *e, const mi355_matmul_args_t *a) {
    if (!dims || !src_stride || !wei_stride || !e || !a || ndims < 2 || ndims > 5) return MI355_INVALID_ARGUMENTS;
    const int64_t MB = dims[0];
    int64_t Kt = 1;
    for (int i = 1; i < ndims; ++i) Kt *= dims[i];
    mi355_matmul_desc_t t = *e;
    t.dst_scale_mode = MI355_DST_SCALE_DIVIDE;
    const int int_path = orc_src_is_int(e->src_dt);
#pragma omp parallel for schedule(static)
    for (int64_t mb = 0; mb < MB; ++mb)
        for (int64_t oc = 0; oc < OC; ++oc) {
            int acc = 0;
            float facc = 0.f;
            for (int64_t k = 0; k < Kt; ++k) {
                int64_t r = k, so = mb * src_stride[0], wo = oc * wei_stride[0];
                for (int i = ndims - 1; i >= 1; --i) {
                    const int64_t idx = r % dims[i];
                    r /= dims[i];
                    so += idx * src_stride[i];
                    wo += idx * wei_stride[i];
                }
                if (int_path) {
                    acc += orc_load_int(e->src_dt, a->src, so) * orc_load_int(e->wei_dt, a->wei, wo);
                } else {
                    const float sv = orc_load_float(e->src_dt, a->src, so);
                    const float wv = orc_load_float(e->wei_dt, a->wei, wo);
                    facc += sv * wv;
                }
            }
            float d = int_path ? (float)acc : facc;
            if (int_path) {
                if (e->src_scale.dt != MI355_DT_UNDEF) d *= orc_load_float(e->src_scale.dt, a->src_scale, 0);
                if (e->wei_scale.dt != MI355_DT_UNDEF)
                    d *= orc_load_float(e->wei_scale.dt, a->wei_scale, e->wei_scale.mask ? oc : 0);
            }
            orc_finish(&t, a, d, 0, mb, oc);
        }
    return MI355_SUCCESS;
}

/* Offset of element k (row-major index over dims[1..]) of row `row` of a tensor
 * [x, ic, spatial...] with the given strides. */
static int64_t orc_ip_off(int ndims, const int64_t *dims, const int64_t *stride, int64_t row, int64_t k) {
    int64_t off = row * stride[0];
    for (int i = ndims - 1; i >= 1; --i) {
        off += (k % dims[i]) * stride[i];
        k /= dims[i];
    }
    return off;
}

/* Inner product, backward by data (ref_inner_product_bwd_data_t::execute_backward_data,
 * src/cpu/ref_inner_product.cpp:100-143):
 *   diff_src[mb, ic, ...] = sum over oc, ascending, of diff_dst[mb, oc] * weights[oc, ic, ...]
 * in f32, stored as diff_src's type.  `dims` are diff_src's dims; dd_stride are
 * the two strides of diff_dst. */
int oracle_inner_product_bwd_data(int ndims, const int64_t *dims, int64_t OC, int dsrc_dt, const int64_t *dsrc_stride,
        void *diff_src, int wei_dt, const int64_t *wei_stride, const void *wei, int dd_dt, const int64_t *dd_stride,
        const void *diff_dst) {
    if (!dims || !dsrc_stride || !wei_stride || !dd_stride || ndims < 2 || ndims > 5) return MI355_INVALID_ARGUMENTS;
    const int64_t MB = dims[0];
    int64_t Kt = 1;
    for (int i = 1; i < ndims; ++i) Kt *= dims[i];
#pragma omp parallel for schedule(static)
    for (int64_t mb = 0; mb < MB; ++mb)
        for (int64_t k = 0; k < Kt; ++k) {
            float ds = 0.f;
            for (int64_t oc = 0; oc < OC; ++oc) {
                const float dd = orc_load_float(dd_dt, diff_dst, mb * dd_stride[0] + oc * dd_stride[1]);
                const float w = orc_load_float(wei_dt, wei, orc_ip_off(ndims, dims, wei_stride, oc, k));
                ds += dd * w;
            }
            orc_store_float(dsrc_dt, ds, diff_src, orc_ip_off(ndims, dims, dsrc_stride, mb, k));
        }
    return MI355_SUCCESS;
}

/* Inner product, backward by weights (ref_inner_product_bwd_weights_t::execute_backward_weights,
 * src/cpu/ref_inner_product.cpp:145-217):
 *   diff_weights[oc, ic, ...] = sum over mb, ascending, of diff_dst[mb, oc] * src[mb, ic, ...]
 *   diff_bias[oc]             = sum over mb, ascending, of diff_dst[mb, oc]       (if diff_bias != NULL)
 * in f32, stored as the outputs' types.  `dims` are src's dims. */
int oracle_inner_product_bwd_weights(int ndims, const int64_t *dims, int64_t OC, int src_dt, const int64_t *src_stride,
        const void *src, int dwei_dt, const int64_t *dwei_stride, void *diff_wei, int dbias_dt, void *diff_bias,
        int dd_dt, const int64_t *dd_stride, const void *diff_dst) {
    if (!dims || !src_stride || !dwei_stride || !dd_stride || ndims < 2 || ndims > 5) return MI355_INVALID_ARGUMENTS;
    const int64_t MB = dims[0];
    int64_t Kt = 1;
    for (int i = 1; i < ndims; ++i) Kt *= dims[i];
#pragma omp parallel for schedule(static)
    for (int64_t oc = 0; oc < OC; ++oc) {
        for (int64_t k = 0; k < Kt; ++k) {
            float dw = 0.f;
            for (int64_t mb = 0; mb < MB; ++mb) {
                const float dd = orc_load_float(dd_dt, diff_dst, mb * dd_stride[0] + oc * dd_stride[1]);
                const float sv = orc_load_float(src_dt, src, orc_ip_off(ndims, dims, src_stride, mb, k));
                dw += dd * sv;
            }
            orc_store_float(dwei_dt, dw, diff_wei, orc_ip_off(ndims, dims, dwei_stride, oc, k));
        }
        if (diff_bias) {
            float db = 0.f;
            for (int64_t mb = 0; mb < MB; ++mb)
                db += orc_load_float(dd_dt, diff_dst, mb * dd_stride[0] + oc * dd_stride[1]);
            orc_store_float(dbias_dt, db, diff_bias, oc);
        }
    }
    return MI355_SUCCESS;
}

/* Scaled dot-product attention, forward: ref_sdpa of src/gpu/intel/sdpa/ref.cl:21-84 loop by loop --
 *   s[k] = sum_h Q[b1, b0, q, h] * K[b1 % kd0, b0 % kd1, h, k]           (f32, h ascending)
 *   s[k] *= scale (the scale read in its type; inverted: 1.f / scale rounded back to that type)
 *   s[k] += mask[b1 % md0, b0 % md1, q, k];  s[k] = exp(s[k]);  sum += s[k]  (k ascending)
 *   s[k] /= sum
 *   dst[b1, b0, q, v] = sum_k V[b1 % vd0, b0 % vd1, k, v] * s[k]          (f32, k ascending)
 * No subtraction of the row maximum, as in the reference.  mask_type 2 / 3: the scores of keys beyond the
 * diagonal (k > q, or k > q + sk - sq) are -inf before the exponential (src/gpu/intel/sdpa/micro.cl:864-878).
 * The mask is indexed modulo its dims in all four positions (the reference: in the first two; the same thing
 * for a mask whose last two dims are full).  dims: {b1, b0, sq, d, sk, dv}; strides in elements, four per tensor. */
int oracle_sdpa(const int64_t *dims, int q_dt, const int64_t *q_st, const void *Q, const int64_t *k_dims01,
        const int64_t *k_st, const void *K, const int64_t *v_dims01, const int64_t *v_st, const void *V, int dst_dt,
        const int64_t *d_st, void *dst, int scale_dt, const void *scale_p, int invert_scale, int mask_type, int mask_dt,
        const int64_t *m_dims, const int64_t *m_st, const void *mask) {
    const int64_t B1 = dims[0], B0 = dims[1], SQ = dims[2], D = dims[3], SK = dims[4], DV = dims[5];
    float scale = 1.f;
    if (scale_dt != MI355_DT_UNDEF) {
        scale = orc_load_float(scale_dt, scale_p, 0);
        if (invert_scale) {
            uint32_t tmp[1] = {0};
            orc_store_float(scale_dt, 1.f / scale, tmp, 0);
            scale = orc_load_float(scale_dt, tmp, 0);
        }
    }
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t b1 = 0; b1 < B1; ++b1)
        for (int64_t b0 = 0; b0 < B0; ++b0) {
            float *s = (float *)malloc(sizeof(float) * (size_t)(SK > 0 ? SK : 1));
            for (int64_t q = 0; q < SQ; ++q) {
                for (int64_t k = 0; k < SK; ++k) {
                    float acc = 0.f;
                    for (int64_t h = 0; h < D; ++h)
                        acc += orc_load_float(q_dt, Q, b1 * q_st[0] + b0 * q_st[1] + q * q_st[2] + h * q_st[3])
                                * orc_load_float(q_dt, K, (b1 % k_dims01[0]) * k_st[0] + (b0 % k_dims01[1]) * k_st[1]
                                        + h * k_st[2] + k * k_st[3]);
                    s[k] = acc;
                }
                float s_sum = 0.f;
                for (int64_t k = 0; k < SK; ++k) {
                    if (scale_dt != MI355_DT_UNDEF) s[k] *= scale;
                    if (mask_type == 1)
                        s[k] += orc_load_float(mask_dt, mask, (b1 % m_dims[0]) * m_st[0] + (b0 % m_dims[1]) * m_st[1]
                                + (q % m_dims[2]) * m_st[2] + (k % m_dims[3]) * m_st[3]);
                    if ((mask_type == 2 && k > q) || (mask_type == 3 && k > q + (SK - SQ))) s[k] = -INFINITY;
                    s[k] = expf(s[k]);
                    s_sum += s[k];
                }
                for (int64_t k = 0; k < SK; ++k) s[k] /= s_sum;
                for (int64_t v = 0; v < DV; ++v) {
                    float acc = 0.f;
                    for (int64_t k = 0; k < SK; ++k)
                        acc += orc_load_float(q_dt, V, (b1 % v_dims01[0]) * v_st[0] + (b0 % v_dims01[1]) * v_st[1]
                                       + k * v_st[2] + v * v_st[3])
                                * s[k];
                    orc_store_float(dst_dt, acc, dst, b1 * d_st[0] + b0 * d_st[1] + q * d_st[2] + v * d_st[3]);
                }
            }
            free(s);
        }
    return MI355_SUCCESS;
}

/* ------------------------------------------------------------- grouped matmul
 * ref_grouped_t::execute, src/cpu/matmul/ref_grouped_gemm.cpp:39-440 -- the
 * offsets validation (:169-212, MI355_INVALID_ARGUMENTS) and the per-group
 * loops (:215-440) in the reference's operation order.  All pointers are host
 * pointers.  Pinned by tests/test_grouped_matmul.py: per-group numpy matmuls on
 * exact data (integer, decompression, fp with power-of-two scales), empty
 * groups, an empty K range that still writes zeros, every binary operand
 * shape, and the offsets the reference refuses. */
int oracle_grouped_matmul(const mi355_grouped_desc_t *d, const mi355_grouped_args_t *a) {
    const int64_t G = d->group_count, N = d->N;
    const int x2 = d->pattern == MI355_GROUPED_2DX2D;
    for (int64_t g = 0; g < G; ++g) {
        if (x2) {
            const int64_t k0 = g == 0 ? 0 : a->src_offsets[g - 1], k1 = a->src_offsets[g];
            if (a->wei_offsets[g] != k1 || (g > 0 && a->wei_offsets[g - 1] != k0) || k0 < 0 || k1 > d->total || k1 < k0)
                return MI355_INVALID_ARGUMENTS;
        } else {
            const int64_t s0 = g == 0 ? 0 : a->src_offsets[g - 1], s1 = a->src_offsets[g];
            const int64_t d0 = g == 0 ? 0 : a->dst_offsets[g - 1], d1 = a->dst_offsets[g];
            if (s0 < 0 || s1 > d->total || s1 < s0 || d0 < 0 || d1 > d->total || d1 < d0) return MI355_INVALID_ARGUMENTS;
            for (int i = 0; i < d->n_post_ops; ++i) {
                const mi355_grouped_post_op_t *po = &d->post_ops[i];
                if (po->kind != MI355_PO_BINARY || !po->grouped) continue;
                const int64_t b0 = g > 0 ? a->po_offsets[i][g - 1] : 0, b1 = a->po_offsets[i][g];
                if (b0 < 0 || b1 > po->bin_m || b1 < b0 || b0 != d0 || b1 != d1) return MI355_INVALID_ARGUMENTS;
            }
        }
    }
    const int int_src = d->src_dt == MI355_DT_S8 || d->src_dt == MI355_DT_U8;
    const int int_wei = d->wei_dt == MI355_DT_S8 || d->wei_dt == MI355_DT_U8 || d->wei_dt == MI355_DT_S4
            || d->wei_dt == MI355_DT_U4;
    const int woq = !int_src && int_wei && d->fpmath_apply_to_int;
    const int64_t Kf = x2 ? 0 : d->K;
#define ORC_NG(dt, gk) ((dt) != MI355_DT_UNDEF && (gk) > 1 ? Kf / (gk) : 1)
    const int64_t ss_ng = ORC_NG(d->src_scale_dt, d->src_scale_gk), ws_ng = ORC_NG(d->wei_scale_dt, d->wei_scale_gk);
    const int64_t sz_ng = ORC_NG(d->src_zp_dt, d->src_zp_gk), wz_ng = ORC_NG(d->wei_zp_dt, d->wei_zp_gk);
#undef ORC_NG
    int64_t nkg = 1;
    if (!x2) {
        nkg = ss_ng > ws_ng ? ss_ng : ws_ng;
        nkg = sz_ng > nkg ? sz_ng : nkg;
        nkg = wz_ng > nkg ? wz_ng : nkg;
    }
#pragma omp parallel for schedule(dynamic)
    for (int64_t g = 0; g < G; ++g) {
        int64_t Mg, Kg, src_start, dst_row0 = 0;
        /* element strides of the inner matmul and the groups' bases (:58-88) */
        int64_t s_sm, s_sk, w_sk, w_sn, d_sm, d_sn, src_base, wei_base, dst_base;
        if (x2) {
            const int64_t k0 = g == 0 ? 0 : a->src_offsets[g - 1];
            Mg = d->M; Kg = a->src_offsets[g] - k0; src_start = k0;
            s_sm = 1; s_sk = d->M; w_sk = N; w_sn = 1; d_sm = d->dst_stride[1]; d_sn = d->dst_stride[2];
            src_base = k0 * d->M; wei_base = k0 * N; dst_base = g * d->dst_stride[0];
        } else {
            const int64_t s0 = g == 0 ? 0 : a->src_offsets[g - 1];
            dst_row0 = g == 0 ? 0 : a->dst_offsets[g - 1];
            Mg = a->src_offsets[g] - s0; Kg = d->K; src_start = s0;
            s_sm = d->K; s_sk = 1; w_sk = d->wei_stride[1]; w_sn = d->wei_stride[2]; d_sm = N; d_sn = 1;
            src_base = s0 * d->K; wei_base = g * d->wei_stride[0]; dst_base = dst_row0 * N;
        }
        if (Mg == 0) continue;
        const int64_t kgs = Kg / nkg;
        for (int64_t m = 0; m < Mg; ++m)
            for (int64_t n = 0; n < N; ++n) {
                float result = 0.0f;
                for (int64_t ig = 0; ig < nkg; ++ig) {
                    float acc = 0.0f;
                    if (int_src || woq) {
                        int zs = 0, zw = 0;
                        float wsc = 1.0f;
                        if (d->src_zp_dt != MI355_DT_UNDEF)
                            zs = orc_load_int(d->src_zp_dt, a->src_zp, (src_start + m) * sz_ng + ig * sz_ng / nkg);
                        if (d->wei_scale_dt != MI355_DT_UNDEF)
                            wsc = orc_load_float(d->wei_scale_dt, a->wei_scale, g * ws_ng * N + (ig * ws_ng / nkg) * N + n);
                        if (d->wei_zp_dt != MI355_DT_UNDEF)
                            zw = orc_load_int(d->wei_zp_dt, a->wei_zp, g * wz_ng * N + (ig * wz_ng / nkg) * N + n);
                        if (int_src) {
                            int acc_int = 0;
                            for (int64_t k = ig * kgs; k < (ig + 1) * kgs; ++k)
                                acc_int += (orc_load_int(d->src_dt, a->src, src_base + m * s_sm + k * s_sk) - zs)
                                        * (orc_load_int(d->wei_dt, a->wei, wei_base + k * w_sk + n * w_sn) - zw);
                            acc = (float)acc_int;
                        } else {
                            for (int64_t k = ig * kgs; k < (ig + 1) * kgs; ++k)
                                acc += orc_load_float(d->src_dt, a->src, src_base + m * s_sm + k * s_sk)
                                        * (float)(orc_load_int(d->wei_dt, a->wei, wei_base + k * w_sk + n * w_sn) - zw);
                        }
                        if (d->src_scale_dt != MI355_DT_UNDEF)
                            acc *= orc_load_float(d->src_scale_dt, a->src_scale, (src_start + m) * ss_ng + ig * ss_ng / nkg);
                        result += acc * wsc;
                    } else {
                        for (int64_t k = ig * kgs; k < (ig + 1) * kgs; ++k)
                            acc += orc_load_float(d->src_dt, a->src, src_base + m * s_sm + k * s_sk)
                                    * orc_load_float(d->wei_dt, a->wei, wei_base + k * w_sk + n * w_sn);
                        if (d->src_scale_dt != MI355_DT_UNDEF)
                            acc *= orc_load_float(d->src_scale_dt, a->src_scale, (src_start + m) * ss_ng + ig * ss_ng / nkg);
                        if (d->wei_scale_dt != MI355_DT_UNDEF)
                            acc *= orc_load_float(d->wei_scale_dt, a->wei_scale, g * ws_ng * N + (ig * ws_ng / nkg) * N + n);
                        result += acc;
                    }
                }
                if (d->bias_dt != MI355_DT_UNDEF) result += orc_load_float(d->bias_dt, a->bias, g * N + n);
                for (int i = 0; i < d->n_post_ops; ++i) {
                    const mi355_grouped_post_op_t *po = &d->post_ops[i];
                    if (po->kind == MI355_PO_ELTWISE) {
                        result = orc_eltwise(po->alg, result, po->alpha, po->beta) * po->scale;
                    } else {
                        int64_t row_base = dst_row0;
                        if (po->grouped) row_base = g > 0 ? a->po_offsets[i][g - 1] : 0;
                        const int per_group = po->bin_m == G && po->bin_n == 1;
                        const int64_t em = per_group ? g : row_base + m, en = po->bin_n > 1 ? n : 0;
                        result = orc_binary(po->alg, result, orc_load_float(po->dt, a->po_arg[i], em * po->bin_n + en));
                    }
                }
                orc_store_float(d->dst_dt, result, a->dst, dst_base + m * d_sm + n * d_sn);
            }
    }
    return MI355_SUCCESS;
}
