// Epilogue of the LDS-tiled MFMA kernels.
//
// The kernels issue their MFMAs with the operands exchanged (weights columns as
// the instruction's A operand, src rows as its B operand), so that the
// accumulators hold the dst tile transposed inside every MFMA tile: a lane owns
// FOUR CONSECUTIVE n OF ONE ROW m per accumulator quad,
//   16x16 tiles: acc[i][j][r]  = dst(m = 16 i + lane % 16, n = 16 j + 4 (lane / 16) + r)
//   32x32 tiles: acc[i][j][r]  = dst(m = 32 i + lane % 32, n = 32 j + 8 (r / 4) + 4 (lane / 32) + r % 4)
// which is exactly the unit the epilogue arithmetic and the dst stores want
// (4 / 8 / 16 bytes of one dst row per lane).  Nothing is transposed through
// LDS and no wavefront waits for another one after the K loop.
//
// Operands of the epilogue:
//   * per column n (weights scales, zero-point compensation terms, per-n bias,
//     one per-n binary post-op operand, dst zero points): converted to f32 / s32
//     once per workgroup into a small LDS table at kernel start -- the loads
//     hide behind the pipeline prologue -- and read back 16 bytes per quad;
//   * per row m (row sums for the weights zero points, per-row src scales):
//     one value per lane and row block, loaded a row block ahead;
//   * one per-element stream (binary post-op src1, the old dst of a sum
//     post-op, a per-element bias; 16- or 32-bit elements): loaded straight
//     into registers a row block ahead, 8 / 16 bytes per lane and quad;
//   * everything else: loaded where it is used, by the general path.
//
// Two paths per wavefront: the fast one (all of the above covers every
// operand, the post-ops are among relu / linear / clip / gelu_tanh / binary
// add|mul / sum, the wavefront's columns lie inside N, dst takes vector stores)
// works on the Q quads of a row block at once with every array index a
// compile-time constant; the general one parks the quads in lane-private LDS and
// interprets any post-op chain quad by quad.
//
// Order of operations: ref_matmul_int8.cpp:275-306 / ref_matmul.cpp:283-331.
#pragma once
#include "mi355_device.hpp"

namespace mi355 {
namespace gemm {

typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef float v4f_t __attribute__((ext_vector_type(4)));
typedef uint4 __attribute__((may_alias)) park_u4_t;

__device__ __forceinline__ int raw_bits(int x) { return x; }
__device__ __forceinline__ int raw_bits(float x) { return __float_as_int(x); }

constexpr int STG_NONE = -1, STG_BIAS = 100, STG_SUM = 101;

// ---- the per-column operand table in LDS: NTAB_SLOTS rows of 256 dwords
constexpr int NT_WSC = 0, NT_CC = 1, NT_C = 2, NT_BIAS = 3, NT_HV = 4, NT_DZP = 5, NTAB_SLOTS = 6;
constexpr int NTAB_COLS = 256;
constexpr int NTAB_BYTES = NTAB_SLOTS * NTAB_COLS * 4;

typedef const v4i_t __attribute__((address_space(3))) *lds_q_ptr_t;
__device__ __forceinline__ v4i_t nt4i(unsigned ntab, int slot, int col) {
    return *(lds_q_ptr_t)(size_t)(ntab + (unsigned)((slot * NTAB_COLS + col) * 4));
}
__device__ __forceinline__ v4f_t nt4f(unsigned ntab, int slot, int col) {
    const v4i_t v = nt4i(ntab, slot, col);
    return v4f_t {__int_as_float(v[0]), __int_as_float(v[1]), __int_as_float(v[2]), __int_as_float(v[3])};
}

// gelu_tanh(s) = 0.5 s (1 + tanh(v)), v = sqrt(2/pi) s (1 + 0.044715 s^2)
// (math_utils.hpp gelu_tanh_fwd), evaluated as s / (1 + exp(-2v)): the same
// real function without the cancellation of 1 + tanh(v) for negative v, in one
// hardware exponential and one reciprocal (a few ulp, like the polynomial
// evaluation of the reference's JIT injector; the generic kernel keeps the
// libm form of the reference's scalar code).
__device__ __forceinline__ float gelu_tanh_fast(float s) {
    const float v = 0.79788458347320556640625f * s * (1.f + 0.044715f * s * s);
    const float e = __builtin_amdgcn_exp2f(-2.8853900817779268f * v); // exp(-2v)
    return s * __builtin_amdgcn_rcpf(1.f + e);
}
// logistic(s) = 1 / (1 + exp(-s)) and swish(s) = s logistic(alpha s)
// (math_utils.hpp logistic_fwd, swish_fwd) the same way.  Where s is negative
// the result is exp(s) to first order, so the exponential has to be good to a
// few ulp by itself: the rounding of the product s log2(e) (|s| 2^-24 in the
// exponent) is recovered by an fma and applied to first order,
// exp2(hi + lo) = exp2(hi) (1 + lo ln 2).  exp(-s) overflows to infinity where
// the reference returns 0 outright, and the reciprocal of that is the same 0.
__device__ __forceinline__ float logistic_fast(float s) {
    const float c = -1.44269502162933349609375f; // -log2(e) rounded; the rest of it follows
    const float hi = c * s;
    float lo = __builtin_fmaf(c, s, -hi);
    lo = __builtin_fmaf(-1.92596299e-8f, s, lo);
    float e = __builtin_amdgcn_exp2f(hi);
    // (outside: e is 0 or infinity, or s is not finite, and the correction would make NaN of it)
    if (fabsf(hi) < 126.f) e = __builtin_fmaf(e, lo * 0.693147182464599609375f, e);
    return __builtin_amdgcn_rcpf(1.f + e);
}

// x / s by two Newton corrections of x * (1 / s):
//   q0 = x y, r0 = x - s q0 (one fma, exact), q1 = q0 + r0 y, r1 = x - s q1, q = q1 + r1 y
// with y = 1 / s correctly rounded (one IEEE division per lane, outside the
// loop).  q1 is within an ulp of x / s, and then the last step returns the
// correctly rounded quotient (Markstein's theorem for division by fma
// correction: y correctly rounded, q1 faithful, the remainder exact) -- five
// instructions instead of the dozen of an IEEE division.  Used for integer dst
// types only, with 2^-20 <= |s| <= 2^20 and |x| < 2^100 (NaN excluded):
//   * 2^-90 <= |x| < 2^100: nothing under- or overflows, the remainders are
//     exact, the result is the IEEE quotient (checked on the host for the
//     benchmark's scale over every such x, and for random scales);
//   * |x| < 2^-90: every intermediate stays below 2^-69, so the quotient, like
//     the IEEE one, vanishes in the rounding to an integer that follows (a dst
//     zero point is added after the division and absorbs it the same way);
//   * the sign of a zero quotient is not preserved (x = -0 gives +0), which an
//     integer dst does not see.
// A wavefront that holds a larger, infinite or NaN value divides instead.
__device__ __forceinline__ float div_by_fma(float x, float s, float y) {
    const float q0 = x * y;
    const float r0 = __builtin_fmaf(-s, q0, x);
    const float q1 = __builtin_fmaf(r0, y, q0);
    const float r1 = __builtin_fmaf(-s, q1, x);
    return __builtin_fmaf(r1, y, q1);
}
// |x| >= 2^100, infinite or NaN, as one unsigned comparison of the magnitude
// bits; `acc` accumulates the largest magnitude bits of a set of values
__device__ __forceinline__ unsigned mag_bits(float x) { return __float_as_uint(x) & 0x7fffffffu; }
constexpr unsigned DIV_BY_FMA_LIMIT = 0x71800000u; // 2^100

// x clamped to [lo, hi]: a maximum and a minimum (one v_med3_i32 where the
// compiler knows the bounds)
__device__ __forceinline__ int clamp_i32(int x, int lo, int hi) {
    return min(max(x, lo), hi);
}

// Four values to four saturated bytes of one dword (s8: lo = -128, hi = 127; u8: 0, 255)
__device__ __forceinline__ unsigned pack4_i8(const float (&v)[4], int lo, int hi) {
    int q[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) q[e] = clamp_i32((int)__builtin_rintf(v[e]), lo, hi);
    const unsigned lo16 = __builtin_amdgcn_perm((unsigned)q[1], (unsigned)q[0], 0x0c0c0400u);
    const unsigned hi16 = __builtin_amdgcn_perm((unsigned)q[3], (unsigned)q[2], 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi16, lo16, 0x05040100u);
}

struct po_reg_t {
    int kind, alg;
    float alpha, beta, scale, zpf;
};

// Wavefront-uniform description of the epilogue (lives in scalar registers).
struct epi_uniform_t {
    float ds, ds_inv;
    int bias_mode;  // 0 none, 1 per n (table), 2 per element
    int ds_mode;    // 0 none, 1 divide, 2 multiply by reciprocal, 3 divide by fma correction (integer dst)
    int dzp_mode;   // 0 none, 1 present (table)
    int hoisted_po; // post-op whose per-n operand sits in the table, or -1
    int staged;     // STG_NONE, STG_BIAS, STG_SUM or a binary post-op index
    int staged_dt;
    const char *staged_p;
    long st_s0, st_s1; // element strides of the staged stream (stride along n is 1)
    po_reg_t pf0, pf1, pf2; // the leading "simple" post-ops (at most three)
    int nfast;      // how many of them
    int n_po;
    int dst_dt, dst_vec; // dst_vec: four consecutive n leave as one aligned store
    int fast;       // every operand is in the table or staged and every post-op is a register-resident one
    int dynamic;    // MI355_DST_DYNAMIC_*
};

__device__ __forceinline__ bool vec_ok(const void *p, long s0, long s1, int bits) {
    // four consecutive elements must form one aligned 8- or 16-byte vector
    const int bytes4 = bits / 2;
    return (bits == 16 || bits == 32) && (((uintptr_t)p) % bytes4) == 0 && (s0 % 4) == 0
            && (s1 % 4) == 0;
}

__device__ __forceinline__ bool vec_ok_store(const void *p, long s0, long s1, int bits) {
    const int bytes4 = bits / 2; // bytes of four elements
    return (bits == 4 || bits == 8 || bits == 16 || bits == 32) && (((uintptr_t)p) % bytes4) == 0
            && (s0 % 4) == 0 && (s1 % 4) == 0;
}

// the binary post-op whose operand does not depend on the row: first one with
// a zero row stride
template <class PT>
__device__ __forceinline__ int find_hoisted_po(const PT &P) {
    for (int i = 0; i < P.n_po; ++i)
        if (P.po[i].kind == MI355_PO_BINARY && P.po[i].s1 == 0 && P.po[i].alg != MI355_BINARY_SELECT) return i;
    return -1;
}

// Fills the epilogue's rows of the table (bias, per-n binary operand, dst zero
// points) for the tile's 256 columns starting at n0; the kernel's conversion
// fills its own rows with `conv.per_n`.  Called by every thread of the
// workgroup before the K loop; the loop's barriers order it before the reads.
template <int NT, class PT, class Conv>
__device__ __forceinline__ void fill_ntab(const PT &P, const Conv &conv, unsigned ntab, long b, long n0) {
    typedef int __attribute__((address_space(3))) *lds_i_ptr_t;
    static_assert(NT % NTAB_COLS == 0, "every column has a thread");
    const int hp = find_hoisted_po(P);
    // No branch below depends on the thread: thread t fills column t % 256 (with
    // 512 threads two threads store the same values), columns beyond N load from
    // column N - 1 and store neutral values.  (Values that are uniform but merge
    // at the join of a divergent branch would count as divergent from there on.)
    const int col = (int)threadIdx.x & (NTAB_COLS - 1);
    const bool valid = n0 + col < P.N;
    const long n = valid ? n0 + col : P.N - 1;
    lds_i_ptr_t t = (lds_i_ptr_t)(size_t)(ntab + (unsigned)(col * 4));
    float wsc = 1.f, bias = 0.f, hv = 0.f, dzp = 0.f;
    int cc = 0, c = 0;
    conv.per_n(P, b, n, wsc, cc, c);
    if (P.bias_dt != MI355_DT_UNDEF && P.bs[1] == 0) bias = load_float(P.bias_dt, P.bias, b * P.bs[0] + n * P.bs[2]);
    if (hp >= 0) hv = load_float(P.po[hp].dt, P.po[hp].p, b * P.po[hp].s0 + n * P.po[hp].s2);
    if (P.dst_zp.dt != MI355_DT_UNDEF) dzp = (float)((const int *)P.dst_zp.p)[(P.dst_zp.mask & 4) ? n : 0];
    t[NT_WSC * NTAB_COLS] = __float_as_int(valid ? wsc : 1.f);
    t[NT_CC * NTAB_COLS] = valid ? cc : 0;
    t[NT_C * NTAB_COLS] = valid ? c : 0;
    t[NT_BIAS * NTAB_COLS] = __float_as_int(valid ? bias : 0.f);
    t[NT_HV * NTAB_COLS] = __float_as_int(valid ? hv : 0.f);
    t[NT_DZP * NTAB_COLS] = __float_as_int(valid ? dzp : 0.f);
}

// `cols_inside`: the wavefront's columns all lie inside N (operand streams are
// then loaded without column masks)
template <class PT>
__device__ __forceinline__ epi_uniform_t make_uniform(const PT &P, bool cols_inside) {
    epi_uniform_t H;
    H.bias_mode = 0; H.ds_mode = 0; H.dzp_mode = 0; H.staged = STG_NONE;
    H.staged_dt = 0; H.staged_p = nullptr; H.st_s0 = H.st_s1 = 0; H.ds = 1.f; H.ds_inv = 1.f;
    if (P.bias_dt != MI355_DT_UNDEF) H.bias_mode = P.bs[1] == 0 ? 1 : 2;
    H.dynamic = P.dst_dynamic;
    H.dst_dt = P.dst_dt;
    if (P.dst_scale.dt != MI355_DT_UNDEF && !P.dst_dynamic) {
        H.ds = load_float(P.dst_scale.dt, P.dst_scale.p, 0);
        H.ds_inv = 1.f / H.ds;
        H.ds_mode = P.dst_scale_mode == MI355_DST_SCALE_RECIPROCAL ? 2 : 1;
        const bool int_dst = H.dst_dt == MI355_DT_S8 || H.dst_dt == MI355_DT_U8 || H.dst_dt == MI355_DT_S32;
        const float as = fabsf(H.ds);
        if (H.ds_mode == 1 && int_dst && as >= 0x1p-20f && as <= 0x1p20f) H.ds_mode = 3;
    }
    if (P.dst_zp.dt != MI355_DT_UNDEF) H.dzp_mode = 1;
    H.n_po = P.n_po;
    H.dst_vec = P.ds[2] == 1 && vec_ok_store(P.dst, P.ds[0], P.ds[1], dt_bits(P.dst_dt));
    {
        auto grab = [&](int i, po_reg_t &r) -> bool {
            r.kind = 0; r.alg = 0; r.alpha = r.beta = r.zpf = 0.f; r.scale = 1.f;
            if (i >= P.n_po) return false;
            r.kind = P.po[i].kind; r.alg = P.po[i].alg; r.alpha = P.po[i].alpha;
            r.beta = P.po[i].beta; r.scale = P.po[i].scale; r.zpf = (float)P.po[i].zp;
            const bool simple_elt = r.kind == MI355_PO_ELTWISE
                    && (r.alg == MI355_ELTWISE_RELU || r.alg == MI355_ELTWISE_LINEAR
                            || r.alg == MI355_ELTWISE_GELU_TANH || r.alg == MI355_ELTWISE_CLIP
                            || r.alg == MI355_ELTWISE_CLIP_V2 || r.alg == MI355_ELTWISE_SWISH
                            || r.alg == MI355_ELTWISE_LOGISTIC);
            return simple_elt || r.kind == MI355_PO_BINARY || r.kind == MI355_PO_SUM;
        };
        H.nfast = 0;
        if (grab(0, H.pf0)) {
            H.nfast = 1;
            if (grab(1, H.pf1)) {
                H.nfast = 2;
                if (grab(2, H.pf2)) H.nfast = 3;
            } else {
                grab(3 + MI355_MAX_POST_OPS, H.pf2);
            }
        } else {
            grab(3 + MI355_MAX_POST_OPS, H.pf1);
            grab(3 + MI355_MAX_POST_OPS, H.pf2);
        }
    }
    H.hoisted_po = find_hoisted_po(P);
    int first_sum = -1;
    for (int i = 0; i < P.n_po; ++i) {
        const auto &po = P.po[i];
        if (po.kind == MI355_PO_BINARY) {
            if (i != H.hoisted_po && po.s1 != 0 && po.s2 == 1 && H.staged == STG_NONE && cols_inside
                    && vec_ok(po.p, po.s0, po.s1, dt_bits(po.dt))) {
                H.staged = i; H.staged_dt = po.dt; H.staged_p = (const char *)po.p;
                H.st_s0 = po.s0; H.st_s1 = po.s1;
            }
        } else if (po.kind == MI355_PO_SUM && first_sum < 0) {
            first_sum = i;
        }
    }
    if (H.staged == STG_NONE && cols_inside && first_sum >= 0 && P.ds[2] == 1
            && vec_ok(P.dst, P.ds[0], P.ds[1], dt_bits(P.sum_dt))) {
        H.staged = STG_SUM; H.staged_dt = P.sum_dt; H.staged_p = (const char *)P.dst;
        H.st_s0 = P.ds[0]; H.st_s1 = P.ds[1];
    }
    if (H.staged == STG_NONE && cols_inside && H.bias_mode == 2 && P.bs[2] == 1
            && vec_ok(P.bias, P.bs[0], P.bs[1], dt_bits(P.bias_dt))) {
        H.staged = STG_BIAS; H.staged_dt = P.bias_dt; H.staged_p = (const char *)P.bias;
        H.st_s0 = P.bs[0]; H.st_s1 = P.bs[1];
    }
    H.fast = H.n_po == H.nfast && (H.bias_mode != 2 || H.staged == STG_BIAS) && cols_inside && H.dst_vec;
    {
        auto operand_ready = [&](const po_reg_t &r, int i) {
            if (r.kind == MI355_PO_BINARY)
                return (i == H.hoisted_po || i == H.staged) && (r.alg == MI355_BINARY_ADD || r.alg == MI355_BINARY_MUL);
            if (r.kind == MI355_PO_SUM) return H.staged == STG_SUM;
            return true; // grab() admits the five cheap eltwise algorithms only
        };
        const int dd = H.dst_dt;
        if (dd != MI355_DT_S8 && dd != MI355_DT_U8 && dd != MI355_DT_BF16 && dd != MI355_DT_F32 && dd != MI355_DT_S32
                && dd != MI355_DT_F8_E4M3 && dd != MI355_DT_F8_E5M2 && dd != MI355_DT_F16 && dd != MI355_DT_F4_E2M1
                && dd != MI355_DT_S4 && dd != MI355_DT_U4)
            H.fast = 0;
        if (H.nfast > 0 && !operand_ready(H.pf0, 0)) H.fast = 0;
        if (H.nfast > 1 && !operand_ready(H.pf1, 1)) H.fast = 0;
        if (H.nfast > 2 && !operand_ready(H.pf2, 2)) H.fast = 0;
    }
    return H;
}

// decode four packed 16- or 32-bit values
__device__ __forceinline__ void staged4(int dt, const uint4 &raw, float (&y)[4]) {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    switch (dt) {
        case MI355_DT_BF16:
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = u2f((w[e >> 1] >> ((e & 1) * 16)) << 16);
            break;
        case MI355_DT_F16:
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = f16_to_f32((uint16_t)(w[e >> 1] >> ((e & 1) * 16)));
            break;
        case MI355_DT_F32:
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = u2f(w[e]);
            break;
        default: // s32
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = (float)(int)w[e];
            break;
    }
}

// every eltwise algorithm, one copy of the long-tail code (rolled over the
// four values; selects of values, not of addresses)
__device__ __forceinline__ void eltwise4_any(int alg, float (&v)[4], float alpha, float beta,
        float scale) {
    float v0 = v[0], v1 = v[1], v2 = v[2], v3 = v[3];
#pragma unroll 1
    for (int e = 0; e < 4; ++e) {
        const float x = e == 0 ? v0 : e == 1 ? v1 : e == 2 ? v2 : v3;
        const float y = eltwise_f(alg, x, alpha, beta) * scale;
        if (e == 0) v0 = y;
        else if (e == 1) v1 = y;
        else if (e == 2) v2 = y;
        else v3 = y;
    }
    v[0] = v0; v[1] = v1; v[2] = v2; v[3] = v3;
}

// The general path for one quad: bias, any post-op chain, dst scale and zero
// point, every operand loaded where it is used.
template <class PT>
__device__ __forceinline__ void apply_epilogue4(const PT &P, float (&v)[4], long b, long m, long nbase,
        int nvalid) {
    if (P.bias_dt != MI355_DT_UNDEF) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (e < nvalid)
                v[e] += load_float(P.bias_dt, P.bias, b * P.bs[0] + m * P.bs[1] + (nbase + e) * P.bs[2]);
    }
    if (P.n_po > 0) {
        float dst_old[4] = {0.f, 0.f, 0.f, 0.f};
        if (P.sum_dt != MI355_DT_UNDEF) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (e < nvalid)
                    dst_old[e] = load_float(P.sum_dt, P.dst, b * P.ds[0] + m * P.ds[1] + (nbase + e) * P.ds[2]);
        }
#pragma unroll 1
        for (int i = 0; i < P.n_po; ++i) {
            const auto &po = P.po[i];
            const int kind = po.kind;
            if (kind == MI355_PO_ELTWISE) {
                eltwise4_any(po.alg, v, po.alpha, po.beta, po.scale);
            } else if (kind == MI355_PO_BINARY) {
                const int alg = po.alg;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float y = e < nvalid ? load_float(po.dt, po.p, b * po.s0 + m * po.s1 + (nbase + e) * po.s2) : 0.f;
                    v[e] = alg == MI355_BINARY_ADD ? v[e] + y : alg == MI355_BINARY_MUL ? v[e] * y : binary_f(alg, v[e], y);
                }
            } else if (kind == MI355_PO_SUM) {
                const float sc = po.scale, zpf = (float)po.zp;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] += sc * (dst_old[e] - zpf);
            } else if (kind == MI355_PO_PRELU) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (e < nvalid && !(v[e] >= 0))
                        v[e] = ((const float *)po.p)[b * po.s0 + m * po.s1 + (nbase + e) * po.s2] * v[e];
            }
        }
    }
    if (P.dst_dynamic) return; // the group's scale is computed from these values
    if (P.dst_scale.dt != MI355_DT_UNDEF) {
        const float s = load_float(P.dst_scale.dt, P.dst_scale.p, 0);
        if (P.dst_scale_mode == MI355_DST_SCALE_RECIPROCAL) {
            const float r = 1.f / s;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] *= r;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] /= s;
        }
    }
    if (P.dst_zp.dt != MI355_DT_UNDEF) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (e < nvalid) v[e] += (float)((const int *)P.dst_zp.p)[(P.dst_zp.mask & 4) ? nbase + e : 0];
    }
}

// convert four values to the dst type: one dispatch for the four
__device__ __forceinline__ void cvt4(int dt, const float (&v)[4], uint32_t (&w)[4]) {
    switch (dt) {
        case MI355_DT_S8:
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = (uint32_t)(int)__builtin_rintf(sat(v[e], -128.f, 127.f)) & 0xffu;
            break;
        case MI355_DT_U8:
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = (uint32_t)(int)__builtin_rintf(sat(v[e], 0.f, 255.f)) & 0xffu;
            break;
        case MI355_DT_BF16:
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = f32_to_bf16(v[e]);
            break;
        case MI355_DT_F32:
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = f2u(v[e]);
            break;
        case MI355_DT_S32:
#pragma unroll
            for (int e = 0; e < 4; ++e)
                w[e] = (uint32_t)(int)__builtin_rintf(sat(v[e], -2147483648.f, 2147483520.f));
            break;
        case MI355_DT_F4_E2M1:
        case MI355_DT_S4:
        case MI355_DT_U4:
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = nibble_code(dt, v[e]);
            break;
        default:
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = cvt_store_bits(dt, v[e]);
            break;
    }
}

// one quad to dst, `dst_vec`: as one aligned vector store
template <class PT>
__device__ __forceinline__ void store4(const PT &P, int dst_vec, const float (&v)[4], long b,
        long m, long n, int nvalid) {
    const long off = b * P.ds[0] + m * P.ds[1] + n * P.ds[2];
    uint32_t w[4];
    cvt4(P.dst_dt, v, w);
    const int bits = dt_bits(P.dst_dt);
    if (bits == 4) {
        // Two bytes, low nibble first.  The host admits a 4-bit dst only where every quad is whole and starts a
        // byte (unit column stride, N and the other strides multiples of 4); the bytes may start at an odd address.
        if (nvalid == 4) {
            uint8_t *q = (uint8_t *)P.dst + (off >> 1);
            const uint32_t lo = w[0] | (w[1] << 4), hi = w[2] | (w[3] << 4);
            if ((uintptr_t)q & 1) q[0] = (uint8_t)lo, q[1] = (uint8_t)hi;
            else *(uint16_t *)q = (uint16_t)(lo | (hi << 8));
        }
        return;
    }
    if (nvalid == 4 && dst_vec) {
        if (bits == 8) {
            *(uint32_t *)((uint8_t *)P.dst + off) = w[0] | (w[1] << 8) | (w[2] << 16) | (w[3] << 24);
        } else if (bits == 16) {
            uint2 o;
            o.x = w[0] | (w[1] << 16);
            o.y = w[2] | (w[3] << 16);
            *(uint2 *)((uint16_t *)P.dst + off) = o;
        } else {
            uint4 o;
            o.x = w[0]; o.y = w[1]; o.z = w[2]; o.w = w[3];
            *(uint4 *)((uint32_t *)P.dst + off) = o;
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if (e < nvalid) {
            const long o = off + e * P.ds[2];
            if (bits == 8) ((uint8_t *)P.dst)[o] = (uint8_t)w[e];
            else if (bits == 16) ((uint16_t *)P.dst)[o] = (uint16_t)w[e];
            else ((uint32_t *)P.dst)[o] = w[e];
        }
    }
}

// ---- fast path: the Q quads of a row block per dispatch.  Every data-type and
// post-op dispatch below is uniform over the wavefront and is taken once for the
// Q quads.
template <int Q>
__device__ __forceinline__ void eltwiseQ_simple(int alg, float (&v)[Q][4], float alpha, float beta, float scale,
        bool int_dst) {
    if (alg == MI355_ELTWISE_RELU) {
        if (alpha == 0.f && scale == 1.f && int_dst) {
            // an integer dst turns NaN and -0 into 0 either way: one maximum
#pragma unroll
            for (int k = 0; k < Q; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) v[k][e] = fmaxf(v[k][e], 0.f);
        } else {
#pragma unroll
            for (int k = 0; k < Q; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) v[k][e] = (v[k][e] > 0 ? v[k][e] : v[k][e] * alpha) * scale;
        }
    } else if (alg == MI355_ELTWISE_LINEAR) {
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] = (alpha * v[k][e] + beta) * scale;
    } else if (alg == MI355_ELTWISE_GELU_TANH) {
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] = gelu_tanh_fast(v[k][e]) * scale;
    } else if (alg == MI355_ELTWISE_SWISH) {
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] = v[k][e] * logistic_fast(alpha * v[k][e]) * scale;
    } else if (alg == MI355_ELTWISE_LOGISTIC) {
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] = logistic_fast(v[k][e]) * scale;
    } else if (alg == MI355_ELTWISE_CLIP) {
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] = eltwise_f(MI355_ELTWISE_CLIP, v[k][e], alpha, beta) * scale;
    } else {
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] = eltwise_f(MI355_ELTWISE_CLIP_V2, v[k][e], alpha, beta) * scale;
    }
}

// `col[k]`: the quad's first column inside the tile (index into the table);
// `sy`: the staged stream's values for the quads
template <int Q>
__device__ __forceinline__ void apply_epilogueQ(const epi_uniform_t &H, unsigned ntab, const int (&col)[Q],
        float (&v)[Q][4], const float (&sy)[Q][4]) {
    const bool int_dst = H.dst_dt == MI355_DT_S8 || H.dst_dt == MI355_DT_U8 || H.dst_dt == MI355_DT_S32;
    if (H.bias_mode == 1) {
#pragma unroll
        for (int k = 0; k < Q; ++k) {
            const v4f_t bb = nt4f(ntab, NT_BIAS, col[k]);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] += bb[e];
        }
    } else if (H.bias_mode == 2) { // staged
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] += sy[k][e];
    }
    auto fast_op = [&](const po_reg_t &r, int i) __attribute__((always_inline)) {
        if (r.kind == MI355_PO_ELTWISE) {
            eltwiseQ_simple<Q>(r.alg, v, r.alpha, r.beta, r.scale, int_dst);
        } else if (r.kind == MI355_PO_BINARY) {
            const bool add = r.alg == MI355_BINARY_ADD; // else mul: nothing else is on this path
            if (i == H.hoisted_po) {
#pragma unroll
                for (int k = 0; k < Q; ++k) {
                    const v4f_t y = nt4f(ntab, NT_HV, col[k]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[k][e] = add ? v[k][e] + y[e] : v[k][e] * y[e];
                }
            } else {
#pragma unroll
                for (int k = 0; k < Q; ++k)
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[k][e] = add ? v[k][e] + sy[k][e] : v[k][e] * sy[k][e];
            }
        } else { // sum: the old dst is the staged stream
#pragma unroll
            for (int k = 0; k < Q; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) v[k][e] += r.scale * (sy[k][e] - r.zpf);
        }
    };
    if (H.nfast > 0) fast_op(H.pf0, 0);
    if (H.nfast > 1) fast_op(H.pf1, 1);
    if (H.nfast > 2) fast_op(H.pf2, 2);
    if (H.ds_mode == 3) {
        unsigned mx = 0;
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) mx = max(mx, mag_bits(v[k][e]));
        if (__builtin_amdgcn_ballot_w64(mx >= DIV_BY_FMA_LIMIT) == 0) {
#pragma unroll
            for (int k = 0; k < Q; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) v[k][e] = div_by_fma(v[k][e], H.ds, H.ds_inv);
        } else {
#pragma unroll
            for (int k = 0; k < Q; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) v[k][e] /= H.ds;
        }
    } else if (H.ds_mode == 1) {
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] /= H.ds;
    } else if (H.ds_mode == 2) {
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] *= H.ds_inv;
    }
    if (H.dzp_mode) {
#pragma unroll
        for (int k = 0; k < Q; ++k) {
            const v4f_t z = nt4f(ntab, NT_DZP, col[k]);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] += z[e];
        }
    }
}

// The e8m0 scale of a group with largest magnitude amax, and the bits of its
// inverse, by exponent arithmetic: e8m0(x) keeps the exponent byte of x, so
//     scale = e8m0(e8m0(amax) / e8m0(dt_max))  has the byte  ea - em + 127
// (0 when that is below 1: the quotient is subnormal or zero; 255 for a NaN /
// infinite amax), and 1 / scale = 2^(127 - byte), subnormal for byte 254.  The
// same bytes and bits as the reference's two divisions
// (ref_matmul.cpp:343-351, :381).
__device__ __forceinline__ uint8_t mx_scale_byte(float amax, int em, float &inv) {
    const int ea = (int)f32_to_e8m0(amax);
    int sb = ea - em + 127;
    sb = sb < 0 ? 0 : sb;
    if (ea == 255) sb = 255;
    const unsigned ib = sb == 255 ? 0x7fc00000u : sb == 254 ? 0x00400000u : (unsigned)(254 - sb) << 23;
    inv = u2f(ib);
    return (uint8_t)sb;
}

__device__ __forceinline__ float amax4(const float (&v)[4]) {
    return fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
}

// One row of accumulator tiles copied by value.  The row-block pickers select
// their rows with a switch over the run-time block number; were the cases
// identical code on different registers, the compiler would merge them into one
// copy that indexes `acc` with a run-time offset, and all accumulators would
// live in private memory from the first K step on.  The empty asm statements
// keep the cases apart (statements of inline assembly are never merged).
template <class T, int C>
__device__ __forceinline__ void copy_row(const T (&src)[C], T (&dst)[C]) {
#pragma unroll
    for (int j = 0; j < C; ++j) {
        T v = src[j];
        asm volatile("" : "+v"(v));
        dst[j] = v;
    }
}

// Accumulator layouts (operands exchanged, see the top of the file).
//   RB          rows of a row block (one MFMA tile row)
//   NB          row blocks of a wavefront's 128 rows
//   QPG         quads of one lane inside a group of 32 consecutive columns
//   nq<C>()     quads of a lane per row block (C MFMA tiles along n)
//   qcol(k)     first column of quad k inside the wavefront's part
//   quad(a, k)  the four raw accumulators of quad k of row block `a`
//   group_max   maximum over the lanes that share a row and a 32-column group
struct layout16_t {
    static constexpr int RB = 16, NB = 8, QPG = 2;
    template <int C> static constexpr int nq() { return C; }
    static __device__ __forceinline__ int lrow(int lane) { return lane & 15; }
    static __device__ __forceinline__ int qcol(int k, int lane) { return 16 * k + 4 * (lane >> 4); }
    template <class T, int C>
    static __device__ __forceinline__ v4i_t quad(const T (&a)[C], int k) {
        return v4i_t {raw_bits(a[k][0]), raw_bits(a[k][1]), raw_bits(a[k][2]), raw_bits(a[k][3])};
    }
    static __device__ __forceinline__ float group_max(float x) {
        x = fmaxf(x, __shfl_xor(x, 16, 64));
        return fmaxf(x, __shfl_xor(x, 32, 64));
    }
    // the lane that writes the group's scale byte
    static __device__ __forceinline__ bool group_leader(int lane) { return (lane >> 4) == 0; }
    template <class T, int R, int C>
    static __device__ __forceinline__ void pick_rows(const T (&acc)[R][C], int i, T (&a)[C]) {
        static_assert(R == 8, "eight row blocks");
        switch (i) {
            case 0: copy_row(acc[0], a); break;
            case 1: copy_row(acc[1], a); break;
            case 2: copy_row(acc[2], a); break;
            case 3: copy_row(acc[3], a); break;
            case 4: copy_row(acc[4], a); break;
            case 5: copy_row(acc[5], a); break;
            case 6: copy_row(acc[6], a); break;
            default: copy_row(acc[7], a); break;
        }
    }
};

struct layout32_t {
    static constexpr int RB = 32, NB = 4, QPG = 4;
    template <int C> static constexpr int nq() { return 4 * C; }
    static __device__ __forceinline__ int lrow(int lane) { return lane & 31; }
    static __device__ __forceinline__ int qcol(int k, int lane) { return 32 * (k >> 2) + 8 * (k & 3) + 4 * (lane >> 5); }
    template <class T, int C>
    static __device__ __forceinline__ v4i_t quad(const T (&a)[C], int k) {
        const int j = k >> 2, g = k & 3;
        return v4i_t {raw_bits(a[j][4 * g]), raw_bits(a[j][4 * g + 1]), raw_bits(a[j][4 * g + 2]), raw_bits(a[j][4 * g + 3])};
    }
    static __device__ __forceinline__ float group_max(float x) { return fmaxf(x, __shfl_xor(x, 32, 64)); }
    static __device__ __forceinline__ bool group_leader(int lane) { return (lane >> 5) == 0; }
    template <class T, int R, int C>
    static __device__ __forceinline__ void pick_rows(const T (&acc)[R][C], int i, T (&a)[C]) {
        static_assert(R == 4, "four row blocks");
        switch (i) {
            case 0: copy_row(acc[0], a); break;
            case 1: copy_row(acc[1], a); break;
            case 2: copy_row(acc[2], a); break;
            default: copy_row(acc[3], a); break;
        }
    }
};

// Q quads of one row to dst (fast path: vector stores, columns inside N)
template <int Q, class PT>
__device__ __forceinline__ void storeQ(const PT &P, const epi_uniform_t &H, const float (&v)[Q][4], long b,
        long m, bool ok, const long (&n)[Q]) {
    uint32_t w[Q][4];
    const int dt = H.dst_dt;
    const long rowoff = b * P.ds[0] + m * P.ds[1];
    if (dt_bits(dt) == 4) {
        // two bytes a quad, low nibble first; rows and quads start whole bytes (checked by the host), possibly at an
        // odd address.  f4_e2m1 by v_cvt_scalef32_pk_fp4_f32 (nearest even, saturating at +-6 like the software
        // conversion: checked code for code on the device, tests/test_dynamic_dst.py) unless the wavefront holds a
        // NaN, which the software conversion turns into +-6
        bool hw = false;
        if (dt == MI355_DT_F4_E2M1) {
            bool nan = false;
#pragma unroll
            for (int k = 0; k < Q; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) nan |= __builtin_amdgcn_classf(v[k][e], 0x3);
            hw = __builtin_amdgcn_ballot_w64(nan) == 0;
        }
#pragma unroll
        for (int k = 0; k < Q; ++k) {
            uint32_t lo, hi;
            if (hw) {
                unsigned r = 0;
                r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, v[k][0], v[k][1], 1.f, 0);
                r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, v[k][2], v[k][3], 1.f, 1);
                lo = r & 0xffu, hi = (r >> 8) & 0xffu;
            } else {
                uint32_t c[4];
                cvt4(dt, v[k], c);
                lo = c[0] | (c[1] << 4), hi = c[2] | (c[3] << 4);
            }
            uint8_t *q = (uint8_t *)P.dst + ((rowoff + n[k]) >> 1);
            if (!ok) continue;
            if ((uintptr_t)q & 1) q[0] = (uint8_t)lo, q[1] = (uint8_t)hi;
            else *(uint16_t *)q = (uint16_t)(lo | (hi << 8));
        }
        return;
    }
    if (dt == MI355_DT_S8 || dt == MI355_DT_U8) {
        // Round first (v_rndne + the saturating v_cvt_i32_f32, NaN -> 0), clamp as
        // integers (maximum + minimum), pack the four low bytes with byte permutes: the
        // same values as the reference's clamp-then-round (rounding is monotonic and
        // the bounds are integers) in 3 + 3/4 instructions per value.
        const int lo = dt == MI355_DT_S8 ? -128 : 0, hi = dt == MI355_DT_S8 ? 127 : 255;
#pragma unroll
        for (int k = 0; k < Q; ++k) {
            int q[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                q[e] = clamp_i32((int)__builtin_rintf(v[k][e]), lo, hi);
            }
            const unsigned lo16 = __builtin_amdgcn_perm((unsigned)q[1], (unsigned)q[0], 0x0c0c0400u);
            const unsigned hi16 = __builtin_amdgcn_perm((unsigned)q[3], (unsigned)q[2], 0x0c0c0400u);
            const unsigned word = __builtin_amdgcn_perm(hi16, lo16, 0x05040100u);
            if (ok) *(uint32_t *)((uint8_t *)P.dst + rowoff + n[k]) = word;
        }
        return;
    } else if (dt == MI355_DT_BF16) {
        // v_cvt_pk_bf16_f32 rounds to nearest even like the reference's conversion
        // (src/common/bfloat16.cpp:29-49) for normal numbers, zeros and infinities;
        // the reference flushes f32 subnormals to zero and quiets NaNs by setting
        // one bit, so a wavefront that holds any of those (class mask: s/q NaN,
        // +-subnormal) takes the software conversion.  One class test per value
        // and half a conversion instead of a dozen integer operations.
        bool special = false;
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) special |= __builtin_amdgcn_classf(v[k][e], 0x93);
        if (__builtin_amdgcn_ballot_w64(special) == 0) {
            typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
            typedef float f32x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int k = 0; k < Q; ++k) {
                uint2 o;
                o.x = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_t {v[k][0], v[k][1]}, bf16x2_t));
                o.y = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_t {v[k][2], v[k][3]}, bf16x2_t));
                if (ok) *(uint2 *)((uint16_t *)P.dst + rowoff + n[k]) = o;
            }
            return;
        }
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) w[k][e] = f32_to_bf16(v[k][e]);
    } else if (dt == MI355_DT_F32) {
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) w[k][e] = f2u(v[k][e]);
    } else if (dt == MI355_DT_F16) {
        // v_cvt_f16_f32 equals the software conversion (float16.hpp) for every
        // input, NaN payloads included: checked on the device over 4 M f32
        // bit patterns and every exponent's special mantissas
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) w[k][e] = __builtin_bit_cast(uint16_t, (_Float16)v[k][e]);
    } else if (dt == MI355_DT_F8_E4M3 || dt == MI355_DT_F8_E5M2) {
        // The reference converts f32 -> f16 -> fp8, two roundings to nearest even
        // (src/common/float8.cpp:47-126, :216-281).  v_cvt_f16_f32 followed by
        // v_cvt_scalef32_pk_{fp8,bf8}_f16 with scale 1 does the same: checked on
        // the device against the software conversions for every f16 bit pattern
        // and 4 M f32 patterns, the results differ for NaN inputs only (the
        // hardware returns one canonical NaN).  A wavefront that holds a NaN
        // takes the software conversion.
        bool special = false;
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) special |= __builtin_amdgcn_classf(v[k][e], 0x3);
        if (__builtin_amdgcn_ballot_w64(special) == 0) {
            typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
            typedef short s16x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int k = 0; k < Q; ++k) {
                const f16x2_t lo = {(_Float16)v[k][0], (_Float16)v[k][1]}, hi = {(_Float16)v[k][2], (_Float16)v[k][3]};
                s16x2_t r = {0, 0};
                if (dt == MI355_DT_F8_E4M3) {
                    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, lo, 1.f, false);
                    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, hi, 1.f, true);
                } else {
                    r = __builtin_amdgcn_cvt_scalef32_pk_bf8_f16(r, lo, 1.f, false);
                    r = __builtin_amdgcn_cvt_scalef32_pk_bf8_f16(r, hi, 1.f, true);
                }
                if (ok) *(uint32_t *)((uint8_t *)P.dst + rowoff + n[k]) = __builtin_bit_cast(uint32_t, r);
            }
            return;
        }
        if (dt == MI355_DT_F8_E4M3) {
#pragma unroll
            for (int k = 0; k < Q; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) w[k][e] = f32_to_e4m3(v[k][e]);
        } else {
#pragma unroll
            for (int k = 0; k < Q; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) w[k][e] = f32_to_e5m2(v[k][e]);
        }
    } else { // s32 (nothing else is on the fast path)
#pragma unroll
        for (int k = 0; k < Q; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                w[k][e] = (uint32_t)(int)__builtin_rintf(sat(v[k][e], -2147483648.f, 2147483520.f));
    }
    const int bits = dt_bits(dt);
    if (!ok) return;
    if (bits == 8) {
#pragma unroll
        for (int k = 0; k < Q; ++k)
            *(uint32_t *)((uint8_t *)P.dst + rowoff + n[k]) = w[k][0] | (w[k][1] << 8) | (w[k][2] << 16) | (w[k][3] << 24);
    } else if (bits == 16) {
#pragma unroll
        for (int k = 0; k < Q; ++k) {
            uint2 o;
            o.x = w[k][0] | (w[k][1] << 16);
            o.y = w[k][2] | (w[k][3] << 16);
            *(uint2 *)((uint16_t *)P.dst + rowoff + n[k]) = o;
        }
    } else {
#pragma unroll
        for (int k = 0; k < Q; ++k) {
            uint4 o;
            o.x = w[k][0]; o.y = w[k][1]; o.z = w[k][2]; o.w = w[k][3];
            *(uint4 *)((uint32_t *)P.dst + rowoff + n[k]) = o;
        }
    }
}

// Dynamic (MX) quantization of dst for the quads of one row
// (ref_matmul.cpp:338-423): a group is 32 consecutive n of the row = QPG quads
// of this lane and the same quads of its partner lanes.  Writes the e8m0 scale
// of every group and leaves v scaled and saturated, ready for the fp8
// conversion.  All lanes take part in the cross-lane maximum, rows beyond M on
// the data of a valid row; only the stores are masked.
template <class Layout, int Q, bool FP, class PT>
__device__ __forceinline__ void dynamic_quantQ(const PT &P, int dst_dt, float (&v)[Q][4], long b, long m,
        bool ok, const long (&n)[Q], int lane) {
    constexpr int QPG = Layout::QPG;
    const float dt_max = dst_dt == MI355_DT_F8_E4M3 ? 448.f : (dst_dt == MI355_DT_F4_E2M1 ? 6.f : 57344.f);
    if (FP) {
        // groups of 16 columns with an f8_e4m3 scale (ref_matmul.cpp:352-365, :381): the lower and the upper
        // half of the lane's quads of 32 columns, shared with the same partner lanes
        constexpr int HQ = QPG / 2;
#pragma unroll
        for (int g = 0; g < Q / HQ; ++g) {
            float amax = 0.f;
#pragma unroll
            for (int kk = 0; kk < HQ; ++kk) amax = fmaxf(amax, amax4(v[g * HQ + kk]));
            amax = Layout::group_max(amax);
            float scale = amax / dt_max;
            scale = fminf(scale, 448.f);
            scale = fmaxf(scale, 0.125f);
            const uint8_t sbyte = f32_to_e4m3(scale);
            const float inv = 1.f / e4m3_to_f32(sbyte);
#pragma unroll
            for (int kk = 0; kk < HQ; ++kk)
#pragma unroll
                for (int e = 0; e < 4; ++e) v[g * HQ + kk][e] = fminf(fmaxf(v[g * HQ + kk][e] * inv, -dt_max), dt_max);
            if (ok && Layout::group_leader(lane))
                ((uint8_t *)P.dst_scale.p)[quant_off(P.dst_scale, b, m, n[g * HQ] & ~15L, P.M, P.N)] = sbyte;
        }
        return;
    }
    const int em = (int)f32_to_e8m0(dt_max);
#pragma unroll
    for (int g = 0; g < Q / QPG; ++g) {
        float amax = 0.f;
#pragma unroll
        for (int kk = 0; kk < QPG; ++kk) amax = fmaxf(amax, amax4(v[g * QPG + kk]));
        amax = Layout::group_max(amax);
        float inv;
        const uint8_t sbyte = mx_scale_byte(amax, em, inv);
#pragma unroll
        for (int kk = 0; kk < QPG; ++kk)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[g * QPG + kk][e] = fminf(fmaxf(v[g * QPG + kk][e] * inv, -dt_max), dt_max);
        if (ok && Layout::group_leader(lane))
            ((uint8_t *)P.dst_scale.p)[quant_off(P.dst_scale, b, m, n[g * QPG] & ~31L, P.M, P.N)] = sbyte;
    }
}

// A wavefront's 128 x 64 part of a bf16 dst when nothing follows the K sum but the conversion, from accumulators of
// 16 x 16 tiles (a lane holds four consecutive columns of a row): written to dst as whole 128-byte rows.  In the
// accumulator layout a wavefront-wide store touches 16 rows, 8 bytes each; the part goes through the wavefront's 16 KB
// share of the idle tile ring instead -- 8-byte writes at row * 128 + ((slot ^ (row / 2 & 7)) << 4), which spread
// over all banks -- and leaves as 16 stores of 8 whole rows.  False: not this case, nothing was stored.
template <class PT, class V4>
__device__ __forceinline__ bool store_rows_bf16_tile16(const PT &P, const epi_uniform_t &H, unsigned lds_part,
        const V4 (&acc)[8][4], long b, long m_base, long n_base) {
    typedef unsigned v2u_t __attribute__((ext_vector_type(2)));
    typedef unsigned v4u_t __attribute__((ext_vector_type(4)));
    typedef v2u_t __attribute__((address_space(3), may_alias)) *lds_u2_ptr_t;
    typedef v4u_t __attribute__((address_space(3), may_alias)) *lds_u4_ptr_t;
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    if (m_base >= P.M) return true; // nothing of this wavefront's part is inside dst
    if (H.n_po != 0 || H.bias_mode != 0 || H.ds_mode != 0 || H.dzp_mode != 0 || H.dynamic || H.dst_dt != MI355_DT_BF16)
        return false;
    if (((uintptr_t)P.dst & 15) || (P.ds[0] % 8) || (P.ds[1] % 8)) return false;
    const int lane = threadIdx.x & 63, lrow = lane & 15, q = lane >> 4;
    const long rows_left = P.M - m_base;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = 16 * i + lrow;
        bool special = false;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) special |= __builtin_amdgcn_classf(acc[i][j][e], 0x93); // NaN or subnormal
        const bool soft = __builtin_amdgcn_ballot_w64(special) != 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v2u_t o;
            if (!soft) {
                o.x = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_t {acc[i][j][0], acc[i][j][1]}, bf16x2_t));
                o.y = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_t {acc[i][j][2], acc[i][j][3]}, bf16x2_t));
            } else {
                o.x = f32_to_bf16(acc[i][j][0]) | ((unsigned)f32_to_bf16(acc[i][j][1]) << 16);
                o.y = f32_to_bf16(acc[i][j][2]) | ((unsigned)f32_to_bf16(acc[i][j][3]) << 16);
            }
            // columns 16 j + 4 q ..: byte 32 j + 8 q of the row = slot 2 j + q / 2, half q % 2
            const int slot = 2 * j + (q >> 1);
            *(lds_u2_ptr_t)(size_t)(lds_part + (unsigned)(r * 128 + ((slot ^ ((r >> 1) & 7)) << 4) + 8 * (q & 1))) = o;
        }
    }
    // (a wavefront reads back what its own lanes wrote: program order, no barrier)
    char *dbase = (char *)P.dst + (b * P.ds[0] + m_base * P.ds[1] + n_base) * 2;
    const int wr = lane >> 3, wslot = lane & 7;
#pragma unroll
    for (int d = 0; d < 16; ++d) {
        const long r = d * 8 + wr;
        const int chunk = wslot ^ (int)((r >> 1) & 7);
        const v4u_t v = *(lds_u4_ptr_t)(size_t)(lds_part + (unsigned)(d * 1024 + lane * 16));
        if (r < rows_left) __builtin_nontemporal_store(v, (v4u_t *)(dbase + r * P.ds[1] * 2 + chunk * 16));
    }
    return true;
}

// The epilogue of one wavefront's 128 x WCOLS part.
//   park      the idle tile ring: every wavefront owns 16 KB of it (the general path parks
//             Q x 64 x 16 bytes there, the specialised chains stage their part of dst)
//   ntab      LDS byte address of the per-column table (filled before the K loop)
//   m_base    first row of the wavefront's part, n_base its first column, col0 =
//             that column's index inside the tile (the table's index)
//   conv      the kernel's conversion of raw accumulators:
//                 row_t row_data(m)                         per-row operand
//                 quad(raw, row_t, ntab, col, float (&f)[4])
//                 bool hot_chain(P, H, ntab, lds_part, acc, b, m_base, n_base, col0)
//                     the whole epilogue of the wavefront for the chains the kernel
//                     specialises at compile time (false: not one of them)
template <class Layout, int WCOLS, class PT, class T, int R, int C, class Conv>
__device__ __forceinline__ void store_quadrant(const PT &P, char *park, unsigned ntab, const T (&acc)[R][C],
        long b, long m_base, long n_base, int col0, const Conv &conv) {
    constexpr int Q = Layout::template nq<C>();
    constexpr int RB = Layout::RB, NB = Layout::NB, QPG = Layout::QPG;
    static_assert(R == NB, "row blocks");
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int lrow = Layout::lrow(lane);
    const bool cols_inside = n_base + WCOLS <= P.N;
    const epi_uniform_t H = make_uniform(P, cols_inside);
    typedef typename Conv::row_t row_t;

    // the benchmark configurations' chains, specialised at compile time by the kernel
    {
        // the wavefront's share of the idle tile ring: 16 KB
        const unsigned lds_part = (unsigned)(size_t)(__attribute__((address_space(3))) char *)park
                + (unsigned)__builtin_amdgcn_readfirstlane(wave) * 16384u;
        if (H.fast && conv.hot_chain(P, H, ntab, lds_part, acc, b, m_base, n_base, col0)) return;
    }

    if (H.fast) {
        int col[Q];
        long n[Q];
#pragma unroll
        for (int k = 0; k < Q; ++k) {
            col[k] = col0 + Layout::qcol(k, lane);
            n[k] = n_base + Layout::qcol(k, lane);
        }
        const int sbytes = H.staged != STG_NONE ? dt_bits(H.staged_dt) / 8 : 0;
        // the staged stream's quads of a row, as raw 8 or 16 bytes
        auto load_staged = [&](long m, uint4 (&s)[Q]) __attribute__((always_inline)) {
            const char *base = H.staged_p + (b * H.st_s0 + m * H.st_s1 + n_base) * sbytes;
            if (sbytes == 2) {
#pragma unroll
                for (int k = 0; k < Q; ++k) {
                    const uint2 q = *(const uint2 *)(base + Layout::qcol(k, lane) * 2);
                    s[k].x = q.x; s[k].y = q.y; s[k].z = 0; s[k].w = 0;
                }
            } else {
#pragma unroll
                for (int k = 0; k < Q; ++k) s[k] = *(const uint4 *)(base + Layout::qcol(k, lane) * 4);
            }
        };
        auto row_of = [&](int i) { return m_base + i * RB + lrow; };
        auto clamp_row = [&](long m) { return m < P.M ? m : P.M - 1; };
        uint4 snext[Q];
#pragma unroll
        for (int k = 0; k < Q; ++k) snext[k] = make_uint4(0, 0, 0, 0);
        row_t rnext = conv.row_data(clamp_row(row_of(0)));
        if (H.staged != STG_NONE) load_staged(clamp_row(row_of(0)), snext);
#pragma unroll 1
        for (int i = 0; i < NB; ++i) {
            T a[C];
            Layout::pick_rows(acc, i, a);
            const long m = row_of(i);
            const bool ok = m < P.M;
            const row_t rd = rnext;
            uint4 scur[Q];
#pragma unroll
            for (int k = 0; k < Q; ++k) scur[k] = snext[k];
            if (i + 1 < NB) {
                const long mn = clamp_row(row_of(i + 1));
                rnext = conv.row_data(mn);
                if (H.staged != STG_NONE) load_staged(mn, snext);
            }
            float v[Q][4], sy[Q][4];
#pragma unroll
            for (int k = 0; k < Q; ++k) conv.quad(Layout::quad(a, k), rd, ntab, col[k], v[k]);
#pragma unroll
            for (int k = 0; k < Q; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) sy[k][e] = 0.f;
            if (H.staged != STG_NONE) {
                // one dispatch on the data type for the Q quads
                if (H.staged_dt == MI355_DT_BF16) {
#pragma unroll
                    for (int k = 0; k < Q; ++k) staged4(MI355_DT_BF16, scur[k], sy[k]);
                } else if (H.staged_dt == MI355_DT_F32) {
#pragma unroll
                    for (int k = 0; k < Q; ++k) staged4(MI355_DT_F32, scur[k], sy[k]);
                } else if (H.staged_dt == MI355_DT_F16) {
#pragma unroll
                    for (int k = 0; k < Q; ++k) staged4(MI355_DT_F16, scur[k], sy[k]);
                } else {
#pragma unroll
                    for (int k = 0; k < Q; ++k) staged4(MI355_DT_S32, scur[k], sy[k]);
                }
            }
            apply_epilogueQ<Q>(H, ntab, col, v, sy);
            if (H.dynamic == MI355_DST_DYNAMIC_MX) dynamic_quantQ<Layout, Q, false>(P, H.dst_dt, v, b, ok ? m : P.M - 1, ok, n, lane);
            else if (H.dynamic) dynamic_quantQ<Layout, Q, true>(P, H.dst_dt, v, b, ok ? m : P.M - 1, ok, n, lane);
            storeQ<Q>(P, H, v, b, m, ok, n);
        }
        return;
    }

    // ---- general path: the quads of a row block parked in lane-private LDS, then
    // one group of 32 columns at a time through the interpreter
    static_assert(Q * 64 * 16 <= 16384, "a wavefront's share of the ring");
    park_u4_t *pk = (park_u4_t *)(park + wave * 16384); // the same 16 KB share the specialised chains use
#pragma unroll 1
    for (int i = 0; i < NB; ++i) {
        {
            T a[C];
            Layout::pick_rows(acc, i, a);
#pragma unroll
            for (int k = 0; k < Q; ++k) {
                const v4i_t q = Layout::quad(a, k);
                pk[k * 64 + lane] = make_uint4((unsigned)q[0], (unsigned)q[1], (unsigned)q[2], (unsigned)q[3]);
            }
        }
        const long m = m_base + i * RB + lrow;
        const bool okm = m < P.M;
        const long mv = okm ? m : P.M - 1;
        const row_t rd = conv.row_data(mv);
        const float dt_max = P.dst_dt == MI355_DT_F8_E4M3 ? 448.f : (P.dst_dt == MI355_DT_F4_E2M1 ? 6.f : 57344.f);
        const int em = (int)f32_to_e8m0(dt_max);
#pragma unroll 1
        for (int g = 0; g < Q / QPG; ++g) {
            float v[QPG][4];
            long nq[QPG];
            int nvalid[QPG];
            float amax = 0.f;
#pragma unroll
            for (int kk = 0; kk < QPG; ++kk) {
                const int k = g * QPG + kk;
                const int qc = Layout::qcol(k, lane);
                nq[kk] = n_base + qc;
                const long left = P.N - nq[kk];
                nvalid[kk] = left >= 4 ? 4 : left > 0 ? (int)left : 0;
                const uint4 raw = pk[k * 64 + lane];
                conv.quad(v4i_t {(int)raw.x, (int)raw.y, (int)raw.z, (int)raw.w}, rd, ntab, col0 + qc, v[kk]);
                if (nvalid[kk] > 0) apply_epilogue4(P, v[kk], b, mv, nq[kk], nvalid[kk]);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (e >= nvalid[kk]) v[kk][e] = 0.f;
                amax = fmaxf(amax, amax4(v[kk]));
            }
            if (H.dynamic == MI355_DST_DYNAMIC_FP) {
                // groups of 16 columns with an f8_e4m3 scale (ref_matmul.cpp:352-365, :381): the lower and the
                // upper half of this lane's quads of the 32 columns, shared with the same partner lanes.  N is a
                // multiple of 16: a group is whole or absent
                constexpr int HQ = QPG / 2;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    float hmax = 0.f;
#pragma unroll
                    for (int kk = 0; kk < HQ; ++kk) hmax = fmaxf(hmax, amax4(v[h * HQ + kk]));
                    hmax = Layout::group_max(hmax);
                    float scale = hmax / dt_max;
                    scale = fminf(scale, 448.f);
                    scale = fmaxf(scale, 0.125f);
                    const uint8_t sbyte = f32_to_e4m3(scale);
                    const float inv = 1.f / e4m3_to_f32(sbyte);
#pragma unroll
                    for (int kk = 0; kk < HQ; ++kk)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            v[h * HQ + kk][e] = fminf(fmaxf(v[h * HQ + kk][e] * inv, -dt_max), dt_max);
                    if (okm && nvalid[h * HQ] > 0 && Layout::group_leader(lane))
                        ((uint8_t *)P.dst_scale.p)[quant_off(P.dst_scale, b, m, nq[h * HQ] & ~15L, P.M, P.N)] = sbyte;
                }
            } else if (H.dynamic) {
                // N is a multiple of 32: a group is whole or absent
                amax = Layout::group_max(amax);
                float inv;
                const uint8_t sbyte = mx_scale_byte(amax, em, inv);
#pragma unroll
                for (int kk = 0; kk < QPG; ++kk)
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[kk][e] = fminf(fmaxf(v[kk][e] * inv, -dt_max), dt_max);
                if (okm && nvalid[0] > 0 && Layout::group_leader(lane))
                    ((uint8_t *)P.dst_scale.p)[quant_off(P.dst_scale, b, m, nq[0] & ~31L, P.M, P.N)] = sbyte;
            }
#pragma unroll
            for (int kk = 0; kk < QPG; ++kk)
                if (okm && nvalid[kk] > 0) store4(P, H.dst_vec, v[kk], b, m, nq[kk], nvalid[kk]);
        }
    }
}

} // namespace gemm
} // namespace mi355
