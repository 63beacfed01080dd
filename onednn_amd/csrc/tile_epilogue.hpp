// Epilogue of the LDS-tiled MFMA kernels.
//
// After the K loop every wavefront owns a 128 x WCOLS part of the tile in
// accumulator registers (WCOLS = 128 with four wavefronts per workgroup, 64
// with eight).  It leaves through LDS in four 32-row slabs; afterwards each
// lane owns four consecutive n of one row, so dst goes out in coalesced
// 4/8/16-byte stores and the per-element epilogue code exists once, in a
// rolled loop over the row groups of a slab.
//
// With one wavefront per SIMD nothing hides memory latency inside that loop,
// so every operand that does not depend on the row is loaded once per lane
// before it (dst scale, dst zero points, per-n bias, one per-n binary
// operand), and one per-element operand stream (the src1 tensor of a binary
// post-op, the old dst of a sum post-op, or a per-element bias) is prefetched
// a whole slab ahead into an LDS staging area with 16 loads in flight.
// Anything beyond that is still computed exactly, with loads inside the loop.
//
// Order of operations: ref_matmul_int8.cpp:275-306 / ref_matmul.cpp:283-331.
#pragma once
#include "mi355_device.hpp"

namespace mi355 {
namespace gemm {

typedef int v4i_t __attribute__((ext_vector_type(4)));
// The accumulator slab in LDS is written one dword at a time and read back as
// 16-byte vectors: both accesses go through may_alias types, otherwise
// type-based alias analysis lets the reads move above the writes.
typedef int __attribute__((may_alias)) slab_int_t;
typedef int __attribute__((ext_vector_type(4), may_alias)) slab_v4i_t;
typedef uint4 __attribute__((may_alias)) stage_u4_t;

__device__ __forceinline__ int raw_bits(int x) { return x; }
__device__ __forceinline__ int raw_bits(float x) { return __float_as_int(x); }

constexpr int STG_NONE = -1, STG_BIAS = 100, STG_SUM = 101;

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

struct po_reg_t {
    int kind, alg;
    float alpha, beta, scale, zpf;
};

struct epi_hoist_t {
    float bias4[4];
    float hv4[4];   // hoisted per-n operand of post-op `hoisted_po`
    float dzp4[4];
    float ds, ds_inv;
    int bias_mode;  // 0 none, 1 hoisted, 2 per element
    int ds_mode;    // 0 none, 1 divide, 2 multiply by reciprocal
    int dzp_mode;   // 0 none, 1 present
    int hoisted_po; // post-op index or -1
    int staged;     // STG_NONE, STG_BIAS, STG_SUM or a binary post-op index
    int staged_dt;
    const char *staged_p;
    long st_s0, st_s1; // element strides of the staged stream (stride along n is 1)
    // the leading "simple" post-ops (at most three), resident in registers
    po_reg_t pf0, pf1, pf2;
    int nfast; // how many of them; the rest run through the generic loop
    int n_po;
    int dst_dt, dst_vec; // dst_vec: four consecutive n leave as one aligned store
    int batchable;       // every operand is hoisted or staged and every post-op is a register-resident one
    int dynamic;         // MI355_DST_DYNAMIC_*: the dst scale is an output, computed per 32 columns of a row
};

__device__ __forceinline__ bool vec_ok(const void *p, long s0, long s1, int bits) {
    // four consecutive elements must form one aligned 8- or 16-byte vector
    const int bytes4 = bits / 2;
    return (bits == 16 || bits == 32) && (((uintptr_t)p) % bytes4) == 0 && (s0 % 4) == 0
            && (s1 % 4) == 0;
}

__device__ __forceinline__ bool vec_ok_store(const void *p, long s0, long s1, int bits) {
    const int bytes4 = bits / 2; // bytes of four elements
    const long e4 = bits == 8 ? 4 : 4; // strides are in elements: need multiples of 4
    return (bits == 8 || bits == 16 || bits == 32) && (((uintptr_t)p) % bytes4) == 0
            && (s0 % e4) == 0 && (s1 % e4) == 0;
}

template <class PT>
__device__ __forceinline__ epi_hoist_t make_hoist(const PT &P, long b, long nbase, int nvalid,
        bool interior) {
    epi_hoist_t H;
    H.bias_mode = 0; H.ds_mode = 0; H.dzp_mode = 0; H.hoisted_po = -1; H.staged = STG_NONE;
    H.staged_dt = 0; H.staged_p = nullptr; H.st_s0 = H.st_s1 = 0; H.ds = 1.f; H.ds_inv = 1.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) { H.bias4[e] = 0.f; H.hv4[e] = 0.f; H.dzp4[e] = 0.f; }
    if (P.bias_dt != MI355_DT_UNDEF) {
        if (P.bs[1] == 0) {
            H.bias_mode = 1;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (e < nvalid) H.bias4[e] = load_float(P.bias_dt, P.bias, b * P.bs[0] + (nbase + e) * P.bs[2]);
        } else {
            H.bias_mode = 2;
        }
    }
    H.dynamic = P.dst_dynamic;
    if (P.dst_scale.dt != MI355_DT_UNDEF && !P.dst_dynamic) {
        H.ds = load_float(P.dst_scale.dt, P.dst_scale.p, 0);
        H.ds_inv = 1.f / H.ds;
        H.ds_mode = P.dst_scale_mode == MI355_DST_SCALE_RECIPROCAL ? 2 : 1;
    }
    if (P.dst_zp.dt != MI355_DT_UNDEF) {
        H.dzp_mode = 1;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (e < nvalid)
                H.dzp4[e] = (float)((const int *)P.dst_zp.p)[(P.dst_zp.mask & 4) ? nbase + e : 0];
    }
    H.n_po = P.n_po;
    H.dst_dt = P.dst_dt;
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
                            || r.alg == MI355_ELTWISE_CLIP_V2);
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
    int first_sum = -1;
    for (int i = 0; i < P.n_po; ++i) {
        const auto &po = P.po[i];
        if (po.kind == MI355_PO_BINARY) {
            if (po.s1 == 0 && H.hoisted_po < 0) {
                H.hoisted_po = i;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (e < nvalid) H.hv4[e] = load_float(po.dt, po.p, b * po.s0 + (nbase + e) * po.s2);
            } else if (po.s1 != 0 && po.s2 == 1 && H.staged == STG_NONE && interior
                    && vec_ok(po.p, po.s0, po.s1, dt_bits(po.dt))) {
                H.staged = i; H.staged_dt = po.dt; H.staged_p = (const char *)po.p;
                H.st_s0 = po.s0; H.st_s1 = po.s1;
            }
        } else if (po.kind == MI355_PO_SUM && first_sum < 0) {
            first_sum = i;
        }
    }
    if (H.staged == STG_NONE && interior && first_sum >= 0 && P.ds[2] == 1
            && vec_ok(P.dst, P.ds[0], P.ds[1], dt_bits(P.sum_dt))) {
        H.staged = STG_SUM; H.staged_dt = P.sum_dt; H.staged_p = (const char *)P.dst;
        H.st_s0 = P.ds[0]; H.st_s1 = P.ds[1];
    }
    if (H.staged == STG_NONE && interior && H.bias_mode == 2 && P.bs[2] == 1
            && vec_ok(P.bias, P.bs[0], P.bs[1], dt_bits(P.bias_dt))) {
        H.staged = STG_BIAS; H.staged_dt = P.bias_dt; H.staged_p = (const char *)P.bias;
        H.st_s0 = P.bs[0]; H.st_s1 = P.bs[1];
    }
    // The batched epilogue (several row quads per dispatch) needs every operand in
    // registers or in the staging area: no loads inside the loop.
    H.batchable = H.n_po == H.nfast && (H.bias_mode != 2 || H.staged == STG_BIAS) && nvalid == 4 && H.dst_vec;
    {
        auto operand_ready = [&](const po_reg_t &r, int i) {
            if (r.kind == MI355_PO_BINARY)
                return (i == H.hoisted_po || i == H.staged) && (r.alg == MI355_BINARY_ADD || r.alg == MI355_BINARY_MUL);
            if (r.kind == MI355_PO_SUM) return H.staged == STG_SUM;
            return true; // grab() admits the five cheap eltwise algorithms only
        };
        const int dd = H.dst_dt;
        if (dd != MI355_DT_S8 && dd != MI355_DT_U8 && dd != MI355_DT_BF16 && dd != MI355_DT_F32 && dd != MI355_DT_S32
                && dd != MI355_DT_F8_E4M3 && dd != MI355_DT_F8_E5M2 && dd != MI355_DT_F16)
            H.batchable = 0;
        if (H.nfast > 0 && !operand_ready(H.pf0, 0)) H.batchable = 0;
        if (H.nfast > 1 && !operand_ready(H.pf1, 1)) H.batchable = 0;
        if (H.nfast > 2 && !operand_ready(H.pf2, 2)) H.batchable = 0;
    }
    return H;
}

// decode four packed 16- or 32-bit values (one dispatch for the four)
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

// eltwise on four values: one dispatch, four bodies (the cheap algorithms)
__device__ __forceinline__ void eltwise4_simple(int alg, float (&v)[4], float alpha, float beta,
        float scale) {
    if (alg == MI355_ELTWISE_RELU) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (v[e] > 0 ? v[e] : v[e] * alpha) * scale;
    } else if (alg == MI355_ELTWISE_LINEAR) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (alpha * v[e] + beta) * scale;
    } else if (alg == MI355_ELTWISE_GELU_TANH) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = gelu_tanh_fast(v[e]) * scale;
    } else if (alg == MI355_ELTWISE_CLIP) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = eltwise_f(MI355_ELTWISE_CLIP, v[e], alpha, beta) * scale;
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = eltwise_f(MI355_ELTWISE_CLIP_V2, v[e], alpha, beta) * scale;
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

template <class PT>
__device__ __forceinline__ void apply_epilogue4(const PT &P, const epi_hoist_t &H, float (&v)[4],
        long b, long m, long nbase, int nvalid, const uint4 &stg) {
    float sy[4] = {0.f, 0.f, 0.f, 0.f};
    if (H.staged != STG_NONE) staged4(H.staged_dt, stg, sy);
    if (H.bias_mode == 1) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += H.bias4[e];
    } else if (H.bias_mode == 2) {
        if (H.staged == STG_BIAS) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += sy[e];
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (e < nvalid)
                    v[e] += load_float(P.bias_dt, P.bias, b * P.bs[0] + m * P.bs[1] + (nbase + e) * P.bs[2]);
        }
    }
    if (H.n_po > 0) {
        float dst_old[4] = {0.f, 0.f, 0.f, 0.f};
        if (P.sum_dt != MI355_DT_UNDEF) {
            if (H.staged == STG_SUM) {
#pragma unroll
                for (int e = 0; e < 4; ++e) dst_old[e] = sy[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (e < nvalid)
                        dst_old[e] = load_float(P.sum_dt, P.dst,
                                b * P.ds[0] + m * P.ds[1] + (nbase + e) * P.ds[2]);
            }
        }
        auto binary_operand = [&](int i, float (&y)[4]) {
            if (i == H.hoisted_po) {
#pragma unroll
                for (int e = 0; e < 4; ++e) y[e] = H.hv4[e];
            } else if (i == H.staged) {
#pragma unroll
                for (int e = 0; e < 4; ++e) y[e] = sy[e];
            } else {
                const auto &po = P.po[i];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    y[e] = e < nvalid ? load_float(po.dt, po.p, b * po.s0 + m * po.s1 + (nbase + e) * po.s2)
                                      : 0.f;
            }
        };
        auto binary4 = [&](int alg, const float (&y)[4]) {
            if (alg == MI355_BINARY_ADD) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] + y[e];
            } else if (alg == MI355_BINARY_MUL) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] * y[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = binary_f(alg, v[e], y[e]);
            }
        };
        auto fast_op = [&](const po_reg_t &r, int i) {
            if (r.kind == MI355_PO_ELTWISE) {
                eltwise4_simple(r.alg, v, r.alpha, r.beta, r.scale);
            } else if (r.kind == MI355_PO_BINARY) {
                float y[4];
                binary_operand(i, y);
                binary4(r.alg, y);
            } else { // sum
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] += r.scale * (dst_old[e] - r.zpf);
            }
        };
        if (H.nfast > 0) fast_op(H.pf0, 0);
        if (H.nfast > 1) fast_op(H.pf1, 1);
        if (H.nfast > 2) fast_op(H.pf2, 2);
#pragma unroll 1
        for (int i = H.nfast; i < H.n_po; ++i) {
            const auto &po = P.po[i];
            const int kind = po.kind;
            if (kind == MI355_PO_ELTWISE) {
                eltwise4_any(po.alg, v, po.alpha, po.beta, po.scale);
            } else if (kind == MI355_PO_BINARY) {
                float y[4];
                binary_operand(i, y);
                binary4(po.alg, y);
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
    if (H.ds_mode == 1) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] /= H.ds;
    } else if (H.ds_mode == 2) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] *= H.ds_inv;
    }
    if (H.dzp_mode) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += H.dzp4[e];
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
        default:
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = cvt_store_bits(dt, v[e]);
            break;
    }
}

template <class PT>
__device__ __forceinline__ void store4(const PT &P, const epi_hoist_t &H, const float (&v)[4], long b,
        long m, long n, int nvalid) {
    const long off = b * P.ds[0] + m * P.ds[1] + n * P.ds[2];
    uint32_t w[4];
    cvt4(H.dst_dt, v, w);
    const int bits = dt_bits(H.dst_dt);
    if (nvalid == 4 && H.dst_vec) {
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

// ---- batched form: NQ row quads per dispatch.  Every data-type and post-op
// dispatch below is uniform over the wavefront and is taken once for the NQ
// quads, and the quads' LDS reads and stores overlap; with one wavefront per
// SIMD a dispatch per quad leaves the SIMD idle through every branch.
template <int NQ>
__device__ __forceinline__ void eltwiseQ_simple(int alg, float (&v)[NQ][4], float alpha, float beta, float scale) {
    if (alg == MI355_ELTWISE_RELU) {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] = (v[k][e] > 0 ? v[k][e] : v[k][e] * alpha) * scale;
    } else if (alg == MI355_ELTWISE_LINEAR) {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] = (alpha * v[k][e] + beta) * scale;
    } else if (alg == MI355_ELTWISE_GELU_TANH) {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] = gelu_tanh_fast(v[k][e]) * scale;
    } else if (alg == MI355_ELTWISE_CLIP) {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] = eltwise_f(MI355_ELTWISE_CLIP, v[k][e], alpha, beta) * scale;
    } else {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] = eltwise_f(MI355_ELTWISE_CLIP_V2, v[k][e], alpha, beta) * scale;
    }
}

template <int NQ>
__device__ __forceinline__ void apply_epilogueQ(const epi_hoist_t &H, float (&v)[NQ][4], const uint4 (&stg)[NQ]) {
    float sy[NQ][4];
#pragma unroll
    for (int k = 0; k < NQ; ++k)
#pragma unroll
        for (int e = 0; e < 4; ++e) sy[k][e] = 0.f;
    if (H.staged != STG_NONE) {
        // every array index below is a compile-time constant: a rolled loop over
        // the quads would put these arrays into private memory
        if (H.staged_dt == MI355_DT_BF16) {
#pragma unroll
            for (int k = 0; k < NQ; ++k) staged4(MI355_DT_BF16, stg[k], sy[k]);
        } else if (H.staged_dt == MI355_DT_F32) {
#pragma unroll
            for (int k = 0; k < NQ; ++k) staged4(MI355_DT_F32, stg[k], sy[k]);
        } else if (H.staged_dt == MI355_DT_F16) {
#pragma unroll
            for (int k = 0; k < NQ; ++k) staged4(MI355_DT_F16, stg[k], sy[k]);
        } else {
#pragma unroll
            for (int k = 0; k < NQ; ++k) staged4(MI355_DT_S32, stg[k], sy[k]);
        }
    }
    if (H.bias_mode == 1) {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] += H.bias4[e];
    } else if (H.bias_mode == 2) { // staged
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] += sy[k][e];
    }
    auto fast_op = [&](const po_reg_t &r, int i) __attribute__((always_inline)) {
        if (r.kind == MI355_PO_ELTWISE) {
            eltwiseQ_simple<NQ>(r.alg, v, r.alpha, r.beta, r.scale);
        } else if (r.kind == MI355_PO_BINARY) {
            const bool hoisted = i == H.hoisted_po;
            if (r.alg == MI355_BINARY_ADD) {
#pragma unroll
                for (int k = 0; k < NQ; ++k)
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[k][e] = v[k][e] + (hoisted ? H.hv4[e] : sy[k][e]);
            } else { // mul (nothing else is batchable)
#pragma unroll
                for (int k = 0; k < NQ; ++k)
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[k][e] = v[k][e] * (hoisted ? H.hv4[e] : sy[k][e]);
            }
        } else { // sum: the old dst is the staged stream
#pragma unroll
            for (int k = 0; k < NQ; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) v[k][e] += r.scale * (sy[k][e] - r.zpf);
        }
    };
    if (H.nfast > 0) fast_op(H.pf0, 0);
    if (H.nfast > 1) fast_op(H.pf1, 1);
    if (H.nfast > 2) fast_op(H.pf2, 2);
    if (H.ds_mode == 1) {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] /= H.ds;
    } else if (H.ds_mode == 2) {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] *= H.ds_inv;
    }
    if (H.dzp_mode) {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] += H.dzp4[e];
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

// Dynamic (MX) quantization of dst for NQ quads (ref_matmul.cpp:338-423): a
// group is 32 consecutive n of one row = the quads of 8 consecutive lanes
// (`lcol` is the lane's quad number in its row).  Writes the e8m0 scale of
// every group and leaves v scaled and saturated, ready for the fp8 conversion.
template <int NQ, class PT>
__device__ __forceinline__ void dynamic_quantQ(const PT &P, const epi_hoist_t &H, float (&v)[NQ][4], long b,
        const long (&m)[NQ], long n, const bool (&ok)[NQ], int lcol) {
    const float dt_max = H.dst_dt == MI355_DT_F8_E4M3 ? 448.f : 57344.f;
    const int em = (int)f32_to_e8m0(dt_max);
#pragma unroll
    for (int k = 0; k < NQ; ++k) {
        float amax = fmaxf(fmaxf(fabsf(v[k][0]), fabsf(v[k][1])), fmaxf(fabsf(v[k][2]), fabsf(v[k][3])));
        amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
        float inv;
        const uint8_t sbyte = mx_scale_byte(amax, em, inv);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[k][e] = fminf(fmaxf(v[k][e] * inv, -dt_max), dt_max);
        if (ok[k] && (lcol & 7) == 0) ((uint8_t *)P.dst_scale.p)[quant_off(P.dst_scale, b, m[k], n, P.M, P.N)] = sbyte;
    }
}

// four full quads (nvalid == 4, vector stores allowed) to dst; `ok[k]` masks rows beyond M
template <int NQ, class PT>
__device__ __forceinline__ void storeQ(const PT &P, const epi_hoist_t &H, const float (&v)[NQ][4], long b,
        const long (&m)[NQ], long n, const bool (&ok)[NQ]) {
    uint32_t w[NQ][4];
    const int dt = H.dst_dt;
    if (dt == MI355_DT_S8 || dt == MI355_DT_U8) {
        // Round first (v_rndne + the saturating v_cvt_i32_f32, NaN -> 0), clamp as
        // integers, pack the four low bytes with byte permutes: the same values as
        // the reference's clamp-then-round (rounding is monotonic and the bounds
        // are integers) in 3 + 3/4 instructions per value instead of 7 + 7/4.
        const int lo = dt == MI355_DT_S8 ? -128 : 0, hi = dt == MI355_DT_S8 ? 127 : 255;
        const long off0b = b * P.ds[0] + n;
#pragma unroll
        for (int k = 0; k < NQ; ++k) {
            int q[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int r = (int)__builtin_rintf(v[k][e]);
                q[e] = r < lo ? lo : (r > hi ? hi : r);
            }
            const unsigned lo16 = __builtin_amdgcn_perm((unsigned)q[1], (unsigned)q[0], 0x0c0c0400u);
            const unsigned hi16 = __builtin_amdgcn_perm((unsigned)q[3], (unsigned)q[2], 0x0c0c0400u);
            const unsigned word = __builtin_amdgcn_perm(hi16, lo16, 0x05040100u);
            if (ok[k]) *(uint32_t *)((uint8_t *)P.dst + off0b + m[k] * P.ds[1]) = word;
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
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) special |= __builtin_amdgcn_classf(v[k][e], 0x93);
        if (__builtin_amdgcn_ballot_w64(special) == 0) {
            typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
            typedef float f32x2_t __attribute__((ext_vector_type(2)));
            const long off0b = b * P.ds[0] + n;
#pragma unroll
            for (int k = 0; k < NQ; ++k) {
                uint2 o;
                o.x = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_t {v[k][0], v[k][1]}, bf16x2_t));
                o.y = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_t {v[k][2], v[k][3]}, bf16x2_t));
                if (ok[k]) *(uint2 *)((uint16_t *)P.dst + off0b + m[k] * P.ds[1]) = o;
            }
            return;
        }
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) w[k][e] = f32_to_bf16(v[k][e]);
    } else if (dt == MI355_DT_F32) {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) w[k][e] = f2u(v[k][e]);
    } else if (dt == MI355_DT_F16) {
        // v_cvt_f16_f32 equals the software conversion (float16.hpp) for every
        // input, NaN payloads included: checked on the device over 4 M f32
        // bit patterns and every exponent's special mantissas
#pragma unroll
        for (int k = 0; k < NQ; ++k)
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
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) special |= __builtin_amdgcn_classf(v[k][e], 0x3);
        if (__builtin_amdgcn_ballot_w64(special) == 0) {
            typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
            typedef short s16x2_t __attribute__((ext_vector_type(2)));
            const long off0b = b * P.ds[0] + n;
#pragma unroll
            for (int k = 0; k < NQ; ++k) {
                const f16x2_t lo = {(_Float16)v[k][0], (_Float16)v[k][1]}, hi = {(_Float16)v[k][2], (_Float16)v[k][3]};
                s16x2_t r = {0, 0};
                if (dt == MI355_DT_F8_E4M3) {
                    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, lo, 1.f, false);
                    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, hi, 1.f, true);
                } else {
                    r = __builtin_amdgcn_cvt_scalef32_pk_bf8_f16(r, lo, 1.f, false);
                    r = __builtin_amdgcn_cvt_scalef32_pk_bf8_f16(r, hi, 1.f, true);
                }
                if (ok[k]) *(uint32_t *)((uint8_t *)P.dst + off0b + m[k] * P.ds[1]) = __builtin_bit_cast(uint32_t, r);
            }
            return;
        }
        if (dt == MI355_DT_F8_E4M3) {
#pragma unroll
            for (int k = 0; k < NQ; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) w[k][e] = f32_to_e4m3(v[k][e]);
        } else {
#pragma unroll
            for (int k = 0; k < NQ; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) w[k][e] = f32_to_e5m2(v[k][e]);
        }
    } else { // s32 (nothing else is batchable)
#pragma unroll
        for (int k = 0; k < NQ; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                w[k][e] = (uint32_t)(int)__builtin_rintf(sat(v[k][e], -2147483648.f, 2147483520.f));
    }
    const int bits = dt_bits(dt);
    const long off0 = b * P.ds[0] + n;
    if (bits == 8) {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
            if (ok[k])
                *(uint32_t *)((uint8_t *)P.dst + off0 + m[k] * P.ds[1])
                        = w[k][0] | (w[k][1] << 8) | (w[k][2] << 16) | (w[k][3] << 24);
    } else if (bits == 16) {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
            if (ok[k]) {
                uint2 o;
                o.x = w[k][0] | (w[k][1] << 16);
                o.y = w[k][2] | (w[k][3] << 16);
                *(uint2 *)((uint16_t *)P.dst + off0 + m[k] * P.ds[1]) = o;
            }
    } else {
#pragma unroll
        for (int k = 0; k < NQ; ++k)
            if (ok[k]) {
                uint4 o;
                o.x = w[k][0]; o.y = w[k][1]; o.z = w[k][2]; o.w = w[k][3];
                *(uint4 *)((uint32_t *)P.dst + off0 + m[k] * P.ds[1]) = o;
            }
    }
}

// One row of accumulator tiles copied by value.  The slab writers pick their rows
// with a switch over the run-time slab number; were the cases identical code on
// different addresses, the compiler would merge them into one copy that indexes
// `acc` with a run-time offset, and all accumulators would live in private memory
// from the first K step on.  The empty asm statements keep the cases apart
// (statements of inline assembly are never merged).
template <class T, int C>
__device__ __forceinline__ void copy_row(const T (&src)[C], T (&dst)[C]) {
#pragma unroll
    for (int j = 0; j < C; ++j) {
        T v = src[j];
        asm volatile("" : "+v"(v));
        dst[j] = v;
    }
}

// Accumulator layouts: how a wavefront's 128x128 quadrant sits in registers
// and how one 32-row slab of it is written to LDS as [32 rows][128 cols] s32.
//
// 32x32 MFMA tiles, acc[4][4] of 16 registers: register r of tile (i, j) holds
// row 32i + 8*(r/4) + 4*(lane/32) + r%4, column 32j + lane%32.
struct layout32_t {
    template <class T, int R, int C>
    static __device__ __forceinline__ void write_slab(const T (&acc)[R][C], int s, slab_int_t *wl, int lane) {
        constexpr int WCOLS = C * 32;
        // The stores are written as ds_write_b32 instructions by hand.  Left to
        // the compiler (ROCm 7.2) they were merged into ds_write2_b32 pairs, and
        // two stores per tile of this layout came out with their first offset
        // divided by four and landed in other cells of the slab (the parity
        // tests caught it); as volatile stores they stayed single but each one
        // was followed by a wait for the LDS queue to drain, 11-12 us per slab.
        const unsigned base = (unsigned)(size_t)(__attribute__((address_space(3))) char *)(char *)wl
                + (unsigned)(((lane >> 5) * 4 * WCOLS + (lane & 31)) * 4);
        T a[C];
        pick_rows(acc, s, a);
#pragma unroll
        for (int j = 0; j < C; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const unsigned addr = base + (unsigned)((((r >> 2) * 8 + (r & 3)) * WCOLS + j * 32) * 4);
                asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(raw_bits(a[j][r])) : "memory");
            }
        // the wavefront reads its own slab next: LDS operations of one
        // wavefront complete in order, the wait only keeps the compiler's own
        // counter bookkeeping (which does not see these stores) conservative
        asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
    }
    template <class T, int R, int C>
    static __device__ __forceinline__ void pick_rows(const T (&acc)[R][C], int s, T (&a)[C]) {
        switch (s) {
            case 0: copy_row(acc[0], a); break;
            case 1: copy_row(acc[1], a); break;
            case 2: copy_row(acc[2], a); break;
            default: copy_row(acc[3], a); break;
        }
    }
};

// 16x16 MFMA tiles, acc[8][8] of 4 registers: register r of tile (i, j) holds
// row 16i + 4*(lane/16) + r, column 16j + lane%16.
struct layout16_t {
    template <class T, int R, int C>
    static __device__ __forceinline__ void write_slab(const T (&acc)[R][C], int s, slab_int_t *wl, int lane) {
        constexpr int WCOLS = C * 16;
        slab_int_t *vw = wl;
        T a0[C], a1[C];
        switch (s) {
            case 0: copy_row(acc[0], a0); copy_row(acc[1], a1); break;
            case 1: copy_row(acc[2], a0); copy_row(acc[3], a1); break;
            case 2: copy_row(acc[4], a0); copy_row(acc[5], a1); break;
            default: copy_row(acc[6], a0); copy_row(acc[7], a1); break;
        }
#pragma unroll
        for (int j = 0; j < C; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                vw[((lane >> 4) * 4 + r) * WCOLS + j * 16 + (lane & 15)] = raw_bits(a0[j][r]);
                vw[(16 + (lane >> 4) * 4 + r) * WCOLS + j * 16 + (lane & 15)] = raw_bits(a1[j][r]);
            }
    }
};

// `conv.row(raw, m, f)` turns four raw accumulators of row m into the f32
// values that enter the epilogue.
// smem: one accumulator slab per wavefront (32 rows x WCOLS x 4 bytes), then
// as much again for operand staging.
// WCOLS: columns of the wavefront's part; NW: wavefronts of the workgroup.
template <class Layout, int WCOLS, int NW, class PT, class Acc, class Conv>
__device__ __forceinline__ void store_quadrant(const PT &P, char *smem, const Acc &acc,
        long b, long m_base, long n_base_wave, bool interior, const Conv &conv) {
    constexpr int LPR = WCOLS / 4;     // lanes per row: four consecutive n each
    constexpr int RPP = 64 / LPR;      // rows per pass of the wavefront
    constexpr int PASSES = 32 / RPP;   // passes per 32-row slab
    constexpr int SLAB_INTS = 32 * WCOLS;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int lrow = lane / LPR, lcol = lane % LPR;
    slab_int_t *wl = (slab_int_t *)smem + wave * SLAB_INTS;
    stage_u4_t *stg = (stage_u4_t *)(smem + NW * SLAB_INTS * 4) + wave * (PASSES * 64);
    const long nbase = n_base_wave + lcol * 4;
    int nvalid = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e)
        if (nbase + e < P.N) nvalid = e + 1;
    const epi_hoist_t H = make_hoist(P, b, nbase, nvalid, interior);
    const int sbytes = dt_bits(H.staged_dt) / 8;

    // rolled over the four slabs: the epilogue arithmetic exists once
#pragma unroll 1
    for (int i = 0; i < 4; ++i) {
        if (H.staged != STG_NONE) {
            // PASSES independent vector loads in flight, then park them in LDS
            uint4 tmp[PASSES];
            const char *base = H.staged_p
                    + (b * H.st_s0 + (m_base + i * 32 + lrow) * H.st_s1 + nbase) * sbytes;
            if (sbytes == 2) {
#pragma unroll
                for (int it = 0; it < PASSES; ++it) {
                    const uint2 q = *(const uint2 *)(base + (long)it * RPP * H.st_s1 * 2);
                    tmp[it].x = q.x; tmp[it].y = q.y; tmp[it].z = 0; tmp[it].w = 0;
                }
            } else {
#pragma unroll
                for (int it = 0; it < PASSES; ++it)
                    tmp[it] = *(const uint4 *)(base + (long)it * RPP * H.st_s1 * 4);
            }
#pragma unroll
            for (int it = 0; it < PASSES; ++it) stg[it * 64 + lane] = tmp[it];
        }
        Layout::write_slab(acc, i, wl, lane);
        if (H.batchable) {
            constexpr int NQ = 4;
#pragma unroll 1
            for (int it0 = 0; it0 < PASSES; it0 += NQ) {
                v4i_t raw[NQ];
                uint4 sv[NQ];
                long m[NQ];
                bool ok[NQ];
#pragma unroll
                for (int k = 0; k < NQ; ++k) {
                    const int row = (it0 + k) * RPP + lrow;
                    m[k] = m_base + i * 32 + row;
                    ok[k] = m[k] < P.M;
                    raw[k] = *(const slab_v4i_t *)&wl[row * WCOLS + lcol * 4];
                    sv[k] = make_uint4(0, 0, 0, 0);
                }
                if (H.staged != STG_NONE) {
#pragma unroll
                    for (int k = 0; k < NQ; ++k) sv[k] = stg[(it0 + k) * 64 + lane];
                }
                float v[NQ][4];
#pragma unroll
                for (int k = 0; k < NQ; ++k) conv.row(raw[k], ok[k] ? m[k] : m_base, v[k]);
                apply_epilogueQ<NQ>(H, v, sv);
                if (H.dynamic) dynamic_quantQ<NQ>(P, H, v, b, m, nbase, ok, lcol);
                storeQ<NQ>(P, H, v, b, m, nbase, ok);
            }
            continue;
        }
        if (H.dynamic) {
            // Dynamic (MX) quantization of dst, ref_matmul.cpp:338-423: a group is
            // 32 consecutive n of one row = 8 consecutive lanes of this layout
            // (four n each; a wavefront's columns start at a multiple of 64 and
            // N % 32 == 0, so a group is whole or absent).  All lanes run the
            // arithmetic and the cross-lane maximum, rows beyond M on the data of
            // a valid row; only the stores are masked.
            const float dt_max = H.dst_dt == MI355_DT_F8_E4M3 ? 448.f : 57344.f;
            const int em = (int)f32_to_e8m0(dt_max);
#pragma unroll 1
            for (int it = 0; it < PASSES; ++it) {
                const int row = it * RPP + lrow;
                const long m = m_base + i * 32 + row;
                const bool ok = m < P.M && nvalid > 0;
                const long mv = m < P.M ? m : P.M - 1;
                const v4i_t raw = *(const slab_v4i_t *)&wl[row * WCOLS + lcol * 4];
                uint4 sv = make_uint4(0, 0, 0, 0);
                if (H.staged != STG_NONE) sv = stg[it * 64 + lane];
                float v[4] = {0.f, 0.f, 0.f, 0.f};
                if (nvalid > 0) {
                    conv.row(raw, mv, v);
                    apply_epilogue4(P, H, v, b, mv, nbase, nvalid, sv);
                }
                float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
                amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
                amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
                amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
                float inv;
                const uint8_t sbyte = mx_scale_byte(amax, em, inv);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = fminf(fmaxf(v[e] * inv, -dt_max), dt_max);
                if (ok) {
                    if ((lcol & 7) == 0)
                        ((uint8_t *)P.dst_scale.p)[quant_off(P.dst_scale, b, m, nbase, P.M, P.N)] = sbyte;
                    store4(P, H, v, b, m, nbase, nvalid);
                }
            }
            continue;
        }
#pragma unroll 1
        for (int it = 0; it < PASSES; ++it) {
            const int row = it * RPP + lrow;
            const long m = m_base + i * 32 + row;
            const v4i_t raw = *(const slab_v4i_t *)&wl[row * WCOLS + lcol * 4];
            uint4 sv = make_uint4(0, 0, 0, 0);
            if (H.staged != STG_NONE) sv = stg[it * 64 + lane];
            if (m < P.M && nvalid > 0) {
                float v[4];
                conv.row(raw, m, v);
                apply_epilogue4(P, H, v, b, m, nbase, nvalid, sv);
                store4(P, H, v, b, m, nbase, nvalid);
            }
        }
    }
}

} // namespace gemm
} // namespace mi355
