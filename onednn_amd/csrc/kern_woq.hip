// "hip:woq_gemv" -- bandwidth-bound skinny GEMM for weight-only-quantized
// decode: bf16 activations (M <= 32 rows) times 4-bit weights [K][N] with N
// contiguous (tag ab: two n per byte, low nibble = even n), per-group scales
// and zero points along K, fpmath "apply_to_int" weight decompression.
//
// Semantics (ref_matmul_t, src/cpu/matmul/ref_matmul.cpp:179-235, weights
// decompression branch :193-214):
//     w[k,n]  = (f32(wei[k,n]) - f32(zp[k/G,n])) * f32(scale[k/G,n])
//     dst[m,n] = sum_k f32(src[m,k]) * w[k,n]          (f32 accumulation)
// evaluated here as
//     dst[m,n] = sum_g scale[g,n] * ( sum_{k in g} src[m,k] * (128 + wei[k,n])
//                                     - (128 + zp[g,n]) * sum_{k in g} src[m,k] )
// which is the same real number; the rounding differs (f32 accumulation order,
// and the group factor applied once per group instead of once per weight).
// The result is compared with the reference under the bf16 threshold plus the
// forward error bound of the K sum, like the reference's own JIT path, which
// rounds every decompressed weight to bf16
// (src/cpu/x64/matmul/brgemm_matmul_copy_utils.cpp:2870-2896).
//
// Why this form: the HBM stream is 4 bits per weight and the budget is ~1.4
// VALU operations per weight at 8 TB/s.  "128 + nibble" is an exact bf16 that
// costs one v_and_or per *two* weights (0x4300 | nibble, two lanes of a dword
// at once), the products run on the bf16 matrix cores, and the per-weight
// subtract/multiply of the naive formula moves to once per group and column.
//
// Data flow per wavefront step (16 k-rows x 16 lanes x 8*CHD columns):
//   lane (c = lane%16, q = lane/16) loads CHD dwords of rows k0+4q .. k0+4q+3 at
//   column chunk c; every dword yields four bf16 pairs (n, n+4) by shift+and_or;
//   the four rows of one pair are the B operand of v_mfma_f32_16x16x32_bf16
//   (MFMA k-slot 2t+h <-> row 4q+t, column half h); the A operand interleaves
//   zeros, (s,0,s,0,..) or (0,s,0,s,..), so that one MFMA yields column n and a
//   second one column n+4.  An MFMA against an all-ones B gives sum_k src[m,k].
//
// Work split: grid = column chunks x K splits; the 4 wavefronts of a workgroup
// take consecutive K sub-ranges, reduce through LDS, and the workgroup writes
// one f32 partial [M][chunk] to scratch.  The last workgroup to arrive for a
// chunk (epoch-stamped arrival counter in scratch, so scratch needs no
// initialisation) adds the partials in split order -- deterministic -- and runs
// the shared epilogue.
#include <stdlib.h>

#include <atomic>

#include "kernels.hpp"

namespace mi355 {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

constexpr int COUNTER_BYTES = 4096; // up to 1024 column chunks

struct woq_extra_t {
    unsigned *counters; // [chunks] epoch-stamped arrival counters
    float *partials;    // [ksplit][M][N]
    unsigned epoch;     // 24-bit, never 0
    int ksplit;         // K splits across workgroups
    int krange;         // k per workgroup (multiple of 64)
    int G;              // k per quantization group (multiple of 16), K if ungrouped
    int sc_grouped, zp_grouped; // parameter has a K dimension
    int zp_common;      // single zero point
    int signed_w;       // s4 weights
};

__device__ __forceinline__ v8bf as_bf(const v4i &x) { return __builtin_bit_cast(v8bf, x); }

// NPL consecutive parameter values held as raw 32-bit words -> f32; one
// data-type dispatch, fully unrolled bodies (static register indices)
template <int NPL>
__device__ __forceinline__ void decode_raw(int dt, const uint4 (&r)[NPL / 4], float (&out)[NPL]) {
    unsigned w[NPL];
#pragma unroll
    for (int i = 0; i < NPL / 4; ++i) {
        w[4 * i] = r[i].x; w[4 * i + 1] = r[i].y; w[4 * i + 2] = r[i].z; w[4 * i + 3] = r[i].w;
    }
    switch (dt) {
        case MI355_DT_F32:
#pragma unroll
            for (int i = 0; i < NPL; ++i) out[i] = u2f(w[i]);
            break;
        case MI355_DT_S32:
#pragma unroll
            for (int i = 0; i < NPL; ++i) out[i] = (float)(int)w[i];
            break;
        case MI355_DT_BF16:
#pragma unroll
            for (int i = 0; i < NPL; ++i) out[i] = u2f((w[i / 2] >> ((i & 1) * 16)) << 16);
            break;
        case MI355_DT_F16:
#pragma unroll
            for (int i = 0; i < NPL; ++i) out[i] = f16_to_f32((uint16_t)(w[i / 2] >> ((i & 1) * 16)));
            break;
        case MI355_DT_S8:
#pragma unroll
            for (int i = 0; i < NPL; ++i) out[i] = (float)(int)(int8_t)((w[i / 4] >> ((i & 3) * 8)) & 0xffu);
            break;
        case MI355_DT_U8:
#pragma unroll
            for (int i = 0; i < NPL; ++i) out[i] = (float)((w[i / 4] >> ((i & 3) * 8)) & 0xffu);
            break;
        case MI355_DT_S4:
#pragma unroll
            for (int i = 0; i < NPL; ++i) out[i] = (float)s4_to_int((uint8_t)((w[i / 8] >> ((i & 7) * 4)) & 0xfu));
            break;
        default: // u4
#pragma unroll
            for (int i = 0; i < NPL; ++i) out[i] = (float)((w[i / 8] >> ((i & 7) * 4)) & 0xfu);
            break;
    }
}

// NWV wavefronts per workgroup share one column chunk and split its K range.
template <int CHD, int MT, int NWV>
__global__ void __launch_bounds__(NWV * 64) woq_gemv_kernel(const problem_t P_, const woq_extra_t X) {
    const auto &P = MI355_KERNARG_PROBLEM();
    extern __shared__ __attribute__((aligned(16))) float red[]; // [4][M][NW]
    constexpr int NPL = CHD * 8;      // columns per lane
    constexpr int NW = 16 * NPL;      // columns per wavefront / workgroup
    constexpr int NP = CHD * 4;       // bf16 pairs per lane per row
    constexpr int WOQ_NT = NWV * 64;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int c = lane & 15, q = lane >> 4;
    const int chunk = blockIdx.x, split = blockIdx.y;
    const long N = P.N, K = P.K;
    const int M = (int)P.M;
    const long n_lane = (long)chunk * NW + c * NPL; // first column of this lane
    const bool lane_on = n_lane < N;                // N is a multiple of NPL

    // K sub-range of this wavefront: quarter of the workgroup's range, in 16-row steps
    const int kr4 = X.krange / NWV;
    long kb = (long)split * X.krange + (long)wave * kr4;
    long ke = kb + kr4;
    if (ke > K) ke = K;

    const uint8_t *wei = (const uint8_t *)P.wei;
    const long row_bytes = N / 2;
    const uint16_t *src = (const uint16_t *)P.src;
    const long lds = P.ss[1];

    v4f acc[NP][2][MT], rs[MT];
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc[p][h][mt] = v4f {0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) rs[mt] = v4f {0.f, 0.f, 0.f, 0.f};

    struct step_t {
        unsigned w[4][CHD]; // rows 4q+t, dwords of this lane's chunk
        uint2 a[MT];        // src[m][k0+4q .. +3] as four bf16
    };
    auto load_step = [&](step_t &s, long k0) __attribute__((always_inline)) {
        const long kr = k0 + 4 * q;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            const uint8_t *p = wei + (kr + tt) * row_bytes + n_lane / 2;
            if (CHD == 4) {
                uint4 v = lane_on ? *(const uint4 *)p : make_uint4(0, 0, 0, 0);
                s.w[tt][0] = v.x; s.w[tt][1 % CHD] = v.y; s.w[tt][2 % CHD] = v.z; s.w[tt][3 % CHD] = v.w;
            } else if (CHD == 2) {
                uint2 v = lane_on ? *(const uint2 *)p : make_uint2(0, 0);
                s.w[tt][0] = v.x; s.w[tt][1 % CHD] = v.y;
            } else {
                s.w[tt][0] = lane_on ? *(const unsigned *)p : 0u;
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + c;
            s.a[mt] = m < M ? *(const uint2 *)(src + (long)m * lds + kr) : make_uint2(0, 0);
        }
    };

    const unsigned sx = X.signed_w ? 0x88888888u : 0u; // s4 -> offset-binary
    const v4i ones = {0x3F803F80, 0x3F803F80, 0x3F803F80, 0x3F803F80};
    auto compute_step = [&](const step_t &s) __attribute__((always_inline)) {
        v4i aa[MT], ab[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const unsigned x = s.a[mt].x, y = s.a[mt].y;
            aa[mt] = v4i {(int)(x & 0xffffu), (int)(x >> 16), (int)(y & 0xffffu), (int)(y >> 16)};
            ab[mt] = v4i {(int)(x << 16), (int)(x & 0xffff0000u), (int)(y << 16), (int)(y & 0xffff0000u)};
            rs[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf(aa[mt]), as_bf(ones), rs[mt], 0, 0, 0);
        }
#pragma unroll
        for (int d = 0; d < CHD; ++d) {
#pragma unroll
            for (int sh = 0; sh < 4; ++sh) {
                v4i b;
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
                    b[tt] = (int)((((s.w[tt][d] ^ sx) >> (4 * sh)) & 0x000F000Fu) | 0x43004300u);
                const int p = d * 4 + sh;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc[p][0][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf(aa[mt]), as_bf(b), acc[p][0][mt], 0, 0, 0);
                    acc[p][1][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf(ab[mt]), as_bf(b), acc[p][1][mt], 0, 0, 0);
                }
            }
        }
    };

    // Quantization parameters of one group for this lane's NPL columns, fetched
    // as raw vectors (no data-type dispatch between the loads, so they are all
    // in flight together) when the group starts and decoded when it ends.
    constexpr int RAWQ = NPL / 4; // uint4 registers for NPL 32-bit values
    struct qraw_t {
        uint4 s[RAWQ], z[RAWQ];
    };
    const int sc_bits = dt_bits(P.wei_scale.dt), zp_bits = dt_bits(P.wei_zp.dt);
    const bool with_sc = P.wei_scale.dt != MI355_DT_UNDEF, with_zp = P.wei_zp.dt != MI355_DT_UNDEF;
    auto load_raw = [&](uint4 (&r)[RAWQ], const void *base, long elem_off, int bits) {
        // NPL consecutive elements of `bits` bits starting at element elem_off
        const char *p = (const char *)base + elem_off * bits / 8;
        const int bytes = NPL * bits / 8;
#pragma unroll
        for (int i = 0; i < RAWQ; ++i) {
            r[i] = make_uint4(0, 0, 0, 0);
            if (i * 16 + 16 <= bytes) r[i] = *(const uint4 *)(p + i * 16);
            else if (i * 16 + 8 <= bytes) {
                const uint2 v = *(const uint2 *)(p + i * 16);
                r[i].x = v.x; r[i].y = v.y;
            } else if (i * 16 + 4 <= bytes) r[i].x = *(const unsigned *)(p + i * 16);
        }
    };
    auto fetch_group = [&](qraw_t &qr, long g) __attribute__((always_inline)) {
        if (!lane_on) return;
        if (with_sc) load_raw(qr.s, P.wei_scale.p, (X.sc_grouped ? g * N : 0) + n_lane, sc_bits);
        if (with_zp && !X.zp_common) load_raw(qr.z, P.wei_zp.p, (X.zp_grouped ? g * N : 0) + n_lane, zp_bits);
    };
    const float zp_common_val = (with_zp && X.zp_common) ? load_float(P.wei_zp.dt, P.wei_zp.p, 0) : 0.f;

    // fold one finished group into this wavefront's LDS slice:
    //   red[wave][m][n] (+)= scale * (acc - (128 + zp) * rowsum)
    bool first_flush = true;
    auto flush_group = [&](const qraw_t &qr) __attribute__((always_inline)) {
        float sc[NPL], zc[NPL];
        const float zbase = (X.signed_w ? 136.f : 128.f) + zp_common_val;
#pragma unroll
        for (int i = 0; i < NPL; ++i) { sc[i] = 1.f; zc[i] = 0.f; }
        if (with_sc && lane_on) decode_raw<NPL>(P.wei_scale.dt, qr.s, sc);
        if (with_zp && !X.zp_common && lane_on) decode_raw<NPL>(P.wei_zp.dt, qr.z, zc);
#pragma unroll
        for (int i = 0; i < NPL; ++i) zc[i] += zbase;
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int i = (p / 4) * 8 + h * 4 + (p % 4); // column of (pair p, half h)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int m = mt * 16 + q * 4 + r;
                        if (m < M) {
                            float *slot = &red[((long)wave * M + m) * NW + c * NPL + i];
                            const float tmp = __builtin_fmaf(-zc[i], rs[mt][r], acc[p][h][mt][r]);
                            *slot = first_flush ? sc[i] * tmp : __builtin_fmaf(sc[i], tmp, *slot);
                        }
                        acc[p][h][mt][r] = 0.f;
                    }
            }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) rs[mt] = v4f {0.f, 0.f, 0.f, 0.f};
        first_flush = false;
    };

    if (kb < ke) {
        // Super-steps of SS steps: all weight and src loads of a super-step are
        // issued before its first MFMA, so one wavefront keeps SS * 4 row loads
        // in flight (HBM latency is hidden by depth, not by occupancy: the
        // accumulators leave room for one wavefront per SIMD only).
        constexpr int SS = 4;
        step_t sb[SS];
        qraw_t qr;
        long g_cur = kb / X.G;
        fetch_group(qr, g_cur);
        for (long k = kb; k < ke; k += 16 * SS) {
#pragma unroll
            for (int i = 0; i < SS; ++i)
                if (k + 16 * i < ke) load_step(sb[i], k + 16 * i);
#pragma unroll
            for (int i = 0; i < SS; ++i) {
                const long kk = k + 16 * i;
                if (kk < ke) {
                    if (kk / X.G != g_cur) {
                        flush_group(qr);
                        g_cur = kk / X.G;
                        fetch_group(qr, g_cur);
                    }
#ifndef MI355_DBG_WOQ_NOCOMPUTE
                    compute_step(sb[i]);
#else
                    acc[0][0][0][0] += __uint_as_float(sb[i].w[0][0] ^ sb[i].w[1][0] ^ sb[i].w[2][1] ^ sb[i].w[3][1] ^ sb[i].a[0].x);
#endif
                }
            }
        }
        flush_group(qr);
    }
    if (first_flush) flush_group(qraw_t {}); // empty K range: contribute zeros
    // ---- reduce the wavefronts' LDS slices: red[wave][m][n_local]
    __syncthreads();
    const long n0 = (long)chunk * NW;
    float *part = X.partials + (long)split * M * N;
    const bool direct = X.ksplit == 1;
    for (int idx = t; idx < M * NW; idx += WOQ_NT) {
        const int m = idx / NW, nl = idx % NW;
        if (n0 + nl >= N) continue;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < NWV; ++w) v += red[((long)w * M + m) * NW + nl];
        if (direct) epilogue_store(P, v, 0, m, n0 + nl);
        else __hip_atomic_store(part + (long)m * N + n0 + nl, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (direct) return;
#ifdef MI355_DBG_WOQ_NOFINAL
    return;
#endif

    // ---- arrival counter: the last workgroup of this chunk finishes the job
    // The partial sums were written with device-coherent (agent-scope atomic)
    // stores; waiting for them to complete orders them before the arrival
    // below without a device-wide cache write-back.
    __shared__ int is_last;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (t == 0) {
        unsigned *ctr = X.counters + chunk;
        unsigned old = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        unsigned want;
        do {
            // a stamp from another launch (or uninitialised memory) counts as zero arrivals
            const unsigned cnt = (old >> 8) == X.epoch ? (old & 0xffu) : 0u;
            want = (X.epoch << 8) | (cnt + 1u);
        } while (!__hip_atomic_compare_exchange_strong(ctr, &old, want, __ATOMIC_RELAXED,
                __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        is_last = (int)((want & 0xffu) == (unsigned)X.ksplit);
    }
    __syncthreads();
    if (!is_last) return;
    for (int idx = t; idx < M * NW; idx += WOQ_NT) {
        const int m = idx / NW, nl = idx % NW;
        if (n0 + nl >= N) continue;
        float v = 0.f;
        const float *pp = X.partials + (long)m * N + n0 + nl;
        const long sstride = (long)M * N;
        int s = 0;
        for (; s + 8 <= X.ksplit; s += 8) {
            float tv[8];
#pragma unroll
            for (int j = 0; j < 8; ++j)
                tv[j] = __hip_atomic_load(pp + (s + j) * sstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int j = 0; j < 8; ++j) v += tv[j];
        }
        for (; s < X.ksplit; ++s)
            v += __hip_atomic_load(pp + s * sstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        epilogue_store(P, v, 0, m, n0 + nl);
    }
}

struct woq_plan_t {
    int chd, mt, nwv, ksplit, krange, chunks;
    size_t lds_bytes, total;
};

woq_plan_t make_plan(const mi355_matmul_desc_t &d) {
    woq_plan_t p {};
    p.mt = d.M > 16 ? 2 : 1;
    // Wide-N problems: 16 lanes x 8 columns per workgroup and the whole K range
    // inside it (16 wavefronts, or 8 for two M tiles) -- no cross-workgroup
    // reduction at all.  Narrow-N problems: wider chunks, K split over
    // workgroups, partial sums through scratch.
    const long chunks1 = (d.N + 127) / 128;
    // (measured on MI355X: the whole-K form is latency-bound, 38 us against 25 us
    // for the split form on 4096 x 14336, so it is opt-in for now)
    const bool whole_k = chunks1 >= 96 && d.K >= 1024 && getenv("MI355_WOQ_WHOLE_K") != nullptr;
    long krange;
    if (whole_k) {
        p.chd = 1;
        p.nwv = p.mt == 2 ? 8 : 16;
        p.chunks = (int)chunks1;
        krange = (d.K + 16 * p.nwv - 1) / (16 * p.nwv) * (16 * p.nwv);
    } else {
        p.chd = 2;
        p.nwv = 4;
        const int nw = 16 * p.chd * 8;
        p.chunks = (int)((d.N + nw - 1) / nw);
        // K range per workgroup: a power-of-two multiple of 64, the smallest that
        // keeps the grid near two workgroups per CU; larger M gets longer ranges
        // (each split costs M*N*4 bytes of partial-sum traffic)
        const long min_range = d.M <= 2 ? 64 : d.M <= 8 ? 256 : 512;
        krange = 64;
        const long kmax = (d.K + 63) / 64 * 64;
        while (krange < kmax && (krange < min_range || p.chunks * ((d.K + krange - 1) / krange) > 512))
            krange *= 2;
        if (const char *e = getenv("MI355_WOQ_KRANGE")) krange = atol(e); // tuning aid
        if (krange > kmax) krange = kmax;
    }
    int ksplit = (int)((d.K + krange - 1) / krange);
    while (ksplit > 255) {
        krange *= 2;
        ksplit = (int)((d.K + krange - 1) / krange);
    }
    p.ksplit = ksplit;
    p.krange = (int)krange;
    p.lds_bytes = (size_t)p.nwv * d.M * (16 * p.chd * 8) * sizeof(float);
    p.total = COUNTER_BYTES + (ksplit > 1 ? (size_t)ksplit * d.M * d.N * sizeof(float) : 0);
    return p;
}

std::atomic<unsigned> g_epoch {1};

bool param_layout_ok(const mi355_quant_t &q, long K, bool allow_common, long *G) {
    // per-n with or without groups along K, or a single common value
    *G = K;
    if (q.dt == MI355_DT_UNDEF) return true;
    if (q.mask & 1) return false;
    if (q.mask == 0) return allow_common;
    if (!(q.mask & 4) || q.group[1] != 1) return false;
    if (q.mask & 2) {
        if (q.group[0] % 16 != 0) return false;
        *G = q.group[0];
    }
    return true;
}

} // namespace

int woq_supported(const mi355_matmul_desc_t &d) {
    if (d.src_dt != MI355_DT_BF16 || !is_int4_dt(d.wei_dt) || !d.fpmath_apply_to_int)
        return MI355_UNIMPLEMENTED;
    if (dt_bits(d.dst_dt) < 8) return MI355_UNIMPLEMENTED;
    if (d.batch != 1 || d.M < 1 || d.M > 32) return MI355_UNIMPLEMENTED;
    if (d.K % 16 != 0 || d.N % 16 != 0 || d.K < 16) return MI355_UNIMPLEMENTED;
    if (d.src_stride[2] != 1 || d.src_stride[1] % 4 != 0) return MI355_UNIMPLEMENTED;
    if (d.wei_stride[2] != 1 || d.wei_stride[1] != d.N) return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.src_scale) || !quant_absent(d.src_zp) || !quant_absent(d.src_pr))
        return MI355_UNIMPLEMENTED;
    long gs, gz;
    if (!param_layout_ok(d.wei_scale, d.K, false, &gs)) return MI355_UNIMPLEMENTED;
    if (!param_layout_ok(d.wei_zp, d.K, true, &gz)) return MI355_UNIMPLEMENTED;
    // one group size along K for both parameters
    const bool sg = !quant_absent(d.wei_scale) && (d.wei_scale.mask & 2);
    const bool zg = !quant_absent(d.wei_zp) && (d.wei_zp.mask & 2);
    if (sg && zg && gs != gz) return MI355_UNIMPLEMENTED;
    if ((d.N + 127) / 128 > COUNTER_BYTES / 4) return MI355_UNIMPLEMENTED;
    return MI355_SUCCESS;
}

size_t woq_scratch_bytes(const mi355_matmul_desc_t &d) {
    return make_plan(d).total;
}

int woq_launch(const mi355_matmul_desc_t &d, const problem_t &P, void *scratch, hipStream_t stream) {
    const woq_plan_t plan = make_plan(d);
    if (!scratch) {
        set_error("woq_gemv: %zu bytes of scratch required", plan.total);
        return MI355_INVALID_ARGUMENTS;
    }
    woq_extra_t X {};
    X.counters = (unsigned *)scratch;
    X.partials = (float *)((char *)scratch + COUNTER_BYTES);
    X.epoch = (g_epoch.fetch_add(1) % 0xFFFFFEu) + 1u;
    X.ksplit = plan.ksplit;
    X.krange = plan.krange;
    const bool sg = !quant_absent(d.wei_scale) && (d.wei_scale.mask & 2);
    const bool zg = !quant_absent(d.wei_zp) && (d.wei_zp.mask & 2);
    X.G = (int)(sg ? d.wei_scale.group[0] : zg ? d.wei_zp.group[0] : d.K);
    X.sc_grouped = sg;
    X.zp_grouped = zg;
    X.zp_common = !quant_absent(d.wei_zp) && d.wei_zp.mask == 0;
    X.signed_w = d.wei_dt == MI355_DT_S4;
    dim3 grid((unsigned)plan.chunks, (unsigned)plan.ksplit, 1);
    auto go = [&](auto kern) __attribute__((always_inline)) {
        if (plan.lds_bytes > 65536) {
            if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                        (int)plan.lds_bytes) != hipSuccess) {
                set_error("woq_gemv: cannot reserve %zu bytes of LDS", plan.lds_bytes);
                return MI355_RUNTIME_ERROR;
            }
        }
        hipLaunchKernelGGL(kern, grid, dim3(plan.nwv * 64), plan.lds_bytes, stream, P, X);
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
    };
    if (plan.nwv == 16) return go(woq_gemv_kernel<1, 1, 16>);
    if (plan.nwv == 8) return go(woq_gemv_kernel<1, 2, 8>);
    if (plan.mt == 2) return go(woq_gemv_kernel<2, 2, 4>);
    return go(woq_gemv_kernel<2, 1, 4>);
}

} // namespace mi355
