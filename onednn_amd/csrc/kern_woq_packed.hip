// "hip:woq_packed" -- the weight-only-quantized decode of kern_woq.hip over
// weights in the MI355_WEI_PACK_WOQ64 layout: bf16 activations (M <= 32 rows)
// times 4-bit weights, per-group scales and zero points along K, fpmath
// "apply_to_int" weight decompression.
//
// Semantics (ref_matmul_t, src/cpu/matmul/ref_matmul.cpp:179-235, weights
// decompression branch :193-214) and the evaluation
//     dst[m,n] = sum_g scale[g,n] * ( sum_{k in g} src[m,k] * (128 + wei[k,n])
//                                     - (128 + zp[g,n]) * sum_{k in g} src[m,k] )
// are those of "hip:woq_gemv"; so is the comparison with the reference (bf16
// threshold plus the forward error bound of the K sum).
//
// What the layout buys.  A 64-column chunk holds all of K contiguously, so one
// workgroup owns 64 columns of dst and all of K: no K split across workgroups,
// no partial sums in memory, no second kernel, and N / 64 workgroups fill the
// device for the decode shapes (224 for N = 14336).  A wavefront reads 32 rows
// x 64 columns as one 1 KB run, 16 bytes per lane.  Lane (q = lane / 16,
// j = lane % 16) receives, for each of the four 16-column blocks t, one dword
// with rows 8q .. 8q+7 of column 16t + j, nibbles ordered so that
//     ((dword >> 4u) & 0x000F000F) | 0x43004300,   u = 0..3
// are the eight bf16 values 128 + w in matrix-core order: one dword is the
// whole B operand of a lane for one v_mfma_f32_16x16x32_bf16, with no
// zero-interleaved A operand (half the matrix-core work of the plain layout).
// The A operand is 16 bytes of a src row, the same k order by construction.
//
// The eight wavefronts of a workgroup split K, keep their sums in registers
// across quantization groups and add them through LDS at the end, in wavefront
// order: results do not depend on timing.
#include "kernels.hpp"
#include "tile_epilogue.hpp"

#include <type_traits>

namespace mi355 {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

constexpr int NWV = 8;         // wavefronts per workgroup
constexpr int CHUNK = 64;      // columns per workgroup
constexpr int KBLK = 32;       // rows per step (one MFMA depth)
constexpr int NO_GROUPS = 1 << 30;

struct woqp_extra_t {
    const uint8_t *wei;  // packed, K * N / 2 bytes
    const uint8_t *src;  // bf16 [M][src_ld]
    const uint8_t *sc, *zp; // weights scales / zero points (NULL when absent)
    int M, N, K, src_ld;
    int kbw;             // 32-row blocks per wavefront
    int spg;             // 32-row blocks per quantization group, NO_GROUPS without groups
    int sc_dt, zp_dt;    // MI355_DT_UNDEF when absent (sc / zp then point at any readable memory)
    int sc_bits, zp_bits; // bits per element, 0 when absent (every lane then reads the first dword)
    int sc_grouped, zp_grouped; // parameter has a K dimension
    int zp_common;       // single zero point
    int signed_w;        // s4 weights
};

__device__ __forceinline__ v8bf as_bf(const v4i &x) { return __builtin_bit_cast(v8bf, x); }

// Quantization parameters are fetched as the aligned dword that holds the
// element (no branch on the data type next to the load, so a fetch never waits
// for its own data); the element is cut out when the group is flushed.
__device__ __forceinline__ unsigned param_word(const uint8_t *p, int bits, long idx) {
    // (pointer arithmetic on p, not an address rebuilt from an integer: the
    // load stays a global one)
    const long off = (idx * bits) >> 3;
    return *(const unsigned *)(p + (off - (long)(((uintptr_t)p + (size_t)off) & 3)));
}

__device__ __forceinline__ unsigned param_cut(const uint8_t *p, int bits, long idx, unsigned word) {
    const uintptr_t addr = (uintptr_t)p + (size_t)((idx * bits) >> 3);
    const unsigned sh = (unsigned)(addr & 3) * 8u + (unsigned)((idx * bits) & 4);
    return (word >> sh) & (0xffffffffu >> ((32 - bits) & 31));
}

__device__ __forceinline__ float decode_scale(int dt, unsigned raw) {
    switch (dt) {
        case MI355_DT_F32: return u2f(raw);
        case MI355_DT_BF16: return u2f(raw << 16);
        case MI355_DT_F16: return f16_to_f32((uint16_t)raw);
        default: return 1.f;
    }
}

__device__ __forceinline__ float decode_zp(int dt, unsigned raw) {
    switch (dt) {
        case MI355_DT_S32: return (float)(int)raw;
        case MI355_DT_U8: return (float)raw;
        case MI355_DT_S8: return (float)(int)(int8_t)raw;
        case MI355_DT_U4: return (float)raw;
        case MI355_DT_S4: return (float)((int)(raw ^ 8u) - 8);
        default: return 0.f;
    }
}

// MT 16-row tiles of activations; SS steps per super-step (all of its loads
// are issued before its first MFMA); SPG steps per quantization group when a
// super-step holds whole groups, 0 when a group holds whole super-steps.
template <int MT, int SS, int SPG>
__global__ void __launch_bounds__(NWV * 64) woqp_kernel(const problem_t P_, const woqp_extra_t X) {
    __shared__ v4f red4[NWV * MT * 4 * 64];
    constexpr int NGS = SPG ? SS / SPG : 1; // groups per super-step
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int j = lane & 15, q = lane >> 4;
    const int chunk = blockIdx.x;
    const int N = X.N, K = X.K, M = X.M;
    const int KB = K / KBLK;
    const int kb0 = wave * X.kbw;
    const int kb1 = kb0 + X.kbw < KB ? kb0 + X.kbw : KB;

    const uint8_t *wlane = X.wei + (long)chunk * K * (CHUNK / 2) + lane * 16;
    // MFMA rows beyond M read the last valid row: an output row depends on its
    // own src row only, and those results are never stored
    unsigned src_lane_off[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + j < M ? mt * 16 + j : M - 1;
        src_lane_off[mt] = (unsigned)(m * X.src_ld * 2 + q * 16);
    }
    // quantization parameters: lane l fetches column l of the chunk, the
    // columns a lane accumulates (16t + j) come from lanes 16t + j at the flush
    const long n_param = (long)chunk * CHUNK + lane;

    v4f acc[MT][4], rsum[MT], tot[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        rsum[mt] = v4f {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) acc[mt][tt] = tot[mt][tt] = v4f {0.f, 0.f, 0.f, 0.f};
    }
    int rows_used[MT]; // rows of a quad that can hold data in tile mt (uniform: 4 unless M is below 4 there)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) rows_used[mt] = M - 16 * mt;

    // 0x4300 | nibble = bf16(128 + nibble).  The constant is kept in a vector
    // register: a VOP3 instruction takes one scalar operand at most, so
    // (x & mask) | magic fuses into v_and_or_b32 only when `magic` is not scalar.
    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));
    const v4i ones = {0x3F803F80, 0x3F803F80, 0x3F803F80, 0x3F803F80};
    const unsigned flip = X.signed_w ? 0x88888888u : 0u; // s4 -> offset-binary
    const float zbase = X.signed_w ? 136.f : 128.f;

    auto compute_step = [&](const v4u &w, const v4u (&a)[MT]) __attribute__((always_inline)) {
        v4i av[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            av[mt] = v4i {(int)a[mt][0], (int)a[mt][1], (int)a[mt][2], (int)a[mt][3]};
            rsum[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf(av[mt]), as_bf(ones), rsum[mt], 0, 0, 0);
        }
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            const unsigned d = w[tt] ^ flip;
            v4i b;
#pragma unroll
            for (int u = 0; u < 4; ++u) b[u] = (int)(((d >> (4 * u)) & 0x000F000Fu) | magic);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                acc[mt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf(av[mt]), as_bf(b), acc[mt][tt], 0, 0, 0);
        }
    };

    // element index of this lane's parameters of group g
    auto sc_index = [&](int g) __attribute__((always_inline)) { return (X.sc_grouped ? (long)g * N : 0) + n_param; };
    auto zp_index = [&](int g) __attribute__((always_inline)) {
        return X.zp_common ? 0 : (X.zp_grouped ? (long)g * N : 0) + n_param;
    };
    auto fetch_params = [&](unsigned &word_s, unsigned &word_z, int g) __attribute__((always_inline)) {
        word_s = param_word(X.sc, X.sc_bits, sc_index(g));
        word_z = param_word(X.zp, X.zp_bits, zp_index(g));
    };

    // tot += scale * (acc - (128 + zp) * rowsum) for one finished group
    auto flush_group = [&](unsigned word_s, unsigned word_z, int g) __attribute__((always_inline)) {
        const float s = decode_scale(X.sc_dt, param_cut(X.sc, X.sc_bits, sc_index(g), word_s));
        const float z = decode_zp(X.zp_dt, param_cut(X.zp, X.zp_bits, zp_index(g), word_z)) + zbase;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            const float st = __shfl(s, tt * 16 + j, 64);
            const float zt = __shfl(z, tt * 16 + j, 64);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (r < rows_used[mt]) tot[mt][tt][r] += st * __builtin_fmaf(-zt, rsum[mt][r], acc[mt][tt][r]);
                acc[mt][tt] = v4f {0.f, 0.f, 0.f, 0.f};
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) rsum[mt] = v4f {0.f, 0.f, 0.f, 0.f};
    };

    // One super-step.  Issue order: the groups' parameters (few bytes, needed
    // last -- loads return in order, so they must not queue behind the weights),
    // the activations, the weights; then the MFMAs step by step as their loads
    // arrive.  FULL = all SS steps present (no guards in the common case).
    auto super_step = [&](int kb, int ns, auto full) __attribute__((always_inline)) {
        constexpr bool FULL = decltype(full)::value;
        unsigned raw_s[NGS], raw_z[NGS];
#pragma unroll
        for (int gi = 0; gi < NGS; ++gi)
            if (FULL || gi * (SPG ? SPG : SS) < ns) fetch_params(raw_s[gi], raw_z[gi], (kb + gi * SPG) / X.spg);
        v4u a[SS][MT], w[SS];
#pragma unroll
        for (int i = 0; i < SS; ++i)
            if (FULL || i < ns) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    a[i][mt] = *(const v4u *)(X.src + (long)(kb + i) * (KBLK * 2) + src_lane_off[mt]);
            }
        // the weights are read once: non-temporal loads keep them from
        // displacing the activations and parameters in the caches
#pragma unroll
        for (int i = 0; i < SS; ++i)
            if (FULL || i < ns) w[i] = __builtin_nontemporal_load((const v4u *)(wlane + (long)(kb + i) * (KBLK * CHUNK / 2)));
        // every load of the super-step is in flight before its first MFMA
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < SS; ++i)
            if (FULL || i < ns) {
                compute_step(w[i], a[i]);
                if constexpr (SPG != 0) {
                    if ((i + 1) % SPG == 0) flush_group(raw_s[i / SPG], raw_z[i / SPG], (kb + i) / X.spg);
                }
            }
        if constexpr (SPG == 0) {
            if ((kb + ns) % X.spg == 0 || kb + ns >= kb1) flush_group(raw_s[0], raw_z[0], kb / X.spg);
        }
    };

    for (int kb = kb0; kb < kb1; kb += SS) {
        const int ns = kb1 - kb < SS ? kb1 - kb : SS;
        if (ns == SS)
            super_step(kb, ns, std::true_type {});
        else
            super_step(kb, ns, std::false_type {});
    }

    // ---- add the wavefronts' sums in wavefront order and store.  LDS holds
    // [wavefront][row][column] floats; a thread then owns four consecutive
    // columns of one row and runs the four-wide epilogue of the GEMM tiles.
    float *red = (float *)red4;
    constexpr int WSTRIDE = MT * 16 * CHUNK; // floats per wavefront
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                red[wave * WSTRIDE + (mt * 16 + 4 * q + r) * CHUNK + tt * 16 + j] = tot[mt][tt][r];
    __syncthreads();
    const auto &P = MI355_KERNARG_PROBLEM();
    if (M <= 8) {
        // few rows: one element per thread, 64 consecutive columns per
        // wavefront (the four-wide path below starts later: it gathers the
        // epilogue's operands first, which a single pass does not win back)
        const int m = t >> 6, nl = t & 63;
        if (m >= M) return;
        const float *cell = red + m * CHUNK + nl;
        float v = cell[0];
#pragma unroll
        for (int wv = 1; wv < NWV; ++wv) v += cell[wv * WSTRIDE];
        epilogue_store(P, v, 0, m, chunk * CHUNK + nl);
        return;
    }
#pragma unroll 1
    for (int e = t; e < MT * 16 * (CHUNK / 4); e += NWV * 64) {
        const int m = e >> 4, nq = e & 15;
        if (m >= M) continue;
        const v4f *cell = (const v4f *)(red + m * CHUNK + nq * 4);
        v4f sum = cell[0];
#pragma unroll
        for (int wv = 1; wv < NWV; ++wv) sum += cell[wv * (WSTRIDE / 4)];
        float v[4] = {sum[0], sum[1], sum[2], sum[3]};
        const long n = (long)chunk * CHUNK + nq * 4;
        gemm::apply_epilogue4(P, v, 0, m, n, 4);
        gemm::store4(P, P.ds[2] == 1 && gemm::vec_ok_store(P.dst, P.ds[0], P.ds[1], dt_bits(P.dst_dt)), v, 0, m, n, 4);
    }
}

int scale_ok(int dt) {
    return dt == MI355_DT_UNDEF || dt == MI355_DT_F32 || dt == MI355_DT_BF16 || dt == MI355_DT_F16;
}

int zp_ok(int dt) {
    return dt == MI355_DT_UNDEF || dt == MI355_DT_S32 || dt == MI355_DT_S8 || dt == MI355_DT_U8 || dt == MI355_DT_S4
            || dt == MI355_DT_U4;
}

bool param_layout_ok(const mi355_quant_t &q, long K, bool allow_common, long *G) {
    // per-n with or without groups along K, or a single common value
    *G = K;
    if (q.dt == MI355_DT_UNDEF) return true;
    if (q.mask & 1) return false;
    if (q.mask == 0) return allow_common;
    if (!(q.mask & 4) || q.group[1] != 1) return false;
    if (q.mask & 2) *G = q.group[0];
    return true;
}

// group size along K of the problem (K without groups); 0 if the two
// parameters disagree or their layout is not covered
long group_rows(const mi355_matmul_desc_t &d) {
    long gs, gz;
    if (!param_layout_ok(d.wei_scale, d.K, false, &gs)) return 0;
    if (!param_layout_ok(d.wei_zp, d.K, true, &gz)) return 0;
    const bool sg = !quant_absent(d.wei_scale) && (d.wei_scale.mask & 2);
    const bool zg = !quant_absent(d.wei_zp) && (d.wei_zp.mask & 2);
    if (sg && zg && gs != gz) return 0;
    return sg ? gs : zg ? gz : d.K;
}

// super-step geometry for a tile count and a group size (in 32-row blocks)
struct woqp_geo_t {
    int ss, spg; // template arguments; ss == 0: not covered
};

woqp_geo_t pick_geo(int mt, long G, long K) {
    const int ss_max = mt == 1 ? 16 : 8;
    if (G == K) return {ss_max, 0};
    if (G % KBLK != 0) return {0, 0};
    const long spg = G / KBLK;
    if (spg <= ss_max && (spg & (spg - 1)) == 0) {
        const int ss = (int)(4 * spg < ss_max ? 4 * spg : ss_max);
        // a group that fills the super-step is the spanning case
        return {ss, spg == ss ? 0 : (int)spg};
    }
    if (spg % ss_max == 0) return {ss_max, 0};
    return {0, 0};
}

} // namespace

int woqp_supported(const mi355_matmul_desc_t &d) {
    if (!woq64_layout_ok(d)) return MI355_UNIMPLEMENTED;
    if (d.src_dt != MI355_DT_BF16 || !d.fpmath_apply_to_int) return MI355_UNIMPLEMENTED;
    if (dt_bits(d.dst_dt) < 8) return MI355_UNIMPLEMENTED;
    if (d.M < 1 || d.M > 32) return MI355_UNIMPLEMENTED;
    // 16-byte loads of src rows at 32-bit byte offsets
    if (d.src_stride[2] != 1 || d.src_stride[1] % 8 != 0 || d.src_stride[1] >= (1L << 25)) return MI355_UNIMPLEMENTED;
    if (d.K * d.N / 2 >= (1L << 40)) return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.src_scale) || !quant_absent(d.src_zp) || !quant_absent(d.src_pr))
        return MI355_UNIMPLEMENTED;
    if (!scale_ok(d.wei_scale.dt) || !zp_ok(d.wei_zp.dt)) return MI355_UNIMPLEMENTED;
    const long G = group_rows(d);
    if (G == 0) return MI355_UNIMPLEMENTED;
    if (pick_geo(d.M <= 16 ? 1 : 2, G, d.K).ss == 0) return MI355_UNIMPLEMENTED;
    return MI355_SUCCESS;
}

int woqp_launch(const mi355_matmul_desc_t &d, const problem_t &P, hipStream_t stream) {
    if (((uintptr_t)P.src | (uintptr_t)P.wei) & 15) {
        set_error("woq_packed: src and weights must be 16-byte aligned");
        return MI355_INVALID_ARGUMENTS;
    }
    const int mt = d.M <= 16 ? 1 : 2;
    const long G = group_rows(d);
    const woqp_geo_t geo = pick_geo(mt, G, d.K);
    woqp_extra_t X {};
    X.wei = (const uint8_t *)P.wei;
    X.src = (const uint8_t *)P.src;
    X.M = (int)d.M; X.N = (int)d.N; X.K = (int)d.K;
    X.src_ld = (int)d.src_stride[1];
    X.spg = G == d.K ? NO_GROUPS : (int)(G / KBLK);
    // K range of a wavefront: whole groups when a super-step holds groups,
    // whole super-steps when a group holds super-steps
    const long unit = geo.spg ? geo.spg : (G == d.K ? 1 : geo.ss);
    const long KB = d.K / KBLK;
    X.kbw = (int)(((KB + NWV - 1) / NWV + unit - 1) / unit * unit);
    X.sc_dt = d.wei_scale.dt;
    X.zp_dt = d.wei_zp.dt;
    // an absent parameter is fetched from src (any readable memory) and ignored
    X.sc = X.sc_dt ? (const uint8_t *)P.wei_scale.p : (const uint8_t *)P.src;
    X.zp = X.zp_dt ? (const uint8_t *)P.wei_zp.p : (const uint8_t *)P.src;
    X.sc_bits = X.sc_dt ? dt_bits(X.sc_dt) : 0;
    X.zp_bits = X.zp_dt ? dt_bits(X.zp_dt) : 0;
    X.sc_grouped = X.sc_dt && (d.wei_scale.mask & 2);
    X.zp_grouped = X.zp_dt && (d.wei_zp.mask & 2);
    X.zp_common = X.zp_dt && d.wei_zp.mask == 0;
    X.signed_w = d.wei_dt == MI355_DT_S4;
    const dim3 grid((unsigned)(d.N / CHUNK)), block(NWV * 64);
#define MI355_WOQP_CASE(MT_, SS_, SPG_) \
    if (mt == MT_ && geo.ss == SS_ && geo.spg == SPG_) { \
        hipLaunchKernelGGL((woqp_kernel<MT_, SS_, SPG_>), grid, block, 0, stream, P, X); \
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR; \
    }
    MI355_WOQP_CASE(1, 4, 1)
    MI355_WOQP_CASE(1, 8, 2)
    MI355_WOQP_CASE(1, 16, 4)
    MI355_WOQP_CASE(1, 16, 8)
    MI355_WOQP_CASE(1, 16, 0)
    MI355_WOQP_CASE(2, 4, 1)
    MI355_WOQP_CASE(2, 8, 2)
    MI355_WOQP_CASE(2, 8, 4)
    MI355_WOQP_CASE(2, 8, 0)
#undef MI355_WOQP_CASE
    set_error("woq_packed: no kernel for %d tiles, super-step %d, group %d", mt, geo.ss, geo.spg);
    return MI355_UNIMPLEMENTED;
}

} // namespace mi355
