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
// Data flow per wavefront step (16 k-rows x 16 lanes x 16 columns):
//   lane (c = lane%16, q = lane/16) loads two dwords of rows k0+4q .. k0+4q+3 at
//   column chunk c; every dword yields four bf16 pairs (n, n+4) by shift+and_or;
//   the four rows of one pair are the B operand of v_mfma_f32_16x16x32_bf16
//   (MFMA k-slot 2t+h <-> row 4q+t, column half h); the A operand interleaves
//   zeros, (s,0,s,0,..) or (0,s,0,s,..), so that one MFMA yields column n and a
//   second one column n+4.  An MFMA against an all-ones B gives sum_k src[m,k].
//
// Work split: grid = column chunks x K splits, sized to one workgroup per CU
// (a CU sustains ~35 GB/s of misses, so every CU has to pull its share, and
// row segments shorter than a 128-byte line are fetched whole: chunks are 256
// columns wide).  A wavefront keeps the weight loads of four 16-row steps in
// flight ahead of the MFMAs, and the wavefronts of a workgroup reduce through
// LDS into one f32 partial [row quad][chunk] in scratch.  A second small
// kernel adds the partials of all splits in split order -- deterministic -- and
// runs the shared epilogue; measured on MI355X it costs no more than a
// last-workgroup-finishes scheme with arrival counters for one row of
// activations and half as much for 32 rows, and it keeps no state between
// launches.
#include "kernels.hpp"

namespace mi355 {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

// CHD = dwords of nibbles per lane and row: 2 (16 columns per lane, 256 per
// workgroup) or 4 (32 columns per lane, 512 per workgroup)

// Everything the main loop needs, gathered in one argument so that the kernel
// starts with a single block of scalar loads: the first weight load must not
// wait behind a chain of dependent argument fetches.
struct woq_extra_t {
    const uint8_t *wei;  // [K][N/2]
    const uint8_t *src;  // bf16 [M][src_ld]
    const uint8_t *sc, *zp; // weights scales / zero points (NULL when absent)
    float *partials;     // [ksplit][chunks][unit][4]: row quads in the order of the LDS reduction
    int M, N, K, src_ld;
    int row_bytes;       // N / 2
    int krange;          // k per workgroup (multiple of 16 * wavefronts)
    int ksplit;          // K splits across workgroups
    int G;               // k per quantization group (multiple of 16), K if ungrouped
    int sc_dt, zp_dt;    // MI355_DT_UNDEF when absent
    int sc_grouped, zp_grouped; // parameter has a K dimension
    int zp_common;       // single zero point
    int signed_w;        // s4 weights
};

__device__ __forceinline__ v8bf as_bf(const v4i &x) { return __builtin_bit_cast(v8bf, x); }

// NPL consecutive parameter values of BITS bits each, as raw dwords
template <int NPL, int BITS>
struct raw_t {
    static constexpr int DW = BITS ? NPL * BITS / 32 : 1;
    unsigned w[DW];
};

template <int NPL, int BITS>
__device__ __forceinline__ void load_raw(raw_t<NPL, BITS> &r, const uint8_t *p) {
    if constexpr (raw_t<NPL, BITS>::DW == 2) {
        const uint2 v = *(const uint2 *)p;
        r.w[0] = v.x; r.w[1] = v.y;
    } else if constexpr (BITS != 0) {
#pragma unroll
        for (int i = 0; i < raw_t<NPL, BITS>::DW / 4; ++i) {
            const uint4 v = *(const uint4 *)(p + 16 * i);
            r.w[4 * i] = v.x; r.w[4 * i + 1] = v.y; r.w[4 * i + 2] = v.z; r.w[4 * i + 3] = v.w;
        }
    }
}

// scales: f32 (32 bits) or bf16 / f16 (16 bits)
template <int NPL, int BITS>
__device__ __forceinline__ void decode_scales(int dt, const raw_t<NPL, BITS> &r, float (&out)[NPL]) {
    if constexpr (BITS == 32) {
#pragma unroll
        for (int i = 0; i < NPL; ++i) out[i] = u2f(r.w[i]);
    } else if constexpr (BITS == 16) {
        if (dt == MI355_DT_BF16) {
#pragma unroll
            for (int i = 0; i < NPL; ++i) out[i] = u2f((r.w[i / 2] >> ((i & 1) * 16)) << 16);
        } else {
#pragma unroll
            for (int i = 0; i < NPL; ++i) out[i] = f16_to_f32((uint16_t)(r.w[i / 2] >> ((i & 1) * 16)));
        }
    } else {
#pragma unroll
        for (int i = 0; i < NPL; ++i) out[i] = 1.f;
    }
}

// zero points: s32 (32 bits), s8 / u8 (8 bits), s4 / u4 (4 bits)
template <int NPL, int BITS>
__device__ __forceinline__ void decode_zps(int dt, const raw_t<NPL, BITS> &r, float (&out)[NPL]) {
    if constexpr (BITS == 32) {
#pragma unroll
        for (int i = 0; i < NPL; ++i) out[i] = (float)(int)r.w[i];
    } else if constexpr (BITS == 8) {
        if (dt == MI355_DT_U8) {
#pragma unroll
            for (int i = 0; i < NPL; ++i) out[i] = (float)((r.w[i / 4] >> ((i & 3) * 8)) & 0xffu);
        } else {
#pragma unroll
            for (int i = 0; i < NPL; ++i) out[i] = (float)(int)(int8_t)((r.w[i / 4] >> ((i & 3) * 8)) & 0xffu);
        }
    } else if constexpr (BITS == 4) {
        // s4 as offset-binary: (nibble ^ 8) - 8
        const unsigned flip = dt == MI355_DT_S4 ? 0x88888888u : 0u;
        const float bias = dt == MI355_DT_S4 ? -8.f : 0.f;
#pragma unroll
        for (int i = 0; i < NPL; ++i) out[i] = (float)(((r.w[i / 8] ^ flip) >> ((i & 7) * 4)) & 0xfu) + bias;
    } else {
#pragma unroll
        for (int i = 0; i < NPL; ++i) out[i] = 0.f;
    }
}

// CHD dwords per lane and row; MT 16-row tiles of activations; NWV wavefronts
// per workgroup share one column chunk and split its K range; SS = 16-row steps
// of one super-step; SCB / ZPB = bits per scale / zero point (0 = absent).
template <int CHD, int MT, int NWV, int SS, int SCB, int ZPB>
__global__ void __launch_bounds__(NWV * 64) woq_gemv_kernel(const problem_t P_, const woq_extra_t X) {
    extern __shared__ __attribute__((aligned(16))) float red[]; // [NWV][row quads][NW] x 4 floats
    constexpr int NPL = CHD * 8; // columns per lane
    constexpr int NW = 16 * NPL; // columns per wavefront / workgroup: 128- or 256-byte row segments
    constexpr int NP = CHD * 4;  // bf16 pairs per lane per row
    typedef unsigned vwu __attribute__((ext_vector_type(CHD)));
    constexpr int PF = SS < 4 ? SS : 4; // weight steps in flight ahead of the MFMAs
    constexpr int WOQ_NT = NWV * 64;
    const int t = threadIdx.x, lane = t & 63;
    // uniform: addresses below split into a scalar base and one 32-bit lane offset
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int c = lane & 15, q = lane >> 4;
    const int chunk = blockIdx.x, split = blockIdx.y;
    const int N = X.N, K = X.K, M = X.M;
    // Lanes whose columns lie beyond N (last chunk) and MFMA rows beyond M read
    // the last valid columns / row instead: every output element depends on its
    // own row and column only, and those results are never stored.
    const int n_lane = chunk * NW + c * NPL;
    const int n_ld = n_lane < N - NPL ? n_lane : N - NPL;

    // K sub-range of this wavefront: its share of the workgroup's range, in 16-row steps
    const int krw = X.krange / NWV;
    const int kb = split * X.krange + wave * krw;
    const int ke = kb + krw < K ? kb + krw : K;

    v4f acc[NP][2][MT], rs[MT];
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[p][h][mt] = v4f {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) rs[mt] = v4f {0.f, 0.f, 0.f, 0.f};

    struct step_t {
        vwu w[4];    // rows 4q+t, the dwords of this lane's columns
        uint2 a[MT]; // src[m][k0+4q .. +3] as four bf16
    };
    const unsigned wei_lane_off = (unsigned)(4 * q * X.row_bytes + n_ld / 2);
    unsigned src_lane_off[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + c < M ? mt * 16 + c : M - 1;
        src_lane_off[mt] = (unsigned)(m * X.src_ld * 2 + 4 * q * 2);
    }
    auto load_src = [&](step_t &s, int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) s.a[mt] = *(const uint2 *)(X.src + (long)k0 * 2 + src_lane_off[mt]);
    };
    // the weights are read once: non-temporal loads keep them from displacing
    // the activations and parameters in the caches
    auto load_wei = [&](step_t &s, int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
            s.w[tt] = __builtin_nontemporal_load((const vwu *)(X.wei + (long)(k0 + tt) * X.row_bytes + wei_lane_off));
    };

    // 0x4300 | nibble = bf16(128 + nibble).  The constant is kept in a vector
    // register: a VOP3 instruction takes one scalar operand at most, so
    // (x & mask) | magic fuses into v_and_or_b32 only when `magic` is not scalar.
    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));
    const v4i ones = {0x3F803F80, 0x3F803F80, 0x3F803F80, 0x3F803F80};
    auto compute_step = [&](step_t &s) __attribute__((always_inline)) {
        if (X.signed_w) { // s4 -> offset-binary
#pragma unroll
            for (int tt = 0; tt < 4; ++tt) s.w[tt] ^= (vwu)(0x88888888u);
        }
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
                for (int tt = 0; tt < 4; ++tt) b[tt] = (int)(((s.w[tt][d] >> (4 * sh)) & 0x000F000Fu) | magic);
                const int p = d * 4 + sh;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc[p][0][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf(aa[mt]), as_bf(b), acc[p][0][mt], 0, 0, 0);
                    acc[p][1][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf(ab[mt]), as_bf(b), acc[p][1][mt], 0, 0, 0);
                }
            }
        }
    };

    // Quantization parameters of one group for this lane's columns: raw loads
    // when the group starts, decoded when it ends.
    struct qraw_t {
        raw_t<NPL, SCB> s;
        raw_t<NPL, ZPB> z;
    };
    auto fetch_group = [&](qraw_t &qr, int g) __attribute__((always_inline)) {
        if constexpr (SCB != 0)
            load_raw<NPL, SCB>(qr.s, X.sc + ((long)(X.sc_grouped ? g : 0) * N * SCB / 8 + (unsigned)(n_ld * SCB / 8)));
        if constexpr (ZPB != 0) {
            if (X.zp_common) // element 0 for every column
                qr.z.w[0] = ZPB == 32 ? *(const unsigned *)X.zp : (unsigned)*X.zp;
            else
                load_raw<NPL, ZPB>(qr.z, X.zp + ((long)(X.zp_grouped ? g : 0) * N * ZPB / 8 + (unsigned)(n_ld * ZPB / 8)));
        }
    };

    // Rows are handled in quads (the four rows a lane holds of one MFMA tile):
    // MQ quads in all, MQ0 of them in the first 16-row tile.
    const int MQ = (M + 3) / 4, MQ0 = MQ < 4 ? MQ : 4;
    // fold one finished group into this wavefront's LDS slice, one 16-byte
    // write per column and row quad:
    //   red[wave][tile][slot][quad] (+)= scale * (acc - (128 + zp) * rowsum)
    // column i of lane c sits at slot i * 16 + c, so the lanes of a write
    // cover consecutive 16-byte words (no bank conflicts)
    v4f *red4 = (v4f *)red;
    int rows_used[MT]; // rows of a quad that can hold data in tile mt (4 unless M is below 4 there)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) rows_used[mt] = M - 16 * mt < 4 ? M - 16 * mt : 4;
    bool first_flush = true;
    auto flush_group = [&](const qraw_t &qr) __attribute__((always_inline)) {
        float sc[NPL], zc[NPL];
        decode_scales<NPL, SCB>(X.sc_dt, qr.s, sc);
        decode_zps<NPL, ZPB>(X.zp_dt, qr.z, zc);
        if (ZPB != 0 && X.zp_common) {
#pragma unroll
            for (int i = 1; i < NPL; ++i) zc[i] = zc[0];
        }
        const float zbase = X.signed_w ? 136.f : 128.f;
#pragma unroll
        for (int i = 0; i < NPL; ++i) zc[i] += zbase;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int mqt = mt ? MQ - MQ0 : MQ0; // quads of this tile
            if (q < mqt) {
                v4f *col = red4 + (wave * MQ + (mt ? MQ0 : 0)) * NW + c * mqt + q;
#pragma unroll
                for (int p = 0; p < NP; ++p)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int i = (p / 4) * 8 + h * 4 + (p % 4); // column of (pair p, half h)
                        v4f val = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (r < rows_used[mt]) // uniform: skips the padding rows of small M
                                val[r] = sc[i] * __builtin_fmaf(-zc[i], rs[mt][r], acc[p][h][mt][r]);
                        v4f *slot = col + i * 16 * mqt;
                        *slot = first_flush ? val : *slot + val;
                    }
            }
        }
        first_flush = false;
    };
    auto clear_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[p][h][mt] = v4f {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) rs[mt] = v4f {0.f, 0.f, 0.f, 0.f};
    };

    // The K range of the wavefront is walked one quantization group at a time;
    // inside a group, super-steps of SS steps.  Issue order: the group's
    // parameters (few bytes, needed last: loads return in order, so they must
    // not queue behind the weights), the activations, then the weight rows PF
    // steps ahead of the MFMAs that consume them.
    for (int k = kb; k < ke;) {
        const int g = k / X.G;
        const int kend = (g + 1) * X.G < ke ? (g + 1) * X.G : ke;
        qraw_t qr;
        fetch_group(qr, g);
        for (; k + 16 * SS <= kend; k += 16 * SS) {
            step_t sb[SS];
#pragma unroll
            for (int i = 0; i < SS; ++i) load_src(sb[i], k + 16 * i);
#pragma unroll
            for (int i = 0; i < PF; ++i) load_wei(sb[i], k + 16 * i);
#pragma unroll
            for (int i = 0; i < SS; ++i) {
                if (i + PF < SS) load_wei(sb[i + PF], k + 16 * (i + PF));
                compute_step(sb[i]);
            }
        }
        for (; k < kend; k += 16) { // remainder of the group, one step at a time
            step_t s1;
            load_src(s1, k);
            load_wei(s1, k);
            compute_step(s1);
        }
        flush_group(qr);
        if (k < ke) clear_acc();
    }
    if (first_flush) { // empty K range: contribute zeros
        for (int u = lane; u < MQ * NW; u += 64) red4[wave * MQ * NW + u] = v4f {0.f, 0.f, 0.f, 0.f};
    }
    // ---- reduce the wavefronts' LDS slices.  A unit is one 16-byte word: four
    // rows of one column, in the order the flush wrote them; the partial sums
    // in scratch keep that order, [split][chunk][unit].
    __syncthreads();
    const int n0 = chunk * NW;
    const int units = MQ * NW;
    auto wave_sum = [&](int u) __attribute__((always_inline)) {
        v4f v = red4[u];
#pragma unroll
        for (int w = 1; w < NWV; ++w) v += red4[w * units + u];
        return v;
    };
    const auto &P = MI355_KERNARG_PROBLEM();
    if (X.ksplit > 1) { // plain stores: the kernel boundary publishes them to the second pass
        v4f *part = (v4f *)X.partials + ((long)split * gridDim.x + chunk) * units;
        for (int u = t; u < units; u += WOQ_NT) part[u] = wave_sum(u);
        return;
    }
    // a single split: finish here
    for (int u0 = t; u0 < units; u0 += WOQ_NT) {
        const v4f v = wave_sum(u0);
        // unit -> (tile, slot, quad) -> column and rows
        int u = u0, mt = 0, mqt = MQ0;
        if (u >= MQ0 * NW) {
            u -= MQ0 * NW;
            mt = 1;
            mqt = MQ - MQ0;
        }
        const int slot = u / mqt, mq = u % mqt;
        const int n = n0 + (slot % 16) * NPL + slot / 16;
        if (n >= N) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = mt * 16 + mq * 4 + r;
            if (m < M) epilogue_store(P, v[r], 0, m, n);
        }
    }
}

// Second pass: the partial sums of all splits are added in split order, one
// thread per row quad and column over the whole device.
template <int CHD>
__global__ void __launch_bounds__(256) woq_reduce_kernel(const problem_t P_, const woq_extra_t X, int chunks) {
    const auto &P = MI355_KERNARG_PROBLEM();
    constexpr int NPL = CHD * 8, NW = 16 * NPL;
    const int M = X.M, N = X.N;
    const int MQ = (M + 3) / 4, MQ0 = MQ < 4 ? MQ : 4;
    const int units = MQ * NW;
    const long g = (long)blockIdx.x * 256 + threadIdx.x;
    if (g >= (long)chunks * units) return;
    const int chunk = (int)(g / units);
    int u = (int)(g % units);
    const v4f *pp = (const v4f *)X.partials + g;
    const long sstride = (long)chunks * units;
    v4f v = {0.f, 0.f, 0.f, 0.f};
    int s = 0;
    for (; s + 4 <= X.ksplit; s += 4) {
        v4f tv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) tv[j] = pp[(s + j) * sstride];
#pragma unroll
        for (int j = 0; j < 4; ++j) v += tv[j];
    }
    for (; s < X.ksplit; ++s) v += pp[s * sstride];
    int mt = 0, mqt = MQ0;
    if (u >= MQ0 * NW) {
        u -= MQ0 * NW;
        mt = 1;
        mqt = MQ - MQ0;
    }
    const int slot = u / mqt, mq = u % mqt;
    const int n = chunk * NW + (slot % 16) * NPL + slot / 16;
    if (n >= N) return;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int m = mt * 16 + mq * 4 + r;
        if (m < M) epilogue_store(P, v[r], 0, m, n);
    }
}

// Launch geometry.  One workgroup per CU is the target: the grid never exceeds
// the CU count, so every load of the problem is issued by the first and only
// wave of workgroups.
struct woq_plan_t {
    int chd, mt, nwv, ksplit, krange, chunks;
    size_t lds_bytes, total;
};

constexpr int TARGET_WGS = 256;

woq_plan_t make_plan(const mi355_matmul_desc_t &d) {
    woq_plan_t p {};
    // M <= 16: one 16-row tile, 8 wavefronts; M <= 32: two tiles, 4 wavefronts.
    // Both keep the LDS reduction buffer [wavefronts][M][256] within 128 KB.
    // (Measured on MI355X for M = 1 at 4096 x 14336, against 12-13 us for this
    // shape: 512-column chunks with 16-byte loads and one wavefront per SIMD
    // 16 us, 4 wavefronts x 16 steps 22 us, 16 wavefronts x 4 steps 19 us -- two
    // wavefronts per SIMD overlap one's nibble unpacking with the other's MFMAs.)
    p.chd = 2;
    p.mt = d.M <= 16 ? 1 : 2;
    p.nwv = d.M <= 16 ? 8 : 4;
    const int NW = 16 * 8 * p.chd;
    p.chunks = (int)((d.N + NW - 1) / NW);
    // K range per workgroup: a multiple of 16 rows per wavefront
    const long unit = 16L * p.nwv;
    long ksplit = TARGET_WGS / p.chunks;
    if (ksplit < 1) ksplit = 1;
    long krange = ((d.K + ksplit - 1) / ksplit + unit - 1) / unit * unit;
    // every split costs M*N*4 bytes of partial sums each way: keep the K range
    // of a split at least 8 rows per row of activations
    while (krange < d.K && krange < 8L * d.M * p.nwv) krange += unit;
    ksplit = (d.K + krange - 1) / krange;
    p.ksplit = (int)ksplit;
    p.krange = (int)krange;
    const size_t m4 = (size_t)(d.M + 3) / 4 * 4; // rows in quads
    p.lds_bytes = (size_t)p.nwv * m4 * NW * sizeof(float);
    p.total = ksplit > 1 ? (size_t)ksplit * p.chunks * NW * m4 * sizeof(float) : 0;
    return p;
}

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

int scale_bits(int dt) {
    return dt == MI355_DT_UNDEF ? 0 : dt == MI355_DT_F32 ? 32 : (dt == MI355_DT_BF16 || dt == MI355_DT_F16) ? 16 : -1;
}

int zp_bits(int dt) {
    return dt == MI355_DT_UNDEF ? 0
            : dt == MI355_DT_S32 ? 32
            : (dt == MI355_DT_S8 || dt == MI355_DT_U8) ? 8
            : (dt == MI355_DT_S4 || dt == MI355_DT_U4) ? 4 : -1;
}

template <int CHD, int MT, int NWV, int SS>
int launch_variant(int scb, int zpb, dim3 grid, size_t lds, hipStream_t stream, const problem_t &P,
        const woq_extra_t &X) {
    auto go = [&](auto kern) __attribute__((always_inline)) -> int {
        if (lds > 65536) {
            if (const int st = ensure_dynamic_lds((const void *)kern, (int)lds, "woq_gemv")) return st;
        }
        hipLaunchKernelGGL(kern, grid, dim3(NWV * 64), lds, stream, P, X);
        if (X.ksplit > 1) {
            const long total = (long)grid.x * ((X.M + 3) / 4) * (16 * 8 * CHD);
            hipLaunchKernelGGL(woq_reduce_kernel<CHD>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                    P, X, (int)grid.x);
        }
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
    };
#define MI355_WOQ_CASE(S, Z) \
    if (scb == S && zpb == Z) return go(woq_gemv_kernel<CHD, MT, NWV, SS, S, Z>)
    MI355_WOQ_CASE(16, 4);
    MI355_WOQ_CASE(16, 8);
    MI355_WOQ_CASE(16, 32);
    MI355_WOQ_CASE(16, 0);
    MI355_WOQ_CASE(32, 4);
    MI355_WOQ_CASE(32, 8);
    MI355_WOQ_CASE(32, 32);
    MI355_WOQ_CASE(32, 0);
    MI355_WOQ_CASE(0, 4);
    MI355_WOQ_CASE(0, 8);
    MI355_WOQ_CASE(0, 32);
    MI355_WOQ_CASE(0, 0);
#undef MI355_WOQ_CASE
    set_error("woq_gemv: no kernel for %d-bit scales and %d-bit zero points", scb, zpb);
    return MI355_UNIMPLEMENTED;
}

} // namespace

int woq_supported(const mi355_matmul_desc_t &d) {
    if (d.src_dt != MI355_DT_BF16 || !is_int4_dt(d.wei_dt) || !d.fpmath_apply_to_int)
        return MI355_UNIMPLEMENTED;
    if (d.wei_packing != MI355_WEI_PACK_NONE) return MI355_UNIMPLEMENTED;
    if (dt_bits(d.dst_dt) < 8) return MI355_UNIMPLEMENTED;
    if (d.batch != 1 || d.M < 1 || d.M > 32) return MI355_UNIMPLEMENTED;
    if (d.K % 16 != 0 || d.N % 16 != 0 || d.K < 16) return MI355_UNIMPLEMENTED;
    // 32-bit byte offsets into src and into a weights row
    if (d.src_stride[2] != 1 || d.src_stride[1] % 4 != 0 || d.src_stride[1] >= (1L << 25)) return MI355_UNIMPLEMENTED;
    if (d.wei_stride[2] != 1 || d.wei_stride[1] != d.N || d.N >= (1L << 28)) return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.src_scale) || !quant_absent(d.src_zp) || !quant_absent(d.src_pr))
        return MI355_UNIMPLEMENTED;
    if (scale_bits(d.wei_scale.dt) < 0 || zp_bits(d.wei_zp.dt) < 0) return MI355_UNIMPLEMENTED;
    long gs, gz;
    if (!param_layout_ok(d.wei_scale, d.K, false, &gs)) return MI355_UNIMPLEMENTED;
    if (!param_layout_ok(d.wei_zp, d.K, true, &gz)) return MI355_UNIMPLEMENTED;
    // one group size along K for both parameters
    const bool sg = !quant_absent(d.wei_scale) && (d.wei_scale.mask & 2);
    const bool zg = !quant_absent(d.wei_zp) && (d.wei_zp.mask & 2);
    if (sg && zg && gs != gz) return MI355_UNIMPLEMENTED;
    return MI355_SUCCESS;
}

size_t woq_scratch_bytes(const mi355_matmul_desc_t &d) {
    return make_plan(d).total;
}

int woq_launch(const mi355_matmul_desc_t &d, const problem_t &P, void *scratch, hipStream_t stream) {
    const woq_plan_t plan = make_plan(d);
    if (plan.total && !scratch) {
        set_error("woq_gemv: %zu bytes of scratch required", plan.total);
        return MI355_INVALID_ARGUMENTS;
    }
    woq_extra_t X {};
    X.wei = (const uint8_t *)P.wei;
    X.src = (const uint8_t *)P.src;
    X.partials = (float *)scratch;
    X.M = (int)d.M; X.N = (int)d.N; X.K = (int)d.K;
    X.src_ld = (int)d.src_stride[1];
    X.row_bytes = (int)(d.N / 2);
    X.ksplit = plan.ksplit;
    X.krange = plan.krange;
    const bool sg = !quant_absent(d.wei_scale) && (d.wei_scale.mask & 2);
    const bool zg = !quant_absent(d.wei_zp) && (d.wei_zp.mask & 2);
    X.G = (int)(sg ? d.wei_scale.group[0] : zg ? d.wei_zp.group[0] : d.K);
    X.sc_dt = d.wei_scale.dt;
    X.zp_dt = d.wei_zp.dt;
    X.sc = X.sc_dt ? (const uint8_t *)P.wei_scale.p : nullptr;
    X.zp = X.zp_dt ? (const uint8_t *)P.wei_zp.p : nullptr;
    X.sc_grouped = sg;
    X.zp_grouped = zg;
    X.zp_common = X.zp_dt && d.wei_zp.mask == 0;
    X.signed_w = d.wei_dt == MI355_DT_S4;
    const dim3 grid((unsigned)plan.chunks, (unsigned)plan.ksplit, 1);
    const int scb = scale_bits(X.sc_dt), zpb = zp_bits(X.zp_dt);
    if (plan.mt == 1) return launch_variant<2, 1, 8, 8>(scb, zpb, grid, plan.lds_bytes, stream, P, X);
    return launch_variant<2, 2, 4, 8>(scb, zpb, grid, plan.lds_bytes, stream, P, X);
}

} // namespace mi355
