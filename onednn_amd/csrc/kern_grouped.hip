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
//
// Further down: "hip:mfma_grouped_k" (the variable-K pattern) and
// "hip:mfma_grouped" (the variable-M pattern) on the matrix cores.
#include "kernels.hpp"
#include <cstdlib>
#include <cstring>

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

// ---- "hip:mfma_grouped_k" -- the variable-K pattern (the weights' gradient of
// a mixture-of-experts layer: dst[g] = src[:, k0:k1] x wei[k0:k1, :]) on the
// matrix cores.
//
// Both operands arrive with K outermost -- src as [total_K][M], weights as
// [total_K][N] -- the opposite of what the 16-bit matrix instructions want (a
// lane's elements consecutive along K).  v_mfma_f32_16x16x4_f32 takes ONE
// element per lane and operand, lane (i, q) supplying row (column) i at k = q,
// so the operands go from global memory to the instruction with no transpose at
// all: a lane loads the four consecutive rows 4 i .. 4 i + 3 of k = q in one
// instruction (16 bytes of f32, 8 of bf16 / f16, widened in registers) and each
// of the four values feeds a different fragment.  Fragment r therefore holds the
// rows 4 i + r of a wavefront's 64, and fragment c of the weights the columns
// 4 j + c: in the 16 accumulators lane (j, q) finds, for each of its rows, the
// columns 4 j .. 4 j + 3 side by side, which is one 16-byte store.  With the
// short groups of expert routing the work is bound by dst (G x M x N elements
// written against (M + N) x total_K read) and the f32 rate of the matrix cores
// is enough; bf16 / f16 tensors with columns in eights go through LDS to the
// 16-bit instructions instead (grouped_k_lds_kernel, further down).
//
// A workgroup of four wavefronts owns 128 x 128 of one group's dst (64 x 64 a
// wavefront) and walks the group's k range a step at a time, DEPTH steps in
// flight.  A dst stored with rows contiguous ("acb") is the same problem with
// the operands exchanged, which the launch does.
typedef int g4i __attribute__((ext_vector_type(4)));
typedef int g8i __attribute__((ext_vector_type(8)));
typedef unsigned g2u __attribute__((ext_vector_type(2)));
typedef unsigned g4u __attribute__((ext_vector_type(4)));
typedef float g4f __attribute__((ext_vector_type(4)));
typedef __bf16 g8bf __attribute__((ext_vector_type(8)));
typedef _Float16 g8h __attribute__((ext_vector_type(8)));

struct grouped_k_dev_t {
    const void *a, *b;           // [total][MA] and [total][NB]
    const int32_t *offsets;      // cumulative k per group
    void *dst;
    long MA, NB, total;
    long dst_g, dst_ld;          // element strides of dst: group, row of A
    int tiles_n;
    int run;                     // column tiles a workgroup of the LDS kernel takes in turn
};

typedef unsigned gk_u2 __attribute__((ext_vector_type(2)));
typedef float gk_f4 __attribute__((ext_vector_type(4)));

// What a lane holds of one step (4 k) of one operand of v_mfma_f32_16x16x4_f32: four consecutive rows of
// k = kb + q, one load of 16 bytes (f32) or 8 (bf16 / f16, widened when the fragment is taken).
template <int DT>
struct gk_step_t {
    static constexpr int NRAW = DT == MI355_DT_F32 ? 2 : 1; // 8-byte pieces
    gk_u2 raw[NRAW];

    __device__ __forceinline__ void load(const void *base, long ld, long kb, long k1, int q, long first, bool in) {
        const long k = kb + q;
        if (DT == MI355_DT_F32) {
            gk_f4 v = {0.f, 0.f, 0.f, 0.f};
            if (in && k < k1) v = *(const gk_f4 *)((const float *)base + k * ld + first);
            raw[0] = gk_u2 {f2u(v.x), f2u(v.y)};
            raw[NRAW - 1] = gk_u2 {f2u(v.z), f2u(v.w)};
        } else {
            raw[0] = gk_u2 {0u, 0u};
            if (in && k < k1) raw[0] = *(const gk_u2 *)((const uint16_t *)base + k * ld + first);
        }
    }
    // the element of row (column) 4 i + r
    __device__ __forceinline__ float frag(int r) const {
        if (DT == MI355_DT_F32) return u2f(r == 0 ? raw[0].x : r == 1 ? raw[0].y : r == 2 ? raw[NRAW - 1].x : raw[NRAW - 1].y);
        const unsigned w = (r & 2) ? raw[0].y : raw[0].x;
        if (DT == MI355_DT_BF16) return u2f((r & 1) ? (w & 0xffff0000u) : (w << 16));
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 h = __builtin_bit_cast(h2, w);
        return (r & 1) ? (float)h.y : (float)h.x;
    }
};

// Four rows (columns) of each of eight consecutive k -- raw[t] = rows 4 i .. 4 i + 3 of k = 8 q + t, two to a
// dword -- into the eight consecutive k of row 4 i + r that v_mfma_f32_16x16x32_{bf16,f16} takes: a 4 x 8
// transpose inside the lane, 4 v_perm_b32 a fragment.
__device__ __forceinline__ g4u gk_frag16(const gk_u2 (&raw)[8], int r) {
    const unsigned sel = (r & 1) ? 0x07060302u : 0x05040100u;
    g4u o;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const unsigned lo = (r & 2) ? raw[2 * d].y : raw[2 * d].x;
        const unsigned hi = (r & 2) ? raw[2 * d + 1].y : raw[2 * d + 1].x;
        o[d] = __builtin_amdgcn_perm(hi, lo, sel);
    }
    return o;
}

// lane (j, q) of a wavefront's 64 x 64: acc[r][c][e] is row 4 (4 q + e) + r, column 4 j + c
template <int DT>
__device__ __forceinline__ void gk_store(const grouped_k_dev_t &P, const gk_f4 (&acc)[4][4], long g, long m_w, long n_w,
        int j, int q) {
    const long col = n_w + 4 * j;
    // dst is written once and not read again by the launch: non-temporal stores, which do not take lines of the
    // L2s (a quarter faster on a launch that writes 1.3 GB: 0.325 -> 0.25 ms)
    // bf16: v_cvt_pk_bf16_f32 unless the wavefront holds a NaN or an f32 subnormal, which the software conversion
    // (the reference's: subnormals flush, NaNs are quieted its way) treats differently
    bool hw = false;
    if (DT == MI355_DT_BF16) {
        bool special = false;
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int e = 0; e < 4; ++e) special |= __builtin_amdgcn_classf(acc[r][c][e], 0x93);
        hw = __builtin_amdgcn_ballot_w64(special) == 0;
    }
    if (col >= P.NB) return;
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const long row = m_w + 4 * (4 * q + e) + r;
            if (row >= P.MA) continue;
            const long off = g * P.dst_g + row * P.dst_ld + col;
            const float v0 = acc[r][0][e], v1 = acc[r][1][e], v2 = acc[r][2][e], v3 = acc[r][3][e];
            if (DT == MI355_DT_F32) {
                __builtin_nontemporal_store(gk_f4 {v0, v1, v2, v3}, (gk_f4 *)((float *)P.dst + off));
            } else if (DT == MI355_DT_BF16 && hw) {
                typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
                typedef float f32x2_t __attribute__((ext_vector_type(2)));
                gk_u2 o;
                o.x = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_t {v0, v1}, bf16x2_t));
                o.y = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_t {v2, v3}, bf16x2_t));
                __builtin_nontemporal_store(o, (gk_u2 *)((uint16_t *)P.dst + off));
            } else {
                gk_u2 o;
                o.x = (cvt_store_bits(DT, v0) & 0xffffu) | (cvt_store_bits(DT, v1) << 16);
                o.y = (cvt_store_bits(DT, v2) & 0xffffu) | (cvt_store_bits(DT, v3) << 16);
                __builtin_nontemporal_store(o, (gk_u2 *)((uint16_t *)P.dst + off));
            }
        }
}

template <int DT>
__global__ void __launch_bounds__(256) grouped_k_tile_kernel(const grouped_k_dev_t P) {
    typedef gk_f4 f4;
    typedef gk_step_t<DT> step_t;
    constexpr int DEPTH = 4, KSTEP = 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, q = lane >> 4;
    const long g = blockIdx.y;
    const long m_w = (long)(blockIdx.x / P.tiles_n) * 128 + (wave >> 1) * 64;
    const long n_w = (long)(blockIdx.x % P.tiles_n) * 128 + (wave & 1) * 64;
    long k0 = g > 0 ? (long)P.offsets[g - 1] : 0, k1 = P.offsets[g];
    if (k0 < 0) k0 = 0;
    if (k1 > P.total) k1 = P.total;
    // a wavefront whose rows or columns are all outside has nothing to store
    if (m_w >= P.MA || n_w >= P.NB) return;
    const bool a_in = m_w + 4 * i < P.MA, b_in = n_w + 4 * i < P.NB; // (MA and NB are multiples of 4)

    f4 acc[4][4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[r][c] = f4 {0.f, 0.f, 0.f, 0.f};

    step_t sa[DEPTH], sb[DEPTH];
    auto fetch = [&](int slot, long kb) { // (past the range: zeros, no loads)
        sa[slot].load(P.a, P.MA, kb, k1, q, m_w + 4 * i, a_in);
        sb[slot].load(P.b, P.NB, kb, k1, q, n_w + 4 * i, b_in);
    };
#pragma unroll
    for (int s = 0; s < DEPTH; ++s) fetch(s, k0 + KSTEP * s);
    for (long kb = k0; kb < k1; kb += KSTEP * DEPTH) {
#pragma unroll
        for (int s = 0; s < DEPTH; ++s) {
            float a[4], b[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) a[e] = sa[s].frag(e), b[e] = sb[s].frag(e);
            fetch(s, kb + KSTEP * (s + DEPTH));
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    acc[r][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[r], b[c], acc[r][c], 0, 0, 0);
        }
    }

    gk_store<DT>(P, acc, g, m_w, n_w, i, q);
}

// ---- "hip:mfma_grouped" -- the 2Dx3D pattern on the matrix cores for fp8,
// bf16, f16 and s8 operands with K-contiguous weights ([G][N][K], tag acb), no
// groups along K in the scales, no zero points.
//
// Mixture-of-experts groups are short (tens of rows against weights of K x N
// per group), so the work is streaming every active group's weights once: HBM
// bound.  A workgroup owns one (group, BM rows, BN columns) tile and walks K:
//   * the four wavefronts take the K steps (128 bytes per row) in turn, each
//     over the whole tile, so src and weights are both read once per
//     workgroup; the accumulators meet in LDS (eight wavefronts measured
//     slower on every shape);
//   * a tile holds up to MTMAX fragments of 16 rows; the walk is compiled per
//     fragment count and the tile's own count picks one, so a group of 20 rows
//     loads and multiplies two fragments, not MTMAX;
//   * operands go from global memory straight to registers, a load instruction
//     fetching the whole 128-byte lines of 8 rows (what a compute unit can keep
//     in flight is counted in line requests: half lines halve it); after an
//     exchange between lanes j and j +- 8, lane (j, q) of a fragment holds
//     bytes 16 q .. 16 q + 15 and 64 + 16 q .. 64 + 16 q + 15 of row j's step,
//     for src and weights alike, so whichever K slots of the instruction those
//     bytes land in, the dot product is the same: one
//     v_mfma_f32_16x16x128_f8f6f4 per fragment pair for fp8, two
//     v_mfma_f32_16x16x32_{bf16,f16} for the 16-bit types;
//   * D steps are in flight per wavefront (registers); weights are loaded
//     non-temporally, src rows stay in the caches for the group's other tiles.
// The grid is (column tiles, tile slots): slot s is the s-th (group, row
// block) in group order.  A workgroup finds its slot by a block-wide prefix
// sum over the groups' row-block counts (the offsets live on the device); the
// host sizes the grid by the upper bound total_M / BM + min(G, total_M).

enum { GM_F8 = 0, GM_BF16 = 1, GM_F16 = 2, GM_MXF8 = 3, GM_MXF4 = 4, GM_I8 = 5 };
// GM_I8: s8 x s8, the sums are s32 (kept in the accumulator registers' bits and added as integers wherever
// partial sums meet); they turn into f32 once, after the last addition -- ref_grouped_t's `acc = f32(s32 sum)`
// (src/cpu/matmul/ref_grouped_gemm.cpp:258-330), so the tiles agree with it bit for bit on any data.

// GM_MXF8 / GM_MXF4: e8m0 scales per 32 consecutive k on both operands, applied by the instruction
// (v_mfma_scale_f32_16x16x128_f8f6f4).  Lane (j, q) supplies the scale of block q of row j.  Its data
// are, for fp8, k 16 q .. 16 q + 15 and 64 + 16 q .. 64 + 16 q + 15 (chunks q and 4 + q of the step, as
// without scales: the instruction takes the halves of blocks q / 2 and 2 + q / 2 from it and their scales
// from the lanes that own those blocks); for fp4 a 16-byte chunk is a block and chunks q and 4 + q feed two
// instructions.  (Found by measurement: with a lane holding one whole fp8 block the scales came out wrong.)
template <int MODE>
struct gmode_t {
    static constexpr int EBITS = (MODE == GM_BF16 || MODE == GM_F16) ? 16 : (MODE == GM_MXF4 ? 4 : 8);
    static constexpr int SB = MODE == GM_MXF8 ? 1 : (MODE == GM_MXF4 ? 2 : 0); // scale dwords per step and row
    static constexpr bool MX = SB != 0;
    static constexpr int BPS = 4 * SB;                                          // blocks of 32 k per 128-byte step
    __device__ static __forceinline__ long bytes(long elems) { return elems * EBITS / 8; }
    // the two chunks of a step lane (j, q) ends up with
    __device__ static __forceinline__ int chunk_lo(int q) { return q; }
    __device__ static __forceinline__ int chunk_hi(int q) { return 4 + q; }
    // the chunk lane (j, q) fetches (of rows j % 8 and 8 + j % 8) before the exchange
    __device__ static __forceinline__ int chunk_fetch(int q, int half) { return q + 4 * half; }
};

// weights fragment first: the tile comes out transposed, a lane holds four
// consecutive n (4 * (lane / 16) + e) of row lane % 16.  sw / sa: the lane's e8m0 scale bytes (MX modes).
template <int MODE, int FA, int FB>
__device__ __forceinline__ g4f grouped_mma(const g8i &w, const g8i &a, g4f c, const int *sw = nullptr,
        const int *sa = nullptr) {
    if constexpr (MODE == GM_F8) {
        return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w, a, c, FB, FA, 0, 0, 0, 0);
    } else if constexpr (MODE == GM_MXF8) {
        return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w, a, c, FB, FA, 0, sw[0], 0, sa[0]);
    } else if constexpr (MODE == GM_I8) {
        const g4i wl = {w[0], w[1], w[2], w[3]}, wh = {w[4], w[5], w[6], w[7]};
        const g4i al = {a[0], a[1], a[2], a[3]}, ah = {a[4], a[5], a[6], a[7]};
        g4i ci = __builtin_bit_cast(g4i, c);
        ci = __builtin_amdgcn_mfma_i32_16x16x64_i8(wl, al, ci, 0, 0, 0);
        ci = __builtin_amdgcn_mfma_i32_16x16x64_i8(wh, ah, ci, 0, 0, 0);
        return __builtin_bit_cast(g4f, ci);
    } else if constexpr (MODE == GM_MXF4) {
        const g8i wl = {w[0], w[1], w[2], w[3], 0, 0, 0, 0}, wh = {w[4], w[5], w[6], w[7], 0, 0, 0, 0};
        const g8i al = {a[0], a[1], a[2], a[3], 0, 0, 0, 0}, ah = {a[4], a[5], a[6], a[7], 0, 0, 0, 0};
        c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wl, al, c, 4, 4, 0, sw[0], 0, sa[0]);
        return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wh, ah, c, 4, 4, 0, sw[1], 0, sa[1]);
    } else {
        const g4i wl = {w[0], w[1], w[2], w[3]}, wh = {w[4], w[5], w[6], w[7]};
        const g4i al = {a[0], a[1], a[2], a[3]}, ah = {a[4], a[5], a[6], a[7]};
        if constexpr (MODE == GM_BF16) {
            c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    __builtin_bit_cast(g8bf, wl), __builtin_bit_cast(g8bf, al), c, 0, 0, 0);
            return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    __builtin_bit_cast(g8bf, wh), __builtin_bit_cast(g8bf, ah), c, 0, 0, 0);
        } else {
            c = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                    __builtin_bit_cast(g8h, wl), __builtin_bit_cast(g8h, al), c, 0, 0, 0);
            return __builtin_amdgcn_mfma_f32_16x16x32_f16(
                    __builtin_bit_cast(g8h, wh), __builtin_bit_cast(g8h, ah), c, 0, 0, 0);
        }
    }
}

// what a workgroup knows about its tile (uniform over the workgroup)
struct gtile_t {
    long g, m_base, rows; // group, first row of the tile inside the group, rows of the group
    long dst0, src0;      // first row of the group in dst / src
    long n0;              // first column of the tile
};

// The weights' scales of one step for NT * 16 columns, [G][K / 32][N] with N contiguous: lane (j, q)
// fetches the dword of columns 4 j .. 4 j + 3 of block row q (and 4 + q for fp4); the byte lane (j, q)
// needs for fragment jn -- column 16 jn + j, block q -- sits in lane (4 jn + j / 4, q), byte j % 4.
template <int MODE, int NT>
struct gscale_b_t {
    using Mo = gmode_t<MODE>;
    const char *base; // scales of this group at the tile's first column (uniform)
    uint32_t off;     // lane part: block row q, dword of columns
    long N;
    __device__ __forceinline__ void init(const grouped_dev_t &P, const gtile_t &T, long n_first, int lane) {
        const int j = lane & 15, q = lane >> 4;
        N = P.d.N;
        const long kb = P.d.K / 32;
        int jj = j < 4 * NT ? j : 4 * NT - 1;
        long col = n_first + 4 * jj;
        col = col <= N - 4 ? col : N - 4; // N is a multiple of 4: a dword is inside or outside as a whole
        base = (const char *)P.a.wei_scale + T.g * kb * N;
        off = (uint32_t)(q * N + col);
    }
    __device__ __forceinline__ void load(long step, int (&raw)[2]) const {
#pragma unroll
        for (int h = 0; h < Mo::SB; ++h) raw[h] = *(const int *)(base + (step * Mo::BPS + 4 * h) * N + off);
    }
    __device__ __forceinline__ void pick(const int (&raw)[2], int jn, int lane, int (&out)[2]) const {
        const int j = lane & 15, q = lane >> 4;
        const int from = 4 * (16 * q + 4 * jn + (j >> 2));
#pragma unroll
        for (int h = 0; h < Mo::SB; ++h) out[h] = (__builtin_amdgcn_ds_bpermute(from, raw[h]) >> (8 * (j & 3))) & 0xff;
    }
};

// rows of group g that both src and dst hold, and where they start; offsets
// that leave [0, total] or run backwards give fewer rows, never an access
// outside the tensors
__device__ __forceinline__ long grouped_rows(const grouped_dev_t &P, long g, long &dst0, long &src0) {
    const long total = P.d.total;
    auto clamp = [&](long v) { return v < 0 ? 0 : (v > total ? total : v); };
    dst0 = g > 0 ? clamp(P.a.dst_offsets[g - 1]) : 0;
    src0 = g > 0 ? clamp(P.a.src_offsets[g - 1]) : 0;
    const long nd = clamp(P.a.dst_offsets[g]) - dst0, ns = clamp(P.a.src_offsets[g]) - src0;
    const long n = nd < ns ? nd : ns;
    return n > 0 ? n : 0;
}

// One wavefront's share of a tile's K walk: steps wk, wk + WK, .. of 128 bytes per
// row for MF fragments of 16 src rows against NT fragments of 16 weights rows,
// D steps in flight.  Leaves the MF x NT accumulators in `part`.  NTL: the weights are loaded non-temporally
// (they are read once); only when every row starts on a 128-byte line -- otherwise a step's last line is also
// the next step's first and has to stay in the caches (measured: 75 -> 98 us on K = 2880).
template <int MODE, int FA, int FB, int MF, int NT, int D, int WK, bool NTL>
__device__ __forceinline__ void grouped_walk(const grouped_dev_t &P, const gtile_t &T, g4f *part, int wk, int lane) {
    using Mo = gmode_t<MODE>;
    const mi355_grouped_desc_t &Dd = P.d;
    const int j = lane & 15, q = lane >> 4;
    const long row_bytes = Mo::bytes(Dd.K);
    // A load instruction fetches whole 128-byte lines: 8 rows x 8 chunks of 16
    // bytes.  Lane (j, q) fetches one chunk of rows j % 8 and 8 + j % 8 of a
    // fragment; lanes j and j +- 8 then exchange one of the two so that lane
    // (j, q) holds two chunks of row j (which ones: gmode_t).
    const int half = j >> 3;
    const uint32_t chunk = 16 * Mo::chunk_fetch(q, half);
    const long pitch_b = Mo::bytes(Dd.wei_stride[2]);
    const char *abase = (const char *)P.a.src + (T.src0 + T.m_base) * row_bytes;
    const char *bbase = (const char *)P.a.wei + Mo::bytes(T.g * Dd.wei_stride[0] + T.n0 * Dd.wei_stride[2]);
    uint32_t aoff[MF][2], boff[NT][2];
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            long m = T.m_base + 16 * i + 8 * h + (j & 7);
            m = m < T.rows ? m : T.rows - 1; // rows beyond the group read its last one (never stored)
            aoff[i][h] = (uint32_t)((m - T.m_base) * row_bytes) + chunk;
        }
#pragma unroll
    for (int jn = 0; jn < NT; ++jn)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            long n = T.n0 + 16 * jn + 8 * h + (j & 7);
            n = n < Dd.N ? n : Dd.N - 1;
            boff[jn][h] = (uint32_t)((n - T.n0) * pitch_b) + chunk;
        }
    // MX: the src scales of row 16 i + j ([total_M][K / 32], a dword or two per step) and the weights' scales
    const long kblocks = Dd.K / 32;
    const char *sabase = Mo::MX ? (const char *)P.a.src_scale + (T.src0 + T.m_base) * kblocks : nullptr;
    uint32_t saoff[MF];
    gscale_b_t<MODE, NT> SBs;
    if constexpr (Mo::MX) {
#pragma unroll
        for (int i = 0; i < MF; ++i) {
            long m = T.m_base + 16 * i + j;
            m = m < T.rows ? m : T.rows - 1;
            saoff[i] = (uint32_t)((m - T.m_base) * kblocks);
        }
        SBs.init(P, T, T.n0, lane);
    }
    struct stage_t {
        g4i a[MF][2], b[NT][2];
        int sa[MF][2], sb[2];
    };
    // step_off: byte offset of the step in a row (uniform)
    auto load = [&](long step_off, uint32_t back) __attribute__((always_inline)) {
        stage_t f;
#pragma unroll
        for (int jn = 0; jn < NT; ++jn)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const g4i *bp = (const g4i *)(bbase + step_off + (boff[jn][h] - back));
                f.b[jn][h] = NTL ? __builtin_nontemporal_load(bp) : *bp;
            }
#pragma unroll
        for (int i = 0; i < MF; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h) f.a[i][h] = *(const g4i *)(abase + step_off + (aoff[i][h] - back));
        if constexpr (Mo::MX) {
            const long step = step_off >> 7;
            SBs.load(step, f.sb);
#pragma unroll
            for (int i = 0; i < MF; ++i)
#pragma unroll
                for (int h = 0; h < Mo::SB; ++h) f.sa[i][h] = *(const int *)(sabase + step * Mo::BPS + 4 * h + saoff[i]);
        }
        return f;
    };
    // the exchange between lanes j and j +- 8 (a rotation by 8 inside each row of 16 lanes)
    auto settle = [&](const g4i (&r)[2]) __attribute__((always_inline)) {
        g8i out;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int send = half ? r[0][e] : r[1][e];
            const int recv = __builtin_amdgcn_update_dpp(0, send, 0x128 /* row_ror:8 */, 0xf, 0xf, false);
            out[e] = half ? recv : r[0][e];
            out[4 + e] = half ? r[1][e] : recv;
        }
        return out;
    };
    g4f acc[MF][NT];
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
        for (int jn = 0; jn < NT; ++jn) acc[i][jn] = g4f {0.f, 0.f, 0.f, 0.f};
    auto compute = [&](const stage_t &f) __attribute__((always_inline)) {
        g8i a[MF];
        int sa[MF][2];
#pragma unroll
        for (int i = 0; i < MF; ++i) {
            a[i] = settle(f.a[i]);
#pragma unroll
            for (int h = 0; h < 2; ++h) sa[i][h] = Mo::MX ? (f.sa[i][h] >> (8 * q)) & 0xff : 0; // block q (4 + q) of the step
        }
#pragma unroll
        for (int jn = 0; jn < NT; ++jn) {
            const g8i w = settle(f.b[jn]);
            int sw[2] = {0, 0};
            if constexpr (Mo::MX) SBs.pick(f.sb, jn, lane, sw);
#pragma unroll
            for (int i = 0; i < MF; ++i) acc[i][jn] = grouped_mma<MODE, FA, FB>(w, a[i], acc[i][jn], sw, sa[i]);
        }
    };

    const long nfull = row_bytes / 128;
    const int tail = (int)(row_bytes % 128); // a multiple of 32
    if (nfull > wk) {
        // this wavefront's steps: wk + WK * c, c < count; whole rounds of D run
        // without a condition (loads beyond the end repeat the last step)
        const long count = (nfull - wk + WK - 1) / WK;
        // workgroups start at different places of K and wrap around: walking in step, they
        // would all ask the same few memory channels at a time when K is a power of two
        const long c0 = (long)((blockIdx.x * 5u + blockIdx.y * 3u) % (unsigned long)count);
        auto step_off = [&](long c) {
            long cr = (c < count ? c : count - 1) + c0;
            cr = cr >= count ? cr - count : cr;
            return (wk + WK * cr) * 128;
        };
        stage_t st[D];
#pragma unroll
        for (int d = 0; d < D; ++d) st[d] = load(step_off(d), 0);
        long c = 0;
        for (; c + D <= count; c += D) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                compute(st[d]);
                st[d] = load(step_off(c + D + d), 0);
                // keep the rounds apart: the scheduler would otherwise start the next
                // stage's products early and wait for every load in flight
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int d = 0; d < D; ++d)
            if (c + d < count) compute(st[d]);
    }
    if (tail != 0 && wk == (int)(nfull % WK)) {
        // a chunk beyond K: the lane reads the step's first chunk instead and hands on zeros
        const bool in = chunk + 16 <= (uint32_t)tail;
        stage_t f = load(nfull * 128, in ? 0 : chunk);
        if (!in) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int i = 0; i < MF; ++i) f.a[i][h] = g4i {0, 0, 0, 0};
#pragma unroll
                for (int jn = 0; jn < NT; ++jn) f.b[jn][h] = g4i {0, 0, 0, 0};
            }
        }
        compute(f);
    }
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
        for (int jn = 0; jn < NT; ++jn) part[((wk * MF + i) * NT + jn) * 64 + lane] = acc[i][jn];
}

// The same walk for row-major weights ([G][K][N], tag abc: a k row holds its N columns) of the 16-bit types, 64
// columns a tile.  A column's eight consecutive k lie a row pitch apart, so a lane fetches 8 bytes -- four columns
// 4 j .. 4 j + 3 -- of each of the rows k = 8 q .. 8 q + 7 and 32 + 8 q .. (a load instruction covers whole lines:
// four rows x 128 bytes) and turns them inside the lane (`gk_frag16`) into the four fragments it needs: fragment
// c holds column 4 j + c in lane (j, q).  The matrix instruction does not mind which 16 columns share a fragment;
// the accumulators -- acc[i][c][e] is src row 16 i + j, column 16 q + 4 e + c -- are written to `part` in the
// arrangement of the K-contiguous walk (unit q, lane (j, e), element c), so the same epilogue follows.
template <int MODE, int MF, int D, int WK, bool NTL>
__device__ __forceinline__ void grouped_walk_bt(const grouped_dev_t &P, const gtile_t &T, g4f *part, int wk, int lane) {
    constexpr int NT = 4;
    using Mo = gmode_t<MODE>;
    static_assert(Mo::EBITS == 16, "row-major weights: bf16 / f16 only");
    const mi355_grouped_desc_t &Dd = P.d;
    const int j = lane & 15, q = lane >> 4, half = j >> 3;
    const long row_bytes = 2 * Dd.K;
    const uint32_t chunk = 16 * Mo::chunk_fetch(q, half);
    const char *abase = (const char *)P.a.src + (T.src0 + T.m_base) * row_bytes;
    uint32_t aoff[MF][2];
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            long m = T.m_base + 16 * i + 8 * h + (j & 7);
            m = m < T.rows ? m : T.rows - 1;
            aoff[i][h] = (uint32_t)((m - T.m_base) * row_bytes) + chunk;
        }
    const long pitch_b = 2 * Dd.wei_stride[1];
    long col = T.n0 + 4 * j;
    col = col <= Dd.N - 4 ? col : Dd.N - 4; // N is a multiple of 4; columns beyond N are never stored
    const char *bbase = (const char *)P.a.wei + 2 * (T.g * Dd.wei_stride[0] + col) + 8 * q * pitch_b;
    struct stage_t {
        g4i a[MF][2];
        gk_u2 b[2][8];
    };
    // k0: the step's first k (uniform)
    auto load = [&](long k0) __attribute__((always_inline)) {
        stage_t f;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const gk_u2 *bp = (const gk_u2 *)(bbase + (k0 + 32 * h + r) * pitch_b);
                f.b[h][r] = NTL ? __builtin_nontemporal_load(bp) : *bp;
            }
#pragma unroll
        for (int i = 0; i < MF; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h) f.a[i][h] = *(const g4i *)(abase + 2 * k0 + aoff[i][h]);
        return f;
    };
    auto settle = [&](const g4i (&r)[2]) __attribute__((always_inline)) {
        g8i out;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int send = half ? r[0][e] : r[1][e];
            const int recv = __builtin_amdgcn_update_dpp(0, send, 0x128 /* row_ror:8 */, 0xf, 0xf, false);
            out[e] = half ? recv : r[0][e];
            out[4 + e] = half ? r[1][e] : recv;
        }
        return out;
    };
    g4f acc[MF][NT];
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
        for (int c = 0; c < NT; ++c) acc[i][c] = g4f {0.f, 0.f, 0.f, 0.f};
    auto compute = [&](const stage_t &f) __attribute__((always_inline)) {
        g8i a[MF];
#pragma unroll
        for (int i = 0; i < MF; ++i) a[i] = settle(f.a[i]);
#pragma unroll
        for (int c = 0; c < NT; ++c) {
            const g4u lo = gk_frag16(f.b[0], c), hi = gk_frag16(f.b[1], c);
            const g8i w = {(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
#pragma unroll
            for (int i = 0; i < MF; ++i) acc[i][c] = grouped_mma<MODE, 0, 0>(w, a[i], acc[i][c]);
        }
    };

    const long nfull = Dd.K / 64;
    const int tail = (int)(Dd.K % 64); // a multiple of 16
    if (nfull > wk) {
        const long count = (nfull - wk + WK - 1) / WK;
        const long c0 = (long)((blockIdx.x * 5u + blockIdx.y * 3u) % (unsigned long)count);
        auto step_k0 = [&](long c) {
            long cr = (c < count ? c : count - 1) + c0;
            cr = cr >= count ? cr - count : cr;
            return (wk + WK * cr) * 64;
        };
        stage_t st[D];
#pragma unroll
        for (int d = 0; d < D; ++d) st[d] = load(step_k0(d));
        long c = 0;
        for (; c + D <= count; c += D) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                compute(st[d]);
                st[d] = load(step_k0(c + D + d));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int d = 0; d < D; ++d)
            if (c + d < count) compute(st[d]);
    }
    if (tail != 0 && wk == (int)(nfull % WK)) {
        // k beyond K: zeros on both sides (a product with a zero operand would still be NaN against an infinity)
        stage_t f;
        const long k0 = nfull * 64;
        const bool in = chunk + 16 <= (uint32_t)(2 * tail);
#pragma unroll
        for (int i = 0; i < MF; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                f.a[i][h] = g4i {0, 0, 0, 0};
                if (in) f.a[i][h] = *(const g4i *)(abase + 2 * k0 + aoff[i][h]);
            }
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                f.b[h][r] = gk_u2 {0u, 0u};
                if (32 * h + 8 * q + r < tail) f.b[h][r] = *(const gk_u2 *)(bbase + (k0 + 32 * h + r) * pitch_b);
            }
        compute(f);
    }
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e)
            part[((wk * MF + i) * NT + q) * 64 + j + 16 * e] = g4f {acc[i][0][e], acc[i][1][e], acc[i][2][e], acc[i][3][e]};
}

// Which (group, row block) is slot `slot`: a block-wide prefix sum over the
// groups' row-block counts.  False (for the whole workgroup) beyond the last tile.
template <int BM, int NW>
__device__ __forceinline__ bool grouped_find_tile(const grouped_dev_t &P, int slot, gtile_t &T) {
    __shared__ int pick[2];
    __shared__ int wave_tot[NW];
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const long G = P.d.group_count;
    const long per = (G + 64 * NW - 1) / (64 * NW); // groups per thread
    auto blocks_of = [&](long g) {
        long d0, s0;
        return (int)((grouped_rows(P, g, d0, s0) + BM - 1) / BM);
    };
    int local = 0;
    for (long i = 0; i < per; ++i) {
        const long g = (long)t * per + i;
        if (g < G) local += blocks_of(g);
    }
    int x = local;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int y = __shfl_up(x, o, 64);
        if (lane >= o) x += y;
    }
    if (t == 0) pick[0] = -1;
    if (lane == 63) wave_tot[wave] = x;
    __syncthreads();
    int before = x - local;
    for (int w = 0; w < wave; ++w) before += wave_tot[w];
    for (long i = 0; i < per; ++i) {
        const long g = (long)t * per + i;
        if (g < G) {
            const int nb = blocks_of(g);
            if (slot >= before && slot < before + nb) {
                pick[0] = (int)g;
                pick[1] = slot - before;
            }
            before += nb;
        }
    }
    __syncthreads();
    T.g = __builtin_amdgcn_readfirstlane(pick[0]);
    if (T.g < 0) return false;
    T.m_base = (long)__builtin_amdgcn_readfirstlane(pick[1]) * BM;
    T.rows = grouped_rows(P, T.g, T.dst0, T.src0); // > m_base
    return true;
}

// Scales, bias, post-ops, conversion and store of four consecutive columns nb .. nb + 3 of row m
// (a lane's share of a 16 x 16 unit).
__device__ __forceinline__ void grouped_store_quad(const grouped_dev_t &P, const gtile_t &T, g4f sum, long m, long nb) {
    const mi355_grouped_desc_t &Dd = P.d;
    const long N = Dd.N;
    if (m >= T.rows || nb >= N) return;
    // scales with groups along K (the MX modes) were applied by the matrix instruction
    // (a group that spans all of K is one scale per row / per group and column: no groups along K)
    const bool with_ss = Dd.src_scale_dt != MI355_DT_UNDEF && (Dd.src_scale_gk <= 1 || Dd.src_scale_gk == Dd.K);
    const bool with_ws = Dd.wei_scale_dt != MI355_DT_UNDEF && (Dd.wei_scale_gk <= 1 || Dd.wei_scale_gk == Dd.K);
    const int dbits = dt_bits(Dd.dst_dt);
    const bool vec_ok = N % 4 == 0 && ((uintptr_t)P.a.dst % 16) == 0;
    const float ss = with_ss ? load_float(Dd.src_scale_dt, P.a.src_scale, T.src0 + m) : 1.f;
    const int nvalid = N - nb < 4 ? (int)(N - nb) : 4;
    uint32_t bits[4] = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if (e < nvalid) {
            float v = sum[e];
            if (with_ss) v *= ss;
            if (with_ws) v *= load_float(Dd.wei_scale_dt, P.a.wei_scale, T.g * N + nb + e);
            v = grouped_finish(P, v, T.g, m, nb + e, T.dst0);
            bits[e] = cvt_store_bits(Dd.dst_dt, v);
        }
    }
    const long off = (T.dst0 + m) * N + nb;
    if (vec_ok && nvalid == 4) {
        if (dbits == 32)
            *(g4u *)((char *)P.a.dst + off * 4) = g4u {bits[0], bits[1], bits[2], bits[3]};
        else
            *(g2u *)((char *)P.a.dst + off * 2) = g2u {bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16)};
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (e < nvalid) {
                if (dbits == 32) ((uint32_t *)P.a.dst)[off + e] = bits[e];
                else ((uint16_t *)P.a.dst)[off + e] = (uint16_t)bits[e];
            }
        }
    }
}

// BT: row-major weights (`grouped_walk_bt`)
template <int MODE, int FA, int FB, int MTMAX, int NT, int D, int NW, int OCC, bool BT = false>
__global__ void __launch_bounds__(64 * NW, OCC) grouped_tile_kernel(const grouped_dev_t P) {
    constexpr int BM = 16 * MTMAX, BN = 16 * NT;
    extern __shared__ g4f part[]; // [wavefront][fragment row][fragment column][lane]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    gtile_t T;
    if (!grouped_find_tile<BM, NW>(P, blockIdx.y, T)) return;
    T.n0 = (long)blockIdx.x * BN;
    const long here = T.rows - T.m_base < BM ? T.rows - T.m_base : BM;
    const int mf = __builtin_amdgcn_readfirstlane((int)((here + 15) / 16)); // fragments of 16 rows the tile holds

    // ---- K: the wavefronts take the 128-byte steps in turn, each over the whole tile
    const bool whole_lines = gmode_t<MODE>::bytes(P.d.wei_stride[BT ? 1 : 2]) % 128 == 0;
#define MI355_GROUPED_WALK(MF_) \
    do { \
        if constexpr (BT) { \
            if (whole_lines) grouped_walk_bt<MODE, MF_, D, NW, true>(P, T, part, wave, lane); \
            else grouped_walk_bt<MODE, MF_, D, NW, false>(P, T, part, wave, lane); \
        } else { \
            if (whole_lines) grouped_walk<MODE, FA, FB, MF_, NT, D, NW, true>(P, T, part, wave, lane); \
            else grouped_walk<MODE, FA, FB, MF_, NT, D, NW, false>(P, T, part, wave, lane); \
        } \
    } while (0)
    switch (mf) {
        case 1: MI355_GROUPED_WALK(1); break;
        case 2:
            if constexpr (MTMAX >= 2) MI355_GROUPED_WALK(2);
            break;
        case 3:
            if constexpr (MTMAX >= 3) MI355_GROUPED_WALK(3);
            break;
        default:
            if constexpr (MTMAX >= 4) MI355_GROUPED_WALK(4);
            break;
    }
#undef MI355_GROUPED_WALK
    __syncthreads();

    // ---- the 16 x 16 units of the tile are finished by the wavefronts in
    // turn (one copy of the scales / bias / post-op / conversion code): lane
    // (j, q) holds row j, columns 4 q .. 4 q + 3 of a unit
    const int j = lane & 15, q = lane >> 4;
#pragma nounroll
    for (int u = wave; u < mf * NT; u += NW) {
        const int i = u / NT, jn = u % NT;
        g4f sum = part[u * 64 + lane];
        if constexpr (MODE == GM_I8) {
            g4i isum = __builtin_bit_cast(g4i, sum);
#pragma unroll
            for (int w = 1; w < NW; ++w) isum += __builtin_bit_cast(g4i, part[(w * mf * NT + u) * 64 + lane]);
            sum = g4f {(float)isum[0], (float)isum[1], (float)isum[2], (float)isum[3]};
        } else {
#pragma unroll
            for (int w = 1; w < NW; ++w) sum += part[(w * mf * NT + u) * 64 + lane];
        }
        grouped_store_quad(P, T, sum, T.m_base + 16 * i + j, T.n0 + 16 * jn + 4 * q);
    }
}

// ---- the second tile shape of "hip:mfma_grouped": columns split between the
// wavefronts, src rows shared through LDS.
//
// A workgroup owns (group, up to 16 * MTMAX rows, 256 columns); each of its four
// wavefronts owns 64 columns (four fragments) and walks all of K with D steps
// of its weights in flight in registers (whole-line loads + lane exchange as
// above).  The src rows of the tile are needed by all four wavefronts: they
// are brought to LDS once per workgroup, 512 bytes of K (four steps) per row at
// a time, by direct-to-LDS loads that fetch whole lines (8 rows x 128 bytes per
// instruction), double buffered, one barrier per four steps.  Per byte of
// weights a quarter of the src traffic of the 64-column tiles goes through the
// vector memory path, which is what bounds these kernels.
//
// LDS layout of one (fragment, step) block of 16 rows x 128 bytes: the 16-byte
// chunk c of row r sits in slot 8 r + (c ^ (r / 2)); a direct-to-LDS
// instruction fills 64 consecutive slots, so its lane L fetches row L / 8 (of
// the block's lower or upper half), chunk (L % 8) ^ (row / 2); the fragment
// read of lanes (j, q) -- slots 8 j + (q ^ (j / 2)) -- touches every bank once
// per 16 lanes.
typedef const g4i __attribute__((address_space(3))) *lds_g4i_ptr_t;
typedef g4f __attribute__((address_space(3))) *lds_g4f_ptr_t;

// lane i brings 16 bytes from sbase + voff to LDS byte address lds_addr + 16 i
__device__ __forceinline__ void grouped_dma16(const void *sbase, unsigned voff, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(sbase)
                 : "memory", "m0");
}

// ---- the variable-K pattern, long groups of bf16 / f16: the operands of a 128 x 128 tile go through LDS.
//
// Per step of 32 k the workgroup needs 32 rows of 256 bytes of each operand.  They are fetched by direct-to-LDS
// instructions (a wavefront's instruction brings four rows, 1 KB; no registers are held while a stage is in
// flight, so NST - 1 stages are), once per workgroup instead of once per wavefront.  A block of four rows takes
// GK_BLOCK = 1024 + 64 bytes of LDS: lane (i, q) reads row 8 q + t, bytes 8 i .. 8 i + 7 of its wavefront's half,
// and two blocks further on (q + 1) is 128 bytes further on in the banks, so the four q of a read share the 64
// banks two by two, which is what 512 bytes cost anyway.  gk_frag16 transposes inside the lane.
// Rows past the group's end are fetched from its last row (any valid address) and the lanes clear their
// fragments' k slots past the end on both operands; columns past the tensors' edge are fetched from column 0 of
// the tile and only reach accumulators that are not stored.
// NST stages: 4 for long groups; 2 where the groups are a step or two (three workgroups fit a compute unit then,
// and what a workgroup waits for is the latency of its only fetch).
constexpr int GK_BLOCK = 1024 + 64, GK_OPERAND = 8 * GK_BLOCK, GK_STAGE = 2 * GK_OPERAND;

// s_waitcnt vmcnt(n) for the counts the kernel below uses (the instruction takes an immediate)
__device__ __forceinline__ void gk_wait_vm(int n) {
    switch (n) {
        case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
        case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
        case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
        case 16: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
        case 20: asm volatile("s_waitcnt vmcnt(20)" ::: "memory"); break;
        case 24: asm volatile("s_waitcnt vmcnt(24)" ::: "memory"); break;
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
}

template <int DT, int GK_NST>
__global__ void __launch_bounds__(256) grouped_k_lds_kernel(const grouped_k_dev_t P) {
    typedef gk_f4 f4;
    extern __shared__ __attribute__((aligned(16))) unsigned char gk_smem[];
    const unsigned lds0 = (unsigned)(uintptr_t)gk_smem;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, q = lane >> 4;
    const long g = blockIdx.y;
    // a workgroup takes a run of `run` column tiles of one row of tiles, one after the other
    const int runs_n = (P.tiles_n + P.run - 1) / P.run;
    const long m_t = (long)(blockIdx.x / runs_n) * 128;
    const int tn0 = (int)(blockIdx.x % runs_n) * P.run;
    const int count = P.tiles_n - tn0 < P.run ? P.tiles_n - tn0 : P.run;
    const long m_w = m_t + (wave >> 1) * 64;
    long k0 = g > 0 ? (long)P.offsets[g - 1] : 0, k1 = P.offsets[g];
    if (k0 < 0) k0 = 0;
    if (k1 > P.total) k1 = P.total;
    const long nsteps = k0 < k1 ? (k1 - k0 + 31) / 32 : 0;

    // this lane's part of a block: row lane / 16 of its four, the 16 bytes of columns 8 (lane % 16) ..
    const long ca = m_t + 8 * i < P.MA ? 8 * i : 0;
    const unsigned char *abase = (const unsigned char *)P.a + (k0 * P.MA + m_t) * 2;
    const long last = k1 - 1 - k0;
    auto issue = [&](long n_t, long step) {
        const unsigned cb = n_t + 8 * i < P.NB ? 16 * i : 0;
        const unsigned char *bbase = (const unsigned char *)P.b + (k0 * P.NB + n_t) * 2;
        const unsigned slot = lds0 + (unsigned)(step % GK_NST) * GK_STAGE;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int blk = 2 * wave + h;
            long row = step * 32 + 4 * blk + q;
            row = row < last ? row : last;
            grouped_dma16(abase, (unsigned)((row * P.MA + ca) * 2), slot + blk * GK_BLOCK);
            grouped_dma16(bbase, (unsigned)(row * P.NB * 2) + cb, slot + GK_OPERAND + blk * GK_BLOCK);
        }
    };
    auto first_stages = [&](long n_t) {
#pragma unroll
        for (int s = 0; s < GK_NST - 1; ++s)
            if (s < nsteps) issue(n_t, s);
    };
    const unsigned a_rd = (unsigned)(2 * q * GK_BLOCK + ((wave >> 1) * 64 + 4 * i) * 2);
    const unsigned b_rd = (unsigned)(GK_OPERAND + 2 * q * GK_BLOCK + ((wave & 1) * 64 + 4 * i) * 2);

    first_stages((long)tn0 * 128);
    int stores_behind = 0; // store instructions of this wavefront issued after the tile's first stages (-1: some)
#pragma nounroll
    for (int tp = 0; tp < count; ++tp) {
        const long n_t = (long)(tn0 + tp) * 128;
        f4 acc[4][4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[r][c] = f4 {0.f, 0.f, 0.f, 0.f};
        for (long step = 0; step < nsteps; ++step) {
            // this wavefront's part of the stage has landed; after the barrier everyone's has, and
            // everyone is done reading the stage that the next instructions overwrite
            // (four instructions a stage and wavefront; stages past the group's end are not fetched, so
            // towards the end fewer are behind this one)
            const long behind = nsteps - step - 1;
            const int stages_behind = behind >= GK_NST - 2 ? GK_NST - 2 : (int)behind;
            // Memory instructions complete in the order of issue, stores included: when the previous tile
            // was a whole one, exactly 16 store instructions of this wavefront follow the first stages in the
            // queue and need not be waited for (otherwise their number depends on the edges: wait for all)
            if (__builtin_expect(step < GK_NST - 1 && stores_behind != 0, 0)) {
                if (stores_behind == 16) gk_wait_vm(4 * stages_behind + 16);
                else gk_wait_vm(0);
            } else if (behind >= GK_NST - 2) {
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(4 * (GK_NST - 2)) : "memory");
            } else if (behind == 1) {
                asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
            } else {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
            __syncthreads();
            if (step + GK_NST - 1 < nsteps) issue(n_t, step + GK_NST - 1);
            const unsigned slot = (unsigned)(step % GK_NST) * GK_STAGE;
            gk_u2 ra[8], rb[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const unsigned off = slot + (t >> 2) * GK_BLOCK + (t & 3) * 256;
                ra[t] = *(const gk_u2 *)(gk_smem + a_rd + off);
                rb[t] = *(const gk_u2 *)(gk_smem + b_rd + off);
            }
            g4u a[4], b[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) a[e] = gk_frag16(ra, e), b[e] = gk_frag16(rb, e);
            const long left = k1 - k0 - step * 32 - 8 * q; // k slots of this lane inside the group
            if (step == nsteps - 1 && (k1 - k0) % 32 != 0) {
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const unsigned keep = left >= 2 * d + 2 ? 0xffffffffu : (left == 2 * d + 1 ? 0xffffu : 0u);
#pragma unroll
                    for (int e = 0; e < 4; ++e) a[e][d] &= keep, b[e][d] &= keep;
                }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if (DT == MI355_DT_BF16)
                        acc[r][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(g8bf, a[r]),
                                __builtin_bit_cast(g8bf, b[c]), acc[r][c], 0, 0, 0);
                    else
                        acc[r][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(g8h, a[r]),
                                __builtin_bit_cast(g8h, b[c]), acc[r][c], 0, 0, 0);
                }
        }
        // The next tile's first stages go out before this tile's stores: a compute unit's memory instructions
        // are served in order, so a fetch issued behind 32 KB of stores waits for all of them (a workgroup a
        // tile measured fetch + arithmetic + stores end to end, nothing hidden); this way the fetch is done by
        // the time the stores are, and the store queue stays fed.
        if (tp + 1 < count && nsteps > 0) {
            __syncthreads(); // everyone has read this tile's last stage
            first_stages(n_t + 128);
        }
        const long n_w = n_t + (wave & 1) * 64;
        if (m_w < P.MA && n_w < P.NB) gk_store<DT>(P, acc, g, m_w, n_w, i, q);
        stores_behind = m_w >= P.MA || n_w >= P.NB ? 0 : (m_w + 64 <= P.MA && n_w + 64 <= P.NB ? 16 : -1);
    }
}

// NT: fragments of 16 columns per wavefront.  Leaves the wavefront's MF x NT accumulators in LDS at
// lds0 + (wave * MF * NT + unit) * 1024.
template <int MODE, int FA, int FB, int MF, int NT, int D>
__device__ __forceinline__ void grouped_walk_nsplit(const grouped_dev_t &P, const gtile_t &T, unsigned lds0, int wave,
        int lane) {
    constexpr int CH = 4; // steps per src chunk in LDS
    static_assert(CH % D == 0, "a step's register stage must not depend on the chunk");
    using Mo = gmode_t<MODE>;
    constexpr unsigned ABUF = MF * CH * 2048; // bytes of one src buffer
    constexpr unsigned SBUF = Mo::SB * 1024;    // MX: the src scales of a chunk, 16 bytes (two of them for fp4) per row
    const mi355_grouped_desc_t &Dd = P.d;
    const int j = lane & 15, q = lane >> 4;
    const long row_bytes = Mo::bytes(Dd.K);
    const long nfull = row_bytes / 128;
    const int tail = (int)(row_bytes % 128); // a multiple of 32
    const long nsteps = nfull + (tail != 0);
    const long nchunks = (nsteps + CH - 1) / CH;

    // ---- weights: as in grouped_walk, for this wavefront's 64 columns
    const int half = j >> 3;
    const uint32_t chunk = 16 * Mo::chunk_fetch(q, half);
    const long pitch_b = Mo::bytes(Dd.wei_stride[2]);
    const char *bbase = (const char *)P.a.wei + Mo::bytes(T.g * Dd.wei_stride[0] + T.n0 * Dd.wei_stride[2]);
    uint32_t boff[NT][2];
#pragma unroll
    for (int jn = 0; jn < NT; ++jn)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            long n = T.n0 + 16 * NT * wave + 16 * jn + 8 * h + (j & 7);
            n = n < Dd.N ? n : Dd.N - 1;
            boff[jn][h] = (uint32_t)((n - T.n0) * pitch_b) + chunk;
        }
    struct stage_t {
        g4i b[NT][2];
        int sb[2];
    };
    gscale_b_t<MODE, NT> SBs;
    if constexpr (Mo::MX) SBs.init(P, T, T.n0 + 16 * NT * wave, lane);
    // A lane whose chunk lies beyond K in the tail step fetches the step's first chunk
    // instead (the tail holds at least 32 bytes); steps beyond the last repeat it.
    const uint32_t b_back = chunk + 16 <= (uint32_t)tail ? 0 : chunk;
    auto load_b = [&](long s) __attribute__((always_inline)) {
        stage_t f;
        s = s < nsteps ? s : nsteps - 1;
        const uint32_t back = s >= nfull ? b_back : 0;
#pragma unroll
        for (int jn = 0; jn < NT; ++jn)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                f.b[jn][h] = __builtin_nontemporal_load((const g4i *)(bbase + s * 128 + (boff[jn][h] - back)));
        if constexpr (Mo::MX) SBs.load(s, f.sb);
        return f;
    };
    auto settle = [&](const g4i (&r)[2]) __attribute__((always_inline)) {
        g8i out;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int send = half ? r[0][e] : r[1][e];
            const int recv = __builtin_amdgcn_update_dpp(0, send, 0x128 /* row_ror:8 */, 0xf, 0xf, false);
            out[e] = half ? recv : r[0][e];
            out[4 + e] = half ? r[1][e] : recv;
        }
        return out;
    };

    // ---- src: this wavefront's share of a chunk's direct-to-LDS loads.  Instruction
    // wave + 4 x of the chunk's 2 * MF * CH fills half (wave % 2) of block (wave + 4 x) / 2
    // = (fragment, step); the row and chunk a lane fetches are the same in all of them.
    constexpr int NDMA = 2 * MF * CH / 4;
    const char *abase = (const char *)P.a.src + (T.src0 + T.m_base) * row_bytes;
    const int a_r = 8 * (wave & 1) + (lane >> 3);
    const uint32_t a_chunk = 16 * ((lane & 7) ^ (a_r >> 1));
    const uint32_t a_back = a_chunk + 16 <= (uint32_t)tail ? 0 : a_chunk;
    uint32_t a_row[NDMA]; // byte offset of the lane's row, per instruction (the fragment differs)
#pragma unroll
    for (int x = 0; x < NDMA; ++x) {
        const int i = ((wave + 4 * x) >> 1) / CH;
        long m = T.m_base + 16 * i + a_r;
        m = m < T.rows ? m : T.rows - 1; // rows beyond the group read its last one (never stored)
        a_row[x] = (uint32_t)((m - T.m_base) * row_bytes);
    }
    // MX: wavefront 3 also brings the chunk's src scales, lane L those of row L of the tile: 16 bytes = four steps
    // of four blocks (fp8); for fp4 (eight blocks a step) a second instruction brings the next 16
    const long kblocks = Dd.K / 32;
    const char *sabase = Mo::MX ? (const char *)P.a.src_scale + (T.src0 + T.m_base) * kblocks : nullptr;
    uint32_t sa_row = 0;
    if constexpr (Mo::MX) {
        long m = T.m_base + lane;
        m = m < T.rows ? m : T.rows - 1;
        sa_row = (uint32_t)((m - T.m_base) * kblocks);
    }
    auto issue_a = [&](long c, int which) __attribute__((always_inline)) {
        const unsigned buf = lds0 + (unsigned)which * ABUF;
#pragma unroll
        for (int x = 0; x < NDMA; ++x) {
            const int inst = wave + 4 * x, blk = inst >> 1;
            long s = c * CH + blk % CH;
            s = s < nsteps ? s : nsteps - 1;
            const uint32_t voff = a_row[x] + a_chunk - (s >= nfull ? a_back : 0);
            grouped_dma16(abase + s * 128, voff, buf + (unsigned)blk * 2048 + (unsigned)(inst & 1) * 1024);
        }
        if constexpr (Mo::MX) {
            if (wave == 3) {
#pragma unroll
                for (int h = 0; h < Mo::SB; ++h)
                    grouped_dma16(sabase + c * (CH * Mo::BPS) + 16 * h, sa_row,
                            lds0 + 2 * ABUF + (unsigned)which * SBUF + (unsigned)h * 1024);
            }
        }
    };
    const unsigned a_lo = 16 * (8 * j + (Mo::chunk_lo(q) ^ (j >> 1))), a_hi = 16 * (8 * j + (Mo::chunk_hi(q) ^ (j >> 1)));
    const bool lo_in = 16 * q + 16 <= tail, hi_in = 64 + 16 * q + 16 <= tail; // the lane's chunks in the tail step

    g4f acc[MF][NT];
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
        for (int jn = 0; jn < NT; ++jn) acc[i][jn] = g4f {0.f, 0.f, 0.f, 0.f};

    // chunks are walked from a place of K that differs between workgroups, wrapping around
    // (see grouped_walk); x counts chunks in walking order, p steps
    const long c0 = (long)((blockIdx.x * 5u + blockIdx.y * 3u) % (unsigned long)nchunks);
    auto chunk_at = [&](long x) {
        const long cr = x + c0;
        return cr >= nchunks ? cr - nchunks : cr;
    };
    auto step_at = [&](long p) {
        p = p < nchunks * CH ? p : nchunks * CH - 1;
        return chunk_at(p / CH) * CH + p % CH;
    };
    stage_t st[D];
    issue_a(chunk_at(0), 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int d = 0; d < D; ++d) st[d] = load_b(step_at(d));
    for (long x = 0; x < nchunks; ++x) {
        // memory operations return in order: once at most the D stages of weights issued
        // after this wavefront's part of the chunk are in flight, that part has landed
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(D * (NT * 2 + Mo::SB)) : "memory");
        __syncthreads();
        if (x + 1 < nchunks) issue_a(chunk_at(x + 1), (x + 1) & 1); // into the buffer whose readers passed the barrier
        __builtin_amdgcn_sched_barrier(0);
        const unsigned buf = lds0 + (unsigned)(x & 1) * ABUF;
        const long c = chunk_at(x);
#pragma unroll
        for (int t = 0; t < CH; ++t) {
            const long s = c * CH + t;
            if (s < nsteps) {
                g8i a[MF];
#pragma unroll
                for (int i = 0; i < MF; ++i) {
                    const unsigned blk = buf + (unsigned)(i * CH + t) * 2048;
                    const g4i lo = *(lds_g4i_ptr_t)(size_t)(blk + a_lo), hi = *(lds_g4i_ptr_t)(size_t)(blk + a_hi);
                    a[i] = g8i {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                }
                int sa[MF][2];
#pragma unroll
                for (int i = 0; i < MF; ++i)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        sa[i][h] = 0;
                        if constexpr (Mo::MX) {
                            if (h < Mo::SB) {
                                // row 16 i + j, the dword of this step's blocks (fp4: 0..3 and 4..7), byte q
                                const unsigned at = lds0 + 2 * ABUF + (unsigned)(x & 1) * SBUF + (unsigned)h * 1024
                                        + (unsigned)(16 * i + j) * 16 + (unsigned)((t * Mo::SB + h) % 4) * 4;
                                // fp4: steps 0, 1 sit in the first 16 bytes of the row, steps 2, 3 in the second
                                const unsigned at4 = lds0 + 2 * ABUF + (unsigned)(x & 1) * SBUF
                                        + (unsigned)((t * 2 + h) / 4) * 1024 + (unsigned)(16 * i + j) * 16
                                        + (unsigned)((t * 2 + h) % 4) * 4;
                                const int raw = *(const int __attribute__((address_space(3))) *)(size_t)(Mo::SB == 2 ? at4 : at);
                                sa[i][h] = (raw >> (8 * q)) & 0xff;
                            }
                        }
                    }
                const bool is_tail = s >= nfull;
                if (is_tail) {
#pragma unroll
                    for (int i = 0; i < MF; ++i)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            if (!lo_in) a[i][e] = 0;
                            if (!hi_in) a[i][4 + e] = 0;
                        }
                }
#pragma unroll
                for (int jn = 0; jn < NT; ++jn) {
                    g8i w = settle(st[t % D].b[jn]);
                    if (is_tail) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            if (!lo_in) w[e] = 0;
                            if (!hi_in) w[4 + e] = 0;
                        }
                    }
                    int sw[2] = {0, 0};
                    if constexpr (Mo::MX) SBs.pick(st[t % D].sb, jn, lane, sw);
#pragma unroll
                    for (int i = 0; i < MF; ++i) acc[i][jn] = grouped_mma<MODE, FA, FB>(w, a[i], acc[i][jn], sw, sa[i]);
                }
            }
            st[t % D] = load_b(step_at(x * CH + t + D));
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    __syncthreads(); // every wavefront is done with the src buffers
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
        for (int jn = 0; jn < NT; ++jn)
            *(lds_g4f_ptr_t)(size_t)(lds0 + (unsigned)((wave * MF * NT + i * NT + jn) * 64 + lane) * 16) = acc[i][jn];
}

template <int MODE, int FA, int FB, int MTMAX, int NT, int D>
__global__ void __launch_bounds__(256, 2) grouped_nsplit_kernel(const grouped_dev_t P) {
    constexpr int BM = 16 * MTMAX, BN = 64 * NT;
    extern __shared__ g4f part[]; // two src buffers of MTMAX * 8 KB; afterwards the accumulators
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)part;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    gtile_t T;
    if (!grouped_find_tile<BM, 4>(P, blockIdx.y, T)) return;
    T.n0 = (long)blockIdx.x * BN;
    const long here = T.rows - T.m_base < BM ? T.rows - T.m_base : BM;
    const int mf = __builtin_amdgcn_readfirstlane((int)((here + 15) / 16));
    // tiles of one or two fragments have registers left for four steps of weights in flight
    constexpr int D2 = D;
    switch (mf) {
        case 1: grouped_walk_nsplit<MODE, FA, FB, 1, NT, D2>(P, T, lds0, wave, lane); break;
        case 2:
            if constexpr (MTMAX >= 2) grouped_walk_nsplit<MODE, FA, FB, 2, NT, D2>(P, T, lds0, wave, lane);
            break;
        case 3:
            if constexpr (MTMAX >= 3) grouped_walk_nsplit<MODE, FA, FB, 3, NT, D>(P, T, lds0, wave, lane);
            break;
        default:
            if constexpr (MTMAX >= 4) grouped_walk_nsplit<MODE, FA, FB, 4, NT, D>(P, T, lds0, wave, lane);
            break;
    }
    // a wavefront finishes its own columns, one 16 x 16 unit at a time (one copy of the code)
    const int j = lane & 15, q = lane >> 4;
#pragma nounroll
    for (int u = 0; u < mf * NT; ++u) {
        const int i = u / NT, jn = u % NT;
        g4f sum = *(lds_g4f_ptr_t)(size_t)(lds0 + (unsigned)((wave * mf * NT + u) * 64 + lane) * 16);
        if constexpr (MODE == GM_I8) {
            const g4i isum = __builtin_bit_cast(g4i, sum);
            sum = g4f {(float)isum[0], (float)isum[1], (float)isum[2], (float)isum[3]};
        }
        grouped_store_quad(P, T, sum, T.m_base + 16 * i + j, T.n0 + 16 * NT * wave + 16 * jn + 4 * q);
    }
}

bool fp_plain(int dt) { return dt == MI355_DT_F32 || dt == MI355_DT_BF16 || dt == MI355_DT_F16; }
bool fp_any(int dt) {
    return fp_plain(dt) || dt == MI355_DT_F8_E4M3 || dt == MI355_DT_F8_E5M2 || dt == MI355_DT_F4_E2M1;
}

bool f8_dt(int dt) { return dt == MI355_DT_F8_E4M3 || dt == MI355_DT_F8_E5M2; }

// the tile shapes of the matrix-core kernel: rows (16 * MTMAX) x columns (16 * NT)
struct gshape_t {
    int bm, bn;
};
constexpr gshape_t GSHAPES[5] = {{0, 0}, {16, 32}, {48, 64}, {64, 256}, {48, 64}};

// 0: the thread-per-element kernel; 1: 16 x 32 tiles, K split between the
// wavefronts (groups of a row or two: many small workgroups); 2: 48 x 64, K
// split, two workgroups per compute unit; 3: 64 x 256, columns split, src rows
// through LDS; 4: 48 x 64 for row-major weights of the 16-bit types (a 16 x 64 shape with four steps in flight
// measured the same on groups of one row).  Decided on the descriptor.
// *mx_out: the plan is one of the MX modes (scales inside the instruction); every other plan has
// no groups along K (a group size of K counts as none) and applies its scales after the K sum.
int tile_plan(const mi355_grouped_desc_t &d, bool *mx_out = nullptr) {
    if (mx_out) *mx_out = false;
    if (d.pattern != MI355_GROUPED_2DX3D) return 0;
    const int force = tuning(TUNE_GROUPED_IMPL);
    if (force == TUNE_REF) return 0;
    const bool f8 = f8_dt(d.src_dt) && f8_dt(d.wei_dt);
    const bool f4 = d.src_dt == MI355_DT_F4_E2M1 && d.wei_dt == MI355_DT_F4_E2M1;
    const bool h16 = d.src_dt == d.wei_dt && (d.src_dt == MI355_DT_BF16 || d.src_dt == MI355_DT_F16);
    const bool i8 = d.src_dt == MI355_DT_S8 && d.wei_dt == MI355_DT_S8; // (u8 src would need the weights' column sums)
    if (!f8 && !h16 && !f4 && !i8) return 0;
    const long ebits = f4 ? 4 : (f8 ? 8 : 16);
    auto bytes = [&](long elems) { return elems * ebits / 8; };
    auto k_groups = [&](int dt, long gk) { return dt != MI355_DT_UNDEF && gk > 1 && gk != d.K; };
    const long active = d.group_count < d.total ? d.group_count : d.total;
    if (h16 && d.wei_stride[2] == 1 && d.wei_stride[1] >= d.N && !(d.wei_stride[1] == 1 && d.wei_stride[2] >= d.K)) {
        // row-major weights: a lane reads 8 bytes of a k row (four columns), 16 of a src row
        if (d.N % 4 != 0 || d.wei_stride[1] % 4 != 0 || d.wei_stride[0] % 4 != 0 || d.K % 16 != 0) return 0;
        if (d.src_zp_dt != MI355_DT_UNDEF || d.wei_zp_dt != MI355_DT_UNDEF) return 0;
        if (k_groups(d.src_scale_dt, d.src_scale_gk) || k_groups(d.wei_scale_dt, d.wei_scale_gk)) return 0;
        if (2 * d.K * GSHAPES[4].bm >= (1L << 32)) return 0; // 32-bit offsets of the src rows inside a tile
        if (d.total / GSHAPES[4].bm + active > 65535) return 0;
        return 4;
    }
    if (d.wei_stride[1] != 1 || d.wei_stride[2] < d.K) return 0; // otherwise K-contiguous weights only
    if (bytes(d.wei_stride[2]) % 16 != 0 || bytes(d.wei_stride[0]) % 16 != 0 || bytes(d.K) % 32 != 0 || d.K % 2 != 0) return 0;
    if (bytes(d.wei_stride[2]) > (1L << 24)) return 0; // 32-bit offsets inside a tile
    if (d.src_zp_dt != MI355_DT_UNDEF || d.wei_zp_dt != MI355_DT_UNDEF) return 0;
    const bool sg = k_groups(d.src_scale_dt, d.src_scale_gk), wg = k_groups(d.wei_scale_dt, d.wei_scale_gk);
    // MX: e8m0 scales per 32 k on both operands of fp8 / fp4 tensors, applied by the instruction; whole
    // 512-byte chunks of K (16 or 32 scale bytes a row), dword loads of the weights' scales along N
    const bool mx = sg && wg && (f8 || f4) && d.src_scale_dt == MI355_DT_E8M0 && d.wei_scale_dt == MI355_DT_E8M0
            && d.src_scale_gk == 32 && d.wei_scale_gk == 32 && bytes(d.K) % 512 == 0 && d.N % 4 == 0;
    if ((sg || wg) && !mx) return 0;
    if (f4 && !mx) return 0;
    // Groups of a row or two: the small tiles.  Otherwise the 256-column tiles (a quarter of
    // the src traffic per byte of weights), unless they are too few to fill the device or
    // the rows are not whole lines (K not a multiple of 128 bytes: measured slower there).
    int plan = 3;
    if (d.total <= 2 * d.group_count) plan = 1;
    else if (bytes(d.K) % 128 != 0 || (d.N + 255) / 256 * active < 256) plan = 2;
    if (force == TUNE_SHORT) plan = 1;
    if (force == TUNE_TALL) plan = 2;
    if (force == TUNE_WIDE) plan = 3;
    if (d.total / GSHAPES[plan].bm + active > 65535) return 0;
    if (mx_out) *mx_out = mx;
    return plan;
}

// The variable-K pattern on the matrix cores: 0 = no, 1 = dst rows are rows of src ("abc"), 2 = dst rows are
// columns of the weights ("acb": the operands change places).
int k_tile_plan(const mi355_grouped_desc_t &d) {
    if (d.pattern != MI355_GROUPED_2DX2D) return 0;
    if (tuning(TUNE_GROUPED_IMPL) == TUNE_REF) return 0;
    if (d.src_dt != MI355_DT_F32 && d.src_dt != MI355_DT_BF16 && d.src_dt != MI355_DT_F16) return 0;
    // a lane reads four consecutive rows (columns) and stores four consecutive dst elements
    if (d.M % 4 != 0 || d.N % 4 != 0 || d.dst_stride[0] % 4 != 0) return 0;
    if (d.group_count > 65535) return 0;
    if (((d.M + 127) / 128) * ((d.N + 127) / 128) >= (1L << 31)) return 0;
    if (d.dst_stride[2] == 1 && d.dst_stride[1] >= d.N && d.dst_stride[1] % 4 == 0) return 1;
    if (d.dst_stride[1] == 1 && d.dst_stride[2] >= d.M && d.dst_stride[2] % 4 == 0) return 2;
    return 0;
}

int launch_k_tiles(int plan, const grouped_dev_t &G, hipStream_t stream) {
    const mi355_grouped_desc_t &d = G.d;
    grouped_k_dev_t P;
    const bool swap = plan == 2;
    P.a = swap ? G.a.wei : G.a.src;
    P.b = swap ? G.a.src : G.a.wei;
    P.MA = swap ? d.N : d.M;
    P.NB = swap ? d.M : d.N;
    P.offsets = G.a.src_offsets;
    P.dst = G.a.dst;
    P.total = d.total;
    P.dst_g = d.dst_stride[0];
    P.dst_ld = swap ? d.dst_stride[2] : d.dst_stride[1];
    P.tiles_n = (int)((P.NB + 127) / 128);
    P.run = 1;
    const long tiles_m = (P.MA + 127) / 128;
    dim3 grid((unsigned)(tiles_m * P.tiles_n), (unsigned)d.group_count);
    // bf16 / f16 through LDS and the 16-bit instructions (measured faster at every group length) where columns
    // can be fetched eight at a time and 32-bit offsets reach across a group; otherwise the f32 instruction
    const bool h16 = d.src_dt != MI355_DT_F32;
    bool lds_path = h16 && P.MA % 8 == 0 && P.NB % 8 == 0 && d.total * (P.MA > P.NB ? P.MA : P.NB) * 2 < (1L << 32);
    if (tuning(TUNE_GROUPED_IMPL) == TUNE_SHORT) lds_path = false;
    if (lds_path) {
        const bool brief = d.total <= 48 * d.group_count; // (k per group on average)
        // runs of up to 8 column tiles a workgroup, while some thousands of workgroups remain
        const long tiles = tiles_m * P.tiles_n * d.group_count;
        while (P.run < 8 && P.run * 2 <= P.tiles_n && tiles / (P.run * 2) >= 3072) P.run *= 2;
        // (the tuning switch: "tall" a tile a workgroup, "wide" runs of 8 whatever the size)
        if (tuning(TUNE_GROUPED_IMPL) == TUNE_TALL) P.run = 1;
        if (tuning(TUNE_GROUPED_IMPL) == TUNE_WIDE) P.run = P.tiles_n < 8 ? P.tiles_n : 8;
        grid.x = (unsigned)(tiles_m * ((P.tiles_n + P.run - 1) / P.run));
        auto launch = [&](auto kern, int nst) {
            const int lds = nst * GK_STAGE;
            if (const int st = ensure_dynamic_lds((const void *)kern, lds, "mfma_grouped_k")) return st;
            hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, P);
            return hipGetLastError() == hipSuccess ? (int)MI355_SUCCESS : (int)MI355_RUNTIME_ERROR;
        };
        if (d.src_dt == MI355_DT_BF16)
            return brief ? launch(grouped_k_lds_kernel<MI355_DT_BF16, 2>, 2) : launch(grouped_k_lds_kernel<MI355_DT_BF16, 4>, 4);
        return brief ? launch(grouped_k_lds_kernel<MI355_DT_F16, 2>, 2) : launch(grouped_k_lds_kernel<MI355_DT_F16, 4>, 4);
    }
    if (d.src_dt == MI355_DT_F32)
        hipLaunchKernelGGL(grouped_k_tile_kernel<MI355_DT_F32>, grid, dim3(256), 0, stream, P);
    else if (d.src_dt == MI355_DT_BF16)
        hipLaunchKernelGGL(grouped_k_tile_kernel<MI355_DT_BF16>, grid, dim3(256), 0, stream, P);
    else
        hipLaunchKernelGGL(grouped_k_tile_kernel<MI355_DT_F16>, grid, dim3(256), 0, stream, P);
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
}

template <int MODE, int FA, int FB>
int launch_tiles(int plan, const grouped_dev_t &P, hipStream_t stream) {
    const mi355_grouped_desc_t &d = P.d;
    const long active = d.group_count < d.total ? d.group_count : d.total;
    const gshape_t sh = GSHAPES[plan];
    dim3 grid((unsigned)((d.N + sh.bn - 1) / sh.bn), (unsigned)(d.total / sh.bm + active));
    auto go = [&](auto kern, int mtmax, int nt, int nw) -> int {
        const int lds = nw * mtmax * nt * 64 * 16;
        if (const int st = ensure_dynamic_lds((const void *)kern, lds, "mfma_grouped")) return st;
        hipLaunchKernelGGL(kern, grid, dim3(64 * nw), lds, stream, P);
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
    };
    if (plan == 4) {
        if constexpr (MODE == GM_BF16 || MODE == GM_F16) return go(grouped_tile_kernel<MODE, 0, 0, 3, 4, 2, 4, 2, true>, 3, 4, 4);
        return MI355_RUNTIME_ERROR;
    }
    if (plan == 1) return go(grouped_tile_kernel<MODE, FA, FB, 1, 2, 4, 4, 1>, 1, 2, 4);
    // (the MX modes hold their scales too and do not fit two workgroups' registers)
    if (plan == 2) return go(grouped_tile_kernel<MODE, FA, FB, 3, 4, 2, 4, gmode_t<MODE>::MX ? 1 : 2>, 3, 4, 4);
    // two src buffers of 4 fragments x 4 steps (the accumulators fit the same space) + the MX scales of two chunks
    {
        auto kern = grouped_nsplit_kernel<MODE, FA, FB, 4, 4, 2>;
        const int lds = 2 * 4 * 4 * 2048 + 2 * gmode_t<MODE>::SB * 1024;
        if (const int st = ensure_dynamic_lds((const void *)kern, lds, "mfma_grouped")) return st;
        hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, P);
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
    }
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

extern "C" const char *mi355_grouped_matmul_impl(const mi355_grouped_desc_t *d) {
    if (!d || mi355_grouped_matmul_query(d) != MI355_SUCCESS) return "";
    if (k_tile_plan(*d) != 0) return "hip:mfma_grouped_k";
    return tile_plan(*d) != 0 ? "hip:mfma_grouped" : "hip:ref_grouped:any";
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
    // the tiles read 16 bytes at a time
    const bool aligned = (uintptr_t)a->src % 16 == 0 && (uintptr_t)a->wei % 16 == 0
            && (d->src_scale_gk <= 1 || ((uintptr_t)a->src_scale % 16 == 0 && (uintptr_t)a->wei_scale % 4 == 0));
    bool mx = false;
    const int plan = aligned ? tile_plan(*d, &mx) : 0;
    if (plan != 0) {
        hipStream_t s = (hipStream_t)stream;
        const int fa = d->src_dt == MI355_DT_F8_E5M2, fb = d->wei_dt == MI355_DT_F8_E5M2;
        if (d->src_dt == MI355_DT_BF16) return launch_tiles<GM_BF16, 0, 0>(plan, P, s);
        if (d->src_dt == MI355_DT_F16) return launch_tiles<GM_F16, 0, 0>(plan, P, s);
        if (d->src_dt == MI355_DT_F4_E2M1) return launch_tiles<GM_MXF4, 0, 0>(plan, P, s);
        if (d->src_dt == MI355_DT_S8) return launch_tiles<GM_I8, 0, 0>(plan, P, s);
        if (mx) {
            if (!fa && !fb) return launch_tiles<GM_MXF8, 0, 0>(plan, P, s);
            if (fa && fb) return launch_tiles<GM_MXF8, 1, 1>(plan, P, s);
            if (fa) return launch_tiles<GM_MXF8, 1, 0>(plan, P, s);
            return launch_tiles<GM_MXF8, 0, 1>(plan, P, s);
        }
        if (!fa && !fb) return launch_tiles<GM_F8, 0, 0>(plan, P, s);
        if (fa && fb) return launch_tiles<GM_F8, 1, 1>(plan, P, s);
        if (fa) return launch_tiles<GM_F8, 1, 0>(plan, P, s);
        return launch_tiles<GM_F8, 0, 1>(plan, P, s);
    }
    if (const int kplan = k_tile_plan(*d)) {
        // (the tiles read and write 16 bytes at a time)
        if ((uintptr_t)a->src % 16 == 0 && (uintptr_t)a->wei % 16 == 0 && (uintptr_t)a->dst % 16 == 0)
            return launch_k_tiles(kplan, P, (hipStream_t)stream);
    }
    if (x3)
        hipLaunchKernelGGL(grouped_2dx3d_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, P);
    else
        hipLaunchKernelGGL(grouped_2dx2d_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, P);
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
}
