// "hip:mfma_i8" -- LDS-tiled int8 GEMM on the gfx950 matrix cores
// (v_mfma_i32_16x16x64_i8) with the zero-point compensation folded into an
// s32 row/column-sum correction and the reference's epilogue fused in.
//
// Replaces, for integer src and weights, the reference's brgemm int8 path
// (src/cpu/x64/matmul/brgemm_matmul.cpp:658-1027: copy_B with s8s8/zp
// compensation + AMX/VNNI microkernel + jit_brgemm_post_ops) and computes the
// same values as ref_matmul_int8_t (src/cpu/matmul/ref_matmul_int8.cpp:174-306)
// when there is a single group along K:
//   acc[m,n] = sum_k (src[m,k] - zs) * (wei[k,n] - zw[n])          (s32)
//            = sum_k s'w' + a*colsum'[n] + c[n]*rowsum'[m] + K*a*c[n]
//     with s' = src - off_s, w' = wei - off_w the bytes re-biased to s8
//     (off = 128 for u8, 0 for s8), a = off_s - zs, c[n] = off_w - zw[n];
//   d = (float)acc * src_scale * wei_scale[n]  -> shared epilogue.
#include "gemm_core.hpp"

#include <cstdlib>
#include <cstring>

namespace mi355 {

namespace {

using namespace gemm;
// 1: the loop that reads a stage ahead instead of the two-group loop.  Both pass the parity tests and measured the
// same on the 8192^3 configuration (0.4560 against 0.4566 ms, same box): the kernel's time is set by the energy of
// its data movement, not by how the wavefronts take turns.
#ifndef MI355_I8_AHEAD
#define MI355_I8_AHEAD 0
#endif
constexpr int BK = BKB;       // int8: one byte per K element
using i8_geo_t = geo_t<8, 256>;
constexpr int NSTAGE = i8_geo_t::NSTAGE;

struct i8_extra_t {
    const int8_t *bt; // weights as [N][K] bytes, K contiguous
    long ldb;         // bytes between consecutive n
    long bt_bstride;  // bytes between batches (0 = broadcast)
    const int *colsum; // [Bw][N] sum_k w'  (null when a == 0)
    const int *rowsum; // [Bs][M] sum_k s'  (null when c == 0)
    int tiles_m, tiles_n;
};

struct i8_ctx_t {};

// v_mfma_i32_16x16x64_i8: lane l supplies row l%16, K bytes 16*(l/16)..+16, so
// one instruction consumes the whole 64-byte K extent of a stage for a 16x16
// tile.  (Measured on MI355X: this shape sustains ~4.0 POPS, the 32x32x32
// shape ~3.0 POPS.)
template <bool SRC_U8, bool WEI_U8, class G_>
struct i8_mma_t {
    using G = G_;
    static constexpr int EXTRA_DMAS = 0;
    __device__ static __forceinline__ void issue_extra(const i8_ctx_t &, int, int, int, int) {}
    static constexpr int ROWS = 8, COLS = G::WCOLS / 16, A_READS = 1, B_READS = 1;
    struct frag_t {
        v4i a[ROWS], b[COLS];
    };
    // fragments whose products are zero: a u8 operand is re-biased by 128 where
    // it is used, so its zero is the byte 0x80
    __device__ static __forceinline__ frag_t zero_frag() {
        frag_t f;
        const int za = SRC_U8 ? (int)0x80808080 : 0, zb = WEI_U8 ? (int)0x80808080 : 0;
#pragma unroll
        for (int i = 0; i < ROWS; ++i) f.a[i] = v4i {za, za, za, za};
#pragma unroll
        for (int j = 0; j < COLS; ++j) f.b[j] = v4i {zb, zb, zb, zb};
        return f;
    }
    // Per-lane LDS offsets of fragment 0 of both operands.  Fragment i is 16 rows
    // further: the swizzle depends on the row modulo 16 only, so it is the same
    // address plus i KB, which goes into the offset field of the read.
    struct addr_t {
        unsigned a, b;
    };
    __device__ static __forceinline__ addr_t lane_addr(int wm, int wn, int lane) {
        const int frow = lane & 15, fch = lane >> 4;
        return addr_t {(unsigned)swz(wm * 128 + frow, fch), (unsigned)(B_OFF + swz(wn * G::WCOLS + frow, fch))};
    }
    __device__ static __forceinline__ void load_b(frag_t &f, const unsigned (&S)[1], const addr_t &ad,
            const i8_ctx_t &, int) {
#pragma unroll
        for (int j = 0; j < COLS; ++j) f.b[j] = lds_read16(S[0] + ad.b + j * 1024);
    }
    __device__ static __forceinline__ void load_a(frag_t &f, int i, const unsigned (&S)[1], const addr_t &ad,
            const i8_ctx_t &, int) {
        f.a[i] = lds_read16(S[0] + ad.a + i * 1024);
    }
    // The loop that reads a stage ahead (gemm_core.hpp): a u8 operand is
    // re-biased in place when its stage's turn comes, and the instruction is
    // written out with the accumulator tied to one operand -- left to itself the
    // compiler accumulates out of place in a loop that alternates between two
    // fragment sets and then copies accumulators around in every iteration.  (No
    // wait states are owed inside the loop: an accumulator is next touched 31
    // instructions later, and a VALU result may feed the following MFMA.)
    static constexpr bool READS_AHEAD = MI355_I8_AHEAD && G::NSTAGE >= 4;
    __device__ static __forceinline__ void load_b_one(frag_t &f, int j, const unsigned (&S)[1], const addr_t &ad,
            const i8_ctx_t &, int) {
        f.b[j] = lds_read16(S[0] + ad.b + j * 1024);
    }
    __device__ static __forceinline__ void prepare(frag_t &f) {
        if (SRC_U8) {
#pragma unroll
            for (int i = 0; i < ROWS; ++i) f.a[i] ^= (int)0x80808080;
        }
        if (WEI_U8) {
#pragma unroll
            for (int j = 0; j < COLS; ++j) f.b[j] ^= (int)0x80808080;
        }
    }
    __device__ static __forceinline__ void mma_row(v4i (&acc)[ROWS][COLS], const frag_t &f, int i,
            const i8_ctx_t &, int) {
        if constexpr (READS_AHEAD) {
#pragma unroll
            for (int j = 0; j < COLS; ++j)
                asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(acc[i][j]) : "v"(f.b[j]), "v"(f.a[i]));
        } else {
            const v4i a = SRC_U8 ? (f.a[i] ^ (int)0x80808080) : f.a[i];
#pragma unroll
            for (int j = 0; j < COLS; ++j) {
                const v4i b = WEI_U8 ? (f.b[j] ^ (int)0x80808080) : f.b[j];
                // operands exchanged: the tile comes out transposed, a lane holds four
                // consecutive n of one row (tile_epilogue.hpp)
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b, a, acc[i][j], 0, 0, 0);
            }
        }
    }
};

// raw s32 accumulator -> f32 entering the shared epilogue
struct i8_conv_t {
    typedef int row_t;
    float ssc;
    bool with_src_sc, with_wei_sc, has_comp;
    const int *rowsum; // already offset to this batch, or null
    const int *colsum; // already offset to this batch, or null
    int a_c, off_w, Kc;
    long bw;
    // the per-column operands of the table: weights scale, a * colsum'[n] + K a c[n], c[n]
    template <class PT>
    __device__ __forceinline__ void per_n(const PT &P, long, long n, float &wsc, int &cc, int &c) const {
        c = off_w;
        if (P.wei_zp.dt != MI355_DT_UNDEF)
            c -= load_int(P.wei_zp.dt, P.wei_zp.p, quant_off(P.wei_zp, bw, 0, n, P.K, P.N));
        cc = (a_c != 0 ? a_c * colsum[n] : 0) + Kc * a_c * c;
        if (with_wei_sc)
            wsc = load_float(P.wei_scale.dt, P.wei_scale.p, quant_off(P.wei_scale, bw, 0, n, P.K, P.N));
    }
    __device__ __forceinline__ int row_data(long m) const { return rowsum ? rowsum[m] : 0; }

    // The chain of the compute-bound int8 configuration and its neighbours, fully
    // unrolled over the wavefront's 8 x 4 accumulator tiles with every choice a
    // template parameter:
    //   f32(acc) * src_scale * wei_scale[n]  [-> max(., 0)]  [-> / dst_scale]  -> s8 / u8
    // (no compensation terms, no bias, no zero points).  Per element: convert, two
    // multiplications, maximum, five operations of the fma-corrected division,
    // round, convert, clamp, 3/4 of a byte permute.
    template <bool RELU, int DS, class PT>
    __device__ __forceinline__ void hot_store(const PT &P, const epi_uniform_t &H, unsigned ntab,
            const v4i (&acc)[8][4], long b, long m_base, long n_base, int col0) const {
        const int lane = threadIdx.x & 63, lrow = lane & 15, cq = 4 * (lane >> 4);
        v4f_t w[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) w[k] = nt4f(ntab, NT_WSC, col0 + 16 * k + cq);
        const int lo = H.dst_dt == MI355_DT_S8 ? -128 : 0, hi = H.dst_dt == MI355_DT_S8 ? 127 : 255;
        uint8_t *dcol = (uint8_t *)P.dst + b * P.ds[0] + n_base + cq;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const long m = m_base + 16 * i + lrow;
            float x[4][4];
            unsigned mx = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float t = (float)acc[i][k][e] * ssc;
                    t *= w[k][e];
                    if (RELU) t = fmaxf(t, 0.f); // an integer dst turns NaN and -0 into 0 either way
                    if (DS == 2) t *= H.ds_inv;
                    if (DS == 3) mx = max(mx, mag_bits(t));
                    x[k][e] = t;
                }
            if (DS == 3) {
                if (__builtin_amdgcn_ballot_w64(mx >= DIV_BY_FMA_LIMIT) == 0) {
#pragma unroll
                    for (int k = 0; k < 4; ++k)
#pragma unroll
                        for (int e = 0; e < 4; ++e) x[k][e] = div_by_fma(x[k][e], H.ds, H.ds_inv);
                } else {
#pragma unroll
                    for (int k = 0; k < 4; ++k)
#pragma unroll
                        for (int e = 0; e < 4; ++e) x[k][e] /= H.ds;
                }
            }
            unsigned word[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) word[k] = pack4_i8(x[k], lo, hi);
            if (m < P.M) {
                uint8_t *d = dcol + m * P.ds[1];
#pragma unroll
                for (int k = 0; k < 4; ++k) *(uint32_t *)(d + 16 * k) = word[k];
            }
        }
    }
    template <class PT>
    __device__ __forceinline__ bool hot_chain(const PT &P, const epi_uniform_t &H, unsigned ntab, unsigned,
            const v4i (&acc)[8][4], long b, long m_base, long n_base, int col0) const {
        const bool relu0 = H.n_po == 1 && H.pf0.kind == MI355_PO_ELTWISE && H.pf0.alg == MI355_ELTWISE_RELU
                && H.pf0.alpha == 0.f && H.pf0.scale == 1.f;
        if (has_comp || !with_src_sc || !with_wei_sc || H.bias_mode != 0 || H.dzp_mode != 0 || H.dynamic
                || (H.n_po != 0 && !relu0) || H.ds_mode == 1 || (H.dst_dt != MI355_DT_S8 && H.dst_dt != MI355_DT_U8))
            return false;
        if (relu0) {
            if (H.ds_mode == 0) hot_store<true, 0>(P, H, ntab, acc, b, m_base, n_base, col0);
            else if (H.ds_mode == 2) hot_store<true, 2>(P, H, ntab, acc, b, m_base, n_base, col0);
            else hot_store<true, 3>(P, H, ntab, acc, b, m_base, n_base, col0);
        } else {
            if (H.ds_mode == 0) hot_store<false, 0>(P, H, ntab, acc, b, m_base, n_base, col0);
            else if (H.ds_mode == 2) hot_store<false, 2>(P, H, ntab, acc, b, m_base, n_base, col0);
            else hot_store<false, 3>(P, H, ntab, acc, b, m_base, n_base, col0);
        }
        return true;
    }
    __device__ __forceinline__ void quad(const v4i_t &raw, int rs, unsigned ntab, int col, float (&f)[4]) const {
        int v[4] = {raw[0], raw[1], raw[2], raw[3]};
        if (has_comp) {
            const v4i_t cc = nt4i(ntab, NT_CC, col), c = nt4i(ntab, NT_C, col);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += cc[e] + c[e] * rs;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) f[e] = (float)v[e];
        if (with_src_sc) {
#pragma unroll
            for (int e = 0; e < 4; ++e) f[e] *= ssc;
        }
        if (with_wei_sc) {
            const v4f_t w = nt4f(ntab, NT_WSC, col);
#pragma unroll
            for (int e = 0; e < 4; ++e) f[e] *= w[e];
        }
    }
};

extern __shared__ __attribute__((aligned(16))) char i8_smem[];

template <bool SRC_U8, bool WEI_U8, class G>
__global__ void __launch_bounds__(G::NT) __attribute__((amdgpu_waves_per_eu(G::NW * G::WG_PER_CU / 4))) i8_gemm_kernel(const problem_t P_, const i8_extra_t X) {
    using Mma = i8_mma_t<SRC_U8, WEI_U8, G>;
    const auto &P = MI355_KERNARG_PROBLEM();
    char *smem = i8_smem;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = G::wm(wave), wn = G::wn(wave);
    const long b = blockIdx.z;
    const tile_pos_t tp = tile_position<G>((int)blockIdx.x, X.tiles_m, X.tiles_n);
    const long m0 = tp.m0, n0 = tp.n0;

    const long lda = P.ss[1];
    const char *A = (const char *)P.src + (P.ss[0] ? b * P.ss[0] : 0) + m0 * lda;
    const char *Bt = (const char *)X.bt + b * X.bt_bstride + n0 * X.ldb;

    // ---- the epilogue's per-column operands go into their LDS table now: the
    // loads hide behind the pipeline prologue
    const long bs = P.ss[0] ? b : 0, bw = P.ws[0] ? b : 0;
    const int off_s = SRC_U8 ? 128 : 0, off_w = WEI_U8 ? 128 : 0;
    i8_conv_t cv;
    cv.a_c = off_s;
    if (P.src_zp.dt != MI355_DT_UNDEF) cv.a_c -= load_int(P.src_zp.dt, P.src_zp.p, 0);
    cv.off_w = off_w;
    cv.Kc = (int)P.K;
    cv.bw = bw;
    cv.with_src_sc = P.src_scale.dt != MI355_DT_UNDEF;
    cv.with_wei_sc = P.wei_scale.dt != MI355_DT_UNDEF;
    cv.ssc = cv.with_src_sc ? load_float(P.src_scale.dt, P.src_scale.p, 0) : 1.f;
    cv.rowsum = X.rowsum ? X.rowsum + bs * P.M : nullptr;
    cv.colsum = X.colsum ? X.colsum + bw * P.N : nullptr;
    cv.has_comp = X.rowsum != nullptr || X.colsum != nullptr || cv.a_c != 0 || WEI_U8 || P.wei_zp.dt != MI355_DT_UNDEF;
    const unsigned ntab = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem + G::NSTAGE * G::STAGE_BYTES;
    fill_ntab<G::NT>(P, cv, ntab, b, n0);

    v4i acc[Mma::ROWS][Mma::COLS];
#pragma unroll
    for (int i = 0; i < Mma::ROWS; ++i)
#pragma unroll
        for (int j = 0; j < Mma::COLS; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0;

    main_loop<G::NSTAGE, 1, Mma>(acc, smem, A, Bt, lda, X.ldb, P.M - m0, P.N - n0,
            (int)(P.K / BK), i8_ctx_t {});

    store_quadrant<layout16_t, G::WCOLS>(P, smem, ntab, acc, b, m0 + wm * 128, n0 + wn * G::WCOLS, wn * G::WCOLS, cv);
}


// ---- few tiles or a K that is not a multiple of the stage: 32 x 32 dst tiles
// without LDS staging.  The 256 x 256 tiles above leave the device idle when
// M x N holds only a handful of them (4 workgroups for 256 x 1024), and their
// stage loads want K in units of 64.  Here a workgroup of four wavefronts owns a
// 32 x 32 tile, the wavefronts take every fourth 64-byte step of K, each lane
// loads its MFMA operands (16 bytes of a src row, 16 bytes of a weights
// column, K contiguous in both) straight from memory, four steps ahead of the
// matrix cores, and a step beyond K's last 16 bytes is filled with the
// operand's zero.  The column sums of the weights and the row sums of src that
// the zero-point correction needs come out of two more MFMAs per operand tile
// against all-ones bytes, in the accumulators' own lane layout: no pre-pass
// kernels.  The four wavefronts' sums are added through LDS in wavefront order
// (integer: exact in any order), converted like the large tiles' and finished
// by the general epilogue.
constexpr int ST = 32;     // rows and columns of a small tile
constexpr int SNW = 4;     // wavefronts of its workgroup

template <bool SRC_U8, bool WEI_U8>
__global__ void __launch_bounds__(SNW * 64) i8_small_kernel(const problem_t P_, const i8_extra_t X) {
    // [wavefront][slot][lane]; slots: 16 accumulators, 8 column sums, 8 row sums
    __shared__ int part[SNW][32][64];
    const auto &P = MI355_KERNARG_PROBLEM();
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int j = lane & 15, q = lane >> 4;
    const long b = blockIdx.z;
    const long m0 = (long)(blockIdx.x / X.tiles_n) * ST, n0 = (long)(blockIdx.x % X.tiles_n) * ST;
    const long M = P.M, N = P.N, K = P.K;
    const long lda = P.ss[1];
    const char *A = (const char *)P.src + (P.ss[0] ? b * P.ss[0] : 0);
    const char *Bt = (const char *)X.bt + b * X.bt_bstride;
    // rows and columns beyond the edge read the last valid one (never stored)
    const char *arow[2], *bcol[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const long m = m0 + 16 * i + j < M ? m0 + 16 * i + j : M - 1;
        const long n = n0 + 16 * i + j < N ? n0 + 16 * i + j : N - 1;
        arow[i] = A + m * lda + 16 * q;
        bcol[i] = Bt + n * X.ldb + 16 * q;
    }
    const int a_fill = SRC_U8 ? (int)0x80808080 : 0, b_fill = WEI_U8 ? (int)0x80808080 : 0;
    struct frag_t {
        v4i a[2], b[2];
    };
    // K is a multiple of 16: a lane's 16 bytes are inside K or beyond it
    auto load = [&](long step) __attribute__((always_inline)) {
        frag_t f;
        const long k = step * 64;
        const bool in = k + 16 * q < K;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            f.a[i] = v4i {a_fill, a_fill, a_fill, a_fill};
            f.b[i] = v4i {b_fill, b_fill, b_fill, b_fill};
            if (in) {
                f.a[i] = *(const v4i *)(arow[i] + k);
                f.b[i] = *(const v4i *)(bcol[i] + k);
            }
        }
        return f;
    };
    v4i acc[2][2], cs[2], rs[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        cs[i] = rs[i] = v4i {0, 0, 0, 0};
#pragma unroll
        for (int jn = 0; jn < 2; ++jn) acc[i][jn] = v4i {0, 0, 0, 0};
    }
    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
    const long nsteps = (K + 63) / 64;
    // SD of the wavefront's steps are in flight: a launch of a few hundred tiles lasts a handful of memory
    // latencies, and with one step ahead every step of a wavefront cost one of them
    constexpr int SD = 4;
    auto multiply = [&](const frag_t &cur) __attribute__((always_inline)) {
        v4i a[2], w[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            a[i] = SRC_U8 ? (cur.a[i] ^ (int)0x80808080) : cur.a[i];
            w[i] = WEI_U8 ? (cur.b[i] ^ (int)0x80808080) : cur.b[i];
        }
        // operands exchanged as in the large tiles: a lane holds four
        // consecutive n (4 * (lane / 16) + e) of row lane % 16
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int jn = 0; jn < 2; ++jn)
                acc[i][jn] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[jn], a[i], acc[i][jn], 0, 0, 0);
            cs[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[i], ones, cs[i], 0, 0, 0); // [e]: column 4 * (lane / 16) + e
            rs[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, a[i], rs[i], 0, 0, 0); // every e: row lane % 16
        }
    };
    long step = wave;
    frag_t st[SD];
#pragma unroll
    for (int d = 0; d < SD; ++d) {
        const long sl = step + (long)d * SNW;
        st[d] = load(sl < nsteps ? sl : 0);
    }
    for (; step + (long)(SD - 1) * SNW < nsteps; step += (long)SD * SNW) {
#pragma unroll
        for (int d = 0; d < SD; ++d) {
            multiply(st[d]);
            const long sl = step + (long)(SD + d) * SNW;
            if (sl < nsteps) st[d] = load(sl); // (uniform over the wavefront)
        }
    }
#pragma unroll
    for (int d = 0; d < SD; ++d)
        if (step + (long)d * SNW < nsteps) multiply(st[d]);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
#pragma unroll
            for (int jn = 0; jn < 2; ++jn) part[wave][i * 8 + jn * 4 + e][lane] = acc[i][jn][e];
            part[wave][16 + i * 4 + e][lane] = cs[i][e];
            part[wave][24 + i * 4 + e][lane] = rs[i][e];
        }
    }
    __syncthreads();
    // thread (unit = i, jn; lane): the quad of row m0 + 16 i + lane % 16,
    // columns n0 + 16 jn + 4 (lane / 16) ..
    const int unit = t >> 6, ui = unit >> 1, ujn = unit & 1;
    int sum[4] = {0, 0, 0, 0}, csum[4] = {0, 0, 0, 0}, rsum = 0;
#pragma unroll
    for (int wv = 0; wv < SNW; ++wv) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            sum[e] += part[wv][ui * 8 + ujn * 4 + e][lane];
            csum[e] += part[wv][16 + ujn * 4 + e][lane];
        }
        rsum += part[wv][24 + ui * 4][lane];
    }
    const long m = m0 + 16 * ui + j, nbase = n0 + 16 * ujn + 4 * q;
    if (m >= M || nbase >= N) return;
    const int nvalid = N - nbase < 4 ? (int)(N - nbase) : 4;
    const long bw = P.ws[0] ? b : 0;
    int a_c = SRC_U8 ? 128 : 0;
    if (P.src_zp.dt != MI355_DT_UNDEF) a_c -= load_int(P.src_zp.dt, P.src_zp.p, 0);
    const bool with_src_sc = P.src_scale.dt != MI355_DT_UNDEF, with_wei_sc = P.wei_scale.dt != MI355_DT_UNDEF;
    const float ssc = with_src_sc ? load_float(P.src_scale.dt, P.src_scale.p, 0) : 1.f;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if (e < nvalid) {
            const long n = nbase + e;
            int c = WEI_U8 ? 128 : 0;
            if (P.wei_zp.dt != MI355_DT_UNDEF)
                c -= load_int(P.wei_zp.dt, P.wei_zp.p, quant_off(P.wei_zp, bw, 0, n, P.K, P.N));
            // the large tiles' order: a * colsum + K * a * c, then + c * rowsum
            const int cc = a_c * csum[e] + (int)K * a_c * c;
            float f = (float)(sum[e] + (cc + c * rsum));
            if (with_src_sc) f *= ssc;
            if (with_wei_sc)
                f *= load_float(P.wei_scale.dt, P.wei_scale.p, quant_off(P.wei_scale, bw, 0, n, P.K, P.N));
            v[e] = f;
        }
    }
    apply_epilogue4(P, v, b, m, nbase, nvalid);
    store4(P, P.ds[2] == 1 && vec_ok_store(P.dst, P.ds[0], P.ds[1], dt_bits(P.dst_dt)), v, b, m, nbase, nvalid);
}

// out[r] = sum_k (bytes[r][k] ^ flip) as signed bytes; one wave per row
__global__ void __launch_bounds__(256) i8_rowsum_kernel(const int8_t *p, long rows, long K,
        long ld, int flip, int *out) {
    const long r = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const int lane = threadIdx.x & 63;
    const int8_t *row = p + r * ld;
    int s = 0;
    const long k16 = K / 16 * 16;
    for (long k = lane * 16; k < k16; k += 64 * 16) {
        v4i v = *(const v4i *)(row + k);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int w = v[i] ^ flip;
            s += (int)(int8_t)(w & 0xff) + (int)(int8_t)((w >> 8) & 0xff)
                    + (int)(int8_t)((w >> 16) & 0xff) + (w >> 24);
        }
    }
    for (long k = k16 + lane; k < K; k += 64) s += (int)(int8_t)(row[k] ^ (flip & 0xff));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_down(s, o, 64);
    if (lane == 0) out[r] = s;
}

struct i8_plan_t {
    bool small; // 32 x 32 tiles
    bool need_transpose, need_colsum, need_rowsum;
    size_t off_bt, off_colsum, off_rowsum, total;
    long Bw, Bs;
};

i8_plan_t make_plan(const mi355_matmul_desc_t &d) {
    i8_plan_t p {};
    p.Bw = d.wei_stride[0] ? d.batch : 1;
    p.Bs = d.src_stride[0] ? d.batch : 1;
    p.need_transpose = !(d.wei_stride[1] == 1);
    // the small tiles when the LDS tiles would occupy too little of the device
    // (measured with K = 1024 / 4096 against the 256 x 128 tiles, which take 16.7 /
    // 35 us for anything up to 128 large tiles: the small tiles take 14.5 / 30.3 us
    // at 12 large tiles, 17.2 / 37.5 at 16, 22.4 / 53.5 at 20), or when the LDS
    // tiles cannot step through K (the small tiles compute their own sums and have
    // no dynamic dst quantization)
    const long big_tiles = ((d.M + BM - 1) / BM) * ((d.N + i8_geo_t::BN - 1) / i8_geo_t::BN) * d.batch;
    const long crossover = 16;
    p.small = !d.dst_scale_dynamic && (big_tiles < crossover || d.K % BK != 0);
    // the MI355_I8_TILES switch overrides the choice where both can run (tests and
    // tuning): large = the LDS tiles, 256 x 128 or 256 x 256 by the number of
    // tiles; wide = the 256 x 256 ones
    const int force = tuning(TUNE_I8_TILES);
    if ((force == TUNE_LARGE || force == TUNE_WIDE || force == TUNE_NARROW) && d.K % BK == 0) p.small = false;
    if (force == TUNE_SMALL && !d.dst_scale_dynamic) p.small = true;
    // a = off_s - zs can be non-zero whenever src is u8 or has a zero point;
    // c likewise for the weights.  The small tiles compute their own sums: a
    // problem they run on K-contiguous weights needs no scratch at all.
    p.need_colsum = !p.small && (d.src_dt == MI355_DT_U8 || !quant_absent(d.src_zp));
    p.need_rowsum = !p.small && (d.wei_dt == MI355_DT_U8 || !quant_absent(d.wei_zp));
    // where a scratch buffer exists anyway its layout is that of the LDS tiles
    // (the sums are 4 (M + N) bytes), whichever tiles run
    const bool colsum = p.need_colsum || (p.need_transpose && (d.src_dt == MI355_DT_U8 || !quant_absent(d.src_zp)));
    const bool rowsum = p.need_rowsum || (p.need_transpose && (d.wei_dt == MI355_DT_U8 || !quant_absent(d.wei_zp)));
    size_t off = 0;
    p.off_bt = off;
    if (p.need_transpose) off += align_up((size_t)p.Bw * d.N * d.K, 256);
    p.off_colsum = off;
    if (colsum) off += align_up((size_t)p.Bw * d.N * 4, 256);
    p.off_rowsum = off;
    if (rowsum) off += align_up((size_t)p.Bs * d.M * 4, 256);
    p.total = off;
    return p;
}

} // namespace

int i8_supported(const mi355_matmul_desc_t &d) {
    if (!is_int8_dt(d.src_dt) || !is_int8_dt(d.wei_dt)) return MI355_UNIMPLEMENTED;
    if (dt_bits(d.dst_dt) < 8) return MI355_UNIMPLEMENTED;
    // (a K that is not a multiple of the large tiles' stage runs on the small
    // tiles, whose 16-byte operand loads are whole inside K or beyond it)
    if (d.K < 16 || d.K % 16 != 0) return MI355_UNIMPLEMENTED;
    if (d.K % BK != 0 && d.dst_scale_dynamic) return MI355_UNIMPLEMENTED;
    if (d.src_stride[2] != 1 || d.src_stride[1] % 16 != 0) return MI355_UNIMPLEMENTED;
    if (d.src_stride[0] % 16 != 0) return MI355_UNIMPLEMENTED;
    const bool k_major = d.wei_stride[1] == 1 && d.wei_stride[2] % 16 == 0
            && d.wei_stride[0] % 16 == 0;
    const bool n_major = d.wei_stride[2] == 1;
    if (!k_major && !n_major) return MI355_UNIMPLEMENTED;
    // single group along K, per-tensor src parameters, per-tensor or per-N
    // weights parameters
    if (!quant_absent(d.src_pr)) return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.src_scale) && (d.src_scale.mask != 0)) return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.src_zp) && (d.src_zp.mask != 0)) return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.wei_scale)
            && ((d.wei_scale.mask & 2) || d.wei_scale.group[0] > 1 || d.wei_scale.group[1] > 1))
        return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.wei_zp)
            && ((d.wei_zp.mask & 2) || d.wei_zp.group[0] > 1 || d.wei_zp.group[1] > 1))
        return MI355_UNIMPLEMENTED;
    if (d.batch > 65535) return MI355_UNIMPLEMENTED;
    return MI355_SUCCESS;
}

size_t i8_scratch_bytes(const mi355_matmul_desc_t &d) {
    return make_plan(d).total;
}

int i8_launch(const mi355_matmul_desc_t &d, const problem_t &P, void *scratch,
        hipStream_t stream) {
    const i8_plan_t plan = make_plan(d);
    if (plan.total > 0 && !scratch) {
        set_error("mfma_i8: %zu bytes of scratch required", plan.total);
        return MI355_INVALID_ARGUMENTS;
    }
    char *sc = (char *)scratch;
    i8_extra_t X {};
    const bool src_u8 = d.src_dt == MI355_DT_U8, wei_u8 = d.wei_dt == MI355_DT_U8;
    if (plan.need_transpose) {
        uint8_t *bt = (uint8_t *)(sc + plan.off_bt);
        transpose_bytes(P.wei, d.K, d.N, d.wei_stride[1], d.wei_stride[0], bt, d.K, d.N * d.K,
                plan.Bw, stream);
        X.bt = (const int8_t *)bt;
        X.ldb = d.K;
        X.bt_bstride = plan.Bw > 1 ? d.N * d.K : 0;
    } else {
        X.bt = (const int8_t *)P.wei;
        X.ldb = d.wei_stride[2];
        X.bt_bstride = d.wei_stride[0];
    }
    if (plan.need_colsum) {
        int *cs = (int *)(sc + plan.off_colsum);
        for (long b = 0; b < plan.Bw; ++b)
            hipLaunchKernelGGL(i8_rowsum_kernel, dim3((unsigned)((d.N + 3) / 4)), dim3(256), 0,
                    stream, X.bt + b * X.bt_bstride, d.N, d.K, X.ldb,
                    wei_u8 ? (int)0x80808080 : 0, cs + b * d.N);
        X.colsum = cs;
    }
    if (plan.need_rowsum) {
        int *rs = (int *)(sc + plan.off_rowsum);
        for (long b = 0; b < plan.Bs; ++b)
            hipLaunchKernelGGL(i8_rowsum_kernel, dim3((unsigned)((d.M + 3) / 4)), dim3(256), 0,
                    stream, (const int8_t *)P.src + b * d.src_stride[0], d.M, d.K,
                    d.src_stride[1], src_u8 ? (int)0x80808080 : 0, rs + b * d.M);
        X.rowsum = rs;
    }
    const bool su = d.src_dt == MI355_DT_U8, wu = d.wei_dt == MI355_DT_U8;
    if (plan.small) {
        X.tiles_m = (int)((d.M + ST - 1) / ST);
        X.tiles_n = (int)((d.N + ST - 1) / ST);
        const long tiles = (long)X.tiles_m * X.tiles_n;
        if (tiles >= (1L << 31)) {
            set_error("mfma_i8: %ld small tiles exceed the grid", tiles);
            return MI355_UNIMPLEMENTED;
        }
        const dim3 sgrid((unsigned)tiles, 1, (unsigned)d.batch);
        auto go_small = [&](auto kern) -> int {
            hipLaunchKernelGGL(kern, sgrid, dim3(SNW * 64), 0, stream, P, X);
            return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
        };
        if (su && wu) return go_small(i8_small_kernel<true, true>);
        if (su) return go_small(i8_small_kernel<true, false>);
        if (wu) return go_small(i8_small_kernel<false, true>);
        return go_small(i8_small_kernel<false, false>);
    }
    X.tiles_m = (int)((d.M + BM - 1) / BM);
    X.tiles_n = (int)((d.N + i8_geo_t::BN - 1) / i8_geo_t::BN);
    // Up to 128 large tiles leave half of the CUs or more idle: 256 x 128 tiles of four wavefronts, two workgroups a
    // CU, put twice as many to work (a wavefront's part, 128 x 64, its fragments and the epilogue are the same).
    // MI355_I8_TILES=wide keeps the 256 x 256 tiles.
    using narrow_t = geo_t<4, 128>;
    const int force = tuning(TUNE_I8_TILES);
    if (force == TUNE_NARROW || ((long)X.tiles_m * X.tiles_n * d.batch <= 128 && d.N > 128 && force != TUNE_WIDE)) {
        X.tiles_n = (int)((d.N + narrow_t::BN - 1) / narrow_t::BN);
        dim3 grid((unsigned)(X.tiles_m * X.tiles_n), 1, (unsigned)d.batch);
        constexpr int smem_bytes = narrow_t::NSTAGE * narrow_t::STAGE_BYTES + NTAB_BYTES;
        auto go = [&](auto kern) -> int {
            if (const int st = ensure_dynamic_lds((const void *)kern, smem_bytes, "mfma_i8")) return st;
            hipLaunchKernelGGL(kern, grid, dim3(narrow_t::NT), smem_bytes, stream, P, X);
            return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
        };
        if (su && wu) return go(i8_gemm_kernel<true, true, narrow_t>);
        if (su) return go(i8_gemm_kernel<true, false, narrow_t>);
        if (wu) return go(i8_gemm_kernel<false, true, narrow_t>);
        return go(i8_gemm_kernel<false, false, narrow_t>);
    }
    dim3 grid((unsigned)(X.tiles_m * X.tiles_n), 1, (unsigned)d.batch);
    constexpr int smem_bytes = NSTAGE * i8_geo_t::STAGE_BYTES + NTAB_BYTES;
    auto go = [&](auto kern) -> int {
        if (const int st = ensure_dynamic_lds((const void *)kern, smem_bytes, "mfma_i8")) return st;
        hipLaunchKernelGGL(kern, grid, dim3(i8_geo_t::NT), smem_bytes, stream, P, X);
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
    };
    if (su && wu) return go(i8_gemm_kernel<true, true, i8_geo_t>);
    if (su) return go(i8_gemm_kernel<true, false, i8_geo_t>);
    if (wu) return go(i8_gemm_kernel<false, true, i8_geo_t>);
    return go(i8_gemm_kernel<false, false, i8_geo_t>);
}

} // namespace mi355
