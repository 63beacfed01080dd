// "hip:mfma_mxf4" -- MXFP4 GEMM: f4_e2m1 x f4_e2m1 with e8m0 block scales over
// 32 consecutive K on both operands, f32 accumulation, on the gfx950
// block-scaled matrix instruction v_mfma_scale_f32_16x16x128_f8f6f4.
//
// Semantics: ref_matmul_t with group_k = 32 (src/cpu/matmul/ref_matmul.cpp:
// 168-236; the Intel GPU reference kernel src/gpu/intel/matmul/ref.cl:200-262
// is the in-tree implementation that runs it):
//   for each block g of 32 k:  acc = sum_j src*wei  (exact in f32)
//                              acc *= 2^(ss-127); acc *= 2^(ws-127); res += acc
// One MFMA covers 128 k = four blocks; lane l carries row l%16 and block l/16,
// i.e. exactly one MX block and one scale byte per operand per lane.  Only the
// rounding of the cross-block f32 additions can differ from the reference.
//
// Operand bytes are K-contiguous nibble pairs; the order of the two nibbles
// inside a byte is irrelevant as long as both operands agree, because all 32
// elements of a block share one scale.
//
// Scales ride along with the tile stages: per stage and operand one extra
// direct-to-LDS load per wavefront brings the 4 scale bytes (one dword) of
// each of its 64 rows.  Two small pre-pass kernels of the launch put both
// operands' scales into a stage-major order, [K/128][rows] dwords, so that this
// load is 256 contiguous bytes: from the plain layouts (src [M][K/32] bytes, a
// row's dword of a stage 256 bytes from the next row's at K = 8192) the same
// load touched 64 cache lines for 256 useful bytes, and the scales made as many
// requests to the L2 as the tiles themselves.
#include "gemm_core.hpp"

namespace mi355 {
namespace {

using namespace gemm;
#ifndef MI355_MXF4_NW
#define MI355_MXF4_NW 8
#endif
#ifndef MI355_MXF4_AHEAD
#define MI355_MXF4_AHEAD 1
#endif
using mx_geo_t = geo_t<MI355_MXF4_NW, 256>;
constexpr int NSTAGE = mx_geo_t::NSTAGE;
constexpr int SCALE_OFF = NSTAGE * mx_geo_t::STAGE_BYTES; // scale ring after the tile ring
constexpr int SCALE_STAGE = (BM + mx_geo_t::BN) * 4;      // 256 dwords A + BN dwords B
constexpr int SMEM_RING_BYTES = SCALE_OFF + NSTAGE * SCALE_STAGE;
constexpr int SMEM_BYTES = SMEM_RING_BYTES + NTAB_BYTES;

struct mxf4_extra_t {
    const char *bt;       // weights [N][K/2] bytes
    long ldb, bt_bstride; // bytes
    const char *sa;       // src scales, stage-major copy: [K/128][M] dwords, this batch added in-kernel
    const char *sb;       // weights scales, stage-major copy: [K/128][N] dwords
    long sa_bstride, sb_bstride;
    long sa_pitch, sb_pitch; // bytes between stages: 4 M, 4 N
    int tiles_m, tiles_n;
};

struct mxf4_ctx_t {
    const char *sa_tile, *sb_tile; // scale dword of tile row 0, stage 0
    long sa_pitch, sb_pitch;       // bytes between stages
    unsigned voff_a, voff_b;       // this lane's row offset in the scale arrays
    const char *s_tile;            // eight wavefronts: the one operand this wavefront brings
    long s_pitch;
    unsigned voff_s;
    unsigned lds_scale0;           // LDS byte address of the scale ring
    unsigned lds0;                 // LDS byte address of the tile ring
};

template <class G_>
struct mxf4_mma_t {
    using G = G_;
    static constexpr int EXTRA_DMAS = G::NW == 4 ? 2 : 1;
    static constexpr int BBLK = G::BN / 64; // 64-row blocks of B^T scales
    // four wavefronts: wave w brings the scale dwords of tile rows [64w, 64w+64)
    // of A and those of block w % BBLK of B^T (with BN = 128 two wavefronts
    // bring the same block: every wavefront issues the same number of loads,
    // which the outstanding-load accounting relies on); eight wavefronts:
    // waves 0-3 bring those of A, waves 4-7 those of B^T
    __device__ static __forceinline__ void issue_extra(const mxf4_ctx_t &c, int g, int slot, int wave,
            int) {
        const unsigned dst = c.lds_scale0 + slot * SCALE_STAGE + wave * 256;
        if (G::NW == 4) {
            dma4(c.sa_tile + (long)g * c.sa_pitch, c.voff_a, dst);
            dma4(c.sb_tile + (long)g * c.sb_pitch, c.voff_b,
                    c.lds_scale0 + slot * SCALE_STAGE + 1024 + (wave % BBLK) * 256);
        } else {
            dma4(c.s_tile + (long)g * c.s_pitch, c.voff_s, dst);
        }
    }
    static constexpr int ROWS = 8, COLS = G::WCOLS / 16, A_READS = 2, B_READS = 2; // data + scale dword
    static constexpr int SA = ROWS / 4, SB = (COLS + 3) / 4; // scale dwords: one per four fragments
    struct frag_t {
        v4i a[ROWS], b[COLS];
        int sa[SA], sb[SB];
    };
    __device__ static __forceinline__ frag_t zero_frag() { return frag_t {}; } // e2m1 zero is all-zero bits
    // LDS byte address of the scale dwords that belong to the stage at S[0]
    __device__ static __forceinline__ unsigned scales(const unsigned (&S)[1], const mxf4_ctx_t &c) {
        const unsigned slot = (S[0] - c.lds0) / G::STAGE_BYTES;
        return c.lds_scale0 + slot * SCALE_STAGE;
    }
    // Per-lane LDS offsets of fragment 0 (data; fragment i is 16 rows further) and of
    // the scale dword of the lane's first group of 64 rows.  A group of 64 rows holds
    // its stage's scales as 64 dwords, dword 4 r + q = the bytes of block q of rows r,
    // 16 + r, 32 + r and 48 + r (the pre-pass kernels of the launch write that order):
    // lane (r, q) of an MFMA operand reads one dword and has the scale bytes of four
    // fragments, which the instruction picks by its op_sel bits -- a dword and a read
    // per four fragments, nothing to shift or mask.
    struct addr_t {
        unsigned a, b, sa, sb;
    };
    __device__ static __forceinline__ addr_t lane_addr(int wm, int wn, int lane) {
        const int frow = lane & 15, q = lane >> 4;
        const int ra = wm * 128 + frow, rb = wn * G::WCOLS + frow;
        const int cell = (frow * 4 + q) * 4;
        return addr_t {(unsigned)swz(ra, q), (unsigned)(B_OFF + swz(rb, q)), (unsigned)(wm * 2 * 256 + cell),
                (unsigned)(1024 + (wn * G::WCOLS / 64) * 256 + cell)};
    }
    static constexpr bool READS_AHEAD = MI355_MXF4_AHEAD;
    __device__ static __forceinline__ void prepare(frag_t &) {}
    __device__ static __forceinline__ void load_b_one(frag_t &f, int j, const unsigned (&S)[1], const addr_t &ad,
            const mxf4_ctx_t &c, int) {
        f.b[j] = lds_read16(S[0] + ad.b + j * 1024);
        if (j % 4 == 0) f.sb[j / 4] = (int)lds_read4(scales(S, c) + ad.sb + (j / 4) * 256);
    }
    __device__ static __forceinline__ void load_b(frag_t &f, const unsigned (&S)[1], const addr_t &ad,
            const mxf4_ctx_t &c, int g) {
#pragma unroll
        for (int j = 0; j < COLS; ++j) load_b_one(f, j, S, ad, c, g);
    }
    __device__ static __forceinline__ void load_a(frag_t &f, int i, const unsigned (&S)[1], const addr_t &ad,
            const mxf4_ctx_t &c, int) {
        f.a[i] = lds_read16(S[0] + ad.a + i * 1024);
        if (i % 4 == 0) f.sa[i / 4] = (int)lds_read4(scales(S, c) + ad.sa + (i / 4) * 256);
    }
    // The instruction is written out with the accumulator tied to one operand: left
    // to itself the compiler accumulates out of place in the loops that alternate
    // between fragment sets or wavefront groups and then moves accumulators through
    // scratch memory in every iteration (one wavefront per SIMD: the accumulation
    // registers; two: plain ones, which the epilogue can work on directly).  No
    // wait states are owed inside the loop: an accumulator is next touched 31 or 63
    // instructions later.  OW / OS: the byte of the scale dwords that belongs to the
    // weights / src fragment (op_sel bit 0, op_sel_hi bit 1 of each).
    template <int OW, int OS>
    __device__ static __forceinline__ void mma_one(v4f &acc, const v4i &w, const v4i &s, int sw, int ss) {
        // operands exchanged: the tile comes out transposed, a lane holds four
        // consecutive n of one row (tile_epilogue.hpp)
        if constexpr (G::NW == 4)
            asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[%5,%6,0] op_sel_hi:[%7,%8,0] cbsz:4 blgp:4"
                         : "+a"(acc)
                         : "v"(w), "v"(s), "v"(sw), "v"(ss), "n"(OW & 1), "n"(OS & 1), "n"(OW >> 1), "n"(OS >> 1));
        else
            asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[%5,%6,0] op_sel_hi:[%7,%8,0] cbsz:4 blgp:4"
                         : "+v"(acc)
                         : "v"(w), "v"(s), "v"(sw), "v"(ss), "n"(OW & 1), "n"(OS & 1), "n"(OW >> 1), "n"(OS >> 1));
    }
    template <int I, int J>
    __device__ static __forceinline__ void mma_cols(v4f (&acc)[ROWS][COLS], const frag_t &f) {
        if constexpr (J < COLS) {
            mma_one<J % 4, I % 4>(acc[I][J], f.b[J], f.a[I], f.sb[J / 4], f.sa[I / 4]);
            mma_cols<I, J + 1>(acc, f);
        }
    }
    template <int I>
    __device__ static __forceinline__ void mma_rows(v4f (&acc)[ROWS][COLS], const frag_t &f, int i) {
        if constexpr (I < ROWS) {
            if (i == I) mma_cols<I, 0>(acc, f);
            else mma_rows<I + 1>(acc, f, i);
        }
    }
    // K that ends inside a stage (gemm_core.hpp tail_step): the lane's chunk is block lane / 16 of the stage
    static constexpr bool K_TAIL = true;
    __device__ static __forceinline__ void zero_tail(frag_t &f, int nz, int lane) {
        const bool z = (lane >> 4) < nz;
#pragma unroll
        for (int i = 0; i < ROWS; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) f.a[i][e] = z ? 0 : f.a[i][e];
#pragma unroll
        for (int j = 0; j < COLS; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) f.b[j][e] = z ? 0 : f.b[j][e];
    }
    // (i is a constant after unrolling: the chain of comparisons folds away)
    __device__ static __forceinline__ void mma_row(v4f (&acc)[ROWS][COLS], const frag_t &f, int i,
            const mxf4_ctx_t &, int) {
        mma_rows<0>(acc, f, i);
    }
};

struct mxf4_conv_t {
    typedef int row_t;
    template <class PT>
    __device__ __forceinline__ void per_n(const PT &, long, long, float &, int &, int &) const {}
    __device__ __forceinline__ int row_data(long) const { return 0; }
    // The configuration's own chain: the accumulators as they are -> bf16, no bias, no post-ops.  Global memory sees
    // whole 128-byte rows only: in the accumulator layout a lane owns 8 bytes of a dst row and a wavefront-wide store
    // touches 16 rows, 32 bytes each (the memory pipeline's cost is per line touched).  The wavefront's 128 x 64 part
    // goes through its 16 KB share of the idle tile ring instead -- 8-byte writes at row * 128 + ((slot ^ (row / 2 & 7))
    // << 4), which spread over all banks -- and leaves as 16 stores of 8 whole rows.
    template <class PT>
    __device__ __forceinline__ bool hot_chain(const PT &P, const epi_uniform_t &H, unsigned, unsigned lds_part,
            const v4f (&acc)[8][4], long b, long m_base, long n_base, int) const {
        return store_rows_bf16_tile16(P, H, lds_part, acc, b, m_base, n_base);
    }
    template <class PT, class Acc>
    __device__ __forceinline__ bool hot_chain(const PT &, const epi_uniform_t &, unsigned, unsigned, const Acc &, long,
            long, long, int) const {
        return false;
    }
    __device__ __forceinline__ void quad(const v4i_t &raw, int, unsigned, int, float (&f)[4]) const {
#pragma unroll
        for (int e = 0; e < 4; ++e) f[e] = __int_as_float(raw[e]);
    }
};

extern __shared__ __attribute__((aligned(16))) char mxf4_smem[];

template <class G>
__global__ void __launch_bounds__(G::NT) __attribute__((amdgpu_waves_per_eu(G::NW * G::WG_PER_CU / 4))) mxf4_gemm_kernel(const problem_t P_, const mxf4_extra_t X) {
    using Mma = mxf4_mma_t<G>;
    const auto &P = MI355_KERNARG_PROBLEM();
    char *smem = mxf4_smem;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = G::wm(wave), wn = G::wn(wave);
    const long b = blockIdx.z;
    const tile_pos_t tp = tile_position<G>((int)blockIdx.x, X.tiles_m, X.tiles_n);
    const long m0 = tp.m0, n0 = tp.n0;

    const long lda = P.ss[1] / 2; // bytes per src row
    const char *A = (const char *)P.src + (P.ss[0] ? b * (P.ss[0] / 2) : 0) + m0 * lda;
    const char *Bt = X.bt + b * X.bt_bstride + n0 * X.ldb;

    mxf4_ctx_t ctx;
    ctx.lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem;
    ctx.lds_scale0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem + SCALE_OFF;
    ctx.sa_tile = X.sa + b * X.sa_bstride + m0 * 4;
    ctx.sb_tile = X.sb + b * X.sb_bstride + n0 * 4;
    ctx.sa_pitch = X.sa_pitch;
    ctx.sb_pitch = X.sb_pitch;
    {
        // (the packed scales are padded to whole tiles of 256 rows: nothing to clamp)
        const long ra = (wave & 3) * 64 + lane, rb = ((wave & 3) % (G::BN / 64)) * 64 + lane;
        ctx.voff_a = (unsigned)(ra * 4);
        ctx.voff_b = (unsigned)(rb * 4);
        const bool brings_a = __builtin_amdgcn_readfirstlane(wave) < 4; // uniform: the base stays scalar
        ctx.s_tile = brings_a ? ctx.sa_tile : ctx.sb_tile;
        ctx.s_pitch = brings_a ? ctx.sa_pitch : ctx.sb_pitch;
        ctx.voff_s = brings_a ? ctx.voff_a : ctx.voff_b;
    }

    // the epilogue's per-column operands go into their LDS table now
    const unsigned ntab = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem + SMEM_RING_BYTES;
    fill_ntab<G::NT>(P, mxf4_conv_t {}, ntab, b, n0);

    v4f acc[Mma::ROWS][Mma::COLS];
#pragma unroll
    for (int i = 0; i < Mma::ROWS; ++i)
#pragma unroll
        for (int j = 0; j < Mma::COLS; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    main_loop<NSTAGE, 1, Mma>(acc, smem, A, Bt, lda, X.ldb, P.M - m0, P.N - n0,
            (int)(P.K / 128), ctx);
    // the rest of a K that is whole blocks of 32 but not whole stages of 128: the row's last 64 bytes, the blocks
    // multiplied before zeroed; the scales of those four blocks are the stage after the whole ones in the packed order
    if (const int rem = (int)(P.K % 128))
        tail_step<Mma>(acc, smem, A + P.K / 2 - BKB, Bt + P.K / 2 - BKB, lda, X.ldb, P.M - m0, P.N - n0,
                (128 - rem) / 32, (int)(P.K / 128), ctx);

    store_quadrant<layout16_t, G::WCOLS>(P, smem, ntab, acc, b, m0 + wm * 128, n0 + wn * G::WCOLS, wn * G::WCOLS,
            mxf4_conv_t {});
}

// in: [R][C] nibbles, C contiguous (two per byte)  ->  out: [C][R] nibbles
__global__ void __launch_bounds__(256) transpose_nibbles_kernel(const uint8_t *in, long R, long C,
        long in_bstride, uint8_t *out, long out_bstride) {
    in += blockIdx.z * in_bstride;
    out += blockIdx.z * out_bstride;
    // one thread per output byte: column c, rows 2r and 2r+1
    const long total = C * (R / 2);
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
            i += (long)gridDim.x * blockDim.x) {
        const long c = i / (R / 2), r2 = i % (R / 2);
        const uint8_t b0 = in[((2 * r2) * C + c) >> 1], b1 = in[((2 * r2 + 1) * C + c) >> 1];
        const uint8_t lo = (c & 1) ? (b0 >> 4) : (b0 & 0xf), hi = (c & 1) ? (b1 >> 4) : (b1 & 0xf);
        out[c * (R / 2) + r2] = (uint8_t)(lo | (hi << 4));
    }
}

// e8m0 scales of `rows` rows x KB blocks of 32 k, element (r, kb) at in[r * rs + kb * ks], into the order the tile
// kernel loads: per stage of 128 k (four blocks) and group of 64 rows 64 dwords, dword 4 r + q = the bytes of block q
// of rows r, 16 + r, 32 + r, 48 + r of the group; groups padded to whole tiles of 256 rows (rows beyond the last
// repeat it).  out[stage][group][64] dwords.
// Rows contiguous in the input (weights scales [K/32][N], rs = 1): a thread per dword.
__global__ void __launch_bounds__(256) mx_scales_rows_kernel(const uint8_t *in, long rows, long prows, long KB, long ks,
        long in_bstride, uint32_t *out, long out_bstride) {
    in += blockIdx.z * in_bstride;
    out += blockIdx.z * out_bstride;
    const long nst = (KB + 3) / 4, total = prows * nst;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const long st = i / prows, w = i % prows, grp = w / 64;
        const int cell = (int)(w % 64), r = cell >> 2, q = cell & 3;
        // a last stage that K does not fill holds the last four blocks (the tile kernel multiplies the row's last
        // 64 bytes there)
        const long blk = 4 * st + 4 <= KB ? 4 * st + q : KB - 4 + q;
        uint32_t v = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            long row = grp * 64 + 16 * e + r;
            row = row < rows ? row : rows - 1;
            v |= (uint32_t)in[blk * ks + row] << (8 * e);
        }
        out[i] = v;
    }
}
// Blocks contiguous in the input (src scales [M][K/32], ks = 1): a workgroup moves 64 rows x 16 stages through LDS,
// 64 contiguous bytes of a row in, 256 contiguous bytes of a stage and group out.
__global__ void __launch_bounds__(256) mx_scales_blocks_kernel(const uint8_t *in, long rows, long prows, long KB, long rs,
        long in_bstride, uint32_t *out, long out_bstride) {
    __shared__ uint32_t tile[16][65]; // [stage][row]: the row's four block bytes of the stage
    in += blockIdx.z * in_bstride;
    out += blockIdx.z * out_bstride;
    const long grp = blockIdx.x, r0 = grp * 64, q0 = (long)blockIdx.y * 16, nq = (KB + 3) / 4;
    const int t = threadIdx.x;
    const bool aligned = ((uintptr_t)in & 3) == 0 && (rs & 3) == 0;
    {
        const int r = t >> 2, c = t & 3; // row, group of four stages
        const long row = r0 + r < rows ? r0 + r : rows - 1;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const long q = q0 + 4 * c + e;
            // (a last stage that K does not fill: the row's last four blocks)
            const uint8_t *p = in + row * rs + (4 * q + 4 <= KB ? 4 * q : KB - 4);
            uint32_t v = 0u;
            if (q < nq) {
                if (aligned) v = *(const uint32_t *)p;
                else v = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
            }
            tile[4 * c + e][r] = v;
        }
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int st = (t >> 6) + 4 * e, cell = t & 63, r = cell >> 2, q = cell & 3;
        if (q0 + st < nq) {
            uint32_t v = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k) v |= ((tile[st][16 * k + r] >> (8 * q)) & 0xffu) << (8 * k);
            out[(q0 + st) * prows + grp * 64 + cell] = v;
        }
    }
}

struct mxf4_plan_t {
    bool need_transpose;
    size_t off_bt, off_sb, off_sa, total;
    long Bw, Bsb, Bsa;
    long pm, pn; // M, N rounded up to whole tiles
    long nst;
};

mxf4_plan_t make_plan(const mi355_matmul_desc_t &d) {
    mxf4_plan_t p {};
    p.Bw = d.wei_stride[0] ? d.batch : 1;
    p.Bsb = (d.wei_scale.mask & 1) ? p.Bw : 1;
    p.need_transpose = !(d.wei_stride[1] == 1);
    size_t off = 0;
    p.off_bt = off;
    if (p.need_transpose) off += align_up((size_t)p.Bw * d.N * d.K / 2, 256);
    // the scales in the tile kernel's order, rows padded to whole tiles
    p.pn = (d.N + 255) / 256 * 256;
    p.pm = (d.M + 255) / 256 * 256;
    p.off_sb = off;
    p.nst = (d.K + 127) / 128; // stages, one scale dword per row and stage
    off += align_up((size_t)p.Bsb * p.pn * p.nst * 4, 256);
    p.Bsa = ((d.src_scale.mask & 1) && d.src_stride[0]) ? d.batch : 1;
    p.off_sa = off;
    off += align_up((size_t)p.Bsa * p.pm * p.nst * 4, 256);
    p.total = off;
    return p;
}

} // namespace

int mxf4_supported(const mi355_matmul_desc_t &d) {
    if (d.src_dt != MI355_DT_F4_E2M1 || d.wei_dt != MI355_DT_F4_E2M1) return MI355_UNIMPLEMENTED;
    if (dt_bits(d.dst_dt) < 8 && !tile_nibble_dst_ok(d)) return MI355_UNIMPLEMENTED;
    // whole MX blocks; a K that ends inside a stage of 128 takes one unpipelined step more per tile
    if (d.K < 128 || d.K % 32 != 0) return MI355_UNIMPLEMENTED;
    if (d.src_stride[2] != 1 || d.src_stride[1] % 32 != 0 || d.src_stride[0] % 32 != 0)
        return MI355_UNIMPLEMENTED;
    const bool k_major = d.wei_stride[1] == 1 && d.wei_stride[2] % 32 == 0 && d.wei_stride[0] % 32 == 0;
    const bool n_major = d.wei_stride[2] == 1 && d.wei_stride[1] == d.N && d.N % 2 == 0
            && (d.wei_stride[0] == 0 || d.wei_stride[0] == d.K * d.N);
    if (!k_major && !n_major) return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.src_zp) || !quant_absent(d.wei_zp) || !quant_absent(d.src_pr))
        return MI355_UNIMPLEMENTED;
    // MX scales on both operands: e8m0, one per 32 consecutive k
    const mi355_quant_t &ss = d.src_scale, &ws = d.wei_scale;
    if (ss.dt != MI355_DT_E8M0 || (ss.mask & 6) != 6 || ss.group[0] != 1 || ss.group[1] != 32)
        return MI355_UNIMPLEMENTED;
    if (ws.dt != MI355_DT_E8M0 || (ws.mask & 6) != 6 || ws.group[0] != 32 || ws.group[1] != 1)
        return MI355_UNIMPLEMENTED;
    if (d.batch > 65535) return MI355_UNIMPLEMENTED;
    return MI355_SUCCESS;
}

size_t mxf4_scratch_bytes(const mi355_matmul_desc_t &d) {
    return make_plan(d).total;
}

int mxf4_launch(const mi355_matmul_desc_t &d, const problem_t &P, void *scratch, hipStream_t stream) {
    const mxf4_plan_t plan = make_plan(d);
    if (!scratch) {
        set_error("mfma_mxf4: %zu bytes of scratch required", plan.total);
        return MI355_INVALID_ARGUMENTS;
    }
    char *sc = (char *)scratch;
    mxf4_extra_t X {};
    if (plan.need_transpose) {
        const long total = d.N * (d.K / 2);
        long blocks = (total + 255) / 256;
        if (blocks > 65535) blocks = 65535;
        hipLaunchKernelGGL(transpose_nibbles_kernel, dim3((unsigned)blocks, 1, (unsigned)plan.Bw),
                dim3(256), 0, stream, (const uint8_t *)P.wei, d.K, d.N, d.wei_stride[0] / 2,
                (uint8_t *)(sc + plan.off_bt), d.N * d.K / 2);
        X.bt = sc + plan.off_bt;
        X.ldb = d.K / 2;
        X.bt_bstride = plan.Bw > 1 ? d.N * d.K / 2 : 0;
    } else {
        X.bt = (const char *)P.wei;
        X.ldb = d.wei_stride[2] / 2;
        X.bt_bstride = d.wei_stride[0] / 2;
    }
    // scales into the tile kernel's order (see mx_scales_rows_kernel)
    const long kb = d.K / 32;
    {
        long blocks = (plan.pn * plan.nst + 255) / 256;
        if (blocks > 65535) blocks = 65535;
        hipLaunchKernelGGL(mx_scales_rows_kernel, dim3((unsigned)blocks, 1, (unsigned)plan.Bsb), dim3(256), 0, stream,
                (const uint8_t *)P.wei_scale.p, d.N, plan.pn, kb, d.N, kb * d.N, (uint32_t *)(sc + plan.off_sb),
                plan.pn * plan.nst);
        hipLaunchKernelGGL(mx_scales_blocks_kernel,
                dim3((unsigned)(plan.pm / 64), (unsigned)((plan.nst + 15) / 16), (unsigned)plan.Bsa), dim3(256), 0, stream,
                (const uint8_t *)P.src_scale.p, d.M, plan.pm, kb, kb, d.M * kb, (uint32_t *)(sc + plan.off_sa),
                plan.pm * plan.nst);
    }
    X.sb = sc + plan.off_sb;
    X.sb_bstride = plan.Bsb > 1 ? plan.pn * plan.nst * 4 : 0;
    X.sb_pitch = plan.pn * 4;
    X.sa = sc + plan.off_sa;
    X.sa_bstride = plan.Bsa > 1 ? plan.pm * plan.nst * 4 : 0;
    X.sa_pitch = plan.pm * 4;
    X.tiles_m = (int)((d.M + BM - 1) / BM);
    X.tiles_n = (int)((d.N + mx_geo_t::BN - 1) / mx_geo_t::BN);
    dim3 grid((unsigned)(X.tiles_m * X.tiles_n), 1, (unsigned)d.batch);
    if (const int st = ensure_dynamic_lds((const void *)mxf4_gemm_kernel<mx_geo_t>, SMEM_BYTES, "mfma_mxf4")) return st;
    hipLaunchKernelGGL(mxf4_gemm_kernel<mx_geo_t>, grid, dim3(mx_geo_t::NT), SMEM_BYTES, stream, P, X);
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
}

} // namespace mi355
