// "hip:mfma_f8" -- LDS-tiled fp8 GEMM (OCP e4m3 / e5m2 operands, f32
// accumulation) on the gfx950 matrix cores, v_mfma_f32_32x32x64_f8f6f4, with
// the reference's epilogue fused in.
//
// Semantics: ref_matmul_t (src/cpu/matmul/ref_matmul.cpp:168-331) for f8 src
// and weights with per-tensor / per-row src scales and per-tensor / per-n
// weights scales.  The reference scales every product before summing
// (its "group" is a single k when no K groups exist); this kernel sums the
// exact e4m3 x e4m3 products in f32 on the matrix cores and applies
//   acc * src_scale * wei_scale
// once, which differs only in rounding and is covered by the f32/bf16
// comparison thresholds.
//
// MFMA shape: v_mfma_f32_32x32x64_f8f6f4.  Measured on MI355X with random
// operands the 16x16x128 shape sustains ~4.9 PFLOP/s against ~4.3 for this
// one, but it consumes 128 bytes of K per instruction: two 32 KB stages at a
// time, which leaves room for two such groups in LDS and a prefetch distance
// of one group, shorter than the memory latency (measured 175 us per 256x256
// tile at K = 8192).  The 32x32x64 shape consumes one 64-byte stage like the
// int8 kernel and keeps three stages in flight.
//
// "hip:mfma_h16" -- the same tiles for bf16 x bf16, f16 x f16 and f32 x f32 operands
// (ref_matmul_t's f32 sum of exact products): a 64-byte stage is 32 elements of
// K, two v_mfma_f32_32x32x16_{bf16,f16} per fragment pair in the time of the
// one fp8 instruction, so the data path (DMA, LDS ring, fragment reads,
// epilogue) is shared unchanged; a lane's two 16-byte chunks of a stage feed
// the two instructions, the same chunks for both operands, so the order in
// which the 32 k of a stage meet does not matter.
#include "gemm_core.hpp"

namespace mi355 {
namespace {

using namespace gemm;
constexpr int KSTEP = 1;
using f8_geo_t = geo_t<8, 256>;
using mxf8_geo_t = geo_t<4, 256>; // the block-scaled variant: see mxf8_mma_t
constexpr int NSTAGE = f8_geo_t::NSTAGE; // one stage (K = 64) per step

struct f8_extra_t {
    const char *bt; // weights as [N][K] bytes, K contiguous
    long ldb, bt_bstride;
    int tiles_m, tiles_n;
    // MX variant: e8m0 scales per 32 k, src [M][K/32], weights transposed to [N][K/32]
    const char *sa, *sb;
    long sa_bstride, sb_bstride;
};

struct f8_ctx_t {};

// cbsz / blgp operand format codes of the f8f6f4 MFMA: 0 = e4m3, 1 = e5m2
template <int FMT_A, int FMT_B, class G_>
struct f8_mma_t {
    using G = G_;
    static constexpr int ELEM_BYTES = 1;
    static constexpr bool HOT = FMT_A == 0 && FMT_B == 0;
    static constexpr int EXTRA_DMAS = 0;
    __device__ static __forceinline__ void issue_extra(const f8_ctx_t &, int, int, int, int) {}
    static constexpr int ROWS = 4, COLS = G::WCOLS / 32, A_READS = 2, B_READS = 2;
    struct frag_t {
        v8i a[ROWS], b[COLS];
    };
    __device__ static __forceinline__ frag_t zero_frag() { return frag_t {}; } // fp8 zero is all-zero bits
    // lane l supplies row l%32 and K bytes 32*(l/32) .. +32 of the stage: two
    // 16-byte chunks.  Per-lane LDS offsets of fragment 0; fragment i is 32 rows
    // (2 KB) further with the same swizzle.
    struct addr_t {
        unsigned a0, a1, b0, b1;
    };
    __device__ static __forceinline__ addr_t lane_addr(int wm, int wn, int lane) {
        const int frow = lane & 31, c0 = (lane >> 5) * 2;
        const int ra = wm * 128 + frow, rb = wn * G::WCOLS + frow;
        return addr_t {(unsigned)swz(ra, c0), (unsigned)swz(ra, c0 + 1), (unsigned)(B_OFF + swz(rb, c0)),
                (unsigned)(B_OFF + swz(rb, c0 + 1))};
    }
    __device__ static __forceinline__ v8i read32(unsigned lo_addr, unsigned hi_addr) {
        const v4i lo = lds_read16(lo_addr), hi = lds_read16(hi_addr);
        return v8i {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
    __device__ static __forceinline__ void load_b(frag_t &f, const unsigned (&S)[1], const addr_t &ad,
            const f8_ctx_t &, int) {
#pragma unroll
        for (int j = 0; j < COLS; ++j) f.b[j] = read32(S[0] + ad.b0 + j * 2048, S[0] + ad.b1 + j * 2048);
    }
    __device__ static __forceinline__ void load_a(frag_t &f, int i, const unsigned (&S)[1], const addr_t &ad,
            const f8_ctx_t &, int) {
        f.a[i] = read32(S[0] + ad.a0 + i * 2048, S[0] + ad.a1 + i * 2048);
    }
    __device__ static __forceinline__ void mma_row(v16f (&acc)[ROWS][COLS], const frag_t &f, int i,
            const f8_ctx_t &, int) {
#pragma unroll
        for (int j = 0; j < COLS; ++j)
            // operands exchanged: the tile comes out transposed, a lane holds four
            // consecutive n of one row per accumulator quad (tile_epilogue.hpp)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    f.b[j], f.a[i], acc[i][j], FMT_B, FMT_A, 0, 0, 0, 0);
    }
};

// MXFP8: the fp8 policy with e8m0 scales per 32 k on both operands, applied by
// the instruction itself (v_mfma_scale_f32_32x32x64_f8f6f4): ref_matmul_t with
// group_k = 32 -- acc = sum of a block's 32 products, acc *= 2^(ss-127),
// acc *= 2^(ws-127), res += acc (src/cpu/matmul/ref_matmul.cpp:168-236).
// A 64-byte stage is two blocks; lanes 0-31 supply the scale byte of the
// stage's first block of their row, lanes 32-63 that of the second.  The scale
// bytes ride along with the tile stages as in the MXFP4 family: one direct-to-LDS
// dword per row and stage -- the dword that holds the stage's two bytes, so two
// consecutive stages fetch the same one.  Four wavefronts of 128 x 128 (the
// geometry of the MXFP4 family): with eight, the scale operands on top of the
// fp8 policy's registers put spills into the K loop (6.5 GB of scratch writes
// per 8192^3 launch, 0.4 PFLOP/s).
struct mxf8_ctx_t {
    const char *sa_tile, *sb_tile; // first scale byte of tile row 0 of each operand
    unsigned voff_a, voff_b;       // this lane's row offset in the scale arrays
    unsigned lds_scale0;           // LDS byte address of the scale ring
    unsigned lds0;                 // LDS byte address of the tile ring
};

// SPLIT: which 16-byte chunks of a stage a lane's register halves hold.  The
// instruction reads the first halves of all lanes as k 0..31 and the second
// halves as k 32..63 (lane group h: bytes 16h..16h+15 of each), while it takes
// block h's scale from lane group h -- so for scaled operands a lane holds
// chunks h and 2 + h (SPLIT), not the contiguous 2h, 2h + 1 that serve when
// no scale distinguishes the blocks (established on the device: exact data
// with a scale of its own per block match the oracle bit for bit this way and
// differ the other way).
template <int FMT_A, int FMT_B, bool SPLIT, class G_>
struct mxf8_mma_t {
    using G = G_;
    static constexpr int ELEM_BYTES = 1;
    static constexpr bool HOT = false;
    static constexpr int EXTRA_DMAS = 2;
    static constexpr int SCALE_STAGE = (BM + G::BN) * 4;
    static_assert(G::NW == 4 && G::BN == 256, "wavefront w brings the scale dwords of rows 64 w .. 64 w + 63 of A and of B^T");
    __device__ static __forceinline__ void issue_extra(const mxf8_ctx_t &c, int g, int slot, int wave, int) {
        const unsigned dst = c.lds_scale0 + slot * SCALE_STAGE + wave * 256;
        dma4(c.sa_tile + (long)(g >> 1) * 4, c.voff_a, dst);
        dma4(c.sb_tile + (long)(g >> 1) * 4, c.voff_b, dst + BM * 4);
    }
    static constexpr int ROWS = 4, COLS = G::WCOLS / 32, A_READS = 3, B_READS = 3;
    struct frag_t {
        v8i a[ROWS], b[COLS];
        int sa[ROWS], sb[COLS];
    };
    __device__ static __forceinline__ frag_t zero_frag() { return frag_t {}; }
    struct addr_t {
        unsigned a0, a1, b0, b1, sa, sb, shift;
    };
    __device__ static __forceinline__ addr_t lane_addr(int wm, int wn, int lane) {
        const int frow = lane & 31, h = lane >> 5;
        const int c0 = SPLIT ? h : 2 * h, c1 = SPLIT ? 2 + h : 2 * h + 1;
        const int ra = wm * 128 + frow, rb = wn * G::WCOLS + frow;
        return addr_t {(unsigned)swz(ra, c0), (unsigned)swz(ra, c1), (unsigned)(B_OFF + swz(rb, c0)),
                (unsigned)(B_OFF + swz(rb, c1)), (unsigned)(ra * 4), (unsigned)((BM + rb) * 4), (unsigned)(h * 8)};
    }
    __device__ static __forceinline__ unsigned scales(const unsigned (&S)[1], const mxf8_ctx_t &c) {
        const unsigned slot = (S[0] - c.lds0) / G::STAGE_BYTES;
        return c.lds_scale0 + slot * SCALE_STAGE;
    }
    __device__ static __forceinline__ void load_b(frag_t &f, const unsigned (&S)[1], const addr_t &ad,
            const mxf8_ctx_t &c, int g) {
        const unsigned sc = scales(S, c), sh = ad.shift + 16 * (g & 1);
#pragma unroll
        for (int j = 0; j < COLS; ++j) {
            f.b[j] = f8_mma_t<0, 0, G_>::read32(S[0] + ad.b0 + j * 2048, S[0] + ad.b1 + j * 2048);
            f.sb[j] = (int)((lds_read4(sc + ad.sb + j * 128) >> sh) & 0xffu);
        }
    }
    __device__ static __forceinline__ void load_a(frag_t &f, int i, const unsigned (&S)[1], const addr_t &ad,
            const mxf8_ctx_t &c, int g) {
        const unsigned sc = scales(S, c), sh = ad.shift + 16 * (g & 1);
        f.a[i] = f8_mma_t<0, 0, G_>::read32(S[0] + ad.a0 + i * 2048, S[0] + ad.a1 + i * 2048);
        f.sa[i] = (int)((lds_read4(sc + ad.sa + i * 128) >> sh) & 0xffu);
    }
    __device__ static __forceinline__ void mma_row(v16f (&acc)[ROWS][COLS], const frag_t &f, int i,
            const mxf8_ctx_t &, int) {
#pragma unroll
        for (int j = 0; j < COLS; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    f.b[j], f.a[i], acc[i][j], FMT_B, FMT_A, 0, f.sb[j], 0, f.sa[i]);
    }
};

typedef __bf16 v8bf_t __attribute__((ext_vector_type(8)));
typedef _Float16 v8h_t __attribute__((ext_vector_type(8)));

// bf16 (BF16) or f16 operands: the fp8 policy's addresses and reads; a fragment
// is its two 16-byte chunks, each the operand of one 32x32x16 instruction
template <bool BF16, class G_>
struct h16_mma_t {
    using G = G_;
    static constexpr int ELEM_BYTES = 2;
    static constexpr bool HOT = BF16; // the whole-row bf16 epilogue chains of the fp8 family
    static constexpr int EXTRA_DMAS = 0;
    __device__ static __forceinline__ void issue_extra(const f8_ctx_t &, int, int, int, int) {}
    static constexpr int ROWS = 4, COLS = G::WCOLS / 32, A_READS = 2, B_READS = 2;
    struct frag_t {
        v4i a[ROWS][2], b[COLS][2];
    };
    __device__ static __forceinline__ frag_t zero_frag() { return frag_t {}; }
    using addr_t = typename f8_mma_t<0, 0, G_>::addr_t;
    __device__ static __forceinline__ addr_t lane_addr(int wm, int wn, int lane) {
        return f8_mma_t<0, 0, G_>::lane_addr(wm, wn, lane);
    }
    __device__ static __forceinline__ void load_b(frag_t &f, const unsigned (&S)[1], const addr_t &ad,
            const f8_ctx_t &, int) {
#pragma unroll
        for (int j = 0; j < COLS; ++j) {
            f.b[j][0] = lds_read16(S[0] + ad.b0 + j * 2048);
            f.b[j][1] = lds_read16(S[0] + ad.b1 + j * 2048);
        }
    }
    __device__ static __forceinline__ void load_a(frag_t &f, int i, const unsigned (&S)[1], const addr_t &ad,
            const f8_ctx_t &, int) {
        f.a[i][0] = lds_read16(S[0] + ad.a0 + i * 2048);
        f.a[i][1] = lds_read16(S[0] + ad.a1 + i * 2048);
    }
    __device__ static __forceinline__ void mma_row(v16f (&acc)[ROWS][COLS], const frag_t &f, int i,
            const f8_ctx_t &, int) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < COLS; ++j) {
                // operands exchanged, as in the fp8 policy: the tile comes out transposed
                if constexpr (BF16)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf_t, f.b[j][h]),
                            __builtin_bit_cast(v8bf_t, f.a[i][h]), acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h_t, f.b[j][h]),
                            __builtin_bit_cast(v8h_t, f.a[i][h]), acc[i][j], 0, 0, 0);
            }
    }
};

// f32 x f32: a 64-byte stage is 16 elements of K, eight v_mfma_f32_32x32x2_f32 per
// fragment pair (instruction t takes dword t of the lane's eight: k = t from the
// lower half of the lanes, k = 8 + t from the upper one, on both operands alike).
// Eight times the matrix-core cycles of the other policies per stage: this one
// is bound by the f32 instruction's own rate (157 TFLOP/s), not by the data path.
template <class G_>
struct f32_mma_t {
    using G = G_;
    static constexpr int ELEM_BYTES = 4;
    static constexpr bool HOT = false;
    static constexpr int EXTRA_DMAS = 0;
    __device__ static __forceinline__ void issue_extra(const f8_ctx_t &, int, int, int, int) {}
    static constexpr int ROWS = 4, COLS = G::WCOLS / 32, A_READS = 2, B_READS = 2;
    struct frag_t {
        v8i a[ROWS], b[COLS];
    };
    __device__ static __forceinline__ frag_t zero_frag() { return frag_t {}; }
    using base_t = f8_mma_t<0, 0, G_>;
    using addr_t = typename base_t::addr_t;
    __device__ static __forceinline__ addr_t lane_addr(int wm, int wn, int lane) { return base_t::lane_addr(wm, wn, lane); }
    __device__ static __forceinline__ void load_b(frag_t &f, const unsigned (&S)[1], const addr_t &ad,
            const f8_ctx_t &, int) {
#pragma unroll
        for (int j = 0; j < COLS; ++j) f.b[j] = base_t::read32(S[0] + ad.b0 + j * 2048, S[0] + ad.b1 + j * 2048);
    }
    __device__ static __forceinline__ void load_a(frag_t &f, int i, const unsigned (&S)[1], const addr_t &ad,
            const f8_ctx_t &, int) {
        f.a[i] = base_t::read32(S[0] + ad.a0 + i * 2048, S[0] + ad.a1 + i * 2048);
    }
    __device__ static __forceinline__ void mma_row(v16f (&acc)[ROWS][COLS], const frag_t &f, int i,
            const f8_ctx_t &, int) {
#pragma unroll
        for (int t = 0; t < 8; ++t)
#pragma unroll
            for (int j = 0; j < COLS; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__int_as_float(f.b[j][t]), __int_as_float(f.a[i][t]),
                        acc[i][j], 0, 0, 0);
    }
};

// HOT: whether the kernel instantiation carries the compile-time specialised
// chains (e4m3 x e4m3 only: each one multiplies the code of the epilogue)
template <bool HOT>
struct f8_conv_t {
    typedef float row_t;
    float ssc_common;
    const void *ssc_p; // per-row src scales (already offset to this batch) or null
    int ssc_dt;
    bool with_src_sc, with_wei_sc;
    long bw;
    template <class PT>
    __device__ __forceinline__ void per_n(const PT &P, long, long n, float &wsc, int &, int &) const {
        if (with_wei_sc)
            wsc = load_float(P.wei_scale.dt, P.wei_scale.p, quant_off(P.wei_scale, bw, 0, n, P.K, P.N));
    }
    __device__ __forceinline__ float row_data(long m) const {
        return ssc_p ? load_float(ssc_dt, ssc_p, m) : ssc_common;
    }

    // The chain of the fp8 up-projection configuration and its subsets, fully
    // unrolled over the wavefront's 4 x 2 accumulator tiles with every choice a
    // template parameter:
    //   acc * src_scale * wei_scale[n]  [+ bias[n]]  [-> gelu_tanh]  [+ bf16 residual]  -> bf16
    //
    // Global memory sees whole 128-byte rows only.  In the accumulator layout a
    // lane owns 8 bytes of a dst row and a wavefront-wide access touches 32 rows,
    // 16 bytes each: the memory pipeline takes a cycle per row touched, and 512
    // such loads plus 512 such stores per tile cost ~10 us each.  Instead the
    // wavefront's 128 x 64 part of the residual (16 KB) comes into its own share
    // of the (now idle) tile ring by 16 direct-to-LDS DMAs of 8 whole rows, all in
    // flight at once; every quad is read from there, and the bf16 result is
    // written back over it (same lane, same address); at the end the part leaves
    // LDS as 16 stores of 8 whole rows.  LDS rows are 128 bytes with the eight
    // 16-byte chunks XOR-swizzled by the row number (on the global-address side of
    // the DMA and of the final stores), which keeps both access patterns free of
    // bank conflicts.
    template <bool BIAS, bool GELU, bool ADD, class PT, int C>
    __device__ __forceinline__ void hot_store(const PT &P, const epi_uniform_t &H, unsigned ntab, unsigned lds_part,
            const v16f (&acc)[4][C], long b, long m_base, long n_base, int col0) const {
        static_assert(C == 2, "a wavefront's part is 128 rows of 128 bytes");
        typedef unsigned v2u_t __attribute__((ext_vector_type(2)));
        typedef unsigned v4u_t __attribute__((ext_vector_type(4)));
        typedef v2u_t __attribute__((address_space(3), may_alias)) *lds_u2_ptr_t;
        typedef v4u_t __attribute__((address_space(3), may_alias)) *lds_u4_ptr_t;
        const int lane = threadIdx.x & 63, lrow = lane & 31, half = lane >> 5;
        const long rows_left = P.M - m_base; // > 0, checked by the caller
        // whole-row accesses: lane -> (row d * 8 + lane / 8, chunk slot lane % 8); the slot holds
        // the row's chunk slot ^ (row & 7)
        const int wr = lane >> 3, wslot = lane & 7;
        if (ADD) {
            const char *rbase = scalar_ptr(H.staged_p + (b * H.st_s0 + m_base * H.st_s1 + n_base) * 2);
#pragma unroll
            for (int d = 0; d < 16; ++d) {
                long r = d * 8 + wr;
                const int chunk = wslot ^ (int)(r & 7);
                r = r < rows_left ? r : rows_left - 1;
                dma16(rbase, (unsigned)(r * H.st_s1 * 2 + chunk * 16), lds_part + d * 1024);
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = u / 2, j = u % 2;
            if (ADD && j == 0) { // the four DMAs of this row block have landed
                if (i == 0) wait_vmcnt<12>();
                else if (i == 1) wait_vmcnt<8>();
                else if (i == 2) wait_vmcnt<4>();
                else wait_vmcnt<0>();
                asm volatile("" ::: "memory"); // no LDS read moves above the wait
            }
            const int r = 32 * i + lrow;
            float x[4][4];
            bool special = false;
            unsigned cell[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                cell[g] = lds_part + (unsigned)(r * 128 + (((4 * j + g) ^ (r & 7)) << 4) + 8 * half);
                // keeps the table reads of every tile apart: merged, the 32 columns'
                // operands of all tiles would stay in registers
                int col = col0 + 32 * j + 8 * g + 4 * half;
                asm volatile("" : "+v"(col));
                v4f_t w = {1.f, 1.f, 1.f, 1.f}, bb = {0.f, 0.f, 0.f, 0.f};
                if (with_wei_sc) w = nt4f(ntab, NT_WSC, col);
                if (BIAS) bb = nt4f(ntab, NT_BIAS, col);
                float y[4] = {0.f, 0.f, 0.f, 0.f};
                if (ADD) {
                    const v2u_t q = *(lds_u2_ptr_t)(size_t)cell[g];
                    y[0] = u2f(q.x << 16); y[1] = u2f(q.x & 0xffff0000u);
                    y[2] = u2f(q.y << 16); y[3] = u2f(q.y & 0xffff0000u);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float t = acc[i][j][4 * g + e];
                    if (with_src_sc) t *= ssc_common;
                    if (with_wei_sc) t *= w[e];
                    if (BIAS) t += bb[e];
                    if (GELU) t = gelu_tanh_fast(t);
                    if (ADD) t += y[e];
                    special |= __builtin_amdgcn_classf(t, 0x93); // NaN or subnormal: software conversion
                    x[g][e] = t;
                }
            }
            typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
            typedef float f32x2_t __attribute__((ext_vector_type(2)));
            v2u_t o[4];
            if (__builtin_amdgcn_ballot_w64(special) == 0) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    o[g].x = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_t {x[g][0], x[g][1]}, bf16x2_t));
                    o[g].y = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_t {x[g][2], x[g][3]}, bf16x2_t));
                }
            } else {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    o[g].x = f32_to_bf16(x[g][0]) | ((unsigned)f32_to_bf16(x[g][1]) << 16);
                    o[g].y = f32_to_bf16(x[g][2]) | ((unsigned)f32_to_bf16(x[g][3]) << 16);
                }
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) *(lds_u2_ptr_t)(size_t)cell[g] = o[g];
        }
        // the finished part, 8 whole rows per store
        char *dbase = (char *)P.dst + (b * P.ds[0] + m_base * P.ds[1] + n_base) * 2;
#pragma unroll
        for (int d = 0; d < 16; ++d) {
            const long r = d * 8 + wr;
            const int chunk = wslot ^ (int)(r & 7);
            const v4u_t q = *(lds_u4_ptr_t)(size_t)(lds_part + (unsigned)(d * 1024 + lane * 16));
            // written once, never read again by this launch: non-temporal
            if (r < rows_left) __builtin_nontemporal_store(q, (v4u_t *)(dbase + r * P.ds[1] * 2 + chunk * 16));
        }
    }
    template <class PT, int C>
    __device__ __forceinline__ bool hot_chain(const PT &P, const epi_uniform_t &H, unsigned ntab, unsigned lds_part,
            const v16f (&acc)[4][C], long b, long m_base, long n_base, int col0) const {
        if constexpr (C != 2) { // the whole-row chains are laid out for a 128 x 64 part
            return false;
        } else {
        if (m_base >= P.M) return true; // nothing of this wavefront's part is inside dst
        // 16-byte row pieces of dst and of the residual
        if (((uintptr_t)P.dst & 15) || (P.ds[0] % 8) || (P.ds[1] % 8)) return false;
        if (H.staged != STG_NONE && (((uintptr_t)H.staged_p & 15) || (H.st_s0 % 8) || (H.st_s1 % 8))) return false;
        if (!HOT || ssc_p || H.bias_mode == 2 || H.ds_mode != 0 || H.dzp_mode != 0 || H.dynamic || H.dst_dt != MI355_DT_BF16
                || H.n_po > 2)
            return false;
        auto is_gelu = [](const po_reg_t &r) {
            return r.kind == MI355_PO_ELTWISE && r.alg == MI355_ELTWISE_GELU_TANH && r.scale == 1.f;
        };
        auto is_res = [&](const po_reg_t &r, int i) {
            return r.kind == MI355_PO_BINARY && r.alg == MI355_BINARY_ADD && i == H.staged && H.staged_dt == MI355_DT_BF16;
        };
        bool gelu = false, add = false;
        if (H.n_po == 1) {
            gelu = is_gelu(H.pf0);
            add = is_res(H.pf0, 0);
            if (!gelu && !add) return false;
        } else if (H.n_po == 2) {
            gelu = is_gelu(H.pf0);
            add = is_res(H.pf1, 1);
            if (!gelu || !add) return false;
        }
        const bool bias = H.bias_mode == 1;
#define MI355_F8_HOT(B, G, A) hot_store<B, G, A>(P, H, ntab, lds_part, acc, b, m_base, n_base, col0)
        if (bias) {
            if (gelu) { if (add) MI355_F8_HOT(true, true, true); else MI355_F8_HOT(true, true, false); }
            else { if (add) MI355_F8_HOT(true, false, true); else MI355_F8_HOT(true, false, false); }
        } else {
            if (gelu) { if (add) MI355_F8_HOT(false, true, true); else MI355_F8_HOT(false, true, false); }
            else { if (add) MI355_F8_HOT(false, false, true); else MI355_F8_HOT(false, false, false); }
        }
#undef MI355_F8_HOT
        return true;
        }
    }
    __device__ __forceinline__ void quad(const v4i_t &raw, float ssc, unsigned ntab, int col, float (&f)[4]) const {
#pragma unroll
        for (int e = 0; e < 4; ++e) f[e] = __int_as_float(raw[e]);
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

extern __shared__ __attribute__((aligned(16))) char f8_smem[];

template <class Mma>
__global__ void __launch_bounds__(Mma::G::NT) __attribute__((amdgpu_waves_per_eu(Mma::G::NW * Mma::G::WG_PER_CU / 4))) f8_gemm_kernel(const problem_t P_, const f8_extra_t X) {
    using G = typename Mma::G;
    constexpr int EB = Mma::ELEM_BYTES;
    const auto &P = MI355_KERNARG_PROBLEM();
    char *smem = f8_smem;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = G::wm(wave), wn = G::wn(wave);
    const long b = blockIdx.z;
    const tile_pos_t tp = tile_position<G>((int)blockIdx.x, X.tiles_m, X.tiles_n);
    const long m0 = tp.m0, n0 = tp.n0;

    const long lda = P.ss[1] * EB; // bytes, like X.ldb and X.bt_bstride
    const char *A = (const char *)P.src + (P.ss[0] ? b * P.ss[0] * EB : 0) + m0 * lda;
    const char *Bt = X.bt + b * X.bt_bstride + n0 * X.ldb;

    const long bs = P.ss[0] ? b : 0, bw = P.ws[0] ? b : 0;
    f8_conv_t<Mma::HOT> cv;
    cv.with_src_sc = P.src_scale.dt != MI355_DT_UNDEF;
    cv.with_wei_sc = P.wei_scale.dt != MI355_DT_UNDEF;
    cv.ssc_common = 1.f;
    cv.ssc_p = nullptr;
    cv.ssc_dt = P.src_scale.dt;
    cv.bw = bw;
    if (cv.with_src_sc) {
        if (P.src_scale.mask & 2)
            cv.ssc_p = (const char *)P.src_scale.p
                    + ((P.src_scale.mask & 1) ? bs * P.M : 0) * (dt_bits(P.src_scale.dt) / 8);
        else
            cv.ssc_common = load_float(P.src_scale.dt, P.src_scale.p, (P.src_scale.mask & 1) ? bs : 0);
    }
    // the epilogue's per-column operands go into their LDS table now: the loads
    // hide behind the pipeline prologue
    const unsigned ntab = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem + NSTAGE * G::STAGE_BYTES;
    fill_ntab<G::NT>(P, cv, ntab, b, n0);

    v16f acc[Mma::ROWS][Mma::COLS];
#pragma unroll
    for (int i = 0; i < Mma::ROWS; ++i)
#pragma unroll
        for (int j = 0; j < Mma::COLS; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    main_loop<NSTAGE, KSTEP, Mma>(acc, smem, A, Bt, lda, X.ldb, P.M - m0,
            P.N - n0, (int)(P.K * EB / (BKB * KSTEP)), f8_ctx_t {});

    store_quadrant<layout32_t, G::WCOLS>(P, smem, ntab, acc, b, m0 + wm * 128, n0 + wn * G::WCOLS, wn * G::WCOLS, cv);
}

template <class Mma>
__global__ void __launch_bounds__(Mma::G::NT) __attribute__((amdgpu_waves_per_eu(Mma::G::NW * Mma::G::WG_PER_CU / 4))) mxf8_gemm_kernel(const problem_t P_, const f8_extra_t X) {
    using G = typename Mma::G;
    const auto &P = MI355_KERNARG_PROBLEM();
    char *smem = f8_smem;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = G::wm(wave), wn = G::wn(wave);
    const long b = blockIdx.z;
    const tile_pos_t tp = tile_position<G>((int)blockIdx.x, X.tiles_m, X.tiles_n);
    const long m0 = tp.m0, n0 = tp.n0;

    const long lda = P.ss[1];
    const long kb = P.K / 32; // scale bytes per row
    const char *A = (const char *)P.src + (P.ss[0] ? b * P.ss[0] : 0) + m0 * lda;
    const char *Bt = X.bt + b * X.bt_bstride + n0 * X.ldb;

    mxf8_ctx_t ctx;
    ctx.lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem;
    ctx.lds_scale0 = ctx.lds0 + NSTAGE * G::STAGE_BYTES;
    ctx.sa_tile = X.sa + b * X.sa_bstride + m0 * kb;
    ctx.sb_tile = X.sb + b * X.sb_bstride + n0 * kb;
    {
        long ra = wave * 64 + lane, rb = wave * 64 + lane;
        if (ra > P.M - m0 - 1) ra = P.M - m0 - 1;
        if (rb > P.N - n0 - 1) rb = P.N - n0 - 1;
        ctx.voff_a = (unsigned)(ra * kb);
        ctx.voff_b = (unsigned)(rb * kb);
    }
    f8_conv_t<false> cv;
    cv.with_src_sc = cv.with_wei_sc = false; // the scales are operands of the instruction
    cv.ssc_common = 1.f;
    cv.ssc_p = nullptr;
    cv.ssc_dt = MI355_DT_UNDEF;
    cv.bw = 0;
    const unsigned ntab = ctx.lds_scale0 + NSTAGE * Mma::SCALE_STAGE;
    fill_ntab<G::NT>(P, cv, ntab, b, n0);

    v16f acc[Mma::ROWS][Mma::COLS];
#pragma unroll
    for (int i = 0; i < Mma::ROWS; ++i)
#pragma unroll
        for (int j = 0; j < Mma::COLS; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    main_loop<NSTAGE, KSTEP, Mma>(acc, smem, A, Bt, lda, X.ldb, P.M - m0, P.N - n0, (int)(P.K / (BKB * KSTEP)), ctx);

    store_quadrant<layout32_t, G::WCOLS>(P, smem, ntab, acc, b, m0 + wm * 128, n0 + wn * G::WCOLS, wn * G::WCOLS, cv);
}

struct f8_plan_t {
    bool need_transpose, mx;
    size_t off_sb, total;
    long Bw, Bsb;
};

// MX: e8m0 scales per 32 consecutive k on both operands
bool f8_is_mx(const mi355_matmul_desc_t &d) {
    const mi355_quant_t &ss = d.src_scale, &ws = d.wei_scale;
    return ss.dt == MI355_DT_E8M0 && (ss.mask & 6) == 6 && ss.group[0] == 1 && ss.group[1] == 32
            && ws.dt == MI355_DT_E8M0 && (ws.mask & 6) == 6 && ws.group[0] == 32 && ws.group[1] == 1;
}

f8_plan_t make_plan(const mi355_matmul_desc_t &d) {
    f8_plan_t p {};
    p.Bw = d.wei_stride[0] ? d.batch : 1;
    p.need_transpose = !(d.wei_stride[1] == 1);
    p.mx = f8_is_mx(d);
    p.Bsb = (d.wei_scale.mask & 1) ? p.Bw : 1;
    size_t off = p.need_transpose ? align_up((size_t)p.Bw * d.N * d.K, 256) : 0;
    p.off_sb = off;
    if (p.mx) off += align_up((size_t)p.Bsb * d.N * (d.K / 32), 256); // weights scales as [N][K/32]
    p.total = off;
    return p;
}

} // namespace

int f8_supported(const mi355_matmul_desc_t &d) {
    if (!is_f8_dt(d.src_dt) || !is_f8_dt(d.wei_dt)) return MI355_UNIMPLEMENTED;
    if (dt_bits(d.dst_dt) < 8) return MI355_UNIMPLEMENTED;
    if (d.K < BKB * KSTEP || d.K % (BKB * KSTEP) != 0) return MI355_UNIMPLEMENTED;
    if (d.src_stride[2] != 1 || d.src_stride[1] % 16 != 0 || d.src_stride[0] % 16 != 0)
        return MI355_UNIMPLEMENTED;
    const bool k_major = d.wei_stride[1] == 1 && d.wei_stride[2] % 16 == 0 && d.wei_stride[0] % 16 == 0;
    const bool n_major = d.wei_stride[2] == 1;
    if (!k_major && !n_major) return MI355_UNIMPLEMENTED;
    // no zero points on this path, scales without groups and without a K mask
    if (!quant_absent(d.src_zp) || !quant_absent(d.wei_zp) || !quant_absent(d.src_pr))
        return MI355_UNIMPLEMENTED;
    if (f8_is_mx(d)) {
        // a stage fetches the dword that holds its two scale bytes: rows of whole dwords, static dst quantization
        if (d.K % 128 != 0 || d.dst_scale_dynamic != MI355_DST_DYNAMIC_NONE) return MI355_UNIMPLEMENTED;
        if (d.batch > 65535) return MI355_UNIMPLEMENTED;
        return MI355_SUCCESS;
    }
    if (!quant_absent(d.src_scale)
            && ((d.src_scale.mask & 4) || d.src_scale.group[0] > 1 || d.src_scale.group[1] > 1))
        return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.wei_scale)
            && ((d.wei_scale.mask & 2) || d.wei_scale.group[0] > 1 || d.wei_scale.group[1] > 1))
        return MI355_UNIMPLEMENTED;
    if (d.batch > 65535) return MI355_UNIMPLEMENTED;
    return MI355_SUCCESS;
}

size_t f8_scratch_bytes(const mi355_matmul_desc_t &d) {
    return make_plan(d).total;
}

int f8_launch(const mi355_matmul_desc_t &d, const problem_t &P, void *scratch, hipStream_t stream) {
    const f8_plan_t plan = make_plan(d);
    if (plan.total > 0 && !scratch) {
        set_error("mfma_f8: %zu bytes of scratch required", plan.total);
        return MI355_INVALID_ARGUMENTS;
    }
    f8_extra_t X {};
    if (plan.need_transpose) {
        transpose_bytes(P.wei, d.K, d.N, d.wei_stride[1], d.wei_stride[0], scratch, d.K, d.N * d.K,
                plan.Bw, stream);
        X.bt = (const char *)scratch;
        X.ldb = d.K;
        X.bt_bstride = plan.Bw > 1 ? d.N * d.K : 0;
    } else {
        X.bt = (const char *)P.wei;
        X.ldb = d.wei_stride[2];
        X.bt_bstride = d.wei_stride[0];
    }
    X.tiles_m = (int)((d.M + BM - 1) / BM);
    X.tiles_n = (int)((d.N + f8_geo_t::BN - 1) / f8_geo_t::BN);
    dim3 grid((unsigned)(X.tiles_m * X.tiles_n), 1, (unsigned)d.batch);
    constexpr int smem_bytes = NSTAGE * f8_geo_t::STAGE_BYTES + NTAB_BYTES;
    auto go = [&](auto kern) -> int {
        if (const int st = ensure_dynamic_lds((const void *)kern, smem_bytes, "mfma_f8")) return st;
        hipLaunchKernelGGL(kern, grid, dim3(f8_geo_t::NT), smem_bytes, stream, P, X);
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
    };
    const int fa = d.src_dt == MI355_DT_F8_E5M2, fb = d.wei_dt == MI355_DT_F8_E5M2;
    if (plan.mx) {
        if (((uintptr_t)P.src_scale.p & 3) != 0) {
            set_error("mfma_f8: MX src scales must be 4-byte aligned");
            return MI355_INVALID_ARGUMENTS;
        }
        const long kb = d.K / 32;
        char *sb = (char *)scratch + plan.off_sb;
        transpose_bytes(P.wei_scale.p, kb, d.N, d.N, kb * d.N, sb, kb, d.N * kb, plan.Bsb, stream);
        X.sb = sb;
        X.sb_bstride = plan.Bsb > 1 ? d.N * kb : 0;
        X.sa = (const char *)P.src_scale.p;
        X.sa_bstride = ((d.src_scale.mask & 1) && d.src_stride[0]) ? d.M * kb : 0;
        constexpr int mx_smem = NSTAGE * mxf8_geo_t::STAGE_BYTES + NSTAGE * (BM + mxf8_geo_t::BN) * 4 + NTAB_BYTES;
        static_assert(mxf8_geo_t::NSTAGE == NSTAGE && mxf8_geo_t::BN == f8_geo_t::BN, "one ring depth and tile width");
        auto go_mx = [&](auto kern) -> int {
            if (const int st = ensure_dynamic_lds((const void *)kern, mx_smem, "mfma_f8")) return st;
            hipLaunchKernelGGL(kern, grid, dim3(mxf8_geo_t::NT), mx_smem, stream, P, X);
            return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
        };
        if (fa && fb) return go_mx(mxf8_gemm_kernel<mxf8_mma_t<1, 1, true, mxf8_geo_t>>);
        if (fa) return go_mx(mxf8_gemm_kernel<mxf8_mma_t<1, 0, true, mxf8_geo_t>>);
        if (fb) return go_mx(mxf8_gemm_kernel<mxf8_mma_t<0, 1, true, mxf8_geo_t>>);
        return go_mx(mxf8_gemm_kernel<mxf8_mma_t<0, 0, true, mxf8_geo_t>>);
    }
    if (fa && fb) return go(f8_gemm_kernel<f8_mma_t<1, 1, f8_geo_t>>);
    if (fa) return go(f8_gemm_kernel<f8_mma_t<1, 0, f8_geo_t>>);
    if (fb) return go(f8_gemm_kernel<f8_mma_t<0, 1, f8_geo_t>>);
    return go(f8_gemm_kernel<f8_mma_t<0, 0, f8_geo_t>>);
}

// ---- bf16 / f16 / f32
static bool h16_k_major(const mi355_matmul_desc_t &d) {
    const int AL = 16 / (dt_bits(d.src_dt) / 8);
    return d.wei_stride[1] == 1 && d.wei_stride[2] % AL == 0 && d.wei_stride[0] % AL == 0;
}

int h16_supported(const mi355_matmul_desc_t &d) {
    if (d.src_dt != d.wei_dt || (d.src_dt != MI355_DT_BF16 && d.src_dt != MI355_DT_F16 && d.src_dt != MI355_DT_F32))
        return MI355_UNIMPLEMENTED;
    if (dt_bits(d.dst_dt) < 8) return MI355_UNIMPLEMENTED;
    const int EB = dt_bits(d.src_dt) / 8;   // bytes per element
    const int KE = BKB * KSTEP / EB, AL = 16 / EB; // elements of K per stage; elements per 16 bytes
    if (d.K < KE || d.K % KE != 0) return MI355_UNIMPLEMENTED;
    // 16-byte row pieces
    if (d.src_stride[2] != 1 || d.src_stride[1] % AL != 0 || d.src_stride[0] % AL != 0) return MI355_UNIMPLEMENTED;
    // K-contiguous weights (what format_tag::any resolves to) are read in place; N-contiguous ones are
    // transposed into scratch by a pre-pass of every launch
    const bool k_major = h16_k_major(d);
    const bool n_major = d.wei_stride[2] == 1;
    if (!k_major && !n_major) return MI355_UNIMPLEMENTED;
    // byte offsets inside a tile are 32-bit
    const long ldb = k_major ? d.wei_stride[2] : d.K;
    if (d.src_stride[1] * EB * BM >= (1L << 31) || ldb * EB * f8_geo_t::BN >= (1L << 31)) return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.src_zp) || !quant_absent(d.wei_zp) || !quant_absent(d.src_pr)) return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.src_scale)
            && ((d.src_scale.mask & 4) || d.src_scale.group[0] > 1 || d.src_scale.group[1] > 1))
        return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.wei_scale)
            && ((d.wei_scale.mask & 2) || d.wei_scale.group[0] > 1 || d.wei_scale.group[1] > 1))
        return MI355_UNIMPLEMENTED;
    if (d.batch > 65535) return MI355_UNIMPLEMENTED;
    return MI355_SUCCESS;
}

size_t h16_scratch_bytes(const mi355_matmul_desc_t &d) {
    const long Bw = d.wei_stride[0] ? d.batch : 1;
    return h16_k_major(d) ? 0 : align_up((size_t)Bw * d.N * d.K * (dt_bits(d.src_dt) / 8), 256);
}

int h16_launch(const mi355_matmul_desc_t &d, const problem_t &P, void *scratch, hipStream_t stream) {
    f8_extra_t X {};
    const long EB = dt_bits(d.src_dt) / 8;
    const size_t need = h16_scratch_bytes(d);
    if (need > 0) {
        if (!scratch) {
            set_error("mfma_h16: %zu bytes of scratch required", need);
            return MI355_INVALID_ARGUMENTS;
        }
        // [Bw][K][N] with N contiguous -> [Bw][N][K] with K contiguous: the reorder's tiled kernel
        const long Bw = d.wei_stride[0] ? d.batch : 1;
        mi355_reorder_desc_t rd {};
        rd.ndims = 3;
        rd.src_dt = rd.dst_dt = d.wei_dt;
        rd.dims[0] = Bw; rd.dims[1] = d.K; rd.dims[2] = d.N;
        rd.src_stride[0] = d.wei_stride[0]; rd.src_stride[1] = d.wei_stride[1]; rd.src_stride[2] = 1;
        rd.dst_stride[0] = d.N * d.K; rd.dst_stride[1] = 1; rd.dst_stride[2] = d.K;
        rd.src_scale.group[0] = rd.src_scale.group[1] = rd.dst_scale.group[0] = rd.dst_scale.group[1] = 1;
        rd.src_zp.group[0] = rd.src_zp.group[1] = rd.dst_zp.group[0] = rd.dst_zp.group[1] = 1;
        mi355_reorder_args_t ra {};
        ra.src = P.wei;
        ra.dst = scratch;
        if (const int st = mi355_reorder_launch(&rd, &ra, stream)) return st;
        X.bt = (const char *)scratch;
        X.ldb = d.K * EB;
        X.bt_bstride = Bw > 1 ? d.N * d.K * EB : 0;
    } else {
        X.bt = (const char *)P.wei;
        X.ldb = d.wei_stride[2] * EB;
        X.bt_bstride = d.wei_stride[0] * EB;
    }
    X.tiles_m = (int)((d.M + BM - 1) / BM);
    X.tiles_n = (int)((d.N + f8_geo_t::BN - 1) / f8_geo_t::BN);
    dim3 grid((unsigned)(X.tiles_m * X.tiles_n), 1, (unsigned)d.batch);
    constexpr int smem_bytes = NSTAGE * f8_geo_t::STAGE_BYTES + NTAB_BYTES;
    auto go = [&](auto kern) -> int {
        if (const int st = ensure_dynamic_lds((const void *)kern, smem_bytes, "mfma_h16")) return st;
        hipLaunchKernelGGL(kern, grid, dim3(f8_geo_t::NT), smem_bytes, stream, P, X);
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
    };
    if (d.src_dt == MI355_DT_BF16) return go(f8_gemm_kernel<h16_mma_t<true, f8_geo_t>>);
    if (d.src_dt == MI355_DT_F32) return go(f8_gemm_kernel<f32_mma_t<f8_geo_t>>);
    return go(f8_gemm_kernel<h16_mma_t<false, f8_geo_t>>);
}

} // namespace mi355
