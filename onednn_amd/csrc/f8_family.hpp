// What the fp8 family ("hip:mfma_f8", kern_f8.hip) and the unquantized float family ("hip:mfma_h16",
// kern_h16.hip) share: the kernel, templated over an operand policy; the fp8 policy, whose addresses and
// fragment reads the other policies reuse; the scale handling and the compile-time epilogue chains.
#pragma once
#include <type_traits>

#include "gemm_core.hpp"

namespace mi355 {
namespace {

using namespace gemm;
constexpr int KSTEP = 1;
using f8_geo_t = geo_t<8, 256>;
constexpr int NSTAGE = f8_geo_t::NSTAGE; // one stage (K = 64) per step

struct f8_extra_t {
    const char *bt; // weights as [N][K] bytes, K contiguous
    long ldb, bt_bstride;
    int tiles_m, tiles_n;
    // MX variant: the e8m0 scales per 32 k of both operands, packed by a pre-pass of the launch into the order the
    // wavefronts load them (mxf8_mma_t in kern_f8.hip); strides in bytes, nst = stages of K (a tail stage included)
    const char *sa, *sb;
    long sa_bstride, sb_bstride;
    int nst;
};

struct f8_ctx_t {};

// cbsz / blgp operand format codes of the f8f6f4 MFMA: 0 = e4m3, 1 = e5m2
template <int FMT_A, int FMT_B, class G_>
struct f8_mma_t {
    using G = G_;
    static constexpr int ELEM_BYTES = 1;
    static constexpr int HOT = FMT_A == 0 && FMT_B == 0 ? 2 : 0;
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
    // K that ends inside a stage (gemm_core.hpp tail_step): the lane's two chunks are
    // 2 (lane / 32) and the next one; chunks below nz are zeroed in both operands
    // (fp8 zero is all-zero bits; both, so that no Inf or NaN among the bytes that were
    // multiplied before meets a zero)
    static constexpr bool K_TAIL = true;
    __device__ static __forceinline__ void zero_tail(frag_t &f, int nz, int lane) {
        const int c0 = (lane >> 5) * 2;
        const bool z0 = c0 < nz, z1 = c0 + 1 < nz;
#pragma unroll
        for (int i = 0; i < ROWS; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                f.a[i][e] = z0 ? 0 : f.a[i][e];
                f.a[i][4 + e] = z1 ? 0 : f.a[i][4 + e];
            }
#pragma unroll
        for (int j = 0; j < COLS; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                f.b[j][e] = z0 ? 0 : f.b[j][e];
                f.b[j][4 + e] = z1 ? 0 : f.b[j][4 + e];
            }
    }
};

// HOT: whether the kernel instantiation carries the compile-time specialised
// chains (e4m3 x e4m3 only: each one multiplies the code of the epilogue): 0 none, 1 the gelu_tanh / residual
// ones, 2 the swish / gate ones as well
template <int HOT>
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
    // and, SW != 0 (the plain fp8 kernel only: HOT == 2), the gated feed-forward layer of the Llama family,
    //   ...  [+ bias[n]]  -> swish  [* bf16 gate (SW == 2)]  -> bf16
    //   ...  [+ bias[n]]  [-> gelu_tanh]  * bf16 gate (SW == 3: GeGLU, or a plain gate)  -> bf16
    // where ADD stands for "a staged bf16 operand".  (The SW == 0 instantiations are what the block-scaled
    // kernel carries, and their code is kept as it was: that kernel's main loop sits at the register limit and
    // any change to its epilogue moved spills into it, 0.55 -> 1.2 ms.)
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
    // 16-byte chunks XOR-swizzled by bits 1-3 of the row number (on the
    // global-address side of the DMA and of the final stores), which keeps both
    // access patterns free of bank conflicts.
    template <bool BIAS, bool GELU, bool ADD, int SW = 0, class PT, int C>
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
        // the row's chunk slot ^ ((row >> 1) & 7): a row is 32 banks, so bit 0 of the row picks
        // the half of the 64 banks and bits 1-3 the 16-byte slot inside it -- the 8-byte accesses
        // of the 32 rows of an accumulator tile then spread over all banks (with row & 7 they
        // used half of them: SQ_LDS_BANK_CONFLICT was 18 % of the LDS cycles of the kernel)
        const int wr = lane >> 3, wslot = lane & 7;
        if (ADD) {
            const char *rbase = scalar_ptr(H.staged_p + (b * H.st_s0 + m_base * H.st_s1 + n_base) * 2);
#pragma unroll
            for (int d = 0; d < 16; ++d) {
                long r = d * 8 + wr;
                const int chunk = wslot ^ (int)((r >> 1) & 7);
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
                cell[g] = lds_part + (unsigned)(r * 128 + (((4 * j + g) ^ ((r >> 1) & 7)) << 4) + 8 * half);
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
                    if (SW == 1 || SW == 2) t = t * logistic_fast(H.pf0.alpha * t);
                    if (ADD) {
                        if (SW >= 2) t *= y[e];
                        else t += y[e];
                    }
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
            const int chunk = wslot ^ (int)((r >> 1) & 7);
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
        if constexpr (HOT >= 2) {
            // swish, alone or followed by the multiplication with a staged bf16 tensor
            const bool swish = H.n_po >= 1 && H.pf0.kind == MI355_PO_ELTWISE && H.pf0.alg == MI355_ELTWISE_SWISH
                    && H.pf0.scale == 1.f;
            const bool gate = H.n_po == 2 && H.pf1.kind == MI355_PO_BINARY && H.pf1.alg == MI355_BINARY_MUL
                    && H.staged == 1 && H.staged_dt == MI355_DT_BF16;
            // gelu_tanh, or nothing, followed by that multiplication
            const bool gelu_first = H.n_po == 2 && H.pf0.kind == MI355_PO_ELTWISE && H.pf0.alg == MI355_ELTWISE_GELU_TANH
                    && H.pf0.scale == 1.f;
            const bool gate_alone = H.n_po == 1 && H.pf0.kind == MI355_PO_BINARY && H.pf0.alg == MI355_BINARY_MUL
                    && H.staged == 0 && H.staged_dt == MI355_DT_BF16;
            if ((gelu_first && gate) || gate_alone) {
                const bool with_bias = H.bias_mode == 1;
#define MI355_F8_GATED(B, G) hot_store<B, G, true, 3>(P, H, ntab, lds_part, acc, b, m_base, n_base, col0)
                if (with_bias) { if (gelu_first) MI355_F8_GATED(true, true); else MI355_F8_GATED(true, false); }
                else { if (gelu_first) MI355_F8_GATED(false, true); else MI355_F8_GATED(false, false); }
#undef MI355_F8_GATED
                return true;
            }
            if (swish && (H.n_po == 1 || gate)) {
                const bool with_bias = H.bias_mode == 1;
#define MI355_F8_GATED(B, A, S) hot_store<B, false, A, S>(P, H, ntab, lds_part, acc, b, m_base, n_base, col0)
                if (with_bias) { if (gate) MI355_F8_GATED(true, true, 2); else MI355_F8_GATED(true, false, 1); }
                else { if (gate) MI355_F8_GATED(false, true, 2); else MI355_F8_GATED(false, false, 1); }
#undef MI355_F8_GATED
                return true;
            }
        }
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
    // the 16 x 16 tiles of the 16-bit policies: whole rows for a plain bf16 dst (tile_epilogue.hpp)
    template <class PT>
    __device__ __forceinline__ bool hot_chain(const PT &P, const epi_uniform_t &H, unsigned, unsigned lds_part,
            const v4f (&acc)[8][4], long b, long m_base, long n_base, int) const {
        if (ssc_p || with_src_sc || with_wei_sc) return false;
        return store_rows_bf16_tile16(P, H, lds_part, acc, b, m_base, n_base);
    }
    // other accumulator shapes without compile-time chains
    template <class PT, class Acc>
    __device__ __forceinline__ bool hot_chain(const PT &, const epi_uniform_t &, unsigned, unsigned, const Acc &, long, long,
            long, int) const {
        return false;
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

// accumulator tile of a policy: 32 x 32 (sixteen registers) unless it declares TILE16
template <class Mma, class = void>
struct acc_of {
    typedef v16f type;
    typedef layout32_t layout;
    static constexpr int N = 16;
};
template <class Mma>
struct acc_of<Mma, std::enable_if_t<Mma::TILE16>> {
    typedef v4f type;
    typedef layout16_t layout;
    static constexpr int N = 4;
};

// block-scaled policies (MX = true) bring a context of their own and LDS behind the tile ring
template <class Mma, class = void>
struct mx_of : std::false_type {
    static constexpr int EXTRA_LDS = 0;
    __device__ static __forceinline__ f8_ctx_t make_ctx(const f8_extra_t &, unsigned, long, long, long, int) { return {}; }
};
template <class Mma>
struct mx_of<Mma, std::enable_if_t<Mma::MX>> : std::true_type {
    static constexpr int EXTRA_LDS = Mma::EXTRA_LDS;
    __device__ static __forceinline__ auto make_ctx(const f8_extra_t &X, unsigned lds0, long b, long m0, long n0, int wave) {
        return Mma::make_ctx(X, lds0, b, m0, n0, wave);
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
    // (block scales are operands of the instruction: nothing of them is left for the epilogue)
    cv.with_src_sc = !mx_of<Mma>::value && P.src_scale.dt != MI355_DT_UNDEF;
    cv.with_wei_sc = !mx_of<Mma>::value && P.wei_scale.dt != MI355_DT_UNDEF;
    cv.ssc_common = 1.f;
    cv.ssc_p = nullptr;
    cv.ssc_dt = mx_of<Mma>::value ? (int)MI355_DT_UNDEF : P.src_scale.dt;
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
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem;
    const unsigned ntab = lds0 + G::NSTAGE * G::STAGE_BYTES + mx_of<Mma>::EXTRA_LDS;
    fill_ntab<G::NT>(P, cv, ntab, b, n0);
    const auto ctx = mx_of<Mma>::make_ctx(X, lds0, b, m0, n0, __builtin_amdgcn_readfirstlane(wave));

    typename acc_of<Mma>::type acc[Mma::ROWS][Mma::COLS];
#pragma unroll
    for (int i = 0; i < Mma::ROWS; ++i)
#pragma unroll
        for (int j = 0; j < Mma::COLS; ++j)
#pragma unroll
            for (int r = 0; r < acc_of<Mma>::N; ++r) acc[i][j][r] = 0.f;

    const long kbytes = P.K * EB;
    main_loop<G::NSTAGE, KSTEP, Mma>(acc, smem, A, Bt, lda, X.ldb, P.M - m0,
            P.N - n0, (int)(kbytes / (BKB * KSTEP)), ctx);
    if constexpr (has_k_tail<Mma>::value) {
        // the rest of a K that is whole 16-byte chunks but not whole stages
        const int rem = (int)(kbytes % BKB);
        if (rem != 0)
            tail_step<Mma>(acc, smem, A + kbytes - BKB, Bt + kbytes - BKB, lda, X.ldb, P.M - m0, P.N - n0,
                    (BKB - rem) / 16, (int)(kbytes / BKB), ctx);
    }

    store_quadrant<typename acc_of<Mma>::layout, G::WCOLS>(P, smem, ntab, acc, b, m0 + wm * 128, n0 + wn * G::WCOLS,
            wn * G::WCOLS, cv);
}

} // namespace
} // namespace mi355
