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
// each of its 64 rows; weights scales [K/32][N] are transposed to [N][K/32]
// by a pre-pass so both sides look alike.
#include "gemm_core.hpp"

namespace mi355 {
namespace {

using namespace gemm;
using mx_geo_t = geo_t<4, 256>;
constexpr int NSTAGE = mx_geo_t::NSTAGE;
constexpr int SCALE_OFF = NSTAGE * mx_geo_t::STAGE_BYTES; // scale ring after the tile ring
constexpr int SCALE_STAGE = (BM + mx_geo_t::BN) * 4;      // 256 dwords A + BN dwords B
constexpr int SMEM_RING_BYTES = SCALE_OFF + NSTAGE * SCALE_STAGE;
constexpr int SMEM_BYTES = SMEM_RING_BYTES + NTAB_BYTES;

struct mxf4_extra_t {
    const char *bt;       // weights [N][K/2] bytes
    long ldb, bt_bstride; // bytes
    const char *sa;       // src scales [M][K/32] bytes, this batch added in-kernel
    const char *sb;       // weights scales [N][K/32] bytes (transposed copy)
    long sa_bstride, sb_bstride;
    int tiles_m, tiles_n;
};

struct mxf4_ctx_t {
    const char *sa_tile, *sb_tile; // first scale byte of tile row 0
    unsigned voff_a, voff_b;       // this lane's row offset in the scale arrays
    const char *s_tile;            // eight wavefronts: the one operand this wavefront brings
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
            dma4(c.sa_tile + (long)g * 4, c.voff_a, dst);
            dma4(c.sb_tile + (long)g * 4, c.voff_b,
                    c.lds_scale0 + slot * SCALE_STAGE + 1024 + (wave % BBLK) * 256);
        } else {
            dma4(c.s_tile + (long)g * 4, c.voff_s, dst);
        }
    }
    static constexpr int ROWS = 8, COLS = G::WCOLS / 16, A_READS = 2, B_READS = 2; // data + scale dword
    struct frag_t {
        v4i a[ROWS], b[COLS];
        int sa[ROWS], sb[COLS];
    };
    __device__ static __forceinline__ frag_t zero_frag() { return frag_t {}; } // e2m1 zero is all-zero bits
    // LDS byte address of the scale dwords that belong to the stage at S[0]
    __device__ static __forceinline__ unsigned scales(const unsigned (&S)[1], const mxf4_ctx_t &c) {
        const unsigned slot = (S[0] - c.lds0) / G::STAGE_BYTES;
        return c.lds_scale0 + slot * SCALE_STAGE;
    }
    // Per-lane LDS offsets of fragment 0 (data) and of its scale dword, and the
    // bit position of this lane's scale byte; fragment i is 16 rows further.
    struct addr_t {
        unsigned a, b, sa, sb, shift;
    };
    __device__ static __forceinline__ addr_t lane_addr(int wm, int wn, int lane) {
        const int frow = lane & 15, q = lane >> 4;
        const int ra = wm * 128 + frow, rb = wn * G::WCOLS + frow;
        return addr_t {(unsigned)swz(ra, q), (unsigned)(B_OFF + swz(rb, q)), (unsigned)(ra * 4),
                (unsigned)((256 + rb) * 4), (unsigned)(q * 8)};
    }
    __device__ static __forceinline__ void load_b(frag_t &f, const unsigned (&S)[1], const addr_t &ad,
            const mxf4_ctx_t &c, int) {
        const unsigned sc = scales(S, c);
#pragma unroll
        for (int j = 0; j < COLS; ++j) {
            f.b[j] = lds_read16(S[0] + ad.b + j * 1024);
            f.sb[j] = (int)((lds_read4(sc + ad.sb + j * 64) >> ad.shift) & 0xffu);
        }
    }
    __device__ static __forceinline__ void load_a(frag_t &f, int i, const unsigned (&S)[1], const addr_t &ad,
            const mxf4_ctx_t &c, int) {
        const unsigned sc = scales(S, c);
        f.a[i] = lds_read16(S[0] + ad.a + i * 1024);
        f.sa[i] = (int)((lds_read4(sc + ad.sa + i * 64) >> ad.shift) & 0xffu);
    }
    __device__ static __forceinline__ void mma_row(v4f (&acc)[ROWS][COLS], const frag_t &f, int i,
            const mxf4_ctx_t &, int) {
        const v8i a = {f.a[i][0], f.a[i][1], f.a[i][2], f.a[i][3], 0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < COLS; ++j) {
            const v8i bb = {f.b[j][0], f.b[j][1], f.b[j][2], f.b[j][3], 0, 0, 0, 0};
            // operands exchanged: the tile comes out transposed, a lane holds four
            // consecutive n of one row (tile_epilogue.hpp)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                    bb, a, acc[i][j], 4, 4, 0, f.sb[j], 0, f.sa[i]);
        }
    }
};

struct mxf4_conv_t {
    typedef int row_t;
    template <class PT>
    __device__ __forceinline__ void per_n(const PT &, long, long, float &, int &, int &) const {}
    __device__ __forceinline__ int row_data(long) const { return 0; }
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
    const long kb = P.K / 32;     // scale bytes per row
    const char *A = (const char *)P.src + (P.ss[0] ? b * (P.ss[0] / 2) : 0) + m0 * lda;
    const char *Bt = X.bt + b * X.bt_bstride + n0 * X.ldb;

    mxf4_ctx_t ctx;
    ctx.lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem;
    ctx.lds_scale0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem + SCALE_OFF;
    ctx.sa_tile = X.sa + b * X.sa_bstride + m0 * kb;
    ctx.sb_tile = X.sb + b * X.sb_bstride + n0 * kb;
    {
        long ra = (wave & 3) * 64 + lane, rb = ((wave & 3) % (G::BN / 64)) * 64 + lane;
        if (ra > P.M - m0 - 1) ra = P.M - m0 - 1;
        if (rb > P.N - n0 - 1) rb = P.N - n0 - 1;
        ctx.voff_a = (unsigned)(ra * kb);
        ctx.voff_b = (unsigned)(rb * kb);
        const bool brings_a = __builtin_amdgcn_readfirstlane(wave) < 4; // uniform: the base stays scalar
        ctx.s_tile = brings_a ? ctx.sa_tile : ctx.sb_tile;
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

struct mxf4_plan_t {
    bool need_transpose;
    size_t off_bt, off_sb, total;
    long Bw, Bsb;
};

mxf4_plan_t make_plan(const mi355_matmul_desc_t &d) {
    mxf4_plan_t p {};
    p.Bw = d.wei_stride[0] ? d.batch : 1;
    p.Bsb = (d.wei_scale.mask & 1) ? p.Bw : 1;
    p.need_transpose = !(d.wei_stride[1] == 1);
    size_t off = 0;
    p.off_bt = off;
    if (p.need_transpose) off += align_up((size_t)p.Bw * d.N * d.K / 2, 256);
    p.off_sb = off;
    off += align_up((size_t)p.Bsb * d.N * (d.K / 32), 256);
    p.total = off;
    return p;
}

} // namespace

int mxf4_supported(const mi355_matmul_desc_t &d) {
    if (d.src_dt != MI355_DT_F4_E2M1 || d.wei_dt != MI355_DT_F4_E2M1) return MI355_UNIMPLEMENTED;
    if (dt_bits(d.dst_dt) < 8) return MI355_UNIMPLEMENTED;
    if (d.K < 128 || d.K % 128 != 0) return MI355_UNIMPLEMENTED;
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
    // weights scales [K/32][N] -> [N][K/32]
    const long kb = d.K / 32;
    transpose_bytes(P.wei_scale.p, kb, d.N, d.N, kb * d.N, sc + plan.off_sb, kb, d.N * kb, plan.Bsb,
            stream);
    X.sb = sc + plan.off_sb;
    X.sb_bstride = plan.Bsb > 1 ? d.N * kb : 0;
    X.sa = (const char *)P.src_scale.p;
    X.sa_bstride = ((d.src_scale.mask & 1) && d.src_stride[0]) ? d.M * kb : 0;
    X.tiles_m = (int)((d.M + BM - 1) / BM);
    X.tiles_n = (int)((d.N + mx_geo_t::BN - 1) / mx_geo_t::BN);
    dim3 grid((unsigned)(X.tiles_m * X.tiles_n), 1, (unsigned)d.batch);
    if (const int st = ensure_dynamic_lds((const void *)mxf4_gemm_kernel<mx_geo_t>, SMEM_BYTES, "mfma_mxf4")) return st;
    hipLaunchKernelGGL(mxf4_gemm_kernel<mx_geo_t>, grid, dim3(mx_geo_t::NT), SMEM_BYTES, stream, P, X);
    return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
}

} // namespace mi355
