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
#include <cstring>
#include "f8_family.hpp"

namespace mi355 {
namespace {

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
    // whole 16-byte chunks of K; a K that ends inside a 64-byte stage takes one unpipelined step more per tile
    if (d.K < BKB * KSTEP || d.K % 16 != 0) return MI355_UNIMPLEMENTED;
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
    // Up to 128 tiles leave half of the CUs or more idle: 256 x 128 tiles of four wavefronts, two workgroups a CU, put
    // twice as many to work (a wavefront's part, 128 x 64, its fragments and the epilogue are the same).  MI355_F8_TILES=wide keeps the 256 x 256 tiles.
    const int force = tuning(TUNE_F8_TILES); // wide / narrow: one geometry whatever the size (tests, tuning)
    if (force == TUNE_NARROW || ((long)X.tiles_m * X.tiles_n * d.batch <= 128 && d.N > 128 && force != TUNE_WIDE))
        return f8_launch_narrow(fa, fb, P, X.bt, X.ldb, X.bt_bstride, (unsigned)d.batch, stream);
    if (fa && fb) return go(f8_gemm_kernel<f8_mma_t<1, 1, f8_geo_t>>);
    if (fa) return go(f8_gemm_kernel<f8_mma_t<1, 0, f8_geo_t>>);
    if (fb) return go(f8_gemm_kernel<f8_mma_t<0, 1, f8_geo_t>>);
    return go(f8_gemm_kernel<f8_mma_t<0, 0, f8_geo_t>>);
}

} // namespace mi355
