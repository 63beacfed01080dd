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
//
// A 64-byte stage is two blocks; the instruction takes block h's scale from the lanes 32 h .. 32 h + 31 (lane
// l: row l % 32 of the fragment) and reads the first register halves of all lanes as k 0..31, the second halves
// as k 32..63 -- so a lane holds the 16-byte chunks h and 2 + h of the stage, not 2 h and 2 h + 1 as in the
// unscaled policy (established on the device: exact data with a scale of its own per block match the oracle bit
// for bit this way and differ the other way).  Which byte of the scale register counts is picked by op_sel.
//
// The scales reach a wavefront the way the MXFP4 family's do: a pre-pass of the launch packs them, per stage and
// block of rows, into the 64 dwords a wavefront loads for that stage -- dword l holds, for the lane's row l % 32 and
// block l / 32, the bytes of the block's up to four fragments (rows +0, +32, +64, +96) -- so that one 4-byte LDS
// read per operand and stage feeds all of a wavefront's MFMAs and no shift or mask touches the scales.  Blocks of
// 128 rows of src (a wavefront's four fragments), of 64 columns of weights (its two).  The packed scales of a
// stage -- 2 blocks of A, 4 of B^T, 256 bytes each -- ride along with the tile ring, one direct-to-LDS dword per
// lane and stage for six of the eight wavefronts (the other two repeat two of them: every wavefront issues the
// same number of loads per stage, which the loop's load counting relies on).  The geometry, loop and epilogue are
// the unscaled kernel's (eight wavefronts, whole-row bf16 chains); a K that ends inside a stage takes the family's
// tail step, the pre-pass giving that stage the scales of its window (K - 64 ..) with the neutral byte for the
// block that was multiplied before.
struct mxf8_ctx_t {
    const char *s_blk;     // packed scales of the block this wavefront brings in, stage 0
    unsigned lds_scale0;   // LDS byte address of the scale ring
    unsigned lds0;         // LDS byte address of the tile ring
};

template <int FMT_A, int FMT_B, class G_>
struct mxf8_mma_t {
    using G = G_;
    static constexpr int ELEM_BYTES = 1;
    static constexpr int HOT = FMT_A == 0 && FMT_B == 0 ? 1 : 0;
    static constexpr bool MX = true;
    static constexpr int EXTRA_DMAS = 1;
    static constexpr int SCALE_STAGE = 6 * 256; // two blocks of A, four of B^T
    static constexpr int EXTRA_LDS = G::NSTAGE * SCALE_STAGE;
    static_assert(G::NW == 8 && G::BN == 256 && BM == 256, "blocks of 128 rows / 64 columns per wavefront part");
    typedef mxf8_ctx_t ctx_t;
    // where wavefront `wave` puts its block inside a stage of the scale ring
    __device__ static __forceinline__ unsigned blk_off(int wave) {
        return wave >= 2 && wave < 6 ? 512u + (unsigned)(wave - 2) * 256u : (unsigned)(wave & 1) * 256u;
    }
    __device__ static __forceinline__ mxf8_ctx_t make_ctx(const f8_extra_t &X, unsigned lds0, long b, long m0, long n0,
            int wave) {
        mxf8_ctx_t c;
        c.lds0 = lds0;
        c.lds_scale0 = lds0 + G::NSTAGE * G::STAGE_BYTES;
        const bool of_b = wave >= 2 && wave < 6;
        const char *p = of_b ? X.sb + b * X.sb_bstride + ((n0 >> 6) + (wave - 2)) * (long)X.nst * 256
                             : X.sa + b * X.sa_bstride + ((m0 >> 7) + (wave & 1)) * (long)X.nst * 256;
        c.s_blk = scalar_ptr(p);
        return c;
    }
    __device__ static __forceinline__ void issue_extra(const mxf8_ctx_t &c, int g, int slot, int wave, int lane) {
        dma4(c.s_blk + (long)g * 256, (unsigned)lane * 4u, c.lds_scale0 + slot * SCALE_STAGE + blk_off(wave));
    }
    static constexpr int ROWS = 4, COLS = G::WCOLS / 32, A_READS = 3, B_READS = 3;
    static_assert(COLS == 2, "a wavefront's part is 128 x 64");
    struct frag_t {
        v8i a[ROWS], b[COLS];
        int sa, sb; // byte i: the scale of fragment i
    };
    __device__ static __forceinline__ frag_t zero_frag() { return frag_t {}; }
    struct addr_t {
        unsigned a0, a1, b0, b1, sa, sb;
    };
    __device__ static __forceinline__ addr_t lane_addr(int wm, int wn, int lane) {
        const int frow = lane & 31, h = lane >> 5;
        const int ra = wm * 128 + frow, rb = wn * G::WCOLS + frow;
        return addr_t {(unsigned)swz(ra, h), (unsigned)swz(ra, 2 + h), (unsigned)(B_OFF + swz(rb, h)),
                (unsigned)(B_OFF + swz(rb, 2 + h)), (unsigned)(wm * 256 + lane * 4), (unsigned)(512 + wn * 256 + lane * 4)};
    }
    __device__ static __forceinline__ unsigned scales(const unsigned (&S)[1], const mxf8_ctx_t &c) {
        const unsigned slot = (S[0] - c.lds0) / G::STAGE_BYTES;
        return c.lds_scale0 + slot * SCALE_STAGE;
    }
    __device__ static __forceinline__ void load_b(frag_t &f, const unsigned (&S)[1], const addr_t &ad,
            const mxf8_ctx_t &c, int) {
#pragma unroll
        for (int j = 0; j < COLS; ++j)
            f.b[j] = f8_mma_t<0, 0, G_>::read32(S[0] + ad.b0 + j * 2048, S[0] + ad.b1 + j * 2048);
        f.sb = (int)lds_read4(scales(S, c) + ad.sb);
    }
    __device__ static __forceinline__ void load_a(frag_t &f, int i, const unsigned (&S)[1], const addr_t &ad,
            const mxf8_ctx_t &c, int) {
        f.a[i] = f8_mma_t<0, 0, G_>::read32(S[0] + ad.a0 + i * 2048, S[0] + ad.a1 + i * 2048);
        if (i == 0) f.sa = (int)lds_read4(scales(S, c) + ad.sa);
    }
    template <int I, int J>
    __device__ static __forceinline__ void mma_one(v16f (&acc)[ROWS][COLS], const frag_t &f) {
        // operands exchanged as in the unscaled policy: weights first
        acc[I][J] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.b[J], f.a[I], acc[I][J], FMT_B, FMT_A, J, f.sb, I, f.sa);
    }
    __device__ static __forceinline__ void mma_row(v16f (&acc)[ROWS][COLS], const frag_t &f, int i,
            const mxf8_ctx_t &, int) {
        switch (i) {
            case 0: mma_one<0, 0>(acc, f); mma_one<0, 1>(acc, f); break;
            case 1: mma_one<1, 0>(acc, f); mma_one<1, 1>(acc, f); break;
            case 2: mma_one<2, 0>(acc, f); mma_one<2, 1>(acc, f); break;
            default: mma_one<3, 0>(acc, f); mma_one<3, 1>(acc, f); break;
        }
    }
    // K that ends inside a stage (gemm_core.hpp tail_step): the lane's chunks are h and 2 + h; chunks below nz
    // are zeroed in both operands (their block's scale in the packed tail stage is the neutral byte)
    static constexpr bool K_TAIL = true;
    __device__ static __forceinline__ void zero_tail(frag_t &f, int nz, int lane) {
        const int h = lane >> 5;
        const bool z0 = h < nz, z1 = 2 + h < nz;
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

// The pre-pass: dword (block, stage g, lane l) of the packed scales holds, in byte i < frags, the scale of row
// 32 * frags * block + 32 i + l % 32 for the stage's block l / 32 (blocks 2 g, 2 g + 1 of the row; the tail stage
// of a K that is an odd number of blocks covers blocks kb - 2, kb - 1 and gives the first one, multiplied before,
// the neutral byte); rows beyond the tensor and unused bytes hold the neutral byte too.  `in`: e8m0 bytes, element
// (row, block) at row * row_stride + block * k_stride (src scales [M][K/32], weights scales [K/32][N]).
__global__ void __launch_bounds__(256) mxf8_pack_scales_kernel(const uint8_t *in, long rows, long kb, long row_stride,
        long k_stride, long in_bstride, uint32_t *out, long out_bstride, int nst, int frags, long nblk) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= nblk * nst * 64) return;
    const int l = (int)(idx & 63), h = l >> 5;
    const long g = (idx >> 6) % nst, blk = (idx >> 6) / nst;
    const long full = kb / 2;
    const long kblk = g < full ? 2 * g + h : (h == 0 ? -1 : kb - 1);
    const uint8_t *src = in + (long)blockIdx.y * in_bstride;
    uint32_t word = 0;
    for (int i = 0; i < 4; ++i) {
        const long row = blk * 32 * frags + 32 * i + (l & 31);
        uint32_t byte = 127;
        if (i < frags && row < rows && kblk >= 0) byte = src[row * row_stride + kblk * k_stride];
        word |= byte << (8 * i);
    }
    out[(long)blockIdx.y * out_bstride + idx] = word;
}

struct f8_plan_t {
    bool need_transpose, mx;
    size_t off_sa, off_sb, total;
    long Bw, Bsa, Bsb;
    long nst, blk_a, blk_b; // MX: stages of K, blocks of 128 src rows / 64 columns
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
    p.Bsa = ((d.src_scale.mask & 1) && d.src_stride[0]) ? d.batch : 1;
    size_t off = p.need_transpose ? align_up((size_t)p.Bw * d.N * d.K, 256) : 0;
    if (p.mx) { // the packed scales of both operands
        p.nst = (d.K + BKB - 1) / BKB;
        p.blk_a = (d.M + 127) / 128 + 1; // (a tile of 256 rows reads two blocks whatever M is)
        p.blk_b = (d.N + 255) / 256 * 4;
        p.off_sa = off;
        off += align_up((size_t)p.Bsa * p.blk_a * p.nst * 256, 256);
        p.off_sb = off;
        off += align_up((size_t)p.Bsb * p.blk_b * p.nst * 256, 256);
    }
    p.total = off;
    return p;
}

} // namespace

int f8_supported(const mi355_matmul_desc_t &d) {
    if (!is_f8_dt(d.src_dt) || !is_f8_dt(d.wei_dt)) return MI355_UNIMPLEMENTED;
    if (dt_bits(d.dst_dt) < 8 && !tile_nibble_dst_ok(d)) return MI355_UNIMPLEMENTED;
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
        // whole blocks of 32 k (a K that ends inside a 64-byte stage takes the tail step), static dst quantization
        if (d.K % 32 != 0 || d.dst_scale_dynamic != MI355_DST_DYNAMIC_NONE) return MI355_UNIMPLEMENTED;
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
        const long kb = d.K / 32;
        char *sa = (char *)scratch + plan.off_sa, *sb = (char *)scratch + plan.off_sb;
        auto pack = [&](const void *in, long rows, long row_stride, long k_stride, long in_bstride, char *out, int frags,
                            long nblk, long batches) {
            const long n = nblk * plan.nst * 64;
            hipLaunchKernelGGL(mxf8_pack_scales_kernel, dim3((unsigned)((n + 255) / 256), (unsigned)batches), dim3(256), 0,
                    stream, (const uint8_t *)in, rows, kb, row_stride, k_stride, in_bstride, (uint32_t *)out, n,
                    (int)plan.nst, frags, nblk);
        };
        pack(P.src_scale.p, d.M, kb, 1, d.M * kb, sa, 4, plan.blk_a, plan.Bsa);
        pack(P.wei_scale.p, d.N, 1, d.N, kb * d.N, sb, 2, plan.blk_b, plan.Bsb);
        if (hipGetLastError() != hipSuccess) return MI355_RUNTIME_ERROR;
        X.sa = sa;
        X.sb = sb;
        X.sa_bstride = plan.Bsa > 1 ? plan.blk_a * plan.nst * 256 : 0;
        X.sb_bstride = plan.Bsb > 1 ? plan.blk_b * plan.nst * 256 : 0;
        X.nst = (int)plan.nst;
        constexpr int mx_smem = NSTAGE * f8_geo_t::STAGE_BYTES + mxf8_mma_t<0, 0, f8_geo_t>::EXTRA_LDS + NTAB_BYTES;
        auto go_mx = [&](auto kern) -> int {
            if (const int st = ensure_dynamic_lds((const void *)kern, mx_smem, "mfma_f8")) return st;
            hipLaunchKernelGGL(kern, grid, dim3(f8_geo_t::NT), mx_smem, stream, P, X);
            return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
        };
        if (fa && fb) return go_mx(f8_gemm_kernel<mxf8_mma_t<1, 1, f8_geo_t>>);
        if (fa) return go_mx(f8_gemm_kernel<mxf8_mma_t<1, 0, f8_geo_t>>);
        if (fb) return go_mx(f8_gemm_kernel<mxf8_mma_t<0, 1, f8_geo_t>>);
        return go_mx(f8_gemm_kernel<mxf8_mma_t<0, 0, f8_geo_t>>);
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
