// "hip:mfma_h16" -- the same tiles for bf16 x bf16, f16 x f16 and f32 x f32 operands
// (ref_matmul_t's f32 sum of exact products): a 64-byte stage is 32 elements of
// K, one v_mfma_f32_16x16x32_{bf16,f16} per pair of 16-row fragments, in the
// matrix cycles of the fp8 family's instruction per stage, so the data path
// (DMA, LDS ring, epilogue) is shared unchanged.
#include "f8_family.hpp"

namespace mi355 {
namespace {

typedef __bf16 v8bf_t __attribute__((ext_vector_type(8)));
typedef _Float16 v8h_t __attribute__((ext_vector_type(8)));

// bf16 (BF16) or f16 operands on the 16 x 16 x 32 instruction: a lane's one
// 16-byte chunk of a stage (row lane % 16, chunk lane / 16) is the whole
// operand.  The 32 x 32 x 16 shape (two instructions per fragment pair of the
// fp8 policy's layout) costs the same matrix cycles and LDS bytes per stage, but
// sustains 1.53 instead of 1.85 PFLOP/s on random operand bits (the clock the
// power manager allows, `bench.py --calib-mfma`): 0.90 against 0.84 ms on
// 8192^3, the fp8 family's whole-row bf16 epilogue included.
template <bool BF16, class G_>
struct h16x16_mma_t {
    using G = G_;
    static constexpr bool TILE16 = true;
    static constexpr int ELEM_BYTES = 2;
    static constexpr bool HOT = false;
    static constexpr int EXTRA_DMAS = 0;
    __device__ static __forceinline__ void issue_extra(const f8_ctx_t &, int, int, int, int) {}
    static constexpr int ROWS = 8, COLS = G::WCOLS / 16, A_READS = 1, B_READS = 1;
    struct frag_t {
        v4i a[ROWS], b[COLS];
    };
    __device__ static __forceinline__ frag_t zero_frag() { return frag_t {}; }
    struct addr_t {
        unsigned a, b;
    };
    __device__ static __forceinline__ addr_t lane_addr(int wm, int wn, int lane) {
        const int frow = lane & 15, q = lane >> 4;
        const int ra = wm * 128 + frow, rb = wn * G::WCOLS + frow;
        return addr_t {(unsigned)swz(ra, q), (unsigned)(B_OFF + swz(rb, q))};
    }
    __device__ static __forceinline__ void load_b(frag_t &f, const unsigned (&S)[1], const addr_t &ad,
            const f8_ctx_t &, int) {
#pragma unroll
        for (int j = 0; j < COLS; ++j) f.b[j] = lds_read16(S[0] + ad.b + j * 1024);
    }
    __device__ static __forceinline__ void load_a(frag_t &f, int i, const unsigned (&S)[1], const addr_t &ad,
            const f8_ctx_t &, int) {
        f.a[i] = lds_read16(S[0] + ad.a + i * 1024);
    }
    __device__ static __forceinline__ void mma_row(v4f (&acc)[ROWS][COLS], const frag_t &f, int i,
            const f8_ctx_t &, int) {
#pragma unroll
        for (int j = 0; j < COLS; ++j) {
            // operands exchanged: the tile comes out transposed (a lane holds four consecutive n of one row)
            if constexpr (BF16)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf_t, f.b[j]),
                        __builtin_bit_cast(v8bf_t, f.a[i]), acc[i][j], 0, 0, 0);
            else
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h_t, f.b[j]),
                        __builtin_bit_cast(v8h_t, f.a[i]), acc[i][j], 0, 0, 0);
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

} // namespace

// ---- bf16 / f16 / f32
namespace {
// zeroes bytes [from, pitch) of every row: the K padding of an operand copy
__global__ void __launch_bounds__(256) h16_zero_tail_kernel(uint16_t *base, long rows, long pitch16, long from16) {
    const long per = pitch16 - from16, total = rows * per;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256)
        base[(i / per) * pitch16 + from16 + i % per] = 0;
}
} // namespace

// f32 operands under fpmath_mode bf16 / f16 / any (dnnl_fpmath_mode_t 1 / 2 / 3): the attribute allows an implicit
// down-conversion (doc/programming_model/attributes_fpmath_mode.md), so both operands are converted into scratch by
// two reorder launches -- the weights into the K-contiguous layout on the way -- and the 16-bit policy multiplies
// them: eight times the matrix-core rate of the f32 instruction.  0 = no down-conversion.
static int h16_down_dt(const mi355_matmul_desc_t &d) {
    if (d.src_dt != MI355_DT_F32 || d.wei_dt != MI355_DT_F32) return 0;
    if (d.fpmath_mode == 1 || d.fpmath_mode == 3) return MI355_DT_BF16;
    if (d.fpmath_mode == 2) return MI355_DT_F16;
    return 0;
}

// How a problem reaches the tiles.  An operand is read where it lies when it is K-contiguous with 16-byte aligned
// rows and K fills whole 64-byte stages; otherwise a reorder launch copies it into scratch as dense K-contiguous
// rows of Kp = K rounded up to whole stages (converted on the way under fpmath, transposed on the way for
// N-contiguous weights), the padding zeroed -- so any K and any plain layout with a unit stride runs here, at the
// price of the copy.
struct h16_plan_t {
    bool ok, woq;
    int op_dt;
    long EB, Kp, Bs, Bw;
    bool copy_src, copy_wei;
    size_t off_wei, total;
};

static h16_plan_t h16_plan(const mi355_matmul_desc_t &d) {
    h16_plan_t p {};
    if (d.K < 1) return p;
    p.Bs = d.src_stride[0] ? d.batch : 1;
    p.Bw = d.wei_stride[0] ? d.batch : 1;
    const int down = h16_down_dt(d);
    p.woq = d.src_dt != d.wei_dt; // 8- or 4-bit integer weights under a 16-bit src (checked by h16_supported)
    p.op_dt = down ? down : d.src_dt;
    p.EB = dt_bits(p.op_dt) / 8;
    const long KE = BKB * KSTEP / p.EB, AL = 16 / p.EB;
    p.Kp = (d.K + KE - 1) / KE * KE;
    const bool pad = p.Kp != d.K;
    const bool src_direct = !down && !pad && d.src_stride[2] == 1 && d.src_stride[1] % AL == 0 && d.src_stride[0] % AL == 0;
    const bool wei_direct = !down && !pad && !p.woq && d.wei_stride[1] == 1 && d.wei_stride[2] % AL == 0
            && d.wei_stride[0] % AL == 0;
    p.copy_src = !src_direct;
    p.copy_wei = !wei_direct;
    // the copies come from the reorder's direct or tiled kernels: a unit stride on the way in
    if (p.copy_src && d.src_stride[2] != 1 && d.src_stride[1] != 1) return p;
    if (p.copy_wei && d.wei_stride[2] != 1 && d.wei_stride[1] != 1) return p;
    // byte offsets inside a tile are 32-bit
    const long lda = p.copy_src ? p.Kp : d.src_stride[1], ldb = p.copy_wei ? p.Kp : d.wei_stride[2];
    if (lda * p.EB * BM >= (1L << 31) || ldb * p.EB * f8_geo_t::BN >= (1L << 31)) return p;
    size_t off = 0;
    if (p.copy_src) off += align_up((size_t)p.Bs * d.M * p.Kp * p.EB, 256);
    p.off_wei = off;
    if (p.copy_wei) off += align_up((size_t)p.Bw * d.N * p.Kp * p.EB, 256);
    p.total = off;
    p.ok = true;
    return p;
}

// Weight-only quantization beyond the decode kernels' 32 rows (prefill): s4 / u4 / s8 / u8 weights under a bf16 / f16
// src with fpmath apply_to_int.  The weights' copy is written by the reorder with the weights' scales and zero points
// as its src parameters -- (w - zp) * scale rounded to the src type, what the reference's JIT path multiplies
// (brgemm_matmul_copy_utils.cpp:2870-2896) -- and the 16-bit tiles run without them.
static bool h16_woq(const mi355_matmul_desc_t &d) {
    if (d.src_dt != MI355_DT_BF16 && d.src_dt != MI355_DT_F16) return false;
    if (d.wei_dt != MI355_DT_S4 && d.wei_dt != MI355_DT_U4 && d.wei_dt != MI355_DT_S8 && d.wei_dt != MI355_DT_U8) return false;
    if (!d.fpmath_apply_to_int || d.wei_packing != MI355_WEI_PACK_NONE) return false;
    if (!quant_absent(d.src_scale) || !quant_absent(d.src_zp) || !quant_absent(d.src_pr)) return false;
    const int sdt = d.wei_scale.dt, zdt = d.wei_zp.dt;
    if (sdt != MI355_DT_UNDEF && sdt != MI355_DT_F32 && sdt != MI355_DT_BF16 && sdt != MI355_DT_F16) return false;
    if (zdt != MI355_DT_UNDEF && zdt != MI355_DT_S32 && zdt != MI355_DT_S8 && zdt != MI355_DT_U8 && zdt != MI355_DT_S4
            && zdt != MI355_DT_U4)
        return false;
    for (const mi355_quant_t *q : {&d.wei_scale, &d.wei_zp})
        if (q->dt != MI355_DT_UNDEF
                && ((q->group[0] > 1 && d.K % q->group[0]) || (q->group[1] > 1 && d.N % q->group[1])))
            return false;
    // 4-bit weights: whole bytes along the contiguous dim
    if (dt_bits(d.wei_dt) == 4 && ((d.wei_stride[2] == 1 ? d.N : d.K) % 2)) return false;
    return true;
}

int h16_supported(const mi355_matmul_desc_t &d) {
    if (dt_bits(d.dst_dt) < 8) return MI355_UNIMPLEMENTED;
    if (d.batch > 65535) return MI355_UNIMPLEMENTED;
    if (h16_woq(d)) return h16_plan(d).ok ? MI355_SUCCESS : MI355_UNIMPLEMENTED;
    if (d.src_dt != d.wei_dt || (d.src_dt != MI355_DT_BF16 && d.src_dt != MI355_DT_F16 && d.src_dt != MI355_DT_F32))
        return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.src_zp) || !quant_absent(d.wei_zp) || !quant_absent(d.src_pr)) return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.src_scale)
            && ((d.src_scale.mask & 4) || d.src_scale.group[0] > 1 || d.src_scale.group[1] > 1))
        return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.wei_scale)
            && ((d.wei_scale.mask & 2) || d.wei_scale.group[0] > 1 || d.wei_scale.group[1] > 1))
        return MI355_UNIMPLEMENTED;
    if (d.batch > 65535) return MI355_UNIMPLEMENTED;
    return h16_plan(d).ok ? MI355_SUCCESS : MI355_UNIMPLEMENTED;
}

size_t h16_scratch_bytes(const mi355_matmul_desc_t &d) {
    const h16_plan_t p = h16_plan(d);
    return p.ok ? p.total : 0;
}

// [B][R][C] with the given strides -> [B][R][ld] (or, transposed, [B][C][ld]) of data type `to`, ld >= the row
// length; the columns beyond it are zeroed
static int h16_convert(const void *in, int from, long B, long R, long C, const int64_t *stride, bool transposed, int to,
        void *out, long ld, hipStream_t stream, const mi355_quant_t *scale = nullptr, const void *scale_p = nullptr,
        const mi355_quant_t *zp = nullptr, const void *zp_p = nullptr) {
    const long rows = transposed ? C : R, cols = transposed ? R : C;
    mi355_reorder_desc_t rd {};
    rd.ndims = 3;
    rd.src_dt = from;
    rd.dst_dt = to;
    rd.dims[0] = B; rd.dims[1] = R; rd.dims[2] = C;
    rd.src_stride[0] = stride[0]; rd.src_stride[1] = stride[1]; rd.src_stride[2] = stride[2];
    rd.dst_stride[0] = rows * ld;
    rd.dst_stride[1] = transposed ? 1 : ld;
    rd.dst_stride[2] = transposed ? ld : 1;
    rd.src_scale.group[0] = rd.src_scale.group[1] = rd.dst_scale.group[0] = rd.dst_scale.group[1] = 1;
    rd.src_zp.group[0] = rd.src_zp.group[1] = rd.dst_zp.group[0] = rd.dst_zp.group[1] = 1;
    mi355_reorder_args_t ra {};
    ra.src = in;
    ra.dst = out;
    if (scale && scale->dt != MI355_DT_UNDEF) {
        rd.src_scale = *scale;
        ra.src_scale = scale_p;
    }
    if (zp && zp->dt != MI355_DT_UNDEF) {
        rd.src_zp = *zp;
        ra.src_zp = zp_p;
    }
    if (const int st = mi355_reorder_launch(&rd, &ra, stream)) return st;
    if (ld > cols) {
        const long units = dt_bits(to) / 16; // 16-bit words per element
        const long total = B * rows * (ld - cols) * units;
        long blocks = (total + 255) / 256;
        if (blocks > 65535) blocks = 65535;
        hipLaunchKernelGGL(h16_zero_tail_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (uint16_t *)out, B * rows,
                ld * units, cols * units);
        if (hipGetLastError() != hipSuccess) return MI355_RUNTIME_ERROR;
    }
    return MI355_SUCCESS;
}

int h16_launch(const mi355_matmul_desc_t &d, const problem_t &P_in, void *scratch, hipStream_t stream) {
    const h16_plan_t plan = h16_plan(d);
    if (!plan.ok) {
        set_error("mfma_h16: the problem is not one this family takes");
        return MI355_UNIMPLEMENTED;
    }
    if (plan.total > 0 && !scratch) {
        set_error("mfma_h16: %zu bytes of scratch required", plan.total);
        return MI355_INVALID_ARGUMENTS;
    }
    f8_extra_t X {};
    problem_t P = P_in;
    const long EB = plan.EB;
    char *a_copy = (char *)scratch, *b_copy = (char *)scratch + plan.off_wei;
    if (plan.copy_src) {
        if (const int st = h16_convert(P.src, d.src_dt, plan.Bs, d.M, d.K, d.src_stride, false, plan.op_dt, a_copy, plan.Kp,
                    stream))
            return st;
        P.src = a_copy;
        P.ss[0] = plan.Bs > 1 ? d.M * plan.Kp : 0; P.ss[1] = plan.Kp; P.ss[2] = 1;
    }
    if (plan.copy_wei) {
        if (const int st = h16_convert(P.wei, d.wei_dt, plan.Bw, d.K, d.N, d.wei_stride, true, plan.op_dt, b_copy, plan.Kp,
                    stream, plan.woq ? &d.wei_scale : nullptr, P.wei_scale.p, plan.woq ? &d.wei_zp : nullptr, P.wei_zp.p))
            return st;
        if (plan.woq) P.wei_scale.dt = P.wei_zp.dt = MI355_DT_UNDEF; // applied by the copy
        X.bt = b_copy;
        X.ldb = plan.Kp * EB;
        X.bt_bstride = plan.Bw > 1 ? d.N * plan.Kp * EB : 0;
    } else {
        X.bt = (const char *)P.wei;
        X.ldb = d.wei_stride[2] * EB;
        X.bt_bstride = d.wei_stride[0] * EB;
    }
    P.src_dt = P.wei_dt = plan.op_dt;
    P.K = plan.Kp; // the padding multiplies zeros by zeros
    X.tiles_m = (int)((d.M + BM - 1) / BM);
    X.tiles_n = (int)((d.N + f8_geo_t::BN - 1) / f8_geo_t::BN);
    dim3 grid((unsigned)(X.tiles_m * X.tiles_n), 1, (unsigned)d.batch);
    constexpr int smem_bytes = NSTAGE * f8_geo_t::STAGE_BYTES + NTAB_BYTES;
    auto go = [&](auto kern) -> int {
        if (const int st = ensure_dynamic_lds((const void *)kern, smem_bytes, "mfma_h16")) return st;
        hipLaunchKernelGGL(kern, grid, dim3(f8_geo_t::NT), smem_bytes, stream, P, X);
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
    };
    if (plan.op_dt == MI355_DT_BF16) return go(f8_gemm_kernel<h16x16_mma_t<true, f8_geo_t>>);
    if (plan.op_dt == MI355_DT_F32) return go(f8_gemm_kernel<f32_mma_t<f8_geo_t>>);
    return go(f8_gemm_kernel<h16x16_mma_t<false, f8_geo_t>>);
}

} // namespace mi355
