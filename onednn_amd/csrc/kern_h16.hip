// "hip:mfma_h16" -- the same tiles for bf16 x bf16, f16 x f16 and f32 x f32 operands
// (ref_matmul_t's f32 sum of exact products): a 64-byte stage is 32 elements of
// K, one v_mfma_f32_16x16x32_{bf16,f16} per pair of 16-row fragments, in the
// matrix cycles of the fp8 family's instruction per stage, so the data path
// (DMA, LDS ring, epilogue) is shared unchanged.
#include <cstdlib>
#include <cstring>
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

// Decompression of row-major 4-bit weights [K][N] (two n per byte, low nibble = even n) into the K-contiguous 16-bit
// copy the tiles read, [N][K]: value = (w - zp[k / gk][n]) * scale[k / gk][n], the reorder's arithmetic (integer
// subtraction, one f32 multiplication, round to nearest even).  A workgroup owns 64 k x 256 n: a thread loads the
// 16 bytes (32 columns) of two adjacent k rows -- eight lanes a whole 128-byte line -- takes the scales and zero
// points of its columns from LDS (fetched once per workgroup), packs the two k of a column into one dword and parks it in LDS at dword column
// (k / 2) ^ 4 (n / 32) of row n, which spreads a store instruction over all banks and keeps every aligned group of
// four columns together; the tile then leaves as whole 128-byte rows.  The generic tiled reorder took 0.36 ms for
// 4096 x 14336 weights with grouped parameters; this kernel moves the same 29 MB in and 117 MB out.
struct woq_dq_t {
    const uint8_t *wei;  // [K][ldw / 2] bytes
    uint16_t *out;       // [N][ldo]
    const void *sc, *zp; // [K / gk or 1][N or 1], null = absent
    long ldw, ldo;       // elements
    int K, N;
    int sc_dt, zp_dt;
    int sc_gk, zp_gk;    // rows of k per parameter row; 0 = one row for all k
    int sc_per_n, zp_per_n;
    int signed_w, out_bf16;
};

typedef uint32_t woq_u4v __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(256) woq_dequant_kernel(const woq_dq_t A) {
    typedef woq_u4v u4v;
    __shared__ __attribute__((aligned(16))) uint32_t tile[256 * 32];
    const int t = threadIdx.x;
    const int k0 = blockIdx.y * 64, n0 = blockIdx.x * 256;
    const int c = t & 7, kp = t >> 3;            // columns n0 + 32 c .. + 31, rows k0 + 2 kp and + 1
    const int nb = n0 + 32 * c;
    const long k = k0 + 2 * kp;
    const u4v w0 = __builtin_nontemporal_load((const u4v *)(A.wei + (k * A.ldw + nb) / 2));
    const u4v w1 = __builtin_nontemporal_load((const u4v *)(A.wei + ((k + 1) * A.ldw + nb) / 2));
    // The 64 rows of k share their parameters (groups are whole 64s): thread t fetches those of column n0 + t once
    // for the workgroup -- 32 threads per column block asking for the same 80 bytes each was most of what the
    // vector-memory path had to serve.
    __shared__ __attribute__((aligned(16))) float s_sc[256];
    __shared__ __attribute__((aligned(16))) int s_zp[256];
    {
        float scv = 1.f;
        int zpv = 0;
        if (A.sc)
            scv = load_float(A.sc_dt, A.sc,
                    (A.sc_gk ? (k0 / A.sc_gk) * (long)(A.sc_per_n ? A.N : 1) : 0) + (A.sc_per_n ? n0 + t : 0));
        if (A.zp)
            zpv = load_int(A.zp_dt, A.zp,
                    (A.zp_gk ? (k0 / A.zp_gk) * (long)(A.zp_per_n ? A.N : 1) : 0) + (A.zp_per_n ? n0 + t : 0));
        s_sc[t] = scv;
        s_zp[t] = zpv;
    }
    __syncthreads();
    float sc[32];
    int zp[32];
#pragma unroll
    for (int e = 0; e < 32; e += 4) {
        const float4 a = *(const float4 *)&s_sc[32 * c + e];
        const int4 z = *(const int4 *)&s_zp[32 * c + e];
        sc[e] = a.x, sc[e + 1] = a.y, sc[e + 2] = a.z, sc[e + 3] = a.w;
        zp[e] = z.x, zp[e + 1] = z.y, zp[e + 2] = z.z, zp[e + 3] = z.w;
    }
    const uint32_t d0[4] = {w0.x, w0.y, w0.z, w0.w}, d1[4] = {w1.x, w1.y, w1.z, w1.w};
    const int sx = A.signed_w ? 8 : 0; // (b ^ 8) - 8 sign-extends a nibble
    // bf16: v_cvt_pk_bf16_f32 rounds to nearest even like the software conversion for normal numbers, zeros and
    // infinities; that one flushes f32 subnormals and quiets NaNs its own way, so a wavefront that meets either
    // (class mask: s/q NaN, +-subnormal) redoes its part in software
    bool special = false;
    if (A.out_bf16) {
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
        typedef float f32x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int e = 0; e < 32; ++e) {
            const int v0 = (int)(((d0[e >> 3] >> (4 * (e & 7))) & 15) ^ sx) - sx;
            const int v1 = (int)(((d1[e >> 3] >> (4 * (e & 7))) & 15) ^ sx) - sx;
            const float f0 = sc[e] * (float)(v0 - zp[e]), f1 = sc[e] * (float)(v1 - zp[e]);
            special |= __builtin_amdgcn_classf(f0, 0x93) | __builtin_amdgcn_classf(f1, 0x93);
            tile[(32 * c + e) * 32 + (kp ^ (4 * c))]
                    = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_t {f0, f1}, bf16x2_t));
        }
    }
    if (!A.out_bf16 || __builtin_amdgcn_ballot_w64(special) != 0) {
#pragma unroll
        for (int e = 0; e < 32; ++e) {
            const int v0 = (int)(((d0[e >> 3] >> (4 * (e & 7))) & 15) ^ sx) - sx;
            const int v1 = (int)(((d1[e >> 3] >> (4 * (e & 7))) & 15) ^ sx) - sx;
            const float f0 = sc[e] * (float)(v0 - zp[e]), f1 = sc[e] * (float)(v1 - zp[e]);
            const unsigned lo = A.out_bf16 ? f32_to_bf16(f0) : f32_to_f16(f0), hi = A.out_bf16 ? f32_to_bf16(f1) : f32_to_f16(f1);
            tile[(32 * c + e) * 32 + (kp ^ (4 * c))] = lo | (hi << 16);
        }
    }
    __syncthreads();
    const int q = t & 7, r = t >> 3; // write: row r + 32 pass, dwords of the physical group q
#pragma unroll
    for (int pass = 0; pass < 8; ++pass) {
        const int row = r + 32 * pass, cc = row >> 5;
        const u4v v = *(const u4v *)&tile[row * 32 + 4 * q];
        // physical group q of this row holds the logical dword columns 4 (q ^ cc) .. + 3, i.e. k0 + 8 (q ^ cc) .. + 7
        __builtin_nontemporal_store(v, (u4v *)(A.out + (long)(n0 + row) * A.ldo + k0 + 8 * (q ^ cc)));
    }
}

// The same for K-contiguous 4-bit weights [N][K] (two k per byte): no transposition.  A workgroup owns 256 k x 32 n;
// thread (c = t % 8, r = t / 8) takes the dwords c, c + 8, c + 16, c + 24 of row r's 128 bytes, so that the eight
// lanes of a row write 128 contiguous bytes with every store instruction (the reads, a quarter of the traffic, come
// in 32-byte pieces instead).  The eight k of a dword share their parameters (groups along k are multiples of 64).
__global__ void __launch_bounds__(256) woq_dequant_kmajor_kernel(const woq_dq_t A) {
    const int t = threadIdx.x, c = t & 7;
    const int n = blockIdx.y * 32 + (t >> 3);
    if (n >= A.N) return;
    const long k0 = (long)blockIdx.x * 256;
    const uint32_t *row = (const uint32_t *)(A.wei + ((long)n * A.ldw + k0) / 2);
    uint32_t d[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) d[j] = __builtin_nontemporal_load(row + c + 8 * j);
    const int sx = A.signed_w ? 8 : 0;
    long sg = -1, zg = -1;
    float sc = 1.f;
    int zp = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const long k = k0 + 8 * (c + 8 * j);
        const long sgj = A.sc_gk ? k / A.sc_gk : 0, zgj = A.zp_gk ? k / A.zp_gk : 0;
        if (A.sc && sgj != sg) sc = load_float(A.sc_dt, A.sc, sgj * (A.sc_per_n ? A.N : 1) + (A.sc_per_n ? n : 0)), sg = sgj;
        if (A.zp && zgj != zg) zp = load_int(A.zp_dt, A.zp, zgj * (A.zp_per_n ? A.N : 1) + (A.zp_per_n ? n : 0)), zg = zgj;
        uint32_t h[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int v = (int)(((d[j] >> (4 * e)) & 15) ^ sx) - sx;
            const float f = sc * (float)(v - zp);
            h[e] = A.out_bf16 ? f32_to_bf16(f) : f32_to_f16(f);
        }
        woq_u4v o;
        o.x = h[0] | (h[1] << 16), o.y = h[2] | (h[3] << 16), o.z = h[4] | (h[5] << 16), o.w = h[6] | (h[7] << 16);
        __builtin_nontemporal_store(o, (woq_u4v *)(A.out + (long)n * A.ldo + k));
    }
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

// the dedicated kernels' conditions: 4-bit weights of one batch in whole tiles (row-major: 64 k x 256 n, returns 1;
// K-contiguous: K in whole 256s, returns 2), parameters per tensor, per column, or per group of whole 64s of k and
// column; 0 = the reorder
static int h16_woq_fast(const mi355_matmul_desc_t &d, const h16_plan_t &p) {
    if (!p.woq || dt_bits(d.wei_dt) != 4 || p.Bw != 1 || p.Kp != d.K) return 0;
    if (d.K >= (1L << 31) || d.N >= (1L << 31)) return 0;
    for (const mi355_quant_t *q : {&d.wei_scale, &d.wei_zp}) {
        if (q->dt == MI355_DT_UNDEF) continue;
        const int m = q->mask & 6;
        if ((q->mask & 1) || q->group[1] > 1) return 0;
        if (m == 2) return 0;                                                       // per k only
        if ((m & 2) && (q->group[0] < 64 || q->group[0] % 64 != 0)) return 0;       // whole 64s of k share a parameter
    }
    if (d.wei_stride[2] == 1 && d.wei_stride[1] % 32 == 0 && d.K % 64 == 0 && d.N % 256 == 0) return 1;
    if (d.wei_stride[1] == 1 && d.wei_stride[2] % 8 == 0 && d.K % 256 == 0 && (d.N + 31) / 32 <= 65535) return 2;
    return 0;
}

int h16_supported(const mi355_matmul_desc_t &d) {
    if (dt_bits(d.dst_dt) < 8 && !tile_nibble_dst_ok(d)) return MI355_UNIMPLEMENTED;
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
    const int fast = plan.copy_wei ? h16_woq_fast(d, plan) : 0;
    const uintptr_t align = fast == 1 ? ((uintptr_t)P.wei | (uintptr_t)P.wei_scale.p | (uintptr_t)P.wei_zp.p) & 15
                                      : (uintptr_t)P.wei & 3;
    if (fast && align == 0) {
        woq_dq_t A {};
        A.wei = (const uint8_t *)P.wei;
        A.out = (uint16_t *)b_copy;
        A.ldw = fast == 1 ? d.wei_stride[1] : d.wei_stride[2];
        A.ldo = plan.Kp;
        A.K = (int)d.K; A.N = (int)d.N;
        auto param = [&](const mi355_quant_t &q, const void *ptr, const void *&p_, int &dt, int &gk, int &per_n) {
            p_ = q.dt != MI355_DT_UNDEF ? ptr : nullptr;
            dt = q.dt;
            gk = (q.mask & 2) ? (int)q.group[0] : 0;
            per_n = (q.mask & 4) ? 1 : 0;
        };
        param(d.wei_scale, P.wei_scale.p, A.sc, A.sc_dt, A.sc_gk, A.sc_per_n);
        param(d.wei_zp, P.wei_zp.p, A.zp, A.zp_dt, A.zp_gk, A.zp_per_n);
        A.signed_w = d.wei_dt == MI355_DT_S4;
        A.out_bf16 = plan.op_dt == MI355_DT_BF16;
        if (fast == 1)
            hipLaunchKernelGGL(woq_dequant_kernel, dim3((unsigned)(d.N / 256), (unsigned)(d.K / 64)), dim3(256), 0, stream, A);
        else
            hipLaunchKernelGGL(woq_dequant_kmajor_kernel, dim3((unsigned)(d.K / 256), (unsigned)((d.N + 31) / 32)), dim3(256),
                    0, stream, A);
        if (hipGetLastError() != hipSuccess) return MI355_RUNTIME_ERROR;
    } else if (plan.copy_wei) {
        if (const int st = h16_convert(P.wei, d.wei_dt, plan.Bw, d.K, d.N, d.wei_stride, true, plan.op_dt, b_copy, plan.Kp,
                    stream, plan.woq ? &d.wei_scale : nullptr, P.wei_scale.p, plan.woq ? &d.wei_zp : nullptr, P.wei_zp.p))
            return st;
    }
    if (plan.copy_wei) {
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
    // Few tiles (prefill at a few hundred rows): 256 x 128 tiles of four wavefronts, two workgroups a CU, put twice
    // the CUs to work; a wavefront's part, 128 x 64, and with it the fragments and the epilogue are the same.
    using narrow_t = geo_t<4, 128>;
    // (the MI355_H16_TILES switch keeps the 256 x 256 tiles: tests, tuning)
    if (plan.op_dt != MI355_DT_F32 && (long)X.tiles_m * X.tiles_n * d.batch <= 128 && d.N > 128
            && tuning(TUNE_H16_TILES) != TUNE_WIDE) {
        X.tiles_n = (int)((d.N + narrow_t::BN - 1) / narrow_t::BN);
        dim3 grid((unsigned)(X.tiles_m * X.tiles_n), 1, (unsigned)d.batch);
        constexpr int smem_bytes = narrow_t::NSTAGE * narrow_t::STAGE_BYTES + NTAB_BYTES;
        auto go = [&](auto kern) -> int {
            if (const int st = ensure_dynamic_lds((const void *)kern, smem_bytes, "mfma_h16")) return st;
            hipLaunchKernelGGL(kern, grid, dim3(narrow_t::NT), smem_bytes, stream, P, X);
            return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
        };
        if (plan.op_dt == MI355_DT_BF16) return go(f8_gemm_kernel<h16x16_mma_t<true, narrow_t>>);
        return go(f8_gemm_kernel<h16x16_mma_t<false, narrow_t>>);
    }
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
