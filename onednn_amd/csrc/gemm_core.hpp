// LDS-tiled MFMA GEMM core shared by the int8, fp8 and MXFP4 kernel families.
//
// Shape of the computation (one workgroup = 4 wavefronts = one 256x256 dst
// tile, each wavefront a 128x128 quadrant held in 256 accumulator registers):
//
//   HBM/L2 --global_load_lds_dwordx4--> LDS ring of NSTAGE stages
//       stage = A[256 rows][64 B of K] + B^T[256 rows][64 B of K]  (32 KB)
//   LDS --ds_read_b128--> MFMA operands --v_mfma--> accumulators
//   accumulators --LDS slab transpose--> fused epilogue --> wide dst stores
//
// Both operands are consumed K-contiguous ("A" rows are src rows, "B^T" rows
// are weight columns).  Loads bypass the register file (direct-to-LDS DMA);
// each wavefront-wide DMA moves 64 x 16 B = 16 rows x 64 B.  Inside a row the
// four 16-byte chunks are XOR-swizzled with the row number so the ds_read_b128
// of an MFMA operand (32 or 16 consecutive rows, one chunk) is free of bank
// conflicts; the swizzle is applied on the global-address side of the DMA.
//
// Pipeline per K step kt (ring slot kt % NSTAGE):
//   s_waitcnt vmcnt(..)   own DMAs of stage kt landed
//   s_barrier             everybody's did, and everybody finished stage kt-1
//   issue DMAs for stage kt+NSTAGE-1 into the slot stage kt-1 used
//   ds_read + MFMA over stage kt
//
// The DMA instructions are emitted through inline assembly so that the
// outstanding-load counter is managed by hand (a prefetch distance of
// NSTAGE-1 stages needs "wait until at most N loads are in flight").
#pragma once
#include "kernels.hpp"
#include "tile_epilogue.hpp"

namespace mi355 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

namespace gemm {

constexpr int BM = 256, BN = 256;
constexpr int BKB = 64;               // bytes of K per row per stage
constexpr int NT = 256;               // threads per workgroup
constexpr int STAGE_BYTES = (BM + BN) * BKB; // 32 KB
constexpr int B_OFF = BM * BKB;       // B^T tile offset inside a stage

// chunk swizzle: conflict-free for ds_read_b128 over 8 or 16 consecutive rows
__device__ __forceinline__ int swz_f(int row) { return ((row >> 1) & 3) ^ ((row >> 3) & 1); }
__device__ __forceinline__ int swz(int row, int chunk) {
    return row * BKB + ((chunk ^ swz_f(row)) << 4);
}

// 4 bytes per lane: LDS byte address lds_addr + 4*i
__device__ __forceinline__ void dma4(const void *sbase, unsigned voff, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(sbase)
                 : "memory", "m0");
}

// one wavefront-wide direct-to-LDS load: lane i brings 16 bytes from
// sbase + voff to LDS byte address lds_addr + 16*i
__device__ __forceinline__ void dma16(const void *sbase, unsigned voff, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(sbase)
                 : "memory", "m0");
}

// LDS reads through explicit 32-bit LDS addresses: a generic pointer that the
// compiler cannot prove to be shared memory (one selected between two stages,
// say) turns every ds_read into a flat load through the vector memory path.
typedef const v4i __attribute__((address_space(3))) *lds_v4i_ptr_t;
typedef const unsigned __attribute__((address_space(3))) *lds_u32_ptr_t;
__device__ __forceinline__ v4i lds_read16(unsigned addr) { return *(lds_v4i_ptr_t)(size_t)addr; }
__device__ __forceinline__ unsigned lds_read4(unsigned addr) { return *(lds_u32_ptr_t)(size_t)addr; }

// s_waitcnt vmcnt(n) only (expcnt / lgkmcnt left at their maxima)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | ((N >> 4) << 14));
}

struct tile_pos_t {
    long m0, n0;
};

// XCD-aware tile order.  Consecutive workgroup ids land on different XCDs
// (8 of them, each with a private L2); give every XCD one contiguous run of
// tiles, walked in bands of GM tile rows so that concurrently resident tiles
// share A rows and B columns in that L2.
__device__ __forceinline__ tile_pos_t tile_position(int tiles_m, int tiles_n) {
    const int nwg = gridDim.x, id = blockIdx.x;
    const int per = nwg / 8;
    const int tile = (nwg % 8 == 0) ? (id % 8) * per + id / 8 : id;
    constexpr int GM = 8;
    const int band = tile / (GM * tiles_n);
    const int band_rows = min(GM, tiles_m - band * GM);
    const int in_band = tile - band * GM * tiles_n;
    tile_pos_t p;
    p.m0 = (long)(band * GM + in_band % band_rows) * BM;
    p.n0 = (long)(in_band / band_rows) * BN;
    return p;
}

// Per-thread DMA plan: wave w owns tile rows [64w, 64w+64) of A and of B^T,
// four DMAs each per stage.
struct dma_plan_t {
    unsigned voff_a[4], voff_b[4]; // byte offsets from the scalar tile base
    unsigned lds_a[4], lds_b[4];   // LDS byte offsets inside a stage
};

__device__ __forceinline__ dma_plan_t make_dma_plan(int wave, int lane, long rows_a_left,
        long rows_b_left, long lda, long ldb) {
    dma_plan_t p;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = (wave * 4 + i) * 16 + (lane >> 2);
        const int chunk = (lane & 3) ^ swz_f(row);
        long ra = row, rb = row;
        if (ra > rows_a_left - 1) ra = rows_a_left - 1;
        if (rb > rows_b_left - 1) rb = rows_b_left - 1;
        p.voff_a[i] = (unsigned)(ra * lda + chunk * 16);
        p.voff_b[i] = (unsigned)(rb * ldb + chunk * 16);
        p.lds_a[i] = (unsigned)((wave * 4 + i) * 1024);
        p.lds_b[i] = (unsigned)(B_OFF + (wave * 4 + i) * 1024);
    }
    return p;
}

__device__ __forceinline__ void issue_stage(const dma_plan_t &p, const char *a_base,
        const char *b_base, unsigned lds_stage) {
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16(a_base, p.voff_a[i], lds_stage + p.lds_a[i]);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16(b_base, p.voff_b[i], lds_stage + p.lds_b[i]);
}

// Main loop.  The ring holds NSTAGE stages; one iteration consumes KSTEP of
// them (a "group": KSTEP * 64 bytes of K), so NSTAGE / KSTEP groups rotate.
// Per group g:
//   s_waitcnt vmcnt(..)   own DMAs of group g landed
//   s_barrier             everybody's did, and everybody finished group g-1
//   DMA group g+NG-1      into the slots group g-1 used
//   ds_read + MFMA over group g
// `Mma` supplies frag_t, load_b(frag, S, wn, lane, ctx, g) for the 8 B^T
// fragments, load_a(frag, i, S, wm, lane, ctx, g) for A fragment i (S[k] is the
// LDS byte address of the k-th stage of the group), mma_row(acc, frag, i, ctx, g)
// for the COLS MFMAs of A fragment i (ROWS x COLS MFMA tiles per quadrant),
// and A_READS / B_READS = LDS read instructions per fragment.
// a_tile / b_tile point at the first K byte of tile row 0.
template <int NSTAGE, int KSTEP, class Mma, class Acc, class Ctx>
__device__ __forceinline__ void main_loop(Acc &acc, char *smem, const char *a_tile,
        const char *b_tile, long lda, long ldb, long rows_a_left, long rows_b_left, int ngroups,
        const Ctx &ctx) {
    constexpr int NG = NSTAGE / KSTEP;           // groups in the ring
    constexpr int GROUP_BYTES = KSTEP * STAGE_BYTES;
    constexpr int GROUP_DMAS = KSTEP * 8 + Mma::EXTRA_DMAS;
    static_assert(NSTAGE % KSTEP == 0 && NG >= 2 && NG <= 5, "ring depth");
    static_assert((NG - 2) * GROUP_DMAS < 64, "vmcnt range");
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem;
    const dma_plan_t plan = make_dma_plan(wave, lane, rows_a_left, rows_b_left, lda, ldb);

    // DMA number i (0..7) of every stage of group g: A row blocks first, then B^T
    auto issue_part = [&](int g, int slot, int i) __attribute__((always_inline)) {
#pragma unroll
        for (int k = 0; k < KSTEP; ++k) {
            const long koff = ((long)g * KSTEP + k) * BKB;
            const unsigned lds_stage = lds0 + slot * GROUP_BYTES + k * STAGE_BYTES;
            if (i < 4) dma16(a_tile + koff, plan.voff_a[i], lds_stage + plan.lds_a[i]);
            else dma16(b_tile + koff, plan.voff_b[i - 4], lds_stage + plan.lds_b[i - 4]);
        }
        if (i == 7) Mma::issue_extra(ctx, g, slot, wave, lane);
    };

    // prologue: groups 0 .. NG-2 in flight
#pragma unroll
    for (int s = 0; s < NG - 1; ++s)
        if (s < ngroups) {
#pragma unroll
            for (int i = 0; i < 8; ++i) issue_part(s, s, i);
        }

    int slot = 0;
    // One group: all B fragments and the first two A fragments, then per A
    // fragment i its row of MFMAs, with the load of A fragment i+2 and a share
    // of the DMAs of group g+NG-1 issued ahead of them (a burst of DMAs right
    // after the barrier queues up at the address unit while the matrix cores
    // idle: measured 250 ns of a 950 ns step).  The DMA shares sit in small
    // conditional blocks and the loop is not unrolled: with a branch-free or
    // rotated body the register allocator starts copying the 256 accumulators
    // around in every iteration.
#pragma nounroll
    for (int g = 0; g < ngroups; ++g) {
        // groups g+1 .. g+NG-2 may stay in flight
        if (g + NG - 2 < ngroups) wait_vmcnt<(NG - 2) * GROUP_DMAS>();
        else wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
        int nslot = slot + NG - 1;
        if (nslot >= NG) nslot -= NG;
        unsigned S[KSTEP]; // LDS byte addresses of the group's stages
#pragma unroll
        for (int k = 0; k < KSTEP; ++k) S[k] = lds0 + slot * GROUP_BYTES + k * STAGE_BYTES;
        const bool dma = g + NG - 1 < ngroups;
        typename Mma::frag_t f;
        constexpr int ROWS = Mma::ROWS, COLS = Mma::COLS; // MFMA tiles of the quadrant
        constexpr int DPR = 8 / ROWS;                     // DMAs per row of MFMAs
        // A fragment 0 first: LDS reads return in order, so the first MFMA can go
        // as soon as it and the first B fragment are in
        Mma::load_a(f, 0, S, wm, lane, ctx, g);
        Mma::load_b(f, S, wn, lane, ctx, g);
        Mma::load_a(f, 1, S, wm, lane, ctx, g);
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
            if (dma) {
#pragma unroll
                for (int d = 0; d < DPR; ++d) issue_part(g + NG - 1, nslot, i * DPR + d);
            }
            if (i + 2 < ROWS) Mma::load_a(f, i + 2, S, wm, lane, ctx, g);
            Mma::mma_row(acc, f, i, ctx, g);
        }
        if (++slot == NG) slot = 0;
    }
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
}

} // namespace gemm
} // namespace mi355
