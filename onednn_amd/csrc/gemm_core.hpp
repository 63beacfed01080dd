// LDS-tiled MFMA GEMM core shared by the int8, fp8 and MXFP4 kernel families.
//
// Shape of the computation: one workgroup = one 256x256 dst tile, split over
// either 4 wavefronts (a 128x128 part each, 256 accumulator registers, one
// wavefront per SIMD) or 8 wavefronts (128x64 each, 128 accumulator registers,
// two wavefronts per SIMD that fill each other's LDS and barrier waits):
//
//   HBM/L2 --global_load_lds_dwordx4--> LDS ring of NSTAGE stages
//       stage = A[256 rows][64 B of K] + B^T[256 rows][64 B of K]  (32 KB)
//   LDS --ds_read_b128--> MFMA operands --v_mfma--> accumulators
//   accumulators --fused epilogue, straight from the registers (the MFMA operands are
//       exchanged, so a lane holds four consecutive n of a row)--> dst stores
//
// Both operands are consumed K-contiguous ("A" rows are src rows, "B^T" rows
// are weight columns).  Loads bypass the register file (direct-to-LDS DMA);
// each wavefront-wide DMA moves 64 x 16 B = 16 rows x 64 B.  Inside a row the
// four 16-byte chunks are XOR-swizzled with the row number so the ds_read_b128
// of an MFMA operand (32 or 16 consecutive rows, one chunk) is free of bank
// conflicts; the swizzle is applied on the global-address side of the DMA.
//
// Pipeline per K step kt (ring slot kt % NSTAGE), in its plainest form:
//   s_waitcnt vmcnt(..)   own DMAs of stage kt landed
//   s_barrier             everybody's did, and everybody finished stage kt-1
//   issue DMAs for stage kt+NSTAGE-1 into the slot stage kt-1 used
//   ds_read + MFMA over stage kt
// Three loops build on it: main_loop (four wavefronts, fragments read inside the
// step), main_loop_two_groups (eight wavefronts in two groups half a step apart)
// and main_loop_ahead (fragments of the next stage read into a second register
// set while the current one is multiplied).
//
// The DMA instructions are emitted through inline assembly so that the
// outstanding-load counter is managed by hand (a prefetch distance of
// NSTAGE-1 stages needs "wait until at most N loads are in flight").
#pragma once
#include <type_traits>

#include "kernels.hpp"
#include "tile_epilogue.hpp"

namespace mi355 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

namespace gemm {

constexpr int BM = 256;               // rows of a workgroup's dst tile
constexpr int BKB = 64;               // bytes of K per row per stage
constexpr int B_OFF = BM * BKB;       // B^T tile offset inside a stage

// Tile geometry: a workgroup of NW wavefronts computes a 256 x BN dst tile, two
// wavefronts along m (128 rows each) and NW/2 along n.
//   geo_t<4, 256>  128x128 per wavefront (256 accumulators), one wavefront per
//                  SIMD: the fewest LDS bytes per MFMA (64 KB of fragment reads
//                  per K step and CU), nothing to hide LDS latency behind
//   geo_t<8, 256>  128x64 per wavefront, two wavefronts per SIMD in two groups
//                  that alternate between reading and multiplying (96 KB of
//                  fragment reads per K step)
//   geo_t<4, 128>  256x128 tiles of four wavefronts, two workgroups per CU: for
//                  problems of at most 128 large tiles, where it puts twice the
//                  CUs to work; with every CU busy it measured 10-30 % slower
//                  (1.5x the stage loads per MFMA; fp8 4096x8192x28672: 1.04
//                  against 0.91 ms)
// Each kernel family uses the one measured faster on its headline shape.
template <int NW_, int BN_>
struct geo_t {
    static constexpr int NW = NW_, NT = 64 * NW_, BN = BN_;
    static constexpr int WN = NW_ / 2;        // wavefronts along n
    static constexpr int WCOLS = BN_ / WN;    // columns of a wavefront's part
    static constexpr int DPA = (BM / 16) / NW_;  // A DMAs per stage and wavefront
    static constexpr int DPB = (BN_ / 16) / NW_; // B^T DMAs per stage and wavefront
    static constexpr int DPS = DPA + DPB;
    static constexpr int STAGE_BYTES = (BM + BN_) * BKB;
    static constexpr int NSTAGE = BN_ == 256 ? 4 : 3; // ring depth: 128 KB or 72 KB
    static constexpr int WG_PER_CU = BN_ == 256 ? 1 : 2;
    // the epilogue needs the ring's memory: accumulator slabs + operand staging
    static_assert(NSTAGE * STAGE_BYTES >= 2 * NW_ * 32 * WCOLS * 4, "epilogue LDS");
    __device__ static __forceinline__ int wm(int wave) { return wave / WN; }
    __device__ static __forceinline__ int wn(int wave) { return wave % WN; }
};

// Chunk swizzle.  Measured on MI355X with a read-only micro-benchmark over all
// XOR-of-row-bits functions: this one is free of bank conflicts for both
// fragment read patterns in use (16 rows x 4 chunks across the 64 lanes, the
// 16x16 MFMA shapes; 32 rows x 2 chunks in two reads, the 32x32 shape), where
// e.g. ((row >> 1) & 3) ^ ((row >> 3) & 1) costs the 16-row pattern a factor
// of two (SQ_LDS_BANK_CONFLICT = half of SQ_LDS_IDX_ACTIVE in the int8 kernel).
__device__ __forceinline__ int swz_f(int row) {
    return ((row >> 2) & 1) | ((((row >> 2) ^ (row >> 3)) & 1) << 1);
}
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

// A workgroup-uniform value pinned to scalar registers: the DMA's base operand
// must be an SGPR pair, and a uniform value that merges at the join of divergent
// code ahead of the K loop counts as divergent from there on.  The value passes
// through an empty asm statement as a vector register, which hides from the
// compiler that it is uniform (it would fold a readfirstlane of a known-uniform
// value away, wherever it keeps it); the readfirstlane itself is the builtin, so
// that the compiler places the wait states the instruction needs after a VALU
// write of its source and before a memory instruction reads its result (an
// inline-assembly v_readfirstlane gets none of them: it read a stale register
// right behind the v_mov that fed it).
__device__ __forceinline__ int scalar_int(int x) {
    asm volatile("" : "+v"(x));
    int r = __builtin_amdgcn_readfirstlane(x);
    // the result may go straight into the base operand of a DMA written in inline
    // assembly, whose wait states after a VALU write of an SGPR (five before a
    // memory instruction reads it) the compiler cannot place either
    asm volatile("s_nop 4" : "+s"(r));
    return r;
}
__device__ __forceinline__ const char *scalar_ptr(const char *p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = (uint32_t)scalar_int((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)scalar_int((int)(uint32_t)(v >> 32));
    return (const char *)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

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
// (A persistent form, one workgroup per CU walking ids blockIdx.x + k * gridDim.x,
// measured the same as one workgroup per tile: the turnover between tiles is
// ~6 us of 130.)
template <class G>
__device__ __forceinline__ tile_pos_t tile_position(int id, int tiles_m, int tiles_n) {
    const int nwg = tiles_m * tiles_n;
    const int per = nwg / 8;
    const int tile = (nwg % 8 == 0) ? (id % 8) * per + id / 8 : id;
    constexpr int GM = 8; // measured: 4 and 8 alike, 16 is 2 % and 32 is 7 % slower on the int8 headline shape
    const int band = tile / (GM * tiles_n);
    const int band_rows = min(GM, tiles_m - band * GM);
    const int in_band = tile - band * GM * tiles_n;
    tile_pos_t p;
    p.m0 = (long)(band * GM + in_band % band_rows) * BM;
    p.n0 = (long)(in_band / band_rows) * G::BN;
    return p;
}

// Per-thread DMA plan: wave w owns DPA blocks of 16 tile rows of A and DPB of
// B^T, one DMA each per stage.
template <int DPA, int DPB>
struct dma_plan_t {
    unsigned voff_a[DPA], voff_b[DPB]; // byte offsets from the scalar tile base
    unsigned lds_a[DPA], lds_b[DPB];   // LDS byte offsets inside a stage
};

template <int DPA, int DPB>
__device__ __forceinline__ dma_plan_t<DPA, DPB> make_dma_plan(int wave, int lane, long rows_a_left,
        long rows_b_left, long lda, long ldb) {
    dma_plan_t<DPA, DPB> p;
#pragma unroll
    for (int i = 0; i < DPA; ++i) {
        const int row = (wave * DPA + i) * 16 + (lane >> 2);
        const int chunk = (lane & 3) ^ swz_f(row);
        long ra = row;
        if (ra > rows_a_left - 1) ra = rows_a_left - 1;
        p.voff_a[i] = (unsigned)(ra * lda + chunk * 16);
        p.lds_a[i] = (unsigned)((wave * DPA + i) * 1024);
    }
#pragma unroll
    for (int i = 0; i < DPB; ++i) {
        const int row = (wave * DPB + i) * 16 + (lane >> 2);
        const int chunk = (lane & 3) ^ swz_f(row);
        long rb = row;
        if (rb > rows_b_left - 1) rb = rows_b_left - 1;
        p.voff_b[i] = (unsigned)(rb * ldb + chunk * 16);
        p.lds_b[i] = (unsigned)(B_OFF + (wave * DPB + i) * 1024);
    }
    return p;
}

// operand policies that supply load_b_one (one B^T fragment at a time) run the
// four-wavefront loop that reads a stage ahead
template <class Mma, class = void>
struct reads_ahead : std::false_type {};
template <class Mma>
struct reads_ahead<Mma, std::enable_if_t<Mma::READS_AHEAD>> : std::true_type {};

// s_waitcnt lgkmcnt(0) only
__device__ __forceinline__ void wait_lds_reads() {
    __builtin_amdgcn_s_waitcnt(0xC07F);
}

// workgroup barrier that neither memory accesses nor MFMAs are scheduled across
__device__ __forceinline__ void phase_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
}

// Main loop for eight wavefronts, two per SIMD, in two groups of four that run
// half a K step apart.  Both groups meet at one workgroup barrier per step; in
// the interval after barrier g
//   group 0:  reads stage g from LDS, then its MFMAs of stage g
//   group 1:  its MFMAs of stage g-1 (fragments read in the previous interval),
//             then reads stage g
// so on every SIMD one wavefront has MFMAs to issue while the other one waits
// for LDS, with every wavefront's instruction stream in plain program order:
// nothing depends on how the compiler interleaves reads with MFMAs.  Both
// groups read stage g in the same interval, so one barrier per step covers
// both conditions: every wavefront waits for its own DMAs of stage g before
// barrier g (then all of stage g is in LDS), and has its reads of stage g-1
// back before it (then that slot may be overwritten by the DMAs of stage
// g+NG-1, which are issued after the barrier).  Group 1 runs one more
// iteration for its last MFMAs.
template <int NSTAGE, int KSTEP, class Mma, class Acc, class Ctx>
__device__ __forceinline__ void main_loop_two_groups(Acc &acc, char *smem, const char *a_tile_,
        const char *b_tile_, long lda, long ldb, long rows_a_left, long rows_b_left, int ngroups_,
        const Ctx &ctx) {
    using G = typename Mma::G;
    const char *a_tile = scalar_ptr(a_tile_), *b_tile = scalar_ptr(b_tile_);
    // (a uniform value merged from two loads at the join of divergent code ahead of
    // the loop counts as divergent, and the stage offsets derive from it)
    const int ngroups = scalar_int(ngroups_);
    static_assert(G::NW == 8, "two groups of four wavefronts");
    constexpr int NG = NSTAGE / KSTEP;
    constexpr int STAGE_BYTES = G::STAGE_BYTES, GROUP_BYTES = KSTEP * STAGE_BYTES;
    constexpr int DPA = G::DPA, DPB = G::DPB, DPS = G::DPS;
    constexpr int GROUP_DMAS = KSTEP * DPS + Mma::EXTRA_DMAS;
    static_assert(NSTAGE % KSTEP == 0 && NG >= 3 && NG <= 5, "ring depth");
    static_assert((NG - 2) * GROUP_DMAS < 64, "vmcnt range");
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const typename Mma::addr_t AD = Mma::lane_addr(G::wm(wave), G::wn(wave), lane);
    const bool late = wave >= 4; // group 1
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem;
    const dma_plan_t<DPA, DPB> plan = make_dma_plan<DPA, DPB>(wave, lane, rows_a_left, rows_b_left, lda, ldb);

    auto issue_part = [&](int g, int slot, int i) __attribute__((always_inline)) {
#pragma unroll
        for (int k = 0; k < KSTEP; ++k) {
            const long koff = ((long)g * KSTEP + k) * BKB;
            const unsigned lds_stage = lds0 + slot * GROUP_BYTES + k * STAGE_BYTES;
            if (i < DPA) dma16(a_tile + koff, plan.voff_a[i], lds_stage + plan.lds_a[i]);
            else dma16(b_tile + koff, plan.voff_b[i - DPA], lds_stage + plan.lds_b[i - DPA]);
        }
        if (i == DPS - 1) Mma::issue_extra(ctx, g, slot, wave, lane);
    };
    // the MFMAs of one stage with the DMAs of stage gd spread between the rows:
    // a DMA instruction can wait tens of cycles for the address unit, which
    // passes unnoticed behind a row of MFMAs
    // Past the last stage the DMAs are issued all the same, clamped to the last
    // stage and into a slot nobody reads again: the MFMA sequence stays one
    // basic block (conditional blocks between the rows make the register
    // allocator spill accumulators), and every stage is followed by the same
    // number of loads, so one outstanding-load count fits every iteration.
    auto mma_stage = [&](const typename Mma::frag_t &f, int gm, int gd, int dslot) __attribute__((always_inline)) {
        const int gdc = gd < ngroups ? gd : ngroups - 1;
#pragma unroll
        for (int i = 0; i < Mma::ROWS; ++i) {
            Mma::mma_row(acc, f, i, ctx, gm);
#pragma unroll
            for (int d = 0; d < DPS; ++d)
                if (d * Mma::ROWS / DPS == i) issue_part(gdc, dslot, d);
            __builtin_amdgcn_sched_barrier(0); // or the DMAs all move to the front
        }
    };

#pragma unroll
    for (int s = 0; s < NG - 1; ++s) {
        const int sc = s < ngroups ? s : ngroups - 1;
#pragma unroll
        for (int i = 0; i < DPS; ++i) issue_part(sc, s, i);
    }

    int slot = 0;
    // Group 1 carries the fragments from one iteration to the next; they start
    // as the operands' zero (Mma::zero_frag: bytes the MFMA row reads as 0 --
    // not all-zero bits for an operand type whose bytes are re-biased at use), so
    // that its first iteration, which has no stage to multiply yet, adds zero
    // products instead of branching around the MFMAs (one MFMA sequence on every
    // path keeps the accumulators where they are).
    typename Mma::frag_t f = Mma::zero_frag();
    const int niter = ngroups + (late ? 1 : 0);
    auto read_stage = [&](int g) __attribute__((always_inline)) {
        unsigned S[KSTEP];
#pragma unroll
        for (int k = 0; k < KSTEP; ++k) S[k] = lds0 + slot * GROUP_BYTES + k * STAGE_BYTES;
        Mma::load_a(f, 0, S, AD, ctx, g);
        Mma::load_b(f, S, AD, ctx, g);
#pragma unroll
        for (int i = 1; i < Mma::ROWS; ++i) Mma::load_a(f, i, S, AD, ctx, g);
    };
#pragma nounroll
    for (int g = 0; g < niter; ++g) {
        // own DMAs of stage g landed; those of NG-2 later stages may stay in flight
        wait_vmcnt<(NG - 2) * GROUP_DMAS>();
        if (late) wait_lds_reads();
        phase_barrier();
        int nslot = slot + NG - 1; // the slot stage g-1 used: free after this barrier
        if (nslot >= NG) nslot -= NG;
        if (!late) read_stage(g);
        __builtin_amdgcn_sched_barrier(0);
        // Group 1 gets the matrix core first: its MFMAs were ready at the barrier,
        // and its reads for the next interval come after them.  At equal priority
        // group 0, which starts ~125 ns later, is served first all the same and
        // group 1's reads end up after all MFMAs of the step, with the matrix core
        // idle (time stamps: 545 ns for group 1's block against 285 ns for group 0's;
        // with the priority 300 against 480, and 1.5-2 % less time per launch).
        if (late) __builtin_amdgcn_s_setprio(3);
        mma_stage(f, g, g + NG - 1, nslot); // group 0: stage g; group 1: stage g-1
        if (late) __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
        if (late && g < ngroups) read_stage(g);
        if (++slot == NG) slot = 0;
    }
    if (!late) phase_barrier(); // the barrier of group 1's last iteration
    // every DMA has landed (the clamped ones included) before the ring's memory
    // is used for something else
    wait_vmcnt<0>();
    phase_barrier();
}

// Main loop for four wavefronts, one per SIMD, with the fragments of the next
// stage read while the current one is multiplied.  A single wavefront per SIMD
// has nobody to cover for it: whatever it waits for, the matrix core waits
// too.  So nothing a stage's MFMAs need is requested inside that stage -- its
// fragments were read from LDS into a second set of registers during the
// previous stage's MFMAs (a stage's fragments are 64-80 registers; one
// wavefront per SIMD has 512), and the only wait between two stages' MFMAs is
// the workgroup barrier itself.
//
// Ring of NSTAGE slots, stage s in slot s % NSTAGE.  At the barrier of
// iteration g
//   every wavefront holds stage g in registers (read during iteration g-1):
//     slot g % NSTAGE is free and takes the DMAs of stage g + NSTAGE;
//   every wavefront's DMAs of stage g+1 have landed (each waited for its own
//     before the barrier): it is read from LDS during this iteration;
//   stages g+2 .. g+NSTAGE-1 stay in flight: NSTAGE-2 stages of lead, as with
//     the ring used the plain way, at one more stage of registers.
// The loop is unrolled by two so that the two fragment sets keep their
// registers (the sets swap roles, not contents); an odd stage count ends with
// one more copy of the body.  Past the last stage the DMAs are issued all the
// same, clamped to the last stage and into a slot nobody reads again, and the
// reads fetch whatever the next slot holds: every iteration is the same
// straight-line code and one outstanding-load count fits all of them.
template <int NSTAGE, class Mma, class Acc, class Ctx>
__device__ __forceinline__ void main_loop_ahead(Acc &acc, char *smem, const char *a_tile_, const char *b_tile_,
        long lda, long ldb, long rows_a_left, long rows_b_left, int nstages_, const Ctx &ctx) {
    using G = typename Mma::G;
    const char *a_tile = scalar_ptr(a_tile_), *b_tile = scalar_ptr(b_tile_);
    const int nstages = scalar_int(nstages_);
    constexpr int STAGE_BYTES = G::STAGE_BYTES;
    constexpr int DPA = G::DPA, DPB = G::DPB, DPS = G::DPS;
    constexpr int STAGE_DMAS = DPS + Mma::EXTRA_DMAS;
    constexpr int ROWS = Mma::ROWS, COLS = Mma::COLS;
    static_assert(NSTAGE >= 3 && (NSTAGE - 1) * STAGE_DMAS < 64, "vmcnt range");
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const typename Mma::addr_t AD = Mma::lane_addr(G::wm(wave), G::wn(wave), lane);
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem;
    const dma_plan_t<DPA, DPB> plan = make_dma_plan<DPA, DPB>(wave, lane, rows_a_left, rows_b_left, lda, ldb);

    auto issue_part = [&](int s, int slot, int i) __attribute__((always_inline)) {
        const long koff = (long)s * BKB;
        const unsigned lds_stage = lds0 + slot * STAGE_BYTES;
        if (i < DPA) dma16(a_tile + koff, plan.voff_a[i], lds_stage + plan.lds_a[i]);
        else dma16(b_tile + koff, plan.voff_b[i - DPA], lds_stage + plan.lds_b[i - DPA]);
        if (i == DPS - 1) Mma::issue_extra(ctx, s, slot, wave, lane);
    };

#pragma unroll
    for (int s = 0; s < NSTAGE; ++s) {
        const int sc = s < nstages ? s : nstages - 1;
#pragma unroll
        for (int i = 0; i < DPS; ++i) issue_part(sc, s, i);
    }
    typename Mma::frag_t f0, f1;
    wait_vmcnt<(NSTAGE - 1) * STAGE_DMAS>();
    phase_barrier();
    {
        const unsigned S[1] = {lds0};
#pragma unroll
        for (int j = 0; j < COLS; ++j) Mma::load_b_one(f0, j, S, AD, ctx, 0);
#pragma unroll
        for (int i = 0; i < ROWS; ++i) Mma::load_a(f0, i, S, AD, ctx, 0);
    }

#ifdef MI355_ABLATE_READS
    wait_lds_reads();
    f1 = f0; // both sets hold real operand bits
#endif
    int slot = 0; // of stage g
    // iteration g: multiply `cur` (stage g), read stage g+1 into `nxt`, DMA stage g+NSTAGE
    auto step = [&](int g, typename Mma::frag_t &cur, typename Mma::frag_t &nxt) __attribute__((always_inline)) {
        wait_vmcnt<(NSTAGE - 2) * STAGE_DMAS>();
        wait_lds_reads();
        phase_barrier();
        Mma::prepare(cur);
        int rslot = slot + 1;
        if (rslot == NSTAGE) rslot = 0;
        const unsigned S[1] = {lds0 + rslot * STAGE_BYTES};
        const int sd = g + NSTAGE < nstages ? g + NSTAGE : nstages - 1;
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
            // (MI355_ABLATE_READS / MI355_ABLATE_DMA: measurement builds that leave the fragment reads / the
            // stage loads out of the loop -- wrong results, the same MFMAs -- to price each by itself)
#ifndef MI355_ABLATE_READS
            Mma::load_a(nxt, i, S, AD, ctx, g + 1);
#pragma unroll
            for (int j = 0; j < COLS; ++j)
                if (j * ROWS / COLS == i) Mma::load_b_one(nxt, j, S, AD, ctx, g + 1);
#endif
#ifndef MI355_ABLATE_DMA
#pragma unroll
            for (int d = 0; d < DPS; ++d)
                if (d * ROWS / DPS == i) issue_part(sd, slot, d);
#endif
            Mma::mma_row(acc, cur, i, ctx, g);
            __builtin_amdgcn_sched_barrier(0); // keeps the reads and DMAs spread between the rows
        }
        slot = rslot;
    };
    int g = 0;
#pragma nounroll
    for (; g + 1 < nstages; g += 2) {
        step(g, f0, f1);
        step(g + 1, f1, f0);
    }
    if (g < nstages) step(g, f0, f1);
    // every DMA has landed (the clamped ones included) and every read is back
    // before the ring's memory is used for something else; the wait states
    // between the last MFMA and the first read of its result, which the compiler
    // cannot count for an MFMA written as inline assembly
    wait_vmcnt<0>();
    wait_lds_reads();
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    phase_barrier();
}

// operand policies that supply zero_tail take a K that ends inside a stage
template <class Mma, class = void>
struct has_k_tail : std::false_type {};
template <class Mma>
struct has_k_tail<Mma, std::enable_if_t<Mma::K_TAIL>> : std::true_type {};

// The end of a K that does not fill its last stage, after the main loop has
// taken the whole stages: one more stage whose 64 bytes per row are the LAST 64
// bytes of the row -- a_win / b_win point 64 bytes before the row's end, so no
// byte beyond the row is touched -- of which the first `nz` 16-byte chunks were
// multiplied already and are zeroed in the fragments of both operands
// (Mma::zero_tail; both operands hold the same k in the same place, so the
// shift inside the stage does not matter to the products).  g_tail = the number
// of whole stages = the tail's stage number for the policy's own loads.  Not pipelined: it
// costs a problem with such a K a few microseconds per tile and the others
// nothing.  The ring is idle on entry and on return.
template <class Mma, class Acc, class Ctx>
__device__ __forceinline__ void tail_step(Acc &acc, char *smem, const char *a_win_, const char *b_win_, long lda,
        long ldb, long rows_a_left, long rows_b_left, int nz_, int g_tail, const Ctx &ctx) {
    using G = typename Mma::G;
    const char *a_win = scalar_ptr(a_win_), *b_win = scalar_ptr(b_win_);
    const int nz = scalar_int(nz_);
    constexpr int DPA = G::DPA, DPB = G::DPB;
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const typename Mma::addr_t AD = Mma::lane_addr(G::wm(wave), G::wn(wave), lane);
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem;
    const dma_plan_t<DPA, DPB> plan = make_dma_plan<DPA, DPB>(wave, lane, rows_a_left, rows_b_left, lda, ldb);
#pragma unroll
    for (int i = 0; i < DPA; ++i) dma16(a_win, plan.voff_a[i], lds0 + plan.lds_a[i]);
#pragma unroll
    for (int i = 0; i < DPB; ++i) dma16(b_win, plan.voff_b[i], lds0 + plan.lds_b[i]);
    Mma::issue_extra(ctx, g_tail, 0, wave, lane); // what rides along with stage number g_tail (block scales)
    wait_vmcnt<0>();
    phase_barrier();
    typename Mma::frag_t f;
    const unsigned S[1] = {lds0};
    Mma::load_b(f, S, AD, ctx, 0);
#pragma unroll
    for (int i = 0; i < Mma::ROWS; ++i) Mma::load_a(f, i, S, AD, ctx, 0);
    wait_lds_reads();
    Mma::zero_tail(f, nz, lane);
#pragma unroll
    for (int i = 0; i < Mma::ROWS; ++i) Mma::mma_row(acc, f, i, ctx, 0);
    phase_barrier();
}

// Main loop.  The ring holds NSTAGE stages; one iteration consumes KSTEP of
// them (a "group": KSTEP * 64 bytes of K), so NSTAGE / KSTEP groups rotate.
// Per group g:
//   s_waitcnt vmcnt(..)   own DMAs of group g landed
//   s_barrier             everybody's did, and everybody finished group g-1
//   DMA group g+NG-1      into the slots group g-1 used
//   ds_read + MFMA over group g
// `Mma` supplies the tile geometry G, frag_t, addr_t lane_addr(wm, wn, lane)
// (this lane's LDS offsets of fragment 0 of both operands inside a stage; the
// other fragments are constant offsets from it, which ride in the offset field
// of the reads instead of one address register per fragment), load_b(frag, S,
// addr, ctx, g) for the B^T fragments, load_a(frag, i, S, addr, ctx, g) for A
// fragment i (S[k] is the LDS byte address of the k-th stage of the group),
// mma_row(acc, frag, i, ctx, g) for the COLS MFMAs of A fragment i (ROWS x COLS
// MFMA tiles per wavefront), and A_READS / B_READS = LDS read instructions per
// fragment.
// a_tile / b_tile point at the first K byte of tile row 0.
template <int NSTAGE, int KSTEP, class Mma, class Acc, class Ctx>
__device__ __forceinline__ void main_loop(Acc &acc, char *smem, const char *a_tile_,
        const char *b_tile_, long lda, long ldb, long rows_a_left, long rows_b_left, int ngroups_,
        const Ctx &ctx) {
    using G = typename Mma::G;
    const char *a_tile = scalar_ptr(a_tile_), *b_tile = scalar_ptr(b_tile_);
    // (a uniform value merged from two loads at the join of divergent code ahead of
    // the loop counts as divergent, and the stage offsets derive from it)
    const int ngroups = scalar_int(ngroups_);
    constexpr int NG = NSTAGE / KSTEP;           // groups in the ring
    constexpr int STAGE_BYTES = G::STAGE_BYTES, GROUP_BYTES = KSTEP * STAGE_BYTES;
    if constexpr (NSTAGE >= 4 && KSTEP == 1 && reads_ahead<Mma>::value) {
        main_loop_ahead<NSTAGE, Mma>(acc, smem, a_tile_, b_tile_, lda, ldb, rows_a_left, rows_b_left, ngroups_, ctx);
        return;
    }
    if constexpr (G::NW == 8) {
        main_loop_two_groups<NSTAGE, KSTEP, Mma>(acc, smem, a_tile_, b_tile_, lda, ldb, rows_a_left,
                rows_b_left, ngroups_, ctx);
        return;
    }
    constexpr int DPA = G::DPA, DPB = G::DPB, DPS = G::DPS;
    constexpr int GROUP_DMAS = KSTEP * DPS + Mma::EXTRA_DMAS;
    static_assert(NSTAGE % KSTEP == 0 && NG >= 2 && NG <= 5, "ring depth");
    static_assert((NG - 2) * GROUP_DMAS < 64, "vmcnt range");
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const typename Mma::addr_t AD = Mma::lane_addr(G::wm(wave), G::wn(wave), lane);
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)smem;
    const dma_plan_t<DPA, DPB> plan = make_dma_plan<DPA, DPB>(wave, lane, rows_a_left, rows_b_left, lda, ldb);

    // DMA number i (0..DPS-1) of every stage of group g: A row blocks first, then B^T
    auto issue_part = [&](int g, int slot, int i) __attribute__((always_inline)) {
#pragma unroll
        for (int k = 0; k < KSTEP; ++k) {
            const long koff = ((long)g * KSTEP + k) * BKB;
            const unsigned lds_stage = lds0 + slot * GROUP_BYTES + k * STAGE_BYTES;
            if (i < DPA) dma16(a_tile + koff, plan.voff_a[i], lds_stage + plan.lds_a[i]);
            else dma16(b_tile + koff, plan.voff_b[i - DPA], lds_stage + plan.lds_b[i - DPA]);
        }
        if (i == DPS - 1) Mma::issue_extra(ctx, g, slot, wave, lane);
    };

    // prologue: groups 0 .. NG-2 in flight
#pragma unroll
    for (int s = 0; s < NG - 1; ++s)
        if (s < ngroups) {
#pragma unroll
            for (int i = 0; i < DPS; ++i) issue_part(s, s, i);
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
        // A fragment 0 first: LDS reads return in order, so the first MFMA can go
        // as soon as it and the first B fragment are in
        Mma::load_a(f, 0, S, AD, ctx, g);
        Mma::load_b(f, S, AD, ctx, g);
        Mma::load_a(f, 1, S, AD, ctx, g);
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
            if (dma) {
#pragma unroll
                for (int d = 0; d < DPS; ++d) // spread evenly over the rows
                    if (d * ROWS / DPS == i) issue_part(g + NG - 1, nslot, d);
            }
            if (i + 2 < ROWS) Mma::load_a(f, i + 2, S, AD, ctx, g);
            Mma::mma_row(acc, f, i, ctx, g);
        }
        if (++slot == NG) slot = 0;
    }
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
}

} // namespace gemm
} // namespace mi355
