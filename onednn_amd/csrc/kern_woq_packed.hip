// "hip:woq_packed" -- the weight-only-quantized decode of kern_woq.hip over
// weights in the MI355_WEI_PACK_WOQ64 layout: bf16 activations (M <= 32 rows)
// times 4-bit weights, per-group scales and zero points along K, fpmath
// "apply_to_int" weight decompression.
//
// Semantics (ref_matmul_t, src/cpu/matmul/ref_matmul.cpp:179-235, weights
// decompression branch :193-214) and the evaluation
//     dst[m,n] = sum_g scale[g,n] * ( sum_{k in g} src[m,k] * (128 + wei[k,n])
//                                     - (128 + zp[g,n]) * sum_{k in g} src[m,k] )
// are those of "hip:woq_gemv"; so is the comparison with the reference (bf16
// threshold plus the forward error bound of the K sum).
//
// What the layout buys.  A 64-column chunk holds all of K contiguously, so one
// workgroup owns 64 columns of dst and all of K: no K split across workgroups,
// no partial sums in memory, no second kernel, and N / 64 workgroups fill the
// device for the decode shapes (224 for N = 14336).  A wavefront reads 32 rows
// x 64 columns as one 1 KB run, 16 bytes per lane.  Lane (q = lane / 16,
// j = lane % 16) receives, for each of the four 16-column blocks t, one dword
// with rows 8q .. 8q+7 of column 16t + j, nibbles ordered so that
//     ((dword >> 4u) & 0x000F000F) | 0x43004300,   u = 0..3
// are the eight bf16 values 128 + w in matrix-core order: one dword is the
// whole B operand of a lane for one v_mfma_f32_16x16x32_bf16, with no
// zero-interleaved A operand (half the matrix-core work of the plain layout).
// The A operand is 16 bytes of a src row, the same k order by construction.
//
// The wavefronts of a workgroup (16 for M <= 16, 8 above) split K, keep their
// sums in registers across quantization groups and add them through LDS at the
// end, in wavefront order: results do not depend on timing.
//
// The launch lasts a few microseconds, so what a wavefront does before its
// loads are in flight and after its last data arrive is as visible as the
// stream itself:
//  - the loop's operands are the first 112 bytes of the kernel arguments and
//    are fetched with one burst of scalar loads; the problem description is
//    read only by the general epilogue;
//  - a problem with nothing after the K sum but the conversion to f32 / bf16 /
//    f16 (no bias, post-ops, dst scale or zero point) runs a kernel whose end
//    is a sum over the wavefronts and one store: no further argument fetch, no
//    instruction-cache misses on an epilogue interpreter;
//  - a wavefront's loads return as one burst, late ones last, and its whole
//    unpack + MFMA work then follows that burst: more wavefronts with fewer
//    steps each keep this tail short;
//  - the parameter decode at a group's end is straight-line code (candidate
//    conversions selected by uniform masks), no data-type switch.
#include "kernels.hpp"
#include "tile_epilogue.hpp"

#include <type_traits>

// Measurement builds (wrong results, timing only; `make EXTRA=-DMI355_WOQP_ABL=n OBJDIR=... OUT=...`): what a launch
// costs with one part of the kernel taken out.  1: every unit reads the activations of the wavefront's first unit
// (no activation traffic beyond the caches); 2: every unit reads the weights of the first unit (a quarter of the
// weights' bytes); 3: no flush of the groups; 4: no LDS staging of the activations; 5: no unpacking; 6: loads,
// waits, the sum over the wavefronts and the store only.
#ifndef MI355_WOQP_ABL
#define MI355_WOQP_ABL 0
#endif
namespace mi355 {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned v16u __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

constexpr int CHUNK = 64;      // columns per workgroup
constexpr int KBLK = 32;       // rows per step (one MFMA depth)
constexpr int NO_GROUPS = 1 << 30;

struct woqp_extra_t {
    const uint8_t *wei;  // packed, K * N / 2 bytes
    const uint8_t *src;  // bf16 [M][src_ld]
    const uint8_t *sc, *zp; // weights scales / zero points (NULL when absent)
    uint8_t *dst;        // the plain store: dst_dt in {f32, bf16, f16}, rows dst_ld elements apart
    int dst_dt, dst_ld;
    int M, N, K, src_ld;
    int kbw;             // 32-row blocks per wavefront
    int spg;             // 32-row blocks per quantization group, NO_GROUPS without groups
    int sc_dt, zp_dt;    // MI355_DT_UNDEF when absent (sc / zp then point at any readable memory)
    int sc_bits, zp_bits; // bits per element, 0 when absent (every lane then reads the first dword)
    int sc_grouped, zp_grouped; // parameter has a K dimension
    int zp_common;       // single zero point
    int signed_w;        // s4 weights
    int pad[6];
};
static_assert(sizeof(woqp_extra_t) == 128, "fetched as two 64-byte scalar loads");

// the one kernel argument: the loop's operands first
struct woqp_args_t {
    woqp_extra_t X;
    problem_t P;
};
typedef const __attribute__((address_space(4))) woqp_args_t kernarg_woqp_t;

__device__ __forceinline__ v8bf as_bf(const v4i &x) { return __builtin_bit_cast(v8bf, x); }

// Loads through pointers of the global address space.  The kernel's pointers come out of a block of scalar
// registers filled by inline assembly, so the compiler cannot tell that they point to global memory and would
// emit flat loads: those count on the LDS counter as well as on the vector-memory counter, and every wait for an
// LDS access (the activations' staging) then waits for every load in flight -- the next unit's included.
// An address is a wavefront-uniform base (scalar registers) plus a lane's 32-bit byte offset plus a constant:
// the form a global load takes as it is (base in a scalar pair, offset in one vector register, the constant in
// the instruction), so stepping along K costs scalar additions only.
typedef const uint8_t __attribute__((address_space(1))) *global_bytes_t;
typedef const v4u __attribute__((address_space(1))) *global_v4u_ptr_t;
typedef const unsigned __attribute__((address_space(1))) *global_u32_ptr_t;
__device__ __forceinline__ global_bytes_t gaddr(const uint8_t *base, unsigned voff, int imm) {
    return (global_bytes_t)(uintptr_t)base + voff + imm;
}
// Marks a base as wavefront-uniform for the compiler (a no-op on a value that is in scalar registers already):
// without it loop strength reduction folds the lane's offset into a per-lane 64-bit pointer per stream, kept in
// vector registers across the loop.
__device__ __forceinline__ const uint8_t *uniform_ptr(const uint8_t *p) {
    const uintptr_t v = (uintptr_t)p;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    return (const uint8_t *)(((uintptr_t)hi << 32) | lo);
}
// A lane's offset as a value defined where it is used: its zero-extension then stays next to the load instead of
// being hoisted out of the loop as a 64-bit pair, and the load keeps the scalar-base form.
__device__ __forceinline__ unsigned here(unsigned voff) {
    asm volatile("" : "+v"(voff));
    return voff;
}
__device__ __forceinline__ v4u gload16(const uint8_t *base, unsigned voff, int imm = 0) {
    return *(global_v4u_ptr_t)gaddr(base, voff, imm);
}
__device__ __forceinline__ v4u gload16_nt(const uint8_t *base, unsigned voff, int imm = 0) {
    return __builtin_nontemporal_load((global_v4u_ptr_t)gaddr(base, voff, imm));
}
__device__ __forceinline__ unsigned gload4(const uint8_t *base, unsigned voff) {
    return *(global_u32_ptr_t)gaddr(base, voff, 0);
}

// The main loop's loads are written as instructions of their own and waited for by hand.  The counter of
// outstanding loads is waited for by position from the end of the queue; where one piece of code is reached with
// and without the next unit's loads behind the current one's, the compiler has to assume "without" and would wait
// for the next unit as well -- no overlap of one unit's loads with the other's arithmetic.  Here the wait is picked
// by a uniform branch on what is behind.  Between the first of these loads and the last of these waits the kernel
// must not contain other vector-memory instructions: no spilled registers in particular (the build of this file
// shows none).
template <int N>
__device__ __forceinline__ void wait_vm() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N));
}
__device__ __forceinline__ void aload4(unsigned &d, const uint8_t *base, unsigned voff) {
    asm volatile("global_load_dword %0, %1, %2" : "=&v"(d) : "v"(voff), "s"(base));
}
template <int IMM>
__device__ __forceinline__ void aload16(v4u &d, const uint8_t *base, unsigned voff) {
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=&v"(d) : "v"(voff), "s"(base), "n"(IMM));
}
template <int IMM>
__device__ __forceinline__ void aload16_nt(v4u &d, const uint8_t *base, unsigned voff) {
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3 nt" : "=&v"(d) : "v"(voff), "s"(base), "n"(IMM));
}
// a value loaded above is used only after the wait that precedes this
template <class T>
__device__ __forceinline__ void arrived(T &x) {
    asm volatile("" : "+v"(x));
}
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I> {});
        static_for<I + 1, N>(f);
    }
}

// Quantization parameters are fetched as the aligned dword that holds the
// element (no branch on the data type next to the load, so a fetch never waits
// for its own data); the element is cut out when the group is flushed.  A row
// of parameters (one group, N elements) is a multiple of four bytes, so a
// lane's offset inside the row, the shift and the mask are the same for every
// group and a fetch costs one scalar multiply-add and the load.
struct param_lane_t {
    const uint8_t *base; // aligned down to four bytes
    long pitch;          // bytes between groups, 0 without groups
    unsigned voff, sh, mask;
};

__device__ __forceinline__ param_lane_t param_setup(const uint8_t *p, int bits, long n, bool grouped, long N) {
    param_lane_t L;
    const unsigned mis = (unsigned)((uintptr_t)p & 3);
    const long bitoff = n * bits;
    const unsigned byte = (unsigned)(bitoff >> 3) + mis;
    L.base = p - mis;
    L.pitch = grouped ? N * bits / 8 : 0;
    L.voff = byte & ~3u;
    L.sh = (byte & 3) * 8u + ((unsigned)bitoff & 4u);
    L.mask = 0xffffffffu >> ((32 - bits) & 31);
    return L;
}

__device__ __forceinline__ unsigned param_word(const param_lane_t &L, int g) {
    return gload4(uniform_ptr(L.base + g * L.pitch), here(L.voff));
}

__device__ __forceinline__ unsigned param_cut(const param_lane_t &L, unsigned word) { return (word >> L.sh) & L.mask; }

// Straight-line decodes: every candidate is a couple of instructions and the
// data type is uniform, so selects cost less than branches.
__device__ __forceinline__ float decode_scale(int dt, unsigned raw) {
    const float h = (float)__builtin_bit_cast(_Float16, (unsigned short)raw);
    float r = u2f(raw << (dt == MI355_DT_BF16 ? 16 : 0));
    r = dt == MI355_DT_F16 ? h : r;
    return dt == MI355_DT_UNDEF ? 1.f : r;
}

// raw holds `bits` bits, zero-extended
__device__ __forceinline__ float decode_zp(int dt, int bits, unsigned raw) {
    const int sh = (32 - bits) & 31;
    const unsigned x = raw << sh;
    const bool sgn = dt == MI355_DT_S32 || dt == MI355_DT_S8 || dt == MI355_DT_S4;
    const int v = sgn ? (int)x >> sh : (int)(x >> sh);
    return dt == MI355_DT_UNDEF ? 0.f : (float)v;
}

// MT 16-row tiles of activations; SS steps per super-step (all of its loads
// are issued before its first MFMA); SPG steps per quantization group when a
// super-step holds whole groups, 0 when a group holds whole super-steps.
// NWV wavefronts per workgroup.  PLAIN: nothing follows the K sum but the
// conversion to the dst type.
template <int NWV, int MT, int SS, int SPG, bool PLAIN>
__global__ void __launch_bounds__(NWV * 64)
        woqp_kernel(const std::conditional_t<PLAIN, woqp_extra_t, woqp_args_t> A_) {
    __shared__ v4f red4[NWV * MT * 4 * 64];
    // the loop's operands in one burst of scalar loads (left to itself the
    // compiler fetches each field where it is first used, a round trip through
    // the scalar cache each)
    struct raw_args_t {
        v16u lo, hi;
    } raw;
    asm volatile("s_load_dwordx16 %0, %2, 0x0\n\ts_load_dwordx16 %1, %2, 0x40\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(raw.lo), "=&s"(raw.hi)
                 : "s"(__builtin_amdgcn_kernarg_segment_ptr()));
    const woqp_extra_t X = __builtin_bit_cast(woqp_extra_t, raw);
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int j = lane & 15, q = lane >> 4;
    const int chunk = blockIdx.x;
    const int N = X.N, K = X.K, M = X.M;
    const int KB = K / KBLK;
    const int kb0 = wave * X.kbw;
    const int kb1 = kb0 + X.kbw < KB ? kb0 + X.kbw : KB;

    const uint8_t *wbase = X.wei + (long)chunk * K * (CHUNK / 2); // uniform; the lane's share starts at lane * 16
    const unsigned wlane = (unsigned)lane * 16u;
    // MFMA rows beyond M read the last valid row: an output row depends on its
    // own src row only, and those results are never stored
    constexpr bool ALDS = MT == 2;
    static_assert(SS % 2 == 0, "activations are loaded for pairs of steps");
    // ALDS: the loader's lane = row + 8 * slot over eight rows and two steps; else the lane's operand row
    const int lr = lane & 7, lc = lane >> 3;
    unsigned src_off[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int row = ALDS ? mt * 16 + 8 * h + lr : mt * 16 + j;
            const int m = row < M ? row : M - 1;
            src_off[mt][h] = (unsigned)(m * X.src_ld * 2 + (ALDS ? lc : q) * 16);
        }
    // quantization parameters: lane l fetches column l of the chunk, the
    // columns a lane accumulates (16t + j) come from lanes 16t + j at the flush
    const long n_param = (long)chunk * CHUNK + lane;
    const param_lane_t Lsc = param_setup(X.sc, X.sc_bits, n_param, X.sc_grouped, N);
    const param_lane_t Lzp = param_setup(X.zp, X.zp_bits, X.zp_common ? 0 : n_param, X.zp_grouped, N);
    auto fetch_params = [&](unsigned &word_s, unsigned &word_z, int g) __attribute__((always_inline)) {
        word_s = param_word(Lsc, g);
        word_z = param_word(Lzp, g);
    };

    // A unit: the steps whose loads are issued together, before the first of them is multiplied.  One tile of
    // rows: a super-step.  Two tiles: half a super-step, and the next unit is requested before the current one is
    // multiplied (a wavefront has two super-steps or more there, and with one in flight at a time the memory
    // pipeline would drain while each is multiplied): the same registers hold loads in flight all the time.
    constexpr bool PIPE = MT == 2 && (SS / 2) % 2 == 0 && (SPG == 0 || (SS / 2) % (SPG ? SPG : 1) == 0);
    constexpr int U = PIPE ? SS / 2 : SS;                // steps per unit
    constexpr int NGU = SPG ? (U / (SPG ? SPG : 1) > 0 ? U / (SPG ? SPG : 1) : 1) : 1; // groups per unit
    struct unit_t {
        unsigned raw_s[NGU], raw_z[NGU];
        // a[p][mt][h]: ALDS: pair p of steps, rows 8h .. 8h + 7; else step 2p + h in operand order
        v4u a[U / 2][MT][2], w[U];
    };
    // Issue order: the groups' parameters (few bytes, needed last -- loads return in order, so they must not queue
    // behind the weights), the activations, the weights; the MFMAs then follow step by step as their loads arrive.
    //
    // Activations.  The MFMA operand of a step is 16 rows x 64 bytes; loaded
    // that way every instruction touches 16 half lines, the other halves are
    // fetched again for the next step, and the launch time grows by 0.35 us per
    // row of src.  With two tiles (ALDS) a load covers two steps of eight rows
    // instead, whole 128-byte lines (lane = row + 8 * slot), and a pair of
    // steps is brought into operand order through 2 KB of LDS per tile and
    // wavefront when its turn comes: slot c of row r is stored at c ^ (r & 7),
    // so the eight lanes that write or read together fall into eight different
    // slots.  The detour costs 0.8 us per launch and halves the growth per row:
    // it pays above 16 rows.
    constexpr int NLOADS = 2 * NGU + MT * U + U; // per unit, in this order: parameters, activations, weights
    auto issue_unit = [&](unit_t &u, int kbu) __attribute__((always_inline)) {
        // (whole groups inside the unit: the group size is SPG)
        const int g0 = SPG ? kbu / (SPG ? SPG : 1) : kbu / X.spg;
        static_for<0, NGU>([&](auto GI) {
            constexpr int gi = decltype(GI)::value;
            aload4(u.raw_s[gi], uniform_ptr(Lsc.base + (g0 + gi) * Lsc.pitch), Lsc.voff);
            aload4(u.raw_z[gi], uniform_ptr(Lzp.base + (g0 + gi) * Lzp.pitch), Lzp.voff);
        });
#if MI355_WOQP_ABL == 1
        const uint8_t *sb = uniform_ptr(X.src + (long)kb0 * (KBLK * 2));
#else
        const uint8_t *sb = uniform_ptr(X.src + (long)kbu * (KBLK * 2));
#endif
        static_for<0, U / 2>([&](auto P) {
            constexpr int p = decltype(P)::value;
            static_for<0, MT>([&](auto MT_) {
                constexpr int mt = decltype(MT_)::value;
                aload16<(ALDS ? 2 * p : 2 * p) * (KBLK * 2)>(u.a[p][mt][0], sb, src_off[mt][0]);
                aload16<(ALDS ? 2 * p : 2 * p + 1) * (KBLK * 2)>(u.a[p][mt][1], sb, src_off[mt][1]);
            });
        });
        // the weights are read once: non-temporal loads keep them from
        // displacing the activations and parameters in the caches
#if MI355_WOQP_ABL == 2
        const uint8_t *wb = wbase + (long)kb0 * (KBLK * CHUNK / 2);
#else
        const uint8_t *wb = wbase + (long)kbu * (KBLK * CHUNK / 2);
#endif
        static_for<0, U>([&](auto I) { // (the constant of an instruction reaches 4 KB: four steps per scalar base)
            constexpr int i = decltype(I)::value;
            aload16_nt<(i % 4) * (KBLK * CHUNK / 2)>(u.w[i], uniform_ptr(wb + (i / 4) * (4 * KBLK * CHUNK / 2)), wlane);
        });
    };
    // The wavefront's first unit is requested before anything else is set up: the stream is what the launch waits
    // for, the rest of the prologue (staging indices, sums, constants) runs under it.
    unit_t ua;
    int kb = kb0;
    bool have_a = kb + U <= kb1;
    if (have_a) issue_unit(ua, kb);
    __builtin_amdgcn_sched_barrier(0);

    int wr_idx[2], rd_idx[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        wr_idx[h] = (8 * h + lr) * 8 + (lc ^ lr);
        rd_idx[h] = j * 8 + ((4 * h + q) ^ (j & 7));
    }
    v4u *stage = (v4u *)red4 + wave * (MT * 128);

    v4f acc[MT][4], rsum[MT], tot[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        // (with whole groups inside a unit every group's first step starts its sums from a zero operand)
        if constexpr (SPG == 0) rsum[mt] = v4f {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            if constexpr (SPG == 0) acc[mt][tt] = v4f {0.f, 0.f, 0.f, 0.f};
            tot[mt][tt] = v4f {0.f, 0.f, 0.f, 0.f};
        }
    }
    // 0x4300 | nibble = bf16(128 + nibble).  The constant is kept in a vector
    // register: a VOP3 instruction takes one scalar operand at most, so
    // (x & mask) | magic fuses into v_and_or_b32 only when `magic` is not scalar.
    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));
    const v4i ones = {0x3F803F80, 0x3F803F80, 0x3F803F80, 0x3F803F80};
    const unsigned flip = X.signed_w ? 0x88888888u : 0u; // s4 -> offset-binary
    const float zbase = X.signed_w ? 136.f : 128.f;
    // s4 weights go to offset-binary before they are unpacked: a uniform branch around the exclusive-ors, so the
    // unsigned case does not pay an instruction per dword for them
    auto flip_signed = [&](auto &ws) __attribute__((always_inline)) {
        if (flip != 0) {
            asm volatile("" ::: "memory");
            for (auto &wv : ws) wv ^= flip;
        }
    };

    // `first`: the step opens a quantization group (sums start from zero)
    auto compute_step = [&](const v4u &w, const v4u (&a)[MT], bool first) __attribute__((always_inline)) {
#if MI355_WOQP_ABL == 6
        // (timing build: the loads and waits only)
        tot[0][0][0] += u2f(w[0] ^ w[1] ^ w[2] ^ w[3] ^ a[0][0] ^ a[MT - 1][3]);
        return;
#endif
        v4i av[MT];
        const v4f zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            av[mt] = v4i {(int)a[mt][0], (int)a[mt][1], (int)a[mt][2], (int)a[mt][3]};
            rsum[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf(av[mt]), as_bf(ones), first ? zero : rsum[mt], 0, 0, 0);
        }
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            const unsigned d = w[tt];
            v4i b;
#pragma unroll
            for (int u = 0; u < 4; ++u)
                b[u] = MI355_WOQP_ABL == 5 ? (int)(d + u) : (int)(((d >> (4 * u)) & 0x000F000Fu) | magic);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                acc[mt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf(av[mt]), as_bf(b), first ? zero : acc[mt][tt], 0, 0, 0);
        }
    };

    // tot += scale * (acc - (128 + zp) * rowsum) for one finished group (rows
    // beyond M hold the sums of row M - 1: finite, never stored).  ZERO: the
    // next step does not start the sums from zero by itself.
    auto flush_group = [&](unsigned word_s, unsigned word_z, bool zero_sums) __attribute__((always_inline)) {
#if MI355_WOQP_ABL == 3 || MI355_WOQP_ABL == 6
        if (word_s != 0x12345678u) return; // (timing build: practically never flushes)
#endif
        const float s = decode_scale(X.sc_dt, param_cut(Lsc, word_s));
        const float z = decode_zp(X.zp_dt, X.zp_bits, param_cut(Lzp, word_z)) + zbase;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            const float st = __shfl(s, tt * 16 + j, 64);
            const float zt = __shfl(z, tt * 16 + j, 64);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    tot[mt][tt][r] = __builtin_fmaf(st, __builtin_fmaf(-zt, rsum[mt][r], acc[mt][tt][r]), tot[mt][tt][r]);
                if (zero_sums) acc[mt][tt] = v4f {0.f, 0.f, 0.f, 0.f};
            }
        }
        if (zero_sums) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) rsum[mt] = v4f {0.f, 0.f, 0.f, 0.f};
        }
    };

    // `behind`: the next unit's loads were issued after this unit's
    auto consume_unit = [&](unit_t &u, int kbu, bool behind) __attribute__((always_inline)) {
        // at most n of this unit's loads still outstanding
        auto wait_left = [&](auto N_) __attribute__((always_inline)) {
            constexpr int n = decltype(N_)::value;
            if (behind) wait_vm<n + NLOADS>();
            else wait_vm<n>();
        };
        if (flip != 0) { // s4 weights go to offset-binary before they are unpacked
            wait_left(std::integral_constant<int, 0> {});
            static_for<0, U>([&](auto I) {
                arrived(u.w[decltype(I)::value]);
                u.w[decltype(I)::value] ^= flip;
            });
        }
        static_for<0, U / 2>([&](auto P) {
            constexpr int p = decltype(P)::value;
            v4u as[2][MT];
            wait_left(std::integral_constant<int, NLOADS - (2 * NGU + (p + 1) * 2 * MT)> {});
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                arrived(u.a[p][mt][0]);
                arrived(u.a[p][mt][1]);
            }
            if constexpr (ALDS && MI355_WOQP_ABL != 4 && MI355_WOQP_ABL != 6) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                    for (int h = 0; h < 2; ++h) stage[mt * 128 + wr_idx[h]] = u.a[p][mt][h];
                }
#pragma unroll
                for (int sx = 0; sx < 2; ++sx)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) as[sx][mt] = stage[mt * 128 + rd_idx[sx]];
            } else {
#pragma unroll
                for (int sx = 0; sx < 2; ++sx)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) as[sx][mt] = u.a[p][mt][sx];
            }
            static_for<0, 2>([&](auto SX) {
                constexpr int sx = decltype(SX)::value;
                constexpr int i = 2 * p + sx;
                wait_left(std::integral_constant<int, U - 1 - i> {});
                arrived(u.w[i]);
                // with whole groups inside the unit a group's first step
                // is known at compile time and starts from a zero operand
                compute_step(u.w[i], as[sx], SPG != 0 && i % (SPG ? SPG : 1) == 0);
                if constexpr (SPG != 0) {
                    if constexpr ((i + 1) % (SPG ? SPG : 1) == 0) { // (the parameters came before the weights)
                        arrived(u.raw_s[i / SPG]);
                        arrived(u.raw_z[i / SPG]);
                        flush_group(u.raw_s[i / SPG], u.raw_z[i / SPG], false);
                    }
                }
            });
        });
        if constexpr (SPG == 0) {
            arrived(u.raw_s[0]);
            arrived(u.raw_z[0]);
            if ((kbu + U) % X.spg == 0 || kbu + U >= kb1) flush_group(u.raw_s[0], u.raw_z[0], true);
        }
    };

    if constexpr (PIPE) {
        if (have_a) {
            unit_t ub;
            while (true) {
                const bool more_b = kb + 2 * U <= kb1;
                if (more_b) issue_unit(ub, kb + U);
                consume_unit(ua, kb, more_b);
                kb += U;
                if (!more_b) break;
                const bool more_a = kb + 2 * U <= kb1;
                if (more_a) issue_unit(ua, kb + U);
                consume_unit(ub, kb, more_a);
                kb += U;
                if (!more_a) break;
            }
        }
    } else {
        // (the first unit apart from the loop: as one loop with the issue at its end the 16-wavefront variants
        // run out of their 128 registers)
        if (have_a) {
            consume_unit(ua, kb, false);
            kb += U;
        }
        for (; kb + U <= kb1; kb += U) {
            unit_t un;
            issue_unit(un, kb);
            consume_unit(un, kb, false);
        }
    }
    if (kb < kb1) {
        // ragged end of K: one step at a time, parameters fetched when the
        // group ends
        if constexpr (SPG != 0) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                rsum[mt] = v4f {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int tt = 0; tt < 4; ++tt) acc[mt][tt] = v4f {0.f, 0.f, 0.f, 0.f};
            }
        }
#pragma unroll 1
        for (; kb < kb1; ++kb) {
            v4u a1[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int m = mt * 16 + j < M ? mt * 16 + j : M - 1;
                a1[mt] = gload16(X.src + (long)kb * (KBLK * 2), (unsigned)(m * X.src_ld * 2 + q * 16));
            }
            v4u w1[1] = {gload16_nt(wbase + (long)kb * (KBLK * CHUNK / 2), wlane)};
            flip_signed(w1);
            compute_step(w1[0], a1, false);
            if ((kb + 1) % X.spg == 0 || kb + 1 == kb1) {
                unsigned word_s, word_z;
                fetch_params(word_s, word_z, kb / X.spg);
                flush_group(word_s, word_z, true);
            }
        }
    }

    // ---- add the wavefronts' sums in wavefront order and store.  LDS holds
    // [wavefront][row][column] floats; a thread then owns four consecutive
    // columns of one row and runs the four-wide epilogue of the GEMM tiles.
    if constexpr (ALDS) __syncthreads(); // the sums take the memory the activations were staged in
    float *red = (float *)red4;
    constexpr int WSTRIDE = MT * 16 * CHUNK; // floats per wavefront
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                red[wave * WSTRIDE + (mt * 16 + 4 * q + r) * CHUNK + tt * 16 + j] = tot[mt][tt][r];
    __syncthreads();
    if constexpr (PLAIN) {
        // one element per thread, 64 consecutive columns per wavefront
#pragma unroll 1
        for (int e = t; e < M * CHUNK; e += NWV * 64) {
            const int m = e >> 6, nl = e & 63;
            const float *cell = red + m * CHUNK + nl;
            float v = cell[0];
#pragma unroll
            for (int wv = 1; wv < NWV; ++wv) v += cell[wv * WSTRIDE];
            const unsigned bits = X.dst_dt == MI355_DT_F32 ? f2u(v)
                    : X.dst_dt == MI355_DT_BF16 ? (unsigned)f32_to_bf16(v) : (unsigned)f32_to_f16(v);
            const long off = (long)m * X.dst_ld + chunk * CHUNK + nl;
            if (X.dst_dt == MI355_DT_F32)
                ((unsigned __attribute__((address_space(1))) *)(uintptr_t)X.dst)[off] = bits;
            else
                ((uint16_t __attribute__((address_space(1))) *)(uintptr_t)X.dst)[off] = (uint16_t)bits;
        }
        return;
    } else {
    const auto &P = (*(kernarg_woqp_t *)__builtin_amdgcn_kernarg_segment_ptr()).P;
    if (M <= 8) {
        // few rows: one element per thread (the four-wide path below gathers
        // the epilogue's operands first, which a single pass does not win back)
#pragma unroll 1
        for (int e = t; e < M * CHUNK; e += NWV * 64) {
            const int m = e >> 6, nl = e & 63;
            const float *cell = red + m * CHUNK + nl;
            float v = cell[0];
#pragma unroll
            for (int wv = 1; wv < NWV; ++wv) v += cell[wv * WSTRIDE];
            epilogue_store(P, v, 0, m, chunk * CHUNK + nl);
        }
        return;
    }
#pragma unroll 1
    for (int e = t; e < MT * 16 * (CHUNK / 4); e += NWV * 64) {
        const int m = e >> 4, nq = e & 15;
        if (m >= M) continue;
        const v4f *cell = (const v4f *)(red + m * CHUNK + nq * 4);
        v4f sum = cell[0];
#pragma unroll
        for (int wv = 1; wv < NWV; ++wv) sum += cell[wv * (WSTRIDE / 4)];
        float v[4] = {sum[0], sum[1], sum[2], sum[3]};
        const long n = (long)chunk * CHUNK + nq * 4;
        gemm::apply_epilogue4(P, v, 0, m, n, 4);
        gemm::store4(P, P.ds[2] == 1 && gemm::vec_ok_store(P.dst, P.ds[0], P.ds[1], dt_bits(P.dst_dt)), v, 0, m, n, 4);
    }
    }
}

int scale_ok(int dt) {
    return dt == MI355_DT_UNDEF || dt == MI355_DT_F32 || dt == MI355_DT_BF16 || dt == MI355_DT_F16;
}

int zp_ok(int dt) {
    return dt == MI355_DT_UNDEF || dt == MI355_DT_S32 || dt == MI355_DT_S8 || dt == MI355_DT_U8 || dt == MI355_DT_S4
            || dt == MI355_DT_U4;
}

bool param_layout_ok(const mi355_quant_t &q, long K, bool allow_common, long *G) {
    // per-n with or without groups along K, or a single common value
    *G = K;
    if (q.dt == MI355_DT_UNDEF) return true;
    if (q.mask & 1) return false;
    if (q.mask == 0) return allow_common;
    if (!(q.mask & 4) || q.group[1] != 1) return false;
    if (q.mask & 2) *G = q.group[0];
    return true;
}

// group size along K of the problem (K without groups); 0 if the two
// parameters disagree or their layout is not covered
long group_rows(const mi355_matmul_desc_t &d) {
    long gs, gz;
    if (!param_layout_ok(d.wei_scale, d.K, false, &gs)) return 0;
    if (!param_layout_ok(d.wei_zp, d.K, true, &gz)) return 0;
    const bool sg = !quant_absent(d.wei_scale) && (d.wei_scale.mask & 2);
    const bool zg = !quant_absent(d.wei_zp) && (d.wei_zp.mask & 2);
    if (sg && zg && gs != gz) return 0;
    return sg ? gs : zg ? gz : d.K;
}

// super-step geometry for a tile count and a group size (in 32-row blocks)
struct woqp_geo_t {
    int ss, spg; // template arguments; ss == 0: not covered
};

// Wavefronts per workgroup.  One tile of rows: 16 wavefronts of 8 steps each
// at K = 4096 (a wavefront's work after its last data arrive is what ends the
// launch); two tiles, or groups of fewer than 128 rows (more parameter words in
// flight): 8 wavefronts, the register budget of two per SIMD.
int wavefronts(int mt, long G, long K) { return mt == 1 && (G == K || G >= 4 * KBLK) ? 16 : 8; }

woqp_geo_t pick_geo(int mt, long G, long K) {
    const int ss_max = mt == 1 && wavefronts(mt, G, K) == 8 ? 16 : 8;
    if (G == K) return {ss_max, 0};
    if (G % KBLK != 0) return {0, 0};
    const long spg = G / KBLK;
    if (spg <= ss_max && (spg & (spg - 1)) == 0) {
        // (two tiles of rows and groups of 64: units of two steps -- with four, and two groups' parameters per
        // unit, the kernel does not fit the registers of two wavefronts per SIMD)
        const int ss = mt == 2 && spg == 2 ? 4 : (int)(4 * spg < ss_max ? 4 * spg : ss_max);
        // a group that fills the super-step is the spanning case
        return {ss, spg == ss ? 0 : (int)spg};
    }
    if (spg % ss_max == 0) return {ss_max, 0};
    return {0, 0};
}

} // namespace

int woqp_supported(const mi355_matmul_desc_t &d) {
    if (!woq64_layout_ok(d)) return MI355_UNIMPLEMENTED;
    if (d.src_dt != MI355_DT_BF16 || !d.fpmath_apply_to_int) return MI355_UNIMPLEMENTED;
    if (dt_bits(d.dst_dt) < 8) return MI355_UNIMPLEMENTED;
    if (d.M < 1 || d.M > 32) return MI355_UNIMPLEMENTED;
    // 16-byte loads of src rows at 32-bit byte offsets
    if (d.src_stride[2] != 1 || d.src_stride[1] % 8 != 0 || d.src_stride[1] >= (1L << 25)) return MI355_UNIMPLEMENTED;
    if (d.K * d.N / 2 >= (1L << 40)) return MI355_UNIMPLEMENTED;
    if (!quant_absent(d.src_scale) || !quant_absent(d.src_zp) || !quant_absent(d.src_pr))
        return MI355_UNIMPLEMENTED;
    if (!scale_ok(d.wei_scale.dt) || !zp_ok(d.wei_zp.dt)) return MI355_UNIMPLEMENTED;
    const long G = group_rows(d);
    if (G == 0) return MI355_UNIMPLEMENTED;
    if (pick_geo(d.M <= 16 ? 1 : 2, G, d.K).ss == 0) return MI355_UNIMPLEMENTED;
    return MI355_SUCCESS;
}

int woqp_launch(const mi355_matmul_desc_t &d, const problem_t &P, hipStream_t stream) {
    if (((uintptr_t)P.src | (uintptr_t)P.wei) & 15) {
        set_error("woq_packed: src and weights must be 16-byte aligned");
        return MI355_INVALID_ARGUMENTS;
    }
    const int mt = d.M <= 16 ? 1 : 2;
    const long G = group_rows(d);
    const woqp_geo_t geo = pick_geo(mt, G, d.K);
    const int nw = wavefronts(mt, G, d.K);
    // nothing after the K sum but the conversion?
    const bool plain = P.bias_dt == MI355_DT_UNDEF && P.n_po == 0 && !P.dst_dynamic
            && P.dst_scale.dt == MI355_DT_UNDEF && P.dst_zp.dt == MI355_DT_UNDEF && P.ds[2] == 1
            && (P.dst_dt == MI355_DT_F32 || P.dst_dt == MI355_DT_BF16 || P.dst_dt == MI355_DT_F16)
            && P.ds[1] < (1L << 31);
    woqp_args_t A;
    A.P = P;
    woqp_extra_t &X = A.X;
    X = woqp_extra_t {};
    X.dst = (uint8_t *)P.dst;
    X.dst_dt = P.dst_dt;
    X.dst_ld = (int)P.ds[1];
    X.wei = (const uint8_t *)P.wei;
    X.src = (const uint8_t *)P.src;
    X.M = (int)d.M; X.N = (int)d.N; X.K = (int)d.K;
    X.src_ld = (int)d.src_stride[1];
    X.spg = G == d.K ? NO_GROUPS : (int)(G / KBLK);
    // K range of a wavefront: whole groups when a super-step holds groups,
    // whole super-steps when a group holds super-steps
    const long unit = geo.spg ? geo.spg : (G == d.K ? 1 : geo.ss);
    const long KB = d.K / KBLK;
    X.kbw = (int)(((KB + nw - 1) / nw + unit - 1) / unit * unit);
    X.sc_dt = d.wei_scale.dt;
    X.zp_dt = d.wei_zp.dt;
    // an absent parameter is fetched from src (any readable memory) and ignored
    X.sc = X.sc_dt ? (const uint8_t *)P.wei_scale.p : (const uint8_t *)P.src;
    X.zp = X.zp_dt ? (const uint8_t *)P.wei_zp.p : (const uint8_t *)P.src;
    X.sc_bits = X.sc_dt ? dt_bits(X.sc_dt) : 0;
    X.zp_bits = X.zp_dt ? dt_bits(X.zp_dt) : 0;
    X.sc_grouped = X.sc_dt && (d.wei_scale.mask & 2);
    X.zp_grouped = X.zp_dt && (d.wei_zp.mask & 2);
    X.zp_common = X.zp_dt && d.wei_zp.mask == 0;
    X.signed_w = d.wei_dt == MI355_DT_S4;
    const dim3 grid((unsigned)(d.N / CHUNK)), block(nw * 64);
#define MI355_WOQP_CASE(NW_, MT_, SS_, SPG_) \
    if (nw == NW_ && mt == MT_ && geo.ss == SS_ && geo.spg == SPG_) { \
        if (plain) \
            hipLaunchKernelGGL((woqp_kernel<NW_, MT_, SS_, SPG_, true>), grid, block, 0, stream, A.X); \
        else \
            hipLaunchKernelGGL((woqp_kernel<NW_, MT_, SS_, SPG_, false>), grid, block, 0, stream, A); \
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR; \
    }
    MI355_WOQP_CASE(16, 1, 8, 4)
    MI355_WOQP_CASE(16, 1, 8, 0)
    MI355_WOQP_CASE(8, 1, 4, 1)
    MI355_WOQP_CASE(8, 1, 8, 2)
    MI355_WOQP_CASE(8, 2, 4, 1)
    MI355_WOQP_CASE(8, 2, 4, 2)
    MI355_WOQP_CASE(8, 2, 8, 4)
    MI355_WOQP_CASE(8, 2, 8, 0)
#undef MI355_WOQP_CASE
    set_error("woq_packed: no kernel for %d tiles, super-step %d, group %d", mt, geo.ss, geo.spg);
    return MI355_UNIMPLEMENTED;
}

} // namespace mi355
