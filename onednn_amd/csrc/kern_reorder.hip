// "hip:reorder" -- the reorder primitive for plain strided tensors: layout
// change (any permutation of dims), data-type conversion and (de)quantization
// in one pass over the data.  Bound: HBM.
//
// Arithmetic per element, in the reference's order (generic reorder
// simple_reorder_impl_t<..., spec::reference>::execute,
// src/cpu/reorder/simple_reorder.hpp:2579-2661; 4-bit sources :2291-2425,
// 4-bit destinations :2168-2288):
//   d = src_scale * (src - src_zp)      integer sources subtract as integers
//   d += beta * dst_old                 sum post-op
//   d = d / dst_scale + dst_zp          only when a dst scale or zero point is set
//   dst = saturate_and_round<dst_dt>(d) (src/cpu/simple_q10n.hpp:41-81)
// e8m0 sources are converted without arithmetic (:2645-2655).
//
// Two general kernels:
//   direct  the unit-stride dim of dst is also unit-stride in src (or no dim
//           is): consecutive lanes walk that dim, four elements per lane when
//           it divides, stores packed to 2 / 4 / 8 / 16 bytes.
//   tiled   src and dst are unit-stride along different dims (a transposition):
//           a 64x64 tile of the two dims goes through LDS, read with lanes
//           along the src dim and written with lanes along the dst dim, so
//           both sides move whole cache lines.
// and dedicated ones for what the matmul path does with a reorder:
//   rows          quantization of activations / weights (float src, 8-bit dst,
//                 scales per tensor or per column), data types as template
//                 parameters, parameters fetched once per lane
//   transpose8(w) 8-bit transposition in registers (the layout change of
//                 int8 / fp8 weights), 64 x 64 or 128 x 128 tiles
//   pack_woq64    4-bit weights into the packed decode layout
// MI355_REORDER_GENERIC=1 in the environment keeps rows and transpose8w out.
#include "kernels.hpp"
#include "tile_epilogue.hpp" // div_by_fma

namespace mi355 {
namespace {

constexpr int RD = MI355_REORDER_MAX_DIMS;
constexpr int NQ = 3; // src scales, dst scales, src zero points (dst zero point is one value)

// One logical dim as the kernels see it: extent, element strides of both
// tensors and, per quantization parameter tensor, its stride along this dim
// (0 = broadcast) and the group size (logical indices per parameter).
struct rdim_t {
    unsigned n;
    unsigned qg[NQ];
    long ss, ds;
    long qs[NQ];
};

struct reorder_t {
    int src_dt, dst_dt;
    float beta;
    int n_outer;        // dims besides `a` (and `b` in the tiled kernel)
    const void *src;
    void *dst;
    const void *qp[NQ]; // parameter tensors, null = absent
    const void *dst_zp; // one s32, null = absent
    int qdt[NQ];
    int elems;          // elements per lane along `a`: 1, 2 or 4
    int src_vec;        // the `elems` src elements of a lane are one aligned vector load
    int packed;         // ... and the dst elements one aligned vector store
    int plain_copy;     // same data type, no attributes
    rdim_t a;           // the dim lanes walk: smallest dst stride
    rdim_t b;           // tiled kernel: the dim with src stride 1
    rdim_t outer[RD];   // the remaining dims, any order
    unsigned outer_total;
    unsigned tiles_a, tiles_b;
};

__device__ __forceinline__ bool is_int_dt(int dt) {
    return dt == MI355_DT_S32 || dt == MI355_DT_S8 || dt == MI355_DT_U8 || dt == MI355_DT_S4
            || dt == MI355_DT_U4;
}

struct rbase_t { // offsets contributed by the outer dims
    long so, dof;
    long q[NQ];
};

// (RT: the structure is read in place from the kernel argument segment)
template <class RT>
__device__ __forceinline__ rbase_t outer_base(const RT &R, unsigned o) {
    rbase_t B;
    B.so = 0; B.dof = 0;
#pragma unroll
    for (int k = 0; k < NQ; ++k) B.q[k] = 0;
    for (int i = 0; i < R.n_outer; ++i) {
        const unsigned n = R.outer[i].n;
        const unsigned q = o / n, r = o - q * n;
        o = q;
        B.so += (long)r * R.outer[i].ss;
        B.dof += (long)r * R.outer[i].ds;
#pragma unroll
        for (int k = 0; k < NQ; ++k)
            if (R.outer[i].qs[k]) B.q[k] += (long)(r / R.outer[i].qg[k]) * R.outer[i].qs[k];
    }
    return B;
}

template <class DT_>
__device__ __forceinline__ void add_dim(rbase_t &B, const DT_ &d, unsigned i) {
    B.so += (long)i * d.ss;
    B.dof += (long)i * d.ds;
#pragma unroll
    for (int k = 0; k < NQ; ++k)
        if (d.qs[k]) B.q[k] += (long)(d.qg[k] == 1 ? i : i / d.qg[k]) * d.qs[k];
}

// offsets of the N consecutive indices i .. i+N-1 along dim d
template <int N, class DT_>
__device__ __forceinline__ void add_dim_run(rbase_t (&B)[N], const rbase_t &B0, const DT_ &d, unsigned i) {
    B[0] = B0;
    add_dim(B[0], d, i);
#pragma unroll
    for (int e = 1; e < N; ++e) {
        B[e].so = B[e - 1].so + d.ss;
        B[e].dof = B[e - 1].dof + d.ds;
#pragma unroll
        for (int k = 0; k < NQ; ++k) {
            B[e].q[k] = B[e - 1].q[k];
            if (d.qs[k]) {
                if (d.qg[k] == 1) B[e].q[k] += d.qs[k];
                else B[e].q[k] = B0.q[k] + (long)((i + e) / d.qg[k]) * d.qs[k];
            }
        }
    }
}

// raw storage bits of one element -> its value (8-bit and wider types)
__device__ __forceinline__ float raw_to_float(int dt, uint32_t w) {
    switch (dt) {
        case MI355_DT_F32: return u2f(w);
        case MI355_DT_BF16: return bf16_to_f32((uint16_t)w);
        case MI355_DT_F16: return f16_to_f32((uint16_t)w);
        case MI355_DT_F8_E4M3: return e4m3_to_f32((uint8_t)w);
        case MI355_DT_F8_E5M2: return e5m2_to_f32((uint8_t)w);
        case MI355_DT_E8M0: return e8m0_to_f32((uint8_t)w);
        case MI355_DT_F4_E2M1: return e2m1_to_f32((uint8_t)(w & 0xf));
        default: return 0.f;
    }
}
__device__ __forceinline__ int raw_to_int(int dt, uint32_t w) {
    switch (dt) {
        case MI355_DT_S32: return (int)w;
        case MI355_DT_S8: return (int)(int8_t)w;
        case MI355_DT_U8: return (int)(uint8_t)w;
        case MI355_DT_S4: return s4_to_int((uint8_t)(w & 0xf));
        default: return (int)(w & 0xf); // u4
    }
}

__device__ __forceinline__ uint32_t load_raw(int dt, const void *p, long off) {
    const int bits = dt_bits(dt);
    if (bits == 32) return ((const uint32_t *)p)[off];
    if (bits == 16) return ((const uint16_t *)p)[off];
    if (bits == 8) return ((const uint8_t *)p)[off];
    return nibble_get(p, off);
}

// The reference's arithmetic (see the head of this file) on N elements at once:
// raw[e] holds the src storage bits, B[e] the offsets of element e in every
// tensor.  Every data-type dispatch is uniform over the wavefront and is taken
// once for the N elements.
template <int N>
__device__ __forceinline__ void load_raw_vec(int dt, const void *p, long off, uint32_t (&w)[N]);

// How a unit finds its quantization parameters:
//   GENERIC  every element has its own offsets B[e] into every tensor;
//   SIMPLE   no scales, zero points or sum (a pure change of type and layout):
//            B is not read;
//   QVEC     no sum, and every parameter tensor is either constant along the
//            unit or holds its N values consecutively and aligned: B[0] only,
//            one (vector) load per parameter.
enum { MODE_GENERIC = 0, MODE_SIMPLE = 1, MODE_QVEC = 2 };

// the N values of parameter k (0 src scale, 1 dst scale, 2 src zero point)
template <int N, int MODE, class RT>
__device__ __forceinline__ void param_values(const RT &R, int k, const rbase_t (&B)[N], float (&out)[N]) {
    const int dt = R.qdt[k];
    if constexpr (MODE == MODE_QVEC) {
        if (R.a.qs[k] == 0) {
            const float v = load_float(dt, R.qp[k], B[0].q[k]);
#pragma unroll
            for (int e = 0; e < N; ++e) out[e] = v;
        } else {
            uint32_t pr[N];
            load_raw_vec<N>(dt, R.qp[k], B[0].q[k], pr);
            if (is_int_dt(dt)) {
#pragma unroll
                for (int e = 0; e < N; ++e) out[e] = (float)raw_to_int(dt, pr[e]);
            } else if (dt == MI355_DT_F32) {
#pragma unroll
                for (int e = 0; e < N; ++e) out[e] = u2f(pr[e]);
            } else {
#pragma unroll
                for (int e = 0; e < N; ++e) out[e] = raw_to_float(dt, pr[e]);
            }
        }
    } else if (dt == MI355_DT_F32) {
#pragma unroll
        for (int e = 0; e < N; ++e) out[e] = ((const float *)R.qp[k])[B[e].q[k]];
    } else {
#pragma unroll
        for (int e = 0; e < N; ++e) out[e] = load_float(dt, R.qp[k], B[e].q[k]);
    }
}

template <int N, int MODE = MODE_GENERIC, class RT>
__device__ __forceinline__ void convert(const RT &R, const uint32_t (&raw)[N], const rbase_t (&B)[N], uint32_t (&w)[N]) {
    constexpr bool SIMPLE = MODE == MODE_SIMPLE;
    if (R.plain_copy) { // same type, no attributes: the bits move unchanged
#pragma unroll
        for (int e = 0; e < N; ++e) w[e] = raw[e];
        return;
    }
    float x[N];
    const int sdt = R.src_dt;
    if (is_int_dt(sdt)) {
        int v[N];
        if (sdt == MI355_DT_S8) {
#pragma unroll
            for (int e = 0; e < N; ++e) v[e] = (int)(int8_t)raw[e];
        } else if (sdt == MI355_DT_U8) {
#pragma unroll
            for (int e = 0; e < N; ++e) v[e] = (int)(uint8_t)raw[e];
        } else if (sdt == MI355_DT_S32) {
#pragma unroll
            for (int e = 0; e < N; ++e) v[e] = (int)raw[e];
        } else if (sdt == MI355_DT_S4) {
#pragma unroll
            for (int e = 0; e < N; ++e) v[e] = s4_to_int((uint8_t)(raw[e] & 0xf));
        } else {
#pragma unroll
            for (int e = 0; e < N; ++e) v[e] = (int)(raw[e] & 0xf);
        }
        if constexpr (!SIMPLE) {
            if (R.qp[2]) {
                float zp[N];
                param_values<N, MODE>(R, 2, B, zp);
#pragma unroll
                for (int e = 0; e < N; ++e) v[e] -= (int)zp[e];
            }
        }
#pragma unroll
        for (int e = 0; e < N; ++e) x[e] = (float)v[e];
    } else if (sdt == MI355_DT_F32) {
#pragma unroll
        for (int e = 0; e < N; ++e) x[e] = u2f(raw[e]);
    } else if (sdt == MI355_DT_BF16) {
#pragma unroll
        for (int e = 0; e < N; ++e) x[e] = bf16_to_f32((uint16_t)raw[e]);
    } else if (sdt == MI355_DT_F16) {
#pragma unroll
        for (int e = 0; e < N; ++e) x[e] = f16_to_f32((uint16_t)raw[e]);
    } else {
#pragma unroll
        for (int e = 0; e < N; ++e) x[e] = raw_to_float(sdt, raw[e]);
    }
    if (!SIMPLE && sdt != MI355_DT_E8M0) { // e8m0 sources are converted without arithmetic
        if (R.qp[0]) {
            float sc[N];
            param_values<N, MODE>(R, 0, B, sc);
#pragma unroll
            for (int e = 0; e < N; ++e) x[e] = sc[e] * x[e];
        }
        if constexpr (MODE == MODE_GENERIC) {
            if (R.beta != 0.f) {
#pragma unroll
                for (int e = 0; e < N; ++e) x[e] += R.beta * load_float(R.dst_dt, R.dst, B[e].dof);
            }
        }
        if (R.qp[1] || R.dst_zp) {
            const float dzp = R.dst_zp ? (float)*(const int *)R.dst_zp : 0.f;
            if (R.qp[1]) {
                float sc[N];
                param_values<N, MODE>(R, 1, B, sc);
#pragma unroll
                for (int e = 0; e < N; ++e) x[e] = x[e] / sc[e] + dzp;
            } else {
#pragma unroll
                for (int e = 0; e < N; ++e) x[e] = x[e] / 1.f + dzp;
            }
        }
    }
    const int ddt = R.dst_dt;
    if (ddt == MI355_DT_S8) {
#pragma unroll
        for (int e = 0; e < N; ++e) w[e] = (uint32_t)(int)__builtin_rintf(sat(x[e], -128.f, 127.f)) & 0xffu;
    } else if (ddt == MI355_DT_U8) {
#pragma unroll
        for (int e = 0; e < N; ++e) w[e] = (uint32_t)(int)__builtin_rintf(sat(x[e], 0.f, 255.f)) & 0xffu;
    } else if (ddt == MI355_DT_F32) {
#pragma unroll
        for (int e = 0; e < N; ++e) w[e] = f2u(x[e]);
    } else if (ddt == MI355_DT_BF16) {
#pragma unroll
        for (int e = 0; e < N; ++e) w[e] = f32_to_bf16(x[e]);
    } else if (ddt == MI355_DT_F16) {
#pragma unroll
        for (int e = 0; e < N; ++e) w[e] = f32_to_f16(x[e]);
    } else if (ddt == MI355_DT_S4) {
#pragma unroll
        for (int e = 0; e < N; ++e) w[e] = (uint32_t)(int)__builtin_rintf(sat(x[e], -8.f, 7.f)) & 0xfu;
    } else if (ddt == MI355_DT_U4) {
#pragma unroll
        for (int e = 0; e < N; ++e) w[e] = (uint32_t)(int)__builtin_rintf(sat(x[e], 0.f, 15.f)) & 0xfu;
    } else if (ddt == MI355_DT_F4_E2M1) {
#pragma unroll
        for (int e = 0; e < N; ++e) w[e] = f32_to_e2m1(x[e]);
    } else {
#pragma unroll
        for (int e = 0; e < N; ++e) w[e] = cvt_store_bits(ddt, x[e]);
    }
}

// N consecutive elements of BITS bits each as raw dwords: one access of
// N * BITS / 8 bytes when that is at most 16 bytes, several 16-byte ones
// otherwise.  The address is a multiple of the access size.
template <int N, int BITS>
struct vec_io_t {
    static constexpr int TOTAL = N * BITS;            // bits
    static constexpr int D = TOTAL >= 32 ? TOTAL / 32 : 1; // dwords
    static __device__ __forceinline__ void load(const void *p, long off, uint32_t (&w)[N]) {
        const char *q = (const char *)p + off * BITS / 8;
        uint32_t dw[D];
        if constexpr (TOTAL >= 128) {
#pragma unroll
            for (int c = 0; c < D / 4; ++c) {
                const uint4 v = ((const uint4 *)q)[c];
                dw[4 * c] = v.x; dw[4 * c + 1] = v.y; dw[4 * c + 2] = v.z; dw[4 * c + 3] = v.w;
            }
        } else if constexpr (TOTAL == 64) {
            const uint2 v = *(const uint2 *)q;
            dw[0] = v.x; dw[1] = v.y;
        } else if constexpr (TOTAL == 32) {
            dw[0] = *(const uint32_t *)q;
        } else {
            dw[0] = *(const uint16_t *)q;
        }
#pragma unroll
        for (int e = 0; e < N; ++e)
            w[e] = BITS == 32 ? dw[e] : (dw[e * BITS / 32] >> (e * BITS % 32)) & (0xffffffffu >> (32 - BITS));
    }
    static __device__ __forceinline__ void store(void *p, long off, const uint32_t (&w)[N]) {
        char *q = (char *)p + off * BITS / 8;
        uint32_t dw[D];
#pragma unroll
        for (int c = 0; c < D; ++c) dw[c] = 0;
#pragma unroll
        for (int e = 0; e < N; ++e) dw[e * BITS / 32] |= BITS == 32 ? w[e] : w[e] << (e * BITS % 32);
        if constexpr (TOTAL >= 128) {
#pragma unroll
            for (int c = 0; c < D / 4; ++c) {
                uint4 v;
                v.x = dw[4 * c]; v.y = dw[4 * c + 1]; v.z = dw[4 * c + 2]; v.w = dw[4 * c + 3];
                ((uint4 *)q)[c] = v;
            }
        } else if constexpr (TOTAL == 64) {
            uint2 v;
            v.x = dw[0]; v.y = dw[1];
            *(uint2 *)q = v;
        } else if constexpr (TOTAL == 32) {
            *(uint32_t *)q = dw[0];
        } else {
            *(uint16_t *)q = (uint16_t)dw[0];
        }
    }
};

// store N consecutive dst elements starting at element offset off; `packed`:
// they may leave as one aligned vector (N >= 4)
template <int N>
__device__ __forceinline__ void store_bits(int dt, void *dst, long off, const uint32_t (&w)[N], bool packed) {
    const int bits = dt_bits(dt);
    if constexpr (N >= 4) {
        if (packed) {
            if (bits == 4) vec_io_t<N, 4>::store(dst, off, w);
            else if (bits == 8) vec_io_t<N, 8>::store(dst, off, w);
            else if (bits == 16) vec_io_t<N, 16>::store(dst, off, w);
            else vec_io_t<N, 32>::store(dst, off, w);
            return;
        }
    }
    if (bits == 4) {
        // off is even and the N nibbles fill whole bytes
        uint8_t *p = (uint8_t *)dst + (off >> 1);
#pragma unroll
        for (int e = 0; e + 1 < N; e += 2) p[e >> 1] = (uint8_t)(w[e] | (w[e + 1] << 4));
        return;
    }
#pragma unroll
    for (int e = 0; e < N; ++e) {
        if (bits == 8) ((uint8_t *)dst)[off + e] = (uint8_t)w[e];
        else if (bits == 16) ((uint16_t *)dst)[off + e] = (uint16_t)w[e];
        else ((uint32_t *)dst)[off + e] = w[e];
    }
}

// N consecutive src elements as vector loads (off is a multiple of N)
template <int N>
__device__ __forceinline__ void load_raw_vec(int dt, const void *p, long off, uint32_t (&w)[N]) {
    const int bits = dt_bits(dt);
    if (bits == 32) vec_io_t<N, 32>::load(p, off, w);
    else if (bits == 16) vec_io_t<N, 16>::load(p, off, w);
    else if (bits == 8) vec_io_t<N, 8>::load(p, off, w);
    else vec_io_t<N, 4>::load(p, off, w);
}

// One unit = E consecutive elements along the dim `a` (dst stride 1 when
// E > 1) of one outer index; units are numbered (outer, chunk of a) and walked
// with a grid stride.  A lane issues the loads of its next unit before it
// converts and stores the current one: with a single unit in flight per lane a
// plain s8 copy ran at 1.7 TB/s.
template <int E, int MODE>
__global__ void __launch_bounds__(256) reorder_direct_kernel(const reorder_t R_) {
    const auto &R = *(const __attribute__((address_space(4))) reorder_t *)__builtin_amdgcn_kernarg_segment_ptr();
    constexpr bool SIMPLE = MODE == MODE_SIMPLE;
    const unsigned units = R.a.n / E;
    const unsigned long total = (unsigned long)R.outer_total * units;
    const unsigned long stride = (unsigned long)gridDim.x * 256;
    // offsets of unit f (recomputed where needed rather than kept across the
    // loads).  SIMPLE: only the src and dst offsets of the unit's first element;
    // the per-element offsets into the parameter tensors are most of the
    // integer work of a unit otherwise.
    auto bases = [&](unsigned long f, rbase_t (&B)[E]) __attribute__((always_inline)) {
        unsigned o, u;
        if (total >> 32) {
            o = (unsigned)(f / units);
            u = (unsigned)(f - (unsigned long)o * units);
        } else {
            o = (unsigned)f / units;
            u = (unsigned)f - o * units;
        }
        if constexpr (SIMPLE) {
            long so = (long)(u * E) * R.a.ss, dof = (long)(u * E) * R.a.ds;
            for (int i = 0; i < R.n_outer; ++i) {
                const unsigned n = R.outer[i].n;
                const unsigned q = o / n, r = o - q * n;
                o = q;
                so += (long)r * R.outer[i].ss;
                dof += (long)r * R.outer[i].ds;
            }
            B[0].so = so;
            B[0].dof = dof;
        } else if constexpr (MODE == MODE_QVEC) {
            B[0] = outer_base(R, o);
            add_dim(B[0], R.a, u * E);
        } else {
            const rbase_t B0 = outer_base(R, o);
            add_dim_run<E>(B, B0, R.a, u * E);
        }
    };
    auto fetch = [&](unsigned long f, uint32_t (&raw)[E]) __attribute__((always_inline)) {
        rbase_t B[E];
        bases(f, B);
        bool loaded = false;
        if constexpr (E >= 4) {
            if (R.src_vec) {
                load_raw_vec<E>(R.src_dt, R.src, B[0].so, raw);
                loaded = true;
            }
        }
        if (!loaded) {
#pragma unroll
            for (int e = 0; e < E; ++e)
                raw[e] = load_raw(R.src_dt, R.src, MODE != MODE_GENERIC ? B[0].so + (long)e * R.a.ss : B[e].so);
        }
    };
    unsigned long f = (unsigned long)blockIdx.x * 256 + threadIdx.x;
    if (f >= total) return;
    uint32_t raw[E];
    fetch(f, raw);
    while (true) {
        const unsigned long fn = f + stride;
        uint32_t next[E];
#pragma unroll
        for (int e = 0; e < E; ++e) next[e] = 0;
        if (fn < total) fetch(fn, next);
        rbase_t B[E];
        bases(f, B);
        uint32_t w[E];
        convert<E, MODE>(R, raw, B, w);
        store_bits<E>(R.dst_dt, R.dst, B[0].dof, w, R.packed);
        if (fn >= total) break;
#pragma unroll
        for (int e = 0; e < E; ++e) raw[e] = next[e];
        f = fn;
    }
}

// Row quantization: float src (f32 / bf16 / f16) to an 8-bit dst (s8 / u8 /
// e4m3 / e5m2), both unit-stride along `a`, at most one outer dim (rows), no
// sum, no src zero point, f32 scales per tensor or per column.  This is what
// quantizing activations or weights is, and the generic direct kernel spends
// some 45 instructions per element on it (per-unit offsets, parameter loads
// and data-type dispatch).  Here a workgroup owns 1024 columns -- a lane four
// consecutive ones -- for a block of rows: the scales and, for integer dst, the
// reciprocals of the dst scales are fetched once per lane, the data types are
// template parameters, four rows are in flight per lane, and every load or
// store instruction moves whole 128-byte lines.  The arithmetic is convert()'s:
// x = src_scale * x; x = x / dst_scale + dst_zp; saturate, round to nearest
// even.  For integer dst the division is div_by_fma where its conditions hold
// (the IEEE quotient bit for bit where the rounding to an integer can see it).
template <int SDT, int DDT>
__global__ void __launch_bounds__(256) reorder_rows_kernel(const reorder_t R_, unsigned rows_per_wg) {
    const auto &R = *(const __attribute__((address_space(4))) reorder_t *)__builtin_amdgcn_kernarg_segment_ptr();
    typedef uint32_t u4v __attribute__((ext_vector_type(4)));
    typedef uint32_t u2v __attribute__((ext_vector_type(2)));
    constexpr bool INT_DST = DDT == MI355_DT_S8 || DDT == MI355_DT_U8;
    constexpr int U = 4;
    const unsigned a = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (a >= R.a.n) return;
    const unsigned rows = R.n_outer ? R.outer[0].n : 1;
    const long rs = R.n_outer ? R.outer[0].ss : 0, rd = R.n_outer ? R.outer[0].ds : 0;
    const unsigned r0 = blockIdx.y * rows_per_wg;
    const unsigned r1 = min(rows, r0 + rows_per_wg);
    float s0[4], s1[4], y1[4];
    bool fast = INT_DST;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        s0[e] = R.qp[0] ? ((const float *)R.qp[0])[R.a.qs[0] ? a + e : 0] : 1.f;
        s1[e] = R.qp[1] ? ((const float *)R.qp[1])[R.a.qs[1] ? a + e : 0] : 1.f;
        y1[e] = 1.f / s1[e];
        const float m = __builtin_fabsf(s1[e]);
        fast = fast && m >= 0x1p-20f && m <= 0x1p20f;
    }
    const bool with_s0 = R.qp[0] != nullptr, with_div = R.qp[1] != nullptr || R.dst_zp != nullptr;
    const float dzp = R.dst_zp ? (float)*(const int *)R.dst_zp : 0.f;
    const char *src = (const char *)R.src + (long)a * (dt_bits(SDT) / 8);
    uint8_t *dst = (uint8_t *)R.dst + a;
    for (unsigned r = r0; r < r1; r += U) {
        uint32_t raw[U][4];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned rr = min(r + u, r1 - 1); // a row past the block repeats the last one (and is not stored)
            const char *p = src + (long)rr * rs * (dt_bits(SDT) / 8);
            if constexpr (SDT == MI355_DT_F32) {
                const u4v v = __builtin_nontemporal_load((const u4v *)p);
                raw[u][0] = v.x; raw[u][1] = v.y; raw[u][2] = v.z; raw[u][3] = v.w;
            } else {
                const u2v v = __builtin_nontemporal_load((const u2v *)p);
                raw[u][0] = v.x & 0xffffu; raw[u][1] = v.x >> 16; raw[u][2] = v.y & 0xffffu; raw[u][3] = v.y >> 16;
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (r + u >= r1) break;
            float x[4];
            unsigned mag = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                x[e] = raw_to_float(SDT, raw[u][e]);
                if (with_s0) x[e] = s0[e] * x[e];
                mag = max(mag, gemm::mag_bits(x[e]));
            }
            if (with_div) {
                if (fast && mag < gemm::DIV_BY_FMA_LIMIT) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) x[e] = gemm::div_by_fma(x[e], s1[e], y1[e]) + dzp;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) x[e] = x[e] / s1[e] + dzp;
                }
            }
            uint32_t w = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                uint32_t b;
                if constexpr (DDT == MI355_DT_S8) b = (uint32_t)(int)__builtin_rintf(sat(x[e], -128.f, 127.f)) & 0xffu;
                else if constexpr (DDT == MI355_DT_U8) b = (uint32_t)(int)__builtin_rintf(sat(x[e], 0.f, 255.f)) & 0xffu;
                else b = cvt_store_bits(DDT, x[e]) & 0xffu;
                w |= b << (8 * e);
            }
            __builtin_nontemporal_store(w, (uint32_t *)(dst + (long)(r + u) * rd));
        }
    }
}

// 64 x 64 tile over (b, a): b has src stride 1, a has dst stride 1.  grid: x
// over the tiles, y over the outer index.  MODE as in the direct kernel; the
// modes other than MODE_GENERIC want the extent of a to be a multiple of four
// (a lane's four rows are then all inside or all outside the tensor).
template <int MODE>
__global__ void __launch_bounds__(256) reorder_tiled_kernel(const reorder_t R_) {
    const auto &R = *(const __attribute__((address_space(4))) reorder_t *)__builtin_amdgcn_kernarg_segment_ptr();
    __shared__ uint32_t tile[64][65];
    const unsigned ntiles = R.tiles_a * R.tiles_b;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (unsigned o = blockIdx.y; o < R.outer_total; o += gridDim.y) {
        const rbase_t B0 = outer_base(R, o);
        for (unsigned t = blockIdx.x; t < ntiles; t += gridDim.x) {
            const unsigned tb = t % R.tiles_b, ta = t / R.tiles_b;
            const unsigned b0 = tb * 64, a0 = ta * 64;
            // read: lanes along b (src unit stride)
            // (four rows per pass: four loads in flight, one dispatch for the four)
            for (int i0 = ty * 4; i0 < 64; i0 += 16) {
                rbase_t B[4];
                uint32_t raw[4], v[4];
                const unsigned ib = b0 + tx < R.b.n ? b0 + tx : R.b.n - 1; // clamped, masked below
                if constexpr (MODE == MODE_GENERIC) {
                    rbase_t Bb = B0;
                    add_dim(Bb, R.b, ib);
                    if (a0 + i0 + 4 <= R.a.n) {
                        add_dim_run<4>(B, Bb, R.a, a0 + i0);
                    } else { // ragged last tile along a: clamped, masked below
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            B[k] = Bb;
                            add_dim(B[k], R.a, a0 + i0 + k < R.a.n ? a0 + i0 + k : R.a.n - 1);
                        }
                    }
#pragma unroll
                    for (int k = 0; k < 4; ++k) raw[k] = load_raw(R.src_dt, R.src, B[k].so);
                } else {
                    const unsigned ia = a0 + i0 < R.a.n ? a0 + i0 : R.a.n - 4; // clamped, masked below
                    if constexpr (MODE == MODE_SIMPLE) {
                        B[0].so = B0.so + (long)ib * R.b.ss + (long)ia * R.a.ss;
                    } else {
                        B[0] = B0;
                        add_dim(B[0], R.b, ib);
                        add_dim(B[0], R.a, ia);
                    }
#pragma unroll
                    for (int k = 0; k < 4; ++k) raw[k] = load_raw(R.src_dt, R.src, B[0].so + (long)k * R.a.ss);
                }
                convert<4, MODE>(R, raw, B, v);
#pragma unroll
                for (int k = 0; k < 4; ++k) tile[i0 + k][tx] = v[k];
            }
            __syncthreads();
            // write: lanes along a (dst unit stride), four elements each
            const int lx = (threadIdx.x & 15) * 4, ly = threadIdx.x >> 4;
            for (int i = ly; i < 64; i += 16) {
                const unsigned ib = b0 + i, ia = a0 + lx;
                if (ib < R.b.n && ia < R.a.n) {
                    const long dof = B0.dof + (long)ib * R.b.ds + (long)ia * R.a.ds;
                    const uint32_t w[4] = {tile[lx][i], tile[lx + 1][i], tile[lx + 2][i], tile[lx + 3][i]};
                    if (ia + 4 <= R.a.n) {
                        store_bits<4>(R.dst_dt, R.dst, dof, w, R.packed);
                    } else { // ragged edge: the extent is even for 4-bit types
                        const int left = (int)(R.a.n - ia);
                        if (dt_bits(R.dst_dt) == 4) {
                            const uint32_t w2[2] = {w[0], w[1]};
                            if (left >= 2) store_bits<2>(R.dst_dt, R.dst, dof, w2, false);
                        } else {
                            for (int e = 0; e < left; ++e) {
                                const uint32_t w1[1] = {w[e]};
                                store_bits<1>(R.dst_dt, R.dst, dof + e, w1, false);
                            }
                        }
                    }
                }
            }
            __syncthreads();
        }
    }
}

// Transposition of 8-bit elements without attributes (the layout change of
// int8 / fp8 weights that format_tag::any asks for): 64 x 64 tile over (a, b),
// b has src stride 1, a has dst stride 1, both extents multiples of 64.  A
// thread loads a 4 x 4 block as four dwords, transposes it in registers with
// eight byte permutes and parks the four result dwords in LDS; the tile then
// leaves as 16-byte stores along a.
__global__ void __launch_bounds__(256) transpose8_kernel(const reorder_t R_) {
    const auto &R = *(const __attribute__((address_space(4))) reorder_t *)__builtin_amdgcn_kernarg_segment_ptr();
    constexpr int PITCH = 17; // dwords per LDS row (16 + 1: spreads the banks)
    __shared__ uint32_t tile[64 * PITCH];
    const unsigned ntiles = R.tiles_a * R.tiles_b;
    const int bi = threadIdx.x & 15, ai = threadIdx.x >> 4; // read: block (4 ai .. +3, 4 bi .. +3)
    const int wb = threadIdx.x >> 2, wq = threadIdx.x & 3;  // write: row b, 16 bytes of a
    const uint8_t *src = (const uint8_t *)R.src;
    uint8_t *dst = (uint8_t *)R.dst;
    for (unsigned o = blockIdx.y; o < R.outer_total; o += gridDim.y) {
        long so = 0, dof = 0;
        {
            unsigned oo = o;
            for (int i = 0; i < R.n_outer; ++i) {
                const unsigned n = R.outer[i].n;
                const unsigned q = oo / n, r = oo - q * n;
                oo = q;
                so += (long)r * R.outer[i].ss;
                dof += (long)r * R.outer[i].ds;
            }
        }
        for (unsigned t = blockIdx.x; t < ntiles; t += gridDim.x) {
            const unsigned tb = t % R.tiles_b, ta = t / R.tiles_b;
            const long a0 = (long)ta * 64, b0 = (long)tb * 64;
            const uint8_t *p = src + so + (a0 + 4 * ai) * R.a.ss + b0 + 4 * bi;
            const uint32_t r0 = *(const uint32_t *)p, r1 = *(const uint32_t *)(p + R.a.ss),
                           r2 = *(const uint32_t *)(p + 2 * R.a.ss), r3 = *(const uint32_t *)(p + 3 * R.a.ss);
            // byte k of r_i is element (a + i, b + k); T_k collects byte k of the four rows
            const uint32_t x0 = __builtin_amdgcn_perm(r1, r0, 0x05010400u), x1 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
            const uint32_t y0 = __builtin_amdgcn_perm(r3, r2, 0x05010400u), y1 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
            tile[(4 * bi + 0) * PITCH + ai] = __builtin_amdgcn_perm(y0, x0, 0x05040100u);
            tile[(4 * bi + 1) * PITCH + ai] = __builtin_amdgcn_perm(y0, x0, 0x07060302u);
            tile[(4 * bi + 2) * PITCH + ai] = __builtin_amdgcn_perm(y1, x1, 0x05040100u);
            tile[(4 * bi + 3) * PITCH + ai] = __builtin_amdgcn_perm(y1, x1, 0x07060302u);
            __syncthreads();
            uint4 v;
            v.x = tile[wb * PITCH + 4 * wq]; v.y = tile[wb * PITCH + 4 * wq + 1];
            v.z = tile[wb * PITCH + 4 * wq + 2]; v.w = tile[wb * PITCH + 4 * wq + 3];
            *(uint4 *)(dst + dof + (b0 + wb) * R.b.ds + a0 + 16 * wq) = v;
            __syncthreads();
        }
    }
}

// The same transposition on 128 x 128 tiles, for extents that are multiples of
// 128 and 16-byte aligned rows: every load instruction fetches the whole
// 128-byte lines of eight src rows and every store instruction writes the
// whole lines of eight dst rows, so no line is touched by two workgroups
// (with 64-byte tile rows every src line was fetched twice, by workgroups on
// different L2s).  A thread loads 4 rows x 16 bytes, transposes the four
// 4 x 4 blocks in registers and parks 16 dwords in LDS; dword column c of
// tile row b sits at (c + 8 (b / 16)) % 32, which spreads a store instruction
// over all banks and keeps the 16-byte reads aligned.
__global__ void __launch_bounds__(256) transpose8w_kernel(const reorder_t R_) {
    const auto &R = *(const __attribute__((address_space(4))) reorder_t *)__builtin_amdgcn_kernarg_segment_ptr();
    __shared__ __attribute__((aligned(16))) uint32_t tile[128 * 32];
    const unsigned tiles_b = R.b.n / 128, ntiles = (R.a.n / 128) * tiles_b;
    const int bi = threadIdx.x & 7, ag = threadIdx.x >> 3; // read: rows 4 ag .. +3, bytes 16 bi .. +15
    const int wq = threadIdx.x & 7, wr = threadIdx.x >> 3; // write: row wr + 32 pass, bytes 16 wq .. +15
    const uint8_t *src = (const uint8_t *)R.src;
    uint8_t *dst = (uint8_t *)R.dst;
    for (unsigned o = blockIdx.y; o < R.outer_total; o += gridDim.y) {
        long so = 0, dof = 0;
        {
            unsigned oo = o;
            for (int i = 0; i < R.n_outer; ++i) {
                const unsigned n = R.outer[i].n;
                const unsigned q = oo / n, r = oo - q * n;
                oo = q;
                so += (long)r * R.outer[i].ss;
                dof += (long)r * R.outer[i].ds;
            }
        }
        for (unsigned t = blockIdx.x; t < ntiles; t += gridDim.x) {
            const unsigned tb = t % tiles_b, ta = t / tiles_b;
            const long a0 = (long)ta * 128, b0 = (long)tb * 128;
            const uint8_t *p = src + so + (a0 + 4 * ag) * R.a.ss + b0 + 16 * bi;
            typedef uint32_t u4v __attribute__((ext_vector_type(4)));
            u4v r[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) r[i] = __builtin_nontemporal_load((const u4v *)(p + i * R.a.ss));
            const int col = (ag + 8 * (bi & 3)) & 31;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t r0 = k == 0 ? r[0].x : k == 1 ? r[0].y : k == 2 ? r[0].z : r[0].w;
                const uint32_t r1 = k == 0 ? r[1].x : k == 1 ? r[1].y : k == 2 ? r[1].z : r[1].w;
                const uint32_t r2 = k == 0 ? r[2].x : k == 1 ? r[2].y : k == 2 ? r[2].z : r[2].w;
                const uint32_t r3 = k == 0 ? r[3].x : k == 1 ? r[3].y : k == 2 ? r[3].z : r[3].w;
                // byte j of r_i is element (a + i, b + 4 k + j); T_j collects byte j of the four rows
                const uint32_t x0 = __builtin_amdgcn_perm(r1, r0, 0x05010400u), x1 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
                const uint32_t y0 = __builtin_amdgcn_perm(r3, r2, 0x05010400u), y1 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
                const int row = 16 * bi + 4 * k;
                tile[(row + 0) * 32 + col] = __builtin_amdgcn_perm(y0, x0, 0x05040100u);
                tile[(row + 1) * 32 + col] = __builtin_amdgcn_perm(y0, x0, 0x07060302u);
                tile[(row + 2) * 32 + col] = __builtin_amdgcn_perm(y1, x1, 0x05040100u);
                tile[(row + 3) * 32 + col] = __builtin_amdgcn_perm(y1, x1, 0x07060302u);
            }
            __syncthreads();
#pragma unroll
            for (int pass = 0; pass < 4; ++pass) {
                const int b = wr + 32 * pass;
                const u4v v = *(const u4v *)&tile[b * 32 + ((4 * wq + 8 * ((b >> 4) & 3)) & 31)];
                __builtin_nontemporal_store(v, (u4v *)(dst + dof + (b0 + b) * R.b.ds + a0 + 16 * wq));
            }
            __syncthreads();
        }
    }
}

bool dt_ok(int dt) {
    switch (dt) {
        case MI355_DT_F16: case MI355_DT_BF16: case MI355_DT_F32: case MI355_DT_S32: case MI355_DT_S8:
        case MI355_DT_U8: case MI355_DT_F8_E5M2: case MI355_DT_F8_E4M3: case MI355_DT_S4: case MI355_DT_U4:
        case MI355_DT_E8M0: case MI355_DT_F4_E2M1: return true;
        default: return false;
    }
}

// strides of a quantization parameter tensor along the tensor's dims: dense
// row-major over the masked dims, the last two divided by the groups
// (quant_entry_t::get_md, src/common/primitive_attr_quant.hpp:116-140)
void quant_strides(const mi355_quant_t &m, int ndims, const int64_t *dims, long (&stride)[RD], long (&group)[RD]) {
    long st = 1;
    for (int d = RD - 1; d >= 0; --d) {
        stride[d] = 0;
        group[d] = 1;
        if (d >= ndims || m.dt == MI355_DT_UNDEF) continue;
        if (d == ndims - 2) group[d] = m.group[0];
        if (d == ndims - 1) group[d] = m.group[1];
        if (m.mask & (1 << d)) {
            stride[d] = st;
            st *= dims[d] / group[d];
        }
    }
}

int check(const mi355_reorder_desc_t *d) {
    if (!d) {
        set_error("null descriptor");
        return MI355_INVALID_ARGUMENTS;
    }
    if (d->ndims < 1 || d->ndims > RD || !dt_ok(d->src_dt) || !dt_ok(d->dst_dt)) {
        set_error("reorder: bad rank or data type");
        return MI355_INVALID_ARGUMENTS;
    }
    for (int i = 0; i < d->ndims; ++i)
        if (d->dims[i] < 0 || d->src_stride[i] < 0 || d->dst_stride[i] < 0) {
            set_error("reorder: negative dimension or stride");
            return MI355_INVALID_ARGUMENTS;
        }
    const mi355_quant_t *qs[4] = {&d->src_scale, &d->dst_scale, &d->src_zp, &d->dst_zp};
    for (const mi355_quant_t *q : qs) {
        if (q->dt == MI355_DT_UNDEF) continue;
        if (!dt_ok(q->dt) || q->group[0] < 1 || q->group[1] < 1 || (q->mask >> d->ndims)) {
            set_error("reorder: bad quantization parameter");
            return MI355_INVALID_ARGUMENTS;
        }
        const long g0 = q->group[0], g1 = q->group[1];
        if ((g0 > 1 && (d->ndims < 2 || d->dims[d->ndims - 2] % g0)) || (g1 > 1 && d->dims[d->ndims - 1] % g1)) {
            set_error("reorder: groups do not divide the dims");
            return MI355_INVALID_ARGUMENTS;
        }
    }
    // zero points only with integer data (src/common/reorder.cpp:96-103)
    auto integral = [](int dt) {
        return dt == MI355_DT_S32 || dt == MI355_DT_S8 || dt == MI355_DT_U8 || dt == MI355_DT_S4
                || dt == MI355_DT_U4;
    };
    if ((d->src_zp.dt != MI355_DT_UNDEF && !integral(d->src_dt))
            || (d->dst_zp.dt != MI355_DT_UNDEF && !integral(d->dst_dt))) {
        set_error("reorder: zero points need an integer data type");
        return MI355_INVALID_ARGUMENTS;
    }
    if (d->dst_scale.dt != MI355_DT_UNDEF && (d->dst_scale.group[0] > 1 || d->dst_scale.group[1] > 1))
        return MI355_UNIMPLEMENTED; // src/common/reorder.cpp:145
    if (d->dst_zp.dt != MI355_DT_UNDEF && (d->dst_zp.mask != 0 || d->dst_zp.dt != MI355_DT_S32))
        return MI355_UNIMPLEMENTED;
    // 4-bit dst: two elements share a byte, so the lanes must own whole bytes:
    // a unit-stride dim of even size and even strides elsewhere
    if (dt_bits(d->dst_dt) == 4) {
        int unit = -1;
        for (int i = 0; i < d->ndims; ++i)
            if (d->dst_stride[i] == 1 && d->dims[i] > 1) unit = i;
        if (unit < 0 || d->dims[unit] % 2) return MI355_UNIMPLEMENTED;
        for (int i = 0; i < d->ndims; ++i)
            if (i != unit && d->dims[i] > 1 && d->dst_stride[i] % 2) return MI355_UNIMPLEMENTED;
        if (d->beta != 0.f) return MI355_UNIMPLEMENTED;
    }
    return MI355_SUCCESS;
}

// ---- plain 4-bit weights -> MI355_WEI_PACK_WOQ64, the one reorder whose dst
// is not a plain strided tensor at heart: the generic kernels above handle its
// six-dim view correctly but four nibbles at a time.  One thread writes the 16
// bytes one lane of the decode kernel reads: rows 8kq .. 8kq+7 of the columns
// 64c + 16t + j, t = 0..3.
//   ROW_MAJOR: src [K][N], row pitch `pitch` bytes: the thread reads the 32
//     bytes of its chunk in each of the 8 rows (shared by the 16 threads of
//     the same (c, kq): cache hits) and picks nibble j of every 8-byte block.
//   else: src [N][K], column pitch `pitch` bytes: the 8 rows of a column are
//     one dword, its even nibbles go to the low half, the odd ones to the high.
template <bool ROW_MAJOR>
__global__ void __launch_bounds__(256) pack_woq64_kernel(const uint8_t *src, uint8_t *dst, int K, int N, long pitch) {
    const long g = (long)blockIdx.x * 256 + threadIdx.x; // (c, kq, j), j fastest: 16 bytes of dst each
    const long total = (long)(N / 64) * (K / 8) * 16;
    if (g >= total) return;
    const int j = (int)(g & 15);
    const long ckq = g >> 4;
    const int kq = (int)(ckq % (K / 8));
    const int c = (int)(ckq / (K / 8));
    unsigned out[4] = {0u, 0u, 0u, 0u};
    if (ROW_MAJOR) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const uint4 *row = (const uint4 *)(src + (long)(kq * 8 + r) * pitch + c * 32);
            const uint4 lo = row[0], hi = row[1];
            const unsigned long long blk[4] = {lo.x | ((unsigned long long)lo.y << 32), lo.z | ((unsigned long long)lo.w << 32),
                    hi.x | ((unsigned long long)hi.y << 32), hi.z | ((unsigned long long)hi.w << 32)};
            const int pos = (r & 1) * 4 + (r >> 1);
#pragma unroll
            for (int t = 0; t < 4; ++t) out[t] |= (unsigned)((blk[t] >> (4 * j)) & 0xfull) << (4 * pos);
        }
    } else {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const unsigned w = *(const unsigned *)(src + (long)(c * 64 + t * 16 + j) * pitch + kq * 4);
            unsigned even = w & 0x0f0f0f0fu, odd = (w >> 4) & 0x0f0f0f0fu; // nibbles k = 0,2,4,6 / 1,3,5,7, one per byte
            // compact four byte-spaced nibbles into 16 bits
            even = (even | (even >> 4)) & 0x00ff00ffu;
            even = (even | (even >> 8)) & 0x0000ffffu;
            odd = (odd | (odd >> 4)) & 0x00ff00ffu;
            odd = (odd | (odd >> 8)) & 0x0000ffffu;
            out[t] = even | (odd << 16);
        }
    }
    uint4 o;
    o.x = out[0]; o.y = out[1]; o.z = out[2]; o.w = out[3];
    *(uint4 *)(dst + g * 16) = o;
}

// the six-dim view mi355_wei_pack_reorder_dims writes, with a src the kernel
// above can read: returns 1 (row-major src), 2 (column-major src) or 0
int woq64_fast_path(const mi355_reorder_desc_t &d, const mi355_reorder_args_t &a, long *K, long *N, long *pitch) {
    if (d.ndims != 6 || d.src_dt != d.dst_dt || dt_bits(d.src_dt) != 4 || d.beta != 0.f) return 0;
    if (d.src_scale.dt != MI355_DT_UNDEF || d.dst_scale.dt != MI355_DT_UNDEF || d.src_zp.dt != MI355_DT_UNDEF
            || d.dst_zp.dt != MI355_DT_UNDEF)
        return 0;
    if (d.dims[1] != 4 || d.dims[2] != 2 || d.dims[4] != 4 || d.dims[5] != 16) return 0;
    *K = d.dims[0] * 8;
    *N = d.dims[3] * 64;
    if (*K % 32 || *K >= (1L << 31) || *N >= (1L << 31)) return 0;
    const int64_t ds[6] = {512, 1, 4, *K * 64, 8, 32};
    for (int i = 0; i < 6; ++i)
        if (d.dst_stride[i] != ds[i]) return 0;
    const int64_t sk = d.src_stride[2], sn = d.src_stride[5];
    const int64_t ss[6] = {8 * sk, 2 * sk, sk, 64 * sn, 16 * sn, sn};
    for (int i = 0; i < 6; ++i)
        if (d.src_stride[i] != ss[i]) return 0;
    if (((uintptr_t)a.dst & 15) != 0) return 0;
    if (sn == 1 && sk >= *N && sk % 32 == 0 && ((uintptr_t)a.src & 15) == 0) {
        *pitch = sk / 2;
        return 1;
    }
    if (sk == 1 && sn >= *K && sn % 8 == 0 && ((uintptr_t)a.src & 3) == 0) {
        *pitch = sn / 2;
        return 2;
    }
    return 0;
}

} // namespace
} // namespace mi355

using namespace mi355;

extern "C" int mi355_reorder_query(const mi355_reorder_desc_t *desc) {
    return check(desc);
}

extern "C" int mi355_reorder_launch(const mi355_reorder_desc_t *desc, const mi355_reorder_args_t *args,
        void *stream) {
    const int st = check(desc);
    if (st != MI355_SUCCESS) return st;
    if (!args) {
        set_error("null arguments");
        return MI355_INVALID_ARGUMENTS;
    }
    const mi355_reorder_desc_t &d = *desc;
    long total = 1;
    for (int i = 0; i < d.ndims; ++i) total *= d.dims[i];
    if (total == 0) return MI355_SUCCESS;
    if (!args->src || !args->dst) {
        set_error("reorder: null tensor");
        return MI355_INVALID_ARGUMENTS;
    }
    const mi355_quant_t *qs[4] = {&d.src_scale, &d.dst_scale, &d.src_zp, &d.dst_zp};
    const void *qp[4] = {args->src_scale, args->dst_scale, args->src_zp, args->dst_zp};
    for (int i = 0; i < 4; ++i)
        if (qs[i]->dt != MI355_DT_UNDEF && !qp[i]) {
            set_error("reorder: a declared scale or zero point tensor is null");
            return MI355_INVALID_ARGUMENTS;
        }
    for (int i = 0; i < d.ndims; ++i)
        if (d.dims[i] >= (1L << 31)) return MI355_UNIMPLEMENTED;
    {
        long K = 0, N = 0, pitch = 0;
        const int fast = woq64_fast_path(d, *args, &K, &N, &pitch);
        if (fast) {
            const long threads = (N / 64) * (K / 8) * 16;
            const dim3 grid((unsigned)((threads + 255) / 256)), block(256);
            if (fast == 1)
                hipLaunchKernelGGL(pack_woq64_kernel<true>, grid, block, 0, (hipStream_t)stream,
                        (const uint8_t *)args->src, (uint8_t *)args->dst, (int)K, (int)N, pitch);
            else
                hipLaunchKernelGGL(pack_woq64_kernel<false>, grid, block, 0, (hipStream_t)stream,
                        (const uint8_t *)args->src, (uint8_t *)args->dst, (int)K, (int)N, pitch);
            if (hipGetLastError() != hipSuccess) {
                set_error("reorder: launch failed");
                return MI355_RUNTIME_ERROR;
            }
            return MI355_SUCCESS;
        }
    }

    reorder_t R {};
    R.src_dt = d.src_dt;
    R.dst_dt = d.dst_dt;
    R.beta = d.beta;
    R.src = args->src;
    R.dst = args->dst;
    long qstride[NQ][RD], qgroup[NQ][RD];
    for (int k = 0; k < NQ; ++k) {
        quant_strides(*qs[k], d.ndims, d.dims, qstride[k], qgroup[k]);
        R.qp[k] = qs[k]->dt != MI355_DT_UNDEF ? qp[k] : nullptr;
        R.qdt[k] = qs[k]->dt;
    }
    R.dst_zp = d.dst_zp.dt != MI355_DT_UNDEF ? args->dst_zp : nullptr;
    auto make_dim = [&](int i) {
        rdim_t r {};
        r.n = (unsigned)d.dims[i];
        r.ss = d.src_stride[i];
        r.ds = d.dst_stride[i];
        for (int k = 0; k < NQ; ++k) {
            r.qs[k] = qstride[k][i];
            r.qg[k] = (unsigned)qgroup[k][i];
        }
        return r;
    };
    // dims of extent > 1, ordered by dst stride; neighbours that are contiguous
    // in both tensors (and in every parameter tensor) merge into one dim, so a
    // plain conversion of a dense tensor becomes one long row
    rdim_t v[RD];
    int nv = 0;
    for (int i = 0; i < d.ndims; ++i)
        if (d.dims[i] > 1) v[nv++] = make_dim(i);
    for (int x = 0; x < nv; ++x)
        for (int y = x + 1; y < nv; ++y)
            if (v[y].ds < v[x].ds) {
                const rdim_t t = v[x];
                v[x] = v[y];
                v[y] = t;
            }
    for (int x = 0; x + 1 < nv;) {
        const rdim_t &in = v[x], &out = v[x + 1];
        bool ok = out.ss == in.ss * (long)in.n && out.ds == in.ds * (long)in.n
                && (long)in.n * (long)out.n < (1L << 31);
        for (int k = 0; k < NQ && ok; ++k)
            ok = (in.qs[k] == 0 && out.qs[k] == 0)
                    || (in.qg[k] == 1 && out.qg[k] == 1 && in.qs[k] != 0 && out.qs[k] == in.qs[k] * (long)in.n);
        if (!ok) {
            ++x;
            continue;
        }
        v[x].n = in.n * out.n;
        for (int y = x + 1; y + 1 < nv; ++y) v[y] = v[y + 1];
        --nv;
    }
    if (nv == 0) { // a single element
        v[0] = make_dim(d.ndims - 1);
        nv = 1;
    }
    // v[0] has the smallest dst stride: the dim lanes walk.  A transposition:
    // src is unit-stride along another dim.
    const int da = 0;
    int db = -1;
    for (int i = 1; i < nv; ++i)
        if (v[i].ss == 1) db = i;
    const bool tiled = v[da].ds == 1 && db > 0 && v[da].n >= 16 && v[db].n >= 16;
    if (!tiled) db = -1;
    R.a = v[da];
    if (tiled) R.b = v[db];
    long outer = 1;
    for (int i = 1; i < nv; ++i)
        if (i != db) {
            R.outer[R.n_outer++] = v[i];
            outer *= v[i].n;
        }
    if (outer >= (1L << 31)) return MI355_UNIMPLEMENTED;
    R.outer_total = (unsigned)outer;

    // MI355_REORDER_GENERIC=1 keeps the dedicated kernels (row quantization, whole-line transposition) out: for
    // measurements and tests of the kernels behind them
    static const bool generic_only = getenv("MI355_REORDER_GENERIC") != nullptr;
    const int dbits = dt_bits(d.dst_dt), sbits = dt_bits(d.src_dt);
    // E elements per lane along `a` as one aligned vector (several 16-byte ones
    // beyond 16 bytes): unit stride, an extent that divides, every other stride
    // and the pointer aligned to it
    auto vec_ok = [&](const void *p, bool src_side, int bits, int E) {
        const long sa = src_side ? v[da].ss : v[da].ds;
        if (sa != 1 || v[da].n % E) return false;
        long bytes = (long)E * bits / 8;
        if (bytes > 16) bytes = 16;
        if (bytes < 1) bytes = 1;
        if ((uintptr_t)p % (size_t)bytes) return false;
        for (int i = 1; i < nv; ++i)
            if ((src_side ? v[i].ss : v[i].ds) % E) return false;
        return true;
    };
    R.plain_copy = d.src_dt == d.dst_dt && d.beta == 0.f && d.src_scale.dt == MI355_DT_UNDEF
            && d.dst_scale.dt == MI355_DT_UNDEF && d.src_zp.dt == MI355_DT_UNDEF && d.dst_zp.dt == MI355_DT_UNDEF;
    // direct kernel: the widest E in {16, 8, 4} whose narrower side is at most
    // 16 bytes and whose wider side at most 64 bytes per lane
    int E = 1;
    if (!tiled) {
        const int narrow = dbits < sbits ? dbits : sbits, wide = dbits < sbits ? sbits : dbits;
        for (int cand = 16; cand >= 4 && E == 1; cand /= 2)
            if (cand * narrow <= 128 && cand * wide <= 256 && vec_ok(R.dst, false, dbits, cand)) E = cand;
        if (E == 1 && dbits == 4) E = 2;
    } else {
        E = 4;
    }
    R.packed = E >= 4 && vec_ok(R.dst, false, dbits, E);
    R.src_vec = E >= 4 && vec_ok(R.src, true, sbits, E);
    hipStream_t hs = (hipStream_t)stream;
    const unsigned gy = (unsigned)(outer < 65535 ? outer : 65535);
    if (tiled) {
        R.tiles_a = (R.a.n + 63) / 64;
        R.tiles_b = (R.b.n + 63) / 64;
        R.elems = 4;
        long gx = (long)R.tiles_a * R.tiles_b;
        if (gx > (1 << 20)) gx = 1 << 20;
        // 8-bit transposition without attributes: whole tiles, dword loads along b, 16-byte stores along a
        bool t8 = R.plain_copy && dbits == 8 && R.a.n % 64 == 0 && R.b.n % 64 == 0 && R.a.ss % 4 == 0
                && R.b.ds % 16 == 0 && (uintptr_t)R.src % 4 == 0 && (uintptr_t)R.dst % 16 == 0;
        for (int i = 0; i < R.n_outer && t8; ++i)
            if (R.outer[i].ss % 4 || R.outer[i].ds % 16) t8 = false;
        const bool simple = d.beta == 0.f && d.src_scale.dt == MI355_DT_UNDEF && d.dst_scale.dt == MI355_DT_UNDEF
                && d.src_zp.dt == MI355_DT_UNDEF && d.dst_zp.dt == MI355_DT_UNDEF;
        // a lane converts four consecutive a at one b: every parameter tensor constant
        // along a, or its four values consecutive and aligned
        bool qvec = !simple && d.beta == 0.f;
        for (int k = 0; k < 3 && qvec; ++k) {
            if (!R.qp[k] || R.a.qs[k] == 0) continue;
            const long bytes = 4L * dt_bits(R.qdt[k]) / 8;
            if (R.a.qs[k] != 1 || R.a.qg[k] != 1 || (uintptr_t)R.qp[k] % (size_t)bytes || R.b.qs[k] % 4) qvec = false;
            for (int i = 0; i < R.n_outer && qvec; ++i)
                if (R.outer[i].qs[k] % 4) qvec = false;
        }
        // ... and whole 128-byte lines on both sides where the extents and the row pitches allow
        bool t8w = t8 && R.a.n % 128 == 0 && R.b.n % 128 == 0 && R.a.ss % 16 == 0 && (uintptr_t)R.src % 16 == 0
                && !generic_only;
        for (int i = 0; i < R.n_outer && t8w; ++i)
            if (R.outer[i].ss % 16) t8w = false;
        const dim3 grid((unsigned)gx, gy), block(256);
        if (t8w) {
            long gw = (long)(R.a.n / 128) * (R.b.n / 128);
            if (gw > (1 << 20)) gw = 1 << 20;
            hipLaunchKernelGGL(transpose8w_kernel, dim3((unsigned)gw, gy), block, 0, hs, R);
        } else if (t8) hipLaunchKernelGGL(transpose8_kernel, grid, block, 0, hs, R);
        else if (R.a.n % 4 == 0 && simple) hipLaunchKernelGGL(reorder_tiled_kernel<MODE_SIMPLE>, grid, block, 0, hs, R);
        else if (R.a.n % 4 == 0 && qvec) hipLaunchKernelGGL(reorder_tiled_kernel<MODE_QVEC>, grid, block, 0, hs, R);
        else hipLaunchKernelGGL(reorder_tiled_kernel<MODE_GENERIC>, grid, block, 0, hs, R);
    } else {
        // row quantization (float src, 8-bit dst, per-tensor / per-column f32 scales): the dedicated kernel
        {
            const bool src_ok = d.src_dt == MI355_DT_F32 || d.src_dt == MI355_DT_BF16 || d.src_dt == MI355_DT_F16;
            const bool dst_ok = d.dst_dt == MI355_DT_S8 || d.dst_dt == MI355_DT_U8 || d.dst_dt == MI355_DT_F8_E4M3
                    || d.dst_dt == MI355_DT_F8_E5M2;
            const long sbytes = 4L * sbits / 8;
            bool rows_ok = src_ok && dst_ok && d.beta == 0.f && R.n_outer <= 1 && R.a.ss == 1 && R.a.ds == 1
                    && R.a.n % 4 == 0 && !R.qp[2] && (uintptr_t)R.src % (size_t)sbytes == 0 && (uintptr_t)R.dst % 4 == 0
                    && !generic_only;
            if (rows_ok && R.n_outer == 1) rows_ok = R.outer[0].ss % 4 == 0 && R.outer[0].ds % 4 == 0;
            for (int k = 0; k < 2 && rows_ok; ++k) {
                if (!R.qp[k]) continue;
                rows_ok = R.qdt[k] == MI355_DT_F32 && (R.a.qs[k] == 0 || (R.a.qs[k] == 1 && R.a.qg[k] == 1))
                        && (R.n_outer == 0 || R.outer[0].qs[k] == 0);
            }
            if (rows_ok) {
                const unsigned rows = R.n_outer ? R.outer[0].n : 1;
                const unsigned chunks = (unsigned)((R.a.n / 4 + 255) / 256);
                // some 4096 workgroups, at least four rows (one round of loads) each
                unsigned per = (unsigned)(((unsigned long)rows * chunks + 4095) / 4096);
                per = per < 4 ? 4 : (per + 3) / 4 * 4;
                const dim3 rgrid(chunks, (rows + per - 1) / per), block(256);
                if (rgrid.y <= 65535) {
#define MI355_ROWS_CASE(S_, D_) \
    if (d.src_dt == S_ && d.dst_dt == D_) hipLaunchKernelGGL((reorder_rows_kernel<S_, D_>), rgrid, block, 0, hs, R, per);
#define MI355_ROWS_SRC(S_) \
    MI355_ROWS_CASE(S_, MI355_DT_S8) MI355_ROWS_CASE(S_, MI355_DT_U8) MI355_ROWS_CASE(S_, MI355_DT_F8_E4M3) \
    MI355_ROWS_CASE(S_, MI355_DT_F8_E5M2)
                    MI355_ROWS_SRC(MI355_DT_F32)
                    MI355_ROWS_SRC(MI355_DT_BF16)
                    MI355_ROWS_SRC(MI355_DT_F16)
#undef MI355_ROWS_SRC
#undef MI355_ROWS_CASE
                    if (hipGetLastError() != hipSuccess) {
                        set_error("reorder: launch failed");
                        return MI355_RUNTIME_ERROR;
                    }
                    return MI355_SUCCESS;
                }
            }
        }
        R.elems = E;
        // units of all outer indices in one grid-stride walk; enough workgroups
        // to fill the device a few times over, each lane several units
        const long total_units = outer * ((long)R.a.n / E);
        long gx = (total_units + 255) / 256;
        if (gx > 256 * 16) gx = 256 * 16;
        if (gx < 1) gx = 1;
        const dim3 grid((unsigned)gx), block(256);
        const bool simple = d.beta == 0.f && d.src_scale.dt == MI355_DT_UNDEF && d.dst_scale.dt == MI355_DT_UNDEF
                && d.src_zp.dt == MI355_DT_UNDEF && d.dst_zp.dt == MI355_DT_UNDEF;
        // every parameter tensor constant along a unit, or its E values consecutive and aligned
        bool qvec = !simple && d.beta == 0.f && E >= 4;
        for (int k = 0; k < 3 && qvec; ++k) {
            if (!R.qp[k] || R.a.qs[k] == 0) continue;
            const int pbits = dt_bits(R.qdt[k]);
            long bytes = (long)E * pbits / 8;
            if (bytes > 16) bytes = 16;
            if (bytes < 1) bytes = 1;
            if (R.a.qs[k] != 1 || R.a.qg[k] != 1 || (uintptr_t)R.qp[k] % (size_t)bytes) qvec = false;
            for (int i = 0; i < R.n_outer && qvec; ++i)
                if (R.outer[i].qs[k] % E) qvec = false;
        }
        const int mode = simple ? MODE_SIMPLE : qvec ? MODE_QVEC : MODE_GENERIC;
#define MI355_REORDER_CASE(E_) \
    if (E == E_) { \
        if (mode == MODE_SIMPLE) hipLaunchKernelGGL((reorder_direct_kernel<E_, MODE_SIMPLE>), grid, block, 0, hs, R); \
        else if (mode == MODE_QVEC) hipLaunchKernelGGL((reorder_direct_kernel<E_, MODE_QVEC>), grid, block, 0, hs, R); \
        else hipLaunchKernelGGL((reorder_direct_kernel<E_, MODE_GENERIC>), grid, block, 0, hs, R); \
    }
        MI355_REORDER_CASE(16)
        MI355_REORDER_CASE(8)
        MI355_REORDER_CASE(4)
        MI355_REORDER_CASE(2)
        MI355_REORDER_CASE(1)
#undef MI355_REORDER_CASE
    }
    if (hipGetLastError() != hipSuccess) {
        set_error("reorder: launch failed");
        return MI355_RUNTIME_ERROR;
    }
    return MI355_SUCCESS;
}

extern "C" int mi355_wei_pack_reorder_dims(int packing, int64_t K, int64_t N, int64_t src_stride_k,
        int64_t src_stride_n, mi355_reorder_desc_t *desc) {
    using namespace mi355;
    if (!desc || packing != MI355_WEI_PACK_WOQ64 || K <= 0 || N <= 0 || K % 32 || N % 64) {
        set_error("weights packing %d does not fit K = %ld, N = %ld", packing, (long)K, (long)N);
        return MI355_INVALID_ARGUMENTS;
    }
    // k = 8 * kq + 2 * r_hi + r_lo, n = 64 * c + 16 * t + j; dims in the order
    // (kq, r_hi, r_lo, c, t, j)
    const int64_t dims[6] = {K / 8, 4, 2, N / 64, 4, 16};
    const int64_t ss[6] = {8 * src_stride_k, 2 * src_stride_k, src_stride_k, 64 * src_stride_n, 16 * src_stride_n,
            src_stride_n};
    const int64_t ds[6] = {512, 1, 4, K * 64, 8, 32};
    desc->ndims = 6;
    for (int i = 0; i < 6; ++i) {
        desc->dims[i] = dims[i];
        desc->src_stride[i] = ss[i];
        desc->dst_stride[i] = ds[i];
    }
    return MI355_SUCCESS;
}
