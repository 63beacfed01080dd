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
// Two kernels:
//   direct  the unit-stride dim of dst is also unit-stride in src (or no dim
//           is): consecutive lanes walk that dim, four elements per lane when
//           it divides, stores packed to 2 / 4 / 8 / 16 bytes.
//   tiled   src and dst are unit-stride along different dims (a transposition):
//           a 64x64 tile of the two dims goes through LDS, read with lanes
//           along the src dim and written with lanes along the dst dim, so
//           both sides move whole cache lines.
#include "kernels.hpp"

namespace mi355 {
namespace {

constexpr int RD = MI355_REORDER_MAX_DIMS;

struct rq_t { // one quantization parameter tensor
    const void *p;
    int dt;
    int present;
    long stride[RD]; // element stride of the parameter tensor per dim, 0 = broadcast
    long group[RD];  // logical indices per parameter along the dim
};

struct reorder_t {
    int ndims, src_dt, dst_dt;
    float beta;
    const void *src;
    void *dst;
    long dims[RD], ss[RD], ds[RD];
    // walk order: dims sorted by ascending dst stride; order[0] is the inner dim
    int order[RD];
    rq_t src_scale, dst_scale, src_zp, dst_zp;
    long total;     // logical elements
    int inner_elems; // elements per lane along order[0] (direct kernel)
    // tiled kernel: the two tile dims and the number of tiles along each
    int dim_s, dim_d;
    long tiles_s, tiles_d, outer;
};

__device__ __forceinline__ bool is_int_dt(int dt) {
    return dt == MI355_DT_S32 || dt == MI355_DT_S8 || dt == MI355_DT_U8 || dt == MI355_DT_S4
            || dt == MI355_DT_U4;
}

// idx[dim] = v / idx[dim] += v without a run-time array index (which would move
// the index vector to private memory)
__device__ __forceinline__ void idx_set(long (&idx)[RD], int dim, long v) {
#pragma unroll
    for (int d = 0; d < RD; ++d)
        if (d == dim) idx[d] = v;
}
__device__ __forceinline__ void idx_add(long (&idx)[RD], int dim, long v) {
#pragma unroll
    for (int d = 0; d < RD; ++d)
        if (d == dim) idx[d] += v;
}

// (RT / QT: the structures are read in place from the kernel argument segment)
template <class QT>
__device__ __forceinline__ long rq_off(const QT &q, const long (&idx)[RD], int ndims) {
    long off = 0;
#pragma unroll
    for (int d = 0; d < RD; ++d)
        if (d < ndims && q.stride[d]) off += (idx[d] / q.group[d]) * q.stride[d];
    return off;
}

// the converted element at logical index idx, as the raw bits of the dst type
template <class RT>
__device__ __forceinline__ uint32_t reorder_value(const RT &R, const long (&idx)[RD]) {
    long so = 0, dof = 0;
#pragma unroll
    for (int d = 0; d < RD; ++d)
        if (d < R.ndims) {
            so += idx[d] * R.ss[d];
            dof += idx[d] * R.ds[d];
        }
    float x;
    if (R.src_dt == MI355_DT_E8M0) {
        x = load_float(MI355_DT_E8M0, R.src, so);
    } else {
        int zp = 0;
        if (R.src_zp.present)
            zp = (int)load_float(R.src_zp.dt, R.src_zp.p, rq_off(R.src_zp, idx, R.ndims));
        if (is_int_dt(R.src_dt)) x = (float)(load_int(R.src_dt, R.src, so) - zp);
        else x = load_float(R.src_dt, R.src, so) - (float)zp;
        if (R.src_scale.present)
            x = load_float(R.src_scale.dt, R.src_scale.p, rq_off(R.src_scale, idx, R.ndims)) * x;
        if (R.beta != 0.f) x += R.beta * load_float(R.dst_dt, R.dst, dof);
        if (R.dst_scale.present || R.dst_zp.present) {
            float dsc = 1.f;
            int dzp = 0;
            if (R.dst_scale.present)
                dsc = load_float(R.dst_scale.dt, R.dst_scale.p, rq_off(R.dst_scale, idx, R.ndims));
            if (R.dst_zp.present) dzp = load_int(R.dst_zp.dt, R.dst_zp.p, 0);
            x = x / dsc + (float)dzp;
        }
    }
    switch (R.dst_dt) {
        case MI355_DT_S4: return (uint32_t)(int)__builtin_rintf(sat(x, -8.f, 7.f)) & 0xfu;
        case MI355_DT_U4: return (uint32_t)(int)__builtin_rintf(sat(x, 0.f, 15.f)) & 0xfu;
        case MI355_DT_F4_E2M1: return f32_to_e2m1(x);
        default: return cvt_store_bits(R.dst_dt, x);
    }
}

// store n (1, 2 or 4) consecutive dst elements starting at element offset off
template <int N>
__device__ __forceinline__ void store_bits(int dt, void *dst, long off, const uint32_t (&w)[N], bool packed) {
    const int bits = dt_bits(dt);
    if (bits == 4) {
        // off is even and the N nibbles fill whole bytes
        uint8_t *p = (uint8_t *)dst + (off >> 1);
#pragma unroll
        for (int e = 0; e + 1 < N; e += 2) p[e >> 1] = (uint8_t)(w[e] | (w[e + 1] << 4));
        return;
    }
    if (packed && N == 4) {
        if (bits == 8) {
            *(uint32_t *)((uint8_t *)dst + off) = w[0] | (w[1] << 8) | (w[2] << 16) | (w[3] << 24);
        } else if (bits == 16) {
            uint2 o;
            o.x = w[0] | (w[1] << 16);
            o.y = w[2] | (w[3] << 16);
            *(uint2 *)((uint16_t *)dst + off) = o;
        } else {
            uint4 o;
            o.x = w[0]; o.y = w[1]; o.z = w[2]; o.w = w[3];
            *(uint4 *)((uint32_t *)dst + off) = o;
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < N; ++e) {
        if (bits == 8) ((uint8_t *)dst)[off + e] = (uint8_t)w[e];
        else if (bits == 16) ((uint16_t *)dst)[off + e] = (uint16_t)w[e];
        else ((uint32_t *)dst)[off + e] = w[e];
    }
}

// E elements per lane along the inner dim (dst stride 1 when E > 1)
template <int E>
__global__ void __launch_bounds__(256) reorder_direct_kernel(const reorder_t R_) {
    const auto &R = *(const __attribute__((address_space(4))) reorder_t *)__builtin_amdgcn_kernarg_segment_ptr();
    const long units = R.total / E;
    for (long u = (long)blockIdx.x * blockDim.x + threadIdx.x; u < units; u += (long)gridDim.x * blockDim.x) {
        long idx[RD] = {0, 0, 0, 0, 0, 0};
        long rem = u;
#pragma unroll
        for (int k = 0; k < RD; ++k)
            if (k < R.ndims) {
                const int d = R.order[k];
                const long n = k == 0 ? R.dims[d] / E : R.dims[d];
                const long q = rem / n;
                idx_set(idx, d, (rem - q * n) * (k == 0 ? E : 1));
                rem = q;
            }
        const int di = R.order[0];
        long dof = 0;
#pragma unroll
        for (int d = 0; d < RD; ++d)
            if (d < R.ndims) dof += idx[d] * R.ds[d];
        uint32_t w[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            w[e] = reorder_value(R, idx);
            idx_add(idx, di, 1);
        }
        store_bits<E>(R.dst_dt, R.dst, dof, w, true);
    }
}

// 64 x 64 tile over (dim_s, dim_d); one workgroup per tile and outer index
__global__ void __launch_bounds__(256) reorder_tiled_kernel(const reorder_t R_) {
    const auto &R = *(const __attribute__((address_space(4))) reorder_t *)__builtin_amdgcn_kernarg_segment_ptr();
    __shared__ uint32_t tile[64][65];
    const long per_outer = R.tiles_s * R.tiles_d;
    const long ntiles = per_outer * R.outer;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (long t = blockIdx.x; t < ntiles; t += gridDim.x) {
        long idx[RD] = {0, 0, 0, 0, 0, 0};
        long rem = t / per_outer;
        const long in_outer = t - rem * per_outer;
        // the other dims, fastest first in dst order
#pragma unroll
        for (int k = 0; k < RD; ++k)
            if (k < R.ndims) {
                const int d = R.order[k];
                if (d != R.dim_s && d != R.dim_d) {
                    const long q = rem / R.dims[d];
                    idx_set(idx, d, rem - q * R.dims[d]);
                    rem = q;
                }
            }
        const long s0 = (in_outer % R.tiles_s) * 64, d0 = (in_outer / R.tiles_s) * 64;
        // read: lanes along the src unit-stride dim
        for (int i = ty; i < 64; i += 4) {
            idx_set(idx, R.dim_s, s0 + tx);
            idx_set(idx, R.dim_d, d0 + i);
            uint32_t v = 0;
            if (s0 + tx < R.dims[R.dim_s] && d0 + i < R.dims[R.dim_d]) v = reorder_value(R, idx);
            tile[i][tx] = v;
        }
        __syncthreads();
        // write: lanes along the dst unit-stride dim, four elements each
        const int lx = (threadIdx.x & 15) * 4, ly = threadIdx.x >> 4;
        for (int i = ly; i < 64; i += 16) {
            const long is = s0 + i, id = d0 + lx;
            if (is < R.dims[R.dim_s] && id < R.dims[R.dim_d]) {
                idx_set(idx, R.dim_s, is);
                idx_set(idx, R.dim_d, id);
                long dof = 0;
#pragma unroll
                for (int d = 0; d < RD; ++d)
                    if (d < R.ndims) dof += idx[d] * R.ds[d];
                const uint32_t w[4] = {tile[lx][i], tile[lx + 1][i], tile[lx + 2][i], tile[lx + 3][i]};
                if (id + 4 <= R.dims[R.dim_d]) {
                    store_bits<4>(R.dst_dt, R.dst, dof, w, R.inner_elems == 4);
                } else { // ragged edge of the dst dim: dims[dim_d] is even for 4-bit types
                    const int left = (int)(R.dims[R.dim_d] - id);
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

bool dt_ok(int dt) {
    switch (dt) {
        case MI355_DT_F16: case MI355_DT_BF16: case MI355_DT_F32: case MI355_DT_S32: case MI355_DT_S8:
        case MI355_DT_U8: case MI355_DT_F8_E5M2: case MI355_DT_F8_E4M3: case MI355_DT_S4: case MI355_DT_U4:
        case MI355_DT_E8M0: case MI355_DT_F4_E2M1: return true;
        default: return false;
    }
}

// quantization parameter tensor strides over the tensor's dims
// (quant_entry_t::get_md, src/common/primitive_attr_quant.hpp:116-140)
void fill_rq(rq_t &q, const mi355_quant_t &m, const void *p, int ndims, const int64_t *dims) {
    q.p = p;
    q.dt = m.dt;
    q.present = m.dt != MI355_DT_UNDEF;
    long stride = 1;
    for (int d = RD - 1; d >= 0; --d) {
        q.stride[d] = 0;
        q.group[d] = 1;
        if (d >= ndims || !q.present) continue;
        if (d == ndims - 2) q.group[d] = m.group[0];
        if (d == ndims - 1) q.group[d] = m.group[1];
        if (m.mask & (1 << d)) {
            q.stride[d] = stride;
            stride *= dims[d] / q.group[d];
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
    reorder_t R {};
    R.ndims = d.ndims;
    R.src_dt = d.src_dt;
    R.dst_dt = d.dst_dt;
    R.beta = d.beta;
    R.src = args->src;
    R.dst = args->dst;
    R.total = 1;
    for (int i = 0; i < RD; ++i) {
        R.dims[i] = i < d.ndims ? d.dims[i] : 1;
        R.ss[i] = i < d.ndims ? d.src_stride[i] : 0;
        R.ds[i] = i < d.ndims ? d.dst_stride[i] : 0;
        R.order[i] = i;
        R.total *= R.dims[i];
    }
    if (R.total == 0) return MI355_SUCCESS;
    if (!args->src || !args->dst) {
        set_error("reorder: null tensor");
        return MI355_INVALID_ARGUMENTS;
    }
    // walk order: ascending dst stride, dims of size 1 last
    for (int a = 0; a < d.ndims; ++a)
        for (int b = a + 1; b < d.ndims; ++b) {
            const int x = R.order[a], y = R.order[b];
            const bool x_one = R.dims[x] == 1, y_one = R.dims[y] == 1;
            if ((x_one && !y_one) || (x_one == y_one && R.ds[y] < R.ds[x])) {
                R.order[a] = y;
                R.order[b] = x;
            }
        }
    fill_rq(R.src_scale, d.src_scale, args->src_scale, d.ndims, d.dims);
    fill_rq(R.dst_scale, d.dst_scale, args->dst_scale, d.ndims, d.dims);
    fill_rq(R.src_zp, d.src_zp, args->src_zp, d.ndims, d.dims);
    fill_rq(R.dst_zp, d.dst_zp, args->dst_zp, d.ndims, d.dims);
    const mi355_quant_t *qs[4] = {&d.src_scale, &d.dst_scale, &d.src_zp, &d.dst_zp};
    const void *qp[4] = {args->src_scale, args->dst_scale, args->src_zp, args->dst_zp};
    for (int i = 0; i < 4; ++i)
        if (qs[i]->dt != MI355_DT_UNDEF && !qp[i]) {
            set_error("reorder: a declared scale or zero point tensor is null");
            return MI355_INVALID_ARGUMENTS;
        }

    const int di = R.order[0];
    const bool dst_unit = R.ds[di] == 1;
    const int dbits = dt_bits(d.dst_dt);
    // packed stores of four need the pointer and every other stride aligned
    auto packable = [&](int dim) {
        if (R.ds[dim] != 1 || R.dims[dim] % 4) return false;
        const long bytes4 = dbits / 2; // bytes of four elements
        if (dbits != 4 && ((uintptr_t)R.dst % (bytes4 ? bytes4 : 1))) return false;
        for (int i = 0; i < d.ndims; ++i)
            if (i != dim && R.dims[i] > 1 && R.ds[i] % 4) return false;
        return true;
    };
    // a transposition: src is unit-stride along another dim than dst
    int dim_s = -1;
    for (int i = 0; i < d.ndims; ++i)
        if (R.ss[i] == 1 && R.dims[i] > 1) dim_s = i;
    hipStream_t hs = (hipStream_t)stream;
    if (dst_unit && dim_s >= 0 && dim_s != di && R.dims[di] >= 16 && R.dims[dim_s] >= 16) {
        R.dim_s = dim_s;
        R.dim_d = di;
        R.tiles_s = (R.dims[dim_s] + 63) / 64;
        R.tiles_d = (R.dims[di] + 63) / 64;
        R.outer = R.total / (R.dims[dim_s] * R.dims[di]);
        R.inner_elems = packable(di) ? 4 : 1;
        if (dbits == 4 && R.inner_elems != 4) {
            // nibble pairs are stored as bytes: needs even offsets, which check() ensured
            R.inner_elems = 2;
        }
        long blocks = R.tiles_s * R.tiles_d * R.outer;
        if (blocks > (1 << 20)) blocks = 1 << 20;
        hipLaunchKernelGGL(reorder_tiled_kernel, dim3((unsigned)blocks), dim3(256), 0, hs, R);
    } else {
        int E = 1;
        if (dst_unit && packable(di)) E = 4;
        else if (dbits == 4) E = 2;
        R.inner_elems = E;
        const long units = R.total / E;
        long blocks = (units + 255) / 256;
        if (blocks > (1 << 20)) blocks = 1 << 20;
        if (E == 4) hipLaunchKernelGGL(reorder_direct_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, hs, R);
        else if (E == 2) hipLaunchKernelGGL(reorder_direct_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, hs, R);
        else hipLaunchKernelGGL(reorder_direct_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, hs, R);
    }
    if (hipGetLastError() != hipSuccess) {
        set_error("reorder: launch failed");
        return MI355_RUNTIME_ERROR;
    }
    return MI355_SUCCESS;
}
