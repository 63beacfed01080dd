// The reference's MX tutorial (examples/tutorials/matmul/mxfp_matmul.cpp) as a caller of include/dnnl_amd.hpp on a
// GPU engine: MXFP8 everywhere -- e4m3 elements with e8m0 scales per 32 consecutive k on A (row-major) and B
// (column-major), and a dst that the primitive itself quantizes the MX way (quantization_mode::dynamic_mx: e4m3
// elements plus one e8m0 scale per 32 columns, written to DNNL_ARG_ATTR_SCALES | DNNL_ARG_DST).  A is brought to e4m3
// by a reorder from f32, as in the tutorial.  Checked on the host: the scale of every dst block is the power of two
// the MX recipe prescribes for the block's largest magnitude (ref_matmul.cpp:343-351) and every element, multiplied
// back by its scale, is the double-precision result within e4m3's rounding.  Prints "ok <impl>".
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "dnnl_amd.hpp"

using namespace dnnl;

namespace {
template <typename T>
void write_to(const memory &mem, const std::vector<T> &v) {
    T *p = mem.map_data<T>();
    std::memcpy(p, v.data(), v.size() * sizeof(T));
    mem.unmap_data(p);
}
template <typename T>
std::vector<T> read_from(const memory &mem, size_t n) {
    std::vector<T> v(n);
    T *p = mem.map_data<T>();
    std::memcpy(v.data(), p, n * sizeof(T));
    mem.unmap_data(p);
    return v;
}
double e4m3(uint8_t b) { // (0x7f / 0xff are NaN and not generated here)
    const int e = (b >> 3) & 15, m = b & 7;
    const double v = e == 0 ? std::ldexp((double)m, -9) : std::ldexp(1.0 + m / 8.0, e - 7);
    return (b & 0x80) ? -v : v;
}
double e8m0(uint8_t b) { return std::ldexp(1.0, (int)b - 127); }
unsigned seed = 99u;
unsigned next() {
    seed = seed * 1664525u + 1013904223u;
    return seed >> 16;
}
} // namespace

int main() {
    try {
        const memory::dim M = 96, N = 64, K = 128, BLK = 32;
        engine eng(engine::kind::gpu, 0);
        memory::desc a_md({M, K}, memory::data_type::f8_e4m3, {K, 1});
        memory::desc b_md({K, N}, memory::data_type::f8_e4m3, {1, K});
        memory::desc c_md({M, N}, memory::data_type::f8_e4m3, {N, 1});
        const int mask = (1 << 1) | (1 << 0);
        primitive_attr attr;
        attr.set_scales(DNNL_ARG_SRC, mask, {1, 32}, memory::data_type::e8m0);
        attr.set_scales(DNNL_ARG_WEIGHTS, mask, {32, 1}, memory::data_type::e8m0);
        attr.set_scales(DNNL_ARG_DST, mask, {1, 32}, memory::data_type::e8m0, false, quantization_mode::dynamic_mx);
        matmul::primitive_desc pd(eng, a_md, b_md, c_md, attr);
        const std::string impl = pd.impl_info_str();

        stream s(eng);
        // A: f32 values in (-6, 6) through a reorder; what it rounded them to is read back for the check
        std::vector<float> a_f32(M * K);
        for (auto &v : a_f32) v = 12.f * (float)(next() & 0xfff) / 4096.f - 6.f;
        memory a_f32_mem({{M, K}, memory::data_type::f32, {K, 1}}, eng), a_mem(pd.src_desc(), eng);
        write_to(a_f32_mem, a_f32);
        reorder(a_f32_mem, a_mem).execute(s, a_f32_mem, a_mem);
        s.wait();
        const std::vector<uint8_t> a = read_from<uint8_t>(a_mem, M * K);
        for (memory::dim i = 0; i < M * K; ++i)
            if (std::fabs(e4m3(a[i]) - (double)a_f32[i]) > std::fabs((double)a_f32[i]) / 16.0 + 1.0 / 1024.0) {
                std::fprintf(stderr, "reorder: %g became %g\n", a_f32[i], e4m3(a[i]));
                return 2;
            }
        // B: e4m3 bytes over a few binades, stored column by column ([N][K] in memory)
        std::vector<uint8_t> b(N * K), sa(M * (K / BLK)), sb((K / BLK) * N);
        for (auto &v : b) v = (uint8_t)(((next() & 1) << 7) | (0x28 + next() % 0x28));
        for (auto &v : sa) v = (uint8_t)(125 + next() % 4);
        for (auto &v : sb) v = (uint8_t)(125 + next() % 4);
        memory b_mem(pd.weights_desc(), eng), c_mem(pd.dst_desc(), eng);
        memory sa_mem({{M * (K / BLK)}, memory::data_type::e8m0, {1}}, eng);   // [M][K / 32]
        memory sb_mem({{(K / BLK) * N}, memory::data_type::e8m0, {1}}, eng);   // [K / 32][N]
        memory sc_mem({{M * (N / BLK)}, memory::data_type::e8m0, {1}}, eng);   // [M][N / 32], written by the primitive
        write_to(b_mem, b);
        write_to(sa_mem, sa);
        write_to(sb_mem, sb);
        matmul(pd).execute(s,
                {{DNNL_ARG_SRC, a_mem}, {DNNL_ARG_ATTR_SCALES | DNNL_ARG_SRC, sa_mem}, {DNNL_ARG_WEIGHTS, b_mem},
                        {DNNL_ARG_ATTR_SCALES | DNNL_ARG_WEIGHTS, sb_mem}, {DNNL_ARG_DST, c_mem},
                        {DNNL_ARG_ATTR_SCALES | DNNL_ARG_DST, sc_mem}});
        s.wait();
        const std::vector<uint8_t> c = read_from<uint8_t>(c_mem, M * N), sc = read_from<uint8_t>(sc_mem, M * (N / BLK));

        for (memory::dim m = 0; m < M; ++m)
            for (memory::dim nb = 0; nb < N / BLK; ++nb) {
                double ref[32], mag[32], amax = 0.0;
                for (memory::dim j = 0; j < BLK; ++j) {
                    const memory::dim n = nb * BLK + j;
                    ref[j] = mag[j] = 0.0;
                    for (memory::dim k = 0; k < K; ++k) {
                        const double t = e4m3(a[m * K + k]) * e8m0(sa[m * (K / BLK) + k / BLK]) * e4m3(b[n * K + k])
                                * e8m0(sb[(k / BLK) * N + n]);
                        ref[j] += t;
                        mag[j] += std::fabs(t);
                    }
                    amax = std::fmax(amax, std::fabs(ref[j]));
                }
                // 2^floor(log2 amax) / 2^floor(log2 448): the block's largest magnitude lands in [256, 512)
                const double scale = e8m0(sc[m * (N / BLK) + nb]);
                if (!(amax / scale > 255.0 && amax / scale < 513.0)) {
                    std::fprintf(stderr, "block (%ld, %ld): scale %g for a largest magnitude of %g\n", (long)m, (long)nb, scale, amax);
                    return 3;
                }
                for (memory::dim j = 0; j < BLK; ++j) {
                    double x = ref[j] / scale;
                    x = x > 448.0 ? 448.0 : (x < -448.0 ? -448.0 : x); // e4m3 saturates
                    const double got = e4m3(c[m * N + nb * BLK + j]);
                    // half a step of e4m3 (2^-4 relative, 2^-10 among the subnormals) + the f32 sum of K products
                    const double tol = std::fabs(x) / 16.0 + 1.0 / 1024.0 + 2e-5 * mag[j] / scale;
                    if (std::fabs(got - x) > tol) {
                        std::fprintf(stderr, "element (%ld, %ld): %g, not %g (scale %g)\n", (long)m, (long)(nb * BLK + j), got, x, scale);
                        return 4;
                    }
                }
            }
        std::printf("ok %s\n", impl.c_str());
        return 0;
    } catch (const error &e) {
        std::fprintf(stderr, "dnnl::error: %s (status %d)\n", e.message, (int)e.status);
        return 10;
    }
}
