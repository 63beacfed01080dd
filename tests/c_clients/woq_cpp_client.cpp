// The reference's weight-only-quantization tutorial (examples/tutorials/matmul/
// matmul_with_weight_only_quantization.cpp) as a caller of include/dnnl_amd.hpp, on a GPU engine:
//   C_f32 = A_f32 x ((B_s8 - zp_B) * sc_B), scales and zero points per column and per group of K, weights given as
//   format_tag::any and quantized from f32 by a reorder, fpmath strict with apply_to_int;
// then the decode case of the same recipe -- bf16 activations, u4 weights in the layout the primitive picks for
// them, bf16 scales and u8 zero points per group of 128 -- which is what the packed decode kernels serve.
// Both are checked against a host loop in the reference's order (ref_matmul.cpp:193-235: the weight is
// (w - zp) * scale in f32, the products are added in f32 in the order of k).  Prints "ok <impl>, <impl>".
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
uint16_t to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
float from_bf16(uint16_t h) {
    const uint32_t u = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
unsigned seed = 7u;
unsigned next() {
    seed = seed * 1664525u + 1013904223u;
    return seed >> 16;
}
float unit() { return (float)(next() & 0xfff) / 4096.f; }
} // namespace

static int tutorial(const engine &eng, std::string &impl) {
    const memory::dim M = 100, N = 1000, K = 64, G = K / 2, n_groups = K / G;
    memory::desc a_md({M, K}, memory::data_type::f32, {K, 1});
    memory::desc b_md({K, N}, memory::data_type::s8, memory::format_tag::any);
    memory::desc c_md({M, N}, memory::data_type::f32, {N, 1});
    primitive_attr attr;
    attr.set_scales(DNNL_ARG_WEIGHTS, (1 << 0) + (1 << 1), {G, 1}, memory::data_type::f32);
    attr.set_zero_points(DNNL_ARG_WEIGHTS, (1 << 0) + (1 << 1), {G, 1}, memory::data_type::s8);
    attr.set_fpmath_mode(fpmath_mode::strict, true);
    matmul::primitive_desc pd(eng, a_md, b_md, c_md, attr);
    impl = pd.impl_info_str();

    // the weights as the user has them, f32 in [-5, 5]; the reorder rounds them to s8
    std::vector<float> b_f32(K * N);
    for (auto &v : b_f32) v = 10.f * unit() - 5.f;
    memory b_s8_mem(pd.weights_desc(), eng);
    stream s(eng);
    {
        memory b_f32_mem({{K, N}, memory::data_type::f32, memory::format_tag::ab}, eng);
        write_to(b_f32_mem, b_f32);
        reorder(b_f32_mem, b_s8_mem).execute(s, b_f32_mem, b_s8_mem);
        s.wait();
    }
    std::vector<float> a(M * K), sc(n_groups * N);
    std::vector<int8_t> zp(n_groups * N);
    for (auto &v : a) v = unit();
    for (auto &v : sc) v = unit();
    for (auto &v : zp) v = (int8_t)((int)(next() % 11) - 5);
    memory a_mem(a_md, eng), c_mem(c_md, eng);
    // (the tutorial's descriptors: N x groups with N innermost in memory)
    memory sc_mem({{N, n_groups}, memory::data_type::f32, {1, N}}, eng);
    memory zp_mem({{N, n_groups}, memory::data_type::s8, {1, N}}, eng);
    write_to(a_mem, a);
    write_to(sc_mem, sc);
    write_to(zp_mem, zp);
    matmul(pd).execute(s,
            {{DNNL_ARG_SRC, a_mem}, {DNNL_ARG_WEIGHTS, b_s8_mem}, {DNNL_ARG_DST, c_mem},
                    {DNNL_ARG_ATTR_SCALES | DNNL_ARG_WEIGHTS, sc_mem}, {DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_WEIGHTS, zp_mem}});
    s.wait();
    const std::vector<float> c = read_from<float>(c_mem, M * N);
    for (memory::dim m = 0; m < M; ++m)
        for (memory::dim n = 0; n < N; ++n) {
            double ref = 0.0, mag = 0.0;
            for (memory::dim k = 0; k < K; ++k) {
                float q = std::nearbyintf(b_f32[k * N + n]);
                q = q < -128.f ? -128.f : (q > 127.f ? 127.f : q);
                const float w = (q - (float)zp[(k / G) * N + n]) * sc[(k / G) * N + n];
                ref += (double)a[m * K + k] * (double)w;
                mag += std::fabs((double)a[m * K + k] * (double)w);
            }
            // f32 products and K f32 additions against the exact sum
            if (std::fabs((double)c[m * N + n] - ref) > (K + 2) * 6e-8 * mag + 1e-30) {
                std::fprintf(stderr, "tutorial: element (%ld, %ld) is %g, not %g\n", (long)m, (long)n, c[m * N + n], ref);
                return 2;
            }
        }
    return 0;
}

static int decode(const engine &eng, std::string &impl) {
    const memory::dim M = 4, N = 14336, K = 4096, G = 128, n_groups = K / G; // (wide enough for the packed layout)
    memory::desc a_md({M, K}, memory::data_type::bf16, memory::format_tag::ab);
    memory::desc b_md({K, N}, memory::data_type::u4, memory::format_tag::any);
    memory::desc c_md({M, N}, memory::data_type::bf16, memory::format_tag::ab);
    primitive_attr attr;
    attr.set_scales(DNNL_ARG_WEIGHTS, (1 << 0) + (1 << 1), {G, 1}, memory::data_type::bf16);
    attr.set_zero_points(DNNL_ARG_WEIGHTS, (1 << 0) + (1 << 1), {G, 1}, memory::data_type::u8);
    attr.set_fpmath_mode(fpmath_mode::bf16, true);
    matmul::primitive_desc pd(eng, a_md, b_md, c_md, attr);
    impl = pd.impl_info_str();
    if (impl.compare(0, 14, "hip:woq_packed") != 0 || pd.weights_desc().get_format_kind() != memory::format_kind::opaque) {
        std::fprintf(stderr, "decode: format_tag::any weights went to %s\n", impl.c_str());
        return 3;
    }

    std::vector<uint8_t> nib(K * N), packed(K * N / 2), zp(n_groups * N);
    for (auto &v : nib) v = (uint8_t)(next() & 15);
    for (memory::dim i = 0; i < K * N / 2; ++i) packed[i] = (uint8_t)(nib[2 * i] | (nib[2 * i + 1] << 4));
    for (auto &v : zp) v = (uint8_t)(next() & 15);
    std::vector<uint16_t> a(M * K), sc(n_groups * N);
    for (auto &v : a) v = to_bf16(2.f * unit() - 1.f);
    for (auto &v : sc) v = to_bf16(0.01f + 0.05f * unit());

    stream s(eng);
    memory b_user({{K, N}, memory::data_type::u4, memory::format_tag::ab}, eng), b_mem(pd.weights_desc(), eng);
    write_to(b_user, packed);
    reorder(b_user, b_mem).execute(s, b_user, b_mem);
    memory a_mem(a_md, eng), c_mem(c_md, eng);
    memory sc_mem({{n_groups, N}, memory::data_type::bf16, memory::format_tag::ab}, eng);
    memory zp_mem({{n_groups, N}, memory::data_type::u8, memory::format_tag::ab}, eng);
    write_to(a_mem, a);
    write_to(sc_mem, sc);
    write_to(zp_mem, zp);
    matmul(pd).execute(s,
            {{DNNL_ARG_SRC, a_mem}, {DNNL_ARG_WEIGHTS, b_mem}, {DNNL_ARG_DST, c_mem},
                    {DNNL_ARG_ATTR_SCALES | DNNL_ARG_WEIGHTS, sc_mem}, {DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_WEIGHTS, zp_mem}});
    s.wait();
    const std::vector<uint16_t> c = read_from<uint16_t>(c_mem, M * N);
    for (memory::dim m = 0; m < M; ++m)
        for (memory::dim n = 0; n < N; ++n) {
            double ref = 0.0, mag = 0.0;
            for (memory::dim k = 0; k < K; ++k) {
                const float w = ((float)nib[k * N + n] - (float)zp[(k / G) * N + n]) * from_bf16(sc[(k / G) * N + n]);
                ref += (double)from_bf16(a[m * K + k]) * (double)w;
                mag += std::fabs((double)from_bf16(a[m * K + k]) * (double)w);
            }
            // the f32 sum (any order) and one rounding to bf16
            const double tol = (K + 2) * 6e-8 * mag + std::fabs(ref) / 256.0 + 1e-30;
            if (std::fabs((double)from_bf16(c[m * N + n]) - ref) > tol) {
                std::fprintf(stderr, "decode: element (%ld, %ld) is %g, not %g\n", (long)m, (long)n, from_bf16(c[m * N + n]), ref);
                return 3;
            }
        }
    return 0;
}

int main() {
    try {
        engine eng(engine::kind::gpu, 0);
        std::string impl1, impl2;
        if (int rc = tutorial(eng, impl1)) return rc;
        if (int rc = decode(eng, impl2)) return rc;
        std::printf("ok %s, %s\n", impl1.c_str(), impl2.c_str());
        return 0;
    } catch (const error &e) {
        std::fprintf(stderr, "dnnl::error: %s (status %d)\n", e.message, (int)e.status);
        return 10;
    }
}
