// A C++ caller of libdnnl_amd.so through include/dnnl_amd.hpp, written the way the reference's int8 inference
// tutorial is (examples/tutorials/matmul/inference_int8_matmul.cpp): u8 activations, s8 weights handed over as
// format_tag::any and brought into the layout the primitive asks for by a reorder, scales for src / weights (per
// column) / dst, zero points for src and dst, a ReLU post-op; then the same weights under a bf16 matmul with bias.
// Every dst element is checked against a host loop that performs the reference's operations in the reference's
// order (ref_matmul_int8.cpp:241-304).  Also exercised: the exception on an illegal descriptor, allow_empty, the
// implementation iterator, queries of descriptors.  Prints "ok <implementation>" and exits 0.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "dnnl_amd.hpp"

using namespace dnnl;

namespace {
const memory::dim M = 96, K = 192, N = 160;

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
} // namespace

int main() {
    try {
        if (engine::get_count(engine::kind::gpu) == 0) {
            std::fprintf(stderr, "no GPU engine\n");
            return 1;
        }
        engine eng(engine::kind::gpu, 0);
        stream s(eng);
        if (eng.get_kind() != engine::kind::gpu || s.get_engine().get_kind() != engine::kind::gpu) return 1;

        // ---- data
        std::vector<uint8_t> a(M * K);
        std::vector<int8_t> b(K * N);
        std::vector<float> sc_b(N);
        unsigned seed = 2024u;
        auto next = [&]() { seed = seed * 1664525u + 1013904223u; return seed >> 24; };
        for (auto &x : a) x = (uint8_t)next();
        for (auto &x : b) x = (int8_t)((int)(next() % 255) - 127);
        for (memory::dim n = 0; n < N; ++n) sc_b[n] = 0.005f + 0.0001f * (float)(n % 17);
        const float sc_a = 0.02f, sc_c = 0.4f;
        const int32_t zp_a = 131, zp_c = 7;

        // ---- descriptors; the weights' layout is the primitive's choice
        memory::desc a_md({M, K}, memory::data_type::u8, {K, 1});
        memory::desc b_any({K, N}, memory::data_type::s8, memory::format_tag::any);
        memory::desc c_md({M, N}, memory::data_type::u8, {N, 1});
        if (a_md.get_dims() != memory::dims({M, K}) || a_md.get_strides() != memory::dims({K, 1})
                || a_md.get_data_type() != memory::data_type::u8 || a_md.get_size() != (size_t)(M * K))
            return 2;

        primitive_attr attr;
        attr.set_scales_mask(DNNL_ARG_SRC, 0);
        attr.set_scales_mask(DNNL_ARG_WEIGHTS, 1 << 1);
        attr.set_scales_mask(DNNL_ARG_DST, 0);
        attr.set_zero_points_mask(DNNL_ARG_SRC, 0);
        attr.set_zero_points_mask(DNNL_ARG_DST, 0);
        post_ops po;
        po.append_eltwise(algorithm::eltwise_relu, 0.f, 0.f);
        attr.set_post_ops(po);
        if (attr.get_post_ops().len() != 1) return 2;

        // an illegal problem throws, or leaves an empty object when asked to
        bool threw = false;
        try {
            matmul::primitive_desc bad(eng, a_md, memory::desc({K + 1, N}, memory::data_type::s8, memory::format_tag::ab), c_md);
        } catch (const error &e) { threw = e.status == dnnl_invalid_arguments; }
        if (!threw) return 3;
        matmul::primitive_desc none(eng, a_md, memory::desc({K + 1, N}, memory::data_type::s8, memory::format_tag::ab), c_md,
                primitive_attr(), /* allow_empty */ true);
        if (none) return 3;

        matmul::primitive_desc pd(eng, a_md, b_any, c_md, attr);
        const std::string impl = pd.impl_info_str();
        if (pd.weights_desc().get_format_kind() == memory::format_kind::any) return 4; // it has been resolved
        if (pd.src_desc() != a_md || pd.dst_desc() != c_md || !pd.bias_desc().is_zero()) return 4;

        // ---- weights: the caller's row-major tensor into the primitive's layout
        memory b_user({{K, N}, memory::data_type::s8, memory::format_tag::ab}, eng);
        write_to(b_user, b);
        memory b_mem(pd.weights_desc(), eng);
        reorder(b_user, b_mem).execute(s, b_user, b_mem);

        memory a_mem(a_md, eng), c_mem(c_md, eng);
        memory sc_a_mem({{1}, memory::data_type::f32, {1}}, eng), sc_b_mem({{N}, memory::data_type::f32, {1}}, eng);
        memory sc_c_mem({{1}, memory::data_type::f32, {1}}, eng);
        memory zp_a_mem({{1}, memory::data_type::s32, {1}}, eng), zp_c_mem({{1}, memory::data_type::s32, {1}}, eng);
        write_to(a_mem, a);
        write_to(sc_a_mem, std::vector<float> {sc_a});
        write_to(sc_b_mem, sc_b);
        write_to(sc_c_mem, std::vector<float> {sc_c});
        write_to(zp_a_mem, std::vector<int32_t> {zp_a});
        write_to(zp_c_mem, std::vector<int32_t> {zp_c});

        matmul mm(pd);
        mm.execute(s,
                {{DNNL_ARG_SRC, a_mem}, {DNNL_ARG_WEIGHTS, b_mem}, {DNNL_ARG_DST, c_mem},
                        {DNNL_ARG_ATTR_SCALES | DNNL_ARG_SRC, sc_a_mem}, {DNNL_ARG_ATTR_SCALES | DNNL_ARG_WEIGHTS, sc_b_mem},
                        {DNNL_ARG_ATTR_SCALES | DNNL_ARG_DST, sc_c_mem},
                        {DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_SRC, zp_a_mem},
                        {DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_DST, zp_c_mem}});
        s.wait();
        const std::vector<uint8_t> c = read_from<uint8_t>(c_mem, M * N);

        long bad = 0;
        for (memory::dim m = 0; m < M; ++m)
            for (memory::dim n = 0; n < N; ++n) {
                int32_t acc = 0;
                for (memory::dim k = 0; k < K; ++k) acc += ((int32_t)a[m * K + k] - zp_a) * (int32_t)b[k * N + n];
                volatile float d = (float)acc; // (volatile: one rounding per written operation on any host compiler)
                d = d * sc_a;
                d = d * sc_b[n];
                d = d > 0.f ? d : 0.f;
                d = d / sc_c;
                d = d + (float)zp_c;
                float q = d < 0.f ? 0.f : (d > 255.f ? 255.f : d);
                const uint8_t want = (uint8_t)std::nearbyintf(q);
                if (c[m * N + n] != want) ++bad;
            }
        if (bad) {
            std::fprintf(stderr, "int8: %ld of %ld elements differ\n", bad, (long)(M * N));
            return 5;
        }

        // ---- the generic implementation comes next in the list and gives the same bytes
        matmul::primitive_desc pd2(eng, a_md, memory::desc({K, N}, memory::data_type::s8, memory::format_tag::ab), c_md, attr);
        bool more = false;
        while (std::string(pd2.impl_info_str()) != "hip:ref:any" && (more = pd2.next_impl())) {}
        if (std::string(pd2.impl_info_str()) != "hip:ref:any") return 6;
        memory c2_mem(c_md, eng);
        matmul(pd2).execute(s,
                {{DNNL_ARG_SRC, a_mem}, {DNNL_ARG_WEIGHTS, b_user}, {DNNL_ARG_DST, c2_mem},
                        {DNNL_ARG_ATTR_SCALES | DNNL_ARG_SRC, sc_a_mem}, {DNNL_ARG_ATTR_SCALES | DNNL_ARG_WEIGHTS, sc_b_mem},
                        {DNNL_ARG_ATTR_SCALES | DNNL_ARG_DST, sc_c_mem},
                        {DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_SRC, zp_a_mem},
                        {DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_DST, zp_c_mem}});
        s.wait();
        if (read_from<uint8_t>(c2_mem, M * N) != c) return 6;

        // ---- bf16 x bf16 + bias -> f32 on small integers (every sum exact, so any order of additions agrees)
        std::vector<uint16_t> x(M * K), w(K * N);
        std::vector<float> bias(N);
        for (auto &v : x) v = to_bf16((float)((int)(next() % 9) - 4));
        for (auto &v : w) v = to_bf16((float)((int)(next() % 9) - 4));
        for (memory::dim n = 0; n < N; ++n) bias[n] = (float)(n % 5) - 2.f;
        memory::desc x_md({M, K}, memory::data_type::bf16, memory::format_tag::ab);
        memory::desc w_md({K, N}, memory::data_type::bf16, memory::format_tag::ab);
        memory::desc bias_md({1, N}, memory::data_type::f32, memory::format_tag::ab);
        memory::desc y_md({M, N}, memory::data_type::f32, memory::format_tag::ab);
        matmul::primitive_desc pd3(eng, x_md, w_md, bias_md, y_md);
        if (pd3.bias_desc() != bias_md) return 7;
        memory x_mem(x_md, eng), w_mem(w_md, eng), bias_mem(bias_md, eng), y_mem(y_md, eng);
        write_to(x_mem, x);
        write_to(w_mem, w);
        write_to(bias_mem, bias);
        matmul(pd3).execute(s, {{DNNL_ARG_SRC, x_mem}, {DNNL_ARG_WEIGHTS, w_mem}, {DNNL_ARG_BIAS, bias_mem}, {DNNL_ARG_DST, y_mem}});
        s.wait();
        const std::vector<float> y = read_from<float>(y_mem, M * N);
        for (memory::dim m = 0; m < M; ++m)
            for (memory::dim n = 0; n < N; ++n) {
                float acc = 0.f;
                for (memory::dim k = 0; k < K; ++k) acc += from_bf16(x[m * K + k]) * from_bf16(w[k * N + n]);
                if (y[m * N + n] != acc + bias[n]) {
                    std::fprintf(stderr, "bf16: element (%ld, %ld) is %g, not %g\n", (long)m, (long)n, y[m * N + n], acc + bias[n]);
                    return 7;
                }
            }

        std::printf("ok %s, %s\n", impl.c_str(), pd3.impl_info_str());
        return 0;
    } catch (const error &e) {
        std::fprintf(stderr, "dnnl::error: %s (status %d)\n", e.message, (int)e.status);
        return 10;
    }
}
