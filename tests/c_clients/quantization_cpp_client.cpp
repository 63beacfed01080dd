// The reference's dynamic-quantization tutorial (examples/tutorials/matmul/cpu_matmul_quantization.cpp) on a GPU
// engine through include/dnnl_amd.hpp: an f32 matmul; the same product with A quantized to u8 (scale and zero point)
// and B to s8 (scale) by reorders whose quantization parameters arrive at execution, an int8 matmul that takes those
// parameters as src / weights scales and src zero point, and the f32 result quantized to u8 by a third reorder.
// (The tutorial hands host vectors to a CPU engine as memory handles; here the data goes through map / unmap.)
// Checked on the host: the reorders against the reference's formula (simple_reorder.hpp:2579-2661:
// x / scale + zp, saturated, rounded to nearest even), the int8 matmul exactly against the integer sum of what the
// reorders produced, and against the f32 matmul within the bound the two quantization steps imply.
#include <algorithm>
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
template <typename T>
memory scalar(const engine &eng, memory::data_type dt, T value) {
    memory m({{1}, dt, {1}}, eng);
    write_to(m, std::vector<T> {value});
    return m;
}
unsigned seed = 5u;
float unit() {
    seed = seed * 1664525u + 1013904223u;
    return (float)((seed >> 12) & 0xffff) / 65536.f;
}

// f32 -> integer by a reorder with the dst scale (and zero point) as execution arguments
void quantize(const engine &eng, stream &s, const memory &x_f32, memory &x_int, float scale, int32_t zp, bool with_zp) {
    primitive_attr attr;
    attr.set_scales_mask(DNNL_ARG_DST, 0);
    if (with_zp) attr.set_zero_points_mask(DNNL_ARG_DST, 0);
    reorder::primitive_desc pd(eng, x_f32.get_desc(), eng, x_int.get_desc(), attr);
    std::unordered_map<int, memory> args = {{DNNL_ARG_FROM, x_f32}, {DNNL_ARG_TO, x_int},
            {DNNL_ARG_ATTR_SCALES | DNNL_ARG_DST, scalar<float>(eng, memory::data_type::f32, scale)}};
    if (with_zp) args.insert({DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_DST, scalar<int32_t>(eng, memory::data_type::s32, zp)});
    reorder(pd).execute(s, args);
    s.wait();
}
float quantized(float x, float scale, int32_t zp, float lo, float hi) {
    volatile float d = x / scale;
    d = d + (float)zp;
    const float c = d < lo ? lo : (d > hi ? hi : d);
    return std::nearbyintf(c);
}
} // namespace

int main() {
    try {
        const memory::dim M = 10, N = 20, K = 30;
        engine eng(engine::kind::gpu, 0);
        stream s(eng);
        std::vector<float> A(M * K), B(K * N);
        for (auto &v : A) v = 6.f * unit() - 1.f;  // an asymmetric range: u8 with a zero point
        for (auto &v : B) v = 4.f * unit() - 2.f;  // symmetric: s8, zero point 0
        memory::desc a_md({M, K}, memory::data_type::f32, {K, 1}), b_md({K, N}, memory::data_type::f32, {N, 1});
        memory::desc c_md({M, N}, memory::data_type::f32, {N, 1});
        memory a_mem(a_md, eng), b_mem(b_md, eng), c_mem(c_md, eng);
        write_to(a_mem, A);
        write_to(b_mem, B);

        // ---- f32 reference on the device
        matmul::primitive_desc f32_pd(eng, a_md, b_md, c_md);
        matmul(f32_pd).execute(s, {{DNNL_ARG_SRC, a_mem}, {DNNL_ARG_WEIGHTS, b_mem}, {DNNL_ARG_DST, c_mem}});
        s.wait();
        const std::vector<float> C = read_from<float>(c_mem, M * N);

        // ---- quantization parameters from the data, as the tutorial computes them
        const float a_min = *std::min_element(A.begin(), A.end()), a_max = *std::max_element(A.begin(), A.end());
        float b_amax = 0.f;
        for (float v : B) b_amax = std::max(b_amax, std::fabs(v));
        const float scale_A = (a_max - a_min) / 255.f, scale_B = b_amax / 127.f;
        const int32_t zp_A = (int32_t)std::nearbyintf(0.f - a_min / scale_A);

        memory a_u8({{M, K}, memory::data_type::u8, {K, 1}}, eng), b_s8({{K, N}, memory::data_type::s8, {N, 1}}, eng);
        quantize(eng, s, a_mem, a_u8, scale_A, zp_A, true);
        quantize(eng, s, b_mem, b_s8, scale_B, 0, false);
        const std::vector<uint8_t> Aq = read_from<uint8_t>(a_u8, M * K);
        const std::vector<int8_t> Bq = read_from<int8_t>(b_s8, K * N);
        for (memory::dim i = 0; i < M * K; ++i)
            if ((float)Aq[i] != quantized(A[i], scale_A, zp_A, 0.f, 255.f)) {
                std::fprintf(stderr, "reorder to u8: %g became %d\n", A[i], (int)Aq[i]);
                return 2;
            }
        for (memory::dim i = 0; i < K * N; ++i)
            if ((float)Bq[i] != quantized(B[i], scale_B, 0, -128.f, 127.f)) {
                std::fprintf(stderr, "reorder to s8: %g became %d\n", B[i], (int)Bq[i]);
                return 2;
            }

        // ---- the int8 matmul, its quantization parameters given at execution
        primitive_attr attr;
        attr.set_scales_mask(DNNL_ARG_SRC, 0);
        attr.set_scales_mask(DNNL_ARG_WEIGHTS, 0);
        attr.set_zero_points_mask(DNNL_ARG_SRC, 0);
        matmul::primitive_desc q_pd(eng, a_u8.get_desc(), b_s8.get_desc(), c_md, attr);
        const std::string impl = q_pd.impl_info_str();
        memory cq_mem(c_md, eng);
        matmul(q_pd).execute(s,
                {{DNNL_ARG_SRC, a_u8}, {DNNL_ARG_WEIGHTS, b_s8}, {DNNL_ARG_DST, cq_mem},
                        {DNNL_ARG_ATTR_SCALES | DNNL_ARG_SRC, scalar<float>(eng, memory::data_type::f32, scale_A)},
                        {DNNL_ARG_ATTR_SCALES | DNNL_ARG_WEIGHTS, scalar<float>(eng, memory::data_type::f32, scale_B)},
                        {DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_SRC, scalar<int32_t>(eng, memory::data_type::s32, zp_A)}});
        s.wait();
        const std::vector<float> Cq = read_from<float>(cq_mem, M * N);
        float a_amax = std::max(std::fabs(a_min), std::fabs(a_max));
        for (memory::dim m = 0; m < M; ++m)
            for (memory::dim n = 0; n < N; ++n) {
                int32_t acc = 0;
                for (memory::dim k = 0; k < K; ++k) acc += ((int32_t)Aq[m * K + k] - zp_A) * (int32_t)Bq[k * N + n];
                volatile float d = (float)acc;
                d = d * scale_A;
                d = d * scale_B;
                if (Cq[m * N + n] != d) {
                    std::fprintf(stderr, "int8 matmul: element (%ld, %ld) is %g, not %g\n", (long)m, (long)n, Cq[m * N + n], (float)d);
                    return 3;
                }
                // half a step of each operand per product (+ the f32 sums of the reference)
                const float bound = (float)K * (a_amax * scale_B / 2 + b_amax * scale_A / 2 + scale_A * scale_B / 4) + 1e-4f;
                if (std::fabs(Cq[m * N + n] - C[m * N + n]) > bound) {
                    std::fprintf(stderr, "quantized %g against f32 %g exceeds %g\n", Cq[m * N + n], C[m * N + n], bound);
                    return 4;
                }
            }

        // ---- and the result to u8
        const float c_min = *std::min_element(Cq.begin(), Cq.end()), c_max = *std::max_element(Cq.begin(), Cq.end());
        const float scale_C = (c_max - c_min) / 255.f;
        const int32_t zp_C = (int32_t)std::nearbyintf(0.f - c_min / scale_C);
        memory c_u8({{M, N}, memory::data_type::u8, {N, 1}}, eng);
        quantize(eng, s, cq_mem, c_u8, scale_C, zp_C, true);
        const std::vector<uint8_t> Cu = read_from<uint8_t>(c_u8, M * N);
        for (memory::dim i = 0; i < M * N; ++i)
            if ((float)Cu[i] != quantized(Cq[i], scale_C, zp_C, 0.f, 255.f)) {
                std::fprintf(stderr, "reorder of the result: %g became %d\n", Cq[i], (int)Cu[i]);
                return 5;
            }
        std::printf("ok %s\n", impl.c_str());
        return 0;
    } catch (const error &e) {
        std::fprintf(stderr, "dnnl::error: %s (status %d)\n", e.message, (int)e.status);
        return 10;
    }
}
