// Two more of the reference's examples as callers of include/dnnl_amd.hpp on a GPU engine, at their own shapes:
//   examples/primitives/matmul.cpp   batched f32 matmul 3 x (128 x 256) x (256 x 512), bias 1 x 1 x 512, ReLU;
//   examples/primitives/reorder.cpp  f32 -> s8 on a 3 x 3 x 227 x 227 nhwc tensor with a dst scale per channel
//                                    (mask on dim 1, which is the innermost dim in memory).
// The matmul is checked against double-precision loops within the rounding of the f32 sums, the reorder exactly
// against the reference's formula (simple_reorder.hpp:2579-2661: x / scale, saturated, rounded to nearest even).
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
} // namespace

static int matmul_example(const engine &eng, stream &s, std::string &impl) {
    const memory::dim MB = 3, M = 128, K = 256, N = 512;
    std::vector<float> src(MB * M * K), wei(MB * K * N), bias(N);
    for (size_t i = 0; i < src.size(); ++i) src[i] = std::cos((float)i / 10.f);
    for (size_t i = 0; i < wei.size(); ++i) wei[i] = std::sin((float)i * 2.f);
    for (size_t i = 0; i < bias.size(); ++i) bias[i] = std::tanh((float)i);
    memory::desc src_md({MB, M, K}, memory::data_type::f32, memory::format_tag::abc);
    memory::desc wei_md({MB, K, N}, memory::data_type::f32, memory::format_tag::abc);
    memory::desc bias_md({1, 1, N}, memory::data_type::f32, memory::format_tag::abc);
    memory::desc dst_md({MB, M, N}, memory::data_type::f32, memory::format_tag::abc);
    memory src_mem(src_md, eng), wei_mem(wei_md, eng), bias_mem(bias_md, eng), dst_mem(dst_md, eng);
    write_to(src_mem, src);
    write_to(wei_mem, wei);
    write_to(bias_mem, bias);
    post_ops ops;
    ops.append_eltwise(algorithm::eltwise_relu, 0.f, 0.f);
    primitive_attr attr;
    attr.set_post_ops(ops);
    matmul::primitive_desc pd(eng, src_md, wei_md, bias_md, dst_md, attr);
    impl = pd.impl_info_str();
    std::unordered_map<int, memory> args;
    args.insert({DNNL_ARG_SRC, src_mem});
    args.insert({DNNL_ARG_WEIGHTS, wei_mem});
    args.insert({DNNL_ARG_BIAS, bias_mem});
    args.insert({DNNL_ARG_DST, dst_mem});
    matmul(pd).execute(s, args);
    s.wait();
    const std::vector<float> dst = read_from<float>(dst_mem, MB * M * N);
    for (memory::dim b = 0; b < MB; ++b)
        for (memory::dim m = 0; m < M; ++m)
            for (memory::dim n = 0; n < N; ++n) {
                double ref = 0.0, mag = 0.0;
                for (memory::dim k = 0; k < K; ++k) {
                    const double t = (double)src[(b * M + m) * K + k] * (double)wei[(b * K + k) * N + n];
                    ref += t;
                    mag += std::fabs(t);
                }
                ref += bias[n];
                ref = ref > 0.0 ? ref : 0.0;
                if (std::fabs((double)dst[(b * M + m) * N + n] - ref) > (K + 2) * 6e-8 * mag + 1e-6) {
                    std::fprintf(stderr, "matmul: dst(%ld, %ld, %ld) is %g, not %g\n", (long)b, (long)m, (long)n,
                            dst[(b * M + m) * N + n], ref);
                    return 2;
                }
            }
    return 0;
}

static int reorder_example(const engine &eng, stream &s, std::string &impl) {
    const memory::dim N = 3, IC = 3, IH = 227, IW = 227;
    memory::dims dims = {N, IC, IH, IW};
    std::vector<float> src(N * IC * IH * IW), scales(IC);
    for (size_t i = 0; i < src.size(); ++i) src[i] = 100.f * std::cos((float)i / 10.f); // (values that use the s8 range)
    for (memory::dim c = 0; c < IC; ++c) scales[c] = 0.5f + 0.25f * (float)c;
    memory::desc src_md(dims, memory::data_type::f32, memory::format_tag::nhwc);
    memory::desc dst_md(dims, memory::data_type::s8, memory::format_tag::nhwc);
    memory src_mem(src_md, eng), dst_mem(dst_md, eng);
    write_to(src_mem, src);
    primitive_attr attr;
    attr.set_scales_mask(DNNL_ARG_DST, 1 << 1);
    memory scales_mem({{IC}, memory::data_type::f32, memory::format_tag::x}, eng);
    write_to(scales_mem, scales);
    reorder::primitive_desc pd(eng, src_md, eng, dst_md, attr);
    impl = pd.impl_info_str();
    std::unordered_map<int, memory> args;
    args.insert({DNNL_ARG_SRC, src_mem});
    args.insert({DNNL_ARG_DST, dst_mem});
    args.insert({DNNL_ARG_ATTR_SCALES | DNNL_ARG_DST, scales_mem});
    reorder(pd).execute(s, args);
    s.wait();
    const std::vector<int8_t> dst = read_from<int8_t>(dst_mem, src.size());
    for (size_t i = 0; i < src.size(); ++i) {
        volatile float d = src[i] / scales[i % IC]; // nhwc: the channel is the innermost index
        const float c = d < -128.f ? -128.f : (d > 127.f ? 127.f : d);
        if ((float)dst[i] != std::nearbyintf(c)) {
            std::fprintf(stderr, "reorder: element %ld (%g / %g) became %d\n", (long)i, src[i], scales[i % IC], (int)dst[i]);
            return 3;
        }
    }
    return 0;
}

int main() {
    try {
        engine eng(engine::kind::gpu, 0);
        stream s(eng);
        std::string impl1, impl2;
        if (int rc = matmul_example(eng, s, impl1)) return rc;
        if (int rc = reorder_example(eng, s, impl2)) return rc;
        std::printf("ok %s, %s\n", impl1.c_str(), impl2.c_str());
        return 0;
    } catch (const error &e) {
        std::fprintf(stderr, "dnnl::error: %s (status %d)\n", e.message, (int)e.status);
        return 10;
    }
}
