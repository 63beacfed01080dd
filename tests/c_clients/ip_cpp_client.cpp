// The reference's inner-product example (examples/primitives/inner_product.cpp) as a caller of include/dnnl_amd.hpp
// on a GPU engine, same shapes: src 3 x 3 x 227 x 227 in nhwc, the user's weights 96 x 3 x 227 x 227 in oihw handed to
// the primitive as format_tag::any (it answers with the channels-last order of src, so the example's "reorder if the
// descriptors differ" branch runs), bias, ReLU, f32 everywhere; then the two backward primitives on the same
// tensors.  Checked against double-precision loops on the host within the rounding of K f32 additions.
#include <cmath>
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

int main() {
    try {
        engine eng(engine::kind::gpu, 0);
        stream s(eng);
        const memory::dim N = 3, IC = 3, IH = 227, IW = 227, OC = 96, SP = IH * IW, K = IC * SP;
        memory::dims src_dims = {N, IC, IH, IW}, weights_dims = {OC, IC, IH, IW}, bias_dims = {OC}, dst_dims = {N, OC};
        // values by logical index (n / o, c, h, w), as the example generates them by position in its arrays
        std::vector<float> src_nhwc(N * K), wei_oihw(OC * K), bias(OC);
        auto src_at = [&](memory::dim n, memory::dim c, memory::dim p) -> float & { return src_nhwc[(n * SP + p) * IC + c]; };
        for (memory::dim i = 0; i < N * K; ++i) src_nhwc[i] = std::cos((float)i / 10.f);
        for (memory::dim i = 0; i < OC * K; ++i) wei_oihw[i] = std::sin((float)i * 2.f);
        for (memory::dim i = 0; i < OC; ++i) bias[i] = std::tanh((float)i);

        memory::desc src_md(src_dims, memory::data_type::f32, memory::format_tag::nhwc);
        memory::desc bias_md(bias_dims, memory::data_type::f32, memory::format_tag::a);
        memory::desc dst_md(dst_dims, memory::data_type::f32, memory::format_tag::nc);
        memory src_mem(src_md, eng), bias_mem(bias_md, eng), dst_mem(dst_md, eng);
        memory user_weights_mem({weights_dims, memory::data_type::f32, memory::format_tag::oihw}, eng);
        write_to(src_mem, src_nhwc);
        write_to(bias_mem, bias);
        write_to(user_weights_mem, wei_oihw);

        memory::desc any_weights_md(weights_dims, memory::data_type::f32, memory::format_tag::any);
        post_ops ops;
        ops.append_eltwise(algorithm::eltwise_relu, 0.f, 0.f);
        primitive_attr attr;
        attr.set_post_ops(ops);
        inner_product_forward::primitive_desc pd(
                eng, prop_kind::forward_training, src_md, any_weights_md, bias_md, dst_md, attr);
        const std::string impl = pd.impl_info_str();
        memory weights_mem = user_weights_mem;
        if (pd.weights_desc() != user_weights_mem.get_desc()) {
            weights_mem = memory(pd.weights_desc(), eng);
            reorder(user_weights_mem, weights_mem).execute(s, user_weights_mem, weights_mem);
        } else {
            std::fprintf(stderr, "format_tag::any kept oihw under an nhwc src\n");
            return 2;
        }
        inner_product_forward(pd).execute(
                s, {{DNNL_ARG_SRC, src_mem}, {DNNL_ARG_WEIGHTS, weights_mem}, {DNNL_ARG_BIAS, bias_mem}, {DNNL_ARG_DST, dst_mem}});
        s.wait();
        const std::vector<float> dst = read_from<float>(dst_mem, N * OC);
        for (memory::dim n = 0; n < N; ++n)
            for (memory::dim o = 0; o < OC; ++o) {
                double ref = 0.0, mag = 0.0;
                for (memory::dim c = 0; c < IC; ++c)
                    for (memory::dim p = 0; p < SP; ++p) {
                        const double t = (double)src_at(n, c, p) * (double)wei_oihw[(o * IC + c) * SP + p];
                        ref += t;
                        mag += std::fabs(t);
                    }
                ref += bias[o];
                ref = ref > 0.0 ? ref : 0.0;
                // products rounded once, sums of K terms in f32 in some order: a few sqrt(K) ulps of sum |terms|
                const double tol = 8.0 * std::sqrt((double)K) * 6e-8 * mag + 1e-6;
                if (std::fabs((double)dst[n * OC + o] - ref) > tol) {
                    std::fprintf(stderr, "forward: dst(%ld, %ld) is %g, not %g (tolerance %g)\n", (long)n, (long)o, dst[n * OC + o], ref, tol);
                    return 3;
                }
            }

        // ---- backward by data and by weights on the same tensors (plain layouts, no attributes)
        std::vector<float> ddst(N * OC);
        for (memory::dim i = 0; i < N * OC; ++i) ddst[i] = std::sin((float)i * 0.37f);
        memory ddst_mem(dst_md, eng), dsrc_mem(src_md, eng);
        write_to(ddst_mem, ddst);
        inner_product_forward::primitive_desc fwd_hint(eng, prop_kind::forward_training, src_md, pd.weights_desc(), bias_md, dst_md);
        inner_product_backward_data::primitive_desc bd_pd(eng, src_md, pd.weights_desc(), dst_md, fwd_hint);
        inner_product_backward_data(bd_pd).execute(
                s, {{DNNL_ARG_DIFF_DST, ddst_mem}, {DNNL_ARG_WEIGHTS, weights_mem}, {DNNL_ARG_DIFF_SRC, dsrc_mem}});
        memory dwei_mem(pd.weights_desc(), eng), dbias_mem(bias_md, eng);
        inner_product_backward_weights::primitive_desc bw_pd(eng, src_md, pd.weights_desc(), bias_md, dst_md, fwd_hint);
        inner_product_backward_weights(bw_pd).execute(s,
                {{DNNL_ARG_SRC, src_mem}, {DNNL_ARG_DIFF_DST, ddst_mem}, {DNNL_ARG_DIFF_WEIGHTS, dwei_mem},
                        {DNNL_ARG_DIFF_BIAS, dbias_mem}});
        s.wait();
        const std::vector<float> dsrc = read_from<float>(dsrc_mem, N * K), dwei = read_from<float>(dwei_mem, OC * K);
        const std::vector<float> dbias = read_from<float>(dbias_mem, OC);
        // diff_src(n, c, p) = sum_o diff_dst(n, o) w(o, c, p); diff_weights(o, c, p) = sum_n diff_dst(n, o) src(n, c, p):
        // both tensors lie channels-last (p outer, c inner) like src; a sample of positions, every n / o
        for (memory::dim p = 0; p < SP; p += 97)
            for (memory::dim c = 0; c < IC; ++c) {
                for (memory::dim n = 0; n < N; ++n) {
                    double ref = 0.0, mag = 0.0;
                    for (memory::dim o = 0; o < OC; ++o) {
                        const double t = (double)ddst[n * OC + o] * (double)wei_oihw[(o * IC + c) * SP + p];
                        ref += t;
                        mag += std::fabs(t);
                    }
                    if (std::fabs((double)dsrc[(n * SP + p) * IC + c] - ref) > 100 * 6e-8 * mag + 1e-7) {
                        std::fprintf(stderr, "backward data: (%ld, %ld, %ld) is %g, not %g\n", (long)n, (long)c, (long)p,
                                dsrc[(n * SP + p) * IC + c], ref);
                        return 4;
                    }
                }
                for (memory::dim o = 0; o < OC; ++o) {
                    double ref = 0.0, mag = 0.0;
                    for (memory::dim n = 0; n < N; ++n) {
                        const double t = (double)ddst[n * OC + o] * (double)src_at(n, c, p);
                        ref += t;
                        mag += std::fabs(t);
                    }
                    if (std::fabs((double)dwei[(o * SP + p) * IC + c] - ref) > 10 * 6e-8 * mag + 1e-7) {
                        std::fprintf(stderr, "backward weights: (%ld, %ld, %ld) is %g, not %g\n", (long)o, (long)c, (long)p,
                                dwei[(o * SP + p) * IC + c], ref);
                        return 5;
                    }
                }
            }
        for (memory::dim o = 0; o < OC; ++o) {
            double ref = 0.0;
            for (memory::dim n = 0; n < N; ++n) ref += ddst[n * OC + o];
            if (std::fabs((double)dbias[o] - ref) > 1e-6) {
                std::fprintf(stderr, "diff_bias(%ld) is %g, not %g\n", (long)o, dbias[o], ref);
                return 6;
            }
        }
        std::printf("ok %s, %s, %s\n", impl.c_str(), bd_pd.impl_info_str(), bw_pd.impl_info_str());
        return 0;
    } catch (const error &e) {
        std::fprintf(stderr, "dnnl::error: %s (status %d)\n", e.message, (int)e.status);
        return 10;
    }
}
