// Host side of the drop-in: the subset of oneDNN's C API that the matmul
// primitive needs (include/dnnl_amd.h), implemented over the thin C ABI of the
// HIP kernels (include/mi355_matmul.h).  No HIP headers here: device memory,
// streams and launches all go through mi355_* calls.
//
// What is restated from the reference (uxlfoundation/oneDNN v3.14):
//   matmul_desc_init            src/common/matmul.cpp:630-744   (shape rules)
//   matmul_attr_check           src/common/matmul.cpp:261-624   (attribute legality)
//   matmul_pd_t::attr_*_ok      src/common/matmul_pd.hpp:209-397
//   attribute setters' checks   src/common/primitive_attr.cpp:623-720
//   default_accum_data_type     src/common/type_helpers.hpp:515-551
//   pd iteration / next_impl    src/common/primitive_desc_iterator.hpp:37-95
//   execute-argument mapping    src/common/primitive_iface.cpp:244-274,
//                               src/common/matmul_pd.hpp:74-93
// Validation failures return dnnl_invalid_arguments, legal-but-unsupported
// requests dnnl_unimplemented, device failures dnnl_runtime_error, as there.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/dnnl_amd.h"
#include "../../include/mi355_matmul.h"

#define DNNL_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

using dim_t = dnnl_dim_t;

int verbose_level() {
    static int lvl = [] {
        const char *e = getenv("ONEDNN_VERBOSE");
        if (!e) e = getenv("DNNL_VERBOSE");
        if (!e) return 0;
        if (!strcmp(e, "all") || !strcmp(e, "profile") || !strcmp(e, "profile_exec")) return 2;
        return atoi(e);
    }();
    return lvl;
}

dnnl_status_t from_mi355(int st) {
    switch (st) {
        case MI355_SUCCESS: return dnnl_success;
        case MI355_OUT_OF_MEMORY: return dnnl_out_of_memory;
        case MI355_INVALID_ARGUMENTS: return dnnl_invalid_arguments;
        case MI355_UNIMPLEMENTED: return dnnl_unimplemented;
        default: return dnnl_runtime_error;
    }
}

bool dt_valid(int dt) {
    return (dt >= dnnl_f16 && dt <= dnnl_f4_e2m1 && dt != dnnl_f64 && dt != dnnl_boolean) || dt == dnnl_s64;
}
int dt_bits(int dt) {
    switch (dt) {
        case dnnl_f32:
        case dnnl_s32: return 32;
        case dnnl_f16:
        case dnnl_bf16: return 16;
        case dnnl_s4:
        case dnnl_u4:
        case dnnl_f4_e2m1: return 4;
        case dnnl_s64:
        case dnnl_f64: return 64;
        default: return 8;
    }
}
bool is_int_dt(int dt) { return dt == dnnl_s8 || dt == dnnl_u8 || dt == dnnl_s4 || dt == dnnl_u4 || dt == dnnl_s32; }
bool is_int8(int dt) { return dt == dnnl_s8 || dt == dnnl_u8; }
bool is_fp8(int dt) { return dt == dnnl_f8_e4m3 || dt == dnnl_f8_e5m2; }
const char *dt_name(int dt) {
    static const char *n[] = {"undef", "f16", "bf16", "f32", "s32", "s8", "u8", "f64", "bool", "f8_e5m2",
            "f8_e4m3", "s4", "u4", "e8m0", "f4_e2m1"};
    return (dt >= 0 && dt <= 14) ? n[dt] : "?";
}

} // namespace

// ------------------------------------------------------------------ objects
struct dnnl_engine {
    dnnl_engine_kind_t kind;
    size_t index;
};

struct dnnl_stream {
    dnnl_engine_t engine;
    void *hip_stream;
    bool owned = true; // false: the caller's stream (dnnl_amd_interop_stream_create), never destroyed here
};

struct dnnl_memory_desc {
    int ndims = 0;
    dnnl_dims_t dims = {};
    dnnl_dims_t strides = {};
    dnnl_data_type_t dt = dnnl_data_type_undef;
    dnnl_format_kind_t kind = dnnl_format_kind_undef;
    // kind == dnnl_format_kind_opaque: the weights packing (MI355_WEI_PACK_*)
    // that format_tag::any resolved to; strides are meaningless then
    int packing = 0;
    // kind == dnnl_format_kind_sparse: the grouped encoding (memory_desc.cpp:417-472) -- a 2-D tensor that
    // concatenates `group_count` sub-tensors along dims[var_dim], the variable dim outermost in memory
    // (strides say so); a second buffer holds the groups' cumulative ends (s32)
    bool grouped = false;
    int var_dim = 0;
    dim_t group_count = 0;

    bool is_zero() const { return ndims == 0; }
    // a dim or a stride left open until execution (memory_desc_wrapper::has_runtime_dims_or_strides)
    bool has_runtime() const {
        for (int i = 0; i < ndims; ++i)
            if (dims[i] == DNNL_RUNTIME_DIM_VAL || (kind == dnnl_blocked && strides[i] == DNNL_RUNTIME_DIM_VAL)) return true;
        return false;
    }
    dim_t nelems() const {
        if (ndims == 0) return 0;
        dim_t n = 1;
        for (int i = 0; i < ndims; ++i) n *= dims[i];
        return n;
    }
    // logical elements the buffer spans (last offset + 1)
    dim_t span() const {
        if (ndims == 0 || nelems() == 0) return 0;
        dim_t off = 0;
        for (int i = 0; i < ndims; ++i) off += (dims[i] - 1) * strides[i];
        return off + 1;
    }
    size_t size_bytes() const {
        if (has_runtime()) return DNNL_RUNTIME_SIZE_VAL; // memory_desc_wrapper::size, src/common/memory.cpp:62
        if (kind == dnnl_format_kind_opaque) return (size_t)nelems() * dt_bits(dt) / 8; // dense, no padding
        if (grouped) return ((size_t)nelems() * dt_bits(dt) + 7) / 8;                  // the values buffer
        const dim_t s = span();
        return dt_bits(dt) == 4 ? (size_t)(s + 1) / 2 : (size_t)s * (dt_bits(dt) / 8);
    }
    // dense strides in the given order of dims (perm[ndims-1] innermost); a
    // stride outside a runtime dim is a runtime value itself
    // (memory_desc_init_by_strides, src/common/memory_desc.cpp:298-308, :838-845)
    void set_dense(const int *perm = nullptr) {
        dim_t s = 1;
        for (int i = ndims - 1; i >= 0; --i) {
            const int d = perm ? perm[i] : i;
            strides[d] = s;
            if (s == DNNL_RUNTIME_DIM_VAL || dims[d] == DNNL_RUNTIME_DIM_VAL)
                s = DNNL_RUNTIME_DIM_VAL;
            else
                s *= dims[d] == 0 ? 1 : dims[d];
        }
        kind = dnnl_blocked;
    }
    bool operator==(const dnnl_memory_desc &o) const {
        if (ndims != o.ndims || dt != o.dt || kind != o.kind || packing != o.packing) return false;
        if (grouped != o.grouped || (grouped && (var_dim != o.var_dim || group_count != o.group_count))) return false;
        for (int i = 0; i < ndims; ++i)
            if (dims[i] != o.dims[i] || (kind == dnnl_blocked && strides[i] != o.strides[i])) return false;
        return true;
    }
};

struct dnnl_memory {
    dnnl_memory_desc md;
    dnnl_engine_t engine;
    void *handle = nullptr;
    bool owned = false;
    void *mapped = nullptr; // host staging buffer while mapped
    // grouped encoding: buffer 1, the offsets
    void *handle2 = nullptr;
    bool owned2 = false;
    void *mapped2 = nullptr;
    unsigned char scalar[8] = {}; // md.kind == dnnl_format_kind_host_scalar: the value
};

namespace {
struct quant_entry_t {
    int mask = 0;
    dnnl_data_type_t dt = dnnl_data_type_undef;
    int group_ndims = 0;
    dim_t groups[2] = {1, 1};
    dim_t group(int d) const { return group_ndims == 0 ? 1 : groups[d]; }
    dnnl_quantization_mode_t qmode = dnnl_quantization_mode_static_sazp;
    bool on_host = false; // the single value is handed over in a host-scalar memory object
    bool is_mx() const { return qmode == dnnl_quantization_mode_dynamic_mx; }
    bool is_dynamic_fp() const { return qmode == dnnl_quantization_mode_dynamic_fp; }
    bool is_dynamic() const { return is_mx() || is_dynamic_fp(); }
};

struct post_op_entry_t {
    dnnl_primitive_kind_t kind = dnnl_undefined_primitive;
    dnnl_alg_kind_t alg = dnnl_alg_kind_undef;
    float alpha = 0.f, beta = 0.f, scale = 1.f;
    int32_t zero_point = 0;
    dnnl_data_type_t dt = dnnl_data_type_undef;
    dnnl_memory_desc src1;
    dnnl_memory_desc src2; // binary select: the condition
    int mask = 0;
};
} // namespace

struct dnnl_post_ops {
    std::vector<post_op_entry_t> entries;
};

struct dnnl_primitive_attr {
    std::map<int, quant_entry_t> scales, zero_points, reductions;
    dnnl_fpmath_mode_t fpmath = dnnl_fpmath_mode_strict;
    int apply_to_int = 0;
    dnnl_accumulation_mode_t acc_mode = dnnl_accumulation_mode_strict;
    dnnl_scratchpad_mode_t scratchpad_mode = dnnl_scratchpad_mode_library;
    dnnl_post_ops post_ops;
    // dropout_t (src/common/primitive_attr.hpp:185-218): set <=> seed_dt != undef
    dnnl_memory_desc dropout_md;
    dnnl_data_type_t dropout_seed_dt = dnnl_data_type_undef;
    int dropout_use_offset = 0, dropout_host_scalars = 0;
    std::map<int, dnnl_rounding_mode_t> rounding;
    bool with_dropout() const { return dropout_seed_dt != dnnl_data_type_undef; }
    const quant_entry_t *find(const std::map<int, quant_entry_t> &m, int arg) const {
        auto it = m.find(arg);
        return it == m.end() ? nullptr : &it->second;
    }
};

struct dnnl_primitive_desc {
    dnnl_primitive_kind_t kind = dnnl_matmul;
    mi355_reorder_desc_t rdesc; // kind == dnnl_reorder (src / dst hold the two tensors)
    dnnl_engine_t engine = nullptr;
    dnnl_memory_desc src, wei, bias, dst, scratchpad;
    bool with_bias = false;
    dnnl_primitive_attr attr;
    mi355_matmul_desc_t desc;     // impl field = the chosen kernel family
    bool grouped = false;         // grouped (mixture-of-experts) matmul: `gdesc` instead of `desc`
    // inner product: lowered and executed as the matmul [mb, K] x [K, oc] (src, wei, bias, dst and attr above
    // describe that matmul); these are the tensors and the attributes the caller gave and reads back
    bool inner_product = false;
    int prop_kind = 96;           // dnnl_forward_inference
    dnnl_memory_desc ip_src, ip_wei, ip_bias;
    dnnl_primitive_attr ip_attr;
    // inner product backward: dnnl_backward_data (diff_src = diff_dst x weights) or dnnl_backward_weights
    // (diff_weights = diff_dst^T x src, diff_bias = column sums of diff_dst) lowered to a matmul whose src / weights
    // / dst are other execute arguments; ip_src / ip_wei / ip_bias / ip_dst hold (diff_)src, (diff_)weights,
    // diff_bias and diff_dst as the caller describes them
    dnnl_memory_desc ip_dst;
    bool ip_diff_bias = false;
    // scaled dot-product attention (kind == dnnl_amd_sdpa): dst = softmax(scale * Q K + mask) V as two batched
    // matmuls around a row-softmax kernel; the scores and the probabilities live in the primitive's scratchpad
    struct sdpa_t {
        dnnl_memory_desc q, k, v, dst, mask, scale;
        dnnl_memory_desc scores, probs; // dense [b][h][sq][sk]: f32, and the values' type
        bool invert_scale = false, inf_as_zero = false;
        int mask_type = 0;
        std::shared_ptr<dnnl_primitive_desc> kq, vs;
    };
    std::shared_ptr<sdpa_t> sdpa;
    mi355_grouped_desc_t gdesc;
    std::vector<int> impls;       // kernel families that can run it, best first
    size_t impl_pos = 0;
    size_t scratch_bytes = 0;
    std::string impl_name;
    // some dim or stride is DNNL_RUNTIME_DIM_VAL: the descriptor is validated
    // as far as the known values allow, and lowered and dispatched at each
    // execution from the descriptors of the memory objects
    // (exec_ctx_t::memory_mdw, src/common/primitive_exec_types.hpp:112-186)
    bool runtime = false;
    // Batch dims that do not collapse into one stride per tensor (a tensor
    // broadcast over some batch dims only): the leading `outer_n` batch dims
    // are walked on the host, one launch per index, with these element
    // strides; the remaining ones form the batch of a launch.
    // post-op slot of the lowered descriptor -> index of the attribute's post-op and the execute argument it
    // takes (a binary select lowers to two slots: the select with src1, then its condition with src2)
    int po_entry[MI355_MAX_POST_OPS] = {};
    int po_arg_id[MI355_MAX_POST_OPS] = {};
    int outer_n = 0;
    dim_t outer_dims[DNNL_MAX_NDIMS] = {};
    dim_t outer_src[DNNL_MAX_NDIMS] = {}, outer_wei[DNNL_MAX_NDIMS] = {}, outer_dst[DNNL_MAX_NDIMS] = {},
          outer_bias[DNNL_MAX_NDIMS] = {};
    dim_t outer_po[MI355_MAX_POST_OPS][DNNL_MAX_NDIMS] = {};
};

struct dnnl_primitive {
    dnnl_primitive_desc pd;
    dnnl_primitive *sdpa_kq = nullptr, *sdpa_vs = nullptr; // the two matmuls of an attention primitive
    void *scratch = nullptr; // library-mode scratchpad (device)
    std::mutex scratch_mutex;
    // runtime dims: the lowering of the last executed shapes, and the scratch
    // buffers allocated for executions so far (kept until the primitive is
    // destroyed: earlier launches may still be running on their stream)
    // device copies of host-side scalar scales / zero points, refreshed in stream order at each execution
    void *host_scalars = nullptr;
    std::unique_ptr<dnnl_primitive_desc> rt_pd;
    std::vector<void *> rt_scratch;
    size_t rt_scratch_bytes = 0;
    // Executions that use the primitive's own device memory (library-mode
    // scratchpad, host-scalar slots, runtime-dims scratch) are ordered on the
    // device as well as on the host: each records `order_event` behind its
    // launches, and the next one on another stream makes its stream wait for it.
    void *order_event = nullptr;
    void *last_stream = nullptr;
    bool event_recorded = false;
    ~dnnl_primitive() {
        delete sdpa_kq;
        delete sdpa_vs;
        if (scratch) mi355_mem_free(scratch);
        for (void *q : rt_scratch) mi355_mem_free(q);
        if (host_scalars) mi355_mem_free(host_scalars);
        if (order_event) mi355_event_destroy(order_event);
    }
};

namespace {

#define CHECK_ARG(cond) \
    do { \
        if (!(cond)) return dnnl_invalid_arguments; \
    } while (0)
// ONEDNN_AMD_TRACE_UNIMPL=1 names the rule that refused a descriptor (stderr)
static const bool g_trace_unimpl = getenv("ONEDNN_AMD_TRACE_UNIMPL") != nullptr;
#define CHECK_UNIMPL(cond) \
    do { \
        if (!(cond)) { \
            if (g_trace_unimpl) fprintf(stderr, "onednn_amd: unimplemented at %s:%d: !(%s)\n", __FILE__, __LINE__, #cond); \
            return dnnl_unimplemented; \
        } \
    } while (0)
#define IMPLICATION(a, b) (!(a) || (b))

// ------------------------------------------------------------ validation
// matmul_desc_init, src/common/matmul.cpp:630-744
dnnl_status_t check_shapes(const dnnl_memory_desc &s, const dnnl_memory_desc &w, const dnnl_memory_desc *b,
        const dnnl_memory_desc &d) {
    const int nd = d.ndims;
    CHECK_ARG(nd >= 2 && nd <= DNNL_MAX_NDIMS);
    CHECK_ARG(s.ndims == nd && w.ndims == nd);
    CHECK_ARG(IMPLICATION(b, b->ndims == nd));
    const int mi = nd - 2, ni = nd - 1;
    CHECK_ARG(d.dims[mi] == s.dims[mi]);
    CHECK_ARG(d.dims[ni] == w.dims[ni]);
    CHECK_ARG(s.dims[ni] == w.dims[mi]);
    if (b) {
        CHECK_ARG(b->dims[ni] == 1 || b->dims[ni] == d.dims[ni]);
        CHECK_ARG(b->dims[mi] == 1 || b->dims[mi] == d.dims[mi]);
    }
    for (int i = 0; i < nd - 2; ++i) {
        const dim_t sd = s.dims[i], wd = w.dims[i], dd = d.dims[i];
        const dim_t R = DNNL_RUNTIME_DIM_VAL;
        if (sd == R || wd == R || dd == R || (b && b->dims[i] == R)) {
            // a runtime batch dim is runtime in every tensor that has it (matmul.cpp:716-721)
            CHECK_ARG(sd == R && wd == R && dd == R);
            if (b) CHECK_ARG(b->dims[i] == 1 || b->dims[i] == R);
            continue;
        }
        const bool all_eq = sd == wd && wd == dd;
        CHECK_ARG(IMPLICATION(!all_eq, sd == 1 || wd == 1));
        CHECK_ARG(IMPLICATION(sd == 1, dd == wd));
        CHECK_ARG(IMPLICATION(wd == 1, dd == sd));
        if (b) CHECK_ARG(b->dims[i] == 1 || b->dims[i] == dd);
    }
    return dnnl_success;
}

// default_accum_data_type, src/common/type_helpers.hpp:515-551 (forward)
int accum_dt(int src, int wei, int dst) {
    (void)dst;
    if (is_int8(src) && (is_int8(wei) || wei == dnnl_s4 || wei == dnnl_u4)) return dnnl_s32;
    if (src == dnnl_f64) return dnnl_f64;
    return dnnl_f32;
}

// Stand-in for a runtime dim while the attributes of a descriptor with runtime
// dims are checked at creation: divisible by every power-of-two group, like
// DNNL_RUNTIME_DIM_VAL itself in the reference's checks.  The checks run again
// on the real dims at execution.
const dim_t k_probe_dim = (dim_t)1 << 40;

// matmul_attr_check (src/common/matmul.cpp:261-624) plus the generic checks of
// matmul_pd_t::attr_scales_ok / attr_zero_points_ok (matmul_pd.hpp:209-397)
dnnl_status_t check_attr(const dnnl_memory_desc &s, const dnnl_memory_desc &w, const dnnl_memory_desc &d,
        const dnnl_primitive_attr &a) {
    const int nd = s.ndims;
    const dim_t M = s.dims[nd - 2], K = w.dims[nd - 2], N = w.dims[nd - 1];
    const int src_dt = s.dt, wei_dt = w.dt, dst_dt = d.dt;
    const bool src_int8 = is_int8(src_dt), src_fp8 = is_fp8(src_dt), src_fp4 = src_dt == dnnl_f4_e2m1;
    const bool wei_int = wei_dt == dnnl_s8 || wei_dt == dnnl_u8 || wei_dt == dnnl_s4 || wei_dt == dnnl_u4;
    const bool wei_lowp = wei_int || is_fp8(wei_dt) || wei_dt == dnnl_f4_e2m1;
    const int qM = 1 << (nd - 2), qK_src = 1 << (nd - 1);
    const int qK_wei = 1 << (nd - 2), qN = 1 << (nd - 1);
    const int full = (1 << nd) - 1;
    auto divisible = [](dim_t g1, dim_t g2) { return IMPLICATION(g1 > 1 && g2 > 1, g1 % g2 == 0 || g2 % g1 == 0); };

    // zero points and precomputed reductions only with low-precision src
    // (weights zero points also serve weight decompression)
    if (!a.zero_points.empty())
        CHECK_UNIMPL(src_int8 || src_fp8 || src_fp4 || wei_int);
    if (!a.reductions.empty()) CHECK_UNIMPL(src_int8);
    for (auto &kv : a.scales)
        CHECK_UNIMPL(kv.first == DNNL_ARG_SRC || kv.first == DNNL_ARG_WEIGHTS || kv.first == DNNL_ARG_DST);
    for (auto &kv : a.zero_points)
        CHECK_UNIMPL(kv.first == DNNL_ARG_SRC || kv.first == DNNL_ARG_WEIGHTS || kv.first == DNNL_ARG_DST);
    for (auto &kv : a.reductions) CHECK_UNIMPL(kv.first == DNNL_ARG_SRC);

    dim_t src_sg_k = 1, wei_sg_k = 1;
    if (auto q = a.find(a.scales, DNNL_ARG_SRC)) {
        CHECK_UNIMPL(q->mask == 0 || q->mask == qM || q->mask == qK_src || q->mask == qM + qK_src
                || q->mask == full);
        if (q->group_ndims && (q->mask & qK_src)) src_sg_k = q->group(1);
        CHECK_UNIMPL(IMPLICATION(src_sg_k > 1 && src_sg_k < K, src_sg_k % 16 == 0));
        // matmul_pd_t::attr_scales_ok
        CHECK_UNIMPL(IMPLICATION(q->mask & qK_src, q->group_ndims != 0));
        CHECK_UNIMPL(IMPLICATION(q->group_ndims, q->group(0) == 1));
        CHECK_UNIMPL(IMPLICATION(q->group_ndims, K % q->group(1) == 0));
        CHECK_UNIMPL(IMPLICATION(q->mask == qM, q->group_ndims == 0));
        CHECK_UNIMPL(!wei_lowp ? q->group_ndims == 0 : true);
    }
    if (auto q = a.find(a.scales, DNNL_ARG_WEIGHTS)) {
        dim_t gn = 1;
        if (q->group_ndims) {
            CHECK_UNIMPL(wei_lowp);
            if (q->mask & qK_wei) wei_sg_k = q->group(0);
            if (q->mask & qN) gn = q->group(1);
            CHECK_UNIMPL(IMPLICATION(q->group(0) > 1, K % q->group(0) == 0));
            CHECK_UNIMPL(IMPLICATION(q->group(1) > 1, N % q->group(1) == 0));
        }
        CHECK_UNIMPL(IMPLICATION(wei_sg_k > 1 && wei_sg_k < K, wei_sg_k % 16 == 0));
        CHECK_UNIMPL(IMPLICATION(gn > 1 && gn < N, gn % 16 == 0));
        // a K mask on integer weights only for weight decompression
        if (is_int_dt(wei_dt)) {
            const bool decomp = wei_int && IMPLICATION(!is_int_dt(src_dt), a.apply_to_int);
            CHECK_UNIMPL(IMPLICATION(q->mask & qK_wei, decomp));
        }
    }
    if (auto q = a.find(a.scales, DNNL_ARG_DST)) {
        CHECK_UNIMPL(q->mask == 0 || q->mask == qN || q->mask == qM || q->mask == qM + qN || q->mask == full);
        CHECK_UNIMPL(IMPLICATION(q->group_ndims, is_fp8(dst_dt) || dst_dt == dnnl_f4_e2m1));
        CHECK_UNIMPL(IMPLICATION(q->group_ndims, M % q->group(0) == 0 && N % q->group(1) == 0));
        // dynamic_mx: OCP MX flavour only (matmul.cpp:407-424)
        if (q->is_mx()) {
            CHECK_UNIMPL(q->mask == full);
            CHECK_UNIMPL(q->group_ndims == 2 && q->group(1) == 32 && q->group(0) == 1);
            CHECK_UNIMPL(q->dt == dnnl_e8m0);
        }
        // dynamic_fp: the NVFP4 flavour only, f8_e4m3 scales per 16 (matmul.cpp:423-440)
        if (q->is_dynamic_fp()) {
            CHECK_UNIMPL(q->mask == full);
            CHECK_UNIMPL(q->dt == dnnl_f8_e4m3);
            CHECK_UNIMPL(q->group_ndims == 2 && q->group(1) == 16 && q->group(0) == 1);
        }
    }
    // dynamic quantization is a dst scale mode
    for (int arg : {DNNL_ARG_SRC, DNNL_ARG_WEIGHTS})
        if (auto q = a.find(a.scales, arg)) CHECK_UNIMPL(!q->is_dynamic());
    CHECK_UNIMPL(IMPLICATION(src_sg_k > 1, (src_int8 || src_fp8 || src_fp4) && divisible(src_sg_k, wei_sg_k)));

    dim_t src_zg_k = 1, wei_zg_k = 1;
    if (auto q = a.find(a.zero_points, DNNL_ARG_SRC)) {
        CHECK_UNIMPL(q->mask == 0 || q->mask == qK_src || q->mask == qM + qK_src || q->mask == full);
        CHECK_UNIMPL(IMPLICATION(q->mask == full, nd <= 3));
        CHECK_UNIMPL(IMPLICATION(q->mask == full && nd == 3, s.dims[0] == 1));
        if (q->group_ndims && (q->mask & qK_src)) src_zg_k = q->group(1);
        CHECK_UNIMPL(IMPLICATION(src_zg_k > 1 && src_zg_k < K, src_zg_k % 32 == 0));
        CHECK_UNIMPL(IMPLICATION(q->group_ndims, q->group(0) == 1 && K % q->group(1) == 0));
    }
    if (auto q = a.find(a.zero_points, DNNL_ARG_WEIGHTS)) {
        dim_t gn = 1;
        if (q->group_ndims) {
            CHECK_UNIMPL(wei_lowp);
            if (q->mask & qK_wei) wei_zg_k = q->group(0);
            if (q->mask & qN) gn = q->group(1);
            CHECK_UNIMPL(IMPLICATION(q->group(0) > 1, K % q->group(0) == 0));
            CHECK_UNIMPL(IMPLICATION(q->group(1) > 1, N % q->group(1) == 0));
            CHECK_UNIMPL(q->group(0) == 1 || q->group(1) == 1); // one non-unit group
        }
        CHECK_UNIMPL(IMPLICATION(gn > 1, a.apply_to_int));
        CHECK_UNIMPL(IMPLICATION(wei_zg_k > 1 && wei_zg_k < K, wei_zg_k % 16 == 0));
        CHECK_UNIMPL(IMPLICATION(gn > 1 && gn < N, gn % 16 == 0));
        if (q->dt == dnnl_s4 || q->dt == dnnl_u4) {
            CHECK_UNIMPL(IMPLICATION(q->mask & qK_wei, K % 2 == 0));
            CHECK_UNIMPL(IMPLICATION(q->mask & qN, N % 2 == 0));
        }
        CHECK_UNIMPL(q->dt == dnnl_s32 || wei_lowp); // non-s32 zero-point types need low-precision weights
    }
    if (auto q = a.find(a.zero_points, DNNL_ARG_DST)) {
        CHECK_UNIMPL(q->mask == 0 || (d.ndims == 2 && q->mask == (1 << 1)));
        CHECK_UNIMPL(q->group_ndims == 0);
    }
    CHECK_UNIMPL(IMPLICATION(src_zg_k > 1, src_int8 && divisible(src_zg_k, wei_zg_k)));

    if (auto pr = a.find(a.reductions, DNNL_ARG_SRC)) {
        CHECK_UNIMPL(a.find(a.zero_points, DNNL_ARG_WEIGHTS) != nullptr);
        CHECK_UNIMPL(pr->mask == full);
        CHECK_UNIMPL(pr->dt == dnnl_s32);
        if (pr->group_ndims) {
            const dim_t g = pr->group(1);
            dim_t minimal = INT64_MAX;
            dim_t wzk = 1;
            if (auto q = a.find(a.zero_points, DNNL_ARG_WEIGHTS))
                if (q->group_ndims) { wzk = q->group(0); minimal = std::min(minimal, wzk); }
            if (auto q = a.find(a.zero_points, DNNL_ARG_SRC))
                if (q->group_ndims) minimal = std::min(minimal, q->group(1));
            if (auto q = a.find(a.scales, DNNL_ARG_WEIGHTS))
                if (q->group_ndims) minimal = std::min(minimal, q->group(0));
            if (auto q = a.find(a.scales, DNNL_ARG_SRC))
                if (q->group_ndims) minimal = std::min(minimal, q->group(1));
            CHECK_ARG(IMPLICATION(g > 1, src_int8));
            CHECK_ARG(IMPLICATION(g > 1, divisible(g, wzk)));
            CHECK_ARG(IMPLICATION(g > 1, g <= minimal));
            CHECK_UNIMPL(pr->group(0) == 1 && K % g == 0);
        }
    }

    // post-ops: binary, eltwise, prelu, sum (matmul.cpp:606-620)
    for (auto &e : a.post_ops.entries) {
        CHECK_UNIMPL(e.kind == dnnl_binary || e.kind == dnnl_eltwise || e.kind == dnnl_prelu || e.kind == dnnl_sum);
        if (e.kind == dnnl_sum) {
            // check_sum_consistency: same size as dst, zero point only for int8
            CHECK_UNIMPL(IMPLICATION(e.dt != dnnl_data_type_undef, dt_bits(e.dt) == dt_bits(dst_dt)));
            CHECK_UNIMPL(IMPLICATION(e.zero_point != 0, src_int8));
        }
        if (e.kind == dnnl_binary) CHECK_UNIMPL(!e.src1.grouped); // grouped operands: grouped matmul only
        if (e.kind == dnnl_binary) {
            CHECK_ARG(e.src1.ndims == d.ndims);
            for (int i = 0; i < d.ndims; ++i)
                CHECK_ARG(e.src1.dims[i] == 1 || e.src1.dims[i] == d.dims[i] || d.dims[i] == k_probe_dim);
            if (e.alg == dnnl_binary_select) {
                CHECK_ARG(e.src2.ndims == d.ndims);
                for (int i = 0; i < d.ndims; ++i)
                    CHECK_ARG(e.src2.dims[i] == 1 || e.src2.dims[i] == d.dims[i] || d.dims[i] == k_probe_dim);
                CHECK_UNIMPL(e.src2.dt == dnnl_s8 || e.src2.dt == dnnl_u8 || e.src2.dt == dnnl_s32);
            }
        }
    }
    return dnnl_success;
}

// ------------------------------------------------- lowering to the C ABI
// Collapse the batch dims of one operand into a single stride: all broadcast
// (stride 0) or all present and nested.
bool collapse_batch(const dnnl_memory_desc &x, const dnnl_memory_desc &dst, int64_t *bstride, int first = 0) {
    const int nb = dst.ndims - 2;
    *bstride = 0;
    if (nb - first <= 0) return true;
    bool all_one = true, all_full = true;
    for (int i = first; i < nb; ++i) {
        if (x.dims[i] != 1) all_one = false;
        if (x.dims[i] != dst.dims[i]) all_full = false;
    }
    dim_t total = 1;
    for (int i = first; i < nb; ++i) total *= dst.dims[i];
    if (all_one && total > 1) return true; // broadcast
    if (!all_full) return false;
    // offset = sum b_i * stride_i must equal S * (collapsed batch index): every
    // non-unit dim's stride is S times the extent of the dims after it
    // (a dim of extent 1 may carry any stride)
    dim_t inner = 1;
    bool have = false;
    for (int i = nb - 1; i >= first; --i) {
        if (x.dims[i] != 1) {
            if (!have) {
                if (x.strides[i] % inner) return false;
                *bstride = x.strides[i] / inner;
                have = true;
            } else if (x.strides[i] != *bstride * inner) {
                return false;
            }
        }
        inner *= dst.dims[i];
    }
    if (total == 1) *bstride = 0;
    return true;
}

bool lower_quant(const quant_entry_t *q, int nd, int default_dt, mi355_quant_t *out) {
    out->dt = MI355_DT_UNDEF;
    out->mask = 0;
    out->group[0] = out->group[1] = 1;
    if (!q) return true;
    const int batch_bits = (1 << (nd - 2)) - 1;
    const int bm = q->mask & batch_bits;
    if (bm != 0 && bm != batch_bits) return false; // partial batch masks are not lowered
    out->dt = q->dt == dnnl_data_type_undef ? default_dt : q->dt;
    out->mask = (bm ? 1 : 0) | ((q->mask >> (nd - 2)) & 1) << 1 | ((q->mask >> (nd - 1)) & 1) << 2;
    out->group[0] = q->group(0);
    out->group[1] = q->group(1);
    // a group on an unmasked dim carries no information
    if (!(out->mask & 2)) out->group[0] = 1;
    if (!(out->mask & 4)) out->group[1] = 1;
    return true;
}

dnnl_status_t lower(dnnl_primitive_desc &pd) {
    mi355_matmul_desc_t &D = pd.desc;
    memset(&D, 0, sizeof(D));
    const int nd = pd.dst.ndims;
    // the fewest leading batch dims to walk on the host so that the rest collapse in every tensor
    int first = 0;
    {
        auto collapses = [&](int f) {
            int64_t t;
            if (!collapse_batch(pd.src, pd.dst, &t, f) || !collapse_batch(pd.dst, pd.dst, &t, f)) return false;
            if (pd.wei.kind != dnnl_format_kind_opaque && !collapse_batch(pd.wei, pd.dst, &t, f)) return false;
            if (pd.with_bias && !collapse_batch(pd.bias, pd.dst, &t, f)) return false;
            for (const post_op_entry_t &e : pd.attr.post_ops.entries)
                if (e.kind == dnnl_binary
                        && (!collapse_batch(e.src1, pd.dst, &t, f)
                                || (e.alg == dnnl_binary_select && !collapse_batch(e.src2, pd.dst, &t, f))))
                    return false;
            return true;
        };
        while (first < nd - 2 && !collapses(first)) ++first;
    }
    pd.outer_n = first;
    if (first > 0) {
        // parameters indexed by the batch would need the same walk: not offered
        for (const auto *mp : {&pd.attr.scales, &pd.attr.zero_points, &pd.attr.reductions})
            for (const auto &kv : *mp) CHECK_UNIMPL((kv.second.mask & ((1 << (nd - 2)) - 1)) == 0);
        for (const post_op_entry_t &e : pd.attr.post_ops.entries)
            CHECK_UNIMPL(e.kind != dnnl_prelu || (e.mask & ((1 << (nd - 2)) - 1)) == 0);
        bool whole_bytes = true; // a 4-bit tensor is stepped by whole bytes
        auto outer = [&](const dnnl_memory_desc &x, dim_t *out) {
            for (int i = 0; i < first; ++i) {
                out[i] = x.dims[i] == 1 ? 0 : x.strides[i];
                if (dt_bits(x.dt) == 4 && (out[i] & 1)) whole_bytes = false;
            }
        };
        for (int i = 0; i < first; ++i) pd.outer_dims[i] = pd.dst.dims[i];
        outer(pd.src, pd.outer_src); outer(pd.wei, pd.outer_wei); outer(pd.dst, pd.outer_dst);
        if (pd.with_bias) outer(pd.bias, pd.outer_bias);
        for (const post_op_entry_t &e : pd.attr.post_ops.entries) CHECK_UNIMPL(e.alg != dnnl_binary_select || e.kind != dnnl_binary);
        for (size_t i = 0; i < pd.attr.post_ops.entries.size(); ++i)
            if (pd.attr.post_ops.entries[i].kind == dnnl_binary) outer(pd.attr.post_ops.entries[i].src1, pd.outer_po[i]);
        CHECK_UNIMPL(whole_bytes);
    }
    dim_t batch = 1;
    for (int i = first; i < nd - 2; ++i) batch *= pd.dst.dims[i];
    D.batch = batch;
    D.M = pd.dst.dims[nd - 2];
    D.N = pd.dst.dims[nd - 1];
    D.K = pd.src.dims[nd - 1];
    D.src_dt = pd.src.dt; D.wei_dt = pd.wei.dt; D.dst_dt = pd.dst.dt;
    D.bias_dt = pd.with_bias ? (int)pd.bias.dt : (int)MI355_DT_UNDEF;
    auto strides3 = [&](const dnnl_memory_desc &x, int64_t *out) -> bool {
        if (!collapse_batch(x, pd.dst, &out[0], first)) return false;
        out[1] = x.dims[nd - 2] == 1 && pd.dst.dims[nd - 2] != 1 && &x != &pd.src && &x != &pd.wei ? 0 : x.strides[nd - 2];
        out[2] = x.dims[nd - 1] == 1 && pd.dst.dims[nd - 1] != 1 && &x != &pd.src && &x != &pd.wei ? 0 : x.strides[nd - 1];
        return true;
    };
    CHECK_UNIMPL(strides3(pd.src, D.src_stride));
    if (pd.wei.kind == dnnl_format_kind_opaque) {
        CHECK_UNIMPL(nd == 2);
        D.wei_packing = pd.wei.packing;
        D.wei_stride[0] = 0; D.wei_stride[1] = D.N; D.wei_stride[2] = 1; // not read
    } else {
        CHECK_UNIMPL(strides3(pd.wei, D.wei_stride));
    }
    CHECK_UNIMPL(strides3(pd.dst, D.dst_stride));
    if (pd.with_bias) CHECK_UNIMPL(strides3(pd.bias, D.bias_stride));
    const dnnl_primitive_attr &a = pd.attr;
    CHECK_UNIMPL(lower_quant(a.find(a.scales, DNNL_ARG_SRC), nd, dnnl_f32, &D.src_scale));
    CHECK_UNIMPL(lower_quant(a.find(a.scales, DNNL_ARG_WEIGHTS), nd, dnnl_f32, &D.wei_scale));
    CHECK_UNIMPL(lower_quant(a.find(a.scales, DNNL_ARG_DST), nd, dnnl_f32, &D.dst_scale));
    CHECK_UNIMPL(lower_quant(a.find(a.zero_points, DNNL_ARG_SRC), nd, dnnl_s32, &D.src_zp));
    CHECK_UNIMPL(lower_quant(a.find(a.zero_points, DNNL_ARG_WEIGHTS), nd, dnnl_s32, &D.wei_zp));
    CHECK_UNIMPL(lower_quant(a.find(a.zero_points, DNNL_ARG_DST), nd, dnnl_s32, &D.dst_zp));
    CHECK_UNIMPL(lower_quant(a.find(a.reductions, DNNL_ARG_SRC), nd, dnnl_s32, &D.src_pr));
    // a static dst scale is one value; a grouped one is the dynamic (MX) mode
    {
        const quant_entry_t *dq = a.find(a.scales, DNNL_ARG_DST);
        if (dq && dq->is_dynamic()) {
            D.dst_scale_dynamic = dq->is_mx() ? MI355_DST_DYNAMIC_MX : MI355_DST_DYNAMIC_FP;
            CHECK_UNIMPL((is_fp8(pd.dst.dt) || pd.dst.dt == dnnl_f4_e2m1) && D.dst_zp.dt == MI355_DT_UNDEF
                    && D.N % dq->group(1) == 0);
        } else {
            CHECK_UNIMPL(D.dst_scale.dt == MI355_DT_UNDEF || D.dst_scale.mask == 0);
        }
    }
    CHECK_UNIMPL(D.dst_zp.dt == MI355_DT_UNDEF || D.dst_zp.dt == MI355_DT_S32);
    // dropout and stochastic rounding: ref_matmul_t only (ref_matmul.hpp:96-149)
    D.rnd_flags = 0;
    if (a.with_dropout()) {
        CHECK_UNIMPL(first == 0);
        D.rnd_flags |= MI355_RND_DROPOUT;
        if (a.dropout_seed_dt == dnnl_s64) D.rnd_flags |= MI355_RND_SEED_S64;
        if (a.dropout_use_offset) D.rnd_flags |= MI355_RND_DROPOUT_OFFSET;
        if (a.dropout_md.dt != dnnl_data_type_undef) {
            // the mask is laid out like dst (dropout_t::set_default_formats + similar_to)
            const dnnl_memory_desc &mk = a.dropout_md;
            CHECK_UNIMPL(mk.ndims == nd);
            for (int i = 0; i < nd; ++i) CHECK_UNIMPL(mk.dims[i] == pd.dst.dims[i]);
            if (mk.kind != dnnl_format_kind_any)
                for (int i = 0; i < nd; ++i) CHECK_UNIMPL(mk.strides[i] == pd.dst.strides[i]);
            D.rnd_flags |= MI355_RND_DROPOUT_MASK;
        }
    }
    {
        auto it = a.rounding.find(DNNL_ARG_DST);
        if (it != a.rounding.end() && it->second == dnnl_rounding_mode_stochastic) {
            CHECK_UNIMPL(first == 0);
            D.rnd_flags |= MI355_RND_DST_STOCHASTIC;
        }
        for (const auto &kv : a.rounding) CHECK_UNIMPL(kv.first == DNNL_ARG_DST);
    }
    D.fpmath_apply_to_int = a.apply_to_int;
    D.fpmath_mode = a.fpmath;
    D.dst_scale_mode = MI355_DST_SCALE_DIVIDE;
    if (const char *e = getenv("ONEDNN_AMD_DST_SCALE_RECIPROCAL"))
        if (atoi(e)) D.dst_scale_mode = MI355_DST_SCALE_RECIPROCAL;
    int n_slots = (int)a.post_ops.entries.size();
    for (const post_op_entry_t &e : a.post_ops.entries) n_slots += e.kind == dnnl_binary && e.alg == dnnl_binary_select;
    CHECK_UNIMPL(n_slots <= MI355_MAX_POST_OPS);
    D.n_post_ops = n_slots;
    auto operand_strides = [&](const dnnl_memory_desc &x, int64_t *st) -> bool {
        if (!collapse_batch(x, pd.dst, &st[0], first)) return false;
        st[1] = x.dims[nd - 2] == 1 ? 0 : x.strides[nd - 2];
        st[2] = x.dims[nd - 1] == 1 ? 0 : x.strides[nd - 1];
        if (pd.dst.dims[nd - 2] == 1) st[1] = x.strides[nd - 2];
        if (pd.dst.dims[nd - 1] == 1) st[2] = x.strides[nd - 1];
        return true;
    };
    for (int i = 0, ei = 0; i < D.n_post_ops; ++i, ++ei) {
        const post_op_entry_t &e = a.post_ops.entries[ei];
        mi355_post_op_t &o = D.post_ops[i];
        pd.po_entry[i] = ei;
        pd.po_arg_id[i] = e.kind == dnnl_binary ? DNNL_ARG_SRC_1 : e.kind == dnnl_prelu ? DNNL_ARG_WEIGHTS : 0;
        o.alpha = e.alpha; o.beta = e.beta; o.scale = e.scale; o.zero_point = e.zero_point;
        switch (e.kind) {
            case dnnl_sum: o.kind = MI355_PO_SUM; o.dt = e.dt; break;
            case dnnl_eltwise:
                o.kind = MI355_PO_ELTWISE;
                // forward: a *_use_dst_for_bwd algorithm computes what its base one does (primitive_attr_postops.cpp:74-82)
                switch (e.alg) {
                    case dnnl_eltwise_relu_use_dst_for_bwd: o.alg = dnnl_eltwise_relu; break;
                    case dnnl_eltwise_tanh_use_dst_for_bwd: o.alg = dnnl_eltwise_tanh; break;
                    case dnnl_eltwise_elu_use_dst_for_bwd: o.alg = dnnl_eltwise_elu; break;
                    case dnnl_eltwise_sqrt_use_dst_for_bwd: o.alg = dnnl_eltwise_sqrt; break;
                    case dnnl_eltwise_logistic_use_dst_for_bwd: o.alg = dnnl_eltwise_logistic; break;
                    case dnnl_eltwise_exp_use_dst_for_bwd: o.alg = dnnl_eltwise_exp; break;
                    case dnnl_eltwise_clip_v2_use_dst_for_bwd: o.alg = dnnl_eltwise_clip_v2; break;
                    default: o.alg = e.alg; break;
                }
                break;
            case dnnl_binary: {
                o.kind = MI355_PO_BINARY; o.alg = e.alg; o.dt = e.src1.dt;
                if (!operand_strides(e.src1, o.stride)) return dnnl_unimplemented;
                if (e.alg == dnnl_binary_select) {
                    // the condition takes the next slot
                    mi355_post_op_t &c = D.post_ops[++i];
                    c.kind = MI355_PO_SELECT_COND; c.dt = e.src2.dt;
                    if (!operand_strides(e.src2, c.stride)) return dnnl_unimplemented;
                    pd.po_entry[i] = ei;
                    pd.po_arg_id[i] = DNNL_ARG_SRC_2;
                }
            } break;
            case dnnl_prelu: {
                // weights are f32, dims = dst dims under the mask, in the layout
                // the reference gives them (get_prelu_weights_format,
                // src/cpu/primitive_attr_postops.cpp:218-241): ab, acb, acdb,
                // acdeb -- from three dims on, dim 1 is the innermost one
                o.kind = MI355_PO_PRELU; o.dt = dnnl_f32;
                CHECK_UNIMPL(nd <= 5);
                dnnl_memory_desc w;
                w.ndims = nd; w.dt = dnnl_f32;
                for (int d = 0; d < nd; ++d) w.dims[d] = ((e.mask >> d) & 1) ? pd.dst.dims[d] : 1;
                int perm[DNNL_MAX_NDIMS];
                for (int d = 0; d < nd; ++d) perm[d] = d;
                if (nd >= 3) {
                    for (int d = 1; d + 1 < nd; ++d) perm[d] = d + 1;
                    perm[nd - 1] = 1;
                }
                w.set_dense(perm);
                if (!operand_strides(w, o.stride)) return dnnl_unimplemented;
            } break;
            default: return dnnl_unimplemented;
        }
    }
    D.impl = MI355_IMPL_AUTO;
    return dnnl_success;
}

// implementation list of the HIP engine, best first (the role of
// engine_t::get_implementation_list, src/common/engine.hpp:134-137)
const int k_impl_list[] = {MI355_IMPL_WOQ_PACKED, MI355_IMPL_WOQ_GEMV, MI355_IMPL_I8_MFMA, MI355_IMPL_F8_MFMA, MI355_IMPL_MXF4_MFMA,
        MI355_IMPL_H16_MFMA, MI355_IMPL_REF};

dnnl_status_t select_impl(dnnl_primitive_desc &pd) {
    pd.desc.impl = pd.impls[pd.impl_pos];
    pd.impl_name = mi355_matmul_impl_name(pd.desc.impl);
    size_t bytes = 0;
    const int st = mi355_matmul_scratch_bytes(&pd.desc, &bytes);
    if (st != MI355_SUCCESS) return from_mi355(st);
    pd.scratch_bytes = bytes;
    pd.scratchpad = dnnl_memory_desc();
    if (pd.attr.scratchpad_mode == dnnl_scratchpad_mode_user && bytes > 0) {
        pd.scratchpad.ndims = 1;
        pd.scratchpad.dims[0] = (dim_t)bytes;
        pd.scratchpad.dt = dnnl_u8;
        pd.scratchpad.set_dense();
    }
    return dnnl_success;
}

// data type combinations of the reference's two naive implementations
// (ref_matmul.hpp:44-123, ref_matmul_int8.hpp:44-92)
dnnl_status_t check_dtypes(const dnnl_primitive_desc &pd) {
    {
        const int s = pd.src.dt, w = pd.wei.dt, d = pd.dst.dt;
        const bool int_path = is_int8(s);
        if (int_path) {
            CHECK_UNIMPL(is_int8(w) || w == dnnl_s4 || w == dnnl_u4);
            CHECK_UNIMPL(d == dnnl_f32 || d == dnnl_bf16 || d == dnnl_f16 || d == dnnl_s32 || is_int8(d));
            if (pd.with_bias) CHECK_UNIMPL(pd.bias.dt == dnnl_f32 || pd.bias.dt == dnnl_bf16 || pd.bias.dt == dnnl_f16
                    || pd.bias.dt == dnnl_s32 || is_int8(pd.bias.dt));
        } else {
            CHECK_UNIMPL(s == dnnl_f32 || s == dnnl_bf16 || s == dnnl_f16 || is_fp8(s) || s == dnnl_f4_e2m1);
            CHECK_UNIMPL(w == dnnl_f32 || w == dnnl_bf16 || w == dnnl_f16 || is_fp8(w) || w == dnnl_f4_e2m1
                    || is_int8(w) || w == dnnl_s4 || w == dnnl_u4);
            CHECK_UNIMPL(s == w || w == dnnl_bf16 || w == dnnl_f16 || is_fp8(w) || is_int8(w) || w == dnnl_s4
                    || w == dnnl_u4);
            // integer weights under a floating-point src only as weight decompression
            CHECK_UNIMPL(IMPLICATION(is_int8(w) || w == dnnl_s4 || w == dnnl_u4, pd.attr.apply_to_int));
            CHECK_UNIMPL(d == dnnl_f32 || d == dnnl_bf16 || d == dnnl_f16 || is_fp8(d) || is_int8(d) || d == dnnl_f4_e2m1);
            if (pd.with_bias) CHECK_UNIMPL(pd.bias.dt == dnnl_f32 || pd.bias.dt == dnnl_bf16 || pd.bias.dt == dnnl_f16 || is_fp8(pd.bias.dt));
        }
    }
    return dnnl_success;
}

// lowers the descriptor and lists the kernel families that take it, best first
dnnl_status_t dispatch(dnnl_primitive_desc &pd) {
    dnnl_status_t st = lower(pd);
    if (st) return st;
    pd.impls.clear();
    for (int impl : k_impl_list) {
        int chosen = 0;
        if (mi355_matmul_query(&pd.desc, impl, &chosen) == MI355_SUCCESS) pd.impls.push_back(impl);
    }
    if (pd.impls.empty()) return dnnl_unimplemented;
    pd.impl_pos = 0;
    return select_impl(pd);
}

// Runtime dims: the descriptor of this execution.  A tensor whose descriptor
// was created with runtime values takes the descriptor of its memory object
// (exec_ctx_t::memory_mdw, src/common/primitive_exec_types.hpp:112-186), which
// has to agree with every value that was known; then the checks that were
// left open at creation run, the descriptor is lowered and the kernel family
// is chosen.  The result is kept for the next execution with the same shapes.
dnnl_status_t concretize(dnnl_primitive &prim, const std::map<int, dnnl_memory_t> &m, void **scratch) {
    const dnnl_primitive_desc &pd0 = prim.pd;
    // src, weights, dst, bias of this execution
    dnnl_memory_desc now[4] = {pd0.src, pd0.wei, pd0.dst, pd0.bias};
    const int arg_of[4] = {DNNL_ARG_SRC, DNNL_ARG_WEIGHTS, DNNL_ARG_DST, DNNL_ARG_BIAS};
    for (int t = 0; t < 4; ++t) {
        if ((t == 3 && !pd0.with_bias) || !now[t].has_runtime()) continue;
        const dnnl_memory_desc &from = now[t];
        auto it = m.find(arg_of[t]);
        CHECK_ARG(it != m.end() && it->second);
        const dnnl_memory_desc &mm = it->second->md;
        CHECK_ARG(mm.kind == dnnl_blocked && mm.ndims == from.ndims && mm.dt == from.dt);
        for (int i = 0; i < mm.ndims; ++i) {
            CHECK_ARG(from.dims[i] == DNNL_RUNTIME_DIM_VAL || from.dims[i] == mm.dims[i]);
            CHECK_ARG(from.strides[i] == DNNL_RUNTIME_DIM_VAL || from.strides[i] == mm.strides[i] || mm.dims[i] <= 1);
        }
        now[t] = mm;
    }
    const bool same = prim.rt_pd && prim.rt_pd->src == now[0] && prim.rt_pd->wei == now[1] && prim.rt_pd->dst == now[2]
            && (!pd0.with_bias || prim.rt_pd->bias == now[3]);
    if (!same) {
        std::unique_ptr<dnnl_primitive_desc> c(new dnnl_primitive_desc(pd0));
        c->runtime = false;
        c->src = now[0]; c->wei = now[1]; c->dst = now[2]; c->bias = now[3];
        dnnl_status_t st = check_shapes(c->src, c->wei, pd0.with_bias ? &c->bias : nullptr, c->dst);
        if (st) return st;
        st = check_attr(c->src, c->wei, c->dst, c->attr);
        if (st) return st;
        st = dispatch(*c);
        if (st) return st;
        prim.rt_pd = std::move(c);
    }
    const size_t need = prim.rt_pd->scratch_bytes;
    if (need > prim.rt_scratch_bytes) {
        if (mi355_device_set((int)pd0.engine->index) != MI355_SUCCESS) return dnnl_runtime_error;
        void *q = nullptr;
        const int st = mi355_mem_alloc(&q, need);
        if (st != MI355_SUCCESS) return from_mi355(st);
        prim.rt_scratch.push_back(q);
        prim.rt_scratch_bytes = need;
    }
    *scratch = prim.rt_scratch.empty() ? nullptr : prim.rt_scratch.back();
    return dnnl_success;
}

} // namespace

// ================================================================ C API
DNNL_EXPORT dnnl_status_t dnnl_engine_create(dnnl_engine_t *engine, dnnl_engine_kind_t kind, size_t index) {
    CHECK_ARG(engine);
    // this library provides the GPU (HIP) engine only
    CHECK_ARG(kind == dnnl_gpu);
    int n = 0;
    const int rc = mi355_device_count(&n);
    // ONEDNN_AMD_ALLOW_NO_DEVICE=1: descriptor-only engine on a machine without
    // a GPU (primitive descriptors can be created and queried, nothing executes)
    const char *nodev = getenv("ONEDNN_AMD_ALLOW_NO_DEVICE");
    if (!(nodev && atoi(nodev) && index == 0)) {
        if (rc != MI355_SUCCESS) return dnnl_runtime_error;
        CHECK_ARG((int)index < n);
    }
    *engine = new dnnl_engine {kind, index};
    return dnnl_success;
}
DNNL_EXPORT size_t dnnl_engine_get_count(dnnl_engine_kind_t kind) {
    if (kind != dnnl_gpu) return 0;
    int n = 0;
    if (mi355_device_count(&n) != MI355_SUCCESS) return 0;
    return (size_t)n;
}
DNNL_EXPORT dnnl_status_t dnnl_engine_get_kind(dnnl_engine_t engine, dnnl_engine_kind_t *kind) {
    CHECK_ARG(engine && kind);
    *kind = engine->kind;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_engine_destroy(dnnl_engine_t engine) {
    delete engine;
    return dnnl_success;
}

DNNL_EXPORT dnnl_status_t dnnl_stream_create(dnnl_stream_t *stream, dnnl_engine_t engine, unsigned flags) {
    CHECK_ARG(stream && engine);
    CHECK_ARG(flags & (dnnl_stream_in_order | dnnl_stream_out_of_order));
    if (mi355_device_set((int)engine->index) != MI355_SUCCESS) return dnnl_runtime_error;
    void *s = nullptr;
    if (mi355_stream_create(&s) != MI355_SUCCESS) return dnnl_runtime_error;
    *stream = new dnnl_stream {engine, s, true};
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_stream_get_engine(const_dnnl_stream_t stream, dnnl_engine_t *engine) {
    CHECK_ARG(stream && engine);
    *engine = stream->engine;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_stream_wait(dnnl_stream_t stream) {
    CHECK_ARG(stream);
    return from_mi355(mi355_stream_sync(stream->hip_stream));
}
DNNL_EXPORT dnnl_status_t dnnl_stream_destroy(dnnl_stream_t stream) {
    if (stream) {
        if (stream->owned) mi355_stream_destroy(stream->hip_stream);
        delete stream;
    }
    return dnnl_success;
}
// The interoperability pair of the reference's GPU runtimes (dnnl_ocl.h:220-231, dnnl_sycl.h:154-165) for HIP:
// a dnnl stream over the caller's hipStream_t (a framework's current stream; NULL is the default stream), so that
// primitives are ordered with the caller's own kernels -- and recorded when the caller captures that stream.
DNNL_EXPORT dnnl_status_t dnnl_amd_interop_stream_create(dnnl_stream_t *stream, dnnl_engine_t engine, void *hip_stream) {
    CHECK_ARG(stream && engine);
    *stream = new dnnl_stream {engine, hip_stream, false};
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_amd_interop_stream_get_hip_stream(dnnl_stream_t stream, void **hip_stream) {
    CHECK_ARG(stream && hip_stream);
    *hip_stream = stream->hip_stream;
    return dnnl_success;
}

// ---- memory descriptors
static dnnl_status_t md_common(dnnl_memory_desc &md, int ndims, const dnnl_dims_t dims, dnnl_data_type_t dt) {
    CHECK_ARG(ndims > 0 && ndims <= DNNL_MAX_NDIMS && dims);
    CHECK_ARG(dt_valid(dt));
    md.ndims = ndims;
    md.dt = dt;
    for (int i = 0; i < ndims; ++i) {
        CHECK_ARG(dims[i] >= 0 || dims[i] == DNNL_RUNTIME_DIM_VAL);
        md.dims[i] = dims[i];
    }
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_desc_create_with_strides(dnnl_memory_desc_t *memory_desc, int ndims,
        const dnnl_dims_t dims, dnnl_data_type_t data_type, const dnnl_dims_t strides) {
    CHECK_ARG(memory_desc);
    std::unique_ptr<dnnl_memory_desc> md(new dnnl_memory_desc);
    dnnl_status_t st = md_common(*md, ndims, dims, data_type);
    if (st) return st;
    if (!strides) {
        md->set_dense();
    } else {
        for (int i = 0; i < ndims; ++i) {
            CHECK_ARG(strides[i] >= 0 || strides[i] == DNNL_RUNTIME_DIM_VAL);
            md->strides[i] = strides[i];
        }
        md->kind = dnnl_blocked;
        // sub-byte types need an innermost unit stride (memory_desc.cpp, 4-bit rule)
        if (dt_bits(data_type) == 4) {
            bool unit = false;
            for (int i = 0; i < ndims; ++i)
                if (md->strides[i] == 1) unit = true;
            CHECK_ARG(unit);
        }
    }
    *memory_desc = md.release();
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_desc_create_with_tag(dnnl_memory_desc_t *memory_desc, int ndims,
        const dnnl_dims_t dims, dnnl_data_type_t data_type, dnnl_format_tag_t tag) {
    CHECK_ARG(memory_desc);
    std::unique_ptr<dnnl_memory_desc> md(new dnnl_memory_desc);
    if (ndims == 0 || tag == dnnl_format_tag_undef) { // a zero descriptor, memory_desc.cpp:245-250
        *memory_desc = md.release();
        return dnnl_success;
    }
    dnnl_status_t st = md_common(*md, ndims, dims, data_type);
    if (st) return st;
    int perm[DNNL_MAX_NDIMS];
    for (int i = 0; i < ndims; ++i) perm[i] = i;
    switch (tag) {
        case dnnl_format_tag_any:
            // no layout can be picked for dims that are not known (memory_desc.cpp:70-72)
            for (int i = 0; i < ndims; ++i) CHECK_ARG(dims[i] != DNNL_RUNTIME_DIM_VAL);
            md->kind = dnnl_format_kind_any;
            *memory_desc = md.release();
            return dnnl_success;
        case dnnl_a: CHECK_ARG(ndims == 1); break;
        case dnnl_ab: CHECK_ARG(ndims == 2); break;
        case dnnl_abc: CHECK_ARG(ndims == 3); break;
        case dnnl_abcd: CHECK_ARG(ndims == 4); break;
        case dnnl_abcde: CHECK_ARG(ndims == 5); break;
        case dnnl_ba: CHECK_ARG(ndims == 2); perm[0] = 1; perm[1] = 0; break;
        case dnnl_acb: CHECK_ARG(ndims == 3); perm[1] = 2; perm[2] = 1; break;
        case dnnl_abdc: CHECK_ARG(ndims == 4); perm[2] = 3; perm[3] = 2; break;
        case dnnl_acdb: CHECK_ARG(ndims == 4); perm[1] = 2; perm[2] = 3; perm[3] = 1; break;
        case dnnl_acdeb: CHECK_ARG(ndims == 5); perm[1] = 2; perm[2] = 3; perm[3] = 4; perm[4] = 1; break;
        default: return dnnl_unimplemented; // blocked layouts are not offered
    }
    md->set_dense(perm);
    *memory_desc = md.release();
    return dnnl_success;
}
// memory_desc_init_with_grouped_encoding, src/common/memory_desc.cpp:417-472
DNNL_EXPORT dnnl_status_t dnnl_memory_desc_create_with_grouped_encoding(dnnl_memory_desc_t *memory_desc, int ndims,
        const dnnl_dims_t dims, dnnl_data_type_t data_type, int variable_dim_idx, dnnl_dim_t group_count,
        dnnl_data_type_t offsets_dt) {
    CHECK_ARG(memory_desc);
    std::unique_ptr<dnnl_memory_desc> md(new dnnl_memory_desc);
    if (ndims == 0) {
        *memory_desc = md.release();
        return dnnl_success;
    }
    CHECK_UNIMPL(ndims == 2);
    CHECK_ARG(dims && dt_valid(data_type));
    CHECK_ARG(group_count > 0);
    CHECK_ARG(offsets_dt == dnnl_s32);
    CHECK_ARG(variable_dim_idx >= 0 && variable_dim_idx < ndims);
    for (int d = 0; d < ndims; ++d) CHECK_ARG(dims[d] != DNNL_RUNTIME_DIM_VAL && dims[d] > 0);
    md->ndims = ndims;
    md->dt = data_type;
    for (int d = 0; d < ndims; ++d) md->dims[d] = dims[d];
    md->kind = dnnl_format_kind_sparse;
    md->grouped = true;
    md->var_dim = variable_dim_idx;
    md->group_count = group_count;
    // the variable dim is the outermost one: idx 0 -> row-major, idx 1 -> column-major
    md->strides[variable_dim_idx] = dims[1 - variable_dim_idx];
    md->strides[1 - variable_dim_idx] = 1;
    *memory_desc = md.release();
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_desc_clone(dnnl_memory_desc_t *memory_desc, const_dnnl_memory_desc_t existing) {
    CHECK_ARG(memory_desc && existing);
    *memory_desc = new dnnl_memory_desc(*existing);
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_desc_destroy(dnnl_memory_desc_t memory_desc) {
    delete memory_desc;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_desc_query(const_dnnl_memory_desc_t md, dnnl_query_t what, void *result) {
    CHECK_ARG(md && result);
    switch (what) {
        case dnnl_query_ndims_s32: *(int32_t *)result = md->ndims; break;
        case dnnl_query_dims: *(const dnnl_dims_t **)result = &md->dims; break;
        case dnnl_query_data_type: *(dnnl_data_type_t *)result = md->dt; break;
        case dnnl_query_format_kind: *(dnnl_format_kind_t *)result = md->kind; break;
        case dnnl_query_strides:
            if (md->kind != dnnl_blocked) return dnnl_invalid_arguments;
            *(const dnnl_dims_t **)result = &md->strides;
            break;
        case dnnl_query_sparse_encoding:
            *(dnnl_sparse_encoding_t *)result = md->grouped ? dnnl_grouped : dnnl_sparse_encoding_undef;
            break;
        case dnnl_query_nnz_s64: *(int64_t *)result = md->grouped ? md->nelems() : 0; break;
        case dnnl_query_num_handles_s32: *(int32_t *)result = md->grouped ? 2 : 1; break; // memory_desc.cpp:1096
        default: return dnnl_unimplemented;
    }
    return dnnl_success;
}
DNNL_EXPORT int dnnl_memory_desc_equal(const_dnnl_memory_desc_t lhs, const_dnnl_memory_desc_t rhs) {
    if (lhs == rhs) return 1;
    if (!lhs || !rhs) return 0;
    return *lhs == *rhs;
}
DNNL_EXPORT size_t dnnl_memory_desc_get_size(const_dnnl_memory_desc_t md) {
    if (md && md->kind == dnnl_format_kind_host_scalar) return dt_bits(md->dt) / 8;
    if (md && md->grouped) return md->size_bytes();
    if (!md || (md->kind != dnnl_blocked && md->kind != dnnl_format_kind_opaque)) return 0;
    return md->size_bytes();
}
// buffer `index` of a descriptor: a grouped tensor has the values (0) and the s32 offsets (1)
DNNL_EXPORT size_t dnnl_memory_desc_get_size_v2(const_dnnl_memory_desc_t md, int index) {
    if (!md || index < 0) return 0;
    if (index == 0) return dnnl_memory_desc_get_size(md);
    if (md->grouped && index == 1) return (size_t)md->group_count * sizeof(int32_t);
    return 0;
}
DNNL_EXPORT size_t dnnl_data_type_size(dnnl_data_type_t dt) {
    return dt_bits(dt) / 8 ? dt_bits(dt) / 8 : 1;
}

// ---- memory objects
DNNL_EXPORT dnnl_status_t dnnl_memory_create(dnnl_memory_t *memory, const_dnnl_memory_desc_t md,
        dnnl_engine_t engine, void *handle) {
    CHECK_ARG(memory && md && engine);
    CHECK_ARG(md->kind != dnnl_format_kind_any);
    CHECK_ARG(!md->has_runtime()); // src/common/memory.cpp:155
    CHECK_ARG(md->kind != dnnl_format_kind_host_scalar); // :157, dnnl_memory_create_host_scalar makes those
    CHECK_ARG(md->kind != dnnl_format_kind_sparse || md->grouped);
    std::unique_ptr<dnnl_memory> m(new dnnl_memory);
    m->md = *md;
    m->engine = engine;
    if (handle == DNNL_MEMORY_ALLOCATE) {
        if (mi355_device_set((int)engine->index) != MI355_SUCCESS) return dnnl_runtime_error;
        const int st = mi355_mem_alloc(&m->handle, md->size_bytes());
        if (st != MI355_SUCCESS) return from_mi355(st);
        m->owned = true;
    } else {
        m->handle = handle;
    }
    *memory = m.release();
    return dnnl_success;
}
// A memory object over several buffers (src/common/memory.cpp: dnnl_memory_create_v2): only the grouped encoding
// has more than one here.  DNNL_MEMORY_ALLOCATE in a slot lets the library own that buffer.
DNNL_EXPORT dnnl_status_t dnnl_memory_create_v2(dnnl_memory_t *memory, const_dnnl_memory_desc_t md, dnnl_engine_t engine,
        int nhandles, void **handles) {
    CHECK_ARG(memory && md && engine && handles);
    const int need = md->grouped ? 2 : 1;
    CHECK_ARG(nhandles == need);
    dnnl_status_t st = dnnl_memory_create(memory, md, engine, handles[0]);
    if (st != dnnl_success || need == 1) return st;
    dnnl_memory *m = *memory;
    if (handles[1] == DNNL_MEMORY_ALLOCATE) {
        const int rc = mi355_mem_alloc(&m->handle2, dnnl_memory_desc_get_size_v2(md, 1));
        if (rc != MI355_SUCCESS) {
            dnnl_memory_destroy(m);
            *memory = nullptr;
            return from_mi355(rc);
        }
        m->owned2 = true;
    } else {
        m->handle2 = handles[1];
    }
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_get_data_handle_v2(const_dnnl_memory_t memory, void **handle, int index) {
    CHECK_ARG(memory && handle);
    if (index == 0) return dnnl_memory_get_data_handle(memory, handle);
    CHECK_ARG(memory->md.grouped && index == 1);
    *handle = memory->handle2;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_set_data_handle_v2(dnnl_memory_t memory, void *handle, int index) {
    CHECK_ARG(memory);
    if (index == 0) return dnnl_memory_set_data_handle(memory, handle);
    CHECK_ARG(memory->md.grouped && index == 1);
    if (memory->owned2) {
        mi355_mem_free(memory->handle2);
        memory->owned2 = false;
    }
    memory->handle2 = handle;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_map_data_v2(const_dnnl_memory_t cmemory, void **mapped_ptr, int index) {
    if (index == 0) return dnnl_memory_map_data(cmemory, mapped_ptr);
    CHECK_ARG(cmemory && mapped_ptr);
    dnnl_memory *memory = const_cast<dnnl_memory *>(cmemory);
    CHECK_ARG(memory->md.grouped && index == 1 && !memory->mapped2);
    const size_t bytes = dnnl_memory_desc_get_size_v2(&memory->md, 1);
    if (!memory->handle2) {
        *mapped_ptr = nullptr;
        return dnnl_success;
    }
    void *host = malloc(bytes);
    if (!host) return dnnl_out_of_memory;
    const int st = mi355_mem_d2h(host, memory->handle2, bytes, nullptr);
    if (st != MI355_SUCCESS) {
        free(host);
        return from_mi355(st);
    }
    memory->mapped2 = host;
    *mapped_ptr = host;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_unmap_data_v2(const_dnnl_memory_t cmemory, void *mapped_ptr, int index) {
    if (index == 0) return dnnl_memory_unmap_data(cmemory, mapped_ptr);
    CHECK_ARG(cmemory);
    dnnl_memory *memory = const_cast<dnnl_memory *>(cmemory);
    CHECK_ARG(memory->md.grouped && index == 1);
    if (!memory->mapped2) return mapped_ptr ? dnnl_invalid_arguments : dnnl_success;
    CHECK_ARG(mapped_ptr == memory->mapped2);
    const int st = mi355_mem_h2d(memory->handle2, memory->mapped2, dnnl_memory_desc_get_size_v2(&memory->md, 1), nullptr);
    free(memory->mapped2);
    memory->mapped2 = nullptr;
    return from_mi355(st);
}
// src/common/memory.cpp:219-241, :303-333
DNNL_EXPORT dnnl_status_t dnnl_memory_desc_create_host_scalar(dnnl_memory_desc_t *memory_desc, dnnl_data_type_t data_type) {
    CHECK_ARG(memory_desc);
    CHECK_ARG(dt_valid(data_type) && dt_bits(data_type) >= 8);
    std::unique_ptr<dnnl_memory_desc> md(new dnnl_memory_desc);
    md->ndims = 1;
    md->dims[0] = 1;
    md->strides[0] = 1;
    md->dt = data_type;
    md->kind = dnnl_format_kind_host_scalar;
    *memory_desc = md.release();
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_create_host_scalar(dnnl_memory_t *memory, const_dnnl_memory_desc_t md,
        void *scalar_ptr) {
    CHECK_ARG(memory && md && scalar_ptr);
    CHECK_ARG(md->kind == dnnl_format_kind_host_scalar);
    std::unique_ptr<dnnl_memory> m(new dnnl_memory);
    m->md = *md;
    m->engine = nullptr;
    memcpy(m->scalar, scalar_ptr, dt_bits(md->dt) / 8);
    *memory = m.release();
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_get_host_scalar_value(const_dnnl_memory_t memory, void *value) {
    CHECK_ARG(memory && value);
    CHECK_ARG(memory->md.kind == dnnl_format_kind_host_scalar);
    memcpy(value, memory->scalar, dt_bits(memory->md.dt) / 8);
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_set_host_scalar_value(dnnl_memory_t memory, const void *value) {
    CHECK_ARG(memory && value);
    CHECK_ARG(memory->md.kind == dnnl_format_kind_host_scalar);
    memcpy(memory->scalar, value, dt_bits(memory->md.dt) / 8);
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_get_memory_desc(const_dnnl_memory_t memory, const_dnnl_memory_desc_t *md) {
    CHECK_ARG(memory && md);
    *md = &memory->md;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_get_engine(const_dnnl_memory_t memory, dnnl_engine_t *engine) {
    CHECK_ARG(memory && engine);
    *engine = memory->engine;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_map_data(const_dnnl_memory_t cmemory, void **mapped_ptr) {
    CHECK_ARG(cmemory && mapped_ptr);
    dnnl_memory *memory = const_cast<dnnl_memory *>(cmemory);
    CHECK_ARG(!memory->mapped);
    CHECK_ARG(memory->md.kind != dnnl_format_kind_host_scalar); // src/common/memory.cpp:265-297: value accessors only
    const size_t bytes = memory->md.size_bytes();
    if (!memory->handle || bytes == 0) {
        *mapped_ptr = nullptr;
        return dnnl_success;
    }
    void *host = malloc(bytes);
    if (!host) return dnnl_out_of_memory;
    const int st = mi355_mem_d2h(host, memory->handle, bytes, nullptr);
    if (st != MI355_SUCCESS) {
        free(host);
        return from_mi355(st);
    }
    memory->mapped = host;
    *mapped_ptr = host;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_unmap_data(const_dnnl_memory_t cmemory, void *mapped_ptr) {
    CHECK_ARG(cmemory);
    dnnl_memory *memory = const_cast<dnnl_memory *>(cmemory);
    if (!memory->mapped) return mapped_ptr ? dnnl_invalid_arguments : dnnl_success;
    CHECK_ARG(mapped_ptr == memory->mapped);
    const int st = mi355_mem_h2d(memory->handle, memory->mapped, memory->md.size_bytes(), nullptr);
    free(memory->mapped);
    memory->mapped = nullptr;
    return from_mi355(st);
}
DNNL_EXPORT dnnl_status_t dnnl_memory_get_data_handle(const_dnnl_memory_t memory, void **handle) {
    CHECK_ARG(memory && handle);
    CHECK_ARG(memory->md.kind != dnnl_format_kind_host_scalar);
    *handle = memory->handle;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_set_data_handle(dnnl_memory_t memory, void *handle) {
    CHECK_ARG(memory);
    CHECK_ARG(memory->md.kind != dnnl_format_kind_host_scalar);
    if (memory->owned) {
        mi355_mem_free(memory->handle);
        memory->owned = false;
    }
    memory->handle = handle;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_memory_destroy(dnnl_memory_t memory) {
    if (memory) {
        if (memory->mapped) free(memory->mapped);
        if (memory->owned) mi355_mem_free(memory->handle);
        if (memory->mapped2) free(memory->mapped2);
        if (memory->owned2) mi355_mem_free(memory->handle2);
        delete memory;
    }
    return dnnl_success;
}

// ---- attributes
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_create(dnnl_primitive_attr_t *attr) {
    CHECK_ARG(attr);
    *attr = new dnnl_primitive_attr;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_clone(dnnl_primitive_attr_t *attr, const_dnnl_primitive_attr_t existing) {
    CHECK_ARG(attr && existing);
    *attr = new dnnl_primitive_attr(*existing);
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_destroy(dnnl_primitive_attr_t attr) {
    delete attr;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_fpmath_mode_v2(dnnl_primitive_attr_t attr,
        dnnl_fpmath_mode_t mode, int apply_to_int) {
    CHECK_ARG(attr);
    CHECK_ARG(mode >= dnnl_fpmath_mode_strict && mode <= dnnl_fpmath_mode_tf32);
    attr->fpmath = mode;
    attr->apply_to_int = apply_to_int != 0;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_fpmath_mode(dnnl_primitive_attr_t attr, dnnl_fpmath_mode_t mode) {
    return dnnl_primitive_attr_set_fpmath_mode_v2(attr, mode, 0);
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_get_fpmath_mode_v2(const_dnnl_primitive_attr_t attr,
        dnnl_fpmath_mode_t *mode, int *apply_to_int) {
    CHECK_ARG(attr);
    if (mode) *mode = attr->fpmath;
    if (apply_to_int) *apply_to_int = attr->apply_to_int;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_accumulation_mode(dnnl_primitive_attr_t attr,
        dnnl_accumulation_mode_t mode) {
    CHECK_ARG(attr);
    CHECK_ARG(mode >= dnnl_accumulation_mode_strict && mode <= dnnl_accumulation_mode_f16);
    attr->acc_mode = mode;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_get_dropout_v2(const_dnnl_primitive_attr_t attr,
        const_dnnl_memory_desc_t *mask_desc, dnnl_data_type_t *seed_dt, int *use_offset, int *use_host_scalars) {
    CHECK_ARG(attr);
    if (mask_desc) *mask_desc = &attr->dropout_md;
    if (seed_dt) *seed_dt = attr->dropout_seed_dt;
    if (use_offset) *use_offset = attr->dropout_use_offset;
    if (use_host_scalars) *use_host_scalars = attr->dropout_host_scalars;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_get_dropout(const_dnnl_primitive_attr_t attr,
        const_dnnl_memory_desc_t *mask_desc) {
    return dnnl_primitive_attr_get_dropout_v2(attr, mask_desc, nullptr, nullptr, nullptr);
}
// primitive_attr_t::set_dropout, src/common/primitive_attr.cpp:423-438
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_dropout_v2(dnnl_primitive_attr_t attr, const_dnnl_memory_desc_t mask_desc,
        dnnl_data_type_t seed_dt, int use_offset, int use_host_scalars) {
    CHECK_ARG(attr && mask_desc);
    CHECK_ARG(mask_desc->dt == dnnl_u8 || mask_desc->dt == dnnl_data_type_undef);
    CHECK_ARG(seed_dt == dnnl_s32 || seed_dt == dnnl_s64);
    attr->dropout_md = *mask_desc;
    attr->dropout_seed_dt = seed_dt;
    attr->dropout_use_offset = use_offset != 0;
    attr->dropout_host_scalars = use_host_scalars != 0;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_dropout(dnnl_primitive_attr_t attr, const_dnnl_memory_desc_t mask_desc) {
    return dnnl_primitive_attr_set_dropout_v2(attr, mask_desc, dnnl_s32, 0, 0);
}
// rnd_mode_t::set / check, src/common/primitive_attr.hpp:226-258: only dst and the gradients take a non-default mode
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_rounding(dnnl_primitive_attr_t attr, int arg, dnnl_rounding_mode_t mode) {
    CHECK_ARG(attr);
    CHECK_ARG(mode == dnnl_rounding_mode_environment || mode == dnnl_rounding_mode_stochastic);
    if (mode != dnnl_rounding_mode_environment) {
        CHECK_ARG(arg == DNNL_ARG_DST || arg == DNNL_ARG_DIFF_SRC || arg == DNNL_ARG_DIFF_WEIGHTS);
        attr->rounding[arg] = mode;
    }
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_get_rounding(dnnl_primitive_attr_t attr, int arg, dnnl_rounding_mode_t *mode) {
    CHECK_ARG(attr && mode);
    auto it = attr->rounding.find(arg);
    *mode = it == attr->rounding.end() ? dnnl_rounding_mode_environment : it->second;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_scratchpad_mode(dnnl_primitive_attr_t attr,
        dnnl_scratchpad_mode_t mode) {
    CHECK_ARG(attr);
    CHECK_ARG(mode == dnnl_scratchpad_mode_library || mode == dnnl_scratchpad_mode_user);
    attr->scratchpad_mode = mode;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_get_scratchpad_mode(const_dnnl_primitive_attr_t attr,
        dnnl_scratchpad_mode_t *mode) {
    CHECK_ARG(attr && mode);
    *mode = attr->scratchpad_mode;
    return dnnl_success;
}

static dnnl_status_t set_quant(std::map<int, quant_entry_t> &m, int arg, int mask, int group_ndims,
        const dnnl_dims_t group_dims, dnnl_data_type_t dt) {
    CHECK_ARG(arg >= 0 && mask >= 0);
    CHECK_ARG(group_ndims == 0 || group_ndims == 2);
    quant_entry_t q;
    q.mask = mask;
    q.dt = dt;
    q.group_ndims = group_ndims;
    if (group_ndims) {
        CHECK_ARG(group_dims && group_dims[0] > 0 && group_dims[1] > 0);
        q.groups[0] = group_dims[0];
        q.groups[1] = group_dims[1];
    }
    m[arg] = q;
    return dnnl_success;
}
// checks of dnnl_primitive_attr_set_scales_v3, src/common/primitive_attr.cpp:637-663
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_scales(dnnl_primitive_attr_t attr, int arg, int mask,
        int group_ndims, const dnnl_dims_t group_dims, dnnl_data_type_t data_type) {
    CHECK_ARG(attr);
    CHECK_ARG(data_type == dnnl_f32 || data_type == dnnl_bf16 || data_type == dnnl_f16 || data_type == dnnl_e8m0
            || data_type == dnnl_f8_e4m3);
    CHECK_ARG(IMPLICATION(data_type == dnnl_e8m0 || data_type == dnnl_f8_e4m3, mask > 0));
    return set_quant(attr->scales, arg, mask, group_ndims, group_dims, data_type);
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_scales_v3(dnnl_primitive_attr_t attr, int arg, int mask,
        int group_ndims, const dnnl_dims_t group_dims, dnnl_data_type_t data_type, int is_on_host,
        dnnl_quantization_mode_t qmode) {
    CHECK_ARG(attr);
    CHECK_ARG(qmode == dnnl_quantization_mode_static_sazp || qmode == dnnl_quantization_mode_dynamic_mx
            || qmode == dnnl_quantization_mode_dynamic_fp);
    CHECK_ARG(IMPLICATION(is_on_host, mask == 0 && group_ndims == 0));
    const dnnl_status_t st = dnnl_primitive_attr_set_scales(attr, arg, mask, group_ndims, group_dims, data_type);
    if (st == dnnl_success) {
        attr->scales[arg].qmode = qmode;
        attr->scales[arg].on_host = is_on_host != 0;
    }
    return st;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_scales_v2(dnnl_primitive_attr_t attr, int arg, int mask,
        int group_ndims, const dnnl_dims_t group_dims, dnnl_data_type_t data_type, int is_on_host) {
    return dnnl_primitive_attr_set_scales_v3(
            attr, arg, mask, group_ndims, group_dims, data_type, is_on_host, dnnl_quantization_mode_static_sazp);
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_scales_mask(dnnl_primitive_attr_t attr, int arg, int mask) {
    return dnnl_primitive_attr_set_scales(attr, arg, mask, 0, nullptr, dnnl_f32);
}
// checks of dnnl_primitive_attr_set_zero_points_v2, primitive_attr.cpp:684-716
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_zero_points(dnnl_primitive_attr_t attr, int arg, int mask,
        int group_ndims, const dnnl_dims_t group_dims, dnnl_data_type_t data_type) {
    CHECK_ARG(attr);
    CHECK_ARG(data_type == dnnl_s32 || data_type == dnnl_s8 || data_type == dnnl_u8 || data_type == dnnl_s4
            || data_type == dnnl_u4);
    CHECK_ARG(IMPLICATION(data_type == dnnl_s4 || data_type == dnnl_u4, mask > 0));
    CHECK_ARG(IMPLICATION(arg != DNNL_ARG_SRC && arg != DNNL_ARG_WEIGHTS, data_type == dnnl_s32 && group_ndims == 0));
    CHECK_ARG(IMPLICATION(group_ndims > 0, mask > 0));
    return set_quant(attr->zero_points, arg, mask, group_ndims, group_dims, data_type);
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_zero_points_v2(dnnl_primitive_attr_t attr, int arg, int mask,
        int group_ndims, const dnnl_dims_t group_dims, dnnl_data_type_t data_type, int is_on_host) {
    CHECK_ARG(attr);
    CHECK_ARG(IMPLICATION(is_on_host, mask == 0 && group_ndims == 0)); // primitive_attr.cpp:700-702
    const dnnl_status_t st = dnnl_primitive_attr_set_zero_points(attr, arg, mask, group_ndims, group_dims, data_type);
    if (st == dnnl_success) attr->zero_points[arg].on_host = is_on_host != 0;
    return st;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_zero_points_mask(dnnl_primitive_attr_t attr, int arg, int mask) {
    return dnnl_primitive_attr_set_zero_points(attr, arg, mask, 0, nullptr, dnnl_s32);
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_precomputed_reductions(dnnl_primitive_attr_t attr, int arg,
        int mask, int group_ndims, const dnnl_dims_t group_dims, dnnl_data_type_t data_type) {
    CHECK_ARG(attr);
    CHECK_ARG(data_type == dnnl_s32);
    CHECK_ARG(mask > 0);
    return set_quant(attr->reductions, arg, mask, group_ndims, group_dims, data_type);
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_set_post_ops(dnnl_primitive_attr_t attr, const_dnnl_post_ops_t post_ops) {
    CHECK_ARG(attr && post_ops);
    attr->post_ops = *post_ops;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_attr_get_post_ops(const_dnnl_primitive_attr_t attr, const_dnnl_post_ops_t *post_ops) {
    CHECK_ARG(attr && post_ops);
    *post_ops = &attr->post_ops; // borrowed, as in the reference (dnnl.h:683-694)
    return dnnl_success;
}

// ---- post-ops
DNNL_EXPORT dnnl_status_t dnnl_post_ops_create(dnnl_post_ops_t *post_ops) {
    CHECK_ARG(post_ops);
    *post_ops = new dnnl_post_ops;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_post_ops_clone(dnnl_post_ops_t *post_ops, const_dnnl_post_ops_t existing) {
    CHECK_ARG(post_ops && existing);
    *post_ops = new dnnl_post_ops(*existing);
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_post_ops_destroy(dnnl_post_ops_t post_ops) {
    delete post_ops;
    return dnnl_success;
}
DNNL_EXPORT int dnnl_post_ops_len(const_dnnl_post_ops_t post_ops) {
    return post_ops ? (int)post_ops->entries.size() : 0;
}
DNNL_EXPORT dnnl_primitive_kind_t dnnl_post_ops_get_kind(const_dnnl_post_ops_t post_ops, int index) {
    if (!post_ops || index < 0 || index >= (int)post_ops->entries.size()) return dnnl_undefined_primitive;
    return post_ops->entries[index].kind;
}
static bool po_full(const_dnnl_post_ops_t p) { return p->entries.size() >= MI355_MAX_POST_OPS; }
DNNL_EXPORT dnnl_status_t dnnl_post_ops_append_sum(dnnl_post_ops_t post_ops, float scale, int32_t zero_point,
        dnnl_data_type_t data_type) {
    CHECK_ARG(post_ops);
    if (po_full(post_ops)) return dnnl_out_of_memory;
    post_op_entry_t e;
    e.kind = dnnl_sum; e.scale = scale; e.zero_point = zero_point; e.dt = data_type;
    post_ops->entries.push_back(e);
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_post_ops_get_params_sum(const_dnnl_post_ops_t post_ops, int index, float *scale,
        int32_t *zero_point, dnnl_data_type_t *data_type) {
    CHECK_ARG(post_ops && index >= 0 && index < (int)post_ops->entries.size());
    const post_op_entry_t &e = post_ops->entries[index];
    CHECK_ARG(e.kind == dnnl_sum);
    if (scale) *scale = e.scale;
    if (zero_point) *zero_point = e.zero_point;
    if (data_type) *data_type = e.dt;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_post_ops_append_eltwise(dnnl_post_ops_t post_ops, dnnl_alg_kind_t alg, float alpha,
        float beta) {
    CHECK_ARG(post_ops);
    const bool use_dst = alg >= dnnl_eltwise_relu_use_dst_for_bwd && alg <= dnnl_eltwise_clip_v2_use_dst_for_bwd;
    CHECK_ARG((alg >= dnnl_eltwise_relu && alg <= dnnl_eltwise_hardswish) || use_dst);
    // is_eltwise_ok, src/common/math_utils.hpp:432-456
    CHECK_ARG(IMPLICATION(alg == dnnl_eltwise_clip || alg == dnnl_eltwise_clip_v2
                    || alg == dnnl_eltwise_clip_v2_use_dst_for_bwd, beta >= alpha));
    CHECK_ARG(IMPLICATION(alg == dnnl_eltwise_relu_use_dst_for_bwd || alg == dnnl_eltwise_elu_use_dst_for_bwd, alpha >= 0));
    if (po_full(post_ops)) return dnnl_out_of_memory;
    post_op_entry_t e;
    e.kind = dnnl_eltwise; e.alg = alg; e.alpha = alpha; e.beta = beta; e.scale = 1.f;
    post_ops->entries.push_back(e);
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_post_ops_get_params_eltwise(const_dnnl_post_ops_t post_ops, int index,
        dnnl_alg_kind_t *alg, float *alpha, float *beta) {
    CHECK_ARG(post_ops && index >= 0 && index < (int)post_ops->entries.size());
    const post_op_entry_t &e = post_ops->entries[index];
    CHECK_ARG(e.kind == dnnl_eltwise);
    if (alg) *alg = e.alg;
    if (alpha) *alpha = e.alpha;
    if (beta) *beta = e.beta;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_post_ops_append_binary(dnnl_post_ops_t post_ops, dnnl_alg_kind_t alg,
        const_dnnl_memory_desc_t src1_desc) {
    CHECK_ARG(post_ops && src1_desc);
    CHECK_ARG(alg >= dnnl_binary_add && alg <= dnnl_binary_ne);
    // (a grouped operand belongs to a grouped matmul: matmul.cpp:221-231)
    CHECK_ARG(src1_desc->kind == dnnl_blocked || src1_desc->kind == dnnl_format_kind_any || src1_desc->grouped);
    if (po_full(post_ops)) return dnnl_out_of_memory;
    post_op_entry_t e;
    e.kind = dnnl_binary; e.alg = alg; e.src1 = *src1_desc;
    if (e.src1.kind == dnnl_format_kind_any) e.src1.set_dense();
    post_ops->entries.push_back(e);
    return dnnl_success;
}
// post_ops_t::append_binary with a ternary algorithm, src/common/primitive_attr.cpp:888-894
DNNL_EXPORT dnnl_status_t dnnl_post_ops_append_binary_v2(dnnl_post_ops_t post_ops, dnnl_alg_kind_t alg,
        const_dnnl_memory_desc_t src1_desc, const_dnnl_memory_desc_t src2_desc) {
    if (alg != dnnl_binary_select) {
        CHECK_ARG(!src2_desc);
        return dnnl_post_ops_append_binary(post_ops, alg, src1_desc);
    }
    CHECK_ARG(post_ops && src1_desc && src2_desc);
    CHECK_ARG(src1_desc->kind == dnnl_blocked || src1_desc->kind == dnnl_format_kind_any);
    CHECK_ARG(src2_desc->kind == dnnl_blocked || src2_desc->kind == dnnl_format_kind_any);
    if (po_full(post_ops)) return dnnl_out_of_memory;
    post_op_entry_t e;
    e.kind = dnnl_binary; e.alg = alg; e.src1 = *src1_desc; e.src2 = *src2_desc;
    if (e.src1.kind == dnnl_format_kind_any) e.src1.set_dense();
    if (e.src2.kind == dnnl_format_kind_any) e.src2.set_dense();
    post_ops->entries.push_back(e);
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_post_ops_get_params_binary_v2(const_dnnl_post_ops_t post_ops, int index,
        dnnl_alg_kind_t *alg, const_dnnl_memory_desc_t *src1_desc, const_dnnl_memory_desc_t *src2_desc) {
    CHECK_ARG(post_ops && index >= 0 && index < (int)post_ops->entries.size());
    const post_op_entry_t &e = post_ops->entries[index];
    CHECK_ARG(e.kind == dnnl_binary);
    if (alg) *alg = e.alg;
    if (src1_desc) *src1_desc = &e.src1;
    if (src2_desc) *src2_desc = e.alg == dnnl_binary_select ? &e.src2 : nullptr;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_post_ops_get_params_binary(const_dnnl_post_ops_t post_ops, int index,
        dnnl_alg_kind_t *alg, const_dnnl_memory_desc_t *src1_desc) {
    CHECK_ARG(post_ops && index >= 0 && index < (int)post_ops->entries.size());
    const post_op_entry_t &e = post_ops->entries[index];
    CHECK_ARG(e.kind == dnnl_binary);
    if (alg) *alg = e.alg;
    if (src1_desc) *src1_desc = &e.src1;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_post_ops_append_prelu(dnnl_post_ops_t post_ops, int mask) {
    CHECK_ARG(post_ops && mask >= 0);
    if (po_full(post_ops)) return dnnl_out_of_memory;
    post_op_entry_t e;
    e.kind = dnnl_prelu; e.mask = mask;
    post_ops->entries.push_back(e);
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_post_ops_get_params_prelu(const_dnnl_post_ops_t post_ops, int index, int *mask) {
    CHECK_ARG(post_ops && index >= 0 && index < (int)post_ops->entries.size());
    const post_op_entry_t &e = post_ops->entries[index];
    CHECK_ARG(e.kind == dnnl_prelu);
    if (mask) *mask = e.mask;
    return dnnl_success;
}

// ---- matmul primitive descriptor
// ---- grouped (mixture-of-experts) matmul: descriptor rules of grouped_matmul_desc_init and
// grouped_matmul_attr_check (src/common/matmul.cpp:43-259) and the dispatch rules of ref_grouped_t::pd_t::init
// (src/cpu/matmul/ref_grouped_gemm.hpp:60-270), lowered to mi355_grouped_desc_t.
namespace {
bool is_tag_3d(const dnnl_memory_desc &m, bool acb) {
    if (m.kind != dnnl_blocked || m.ndims != 3) return false;
    const dim_t G = m.dims[0], K = m.dims[1], N = m.dims[2];
    (void)G;
    return acb ? (m.strides[0] == K * N && m.strides[1] == 1 && m.strides[2] == K)
               : (m.strides[0] == K * N && m.strides[1] == N && m.strides[2] == 1);
}

dnnl_status_t grouped_pd_init(dnnl_primitive_desc &pd, const dnnl_memory_desc &src, const dnnl_memory_desc &wei_in,
        const dnnl_memory_desc *bias, const dnnl_memory_desc &dst_in) {
    for (const dnnl_memory_desc *m : {&src, &wei_in, &dst_in}) CHECK_ARG(m->kind != dnnl_format_kind_host_scalar);
    // Weights given with format_tag::any (the reference's ref_grouped_t takes abc / acb only): K-contiguous
    // (acb) for the operand types the matrix-core tiles take, as for the plain matmul; row-major otherwise.
    // The caller reads the layout back with dnnl_primitive_desc_query_md and reorders once.
    dnnl_memory_desc wei = wei_in;
    if (wei.kind == dnnl_format_kind_any && wei.ndims == 3 && !wei.grouped) {
        const bool tiles = wei.dt == src.dt
                && (is_fp8(wei.dt) || wei.dt == dnnl_bf16 || wei.dt == dnnl_f16 || wei.dt == dnnl_s8 || wei.dt == dnnl_f4_e2m1);
        const bool both_fp8 = is_fp8(wei.dt) && is_fp8(src.dt);
        if (tiles || both_fp8) {
            const int acb[3] = {0, 2, 1};
            wei.set_dense(acb);
        } else {
            wei.set_dense();
        }
    }
    if (bias) CHECK_ARG(bias->kind != dnnl_format_kind_host_scalar);
    CHECK_UNIMPL(src.grouped);
    const bool x3 = dst_in.grouped && !wei.grouped, x2 = wei.grouped && !dst_in.grouped;
    CHECK_UNIMPL(x3 || x2);
    const dnnl_memory_desc &variant = x3 ? dst_in : wei;
    CHECK_UNIMPL(src.var_dim == (x3 ? 0 : 1) && variant.var_dim == 0);
    CHECK_UNIMPL(src.group_count == variant.group_count);
    const dim_t G = src.group_count;
    CHECK_UNIMPL(src.ndims == 2);
    CHECK_UNIMPL(wei.ndims == (x3 ? 3 : 2));
    CHECK_UNIMPL(dst_in.ndims == (x3 ? 2 : 3));
    CHECK_UNIMPL((x3 ? wei.dims[0] : dst_in.dims[0]) == G);
    CHECK_UNIMPL(src.dims[0] == dst_in.dims[dst_in.ndims - 2]);
    CHECK_UNIMPL(src.dims[1] == wei.dims[wei.ndims - 2]);
    CHECK_UNIMPL(dst_in.dims[dst_in.ndims - 1] == wei.dims[wei.ndims - 1]);
    const dim_t N = wei.dims[wei.ndims - 1];
    dnnl_memory_desc dst = dst_in;
    if (x3) {
        CHECK_UNIMPL(is_tag_3d(wei, false) || is_tag_3d(wei, true)); // dense abc or acb
        if (bias) {
            CHECK_UNIMPL(!bias->grouped && bias->kind == dnnl_blocked && bias->ndims == 2);
            CHECK_UNIMPL(bias->dims[0] == G && bias->dims[1] == N);
            CHECK_UNIMPL(bias->strides[0] == N && bias->strides[1] == 1);
        }
    } else {
        CHECK_UNIMPL(!bias);
        if (dst.kind == dnnl_format_kind_any) dst.set_dense();
        CHECK_UNIMPL(dst.kind == dnnl_blocked);
    }
    CHECK_UNIMPL(accum_dt(src.dt, wei.dt, dst.dt) != dnnl_data_type_undef);

    mi355_grouped_desc_t &D = pd.gdesc;
    memset(&D, 0, sizeof(D));
    D.pattern = x3 ? MI355_GROUPED_2DX3D : MI355_GROUPED_2DX2D;
    D.group_count = G;
    D.total = x3 ? src.dims[0] : src.dims[1];
    D.M = x3 ? 0 : src.dims[0];
    D.K = x3 ? src.dims[1] : 0;
    D.N = N;
    D.src_dt = src.dt; D.wei_dt = wei.dt; D.dst_dt = dst.dt;
    D.bias_dt = bias ? (int)bias->dt : MI355_DT_UNDEF;
    if (x3) for (int i = 0; i < 3; ++i) D.wei_stride[i] = wei.strides[i];
    else for (int i = 0; i < 3; ++i) D.dst_stride[i] = dst.strides[i];

    // ---- attributes (grouped_matmul_attr_check, then the implementation's own rules)
    const dnnl_primitive_attr &a = pd.attr;
    const bool defaults = a.scales.empty() && a.zero_points.empty() && a.reductions.empty() && a.post_ops.entries.empty()
            && a.fpmath == dnnl_fpmath_mode_strict && !a.apply_to_int && a.acc_mode == dnnl_accumulation_mode_strict;
    if (!defaults) {
        CHECK_UNIMPL(x3); // the variable-K pattern takes default attributes only
        CHECK_UNIMPL(a.reductions.empty() && a.acc_mode == dnnl_accumulation_mode_strict);
        auto fp_plain = [](int dt) { return dt == dnnl_f32 || dt == dnnl_bf16 || dt == dnnl_f16; };
        const quant_entry_t *ss = a.find(a.scales, DNNL_ARG_SRC), *ws = a.find(a.scales, DNNL_ARG_WEIGHTS);
        const quant_entry_t *sz = a.find(a.zero_points, DNNL_ARG_SRC), *wz = a.find(a.zero_points, DNNL_ARG_WEIGHTS);
        CHECK_UNIMPL(IMPLICATION(fp_plain(src.dt), !ss));
        CHECK_UNIMPL(IMPLICATION(fp_plain(wei.dt), !ws));
        CHECK_UNIMPL(!a.find(a.scales, DNNL_ARG_DST) && !a.find(a.zero_points, DNNL_ARG_DST));
        for (const auto &kv : a.scales) CHECK_UNIMPL(!kv.second.is_dynamic() && !kv.second.on_host);
        for (const auto &kv : a.zero_points) CHECK_UNIMPL(!kv.second.on_host);
        const dim_t K = D.K;
        auto scale_dt_ok = [](int dt) {
            return dt == dnnl_f32 || dt == dnnl_bf16 || dt == dnnl_f16 || dt == dnnl_e8m0 || dt == dnnl_f8_e4m3
                    || dt == dnnl_f8_e5m2;
        };
        // src: per row (mask M) or per row and K group (mask M|K, groups {1, gK}); weights [G][K][N]: per group and
        // column (mask G|N) or with K groups (mask G|K|N, groups {gK, 1})
        auto src_entry = [&](const quant_entry_t *q, int64_t *gk) -> dnnl_status_t {
            *gk = 0;
            if (!q) return dnnl_success;
            CHECK_UNIMPL(q->mask == 1 || q->mask == 3);
            if (q->group_ndims != 0) {
                CHECK_UNIMPL(q->group(0) == 1 && q->group(1) > 1 && K % q->group(1) == 0);
                *gk = q->group(1);
            }
            CHECK_UNIMPL((q->mask == 3) == (*gk > 1));
            return dnnl_success;
        };
        auto wei_entry = [&](const quant_entry_t *q, int64_t *gk) -> dnnl_status_t {
            *gk = 0;
            if (!q) return dnnl_success;
            CHECK_UNIMPL(q->mask == 5 || q->mask == 7);
            if (q->group_ndims != 0) {
                CHECK_UNIMPL(q->group(0) > 1 && K % q->group(0) == 0 && q->group(1) == 1);
                *gk = q->group(0);
            }
            CHECK_UNIMPL((q->mask == 7) == (*gk > 1));
            return dnnl_success;
        };
        dnnl_status_t st;
        if ((st = src_entry(ss, &D.src_scale_gk)) || (st = wei_entry(ws, &D.wei_scale_gk))
                || (st = src_entry(sz, &D.src_zp_gk)) || (st = wei_entry(wz, &D.wei_zp_gk)))
            return st;
        if (ss) CHECK_UNIMPL(scale_dt_ok(ss->dt));
        if (ws) CHECK_UNIMPL(scale_dt_ok(ws->dt));
        if (sz) CHECK_UNIMPL(is_int8(src.dt) && (sz->dt == dnnl_u8 || sz->dt == dnnl_s8 || sz->dt == dnnl_s32));
        if (wz)
            CHECK_UNIMPL((is_int8(wei.dt) || wei.dt == dnnl_s4 || wei.dt == dnnl_u4)
                    && (wz->dt == dnnl_u8 || wz->dt == dnnl_s8 || wz->dt == dnnl_u4 || wz->dt == dnnl_s4
                            || wz->dt == dnnl_s32));
        if (D.src_scale_gk > 1 && D.wei_scale_gk > 1)
            CHECK_UNIMPL(D.src_scale_gk % D.wei_scale_gk == 0 || D.wei_scale_gk % D.src_scale_gk == 0);
        if (ws && wz) CHECK_UNIMPL((ws->group_ndims ? ws->group(0) : 1) == (wz->group_ndims ? wz->group(0) : 1));
        D.src_scale_dt = ss ? (int)ss->dt : MI355_DT_UNDEF;
        D.wei_scale_dt = ws ? (int)ws->dt : MI355_DT_UNDEF;
        D.src_zp_dt = sz ? (int)sz->dt : MI355_DT_UNDEF;
        D.wei_zp_dt = wz ? (int)wz->dt : MI355_DT_UNDEF;
        D.fpmath_apply_to_int = a.apply_to_int;
        // post-ops: eltwise, and multiplication by a per-group, per-row or per-element operand
        CHECK_UNIMPL(a.post_ops.entries.size() <= MI355_MAX_POST_OPS);
        const dim_t total_M = dst.dims[0];
        for (size_t i = 0; i < a.post_ops.entries.size(); ++i) {
            const post_op_entry_t &e = a.post_ops.entries[i];
            mi355_grouped_post_op_t &po = D.post_ops[i];
            CHECK_UNIMPL(e.kind == dnnl_eltwise || e.kind == dnnl_binary);
            if (e.kind == dnnl_eltwise) {
                po.kind = MI355_PO_ELTWISE;
                po.alg = e.alg; po.alpha = e.alpha; po.beta = e.beta; po.scale = e.scale;
                continue;
            }
            CHECK_UNIMPL(e.alg == dnnl_binary_mul);
            CHECK_ARG(e.src1.ndims == dst.ndims);
            po.kind = MI355_PO_BINARY;
            po.alg = e.alg;
            po.dt = e.src1.dt;
            po.bin_m = e.src1.dims[0];
            po.bin_n = e.src1.dims[1];
            if (e.src1.grouped) {
                CHECK_UNIMPL(e.src1.group_count == dst.group_count && e.src1.var_dim == dst.var_dim);
                CHECK_UNIMPL(po.bin_m == total_M && (po.bin_n == N || po.bin_n == 1));
                po.grouped = 1;
            } else {
                dnnl_memory_desc b = e.src1;
                if (b.kind == dnnl_format_kind_any) b.set_dense();
                CHECK_UNIMPL(b.kind == dnnl_blocked);
                CHECK_UNIMPL(po.bin_n == 1 || (b.strides[0] == po.bin_n && b.strides[1] == 1));
                CHECK_UNIMPL((po.bin_m == G || po.bin_m == total_M) && IMPLICATION(po.bin_m == G, po.bin_n == 1));
                CHECK_UNIMPL(po.bin_n == 1 || po.bin_n == N);
            }
        }
        D.n_post_ops = (int)a.post_ops.entries.size();
    }
    CHECK_UNIMPL(mi355_grouped_matmul_query(&D) == MI355_SUCCESS);
    pd.grouped = true;
    pd.src = src; pd.wei = wei; pd.dst = dst;
    pd.with_bias = bias != nullptr;
    if (bias) pd.bias = *bias;
    pd.impl_name = mi355_grouped_matmul_impl(&D);
    pd.impls.assign(1, MI355_IMPL_REF);
    pd.impl_pos = 0;
    pd.scratch_bytes = 0;
    return dnnl_success;
}
} // namespace

DNNL_EXPORT dnnl_status_t dnnl_matmul_primitive_desc_create(dnnl_primitive_desc_t *primitive_desc,
        dnnl_engine_t engine, const_dnnl_memory_desc_t src_desc, const_dnnl_memory_desc_t weights_desc,
        const_dnnl_memory_desc_t bias_desc, const_dnnl_memory_desc_t dst_desc, const_dnnl_primitive_attr_t attr) {
    CHECK_ARG(primitive_desc && engine);
    CHECK_ARG(src_desc && weights_desc && dst_desc);
    const dnnl_memory_desc *bias = (bias_desc && !bias_desc->is_zero()) ? bias_desc : nullptr;
    if (src_desc->kind == dnnl_format_kind_sparse || weights_desc->kind == dnnl_format_kind_sparse
            || dst_desc->kind == dnnl_format_kind_sparse) {
        std::unique_ptr<dnnl_primitive_desc> gpd(new dnnl_primitive_desc);
        if (attr) gpd->attr = *attr;
        gpd->engine = engine;
        const dnnl_status_t gs = grouped_pd_init(*gpd, *src_desc, *weights_desc, bias, *dst_desc);
        if (gs) return gs;
        if (verbose_level() >= 1)
            fprintf(stderr, "onednn_verbose,v1,primitive,create:dispatch,gpu,matmul,%s\n", gpd->impl_name.c_str());
        *primitive_desc = gpd.release();
        return dnnl_success;
    }
    dnnl_status_t st = check_shapes(*src_desc, *weights_desc, bias, *dst_desc);
    if (st) return st;
    CHECK_ARG(accum_dt(src_desc->dt, weights_desc->dt, dst_desc->dt) != dnnl_data_type_undef);
    std::unique_ptr<dnnl_primitive_desc> pd(new dnnl_primitive_desc);
    if (attr) pd->attr = *attr;
    pd->runtime = src_desc->has_runtime() || weights_desc->has_runtime() || dst_desc->has_runtime()
            || (bias && bias->has_runtime());
    if (pd->runtime) {
        // attribute rules that involve an unknown dim are checked at execution
        dnnl_memory_desc ps = *src_desc, pw = *weights_desc, pdst = *dst_desc;
        for (dnnl_memory_desc *m : {&ps, &pw, &pdst})
            for (int i = 0; i < m->ndims; ++i)
                if (m->dims[i] == DNNL_RUNTIME_DIM_VAL) m->dims[i] = k_probe_dim;
        st = check_attr(ps, pw, pdst, pd->attr);
        for (const post_op_entry_t &e : pd->attr.post_ops.entries)
            if (e.kind == dnnl_binary) CHECK_UNIMPL(!e.src1.has_runtime());
    } else {
        st = check_attr(*src_desc, *weights_desc, *dst_desc, pd->attr);
    }
    if (st) return st;
    pd->engine = engine;
    pd->src = *src_desc; pd->wei = *weights_desc; pd->dst = *dst_desc;
    pd->with_bias = bias != nullptr;
    if (bias) pd->bias = *bias;
    // format `any`: the implementation picks the layout and the caller asks
    // weights_desc() for it, as with the reference's blocked weights
    // (brgemm_matmul_utils.cpp: set_or_check_B_tag).  The MFMA GEMM families
    // consume K-contiguous weight columns, so int8 / fp8 / fp4 / bf16 / f16 / f32 weights resolve
    // to the plain transposed tag (ba, acb, ...); everything else resolves to
    // row-major (matmul_pd_t::set_default_formats, matmul_pd.hpp:419-431).
    bool try_packed = false;
    if (pd->wei.kind == dnnl_format_kind_any) {
        dnnl_memory_desc &w = pd->wei;
        w.set_dense();
        // 4-bit decode weights: the 64-column packing, if the packed decode
        // kernel takes the problem and N gives it enough workgroups to fill
        // the device (decided below, once the descriptor is lowered)
        try_packed = pd->src.dt == dnnl_bf16 && (w.dt == dnnl_s4 || w.dt == dnnl_u4) && pd->attr.apply_to_int
                && w.ndims == 2 && w.dims[1] >= 64 * 128;
        const bool mfma_operands = (is_int8(pd->src.dt) && is_int8(w.dt)) || (is_fp8(pd->src.dt) && is_fp8(w.dt))
                || (pd->src.dt == dnnl_f4_e2m1 && w.dt == dnnl_f4_e2m1)
                || (pd->src.dt == w.dt && (w.dt == dnnl_bf16 || w.dt == dnnl_f16 || w.dt == dnnl_f32));
        if (mfma_operands && w.ndims >= 2) {
            w.strides[w.ndims - 2] = 1;
            w.strides[w.ndims - 1] = w.dims[w.ndims - 2] == 0 ? 1 : w.dims[w.ndims - 2];
        }
    }
    for (dnnl_memory_desc *m : {&pd->src, &pd->dst, &pd->bias})
        if (m->kind == dnnl_format_kind_any) m->set_dense();
    st = check_dtypes(*pd);
    if (st) return st;
    if (pd->runtime) {
        // the kernel family is chosen per execution, from the real shapes
        pd->impls.assign(1, MI355_IMPL_AUTO);
        pd->impl_pos = 0;
        pd->impl_name = "hip:runtime_dims:any";
        pd->desc.impl = MI355_IMPL_AUTO;
        if (verbose_level() >= 1)
            fprintf(stderr, "onednn_verbose,v1,primitive,create:dispatch,gpu,matmul,%s\n", pd->impl_name.c_str());
        *primitive_desc = pd.release();
        return dnnl_success;
    }
    if (try_packed) {
        const dnnl_memory_desc plain = pd->wei;
        pd->wei.kind = dnnl_format_kind_opaque;
        pd->wei.packing = MI355_WEI_PACK_WOQ64;
        for (int i = 0; i < pd->wei.ndims; ++i) pd->wei.strides[i] = 0;
        int chosen = 0;
        if (lower(*pd) != dnnl_success
                || mi355_matmul_query(&pd->desc, MI355_IMPL_WOQ_PACKED, &chosen) != MI355_SUCCESS)
            pd->wei = plain;
    }
    st = dispatch(*pd);
    if (st) return st;
    if (verbose_level() >= 1)
        fprintf(stderr, "onednn_verbose,v1,primitive,create:dispatch,gpu,matmul,%s\n", pd->impl_name.c_str());
    *primitive_desc = pd.release();
    return dnnl_success;
}

// ---- inner product primitive descriptor
namespace {
// memory order of the dims of a plain tensor, outermost first (ties keep the logical order)
void memory_order(const dnnl_memory_desc &md, int *perm) {
    for (int i = 0; i < md.ndims; ++i) perm[i] = i;
    std::stable_sort(perm, perm + md.ndims, [&](int a, int b) { return md.strides[a] > md.strides[b]; });
}
// ip_desc_init, src/common/inner_product.cpp:43-112 (the checks that do not depend on the propagation kind)
dnnl_status_t ip_check_shapes(const dnnl_memory_desc *src, const dnnl_memory_desc *wei, const dnnl_memory_desc *bias,
        const dnnl_memory_desc *dst) {
    CHECK_ARG(src && wei && dst);
    for (const dnnl_memory_desc *m : {src, wei, bias, dst})
        if (m) CHECK_ARG(m->kind != dnnl_format_kind_host_scalar);
    for (const dnnl_memory_desc *m : {src, wei, bias, dst})
        if (m) CHECK_UNIMPL(!m->has_runtime());
    CHECK_ARG(accum_dt(src->dt, wei->dt, dst->dt) != dnnl_data_type_undef);
    CHECK_ARG(wei->nelems() != 0);
    CHECK_ARG(src->ndims >= 2 && src->ndims <= 5);
    CHECK_ARG(dst->ndims == 2);
    CHECK_ARG(wei->ndims == src->ndims);
    if (bias) CHECK_ARG(bias->ndims == 1 && bias->dims[0] == dst->dims[1]);
    CHECK_ARG(src->dims[0] == dst->dims[0]);
    for (int i = 1; i < src->ndims; ++i) CHECK_ARG(src->dims[i] == wei->dims[i]);
    CHECK_ARG(dst->dims[1] == wei->dims[0]);
    return dnnl_success;
}
} // namespace

DNNL_EXPORT dnnl_status_t dnnl_inner_product_forward_primitive_desc_create(dnnl_primitive_desc_t *primitive_desc,
        dnnl_engine_t engine, dnnl_prop_kind_t prop_kind, const_dnnl_memory_desc_t src_desc,
        const_dnnl_memory_desc_t weights_desc, const_dnnl_memory_desc_t bias_desc, const_dnnl_memory_desc_t dst_desc,
        const_dnnl_primitive_attr_t attr) {
    CHECK_ARG(primitive_desc && engine);
    CHECK_ARG(prop_kind == dnnl_forward_training || prop_kind == dnnl_forward_inference);
    const dnnl_memory_desc *bias_in
            = (bias_desc && !bias_desc->is_zero() && bias_desc->kind != dnnl_format_kind_undef) ? bias_desc : nullptr;
    dnnl_status_t st = ip_check_shapes(src_desc, weights_desc, bias_in, dst_desc);
    if (st) return st;
    dnnl_memory_desc src = *src_desc, wei = *weights_desc, dst = *dst_desc, bias;
    if (bias_in) bias = *bias_in;
    const int nd = src.ndims;
    for (const dnnl_memory_desc *m : {&src, &wei, &dst})
        CHECK_UNIMPL(m->kind == dnnl_blocked || m->kind == dnnl_format_kind_any);
    CHECK_UNIMPL(!src.grouped && !wei.grouped && !dst.grouped);

    // ip_attr_check, src/common/inner_product.cpp:114-186; the data types are those of the two naive
    // implementations (ref_inner_product.hpp:52-72, ref_inner_product_int8.hpp:52-66)
    const bool int8 = is_int8(src.dt);
    if (int8) {
        CHECK_UNIMPL(wei.dt == dnnl_s8);
        CHECK_UNIMPL(dst.dt == dnnl_f32 || dst.dt == dnnl_f16 || dst.dt == dnnl_bf16 || dst.dt == dnnl_s32
                || is_int8(dst.dt));
        if (bias_in)
            CHECK_UNIMPL(bias.dt == dnnl_f32 || bias.dt == dnnl_f16 || bias.dt == dnnl_bf16 || bias.dt == dnnl_s32
                    || is_int8(bias.dt));
    } else {
        CHECK_UNIMPL(src.dt == dnnl_f32 || src.dt == dnnl_bf16 || src.dt == dnnl_f16 || is_fp8(src.dt));
        CHECK_UNIMPL(wei.dt == src.dt);
        CHECK_UNIMPL(dst.dt == dnnl_f32 || dst.dt == src.dt);
        if (bias_in) CHECK_UNIMPL(bias.dt == dnnl_f32 || bias.dt == src.dt);
    }
    dnnl_primitive_attr lowered_attr;
    if (attr) {
        const dnnl_primitive_attr &a = *attr;
        CHECK_UNIMPL(a.zero_points.empty() && a.reductions.empty() && !a.with_dropout() && a.rounding.empty());
        const bool scales_allowed = int8 || is_int8(dst.dt) || dst.dt == dnnl_s32; // the gpu-engine rule, :133-137
        CHECK_UNIMPL(IMPLICATION(!a.scales.empty(), scales_allowed));
        for (const auto &kv : a.scales) {
            const quant_entry_t &q = kv.second;
            CHECK_UNIMPL(kv.first == DNNL_ARG_SRC || kv.first == DNNL_ARG_WEIGHTS || kv.first == DNNL_ARG_DST);
            CHECK_UNIMPL(kv.first == DNNL_ARG_WEIGHTS ? (q.mask == 0 || q.mask == 1) : q.mask == 0);
            CHECK_UNIMPL(q.group_ndims == 0 && q.dt == dnnl_f32 && !q.is_dynamic());
            CHECK_UNIMPL(!q.on_host);
            CHECK_UNIMPL(int8); // the implementations read scales on the integer path only
        }
        for (const post_op_entry_t &e : a.post_ops.entries)
            CHECK_UNIMPL(e.kind == dnnl_binary || e.kind == dnnl_eltwise || e.kind == dnnl_prelu || e.kind == dnnl_sum);
        lowered_attr = a;
        auto it = lowered_attr.scales.find(DNNL_ARG_WEIGHTS);
        if (it != lowered_attr.scales.end() && it->second.mask == 1) it->second.mask = 2; // oc is dim 1 of [K, oc]
    }

    // format `any` (cpu_inner_product_fwd_pd_t::set_default_params, src/cpu/cpu_inner_product_pd.hpp:162-209):
    // src and weights share one order of dims; the mb / oc dim never ends up innermost
    int perm[DNNL_MAX_NDIMS];
    auto outer_first = [&](int *pm) {
        if (nd > 1 && pm[nd - 1] == 0) {
            for (int i = nd - 1; i > 0; --i) pm[i] = pm[i - 1];
            pm[0] = 0;
        }
    };
    if (src.kind == dnnl_format_kind_any) {
        if (wei.kind == dnnl_format_kind_any) {
            src.set_dense();
        } else {
            memory_order(wei, perm);
            outer_first(perm);
            src.set_dense(perm);
        }
    }
    if (wei.kind == dnnl_format_kind_any) {
        memory_order(src, perm);
        outer_first(perm);
        wei.set_dense(perm);
    }
    if (dst.kind == dnnl_format_kind_any) dst.set_dense();
    if (bias_in && bias.kind == dnnl_format_kind_any) bias.set_dense();
    if (bias_in) CHECK_UNIMPL(bias.kind == dnnl_blocked);

    // The reduced dims (ic and the spatial ones) as one K: they must be dense, and in the same order, in both
    // tensors.  Dims of extent one do not matter.
    int order[DNNL_MAX_NDIMS], n_inner = 0;
    memory_order(src, perm);
    for (int i = 0; i < nd; ++i)
        if (perm[i] != 0 && src.dims[perm[i]] != 1) order[n_inner++] = perm[i];
    dim_t K = 1, src_ks = 1, wei_ks = 1;
    for (int i = 1; i < nd; ++i) K *= src.dims[i];
    if (n_inner > 0 && K > 0) {
        src_ks = src.strides[order[n_inner - 1]];
        wei_ks = wei.strides[order[n_inner - 1]];
        for (int i = 0; i + 1 < n_inner; ++i) {
            const dim_t inner = src.dims[order[i + 1]];
            CHECK_UNIMPL(src.strides[order[i]] == src.strides[order[i + 1]] * inner);
            CHECK_UNIMPL(wei.strides[order[i]] == wei.strides[order[i + 1]] * inner);
        }
    }
    dnnl_memory_desc src2, wei2, bias2;
    src2.ndims = 2; src2.dt = src.dt; src2.kind = dnnl_blocked;
    src2.dims[0] = src.dims[0]; src2.dims[1] = K;
    src2.strides[0] = src.strides[0]; src2.strides[1] = src_ks;
    wei2.ndims = 2; wei2.dt = wei.dt; wei2.kind = dnnl_blocked;
    wei2.dims[0] = K; wei2.dims[1] = wei.dims[0];
    wei2.strides[0] = wei_ks; wei2.strides[1] = wei.strides[0];
    if (bias_in) {
        bias2.ndims = 2; bias2.dt = bias.dt; bias2.kind = dnnl_blocked;
        bias2.dims[0] = 1; bias2.dims[1] = bias.dims[0];
        bias2.strides[1] = bias.strides[0]; bias2.strides[0] = bias.strides[0] * (bias.dims[0] ? bias.dims[0] : 1);
    }
    dnnl_primitive_desc_t mm = nullptr;
    st = dnnl_matmul_primitive_desc_create(&mm, engine, &src2, &wei2, bias_in ? &bias2 : nullptr, &dst, &lowered_attr);
    if (st) return st;
    mm->inner_product = true;
    mm->prop_kind = (int)prop_kind;
    mm->ip_src = src; mm->ip_wei = wei;
    if (bias_in) mm->ip_bias = bias;
    if (attr) mm->ip_attr = *attr;
    if (verbose_level() >= 1)
        fprintf(stderr, "onednn_verbose,v1,primitive,create:dispatch,gpu,inner_product,%s\n", mm->impl_name.c_str());
    *primitive_desc = mm;
    return dnnl_success;
}

// Inner product, backward (src/common/inner_product.cpp:205-230; the naive implementations
// src/cpu/ref_inner_product.cpp:100-217 and their data types, ref_inner_product.hpp:118-139, :196-218): both are
// matmuls over the tensors as they lie.
//   data:     diff_src[mb, k]     = sum_oc diff_dst[mb, oc] * weights[oc, k]    [mb, oc] x [oc, K]
//   weights:  diff_weights[oc, k] = sum_mb diff_dst[mb, oc] * src[mb, k]        [oc, mb] x [mb, K], src = diff_dst^T
//             diff_bias[oc]       = sum_mb diff_dst[mb, oc]                     column sums, in the reference's order
// k = (ic, spatial) flattened: the reduced dims must be dense and in the same memory order in both tensors that carry
// them, as in the forward lowering.
namespace {
// the flattened K of a tensor [x, ic, spatial...]: element stride of k in `ks`; false if the dims do not flatten
bool ip_flatten(const dnnl_memory_desc &t, const int *order, int n_inner, dim_t *ks) {
    *ks = 1;
    if (n_inner == 0) return true;
    *ks = t.strides[order[n_inner - 1]];
    for (int i = 0; i + 1 < n_inner; ++i)
        if (t.strides[order[i]] != t.strides[order[i + 1]] * t.dims[order[i + 1]]) return false;
    return true;
}
dnnl_status_t ip_backward_create(dnnl_primitive_desc_t *primitive_desc, dnnl_engine_t engine, bool data,
        const dnnl_memory_desc *x_desc /* diff_src | src */, const dnnl_memory_desc *w_desc /* weights | diff_weights */,
        const dnnl_memory_desc *bias_in, const dnnl_memory_desc *ddst_desc, const_dnnl_primitive_attr_t attr) {
    dnnl_memory_desc x = *x_desc, w = *w_desc, dd = *ddst_desc, bias;
    if (bias_in) bias = *bias_in;
    const int nd = x.ndims;
    for (const dnnl_memory_desc *m : {&x, &w, &dd})
        CHECK_UNIMPL(m->kind == dnnl_blocked || m->kind == dnnl_format_kind_any);
    CHECK_UNIMPL(!x.grouped && !w.grouped && !dd.grouped);
    // no attributes on the backward passes of the naive implementations (attr is default or absent)
    if (attr) {
        const dnnl_primitive_attr &a = *attr;
        CHECK_UNIMPL(a.scales.empty() && a.zero_points.empty() && a.reductions.empty() && a.post_ops.entries.empty()
                && !a.with_dropout() && a.rounding.empty());
    }
    auto fp = [](dnnl_data_type_t dt) { return dt == dnnl_f32 || dt == dnnl_bf16 || dt == dnnl_f16; };
    if (data) { // diff_src in {f32, wei}, wei in {f32, bf16, f16}, diff_dst == wei
        CHECK_UNIMPL(fp(w.dt) && dd.dt == w.dt && (x.dt == dnnl_f32 || x.dt == w.dt));
    } else {    // src in {f32, bf16, f16}, diff_dst == src, diff_weights in {f32, src}, diff_bias in {f32, src}
        CHECK_UNIMPL(fp(x.dt) && dd.dt == x.dt && (w.dt == dnnl_f32 || w.dt == x.dt));
        if (bias_in) CHECK_UNIMPL(bias.dt == dnnl_f32 || bias.dt == x.dt);
    }
    // format `any`: as in the forward pass, the two tensors with reduced dims take each other's order
    int perm[DNNL_MAX_NDIMS];
    auto outer_first = [&](int *pm) {
        if (nd > 1 && pm[nd - 1] == 0) {
            for (int i = nd - 1; i > 0; --i) pm[i] = pm[i - 1];
            pm[0] = 0;
        }
    };
    if (x.kind == dnnl_format_kind_any) {
        if (w.kind == dnnl_format_kind_any) {
            x.set_dense();
        } else {
            memory_order(w, perm);
            outer_first(perm);
            x.set_dense(perm);
        }
    }
    if (w.kind == dnnl_format_kind_any) {
        memory_order(x, perm);
        outer_first(perm);
        w.set_dense(perm);
    }
    if (dd.kind == dnnl_format_kind_any) dd.set_dense();
    if (bias_in && bias.kind == dnnl_format_kind_any) bias.set_dense();
    if (bias_in) CHECK_UNIMPL(bias.kind == dnnl_blocked && bias.strides[0] == 1 && dd.strides[1] == 1);

    int order[DNNL_MAX_NDIMS], n_inner = 0;
    memory_order(x, perm);
    for (int i = 0; i < nd; ++i)
        if (perm[i] != 0 && x.dims[perm[i]] != 1) order[n_inner++] = perm[i];
    dim_t K = 1, x_ks = 1, w_ks = 1;
    for (int i = 1; i < nd; ++i) K *= x.dims[i];
    CHECK_UNIMPL(ip_flatten(x, order, n_inner, &x_ks) && ip_flatten(w, order, n_inner, &w_ks));
    const dim_t MB = x.dims[0], OC = w.dims[0];
    auto md2 = [](dnnl_data_type_t dt, dim_t d0, dim_t d1, dim_t s0, dim_t s1) {
        dnnl_memory_desc m;
        m.ndims = 2; m.dt = dt; m.kind = dnnl_blocked;
        m.dims[0] = d0; m.dims[1] = d1; m.strides[0] = s0; m.strides[1] = s1;
        return m;
    };
    dnnl_memory_desc a2, b2, c2;
    if (data) {
        a2 = md2(dd.dt, MB, OC, dd.strides[0], dd.strides[1]);
        b2 = md2(w.dt, OC, K, w.strides[0], w_ks);
        c2 = md2(x.dt, MB, K, x.strides[0], x_ks);
    } else {
        a2 = md2(dd.dt, OC, MB, dd.strides[1], dd.strides[0]);
        b2 = md2(x.dt, MB, K, x.strides[0], x_ks);
        c2 = md2(w.dt, OC, K, w.strides[0], w_ks);
    }
    dnnl_primitive_desc_t mm = nullptr;
    const dnnl_status_t st = dnnl_matmul_primitive_desc_create(&mm, engine, &a2, &b2, nullptr, &c2, nullptr);
    if (st) return st;
    mm->inner_product = true;
    mm->prop_kind = data ? (int)dnnl_backward_data : (int)dnnl_backward_weights;
    mm->ip_src = x; mm->ip_wei = w; mm->ip_dst = dd;
    mm->ip_diff_bias = bias_in != nullptr;
    if (bias_in) mm->ip_bias = bias;
    if (attr) mm->ip_attr = *attr;
    if (verbose_level() >= 1)
        fprintf(stderr, "onednn_verbose,v1,primitive,create:dispatch,gpu,inner_product,%s\n", mm->impl_name.c_str());
    *primitive_desc = mm;
    return dnnl_success;
}
} // namespace

DNNL_EXPORT dnnl_status_t dnnl_inner_product_backward_data_primitive_desc_create(dnnl_primitive_desc_t *primitive_desc,
        dnnl_engine_t engine, const_dnnl_memory_desc_t diff_src_desc, const_dnnl_memory_desc_t weights_desc,
        const_dnnl_memory_desc_t diff_dst_desc, const_dnnl_primitive_desc_t hint_fwd_pd,
        const_dnnl_primitive_attr_t attr) {
    (void)hint_fwd_pd;
    CHECK_ARG(primitive_desc && engine);
    dnnl_status_t st = ip_check_shapes(diff_src_desc, weights_desc, nullptr, diff_dst_desc);
    if (st) return st;
    return ip_backward_create(primitive_desc, engine, true, diff_src_desc, weights_desc, nullptr, diff_dst_desc, attr);
}
DNNL_EXPORT dnnl_status_t dnnl_inner_product_backward_weights_primitive_desc_create(
        dnnl_primitive_desc_t *primitive_desc, dnnl_engine_t engine, const_dnnl_memory_desc_t src_desc,
        const_dnnl_memory_desc_t diff_weights_desc, const_dnnl_memory_desc_t diff_bias_desc,
        const_dnnl_memory_desc_t diff_dst_desc, const_dnnl_primitive_desc_t hint_fwd_pd,
        const_dnnl_primitive_attr_t attr) {
    (void)hint_fwd_pd;
    CHECK_ARG(primitive_desc && engine);
    const dnnl_memory_desc *b = (diff_bias_desc && !diff_bias_desc->is_zero()
            && diff_bias_desc->kind != dnnl_format_kind_undef) ? diff_bias_desc : nullptr;
    dnnl_status_t st = ip_check_shapes(src_desc, diff_weights_desc, b, diff_dst_desc);
    if (st) return st;
    return ip_backward_create(primitive_desc, engine, false, src_desc, diff_weights_desc, b, diff_dst_desc, attr);
}

// Scaled dot-product attention (src/common/sdpa_test_iface.hpp:23-33, sdpa_utils.hpp:51-82 for the shape rules,
// sdpa_pd.hpp, the reference kernel src/gpu/intel/sdpa/ref.cl): forward only, 4-D tensors
//   queries [b][h][sq][d], keys [b][hk][d][sk], values [b][hk][sk][dv], dst [b][h][sq][dv], any strides;
//   mask [..][..][..][..] of dims 1 or the full ones; scale: one value in device memory.
// Lowered to   scores = Q x K (f32)  ->  probs = softmax(scores * scale + mask)  ->  dst = probs x V
// with the matmul families of this library (batch dims b, h; keys / values of one head are broadcast).
DNNL_EXPORT dnnl_status_t dnnl_amd_sdpa_primitive_desc_create(dnnl_primitive_desc_t *primitive_desc, dnnl_engine_t engine,
        const_dnnl_memory_desc_t query_desc, const_dnnl_memory_desc_t key_desc, const_dnnl_memory_desc_t value_desc,
        const_dnnl_memory_desc_t dst_desc, const_dnnl_memory_desc_t mask_desc, const_dnnl_memory_desc_t scale_desc,
        int invert_scale, dnnl_dim_t kv_head_number, int attn_mask_type, dnnl_alg_kind_t softmax_alg,
        dnnl_prop_kind_t prop, const_dnnl_primitive_attr_t attr, const_dnnl_primitive_attr_t kq_attr,
        const_dnnl_primitive_attr_t vs_attr, const_dnnl_memory_desc_t stats_desc) {
    CHECK_ARG(primitive_desc && engine && query_desc && key_desc && value_desc && dst_desc);
    const dnnl_memory_desc &q = *query_desc, &k = *key_desc, &v = *value_desc, &d = *dst_desc;
    // sdpa_desc_check
    const int nd = d.ndims, r = nd - 2, c = nd - 1;
    CHECK_ARG(nd >= 2 && q.ndims == nd && k.ndims == nd && v.ndims == nd);
    CHECK_ARG(q.dims[c] == k.dims[r] && k.dims[c] == v.dims[r] && d.dims[r] == q.dims[r] && d.dims[c] == v.dims[c]);
    const bool with_mask = mask_desc && !mask_desc->is_zero() && mask_desc->dt != dnnl_data_type_undef;
    const bool with_scale = scale_desc && !scale_desc->is_zero() && scale_desc->dt != dnnl_data_type_undef;
    for (const dnnl_memory_desc *md : {&q, &k, &v, &d}) CHECK_ARG(md->kind != dnnl_format_kind_host_scalar);
    if (with_mask) CHECK_ARG(mask_desc->kind != dnnl_format_kind_host_scalar);
    CHECK_ARG(attn_mask_type >= 0 && attn_mask_type <= 3);
    CHECK_ARG(prop == dnnl_forward_inference || prop == dnnl_forward_training);
    // what this implementation takes
    CHECK_UNIMPL(nd == 4);                                   // (as the reference kernel: ref.hpp:50-56)
    CHECK_UNIMPL(prop == dnnl_forward_inference && !(stats_desc && !stats_desc->is_zero()));
    for (const_dnnl_primitive_attr_t a : {attr, kq_attr, vs_attr}) {
        if (!a) continue;                                    // no quantized keys / values, no attributes
        CHECK_UNIMPL(a->scales.empty() && a->zero_points.empty() && a->reductions.empty() && a->post_ops.entries.empty()
                && !a->with_dropout() && a->rounding.empty() && a->scratchpad_mode == dnnl_scratchpad_mode_library);
    }
    auto fp = [](dnnl_data_type_t dt) { return dt == dnnl_f32 || dt == dnnl_bf16 || dt == dnnl_f16; };
    CHECK_UNIMPL(fp(q.dt) && k.dt == q.dt && v.dt == q.dt && fp(d.dt));
    for (const dnnl_memory_desc *md : {&q, &k, &v, &d})
        CHECK_UNIMPL(md->kind == dnnl_blocked && !md->has_runtime() && !md->grouped);
    const dim_t B = q.dims[0], H = q.dims[1], Sq = q.dims[2], Sk = k.dims[3];
    CHECK_ARG(d.dims[0] == B && d.dims[1] == H);
    // keys and values: per head, or one head for all (both ways of grouping query heads agree on these two)
    for (const dnnl_memory_desc *md : {&k, &v}) {
        CHECK_ARG(md->dims[0] == B || md->dims[0] == 1);
        CHECK_UNIMPL(md->dims[1] == H || md->dims[1] == 1);
    }
    CHECK_ARG(kv_head_number <= 0 || kv_head_number == k.dims[1] || k.dims[1] == 1);
    CHECK_UNIMPL(softmax_alg == dnnl_softmax_accurate || (int)softmax_alg == dnnl_amd_softmax_accurate_inf_as_zero);
    const int mask_type = with_mask ? (attn_mask_type == 0 ? 1 : attn_mask_type) : (attn_mask_type == 1 ? 0 : attn_mask_type);
    if (with_mask) {
        CHECK_UNIMPL(mask_type == 1 && mask_desc->ndims == 4 && mask_desc->kind == dnnl_blocked && fp(mask_desc->dt));
        const dim_t full[4] = {B, H, Sq, Sk};
        for (int i = 0; i < 4; ++i) CHECK_ARG(mask_desc->dims[i] == full[i] || mask_desc->dims[i] == 1);
    }
    if (with_scale) {
        CHECK_UNIMPL(scale_desc->kind != dnnl_format_kind_host_scalar && fp(scale_desc->dt));
        CHECK_ARG(scale_desc->nelems() == 1);
    }
    std::unique_ptr<dnnl_primitive_desc> pd(new dnnl_primitive_desc);
    pd->kind = (dnnl_primitive_kind_t)dnnl_amd_sdpa;
    pd->engine = engine;
    pd->prop_kind = (int)prop;
    if (attr) pd->attr = *attr;
    auto S = std::make_shared<dnnl_primitive_desc::sdpa_t>();
    S->q = q; S->k = k; S->v = v; S->dst = d;
    if (with_mask) S->mask = *mask_desc;
    if (with_scale) S->scale = *scale_desc;
    S->invert_scale = invert_scale != 0;
    S->inf_as_zero = (int)softmax_alg == dnnl_amd_softmax_accurate_inf_as_zero;
    S->mask_type = mask_type;
    const dim_t sdims[4] = {B, H, Sq, Sk};
    for (dnnl_memory_desc *md : {&S->scores, &S->probs}) {
        md->ndims = 4;
        md->kind = dnnl_blocked;
        for (int i = 0; i < 4; ++i) md->dims[i] = sdims[i];
        md->set_dense();
    }
    S->scores.dt = dnnl_f32;
    S->probs.dt = v.dt;
    dnnl_primitive_desc_t kq = nullptr, vs = nullptr;
    dnnl_status_t st = dnnl_matmul_primitive_desc_create(&kq, engine, &S->q, &S->k, nullptr, &S->scores, nullptr);
    if (st) return st;
    S->kq.reset(kq);
    st = dnnl_matmul_primitive_desc_create(&vs, engine, &S->probs, &S->v, nullptr, &S->dst, nullptr);
    if (st) return st;
    S->vs.reset(vs);
    pd->src = q; pd->wei = k; pd->dst = d;
    pd->scratch_bytes = ((S->scores.size_bytes() + 255) & ~(size_t)255) + S->probs.size_bytes();
    pd->scratchpad = dnnl_memory_desc(); // library mode only: nothing for the caller to provide
    pd->impl_name = "hip:sdpa(" + kq->impl_name + "," + vs->impl_name + ")";
    pd->sdpa = S;
    if (verbose_level() >= 1)
        fprintf(stderr, "onednn_verbose,v1,primitive,create:dispatch,gpu,sdpa,%s\n", pd->impl_name.c_str());
    *primitive_desc = pd.release();
    return dnnl_success;
}

// ---- reorder primitive descriptor (src/common/reorder.cpp:67-170)
DNNL_EXPORT dnnl_status_t dnnl_reorder_primitive_desc_create(dnnl_primitive_desc_t *reorder_primitive_desc,
        const_dnnl_memory_desc_t src_desc, dnnl_engine_t src_engine, const_dnnl_memory_desc_t dst_desc,
        dnnl_engine_t dst_engine, const_dnnl_primitive_attr_t attr) {
    CHECK_ARG(reorder_primitive_desc && src_desc && dst_desc && src_engine && dst_engine);
    // one device: no cross-engine copies
    CHECK_UNIMPL(src_engine->kind == dnnl_gpu && dst_engine->kind == dnnl_gpu && src_engine->index == dst_engine->index);
    CHECK_ARG(src_desc->kind != dnnl_format_kind_any && dst_desc->kind != dnnl_format_kind_any); // :81-84
    // consistent_with: same logical dims (:91-92)
    CHECK_ARG(src_desc->ndims == dst_desc->ndims && src_desc->ndims >= 1);
    for (int i = 0; i < src_desc->ndims; ++i) CHECK_ARG(src_desc->dims[i] == dst_desc->dims[i]);
    CHECK_UNIMPL(src_desc->ndims <= MI355_REORDER_MAX_DIMS);
    CHECK_UNIMPL(!src_desc->has_runtime() && !dst_desc->has_runtime()); // runtime dims: matmul only
    // opaque (packed) weights: written by a reorder from plain weights of the
    // same data type; reading them back is not offered
    CHECK_UNIMPL(src_desc->kind == dnnl_blocked);
    const bool to_packed = dst_desc->kind == dnnl_format_kind_opaque;
    CHECK_UNIMPL(dst_desc->kind == dnnl_blocked || to_packed);
    if (to_packed) CHECK_UNIMPL(src_desc->ndims == 2 && src_desc->dt == dst_desc->dt);
    std::unique_ptr<dnnl_primitive_desc> pd(new dnnl_primitive_desc);
    if (attr) pd->attr = *attr;
    if (to_packed)
        CHECK_UNIMPL(pd->attr.scales.empty() && pd->attr.zero_points.empty() && pd->attr.post_ops.entries.empty());
    pd->kind = dnnl_reorder;
    pd->engine = dst_engine;
    pd->src = *src_desc;
    pd->dst = *dst_desc;
    const dnnl_primitive_attr &a = pd->attr;
    const int nd = src_desc->ndims;
    // scales / zero points on src and dst only (:106-111); everything else is not a reorder attribute
    for (const auto *m : {&a.scales, &a.zero_points})
        for (const auto &kv : *m)
            CHECK_UNIMPL((kv.first == DNNL_ARG_SRC || kv.first == DNNL_ARG_DST) && !kv.second.on_host);
    CHECK_UNIMPL(a.reductions.empty());
    mi355_reorder_desc_t &r = pd->rdesc;
    memset(&r, 0, sizeof(r));
    r.ndims = nd;
    r.src_dt = (int)src_desc->dt;
    r.dst_dt = (int)dst_desc->dt;
    for (int i = 0; i < nd; ++i) {
        r.dims[i] = src_desc->dims[i];
        r.src_stride[i] = src_desc->strides[i];
        r.dst_stride[i] = dst_desc->strides[i];
    }
    auto lower_q = [&](const quant_entry_t *q, mi355_quant_t &out, dnnl_data_type_t default_dt) -> dnnl_status_t {
        out.dt = MI355_DT_UNDEF;
        out.mask = 0;
        out.group[0] = out.group[1] = 1;
        if (!q) return dnnl_success;
        CHECK_ARG(q->mask >= 0 && (q->mask >> nd) == 0);
        out.dt = (int)(q->dt == dnnl_data_type_undef ? default_dt : q->dt);
        out.mask = q->mask;
        if (q->group_ndims == 2) {
            CHECK_ARG(nd >= 2);
            // groups divide the last two dims and the mask covers both (:118-140)
            CHECK_ARG(IMPLICATION(q->groups[0] > 1, src_desc->dims[nd - 2] % q->groups[0] == 0));
            CHECK_ARG(IMPLICATION(q->groups[1] > 1, src_desc->dims[nd - 1] % q->groups[1] == 0));
            CHECK_ARG((q->mask & (1 << (nd - 1))) && (q->mask & (1 << (nd - 2))));
            out.group[0] = q->groups[0];
            out.group[1] = q->groups[1];
        }
        return dnnl_success;
    };
    dnnl_status_t st;
    if ((st = lower_q(a.find(a.scales, DNNL_ARG_SRC), r.src_scale, dnnl_f32))) return st;
    if ((st = lower_q(a.find(a.scales, DNNL_ARG_DST), r.dst_scale, dnnl_f32))) return st;
    if ((st = lower_q(a.find(a.zero_points, DNNL_ARG_SRC), r.src_zp, dnnl_s32))) return st;
    if ((st = lower_q(a.find(a.zero_points, DNNL_ARG_DST), r.dst_zp, dnnl_s32))) return st;
    // 4-bit sources need a mask for their scales (:113-116)
    if (r.src_scale.dt != MI355_DT_UNDEF && (src_desc->dt == dnnl_s4 || src_desc->dt == dnnl_u4))
        CHECK_ARG(r.src_scale.mask > 0);
    // post-ops: a single sum (simple_po_check, src/cpu/reorder/cpu_reorder_pd.hpp)
    const auto &po = a.post_ops.entries;
    CHECK_UNIMPL(po.size() <= 1);
    if (po.size() == 1) {
        CHECK_UNIMPL(po[0].kind == dnnl_sum && po[0].zero_point == 0);
        r.beta = po[0].scale;
    }
    if (to_packed) {
        const int prc = mi355_wei_pack_reorder_dims(dst_desc->packing, src_desc->dims[0], src_desc->dims[1],
                src_desc->strides[0], src_desc->strides[1], &r);
        if (prc != MI355_SUCCESS) return from_mi355(prc);
    }
    const int rc = mi355_reorder_query(&r);
    if (rc != MI355_SUCCESS) return from_mi355(rc);
    pd->impl_name = "hip:reorder:any";
    pd->impls.assign(1, 0);
    if (verbose_level() >= 1)
        fprintf(stderr, "onednn_verbose,v1,primitive,create:dispatch,gpu,reorder,%s\n", pd->impl_name.c_str());
    *reorder_primitive_desc = pd.release();
    return dnnl_success;
}

DNNL_EXPORT dnnl_status_t dnnl_primitive_desc_clone(dnnl_primitive_desc_t *primitive_desc,
        const_dnnl_primitive_desc_t existing) {
    CHECK_ARG(primitive_desc && existing);
    *primitive_desc = new dnnl_primitive_desc(*existing);
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_desc_next_impl(dnnl_primitive_desc_t pd) {
    CHECK_ARG(pd);
    if (pd->impl_pos + 1 >= pd->impls.size()) return dnnl_last_impl_reached;
    ++pd->impl_pos;
    if (pd->kind == dnnl_reorder) return dnnl_success;
    return select_impl(*pd);
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_desc_get_attr(const_dnnl_primitive_desc_t pd, const_dnnl_primitive_attr_t *attr) {
    CHECK_ARG(pd && attr);
    *attr = pd->inner_product ? &pd->ip_attr : &pd->attr;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_amd_primitive_desc_get_lowered(const_dnnl_primitive_desc_t pd, void *out) {
    CHECK_ARG(pd && out && pd->kind == dnnl_matmul && !pd->runtime);
    memcpy(out, &pd->desc, sizeof(mi355_matmul_desc_t));
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_desc_destroy(dnnl_primitive_desc_t pd) {
    delete pd;
    return dnnl_success;
}
DNNL_EXPORT const_dnnl_memory_desc_t dnnl_primitive_desc_query_md(const_dnnl_primitive_desc_t pd, dnnl_query_t what,
        int index) {
    if (!pd) return nullptr;
    static const dnnl_memory_desc zero_md;
    if (pd->kind == dnnl_reorder) {
        switch (what) {
            case dnnl_query_src_md: return index == 0 ? &pd->src : nullptr;
            case dnnl_query_dst_md: return index == 0 ? &pd->dst : nullptr;
            case dnnl_query_scratchpad_md: return index == 0 ? &pd->scratchpad : nullptr;
            case dnnl_query_exec_arg_md:
                return index == DNNL_ARG_FROM ? &pd->src : index == DNNL_ARG_TO ? &pd->dst
                        : index == DNNL_ARG_SCRATCHPAD ? &pd->scratchpad : nullptr;
            default: return nullptr;
        }
    }
    if (pd->inner_product && pd->prop_kind == (int)dnnl_backward_data) {
        switch (what) {
            case dnnl_query_diff_src_md: return index == 0 ? &pd->ip_src : nullptr;
            case dnnl_query_weights_md: return index == 0 ? &pd->ip_wei : nullptr;
            case dnnl_query_diff_dst_md: return index == 0 ? &pd->ip_dst : nullptr;
            case dnnl_query_src_md: case dnnl_query_dst_md: case dnnl_query_diff_weights_md: return nullptr;
            case dnnl_query_exec_arg_md:
                if (index == DNNL_ARG_DIFF_SRC) return &pd->ip_src;
                if (index == DNNL_ARG_WEIGHTS) return &pd->ip_wei;
                if (index == DNNL_ARG_DIFF_DST) return &pd->ip_dst;
                if (index == DNNL_ARG_SCRATCHPAD) return &pd->scratchpad;
                return nullptr;
            default: break;
        }
    } else if (pd->inner_product && pd->prop_kind == (int)dnnl_backward_weights) {
        switch (what) {
            case dnnl_query_src_md: return index == 0 ? &pd->ip_src : nullptr;
            case dnnl_query_diff_weights_md:
                return index == 0 ? &pd->ip_wei : index == 1 ? (pd->ip_diff_bias ? &pd->ip_bias : &zero_md) : nullptr;
            case dnnl_query_diff_dst_md: return index == 0 ? &pd->ip_dst : nullptr;
            case dnnl_query_weights_md: case dnnl_query_dst_md: case dnnl_query_diff_src_md: return nullptr;
            case dnnl_query_exec_arg_md:
                if (index == DNNL_ARG_SRC) return &pd->ip_src;
                if (index == DNNL_ARG_DIFF_WEIGHTS) return &pd->ip_wei;
                if (index == DNNL_ARG_DIFF_BIAS) return pd->ip_diff_bias ? &pd->ip_bias : &zero_md;
                if (index == DNNL_ARG_DIFF_DST) return &pd->ip_dst;
                if (index == DNNL_ARG_SCRATCHPAD) return &pd->scratchpad;
                return nullptr;
            default: break;
        }
    } else if (pd->inner_product) { // the tensors as the caller describes them; dst is two-dimensional either way
        switch (what) {
            case dnnl_query_src_md: return index == 0 ? &pd->ip_src : nullptr;
            case dnnl_query_weights_md:
                return index == 0 ? &pd->ip_wei : index == 1 ? (pd->with_bias ? &pd->ip_bias : &zero_md) : nullptr;
            case dnnl_query_exec_arg_md:
                if (index == DNNL_ARG_SRC) return &pd->ip_src;
                if (index == DNNL_ARG_WEIGHTS) return &pd->ip_wei;
                if (index == DNNL_ARG_BIAS) return pd->with_bias ? &pd->ip_bias : &zero_md;
                break;
            default: break;
        }
    }
    switch (what) {
        case dnnl_query_src_md: return index == 0 ? &pd->src : nullptr;
        case dnnl_query_weights_md: return index == 0 ? &pd->wei : index == 1 ? (pd->with_bias ? &pd->bias : &zero_md) : nullptr;
        case dnnl_query_dst_md: return index == 0 ? &pd->dst : nullptr;
        case dnnl_query_scratchpad_md: return index == 0 ? &pd->scratchpad : nullptr;
        case dnnl_query_exec_arg_md:
            switch (index) {
                case DNNL_ARG_SRC: return &pd->src;
                case DNNL_ARG_WEIGHTS: return &pd->wei;
                case DNNL_ARG_BIAS: return pd->with_bias ? &pd->bias : &zero_md;
                case DNNL_ARG_DST: return &pd->dst;
                case DNNL_ARG_SCRATCHPAD: return &pd->scratchpad;
                default: return nullptr;
            }
        default: return nullptr;
    }
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_desc_query(const_dnnl_primitive_desc_t pd, dnnl_query_t what, int index,
        void *result) {
    CHECK_ARG(pd && result);
    switch (what) {
        case dnnl_query_engine: *(dnnl_engine_t *)result = pd->engine; break;
        case dnnl_query_primitive_kind:
            *(dnnl_primitive_kind_t *)result = pd->inner_product ? dnnl_inner_product : pd->kind;
            break;
        case dnnl_query_num_of_inputs_s32:
            *(int32_t *)result = pd->kind == dnnl_reorder ? 1 : 2 + (pd->with_bias ? 1 : 0);
            break;
        case dnnl_query_num_of_outputs_s32: *(int32_t *)result = 1; break;
        case dnnl_query_memory_consumption_s64:
            *(int64_t *)result = pd->attr.scratchpad_mode == dnnl_scratchpad_mode_library ? (int64_t)pd->scratch_bytes : 0;
            break;
        case dnnl_query_impl_info_str: *(const char **)result = pd->impl_name.c_str(); break;
        case dnnl_query_prop_kind: *(int *)result = pd->prop_kind; break;
        case dnnl_query_src_md:
        case dnnl_query_weights_md:
        case dnnl_query_dst_md:
        case dnnl_query_scratchpad_md:
        case dnnl_query_exec_arg_md: {
            const_dnnl_memory_desc_t md = dnnl_primitive_desc_query_md(pd, what, index);
            if (!md) return dnnl_invalid_arguments;
            *(const_dnnl_memory_desc_t *)result = md;
        } break;
        default: return dnnl_unimplemented;
    }
    return dnnl_success;
}

// ---- primitive
DNNL_EXPORT dnnl_status_t dnnl_primitive_create(dnnl_primitive_t *primitive, const_dnnl_primitive_desc_t pd) {
    CHECK_ARG(primitive && pd);
    std::unique_ptr<dnnl_primitive> p(new dnnl_primitive);
    p->pd = *pd;
    if (p->pd.attr.scratchpad_mode == dnnl_scratchpad_mode_library && p->pd.scratch_bytes > 0) {
        if (mi355_device_set((int)p->pd.engine->index) != MI355_SUCCESS) return dnnl_runtime_error;
        const int st = mi355_mem_alloc(&p->scratch, p->pd.scratch_bytes);
        if (st != MI355_SUCCESS) return from_mi355(st);
    }
    if (p->pd.sdpa) {
        dnnl_primitive_t kq = nullptr, vs = nullptr;
        dnnl_status_t st = dnnl_primitive_create(&kq, p->pd.sdpa->kq.get());
        if (st == dnnl_success) st = dnnl_primitive_create(&vs, p->pd.sdpa->vs.get());
        p->sdpa_kq = kq;
        p->sdpa_vs = vs;
        if (st != dnnl_success) return st;
    }
    bool any_on_host = false;
    for (const auto *mp : {&p->pd.attr.scales, &p->pd.attr.zero_points})
        for (const auto &kv : *mp) any_on_host |= kv.second.on_host;
    any_on_host |= p->pd.attr.with_dropout() && p->pd.attr.dropout_host_scalars;
    if (any_on_host && p->pd.kind == dnnl_matmul) {
        if (mi355_device_set((int)p->pd.engine->index) != MI355_SUCCESS) return dnnl_runtime_error;
        const int st = mi355_mem_alloc(&p->host_scalars, 128); // 6 quantization slots + 3 dropout slots of 8 bytes
        if (st != MI355_SUCCESS) return from_mi355(st);
    }
    *primitive = p.release();
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_get_primitive_desc(const_dnnl_primitive_t primitive,
        const_dnnl_primitive_desc_t *pd) {
    CHECK_ARG(primitive && pd);
    *pd = &primitive->pd;
    return dnnl_success;
}
DNNL_EXPORT dnnl_status_t dnnl_primitive_destroy(dnnl_primitive_t primitive) {
    delete primitive; // the destructor frees the device memory and the event
    return dnnl_success;
}

DNNL_EXPORT dnnl_status_t dnnl_primitive_execute(const_dnnl_primitive_t cprimitive, dnnl_stream_t stream, int nargs,
        const dnnl_exec_arg_t *args) {
    CHECK_ARG(cprimitive && stream);
    CHECK_ARG(nargs >= 0 && IMPLICATION(nargs > 0, args));
    dnnl_primitive *prim = const_cast<dnnl_primitive *>(cprimitive);
    const dnnl_primitive_desc &pd0 = prim->pd;
    CHECK_ARG(stream->engine == pd0.engine || stream->engine->index == pd0.engine->index);
    std::map<int, dnnl_memory_t> m;
    for (int i = 0; i < nargs; ++i) {
        CHECK_ARG(m.find(args[i].arg) == m.end()); // duplicated argument
        m[args[i].arg] = args[i].memory;
    }
    // inner product backward: the matmul it lowers to takes its src / weights / dst from other arguments
    dnnl_memory_t ip_diff_bias_mem = nullptr, ip_diff_dst_mem = nullptr;
    if (pd0.inner_product && pd0.prop_kind != (int)dnnl_forward_training && pd0.prop_kind != (int)dnnl_forward_inference) {
        auto get = [&](int arg) -> dnnl_memory_t {
            auto it = m.find(arg);
            return it == m.end() ? nullptr : it->second;
        };
        dnnl_memory_t dd = get(DNNL_ARG_DIFF_DST);
        CHECK_ARG(dd);
        ip_diff_dst_mem = dd;
        if (pd0.prop_kind == (int)dnnl_backward_data) {
            dnnl_memory_t ds = get(DNNL_ARG_DIFF_SRC);
            CHECK_ARG(ds && get(DNNL_ARG_WEIGHTS));
            m[DNNL_ARG_SRC] = dd;
            m[DNNL_ARG_DST] = ds;
        } else {
            dnnl_memory_t sr = get(DNNL_ARG_SRC), dw = get(DNNL_ARG_DIFF_WEIGHTS);
            CHECK_ARG(sr && dw);
            ip_diff_bias_mem = get(DNNL_ARG_DIFF_BIAS);
            CHECK_ARG(IMPLICATION(pd0.ip_diff_bias, ip_diff_bias_mem != nullptr));
            if (pd0.ip_src.dims[0] == 0) {
                // an empty batch: the sums over mb are empty, diff_weights and diff_bias are zeros
                // (the loops of src/cpu/ref_inner_product.cpp:165-212 store their initial 0)
                if (mi355_device_set((int)pd0.engine->index) != MI355_SUCCESS) return dnnl_runtime_error;
                int rc0 = dw->handle ? mi355_mem_set(dw->handle, 0, pd0.ip_wei.size_bytes(), stream->hip_stream)
                                     : MI355_INVALID_ARGUMENTS;
                if (rc0 == MI355_SUCCESS && ip_diff_bias_mem && pd0.ip_diff_bias)
                    rc0 = mi355_colsum_launch(nullptr, (int)pd0.ip_dst.dt, 0, pd0.ip_dst.dims[1], pd0.ip_dst.dims[1],
                            ip_diff_bias_mem->handle, (int)pd0.ip_bias.dt, stream->hip_stream);
                return from_mi355(rc0);
            }
            m[DNNL_ARG_SRC] = dd;
            m[DNNL_ARG_WEIGHTS] = sr;
            m[DNNL_ARG_DST] = dw;
        }
    }
    std::unique_lock<std::mutex> lock(prim->scratch_mutex, std::defer_lock);
    // Called before the first use of the primitive's own device memory in this
    // execution: takes the host lock and, if the previous such execution ran on
    // another stream, makes this stream wait for it.
    bool ordered = false;
    auto order_on_device = [&]() {
        if (ordered) return;
        ordered = true;
        if (!lock.owns_lock()) lock.lock();
        if (!prim->order_event) mi355_event_create(&prim->order_event); // the device is current here
        if (prim->order_event && prim->event_recorded && prim->last_stream != stream->hip_stream)
            mi355_stream_wait_event(stream->hip_stream, prim->order_event);
    };
    if (pd0.sdpa) {
        const dnnl_primitive_desc::sdpa_t &S = *pd0.sdpa;
        auto get = [&](int arg) -> dnnl_memory_t {
            auto it = m.find(arg);
            return it == m.end() ? nullptr : it->second;
        };
        dnnl_memory_t q = get(DNNL_ARG_SRC_0), k = get(DNNL_ARG_SRC_1), v = get(DNNL_ARG_SRC_2), d = get(DNNL_ARG_DST);
        dnnl_memory_t mask = get(DNNL_ARG_SHIFT), scale = get(DNNL_ARG_SCALE);
        CHECK_ARG(q && k && v && d);
        CHECK_ARG(IMPLICATION(S.mask_type == 1, mask && mask->handle));
        CHECK_ARG(IMPLICATION(!S.scale.is_zero(), scale && scale->handle));
        if (S.dst.nelems() == 0) return dnnl_success;
        CHECK_ARG(q->handle && k->handle && v->handle && d->handle && prim->scratch);
        if (mi355_device_set((int)pd0.engine->index) != MI355_SUCCESS) return dnnl_runtime_error;
        order_on_device(); // the scores and probabilities belong to the primitive
        dnnl_memory sc_mem, pr_mem;
        sc_mem.md = S.scores; sc_mem.engine = pd0.engine; sc_mem.handle = prim->scratch;
        pr_mem.md = S.probs; pr_mem.engine = pd0.engine;
        pr_mem.handle = (char *)prim->scratch + ((S.scores.size_bytes() + 255) & ~(size_t)255);
        const dnnl_exec_arg_t a1[3] = {{DNNL_ARG_SRC, q}, {DNNL_ARG_WEIGHTS, k}, {DNNL_ARG_DST, &sc_mem}};
        dnnl_status_t st = dnnl_primitive_execute(prim->sdpa_kq, stream, 3, a1);
        if (st != dnnl_success) return st;
        mi355_softmax_desc_t sd;
        memset(&sd, 0, sizeof(sd));
        sd.b = S.scores.dims[0]; sd.h = S.scores.dims[1]; sd.sq = S.scores.dims[2]; sd.sk = S.scores.dims[3];
        sd.out_dt = (int)S.probs.dt;
        sd.scale_dt = S.scale.is_zero() ? (int)MI355_DT_UNDEF : (int)S.scale.dt;
        sd.invert_scale = S.invert_scale;
        sd.mask_type = S.mask_type;
        sd.inf_as_zero = S.inf_as_zero;
        if (S.mask_type == 1) {
            sd.mask_dt = (int)S.mask.dt;
            for (int i = 0; i < 4; ++i) {
                sd.mask_dims[i] = S.mask.dims[i];
                sd.mask_stride[i] = S.mask.strides[i];
            }
        }
        const int rc = mi355_sdpa_softmax_launch(&sd, sc_mem.handle, pr_mem.handle, scale ? scale->handle : nullptr,
                mask ? mask->handle : nullptr, stream->hip_stream);
        if (rc != MI355_SUCCESS) return from_mi355(rc);
        const dnnl_exec_arg_t a2[3] = {{DNNL_ARG_SRC, &pr_mem}, {DNNL_ARG_WEIGHTS, v}, {DNNL_ARG_DST, d}};
        st = dnnl_primitive_execute(prim->sdpa_vs, stream, 3, a2);
        if (prim->order_event && mi355_event_record(prim->order_event, stream->hip_stream) == MI355_SUCCESS) {
            prim->event_recorded = true;
            prim->last_stream = stream->hip_stream;
        }
        return st;
    }
    void *rt_scratch = nullptr;
    if (pd0.runtime) {
        // executions of one primitive with runtime dims are serialised on the
        // host while they enqueue: they share the cached lowering and scratch
        if (mi355_device_set((int)pd0.engine->index) != MI355_SUCCESS) return dnnl_runtime_error;
        order_on_device();
        dnnl_status_t rs = concretize(*prim, m, &rt_scratch);
        if (rs) return rs;
    }
    const dnnl_primitive_desc &pd = pd0.runtime ? *prim->rt_pd : pd0;
    auto handle = [&](int arg, bool required, void **out) -> dnnl_status_t {
        auto it = m.find(arg);
        if (it == m.end() || !it->second) {
            *out = nullptr;
            return required ? dnnl_invalid_arguments : dnnl_success;
        }
        *out = it->second->handle;
        return dnnl_success;
    };
    if (pd.kind == dnnl_reorder) {
        mi355_reorder_args_t R;
        memset(&R, 0, sizeof(R));
        dnnl_status_t rs;
        void *q = nullptr;
        if ((rs = handle(DNNL_ARG_FROM, true, &q))) return rs;
        R.src = q;
        if ((rs = handle(DNNL_ARG_TO, true, &q))) return rs;
        R.dst = q;
        if ((rs = handle(DNNL_ARG_ATTR_SCALES | DNNL_ARG_SRC, pd.rdesc.src_scale.dt != MI355_DT_UNDEF, &q))) return rs;
        R.src_scale = q;
        if ((rs = handle(DNNL_ARG_ATTR_SCALES | DNNL_ARG_DST, pd.rdesc.dst_scale.dt != MI355_DT_UNDEF, &q))) return rs;
        R.dst_scale = q;
        if ((rs = handle(DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_SRC, pd.rdesc.src_zp.dt != MI355_DT_UNDEF, &q))) return rs;
        R.src_zp = q;
        if ((rs = handle(DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_DST, pd.rdesc.dst_zp.dt != MI355_DT_UNDEF, &q))) return rs;
        R.dst_zp = q;
        if (mi355_device_set((int)pd.engine->index) != MI355_SUCCESS) return dnnl_runtime_error;
        const auto t0 = std::chrono::steady_clock::now();
        const int rc = mi355_reorder_launch(&pd.rdesc, &R, stream->hip_stream);
        if (verbose_level() >= 2) {
            mi355_stream_sync(stream->hip_stream);
            const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
            fprintf(stderr, "onednn_verbose,v1,primitive,exec,gpu,reorder,%s,undef,src:%s dst:%s,,,%g\n",
                    pd.impl_name.c_str(), dt_name(pd.src.dt), dt_name(pd.dst.dt), ms);
        }
        return from_mi355(rc);
    }
    if (pd.grouped) {
        // values in buffer 0, the groups' cumulative ends in buffer 1 of the grouped memory objects
        mi355_grouped_args_t GA;
        memset(&GA, 0, sizeof(GA));
        auto mem_of = [&](int arg) -> dnnl_memory_t {
            auto it = m.find(arg);
            return it == m.end() ? nullptr : it->second;
        };
        dnnl_memory_t ms = mem_of(DNNL_ARG_SRC), mw = mem_of(DNNL_ARG_WEIGHTS), md = mem_of(DNNL_ARG_DST);
        CHECK_ARG(ms && mw && md && ms->md.grouped);
        const bool x3 = pd.gdesc.pattern == MI355_GROUPED_2DX3D;
        CHECK_ARG(x3 ? md->md.grouped : mw->md.grouped);
        GA.src = ms->handle; GA.wei = mw->handle; GA.dst = md->handle;
        GA.src_offsets = (const int32_t *)ms->handle2;
        if (x3) GA.dst_offsets = (const int32_t *)md->handle2;
        else GA.wei_offsets = (const int32_t *)mw->handle2;
        void *q = nullptr;
        dnnl_status_t gs;
        if ((gs = handle(DNNL_ARG_BIAS, pd.with_bias, &q))) return gs;
        GA.bias = q;
        if ((gs = handle(DNNL_ARG_ATTR_SCALES | DNNL_ARG_SRC, pd.gdesc.src_scale_dt != MI355_DT_UNDEF, &q))) return gs;
        GA.src_scale = q;
        if ((gs = handle(DNNL_ARG_ATTR_SCALES | DNNL_ARG_WEIGHTS, pd.gdesc.wei_scale_dt != MI355_DT_UNDEF, &q))) return gs;
        GA.wei_scale = q;
        if ((gs = handle(DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_SRC, pd.gdesc.src_zp_dt != MI355_DT_UNDEF, &q))) return gs;
        GA.src_zp = q;
        if ((gs = handle(DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_WEIGHTS, pd.gdesc.wei_zp_dt != MI355_DT_UNDEF, &q))) return gs;
        GA.wei_zp = q;
        for (int i = 0; i < pd.gdesc.n_post_ops; ++i) {
            if (pd.gdesc.post_ops[i].kind != MI355_PO_BINARY) continue;
            dnnl_memory_t mb = mem_of(DNNL_ARG_ATTR_MULTIPLE_POST_OP(i) | DNNL_ARG_SRC_1);
            CHECK_ARG(mb && mb->handle);
            GA.po_arg[i] = mb->handle;
            if (pd.gdesc.post_ops[i].grouped) {
                CHECK_ARG(mb->md.grouped && mb->handle2);
                GA.po_offsets[i] = (const int32_t *)mb->handle2;
            }
        }
        if (mi355_device_set((int)pd.engine->index) != MI355_SUCCESS) return dnnl_runtime_error;
        const auto t0 = std::chrono::steady_clock::now();
        const int rc = mi355_grouped_matmul_launch(&pd.gdesc, &GA, stream->hip_stream);
        if (verbose_level() >= 2) {
            mi355_stream_sync(stream->hip_stream);
            const double ms_ = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
            fprintf(stderr, "onednn_verbose,v1,primitive,exec,gpu,matmul,%s,undef,src:%s wei:%s dst:%s,,grouped:%ld,%g\n",
                    pd.impl_name.c_str(), dt_name(pd.src.dt), dt_name(pd.wei.dt), dt_name(pd.dst.dt),
                    (long)pd.gdesc.group_count, ms_);
        }
        return from_mi355(rc);
    }
    mi355_matmul_args_t A;
    memset(&A, 0, sizeof(A));
    dnnl_status_t st;
    const bool empty = pd.desc.batch == 0 || pd.desc.M == 0 || pd.desc.N == 0 || pd.desc.K == 0;
    void *p = nullptr;
#define TAKE(field, arg, required) \
    do { \
        if ((st = handle(arg, required, &p)) != dnnl_success) return st; \
        A.field = p; \
    } while (0)
    TAKE(src, DNNL_ARG_SRC, true);
    TAKE(wei, DNNL_ARG_WEIGHTS, true);
    TAKE(dst, DNNL_ARG_DST, true);
    TAKE(bias, DNNL_ARG_BIAS, pd.with_bias);
    // a scale / zero point set with is_on_host takes a host-scalar memory object: its value goes to the primitive's
    // device slot in stream order; any other one takes device memory
    int slot = 0;
    auto take_q = [&](const std::map<int, quant_entry_t> &mp, int arg, int flag, const mi355_quant_t &lowered,
                          const void **field) -> dnnl_status_t {
        const quant_entry_t *q = pd.attr.find(mp, arg);
        auto it = m.find(flag | arg);
        dnnl_memory_t mem = it == m.end() ? nullptr : it->second;
        const int my_slot = slot++;
        if (q && q->on_host) {
            CHECK_ARG(mem && mem->md.kind == dnnl_format_kind_host_scalar && (int)mem->md.dt == lowered.dt);
            if (!prim->host_scalars) return dnnl_runtime_error;
            void *dev = (char *)prim->host_scalars + 8 * my_slot;
            order_on_device();
            uint64_t bits = 0;
            memcpy(&bits, mem->scalar, dt_bits(mem->md.dt) / 8);
            const int rc = mi355_mem_store_scalar(dev, bits, dt_bits(mem->md.dt) / 8, stream->hip_stream);
            if (rc != MI355_SUCCESS) return from_mi355(rc);
            *field = dev;
            return dnnl_success;
        }
        CHECK_ARG(!mem || mem->md.kind != dnnl_format_kind_host_scalar);
        void *h = nullptr;
        const dnnl_status_t hs = handle(flag | arg, lowered.dt != MI355_DT_UNDEF, &h);
        *field = h;
        return hs;
    };
    if (mi355_device_set((int)pd.engine->index) != MI355_SUCCESS) return dnnl_runtime_error;
    const dnnl_primitive_attr &at = pd.attr;
    if ((st = take_q(at.scales, DNNL_ARG_SRC, DNNL_ARG_ATTR_SCALES, pd.desc.src_scale, &A.src_scale))) return st;
    if ((st = take_q(at.scales, DNNL_ARG_WEIGHTS, DNNL_ARG_ATTR_SCALES, pd.desc.wei_scale, &A.wei_scale))) return st;
    if ((st = take_q(at.scales, DNNL_ARG_DST, DNNL_ARG_ATTR_SCALES, pd.desc.dst_scale, &A.dst_scale))) return st;
    if ((st = take_q(at.zero_points, DNNL_ARG_SRC, DNNL_ARG_ATTR_ZERO_POINTS, pd.desc.src_zp, &A.src_zp))) return st;
    if ((st = take_q(at.zero_points, DNNL_ARG_WEIGHTS, DNNL_ARG_ATTR_ZERO_POINTS, pd.desc.wei_zp, &A.wei_zp))) return st;
    if ((st = take_q(at.zero_points, DNNL_ARG_DST, DNNL_ARG_ATTR_ZERO_POINTS, pd.desc.dst_zp, &A.dst_zp))) return st;
    TAKE(src_pr, DNNL_ARG_ATTR_PRECOMPUTED_REDUCTIONS | DNNL_ARG_SRC, pd.desc.src_pr.dt != MI355_DT_UNDEF);
    if (pd.desc.rnd_flags & MI355_RND_DROPOUT) {
        // probability, seed and offset: one value each, in device memory or (use_host_scalars) host-scalar objects
        auto take_scalar = [&](int arg, dnnl_data_type_t dt, int my_slot, const void **field) -> dnnl_status_t {
            auto it = m.find(arg);
            dnnl_memory_t mem = it == m.end() ? nullptr : it->second;
            CHECK_ARG(mem && (int)mem->md.dt == (int)dt);
            if (at.dropout_host_scalars) {
                CHECK_ARG(mem->md.kind == dnnl_format_kind_host_scalar);
                if (!prim->host_scalars) return dnnl_runtime_error;
                void *dev = (char *)prim->host_scalars + 8 * my_slot;
                order_on_device();
                uint64_t bits = 0;
                memcpy(&bits, mem->scalar, dt_bits(dt) / 8);
                const int rc = mi355_mem_store_scalar(dev, bits, dt_bits(dt) / 8, stream->hip_stream);
                if (rc != MI355_SUCCESS) return from_mi355(rc);
                *field = dev;
                return dnnl_success;
            }
            CHECK_ARG(mem->md.kind != dnnl_format_kind_host_scalar);
            void *h = nullptr;
            const dnnl_status_t hs = handle(arg, true, &h);
            *field = h;
            return hs;
        };
        if ((st = take_scalar(DNNL_ARG_ATTR_DROPOUT_PROBABILITY, dnnl_f32, 6, &A.dropout_p))) return st;
        if ((st = take_scalar(DNNL_ARG_ATTR_DROPOUT_SEED, at.dropout_seed_dt, 7, &A.dropout_seed))) return st;
        if (pd.desc.rnd_flags & MI355_RND_DROPOUT_OFFSET)
            if ((st = take_scalar(DNNL_ARG_ATTR_DROPOUT_OFFSET, dnnl_s64, 8, &A.dropout_offset))) return st;
        if (pd.desc.rnd_flags & MI355_RND_DROPOUT_MASK) TAKE(dropout_mask, DNNL_ARG_ATTR_DROPOUT_MASK, true);
    }
    for (int i = 0; i < pd.desc.n_post_ops; ++i) {
        if (pd.po_arg_id[i]) {
            if ((st = handle(DNNL_ARG_ATTR_MULTIPLE_POST_OP(pd.po_entry[i]) | pd.po_arg_id[i], true, &p))) return st;
            A.po_arg[i] = p;
        }
    }
#undef TAKE
    if (empty) return dnnl_success;
    if (!A.src || !A.wei || !A.dst) return dnnl_invalid_arguments;

    void *scratch = prim->scratch;
    if (pd0.runtime) {
        scratch = rt_scratch;
    } else if (pd.attr.scratchpad_mode == dnnl_scratchpad_mode_user) {
        if ((st = handle(DNNL_ARG_SCRATCHPAD, pd.scratch_bytes > 0, &scratch))) return st;
    } else if (scratch) {
        // the library-mode scratchpad belongs to the primitive: executions of
        // one primitive object are serialised on the host while they enqueue
        // and, across streams, on the device
        order_on_device();
    }
    if (mi355_device_set((int)pd.engine->index) != MI355_SUCCESS) return dnnl_runtime_error;
    const auto t0 = std::chrono::steady_clock::now();
    int rc = MI355_SUCCESS;
    if (pd.outer_n == 0) {
        rc = mi355_matmul_launch(&pd.desc, &A, scratch, stream->hip_stream);
    } else {
        // one launch per index of the batch dims that are walked on the host (in stream order: they share the scratch)
        dim_t count = 1;
        for (int i = 0; i < pd.outer_n; ++i) count *= pd.outer_dims[i];
        auto shifted = [](const void *base, dim_t elems, int dt) -> const void * {
            return base ? (const char *)base + elems * dt_bits(dt) / 8 : nullptr;
        };
        for (dim_t it = 0; it < count && rc == MI355_SUCCESS; ++it) {
            dim_t idx = it, os = 0, ow = 0, od = 0, ob = 0, op[MI355_MAX_POST_OPS] = {};
            for (int i = pd.outer_n - 1; i >= 0; --i) {
                const dim_t c = idx % pd.outer_dims[i];
                idx /= pd.outer_dims[i];
                os += c * pd.outer_src[i]; ow += c * pd.outer_wei[i]; od += c * pd.outer_dst[i]; ob += c * pd.outer_bias[i];
                for (int k = 0; k < pd.desc.n_post_ops; ++k) op[k] += c * pd.outer_po[k][i];
            }
            mi355_matmul_args_t B = A;
            B.src = shifted(A.src, os, pd.src.dt);
            B.wei = shifted(A.wei, ow, pd.wei.dt);
            B.dst = const_cast<void *>(shifted(A.dst, od, pd.dst.dt));
            if (pd.with_bias) B.bias = shifted(A.bias, ob, pd.bias.dt);
            for (int k = 0; k < pd.desc.n_post_ops; ++k)
                if (pd.desc.post_ops[k].kind == MI355_PO_BINARY) B.po_arg[k] = shifted(A.po_arg[k], op[k], pd.desc.post_ops[k].dt);
            rc = mi355_matmul_launch(&pd.desc, &B, scratch, stream->hip_stream);
        }
    }
    if (rc == MI355_SUCCESS && ip_diff_bias_mem && pd0.ip_diff_bias) {
        // diff_bias[oc] = sum over mb of diff_dst[mb, oc], added in the order of the rows
        CHECK_ARG(ip_diff_bias_mem->handle && ip_diff_dst_mem->handle);
        rc = mi355_colsum_launch(ip_diff_dst_mem->handle, (int)pd0.ip_dst.dt, pd0.ip_dst.dims[0], pd0.ip_dst.dims[1],
                pd0.ip_dst.strides[0], ip_diff_bias_mem->handle, (int)pd0.ip_bias.dt, stream->hip_stream);
    }
    if (ordered && prim->order_event) {
        if (mi355_event_record(prim->order_event, stream->hip_stream) == MI355_SUCCESS) {
            prim->event_recorded = true;
            prim->last_stream = stream->hip_stream;
        }
    }
    if (verbose_level() >= 2) {
        mi355_stream_sync(stream->hip_stream);
        const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        fprintf(stderr, "onednn_verbose,v1,primitive,exec,gpu,%s,%s,undef,src:%s wei:%s dst:%s,,%ldx%ldx%ld:%ldx%ldx%ld,%g\n",
                pd.inner_product ? "inner_product" : "matmul", pd.impl_name.c_str(), dt_name(pd.src.dt), dt_name(pd.wei.dt), dt_name(pd.dst.dt), (long)pd.desc.batch,
                (long)pd.desc.M, (long)pd.desc.K, (long)pd.desc.batch, (long)pd.desc.K, (long)pd.desc.N, ms);
    }
    return from_mi355(rc);
}
