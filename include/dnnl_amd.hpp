/*
 * dnnl_amd.hpp -- the C++ face of dnnl_amd.h: a header-only layer over the C
 * symbols of libdnnl_amd.so with the class and member names of oneDNN's
 * dnnl.hpp (uxlfoundation/oneDNN v3.14, include/oneapi/dnnl/dnnl.hpp and
 * dnnl_common.hpp) for the part of the API the matmul path uses: engine,
 * stream, memory and memory::desc, primitive_attr, post_ops, matmul, reorder,
 * inner_product_forward / _backward_data / _backward_weights.  Code written
 * like the reference's matmul tutorials (the .cpp files of examples/tutorials/matmul)
 * compiles against it after changing the include and asking for a GPU engine.
 *
 * Callers that have oneDNN's own headers keep using them: dnnl.hpp is itself
 * header-only over the same C symbols.  This file is for callers (and tests)
 * that do not have them; it is written from the C API up, not taken from
 * dnnl.hpp.  Each class cites the dnnl.hpp / dnnl_common.hpp declaration whose
 * interface it follows.
 *
 * Objects are reference-counted handles (copies share the C object).  Every
 * failing C call throws dnnl::error carrying the status.
 */
#ifndef DNNL_AMD_HPP
#define DNNL_AMD_HPP

#include "dnnl_amd.h"

#include <cstring>
#include <exception>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

namespace dnnl {

/* dnnl_common.hpp:73-100 */
struct error : public std::exception {
    dnnl_status_t status;
    const char *message;
    error(dnnl_status_t s, const char *m) : status(s), message(m) {}
    const char *what() const noexcept override { return message; }
    static void wrap_c_api(dnnl_status_t s, const char *m) {
        if (s != dnnl_success) throw error(s, m);
    }
};

/* dnnl_common.hpp:290-318 */
enum class status {
    success = dnnl_success,
    out_of_memory = dnnl_out_of_memory,
    invalid_arguments = dnnl_invalid_arguments,
    unimplemented = dnnl_unimplemented,
    last_impl_reached = dnnl_last_impl_reached,
    runtime_error = dnnl_runtime_error,
    not_required = dnnl_not_required,
};

namespace detail {
/* A C handle with shared ownership; `weak` handles are borrowed (the C object belongs to somebody else). */
template <typename T>
class handle {
    std::shared_ptr<typename std::remove_pointer<T>::type> p_;

public:
    handle() = default;
    void reset(T t, dnnl_status_t (*destroy)(T), bool weak = false) {
        if (weak || !destroy) p_.reset(t, [](T) {});
        else p_.reset(t, [destroy](T x) { destroy(x); });
    }
    T get(bool allow_empty = false) const {
        if (!p_ && !allow_empty) throw error(dnnl_invalid_arguments, "object is not initialized");
        return p_.get();
    }
    explicit operator bool() const { return (bool)p_; }
    bool operator==(const handle &o) const { return p_.get() == o.p_.get(); }
    bool operator!=(const handle &o) const { return !(*this == o); }
};
} // namespace detail

/* dnnl_common.hpp:340-420 */
struct engine : public detail::handle<dnnl_engine_t> {
    enum class kind { any = dnnl_any_engine, cpu = dnnl_cpu, gpu = dnnl_gpu };
    engine() = default;
    engine(kind k, size_t index) {
        dnnl_engine_t e = nullptr;
        error::wrap_c_api(dnnl_engine_create(&e, (dnnl_engine_kind_t)k, index), "could not create an engine");
        reset(e, dnnl_engine_destroy);
    }
    engine(dnnl_engine_t borrowed, bool weak) { reset(borrowed, dnnl_engine_destroy, weak); }
    static size_t get_count(kind k) { return dnnl_engine_get_count((dnnl_engine_kind_t)k); }
    kind get_kind() const {
        dnnl_engine_kind_t k;
        error::wrap_c_api(dnnl_engine_get_kind(get(), &k), "could not get an engine's kind");
        return (kind)k;
    }
};

/* dnnl_common.hpp:430-500 */
struct stream : public detail::handle<dnnl_stream_t> {
    enum class flags : unsigned {
        in_order = dnnl_stream_in_order,
        out_of_order = dnnl_stream_out_of_order,
        default_flags = dnnl_stream_default_flags,
    };
    stream() = default;
    stream(const engine &e, flags f = flags::default_flags) {
        dnnl_stream_t s = nullptr;
        error::wrap_c_api(dnnl_stream_create(&s, e.get(), (unsigned)f), "could not create a stream");
        reset(s, dnnl_stream_destroy);
    }
    explicit stream(dnnl_stream_t owned) { reset(owned, dnnl_stream_destroy); }
    engine get_engine() const {
        dnnl_engine_t e = nullptr;
        error::wrap_c_api(dnnl_stream_get_engine(get(), &e), "could not get a stream's engine");
        return engine(e, true);
    }
    stream &wait() {
        error::wrap_c_api(dnnl_stream_wait(get()), "could not wait on a stream");
        return *this;
    }
};

/* The caller's hipStream_t as a dnnl stream and back: what dnnl::ocl_interop::make_stream / get_command_queue
 * (dnnl_ocl.hpp) are for OpenCL queues. */
namespace amd_interop {
inline stream make_stream(const engine &e, void *hip_stream) {
    dnnl_stream_t s = nullptr;
    error::wrap_c_api(dnnl_amd_interop_stream_create(&s, e.get(), hip_stream), "could not create a stream");
    return stream(s);
}
inline void *get_hip_stream(const stream &s) {
    void *h = nullptr;
    error::wrap_c_api(dnnl_amd_interop_stream_get_hip_stream(s.get(), &h), "could not get the HIP stream");
    return h;
}
} // namespace amd_interop

/* dnnl.hpp:770-2700 (struct memory) */
struct memory : public detail::handle<dnnl_memory_t> {
    typedef dnnl_dim_t dim;
    typedef std::vector<dim> dims;

    enum class data_type {
        undef = dnnl_data_type_undef,
        f16 = dnnl_f16,
        bf16 = dnnl_bf16,
        f32 = dnnl_f32,
        s32 = dnnl_s32,
        s8 = dnnl_s8,
        u8 = dnnl_u8,
        f64 = dnnl_f64,
        boolean = dnnl_boolean,
        f8_e5m2 = dnnl_f8_e5m2,
        f8_e4m3 = dnnl_f8_e4m3,
        s4 = dnnl_s4,
        u4 = dnnl_u4,
        e8m0 = dnnl_e8m0,
        f4_e2m1 = dnnl_f4_e2m1,
        f4_e3m0 = dnnl_f4_e3m0,
    };
    enum class format_kind {
        undef = dnnl_format_kind_undef,
        any = dnnl_format_kind_any,
        blocked = dnnl_blocked,
        opaque = dnnl_format_kind_opaque,
    };
    enum class format_tag {
        undef = dnnl_format_tag_undef,
        any = dnnl_format_tag_any,
        a = dnnl_a, ab = dnnl_ab, abc = dnnl_abc, abcd = dnnl_abcd, abcde = dnnl_abcde,
        ba = dnnl_ba, acb = dnnl_acb, abdc = dnnl_abdc, acdb = dnnl_acdb, acdeb = dnnl_acdeb,
        x = dnnl_x, nc = dnnl_nc, tn = dnnl_tn, nt = dnnl_nt, ncw = dnnl_ncw, nwc = dnnl_nwc, nchw = dnnl_nchw,
        nhwc = dnnl_nhwc, ncdhw = dnnl_ncdhw, ndhwc = dnnl_ndhwc, oi = dnnl_oi, io = dnnl_io, oiw = dnnl_oiw,
        owi = dnnl_owi, oihw = dnnl_oihw, ohwi = dnnl_ohwi, oidhw = dnnl_oidhw, odhwi = dnnl_odhwi,
    };

    static size_t data_type_size(data_type dt) { return dnnl_data_type_size((dnnl_data_type_t)dt); }

    /* dnnl.hpp:2790-3300 (memory::desc) */
    struct desc : public detail::handle<dnnl_memory_desc_t> {
        desc() = default; /* the zero descriptor: "no such tensor" */
        desc(const dims &d, data_type dt, format_tag tag, bool allow_empty = false) {
            check_ndims(d);
            dnnl_memory_desc_t md = nullptr;
            const dnnl_status_t st = dnnl_memory_desc_create_with_tag(
                    &md, (int)d.size(), padded(d).data(), (dnnl_data_type_t)dt, (dnnl_format_tag_t)tag);
            if (!allow_empty) error::wrap_c_api(st, "could not construct a memory descriptor using a format tag");
            if (st == dnnl_success) reset(md, dnnl_memory_desc_destroy);
        }
        desc(const dims &d, data_type dt, const dims &strides, bool allow_empty = false) {
            check_ndims(d);
            if (strides.size() != d.size()) throw error(dnnl_invalid_arguments, "dims and strides differ in length");
            dnnl_memory_desc_t md = nullptr;
            const dnnl_status_t st = dnnl_memory_desc_create_with_strides(
                    &md, (int)d.size(), padded(d).data(), (dnnl_data_type_t)dt, padded(strides).data());
            if (!allow_empty) error::wrap_c_api(st, "could not construct a memory descriptor using strides");
            if (st == dnnl_success) reset(md, dnnl_memory_desc_destroy);
        }
        /* a copy of a descriptor that a query returned (owned by this object) */
        explicit desc(const_dnnl_memory_desc_t borrowed) {
            if (!borrowed) return;
            dnnl_memory_desc_t md = nullptr;
            error::wrap_c_api(dnnl_memory_desc_clone(&md, borrowed), "could not clone a memory descriptor");
            reset(md, dnnl_memory_desc_destroy);
        }
        /* experimental in the reference (dnnl.hpp, DNNL_EXPERIMENTAL_GROUPED_MEMORY): memory::desc::grouped */
        static desc grouped(const dims &d, data_type dt, int variable_dim_idx, dim group_count,
                data_type offsets_dt = data_type::s32) {
            check_ndims(d);
            dnnl_memory_desc_t md = nullptr;
            error::wrap_c_api(dnnl_memory_desc_create_with_grouped_encoding(&md, (int)d.size(), padded(d).data(),
                                      (dnnl_data_type_t)dt, variable_dim_idx, group_count, (dnnl_data_type_t)offsets_dt),
                    "could not construct a grouped memory descriptor");
            desc r;
            r.reset(md, dnnl_memory_desc_destroy);
            return r;
        }
        static desc host_scalar(data_type dt) {
            dnnl_memory_desc_t md = nullptr;
            error::wrap_c_api(dnnl_memory_desc_create_host_scalar(&md, (dnnl_data_type_t)dt),
                    "could not construct a host-scalar memory descriptor");
            desc r;
            r.reset(md, dnnl_memory_desc_destroy);
            return r;
        }

        bool is_zero() const { return !*this || get_ndims() == 0; }
        int get_ndims() const { return *this ? query_s32(dnnl_query_ndims_s32) : 0; }
        dims get_dims() const { return query_dims(dnnl_query_dims); }
        dims get_strides() const { return query_dims(dnnl_query_strides); }
        data_type get_data_type() const {
            dnnl_data_type_t dt = dnnl_data_type_undef;
            if (*this) error::wrap_c_api(dnnl_memory_desc_query(get(), dnnl_query_data_type, &dt), "could not query");
            return (data_type)dt;
        }
        format_kind get_format_kind() const {
            dnnl_format_kind_t k = dnnl_format_kind_undef;
            if (*this) error::wrap_c_api(dnnl_memory_desc_query(get(), dnnl_query_format_kind, &k), "could not query");
            return (format_kind)k;
        }
        size_t get_size(int index = 0) const {
            if (!*this) return 0;
            return index == 0 ? dnnl_memory_desc_get_size(get()) : dnnl_memory_desc_get_size_v2(get(), index);
        }
        bool operator==(const desc &o) const {
            if (!*this || !o) return is_zero() && o.is_zero();
            return dnnl_memory_desc_equal(get(), o.get()) != 0;
        }
        bool operator!=(const desc &o) const { return !(*this == o); }
        /* NULL for the zero descriptor: what the C functions take for an absent tensor */
        const_dnnl_memory_desc_t c_or_null() const { return *this ? get() : nullptr; }

    private:
        static void check_ndims(const dims &d) {
            if (d.empty() || d.size() > DNNL_MAX_NDIMS) throw error(dnnl_invalid_arguments, "dimensions are invalid");
        }
        static std::vector<dim> padded(const dims &d) {
            std::vector<dim> v(DNNL_MAX_NDIMS, 0);
            std::memcpy(v.data(), d.data(), d.size() * sizeof(dim));
            return v;
        }
        int query_s32(dnnl_query_t q) const {
            int32_t v = 0;
            error::wrap_c_api(dnnl_memory_desc_query(get(), q, &v), "could not query a memory descriptor");
            return v;
        }
        dims query_dims(dnnl_query_t q) const {
            if (!*this) return {};
            const dnnl_dim_t *p = nullptr;
            error::wrap_c_api(dnnl_memory_desc_query(get(), q, &p), "could not query a memory descriptor");
            const int n = get_ndims();
            return p ? dims(p, p + n) : dims();
        }
    };

    memory() = default;
    /* the library allocates (DNNL_MEMORY_ALLOCATE) */
    memory(const desc &md, const engine &e) : memory(md, e, DNNL_MEMORY_ALLOCATE) {}
    /* `handle`: a device pointer of the caller's, DNNL_MEMORY_NONE or DNNL_MEMORY_ALLOCATE */
    memory(const desc &md, const engine &e, void *handle) {
        dnnl_memory_t m = nullptr;
        error::wrap_c_api(dnnl_memory_create(&m, md.get(), e.get(), handle), "could not create a memory object");
        reset(m, dnnl_memory_destroy);
    }
    /* several buffers (a grouped tensor: values, offsets) */
    memory(const desc &md, const engine &e, std::vector<void *> handles) {
        dnnl_memory_t m = nullptr;
        error::wrap_c_api(dnnl_memory_create_v2(&m, md.get(), e.get(), (int)handles.size(), handles.data()),
                "could not create a memory object");
        reset(m, dnnl_memory_destroy);
    }
    /* a scalar kept on the host (dnnl.hpp: memory(const desc &, T value) for host_scalar descriptors) */
    template <typename T>
    static memory host_scalar(data_type dt, T value) {
        desc md = desc::host_scalar(dt);
        dnnl_memory_t m = nullptr;
        error::wrap_c_api(dnnl_memory_create_host_scalar(&m, md.get(), &value), "could not create a host scalar");
        memory r;
        r.reset(m, dnnl_memory_destroy);
        return r;
    }

    desc get_desc() const {
        const_dnnl_memory_desc_t md = nullptr;
        error::wrap_c_api(dnnl_memory_get_memory_desc(get(), &md), "could not get a memory descriptor");
        return desc(md);
    }
    engine get_engine() const {
        dnnl_engine_t e = nullptr;
        error::wrap_c_api(dnnl_memory_get_engine(get(), &e), "could not get an engine from a memory object");
        return engine(e, true);
    }
    void *get_data_handle(int index = 0) const {
        void *h = nullptr;
        error::wrap_c_api(dnnl_memory_get_data_handle_v2(get(), &h, index), "could not get a data handle");
        return h;
    }
    void set_data_handle(void *h, int index = 0) const {
        error::wrap_c_api(dnnl_memory_set_data_handle_v2(get(), h, index), "could not set a data handle");
    }
    /* a host view of device memory: written back by unmap_data */
    template <typename T = void>
    T *map_data(int index = 0) const {
        void *p = nullptr;
        error::wrap_c_api(dnnl_memory_map_data_v2(get(), &p, index), "could not map memory object data");
        return static_cast<T *>(p);
    }
    void unmap_data(void *mapped, int index = 0) const {
        error::wrap_c_api(dnnl_memory_unmap_data_v2(get(), mapped, index), "could not unmap memory object data");
    }
};

/* dnnl.hpp:130-160 */
enum class scratchpad_mode { library = dnnl_scratchpad_mode_library, user = dnnl_scratchpad_mode_user };
/* dnnl_common.hpp:200-260 */
enum class fpmath_mode {
    strict = dnnl_fpmath_mode_strict,
    bf16 = dnnl_fpmath_mode_bf16,
    f16 = dnnl_fpmath_mode_f16,
    any = dnnl_fpmath_mode_any,
    tf32 = dnnl_fpmath_mode_tf32,
};
enum class accumulation_mode {
    strict = dnnl_accumulation_mode_strict,
    relaxed = dnnl_accumulation_mode_relaxed,
    any = dnnl_accumulation_mode_any,
    s32 = dnnl_accumulation_mode_s32,
    f32 = dnnl_accumulation_mode_f32,
    f16 = dnnl_accumulation_mode_f16,
};
/* dnnl.hpp:163-190 */
enum class prop_kind {
    undef = dnnl_prop_kind_undef,
    forward_training = dnnl_forward_training,
    forward_inference = dnnl_forward_inference,
    forward = dnnl_forward,
    backward = dnnl_backward,
    backward_data = dnnl_backward_data,
    backward_weights = dnnl_backward_weights,
    backward_bias = dnnl_backward_bias,
};
/* dnnl.hpp:193-400: the algorithms post-ops admit */
enum class algorithm {
    undef = dnnl_alg_kind_undef,
    eltwise_relu = dnnl_eltwise_relu,
    eltwise_tanh = dnnl_eltwise_tanh,
    eltwise_elu = dnnl_eltwise_elu,
    eltwise_square = dnnl_eltwise_square,
    eltwise_abs = dnnl_eltwise_abs,
    eltwise_sqrt = dnnl_eltwise_sqrt,
    eltwise_linear = dnnl_eltwise_linear,
    eltwise_soft_relu = dnnl_eltwise_soft_relu,
    eltwise_hardsigmoid = dnnl_eltwise_hardsigmoid,
    eltwise_logistic = dnnl_eltwise_logistic,
    eltwise_exp = dnnl_eltwise_exp,
    eltwise_gelu_tanh = dnnl_eltwise_gelu_tanh,
    eltwise_swish = dnnl_eltwise_swish,
    eltwise_log = dnnl_eltwise_log,
    eltwise_clip = dnnl_eltwise_clip,
    eltwise_clip_v2 = dnnl_eltwise_clip_v2,
    eltwise_pow = dnnl_eltwise_pow,
    eltwise_gelu_erf = dnnl_eltwise_gelu_erf,
    eltwise_round = dnnl_eltwise_round,
    eltwise_mish = dnnl_eltwise_mish,
    eltwise_hardswish = dnnl_eltwise_hardswish,
    binary_add = dnnl_binary_add,
    binary_mul = dnnl_binary_mul,
    binary_max = dnnl_binary_max,
    binary_min = dnnl_binary_min,
    binary_div = dnnl_binary_div,
    binary_sub = dnnl_binary_sub,
    binary_ge = dnnl_binary_ge,
    binary_gt = dnnl_binary_gt,
    binary_le = dnnl_binary_le,
    binary_lt = dnnl_binary_lt,
    binary_eq = dnnl_binary_eq,
    binary_ne = dnnl_binary_ne,
    binary_select = dnnl_binary_select,
};
enum class quantization_mode {
    undef = dnnl_quantization_mode_undef,
    static_sazp = dnnl_quantization_mode_static_sazp,
    dynamic_mx = dnnl_quantization_mode_dynamic_mx,
    dynamic_fp = dnnl_quantization_mode_dynamic_fp,
};
/* dnnl.hpp:520-700 */
enum class query {
    undef = dnnl_query_undef,
    src_md = dnnl_query_src_md,
    diff_src_md = dnnl_query_diff_src_md,
    weights_md = dnnl_query_weights_md,
    diff_weights_md = dnnl_query_diff_weights_md,
    dst_md = dnnl_query_dst_md,
    diff_dst_md = dnnl_query_diff_dst_md,
    scratchpad_md = dnnl_query_scratchpad_md,
    exec_arg_md = dnnl_query_exec_arg_md,
};

/* dnnl.hpp:3480-3900 */
struct post_ops : public detail::handle<dnnl_post_ops_t> {
    post_ops() {
        dnnl_post_ops_t p = nullptr;
        error::wrap_c_api(dnnl_post_ops_create(&p), "could not create post-ops");
        reset(p, dnnl_post_ops_destroy);
    }
    explicit post_ops(const_dnnl_post_ops_t borrowed) {
        dnnl_post_ops_t p = nullptr;
        error::wrap_c_api(dnnl_post_ops_clone(&p, borrowed), "could not clone post-ops");
        reset(p, dnnl_post_ops_destroy);
    }
    int len() const { return dnnl_post_ops_len(get()); }
    dnnl_primitive_kind_t kind(int index) const { return dnnl_post_ops_get_kind(get(), index); }
    void append_sum(float scale = 1.f, int32_t zero_point = 0, memory::data_type dt = memory::data_type::undef) {
        error::wrap_c_api(dnnl_post_ops_append_sum(get(), scale, zero_point, (dnnl_data_type_t)dt),
                "could not append a sum post-op");
    }
    void get_params_sum(int index, float &scale, int32_t &zero_point, memory::data_type &dt) const {
        dnnl_data_type_t c;
        error::wrap_c_api(dnnl_post_ops_get_params_sum(get(), index, &scale, &zero_point, &c), "could not get parameters");
        dt = (memory::data_type)c;
    }
    void append_eltwise(algorithm alg, float alpha, float beta) {
        error::wrap_c_api(dnnl_post_ops_append_eltwise(get(), (dnnl_alg_kind_t)alg, alpha, beta),
                "could not append an elementwise post-op");
    }
    void get_params_eltwise(int index, algorithm &alg, float &alpha, float &beta) const {
        dnnl_alg_kind_t c;
        error::wrap_c_api(dnnl_post_ops_get_params_eltwise(get(), index, &c, &alpha, &beta), "could not get parameters");
        alg = (algorithm)c;
    }
    void append_binary(algorithm alg, const memory::desc &src1) {
        error::wrap_c_api(dnnl_post_ops_append_binary(get(), (dnnl_alg_kind_t)alg, src1.get()),
                "could not append a binary post-op");
    }
    void append_binary(algorithm alg, const memory::desc &src1, const memory::desc &src2) {
        error::wrap_c_api(dnnl_post_ops_append_binary_v2(get(), (dnnl_alg_kind_t)alg, src1.get(), src2.c_or_null()),
                "could not append a binary post-op");
    }
    void get_params_binary(int index, algorithm &alg, memory::desc &src1) const {
        dnnl_alg_kind_t c;
        const_dnnl_memory_desc_t md = nullptr;
        error::wrap_c_api(dnnl_post_ops_get_params_binary(get(), index, &c, &md), "could not get parameters");
        alg = (algorithm)c;
        src1 = memory::desc(md);
    }
    void append_prelu(int mask) {
        error::wrap_c_api(dnnl_post_ops_append_prelu(get(), mask), "could not append a prelu post-op");
    }
    void get_params_prelu(int index, int &mask) const {
        error::wrap_c_api(dnnl_post_ops_get_params_prelu(get(), index, &mask), "could not get parameters");
    }
};

/* dnnl.hpp:3910-4500 */
struct primitive_attr : public detail::handle<dnnl_primitive_attr_t> {
    primitive_attr() {
        dnnl_primitive_attr_t a = nullptr;
        error::wrap_c_api(dnnl_primitive_attr_create(&a), "could not create primitive attributes");
        reset(a, dnnl_primitive_attr_destroy);
    }
    explicit primitive_attr(const_dnnl_primitive_attr_t borrowed) {
        dnnl_primitive_attr_t a = nullptr;
        error::wrap_c_api(dnnl_primitive_attr_clone(&a, borrowed), "could not clone primitive attributes");
        reset(a, dnnl_primitive_attr_destroy);
    }
    void set_fpmath_mode(fpmath_mode mode, bool apply_to_int = false) {
        error::wrap_c_api(dnnl_primitive_attr_set_fpmath_mode_v2(get(), (dnnl_fpmath_mode_t)mode, apply_to_int),
                "could not set the fpmath mode");
    }
    void get_fpmath_mode(fpmath_mode &mode, bool &apply_to_int) const {
        dnnl_fpmath_mode_t m;
        int a = 0;
        error::wrap_c_api(dnnl_primitive_attr_get_fpmath_mode_v2(get(), &m, &a), "could not get the fpmath mode");
        mode = (fpmath_mode)m;
        apply_to_int = a != 0;
    }
    void set_accumulation_mode(accumulation_mode mode) {
        error::wrap_c_api(dnnl_primitive_attr_set_accumulation_mode(get(), (dnnl_accumulation_mode_t)mode),
                "could not set the accumulation mode");
    }
    scratchpad_mode get_scratchpad_mode() const {
        dnnl_scratchpad_mode_t m;
        error::wrap_c_api(dnnl_primitive_attr_get_scratchpad_mode(get(), &m), "could not get the scratchpad mode");
        return (scratchpad_mode)m;
    }
    void set_scratchpad_mode(scratchpad_mode mode) {
        error::wrap_c_api(dnnl_primitive_attr_set_scratchpad_mode(get(), (dnnl_scratchpad_mode_t)mode),
                "could not set the scratchpad mode");
    }
    void set_scales_mask(int arg, int mask) {
        error::wrap_c_api(dnnl_primitive_attr_set_scales_mask(get(), arg, mask), "could not set scales");
    }
    void set_scales(int arg, int mask, const memory::dims &groups, memory::data_type dt = memory::data_type::f32,
            bool is_on_host = false, quantization_mode qmode = quantization_mode::static_sazp) {
        dnnl_dims_t g = {};
        copy_groups(groups, g);
        error::wrap_c_api(dnnl_primitive_attr_set_scales_v3(get(), arg, mask, (int)groups.size(), g,
                                  (dnnl_data_type_t)dt, is_on_host, (dnnl_quantization_mode_t)qmode),
                "could not set scales");
    }
    void set_zero_points_mask(int arg, int mask) {
        error::wrap_c_api(dnnl_primitive_attr_set_zero_points_mask(get(), arg, mask), "could not set zero points");
    }
    void set_zero_points(int arg, int mask, const memory::dims &groups, memory::data_type dt = memory::data_type::s32,
            bool is_on_host = false) {
        dnnl_dims_t g = {};
        copy_groups(groups, g);
        error::wrap_c_api(dnnl_primitive_attr_set_zero_points_v2(
                                  get(), arg, mask, (int)groups.size(), g, (dnnl_data_type_t)dt, is_on_host),
                "could not set zero points");
    }
    void set_precomputed_reductions(int arg, int mask, const memory::dims &groups,
            memory::data_type dt = memory::data_type::s32) {
        dnnl_dims_t g = {};
        copy_groups(groups, g);
        error::wrap_c_api(dnnl_primitive_attr_set_precomputed_reductions(
                                  get(), arg, mask, (int)groups.size(), g, (dnnl_data_type_t)dt),
                "could not set precomputed reductions");
    }
    post_ops get_post_ops() const {
        const_dnnl_post_ops_t p = nullptr;
        error::wrap_c_api(dnnl_primitive_attr_get_post_ops(get(), &p), "could not get post-ops");
        return post_ops(p);
    }
    void set_post_ops(const post_ops &po) {
        error::wrap_c_api(dnnl_primitive_attr_set_post_ops(get(), po.get()), "could not set post-ops");
    }
    void set_dropout(const memory::desc &mask_desc, memory::data_type seed_dt = memory::data_type::s32,
            bool use_offset = false, bool use_host_scalars = false) {
        error::wrap_c_api(dnnl_primitive_attr_set_dropout_v2(get(), mask_desc.c_or_null(), (dnnl_data_type_t)seed_dt,
                                  use_offset, use_host_scalars),
                "could not set dropout");
    }

private:
    static void copy_groups(const memory::dims &groups, dnnl_dims_t out) {
        if (groups.size() > DNNL_MAX_NDIMS) throw error(dnnl_invalid_arguments, "too many group dimensions");
        for (size_t i = 0; i < groups.size(); ++i) out[i] = groups[i];
    }
};

/* dnnl.hpp:4510-4900 (primitive_desc_base) */
struct primitive_desc_base : public detail::handle<dnnl_primitive_desc_t> {
    primitive_desc_base() = default;
    engine get_engine() const {
        dnnl_engine_t e = nullptr;
        error::wrap_c_api(dnnl_primitive_desc_query(get(), dnnl_query_engine, 0, &e), "could not query the engine");
        return engine(e, true);
    }
    const char *impl_info_str() const {
        const char *s = nullptr;
        error::wrap_c_api(dnnl_primitive_desc_query(get(), dnnl_query_impl_info_str, 0, &s),
                "could not query the implementation's name");
        return s;
    }
    /* moves to the next implementation; false when there is none */
    bool next_impl() {
        const dnnl_status_t st = dnnl_primitive_desc_next_impl(get());
        if (st == dnnl_last_impl_reached) return false;
        error::wrap_c_api(st, "could not advance to the next implementation");
        return true;
    }
    memory::desc query_md(query what, int index = 0) const {
        return memory::desc(dnnl_primitive_desc_query_md(get(), (dnnl_query_t)what, index));
    }
    memory::desc src_desc(int index = 0) const { return query_md(query::src_md, index); }
    memory::desc weights_desc(int index = 0) const { return query_md(query::weights_md, index); }
    memory::desc dst_desc(int index = 0) const { return query_md(query::dst_md, index); }
    memory::desc diff_src_desc(int index = 0) const { return query_md(query::diff_src_md, index); }
    memory::desc diff_weights_desc(int index = 0) const { return query_md(query::diff_weights_md, index); }
    memory::desc diff_dst_desc(int index = 0) const { return query_md(query::diff_dst_md, index); }
    memory::desc scratchpad_desc() const { return query_md(query::scratchpad_md, 0); }
    primitive_attr get_primitive_attr() const {
        const_dnnl_primitive_attr_t a = nullptr;
        error::wrap_c_api(dnnl_primitive_desc_get_attr(get(), &a), "could not get attributes");
        return primitive_attr(a);
    }

protected:
    void adopt(dnnl_primitive_desc_t pd, dnnl_status_t st, bool allow_empty, const char *what) {
        if (!allow_empty) error::wrap_c_api(st, what);
        if (st == dnnl_success) reset(pd, dnnl_primitive_desc_destroy);
    }
};

/* dnnl.hpp:400-520 (struct primitive) */
struct primitive : public detail::handle<dnnl_primitive_t> {
    primitive() = default;
    explicit primitive(const primitive_desc_base &pd) {
        dnnl_primitive_t p = nullptr;
        error::wrap_c_api(dnnl_primitive_create(&p, pd.get()), "could not create a primitive");
        reset(p, dnnl_primitive_destroy);
    }
    void execute(const stream &s, const std::unordered_map<int, memory> &args) const {
        std::vector<dnnl_exec_arg_t> c;
        c.reserve(args.size());
        for (const auto &a : args) c.push_back({a.first, a.second.get(true)});
        error::wrap_c_api(dnnl_primitive_execute(get(), s.get(), (int)c.size(), c.data()), "could not execute a primitive");
    }
};

/* dnnl.hpp (struct matmul) */
struct matmul : public primitive {
    struct primitive_desc : public primitive_desc_base {
        primitive_desc() = default;
        primitive_desc(const engine &e, const memory::desc &src, const memory::desc &weights, const memory::desc &dst,
                const primitive_attr &attr = primitive_attr(), bool allow_empty = false)
            : primitive_desc(e, src, weights, memory::desc(), dst, attr, allow_empty) {}
        primitive_desc(const engine &e, const memory::desc &src, const memory::desc &weights, const memory::desc &bias,
                const memory::desc &dst, const primitive_attr &attr = primitive_attr(), bool allow_empty = false) {
            dnnl_primitive_desc_t pd = nullptr;
            const dnnl_status_t st = dnnl_matmul_primitive_desc_create(
                    &pd, e.get(), src.get(), weights.get(), bias.c_or_null(), dst.get(), attr.get());
            adopt(pd, st, allow_empty, "could not create a primitive descriptor for the matmul primitive");
        }
        memory::desc bias_desc() const { return query_md(query::weights_md, 1); }
    };
    matmul() = default;
    explicit matmul(const primitive_desc &pd) : primitive(pd) {}
};

/* dnnl.hpp (struct reorder) */
struct reorder : public primitive {
    struct primitive_desc : public primitive_desc_base {
        primitive_desc() = default;
        primitive_desc(const engine &src_engine, const memory::desc &src, const engine &dst_engine,
                const memory::desc &dst, const primitive_attr &attr = primitive_attr(), bool allow_empty = false) {
            dnnl_primitive_desc_t pd = nullptr;
            const dnnl_status_t st = dnnl_reorder_primitive_desc_create(
                    &pd, src.get(), src_engine.get(), dst.get(), dst_engine.get(), attr.get());
            adopt(pd, st, allow_empty, "could not create a primitive descriptor for a reorder primitive");
        }
        primitive_desc(const memory &src, const memory &dst, const primitive_attr &attr = primitive_attr(),
                bool allow_empty = false)
            : primitive_desc(src.get_engine(), src.get_desc(), dst.get_engine(), dst.get_desc(), attr, allow_empty) {}
    };
    reorder() = default;
    explicit reorder(const primitive_desc &pd) : primitive(pd) {}
    reorder(const memory &src, const memory &dst, const primitive_attr &attr = primitive_attr())
        : primitive(primitive_desc(src, dst, attr)) {}
    using primitive::execute;
    void execute(const stream &s, memory &src, memory &dst) const {
        primitive::execute(s, {{DNNL_ARG_FROM, src}, {DNNL_ARG_TO, dst}});
    }
};

/* dnnl.hpp (struct inner_product_forward) */
struct inner_product_forward : public primitive {
    struct primitive_desc : public primitive_desc_base {
        primitive_desc() = default;
        primitive_desc(const engine &e, prop_kind kind, const memory::desc &src, const memory::desc &weights,
                const memory::desc &bias, const memory::desc &dst, const primitive_attr &attr = primitive_attr(),
                bool allow_empty = false) {
            dnnl_primitive_desc_t pd = nullptr;
            const dnnl_status_t st = dnnl_inner_product_forward_primitive_desc_create(&pd, e.get(),
                    (dnnl_prop_kind_t)kind, src.get(), weights.get(), bias.c_or_null(), dst.get(), attr.get());
            adopt(pd, st, allow_empty, "could not create a primitive descriptor for the inner product forward primitive");
        }
        primitive_desc(const engine &e, prop_kind kind, const memory::desc &src, const memory::desc &weights,
                const memory::desc &dst, const primitive_attr &attr = primitive_attr(), bool allow_empty = false)
            : primitive_desc(e, kind, src, weights, memory::desc(), dst, attr, allow_empty) {}
        memory::desc bias_desc() const { return query_md(query::weights_md, 1); }
    };
    inner_product_forward() = default;
    explicit inner_product_forward(const primitive_desc &pd) : primitive(pd) {}
};

/* dnnl.hpp (struct inner_product_backward_data) */
struct inner_product_backward_data : public primitive {
    struct primitive_desc : public primitive_desc_base {
        primitive_desc() = default;
        primitive_desc(const engine &e, const memory::desc &diff_src, const memory::desc &weights,
                const memory::desc &diff_dst, const inner_product_forward::primitive_desc &hint_fwd_pd,
                const primitive_attr &attr = primitive_attr(), bool allow_empty = false) {
            dnnl_primitive_desc_t pd = nullptr;
            const dnnl_status_t st = dnnl_inner_product_backward_data_primitive_desc_create(&pd, e.get(),
                    diff_src.get(), weights.get(), diff_dst.get(), hint_fwd_pd.get(true), attr.get());
            adopt(pd, st, allow_empty,
                    "could not create a primitive descriptor for the inner product backward propagation primitive");
        }
    };
    inner_product_backward_data() = default;
    explicit inner_product_backward_data(const primitive_desc &pd) : primitive(pd) {}
};

/* dnnl.hpp (struct inner_product_backward_weights) */
struct inner_product_backward_weights : public primitive {
    struct primitive_desc : public primitive_desc_base {
        primitive_desc() = default;
        primitive_desc(const engine &e, const memory::desc &src, const memory::desc &diff_weights,
                const memory::desc &diff_bias, const memory::desc &diff_dst,
                const inner_product_forward::primitive_desc &hint_fwd_pd, const primitive_attr &attr = primitive_attr(),
                bool allow_empty = false) {
            dnnl_primitive_desc_t pd = nullptr;
            const dnnl_status_t st = dnnl_inner_product_backward_weights_primitive_desc_create(&pd, e.get(), src.get(),
                    diff_weights.get(), diff_bias.c_or_null(), diff_dst.get(), hint_fwd_pd.get(true), attr.get());
            adopt(pd, st, allow_empty,
                    "could not create a primitive descriptor for the inner product weights gradient primitive");
        }
        primitive_desc(const engine &e, const memory::desc &src, const memory::desc &diff_weights,
                const memory::desc &diff_dst, const inner_product_forward::primitive_desc &hint_fwd_pd,
                const primitive_attr &attr = primitive_attr(), bool allow_empty = false)
            : primitive_desc(e, src, diff_weights, memory::desc(), diff_dst, hint_fwd_pd, attr, allow_empty) {}
        memory::desc diff_bias_desc() const { return query_md(query::diff_weights_md, 1); }
    };
    inner_product_backward_weights() = default;
    explicit inner_product_backward_weights(const primitive_desc &pd) : primitive(pd) {}
};

} // namespace dnnl

#endif /* DNNL_AMD_HPP */
