/*
 * dnnl_amd.h -- the subset of oneDNN's public C API that the matmul primitive
 * needs, exported by libdnnl_amd.so with the reference's symbol names,
 * signatures and enum values, so that code written against oneDNN's own
 * headers (dnnl.h / dnnl.hpp, which are header-only wrappers over these
 * symbols) links against this library unchanged and only has to ask for a GPU
 * engine.
 *
 * Each declaration cites the reference declaration it reproduces
 * (uxlfoundation/oneDNN v3.14, paths relative to include/oneapi/dnnl/).
 * Callers that already include oneDNN's headers do not need this file; it
 * exists for callers (and tests) that do not have them.
 */
#ifndef DNNL_AMD_H
#define DNNL_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dnnl_common_types.h:44-66 */
typedef enum {
    dnnl_success = 0,
    dnnl_out_of_memory = 1,
    dnnl_invalid_arguments = 2,
    dnnl_unimplemented = 3,
    dnnl_last_impl_reached = 4,
    dnnl_runtime_error = 5,
    dnnl_not_required = 6,
    dnnl_invalid_graph = 7,
    dnnl_invalid_graph_op = 8,
    dnnl_invalid_shape = 9,
    dnnl_invalid_data_type = 10
} dnnl_status_t;

/* dnnl_common_types.h:80-114 */
typedef enum {
    dnnl_data_type_undef = 0,
    dnnl_f16 = 1,
    dnnl_bf16 = 2,
    dnnl_f32 = 3,
    dnnl_s32 = 4,
    dnnl_s8 = 5,
    dnnl_u8 = 6,
    dnnl_f64 = 7,
    dnnl_boolean = 8,
    dnnl_f8_e5m2 = 9,
    dnnl_f8_e4m3 = 10,
    dnnl_s4 = 11,
    dnnl_u4 = 12,
    dnnl_e8m0 = 13,
    dnnl_f4_e2m1 = 14,
    dnnl_f4_e3m0 = 15, /* not offered */
    dnnl_s64 = 16      /* the dropout seed and offset only */
} dnnl_data_type_t;

#define DNNL_MAX_NDIMS 12                  /* dnnl_common_types.h:123 */
typedef int64_t dnnl_dim_t;                /* dnnl_common_types.h:126 */
typedef dnnl_dim_t dnnl_dims_t[DNNL_MAX_NDIMS];
#define DNNL_RUNTIME_DIM_VAL INT64_MIN     /* dnnl_types.h:2331 */
#define DNNL_RUNTIME_SIZE_VAL ((size_t)DNNL_RUNTIME_DIM_VAL) /* dnnl_types.h:2336 */

/* dnnl_common_types.h:137-148 */
typedef enum {
    dnnl_fpmath_mode_strict = 0,
    dnnl_fpmath_mode_bf16,
    dnnl_fpmath_mode_f16,
    dnnl_fpmath_mode_any,
    dnnl_fpmath_mode_tf32
} dnnl_fpmath_mode_t;

/* dnnl_types.h:2470-2486 */
typedef enum {
    dnnl_quantization_mode_undef = 0,
    dnnl_quantization_mode_static_sazp,
    dnnl_quantization_mode_dynamic_mx,
    dnnl_quantization_mode_dynamic_fp
} dnnl_quantization_mode_t;

/* dnnl_common_types.h:157-170 */
typedef enum {
    dnnl_accumulation_mode_strict = 0,
    dnnl_accumulation_mode_relaxed,
    dnnl_accumulation_mode_any,
    dnnl_accumulation_mode_s32,
    dnnl_accumulation_mode_f32,
    dnnl_accumulation_mode_f16
} dnnl_accumulation_mode_t;

/* dnnl_common_types.h:180-187 */
typedef enum { dnnl_any_engine = 0, dnnl_cpu = 1, dnnl_gpu = 2 } dnnl_engine_kind_t;

/* dnnl_common_types.h:206-213 */
typedef enum {
    dnnl_stream_in_order = 0x1U,
    dnnl_stream_out_of_order = 0x2U,
    dnnl_stream_default_flags = dnnl_stream_in_order
} dnnl_stream_flags_t;

#define DNNL_MEMORY_NONE (NULL)                    /* dnnl_common_types.h:253 */
#define DNNL_MEMORY_ALLOCATE ((void *)(size_t)-1)  /* dnnl_common_types.h:257 */

/* dnnl_types.h:45-63 */
typedef enum {
    dnnl_format_kind_undef = 0,
    dnnl_format_kind_any,
    dnnl_blocked,
    dnnl_format_kind_opaque,
    dnnl_format_kind_sparse,     /* the grouped encoding only (dnnl_memory_desc_create_with_grouped_encoding) */
    dnnl_format_kind_host_scalar /* one value that lives in the memory object itself, on the host */
} dnnl_format_kind_t;

/* dnnl_types.h:175-260: the plain tags of the matmul and inner-product tensors, and the activation / weights
 * names the reference gives them (dnnl_types.h:1096-1155) */
typedef enum {
    dnnl_format_tag_undef = 0,
    dnnl_format_tag_any = 1,
    dnnl_a = 2,
    dnnl_ab = 3,
    dnnl_abc = 4,
    dnnl_abcd = 5,
    dnnl_abcde = 6,
    dnnl_ba = 14,
    dnnl_acb = 15,
    dnnl_abdc = 20,
    dnnl_acdb = 22,
    dnnl_acdeb = 33,
    dnnl_x = dnnl_a,
    dnnl_nc = dnnl_ab,
    dnnl_tn = dnnl_ab,
    dnnl_nt = dnnl_ba,
    dnnl_ncw = dnnl_abc,
    dnnl_nwc = dnnl_acb,
    dnnl_nchw = dnnl_abcd,
    dnnl_nhwc = dnnl_acdb,
    dnnl_ncdhw = dnnl_abcde,
    dnnl_ndhwc = dnnl_acdeb,
    dnnl_oi = dnnl_ab,
    dnnl_io = dnnl_ba,
    dnnl_oiw = dnnl_abc,
    dnnl_owi = dnnl_acb,
    dnnl_oihw = dnnl_abcd,
    dnnl_ohwi = dnnl_acdb,
    dnnl_oidhw = dnnl_abcde,
    dnnl_odhwi = dnnl_acdeb
} dnnl_format_tag_t;

/* dnnl_types.h:2057-2101 */
typedef enum {
    dnnl_undefined_primitive = 0,
    dnnl_reorder = 1,
    dnnl_sum = 4,
    dnnl_eltwise = 7,
    dnnl_inner_product = 10,
    dnnl_binary = 13,
    dnnl_matmul = 14,
    dnnl_prelu = 18,
    /* src/common/c_types_map.hpp:2036-2040: internal-only kinds start at 1 << 12; sdpa is the second */
    dnnl_amd_sdpa = (1 << 12) + 1
} dnnl_primitive_kind_t;

/* dnnl_types.h:2029-2049 */
typedef enum {
    dnnl_prop_kind_undef = 0,
    dnnl_forward_training = 64,
    dnnl_forward_inference = 96,
    dnnl_forward = dnnl_forward_training,
    dnnl_backward = 128,
    dnnl_backward_data = 160,
    dnnl_backward_weights = 192,
    dnnl_backward_bias = 193
} dnnl_prop_kind_t;

/* dnnl_types.h:2110-2230: the eltwise and binary algorithms post-ops admit */
typedef enum {
    dnnl_alg_kind_undef = 0,
    dnnl_eltwise_relu = 0x20,
    dnnl_eltwise_tanh,
    dnnl_eltwise_elu,
    dnnl_eltwise_square,
    dnnl_eltwise_abs,
    dnnl_eltwise_sqrt,
    dnnl_eltwise_linear,
    dnnl_eltwise_soft_relu,
    dnnl_eltwise_hardsigmoid,
    dnnl_eltwise_logistic,
    dnnl_eltwise_exp,
    dnnl_eltwise_gelu_tanh,
    dnnl_eltwise_swish,
    dnnl_eltwise_log,
    dnnl_eltwise_clip,
    dnnl_eltwise_clip_v2,
    dnnl_eltwise_pow,
    dnnl_eltwise_gelu_erf,
    dnnl_eltwise_round,
    dnnl_eltwise_mish,
    dnnl_eltwise_hardswish,
    /* the forward computation of the base algorithm (primitive_attr_postops.cpp:74-82) */
    dnnl_eltwise_relu_use_dst_for_bwd = 0x100,
    dnnl_eltwise_tanh_use_dst_for_bwd,
    dnnl_eltwise_elu_use_dst_for_bwd,
    dnnl_eltwise_sqrt_use_dst_for_bwd,
    dnnl_eltwise_logistic_use_dst_for_bwd,
    dnnl_eltwise_exp_use_dst_for_bwd,
    dnnl_eltwise_clip_v2_use_dst_for_bwd,
    dnnl_binary_add = 0x1fff0,
    dnnl_binary_mul = 0x1fff1,
    dnnl_binary_max = 0x1fff2,
    dnnl_binary_min = 0x1fff3,
    dnnl_binary_div = 0x1fff4,
    dnnl_binary_sub = 0x1fff5,
    dnnl_binary_ge = 0x1fff6,
    dnnl_binary_gt = 0x1fff7,
    dnnl_binary_le = 0x1fff8,
    dnnl_binary_lt = 0x1fff9,
    dnnl_binary_eq = 0x1fffa,
    dnnl_binary_ne = 0x1fffb,
    dnnl_binary_select = 0x1fffc, /* ternary: dst = src2 ? dst : src1 (dnnl_post_ops_append_binary_v2) */
    dnnl_softmax_accurate = 0x30000, /* dnnl_types.h:2252 */
    /* src/common/c_types_map.hpp:148-155: internal-only algorithms start at 1 << 12; a row of -inf gives zeros */
    dnnl_amd_softmax_accurate_inf_as_zero = (1 << 12) + 2
} dnnl_alg_kind_t;

/* dnnl_types.h:2448-2458 */
typedef enum { dnnl_scratchpad_mode_library = 0, dnnl_scratchpad_mode_user = 1 } dnnl_scratchpad_mode_t;

/* dnnl_types.h:2460-2467 */
typedef enum { dnnl_rounding_mode_environment = 0, dnnl_rounding_mode_stochastic = 1 } dnnl_rounding_mode_t;

/* dnnl_types.h:2846-2930 */
typedef enum {
    dnnl_query_undef = 0,
    dnnl_query_engine = 1,
    dnnl_query_primitive_kind = 2,
    dnnl_query_num_of_inputs_s32 = 3,
    dnnl_query_num_of_outputs_s32 = 4,
    dnnl_query_memory_consumption_s64 = 6,
    dnnl_query_impl_info_str = 8,
    dnnl_query_prop_kind = 11,
    dnnl_query_strides = 14,
    dnnl_query_src_md = 129,
    dnnl_query_diff_src_md = 130,
    dnnl_query_weights_md = 131,
    dnnl_query_diff_weights_md = 132,
    dnnl_query_dst_md = 133,
    dnnl_query_diff_dst_md = 134,
    dnnl_query_scratchpad_md = 136,
    dnnl_query_exec_arg_md = 255,
    dnnl_query_ndims_s32 = 256,
    dnnl_query_dims = 257,
    dnnl_query_data_type = 258,
    dnnl_query_format_kind = 262,
    dnnl_query_sparse_encoding = 266,
    dnnl_query_nnz_s64 = 267,
    dnnl_query_num_handles_s32 = 268
} dnnl_query_t;

/* dnnl_sparse_encoding_t of include/oneapi/dnnl/dnnl_types.h:67-88 with
 * DNNL_EXPERIMENTAL_GROUPED_MEMORY; only dnnl_grouped is offered. */
typedef enum {
    dnnl_sparse_encoding_undef = 0,
    dnnl_csr,
    dnnl_packed,
    dnnl_coo,
    dnnl_grouped
} dnnl_sparse_encoding_t;

/* execute argument ids, dnnl_types.h:2544-2784 */
#define DNNL_ARG_SRC 1
#define DNNL_ARG_SRC_0 1 /* dnnl_types.h:2544 */
#define DNNL_ARG_SRC_1 2
#define DNNL_ARG_SRC_2 3 /* dnnl_types.h:2562: the condition of a binary select post-op */
#define DNNL_ARG_DST 17
#define DNNL_ARG_SCALE 51 /* dnnl_types.h:2638 */
#define DNNL_ARG_SHIFT 52 /* dnnl_types.h:2640 */
#define DNNL_ARG_DIFF_SRC 129     /* dnnl_types.h:2649-2652 */
#define DNNL_ARG_DIFF_DST 145     /* dnnl_types.h:2676-2679 */
#define DNNL_ARG_DIFF_WEIGHTS 161 /* dnnl_types.h:2697-2700 */
#define DNNL_ARG_DIFF_BIAS 169    /* dnnl_types.h:2724 */
#define DNNL_ARG_WEIGHTS 33
#define DNNL_ARG_BIAS 41
#define DNNL_ARG_SCRATCHPAD 80
/* dnnl_types.h:2737-2750 */
#define DNNL_ARG_ATTR_DROPOUT_OFFSET 507
#define DNNL_ARG_ATTR_ROUNDING_SEED 508 /* accepted and not read: ref_matmul_t seeds the rounding with the dropout seed */
#define DNNL_ARG_ATTR_DROPOUT_MASK 509
#define DNNL_ARG_ATTR_DROPOUT_PROBABILITY 510
#define DNNL_ARG_ATTR_DROPOUT_SEED 511
#define DNNL_ARG_ATTR_PRECOMPUTED_REDUCTIONS 512
#define DNNL_ARG_ATTR_SCALES 4096
#define DNNL_ARG_ATTR_ZERO_POINTS 8192
#define DNNL_ARG_ATTR_MULTIPLE_POST_OP_BASE 32768
#define DNNL_ARG_ATTR_MULTIPLE_POST_OP(idx) (DNNL_ARG_ATTR_MULTIPLE_POST_OP_BASE * ((idx) + 1))

/* opaque handles, dnnl_common_types.h / dnnl_types.h */
typedef struct dnnl_engine *dnnl_engine_t;
typedef struct dnnl_stream *dnnl_stream_t;
typedef const struct dnnl_stream *const_dnnl_stream_t;
typedef struct dnnl_memory_desc *dnnl_memory_desc_t;
typedef const struct dnnl_memory_desc *const_dnnl_memory_desc_t;
typedef struct dnnl_memory *dnnl_memory_t;
typedef const struct dnnl_memory *const_dnnl_memory_t;
typedef struct dnnl_primitive_attr *dnnl_primitive_attr_t;
typedef const struct dnnl_primitive_attr *const_dnnl_primitive_attr_t;
typedef struct dnnl_post_ops *dnnl_post_ops_t;
typedef const struct dnnl_post_ops *const_dnnl_post_ops_t;
typedef struct dnnl_primitive_desc *dnnl_primitive_desc_t;
typedef const struct dnnl_primitive_desc *const_dnnl_primitive_desc_t;
typedef struct dnnl_primitive *dnnl_primitive_t;
typedef const struct dnnl_primitive *const_dnnl_primitive_t;

/* dnnl_types.h:2791-2794 */
typedef struct {
    int arg;
    dnnl_memory_t memory;
} dnnl_exec_arg_t;

/* ---- engine and stream: dnnl_common.h:54-109 ---- */
dnnl_status_t dnnl_engine_create(dnnl_engine_t *engine, dnnl_engine_kind_t kind, size_t index);
dnnl_status_t dnnl_engine_get_kind(dnnl_engine_t engine, dnnl_engine_kind_t *kind);
dnnl_status_t dnnl_engine_destroy(dnnl_engine_t engine);
size_t dnnl_engine_get_count(dnnl_engine_kind_t kind);
dnnl_status_t dnnl_stream_create(dnnl_stream_t *stream, dnnl_engine_t engine, unsigned flags);
dnnl_status_t dnnl_stream_get_engine(const_dnnl_stream_t stream, dnnl_engine_t *engine);
dnnl_status_t dnnl_stream_wait(dnnl_stream_t stream);
dnnl_status_t dnnl_stream_destroy(dnnl_stream_t stream);
/* Interoperability with the caller's HIP stream: what dnnl_ocl_interop_stream_create /
 * dnnl_ocl_interop_stream_get_command_queue (dnnl_ocl.h:220-231) and their SYCL twins (dnnl_sycl.h:154-165) are
 * for the reference's GPU runtimes.  `hip_stream` is a hipStream_t (NULL: the default stream); the dnnl stream does
 * not own it.  Primitives executed on it are ordered with the caller's own work on that stream and are recorded
 * when the caller captures it into a HIP graph (execute then must not need the library-mode scratchpad to grow:
 * use dnnl_scratchpad_mode_user, or execute once before capturing). */
dnnl_status_t dnnl_amd_interop_stream_create(dnnl_stream_t *stream, dnnl_engine_t engine, void *hip_stream);
dnnl_status_t dnnl_amd_interop_stream_get_hip_stream(dnnl_stream_t stream, void **hip_stream);

/* ---- memory descriptors: dnnl.h:1018-1424 ---- */
dnnl_status_t dnnl_memory_desc_create_with_strides(dnnl_memory_desc_t *memory_desc, int ndims,
        const dnnl_dims_t dims, dnnl_data_type_t data_type, const dnnl_dims_t strides);
dnnl_status_t dnnl_memory_desc_create_with_tag(dnnl_memory_desc_t *memory_desc, int ndims,
        const dnnl_dims_t dims, dnnl_data_type_t data_type, dnnl_format_tag_t tag);
dnnl_status_t dnnl_memory_desc_clone(dnnl_memory_desc_t *memory_desc, const_dnnl_memory_desc_t existing);
dnnl_status_t dnnl_memory_desc_destroy(dnnl_memory_desc_t memory_desc);
dnnl_status_t dnnl_memory_desc_query(const_dnnl_memory_desc_t memory_desc, dnnl_query_t what, void *result);

/* Grouped memory (mixture-of-experts): a 2-D tensor that concatenates
 * `group_count` sub-tensors along dims[variable_dim_idx] (index 0: row-major
 * storage, index 1: column-major), with a second buffer of s32 cumulative
 * group ends.  include/oneapi/dnnl/dnnl.h:1155-1193 (experimental in the
 * reference, always present here); src/common/memory_desc.cpp:417-472.
 * A matmul takes grouped src + dense 3-D weights + grouped dst (variable M) or
 * grouped src + grouped weights + dense 3-D dst (variable K):
 * src/common/matmul.cpp:43-259. */
dnnl_status_t dnnl_memory_desc_create_with_grouped_encoding(dnnl_memory_desc_t *memory_desc, int ndims,
        const dnnl_dims_t dims, dnnl_data_type_t data_type, int variable_dim_idx, dnnl_dim_t group_count,
        dnnl_data_type_t offsets_dt);
/* size of buffer `index` (0 values, 1 offsets); dnnl.h:1453 */
size_t dnnl_memory_desc_get_size_v2(const_dnnl_memory_desc_t memory_desc, int index);
int dnnl_memory_desc_equal(const_dnnl_memory_desc_t lhs, const_dnnl_memory_desc_t rhs);
size_t dnnl_memory_desc_get_size(const_dnnl_memory_desc_t memory_desc);
size_t dnnl_data_type_size(dnnl_data_type_t data_type);

/* ---- memory objects: dnnl.h:1482-1705 ---- */
dnnl_status_t dnnl_memory_create(dnnl_memory_t *memory, const_dnnl_memory_desc_t memory_desc,
        dnnl_engine_t engine, void *handle);
/* host-side scalars (dnnl.h:1196-1203, :1506-1520, :1676-1698): the value is copied into the memory object; a scale
 * or zero point set with is_on_host = 1 takes such a memory at execution */
dnnl_status_t dnnl_memory_desc_create_host_scalar(dnnl_memory_desc_t *memory_desc, dnnl_data_type_t data_type);
dnnl_status_t dnnl_memory_create_host_scalar(dnnl_memory_t *memory, const_dnnl_memory_desc_t memory_desc, void *scalar_ptr);
dnnl_status_t dnnl_memory_get_host_scalar_value(const_dnnl_memory_t memory, void *value);
dnnl_status_t dnnl_memory_set_host_scalar_value(dnnl_memory_t memory, const void *value);
dnnl_status_t dnnl_memory_get_memory_desc(const_dnnl_memory_t memory, const_dnnl_memory_desc_t *memory_desc);
dnnl_status_t dnnl_memory_get_engine(const_dnnl_memory_t memory, dnnl_engine_t *engine);
dnnl_status_t dnnl_memory_map_data(const_dnnl_memory_t memory, void **mapped_ptr);
dnnl_status_t dnnl_memory_unmap_data(const_dnnl_memory_t memory, void *mapped_ptr);
dnnl_status_t dnnl_memory_get_data_handle(const_dnnl_memory_t memory, void **handle);
dnnl_status_t dnnl_memory_set_data_handle(dnnl_memory_t memory, void *handle);
/* Memory objects over several buffers (dnnl.h:1503, :1591, :1627, :1660, :1672):
 * a grouped tensor has two, the values (index 0) and the s32 offsets (index 1). */
dnnl_status_t dnnl_memory_create_v2(dnnl_memory_t *memory, const_dnnl_memory_desc_t memory_desc, dnnl_engine_t engine,
        int nhandles, void **handles);
dnnl_status_t dnnl_memory_map_data_v2(const_dnnl_memory_t memory, void **mapped_ptr, int index);
dnnl_status_t dnnl_memory_unmap_data_v2(const_dnnl_memory_t memory, void *mapped_ptr, int index);
dnnl_status_t dnnl_memory_get_data_handle_v2(const_dnnl_memory_t memory, void **handle, int index);
dnnl_status_t dnnl_memory_set_data_handle_v2(dnnl_memory_t memory, void *handle, int index);
dnnl_status_t dnnl_memory_destroy(dnnl_memory_t memory);

/* ---- attributes: dnnl.h:340-720 ---- */
dnnl_status_t dnnl_primitive_attr_create(dnnl_primitive_attr_t *attr);
dnnl_status_t dnnl_primitive_attr_clone(dnnl_primitive_attr_t *attr, const_dnnl_primitive_attr_t existing_attr);
dnnl_status_t dnnl_primitive_attr_destroy(dnnl_primitive_attr_t attr);
dnnl_status_t dnnl_primitive_attr_set_fpmath_mode(dnnl_primitive_attr_t attr, dnnl_fpmath_mode_t mode);
dnnl_status_t dnnl_primitive_attr_set_fpmath_mode_v2(dnnl_primitive_attr_t attr, dnnl_fpmath_mode_t mode,
        int apply_to_int);
dnnl_status_t dnnl_primitive_attr_get_fpmath_mode_v2(const_dnnl_primitive_attr_t attr,
        dnnl_fpmath_mode_t *mode, int *apply_to_int);
dnnl_status_t dnnl_primitive_attr_set_accumulation_mode(dnnl_primitive_attr_t attr, dnnl_accumulation_mode_t mode);
dnnl_status_t dnnl_primitive_attr_set_scratchpad_mode(dnnl_primitive_attr_t attr, dnnl_scratchpad_mode_t mode);
/* dnnl.h:276-329: dropout applied to the matmul result after the bias and before the post-ops
 * (ref_matmul_t, floating-point src, plain row-major dst).  mask_desc: u8 and laid out like dst, or a zero
 * descriptor (no mask is written).  Execute arguments: DNNL_ARG_ATTR_DROPOUT_PROBABILITY (f32),
 * _SEED (seed_dt: s32 or s64), _OFFSET (s64, with use_offset), _MASK; with use_host_scalars the first
 * three are host-scalar memory objects. */
dnnl_status_t dnnl_primitive_attr_get_dropout(const_dnnl_primitive_attr_t attr, const_dnnl_memory_desc_t *mask_desc);
dnnl_status_t dnnl_primitive_attr_set_dropout(dnnl_primitive_attr_t attr, const_dnnl_memory_desc_t mask_desc);
dnnl_status_t dnnl_primitive_attr_get_dropout_v2(const_dnnl_primitive_attr_t attr, const_dnnl_memory_desc_t *mask_desc,
        dnnl_data_type_t *seed_dt, int *use_offset, int *use_host_scalars);
dnnl_status_t dnnl_primitive_attr_set_dropout_v2(dnnl_primitive_attr_t attr, const_dnnl_memory_desc_t mask_desc,
        dnnl_data_type_t seed_dt, int use_offset, int use_host_scalars);
/* dnnl.h:661-679: stochastic rounding of DNNL_ARG_DST (bf16 / f16 / fp8 / f32 dst of ref_matmul_t) */
dnnl_status_t dnnl_primitive_attr_set_rounding(dnnl_primitive_attr_t attr, int arg, dnnl_rounding_mode_t mode);
dnnl_status_t dnnl_primitive_attr_get_rounding(dnnl_primitive_attr_t attr, int arg, dnnl_rounding_mode_t *mode);
dnnl_status_t dnnl_primitive_attr_get_scratchpad_mode(const_dnnl_primitive_attr_t attr,
        dnnl_scratchpad_mode_t *mode);
dnnl_status_t dnnl_primitive_attr_set_scales_mask(dnnl_primitive_attr_t attr, int arg, int mask);
/* dnnl.h:520-553.  With dnnl_quantization_mode_dynamic_mx on DNNL_ARG_DST the
 * (or dnnl_quantization_mode_dynamic_fp, the NVFP4 flavour) the scales memory
 * passed at execution is an output (dnnl.h:546-547); is_on_host = 1 makes the
 * single (mask 0) scale a host-side scalar. */
dnnl_status_t dnnl_primitive_attr_set_scales_v2(dnnl_primitive_attr_t attr, int arg, int mask, int group_ndims,
        const dnnl_dims_t group_dims, dnnl_data_type_t data_type, int is_on_host);
dnnl_status_t dnnl_primitive_attr_set_scales_v3(dnnl_primitive_attr_t attr, int arg, int mask, int group_ndims,
        const dnnl_dims_t group_dims, dnnl_data_type_t data_type, int is_on_host, dnnl_quantization_mode_t qmode);
dnnl_status_t dnnl_primitive_attr_set_scales(dnnl_primitive_attr_t attr, int arg, int mask, int group_ndims,
        const dnnl_dims_t group_dims, dnnl_data_type_t data_type);
dnnl_status_t dnnl_primitive_attr_set_zero_points_mask(dnnl_primitive_attr_t attr, int arg, int mask);
/* dnnl.h:654-659: is_on_host = 1 makes the (single, mask 0) zero point a host-side scalar */
dnnl_status_t dnnl_primitive_attr_set_zero_points_v2(dnnl_primitive_attr_t attr, int arg, int mask, int group_ndims,
        const dnnl_dims_t group_dims, dnnl_data_type_t data_type, int is_on_host);
dnnl_status_t dnnl_primitive_attr_set_zero_points(dnnl_primitive_attr_t attr, int arg, int mask,
        int group_ndims, const dnnl_dims_t group_dims, dnnl_data_type_t data_type);
dnnl_status_t dnnl_primitive_attr_set_precomputed_reductions(dnnl_primitive_attr_t attr, int arg, int mask,
        int group_ndims, const dnnl_dims_t group_dims, dnnl_data_type_t data_type);
dnnl_status_t dnnl_primitive_attr_set_post_ops(dnnl_primitive_attr_t attr, const_dnnl_post_ops_t post_ops);
dnnl_status_t dnnl_primitive_attr_get_post_ops(const_dnnl_primitive_attr_t attr, const_dnnl_post_ops_t *post_ops);

/* ---- post-ops: dnnl.h:730-960 ---- */
dnnl_status_t dnnl_post_ops_create(dnnl_post_ops_t *post_ops);
dnnl_status_t dnnl_post_ops_clone(dnnl_post_ops_t *post_ops, const_dnnl_post_ops_t existing_post_ops);
dnnl_status_t dnnl_post_ops_destroy(dnnl_post_ops_t post_ops);
int dnnl_post_ops_len(const_dnnl_post_ops_t post_ops);
dnnl_primitive_kind_t dnnl_post_ops_get_kind(const_dnnl_post_ops_t post_ops, int index);
dnnl_status_t dnnl_post_ops_append_sum(dnnl_post_ops_t post_ops, float scale, int32_t zero_point,
        dnnl_data_type_t data_type);
dnnl_status_t dnnl_post_ops_get_params_sum(const_dnnl_post_ops_t post_ops, int index, float *scale,
        int32_t *zero_point, dnnl_data_type_t *data_type);
dnnl_status_t dnnl_post_ops_append_eltwise(dnnl_post_ops_t post_ops, dnnl_alg_kind_t alg_kind, float alpha,
        float beta);
dnnl_status_t dnnl_post_ops_get_params_eltwise(const_dnnl_post_ops_t post_ops, int index,
        dnnl_alg_kind_t *alg_kind, float *alpha, float *beta);
dnnl_status_t dnnl_post_ops_append_binary(dnnl_post_ops_t post_ops, dnnl_alg_kind_t alg_kind,
        const_dnnl_memory_desc_t src1_desc);
dnnl_status_t dnnl_post_ops_get_params_binary(const_dnnl_post_ops_t post_ops, int index,
        dnnl_alg_kind_t *alg_kind, const_dnnl_memory_desc_t *src1_desc);
/* dnnl.h: ternary binary post-op (select); src2_desc is NULL for every other algorithm */
dnnl_status_t dnnl_post_ops_append_binary_v2(dnnl_post_ops_t post_ops, dnnl_alg_kind_t alg_kind,
        const_dnnl_memory_desc_t src1_desc, const_dnnl_memory_desc_t src2_desc);
dnnl_status_t dnnl_post_ops_get_params_binary_v2(const_dnnl_post_ops_t post_ops, int index,
        dnnl_alg_kind_t *alg_kind, const_dnnl_memory_desc_t *src1_desc, const_dnnl_memory_desc_t *src2_desc);
dnnl_status_t dnnl_post_ops_append_prelu(dnnl_post_ops_t post_ops, int mask);
dnnl_status_t dnnl_post_ops_get_params_prelu(const_dnnl_post_ops_t post_ops, int index, int *mask);

/* ---- matmul primitive descriptor: dnnl.h:3774-3779 ---- */
dnnl_status_t dnnl_matmul_primitive_desc_create(dnnl_primitive_desc_t *primitive_desc, dnnl_engine_t engine,
        const_dnnl_memory_desc_t src_desc, const_dnnl_memory_desc_t weights_desc,
        const_dnnl_memory_desc_t bias_desc, const_dnnl_memory_desc_t dst_desc,
        const_dnnl_primitive_attr_t attr);

/* ---- inner product primitive descriptor: dnnl.h:2757-2762 (src/common/inner_product.cpp:188-203).
 * src [mb, ic, spatial...] (2 to 5 dims), weights [oc, ic, spatial...], bias [oc], dst [mb, oc]:
 * dst = src flattened to [mb, K] times weights flattened to [oc, K], transposed -- so plain weights are
 * K-contiguous, the layout the matrix-core kernels read at full rate, and the primitive runs on the matmul
 * kernel families (int8 with scales: src mask 0, weights mask 0 or 1, dst mask 0; f32 / bf16 / f16 / fp8
 * without scales; sum, eltwise, binary and prelu post-ops).  src and weights must keep their reduced dims
 * dense and in the same order in memory (nchw with oihw, nhwc with ohwi, ...): `format_tag::any` on either
 * one resolves to the other's order.  Execute arguments: DNNL_ARG_SRC, DNNL_ARG_WEIGHTS, DNNL_ARG_BIAS,
 * DNNL_ARG_DST and the attribute arguments of a matmul. */
dnnl_status_t dnnl_inner_product_forward_primitive_desc_create(dnnl_primitive_desc_t *primitive_desc,
        dnnl_engine_t engine, dnnl_prop_kind_t prop_kind, const_dnnl_memory_desc_t src_desc,
        const_dnnl_memory_desc_t weights_desc, const_dnnl_memory_desc_t bias_desc,
        const_dnnl_memory_desc_t dst_desc, const_dnnl_primitive_attr_t attr);
/* dnnl.h:2781-2787, :2809-2817 (src/common/inner_product.cpp:205-230; the naive implementations
 * src/cpu/ref_inner_product.cpp:100-217): f32 / bf16 / f16 tensors, no attributes; both lower to matmuls over
 * the tensors as they lie -- diff_src = diff_dst x weights; diff_weights = diff_dst^T x src, diff_bias = the
 * column sums of diff_dst in the reference's order of additions.  Execute arguments: DNNL_ARG_DIFF_DST,
 * DNNL_ARG_WEIGHTS, DNNL_ARG_DIFF_SRC / DNNL_ARG_SRC, DNNL_ARG_DIFF_DST, DNNL_ARG_DIFF_WEIGHTS,
 * DNNL_ARG_DIFF_BIAS.  hint_fwd_pd is accepted and not needed. */
dnnl_status_t dnnl_inner_product_backward_data_primitive_desc_create(dnnl_primitive_desc_t *primitive_desc,
        dnnl_engine_t engine, const_dnnl_memory_desc_t diff_src_desc, const_dnnl_memory_desc_t weights_desc,
        const_dnnl_memory_desc_t diff_dst_desc, const_dnnl_primitive_desc_t hint_fwd_pd,
        const_dnnl_primitive_attr_t attr);
dnnl_status_t dnnl_inner_product_backward_weights_primitive_desc_create(dnnl_primitive_desc_t *primitive_desc,
        dnnl_engine_t engine, const_dnnl_memory_desc_t src_desc, const_dnnl_memory_desc_t diff_weights_desc,
        const_dnnl_memory_desc_t diff_bias_desc, const_dnnl_memory_desc_t diff_dst_desc,
        const_dnnl_primitive_desc_t hint_fwd_pd, const_dnnl_primitive_attr_t attr);

/* ---- scaled dot-product attention, forward.  The reference keeps this primitive internal: the C++ function
 * sdpa_primitive_desc_create of src/common/sdpa_test_iface.hpp:23-33 (what its own tests call); this is that
 * function with C linkage, its arguments in the same order (invert_scale as int).  4-D tensors of f32 / bf16 / f16:
 * queries [b][h][sq][d], keys [b][hk][d][sk], values [b][hk][sk][dv], dst [b][h][sq][dv], hk == h or 1, any
 * strides; mask (attn_mask_type 1: a tensor whose dims are 1 or the full ones; 2 / 3: causal from the top left /
 * bottom right, src/common/sdpa_types.hpp:41-55) and scale (one value in device memory) optional.  Execute
 * arguments (sdpa_types.hpp:30-33): queries DNNL_ARG_SRC_0, keys DNNL_ARG_SRC_1, values DNNL_ARG_SRC_2,
 * DNNL_ARG_DST, the mask DNNL_ARG_SHIFT, the scale DNNL_ARG_SCALE.  Not offered (dnnl_unimplemented): training
 * (stats), quantized keys / values (kq_attr, vs_attr), other attributes, 1 < hk < h. ---- */
#define DNNL_ARG_QUERIES DNNL_ARG_SRC_0
#define DNNL_ARG_KEYS DNNL_ARG_SRC_1
#define DNNL_ARG_VALUES DNNL_ARG_SRC_2
#define DNNL_ARG_ATTN_MASK DNNL_ARG_SHIFT
dnnl_status_t dnnl_amd_sdpa_primitive_desc_create(dnnl_primitive_desc_t *primitive_desc, dnnl_engine_t engine,
        const_dnnl_memory_desc_t query_desc, const_dnnl_memory_desc_t key_desc, const_dnnl_memory_desc_t value_desc,
        const_dnnl_memory_desc_t dst_desc, const_dnnl_memory_desc_t mask_desc, const_dnnl_memory_desc_t scale_desc,
        int invert_scale, dnnl_dim_t kv_head_number, int attn_mask_type, dnnl_alg_kind_t softmax_alg,
        dnnl_prop_kind_t prop, const_dnnl_primitive_attr_t attr, const_dnnl_primitive_attr_t kq_attr,
        const_dnnl_primitive_attr_t vs_attr, const_dnnl_memory_desc_t stats_desc);

/* ---- reorder primitive descriptor: dnnl.h:1727-1731.  Execute arguments are
 * DNNL_ARG_FROM / DNNL_ARG_TO (dnnl_types.h:2553,2580) plus the scales and zero
 * points of DNNL_ARG_SRC / DNNL_ARG_DST. ---- */
#define DNNL_ARG_FROM DNNL_ARG_SRC
#define DNNL_ARG_TO DNNL_ARG_DST
dnnl_status_t dnnl_reorder_primitive_desc_create(dnnl_primitive_desc_t *reorder_primitive_desc,
        const_dnnl_memory_desc_t src_desc, dnnl_engine_t src_engine, const_dnnl_memory_desc_t dst_desc,
        dnnl_engine_t dst_engine, const_dnnl_primitive_attr_t attr);

/* ---- primitive descriptors and primitives: dnnl.h:60-243 ---- */
dnnl_status_t dnnl_primitive_desc_clone(dnnl_primitive_desc_t *primitive_desc,
        const_dnnl_primitive_desc_t existing_primitive_desc);
dnnl_status_t dnnl_primitive_desc_next_impl(dnnl_primitive_desc_t primitive_desc);
dnnl_status_t dnnl_primitive_desc_get_attr(const_dnnl_primitive_desc_t primitive_desc,
        const_dnnl_primitive_attr_t *attr);
dnnl_status_t dnnl_primitive_desc_destroy(dnnl_primitive_desc_t primitive_desc);
dnnl_status_t dnnl_primitive_desc_query(const_dnnl_primitive_desc_t primitive_desc, dnnl_query_t what,
        int index, void *result);
const_dnnl_memory_desc_t dnnl_primitive_desc_query_md(const_dnnl_primitive_desc_t primitive_desc,
        dnnl_query_t what, int index);
dnnl_status_t dnnl_primitive_create(dnnl_primitive_t *primitive, const_dnnl_primitive_desc_t primitive_desc);
dnnl_status_t dnnl_primitive_execute(const_dnnl_primitive_t primitive, dnnl_stream_t stream, int nargs,
        const dnnl_exec_arg_t *args);
dnnl_status_t dnnl_primitive_get_primitive_desc(const_dnnl_primitive_t primitive,
        const_dnnl_primitive_desc_t *primitive_desc);
dnnl_status_t dnnl_primitive_destroy(dnnl_primitive_t primitive);

/* ---- extension (no counterpart in dnnl.h): the thin-C-ABI problem description
 * (struct mi355_matmul_desc_t of mi355_matmul.h, passed as void * so that this
 * header stays self-contained) a matmul primitive descriptor without runtime
 * dims lowered to -- shapes, collapsed batch strides, quantization parameter
 * layouts, post-op operand strides.  For tools and tests that inspect what the
 * kernels are given; dnnl_invalid_arguments for a reorder or runtime-dims
 * descriptor. ---- */
dnnl_status_t dnnl_amd_primitive_desc_get_lowered(const_dnnl_primitive_desc_t primitive_desc,
        void *mi355_matmul_desc_out);

#ifdef __cplusplus
}
#endif
#endif /* DNNL_AMD_H */
