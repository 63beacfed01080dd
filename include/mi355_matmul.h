/*
 * mi355_matmul.h -- thin C ABI between the host-side oneDNN-compatible matmul
 * primitive and the hand-written gfx950 (MI355X / CDNA4) HIP kernels.
 *
 * Everything that crosses this boundary is plain C: PODs, raw device pointers,
 * sizes and an opaque stream handle.  No C++ or HIP types appear in the
 * signatures, so the host library (plain g++), a cgo/ctypes caller or a test
 * can bind it without HIP headers.
 *
 * What each piece replaces in the reference (uxlfoundation/oneDNN v3.14):
 *   - mi355_matmul_desc_t   : the information a matmul pd_t holds after
 *                             init(): src/common/matmul_pd.hpp:63-440 (M/N/K,
 *                             data types, strides, qmasks, groups, post-ops).
 *   - mi355_matmul_args_t   : the exec_ctx_t argument map of
 *                             primitive_t::execute, src/common/primitive_exec_types.hpp:112-186
 *                             and the brgemm_post_ops_data_t bundle of
 *                             src/cpu/x64/matmul/brgemm_matmul.cpp:966-981.
 *   - mi355_matmul_launch   : primitive_t::execute(const exec_ctx_t&)
 *                             (src/common/primitive.hpp:54) of the matmul
 *                             implementations ref_matmul_t / ref_matmul_int8_t /
 *                             brgemm_matmul_t.
 *   - mi355_matmul_query    : pd_t::init() dispatch predicate + name()
 *                             (DECLARE_COMMON_PD_T, src/common/primitive_desc.hpp).
 *   - mi355_reorder_*       : the reorder primitive that brings user tensors
 *                             into the layouts / data types the matmul wants
 *                             (src/common/reorder.cpp:67-170,
 *                             src/cpu/reorder/simple_reorder.hpp).
 *   - mi355_mem_* / stream  : memory_storage_t / stream_t of an engine
 *                             (src/common/memory_storage.hpp, src/common/stream.hpp).
 */
#ifndef MI355_MATMUL_H
#define MI355_MATMUL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Data types: numeric values equal dnnl_data_type_t
 * (include/oneapi/dnnl/dnnl_common_types.h:80-114). */
enum {
    MI355_DT_UNDEF = 0,
    MI355_DT_F16 = 1,
    MI355_DT_BF16 = 2,
    MI355_DT_F32 = 3,
    MI355_DT_S32 = 4,
    MI355_DT_S8 = 5,
    MI355_DT_U8 = 6,
    MI355_DT_F64 = 7,
    MI355_DT_BOOLEAN = 8,
    MI355_DT_F8_E5M2 = 9,
    MI355_DT_F8_E4M3 = 10,
    MI355_DT_S4 = 11,
    MI355_DT_U4 = 12,
    MI355_DT_E8M0 = 13,
    MI355_DT_F4_E2M1 = 14
};

/* Status codes: numeric values equal dnnl_status_t
 * (include/oneapi/dnnl/dnnl_common_types.h:44-66). */
enum {
    MI355_SUCCESS = 0,
    MI355_OUT_OF_MEMORY = 1,
    MI355_INVALID_ARGUMENTS = 2,
    MI355_UNIMPLEMENTED = 3,
    MI355_LAST_IMPL_REACHED = 4,
    MI355_RUNTIME_ERROR = 5,
    MI355_NOT_REQUIRED = 6
};

/* Post-op kinds (the four matmul admits, src/common/matmul.cpp:610-612). */
enum {
    MI355_PO_SUM = 1,
    MI355_PO_ELTWISE = 2,
    MI355_PO_BINARY = 3,
    MI355_PO_PRELU = 4,
    /* The condition operand (src2) of the ternary binary post-op
     * MI355_BINARY_SELECT, which must be the entry right before it:
     * v = cond != 0 ? v : src1 (primitive_attr_postops.cpp:44,345-360; the
     * condition is loaded as an integer).  This entry carries dt, stride and
     * po_arg of the condition and computes nothing by itself. */
    MI355_PO_SELECT_COND = 5
};

/* Algorithm kinds: numeric values equal dnnl_alg_kind_t
 * (include/oneapi/dnnl/dnnl_types.h, eltwise 0x20.., binary 0x1fff0..). */
enum {
    MI355_ELTWISE_RELU = 0x20,
    MI355_ELTWISE_TANH = 0x21,
    MI355_ELTWISE_ELU = 0x22,
    MI355_ELTWISE_SQUARE = 0x23,
    MI355_ELTWISE_ABS = 0x24,
    MI355_ELTWISE_SQRT = 0x25,
    MI355_ELTWISE_LINEAR = 0x26,
    MI355_ELTWISE_SOFT_RELU = 0x27,
    MI355_ELTWISE_HARDSIGMOID = 0x28,
    MI355_ELTWISE_LOGISTIC = 0x29,
    MI355_ELTWISE_EXP = 0x2a,
    MI355_ELTWISE_GELU_TANH = 0x2b,
    MI355_ELTWISE_SWISH = 0x2c,
    MI355_ELTWISE_LOG = 0x2d,
    MI355_ELTWISE_CLIP = 0x2e,
    MI355_ELTWISE_CLIP_V2 = 0x2f,
    MI355_ELTWISE_POW = 0x30,
    MI355_ELTWISE_GELU_ERF = 0x31,
    MI355_ELTWISE_ROUND = 0x32,
    MI355_ELTWISE_MISH = 0x33,
    MI355_ELTWISE_HARDSWISH = 0x34,
    MI355_BINARY_ADD = 0x1fff0,
    MI355_BINARY_MUL = 0x1fff1,
    MI355_BINARY_MAX = 0x1fff2,
    MI355_BINARY_MIN = 0x1fff3,
    MI355_BINARY_DIV = 0x1fff4,
    MI355_BINARY_SUB = 0x1fff5,
    MI355_BINARY_GE = 0x1fff6,
    MI355_BINARY_GT = 0x1fff7,
    MI355_BINARY_LE = 0x1fff8,
    MI355_BINARY_LT = 0x1fff9,
    MI355_BINARY_EQ = 0x1fffa,
    MI355_BINARY_NE = 0x1fffb,
    MI355_BINARY_SELECT = 0x1fffc /* generic kernel only; see MI355_PO_SELECT_COND */
};

/* Which arithmetic flavour of "the reference's own matmul" to reproduce where
 * the reference's two CPU implementations differ bit-wise. */
enum {
    /* ref_matmul_int8_t / ref_matmul_t: d /= dst_scale
     * (src/cpu/matmul/ref_matmul_int8.cpp:293-297). */
    MI355_DST_SCALE_DIVIDE = 0,
    /* brgemm_matmul_t: d *= (1.f / dst_scale)
     * (src/cpu/x64/matmul/brgemm_matmul.cpp:703-709). */
    MI355_DST_SCALE_RECIPROCAL = 1
};

/* Dynamic quantization of dst (quantization_mode::dynamic_mx): the scales of
 * DNNL_ARG_DST are an OUTPUT of the primitive.  For every group of 32
 * consecutive n of one dst row (ref_matmul.cpp:338-423; rules
 * src/common/matmul.cpp:407-424: full mask, groups 1 x 32, e8m0 scales)
 *     amax  = max |d| over the group, d after bias and post-ops
 *     scale = e8m0(e8m0(amax) / e8m0(max of dst type)), e8m0(x) = 2^floor(log2 x)
 *             (the exponent byte of x; 2^-127 for a zero exponent)
 *     args->dst_scale[(b, m, n / 32)] = scale       (written, despite the const)
 *     dst = convert(clamp(d * (1 / scale), -max, +max))
 * dst is f8_e4m3, f8_e5m2 or f4_e2m1, N % 32 == 0, no dst zero point.
 *
 * MI355_DST_DYNAMIC_FP (quantization_mode::dynamic_fp, the NVFP4 flavour;
 * ref_matmul.cpp:352-365, rules src/common/matmul.cpp:423-440): groups of 16
 * consecutive n, f8_e4m3 scales
 *     scale = e4m3(min(max(amax / max of dst type, 2^-3), 448))
 *             (2^-3 = epsilon of e4m3, src/common/nstl.hpp:189-191)
 * and the rest as above; N % 16 == 0.
 *
 * A 4-bit dst (f4_e2m1 with static or dynamic scales; s4 / u4 with static ones)
 * is served by the generic kernel: even N, unit n stride and even m / batch
 * strides, so that a thread writes whole bytes (low nibble = even n). */
enum {
    MI355_DST_DYNAMIC_NONE = 0,
    MI355_DST_DYNAMIC_MX = 1,
    MI355_DST_DYNAMIC_FP = 2
};

/* Kernel families (implementation ids). 0 lets the library choose. */
enum {
    MI355_IMPL_AUTO = 0,
    MI355_IMPL_REF = 1,      /* "hip:ref:any": one thread per dst element */
    MI355_IMPL_I8_MFMA = 2,  /* "hip:mfma_i8": LDS-tiled i8 MFMA GEMM */
    MI355_IMPL_F8_MFMA = 3,  /* "hip:mfma_f8": e4m3/e5m2 MFMA GEMM */
    MI355_IMPL_MXF4_MFMA = 4,/* "hip:mfma_mxf4": block-scaled e2m1 MFMA GEMM */
    MI355_IMPL_WOQ_GEMV = 5, /* "hip:woq_gemv": int4/int8 weight-only decode */
    MI355_IMPL_WOQ_PACKED = 6, /* "hip:woq_packed": decode over MI355_WEI_PACK_WOQ64 weights */
    MI355_IMPL_H16_MFMA = 7, /* "hip:mfma_h16": bf16 x bf16 / f16 x f16 / f32 x f32 MFMA GEMM, f32 accumulation */
    MI355_IMPL_COUNT = 8
};

/* Weights packing (mi355_matmul_desc_t.wei_packing): the counterpart of an
 * opaque blocked memory descriptor that dnnl_format_tag_any resolves to
 * (src/common/memory_desc.hpp: format_kind blocked with inner blocks; the
 * reference's brgemm matmul asks for such weights,
 * src/cpu/x64/matmul/brgemm_matmul_utils.cpp:203-330).
 *
 * MI355_WEI_PACK_WOQ64 -- 4-bit weights [K][N], batch 1, K % 32 == 0,
 * N % 64 == 0, K * N / 2 bytes, wei_stride ignored.  Element (k, n) is the
 * nibble (low nibble first within a byte) at nibble offset
 *     (n / 64) * (K * 64)        64-column chunk, all of K contiguous
 *   + (k / 8) * 512              8 rows of the chunk: 256 bytes
 *   + (n % 16) * 32              column within a 16-column block: 16 bytes
 *   + ((n % 64) / 16) * 8        16-column block of the chunk: one dword
 *   + (k % 2) * 4 + (k % 8) / 2  the 8 rows of one column in one dword
 * so that a wavefront reads 32 rows x 64 columns as one 1 KB run, 16 bytes
 * per lane, and every dword unpacks into a matrix-core operand with three
 * shifts.  mi355_reorder_launch writes the layout as a six-dim strided dst
 * (see mi355_wei_pack_reorder_dims). */
enum {
    MI355_WEI_PACK_NONE = 0,
    MI355_WEI_PACK_WOQ64 = 1
};

#define MI355_MAX_POST_OPS 32 /* post_ops_t::post_ops_limit in the reference */

/* A quantization parameter tensor (scales, zero points or precomputed
 * reductions) attached to one matmul argument.  Mirrors quant_entry_t
 * (src/common/primitive_attr_quant.hpp:40-140): a mask over the argument's
 * dimensions, optional groups over the last two dimensions and a data type.
 * The parameter tensor is dense row-major with dims
 *   [ mask&1 ? batch : 1, mask&2 ? D0/group[0] : 1, mask&4 ? D1/group[1] : 1 ]
 * where (D0, D1) are the last two dims of the argument (src: M,K; weights:
 * K,N; dst: M,N) -- quant_entry_t::get_md + matmul_helper_t::get_quant_off
 * (src/cpu/matmul/matmul_utils.hpp:154-173). */
typedef struct mi355_quant {
    int32_t dt;       /* MI355_DT_UNDEF = parameter absent */
    int32_t mask;     /* bit0 batch, bit1 second-to-last dim, bit2 last dim */
    int64_t group[2]; /* >= 1 */
} mi355_quant_t;

typedef struct mi355_post_op {
    int32_t kind; /* MI355_PO_* */
    int32_t alg;  /* eltwise / binary algorithm */
    float alpha, beta;
    float scale;          /* sum scale (eltwise scale is always 1 via the API) */
    int32_t zero_point;   /* sum zero point */
    int32_t dt;           /* binary: src1 dt; sum: dt dst is read as (0 = dst dt) */
    int64_t stride[3];    /* binary src1 / prelu weights element strides over
                             (batch, M, N); 0 on broadcast dims */
} mi355_post_op_t;

/* Dropout and stochastic rounding of ref_matmul_t (src/cpu/matmul/ref_matmul.cpp:61-67,
 * 248-331; ref_dropout src/cpu/primitive_attr_postops.cpp:296-310;
 * stochastic_round_fwd and the Philox generator src/common/math_utils.hpp:458-574).
 * Floating-point src only, the generic kernel only, dst dense row-major.
 *   dropout: after the bias and before the post-ops, element idx (its offset in
 *   dst) is kept when philox(idx, seed[, offset]) > UINT32_MAX * p and scaled by
 *   1 / (1 - p), else zeroed; the keep flags go to the mask.
 *   stochastic rounding of a bf16 / f16 / fp8 dst: random bits below the dst
 *   type's precision are added to the f32 value before truncation; the seed is
 *   the dropout seed (0 without dropout), as in the reference's implementation. */
#define MI355_RND_DROPOUT 1
#define MI355_RND_DROPOUT_MASK 2
#define MI355_RND_SEED_S64 4
#define MI355_RND_DROPOUT_OFFSET 8
#define MI355_RND_DST_STOCHASTIC 16

typedef struct mi355_matmul_desc {
    int64_t batch, M, N, K;
    int32_t src_dt, wei_dt, dst_dt, bias_dt; /* bias_dt UNDEF = no bias */
    /* element strides over (batch, row, col); 4-bit types count nibbles.
     * A batch stride of 0 broadcasts the operand. */
    int64_t src_stride[3];  /* (b, m, k) */
    int64_t wei_stride[3];  /* (b, k, n) */
    int64_t dst_stride[3];  /* (b, m, n) */
    int64_t bias_stride[3]; /* (b, m, n); 0 on broadcast dims */
    mi355_quant_t src_scale, wei_scale, dst_scale;
    mi355_quant_t src_zp, wei_zp, dst_zp;
    mi355_quant_t src_pr; /* precomputed reductions over K of src */
    int32_t fpmath_apply_to_int; /* weight decompression switch */
    int32_t fpmath_mode;         /* dnnl_fpmath_mode_t value: bf16 (1), f16 (2) or any (3) let "hip:mfma_h16"
                                    convert f32 operands to bf16 / f16 / bf16 before it multiplies them */
    int32_t dst_scale_mode;      /* MI355_DST_SCALE_* */
    int32_t n_post_ops;
    mi355_post_op_t post_ops[MI355_MAX_POST_OPS];
    int32_t impl; /* MI355_IMPL_*; AUTO picks the fastest applicable */
    int32_t wei_packing; /* MI355_WEI_PACK_* */
    int32_t dst_scale_dynamic; /* MI355_DST_DYNAMIC_* */
    int32_t rnd_flags;         /* MI355_RND_*: dropout and stochastic rounding */
} mi355_matmul_desc_t;

typedef struct mi355_matmul_args {
    const void *src, *wei, *bias;
    void *dst;
    const void *src_scale, *wei_scale, *dst_scale;
    const void *src_zp, *wei_zp, *dst_zp;
    const void *src_pr;
    const void *po_arg[MI355_MAX_POST_OPS]; /* binary src1 / prelu weights */
    /* MI355_RND_DROPOUT: probability (one f32), seed (one s32 or s64), offset
     * (one s64, with MI355_RND_DROPOUT_OFFSET), all in device memory; the mask
     * (u8, laid out like dst) is written with MI355_RND_DROPOUT_MASK */
    const void *dropout_p, *dropout_seed, *dropout_offset;
    void *dropout_mask;
} mi355_matmul_args_t;

/* ---- device, memory, stream, events (engine / stream / memory_storage) --- */
int mi355_device_count(int *count);
int mi355_device_set(int device);
/* name: gcnArchName; cus: multiProcessorCount; clock_khz; hbm_bytes */
int mi355_device_info(int device, char *name, size_t name_len, int *cus,
        int *clock_khz, int64_t *hbm_bytes, int64_t *l2_bytes);
int mi355_mem_alloc(void **dptr, size_t bytes);
int mi355_mem_free(void *dptr);
int mi355_mem_set(void *dptr, int byte, size_t bytes, void *stream);
int mi355_mem_h2d(void *dptr, const void *hptr, size_t bytes, void *stream);
int mi355_mem_d2h(void *hptr, const void *dptr, size_t bytes, void *stream);
int mi355_mem_d2d(void *dst, const void *src, size_t bytes, void *stream);
int mi355_stream_create(void **stream);
int mi355_stream_destroy(void *stream);
int mi355_stream_sync(void *stream); /* NULL = default stream */
int mi355_event_create(void **event);
int mi355_event_destroy(void *event);
int mi355_event_record(void *event, void *stream);
int mi355_event_sync(void *event);
int mi355_event_elapsed_ms(float *ms, void *start, void *stop);
/* work enqueued on `stream` after this call starts when `event` has completed
 * (the in-order guarantee of a stream, extended across two streams) */
int mi355_stream_wait_event(void *stream, void *event);
/* HIP graphs for launch-bound loops (a decode step is a few microseconds of
 * kernel behind a few microseconds of launch): every *_launch of this library
 * enqueues kernels only -- no allocation, no memset, no copy, nothing read
 * back -- so a stream that is being captured records it.  No counterpart in
 * the reference (its SYCL runtimes leave this to the SYCL graph extension).
 *   mi355_graph_capture_begin(stream)          stream: created, not NULL
 *   ... launches on `stream` (none of them runs) ...
 *   mi355_graph_capture_end(stream, &graph)    the instantiated graph
 *   mi355_graph_launch(graph, stream)          all recorded launches, in order
 * A launch's first call on a process may set a kernel attribute (dynamic LDS
 * size): run each distinct launch once outside the capture first. */
int mi355_graph_capture_begin(void *stream);
int mi355_graph_capture_end(void *stream, void **graph);
int mi355_graph_launch(void *graph, void *stream);
int mi355_graph_destroy(void *graph);
/* writes the low `nbytes` (1, 2, 4 or 8) of `bits` to device memory in stream
 * order, without a host copy: the value travels as a kernel argument, so the
 * call never waits for the stream (a host-side scalar of the attributes) */
int mi355_mem_store_scalar(void *dptr, uint64_t bits, int nbytes, void *stream);
const char *mi355_last_error(void); /* thread-local text of the last failure */

/* Tuning switches for tests and measurements; no counterpart in the reference
 * (its nearest relative is the ONEDNN_MAX_CPU_ISA family of environment
 * controls, src/common/utils.cpp getenv_int_user).  Each switch starts from the
 * environment variable of the same name, read once per process, and afterwards
 * changes only through this call -- launches never read the environment:
 *   MI355_I8_TILES     large | wide | narrow | small   tile geometry of hip:mfma_i8
 *                      (large: the LDS tiles, 256 x 128 or 256 x 256 by the tile count;
 *                      wide: 256 x 256; narrow: 256 x 128; small: 32 x 32 without LDS)
 *   MI355_F8_TILES     wide | narrow          hip:mfma_f8 on 256 x 256 / 256 x 128 tiles
 *   MI355_H16_TILES    wide                   hip:mfma_h16 on 256 x 256 tiles
 *   MI355_GROUPED_IMPL ref | short | tall | wide   grouped matmul kernel (ref: a thread per dst element;
 *                      variable M: 16 x 32, 48 x 64 or 64 x 256 tiles; variable K: short = the f32
 *                      instruction for 16-bit types too, tall / wide = a workgroup takes one / eight
 *                      column tiles in turn)
 *   MI355_GEMM_ORDER   0..63                  tile order of the large GEMMs
 * value NULL, "" or "auto" restores the library's own choice.  A switch can
 * change a problem's scratch need (the 32 x 32 int8 tiles need none, the LDS
 * tiles want column / row sums): set it before mi355_matmul_scratch_bytes, not
 * between that call and the launch.  A change while launches are in progress
 * on other threads takes effect at some launch boundary. */
int mi355_tuning_set(const char *name, const char *value);

/* ---- the matmul path ---------------------------------------------------- */

/* Dispatch predicate: MI355_SUCCESS if kernel family `impl` can run `desc`
 * exactly, MI355_UNIMPLEMENTED if not, MI355_INVALID_ARGUMENTS on nonsense.
 * With impl == AUTO reports the family the launcher would choose in
 * *chosen_impl (may be NULL). */
int mi355_matmul_query(const mi355_matmul_desc_t *desc, int impl,
        int *chosen_impl);

/* Implementation name in oneDNN's "impl_info_str" style, e.g. "hip:mfma_i8". */
const char *mi355_matmul_impl_name(int impl);

/* Bytes of device scratch `mi355_matmul_launch` needs for this problem
 * (0 for most kernels). */
int mi355_matmul_scratch_bytes(const mi355_matmul_desc_t *desc, size_t *bytes);

/* Enqueue the matmul on `stream` (a hipStream_t passed as void*, NULL =
 * default stream).  Asynchronous.  `scratch` may be NULL when
 * mi355_matmul_scratch_bytes reports 0. */
int mi355_matmul_launch(const mi355_matmul_desc_t *desc,
        const mi355_matmul_args_t *args, void *scratch, void *stream);

/* The same launch for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): no
 * counterpart in the reference.  The scratch is a static device array of
 * MI355_NOALLOC_SCRATCH_BYTES inside the library, one per GPU, held until the
 * process ends; the call allocates and frees nothing.  A problem whose
 * mi355_matmul_scratch_bytes exceeds it is refused with
 * MI355_INVALID_ARGUMENTS (mi355_last_error names both sizes).  All calls on
 * one GPU share that array: calls that overlap on one GPU (different streams,
 * or threads) race on it -- order them, or use mi355_matmul_launch with a
 * buffer per stream. */
#define MI355_NOALLOC_SCRATCH_BYTES (8u << 20)
int mi355_matmul_launch_noalloc(const mi355_matmul_desc_t *desc,
        const mi355_matmul_args_t *args, void *stream);

/* ---- reorder: layout and data-type conversion of one tensor -------------- */

#define MI355_REORDER_MAX_DIMS 6

/* What a reorder pd_t holds (src/common/reorder_pd.hpp) for plain strided
 * tensors, with the attributes the reference's generic reorder honours
 * (simple_reorder_impl_t<..., spec::reference>::execute,
 * src/cpu/reorder/simple_reorder.hpp:2579-2661, and its 4-bit variants
 * :2168-2425):
 *   d = src_scale * (src - src_zp);  d += beta * dst_old;
 *   d = d / dst_scale + dst_zp;      dst = saturate_and_round<dst_dt>(d)
 * Scales / zero points are dense row-major tensors over the masked dims with
 * the last two dims divided by the groups (quant_entry_t::get_md), mask bit i
 * = dim i.  Strides are in elements (nibbles for 4-bit types). */
typedef struct mi355_reorder_desc {
    int32_t ndims;
    int32_t src_dt, dst_dt;
    int32_t reserved;
    int64_t dims[MI355_REORDER_MAX_DIMS];
    int64_t src_stride[MI355_REORDER_MAX_DIMS];
    int64_t dst_stride[MI355_REORDER_MAX_DIMS];
    mi355_quant_t src_scale, dst_scale; /* dst_scale: f32, no groups */
    mi355_quant_t src_zp, dst_zp;       /* dst_zp: common s32 */
    float beta;                         /* sum post-op scale, 0 = none */
    int32_t reserved2;
} mi355_reorder_desc_t;

typedef struct mi355_reorder_args {
    const void *src;
    void *dst;
    const void *src_scale, *dst_scale;
    const void *src_zp, *dst_zp;
} mi355_reorder_args_t;

/* MI355_SUCCESS if the reorder kernels compute `desc` exactly,
 * MI355_UNIMPLEMENTED / MI355_INVALID_ARGUMENTS otherwise. */
int mi355_reorder_query(const mi355_reorder_desc_t *desc);

/* Enqueue the reorder on `stream` (primitive_t::execute of the reorder
 * implementations, DNNL_ARG_FROM -> DNNL_ARG_TO).  Asynchronous.  Dedicated
 * kernels serve the reorders of the matmul path (row quantization of float
 * tensors to 8-bit types, 8-bit transposition, 4-bit weights packing), two
 * general ones everything else; MI355_REORDER_GENERIC=1 in the environment
 * (read once per process) keeps the row-quantization and the 128 x 128
 * transposition kernels out, for tests and measurements. */
int mi355_reorder_launch(const mi355_reorder_desc_t *desc,
        const mi355_reorder_args_t *args, void *stream);

/* Writes into desc->ndims / dims / src_stride / dst_stride the six-dim view
 * under which a reorder moves weights [K][N] with element strides
 * (src_stride_k, src_stride_n) into the packed layout `packing`
 * (MI355_WEI_PACK_*); the other fields of `desc` are the caller's.  It is what
 * a reorder into an opaque blocked memory descriptor does in the reference
 * (simple_reorder.hpp, plain -> blocked specializations).
 * MI355_INVALID_ARGUMENTS if K, N do not fit the layout. */
int mi355_wei_pack_reorder_dims(int packing, int64_t K, int64_t N,
        int64_t src_stride_k, int64_t src_stride_n, mi355_reorder_desc_t *desc);

/* ---- grouped matmul (mixture-of-experts): one matmul per group over tensors
 * that concatenate the groups along one dimension, the group boundaries being
 * run-time data on the device.  Replaces ref_grouped_t
 * (src/cpu/matmul/ref_grouped_gemm.cpp:39-440; descriptor rules
 * src/common/matmul.cpp:43-259, ref_grouped_gemm.hpp:60-270):
 *   MI355_GROUPED_2DX3D  src [total_M][K] row-major, grouped along M;
 *                        weights dense [G][K][N] (any strides); dst
 *                        [total_M][N] row-major, grouped like src; optional
 *                        bias [G][N]; scales / zero points / post-ops below
 *   MI355_GROUPED_2DX2D  src [M][total_K] column-major, grouped along K;
 *                        weights [total_K][N] row-major, grouped like src; dst
 *                        dense [G][M][N] (any strides); same floating-point
 *                        type everywhere, nothing else
 * offsets[g] = end of group g along the variable dimension (cumulative, s32,
 * device memory); group g starts at offsets[g - 1] (0 for g = 0).
 * Quantization parameters (2DX3D): src scales / zero points per row,
 * [total_M] or [total_M][K / gk]; weights scales / zero points per group and
 * column, [G][N] or [G][K / gk][N]; gk = 0: no groups along K. */
#define MI355_GROUPED_2DX3D 0
#define MI355_GROUPED_2DX2D 1

typedef struct mi355_grouped_post_op {
    int32_t kind;  /* MI355_PO_ELTWISE or MI355_PO_BINARY (multiplication only) */
    int32_t alg;
    float alpha, beta, scale;
    int32_t dt;          /* binary: data type of the operand */
    int64_t bin_m, bin_n; /* binary: operand dims, [G][1], [total_M][1] or [total_M][N], dense row-major */
    int32_t grouped;     /* binary: the operand is a grouped tensor with offsets of its own */
} mi355_grouped_post_op_t;

typedef struct mi355_grouped_desc {
    int32_t pattern; /* MI355_GROUPED_* */
    int64_t group_count;
    int64_t total;   /* total_M (2DX3D) or total_K (2DX2D) */
    int64_t M;       /* 2DX2D: rows of every group; 2DX3D: unused */
    int64_t K;       /* 2DX3D: depth of every group; 2DX2D: unused */
    int64_t N;
    int32_t src_dt, wei_dt, dst_dt, bias_dt; /* bias_dt UNDEF = no bias */
    int64_t wei_stride[3]; /* 2DX3D: element strides of [G][K][N] */
    int64_t dst_stride[3]; /* 2DX2D: element strides of [G][M][N] */
    int32_t src_scale_dt, wei_scale_dt, src_zp_dt, wei_zp_dt; /* UNDEF = absent */
    int64_t src_scale_gk, wei_scale_gk, src_zp_gk, wei_zp_gk;
    int32_t fpmath_apply_to_int;
    int32_t n_post_ops;
    mi355_grouped_post_op_t post_ops[MI355_MAX_POST_OPS];
} mi355_grouped_desc_t;

typedef struct mi355_grouped_args {
    const void *src, *wei, *bias;
    void *dst;
    const int32_t *src_offsets, *wei_offsets, *dst_offsets; /* wei: 2DX2D; dst: 2DX3D */
    const void *src_scale, *wei_scale, *src_zp, *wei_zp;
    const void *po_arg[MI355_MAX_POST_OPS];
    const int32_t *po_offsets[MI355_MAX_POST_OPS]; /* grouped binary operands */
} mi355_grouped_args_t;

/* MI355_SUCCESS if an implementation takes the problem:
 *   "hip:mfma_grouped"     2DX3D on the matrix cores: fp8 x fp8 (e4m3 / e5m2 in
 *                          any pairing), bf16 x bf16 or f16 x f16 with
 *                          K-contiguous weights ([G][N][K], wei_stride[1] == 1,
 *                          16-byte aligned rows, K a multiple of 32 bytes),
 *                          scales without groups along K, or -- fp8 / f4_e2m1 x
 *                          f4_e2m1 -- e8m0 scales per 32 k on both operands (K a
 *                          multiple of 512 bytes, N of 4); no zero points; bias
 *                          and every post-op of the list.  f32 accumulation in
 *                          the order of the hardware.
 *   "hip:ref_grouped:any"  everything else the descriptor rules allow: a thread
 *                          per dst element in the reference's operation order.
 * The environment variable MI355_GROUPED_IMPL=ref keeps every problem on the
 * second one (short / tall / wide force one of the matrix-core kernel's tile shapes). */
int mi355_grouped_matmul_query(const mi355_grouped_desc_t *desc);

/* Name of the implementation a launch of `desc` uses ("" if none does). */
const char *mi355_grouped_matmul_impl(const mi355_grouped_desc_t *desc);

/* Asynchronous on `stream`; no scratch.  The offsets are not validated (they
 * live on the device): rows outside every group are left untouched, a group
 * whose src and dst ranges differ in length computes the rows both have, and
 * no access leaves the tensors whatever the offsets hold.  Buffers that are
 * not 16-byte aligned run on "hip:ref_grouped:any". */
int mi355_grouped_matmul_launch(const mi355_grouped_desc_t *desc, const mi355_grouped_args_t *args, void *stream);

/* out[c] = sum_r x[r * ld + c] over `rows` rows, added in row order in f32 and
 * stored as out_dt (x_dt, out_dt: f32 / bf16 / f16).  The bias gradient of the
 * inner product, with the operation order of the reference's loop
 * (src/cpu/ref_inner_product.cpp:196-210).  Asynchronous on `stream`. */
int mi355_colsum_launch(const void *x, int x_dt, int64_t rows, int64_t cols, int64_t ld, void *out, int out_dt,
        void *stream);

/* The row softmax between the two matmuls of scaled dot-product attention
 * (ref_sdpa, src/gpu/intel/sdpa/ref.cl:21-84: score * scale, + mask, exp, / sum;
 * causal masks as in micro.cl:864-878: scores of keys beyond the diagonal are
 * -inf).  scores: dense f32 [b][h][sq][sk]; probs: the same shape in out_dt
 * (f32 / bf16 / f16).  The exponentials are taken relative to the row's largest
 * score, which the reference does not do: the same number wherever the
 * reference's exp does not overflow.  A row whose scores are all -inf gives
 * zeros (softmax_accurate_inf_as_zero) or NaN (softmax_accurate). */
typedef struct {
    int64_t b, h, sq, sk;
    int out_dt;
    int scale_dt;        /* MI355_DT_UNDEF: no scale; else one value of f32 / bf16 / f16 in device memory */
    int invert_scale;    /* multiply by 1 / scale, the reciprocal rounded to scale_dt */
    int mask_type;       /* 0 none, 1 buffer, 2 causal from the top left, 3 causal from the bottom right */
    int mask_dt;         /* f32 / bf16 / f16 (mask_type 1) */
    int inf_as_zero;
    int64_t mask_dims[4];   /* element (b % d0, h % d1, q % d2, k % d3) */
    int64_t mask_stride[4]; /* in elements */
} mi355_softmax_desc_t;
int mi355_sdpa_softmax_launch(const mi355_softmax_desc_t *desc, const void *scores, void *probs, const void *scale,
        const void *mask, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355_MATMUL_H */
