// C-ABI entry points: device / memory / stream / event helpers and the matmul
// dispatcher.  See include/mi355_matmul.h for what each replaces in the
// reference.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <stdlib.h>

#include <atomic>
#include <map>
#include <mutex>
#include <utility>

#include "kernels.hpp"

namespace mi355 {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

namespace {
struct tune_name_t {
    const char *name;
    const char *values; // accepted words, blank-separated
};
const tune_name_t TUNE_NAMES[TUNE_COUNT] = {
        {"MI355_I8_TILES", "large wide small narrow"},
        {"MI355_F8_TILES", "wide narrow"},
        {"MI355_H16_TILES", "wide"},
        {"MI355_GROUPED_IMPL", "ref short tall wide"},
        {"MI355_GEMM_ORDER", ""},
};
std::atomic<int> g_tune[TUNE_COUNT];
std::once_flag g_tune_once;

// word -> value; -1 = not a word of this switch.  MI355_GEMM_ORDER takes a small non-negative number.
int tune_parse(int key, const char *v) {
    if (!v || !*v || !strcmp(v, "auto")) return TUNE_AUTO;
    if (key == TUNE_GEMM_ORDER) {
        char *end = nullptr;
        const long x = strtol(v, &end, 10);
        return (end && *end == 0 && x >= 0 && x < 64) ? (int)x : -1;
    }
    static const struct {
        const char *w;
        int val;
    } words[] = {{"large", TUNE_LARGE}, {"wide", TUNE_WIDE}, {"small", TUNE_SMALL}, {"ref", TUNE_REF},
            {"short", TUNE_SHORT}, {"tall", TUNE_TALL}, {"narrow", TUNE_NARROW}};
    for (const auto &w : words) {
        if (strcmp(v, w.w)) continue;
        const char *hit = strstr(TUNE_NAMES[key].values, v);
        return hit ? w.val : -1;
    }
    return -1;
}
void tune_init() {
    for (int k = 0; k < TUNE_COUNT; ++k) {
        const int v = tune_parse(k, getenv(TUNE_NAMES[k].name));
        g_tune[k].store(v < 0 ? TUNE_AUTO : v, std::memory_order_relaxed);
    }
}
} // namespace

int tuning(tune_key_t key) {
    std::call_once(g_tune_once, tune_init);
    return g_tune[key].load(std::memory_order_relaxed);
}

int ensure_dynamic_lds(const void *kernel, int bytes, const char *who) {
    static std::mutex mu;
    static std::map<std::pair<const void *, int>, int> done; // (kernel, device) -> bytes reserved
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        set_error("%s: no current device", who);
        return MI355_RUNTIME_ERROR;
    }
    std::lock_guard<std::mutex> lock(mu);
    auto it = done.find({kernel, dev});
    if (it != done.end() && it->second >= bytes) return MI355_SUCCESS;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
        set_error("%s: cannot reserve %d bytes of LDS", who, bytes);
        return MI355_RUNTIME_ERROR;
    }
    done[{kernel, dev}] = bytes;
    return MI355_SUCCESS;
}

static int hip_status(hipError_t e, const char *what) {
    if (e == hipSuccess) return MI355_SUCCESS;
    set_error("%s: %s", what, hipGetErrorString(e));
    return e == hipErrorOutOfMemory ? MI355_OUT_OF_MEMORY : MI355_RUNTIME_ERROR;
}

static bool dt_known(int dt) {
    return dt >= MI355_DT_F16 && dt <= MI355_DT_F4_E2M1 && dt != MI355_DT_F64
            && dt != MI355_DT_BOOLEAN;
}

static int check_quant(const mi355_quant_t &q, const char *name) {
    if (q.dt == MI355_DT_UNDEF) return MI355_SUCCESS;
    if (!dt_known(q.dt) || q.group[0] < 1 || q.group[1] < 1 || (q.mask & ~7)) {
        set_error("bad quantization parameter %s", name);
        return MI355_INVALID_ARGUMENTS;
    }
    return MI355_SUCCESS;
}

static int validate(const mi355_matmul_desc_t *d) {
    if (!d) {
        set_error("null descriptor");
        return MI355_INVALID_ARGUMENTS;
    }
    if (d->batch < 0 || d->M < 0 || d->N < 0 || d->K < 0) {
        set_error("negative dimension");
        return MI355_INVALID_ARGUMENTS;
    }
    if (!dt_known(d->src_dt) || !dt_known(d->wei_dt) || !dt_known(d->dst_dt)
            || (d->bias_dt != MI355_DT_UNDEF && !dt_known(d->bias_dt))) {
        set_error("unknown data type");
        return MI355_INVALID_ARGUMENTS;
    }
    if (d->n_post_ops < 0 || d->n_post_ops > MI355_MAX_POST_OPS) {
        set_error("bad post-op count");
        return MI355_INVALID_ARGUMENTS;
    }
    for (int i = 0; i < d->n_post_ops; ++i) {
        const int k = d->post_ops[i].kind;
        if (k < MI355_PO_SUM || k > MI355_PO_SELECT_COND) {
            set_error("bad post-op kind at %d", i);
            return MI355_INVALID_ARGUMENTS;
        }
        // a select and its condition come as a pair
        const bool is_select = k == MI355_PO_BINARY && d->post_ops[i].alg == MI355_BINARY_SELECT;
        const bool next_is_cond = i + 1 < d->n_post_ops && d->post_ops[i + 1].kind == MI355_PO_SELECT_COND;
        const bool prev_is_select = i > 0 && d->post_ops[i - 1].kind == MI355_PO_BINARY
                && d->post_ops[i - 1].alg == MI355_BINARY_SELECT;
        if (is_select != next_is_cond || (k == MI355_PO_SELECT_COND) != prev_is_select) {
            set_error("post-op %d: a binary select is followed by its condition entry, which follows nothing else", i);
            return MI355_INVALID_ARGUMENTS;
        }
    }
    if (d->wei_packing != MI355_WEI_PACK_NONE && !woq64_layout_ok(*d)) {
        set_error("weights packing %d needs 4-bit weights, batch 1, K %% 32 == 0 and N %% 64 == 0", d->wei_packing);
        return MI355_INVALID_ARGUMENTS;
    }
    if (d->dst_scale_dynamic != MI355_DST_DYNAMIC_NONE) {
        // src/common/matmul.cpp:407-424
        const mi355_quant_t &q = d->dst_scale;
        const bool mx = d->dst_scale_dynamic == MI355_DST_DYNAMIC_MX, fp = d->dst_scale_dynamic == MI355_DST_DYNAMIC_FP;
        const int g = mx ? 32 : 16;
        const bool ok = (mx || fp) && q.dt == (mx ? MI355_DT_E8M0 : MI355_DT_F8_E4M3)
                && (q.mask & 6) == 6 && (d->batch == 1 || (q.mask & 1)) && q.group[0] == 1 && q.group[1] == g
                && d->N % g == 0 && (is_f8_dt(d->dst_dt) || d->dst_dt == MI355_DT_F4_E2M1) && quant_absent(d->dst_zp);
        if (!ok) {
            set_error("dynamic dst scales: e8m0 with groups 1 x 32 (MX) or f8_e4m3 with groups 1 x 16 (FP), full mask, "
                      "N a multiple of the group, f8 or f4 dst, no dst zero point");
            return MI355_INVALID_ARGUMENTS;
        }
    }
    int st;
    if ((st = check_quant(d->src_scale, "src scale"))) return st;
    if ((st = check_quant(d->wei_scale, "weights scale"))) return st;
    if ((st = check_quant(d->dst_scale, "dst scale"))) return st;
    if ((st = check_quant(d->src_zp, "src zero point"))) return st;
    if ((st = check_quant(d->wei_zp, "weights zero point"))) return st;
    if ((st = check_quant(d->dst_zp, "dst zero point"))) return st;
    if ((st = check_quant(d->src_pr, "src precomputed reduction"))) return st;
    // groups must tile the dimension they apply to
    const struct { const mi355_quant_t *q; long d0, d1; } gs[] = {
            {&d->src_scale, d->M, d->K}, {&d->wei_scale, d->K, d->N},
            {&d->src_zp, d->M, d->K}, {&d->wei_zp, d->K, d->N}, {&d->src_pr, d->M, d->K}};
    for (auto &g : gs) {
        if (g.q->dt == MI355_DT_UNDEF) continue;
        if (((g.q->mask & 2) && g.d0 % g.q->group[0]) || ((g.q->mask & 4) && g.d1 % g.q->group[1])) {
            set_error("quantization group does not divide the dimension");
            return MI355_INVALID_ARGUMENTS;
        }
    }
    if (!quant_absent(d->src_pr) && quant_absent(d->wei_zp)) {
        set_error("precomputed reductions need weights zero points");
        return MI355_INVALID_ARGUMENTS;
    }
    return MI355_SUCCESS;
}

typedef int (*supported_fn)(const mi355_matmul_desc_t &);

static int impl_supported(const mi355_matmul_desc_t &d, int impl) {
    // dynamic dst quantization: the generic kernel and the floating-point GEMM tiles
    if (d.dst_scale_dynamic != MI355_DST_DYNAMIC_NONE && impl != MI355_IMPL_REF && impl != MI355_IMPL_F8_MFMA
            && impl != MI355_IMPL_MXF4_MFMA && impl != MI355_IMPL_H16_MFMA)
        return MI355_UNIMPLEMENTED;
    // the ternary select post-op: generic kernel only
    for (int i = 0; i < d.n_post_ops; ++i)
        if (d.post_ops[i].kind == MI355_PO_SELECT_COND && impl != MI355_IMPL_REF) return MI355_UNIMPLEMENTED;
    // a 4-bit dst: the generic kernel, and the floating-point GEMM tiles where groups of four columns are whole bytes
    if (dt_bits(d.dst_dt) < 8 && impl != MI355_IMPL_REF
            && !((impl == MI355_IMPL_F8_MFMA || impl == MI355_IMPL_MXF4_MFMA || impl == MI355_IMPL_H16_MFMA)
                    && tile_nibble_dst_ok(d)))
        return MI355_UNIMPLEMENTED;
    // dropout and stochastic rounding: generic kernel only
    if (d.rnd_flags != 0 && impl != MI355_IMPL_REF) return MI355_UNIMPLEMENTED;
    switch (impl) {
        case MI355_IMPL_REF: return ref_supported(d);
        case MI355_IMPL_I8_MFMA: return i8_supported(d);
        case MI355_IMPL_F8_MFMA: return f8_supported(d);
        case MI355_IMPL_H16_MFMA: return h16_supported(d);
        case MI355_IMPL_MXF4_MFMA: return mxf4_supported(d);
        case MI355_IMPL_WOQ_GEMV: return woq_supported(d);
        case MI355_IMPL_WOQ_PACKED: return woqp_supported(d);
        default: return MI355_INVALID_ARGUMENTS;
    }
}

// priority order of the implementation list (fastest first, generic last),
// the role of an engine's impl_list_item_t[] in the reference
static const int g_impl_order[] = {MI355_IMPL_WOQ_PACKED, MI355_IMPL_WOQ_GEMV, MI355_IMPL_I8_MFMA, MI355_IMPL_F8_MFMA,
        MI355_IMPL_MXF4_MFMA, MI355_IMPL_H16_MFMA, MI355_IMPL_REF};

static int choose_impl(const mi355_matmul_desc_t &d, int *chosen) {
    if (d.impl != MI355_IMPL_AUTO) {
        const int st = impl_supported(d, d.impl);
        if (st == MI355_SUCCESS && chosen) *chosen = d.impl;
        return st;
    }
    for (int impl : g_impl_order)
        if (impl_supported(d, impl) == MI355_SUCCESS) {
            if (chosen) *chosen = impl;
            return MI355_SUCCESS;
        }
    set_error("no kernel family covers this problem");
    return MI355_UNIMPLEMENTED;
}

static void fill_quant(quant_dev_t &q, const mi355_quant_t &s, const void *p) {
    q.dt = s.dt;
    q.mask = s.mask;
    q.g0 = s.dt == MI355_DT_UNDEF ? 1 : s.group[0];
    q.g1 = s.dt == MI355_DT_UNDEF ? 1 : s.group[1];
    q.p = p;
}

static int build_problem(const mi355_matmul_desc_t &d, const mi355_matmul_args_t &a, problem_t &P) {
    memset(&P, 0, sizeof(P));
    P.B = d.batch; P.M = d.M; P.N = d.N; P.K = d.K;
    P.src_dt = d.src_dt; P.wei_dt = d.wei_dt; P.dst_dt = d.dst_dt; P.bias_dt = d.bias_dt;
    for (int i = 0; i < 3; ++i) {
        P.ss[i] = d.src_stride[i]; P.ws[i] = d.wei_stride[i];
        P.ds[i] = d.dst_stride[i]; P.bs[i] = d.bias_stride[i];
    }
    fill_quant(P.src_scale, d.src_scale, a.src_scale);
    fill_quant(P.wei_scale, d.wei_scale, a.wei_scale);
    fill_quant(P.dst_scale, d.dst_scale, a.dst_scale);
    fill_quant(P.src_zp, d.src_zp, a.src_zp);
    fill_quant(P.wei_zp, d.wei_zp, a.wei_zp);
    fill_quant(P.dst_zp, d.dst_zp, a.dst_zp);
    fill_quant(P.src_pr, d.src_pr, a.src_pr);
    P.apply_to_int = d.fpmath_apply_to_int;
    P.dst_scale_mode = d.dst_scale_mode;
    P.n_po = d.n_post_ops;
    P.sum_dt = MI355_DT_UNDEF;
    P.wei_packing = d.wei_packing;
    P.dst_dynamic = d.dst_scale_dynamic;
    P.src = a.src; P.wei = a.wei; P.bias = a.bias; P.dst = a.dst;
    P.rnd_flags = d.rnd_flags;
    P.drop_p = a.dropout_p; P.drop_seed = a.dropout_seed; P.drop_offset = a.dropout_offset; P.drop_mask = a.dropout_mask;
    if ((d.rnd_flags & MI355_RND_DROPOUT)
            && (!a.dropout_p || !a.dropout_seed || ((d.rnd_flags & MI355_RND_DROPOUT_OFFSET) && !a.dropout_offset)
                    || ((d.rnd_flags & MI355_RND_DROPOUT_MASK) && !a.dropout_mask))) {
        set_error("missing dropout argument (probability, seed, offset or mask)");
        return MI355_INVALID_ARGUMENTS;
    }
    const struct { const mi355_quant_t *q; const void *p; const char *n; } need[] = {
            {&d.src_scale, a.src_scale, "src scale"}, {&d.wei_scale, a.wei_scale, "weights scale"},
            {&d.dst_scale, a.dst_scale, "dst scale"}, {&d.src_zp, a.src_zp, "src zero point"},
            {&d.wei_zp, a.wei_zp, "weights zero point"}, {&d.dst_zp, a.dst_zp, "dst zero point"},
            {&d.src_pr, a.src_pr, "src precomputed reduction"}};
    for (auto &n : need)
        if (n.q->dt != MI355_DT_UNDEF && !n.p) {
            set_error("missing argument: %s", n.n);
            return MI355_INVALID_ARGUMENTS;
        }
    if (!a.src || !a.wei || !a.dst || (d.bias_dt != MI355_DT_UNDEF && !a.bias)) {
        set_error("missing src/weights/dst/bias pointer");
        return MI355_INVALID_ARGUMENTS;
    }
    for (int i = 0; i < d.n_post_ops; ++i) {
        const mi355_post_op_t &s = d.post_ops[i];
        po_dev_t &o = P.po[i];
        o.kind = s.kind; o.alg = s.alg; o.alpha = s.alpha; o.beta = s.beta; o.scale = s.scale;
        o.zp = s.zero_point; o.dt = s.dt;
        o.s0 = s.stride[0]; o.s1 = s.stride[1]; o.s2 = s.stride[2];
        o.p = a.po_arg[i];
        if ((s.kind == MI355_PO_BINARY || s.kind == MI355_PO_PRELU || s.kind == MI355_PO_SELECT_COND) && !o.p) {
            set_error("missing post-op argument %d", i);
            return MI355_INVALID_ARGUMENTS;
        }
        if (s.kind == MI355_PO_SUM && P.sum_dt == MI355_DT_UNDEF)
            P.sum_dt = s.dt ? s.dt : d.dst_dt;
    }
    return MI355_SUCCESS;
}

// Scratch memory of mi355_matmul_launch_noalloc: one array per GPU, part of the
// loaded code object, held until the process ends.  In host code the array's
// name is only a handle for hipGetSymbolAddress; the device address it yields
// (different on every GPU) is what kernels and copies are given.
static __device__ __align__(256) unsigned char g_static_scratch[MI355_NOALLOC_SCRATCH_BYTES];

static int static_scratch_address(void **out) {
    constexpr int MAX_DEVICES = 64;
    static std::mutex mu;
    static void *addr[MAX_DEVICES] = {};
    int dev = 0;
    int st = hip_status(hipGetDevice(&dev), "hipGetDevice");
    if (st) return st;
    if (dev < 0 || dev >= MAX_DEVICES) {
        set_error("device ordinal %d beyond the %d the static scratch table holds", dev, MAX_DEVICES);
        return MI355_RUNTIME_ERROR;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (!addr[dev]) {
        void *p = nullptr;
        st = hip_status(hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_scratch)), "hipGetSymbolAddress");
        if (st) return st;
        addr[dev] = p;
    }
    *out = addr[dev];
    return MI355_SUCCESS;
}

} // namespace mi355

using namespace mi355;

extern "C" {

const char *mi355_last_error(void) { return g_err; }

int mi355_tuning_set(const char *name, const char *value) {
    if (!name) return MI355_INVALID_ARGUMENTS;
    tuning(TUNE_I8_TILES); // the environment first, once
    for (int k = 0; k < TUNE_COUNT; ++k) {
        if (strcmp(name, TUNE_NAMES[k].name)) continue;
        const int v = tune_parse(k, value);
        if (v < 0) {
            set_error("mi355_tuning_set: %s does not take '%s'", name, value);
            return MI355_INVALID_ARGUMENTS;
        }
        g_tune[k].store(v, std::memory_order_relaxed);
        return MI355_SUCCESS;
    }
    set_error("mi355_tuning_set: unknown switch %s", name);
    return MI355_INVALID_ARGUMENTS;
}

int mi355_device_count(int *count) {
    if (!count) return MI355_INVALID_ARGUMENTS;
    return hip_status(hipGetDeviceCount(count), "hipGetDeviceCount");
}

int mi355_device_set(int device) { return hip_status(hipSetDevice(device), "hipSetDevice"); }

int mi355_device_info(int device, char *name, size_t name_len, int *cus, int *clock_khz,
        int64_t *hbm_bytes, int64_t *l2_bytes) {
    hipDeviceProp_t prop;
    const int st = hip_status(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties");
    if (st) return st;
    if (name && name_len) snprintf(name, name_len, "%s", prop.gcnArchName);
    if (cus) *cus = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (hbm_bytes) *hbm_bytes = (int64_t)prop.totalGlobalMem;
    if (l2_bytes) *l2_bytes = (int64_t)prop.l2CacheSize;
    return MI355_SUCCESS;
}

int mi355_mem_alloc(void **dptr, size_t bytes) {
    if (!dptr) return MI355_INVALID_ARGUMENTS;
    *dptr = nullptr;
    if (bytes == 0) return MI355_SUCCESS;
    return hip_status(hipMalloc(dptr, bytes), "hipMalloc");
}
int mi355_mem_free(void *dptr) {
    if (!dptr) return MI355_SUCCESS;
    return hip_status(hipFree(dptr), "hipFree");
}
int mi355_mem_set(void *dptr, int byte, size_t bytes, void *stream) {
    if (bytes == 0) return MI355_SUCCESS;
    return hip_status(hipMemsetAsync(dptr, byte, bytes, (hipStream_t)stream), "hipMemsetAsync");
}
int mi355_mem_h2d(void *dptr, const void *hptr, size_t bytes, void *stream) {
    if (bytes == 0) return MI355_SUCCESS;
    int st = hip_status(hipMemcpyAsync(dptr, hptr, bytes, hipMemcpyHostToDevice, (hipStream_t)stream),
            "hipMemcpyAsync(h2d)");
    if (st) return st;
    // the host buffer is pageable: complete before returning
    return hip_status(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
}
int mi355_mem_d2h(void *hptr, const void *dptr, size_t bytes, void *stream) {
    if (bytes == 0) return MI355_SUCCESS;
    int st = hip_status(hipMemcpyAsync(hptr, dptr, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream),
            "hipMemcpyAsync(d2h)");
    if (st) return st;
    return hip_status(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
}
int mi355_mem_d2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return MI355_SUCCESS;
    return hip_status(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream),
            "hipMemcpyAsync(d2d)");
}
int mi355_stream_create(void **stream) {
    if (!stream) return MI355_INVALID_ARGUMENTS;
    hipStream_t s;
    const int st = hip_status(hipStreamCreate(&s), "hipStreamCreate");
    *stream = st ? nullptr : (void *)s;
    return st;
}
int mi355_stream_destroy(void *stream) {
    if (!stream) return MI355_SUCCESS;
    return hip_status(hipStreamDestroy((hipStream_t)stream), "hipStreamDestroy");
}
int mi355_graph_capture_begin(void *stream) {
    if (!stream) {
        set_error("graph capture needs a created stream");
        return MI355_INVALID_ARGUMENTS;
    }
    // (thread-local: what other host threads call meanwhile does not concern this capture)
    return hip_status(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
}
int mi355_graph_capture_end(void *stream, void **graph) {
    if (!stream || !graph) return MI355_INVALID_ARGUMENTS;
    *graph = nullptr;
    hipGraph_t g = nullptr;
    if (const int st = hip_status(hipStreamEndCapture((hipStream_t)stream, &g), "hipStreamEndCapture")) return st;
    hipGraphExec_t exec = nullptr;
    const int st = hip_status(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0), "hipGraphInstantiate");
    (void)hipGraphDestroy(g);
    if (st) return st;
    *graph = (void *)exec;
    return MI355_SUCCESS;
}
int mi355_graph_launch(void *graph, void *stream) {
    if (!graph) return MI355_INVALID_ARGUMENTS;
    return hip_status(hipGraphLaunch((hipGraphExec_t)graph, (hipStream_t)stream), "hipGraphLaunch");
}
int mi355_graph_destroy(void *graph) {
    if (!graph) return MI355_SUCCESS;
    return hip_status(hipGraphExecDestroy((hipGraphExec_t)graph), "hipGraphExecDestroy");
}
int mi355_stream_sync(void *stream) {
    return hip_status(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
}
int mi355_event_create(void **event) {
    if (!event) return MI355_INVALID_ARGUMENTS;
    hipEvent_t e;
    const int st = hip_status(hipEventCreate(&e), "hipEventCreate");
    *event = st ? nullptr : (void *)e;
    return st;
}
int mi355_event_destroy(void *event) {
    if (!event) return MI355_SUCCESS;
    return hip_status(hipEventDestroy((hipEvent_t)event), "hipEventDestroy");
}
int mi355_event_record(void *event, void *stream) {
    return hip_status(hipEventRecord((hipEvent_t)event, (hipStream_t)stream), "hipEventRecord");
}
int mi355_event_sync(void *event) {
    return hip_status(hipEventSynchronize((hipEvent_t)event), "hipEventSynchronize");
}
int mi355_stream_wait_event(void *stream, void *event) {
    return hip_status(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0), "hipStreamWaitEvent");
}
int mi355_event_elapsed_ms(float *ms, void *start, void *stop) {
    if (!ms) return MI355_INVALID_ARGUMENTS;
    return hip_status(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop), "hipEventElapsedTime");
}

const char *mi355_matmul_impl_name(int impl) {
    switch (impl) {
        case MI355_IMPL_REF: return "hip:ref:any";
        case MI355_IMPL_I8_MFMA: return "hip:mfma_i8:gfx950";
        case MI355_IMPL_F8_MFMA: return "hip:mfma_f8:gfx950";
        case MI355_IMPL_H16_MFMA: return "hip:mfma_h16:gfx950";
        case MI355_IMPL_MXF4_MFMA: return "hip:mfma_mxf4:gfx950";
        case MI355_IMPL_WOQ_GEMV: return "hip:woq_gemv:gfx950";
        case MI355_IMPL_WOQ_PACKED: return "hip:woq_packed:gfx950";
        default: return "undef";
    }
}

int mi355_matmul_query(const mi355_matmul_desc_t *desc, int impl, int *chosen_impl) {
    int st = validate(desc);
    if (st) return st;
    if (impl == MI355_IMPL_AUTO) return choose_impl(*desc, chosen_impl);
    if (impl < MI355_IMPL_REF || impl >= MI355_IMPL_COUNT) {
        set_error("unknown implementation id %d", impl);
        return MI355_INVALID_ARGUMENTS;
    }
    st = impl_supported(*desc, impl);
    if (st == MI355_SUCCESS && chosen_impl) *chosen_impl = impl;
    if (st == MI355_UNIMPLEMENTED) set_error("%s does not cover this problem", mi355_matmul_impl_name(impl));
    return st;
}

int mi355_matmul_scratch_bytes(const mi355_matmul_desc_t *desc, size_t *bytes) {
    if (!bytes) return MI355_INVALID_ARGUMENTS;
    *bytes = 0;
    int st = validate(desc);
    if (st) return st;
    int impl = 0;
    if ((st = choose_impl(*desc, &impl))) return st;
    switch (impl) {
        case MI355_IMPL_I8_MFMA: *bytes = i8_scratch_bytes(*desc); break;
        case MI355_IMPL_F8_MFMA: *bytes = f8_scratch_bytes(*desc); break;
        case MI355_IMPL_H16_MFMA: *bytes = h16_scratch_bytes(*desc); break;
        case MI355_IMPL_MXF4_MFMA: *bytes = mxf4_scratch_bytes(*desc); break;
        case MI355_IMPL_WOQ_GEMV: *bytes = woq_scratch_bytes(*desc); break;
        default: break;
    }
    return MI355_SUCCESS;
}

int mi355_matmul_launch(const mi355_matmul_desc_t *desc, const mi355_matmul_args_t *args,
        void *scratch, void *stream) {
    int st = validate(desc);
    if (st) return st;
    if (!args) {
        set_error("null arguments");
        return MI355_INVALID_ARGUMENTS;
    }
    // zero-dim problems (K == 0 included) are a successful no-op that leaves dst
    // untouched (src/cpu/matmul/ref_matmul_int8.cpp:70-72)
    if (desc->batch == 0 || desc->M == 0 || desc->N == 0 || desc->K == 0) return MI355_SUCCESS;
    int impl = 0;
    if ((st = choose_impl(*desc, &impl))) return st;
    problem_t P;
    if ((st = build_problem(*desc, *args, P))) return st;
    hipStream_t s = (hipStream_t)stream;
    switch (impl) {
        case MI355_IMPL_REF: return ref_launch(P, s);
        case MI355_IMPL_I8_MFMA: return i8_launch(*desc, P, scratch, s);
        case MI355_IMPL_F8_MFMA: return f8_launch(*desc, P, scratch, s);
        case MI355_IMPL_H16_MFMA: return h16_launch(*desc, P, scratch, s);
        case MI355_IMPL_MXF4_MFMA: return mxf4_launch(*desc, P, scratch, s);
        case MI355_IMPL_WOQ_GEMV: return woq_launch(*desc, P, scratch, s);
        case MI355_IMPL_WOQ_PACKED: return woqp_launch(*desc, P, s);
        default: return MI355_UNIMPLEMENTED;
    }
}

int mi355_matmul_launch_noalloc(const mi355_matmul_desc_t *desc, const mi355_matmul_args_t *args,
        void *stream) {
    size_t bytes = 0;
    int st = mi355_matmul_scratch_bytes(desc, &bytes);
    if (st) return st;
    if (bytes > (size_t)MI355_NOALLOC_SCRATCH_BYTES) {
        set_error("mi355_matmul_launch_noalloc: the problem needs %zu bytes of scratch, the static buffer holds %zu "
                  "(use mi355_matmul_launch with a caller-owned buffer, or K-contiguous weights)",
                bytes, (size_t)MI355_NOALLOC_SCRATCH_BYTES);
        return MI355_INVALID_ARGUMENTS;
    }
    void *scratch = nullptr;
    if (bytes > 0 && (st = static_scratch_address(&scratch))) return st;
    // every kernel family writes the part of its scratch it reads within the same
    // launch (transposed weights, row / column sums, split-K partial sums): nothing
    // has to start at zero
    return mi355_matmul_launch(desc, args, scratch, stream);
}

} // extern "C"
