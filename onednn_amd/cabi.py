"""ctypes binding of the thin C ABI (include/mi355_matmul.h).

The structures mirror the header field for field.  Loading fails loudly when
the HIP library has not been built: there is no CPU fallback behind this
module.
"""
import ctypes as C
import os

import numpy as np

MAX_POST_OPS = 32

# data types (dnnl_data_type_t values)
DT_UNDEF, DT_F16, DT_BF16, DT_F32, DT_S32, DT_S8, DT_U8, DT_F64, DT_BOOLEAN = range(9)
DT_F8_E5M2, DT_F8_E4M3, DT_S4, DT_U4, DT_E8M0, DT_F4_E2M1 = 9, 10, 11, 12, 13, 14

DT_NAMES = {
    "undef": DT_UNDEF, "f16": DT_F16, "bf16": DT_BF16, "f32": DT_F32, "s32": DT_S32,
    "s8": DT_S8, "u8": DT_U8, "f8_e5m2": DT_F8_E5M2, "f8_e4m3": DT_F8_E4M3, "s4": DT_S4,
    "u4": DT_U4, "e8m0": DT_E8M0, "f4_e2m1": DT_F4_E2M1,
}
DT_BITS = {DT_F16: 16, DT_BF16: 16, DT_F32: 32, DT_S32: 32, DT_S8: 8, DT_U8: 8,
           DT_F8_E5M2: 8, DT_F8_E4M3: 8, DT_S4: 4, DT_U4: 4, DT_E8M0: 8, DT_F4_E2M1: 4}

SUCCESS, OUT_OF_MEMORY, INVALID_ARGUMENTS, UNIMPLEMENTED, LAST_IMPL_REACHED, RUNTIME_ERROR, NOT_REQUIRED = range(7)

PO_SUM, PO_ELTWISE, PO_BINARY, PO_PRELU, PO_SELECT_COND = 1, 2, 3, 4, 5

ELTWISE = {
    "relu": 0x20, "tanh": 0x21, "elu": 0x22, "square": 0x23, "abs": 0x24, "sqrt": 0x25,
    "linear": 0x26, "soft_relu": 0x27, "hardsigmoid": 0x28, "logistic": 0x29, "exp": 0x2a,
    "gelu_tanh": 0x2b, "swish": 0x2c, "log": 0x2d, "clip": 0x2e, "clip_v2": 0x2f, "pow": 0x30,
    "gelu_erf": 0x31, "round": 0x32, "mish": 0x33, "hardswish": 0x34,
}
BINARY = {
    "add": 0x1fff0, "mul": 0x1fff1, "max": 0x1fff2, "min": 0x1fff3, "div": 0x1fff4,
    "sub": 0x1fff5, "ge": 0x1fff6, "gt": 0x1fff7, "le": 0x1fff8, "lt": 0x1fff9,
    "eq": 0x1fffa, "ne": 0x1fffb, "select": 0x1fffc,
}

DST_SCALE_DIVIDE, DST_SCALE_RECIPROCAL = 0, 1
IMPL_AUTO, IMPL_REF, IMPL_I8_MFMA, IMPL_F8_MFMA, IMPL_MXF4_MFMA, IMPL_WOQ_GEMV, IMPL_WOQ_PACKED = range(7)
IMPL_H16_MFMA = 7
NOALLOC_SCRATCH_BYTES = 8 << 20
WEI_PACK_NONE, WEI_PACK_WOQ64 = 0, 1
DST_DYNAMIC_NONE, DST_DYNAMIC_MX, DST_DYNAMIC_FP = 0, 1, 2


class Quant(C.Structure):
    _fields_ = [("dt", C.c_int32), ("mask", C.c_int32), ("group", C.c_int64 * 2)]


class PostOp(C.Structure):
    _fields_ = [("kind", C.c_int32), ("alg", C.c_int32), ("alpha", C.c_float),
                ("beta", C.c_float), ("scale", C.c_float), ("zero_point", C.c_int32),
                ("dt", C.c_int32), ("stride", C.c_int64 * 3)]


class MatmulDesc(C.Structure):
    _fields_ = [
        ("batch", C.c_int64), ("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64),
        ("src_dt", C.c_int32), ("wei_dt", C.c_int32), ("dst_dt", C.c_int32), ("bias_dt", C.c_int32),
        ("src_stride", C.c_int64 * 3), ("wei_stride", C.c_int64 * 3),
        ("dst_stride", C.c_int64 * 3), ("bias_stride", C.c_int64 * 3),
        ("src_scale", Quant), ("wei_scale", Quant), ("dst_scale", Quant),
        ("src_zp", Quant), ("wei_zp", Quant), ("dst_zp", Quant), ("src_pr", Quant),
        ("fpmath_apply_to_int", C.c_int32), ("fpmath_mode", C.c_int32),
        ("dst_scale_mode", C.c_int32), ("n_post_ops", C.c_int32),
        ("post_ops", PostOp * MAX_POST_OPS),
        ("impl", C.c_int32), ("wei_packing", C.c_int32),
        ("dst_scale_dynamic", C.c_int32), ("rnd_flags", C.c_int32),
    ]


RND_DROPOUT, RND_DROPOUT_MASK, RND_SEED_S64, RND_DROPOUT_OFFSET, RND_DST_STOCHASTIC = 1, 2, 4, 8, 16


class MatmulArgs(C.Structure):
    _fields_ = [
        ("src", C.c_void_p), ("wei", C.c_void_p), ("bias", C.c_void_p), ("dst", C.c_void_p),
        ("src_scale", C.c_void_p), ("wei_scale", C.c_void_p), ("dst_scale", C.c_void_p),
        ("src_zp", C.c_void_p), ("wei_zp", C.c_void_p), ("dst_zp", C.c_void_p),
        ("src_pr", C.c_void_p),
        ("po_arg", C.c_void_p * MAX_POST_OPS),
        ("dropout_p", C.c_void_p), ("dropout_seed", C.c_void_p), ("dropout_offset", C.c_void_p),
        ("dropout_mask", C.c_void_p),
    ]


class GroupedPostOp(C.Structure):
    """mi355_grouped_post_op_t"""
    _fields_ = [("kind", C.c_int32), ("alg", C.c_int32), ("alpha", C.c_float), ("beta", C.c_float),
                ("scale", C.c_float), ("dt", C.c_int32), ("bin_m", C.c_int64), ("bin_n", C.c_int64),
                ("grouped", C.c_int32)]


class GroupedDesc(C.Structure):
    """mi355_grouped_desc_t"""
    _fields_ = [
        ("pattern", C.c_int32), ("group_count", C.c_int64), ("total", C.c_int64), ("M", C.c_int64),
        ("K", C.c_int64), ("N", C.c_int64),
        ("src_dt", C.c_int32), ("wei_dt", C.c_int32), ("dst_dt", C.c_int32), ("bias_dt", C.c_int32),
        ("wei_stride", C.c_int64 * 3), ("dst_stride", C.c_int64 * 3),
        ("src_scale_dt", C.c_int32), ("wei_scale_dt", C.c_int32), ("src_zp_dt", C.c_int32), ("wei_zp_dt", C.c_int32),
        ("src_scale_gk", C.c_int64), ("wei_scale_gk", C.c_int64), ("src_zp_gk", C.c_int64), ("wei_zp_gk", C.c_int64),
        ("fpmath_apply_to_int", C.c_int32), ("n_post_ops", C.c_int32),
        ("post_ops", GroupedPostOp * MAX_POST_OPS),
    ]


class GroupedArgs(C.Structure):
    """mi355_grouped_args_t"""
    _fields_ = [
        ("src", C.c_void_p), ("wei", C.c_void_p), ("bias", C.c_void_p), ("dst", C.c_void_p),
        ("src_offsets", C.c_void_p), ("wei_offsets", C.c_void_p), ("dst_offsets", C.c_void_p),
        ("src_scale", C.c_void_p), ("wei_scale", C.c_void_p), ("src_zp", C.c_void_p), ("wei_zp", C.c_void_p),
        ("po_arg", C.c_void_p * MAX_POST_OPS), ("po_offsets", C.c_void_p * MAX_POST_OPS),
    ]


GROUPED_2DX3D, GROUPED_2DX2D = 0, 1
REORDER_MAX_DIMS = 6


class ReorderDesc(C.Structure):
    """mi355_reorder_desc_t"""
    _fields_ = [
        ("ndims", C.c_int32), ("src_dt", C.c_int32), ("dst_dt", C.c_int32), ("reserved", C.c_int32),
        ("dims", C.c_int64 * REORDER_MAX_DIMS), ("src_stride", C.c_int64 * REORDER_MAX_DIMS),
        ("dst_stride", C.c_int64 * REORDER_MAX_DIMS),
        ("src_scale", Quant), ("dst_scale", Quant), ("src_zp", Quant), ("dst_zp", Quant),
        ("beta", C.c_float), ("reserved2", C.c_int32),
    ]


class ReorderArgs(C.Structure):
    """mi355_reorder_args_t"""
    _fields_ = [
        ("src", C.c_void_p), ("dst", C.c_void_p), ("src_scale", C.c_void_p), ("dst_scale", C.c_void_p),
        ("src_zp", C.c_void_p), ("dst_zp", C.c_void_p),
    ]


# every symbol include/mi355_matmul.h declares
KERNEL_SYMBOLS = [
    "mi355_device_count", "mi355_device_set", "mi355_device_info", "mi355_mem_alloc",
    "mi355_mem_free", "mi355_mem_set", "mi355_mem_h2d", "mi355_mem_d2h", "mi355_mem_d2d",
    "mi355_stream_create", "mi355_stream_destroy", "mi355_stream_sync", "mi355_event_create",
    "mi355_event_destroy", "mi355_event_record", "mi355_event_sync", "mi355_event_elapsed_ms",
    "mi355_stream_wait_event", "mi355_mem_store_scalar",
    "mi355_graph_capture_begin", "mi355_graph_capture_end", "mi355_graph_launch", "mi355_graph_destroy",
    "mi355_last_error", "mi355_matmul_query", "mi355_matmul_impl_name",
    "mi355_matmul_scratch_bytes", "mi355_matmul_launch", "mi355_matmul_launch_noalloc", "mi355_reorder_query",
    "mi355_reorder_launch", "mi355_wei_pack_reorder_dims", "mi355_tuning_set", "mi355_colsum_launch", "mi355_sdpa_softmax_launch",
    "mi355_grouped_matmul_query",
    "mi355_grouped_matmul_launch", "mi355_grouped_matmul_impl",
]

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
KERNEL_LIB_PATH = os.path.join(_PKG_DIR, "lib", "libmi355_matmul.so")
_lib = None


class Mi355Error(RuntimeError):
    def __init__(self, status, msg):
        super().__init__(f"mi355 status {status}: {msg}")
        self.status = status


def load_kernels():
    """Load libmi355_matmul.so (built by onednn_amd/csrc/Makefile)."""
    global _lib
    if _lib is not None:
        return _lib
    path = os.environ.get("MI355_KERNEL_LIB", KERNEL_LIB_PATH)
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `make -C onednn_amd/csrc` "
            "(or __graft_entry__.build()); there is no fallback path")
    lib = C.CDLL(path)
    vp = C.c_void_p
    lib.mi355_last_error.restype = C.c_char_p
    lib.mi355_matmul_impl_name.restype = C.c_char_p
    lib.mi355_matmul_impl_name.argtypes = [C.c_int]
    lib.mi355_tuning_set.argtypes = [C.c_char_p, C.c_char_p]
    lib.mi355_colsum_launch.argtypes = [vp, C.c_int, C.c_int64, C.c_int64, C.c_int64, vp, C.c_int, vp]
    lib.mi355_device_count.argtypes = [C.POINTER(C.c_int)]
    lib.mi355_device_set.argtypes = [C.c_int]
    lib.mi355_device_info.argtypes = [C.c_int, C.c_char_p, C.c_size_t, C.POINTER(C.c_int),
                                      C.POINTER(C.c_int), C.POINTER(C.c_int64),
                                      C.POINTER(C.c_int64)]
    lib.mi355_mem_alloc.argtypes = [C.POINTER(vp), C.c_size_t]
    lib.mi355_mem_free.argtypes = [vp]
    lib.mi355_mem_set.argtypes = [vp, C.c_int, C.c_size_t, vp]
    lib.mi355_mem_h2d.argtypes = [vp, vp, C.c_size_t, vp]
    lib.mi355_mem_d2h.argtypes = [vp, vp, C.c_size_t, vp]
    lib.mi355_mem_d2d.argtypes = [vp, vp, C.c_size_t, vp]
    lib.mi355_stream_create.argtypes = [C.POINTER(vp)]
    lib.mi355_stream_destroy.argtypes = [vp]
    lib.mi355_stream_sync.argtypes = [vp]
    lib.mi355_event_create.argtypes = [C.POINTER(vp)]
    lib.mi355_event_destroy.argtypes = [vp]
    lib.mi355_event_record.argtypes = [vp, vp]
    lib.mi355_event_sync.argtypes = [vp]
    lib.mi355_event_elapsed_ms.argtypes = [C.POINTER(C.c_float), vp, vp]
    lib.mi355_stream_wait_event.argtypes = [vp, vp]
    lib.mi355_graph_capture_begin.argtypes = [vp]
    lib.mi355_graph_capture_end.argtypes = [vp, C.POINTER(vp)]
    lib.mi355_graph_launch.argtypes = [vp, vp]
    lib.mi355_graph_destroy.argtypes = [vp]
    lib.mi355_mem_store_scalar.argtypes = [vp, C.c_uint64, C.c_int, vp]
    lib.mi355_matmul_query.argtypes = [C.POINTER(MatmulDesc), C.c_int, C.POINTER(C.c_int)]
    lib.mi355_matmul_scratch_bytes.argtypes = [C.POINTER(MatmulDesc), C.POINTER(C.c_size_t)]
    lib.mi355_matmul_launch.argtypes = [C.POINTER(MatmulDesc), C.POINTER(MatmulArgs), vp, vp]
    lib.mi355_matmul_launch_noalloc.argtypes = [C.POINTER(MatmulDesc), C.POINTER(MatmulArgs), vp]
    lib.mi355_reorder_query.argtypes = [C.POINTER(ReorderDesc)]
    lib.mi355_reorder_launch.argtypes = [C.POINTER(ReorderDesc), C.POINTER(ReorderArgs), vp]
    lib.mi355_wei_pack_reorder_dims.argtypes = [C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int64,
                                                C.POINTER(ReorderDesc)]
    lib.mi355_grouped_matmul_query.argtypes = [C.POINTER(GroupedDesc)]
    lib.mi355_grouped_matmul_launch.argtypes = [C.POINTER(GroupedDesc), C.POINTER(GroupedArgs), vp]
    lib.mi355_grouped_matmul_impl.argtypes = [C.POINTER(GroupedDesc)]
    lib.mi355_grouped_matmul_impl.restype = C.c_char_p
    _lib = lib
    return lib


def check(status):
    if status != SUCCESS:
        raise Mi355Error(status, load_kernels().mi355_last_error().decode())


def gpu_available():
    try:
        lib = load_kernels()
    except (ImportError, OSError):
        return False
    n = C.c_int(0)
    return lib.mi355_device_count(C.byref(n)) == SUCCESS and n.value > 0


class Stream:
    """A created (non-default) stream."""

    def __init__(self):
        self.lib = load_kernels()
        p = C.c_void_p()
        check(self.lib.mi355_stream_create(C.byref(p)))
        self.ptr = p.value

    def sync(self):
        check(self.lib.mi355_stream_sync(self.ptr))

    def destroy(self):
        if self.ptr:
            self.lib.mi355_stream_destroy(self.ptr)
            self.ptr = None


class Graph:
    """with Graph(stream) as g: <launches on stream>  -- records them; g.launch() replays them in order."""

    def __init__(self, stream):
        self.lib, self.stream, self.exec = load_kernels(), stream, None

    def __enter__(self):
        check(self.lib.mi355_graph_capture_begin(self.stream.ptr))
        return self

    def __exit__(self, *exc):
        p = C.c_void_p()
        st = self.lib.mi355_graph_capture_end(self.stream.ptr, C.byref(p))
        if exc[0] is None:
            check(st)
        self.exec = p.value
        return False

    def launch(self):
        check(self.lib.mi355_graph_launch(self.exec, self.stream.ptr))

    def destroy(self):
        if self.exec:
            self.lib.mi355_graph_destroy(self.exec)
            self.exec = None


class DeviceBuffer:
    """A device allocation owned by Python (hipMalloc / hipFree)."""

    def __init__(self, nbytes):
        self.lib = load_kernels()
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(self.lib.mi355_mem_alloc(C.byref(p), max(self.nbytes, 1)))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, arr):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        if arr.nbytes:
            check(buf.lib.mi355_mem_h2d(buf.ptr, arr.ctypes.data, arr.nbytes, None))
        return buf

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes
        if arr.nbytes:
            check(self.lib.mi355_mem_h2d(self.ptr, arr.ctypes.data, arr.nbytes, None))

    def to_numpy(self, dtype, shape):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        if out.nbytes:
            check(self.lib.mi355_mem_d2h(out.ctypes.data, self.ptr, out.nbytes, None))
        return out

    def free(self):
        if self.ptr:
            self.lib.mi355_mem_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def impl_name(impl):
    return load_kernels().mi355_matmul_impl_name(impl).decode()


def query(desc, impl=IMPL_AUTO):
    """Returns (status, chosen implementation id)."""
    chosen = C.c_int(0)
    st = load_kernels().mi355_matmul_query(C.byref(desc), impl, C.byref(chosen))
    return st, chosen.value


def scratch_bytes(desc):
    n = C.c_size_t(0)
    check(load_kernels().mi355_matmul_scratch_bytes(C.byref(desc), C.byref(n)))
    return n.value


def tuning_set(name, value=None):
    """Set one of the library's tuning switches (MI355_I8_TILES, MI355_F8_TILES, MI355_H16_TILES,
    MI355_GROUPED_IMPL, MI355_GEMM_ORDER); None restores the library's own choice.  The switches start from the
    environment variables of the same names, read once per process."""
    lib = load_kernels()
    check(lib.mi355_tuning_set(name.encode(), None if value is None else str(value).encode()))


class tuning:
    """with tuning("MI355_I8_TILES", "small"): ...  -- the switch is back on the library's choice afterwards."""

    def __init__(self, name, value):
        self.name, self.value = name, value

    def __enter__(self):
        tuning_set(self.name, self.value)
        return self

    def __exit__(self, *exc):
        tuning_set(self.name, None)
        return False
