"""ctypes mirror of the dnnl_* C API subset (include/dnnl_amd.h), shaped after
oneDNN's C++ wrappers (include/oneapi/dnnl/dnnl.hpp: engine, stream,
memory::desc, memory, primitive_attr, post_ops, matmul::primitive_desc,
matmul) so that tests read like the reference's.  Every status other than
success raises `error`, as dnnl::error does.
"""
import ctypes as C
import os

import numpy as np

from . import cabi

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_PKG_DIR, "lib", "libdnnl_amd.so")
_lib = None

MAX_NDIMS = 12
dims_t = C.c_int64 * MAX_NDIMS

# enums (include/dnnl_amd.h)
success, out_of_memory, invalid_arguments, unimplemented, last_impl_reached, runtime_error = range(6)
cpu, gpu = 1, 2
tag_any, tag_a, tag_ab, tag_abc, tag_abcd, tag_ba, tag_acb, tag_abdc = 1, 2, 3, 4, 5, 14, 15, 20
tag_abcde, tag_acdb, tag_acdeb = 6, 22, 33
tag_x, tag_nc, tag_ncw, tag_nwc, tag_nchw, tag_nhwc, tag_ncdhw, tag_ndhwc = 2, 3, 4, 15, 5, 22, 6, 33
tag_oi, tag_io, tag_oiw, tag_owi, tag_oihw, tag_ohwi, tag_oidhw, tag_odhwi = 3, 14, 4, 15, 5, 22, 6, 33
kind_sum, kind_eltwise, kind_binary, kind_matmul, kind_prelu = 4, 7, 13, 14, 18
kind_inner_product = 10
forward_training, forward_inference, backward_data, backward_weights = 64, 96, 160, 192
query_primitive_kind, query_prop_kind = 2, 11
query_impl_info_str, query_src_md, query_weights_md, query_dst_md, query_scratchpad_md = 8, 129, 131, 133, 136
query_diff_src_md, query_diff_weights_md, query_diff_dst_md = 130, 132, 134
query_ndims_s32, query_dims, query_data_type, query_strides, query_memory_consumption = 256, 257, 258, 14, 6
query_format_kind = 262
quantization_mode_undef, quantization_mode_static_sazp, quantization_mode_dynamic_mx, quantization_mode_dynamic_fp = 0, 1, 2, 3
format_kind_undef, format_kind_any, format_kind_blocked, format_kind_opaque = 0, 1, 2, 3
ARG_SRC, ARG_SRC_1, ARG_DST, ARG_WEIGHTS, ARG_BIAS, ARG_SCRATCHPAD = 1, 2, 17, 33, 41, 80
ARG_SRC_2 = 3
ARG_FROM, ARG_TO = ARG_SRC, ARG_DST
ARG_ATTR_PRECOMPUTED_REDUCTIONS, ARG_ATTR_SCALES, ARG_ATTR_ZERO_POINTS = 512, 4096, 8192
ARG_ATTR_DROPOUT_OFFSET, ARG_ATTR_ROUNDING_SEED, ARG_ATTR_DROPOUT_MASK = 507, 508, 509
ARG_ATTR_DROPOUT_PROBABILITY, ARG_ATTR_DROPOUT_SEED = 510, 511
ARG_DIFF_SRC, ARG_DIFF_DST, ARG_DIFF_WEIGHTS, ARG_DIFF_BIAS = 129, 145, 161, 169
ARG_QUERIES, ARG_KEYS, ARG_VALUES, ARG_SCALE, ARG_ATTN_MASK = 1, 2, 3, 51, 52
kind_sdpa = (1 << 12) + 1
softmax_accurate, softmax_accurate_inf_as_zero = 0x30000, (1 << 12) + 2
attn_mask_undef, attn_mask_buffer, attn_mask_top_left, attn_mask_bottom_right = 0, 1, 2, 3
rounding_environment, rounding_stochastic = 0, 1
s64 = 16                               # dnnl_s64: the dropout seed / offset type
scratchpad_library, scratchpad_user = 0, 1
fpmath_strict, fpmath_bf16, fpmath_f16, fpmath_any = 0, 1, 2, 3
MEMORY_ALLOCATE = C.c_void_p(-1 & (2 ** 64 - 1))
RUNTIME_DIM_VAL = -(2 ** 63)           # DNNL_RUNTIME_DIM_VAL, dnnl_types.h:2331
RUNTIME_SIZE_VAL = 2 ** 63             # DNNL_RUNTIME_SIZE_VAL, dnnl_types.h:2336


def ARG_ATTR_MULTIPLE_POST_OP(idx):
    return 32768 * (idx + 1)


class ExecArg(C.Structure):
    _fields_ = [("arg", C.c_int), ("memory", C.c_void_p)]


class error(RuntimeError):
    def __init__(self, status, what):
        super().__init__(f"{what}: status {status}")
        self.status = status


def lib():
    global _lib
    if _lib is None:
        cabi.load_kernels()
        if not os.path.exists(HOST_LIB_PATH):
            raise ImportError(f"{HOST_LIB_PATH} is missing: build it with `make -C onednn_amd/host`")
        _lib = C.CDLL(HOST_LIB_PATH)
        _lib.dnnl_memory_desc_get_size.restype = C.c_size_t
        _lib.dnnl_primitive_desc_query_md.restype = C.c_void_p
        _lib.dnnl_engine_get_count.restype = C.c_size_t
    return _lib


def _check(st, what):
    if st != success:
        raise error(st, what)


def _dims(seq):
    a = dims_t()
    for i, v in enumerate(seq):
        a[i] = v
    return a


class engine:
    def __init__(self, kind=gpu, index=0):
        self.h = C.c_void_p()
        _check(lib().dnnl_engine_create(C.byref(self.h), kind, C.c_size_t(index)), "engine_create")

    def get_kind(self):
        k = C.c_int()
        _check(lib().dnnl_engine_get_kind(self.h, C.byref(k)), "engine_get_kind")
        return k.value


class stream:
    """hip_stream: a hipStream_t of the caller's (an integer; 0 = the default stream) to run on instead of a stream
    of the library's own -- dnnl_amd_interop_stream_create."""

    def __init__(self, eng, flags=1, hip_stream=None):
        self.engine = eng
        self.h = C.c_void_p()
        if hip_stream is None:
            _check(lib().dnnl_stream_create(C.byref(self.h), eng.h, C.c_uint(flags)), "stream_create")
        else:
            _check(lib().dnnl_amd_interop_stream_create(C.byref(self.h), eng.h, C.c_void_p(hip_stream)),
                   "interop_stream_create")

    def wait(self):
        _check(lib().dnnl_stream_wait(self.h), "stream_wait")

    def hip_stream(self):
        p = C.c_void_p()
        _check(lib().dnnl_amd_interop_stream_get_hip_stream(self.h, C.byref(p)), "interop_stream_get_hip_stream")
        return p.value


class memory_desc:
    def __init__(self, dims=None, dt=None, tag=None, strides=None, handle=None):
        self.h = C.c_void_p()
        self.owned = handle is None
        if handle is not None:
            self.h = C.c_void_p(handle)
            return
        nd = len(dims)
        if strides is not None:
            st = lib().dnnl_memory_desc_create_with_strides(C.byref(self.h), nd, _dims(dims), dt, _dims(strides))
        else:
            st = lib().dnnl_memory_desc_create_with_tag(C.byref(self.h), nd, _dims(dims), dt, tag)
        _check(st, "memory_desc_create")

    def get_size(self):
        return lib().dnnl_memory_desc_get_size(self.h)

    def ndims(self):
        v = C.c_int32()
        _check(lib().dnnl_memory_desc_query(self.h, query_ndims_s32, C.byref(v)), "md_query")
        return v.value

    def _vec(self, what):
        p = C.POINTER(dims_t)()
        _check(lib().dnnl_memory_desc_query(self.h, what, C.byref(p)), "md_query")
        return list(p.contents[: self.ndims()])

    def dims(self):
        return self._vec(query_dims)

    def strides(self):
        return self._vec(query_strides)

    def data_type(self):
        v = C.c_int()
        _check(lib().dnnl_memory_desc_query(self.h, query_data_type, C.byref(v)), "md_query")
        return v.value

    def format_kind(self):
        v = C.c_int()
        _check(lib().dnnl_memory_desc_query(self.h, query_format_kind, C.byref(v)), "md_query")
        return v.value


class grouped_memory_desc(memory_desc):
    """dnnl_memory_desc_create_with_grouped_encoding: dims [total_M][K] with
    variable_dim_idx 0 (row-major) or [M][total_K] with 1 (column-major)."""

    def __init__(self, dims, dt, variable_dim_idx, group_count, offsets_dt=None):
        self.h = C.c_void_p()
        self.owned = True
        st = lib().dnnl_memory_desc_create_with_grouped_encoding(
            C.byref(self.h), len(dims), _dims(dims), dt, variable_dim_idx, C.c_int64(group_count),
            cabi.DT_S32 if offsets_dt is None else offsets_dt)
        _check(st, "memory_desc_create_with_grouped_encoding")

    def get_size(self, index=0):
        lib().dnnl_memory_desc_get_size_v2.restype = C.c_size_t
        return lib().dnnl_memory_desc_get_size_v2(self.h, index)

    def num_handles(self):
        v = C.c_int32()
        _check(lib().dnnl_memory_desc_query(self.h, 268, C.byref(v)), "md_query")
        return v.value


class grouped_memory:
    """A grouped tensor on the device: values and the groups' cumulative ends (s32)."""

    def __init__(self, md, eng, values=None, offsets=None):
        self.md, self.engine = md, eng
        self.h = C.c_void_p()
        handles = (C.c_void_p * 2)(MEMORY_ALLOCATE, MEMORY_ALLOCATE)
        _check(lib().dnnl_memory_create_v2(C.byref(self.h), md.h, eng.h, 2, handles), "memory_create_v2")
        if values is not None:
            self.write(values, 0)
        if offsets is not None:
            self.write(np.asarray(offsets, np.int32), 1)

    def write(self, data, index=0):
        data = np.ascontiguousarray(data)
        p = C.c_void_p()
        _check(lib().dnnl_memory_map_data_v2(self.h, C.byref(p), index), "memory_map_data_v2")
        assert data.nbytes <= self.md.get_size(index), (data.nbytes, self.md.get_size(index))
        if data.nbytes:
            C.memmove(p, data.ctypes.data, data.nbytes)
        _check(lib().dnnl_memory_unmap_data_v2(self.h, p, index), "memory_unmap_data_v2")

    def read(self, dtype, index=0):
        p = C.c_void_p()
        _check(lib().dnnl_memory_map_data_v2(self.h, C.byref(p), index), "memory_map_data_v2")
        n = self.md.get_size(index)
        out = np.empty(n // np.dtype(dtype).itemsize, dtype=dtype)
        if n:
            C.memmove(out.ctypes.data, p, n)
        _check(lib().dnnl_memory_unmap_data_v2(self.h, p, index), "memory_unmap_data_v2")
        return out


def zero_memory_desc():
    """A zero memory descriptor (ndims 0: "no tensor")."""
    h = C.c_void_p()
    _check(lib().dnnl_memory_desc_create_with_tag(C.byref(h), 0, _dims([]), 0, 0), "memory_desc_create (zero)")
    return memory_desc(handle=h.value)


class host_scalar:
    """dnnl::memory of a host-side scalar (dnnl_memory_create_host_scalar): the
    value lives in the object; `value` is a numpy scalar of the storage type."""

    def __init__(self, dt, value):
        self.mdh = C.c_void_p()
        _check(lib().dnnl_memory_desc_create_host_scalar(C.byref(self.mdh), dt), "memory_desc_create_host_scalar")
        self.md = memory_desc(handle=self.mdh.value)
        self.h = C.c_void_p()
        v = np.ascontiguousarray(value).reshape(1)
        _check(lib().dnnl_memory_create_host_scalar(C.byref(self.h), self.mdh, C.c_void_p(v.ctypes.data)),
               "memory_create_host_scalar")

    def set(self, value):
        v = np.ascontiguousarray(value).reshape(1)
        _check(lib().dnnl_memory_set_host_scalar_value(self.h, C.c_void_p(v.ctypes.data)), "set_host_scalar_value")

    def get(self, dtype):
        out = np.zeros(1, dtype)
        _check(lib().dnnl_memory_get_host_scalar_value(self.h, C.c_void_p(out.ctypes.data)), "get_host_scalar_value")
        return out[0]


class memory:
    """Device memory; `data` (numpy, raw storage) is uploaded through map/unmap."""

    def __init__(self, md, eng, data=None):
        self.md, self.engine = md, eng
        self.h = C.c_void_p()
        _check(lib().dnnl_memory_create(C.byref(self.h), md.h, eng.h, MEMORY_ALLOCATE), "memory_create")
        if data is not None:
            self.write(data)

    def write(self, data):
        data = np.ascontiguousarray(data)
        p = C.c_void_p()
        _check(lib().dnnl_memory_map_data(self.h, C.byref(p)), "memory_map_data")
        n = self.md.get_size()
        assert data.nbytes <= n, (data.nbytes, n)
        if data.nbytes:
            C.memmove(p, data.ctypes.data, data.nbytes)
        _check(lib().dnnl_memory_unmap_data(self.h, p), "memory_unmap_data")

    def get_data_handle(self):
        """The device pointer (dnnl_memory_get_data_handle)."""
        p = C.c_void_p()
        _check(lib().dnnl_memory_get_data_handle(self.h, C.byref(p)), "memory_get_data_handle")
        return p.value

    def read(self, dtype):
        p = C.c_void_p()
        _check(lib().dnnl_memory_map_data(self.h, C.byref(p)), "memory_map_data")
        n = self.md.get_size()
        out = np.empty(n // np.dtype(dtype).itemsize, dtype=dtype)
        if n:
            C.memmove(out.ctypes.data, p, n)
        _check(lib().dnnl_memory_unmap_data(self.h, p), "memory_unmap_data")
        return out


class post_ops:
    def __init__(self):
        self.h = C.c_void_p()
        _check(lib().dnnl_post_ops_create(C.byref(self.h)), "post_ops_create")

    def append_eltwise(self, alg, alpha=0.0, beta=0.0):
        _check(lib().dnnl_post_ops_append_eltwise(self.h, alg, C.c_float(alpha), C.c_float(beta)), "append_eltwise")

    def append_binary(self, alg, src1_md, src2_md=None):
        if src2_md is not None:
            _check(lib().dnnl_post_ops_append_binary_v2(self.h, alg, src1_md.h, src2_md.h), "append_binary_v2")
            return
        _check(lib().dnnl_post_ops_append_binary(self.h, alg, src1_md.h), "append_binary")

    def append_sum(self, scale=1.0, zero_point=0, dt=0):
        _check(lib().dnnl_post_ops_append_sum(self.h, C.c_float(scale), C.c_int32(zero_point), dt), "append_sum")

    def append_prelu(self, mask):
        _check(lib().dnnl_post_ops_append_prelu(self.h, mask), "append_prelu")

    def len(self):
        return lib().dnnl_post_ops_len(self.h)

    def kind(self, i):
        return lib().dnnl_post_ops_get_kind(self.h, i)


class primitive_attr:
    def __init__(self):
        self.h = C.c_void_p()
        _check(lib().dnnl_primitive_attr_create(C.byref(self.h)), "attr_create")

    def set_scales_mask(self, arg, mask):
        _check(lib().dnnl_primitive_attr_set_scales_mask(self.h, arg, mask), "set_scales_mask")

    def set_scales(self, arg, mask, groups=(), dt=cabi.DT_F32, qmode=None, is_on_host=0):
        if qmode is None and not is_on_host:
            _check(lib().dnnl_primitive_attr_set_scales(self.h, arg, mask, len(groups), _dims(groups), dt), "set_scales")
        else:
            _check(lib().dnnl_primitive_attr_set_scales_v3(
                self.h, arg, mask, len(groups), _dims(groups), dt, is_on_host,
                quantization_mode_static_sazp if qmode is None else qmode), "set_scales_v3")

    def set_zero_points_mask(self, arg, mask):
        _check(lib().dnnl_primitive_attr_set_zero_points_mask(self.h, arg, mask), "set_zero_points_mask")

    def set_zero_points(self, arg, mask, groups=(), dt=cabi.DT_S32, is_on_host=0):
        if is_on_host:
            _check(lib().dnnl_primitive_attr_set_zero_points_v2(
                self.h, arg, mask, len(groups), _dims(groups), dt, is_on_host), "set_zero_points_v2")
            return
        _check(lib().dnnl_primitive_attr_set_zero_points(self.h, arg, mask, len(groups), _dims(groups), dt),
               "set_zero_points")

    def set_precomputed_reductions(self, arg, mask, groups=(), dt=cabi.DT_S32):
        _check(lib().dnnl_primitive_attr_set_precomputed_reductions(self.h, arg, mask, len(groups), _dims(groups), dt),
               "set_precomputed_reductions")

    def set_fpmath_mode(self, mode, apply_to_int=False):
        _check(lib().dnnl_primitive_attr_set_fpmath_mode_v2(self.h, mode, int(apply_to_int)), "set_fpmath_mode")

    def set_post_ops(self, po):
        _check(lib().dnnl_primitive_attr_set_post_ops(self.h, po.h), "set_post_ops")

    def set_scratchpad_mode(self, mode):
        _check(lib().dnnl_primitive_attr_set_scratchpad_mode(self.h, mode), "set_scratchpad_mode")

    def set_dropout(self, mask_md=None, seed_dt=None, use_offset=False, use_host_scalars=False):
        """mask_md None: a zero descriptor (no mask is written).  seed_dt None: the first form of the call."""
        md = mask_md if mask_md is not None else zero_memory_desc()
        if seed_dt is None:
            _check(lib().dnnl_primitive_attr_set_dropout(self.h, md.h), "set_dropout")
        else:
            _check(lib().dnnl_primitive_attr_set_dropout_v2(self.h, md.h, seed_dt, int(use_offset), int(use_host_scalars)),
                   "set_dropout_v2")

    def get_dropout(self):
        """(mask data type, seed data type, use_offset, use_host_scalars)"""
        mdh, dt, off, hs = C.c_void_p(), C.c_int(), C.c_int(), C.c_int()
        _check(lib().dnnl_primitive_attr_get_dropout_v2(self.h, C.byref(mdh), C.byref(dt), C.byref(off), C.byref(hs)),
               "get_dropout_v2")
        return memory_desc(handle=mdh.value).data_type(), dt.value, off.value, hs.value

    def set_rounding(self, arg, mode):
        _check(lib().dnnl_primitive_attr_set_rounding(self.h, arg, mode), "set_rounding")

    def get_rounding(self, arg):
        v = C.c_int()
        _check(lib().dnnl_primitive_attr_get_rounding(self.h, arg, C.byref(v)), "get_rounding")
        return v.value


class matmul_primitive_desc:
    def __init__(self, eng, src_md, weights_md, dst_md, bias_md=None, attr=None):
        self.engine = eng
        self.h = C.c_void_p()
        _check(lib().dnnl_matmul_primitive_desc_create(
            C.byref(self.h), eng.h, src_md.h, weights_md.h, bias_md.h if bias_md else None, dst_md.h,
            attr.h if attr else None), "matmul_primitive_desc_create")

    def impl_info_str(self):
        s = C.c_char_p()
        _check(lib().dnnl_primitive_desc_query(self.h, query_impl_info_str, 0, C.byref(s)), "pd_query")
        return s.value.decode()

    def next_impl(self):
        st = lib().dnnl_primitive_desc_next_impl(self.h)
        if st == last_impl_reached:
            return False
        _check(st, "next_impl")
        return True

    def query_md(self, what, index=0):
        p = lib().dnnl_primitive_desc_query_md(self.h, what, index)
        return memory_desc(handle=p) if p else None

    def scratchpad_desc(self):
        return self.query_md(query_scratchpad_md)

    def lowered_desc(self):
        """The thin-C-ABI problem description the descriptor lowered to
        (dnnl_amd_primitive_desc_get_lowered, an extension of this library)."""
        d = cabi.MatmulDesc()
        _check(lib().dnnl_amd_primitive_desc_get_lowered(self.h, C.byref(d)), "get_lowered")
        return d


class inner_product_forward_primitive_desc(matmul_primitive_desc):
    """dnnl::inner_product_forward::primitive_desc(engine, prop_kind, src_md, weights_md, bias_md, dst_md, attr)"""

    def __init__(self, eng, prop_kind, src_md, weights_md, dst_md, bias_md=None, attr=None):
        self.engine = eng
        self.h = C.c_void_p()
        _check(lib().dnnl_inner_product_forward_primitive_desc_create(
            C.byref(self.h), eng.h, prop_kind, src_md.h, weights_md.h, bias_md.h if bias_md else None, dst_md.h,
            attr.h if attr else None), "inner_product_forward_primitive_desc_create")

    def query_s32(self, what):
        v = C.c_int(0)
        _check(lib().dnnl_primitive_desc_query(self.h, what, 0, C.byref(v)), "pd_query")
        return v.value


class inner_product_backward_data_primitive_desc(inner_product_forward_primitive_desc):
    """dnnl::inner_product_backward_data::primitive_desc(engine, diff_src_md, weights_md, diff_dst_md, hint_fwd_pd,
    attr)"""

    def __init__(self, eng, diff_src_md, weights_md, diff_dst_md, hint_fwd_pd=None, attr=None):
        self.engine = eng
        self.h = C.c_void_p()
        _check(lib().dnnl_inner_product_backward_data_primitive_desc_create(
            C.byref(self.h), eng.h, diff_src_md.h, weights_md.h, diff_dst_md.h,
            hint_fwd_pd.h if hint_fwd_pd else None, attr.h if attr else None),
            "inner_product_backward_data_primitive_desc_create")


class inner_product_backward_weights_primitive_desc(inner_product_forward_primitive_desc):
    """dnnl::inner_product_backward_weights::primitive_desc(engine, src_md, diff_weights_md, diff_bias_md,
    diff_dst_md, hint_fwd_pd, attr)"""

    def __init__(self, eng, src_md, diff_weights_md, diff_dst_md, diff_bias_md=None, hint_fwd_pd=None, attr=None):
        self.engine = eng
        self.h = C.c_void_p()
        _check(lib().dnnl_inner_product_backward_weights_primitive_desc_create(
            C.byref(self.h), eng.h, src_md.h, diff_weights_md.h, diff_bias_md.h if diff_bias_md else None,
            diff_dst_md.h, hint_fwd_pd.h if hint_fwd_pd else None, attr.h if attr else None),
            "inner_product_backward_weights_primitive_desc_create")


class sdpa_primitive_desc(inner_product_forward_primitive_desc):
    """sdpa_primitive_desc_create(engine, query, key, value, dst, mask, scale, invert_scale, kv_head_number,
    attn_mask_type, softmax_alg, prop, attr, kq_attr, vs_attr, stats) of the reference's internal test interface"""

    def __init__(self, eng, q_md, k_md, v_md, dst_md, mask_md=None, scale_md=None, invert_scale=False,
                 kv_head_number=0, attn_mask_type=0, softmax_alg=softmax_accurate, prop=forward_inference, attr=None,
                 kq_attr=None, vs_attr=None, stats_md=None):
        self.engine = eng
        self.h = C.c_void_p()
        h = lambda x: x.h if x is not None else None  # noqa: E731
        _check(lib().dnnl_amd_sdpa_primitive_desc_create(
            C.byref(self.h), eng.h, q_md.h, k_md.h, v_md.h, dst_md.h, h(mask_md), h(scale_md), int(invert_scale),
            C.c_int64(kv_head_number), int(attn_mask_type), int(softmax_alg), int(prop), h(attr), h(kq_attr), h(vs_attr),
            h(stats_md)), "sdpa_primitive_desc_create")


class reorder_primitive_desc(matmul_primitive_desc):
    """dnnl::reorder::primitive_desc(src_engine, src_md, dst_engine, dst_md, attr)"""

    def __init__(self, src_eng, src_md, dst_eng, dst_md, attr=None):
        self.engine = dst_eng
        self.h = C.c_void_p()
        _check(lib().dnnl_reorder_primitive_desc_create(
            C.byref(self.h), src_md.h, src_eng.h, dst_md.h, dst_eng.h, attr.h if attr else None),
            "reorder_primitive_desc_create")


class matmul:
    def __init__(self, pd):
        self.pd = pd
        self.h = C.c_void_p()
        _check(lib().dnnl_primitive_create(C.byref(self.h), pd.h), "primitive_create")

    def execute(self, strm, args):
        arr = (ExecArg * len(args))()
        for i, (k, m) in enumerate(args.items()):
            arr[i].arg = k
            arr[i].memory = m.h
        _check(lib().dnnl_primitive_execute(self.h, strm.h, len(args), arr), "primitive_execute")


class inner_product_forward(matmul):
    """dnnl::inner_product_forward(pd); execute(stream, {ARG_SRC, ARG_WEIGHTS, ARG_BIAS, ARG_DST, ...})"""


class inner_product_backward_data(matmul):
    """dnnl::inner_product_backward_data(pd); execute(stream, {ARG_DIFF_DST, ARG_WEIGHTS, ARG_DIFF_SRC})"""


class inner_product_backward_weights(matmul):
    """dnnl::inner_product_backward_weights(pd); execute(stream, {ARG_DIFF_DST, ARG_SRC, ARG_DIFF_WEIGHTS,
    ARG_DIFF_BIAS})"""


class sdpa(matmul):
    """execute(stream, {ARG_QUERIES, ARG_KEYS, ARG_VALUES, ARG_DST, ARG_ATTN_MASK, ARG_SCALE})"""


class reorder(matmul):
    """dnnl::reorder(pd); execute(stream, {ARG_FROM: src, ARG_TO: dst, ...})"""
