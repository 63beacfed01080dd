"""TEST INFRASTRUCTURE: ctypes binding of the CPU oracle (oracle/liboracle.so).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import
this module; nothing under onednn_amd/ does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from onednn_amd import cabi
from onednn_amd.problem import MatmulProblem, storage_dtype

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "liboracle.so")
FLAG_WEI_BF16 = 1
FLAG_FOLD_SCALES = 2
_lib = None


def build():
    subprocess.check_call(["make", "-C", _DIR, "-s"])


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        build()
    lib = C.CDLL(LIB_PATH)
    lib.oracle_matmul.argtypes = [C.POINTER(cabi.MatmulDesc), C.POINTER(cabi.MatmulArgs),
                                  C.c_int, C.c_void_p, C.c_void_p]
    lib.oracle_int8_acc.argtypes = [C.POINTER(cabi.MatmulDesc), C.POINTER(cabi.MatmulArgs),
                                    C.c_void_p]
    lib.oracle_reorder.argtypes = [C.POINTER(cabi.ReorderDesc), C.POINTER(cabi.ReorderArgs)]
    _lib = lib
    return lib


def _ptr(a):
    return a.ctypes.data if a is not None else None


def host_args(prob: MatmulProblem, dst):
    """MatmulArgs over host arrays; returns (args, keepalive list)."""
    keep = []
    a = cabi.MatmulArgs()

    def hold(x):
        x = np.ascontiguousarray(x)
        keep.append(x)
        return x.ctypes.data

    a.src, a.wei = hold(prob.src), hold(prob.wei)
    if prob.bias is not None:
        a.bias = hold(prob.bias)
    a.dst = dst.ctypes.data
    for name, q in prob.quant.items():
        setattr(a, name, hold(q.data))
    for i, po in enumerate(prob.post_ops):
        if po.data is not None:
            a.po_arg[i] = hold(po.data)
    for name, arr in prob.dropout_buffers().items():
        setattr(a, name, hold(arr))
        if name == "dropout_mask":
            prob._oracle_mask = keep[-1]      # read back by run_oracle_dropout
    return a, keep


def run_oracle(prob: MatmulProblem, flags=0, want_ideal=False):
    """Returns raw dst storage (and, on request, the f64 pre-bias sum and the
    sum of |terms| per dst element, for forward-error bounds)."""
    lib = load()
    dst = prob.initial_dst()
    desc = prob.desc()
    args, keep = host_args(prob, dst)
    n = prob.batch * prob.M * prob.N
    ideal = np.zeros(n, dtype=np.float64) if want_ideal else None
    asum = np.zeros(n, dtype=np.float64) if want_ideal else None
    st = lib.oracle_matmul(C.byref(desc), C.byref(args), flags, _ptr(ideal), _ptr(asum))
    assert st == 0, f"oracle_matmul status {st}"
    del keep
    if want_ideal:
        return dst, ideal, asum
    return dst


def run_oracle_inner_product(prob: MatmulProblem, src, wei):
    """Inner product forward.  `src` / `wei` are numpy arrays (storage type of the
    data type) of the logical shapes [mb, ic, spatial...] / [oc, ic, spatial...]:
    views in any memory order with non-negative strides.  `prob` is the matmul
    [mb, K] x [K, oc] that carries the data types and everything after the sum
    (bias, scales, post-ops, dst); its own src / wei arrays are not read.
    Returns raw dst storage."""
    lib = load()
    lib.oracle_inner_product_fwd.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p,
                                             C.POINTER(cabi.MatmulDesc), C.POINTER(cabi.MatmulArgs)]
    assert src.ndim == wei.ndim and 2 <= src.ndim <= 5 and src.shape[1:] == wei.shape[1:]
    assert min(src.strides) >= 0 and min(wei.strides) >= 0
    dst = prob.initial_dst()
    desc = prob.desc()
    args, keep = host_args(prob, dst)
    args.src, args.wei = src.ctypes.data, wei.ctypes.data
    dims = np.array(src.shape, np.int64)
    ss = np.array([x // src.itemsize for x in src.strides], np.int64)
    ws = np.array([x // wei.itemsize for x in wei.strides], np.int64)
    st = lib.oracle_inner_product_fwd(src.ndim, dims.ctypes.data, wei.shape[0], ss.ctypes.data, ws.ctypes.data,
                                      C.byref(desc), C.byref(args))
    assert st == 0, f"oracle_inner_product_fwd status {st}"
    del keep
    return dst


def _elem_strides(a):
    assert min(a.strides) >= 0
    return np.array([x // a.itemsize for x in a.strides], np.int64)


def run_oracle_inner_product_bwd_data(diff_dst, wei, dsrc_shape, dts, dsrc_order=None):
    """diff_src of the inner product.  `diff_dst` [mb, oc] and `wei` [oc, ic, spatial...] are numpy views (storage
    types) in any memory order; dts = (diff_src, weights, diff_dst) data type names; the result is a view of the
    logical shape `dsrc_shape` whose memory order is `dsrc_order` (a permutation, outermost first; default plain)."""
    lib = load()
    lib.oracle_inner_product_bwd_data.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_void_p,
                                                  C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
    from onednn_amd.problem import storage_dtype
    nd = len(dsrc_shape)
    order = list(dsrc_order) if dsrc_order is not None else list(range(nd))
    store = np.zeros([dsrc_shape[i] for i in order], storage_dtype(cabi.DT_NAMES[dts[0]]))
    out = store.transpose(np.argsort(order))
    dims = np.array(dsrc_shape, np.int64)
    s_o, s_w, s_d = _elem_strides(out), _elem_strides(wei), _elem_strides(diff_dst)
    st = lib.oracle_inner_product_bwd_data(nd, dims.ctypes.data, wei.shape[0], cabi.DT_NAMES[dts[0]], s_o.ctypes.data,
                                           store.ctypes.data, cabi.DT_NAMES[dts[1]], s_w.ctypes.data, wei.ctypes.data,
                                           cabi.DT_NAMES[dts[2]], s_d.ctypes.data, diff_dst.ctypes.data)
    assert st == 0, f"oracle_inner_product_bwd_data status {st}"
    return out


def run_oracle_inner_product_bwd_weights(diff_dst, src, dts, with_bias, dwei_order=None):
    """(diff_weights, diff_bias or None).  `diff_dst` [mb, oc], `src` [mb, ic, spatial...]: numpy views;
    dts = (src, diff_weights, diff_bias, diff_dst) data type names."""
    lib = load()
    lib.oracle_inner_product_bwd_weights.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_void_p,
                                                     C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p,
                                                     C.c_int, C.c_void_p, C.c_void_p]
    from onednn_amd.problem import storage_dtype
    nd, oc = src.ndim, diff_dst.shape[1]
    shape = (oc,) + tuple(src.shape[1:])
    order = list(dwei_order) if dwei_order is not None else list(range(nd))
    store = np.zeros([shape[i] for i in order], storage_dtype(cabi.DT_NAMES[dts[1]]))
    out = store.transpose(np.argsort(order))
    bias = np.zeros(oc, storage_dtype(cabi.DT_NAMES[dts[2]])) if with_bias else None
    dims = np.array(src.shape, np.int64)
    s_s, s_o, s_d = _elem_strides(src), _elem_strides(out), _elem_strides(diff_dst)
    st = lib.oracle_inner_product_bwd_weights(nd, dims.ctypes.data, oc, cabi.DT_NAMES[dts[0]], s_s.ctypes.data,
                                              src.ctypes.data, cabi.DT_NAMES[dts[1]], s_o.ctypes.data, store.ctypes.data,
                                              cabi.DT_NAMES[dts[2]] if with_bias else 0,
                                              bias.ctypes.data if with_bias else None, cabi.DT_NAMES[dts[3]],
                                              s_d.ctypes.data, diff_dst.ctypes.data)
    assert st == 0, f"oracle_inner_product_bwd_weights status {st}"
    return out, bias


def run_oracle_sdpa(q, k, v, dts, scale=None, invert_scale=False, mask=None, mask_type=0, dst_order=None):
    """Scaled dot-product attention.  q [b1][b0][sq][d], k [.][.][d][sk], v [.][.][sk][dv]: numpy views (storage type
    of dts[0]) in any memory order, the first two dims of k / v 1 or full; dts = (q/k/v, dst, scale, mask) data type
    names; scale: a one-element array or None; mask: a 4-D view whose dims are 1 or full (mask_type 1), or None with
    mask_type 2 / 3 for the causal masks.  Returns dst as a view of the logical shape [b1][b0][sq][dv]."""
    lib = load()
    i64p = C.c_void_p
    lib.oracle_sdpa.argtypes = [i64p, C.c_int, i64p, C.c_void_p, i64p, i64p, C.c_void_p, i64p, i64p, C.c_void_p, C.c_int,
                                i64p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, i64p, i64p, C.c_void_p]
    from onednn_amd.problem import storage_dtype
    b1, b0, sq, d = q.shape
    sk, dv = k.shape[3], v.shape[3]
    assert k.shape[2] == d and v.shape[2] == sk
    order = list(dst_order) if dst_order is not None else [0, 1, 2, 3]
    shape = (b1, b0, sq, dv)
    store = np.zeros([shape[i] for i in order], storage_dtype(cabi.DT_NAMES[dts[1]]))
    out = store.transpose(np.argsort(order))
    dims = np.array([b1, b0, sq, d, sk, dv], np.int64)
    kd, vd = np.array(k.shape[:2], np.int64), np.array(v.shape[:2], np.int64)
    sts = [_elem_strides(x) for x in (q, k, v, out)]
    md = np.array(mask.shape if mask is not None else (1, 1, 1, 1), np.int64)
    ms = _elem_strides(mask) if mask is not None else np.zeros(4, np.int64)
    st = lib.oracle_sdpa(dims.ctypes.data, cabi.DT_NAMES[dts[0]], sts[0].ctypes.data, q.ctypes.data, kd.ctypes.data,
                         sts[1].ctypes.data, k.ctypes.data, vd.ctypes.data, sts[2].ctypes.data, v.ctypes.data,
                         cabi.DT_NAMES[dts[1]], sts[3].ctypes.data, store.ctypes.data,
                         cabi.DT_NAMES[dts[2]] if scale is not None else 0,
                         scale.ctypes.data if scale is not None else None, int(invert_scale), int(mask_type),
                         cabi.DT_NAMES[dts[3]] if mask is not None else 0, md.ctypes.data, ms.ctypes.data,
                         mask.ctypes.data if mask is not None else None)
    assert st == 0, f"oracle_sdpa status {st}"
    return out


def run_oracle_dropout(prob: MatmulProblem):
    """(raw dst storage, the dropout mask or None)."""
    prob._oracle_mask = None
    dst = run_oracle(prob)
    return dst, prob._oracle_mask


def philox_block(ctr, key):
    """Philox4x32-10 of the oracle: (4 counter words, 2 key words) -> 4 output words."""
    lib = load()
    c, k, o = (C.c_uint32 * 4)(*ctr), (C.c_uint32 * 2)(*key), (C.c_uint32 * 4)()
    lib.oracle_philox4x32_block(c, k, o)
    return list(o)


def philox(idx, seed, offset):
    lib = load()
    lib.oracle_philox4x32.restype = C.c_uint32
    lib.oracle_philox4x32.argtypes = [C.c_uint64] * 3
    return lib.oracle_philox4x32(idx % 2 ** 64, seed % 2 ** 64, offset % 2 ** 64)


def philox_u32(idx, seed):
    lib = load()
    lib.oracle_philox4x32_u32.restype = C.c_uint32
    lib.oracle_philox4x32_u32.argtypes = [C.c_uint32] * 2
    return lib.oracle_philox4x32_u32(idx % 2 ** 32, seed % 2 ** 32)


def stochastic_round(x, idx, seed, dt):
    lib = load()
    lib.oracle_stochastic_round.restype = C.c_float
    lib.oracle_stochastic_round.argtypes = [C.c_float, C.c_uint32, C.c_uint32, C.c_int]
    return lib.oracle_stochastic_round(float(x), idx % 2 ** 32, seed % 2 ** 32, dt)


def dropout(x, idx, p, seed, offset):
    """(value, keep flag) of oracle_dropout."""
    lib = load()
    lib.oracle_dropout.restype = C.c_float
    lib.oracle_dropout.argtypes = [C.c_float, C.c_void_p, C.c_int64, C.c_float, C.c_int64, C.c_int64]
    mask = np.zeros(idx + 1, np.uint8)
    v = lib.oracle_dropout(float(x), mask.ctypes.data, idx, float(p), seed, offset)
    return v, int(mask[idx])


def run_oracle_dynamic(prob: MatmulProblem, flags=0):
    """Dynamic dst quantization: returns (raw dst storage, raw dst scales)."""
    lib = load()
    dst = prob.initial_dst()
    desc = prob.desc()
    saved = prob.quant["dst_scale"].data
    scales = np.zeros_like(np.ascontiguousarray(saved))
    prob.quant["dst_scale"].data = scales
    try:
        args, keep = host_args(prob, dst)
        st = lib.oracle_matmul(C.byref(desc), C.byref(args), flags, None, None)
    finally:
        prob.quant["dst_scale"].data = saved
    assert st == 0, f"oracle_matmul status {st}"
    del keep
    return dst, scales


def run_int8_acc(prob: MatmulProblem):
    lib = load()
    dst = prob.initial_dst()
    desc = prob.desc()
    args, keep = host_args(prob, dst)
    acc = np.zeros(prob.batch * prob.M * prob.N, dtype=np.int32)
    st = lib.oracle_int8_acc(C.byref(desc), C.byref(args), acc.ctypes.data)
    assert st == 0
    del keep
    return acc


def _cvt(fn, arr, in_dt, out_dt, n_out=None):
    lib = load()
    arr = np.ascontiguousarray(arr, dtype=in_dt)
    n = arr.size if n_out is None else n_out
    out = np.zeros(n if n_out is None else n_out, dtype=out_dt)
    getattr(lib, fn)(C.c_void_p(arr.ctypes.data), C.c_void_p(out.ctypes.data), C.c_int64(n))
    return out


def f32_to_bf16(x): return _cvt("oracle_f32_to_bf16", x, np.float32, np.uint16)
def bf16_to_f32(x): return _cvt("oracle_bf16_to_f32", x, np.uint16, np.float32)
def f32_to_f16(x): return _cvt("oracle_f32_to_f16", x, np.float32, np.uint16)
def f16_to_f32(x): return _cvt("oracle_f16_to_f32", x, np.uint16, np.float32)
def f16_to_e4m3(x): return _cvt("oracle_f16_to_e4m3", x, np.uint16, np.uint8)
def f32_to_e4m3(x): return _cvt("oracle_f32_to_e4m3", x, np.float32, np.uint8)
def e4m3_to_f32(x): return _cvt("oracle_e4m3_to_f32", x, np.uint8, np.float32)
def f16_to_e5m2(x): return _cvt("oracle_f16_to_e5m2", x, np.uint16, np.uint8)
def f32_to_e5m2(x): return _cvt("oracle_f32_to_e5m2", x, np.float32, np.uint8)
def e5m2_to_f32(x): return _cvt("oracle_e5m2_to_f32", x, np.uint8, np.float32)
def f32_to_e8m0(x): return _cvt("oracle_f32_to_e8m0", x, np.float32, np.uint8)
def e8m0_to_f32(x): return _cvt("oracle_e8m0_to_f32", x, np.uint8, np.float32)


def f32_to_e2m1_packed(x):
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros((x.size + 1) // 2, dtype=np.uint8)
    lib.oracle_f32_to_e2m1(C.c_void_p(x.ctypes.data), C.c_void_p(out.ctypes.data), C.c_int64(x.size))
    return out


def nibbles_to_f32(fn, packed, n):
    lib = load()
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    out = np.zeros(n, dtype=np.float32)
    getattr(lib, fn)(C.c_void_p(packed.ctypes.data), C.c_void_p(out.ctypes.data), C.c_int64(n))
    return out


def store_float(dt, x):
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    n_store = (x.size + 1) // 2 if cabi.DT_BITS[dt] == 4 else x.size
    out = np.zeros(n_store, dtype=storage_dtype(dt))
    lib.oracle_store_float(C.c_int(dt), C.c_void_p(x.ctypes.data), C.c_void_p(out.ctypes.data),
                           C.c_int64(x.size))
    return out


def load_float(dt, raw, n):
    lib = load()
    raw = np.ascontiguousarray(raw)
    out = np.zeros(n, dtype=np.float32)
    lib.oracle_load_float(C.c_int(dt), C.c_void_p(raw.ctypes.data), C.c_void_p(out.ctypes.data),
                          C.c_int64(n))
    return out


def eltwise(alg, x, alpha=0.0, beta=0.0):
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros_like(x)
    lib.oracle_eltwise(C.c_int(alg), C.c_float(alpha), C.c_float(beta), C.c_void_p(x.ctypes.data),
                       C.c_void_p(out.ctypes.data), C.c_int64(x.size))
    return out


def binary(alg, x, y):
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.ascontiguousarray(y, dtype=np.float32)
    out = np.zeros_like(x)
    lib.oracle_binary(C.c_int(alg), C.c_void_p(x.ctypes.data), C.c_void_p(y.ctypes.data),
                      C.c_void_p(out.ctypes.data), C.c_int64(x.size))
    return out


def reorder(prob):
    """CPU oracle result of a onednn_amd.reorder.ReorderProblem (raw dst storage)."""
    lib = load()
    d = prob.desc()
    a = cabi.ReorderArgs()
    keep = [np.ascontiguousarray(prob.src)]
    a.src = keep[0].ctypes.data
    dst = prob.new_dst()
    a.dst = dst.ctypes.data
    for name, q in prob.quant.items():
        keep.append(np.ascontiguousarray(q.data))
        setattr(a, name, keep[-1].ctypes.data)
    st = lib.oracle_reorder(C.byref(d), C.byref(a))
    assert st == 0
    return dst


def run_oracle_grouped(prob):
    """Grouped matmul (onednn_amd.grouped.GroupedProblem) on the CPU: returns
    (status, raw dst bytes); the status is the reference's verdict on the
    offsets (ref_grouped_gemm.cpp:169-212)."""
    from onednn_amd import grouped
    lib = load()
    lib.oracle_grouped_matmul.argtypes = [C.POINTER(cabi.GroupedDesc), C.POINTER(cabi.GroupedArgs)]
    lib.oracle_grouped_matmul.restype = C.c_int
    keep = []

    def place(arr):
        arr = np.ascontiguousarray(arr)
        keep.append(arr)
        return arr.ctypes.data

    d = prob.desc()
    a = grouped.fill_args(prob, place)
    dst = prob.initial_dst()
    a.dst = dst.ctypes.data
    st = lib.oracle_grouped_matmul(C.byref(d), C.byref(a))
    del keep
    return st, dst
