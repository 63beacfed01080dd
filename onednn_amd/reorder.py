"""Host-side description of one reorder and its launch through the C ABI.

A ReorderProblem carries what a oneDNN reorder primitive descriptor plus its
execute arguments carry (src/common/reorder.cpp:67-170, reorder_pd.hpp): the
logical dims, the data types and element strides of both tensors, the
quantization attributes (scales / zero points on DNNL_ARG_SRC and DNNL_ARG_DST,
a sum post-op as `beta`) and the host copies of the tensors.
"""
import ctypes as C
from dataclasses import dataclass, field
from typing import Dict, Optional

import numpy as np

from . import cabi
from .problem import QuantParam, storage_dtype, storage_elems


def dense_strides(dims, perm=None):
    """Element strides of a dense tensor whose dims are laid out in memory in
    the order `perm` (outermost first); default: row-major."""
    nd = len(dims)
    perm = list(range(nd)) if perm is None else list(perm)
    strides = [0] * nd
    s = 1
    for d in reversed(perm):
        strides[d] = s
        s *= max(int(dims[d]), 1)
    return tuple(strides)


def span(dims, strides):
    if any(d == 0 for d in dims):
        return 0
    return sum((d - 1) * s for d, s in zip(dims, strides)) + 1


@dataclass
class ReorderProblem:
    dims: tuple
    src_dt: int
    dst_dt: int
    src: np.ndarray                       # raw storage of the src tensor
    src_stride: Optional[tuple] = None    # default row-major
    dst_stride: Optional[tuple] = None
    quant: Dict[str, QuantParam] = field(default_factory=dict)  # src_scale, dst_scale, src_zp, dst_zp
    beta: float = 0.0
    dst_init: Optional[np.ndarray] = None  # prior dst content (sum post-op)
    name: str = ""

    def __post_init__(self):
        self.dims = tuple(int(d) for d in self.dims)
        if self.src_stride is None:
            self.src_stride = dense_strides(self.dims)
        if self.dst_stride is None:
            self.dst_stride = dense_strides(self.dims)

    def desc(self):
        d = cabi.ReorderDesc()
        d.ndims = len(self.dims)
        d.src_dt, d.dst_dt = self.src_dt, self.dst_dt
        for i, v in enumerate(self.dims):
            d.dims[i] = v
            d.src_stride[i] = self.src_stride[i]
            d.dst_stride[i] = self.dst_stride[i]
        for name in ("src_scale", "dst_scale", "src_zp", "dst_zp"):
            q = getattr(d, name)
            q.dt, q.mask = cabi.DT_UNDEF, 0
            q.group[0] = q.group[1] = 1
            if name in self.quant:
                p = self.quant[name]
                q.dt, q.mask = p.dt, p.mask
                q.group[0], q.group[1] = p.groups
        d.beta = self.beta
        return d

    def dst_storage_elems(self):
        return storage_elems(self.dst_dt, span(self.dims, self.dst_stride))

    def new_dst(self):
        n = self.dst_storage_elems()
        if self.dst_init is not None:
            out = np.ascontiguousarray(self.dst_init).reshape(-1).copy()
            assert out.size == n and out.dtype == storage_dtype(self.dst_dt)
            return out
        return np.zeros(n, dtype=storage_dtype(self.dst_dt))


def query(prob):
    d = prob.desc()
    return cabi.load_kernels().mi355_reorder_query(C.byref(d))


class GpuReorder:
    """Device copies of one problem's tensors; launch() enqueues the reorder."""

    def __init__(self, prob: ReorderProblem):
        self.prob = prob
        self.lib = cabi.load_kernels()
        self.desc = prob.desc()
        self.bufs = {"src": cabi.DeviceBuffer.from_numpy(prob.src),
                     "dst": cabi.DeviceBuffer.from_numpy(prob.new_dst())}
        self.args = cabi.ReorderArgs()
        self.args.src, self.args.dst = self.bufs["src"].ptr, self.bufs["dst"].ptr
        for name, q in prob.quant.items():
            self.bufs[name] = cabi.DeviceBuffer.from_numpy(q.data)
            setattr(self.args, name, self.bufs[name].ptr)

    def launch(self, stream=None):
        cabi.check(self.lib.mi355_reorder_launch(C.byref(self.desc), C.byref(self.args), stream))

    def sync(self):
        cabi.check(self.lib.mi355_stream_sync(None))

    def result(self):
        p = self.prob
        return self.bufs["dst"].to_numpy(storage_dtype(p.dst_dt), (p.dst_storage_elems(),))


def run_gpu(prob):
    r = GpuReorder(prob)
    r.launch()
    r.sync()
    return r.result()
