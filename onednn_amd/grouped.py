"""Grouped (mixture-of-experts) matmul through the thin C ABI: the host-side
mirror of `mi355_grouped_desc_t` / `mi355_grouped_args_t`
(include/mi355_matmul.h) -- the problem the reference describes with grouped
memory descriptors (src/common/matmul.cpp:43-259, doc/functional_api/
primitives/matmul.md "Grouped GEMM").

    2Dx3D  src [total_M][K] grouped along M, weights [G][K][N], dst [total_M][N]
    2Dx2D  src [M][total_K] column-major grouped along K, weights [total_K][N]
           grouped along K, dst [G][M][N]

`sizes` are the groups' extents along the variable dimension; offsets are their
cumulative sums (s32), as `dnnl_memory_desc_create_with_grouped_encoding`
documents them.
"""
import ctypes as C
from dataclasses import dataclass, field
from typing import Optional

import numpy as np

from . import cabi


@dataclass
class GroupedQuant:
    dt: int
    data: np.ndarray
    group_k: int = 0            # 0: no groups along K


@dataclass
class GroupedPostOp:
    kind: int                   # cabi.PO_ELTWISE or cabi.PO_BINARY (multiplication)
    alg: int
    alpha: float = 0.0
    beta: float = 0.0
    scale: float = 1.0
    dt: int = 0
    data: Optional[np.ndarray] = None      # binary operand, [bin_m][bin_n] row-major
    bin_m: int = 0
    bin_n: int = 0
    offsets: Optional[np.ndarray] = None   # a grouped operand's own offsets


@dataclass
class GroupedProblem:
    pattern: int
    sizes: list                  # extent of every group along the variable dimension
    N: int
    src_dt: int
    wei_dt: int
    dst_dt: int
    src: np.ndarray              # raw storage
    wei: np.ndarray
    M: int = 0                   # 2Dx2D
    K: int = 0                   # 2Dx3D
    bias_dt: int = cabi.DT_UNDEF
    bias: Optional[np.ndarray] = None
    wei_stride: Optional[tuple] = None   # 2Dx3D, default abc
    dst_stride: Optional[tuple] = None   # 2Dx2D, default abc
    quant: dict = field(default_factory=dict)   # src_scale / wei_scale / src_zp / wei_zp -> GroupedQuant
    post_ops: list = field(default_factory=list)
    apply_to_int: bool = False
    src_offsets: Optional[np.ndarray] = None    # default: cumulative sizes
    other_offsets: Optional[np.ndarray] = None  # dst (2Dx3D) / weights (2Dx2D); default: the same
    name: str = "grouped"

    def __post_init__(self):
        cum = np.cumsum(np.asarray(self.sizes, np.int64)).astype(np.int32)
        if self.src_offsets is None:
            self.src_offsets = cum
        if self.other_offsets is None:
            self.other_offsets = cum.copy()
        self.G = len(self.sizes)
        self.total = int(sum(self.sizes))
        if self.wei_stride is None:
            self.wei_stride = (self.K * self.N, self.N, 1)
        if self.dst_stride is None:
            self.dst_stride = (self.M * self.N, self.N, 1)

    def dst_elems(self):
        if self.pattern == cabi.GROUPED_2DX3D:
            return self.total * self.N
        return (self.G - 1) * self.dst_stride[0] + (self.M - 1) * self.dst_stride[1] + (self.N - 1) * self.dst_stride[2] + 1

    def desc(self):
        d = cabi.GroupedDesc()
        d.pattern, d.group_count, d.total = self.pattern, self.G, self.total
        d.M, d.K, d.N = self.M, self.K, self.N
        d.src_dt, d.wei_dt, d.dst_dt, d.bias_dt = self.src_dt, self.wei_dt, self.dst_dt, self.bias_dt
        for i in range(3):
            d.wei_stride[i] = self.wei_stride[i]
            d.dst_stride[i] = self.dst_stride[i]
        for name in ("src_scale", "wei_scale", "src_zp", "wei_zp"):
            q = self.quant.get(name)
            setattr(d, name + "_dt", q.dt if q else cabi.DT_UNDEF)
            setattr(d, name + "_gk", q.group_k if q else 0)
        d.fpmath_apply_to_int = int(self.apply_to_int)
        d.n_post_ops = len(self.post_ops)
        for i, po in enumerate(self.post_ops):
            e = d.post_ops[i]
            e.kind, e.alg, e.alpha, e.beta, e.scale = po.kind, po.alg, po.alpha, po.beta, po.scale
            e.dt, e.bin_m, e.bin_n, e.grouped = po.dt, po.bin_m, po.bin_n, int(po.offsets is not None)
        return d

    def buffers(self):
        """{name: array} of everything an execution reads."""
        out = {"src": self.src, "wei": self.wei, "src_offsets": self.src_offsets}
        out["dst_offsets" if self.pattern == cabi.GROUPED_2DX3D else "wei_offsets"] = self.other_offsets
        if self.bias is not None:
            out["bias"] = self.bias
        for name, q in self.quant.items():
            out[name] = q.data
        return out

    def initial_dst(self):
        nbytes = (self.dst_elems() * cabi.DT_BITS[self.dst_dt] + 7) // 8
        return np.full(nbytes, 0x5a, np.uint8)   # rows outside every group must stay as they are


def fill_args(prob, place):
    """GroupedArgs whose pointers come from place(array) -> address."""
    a = cabi.GroupedArgs()
    for name, arr in prob.buffers().items():
        setattr(a, name, place(arr))
    for i, po in enumerate(prob.post_ops):
        if po.data is not None:
            a.po_arg[i] = place(po.data)
        if po.offsets is not None:
            a.po_offsets[i] = place(np.asarray(po.offsets, np.int32))
    return a


def run_gpu(prob, stream=None):
    """Launches the problem on the current device; returns dst's raw bytes."""
    lib = cabi.load_kernels()
    d = prob.desc()
    cabi.check(lib.mi355_grouped_matmul_query(C.byref(d)))
    bufs = []

    def place(arr):
        b = cabi.DeviceBuffer.from_numpy(np.ascontiguousarray(arr))
        bufs.append(b)
        return b.ptr

    a = fill_args(prob, place)
    init = prob.initial_dst()
    dst = cabi.DeviceBuffer.from_numpy(init)
    a.dst = dst.ptr
    cabi.check(lib.mi355_grouped_matmul_launch(C.byref(d), C.byref(a), stream))
    cabi.check(lib.mi355_stream_sync(stream))
    out = dst.to_numpy(np.uint8, init.shape)
    for b in bufs + [dst]:
        b.free()
    return out
