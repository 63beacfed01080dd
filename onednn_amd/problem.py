"""Host-side description of one matmul problem and its launch through the C ABI.

A MatmulProblem carries what a oneDNN matmul primitive descriptor plus its
execute arguments carry (src/common/matmul_pd.hpp:63-440; argument table in
doc/functional_api/primitives/matmul.md:47-59): shapes, data types, strides,
quantization attributes, post-ops and the host copies of every tensor.
`run_gpu` uploads the tensors, launches `mi355_matmul_launch` and returns the
raw dst storage.
"""
import ctypes as C
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np

from . import cabi
from . import dtypes as dtp

_STORAGE = {
    cabi.DT_F32: np.float32, cabi.DT_S32: np.int32, cabi.DT_BF16: np.uint16,
    cabi.DT_F16: np.uint16, cabi.DT_S8: np.int8, cabi.DT_U8: np.uint8,
    cabi.DT_F8_E4M3: np.uint8, cabi.DT_F8_E5M2: np.uint8, cabi.DT_E8M0: np.uint8,
    cabi.DT_S4: np.uint8, cabi.DT_U4: np.uint8, cabi.DT_F4_E2M1: np.uint8,
}


def storage_dtype(dt):
    return _STORAGE[dt]


def storage_elems(dt, n_logical):
    """Number of storage elements that hold n_logical values."""
    return (n_logical + 1) // 2 if cabi.DT_BITS[dt] == 4 else n_logical


def strides_for(tag, batch, rows, cols):
    """Element strides (batch, row, col) of a dense tensor; tag 'ab' is
    row-major, 'ba' column-major (oneDNN format tags on the last two dims)."""
    if tag == "ab":
        return (rows * cols, cols, 1)
    if tag == "ba":
        return (rows * cols, 1, rows)
    raise ValueError(tag)


def decode(dt, raw, n):
    """Raw storage -> float32 values (flattened logical-offset order)."""
    raw = np.ascontiguousarray(raw).reshape(-1)
    if dt == cabi.DT_F32:
        return raw.view(np.float32)[:n].astype(np.float32)
    if dt == cabi.DT_S32:
        return raw.view(np.int32)[:n].astype(np.float32)
    if dt == cabi.DT_BF16:
        return dtp.bf16_to_f32(raw.view(np.uint16)[:n])
    if dt == cabi.DT_F16:
        return dtp.f16_bits_to_f32(raw.view(np.uint16)[:n])
    if dt == cabi.DT_S8:
        return raw.view(np.int8)[:n].astype(np.float32)
    if dt == cabi.DT_U8:
        return raw.view(np.uint8)[:n].astype(np.float32)
    if dt == cabi.DT_F8_E4M3:
        return dtp.e4m3_to_f32(raw.view(np.uint8)[:n])
    if dt == cabi.DT_E8M0:
        return dtp.e8m0_to_f32(raw.view(np.uint8)[:n])
    if dt == cabi.DT_F4_E2M1:
        return dtp.E2M1_VALUES[dtp.unpack_nibbles(raw.view(np.uint8), n)]
    if dt == cabi.DT_U4:
        return dtp.unpack_nibbles(raw.view(np.uint8), n).astype(np.float32)
    if dt == cabi.DT_S4:
        return dtp.s4_codes_to_int(dtp.unpack_nibbles(raw.view(np.uint8), n)).astype(np.float32)
    raise ValueError(f"decode: unsupported dt {dt}")


@dataclass
class QuantParam:
    dt: int
    mask: int                      # bit0 batch, bit1 second-to-last dim, bit2 last dim
    data: np.ndarray               # raw storage, dense row-major
    groups: tuple = (1, 1)


@dataclass
class PostOp:
    kind: int
    alg: int = 0
    alpha: float = 0.0
    beta: float = 0.0
    scale: float = 1.0
    zero_point: int = 0
    dt: int = 0
    stride: tuple = (0, 0, 0)
    data: Optional[np.ndarray] = None


def pack_woq64(wei, K, N, stride_k=None, stride_n=1):
    """4-bit weights [K][N] (raw bytes, two elements per byte, low nibble first,
    element strides (stride_k, stride_n)) in the MI355_WEI_PACK_WOQ64 layout:
    memory order [n / 64][k / 8][n % 16][(n % 64) / 16][k % 2][(k % 8) / 2]."""
    assert K % 32 == 0 and N % 64 == 0
    stride_k = N if stride_k is None else stride_k
    raw = np.ascontiguousarray(wei).view(np.uint8).reshape(-1)
    nib = np.empty(raw.size * 2, np.uint8)
    nib[0::2] = raw & 15
    nib[1::2] = raw >> 4
    kn = np.lib.stride_tricks.as_strided(nib, (K, N), (stride_k, stride_n))
    # (kq, r_hi, r_lo, c, t, j) -> (c, kq, j, t, r_lo, r_hi)
    v = kn.reshape(K // 8, 4, 2, N // 64, 4, 16).transpose(3, 0, 5, 4, 2, 1).reshape(-1)
    return (v[0::2] | (v[1::2] << 4)).astype(np.uint8)


@dataclass
class MatmulProblem:
    M: int
    N: int
    K: int
    src_dt: int
    wei_dt: int
    dst_dt: int
    src: np.ndarray
    wei: np.ndarray
    batch: int = 1
    src_stride: Optional[tuple] = None
    wei_stride: Optional[tuple] = None
    dst_stride: Optional[tuple] = None
    bias_dt: int = cabi.DT_UNDEF
    bias: Optional[np.ndarray] = None
    bias_stride: tuple = (0, 0, 1)
    quant: Dict[str, QuantParam] = field(default_factory=dict)  # src_scale, wei_zp, ...
    post_ops: List[PostOp] = field(default_factory=list)
    apply_to_int: bool = False
    fpmath_mode: int = 0
    dst_scale_mode: int = cabi.DST_SCALE_DIVIDE
    impl: int = cabi.IMPL_AUTO
    wei_packing: int = cabi.WEI_PACK_NONE  # `wei` stays plain here; GpuRun uploads it packed
    dst_dynamic: int = cabi.DST_DYNAMIC_NONE  # quant["dst_scale"].data is then an output (its content is ignored)
    dst_init: Optional[np.ndarray] = None   # prior dst content (sum post-op)
    # dropout: {"p": float, "seed": int, "seed_s64": bool, "offset": int or None, "mask": bool}
    dropout: Optional[dict] = None
    dst_stochastic: bool = False            # stochastic rounding of dst
    name: str = ""

    def __post_init__(self):
        if self.src_stride is None:
            self.src_stride = strides_for("ab", self.batch, self.M, self.K)
        if self.wei_stride is None:
            self.wei_stride = strides_for("ab", self.batch, self.K, self.N)
        if self.dst_stride is None:
            self.dst_stride = strides_for("ab", self.batch, self.M, self.N)

    # number of logical dst elements the dst buffer spans
    def dst_span(self):
        if self.batch == 0 or self.M == 0 or self.N == 0:
            return 0
        return ((self.batch - 1) * self.dst_stride[0] + (self.M - 1) * self.dst_stride[1]
                + (self.N - 1) * self.dst_stride[2] + 1)

    def desc(self):
        d = cabi.MatmulDesc()
        d.batch, d.M, d.N, d.K = self.batch, self.M, self.N, self.K
        d.src_dt, d.wei_dt, d.dst_dt, d.bias_dt = self.src_dt, self.wei_dt, self.dst_dt, self.bias_dt
        for i in range(3):
            d.src_stride[i] = self.src_stride[i]
            d.wei_stride[i] = self.wei_stride[i]
            d.dst_stride[i] = self.dst_stride[i]
            d.bias_stride[i] = self.bias_stride[i]
        for name in ("src_scale", "wei_scale", "dst_scale", "src_zp", "wei_zp", "dst_zp", "src_pr"):
            q = getattr(d, name)
            if name in self.quant:
                p = self.quant[name]
                q.dt, q.mask = p.dt, p.mask
                q.group[0], q.group[1] = p.groups
            else:
                q.dt, q.mask = cabi.DT_UNDEF, 0
                q.group[0] = q.group[1] = 1
        d.fpmath_apply_to_int = int(self.apply_to_int)
        d.fpmath_mode = self.fpmath_mode
        d.dst_scale_mode = self.dst_scale_mode
        d.n_post_ops = len(self.post_ops)
        for i, po in enumerate(self.post_ops):
            o = d.post_ops[i]
            o.kind, o.alg, o.alpha, o.beta = po.kind, po.alg, po.alpha, po.beta
            o.scale, o.zero_point, o.dt = po.scale, po.zero_point, po.dt
            for j in range(3):
                o.stride[j] = po.stride[j]
        d.impl = self.impl
        d.wei_packing = self.wei_packing
        d.dst_scale_dynamic = self.dst_dynamic
        d.rnd_flags = self.rnd_flags()
        return d

    def rnd_flags(self):
        f = cabi.RND_DST_STOCHASTIC if self.dst_stochastic else 0
        if self.dropout is not None:
            f |= cabi.RND_DROPOUT
            if self.dropout.get("mask"):
                f |= cabi.RND_DROPOUT_MASK
            if self.dropout.get("seed_s64"):
                f |= cabi.RND_SEED_S64
            if self.dropout.get("offset") is not None:
                f |= cabi.RND_DROPOUT_OFFSET
        return f

    def dropout_buffers(self):
        """{args field: array} of the dropout arguments (the mask zero-filled with 0xee: every byte is written)."""
        if self.dropout is None:
            return {}
        dr = self.dropout
        seed_np = np.int64 if dr.get("seed_s64") else np.int32
        out = {"dropout_p": np.asarray([dr["p"]], np.float32), "dropout_seed": np.asarray([dr["seed"]], seed_np)}
        if dr.get("offset") is not None:
            out["dropout_offset"] = np.asarray([dr["offset"]], np.int64)
        if dr.get("mask"):
            out["dropout_mask"] = np.full(self.dst_span(), 0xee, np.uint8)
        return out

    def initial_dst(self):
        n = storage_elems(self.dst_dt, self.dst_span())
        if self.dst_init is not None:
            out = np.ascontiguousarray(self.dst_init).reshape(-1).copy()
            assert out.dtype == storage_dtype(self.dst_dt) and out.size == n
            return out
        return np.zeros(n, dtype=storage_dtype(self.dst_dt))


class GpuRun:
    """Device-resident copy of a problem: upload once, launch many times."""

    def __init__(self, prob: MatmulProblem, impl=None, stream=None):
        self.lib = cabi.load_kernels()
        self.prob = prob
        self.desc = prob.desc()
        if impl is not None:
            self.desc.impl = impl
        self.stream = stream
        self.bufs = {}
        a = cabi.MatmulArgs()
        self.bufs["src"] = cabi.DeviceBuffer.from_numpy(prob.src)
        wei = prob.wei
        if prob.wei_packing == cabi.WEI_PACK_WOQ64:
            if getattr(prob, "_packed_wei", None) is None:  # several runs may share one problem
                prob._packed_wei = pack_woq64(prob.wei, prob.K, prob.N, prob.wei_stride[1], prob.wei_stride[2])
            wei = prob._packed_wei
        self.bufs["wei"] = cabi.DeviceBuffer.from_numpy(wei)
        a.src, a.wei = self.bufs["src"].ptr, self.bufs["wei"].ptr
        if prob.bias is not None:
            self.bufs["bias"] = cabi.DeviceBuffer.from_numpy(prob.bias)
            a.bias = self.bufs["bias"].ptr
        dst0 = prob.initial_dst()
        self.dst_host_shape = dst0.shape
        self.bufs["dst"] = cabi.DeviceBuffer.from_numpy(dst0)
        a.dst = self.bufs["dst"].ptr
        for name, q in prob.quant.items():
            self.bufs[name] = cabi.DeviceBuffer.from_numpy(q.data)
            setattr(a, name, self.bufs[name].ptr)
        for i, po in enumerate(prob.post_ops):
            if po.data is not None:
                self.bufs[f"po{i}"] = cabi.DeviceBuffer.from_numpy(po.data)
                a.po_arg[i] = self.bufs[f"po{i}"].ptr
        for name, arr in prob.dropout_buffers().items():
            self.bufs[name] = cabi.DeviceBuffer.from_numpy(arr)
            setattr(a, name, self.bufs[name].ptr)
        self.args = a
        st, self.impl = cabi.query(self.desc, self.desc.impl)
        cabi.check(st)
        nbytes = cabi.scratch_bytes(self.desc)
        self.scratch = cabi.DeviceBuffer(nbytes) if nbytes else None

    def reset_dst(self):
        self.bufs["dst"].upload(self.prob.initial_dst())

    def launch(self):
        cabi.check(self.lib.mi355_matmul_launch(
            C.byref(self.desc), C.byref(self.args),
            self.scratch.ptr if self.scratch else None, self.stream))

    def sync(self):
        cabi.check(self.lib.mi355_stream_sync(self.stream))

    def result(self):
        self.sync()
        return self.bufs["dst"].to_numpy(storage_dtype(self.prob.dst_dt), self.dst_host_shape)

    def dropout_mask(self):
        """The keep flags a dropout launch wrote (u8, laid out like dst)."""
        self.sync()
        return self.bufs["dropout_mask"].to_numpy(np.uint8, (self.prob.dst_span(),))

    def dynamic_scales(self):
        """The dst scales a dynamic-quantization launch wrote (raw storage)."""
        self.sync()
        q = self.prob.quant["dst_scale"]
        return self.bufs["dst_scale"].to_numpy(q.data.dtype, q.data.shape)

    def free(self):
        for b in self.bufs.values():
            b.free()
        if self.scratch:
            self.scratch.free()


def run_gpu(prob: MatmulProblem, impl=None):
    """One launch; returns (raw dst storage, implementation name)."""
    run = GpuRun(prob, impl)
    try:
        run.launch()
        return run.result(), cabi.impl_name(run.impl)
    finally:
        run.free()
