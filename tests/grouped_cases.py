"""Grouped (mixture-of-experts) matmul problems on data every type holds exactly,
with their expectation computed group by group in numpy float64 -- exact, so it
pins the oracle's restatement of ref_grouped_t bit for bit.  Shapes follow
tests/benchdnn/inputs/matmul/shapes_grouped and shapes_grouped_2dby2d of the
reference (balanced, unbalanced, one group, empty groups)."""
import numpy as np

from onednn_amd import cabi
from onednn_amd import dtypes as dtp
from onednn_amd.grouped import GroupedPostOp, GroupedProblem, GroupedQuant
from tests.benchdnn_matmul import encode

# --grouped=0:<G>:<sizes>  MxK:GxKxN  (shapes_grouped)
SHAPES_2DX3D = [
    ([8, 8, 8, 8], 64, 32),
    ([2] * 16, 128, 96),
    ([2, 6, 8], 32, 24),
    ([10, 20, 30, 40], 64, 32),
    ([1, 2, 4, 8, 16], 64, 32),
    ([8], 16, 12),
    ([0, 1, 2, 0, 3, 0], 32, 16),
]
# --grouped=1:<G>:<sizes>  MxK:KxN  (shapes_grouped_2dby2d)
SHAPES_2DX2D = [
    ([16, 16, 16, 16], 8, 32),
    ([3, 0, 13, 8], 5, 12),
    ([32], 4, 8),
    ([0, 0, 7], 6, 10),
]
NP_DT = {"f32": np.float32, "bf16": np.float32, "f16": np.float32}


def _vals(rng, dt, shape, full_range=False):
    lo, hi = {cabi.DT_U8: (0, 15), cabi.DT_S8: (-8, 7), cabi.DT_U4: (0, 15), cabi.DT_S4: (-8, 7)}.get(dt, (-4, 4))
    if full_range:
        lo, hi = {cabi.DT_U8: (0, 255), cabi.DT_S8: (-128, 127)}[dt]
    return rng.integers(lo, hi + 1, size=shape).astype(np.float64)


def case_2dx3d(sizes, K, N, src_dt=cabi.DT_F32, wei_dt=cabi.DT_F32, dst_dt=cabi.DT_F32, wtag="abc", bias=False,
               src_scale=None, wei_scale=None, src_zp=None, wei_zp=None, post_ops=(), seed=5, mx=False,
               full_range=False):
    """src_scale / src_zp: None, "row" or a K group size; wei_scale / wei_zp: None, "col" or a K group size.
    post_ops: names out of relu, linear, mul_group, mul_row, mul_full, mul_grouped.
    mx: e8m0 scales per 32 k on both operands (--attr-scales=src:3:e8m0:1x32+wei:7:e8m0:32x1).
    full_range: 8-bit integer operands over their whole range (the expected float64 values are then exact, the
    float32 results of kernel and oracle rounded: compare those two with each other).
    Returns (problem, expected float64 [total_M][N])."""
    rng = np.random.default_rng(seed)
    G, total = len(sizes), int(sum(sizes))
    S = _vals(rng, src_dt, (total, K), full_range)
    W = _vals(rng, wei_dt, (G, K, N), full_range)
    quant = {}
    int_src = src_dt in (cabi.DT_S8, cabi.DT_U8)
    int_wei = wei_dt in (cabi.DT_S8, cabi.DT_U8, cabi.DT_S4, cabi.DT_U4)

    def kgroups(spec):
        return 1 if spec in (None, "row", "col") else K // spec

    ss = np.ones((total, 1))
    if src_scale is not None:
        ss = rng.choice([0.25, 0.5, 1.0, 2.0], size=(total, kgroups(src_scale)))
        quant["src_scale"] = GroupedQuant(cabi.DT_F32, ss.astype(np.float32), 0 if src_scale == "row" else src_scale)
    ws = np.ones((G, 1, N))
    if wei_scale is not None:
        ws = rng.choice([0.125, 0.5, 1.0, 4.0], size=(G, kgroups(wei_scale), N))
        quant["wei_scale"] = GroupedQuant(cabi.DT_BF16, dtp.f32_to_bf16(ws.astype(np.float32)),
                                          0 if wei_scale == "col" else wei_scale)
    if mx:
        ss = rng.choice([0.25, 0.5, 1.0, 2.0], size=(total, K // 32))
        ws = rng.choice([0.125, 0.5, 1.0, 4.0], size=(G, K // 32, N))
        quant["src_scale"] = GroupedQuant(cabi.DT_E8M0, encode(cabi.DT_E8M0, ss), 32)
        quant["wei_scale"] = GroupedQuant(cabi.DT_E8M0, encode(cabi.DT_E8M0, ws), 32)
    zs = np.zeros((total, 1))
    if src_zp is not None:
        zs = rng.integers(-3, 4, size=(total, kgroups(src_zp))).astype(np.float64)
        quant["src_zp"] = GroupedQuant(cabi.DT_S32, zs.astype(np.int32), 0 if src_zp == "row" else src_zp)
    zw = np.zeros((G, 1, N))
    if wei_zp is not None:
        zw = rng.integers(-2, 3, size=(G, kgroups(wei_zp), N)).astype(np.float64)
        quant["wei_zp"] = GroupedQuant(cabi.DT_S8, zw.astype(np.int8), 0 if wei_zp == "col" else wei_zp)

    def expand(x, axis):     # a parameter with g groups along K -> one value per k
        return np.repeat(x, K // x.shape[axis], axis=axis)

    want = np.zeros((total, N))
    start = 0
    for g, mg in enumerate(sizes):
        rows = slice(start, start + mg)
        s_eff = (S[rows] - expand(zs[rows], 1)) * expand(ss[rows], 1)                 # [mg][K]
        w_eff = (W[g] - expand(zw[g], 0)) * expand(ws[g], 0)                          # [K][N]
        want[rows] = s_eff @ w_eff
        start += mg
    b = None
    if bias:
        b = rng.integers(-8, 9, size=(G, N)).astype(np.float64)
        start = 0
        for g, mg in enumerate(sizes):
            want[start:start + mg] += b[g]
            start += mg
    pos = []
    offsets = np.cumsum(sizes).astype(np.int32)
    for name in post_ops:
        if name == "relu":
            pos.append(GroupedPostOp(cabi.PO_ELTWISE, cabi.ELTWISE["relu"]))
            want = np.maximum(want, 0)
        elif name == "linear":
            pos.append(GroupedPostOp(cabi.PO_ELTWISE, cabi.ELTWISE["linear"], alpha=0.5, beta=-1.0))
            want = 0.5 * want - 1.0
        else:
            shape = {"mul_group": (G, 1), "mul_row": (total, 1), "mul_full": (total, N), "mul_grouped": (total, N)}[name]
            y = rng.choice([0.5, 1.0, 2.0, -1.0], size=shape)
            pos.append(GroupedPostOp(cabi.PO_BINARY, cabi.BINARY["mul"], dt=cabi.DT_F32, data=y.astype(np.float32),
                                     bin_m=shape[0], bin_n=shape[1],
                                     offsets=offsets.copy() if name == "mul_grouped" else None))
            # an operand of shape [G][1] is indexed by the group -- also when total_M happens
            # to equal G (ref_grouped_gemm.cpp:421-424)
            per_group = shape == (G, 1)
            want = want * (np.repeat(y, sizes, axis=0) if per_group else y)
    wraw = W if wtag == "abc" else np.ascontiguousarray(np.swapaxes(W, 1, 2))
    p = GroupedProblem(
        pattern=cabi.GROUPED_2DX3D, sizes=list(sizes), K=K, N=N, src_dt=src_dt, wei_dt=wei_dt, dst_dt=dst_dt,
        src=encode(src_dt, S), wei=encode(wei_dt, wraw), bias_dt=cabi.DT_F32 if bias else cabi.DT_UNDEF,
        bias=b.astype(np.float32) if bias else None,
        wei_stride=(K * N, N, 1) if wtag == "abc" else (K * N, 1, K), quant=quant, post_ops=pos,
        apply_to_int=(not int_src) and int_wei, name=f"grouped {sizes} K={K} N={N}")
    return p, want


def case_2dx2d(sizes, M, N, dt=cabi.DT_F32, dtag="abc", seed=6):
    """src [M][total_K] column-major, weights [total_K][N]; dst [G][M][N]."""
    rng = np.random.default_rng(seed)
    G, total = len(sizes), int(sum(sizes))
    S = _vals(rng, dt, (M, total))
    W = _vals(rng, dt, (total, N))
    want = np.zeros((G, M, N))
    k0 = 0
    for g, kg in enumerate(sizes):
        want[g] = S[:, k0:k0 + kg] @ W[k0:k0 + kg]
        k0 += kg
    p = GroupedProblem(
        pattern=cabi.GROUPED_2DX2D, sizes=list(sizes), M=M, N=N, src_dt=dt, wei_dt=dt, dst_dt=dt,
        src=encode(dt, np.ascontiguousarray(S.T)), wei=encode(dt, W),
        dst_stride=(M * N, N, 1) if dtag == "abc" else (M * N, 1, M), name=f"grouped-k {sizes} M={M} N={N}")
    return p, want


def logical_dst(p, raw):
    """dst bytes -> float64 values in logical order ([total_M][N] or [G][M][N])."""
    from onednn_amd.problem import decode
    flat = decode(p.dst_dt, raw, p.dst_elems()).astype(np.float64)
    if p.pattern == cabi.GROUPED_2DX3D:
        return flat.reshape(p.total, p.N)
    g, m, n = np.meshgrid(np.arange(p.G), np.arange(p.M), np.arange(p.N), indexing="ij")
    return flat[g * p.dst_stride[0] + m * p.dst_stride[1] + n * p.dst_stride[2]]
