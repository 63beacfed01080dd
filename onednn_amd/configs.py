"""Synthetic, seeded inputs for the five benchmark configurations.

Each builder returns a MatmulProblem with the data types, layouts, attributes
and value distributions the benchmark definition states; `M/N/K` can be
overridden to get the same problem class at a test-sized shape.  Quantization
parameter layouts follow quant_entry_t::get_md
(src/common/primitive_attr_quant.hpp:116-140): dense row-major over the masked
dims with the last two divided by the group sizes.
"""
import numpy as np

from . import cabi
from . import dtypes as dtp
from .problem import MatmulProblem, PostOp, QuantParam, strides_for

MASK_COMMON = 0
MASK_ROW = 2   # second-to-last dim of the argument
MASK_COL = 4   # last dim of the argument


def _rng(seed, tensor_id):
    return np.random.Generator(np.random.PCG64([seed, tensor_id]))


def config1(M=256, N=1024, K=1024, dst="f32", seed=1, impl=cabi.IMPL_AUTO, wtag="ab"):
    """u8 x s8 -> f32 (or s32): src zero point 128, src scale 0.02, per-N
    weights scales, f32 bias.  dst='s32' drops scales and bias (accumulator
    check)."""
    src = _rng(seed, 1).integers(0, 256, size=(M, K), dtype=np.uint8)
    wei = _rng(seed, 2).integers(-127, 128, size=(K, N), dtype=np.int8)
    if wtag == "ba":
        wei = np.ascontiguousarray(wei.T)
    quant = {"src_zp": QuantParam(cabi.DT_S32, MASK_COMMON, np.array([128], np.int32))}
    bias = None
    bias_dt = cabi.DT_UNDEF
    if dst == "f32":
        quant["src_scale"] = QuantParam(cabi.DT_F32, MASK_COMMON, np.array([0.02], np.float32))
        quant["wei_scale"] = QuantParam(
            cabi.DT_F32, MASK_COL, _rng(seed, 3).uniform(1e-3, 1e-2, size=N).astype(np.float32))
        bias = _rng(seed, 4).uniform(-1, 1, size=N).astype(np.float32)
        bias_dt = cabi.DT_F32
    return MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_U8, wei_dt=cabi.DT_S8,
                         dst_dt=cabi.DT_NAMES[dst], src=src, wei=wei, bias_dt=bias_dt, bias=bias,
                         wei_stride=strides_for(wtag, 1, K, N), quant=quant, impl=impl, name=f"C1-{dst}")


def config2(M=1, N=14336, K=4096, group=128, seed=2, impl=cabi.IMPL_AUTO, wtag="ab"):
    """bf16 x u4 -> bf16 weight-only decode: per-group bf16 scales and u4 zero
    points along K, fpmath bf16 with apply_to_int."""
    src = dtp.f32_to_bf16(_rng(seed, 1).standard_normal((M, K)).astype(np.float32))
    codes = _rng(seed, 2).integers(0, 16, size=(K, N), dtype=np.uint8)
    if wtag == "ab":
        wei = dtp.pack_nibbles(codes)            # two n per byte
    else:
        wei = dtp.pack_nibbles(codes.T.copy())   # two k per byte
    G = K // group
    scales = dtp.f32_to_bf16(_rng(seed, 3).uniform(0.005, 0.02, size=(G, N)).astype(np.float32))
    zps = dtp.pack_nibbles(_rng(seed, 4).integers(0, 16, size=(G, N), dtype=np.uint8))
    quant = {
        "wei_scale": QuantParam(cabi.DT_BF16, MASK_ROW | MASK_COL, scales, (group, 1)),
        "wei_zp": QuantParam(cabi.DT_U4, MASK_ROW | MASK_COL, zps, (group, 1)),
    }
    return MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_BF16, wei_dt=cabi.DT_U4,
                         dst_dt=cabi.DT_BF16, src=src, wei=wei,
                         wei_stride=strides_for(wtag, 1, K, N), quant=quant, apply_to_int=True,
                         fpmath_mode=1, impl=impl, name=f"C2-M{M}")


def woq_variant(M, N, K, group, wei_dt="u4", sc_dt="bf16", zp_dt="u4", zp_kind="grouped", sc_kind="grouped",
                dst_dt="bf16", relu_bias=False, seed=12, wtag="ab"):
    """Weight-only int4 decode in the attribute combinations the reference admits
    (matmul_pd.hpp:131-226): s4 / u4 weights; f32 / bf16 / f16 scales, grouped
    along K or per column; s32 / s8 / u8 / s4 / u4 zero points, grouped, per
    column, one common value, or none; optional f32 bias + ReLU."""
    names = {"f32": cabi.DT_F32, "bf16": cabi.DT_BF16, "f16": cabi.DT_F16, "s32": cabi.DT_S32, "s8": cabi.DT_S8,
             "u8": cabi.DT_U8, "s4": cabi.DT_S4, "u4": cabi.DT_U4}
    src = dtp.f32_to_bf16(_rng(seed, 1).standard_normal((M, K)).astype(np.float32))
    codes = _rng(seed, 2).integers(0, 16, size=(K, N), dtype=np.uint8)  # raw nibbles, s4 reads them as signed
    wei = dtp.pack_nibbles(codes if wtag == "ab" else codes.T.copy())   # two n, or two k, per byte
    G = K // group

    def shaped(kind):
        return {"grouped": ((G, N), MASK_ROW | MASK_COL, (group, 1)), "column": ((N,), MASK_COL, (1, 1)),
                "common": ((1,), MASK_COMMON, (1, 1))}[kind]

    quant = {}
    if sc_kind != "none":
        shape, mask, grp = shaped(sc_kind)
        v = _rng(seed, 3).uniform(0.005, 0.02, size=shape).astype(np.float32)
        raw = {"f32": v, "bf16": dtp.f32_to_bf16(v), "f16": v.astype(np.float16).view(np.uint16)}[sc_dt]
        quant["wei_scale"] = QuantParam(names[sc_dt], mask, raw, grp)
    if zp_kind != "none":
        shape, mask, grp = shaped(zp_kind)
        lo, hi = {"s32": (-20, 21), "s8": (-20, 21), "u8": (0, 21), "s4": (-8, 8), "u4": (0, 16)}[zp_dt]
        z = _rng(seed, 4).integers(lo, hi, size=shape)
        raw = {"s32": z.astype(np.int32), "s8": z.astype(np.int8), "u8": z.astype(np.uint8),
               "s4": dtp.pack_nibbles((z & 0xF).astype(np.uint8)), "u4": dtp.pack_nibbles(z.astype(np.uint8))}[zp_dt]
        quant["wei_zp"] = QuantParam(names[zp_dt], mask, raw, grp)
    kw = {}
    if relu_bias:
        kw["bias_dt"] = cabi.DT_F32
        kw["bias"] = _rng(seed, 5).uniform(-1, 1, size=N).astype(np.float32)
        kw["post_ops"] = [PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"], alpha=0.0, beta=0.0, scale=1.0)]
    return MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_BF16, wei_dt=names[wei_dt], dst_dt=names[dst_dt], src=src,
                         wei=wei, wei_stride=strides_for(wtag, 1, K, N), quant=quant, apply_to_int=True,
                         fpmath_mode=1, name=f"WOQ-{wei_dt}-{sc_dt}/{sc_kind}-{zp_dt}/{zp_kind}-M{M}-{wtag}", **kw)


def config3(M=8192, N=8192, K=8192, seed=3, impl=cabi.IMPL_AUTO, wtag="ab",
            dst_scale_mode=cabi.DST_SCALE_DIVIDE):
    """s8 x s8 -> s8: src scale 0.01, per-N weights scales, dst scale 0.05,
    ReLU, round-to-nearest-even with saturation."""
    src = _rng(seed, 1).integers(-127, 128, size=(M, K), dtype=np.int8)
    wei = _rng(seed, 2).integers(-127, 128, size=(K, N), dtype=np.int8)
    if wtag == "ba":
        wei = np.ascontiguousarray(wei.T)
    quant = {
        "src_scale": QuantParam(cabi.DT_F32, MASK_COMMON, np.array([0.01], np.float32)),
        "wei_scale": QuantParam(cabi.DT_F32, MASK_COL,
                                _rng(seed, 3).uniform(1e-3, 1e-2, size=N).astype(np.float32)),
        "dst_scale": QuantParam(cabi.DT_F32, MASK_COMMON, np.array([0.05], np.float32)),
    }
    po = [PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"], alpha=0.0, beta=0.0, scale=1.0)]
    return MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_S8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_S8,
                         src=src, wei=wei, wei_stride=strides_for(wtag, 1, K, N), quant=quant,
                         post_ops=po, dst_scale_mode=dst_scale_mode, impl=impl, name="C3")


def _quant_e4m3_per_tensor(x):
    amax = np.float32(np.max(np.abs(x)))
    scale = np.float32(amax / np.float32(448.0))
    return dtp.f32_to_e4m3((x / scale).astype(np.float32)), scale


def config4(M=4096, N=28672, K=8192, seed=4, impl=cabi.IMPL_AUTO, wtag="ab"):
    """e4m3 x e4m3 -> bf16 FFN up-projection: per-tensor scales amax/448, bf16
    bias, GELU-tanh, then binary add of a bf16 residual."""
    src, s_scale = _quant_e4m3_per_tensor(_rng(seed, 1).standard_normal((M, K), dtype=np.float32))
    w = _rng(seed, 2).standard_normal((K, N), dtype=np.float32)
    wei, w_scale = _quant_e4m3_per_tensor(w)
    del w
    if wtag == "ba":
        wei = np.ascontiguousarray(wei.T)
    bias = dtp.f32_to_bf16(_rng(seed, 3).uniform(-0.1, 0.1, size=N).astype(np.float32))
    resid = dtp.f32_to_bf16(_rng(seed, 4).standard_normal((M, N), dtype=np.float32))
    quant = {
        "src_scale": QuantParam(cabi.DT_F32, MASK_COMMON, np.array([s_scale], np.float32)),
        "wei_scale": QuantParam(cabi.DT_F32, MASK_COMMON, np.array([w_scale], np.float32)),
    }
    po = [
        PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["gelu_tanh"], scale=1.0),
        PostOp(kind=cabi.PO_BINARY, alg=cabi.BINARY["add"], dt=cabi.DT_BF16,
               stride=(M * N, N, 1), data=resid),
    ]
    return MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_F8_E4M3, wei_dt=cabi.DT_F8_E4M3,
                         dst_dt=cabi.DT_BF16, src=src, wei=wei,
                         wei_stride=strides_for(wtag, 1, K, N), bias_dt=cabi.DT_BF16, bias=bias,
                         quant=quant, post_ops=po, impl=impl, name="C4")


def mx_quantize(x, axis):
    """Block-quantize to e2m1 in blocks of 32 along `axis` with e8m0 scales
    2^floor(log2(block amax / 6)); returns (codes, scale bytes)."""
    x = np.asarray(x, dtype=np.float32)
    xm = np.moveaxis(x, axis, -1)
    shp = xm.shape
    blk = xm.reshape(shp[:-1] + (shp[-1] // 32, 32))
    amax = np.max(np.abs(blk), axis=-1)
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(amax / np.float32(6.0)))
    e = np.where(amax > 0, e, -127.0)
    sb = np.clip(e + 127, 0, 254).astype(np.int32)
    scale = np.ldexp(np.float32(1.0), sb - 127).astype(np.float32)
    q = dtp.f32_to_e2m1_codes((blk / scale[..., None]).astype(np.float32))
    codes = np.moveaxis(q.reshape(shp), -1, axis)
    scales = np.moveaxis(sb.astype(np.uint8), -1, axis) if False else sb.astype(np.uint8)
    return codes, scales


def config5(M=8192, N=8192, K=8192, seed=5, impl=cabi.IMPL_AUTO, wtag="ba"):
    """MXFP4: e2m1 x e2m1 -> bf16 with e8m0 scales per block of 32 along K on
    both operands; weights K-contiguous (tag ba) by default."""
    xs = _rng(seed, 1).standard_normal((M, K), dtype=np.float32)
    s_codes, s_sb = mx_quantize(xs, axis=1)          # scales [M][K/32]
    del xs
    xw = _rng(seed, 2).standard_normal((K, N), dtype=np.float32)
    w_codes, w_sbT = mx_quantize(xw, axis=0)          # blocks along K: [N][K/32]
    del xw
    w_sb = np.ascontiguousarray(w_sbT.T)              # layout [K/32][N]
    src = dtp.pack_nibbles(s_codes)
    if wtag == "ba":
        wei = dtp.pack_nibbles(np.ascontiguousarray(w_codes.T))
    else:
        wei = dtp.pack_nibbles(w_codes)
    quant = {
        "src_scale": QuantParam(cabi.DT_E8M0, MASK_ROW | MASK_COL, s_sb, (1, 32)),
        "wei_scale": QuantParam(cabi.DT_E8M0, MASK_ROW | MASK_COL, w_sb, (32, 1)),
    }
    return MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_F4_E2M1, wei_dt=cabi.DT_F4_E2M1,
                         dst_dt=cabi.DT_BF16, src=src, wei=wei,
                         wei_stride=strides_for(wtag, 1, K, N), quant=quant, impl=impl, name="C5")


def mx_quantize_f8(x, axis):
    """Block-quantize to f8_e4m3 in blocks of 32 along `axis` the OCP-MX way (the rule of the reference's tutorial
    examples/tutorials/matmul/mxfp_matmul.cpp:155-162): scale = 2^(floor(log2 amax) - 8), 8 = the largest exponent
    of e4m3; returns (codes, scale bytes), the scale axis last."""
    x = np.asarray(x, dtype=np.float32)
    xm = np.moveaxis(x, axis, -1)
    shp = xm.shape
    blk = xm.reshape(shp[:-1] + (shp[-1] // 32, 32))
    amax = np.max(np.abs(blk), axis=-1)
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(amax)) - 8
    e = np.where(amax > 0, e, -127.0)
    sb = np.clip(e + 127, 0, 254).astype(np.int32)
    scale = np.ldexp(np.float32(1.0), sb - 127).astype(np.float32)
    q = dtp.f32_to_e4m3(np.clip(blk / scale[..., None], -448, 448).astype(np.float32).reshape(-1)).reshape(shp)
    return np.moveaxis(q, -1, axis), sb.astype(np.uint8)


def config_mxf8(M=8192, N=8192, K=8192, seed=7, impl=cabi.IMPL_AUTO, wtag="ba"):
    """MXFP8: e4m3 x e4m3 -> bf16 with e8m0 scales per block of 32 along K on both operands (the dense sibling of
    the grouped MXFP8 workload; weights K-contiguous by default)."""
    xs = _rng(seed, 1).standard_normal((M, K), dtype=np.float32)
    src, s_sb = mx_quantize_f8(xs, axis=1)            # scales [M][K/32]
    del xs
    xw = _rng(seed, 2).standard_normal((K, N), dtype=np.float32)
    w_codes, w_sbT = mx_quantize_f8(xw, axis=0)        # [K][N] codes, scales [N][K/32]
    del xw
    w_sb = np.ascontiguousarray(w_sbT.T)               # layout [K/32][N]
    wei = np.ascontiguousarray(w_codes.T) if wtag == "ba" else w_codes
    quant = {
        "src_scale": QuantParam(cabi.DT_E8M0, MASK_ROW | MASK_COL, s_sb, (1, 32)),
        "wei_scale": QuantParam(cabi.DT_E8M0, MASK_ROW | MASK_COL, w_sb, (32, 1)),
    }
    return MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_F8_E4M3, wei_dt=cabi.DT_F8_E4M3, dst_dt=cabi.DT_BF16,
                         src=src, wei=wei, wei_stride=strides_for(wtag, 1, K, N), quant=quant, impl=impl, name="M1-mxfp8")


# algorithmic work per configuration
def config_ops(p):
    return 2 * p.batch * p.M * p.N * p.K


def config2_bytes(M, N=14336, K=4096, group=128):
    G = K // group
    return K * N // 2 + G * N * 2 + G * N // 2 + M * K * 2 + M * N * 2


# ---- grouped (mixture-of-experts) matmul: shapes of the reference's
# tests/benchdnn/inputs/matmul/shapes_grouped_moe{,_large}, run there (GPU
# test_matmul_grouped_gpu) as f8_e4m3 x f8_e4m3 -> bf16 with
# --attr-scales=src:1:f32+wei:5:f32 (a scale per src row and per group and
# column) and K-contiguous weights (--wtag=acb).
GROUPED_SHAPES = {
    # DeepSeek-v3 gate/up projection, prefill: 2048x7168 : 256x7168x2048
    "g1": ("DeepSeek-v3-gate/up-proj-prefill", 7168, 2048, [
        5, 8, 3, 7, 7, 3, 2, 8, 7, 6, 7, 4, 5, 10, 8, 6, 9, 3, 7, 9, 9, 8, 10, 11, 6, 10, 13, 5, 7, 7, 8, 10, 8, 6, 8, 13,
        6, 12, 8, 7, 11, 14, 3, 9, 5, 3, 13, 11, 4, 7, 9, 10, 9, 4, 8, 10, 7, 7, 14, 7, 7, 6, 9, 7, 10, 8, 8, 9, 8, 6, 12,
        9, 5, 10, 7, 8, 9, 6, 14, 10, 10, 10, 6, 7, 8, 4, 4, 5, 5, 12, 5, 5, 8, 5, 4, 6, 5, 13, 9, 5, 3, 8, 9, 3, 9, 4, 5,
        5, 9, 8, 8, 8, 10, 9, 7, 12, 6, 7, 5, 9, 11, 9, 11, 11, 12, 9, 10, 9, 9, 6, 6, 7, 2, 8, 5, 18, 10, 4, 4, 13, 10, 8,
        12, 3, 8, 9, 11, 13, 9, 4, 7, 11, 8, 9, 12, 8, 5, 9, 12, 7, 12, 8, 5, 9, 9, 8, 7, 11, 9, 11, 10, 5, 9, 11, 9, 3, 12,
        5, 6, 8, 9, 7, 2, 7, 5, 14, 7, 6, 12, 11, 5, 9, 7, 4, 17, 10, 9, 7, 5, 5, 1, 5, 9, 10, 7, 11, 6, 8, 8, 9, 9, 8, 13,
        9, 10, 6, 12, 7, 7, 7, 11, 4, 5, 9, 8, 9, 13, 7, 9, 8, 13, 5, 17, 8, 7, 9, 10, 9, 10, 8, 13, 7, 11, 8, 7, 9, 4, 8,
        8, 5, 10, 7, 6, 7, 7, 7]),
    # Llama4-Scout gate/up projection, prefill: 512x5120 : 16x5120x8192
    "g2": ("Llama4-Scout-gate/up-proj-prefill", 5120, 8192,
           [28, 31, 37, 31, 30, 27, 34, 45, 40, 25, 33, 22, 34, 39, 34, 22]),
    # DeepSeek-v3 gate/up projection, decode: 8x7168 : 256x7168x2048 (eight groups of one row)
    "g3": ("DeepSeek-v3-gate/up-proj-decode", 7168, 2048,
           [1 if g in (12, 44, 52, 57, 71, 114, 125, 140) else 0 for g in range(256)]),
}


# g4 / g5: the shape of g1 with e8m0 scales per 32 k on both operands (--attr-scales=src:3:e8m0:1x32+wei:7:e8m0:32x1
# of the same test file): MXFP8 (e4m3) and MXFP4 (e2m1) operands
GROUPED_SHAPES["g4"] = ("DeepSeek-v3-gate/up-proj-prefill-mxfp8",) + GROUPED_SHAPES["g1"][1:]
GROUPED_SHAPES["g5"] = ("DeepSeek-v3-gate/up-proj-prefill-mxfp4",) + GROUPED_SHAPES["g1"][1:]
GROUPED_FORMAT = {"g1": "f8", "g2": "f8", "g3": "f8", "g4": "mxf8", "g5": "mxf4"}


def grouped_config(name, seed=9, groups=None, N=None):
    """One of GROUPED_SHAPES as a GroupedProblem with random operands (fp8: finite e4m3 bytes over eight binades;
    fp4: random nibbles) and a bf16 dst; scales per src row and per group and column (f32 in [0.5, 2)) or, for the
    MX formats, e8m0 scales per 32 k (2^-2 .. 2^1).  `groups` / `N`: only the first groups / columns (CPU samples)."""
    from .grouped import GroupedProblem, GroupedQuant
    label, K, n_full, sizes = GROUPED_SHAPES[name]
    fmt = GROUPED_FORMAT[name]
    sizes = list(sizes[:groups] if groups else sizes)
    N = N or n_full
    G, total = len(sizes), int(sum(sizes))
    rng = _rng(seed, 1)

    def fp8(shape):
        return (rng.integers(0, 2, shape, dtype=np.uint8) << 7) | rng.integers(0x20, 0x60, shape, dtype=np.uint8)

    if fmt == "mxf4":
        dt, kb = cabi.DT_F4_E2M1, K // 2
        src, wei = rng.integers(0, 256, (total, kb), dtype=np.uint8), rng.integers(0, 256, (G, N, kb), dtype=np.uint8)
    else:
        dt, kb = cabi.DT_F8_E4M3, K
        src, wei = fp8((total, K)), fp8((G, N, K))
    if fmt == "f8":
        quant = {"src_scale": GroupedQuant(cabi.DT_F32, rng.uniform(0.5, 2.0, total).astype(np.float32), 0),
                 "wei_scale": GroupedQuant(cabi.DT_F32, rng.uniform(0.5, 2.0, (G, N)).astype(np.float32), 0)}
    else:
        quant = {"src_scale": GroupedQuant(cabi.DT_E8M0, rng.integers(125, 129, (total, K // 32), dtype=np.uint8), 32),
                 "wei_scale": GroupedQuant(cabi.DT_E8M0, rng.integers(125, 129, (G, K // 32, N), dtype=np.uint8), 32)}
    return GroupedProblem(pattern=cabi.GROUPED_2DX3D, sizes=sizes, K=K, N=N, src_dt=dt, wei_dt=dt, dst_dt=cabi.DT_BF16,
                          src=src, wei=wei, wei_stride=(K * N, 1, K), quant=quant,
                          name=f"{name.upper()} {label} {total}x{K}:{G}x{K}x{N}")


def grouped_k_config(seed=9, groups=None, M=None, N=None):
    """g6: the weights' gradient of g2's layer -- the variable-K pattern (the reference's shapes_grouped_2dby2d hold
    test sizes only): src [M = 5120][total_K = 512 tokens] column-major, weights [512][N = 8192], both bf16 and
    grouped along K by g2's routing, dst [16][5120][8192] bf16."""
    from .grouped import GroupedProblem
    _, m_full, n_full, sizes = GROUPED_SHAPES["g2"]
    sizes = list(sizes[:groups] if groups else sizes)
    M, N = M or m_full, N or n_full
    total = int(sum(sizes))
    rng = _rng(seed, 2)
    src = dtp.f32_to_bf16(rng.standard_normal(total * M).astype(np.float32)).reshape(total, M)
    wei = dtp.f32_to_bf16(rng.standard_normal(total * N).astype(np.float32)).reshape(total, N)
    return GroupedProblem(pattern=cabi.GROUPED_2DX2D, sizes=sizes, M=M, N=N, src_dt=cabi.DT_BF16, wei_dt=cabi.DT_BF16,
                          dst_dt=cabi.DT_BF16, src=src, wei=wei, dst_stride=(M * N, N, 1),
                          name=f"G6 Llama4-Scout-gate/up-proj-weights-gradient {M}x{total}:{total}x{N} -> {len(sizes)}x{M}x{N}")


def grouped_bytes(p):
    """Algorithmic HBM bytes of a grouped launch: the weights (and their scales) of every group that has rows, src,
    dst, src scales and offsets, each once."""
    if p.pattern == cabi.GROUPED_2DX2D:
        eb = cabi.DT_BITS[p.src_dt] // 8
        return (p.total * (p.M + p.N) + p.G * p.M * p.N) * eb + 8 * p.G
    active = sum(1 for m in p.sizes if m)
    ebits = cabi.DT_BITS[p.wei_dt]
    total = active * p.K * p.N * ebits // 8 + p.total * p.K * ebits // 8 + p.total * p.N * cabi.DT_BITS[p.dst_dt] // 8
    for name, rows in (("src_scale", p.total), ("wei_scale", active * p.N)):
        q = p.quant.get(name)
        if q is not None:
            total += rows * (p.K // q.group_k if q.group_k else 1) * cabi.DT_BITS[q.dt] // 8
    return total + 8 * p.G


def config_h16(M=8192, N=8192, K=8192, dt="bf16", seed=6, impl=cabi.IMPL_AUTO, wtag="ba"):
    """bf16 x bf16 (or f16 x f16, f32 x f32) -> same type, no attributes: the unquantized
    matmul next to the quantized configurations (same tiles, 16-bit operands)."""
    sv = _rng(seed, 1).standard_normal((M, K)).astype(np.float32)
    wv = _rng(seed, 2).standard_normal((K, N)).astype(np.float32)
    if dt == "f32":
        src, wei = sv, wv
    elif dt == "bf16":
        src, wei = dtp.f32_to_bf16(sv.reshape(-1)).reshape(M, K), dtp.f32_to_bf16(wv.reshape(-1)).reshape(K, N)
    else:
        src, wei = sv.astype(np.float16).view(np.uint16), wv.astype(np.float16).view(np.uint16)
    if wtag == "ba":
        wei = np.ascontiguousarray(wei.T)
    return MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_NAMES[dt], wei_dt=cabi.DT_NAMES[dt], dst_dt=cabi.DT_NAMES[dt],
                         src=src, wei=wei, wei_stride=strides_for(wtag, 1, K, N), impl=impl,
                         name=f"{'H2' if dt == 'f32' else 'H1'}-{dt}")
