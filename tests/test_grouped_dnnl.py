"""Grouped (mixture-of-experts) matmul through the dnnl_* API: the descriptor
rules of src/common/matmul.cpp:43-259 and ref_grouped_gemm.hpp:60-270 as status
codes (CPU), and executions against the oracle (GPU)."""
import os

import numpy as np
import pytest

os.environ["ONEDNN_AMD_ALLOW_NO_DEVICE"] = "1"   # descriptor-only engine for the status-code tests

from onednn_amd import cabi, dnnl  # noqa: E402
from tests import grouped_cases as gc  # noqa: E402

F32, BF16, F16, S8, U8, U4, S32 = (cabi.DT_F32, cabi.DT_BF16, cabi.DT_F16, cabi.DT_S8, cabi.DT_U8, cabi.DT_U4,
                                   cabi.DT_S32)


def mds(p):
    """(src, weights, dst, bias) memory descriptors of a GroupedProblem."""
    if p.pattern == cabi.GROUPED_2DX3D:
        src = dnnl.grouped_memory_desc([p.total, p.K], p.src_dt, 0, p.G)
        wei = dnnl.memory_desc([p.G, p.K, p.N], p.wei_dt, strides=list(p.wei_stride))
        dst = dnnl.grouped_memory_desc([p.total, p.N], p.dst_dt, 0, p.G)
        bias = dnnl.memory_desc([p.G, p.N], p.bias_dt, tag=dnnl.tag_ab) if p.bias is not None else None
    else:
        src = dnnl.grouped_memory_desc([p.M, p.total], p.src_dt, 1, p.G)
        wei = dnnl.grouped_memory_desc([p.total, p.N], p.wei_dt, 0, p.G)
        dst = dnnl.memory_desc([p.G, p.M, p.N], p.dst_dt, strides=list(p.dst_stride))
        bias = None
    return src, wei, dst, bias


def attr_of(p):
    """primitive_attr of a GroupedProblem; returns (attr, {execute arg id: (md, data, offsets)})."""
    a = dnnl.primitive_attr()
    extra = {}
    K, N, G, total = p.K, p.N, p.G, p.total
    for name, q in p.quant.items():
        which, kind = name.split("_")
        arg = dnnl.ARG_SRC if which == "src" else dnnl.ARG_WEIGHTS
        if which == "src":
            mask, groups = (3, (1, q.group_k)) if q.group_k else (1, ())
            dims = [total, K // q.group_k] if q.group_k else [total, 1]
        else:
            mask, groups = (7, (q.group_k, 1)) if q.group_k else (5, ())
            dims = [G, K // q.group_k, N] if q.group_k else [G, 1, N]
        if kind == "scale":
            a.set_scales(arg, mask, groups, q.dt)
            flag = dnnl.ARG_ATTR_SCALES
        else:
            a.set_zero_points(arg, mask, groups, q.dt)
            flag = dnnl.ARG_ATTR_ZERO_POINTS
        tag = dnnl.tag_ab if len(dims) == 2 else dnnl.tag_abc
        extra[flag | arg] = (dnnl.memory_desc(dims, q.dt, tag=tag), q.data, None)
    if p.apply_to_int:
        a.set_fpmath_mode(dnnl.fpmath_bf16 if p.src_dt == BF16 else dnnl.fpmath_f16, True)
    if p.post_ops:
        po = dnnl.post_ops()
        for i, op in enumerate(p.post_ops):
            if op.kind == cabi.PO_ELTWISE:
                po.append_eltwise(op.alg, op.alpha, op.beta)
            else:
                if op.offsets is not None:
                    bmd = dnnl.grouped_memory_desc([op.bin_m, op.bin_n], op.dt, 0, G)
                else:
                    bmd = dnnl.memory_desc([op.bin_m, op.bin_n], op.dt, tag=dnnl.tag_ab)
                po.append_binary(op.alg, bmd)
                extra[dnnl.ARG_ATTR_MULTIPLE_POST_OP(i) | dnnl.ARG_SRC_1] = (bmd, op.data, op.offsets)
        a.set_post_ops(po)
    return a, extra


def status_of(fn):
    try:
        fn()
    except dnnl.error as e:
        return e.status
    return dnnl.success


def test_grouped_memory_descriptor_rules():
    """memory_desc_init_with_grouped_encoding, src/common/memory_desc.cpp:417-472"""
    md = dnnl.grouped_memory_desc([9, 256], F32, 0, 3)
    assert md.get_size(0) == 9 * 256 * 4 and md.get_size(1) == 3 * 4 and md.num_handles() == 2
    assert md.format_kind() == 4                                   # dnnl_format_kind_sparse
    assert dnnl.grouped_memory_desc([16, 9], BF16, 1, 3).get_size(0) == 16 * 9 * 2
    assert status_of(lambda: dnnl.grouped_memory_desc([2, 9, 256], F32, 0, 3)) == dnnl.unimplemented   # 2-D only
    assert status_of(lambda: dnnl.grouped_memory_desc([9, 256], F32, 0, 0)) == dnnl.invalid_arguments  # no groups
    assert status_of(lambda: dnnl.grouped_memory_desc([9, 256], F32, 2, 3)) == dnnl.invalid_arguments  # dim index
    assert status_of(lambda: dnnl.grouped_memory_desc([9, 256], F32, 0, 3, offsets_dt=cabi.DT_S8)) == dnnl.invalid_arguments
    assert status_of(lambda: dnnl.grouped_memory_desc([9, 0], F32, 0, 3)) == dnnl.invalid_arguments
    assert status_of(lambda: dnnl.grouped_memory_desc([dnnl.RUNTIME_DIM_VAL, 8], F32, 0, 3)) == dnnl.invalid_arguments


def test_grouped_matmul_descriptor_rules():
    """grouped_matmul_desc_init / grouped_matmul_attr_check (matmul.cpp:52-259)"""
    eng = dnnl.engine(dnnl.gpu, 0)
    G, total, K, N = 3, 9, 32, 16
    src = dnnl.grouped_memory_desc([total, K], F32, 0, G)
    wei = dnnl.memory_desc([G, K, N], F32, tag=dnnl.tag_abc)
    dst = dnnl.grouped_memory_desc([total, N], F32, 0, G)
    pd = dnnl.matmul_primitive_desc(eng, src, wei, dst)
    assert pd.impl_info_str() == "hip:ref_grouped:any"
    assert dnnl.matmul_primitive_desc(eng, src, dnnl.memory_desc([G, K, N], F32, tag=dnnl.tag_acb), dst)

    def make(s=src, w=wei, d=dst, b=None, a=None):
        return status_of(lambda: dnnl.matmul_primitive_desc(eng, s, w, d, bias_md=b, attr=a))

    U = dnnl.unimplemented
    assert make(s=dnnl.memory_desc([total, K], F32, tag=dnnl.tag_ab)) == U             # src must be grouped
    assert make(d=dnnl.memory_desc([total, N], F32, tag=dnnl.tag_ab)) == U             # neither pattern
    assert make(s=dnnl.grouped_memory_desc([total, K], F32, 1, G)) == U                # variable dim of src
    assert make(d=dnnl.grouped_memory_desc([total, N], F32, 0, G + 1)) == U            # group counts differ
    assert make(w=dnnl.memory_desc([G + 1, K, N], F32, tag=dnnl.tag_abc)) == U         # weights' first dim
    assert make(w=dnnl.memory_desc([G, K + 1, N], F32, tag=dnnl.tag_abc)) == U         # K differs
    assert make(d=dnnl.grouped_memory_desc([total, N + 1], F32, 0, G)) == U            # N differs
    assert make(w=dnnl.memory_desc([G, K, N], F32, strides=[K * N * 2, N, 1])) == U    # not dense abc / acb
    assert make(b=dnnl.memory_desc([G, N], F32, tag=dnnl.tag_ab)) == dnnl.success
    assert make(b=dnnl.memory_desc([1, N], F32, tag=dnnl.tag_ab)) == U                 # bias is [G][N]
    assert make(d=dnnl.grouped_memory_desc([total, N], S8, 0, G)) == U                 # dst f32 / bf16 / f16
    # attributes: scales only on low-precision operands, none on dst
    a = dnnl.primitive_attr(); a.set_scales(dnnl.ARG_SRC, 1, (), F32)
    assert make(a=a) == U
    a = dnnl.primitive_attr(); a.set_scales(dnnl.ARG_DST, 0, (), F32)
    assert make(a=a) == U
    s8 = dnnl.grouped_memory_desc([total, K], U8, 0, G)
    w8 = dnnl.memory_desc([G, K, N], S8, tag=dnnl.tag_abc)
    a = dnnl.primitive_attr(); a.set_scales(dnnl.ARG_SRC, 1, (), F32); a.set_scales(dnnl.ARG_WEIGHTS, 5, (), F32)
    assert make(s=s8, w=w8, a=a) == dnnl.success
    a = dnnl.primitive_attr(); a.set_scales(dnnl.ARG_WEIGHTS, 4, (), F32)              # per column only: needs the group dim
    assert make(s=s8, w=w8, a=a) == U
    a = dnnl.primitive_attr(); a.set_scales(dnnl.ARG_WEIGHTS, 7, (16, 1), BF16); a.set_zero_points(dnnl.ARG_WEIGHTS, 7, (8, 1), S8)
    assert make(s=s8, w=w8, a=a) == U                                                  # scale and zero-point groups differ
    a = dnnl.primitive_attr(); a.set_scales(dnnl.ARG_WEIGHTS, 7, (12, 1), BF16)
    assert make(s=s8, w=w8, a=a) == U                                                  # K % group
    # post-ops: eltwise and multiplication only
    po = dnnl.post_ops(); po.append_binary(cabi.BINARY["add"], dnnl.memory_desc([total, N], F32, tag=dnnl.tag_ab))
    a = dnnl.primitive_attr(); a.set_post_ops(po)
    assert make(a=a) == U
    po = dnnl.post_ops(); po.append_binary(cabi.BINARY["mul"], dnnl.memory_desc([G, N], F32, tag=dnnl.tag_ab))
    a = dnnl.primitive_attr(); a.set_post_ops(po)
    assert make(a=a) == U                                                              # per group means [G][1]
    po = dnnl.post_ops(); po.append_binary(cabi.BINARY["mul"], dnnl.memory_desc([G, 1], F32, tag=dnnl.tag_ab))
    a = dnnl.primitive_attr(); a.set_post_ops(po)
    assert make(a=a) == dnnl.success
    po = dnnl.post_ops(); po.append_binary(cabi.BINARY["mul"], dnnl.memory_desc([total], F32, tag=dnnl.tag_a))
    a = dnnl.primitive_attr(); a.set_post_ops(po)
    assert make(a=a) == dnnl.invalid_arguments                                         # operand ndims != dst ndims
    # variable K: default attributes, no bias, one floating-point type
    s2 = dnnl.grouped_memory_desc([8, 40], F32, 1, G)
    w2 = dnnl.grouped_memory_desc([40, N], F32, 0, G)
    d2 = dnnl.memory_desc([G, 8, N], F32, tag=dnnl.tag_abc)
    assert make(s=s2, w=w2, d=d2) == dnnl.success
    assert make(s=s2, w=w2, d=dnnl.memory_desc([G, 8, N], F32, tag=dnnl.tag_any)) == dnnl.success
    assert make(s=s2, w=w2, d=d2, b=dnnl.memory_desc([G, N], F32, tag=dnnl.tag_ab)) == U
    po = dnnl.post_ops(); po.append_eltwise(cabi.ELTWISE["relu"], 0.0, 0.0)
    a = dnnl.primitive_attr(); a.set_post_ops(po)
    assert make(s=s2, w=w2, d=d2, a=a) == U
    assert make(s=s2, w=dnnl.grouped_memory_desc([40, N], BF16, 0, G), d=d2) == U


VARIANTS = [
    {},
    dict(wtag="acb", bias=True),
    dict(src_dt=U8, wei_dt=S8, src_scale="row", wei_scale="col", src_zp="row", wei_zp="col"),
    dict(src_dt=S8, wei_dt=S8, src_scale=8, wei_scale=16, src_zp=16, wei_zp=16),
    dict(src_dt=F16, wei_dt=U4, wei_scale=16, wei_zp=16, dst_dt=F16),
    dict(post_ops=("linear", "mul_grouped"), bias=True),
    dict(post_ops=("relu", "mul_group", "mul_row")),
]


@pytest.mark.gpu
@pytest.mark.parametrize("kw", VARIANTS, ids=lambda kw: ",".join(f"{k}={v}" for k, v in kw.items()) or "plain")
@pytest.mark.parametrize("sizes", [[2, 6, 8], [0, 1, 2, 0, 3, 0]], ids=lambda s: "+".join(map(str, s)))
def test_execute_2dx3d(gpu, oracle, sizes, kw):
    p, _ = gc.case_2dx3d(sizes, 32, 16, **kw)
    st, want = oracle.run_oracle_grouped(p)
    assert st == cabi.SUCCESS
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    smd, wmd, dmd, bmd = mds(p)
    attr, extra = attr_of(p)
    pd = dnnl.matmul_primitive_desc(eng, smd, wmd, dmd, bias_md=bmd, attr=attr)
    assert pd.impl_info_str() == "hip:ref_grouped:any"
    prim = dnnl.matmul(pd)
    dst = dnnl.grouped_memory(dmd, eng, p.initial_dst(), p.other_offsets)
    args = {dnnl.ARG_SRC: dnnl.grouped_memory(smd, eng, p.src, p.src_offsets),
            dnnl.ARG_WEIGHTS: dnnl.memory(wmd, eng, p.wei), dnnl.ARG_DST: dst}
    if p.bias is not None:
        args[dnnl.ARG_BIAS] = dnnl.memory(bmd, eng, p.bias)
    for arg, (md, data, offsets) in extra.items():
        args[arg] = dnnl.grouped_memory(md, eng, data, offsets) if offsets is not None else dnnl.memory(md, eng, data)
    prim.execute(strm, args)
    strm.wait()
    assert np.array_equal(dst.read(np.uint8), want)


@pytest.mark.gpu
@pytest.mark.parametrize("dtag", ["abc", "acb"])
def test_execute_2dx2d(gpu, oracle, dtag):
    p, _ = gc.case_2dx2d([3, 0, 13, 8], 5, 12, dt=BF16, dtag=dtag)
    st, want = oracle.run_oracle_grouped(p)
    assert st == cabi.SUCCESS
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    smd, wmd, dmd, _ = mds(p)
    prim = dnnl.matmul(dnnl.matmul_primitive_desc(eng, smd, wmd, dmd))
    dst = dnnl.memory(dmd, eng, p.initial_dst())
    prim.execute(strm, {dnnl.ARG_SRC: dnnl.grouped_memory(smd, eng, p.src, p.src_offsets),
                        dnnl.ARG_WEIGHTS: dnnl.grouped_memory(wmd, eng, p.wei, p.other_offsets), dnnl.ARG_DST: dst})
    strm.wait()
    assert np.array_equal(dst.read(np.uint8), want)


@pytest.mark.gpu
@pytest.mark.parametrize("sdt,wdt,wtag", [(cabi.DT_F8_E4M3, cabi.DT_F8_E4M3, "acb"), (BF16, BF16, "acb"), (BF16, BF16, "abc"),
                                          (F16, F16, "abc")], ids=["e4m3", "bf16", "bf16 row-major", "f16 row-major"])
def test_execute_2dx3d_on_the_matrix_cores(gpu, oracle, sdt, wdt, wtag):
    """The layout of the reference's GPU grouped tests (--wtag=acb, --attr-scales=src:1:f32+wei:5:f32 for fp8) goes
    to hip:mfma_grouped, and so do row-major (abc) weights of the 16-bit types; exact data, so the oracle's bits are
    the expectation."""
    kw = dict(src_scale="row", wei_scale="col") if sdt == cabi.DT_F8_E4M3 else {}
    p, _ = gc.case_2dx3d([10, 20, 30, 40], 160, 36, src_dt=sdt, wei_dt=wdt, dst_dt=BF16, wtag=wtag, bias=True,
                         post_ops=("relu",), **kw)
    st, want = oracle.run_oracle_grouped(p)
    assert st == cabi.SUCCESS
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    smd, wmd, dmd, bmd = mds(p)
    attr, extra = attr_of(p)
    pd = dnnl.matmul_primitive_desc(eng, smd, wmd, dmd, bias_md=bmd, attr=attr)
    assert pd.impl_info_str() == "hip:mfma_grouped"
    prim = dnnl.matmul(pd)
    dst = dnnl.grouped_memory(dmd, eng, p.initial_dst(), p.other_offsets)
    args = {dnnl.ARG_SRC: dnnl.grouped_memory(smd, eng, p.src, p.src_offsets),
            dnnl.ARG_WEIGHTS: dnnl.memory(wmd, eng, p.wei), dnnl.ARG_DST: dst, dnnl.ARG_BIAS: dnnl.memory(bmd, eng, p.bias)}
    for arg, (md, data, offsets) in extra.items():
        args[arg] = dnnl.memory(md, eng, data)
    prim.execute(strm, args)
    strm.wait()
    assert np.array_equal(dst.read(np.uint8), want)


def test_weights_with_format_any_resolve_to_the_layout_of_the_fast_kernel():
    """Beyond the reference's ref_grouped_t (abc / acb only): `any` weights become K-contiguous (acb) for the
    operand types the matrix-core tiles take -- what format_tag::any does for the plain matmul -- and row-major
    otherwise; the caller reads the layout back and reorders once."""
    eng = dnnl.engine(dnnl.gpu, 0)
    G, total, K, N = 3, 9, 64, 16
    for dt, strides, impl in ((BF16, [K * N, 1, K], "hip:mfma_grouped"), (cabi.DT_F8_E4M3, [K * N, 1, K], "hip:mfma_grouped"),
                              (F32, [K * N, N, 1], "hip:ref_grouped:any")):
        pd = dnnl.matmul_primitive_desc(eng, dnnl.grouped_memory_desc([total, K], dt, 0, G),
                                        dnnl.memory_desc([G, K, N], dt, tag=dnnl.tag_any),
                                        dnnl.grouped_memory_desc([total, N], F32, 0, G))
        assert pd.impl_info_str() == impl
        assert pd.query_md(dnnl.query_weights_md).strides() == strides
