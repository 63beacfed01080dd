"""End to end through the oneDNN-compatible C API (libdnnl_amd.so): engine,
stream, memory objects, attributes, primitive descriptor, primitive, execute
with the reference's argument ids -- results against the CPU oracle."""
import numpy as np
import pytest

from onednn_amd import cabi, configs, dnnl
from onednn_amd.problem import storage_dtype
from tests.helpers import assert_bit_exact, assert_close, assert_decode_close, assert_gemm_close

pytestmark = pytest.mark.gpu
DT = cabi.DT_NAMES


def runtime_md(dims, dt, strides, runtime):
    """The descriptor given to the primitive descriptor: with `runtime` "all"
    every dim is DNNL_RUNTIME_DIM_VAL and the layout is a tag, as in
    tests/gtests/test_matmul.cpp:128-137; with "m" only the row count of src and
    dst is (`dims[0]` is None for those)."""
    R = dnnl.RUNTIME_DIM_VAL
    tag = dnnl.tag_ab if strides[1] == 1 else dnnl.tag_ba
    if runtime == "all":
        return dnnl.memory_desc([R, R], dt, tag=tag)
    if runtime == "m" and dims[0] is None:
        assert tag == dnnl.tag_ab
        return dnnl.memory_desc([R, dims[1]], dt, tag=tag)
    return dnnl.memory_desc([d for d in dims], dt, strides=list(strides))


def run_through_api(p, scratchpad_user=False, runtime=None, reuse=None):
    """Builds the dnnl objects that describe MatmulProblem `p` (2-D, dense).
    `runtime`: see runtime_md; `reuse` = (pd, prim) of an earlier call executes
    that primitive on this problem's shapes."""
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    src_md = dnnl.memory_desc([p.M, p.K], p.src_dt, strides=list(p.src_stride[1:]))
    wei_md = dnnl.memory_desc([p.K, p.N], p.wei_dt, strides=list(p.wei_stride[1:]))
    dst_md = dnnl.memory_desc([p.M, p.N], p.dst_dt, strides=list(p.dst_stride[1:]))
    bias_md = dnnl.memory_desc([1, p.N], p.bias_dt, tag=dnnl.tag_ab) if p.bias is not None else None
    attr = dnnl.primitive_attr()
    args = {}
    name_to = {"src": dnnl.ARG_SRC, "wei": dnnl.ARG_WEIGHTS, "dst": dnnl.ARG_DST}
    for qname, q in p.quant.items():
        which, kind = qname.split("_")
        arg = name_to[which]
        mask2d = q.mask >> 1                       # (row, col) bits of the 2-D argument
        groups = q.groups if q.groups != (1, 1) else ()
        dims = {"src": (p.M, p.K), "wei": (p.K, p.N), "dst": (p.M, p.N)}[which]
        g = q.groups
        qdims = [dims[0] // g[0] if mask2d & 1 else 1, dims[1] // g[1] if mask2d & 2 else 1]
        if kind == "scale":
            attr.set_scales(arg, mask2d, groups, q.dt)
            flag = dnnl.ARG_ATTR_SCALES
        elif kind == "zp":
            attr.set_zero_points(arg, mask2d, groups, q.dt)
            flag = dnnl.ARG_ATTR_ZERO_POINTS
        else:
            attr.set_precomputed_reductions(arg, mask2d, groups, q.dt)
            flag = dnnl.ARG_ATTR_PRECOMPUTED_REDUCTIONS
        qmd = dnnl.memory_desc(qdims, q.dt, tag=dnnl.tag_ab)
        args[flag | arg] = dnnl.memory(qmd, eng, q.data)
    if p.apply_to_int:
        attr.set_fpmath_mode(dnnl.fpmath_bf16, True)
    po = dnnl.post_ops()
    for i, op in enumerate(p.post_ops):
        if op.kind == cabi.PO_ELTWISE:
            po.append_eltwise(op.alg, op.alpha, op.beta)
        elif op.kind == cabi.PO_BINARY:
            dims = [p.M if op.stride[1] else 1, p.N if op.stride[2] else 1]
            bmd = dnnl.memory_desc(dims, op.dt, tag=dnnl.tag_ab)
            po.append_binary(op.alg, bmd)
            args[dnnl.ARG_ATTR_MULTIPLE_POST_OP(i) | dnnl.ARG_SRC_1] = dnnl.memory(bmd, eng, op.data)
        elif op.kind == cabi.PO_SUM:
            po.append_sum(op.scale, op.zero_point, op.dt)
    if p.post_ops:
        attr.set_post_ops(po)
    if scratchpad_user:
        attr.set_scratchpad_mode(dnnl.scratchpad_user)
    if reuse is not None:
        pd, prim = reuse
    elif runtime:
        pd = dnnl.matmul_primitive_desc(
            eng, runtime_md([None, p.K], p.src_dt, p.src_stride[1:], runtime),
            runtime_md([p.K, p.N], p.wei_dt, p.wei_stride[1:], runtime),
            runtime_md([None, p.N], p.dst_dt, p.dst_stride[1:], runtime),
            bias_md=runtime_md([1, p.N], p.bias_dt, (p.N, 1), runtime) if bias_md else None, attr=attr)
        prim = dnnl.matmul(pd)
    else:
        pd = dnnl.matmul_primitive_desc(eng, src_md, wei_md, dst_md, bias_md=bias_md, attr=attr)
        prim = dnnl.matmul(pd)
    args[dnnl.ARG_SRC] = dnnl.memory(src_md, eng, p.src)
    args[dnnl.ARG_WEIGHTS] = dnnl.memory(wei_md, eng, p.wei)
    dst = dnnl.memory(dst_md, eng, p.initial_dst())
    args[dnnl.ARG_DST] = dst
    if p.bias is not None:
        args[dnnl.ARG_BIAS] = dnnl.memory(bias_md, eng, p.bias)
    if scratchpad_user:
        sp = pd.scratchpad_desc()
        if sp.ndims():
            args[dnnl.ARG_SCRATCHPAD] = dnnl.memory(sp, eng)
    prim.execute(strm, args)
    strm.wait()
    return dst.read(storage_dtype(p.dst_dt)), pd.impl_info_str(), (pd, prim, strm, args)


@pytest.mark.parametrize("dst", ["s32", "f32"])
def test_config1_through_the_api(gpu, oracle, dst):
    p = configs.config1(M=256, N=512, K=512, dst=dst)
    got, impl, _ = run_through_api(p)
    assert impl.startswith("hip:mfma_i8")
    assert_bit_exact(p, got, oracle.run_oracle(p), impl)


def test_config3_user_scratchpad_and_next_impl(gpu, oracle):
    p = configs.config3(M=256, N=256, K=512)
    got, impl, keep = run_through_api(p, scratchpad_user=True)
    want = oracle.run_oracle(p)
    assert_bit_exact(p, got, want, impl)
    # the second implementation of the list (generic kernel) gives the same bits
    pd, _, strm, args = keep
    assert pd.next_impl() and pd.impl_info_str() == "hip:ref:any"
    prim2 = dnnl.matmul(pd)
    args[dnnl.ARG_DST].write(p.initial_dst())
    prim2.execute(strm, args)
    strm.wait()
    assert_bit_exact(p, args[dnnl.ARG_DST].read(np.int8), want, "hip:ref:any")


def test_config2_through_the_api(gpu, oracle):
    p = configs.config2(M=8, N=512, K=1024)
    got, impl, _ = run_through_api(p)
    assert impl.startswith("hip:woq_gemv")
    want, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    assert_decode_close(p, got, ideal, asum, what=impl)


def test_config4_through_the_api(gpu, oracle):
    p = configs.config4(M=256, N=256, K=512)
    got, impl, _ = run_through_api(p)
    assert impl.startswith("hip:mfma_f8")
    want, _, asum = oracle.run_oracle(p, want_ideal=True)
    assert_close(p, got, want, abs_sum=asum, transcendental=True, what=impl)


def test_config5_through_the_api(gpu, oracle):
    p = configs.config5(M=256, N=256, K=512)
    got, impl, _ = run_through_api(p)
    assert impl.startswith("hip:mfma_mxf4")
    want, _, asum = oracle.run_oracle(p, want_ideal=True)
    assert_close(p, got, want, abs_sum=asum, what=impl)


def test_missing_argument_is_invalid_arguments(gpu):
    p = configs.config1(M=64, N=64, K=64, dst="s32")
    _, _, (pd, prim, strm, args) = run_through_api(p)
    bad = dict(args)
    del bad[dnnl.ARG_ATTR_ZERO_POINTS | dnnl.ARG_SRC]
    with pytest.raises(dnnl.error) as e:
        prim.execute(strm, bad)
    assert e.value.status == dnnl.invalid_arguments


def test_quantize_and_prepack_weights_with_reorder_then_matmul(gpu, oracle):
    """The flow of the reference's examples (examples/tutorials/matmul/
    inference_int8_matmul.cpp, matmul_with_weight_only_quantization.cpp:181-189):
    weights md with format `any`, ask the matmul pd which layout it wants,
    bring the user's f32 row-major weights there with a reorder that also
    quantizes them, then run the matmul on the reordered memory."""
    from onednn_amd.reorder import ReorderProblem
    from onednn_amd.problem import MatmulProblem, QuantParam
    from oracle import binding as orc
    M, K, N = 256, 512, 384
    r = np.random.default_rng(77)
    w_f32 = r.uniform(-1, 1, size=(K, N)).astype(np.float32)
    wsc = (np.abs(w_f32).max(axis=0) / 127).astype(np.float32)            # per-N scales
    src = r.integers(-100, 100, size=(M, K)).astype(np.int8)
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    src_md = dnnl.memory_desc([M, K], DT["s8"], tag=dnnl.tag_ab)
    wei_any = dnnl.memory_desc([K, N], DT["s8"], tag=dnnl.tag_any)
    dst_md = dnnl.memory_desc([M, N], DT["f32"], tag=dnnl.tag_ab)
    attr = dnnl.primitive_attr()
    attr.set_scales(dnnl.ARG_WEIGHTS, 2)
    pd = dnnl.matmul_primitive_desc(eng, src_md, wei_any, dst_md, attr=attr)
    wei_md = pd.query_md(dnnl.query_weights_md)
    assert wei_md.strides() == [1, K]                                    # K-contiguous for the MFMA kernels
    # reorder: f32 ab -> s8 in the queried layout, dst = src / scale[n]
    user_md = dnnl.memory_desc([K, N], DT["f32"], tag=dnnl.tag_ab)
    rattr = dnnl.primitive_attr()
    rattr.set_scales(dnnl.ARG_DST, 2)
    rpd = dnnl.reorder_primitive_desc(eng, user_md, eng, wei_md, attr=rattr)
    wsc_mem = dnnl.memory(dnnl.memory_desc([1, N], DT["f32"], tag=dnnl.tag_ab), eng, wsc)
    wei_mem = dnnl.memory(wei_md, eng)
    dnnl.reorder(rpd).execute(strm, {dnnl.ARG_FROM: dnnl.memory(user_md, eng, w_f32), dnnl.ARG_TO: wei_mem,
                                     dnnl.ARG_ATTR_SCALES | dnnl.ARG_DST: wsc_mem})
    dst = dnnl.memory(dst_md, eng)
    dnnl.matmul(pd).execute(strm, {dnnl.ARG_SRC: dnnl.memory(src_md, eng, src), dnnl.ARG_WEIGHTS: wei_mem,
                                   dnnl.ARG_DST: dst, dnnl.ARG_ATTR_SCALES | dnnl.ARG_WEIGHTS: wsc_mem})
    strm.wait()
    assert pd.impl_info_str().startswith("hip:mfma_i8")
    # oracle: the same two steps on the CPU
    rp = ReorderProblem(dims=(K, N), src_dt=cabi.DT_F32, dst_dt=cabi.DT_S8, src=w_f32, dst_stride=(1, K),
                        quant={"dst_scale": QuantParam(cabi.DT_F32, 2, wsc)})
    w_q = orc.reorder(rp)
    assert np.array_equal(wei_mem.read(np.int8), w_q)
    assert np.array_equal(w_q.reshape(N, K).T, np.rint(np.clip(w_f32 / wsc[None, :], -128, 127)).astype(np.int8))
    mp = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_S8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_F32, src=src, wei=w_q,
                       wei_stride=(K * N, 1, K), quant={"wei_scale": QuantParam(cabi.DT_F32, 4, wsc)})
    want = oracle.run_oracle(mp)
    assert_close(mp, dst.read(np.float32), want)


def test_prepack_decode_weights_with_reorder_then_matmul(gpu, oracle):
    """format `any` for 4-bit decode weights: the matmul pd answers with an
    opaque packed descriptor, a reorder brings the plain u4 weights there, the
    matmul runs on the packed memory (the flow of the reference's
    matmul_with_weight_only_quantization.cpp:181-189 with blocked weights)."""
    from onednn_amd.problem import pack_woq64
    p = configs.config2(M=8, N=8192, K=512)
    M, K, N = p.M, p.K, p.N
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    src_md = dnnl.memory_desc([M, K], DT["bf16"], tag=dnnl.tag_ab)
    dst_md = dnnl.memory_desc([M, N], DT["bf16"], tag=dnnl.tag_ab)
    attr = dnnl.primitive_attr()
    attr.set_fpmath_mode(dnnl.fpmath_bf16, True)
    attr.set_scales(dnnl.ARG_WEIGHTS, 3, (128, 1), DT["bf16"])
    attr.set_zero_points(dnnl.ARG_WEIGHTS, 3, (128, 1), DT["u4"])
    pd = dnnl.matmul_primitive_desc(eng, src_md, dnnl.memory_desc([K, N], DT["u4"], tag=dnnl.tag_any), dst_md, attr=attr)
    assert pd.impl_info_str().startswith("hip:woq_packed")
    wei_md = pd.query_md(dnnl.query_weights_md)
    assert wei_md.format_kind() == dnnl.format_kind_opaque
    user_md = dnnl.memory_desc([K, N], DT["u4"], tag=dnnl.tag_ab)
    wei_mem = dnnl.memory(wei_md, eng)
    dnnl.reorder(dnnl.reorder_primitive_desc(eng, user_md, eng, wei_md)).execute(
        strm, {dnnl.ARG_FROM: dnnl.memory(user_md, eng, p.wei), dnnl.ARG_TO: wei_mem})
    G = K // 128
    sc_mem = dnnl.memory(dnnl.memory_desc([G, N], DT["bf16"], tag=dnnl.tag_ab), eng, p.quant["wei_scale"].data)
    zp_mem = dnnl.memory(dnnl.memory_desc([G, N], DT["u4"], tag=dnnl.tag_ab), eng, p.quant["wei_zp"].data)
    dst = dnnl.memory(dst_md, eng)
    dnnl.matmul(pd).execute(strm, {dnnl.ARG_SRC: dnnl.memory(src_md, eng, p.src), dnnl.ARG_WEIGHTS: wei_mem,
                                   dnnl.ARG_DST: dst, dnnl.ARG_ATTR_SCALES | dnnl.ARG_WEIGHTS: sc_mem,
                                   dnnl.ARG_ATTR_ZERO_POINTS | dnnl.ARG_WEIGHTS: zp_mem})
    strm.wait()
    assert np.array_equal(wei_mem.read(np.uint8), pack_woq64(p.wei, K, N))
    want, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    assert_decode_close(p, dst.read(np.uint16), ideal, asum, what=pd.impl_info_str())


@pytest.mark.parametrize("flavour", ["mx", "nvfp4"])
def test_dynamic_dst_scales_through_the_api(gpu, oracle, flavour):
    """quantization_mode::dynamic_mx (e8m0 per 32, e4m3 dst) and ::dynamic_fp
    (f8_e4m3 per 16, f4_e2m1 dst: NVFP4) on DNNL_ARG_DST: the scales memory is
    an output of execute (ref_matmul.cpp:338-423)."""
    mx = flavour == "mx"
    G = 32 if mx else 16
    sdt = "e8m0" if mx else "f8_e4m3"
    ddt = "f8_e4m3" if mx else "f4_e2m1"
    from onednn_amd.problem import PostOp, QuantParam
    from oracle import binding as orc
    p = configs.config4(M=64, N=256, K=128)
    p.post_ops = [PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"], alpha=0.0, scale=1.0)]
    p.dst_dt = DT[ddt]
    p.quant["dst_scale"] = QuantParam(DT[sdt], 6, np.zeros((1, p.M, p.N // G), np.uint8), (1, G))
    p.dst_dynamic = cabi.DST_DYNAMIC_MX if mx else cabi.DST_DYNAMIC_FP
    M, K, N = p.M, p.K, p.N
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    src_md = dnnl.memory_desc([M, K], DT["f8_e4m3"], tag=dnnl.tag_ab)
    wei_md = dnnl.memory_desc([K, N], DT["f8_e4m3"], tag=dnnl.tag_ab)
    dst_md = dnnl.memory_desc([M, N], DT[ddt], tag=dnnl.tag_ab)
    assert dst_md.get_size() == (M * N if mx else M * N // 2)
    bias_md = dnnl.memory_desc([1, N], DT["bf16"], tag=dnnl.tag_ab)
    attr = dnnl.primitive_attr()
    attr.set_scales_mask(dnnl.ARG_SRC, 0)
    attr.set_scales_mask(dnnl.ARG_WEIGHTS, 0)
    attr.set_scales(dnnl.ARG_DST, 3, (1, G), DT[sdt],
                    qmode=dnnl.quantization_mode_dynamic_mx if mx else dnnl.quantization_mode_dynamic_fp)
    po = dnnl.post_ops()
    po.append_eltwise(cabi.ELTWISE["relu"], 0.0, 0.0)
    attr.set_post_ops(po)
    pd = dnnl.matmul_primitive_desc(eng, src_md, wei_md, dst_md, bias_md=bias_md, attr=attr)
    # the generic kernel is the one that matches the oracle bit for bit
    while pd.impl_info_str() != "hip:ref:any":
        assert pd.next_impl()
    one = dnnl.memory_desc([1], DT["f32"], tag=dnnl.tag_a)
    sc_md = dnnl.memory_desc([M, N // G], DT[sdt], tag=dnnl.tag_ab)
    sc_mem = dnnl.memory(sc_md, eng)
    dst = dnnl.memory(dst_md, eng)
    dnnl.matmul(pd).execute(strm, {
        dnnl.ARG_SRC: dnnl.memory(src_md, eng, p.src), dnnl.ARG_WEIGHTS: dnnl.memory(wei_md, eng, p.wei),
        dnnl.ARG_BIAS: dnnl.memory(bias_md, eng, p.bias), dnnl.ARG_DST: dst,
        dnnl.ARG_ATTR_SCALES | dnnl.ARG_SRC: dnnl.memory(one, eng, p.quant["src_scale"].data),
        dnnl.ARG_ATTR_SCALES | dnnl.ARG_WEIGHTS: dnnl.memory(one, eng, p.quant["wei_scale"].data),
        dnnl.ARG_ATTR_SCALES | dnnl.ARG_DST: sc_mem})
    strm.wait()
    want, want_sc = orc.run_oracle_dynamic(p)
    assert np.array_equal(sc_mem.read(np.uint8).reshape(-1), np.asarray(want_sc).reshape(-1))
    assert np.array_equal(dst.read(np.uint8).reshape(-1), np.asarray(want).view(np.uint8).reshape(-1))


# ---- runtime dims: one primitive, shapes known at execution only
# (tests/gtests/test_matmul.cpp:544-576,599-660; benchdnn --runtime_dims_masks)
def test_all_runtime_dims_int8_one_primitive_two_shapes(gpu, oracle):
    # the src zero point makes the integer GEMM ask for a scratch buffer (column
    # sums), which a primitive with runtime dims allocates when it executes
    p = configs.config1()
    got, name, (pd, prim, _, _) = run_through_api(p, runtime="all")
    assert name == "hip:runtime_dims:any"
    assert_bit_exact(p, got, oracle.run_oracle(p), name)
    # the same primitive on other shapes
    q = configs.config1(M=37, N=p.N * 2, K=p.K // 2)
    got, _, _ = run_through_api(q, reuse=(pd, prim))
    assert_bit_exact(q, got, oracle.run_oracle(q), name)
    # and back: the cached lowering is replaced, not mixed up
    got, _, _ = run_through_api(p, reuse=(pd, prim))
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


def test_all_runtime_dims_per_column_scales_and_post_ops(gpu, oracle):
    p = configs.config3(M=160, N=288, K=512, wtag="ba")
    got, name, (pd, prim, _, _) = run_through_api(p, runtime="all")
    assert name == "hip:runtime_dims:any"
    assert_bit_exact(p, got, oracle.run_oracle(p), name)
    q = configs.config3(M=512, N=1024, K=1024, wtag="ba")
    got, _, _ = run_through_api(q, reuse=(pd, prim))
    assert_bit_exact(q, got, oracle.run_oracle(q), name)


def test_all_runtime_dims_fp8_with_binary_post_op(gpu, oracle):
    p = configs.config4(M=96, N=256, K=512, wtag="ba")
    got, name, _ = run_through_api(p, runtime="all")
    want, _, asum = oracle.run_oracle(p, want_ideal=True)
    assert_close(p, got, want, abs_sum=asum, transcendental=True, what=name)


def test_runtime_row_count_of_the_decode_matmul(gpu, oracle):
    p = configs.config2(M=1, N=512, K=1024)
    got, name, (pd, prim, _, _) = run_through_api(p, runtime="m")
    assert name == "hip:runtime_dims:any"
    want, _, asum = oracle.run_oracle(p, want_ideal=True)
    assert_close(p, got, want, abs_sum=asum, what=name)
    for M in (8, 33):
        q = configs.config2(M=M, N=512, K=1024)
        got, _, _ = run_through_api(q, reuse=(pd, prim))
        # beyond the decode kernels' 32 rows the weights are decompressed to bf16 before the multiply (the flavour of
        # the reference's JIT path, which fpmath bf16 allows)
        want, _, asum = oracle.run_oracle(q, flags=oracle.FLAG_WEI_BF16 if M > 32 else 0, want_ideal=True)
        assert_close(q, got, want, abs_sum=asum, what=name)


def test_runtime_dims_memory_that_contradicts_the_descriptor(gpu):
    p = configs.config2(M=4, N=512, K=1024)
    _, _, (pd, prim, strm, args) = run_through_api(p, runtime="m")
    eng = dnnl.engine(dnnl.gpu, 0)
    bad = dict(args)
    # K of src differs from the K the descriptor was created with
    bad[dnnl.ARG_SRC] = dnnl.memory(dnnl.memory_desc([4, 512], p.src_dt, tag=dnnl.tag_ab), eng)
    with pytest.raises(dnnl.error) as e:
        prim.execute(strm, bad)
    assert e.value.status == dnnl.invalid_arguments
    # row counts of src and dst disagree
    bad = dict(args)
    bad[dnnl.ARG_SRC] = dnnl.memory(dnnl.memory_desc([5, 1024], p.src_dt, tag=dnnl.tag_ab), eng)
    with pytest.raises(dnnl.error) as e:
        prim.execute(strm, bad)
    assert e.value.status == dnnl.invalid_arguments
    prim.execute(strm, args)                          # the primitive stays usable
    strm.wait()


def test_runtime_batch_dims_and_broadcast_weights(gpu):
    # 3-D: every dim unknown at creation; small integers in f32 are exact, numpy is the check.
    # Second execution: weights with a batch of one, broadcast over src's batch.
    R = dnnl.RUNTIME_DIM_VAL
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    f32 = DT["f32"]
    rt = lambda tag: dnnl.memory_desc([R, R, R], f32, tag=tag)
    pd = dnnl.matmul_primitive_desc(eng, rt(dnnl.tag_abc), rt(dnnl.tag_acb), rt(dnnl.tag_abc))
    prim = dnnl.matmul(pd)
    r = np.random.default_rng(11)
    for B, Bw, M, K, N in ((3, 3, 17, 40, 24), (4, 1, 5, 64, 130)):
        s = r.integers(-4, 5, size=(B, M, K)).astype(np.float32)
        w = r.integers(-4, 5, size=(Bw, K, N)).astype(np.float32)
        dst = dnnl.memory(dnnl.memory_desc([B, M, N], f32, tag=dnnl.tag_abc), eng)
        prim.execute(strm, {dnnl.ARG_SRC: dnnl.memory(dnnl.memory_desc([B, M, K], f32, tag=dnnl.tag_abc), eng, s),
                            dnnl.ARG_WEIGHTS: dnnl.memory(dnnl.memory_desc([Bw, K, N], f32, tag=dnnl.tag_acb), eng,
                                                          np.ascontiguousarray(w.transpose(0, 2, 1))),
                            dnnl.ARG_DST: dst})
        strm.wait()
        assert np.array_equal(dst.read(np.float32).reshape(B, M, N), s @ w)


def test_batch_dims_broadcast_in_part(gpu):
    # numpy broadcasting over the batch dims (matmul.cpp:722-735): src has one of the two batch dims, weights
    # the other; bias and a binary operand broadcast in their own ways.  Small integers in f32: numpy is exact.
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    f32 = DT["f32"]
    r = np.random.default_rng(12)
    M, K, N = 9, 24, 40
    for sb, wb in (((2, 3), (2, 1)), ((1, 3), (2, 1)), ((2, 1), (1, 3)), ((2, 3), (1, 3))):
        B = (max(sb[0], wb[0]), max(sb[1], wb[1]))
        s = r.integers(-4, 5, size=sb + (M, K)).astype(np.float32)
        w = r.integers(-4, 5, size=wb + (K, N)).astype(np.float32)
        bias = r.integers(-4, 5, size=(1, B[1], 1, N)).astype(np.float32)
        other = r.integers(-4, 5, size=(B[0], 1, M, 1)).astype(np.float32)
        mds = [dnnl.memory_desc(list(x.shape), f32, tag=dnnl.tag_abcd) for x in (s, w, bias, other)]
        dst_md = dnnl.memory_desc(list(B) + [M, N], f32, tag=dnnl.tag_abcd)
        attr = dnnl.primitive_attr()
        po = dnnl.post_ops()
        po.append_binary(cabi.BINARY["mul"], mds[3])
        attr.set_post_ops(po)
        pd = dnnl.matmul_primitive_desc(eng, mds[0], mds[1], dst_md, bias_md=mds[2], attr=attr)
        dst = dnnl.memory(dst_md, eng)
        dnnl.matmul(pd).execute(strm, {
            dnnl.ARG_SRC: dnnl.memory(mds[0], eng, s), dnnl.ARG_WEIGHTS: dnnl.memory(mds[1], eng, w),
            dnnl.ARG_BIAS: dnnl.memory(mds[2], eng, bias), dnnl.ARG_DST: dst,
            dnnl.ARG_ATTR_MULTIPLE_POST_OP(0) | dnnl.ARG_SRC_1: dnnl.memory(mds[3], eng, other)})
        strm.wait()
        want = ((s @ w) + bias) * other
        assert np.array_equal(dst.read(np.float32).reshape(want.shape), want), (sb, wb)


def test_host_side_scalar_scales_and_zero_points(gpu, oracle):
    """Scales / zero points set with is_on_host take host-scalar memory objects
    (dnnl.h:494-553,631-659): C3-like int8 problem with a src zero point, all
    four single-valued parameters on the host, per-column weights scales on the
    device.  The value is read at each execution: changing it changes the result."""
    from onednn_amd.problem import QuantParam
    p = configs.config3(M=96, N=160, K=256, wtag="ba")
    p.src_dt = cabi.DT_U8
    p.src = (np.asarray(p.src).view(np.uint8) ^ 0x80).astype(np.uint8)
    p.quant["src_zp"] = QuantParam(cabi.DT_S32, 0, np.array([128], np.int32))
    p.quant["dst_zp"] = QuantParam(cabi.DT_S32, 0, np.array([3], np.int32))
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    mds = {"src": dnnl.memory_desc([p.M, p.K], p.src_dt, strides=list(p.src_stride[1:])),
           "wei": dnnl.memory_desc([p.K, p.N], p.wei_dt, strides=list(p.wei_stride[1:])),
           "dst": dnnl.memory_desc([p.M, p.N], p.dst_dt, strides=list(p.dst_stride[1:]))}
    attr = dnnl.primitive_attr()
    attr.set_scales(dnnl.ARG_SRC, 0, (), DT["f32"], is_on_host=1)
    attr.set_scales(dnnl.ARG_DST, 0, (), DT["f32"], is_on_host=1)
    attr.set_scales(dnnl.ARG_WEIGHTS, 2, (), DT["f32"])
    attr.set_zero_points(dnnl.ARG_SRC, 0, (), DT["s32"], is_on_host=1)
    attr.set_zero_points(dnnl.ARG_DST, 0, (), DT["s32"], is_on_host=1)
    po = dnnl.post_ops()
    for op in p.post_ops:
        po.append_eltwise(op.alg, op.alpha, op.beta)
    attr.set_post_ops(po)
    pd = dnnl.matmul_primitive_desc(eng, mds["src"], mds["wei"], mds["dst"], attr=attr)
    prim = dnnl.matmul(pd)
    scal = {"src_scale": dnnl.host_scalar(DT["f32"], p.quant["src_scale"].data.reshape(-1)[0]),
            "dst_scale": dnnl.host_scalar(DT["f32"], p.quant["dst_scale"].data.reshape(-1)[0]),
            "src_zp": dnnl.host_scalar(DT["s32"], np.int32(128)), "dst_zp": dnnl.host_scalar(DT["s32"], np.int32(3))}
    dst = dnnl.memory(mds["dst"], eng)
    args = {dnnl.ARG_SRC: dnnl.memory(mds["src"], eng, p.src), dnnl.ARG_WEIGHTS: dnnl.memory(mds["wei"], eng, p.wei),
            dnnl.ARG_DST: dst,
            dnnl.ARG_ATTR_SCALES | dnnl.ARG_SRC: scal["src_scale"], dnnl.ARG_ATTR_SCALES | dnnl.ARG_DST: scal["dst_scale"],
            dnnl.ARG_ATTR_SCALES | dnnl.ARG_WEIGHTS: dnnl.memory(dnnl.memory_desc([1, p.N], DT["f32"], tag=dnnl.tag_ab), eng,
                                                                 p.quant["wei_scale"].data),
            dnnl.ARG_ATTR_ZERO_POINTS | dnnl.ARG_SRC: scal["src_zp"], dnnl.ARG_ATTR_ZERO_POINTS | dnnl.ARG_DST: scal["dst_zp"]}
    prim.execute(strm, args)
    strm.wait()
    assert_bit_exact(p, dst.read(np.int8), oracle.run_oracle(p), pd.impl_info_str())
    # new values in the same memory objects, same primitive
    scal["dst_scale"].set(np.float32(0.125))
    scal["dst_zp"].set(np.int32(-5))
    scal["src_zp"].set(np.int32(120))
    p.quant["dst_scale"].data = np.array([0.125], np.float32)
    p.quant["dst_zp"].data = np.array([-5], np.int32)
    p.quant["src_zp"].data = np.array([120], np.int32)
    prim.execute(strm, args)
    strm.wait()
    assert_bit_exact(p, dst.read(np.int8), oracle.run_oracle(p), pd.impl_info_str())
    # a device memory where a host scalar is expected, and the other way round
    bad = dict(args)
    bad[dnnl.ARG_ATTR_SCALES | dnnl.ARG_SRC] = dnnl.memory(dnnl.memory_desc([1], DT["f32"], tag=dnnl.tag_a), eng)
    with pytest.raises(dnnl.error) as e:
        prim.execute(strm, bad)
    assert e.value.status == dnnl.invalid_arguments
    bad = dict(args)
    bad[dnnl.ARG_ATTR_SCALES | dnnl.ARG_WEIGHTS] = dnnl.host_scalar(DT["f32"], np.float32(1))
    with pytest.raises(dnnl.error) as e:
        prim.execute(strm, bad)
    assert e.value.status == dnnl.invalid_arguments


def test_use_dst_for_bwd_eltwise_equals_its_base_algorithm(gpu):
    from onednn_amd.problem import PostOp
    base = {"relu": 0x100, "tanh": 0x101, "elu": 0x102, "sqrt": 0x103, "logistic": 0x104, "exp": 0x105, "clip_v2": 0x106}
    for name, alias in base.items():
        outs = []
        for alg in (cabi.ELTWISE[name], alias):
            p = configs.config1(M=64, N=128, K=128)
            p.post_ops = [PostOp(kind=cabi.PO_ELTWISE, alg=alg, alpha=0.5, beta=2.0, scale=1.0)]
            got, _, _ = run_through_api(p)
            outs.append(np.asarray(got).view(np.uint32))
        assert np.array_equal(outs[0], outs[1]), name


def test_binary_select_post_op(gpu, oracle):
    """dst = cond ? dst : src1 (primitive_attr_postops.cpp:44,345-360): through the C ABI against the oracle, against
    numpy on exact values, and through dnnl_post_ops_append_binary_v2 with DNNL_ARG_SRC_2."""
    from onednn_amd.problem import GpuRun, PostOp
    r = np.random.default_rng(21)
    p = configs.config1(M=48, N=96, K=64, dst="s32")            # exact integer sums
    M, N = p.M, p.N
    other = r.integers(-9, 10, size=(1, N)).astype(np.float32)
    cond = r.integers(-1, 2, size=(M, 1)).astype(np.int8)        # negative values are true as well
    p.post_ops = [PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["linear"], alpha=2.0, beta=1.0, scale=1.0),
                  PostOp(kind=cabi.PO_BINARY, alg=cabi.BINARY["select"], dt=cabi.DT_F32, stride=(0, 0, 1), data=other),
                  PostOp(kind=cabi.PO_SELECT_COND, dt=cabi.DT_S8, stride=(0, 1, 0), data=cond)]
    plain = configs.config1(M=48, N=96, K=64, dst="s32")
    acc = np.asarray(oracle.run_oracle(plain)).view(np.int32).reshape(M, N)
    want_np = np.where(cond != 0, 2 * acc + 1, other.astype(np.int32))
    want = np.asarray(oracle.run_oracle(p)).view(np.int32).reshape(M, N)
    assert np.array_equal(want, want_np)                          # pins the oracle's branch
    run = GpuRun(p, None)
    try:
        run.launch()
        got, name = np.asarray(run.result()).view(np.int32).reshape(M, N), cabi.impl_name(run.impl)
    finally:
        run.free()
    assert name == "hip:ref:any" and np.array_equal(got, want)
    # a select without its condition entry is refused
    bad = configs.config1(M=48, N=96, K=64, dst="s32")
    bad.post_ops = p.post_ops[:2]
    assert cabi.query(bad.desc())[0] == cabi.INVALID_ARGUMENTS
    # the same through the API
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    mds = [dnnl.memory_desc([M, p.K], p.src_dt, tag=dnnl.tag_ab), dnnl.memory_desc([p.K, N], p.wei_dt, strides=list(p.wei_stride[1:])),
           dnnl.memory_desc([M, N], p.dst_dt, tag=dnnl.tag_ab)]
    o_md, c_md = dnnl.memory_desc([1, N], DT["f32"], tag=dnnl.tag_ab), dnnl.memory_desc([M, 1], DT["s8"], tag=dnnl.tag_ab)
    attr = dnnl.primitive_attr()
    attr.set_zero_points_mask(dnnl.ARG_SRC, 0)
    po = dnnl.post_ops()
    po.append_eltwise(cabi.ELTWISE["linear"], 2.0, 1.0)
    po.append_binary(cabi.BINARY["select"], o_md, c_md)
    attr.set_post_ops(po)
    pd = dnnl.matmul_primitive_desc(eng, mds[0], mds[1], mds[2], attr=attr)
    assert pd.impl_info_str() == "hip:ref:any"
    dst = dnnl.memory(mds[2], eng)
    dnnl.matmul(pd).execute(strm, {
        dnnl.ARG_SRC: dnnl.memory(mds[0], eng, p.src), dnnl.ARG_WEIGHTS: dnnl.memory(mds[1], eng, p.wei), dnnl.ARG_DST: dst,
        dnnl.ARG_ATTR_ZERO_POINTS | dnnl.ARG_SRC: dnnl.memory(dnnl.memory_desc([1], DT["s32"], tag=dnnl.tag_a), eng,
                                                             p.quant["src_zp"].data),
        dnnl.ARG_ATTR_MULTIPLE_POST_OP(1) | dnnl.ARG_SRC_1: dnnl.memory(o_md, eng, other),
        dnnl.ARG_ATTR_MULTIPLE_POST_OP(1) | dnnl.ARG_SRC_2: dnnl.memory(c_md, eng, cond)})
    strm.wait()
    assert np.array_equal(dst.read(np.int32).reshape(M, N), want)


def test_one_primitive_two_threads_two_streams(gpu, oracle):
    """primitive_t::execute is const and may run concurrently from several host threads on different streams
    (src/common/primitive.hpp:54).  u8 src + row-major weights: the transposed weights and the column sums live in the
    primitive's own scratchpad, which both executions use -- the second stream waits for the first one's launches."""
    import threading
    p = configs.config1(M=256, N=512, K=512, dst="s32")
    want = np.asarray(oracle.run_oracle(p)).view(np.int32).reshape(p.M, p.N)
    eng = dnnl.engine(dnnl.gpu, 0)
    mds = [dnnl.memory_desc([p.M, p.K], p.src_dt, tag=dnnl.tag_ab), dnnl.memory_desc([p.K, p.N], p.wei_dt, tag=dnnl.tag_ab),
           dnnl.memory_desc([p.M, p.N], p.dst_dt, tag=dnnl.tag_ab)]
    attr = dnnl.primitive_attr()
    attr.set_zero_points_mask(dnnl.ARG_SRC, 0)
    pd = dnnl.matmul_primitive_desc(eng, mds[0], mds[1], mds[2], attr=attr)
    assert pd.impl_info_str().startswith("hip:mfma_i8")
    prim = dnnl.matmul(pd)
    wei = dnnl.memory(mds[1], eng, p.wei)
    zp = dnnl.memory(dnnl.memory_desc([1], DT["s32"], tag=dnnl.tag_a), eng, p.quant["src_zp"].data)
    # each thread multiplies its own src (a row permutation of the problem's) into its own dst
    perms = [np.arange(p.M), np.arange(p.M)[::-1].copy()]
    errors = []

    def worker(t):
        strm = dnnl.stream(eng)
        src = dnnl.memory(mds[0], eng, np.ascontiguousarray(p.src[perms[t]]))
        dst = dnnl.memory(mds[2], eng)
        for it in range(50):
            prim.execute(strm, {dnnl.ARG_SRC: src, dnnl.ARG_WEIGHTS: wei, dnnl.ARG_DST: dst,
                                dnnl.ARG_ATTR_ZERO_POINTS | dnnl.ARG_SRC: zp})
            strm.wait()
            got = dst.read(np.int32).reshape(p.M, p.N)
            if not np.array_equal(got, want[perms[t]]):
                errors.append((t, it, int(np.count_nonzero(got != want[perms[t]]))))
                return

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
