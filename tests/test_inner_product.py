"""Inner product, forward (the backward passes: test_inner_product_backward.py),
on top of the matmul kernels: dst[mb, oc] = sum over (ic, spatial) of src * weights, the caller of the matmul path the reference
lists next to it (src/common/inner_product.cpp, src/cpu/ref_inner_product.cpp,
src/cpu/ref_inner_product_int8.cpp).

CPU part: the oracle's restatement is pinned against numpy (tensordot over the
reduced dims on exact data, every ndims, plain and channels-last layouts; the
scale / bias / dst-scale order on data where another order changes bits), and
the descriptor rules of ip_desc_init / ip_attr_check are checked through the
C API on a descriptor-only engine (status codes, resolved `any` layouts, the
matmul the descriptor lowers to) -- modelled on
tests/gtests/test_inner_product_forward.cpp:100-160,245-330 and
tests/benchdnn/inputs/ip/test_ip_int8, test_ip_ci.

GPU part: execution through libdnnl_amd.so against the oracle: bit-exact for
integer src (s32 sums, then the same f32 operations in the same order) and for
exactly representable float data; random float data within the forward error
bound of a float32 K-sum (helpers.gemm_bound) around a float64 tensordot."""
import os

import numpy as np
import pytest

os.environ.setdefault("ONEDNN_AMD_ALLOW_NO_DEVICE", "1")

from onednn_amd import cabi, dnnl  # noqa: E402
from onednn_amd import dtypes as dtp  # noqa: E402
from onednn_amd.problem import MatmulProblem, PostOp, QuantParam, storage_dtype  # noqa: E402
from tests.helpers import assert_bit_exact, assert_within_bound, gemm_bound, logical  # noqa: E402

DT = cabi.DT_NAMES
MASK_COMMON, MASK_COL = 0, 4
PLAIN = {2: dnnl.tag_ab, 3: dnnl.tag_abc, 4: dnnl.tag_abcd, 5: dnnl.tag_abcde}
CHANNELS_LAST = {2: dnnl.tag_ab, 3: dnnl.tag_acb, 4: dnnl.tag_acdb, 5: dnnl.tag_acdeb}

# (mb, ic, spatial, oc): the reference's own small cases (test_inner_product_forward.cpp EXPAND_SIZES_*,
# inputs/ip/shapes_3d, shapes_bert scaled down) plus ragged sizes
SHAPES = [
    (2, 32, (), 48),
    (5, 17, (), 3),
    (2, 8, (5,), 11),
    (4, 14, (5, 5), 25),
    (2, 32, (6, 6), 48),
    (3, 4, (2, 3, 3), 10),
    (1, 64, (2, 3, 3), 20),
]


def as_layout(logical_arr, channels_last):
    """A view of the logical array whose memory order is plain (a b c ...) or
    channels-last (a c ... b): same logical indexing, different strides."""
    if not channels_last or logical_arr.ndim == 2:
        return np.ascontiguousarray(logical_arr)
    nd = logical_arr.ndim
    order = [0] + list(range(2, nd)) + [1]
    store = np.ascontiguousarray(logical_arr.transpose(order))
    inv = np.argsort(order)
    return store.transpose(inv)


def int_data(seed, shape, dt):
    r = np.random.default_rng(seed)
    if dt == "u8":
        return r.integers(0, 256, size=shape, dtype=np.uint8)
    return r.integers(-128, 128, size=shape, dtype=np.int8)


def small_float_data(seed, shape, dt):
    """Integer values in [-4, 4]: exact in every float type of the path, and so
    is any sum of a few thousand products."""
    v = np.random.default_rng(seed).integers(-4, 5, size=shape).astype(np.float32)
    return encode(v, dt)


def encode(v, dt):
    v = np.asarray(v, np.float32)
    if dt == "f32":
        return v
    if dt == "bf16":
        return dtp.f32_to_bf16(v.reshape(-1)).reshape(v.shape)
    if dt == "f16":
        return v.astype(np.float16).view(np.uint16)
    if dt == "f8_e4m3":
        return dtp.f32_to_e4m3(v.reshape(-1)).reshape(v.shape)
    if dt == "f8_e5m2":
        h = v.astype(np.float16).view(np.uint16)       # e5m2 is the top byte of f16: exact for the values used here
        assert not (h & 0xff).any()
        return (h >> 8).astype(np.uint8)
    raise KeyError(dt)


def ip_problem(mb, ic, sp, oc, sdt, wdt, ddt, *, bias=None, bias_dt="f32", quant=None, post_ops=None,
               dst_init=None):
    K = ic * int(np.prod(sp, dtype=np.int64))
    dummy_s = np.zeros(1, storage_dtype(DT[sdt]))
    dummy_w = np.zeros(1, storage_dtype(DT[wdt]))
    return MatmulProblem(M=mb, N=oc, K=K, src_dt=DT[sdt], wei_dt=DT[wdt], dst_dt=DT[ddt], src=dummy_s, wei=dummy_w,
                         bias_dt=DT[bias_dt] if bias is not None else cabi.DT_UNDEF, bias=bias,
                         quant=quant or {}, post_ops=post_ops or [], dst_init=dst_init, name=f"ip-{sdt}-{wdt}-{ddt}")


def dst_values(p, raw):
    return logical(p, raw).reshape(p.M, p.N)


# ------------------------------------------------------------------ the oracle, pinned
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("channels_last", [False, True])
@pytest.mark.parametrize("sdt", ["u8", "s8"])
def test_oracle_int8_sum_is_tensordot(oracle, shape, channels_last, sdt):
    mb, ic, sp, oc = shape
    src = int_data(1, (mb, ic) + sp, sdt)
    wei = int_data(2, (oc, ic) + sp, "s8")
    p = ip_problem(mb, ic, sp, oc, sdt, "s8", "s32")
    got = oracle.run_oracle_inner_product(p, as_layout(src, channels_last), as_layout(wei, channels_last))
    axes = list(range(1, src.ndim))
    want = np.tensordot(src.astype(np.int64), wei.astype(np.int64), axes=(axes, axes))
    assert np.array_equal(dst_values(p, got).astype(np.int64), want)


def test_oracle_src_and_weights_use_their_own_strides(oracle):
    """A transposed operand fails this: src channels-last against plain weights
    and the other way round give the plain result."""
    mb, ic, sp, oc = 3, 6, (4, 5), 7
    src, wei = int_data(3, (mb, ic) + sp, "s8"), int_data(4, (oc, ic) + sp, "s8")
    p = ip_problem(mb, ic, sp, oc, "s8", "s8", "s32")
    want = np.tensordot(src.astype(np.int64), wei.astype(np.int64), axes=([1, 2, 3], [1, 2, 3]))
    for s_cl, w_cl in ((True, False), (False, True)):
        got = oracle.run_oracle_inner_product(p, as_layout(src, s_cl), as_layout(wei, w_cl))
        assert np.array_equal(dst_values(p, got).astype(np.int64), want)


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16", "f8_e4m3", "f8_e5m2"])
def test_oracle_float_sum_on_exact_data(oracle, dt):
    mb, ic, sp, oc = 4, 14, (5, 5), 25
    sv = np.random.default_rng(5).integers(-4, 5, size=(mb, ic) + sp).astype(np.float32)
    wv = np.random.default_rng(6).integers(-4, 5, size=(oc, ic) + sp).astype(np.float32)
    bias = np.arange(oc, dtype=np.float32) - 7
    p = ip_problem(mb, ic, sp, oc, dt, dt, "f32", bias=bias)
    got = oracle.run_oracle_inner_product(p, as_layout(encode(sv, dt), True), as_layout(encode(wv, dt), True))
    want = np.tensordot(sv.astype(np.float64), wv.astype(np.float64), axes=([1, 2, 3], [1, 2, 3])) + bias
    assert np.array_equal(dst_values(p, got).astype(np.float64), want)


def test_oracle_int8_scale_bias_dst_scale_order(oracle):
    """ref_inner_product_int8.cpp:89-111: ((acc * src_scale) * wei_scale[oc] + bias), post-ops, / dst_scale -- in
    float32, one rounding per operation.  The data make the order visible: folding the two scales into one factor,
    adding the bias before scaling, or multiplying by a reciprocal of the dst scale each change some element."""
    mb, ic, oc = 16, 96, 64
    r = np.random.default_rng(7)
    src, wei = int_data(8, (mb, ic), "u8"), int_data(9, (oc, ic), "s8")
    ss = np.array([0.0123], np.float32)
    ws = r.uniform(1e-3, 1e-2, size=oc).astype(np.float32)
    ds = np.array([0.3], np.float32)
    bias = r.uniform(-1, 1, size=oc).astype(np.float32)
    quant = {"src_scale": QuantParam(cabi.DT_F32, MASK_COMMON, ss), "wei_scale": QuantParam(cabi.DT_F32, MASK_COL, ws),
             "dst_scale": QuantParam(cabi.DT_F32, MASK_COMMON, ds)}
    p = ip_problem(mb, ic, (), oc, "u8", "s8", "f32", bias=bias, quant=quant)
    got = dst_values(p, oracle.run_oracle_inner_product(p, src, wei))
    acc = (src.astype(np.int64) @ wei.astype(np.int64).T).astype(np.float32)
    want = ((acc * ss[0]) * ws[None, :] + bias[None, :]) / ds[0]
    assert want.dtype == np.float32
    assert np.array_equal(got, want)
    folded = (acc * (ss[0] * ws)[None, :] + bias[None, :]) / ds[0]
    recip = ((acc * ss[0]) * ws[None, :] + bias[None, :]) * (np.float32(1) / ds[0])
    bias_first = ((acc + bias[None, :]) * ss[0]) * ws[None, :] / ds[0]
    assert (folded != want).any() and (recip != want).any() and (bias_first != want).any()


def test_oracle_common_weights_scale_and_saturating_dst(oracle):
    mb, ic, oc = 8, 64, 32
    src, wei = int_data(10, (mb, ic), "s8"), int_data(11, (oc, ic), "s8")
    ws = np.array([0.004], np.float32)
    p = ip_problem(mb, ic, (), oc, "s8", "s8", "s8", quant={"wei_scale": QuantParam(cabi.DT_F32, MASK_COMMON, ws)})
    got = dst_values(p, oracle.run_oracle_inner_product(p, src, wei))
    acc = (src.astype(np.int64) @ wei.astype(np.int64).T).astype(np.float32)
    want = np.rint(np.clip(acc * ws[0], -128, 127))
    assert np.array_equal(got, want)
    assert (want == 127).any() and (want == -128).any()


# ------------------------------------------------------------------ descriptor rules (no GPU)
@pytest.fixture(scope="module")
def eng():
    return dnnl.engine(dnnl.gpu, 0)


def status_of(fn):
    try:
        fn()
        return dnnl.success
    except dnnl.error as e:
        return e.status


def md(dims, dt, tag):
    return dnnl.memory_desc(list(dims), DT[dt], tag=tag)


def ip_pd(eng, mb, ic, sp, oc, sdt="s8", wdt="s8", ddt="f32", stag=None, wtag=None, dtag=dnnl.tag_ab, bias=None,
          attr=None, prop=dnnl.forward_inference):
    nd = 2 + len(sp)
    src = md((mb, ic) + tuple(sp), sdt, PLAIN[nd] if stag is None else stag)
    wei = md((oc, ic) + tuple(sp), wdt, PLAIN[nd] if wtag is None else wtag)
    dst = md((mb, oc), ddt, dtag)
    return dnnl.inner_product_forward_primitive_desc(eng, prop, src, wei, dst, bias_md=bias, attr=attr)


def test_queries_describe_the_inner_product(eng):
    pd = ip_pd(eng, 4, 14, (5, 5), 25, bias=md((25,), "f32", dnnl.tag_a), prop=dnnl.forward_training)
    assert pd.query_s32(dnnl.query_primitive_kind) == dnnl.kind_inner_product
    assert pd.query_s32(dnnl.query_prop_kind) == dnnl.forward_training
    assert pd.query_md(dnnl.query_src_md).dims() == [4, 14, 5, 5]
    assert pd.query_md(dnnl.query_weights_md).dims() == [25, 14, 5, 5]
    assert pd.query_md(dnnl.query_weights_md, 1).dims() == [25]
    assert pd.query_md(dnnl.query_dst_md).dims() == [4, 25]
    d = pd.lowered_desc()
    assert (d.batch, d.M, d.N, d.K) == (1, 4, 25, 14 * 25)
    assert tuple(d.src_stride)[1:] == (350, 1) and tuple(d.wei_stride)[1:] == (1, 350)


def test_any_takes_the_other_tensors_order(eng):
    # weights follow src (cpu_inner_product_pd.hpp:185-199), src follows weights (:165-182), both any -> plain
    pd = ip_pd(eng, 2, 8, (3, 5), 6, stag=dnnl.tag_nhwc, wtag=dnnl.tag_any)
    assert pd.query_md(dnnl.query_weights_md).strides() == [8 * 15, 1, 5 * 8, 8]
    pd = ip_pd(eng, 2, 8, (3, 5), 6, stag=dnnl.tag_any, wtag=dnnl.tag_ohwi)
    assert pd.query_md(dnnl.query_src_md).strides() == [8 * 15, 1, 5 * 8, 8]
    pd = ip_pd(eng, 2, 8, (3, 5), 6, stag=dnnl.tag_any, wtag=dnnl.tag_any, dtag=dnnl.tag_any)
    assert pd.query_md(dnnl.query_src_md).strides() == [120, 15, 5, 1]
    assert pd.query_md(dnnl.query_weights_md).strides() == [120, 15, 5, 1]
    assert pd.query_md(dnnl.query_dst_md).strides() == [6, 1]
    # io weights (ic outermost): src must not become column-major -- mb stays the outer dim
    pd = ip_pd(eng, 4, 8, (), 6, stag=dnnl.tag_any, wtag=dnnl.tag_io)
    assert pd.query_md(dnnl.query_src_md).strides() == [8, 1]


def test_channels_last_pairs_lower_to_one_k(eng):
    pd = ip_pd(eng, 2, 8, (3, 5), 6, stag=dnnl.tag_nhwc, wtag=dnnl.tag_ohwi)
    d = pd.lowered_desc()
    assert (d.M, d.N, d.K) == (2, 6, 120)
    assert tuple(d.src_stride)[1:] == (120, 1) and tuple(d.wei_stride)[1:] == (1, 120)
    # different orders of the reduced dims have no common K walk
    assert status_of(lambda: ip_pd(eng, 2, 8, (3, 5), 6, stag=dnnl.tag_nchw, wtag=dnnl.tag_ohwi)) == dnnl.unimplemented
    # ... unless the dims that differ have extent one
    ip_pd(eng, 2, 8, (1, 1), 6, stag=dnnl.tag_nchw, wtag=dnnl.tag_ohwi)


def test_int8_problems_run_on_the_matrix_cores(eng):
    pd = ip_pd(eng, 512, 1024, (), 1024, sdt="u8", ddt="s8")
    assert pd.impl_info_str().startswith("hip:mfma_i8")
    pd = ip_pd(eng, 256, 64, (4, 4), 512, sdt="s8", ddt="f32", stag=dnnl.tag_nhwc, wtag=dnnl.tag_any)
    assert pd.impl_info_str().startswith("hip:mfma_i8")


def test_shape_rules(eng):
    inv = dnnl.invalid_arguments
    f = dnnl.forward_inference

    def create(src, wei, dst, bias=None, prop=f):
        return status_of(lambda: dnnl.inner_product_forward_primitive_desc(eng, prop, src, wei, dst, bias_md=bias))

    s, w, d = md((2, 8, 3), "f32", dnnl.tag_abc), md((6, 8, 3), "f32", dnnl.tag_abc), md((2, 6), "f32", dnnl.tag_ab)
    assert create(s, w, d) == dnnl.success
    assert create(s, w, d, prop=dnnl.backward_data) == inv                       # inner_product.cpp:194-195
    assert create(s, md((6, 8), "f32", dnnl.tag_ab), d) == inv                   # ndims differ
    assert create(s, md((6, 8, 4), "f32", dnnl.tag_abc), d) == inv               # reduced dims differ
    assert create(s, w, md((2, 7), "f32", dnnl.tag_ab)) == inv                   # oc
    assert create(s, w, md((3, 6), "f32", dnnl.tag_ab)) == inv                   # mb
    assert create(s, w, md((2, 6, 1), "f32", dnnl.tag_abc)) == inv               # dst is two-dimensional
    assert create(s, w, d, bias=md((5,), "f32", dnnl.tag_a)) == inv
    assert create(s, w, d, bias=md((1, 6), "f32", dnnl.tag_ab)) == inv           # bias is one-dimensional
    assert create(md((2,), "f32", dnnl.tag_a), md((6,), "f32", dnnl.tag_a), d) == inv
    assert create(md((2, 0, 3), "f32", dnnl.tag_abc), md((6, 0, 3), "f32", dnnl.tag_abc), d) == inv  # empty weights
    assert create(s, w, d, bias=dnnl.zero_memory_desc()) == dnnl.success         # a zero descriptor: no bias


def test_zero_dims(eng):
    # tests/gtests/test_inner_product_forward.cpp:260-283: an empty batch is a valid (no-op) problem, empty weights are not
    ip_pd(eng, 0, 32, (6, 6), 48, sdt="f32", wdt="f32", stag=dnnl.tag_any, wtag=dnnl.tag_any, dtag=dnnl.tag_any)
    assert status_of(lambda: ip_pd(eng, 2, 0, (6, 6), 48, sdt="f32", wdt="f32")) == dnnl.invalid_arguments


def test_float_problems_run_on_the_matrix_cores(eng):
    pd = ip_pd(eng, 128, 2048, (), 1000, sdt="bf16", wdt="bf16", ddt="bf16", wtag=dnnl.tag_any)
    assert pd.impl_info_str().startswith("hip:mfma_h16") and pd.query_md(dnnl.query_weights_md).strides() == [2048, 1]
    pd = ip_pd(eng, 128, 512, (7, 7), 1000, sdt="f32", wdt="f32", ddt="f32", stag=dnnl.tag_nhwc, wtag=dnnl.tag_any)
    assert pd.impl_info_str().startswith("hip:mfma_h16")
    assert pd.query_md(dnnl.query_weights_md).strides() == [25088, 1, 3584, 512]


def test_data_type_rules(eng):
    un = dnnl.unimplemented
    assert status_of(lambda: ip_pd(eng, 2, 8, (), 6, sdt="s8", wdt="u8")) == un        # integer weights are s8
    assert status_of(lambda: ip_pd(eng, 2, 8, (), 6, sdt="bf16", wdt="f32")) == un     # float weights match src
    assert status_of(lambda: ip_pd(eng, 2, 8, (), 6, sdt="bf16", wdt="bf16", ddt="f16")) == un
    for sdt, ddt in (("f32", "f32"), ("bf16", "bf16"), ("bf16", "f32"), ("f16", "f16"), ("f8_e4m3", "f32"),
                     ("f8_e5m2", "f8_e5m2")):
        ip_pd(eng, 2, 8, (), 6, sdt=sdt, wdt=sdt, ddt=ddt)
    for ddt in ("f32", "bf16", "f16", "s32", "s8", "u8"):
        ip_pd(eng, 2, 8, (), 6, sdt="u8", wdt="s8", ddt=ddt)


def test_attribute_rules(eng):
    un = dnnl.unimplemented

    def with_attr(fill, **kw):
        a = dnnl.primitive_attr()
        fill(a)
        return status_of(lambda: ip_pd(eng, 2, 8, (), 6, attr=a, **kw))

    assert with_attr(lambda a: a.set_scales_mask(dnnl.ARG_SRC, 0)) == dnnl.success
    assert with_attr(lambda a: a.set_scales_mask(dnnl.ARG_WEIGHTS, 1)) == dnnl.success
    assert with_attr(lambda a: a.set_scales_mask(dnnl.ARG_DST, 0)) == dnnl.success
    assert with_attr(lambda a: a.set_scales_mask(dnnl.ARG_SRC, 1)) == un               # inner_product.cpp:146-148
    assert with_attr(lambda a: a.set_scales_mask(dnnl.ARG_WEIGHTS, 2)) == un           # :149-152
    assert with_attr(lambda a: a.set_scales_mask(dnnl.ARG_WEIGHTS, 3)) == un
    assert with_attr(lambda a: a.set_scales_mask(dnnl.ARG_DST, 2)) == un               # :153-155
    assert with_attr(lambda a: a.set_scales(dnnl.ARG_SRC, 0, is_on_host=1)) == un      # :159-162
    assert with_attr(lambda a: a.set_zero_points_mask(dnnl.ARG_SRC, 0)) == un          # not in the mask, :128-141
    assert with_attr(lambda a: a.set_scales_mask(dnnl.ARG_SRC, 0), sdt="f32", wdt="f32") == un  # scales: int8 only
    assert with_attr(lambda a: a.set_rounding(dnnl.ARG_DST, dnnl.rounding_stochastic), sdt="f32", wdt="f32",
                     ddt="f32") == un

    def post(a):
        po = dnnl.post_ops()
        po.append_sum(0.5)
        po.append_eltwise(cabi.ELTWISE["relu"], 0.5, 0.0)
        po.append_binary(cabi.BINARY["mul"], md((2, 6), "s8", dnnl.tag_ab))
        po.append_prelu(2)
        a.set_post_ops(po)

    assert with_attr(post) == dnnl.success
    # the caller reads back the attributes it gave (weights mask 1), not the lowered ones
    a = dnnl.primitive_attr()
    a.set_scales_mask(dnnl.ARG_WEIGHTS, 1)
    pd = ip_pd(eng, 2, 8, (), 6, attr=a)
    assert pd.lowered_desc().wei_scale.mask == MASK_COL


# ------------------------------------------------------------------ execution on the device
def run_ip(p, src, wei, sp, stag, wtag, *, post_mem=None, prop=dnnl.forward_inference):
    """Executes the inner product that `p` describes after the sum, on src / wei views (logical shapes, any
    memory order; their storage is uploaded as it lies in memory)."""
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    mb, oc = p.M, p.N
    src_md = dnnl.memory_desc(list(src.shape), p.src_dt, tag=stag)
    wei_md = dnnl.memory_desc(list(wei.shape), p.wei_dt, tag=wtag)
    dst_md = dnnl.memory_desc([mb, oc], p.dst_dt, tag=dnnl.tag_ab)
    bias_md = dnnl.memory_desc([oc], p.bias_dt, tag=dnnl.tag_a) if p.bias is not None else None
    attr = dnnl.primitive_attr()
    args = {}
    for qname, q in p.quant.items():
        which = qname.split("_")[0]
        arg = {"src": dnnl.ARG_SRC, "wei": dnnl.ARG_WEIGHTS, "dst": dnnl.ARG_DST}[which]
        attr.set_scales_mask(arg, 1 if q.mask == MASK_COL else 0)
        qmd = dnnl.memory_desc([q.data.size], q.dt, tag=dnnl.tag_a)
        args[dnnl.ARG_ATTR_SCALES | arg] = dnnl.memory(qmd, eng, q.data)
    po = dnnl.post_ops()
    for i, op in enumerate(p.post_ops):
        if op.kind == cabi.PO_ELTWISE:
            po.append_eltwise(op.alg, op.alpha, op.beta)
        elif op.kind == cabi.PO_SUM:
            po.append_sum(op.scale, op.zero_point, op.dt)
        elif op.kind == cabi.PO_BINARY:
            dims = [mb if op.stride[1] else 1, oc if op.stride[2] else 1]
            bmd = dnnl.memory_desc(dims, op.dt, tag=dnnl.tag_ab)
            po.append_binary(op.alg, bmd)
            args[dnnl.ARG_ATTR_MULTIPLE_POST_OP(i) | dnnl.ARG_SRC_1] = dnnl.memory(bmd, eng, op.data)
    if p.post_ops:
        attr.set_post_ops(po)
    pd = dnnl.inner_product_forward_primitive_desc(eng, prop, src_md, wei_md, dst_md, bias_md=bias_md, attr=attr)
    prim = dnnl.inner_product_forward(pd)

    def storage(view):
        # the bytes in memory order: undo the logical transposition of as_layout
        order = np.argsort([-s for s in view.strides], kind="stable")
        return np.ascontiguousarray(view.transpose(order))

    # a tensor given as format_tag::any lies in memory the way the descriptor resolved it
    if stag == dnnl.tag_any:
        src_md = pd.query_md(dnnl.query_src_md)
    if wtag == dnnl.tag_any:
        wei_md = pd.query_md(dnnl.query_weights_md)
    args[dnnl.ARG_SRC] = dnnl.memory(src_md, eng, storage(src))
    args[dnnl.ARG_WEIGHTS] = dnnl.memory(wei_md, eng, storage(wei))
    dst = dnnl.memory(dst_md, eng, p.initial_dst())
    args[dnnl.ARG_DST] = dst
    if p.bias is not None:
        args[dnnl.ARG_BIAS] = dnnl.memory(bias_md, eng, p.bias)
    prim.execute(strm, args)
    strm.wait()
    return dst.read(storage_dtype(p.dst_dt)), pd.impl_info_str()


def int8_chain(mb, oc, seed, ddt):
    """scales src:common + wei:per_oc + dst:common, f32 bias, sum + relu + binary mul (test_ip_int8's attribute set)"""
    r = np.random.default_rng(seed)
    quant = {"src_scale": QuantParam(cabi.DT_F32, MASK_COMMON, np.array([0.25], np.float32)),
             "wei_scale": QuantParam(cabi.DT_F32, MASK_COL, r.choice([0.0625, 0.125, 0.25], size=oc).astype(np.float32)),
             "dst_scale": QuantParam(cabi.DT_F32, MASK_COMMON, np.array([2.25], np.float32))}
    mul = r.integers(-3, 4, size=(mb, oc), dtype=np.int8)
    post = [PostOp(cabi.PO_BINARY, alg=cabi.BINARY["mul"], dt=cabi.DT_S8, stride=(0, oc, 1), data=mul),
            PostOp(cabi.PO_SUM, scale=0.5), PostOp(cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"], alpha=0.5)]
    bias = r.uniform(-4, 4, size=oc).astype(np.float32)
    init = None
    if ddt == "f32":
        init = r.uniform(-8, 8, size=mb * oc).astype(np.float32)
    elif ddt == "s8":
        init = r.integers(-128, 128, size=mb * oc, dtype=np.int8)
    elif ddt == "u8":
        init = r.integers(0, 256, size=mb * oc, dtype=np.uint8)
    elif ddt == "s32":
        init = r.integers(-1000, 1000, size=mb * oc).astype(np.int32)
    return quant, post, bias, init


@pytest.mark.gpu
@pytest.mark.parametrize("shape", SHAPES + [(64, 128, (), 256), (33, 64, (2, 2), 130)])
@pytest.mark.parametrize("channels_last", [False, True])
@pytest.mark.parametrize("sdt,ddt", [("u8", "s32"), ("s8", "f32"), ("u8", "s8"), ("s8", "u8")])
def test_gpu_int8_bit_exact(gpu, oracle, shape, channels_last, sdt, ddt):
    mb, ic, sp, oc = shape
    src, wei = int_data(21, (mb, ic) + sp, sdt), int_data(22, (oc, ic) + sp, "s8")
    quant, post, bias, init = int8_chain(mb, oc, 23, ddt)
    p = ip_problem(mb, ic, sp, oc, sdt, "s8", ddt, bias=bias, quant=quant, post_ops=post, dst_init=init)
    nd = src.ndim
    tags = CHANNELS_LAST if channels_last else PLAIN
    sv, wv = as_layout(src, channels_last), as_layout(wei, channels_last)
    got, impl = run_ip(p, sv, wv, sp, tags[nd], tags[nd])
    assert_bit_exact(p, got, oracle.run_oracle_inner_product(p, sv, wv), impl)


@pytest.mark.gpu
def test_gpu_int8_bert_shape_on_the_matrix_cores(gpu, oracle):
    """inputs/ip/shapes_bert ic768oc3072 at mb 384, weights with format_tag::any."""
    mb, ic, oc = 384, 768, 3072
    src, wei = int_data(31, (mb, ic), "u8"), int_data(32, (oc, ic), "s8")
    quant, post, bias, init = int8_chain(mb, oc, 33, "s8")
    p = ip_problem(mb, ic, (), oc, "u8", "s8", "s8", bias=bias, quant=quant, post_ops=post, dst_init=init)
    got, impl = run_ip(p, src, wei, (), dnnl.tag_nc, dnnl.tag_any)
    assert impl.startswith("hip:mfma_i8")
    assert_bit_exact(p, got, oracle.run_oracle_inner_product(p, src, wei), impl)


@pytest.mark.gpu
@pytest.mark.parametrize("dt,ddt", [("f32", "f32"), ("bf16", "bf16"), ("bf16", "f32"), ("f16", "f16"),
                                    ("f8_e4m3", "f32"), ("f8_e5m2", "f8_e5m2")])
@pytest.mark.parametrize("shape", [(4, 14, (5, 5), 25), (3, 4, (2, 3, 3), 10), (32, 128, (), 64)])
def test_gpu_float_exact_data(gpu, oracle, dt, ddt, shape):
    mb, ic, sp, oc = shape
    src, wei = small_float_data(41, (mb, ic) + sp, dt), small_float_data(42, (oc, ic) + sp, dt)
    scale = 2.0 ** -6 if ddt.startswith("f8") else 1.0          # keep the sums inside the dst type's exact range
    post = [PostOp(cabi.PO_ELTWISE, alg=cabi.ELTWISE["linear"], alpha=scale, beta=0.0)]
    p = ip_problem(mb, ic, sp, oc, dt, dt, ddt, post_ops=post)
    nd = src.ndim
    sv, wv = as_layout(src, True), as_layout(wei, True)
    got, impl = run_ip(p, sv, wv, sp, CHANNELS_LAST[nd], CHANNELS_LAST[nd], prop=dnnl.forward_training)
    assert_bit_exact(p, got, oracle.run_oracle_inner_product(p, sv, wv), impl)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
def test_gpu_float_random_data_within_bound(gpu, dt):
    mb, ic, sp, oc = 16, 32, (3, 3), 48
    r = np.random.default_rng(51)
    sv = r.standard_normal((mb, ic) + sp).astype(np.float32)
    wv = r.standard_normal((oc, ic) + sp).astype(np.float32)
    src, wei = encode(sv, dt), encode(wv, dt)
    bias = r.uniform(-1, 1, size=oc).astype(np.float32)
    p = ip_problem(mb, ic, sp, oc, dt, dt, "f32", bias=bias,
                   post_ops=[PostOp(cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"], alpha=0.0)])
    got, impl = run_ip(p, src, wei, sp, dnnl.tag_nchw, dnnl.tag_oihw)
    from onednn_amd.problem import decode
    s64 = decode(DT[dt], src.reshape(-1), src.size).astype(np.float64).reshape(mb, -1)
    w64 = decode(DT[dt], wei.reshape(-1), wei.size).astype(np.float64).reshape(oc, -1)
    exact = s64 @ w64.T
    asum = np.abs(s64) @ np.abs(w64).T
    assert_within_bound(p, got, exact, gemm_bound(p.K, asum), impl)
