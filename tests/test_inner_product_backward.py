"""Inner product, backward by data and by weights, on top of the matmul
kernels (src/common/inner_product.cpp:185-330, src/cpu/ref_inner_product.cpp:100-217):
    diff_src[mb, k]     = sum over oc of diff_dst[mb, oc] * weights[oc, k]
    diff_weights[oc, k] = sum over mb of diff_dst[mb, oc] * src[mb, k]
    diff_bias[oc]       = sum over mb of diff_dst[mb, oc]
with k = (ic, spatial) flattened.

CPU part: the oracle's two restatements are pinned against numpy tensordot
over the other index pair on exactly representable data (every ndims, plain
and channels-last layouts, a mixed pair of layouts: a transposed operand or a
wrong reduced index changes every element), and diff_bias against a column sum
and against a sum whose bits depend on the order of the additions.  The
descriptor rules are checked through the C API on a descriptor-only engine --
modelled on tests/gtests/test_inner_product_backward_data.cpp:60-150 and
test_inner_product_backward_weights.cpp:60-200.

GPU part: execution through libdnnl_amd.so against the oracle: bit-exact on
exactly representable data, diff_bias bit-exact on any data (same order of
additions), random data within the forward error bound of a float32 sum
(helpers.gemm_bound) around a float64 tensordot."""
import ctypes as C
import os

import numpy as np
import pytest

os.environ.setdefault("ONEDNN_AMD_ALLOW_NO_DEVICE", "1")

from onednn_amd import cabi, dnnl  # noqa: E402
from onednn_amd.problem import decode, storage_dtype  # noqa: E402
from tests.helpers import gemm_bound  # noqa: E402
from tests.test_inner_product import (CHANNELS_LAST, DT, PLAIN, SHAPES, as_layout, encode, md,  # noqa: E402
                                      small_float_data, status_of)


@pytest.fixture(scope="module")
def eng():
    return dnnl.engine(dnnl.gpu, 0)


def values(dt, view):
    """float64 values of a (possibly permuted) view of raw storage, logical shape kept."""
    flat = np.ascontiguousarray(view).reshape(-1)
    return decode(DT[dt], flat, flat.size).astype(np.float64).reshape(view.shape)


def order_of(channels_last, nd):
    return [0] + list(range(2, nd)) + [1] if channels_last and nd > 2 else list(range(nd))


# ------------------------------------------------------------------ the oracle, pinned
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("channels_last", [False, True])
@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
def test_oracle_backward_data_is_tensordot_over_oc(oracle, shape, channels_last, dt):
    mb, ic, sp, oc = shape
    dd = small_float_data(1, (mb, oc), dt)
    wei = small_float_data(2, (oc, ic) + sp, dt)
    got = oracle.run_oracle_inner_product_bwd_data(dd, as_layout(wei, channels_last), (mb, ic) + sp, (dt, dt, dt),
                                                   order_of(channels_last, 2 + len(sp)))
    want = np.tensordot(values(dt, dd), values(dt, wei), axes=([1], [0]))
    assert got.shape == want.shape and np.array_equal(values(dt, got), want)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("channels_last", [False, True])
@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
def test_oracle_backward_weights_is_tensordot_over_mb(oracle, shape, channels_last, dt):
    mb, ic, sp, oc = shape
    dd = small_float_data(3, (mb, oc), dt)
    src = small_float_data(4, (mb, ic) + sp, dt)
    got, bias = oracle.run_oracle_inner_product_bwd_weights(dd, as_layout(src, channels_last), (dt, dt, dt, dt), True,
                                                            order_of(channels_last, 2 + len(sp)))
    want = np.tensordot(values(dt, dd), values(dt, src), axes=([0], [0]))
    assert got.shape == want.shape and np.array_equal(values(dt, got), want)
    assert np.array_equal(values(dt, bias), values(dt, dd).sum(axis=0))


def test_oracle_backward_tensors_use_their_own_strides(oracle):
    """Inputs in one layout, the output in the other; diff_dst column-major."""
    mb, ic, sp, oc = 3, 6, (4, 5), 7
    dd = small_float_data(5, (mb, oc), "f32")
    dd_t = np.ascontiguousarray(dd.T).T
    wei, src = small_float_data(6, (oc, ic) + sp, "f32"), small_float_data(7, (mb, ic) + sp, "f32")
    want_d = np.tensordot(dd.astype(np.float64), wei.astype(np.float64), axes=([1], [0]))
    want_w = np.tensordot(dd.astype(np.float64), src.astype(np.float64), axes=([0], [0]))
    for in_cl, out_cl in ((True, False), (False, True)):
        got = oracle.run_oracle_inner_product_bwd_data(dd_t, as_layout(wei, in_cl), (mb, ic) + sp, ("f32",) * 3,
                                                       order_of(out_cl, 4))
        assert np.array_equal(got.astype(np.float64), want_d)
        got, _ = oracle.run_oracle_inner_product_bwd_weights(dd_t, as_layout(src, in_cl), ("f32",) * 4, False,
                                                             order_of(out_cl, 4))
        assert np.array_equal(got.astype(np.float64), want_w)


def test_oracle_sums_run_in_ascending_order_in_f32(oracle):
    """1 + 2^-24 + 2^-24 + ... : added one at a time to 1.0f every term is lost; any pairwise or reversed order
    keeps them.  Pins the f32 accumulator and the order of diff_bias, diff_weights (over mb) and diff_src (over oc)."""
    n = 65
    col = np.full(n, 2.0 ** -24, np.float32)
    col[0] = 1.0
    dd = np.stack([col, col[::-1]], axis=1)                          # [mb = n, oc = 2]
    one = np.ones((n, 1), np.float32)
    dw, db = oracle.run_oracle_inner_product_bwd_weights(dd, one, ("f32",) * 4, True)
    rev = np.float32(0)
    for v in col[::-1]:
        rev = np.float32(rev + v)
    assert rev > 1.0
    assert db[0] == 1.0 and db[1] == rev
    assert dw[0, 0] == 1.0 and dw[1, 0] == rev
    # backward data: oc is the reduced index
    ds = oracle.run_oracle_inner_product_bwd_data(np.ascontiguousarray(dd.T), one, (2, 1), ("f32",) * 3)
    assert ds[0, 0] == 1.0 and ds[1, 0] == rev


def test_oracle_output_types_round_once(oracle):
    """f32 sum, one rounding into a bf16 / f16 output."""
    dd = encode(np.array([[1.0, 2.0 ** -9]], np.float32), "bf16")          # [1, 2]
    wei = encode(np.array([[1.0], [1.0]], np.float32), "bf16")             # [2, 1]: 1 + 2^-9 rounds to even -> 1.0
    got = oracle.run_oracle_inner_product_bwd_data(dd, wei, (1, 1), ("bf16", "bf16", "bf16"))
    assert values("bf16", got)[0, 0] == 1.0
    got = oracle.run_oracle_inner_product_bwd_data(dd, wei, (1, 1), ("f32", "bf16", "bf16"))
    assert got[0, 0] == np.float32(1.0 + 2.0 ** -9)


# ------------------------------------------------------------------ descriptor rules (no GPU)
def bwd_d(eng, mb, ic, sp, oc, dt="f32", sdt=None, stag=None, wtag=None, dtag=dnnl.tag_ab, attr=None):
    nd = 2 + len(sp)
    ds = md((mb, ic) + tuple(sp), sdt or dt, PLAIN[nd] if stag is None else stag)
    w = md((oc, ic) + tuple(sp), dt, PLAIN[nd] if wtag is None else wtag)
    dd = md((mb, oc), dt, dtag)
    return dnnl.inner_product_backward_data_primitive_desc(eng, ds, w, dd, attr=attr)


def bwd_w(eng, mb, ic, sp, oc, dt="f32", wdt=None, bdt=None, stag=None, wtag=None, dtag=dnnl.tag_ab, attr=None):
    nd = 2 + len(sp)
    s = md((mb, ic) + tuple(sp), dt, PLAIN[nd] if stag is None else stag)
    dw = md((oc, ic) + tuple(sp), wdt or dt, PLAIN[nd] if wtag is None else wtag)
    dd = md((mb, oc), dt, dtag)
    db = md((oc,), bdt, dnnl.tag_a) if bdt else None
    return dnnl.inner_product_backward_weights_primitive_desc(eng, s, dw, dd, diff_bias_md=db, attr=attr)


def test_queries_describe_the_backward_passes(eng):
    pd = bwd_d(eng, 4, 14, (5, 5), 25)
    assert pd.query_s32(dnnl.query_primitive_kind) == dnnl.kind_inner_product
    assert pd.query_s32(dnnl.query_prop_kind) == dnnl.backward_data
    assert pd.query_md(dnnl.query_diff_src_md).dims() == [4, 14, 5, 5]
    assert pd.query_md(dnnl.query_weights_md).dims() == [25, 14, 5, 5]
    assert pd.query_md(dnnl.query_diff_dst_md).dims() == [4, 25]
    d = pd.lowered_desc()                                            # [mb, oc] x [oc, K]
    assert (d.batch, d.M, d.N, d.K) == (1, 4, 350, 25)
    assert tuple(d.src_stride)[1:] == (25, 1) and tuple(d.wei_stride)[1:] == (350, 1)
    assert tuple(d.dst_stride)[1:] == (350, 1)

    pd = bwd_w(eng, 4, 14, (5, 5), 25, bdt="f32")
    assert pd.query_s32(dnnl.query_prop_kind) == dnnl.backward_weights
    assert pd.query_md(dnnl.query_src_md).dims() == [4, 14, 5, 5]
    assert pd.query_md(dnnl.query_diff_weights_md).dims() == [25, 14, 5, 5]
    assert pd.query_md(dnnl.query_diff_weights_md, 1).dims() == [25]
    assert pd.query_md(dnnl.query_diff_dst_md).dims() == [4, 25]
    d = pd.lowered_desc()                                            # [oc, mb] x [mb, K]: diff_dst read transposed
    assert (d.batch, d.M, d.N, d.K) == (1, 25, 350, 4)
    assert tuple(d.src_stride)[1:] == (1, 25) and tuple(d.wei_stride)[1:] == (350, 1)
    assert d.bias_dt == cabi.DT_UNDEF                                # diff_bias is a reduction of its own


def test_backward_any_takes_the_other_tensors_order(eng):
    pd = bwd_d(eng, 2, 8, (3, 5), 6, stag=dnnl.tag_any, wtag=dnnl.tag_ohwi, dtag=dnnl.tag_any)
    assert pd.query_md(dnnl.query_diff_src_md).strides() == [120, 1, 40, 8]
    assert pd.query_md(dnnl.query_diff_dst_md).strides() == [6, 1]
    pd = bwd_w(eng, 2, 8, (3, 5), 6, stag=dnnl.tag_nhwc, wtag=dnnl.tag_any)
    assert pd.query_md(dnnl.query_diff_weights_md).strides() == [120, 1, 40, 8]
    pd = bwd_d(eng, 2, 8, (3, 5), 6, stag=dnnl.tag_any, wtag=dnnl.tag_any)
    assert pd.query_md(dnnl.query_diff_src_md).strides() == [120, 15, 5, 1]
    assert pd.query_md(dnnl.query_weights_md).strides() == [120, 15, 5, 1]
    # different orders of the flattened dims have no common walk
    assert status_of(lambda: bwd_d(eng, 2, 8, (3, 5), 6, stag=dnnl.tag_nchw, wtag=dnnl.tag_ohwi)) == dnnl.unimplemented


def test_backward_shape_and_type_rules(eng):
    lib = dnnl.lib()
    h = C.c_void_p()
    s, w, d = md((2, 8), "f32", dnnl.tag_ab), md((6, 8), "f32", dnnl.tag_ab), md((2, 6), "f32", dnnl.tag_ab)
    bad = md((3, 6), "f32", dnnl.tag_ab)
    assert lib.dnnl_inner_product_backward_data_primitive_desc_create(
        C.byref(h), eng.h, s.h, w.h, bad.h, None, None) == dnnl.invalid_arguments
    assert lib.dnnl_inner_product_backward_weights_primitive_desc_create(
        C.byref(h), eng.h, s.h, w.h, None, bad.h, None, None) == dnnl.invalid_arguments
    assert lib.dnnl_inner_product_backward_weights_primitive_desc_create(
        C.byref(h), eng.h, s.h, w.h, md((5,), "f32", dnnl.tag_a).h, d.h, None, None) == dnnl.invalid_arguments
    assert lib.dnnl_inner_product_backward_data_primitive_desc_create(
        None, eng.h, s.h, w.h, d.h, None, None) == dnnl.invalid_arguments
    un = dnnl.unimplemented
    # ref_inner_product.hpp:118-139: diff_src is f32 or the weights' type; diff_dst has the weights' type
    for dt in ("f32", "bf16", "f16"):
        bwd_d(eng, 2, 8, (), 6, dt=dt)
        bwd_d(eng, 2, 8, (), 6, dt=dt, sdt="f32")
        bwd_w(eng, 2, 8, (), 6, dt=dt, bdt=dt)
        bwd_w(eng, 2, 8, (), 6, dt=dt, wdt="f32", bdt="f32")
    assert status_of(lambda: bwd_d(eng, 2, 8, (), 6, dt="s8")) == un
    assert status_of(lambda: bwd_d(eng, 2, 8, (), 6, dt="f32", sdt="bf16")) == un
    assert status_of(lambda: bwd_w(eng, 2, 8, (), 6, dt="bf16", wdt="f16")) == un
    assert status_of(lambda: bwd_w(eng, 2, 8, (), 6, dt="f8_e4m3")) == un
    # no attributes on the backward passes
    a = dnnl.primitive_attr()
    a.set_scales_mask(dnnl.ARG_WEIGHTS, 0)
    assert status_of(lambda: bwd_d(eng, 2, 8, (), 6, attr=a)) == un
    bwd_d(eng, 2, 8, (), 6, attr=dnnl.primitive_attr())
    # an empty batch is a valid problem (tests/gtests/test_inner_product_backward_data.cpp:131-136)
    bwd_d(eng, 0, 8, (3, 3), 6)
    bwd_w(eng, 0, 8, (3, 3), 6, bdt="f32")


def test_backward_problems_run_on_the_matrix_cores(eng):
    pd = bwd_d(eng, 128, 2048, (), 1000, dt="bf16")
    assert pd.impl_info_str().startswith("hip:mfma_h16")
    pd = bwd_w(eng, 128, 2048, (), 1000, dt="bf16", wdt="f32", bdt="f32")
    assert pd.impl_info_str().startswith("hip:mfma_h16")


# ------------------------------------------------------------------ execution on the device
def storage(view):
    order = np.argsort([-s for s in view.strides], kind="stable")
    return np.ascontiguousarray(view.transpose(order))


def run_bwd_data(dd, wei, sp, dts, channels_last):
    """(diff_src as a logical-shape array of raw storage, implementation name)"""
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    mb, oc = dd.shape
    ic = wei.shape[1]
    nd = wei.ndim
    tags = CHANNELS_LAST if channels_last else PLAIN
    ds_md = md((mb, ic) + tuple(sp), dts[0], tags[nd])
    w_md = md(wei.shape, dts[1], tags[nd])
    dd_md = md((mb, oc), dts[2], dnnl.tag_ab)
    pd = dnnl.inner_product_backward_data_primitive_desc(eng, ds_md, w_md, dd_md)
    prim = dnnl.inner_product_backward_data(pd)
    order = order_of(channels_last, nd)
    shape = (mb, ic) + tuple(sp)
    init = np.full([shape[i] for i in order], 0x55, np.uint8).repeat(np.dtype(storage_dtype(DT[dts[0]])).itemsize, -1)
    init = init.view(storage_dtype(DT[dts[0]]))
    out = dnnl.memory(ds_md, eng, init)
    prim.execute(strm, {dnnl.ARG_DIFF_DST: dnnl.memory(dd_md, eng, storage(dd)),
                        dnnl.ARG_WEIGHTS: dnnl.memory(w_md, eng, storage(wei)), dnnl.ARG_DIFF_SRC: out})
    strm.wait()
    raw = out.read(storage_dtype(DT[dts[0]])).reshape([shape[i] for i in order])
    return raw.transpose(np.argsort(order)), pd.impl_info_str()


def run_bwd_weights(dd, src, sp, dts, channels_last, with_bias=True):
    """(diff_weights, diff_bias, implementation name)"""
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    mb, oc = dd.shape
    ic = src.shape[1]
    nd = src.ndim
    tags = CHANNELS_LAST if channels_last else PLAIN
    s_md = md(src.shape, dts[0], tags[nd])
    dw_md = md((oc, ic) + tuple(sp), dts[1], tags[nd])
    db_md = md((oc,), dts[2], dnnl.tag_a) if with_bias else None
    dd_md = md((mb, oc), dts[3], dnnl.tag_ab)
    pd = dnnl.inner_product_backward_weights_primitive_desc(eng, s_md, dw_md, dd_md, diff_bias_md=db_md)
    prim = dnnl.inner_product_backward_weights(pd)
    order = order_of(channels_last, nd)
    shape = (oc, ic) + tuple(sp)
    wdt, bdt = storage_dtype(DT[dts[1]]), storage_dtype(DT[dts[2]])
    out = dnnl.memory(dw_md, eng, np.zeros([shape[i] for i in order], wdt))
    args = {dnnl.ARG_DIFF_DST: dnnl.memory(dd_md, eng, storage(dd)), dnnl.ARG_SRC: dnnl.memory(s_md, eng, storage(src)),
            dnnl.ARG_DIFF_WEIGHTS: out}
    if with_bias:
        bias = dnnl.memory(db_md, eng, np.zeros(oc, bdt))
        args[dnnl.ARG_DIFF_BIAS] = bias
    prim.execute(strm, args)
    strm.wait()
    raw = out.read(wdt).reshape([shape[i] for i in order])
    return raw.transpose(np.argsort(order)), bias.read(bdt) if with_bias else None, pd.impl_info_str()


GPU_SHAPES = SHAPES + [(64, 128, (), 256), (33, 64, (2, 2), 130), (256, 512, (), 384)]
TYPES_D = [("f32", "f32"), ("bf16", "bf16"), ("f32", "bf16"), ("f16", "f16"), ("f32", "f16")]   # (diff_src, others)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", GPU_SHAPES)
@pytest.mark.parametrize("channels_last", [False, True])
@pytest.mark.parametrize("odt,dt", TYPES_D)
def test_gpu_backward_data_exact_data(gpu, oracle, shape, channels_last, odt, dt):
    mb, ic, sp, oc = shape
    dd, wei = small_float_data(11, (mb, oc), dt), small_float_data(12, (oc, ic) + sp, dt)
    wv = as_layout(wei, channels_last)
    got, impl = run_bwd_data(dd, wv, sp, (odt, dt, dt), channels_last)
    want = oracle.run_oracle_inner_product_bwd_data(dd, wv, (mb, ic) + sp, (odt, dt, dt),
                                                    order_of(channels_last, wei.ndim))
    assert np.array_equal(np.ascontiguousarray(got), np.ascontiguousarray(want)), impl


@pytest.mark.gpu
@pytest.mark.parametrize("shape", GPU_SHAPES)
@pytest.mark.parametrize("channels_last", [False, True])
@pytest.mark.parametrize("odt,dt", TYPES_D)
def test_gpu_backward_weights_exact_data(gpu, oracle, shape, channels_last, odt, dt):
    mb, ic, sp, oc = shape
    dd, src = small_float_data(13, (mb, oc), dt), small_float_data(14, (mb, ic) + sp, dt)
    sv = as_layout(src, channels_last)
    got, bias, impl = run_bwd_weights(dd, sv, sp, (dt, odt, odt, dt), channels_last)
    want, wbias = oracle.run_oracle_inner_product_bwd_weights(dd, sv, (dt, odt, odt, dt), True,
                                                              order_of(channels_last, src.ndim))
    assert np.array_equal(np.ascontiguousarray(got), np.ascontiguousarray(want)), impl
    assert np.array_equal(bias, wbias), impl


@pytest.mark.gpu
@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
def test_gpu_backward_random_data_within_bound(gpu, oracle, dt):
    mb, ic, sp, oc = 48, 32, (3, 3), 80
    r = np.random.default_rng(61)
    dd = encode(r.standard_normal((mb, oc)).astype(np.float32), dt)
    wei = encode(r.standard_normal((oc, ic) + sp).astype(np.float32), dt)
    src = encode(r.standard_normal((mb, ic) + sp).astype(np.float32), dt)
    d64, w64, s64 = values(dt, dd), values(dt, wei), values(dt, src)

    got, impl = run_bwd_data(dd, wei, sp, ("f32", dt, dt), False)
    exact = np.tensordot(d64, w64, axes=([1], [0]))
    bound = gemm_bound(oc, np.tensordot(np.abs(d64), np.abs(w64), axes=([1], [0])))
    assert (np.abs(got.astype(np.float64) - exact) <= bound).all(), impl
    assert np.abs(got.astype(np.float64) - exact).max() > 0 or dt != "f32"

    got, bias, impl = run_bwd_weights(dd, src, sp, (dt, "f32", "f32", dt), False)
    exact = np.tensordot(d64, s64, axes=([0], [0]))
    bound = gemm_bound(mb, np.tensordot(np.abs(d64), np.abs(s64), axes=([0], [0])))
    assert (np.abs(got.astype(np.float64) - exact) <= bound).all(), impl
    # diff_bias: the same additions in the same order as the reference's loop
    _, wbias = oracle.run_oracle_inner_product_bwd_weights(dd, src, (dt, "f32", "f32", dt), True)
    assert np.array_equal(bias, wbias)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_gpu_diff_bias_in_the_narrow_type_rounds_the_f32_sum_once(gpu, oracle, dt):
    mb, ic, oc = 200, 16, 70
    r = np.random.default_rng(62)
    dd = encode(r.standard_normal((mb, oc)).astype(np.float32), dt)
    src = small_float_data(63, (mb, ic), dt)
    _, bias, _ = run_bwd_weights(dd, src, (), (dt, dt, dt, dt), False)
    _, wbias = oracle.run_oracle_inner_product_bwd_weights(dd, src, (dt, dt, dt, dt), True)
    assert np.array_equal(bias, wbias)


@pytest.mark.gpu
def test_gpu_backward_weights_without_diff_bias_and_empty_batch(gpu, oracle):
    dd, src = small_float_data(64, (8, 24), "f32"), small_float_data(65, (8, 40), "f32")
    got, bias, _ = run_bwd_weights(dd, src, (), ("f32",) * 4, False, with_bias=False)
    want, _ = oracle.run_oracle_inner_product_bwd_weights(dd, src, ("f32",) * 4, False)
    assert bias is None and np.array_equal(got, want)
    # mb = 0: the sums are empty, the outputs are zeros (the memory starts as 0x55 bytes)
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    s_md, dw_md, db_md, dd_md = md((0, 40), "f32", dnnl.tag_ab), md((24, 40), "f32", dnnl.tag_ab), \
        md((24,), "f32", dnnl.tag_a), md((0, 24), "f32", dnnl.tag_ab)
    pd = dnnl.inner_product_backward_weights_primitive_desc(eng, s_md, dw_md, dd_md, diff_bias_md=db_md)
    dw = dnnl.memory(dw_md, eng, np.full(24 * 40, 0x55555555, np.uint32).view(np.float32))
    db = dnnl.memory(db_md, eng, np.full(24, 0x55555555, np.uint32))
    dnnl.inner_product_backward_weights(pd).execute(strm, {
        dnnl.ARG_DIFF_DST: dnnl.memory(dd_md, eng), dnnl.ARG_SRC: dnnl.memory(s_md, eng), dnnl.ARG_DIFF_WEIGHTS: dw,
        dnnl.ARG_DIFF_BIAS: db})
    strm.wait()
    assert not dw.read(np.uint32).any() and not db.read(np.uint32).any()
