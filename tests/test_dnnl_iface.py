"""Interface tests of the dnnl_* C API subset (libdnnl_amd.so) that need no
GPU: a descriptor-only engine (ONEDNN_AMD_ALLOW_NO_DEVICE=1) creates and
queries primitive descriptors.  Modelled on the reference's interface tests
(tests/gtests/test_matmul.cpp:392-680, test_iface_attr_quantization.cpp) and on
the conditions of matmul_desc_init / matmul_attr_check
(src/common/matmul.cpp:261-744): status codes, not numerics."""
import ctypes as C
import os
import re

import pytest

os.environ["ONEDNN_AMD_ALLOW_NO_DEVICE"] = "1"

from onednn_amd import cabi, dnnl  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DT = cabi.DT_NAMES


@pytest.fixture(scope="module")
def eng():
    return dnnl.engine(dnnl.gpu, 0)


def md(dims, dt, tag=None, strides=None):
    if tag is None and strides is None:
        tag = {1: dnnl.tag_a, 2: dnnl.tag_ab, 3: dnnl.tag_abc, 4: dnnl.tag_abcd}[len(dims)]
    return dnnl.memory_desc(dims, DT[dt], tag=tag, strides=strides)


def make_pd(eng, M, K, N, sdt, wdt, ddt, attr=None, bias=None, wtag=dnnl.tag_ab):
    return dnnl.matmul_primitive_desc(eng, md([M, K], sdt), md([K, N], wdt, tag=wtag), md([M, N], ddt),
                                      bias_md=bias, attr=attr)


def status_of(fn):
    try:
        fn()
        return dnnl.success
    except dnnl.error as e:
        return e.status


def test_every_declared_symbol_is_exported():
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "dnnl_amd.h")).read(), flags=re.S)
    names = sorted(set(re.findall(r"\b(dnnl_[a-z0-9_]+)\s*\(", text)))
    assert len(names) >= 55
    lib = dnnl.lib()
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/dnnl_amd.h but not exported"


def test_engine_kinds(eng):
    assert eng.get_kind() == dnnl.gpu
    assert status_of(lambda: dnnl.engine(dnnl.cpu, 0)) == dnnl.invalid_arguments   # no CPU engine here


def test_memory_desc_queries():
    m = md([3, 5, 7], "bf16")
    assert m.ndims() == 3 and m.dims() == [3, 5, 7] and m.strides() == [35, 7, 1]
    assert m.data_type() == DT["bf16"] and m.get_size() == 3 * 5 * 7 * 2
    t = md([4, 6], "s8", tag=dnnl.tag_ba)
    assert t.strides() == [1, 4]
    s = md([4, 6], "f32", strides=[16, 2])
    assert s.get_size() == ((3 * 16 + 5 * 2) + 1) * 4
    n4 = md([4, 6], "u4")
    assert n4.get_size() == 12                      # two nibbles per byte
    assert status_of(lambda: md([4, 6], "u4", strides=[12, 2])) == dnnl.invalid_arguments
    assert status_of(lambda: dnnl.memory_desc([2, 2], 99, tag=dnnl.tag_ab)) == dnnl.invalid_arguments
    assert status_of(lambda: dnnl.memory_desc([2, 2], DT["f32"], tag=dnnl.tag_abc)) == dnnl.invalid_arguments


def test_shape_rules(eng):
    # matmul_desc_init: M, N, K consistency and broadcast rules -> invalid_arguments
    ok = lambda: dnnl.matmul_primitive_desc(eng, md([8, 16], "f32"), md([16, 4], "f32"), md([8, 4], "f32"))
    assert status_of(ok) == dnnl.success
    bad_k = lambda: dnnl.matmul_primitive_desc(eng, md([8, 16], "f32"), md([15, 4], "f32"), md([8, 4], "f32"))
    bad_m = lambda: dnnl.matmul_primitive_desc(eng, md([8, 16], "f32"), md([16, 4], "f32"), md([7, 4], "f32"))
    bad_nd = lambda: dnnl.matmul_primitive_desc(eng, md([8, 16], "f32"), md([1, 16, 4], "f32"), md([8, 4], "f32"))
    for f in (bad_k, bad_m, bad_nd):
        assert status_of(f) == dnnl.invalid_arguments
    # batch broadcast: 3x1 batch dims
    bc = lambda: dnnl.matmul_primitive_desc(eng, md([3, 8, 16], "f32"), md([1, 16, 4], "f32"), md([3, 8, 4], "f32"))
    assert status_of(bc) == dnnl.success
    bad_bc = lambda: dnnl.matmul_primitive_desc(eng, md([3, 8, 16], "f32"), md([2, 16, 4], "f32"), md([3, 8, 4], "f32"))
    assert status_of(bad_bc) == dnnl.invalid_arguments
    # bias must broadcast onto dst and have dst's ndims
    b_ok = lambda: make_pd(eng, 8, 16, 4, "f32", "f32", "f32", bias=md([1, 4], "f32"))
    b_bad = lambda: make_pd(eng, 8, 16, 4, "f32", "f32", "f32", bias=md([1, 3], "f32"))
    b_nd = lambda: make_pd(eng, 8, 16, 4, "f32", "f32", "f32", bias=md([4], "f32"))
    assert status_of(b_ok) == dnnl.success
    assert status_of(b_bad) == dnnl.invalid_arguments and status_of(b_nd) == dnnl.invalid_arguments


def test_attribute_setters_validate():
    a = dnnl.primitive_attr()
    # primitive_attr.cpp:637-716
    assert status_of(lambda: a.set_scales(dnnl.ARG_SRC, 0, dt=DT["s8"])) == dnnl.invalid_arguments
    assert status_of(lambda: a.set_scales(dnnl.ARG_SRC, 0, dt=DT["e8m0"])) == dnnl.invalid_arguments   # needs a mask
    assert status_of(lambda: a.set_scales(dnnl.ARG_WEIGHTS, 3, (32,), DT["f32"])) == dnnl.invalid_arguments  # 0 or 2 group dims
    assert status_of(lambda: a.set_zero_points(dnnl.ARG_WEIGHTS, 0, dt=DT["u4"])) == dnnl.invalid_arguments
    assert status_of(lambda: a.set_zero_points(dnnl.ARG_DST, 2, dt=DT["s8"])) == dnnl.invalid_arguments
    assert status_of(lambda: a.set_zero_points(dnnl.ARG_SRC, -1)) == dnnl.invalid_arguments
    assert status_of(lambda: a.set_scales(dnnl.ARG_WEIGHTS, 3, (128, 1), DT["bf16"])) == dnnl.success
    po = dnnl.post_ops()
    assert status_of(lambda: po.append_eltwise(cabi.ELTWISE["clip"], 2.0, 1.0)) == dnnl.invalid_arguments
    assert status_of(lambda: po.append_eltwise(0x7777)) == dnnl.invalid_arguments
    po.append_eltwise(cabi.ELTWISE["relu"])
    po.append_sum(1.0)
    assert po.len() == 2 and po.kind(0) == dnnl.kind_eltwise and po.kind(1) == dnnl.kind_sum


# (description, src, wei, dst, attr builder, expected status): rows follow matmul_attr_check
def _attr(build):
    a = dnnl.primitive_attr()
    build(a)
    return a


ATTR_CASES = [
    ("src scale common", "u8", "s8", "f32", lambda a: a.set_scales_mask(dnnl.ARG_SRC, 0), dnnl.success),
    ("src scale per-M", "u8", "s8", "f32", lambda a: a.set_scales_mask(dnnl.ARG_SRC, 1), dnnl.success),
    ("src scale per-K without groups", "u8", "s8", "f32", lambda a: a.set_scales_mask(dnnl.ARG_SRC, 2), dnnl.unimplemented),
    ("wei scale per-N", "u8", "s8", "f32", lambda a: a.set_scales_mask(dnnl.ARG_WEIGHTS, 2), dnnl.success),
    ("wei scale K mask on int8 x int8 is decompression-only... allowed for int src", "u8", "s8", "f32",
     lambda a: a.set_scales(dnnl.ARG_WEIGHTS, 3, (32, 1)), dnnl.success),
    ("wei scale K groups not multiple of 16", "u8", "s8", "f32",
     lambda a: a.set_scales(dnnl.ARG_WEIGHTS, 3, (8, 1)), dnnl.unimplemented),
    ("wei scale K mask on bf16 src without apply_to_int", "bf16", "u4", "bf16",
     lambda a: a.set_scales(dnnl.ARG_WEIGHTS, 3, (32, 1), DT["bf16"]), dnnl.unimplemented),
    ("decompression with K-grouped scales and u4 zero points", "bf16", "u4", "bf16",
     lambda a: (a.set_fpmath_mode(dnnl.fpmath_bf16, True), a.set_scales(dnnl.ARG_WEIGHTS, 3, (32, 1), DT["bf16"]),
                a.set_zero_points(dnnl.ARG_WEIGHTS, 3, (32, 1), DT["u4"])), dnnl.success),
    ("wei zp N-groups need apply_to_int", "u8", "s8", "f32",
     lambda a: a.set_zero_points(dnnl.ARG_WEIGHTS, 2, (1, 16), DT["s8"]), dnnl.unimplemented),
    ("src zp per-K groups multiple of 32", "u8", "s8", "f32",
     lambda a: a.set_zero_points(dnnl.ARG_SRC, 3, (1, 32)), dnnl.success),
    ("src zp K group 16 rejected", "u8", "s8", "f32",
     lambda a: a.set_zero_points(dnnl.ARG_SRC, 3, (1, 16)), dnnl.unimplemented),
    ("src zp per-M only rejected", "u8", "s8", "f32", lambda a: a.set_zero_points_mask(dnnl.ARG_SRC, 1), dnnl.unimplemented),
    ("zero points on f32 src", "f32", "f32", "f32", lambda a: a.set_zero_points_mask(dnnl.ARG_SRC, 0), dnnl.unimplemented),
    ("dst zp per-N", "u8", "s8", "u8", lambda a: a.set_zero_points_mask(dnnl.ARG_DST, 2), dnnl.success),
    ("dst zp per-M rejected", "u8", "s8", "u8", lambda a: a.set_zero_points_mask(dnnl.ARG_DST, 1), dnnl.unimplemented),
    ("precomputed reductions need weights zero points", "u8", "s8", "f32",
     lambda a: a.set_precomputed_reductions(dnnl.ARG_SRC, 3, (1, 32)), dnnl.unimplemented),
    ("precomputed reductions with weights zero points", "u8", "s8", "f32",
     lambda a: (a.set_zero_points(dnnl.ARG_WEIGHTS, 3, (32, 1), DT["s8"]),
                a.set_precomputed_reductions(dnnl.ARG_SRC, 3, (1, 32))), dnnl.success),
    ("mx scales on f4", "f4_e2m1", "f4_e2m1", "bf16",
     lambda a: (a.set_scales(dnnl.ARG_SRC, 3, (1, 32), DT["e8m0"]), a.set_scales(dnnl.ARG_WEIGHTS, 3, (32, 1), DT["e8m0"])),
     dnnl.success),
    ("scale on an argument matmul does not have", "u8", "s8", "f32", lambda a: a.set_scales_mask(dnnl.ARG_BIAS, 0),
     dnnl.unimplemented),
]


@pytest.mark.parametrize("case", ATTR_CASES, ids=[c[0] for c in ATTR_CASES])
def test_attribute_legality(eng, case):
    _, s, w, d, build, want = case
    a = _attr(build)
    got = status_of(lambda: make_pd(eng, 64, 128, 64, s, w, d, attr=a))
    assert got == want


def test_unsupported_data_type_mixes(eng):
    assert status_of(lambda: make_pd(eng, 16, 32, 16, "bf16", "u4", "bf16")) == dnnl.unimplemented   # no apply_to_int
    assert status_of(lambda: make_pd(eng, 16, 32, 16, "u8", "f32", "f32")) == dnnl.unimplemented
    assert status_of(lambda: make_pd(eng, 16, 32, 16, "f32", "f32", "s32")) == dnnl.unimplemented
    assert status_of(lambda: make_pd(eng, 16, 32, 16, "f32", "f32", "f32")) == dnnl.success
    assert status_of(lambda: make_pd(eng, 16, 32, 16, "u8", "s8", "f4_e2m1")) == dnnl.unimplemented


def test_implementation_list_and_next_impl(eng):
    a = dnnl.primitive_attr()
    a.set_scales_mask(dnnl.ARG_SRC, 0)
    a.set_scales_mask(dnnl.ARG_WEIGHTS, 2)
    a.set_zero_points_mask(dnnl.ARG_SRC, 0)
    pd = make_pd(eng, 256, 1024, 1024, "u8", "s8", "f32", attr=a, bias=md([1, 1024], "f32"))
    assert pd.impl_info_str().startswith("hip:mfma_i8")
    assert pd.next_impl() and pd.impl_info_str() == "hip:ref:any"
    assert not pd.next_impl()                                  # last_impl_reached
    # K not a multiple of the tile: only the generic kernel applies
    pd = make_pd(eng, 256, 1000, 1024, "u8", "s8", "f32", attr=a)
    assert pd.impl_info_str() == "hip:ref:any"
    # fp8, mxfp4 and int4 decode pick their kernel families
    assert make_pd(eng, 128, 256, 128, "f8_e4m3", "f8_e4m3", "bf16").impl_info_str().startswith("hip:mfma_f8")
    mx = _attr(lambda t: (t.set_scales(dnnl.ARG_SRC, 3, (1, 32), DT["e8m0"]), t.set_scales(dnnl.ARG_WEIGHTS, 3, (32, 1), DT["e8m0"])))
    assert make_pd(eng, 128, 256, 128, "f4_e2m1", "f4_e2m1", "bf16", attr=mx, wtag=dnnl.tag_ba).impl_info_str().startswith("hip:mfma_mxf4")
    wo = _attr(lambda t: (t.set_fpmath_mode(dnnl.fpmath_bf16, True), t.set_scales(dnnl.ARG_WEIGHTS, 3, (128, 1), DT["bf16"]),
                          t.set_zero_points(dnnl.ARG_WEIGHTS, 3, (128, 1), DT["u4"])))
    assert make_pd(eng, 8, 4096, 14336, "bf16", "u4", "bf16", attr=wo).impl_info_str().startswith("hip:woq_gemv")


def test_format_any_is_resolved_by_the_implementation(eng):
    # src / dst: plain row-major (matmul_pd.hpp:419-431); weights: the layout the
    # kernels consume, to be read back through weights_desc() like a blocked
    # layout of the reference -- K-contiguous for the MFMA operand types ...
    pd = dnnl.matmul_primitive_desc(eng, md([8, 16], "s8", tag=dnnl.tag_any), md([16, 4], "s8", tag=dnnl.tag_any),
                                    md([8, 4], "s32", tag=dnnl.tag_any))
    assert pd.query_md(dnnl.query_src_md).strides() == [16, 1]
    assert pd.query_md(dnnl.query_weights_md).strides() == [1, 16]
    assert pd.query_md(dnnl.query_dst_md).strides() == [4, 1]
    pd = dnnl.matmul_primitive_desc(eng, md([2, 8, 128], "f8_e4m3"), md([2, 128, 4], "f8_e4m3", tag=dnnl.tag_any),
                                    md([2, 8, 4], "bf16"))
    assert pd.query_md(dnnl.query_weights_md).strides() == [512, 1, 128]
    # ... for the unquantized float types of the same tiles too ...
    for dt in ("f32", "bf16", "f16"):
        pd = dnnl.matmul_primitive_desc(eng, md([8, 16], dt), md([16, 4], dt, tag=dnnl.tag_any), md([8, 4], dt))
        assert pd.query_md(dnnl.query_weights_md).strides() == [1, 16]
    # ... and row-major for everything else (here: 8-bit weights that a bf16 src decompresses)
    wo = _attr(lambda t: t.set_fpmath_mode(dnnl.fpmath_bf16, True))
    pd = dnnl.matmul_primitive_desc(eng, md([8, 16], "bf16"), md([16, 4], "s8", tag=dnnl.tag_any), md([8, 4], "bf16"),
                                    attr=wo)
    assert pd.query_md(dnnl.query_weights_md).strides() == [4, 1]


def test_format_any_decode_weights_resolve_to_the_packed_layout(eng):
    # 4-bit weights of a decode problem wide enough to fill the device: an
    # opaque descriptor (no strides), dense size, written by a reorder from
    # plain weights of the same type -- the role of a blocked weights layout
    # in the reference (brgemm_matmul_utils.cpp:203-330)
    wo = _attr(lambda t: (t.set_fpmath_mode(dnnl.fpmath_bf16, True), t.set_scales(dnnl.ARG_WEIGHTS, 3, (128, 1), DT["bf16"]),
                          t.set_zero_points(dnnl.ARG_WEIGHTS, 3, (128, 1), DT["u4"])))
    K, N = 4096, 14336
    pd = make_pd(eng, 8, K, N, "bf16", "u4", "bf16", attr=wo, wtag=dnnl.tag_any)
    assert pd.impl_info_str().startswith("hip:woq_packed")
    wmd = pd.query_md(dnnl.query_weights_md)
    assert wmd.format_kind() == dnnl.format_kind_opaque and wmd.get_size() == K * N // 2 and wmd.dims() == [K, N]
    assert status_of(lambda: wmd.strides()) == dnnl.invalid_arguments
    assert pd.next_impl() and pd.impl_info_str() == "hip:ref:any"       # the generic kernel reads the layout too
    # a primitive descriptor built on the queried descriptor is the same problem
    pd2 = dnnl.matmul_primitive_desc(eng, md([8, K], "bf16"), wmd, md([8, N], "bf16"), attr=wo)
    assert pd2.impl_info_str().startswith("hip:woq_packed")
    # the reorder into it: same data type, no attributes
    plain = md([K, N], "u4")
    assert dnnl.reorder_primitive_desc(eng, plain, eng, wmd).impl_info_str() == "hip:reorder:any"
    assert dnnl.reorder_primitive_desc(eng, md([K, N], "u4", tag=dnnl.tag_ba), eng, wmd).impl_info_str() == "hip:reorder:any"
    assert status_of(lambda: dnnl.reorder_primitive_desc(eng, md([K, N], "f32"), eng, wmd)) == dnnl.unimplemented
    assert status_of(lambda: dnnl.reorder_primitive_desc(eng, wmd, eng, plain)) == dnnl.unimplemented
    ra = dnnl.primitive_attr()
    ra.set_scales(dnnl.ARG_DST, 2)
    assert status_of(lambda: dnnl.reorder_primitive_desc(eng, plain, eng, wmd, attr=ra)) == dnnl.unimplemented
    # narrow N, more rows than a decode, or a group size the packed kernel does not take: plain row-major
    assert make_pd(eng, 8, K, 4096, "bf16", "u4", "bf16", attr=wo, wtag=dnnl.tag_any).query_md(dnnl.query_weights_md).strides() == [4096, 1]
    assert make_pd(eng, 64, K, N, "bf16", "u4", "bf16", attr=wo, wtag=dnnl.tag_any).query_md(dnnl.query_weights_md).strides() == [N, 1]
    odd = _attr(lambda t: (t.set_fpmath_mode(dnnl.fpmath_bf16, True), t.set_scales(dnnl.ARG_WEIGHTS, 3, (96, 1), DT["bf16"])))
    assert make_pd(eng, 8, 960, N, "bf16", "u4", "bf16", attr=odd, wtag=dnnl.tag_any).query_md(dnnl.query_weights_md).strides() == [N, 1]
    # explicit row-major weights keep the plain decode kernel
    assert make_pd(eng, 8, K, N, "bf16", "u4", "bf16", attr=wo).impl_info_str().startswith("hip:woq_gemv")


def test_dynamic_mx_dst_scales_rules(eng):
    # dnnl_primitive_attr_set_scales_v3 (primitive_attr.cpp:637-669) and the matmul rules for
    # quantization_mode::dynamic_mx (matmul.cpp:407-424): full mask, groups 1 x 32, e8m0
    def mx(mask=3, groups=(1, 32), dt=DT["e8m0"], arg=dnnl.ARG_DST):
        return _attr(lambda t: t.set_scales(arg, mask, groups, dt, qmode=dnnl.quantization_mode_dynamic_mx))
    pd = make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "f8_e4m3", attr=mx())
    assert pd.impl_info_str().startswith("hip:mfma_f8")
    assert pd.next_impl() and pd.impl_info_str() == "hip:ref:any"
    assert status_of(lambda: make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "f8_e5m2", attr=mx())) == dnnl.success
    assert status_of(lambda: make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "f8_e4m3", attr=mx(groups=(1, 16)))) == dnnl.unimplemented
    assert status_of(lambda: make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "f8_e4m3", attr=mx(mask=2))) == dnnl.unimplemented
    assert status_of(lambda: make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "f8_e4m3", attr=mx(dt=DT["f32"]))) == dnnl.unimplemented
    assert status_of(lambda: make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "bf16", attr=mx())) == dnnl.unimplemented
    assert status_of(lambda: make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "f8_e4m3", attr=mx(arg=dnnl.ARG_SRC, groups=(1, 32)))) == dnnl.unimplemented
    a = dnnl.primitive_attr()
    assert status_of(lambda: a.set_scales(dnnl.ARG_DST, 3, (1, 32), DT["e8m0"], qmode=7)) == dnnl.invalid_arguments
    # quantization_mode::dynamic_fp (matmul.cpp:423-440): the NVFP4 flavour, f8_e4m3 scales per 1 x 16
    def fp(mask=3, groups=(1, 16), dt=DT["f8_e4m3"]):
        return _attr(lambda t: t.set_scales(dnnl.ARG_DST, mask, groups, dt, qmode=dnnl.quantization_mode_dynamic_fp))
    for dst in ("f4_e2m1", "f8_e4m3"):
        pd = make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", dst, attr=fp())
        assert pd.impl_info_str().startswith("hip:mfma_f8")
        assert pd.next_impl() and pd.impl_info_str() == "hip:ref:any"
    assert make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "f4_e2m1", attr=mx()).impl_info_str().startswith("hip:mfma_f8")
    assert status_of(lambda: make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "f4_e2m1", attr=fp(groups=(1, 32)))) == dnnl.unimplemented
    assert status_of(lambda: make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "f4_e2m1", attr=fp(dt=DT["e8m0"]))) == dnnl.unimplemented
    assert status_of(lambda: make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "f4_e2m1", attr=fp(mask=2, groups=()))) == dnnl.unimplemented
    assert status_of(lambda: make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "bf16", attr=fp())) == dnnl.unimplemented
    # a 4-bit dst without dynamic scales: the tiles too (groups of four columns are whole bytes here), else generic
    assert make_pd(eng, 64, 128, 256, "f8_e4m3", "f8_e4m3", "f4_e2m1").impl_info_str().startswith("hip:mfma_f8")
    assert make_pd(eng, 64, 128, 254, "f8_e4m3", "f8_e4m3", "f4_e2m1").impl_info_str() == "hip:ref:any"
    assert status_of(lambda: a.set_scales(dnnl.ARG_DST, 1, (), DT["f32"], is_on_host=1)) == dnnl.invalid_arguments
    assert status_of(lambda: a.set_scales(dnnl.ARG_DST, 0, (), DT["f32"], is_on_host=1)) == dnnl.success


def test_user_scratchpad_is_reported(eng):
    a = dnnl.primitive_attr()
    a.set_scratchpad_mode(dnnl.scratchpad_user)
    a.set_zero_points_mask(dnnl.ARG_SRC, 0)
    pd = make_pd(eng, 256, 1024, 1024, "u8", "s8", "s32", attr=a)     # `ab` weights: layout pre-pass + column sums
    sp = pd.scratchpad_desc()
    assert sp.ndims() == 1 and sp.dims()[0] >= 1024 * 1024
    lib_mode = make_pd(eng, 256, 1024, 1024, "u8", "s8", "s32")
    assert lib_mode.scratchpad_desc().ndims() == 0


def test_reorder_primitive_desc_rules(eng):
    """reorder_primitive_desc_create (src/common/reorder.cpp:67-170): status codes."""
    f32 = md([8, 16], "f32")
    s8t = md([8, 16], "s8", tag=dnnl.tag_ba)
    pd = dnnl.reorder_primitive_desc(eng, f32, eng, s8t)
    assert pd.impl_info_str() == "hip:reorder:any"
    assert pd.query_md(dnnl.query_src_md).data_type() == DT["f32"]
    assert pd.query_md(dnnl.query_dst_md).strides() == [1, 8]
    assert not pd.next_impl()
    # inconsistent dims
    assert status_of(lambda: dnnl.reorder_primitive_desc(eng, f32, eng, md([16, 8], "s8"))) == dnnl.invalid_arguments
    # format any is not a reorder input
    any_md = dnnl.memory_desc([8, 16], DT["s8"], tag=dnnl.tag_any)
    assert status_of(lambda: dnnl.reorder_primitive_desc(eng, f32, eng, any_md)) == dnnl.invalid_arguments
    # zero points only with integer data
    a = dnnl.primitive_attr()
    a.set_zero_points(dnnl.ARG_SRC, 0)
    assert status_of(lambda: dnnl.reorder_primitive_desc(eng, f32, eng, s8t, attr=a)) == dnnl.invalid_arguments
    # scales on src and dst only
    a = dnnl.primitive_attr()
    a.set_scales(dnnl.ARG_WEIGHTS, 0)
    assert status_of(lambda: dnnl.reorder_primitive_desc(eng, f32, eng, s8t, attr=a)) == dnnl.unimplemented
    # groups must divide the dims and the mask must cover the last two dims
    a = dnnl.primitive_attr()
    a.set_scales(dnnl.ARG_SRC, 3, (3, 1))
    u4 = md([8, 16], "u4")
    assert status_of(lambda: dnnl.reorder_primitive_desc(eng, u4, eng, f32, attr=a)) == dnnl.invalid_arguments
    a = dnnl.primitive_attr()
    a.set_scales(dnnl.ARG_SRC, 3, (4, 1), DT["bf16"])
    a.set_zero_points(dnnl.ARG_SRC, 3, (4, 1), DT["u4"])
    assert dnnl.reorder_primitive_desc(eng, u4, eng, f32, attr=a).impl_info_str() == "hip:reorder:any"
    # 4-bit sources need a mask for their scales
    a = dnnl.primitive_attr()
    a.set_scales(dnnl.ARG_SRC, 0)
    assert status_of(lambda: dnnl.reorder_primitive_desc(eng, u4, eng, f32, attr=a)) == dnnl.invalid_arguments


# ---- runtime dims (DNNL_RUNTIME_DIM_VAL): tests/gtests/test_matmul.cpp:128-160,
# :422-427, src/common/memory_desc.cpp:52-72,:298-308, src/common/memory.cpp:62,:155,
# src/common/matmul.cpp:709-736
R = dnnl.RUNTIME_DIM_VAL


def test_memory_desc_with_runtime_dims(eng):
    m = md([R, 7], "f32", tag=dnnl.tag_ab)
    assert m.dims() == [R, 7] and m.strides() == [7, 1]
    m = md([5, R], "f32", tag=dnnl.tag_ab)
    assert m.strides() == [R, 1]                    # a stride outside a runtime dim is a runtime value
    m = md([5, R], "f32", tag=dnnl.tag_ba)
    assert m.strides() == [1, 5]
    m = md([R, R], "s8", tag=dnnl.tag_ba)
    assert m.strides() == [1, R]
    m = md([2, R, 5], "bf16", tag=dnnl.tag_abc)
    assert m.strides() == [R, 5, 1]
    assert m.get_size() == dnnl.RUNTIME_SIZE_VAL
    assert md([R, 4], "f32", strides=[R, 1]).strides() == [R, 1]
    # no layout can be chosen for unknown dims, and no memory object can be made of them
    assert status_of(lambda: md([R, 7], "f32", tag=dnnl.tag_any)) == dnnl.invalid_arguments
    assert status_of(lambda: dnnl.memory(md([R, 7], "f32"), eng)) == dnnl.invalid_arguments
    assert status_of(lambda: md([-3, 7], "f32")) == dnnl.invalid_arguments


def test_matmul_pd_with_runtime_dims(eng):
    pd = dnnl.matmul_primitive_desc(eng, md([R, R], "u8"), md([R, R], "s8", tag=dnnl.tag_ba), md([R, R], "s32"))
    assert pd.impl_info_str() == "hip:runtime_dims:any"
    assert pd.next_impl() is False
    assert pd.query_md(dnnl.query_src_md).dims() == [R, R]
    assert pd.query_md(dnnl.query_weights_md).strides() == [1, R]
    assert pd.scratchpad_desc().ndims() == 0
    dnnl.matmul(pd)                                   # a primitive can be created; it executes on a device only
    # only M unknown (a decode loop): weights known
    pd = dnnl.matmul_primitive_desc(eng, md([R, 256], "bf16"), md([256, 128], "bf16"), md([R, 128], "bf16"))
    assert pd.impl_info_str() == "hip:runtime_dims:any"
    # M, N, K agree as values, runtime included (matmul.cpp:683-688)
    bad = [(md([R, 256], "f32"), md([256, 128], "f32"), md([4, 128], "f32")),
           (md([4, R], "f32"), md([256, 128], "f32"), md([4, 128], "f32")),
           (md([4, 256], "f32"), md([256, R], "f32"), md([4, 128], "f32"))]
    for s, w, d in bad:
        assert status_of(lambda: dnnl.matmul_primitive_desc(eng, s, w, d)) == dnnl.invalid_arguments
    # a runtime batch dim is runtime in src, weights and dst alike (test_matmul.cpp:422-427)
    assert status_of(lambda: dnnl.matmul_primitive_desc(
        eng, md([3, 10, 10], "f32"), md([R, 10, 10], "f32"), md([R, 10, 10], "f32"))) == dnnl.invalid_arguments
    dnnl.matmul_primitive_desc(eng, md([R, 10, 10], "f32"), md([R, 10, 10], "f32"), md([R, 10, 10], "f32"))
    # bias over a runtime batch dim: 1 or runtime
    dnnl.matmul_primitive_desc(eng, md([R, 10, 10], "f32"), md([R, 10, 10], "f32"), md([R, 10, 10], "f32"),
                               bias_md=md([1, 1, 10], "f32"))
    assert status_of(lambda: dnnl.matmul_primitive_desc(
        eng, md([R, 10, 10], "f32"), md([R, 10, 10], "f32"), md([R, 10, 10], "f32"),
        bias_md=md([3, 1, 10], "f32"))) == dnnl.invalid_arguments


def test_attributes_are_checked_with_runtime_dims_too(eng):
    # rules that need no dim value still hold at creation
    a = dnnl.primitive_attr()
    a.set_zero_points(dnnl.ARG_SRC, 0, (), DT["s32"])
    assert status_of(lambda: dnnl.matmul_primitive_desc(            # zero points with a floating-point src
        eng, md([R, R], "f32"), md([R, R], "f32"), md([R, R], "f32"), attr=a)) != dnnl.success
    a = dnnl.primitive_attr()
    a.set_scales(dnnl.ARG_WEIGHTS, 2, (), DT["f32"])
    po = dnnl.post_ops()
    po.append_eltwise(cabi.ELTWISE["relu"], 0.0, 0.0)
    po.append_binary(cabi.BINARY["add"], md([1, 64], "f32"))       # a known src1 under an unknown dst
    a.set_post_ops(po)
    pd = dnnl.matmul_primitive_desc(eng, md([R, R], "s8"), md([R, R], "s8", tag=dnnl.tag_ba), md([R, R], "f32"), attr=a)
    assert pd.impl_info_str() == "hip:runtime_dims:any"
    # data type combinations are known at creation
    assert status_of(lambda: dnnl.matmul_primitive_desc(
        eng, md([R, R], "s8"), md([R, R], "f32"), md([R, R], "f32"))) == dnnl.unimplemented


def test_reorder_with_runtime_dims_is_unimplemented(eng):
    assert status_of(lambda: dnnl.reorder_primitive_desc(
        eng, md([R, 8], "f32"), eng, md([R, 8], "f32"))) == dnnl.unimplemented


def test_host_scalar_memory_and_attributes(eng):
    # dnnl.h:1196-1203,1506-1520,1676-1698; src/common/memory.cpp:157,219-241,265-333; primitive_attr.cpp:655-658,700-702
    import numpy as np
    hs = dnnl.host_scalar(DT["f32"], np.float32(0.25))
    assert hs.md.format_kind() == 5 and hs.md.get_size() == 4           # dnnl_format_kind_host_scalar
    assert hs.get(np.float32) == np.float32(0.25)
    hs.set(np.float32(3.5))
    assert hs.get(np.float32) == np.float32(3.5)
    zp = dnnl.host_scalar(DT["s32"], np.int32(-7))
    assert zp.get(np.int32) == -7
    # an ordinary memory object cannot be made of the descriptor, and the value has no handle and no mapping
    assert status_of(lambda: dnnl.memory(hs.md, eng)) == dnnl.invalid_arguments
    p = C.c_void_p()
    assert dnnl.lib().dnnl_memory_get_data_handle(hs.h, C.byref(p)) == dnnl.invalid_arguments
    assert dnnl.lib().dnnl_memory_map_data(hs.h, C.byref(p)) == dnnl.invalid_arguments
    # only a single value can live on the host
    a = dnnl.primitive_attr()
    assert status_of(lambda: a.set_scales(dnnl.ARG_WEIGHTS, 2, (), DT["f32"], is_on_host=1)) == dnnl.invalid_arguments
    assert status_of(lambda: a.set_zero_points(dnnl.ARG_SRC, 1, (), DT["s32"], is_on_host=1)) == dnnl.invalid_arguments
    a.set_scales(dnnl.ARG_SRC, 0, (), DT["f32"], is_on_host=1)
    a.set_zero_points(dnnl.ARG_SRC, 0, (), DT["s32"], is_on_host=1)
    assert make_pd(eng, 64, 128, 256, "u8", "s8", "f32", attr=a).impl_info_str().startswith("hip:mfma_i8")
    # reorder: device-side parameters only
    r = dnnl.primitive_attr()
    r.set_scales(dnnl.ARG_DST, 0, (), DT["f32"], is_on_host=1)
    assert status_of(lambda: dnnl.reorder_primitive_desc(eng, md([8, 8], "f32"), eng, md([8, 8], "s8"), attr=r)) == dnnl.unimplemented


def test_use_dst_for_bwd_eltwise_post_ops(eng):
    # forward inference computes the base algorithm (primitive_attr_postops.cpp:74-82); the value rules of
    # is_eltwise_ok (math_utils.hpp:442-453) hold at append time
    po = dnnl.post_ops()
    for alg in range(0x100, 0x107):
        po2 = dnnl.post_ops()
        po2.append_eltwise(alg, 0.5, 1.0)
    assert status_of(lambda: po.append_eltwise(0x100, -1.0, 0.0)) == dnnl.invalid_arguments     # relu: alpha >= 0
    assert status_of(lambda: po.append_eltwise(0x102, -1.0, 0.0)) == dnnl.invalid_arguments     # elu
    assert status_of(lambda: po.append_eltwise(0x106, 2.0, 1.0)) == dnnl.invalid_arguments      # clip_v2: beta >= alpha
    assert status_of(lambda: po.append_eltwise(0x107, 0.0, 0.0)) == dnnl.invalid_arguments
    po.append_eltwise(0x100, 0.25, 0.0)
    a = dnnl.primitive_attr()
    a.set_post_ops(po)
    pd = make_pd(eng, 64, 128, 256, "s8", "s8", "f32", attr=a)
    assert pd.impl_info_str().startswith("hip:mfma_i8")           # lowered to plain relu: the fast epilogue takes it


def test_binary_select_post_op_rules(eng):
    # the ternary binary post-op: dnnl_post_ops_append_binary_v2 (primitive_attr.cpp:888-894), dst = src2 ? dst : src1
    sel = cabi.BINARY["select"]
    po = dnnl.post_ops()
    assert status_of(lambda: po.append_binary(sel, md([1, 256], "f32"))) == dnnl.invalid_arguments      # needs src2
    assert status_of(lambda: po.append_binary(cabi.BINARY["add"], md([1, 256], "f32"), md([64, 1], "s8"))) == dnnl.invalid_arguments
    po.append_binary(sel, md([1, 256], "f32"), md([64, 1], "s8"))
    a = dnnl.primitive_attr()
    a.set_post_ops(po)
    assert make_pd(eng, 64, 128, 256, "s8", "s8", "f32", attr=a).impl_info_str() == "hip:ref:any"
    # the condition broadcasts like any binary operand, and is an integer tensor
    po = dnnl.post_ops()
    po.append_binary(sel, md([1, 256], "f32"), md([64, 7], "s8"))
    a = dnnl.primitive_attr()
    a.set_post_ops(po)
    assert status_of(lambda: make_pd(eng, 64, 128, 256, "s8", "s8", "f32", attr=a)) == dnnl.invalid_arguments
    po = dnnl.post_ops()
    po.append_binary(sel, md([1, 256], "f32"), md([64, 256], "f32"))
    a = dnnl.primitive_attr()
    a.set_post_ops(po)
    assert status_of(lambda: make_pd(eng, 64, 128, 256, "s8", "s8", "f32", attr=a)) == dnnl.unimplemented


# ------------------------------------------------- prelu weights layout
def _prelu_pd(eng, dims_dst, K, mask):
    nd = len(dims_dst)
    tags = {2: dnnl.tag_ab, 3: dnnl.tag_abc, 4: dnnl.tag_abcd}
    sdims = list(dims_dst[:-1]) + [K]
    wdims = list(dims_dst[:-2]) + [K, dims_dst[-1]]
    po = dnnl.post_ops()
    po.append_prelu(mask)
    attr = dnnl.primitive_attr()
    attr.set_post_ops(po)
    return dnnl.matmul_primitive_desc(eng, dnnl.memory_desc(sdims, DT["f32"], tag=tags[nd]),
                                      dnnl.memory_desc(wdims, DT["f32"], tag=tags[nd]),
                                      dnnl.memory_desc(list(dims_dst), DT["f32"], tag=tags[nd]), attr=attr)


def test_prelu_weights_follow_the_reference_layout(eng, oracle):
    """get_prelu_weights_format (src/cpu/primitive_attr_postops.cpp:218-241): the
    weights are dims-under-the-mask in ab / acb / acdb -- from three dims on, dim 1
    is innermost.  The lowered strides index an array laid out that way: checked
    by running the oracle on the lowered description against numpy indexing."""
    import numpy as np
    from onednn_amd.problem import MatmulProblem, PostOp
    r = np.random.default_rng(5)
    B, M, N, K = 3, 5, 6, 8
    for mask in (1, 2, 4, 3, 5, 6, 7):                 # bit 0 batch, bit 1 M, bit 2 N
        d = _prelu_pd(eng, (B, M, N), K, mask).lowered_desc()
        db, dm, dn = (B if mask & 1 else 1), (M if mask & 2 else 1), (N if mask & 4 else 1)
        w = r.uniform(-2, 2, size=(db, dn, dm)).astype(np.float32)      # acb: batch, N, M in memory order
        st = tuple(d.post_ops[0].stride)
        assert d.post_ops[0].kind == cabi.PO_PRELU
        src = r.integers(-4, 5, size=(B, M, K)).astype(np.float32)
        wei = r.integers(-4, 5, size=(B, K, N)).astype(np.float32)
        p = MatmulProblem(batch=B, M=M, N=N, K=K, src_dt=cabi.DT_F32, wei_dt=cabi.DT_F32, dst_dt=cabi.DT_F32,
                          src=src, wei=wei, post_ops=[PostOp(kind=cabi.PO_PRELU, dt=cabi.DT_F32, stride=st, data=w)])
        got = oracle.run_oracle(p).reshape(B, M, N)
        v = np.einsum("bmk,bkn->bmn", src, wei)
        wfull = np.broadcast_to(w.transpose(0, 2, 1), (B, M, N))        # logical (b, m, n) view of the acb array
        assert np.array_equal(got, np.where(v >= 0, v, wfull * v)), mask
    # two dims: ab
    d = _prelu_pd(eng, (M, N), K, 3).lowered_desc()
    assert tuple(d.post_ops[0].stride)[1:] == (N, 1)
    # four dims (acdb, dim 1 innermost): the collapsed batch index cannot express a mask over both
    # batch dims together with M or N; masks within what one stride per tensor expresses lower
    assert status_of(lambda: _prelu_pd(eng, (2, 3, M, N), K, 0b1111)) == dnnl.unimplemented
    assert status_of(lambda: _prelu_pd(eng, (2, 3, M, N), K, 0b0111)) == dnnl.unimplemented
    d = _prelu_pd(eng, (2, 3, M, N), K, 0b1100).lowered_desc()          # M and N only: N-major, as acdb says
    assert tuple(d.post_ops[0].stride) == (0, N, 1)
    d = _prelu_pd(eng, (2, 3, M, N), K, 0b0011).lowered_desc()          # both batch dims: memory order a, b
    assert tuple(d.post_ops[0].stride) == (1, 0, 0)
    d = _prelu_pd(eng, (1, 3, M, N), K, 0b1111).lowered_desc()          # one real batch dim, innermost
    assert tuple(d.post_ops[0].stride) == (1, N * 3, 3)


def test_batch_dims_of_extent_one_may_carry_any_stride(eng):
    # [2, 1, M, K] with a stride on the unit dim that does not nest: still one batch stride
    src = dnnl.memory_desc([2, 1, 4, 8], DT["f32"], strides=[32, 7, 8, 1])
    wei = dnnl.memory_desc([2, 1, 8, 6], DT["f32"], strides=[48, 1000, 6, 1])
    dst = dnnl.memory_desc([2, 1, 4, 6], DT["f32"], strides=[24, 24, 6, 1])
    d = dnnl.matmul_primitive_desc(eng, src, wei, dst).lowered_desc()
    assert (d.batch, d.src_stride[0], d.wei_stride[0], d.dst_stride[0]) == (2, 32, 48, 24)
