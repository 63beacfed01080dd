"""Grouped (mixture-of-experts) matmul: the oracle's restatement of
ref_grouped_t (src/cpu/matmul/ref_grouped_gemm.cpp) pinned against per-group
numpy matmuls on exact data (CPU), and the HIP kernel against the oracle through
the C ABI (GPU, bit for bit: same operations in the same order)."""
import ctypes as C

import numpy as np
import pytest

from onednn_amd import cabi
from tests import grouped_cases as gc

F32, BF16, F16 = cabi.DT_F32, cabi.DT_BF16, cabi.DT_F16
S8, U8, S4, U4 = cabi.DT_S8, cabi.DT_U8, cabi.DT_S4, cabi.DT_U4

# (label, builder kwargs) -- the attribute combinations of harness_matmul_grouped_2dby3d
VARIANTS = [
    ("plain", {}),
    ("acb weights + bias", dict(wtag="acb", bias=True)),
    ("bf16", dict(src_dt=BF16, wei_dt=BF16)),
    ("f16", dict(src_dt=F16, wei_dt=F16)),
    ("int8 row / column scales", dict(src_dt=U8, wei_dt=S8, src_scale="row", wei_scale="col")),
    ("int8 zero points", dict(src_dt=S8, wei_dt=U8, src_zp="row", wei_zp="col", wei_scale="col")),
    ("int8 x s4, K-grouped weights", dict(src_dt=U8, wei_dt=S4, wei_scale=16, wei_zp=16, src_scale="row")),
    ("int8, K groups on both sides", dict(src_dt=S8, wei_dt=S8, src_scale=8, wei_scale=16, src_zp=16, wei_zp=16)),
    ("decompression f16 x u4", dict(src_dt=F16, wei_dt=U4, wei_scale=16, wei_zp=16)),
    ("decompression bf16 x s8 per column", dict(src_dt=BF16, wei_dt=S8, wei_scale="col", wei_zp="col")),
    ("fp with scales", dict(src_scale="row", wei_scale="col")),
    ("fp with K-grouped scales", dict(src_scale=16, wei_scale=8)),
    ("relu", dict(post_ops=("relu",))),
    ("per-group factor", dict(post_ops=("mul_group",), bias=True)),
    ("per-row factor", dict(post_ops=("mul_row",))),
    ("per-element factor", dict(post_ops=("mul_full",))),
    ("gate: linear then a grouped factor", dict(post_ops=("linear", "mul_grouped"), bias=True)),
]


def check_exact(p, raw, want):
    got = gc.logical_dst(p, raw)
    assert got.shape == want.shape
    bad = np.argwhere(got != want)
    assert len(bad) == 0, f"{p.name}: {len(bad)} differ, first {bad[0]}: {got[tuple(bad[0])]} vs {want[tuple(bad[0])]}"


@pytest.mark.parametrize("shape", gc.SHAPES_2DX3D, ids=lambda s: "+".join(map(str, s[0])))
@pytest.mark.parametrize("label,kw", VARIANTS, ids=[v[0] for v in VARIANTS])
def test_oracle_2dx3d_against_per_group_numpy(oracle, shape, label, kw):
    sizes, K, N = shape
    p, want = gc.case_2dx3d(sizes, K, N, **kw)
    st, raw = oracle.run_oracle_grouped(p)
    assert st == cabi.SUCCESS
    check_exact(p, raw, want)


@pytest.mark.parametrize("shape", gc.SHAPES_2DX2D, ids=lambda s: "+".join(map(str, s[0])))
@pytest.mark.parametrize("dt", [F32, BF16, F16])
@pytest.mark.parametrize("dtag", ["abc", "acb"])
def test_oracle_2dx2d_against_per_group_numpy(oracle, shape, dt, dtag):
    sizes, M, N = shape
    p, want = gc.case_2dx2d(sizes, M, N, dt=dt, dtag=dtag)
    st, raw = oracle.run_oracle_grouped(p)
    assert st == cabi.SUCCESS
    check_exact(p, raw, want)     # an empty K range writes zeros (ref_grouped_gemm.cpp:252-254)


def test_rows_outside_every_group_stay_untouched(oracle):
    p, want = gc.case_2dx3d([3, 4], 16, 8)
    # the tensors hold 9 rows, the groups cover 7
    p2, _ = gc.case_2dx3d([3, 4, 2], 16, 8)
    p2.sizes, p2.G = [3, 4], 2
    p2.src_offsets = p2.src_offsets[:2].copy()
    p2.other_offsets = p2.other_offsets[:2].copy()
    p2.wei = p2.wei[:2 * 16 * 8]
    st, raw = oracle.run_oracle_grouped(p2)
    assert st == cabi.SUCCESS
    tail = np.asarray(raw).view(np.uint8)[7 * 8 * 4:]
    assert np.all(tail == 0x5a)


@pytest.mark.parametrize("src_off,dst_off", [
    ([4, 3, 9], [4, 7, 9]),        # decreasing
    ([4, 7, 10], [4, 7, 9]),       # beyond total_M
    ([-1, 7, 9], [4, 7, 9]),       # (the end of group 0 is the start of group 1: negative start)
    ([4, 7, 9], [4, 12, 9]),       # dst offsets beyond total_M
])
def test_offsets_the_reference_refuses(oracle, src_off, dst_off):
    p, _ = gc.case_2dx3d([4, 3, 2], 16, 8)
    p.src_offsets = np.asarray(src_off, np.int32)
    p.other_offsets = np.asarray(dst_off, np.int32)
    st, _ = oracle.run_oracle_grouped(p)
    assert st == cabi.INVALID_ARGUMENTS


def test_offsets_the_reference_refuses_2dx2d_and_binary(oracle):
    p, _ = gc.case_2dx2d([5, 6], 4, 8)
    p.other_offsets = np.asarray([5, 10], np.int32)      # weights' offsets differ from src's
    assert oracle.run_oracle_grouped(p)[0] == cabi.INVALID_ARGUMENTS
    p, _ = gc.case_2dx3d([4, 3], 16, 8, post_ops=("mul_grouped",))
    p.post_ops[0].offsets = np.asarray([3, 7], np.int32)  # a grouped operand's offsets differ from dst's
    assert oracle.run_oracle_grouped(p)[0] == cabi.INVALID_ARGUMENTS


def test_query_rules():
    """mi355_grouped_matmul_query mirrors ref_grouped_t::pd_t::init
    (ref_grouped_gemm.hpp:60-270): data types, decompression needs scales and
    apply_to_int, zero points need integer operands, 2Dx2D takes nothing extra."""
    lib = cabi.load_kernels()

    def q(p):
        d = p.desc()
        return lib.mi355_grouped_matmul_query(C.byref(d))

    ok, _ = gc.case_2dx3d([2, 3], 32, 16)
    assert q(ok) == cabi.SUCCESS
    p, _ = gc.case_2dx3d([2, 3], 32, 16, src_dt=U8, wei_dt=S8)
    p.wei_dt = F32                                             # integer src needs integer weights
    assert q(p) == cabi.UNIMPLEMENTED
    p, _ = gc.case_2dx3d([2, 3], 32, 16, src_dt=F16, wei_dt=U4, wei_scale=16)
    assert q(p) == cabi.SUCCESS
    p.apply_to_int = False
    assert q(p) == cabi.UNIMPLEMENTED
    p, _ = gc.case_2dx3d([2, 3], 32, 16, src_dt=F16, wei_dt=U4, wei_scale=16)
    del p.quant["wei_scale"]
    assert q(p) == cabi.UNIMPLEMENTED
    p, _ = gc.case_2dx3d([2, 3], 32, 16, src_zp="row", src_dt=U8, wei_dt=S8)
    p.src_dt, p.wei_dt = F32, F32                              # zero points of a floating-point src
    assert q(p) == cabi.UNIMPLEMENTED
    p, _ = gc.case_2dx3d([2, 3], 32, 16, wei_scale=16)
    p.quant["wei_scale"].group_k = 12                          # K % group != 0
    assert q(p) == cabi.UNIMPLEMENTED
    p, _ = gc.case_2dx3d([2, 3], 32, 16, dst_dt=F32)
    p.dst_dt = S8
    assert q(p) == cabi.UNIMPLEMENTED
    p, _ = gc.case_2dx3d([2, 3], 32, 16, post_ops=("mul_row",))
    p.post_ops[0].alg = cabi.BINARY["add"]                     # only multiplication
    assert q(p) == cabi.UNIMPLEMENTED
    p, _ = gc.case_2dx2d([5, 6], 4, 8)
    assert q(p) == cabi.SUCCESS
    p.wei_dt = BF16                                            # one type everywhere
    assert q(p) == cabi.UNIMPLEMENTED
    p, _ = gc.case_2dx2d([5, 6], 4, 8)
    p.bias_dt = F32
    assert q(p) == cabi.UNIMPLEMENTED


# ---------------------------------------------------------------- GPU parity
@pytest.mark.gpu
@pytest.mark.parametrize("shape", gc.SHAPES_2DX3D, ids=lambda s: "+".join(map(str, s[0])))
@pytest.mark.parametrize("label,kw", VARIANTS, ids=[v[0] for v in VARIANTS])
def test_gpu_2dx3d_bit_exact(gpu, oracle, shape, label, kw):
    from onednn_amd import grouped
    sizes, K, N = shape
    for dst_dt in (F32, BF16):
        p, want = gc.case_2dx3d(sizes, K, N, dst_dt=dst_dt, **kw)
        st, ref = oracle.run_oracle_grouped(p)
        assert st == cabi.SUCCESS
        got = grouped.run_gpu(p)
        assert np.array_equal(got, ref), f"{p.name} {label} dst {dst_dt}"
        if dst_dt == F32:
            check_exact(p, got, want)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", gc.SHAPES_2DX2D, ids=lambda s: "+".join(map(str, s[0])))
@pytest.mark.parametrize("dt", [F32, BF16, F16])
@pytest.mark.parametrize("dtag", ["abc", "acb"])
def test_gpu_2dx2d_bit_exact(gpu, oracle, shape, dt, dtag):
    from onednn_amd import grouped
    sizes, M, N = shape
    p, want = gc.case_2dx2d(sizes, M, N, dt=dt, dtag=dtag)
    st, ref = oracle.run_oracle_grouped(p)
    assert st == cabi.SUCCESS
    got = grouped.run_gpu(p)
    assert np.array_equal(got, ref)


@pytest.mark.gpu
def test_gpu_inexact_data_still_matches_the_oracle_bit_for_bit(gpu, oracle):
    """Random floating-point data, K-grouped scales that are no powers of two,
    tanh-free post-ops: the kernel runs the oracle's operations in the oracle's
    order with one rounding each, so even inexact sums agree bit for bit."""
    from onednn_amd import grouped
    from onednn_amd.grouped import GroupedQuant
    rng = np.random.default_rng(8)
    p, _ = gc.case_2dx3d([5, 0, 17, 9], 64, 40, src_scale=16, wei_scale=32, bias=True, post_ops=("linear", "mul_row"))
    p.src = rng.standard_normal((31, 64)).astype(np.float32)
    p.wei = rng.standard_normal((4, 64, 40)).astype(np.float32)
    p.quant["src_scale"] = GroupedQuant(cabi.DT_F32, rng.uniform(0.3, 1.7, (31, 4)).astype(np.float32), 16)
    p.quant["wei_scale"] = GroupedQuant(cabi.DT_F32, rng.uniform(0.3, 1.7, (4, 2, 40)).astype(np.float32), 32)
    st, ref = oracle.run_oracle_grouped(p)
    assert st == cabi.SUCCESS
    assert np.array_equal(grouped.run_gpu(p), ref)


@pytest.mark.gpu
def test_gpu_is_memory_safe_on_offsets_the_reference_refuses(gpu):
    """The launch does not validate offsets (they live on the device): whatever
    they hold, the kernel stays inside the tensors and leaves rows outside every
    group untouched."""
    from onednn_amd import grouped
    p, _ = gc.case_2dx3d([4, 3, 2], 16, 8)
    p.src_offsets = np.asarray([4, 100000, 9], np.int32)
    p.other_offsets = np.asarray([4, 3, 7], np.int32)
    out = grouped.run_gpu(p)
    assert out.shape == p.initial_dst().shape
    assert np.all(out[7 * 8 * 4:] == 0x5a)       # rows 7, 8 belong to no dst group
