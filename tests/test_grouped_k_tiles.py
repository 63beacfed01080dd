"""The variable-K grouped pattern on the matrix cores ("hip:mfma_grouped_k"):
dst[g] = src[:, k0:k1] x wei[k0:k1, :] for f32 / bf16 / f16 tensors, both dst
layouts.

  * data every type holds exactly (any summation order gives the same bits):
    against the oracle -- ref_grouped_t's loop
    (src/cpu/matmul/ref_grouped_gemm.cpp:215-440) -- bit for bit, over tiles
    with row and column tails, several tiles a group, groups of 0, 1, 3 ... k
    (k ranges that are no multiples of the instruction's 4 or of the 16 in
    flight), more than one tile along both dimensions;
  * random data: against per-group float64 products within
    tests.helpers.gemm_bound (float32 sums of exact or once-rounded products in
    the hardware's order) plus one rounding to the dst type;
  * a weights-gradient shape at full size: against the thread-per-element
    kernel within the same bound."""
import ctypes as C

import numpy as np
import pytest

from onednn_amd import cabi
from onednn_amd.problem import decode
from tests import grouped_cases as gc
from tests.benchdnn_matmul import encode
from tests.helpers import U, gemm_bound

F32, BF16, F16 = cabi.DT_F32, cabi.DT_BF16, cabi.DT_F16
HALF_ULP = {F32: 2.0 ** -24, BF16: 2.0 ** -8, F16: 2.0 ** -11}

SHAPES = [
    ([16, 16, 16, 16], 8, 32),
    ([3, 0, 13, 8], 4, 12),
    ([32], 4, 8),
    ([0, 0, 7], 132, 68),                 # tails on both sides of a second tile
    ([1, 2, 3, 4, 5, 17, 64, 0, 33], 64, 128),
    ([40, 1], 260, 136),                  # 3 x 2 tiles a group
    ([5] * 70, 16, 20),
    ([0, 31, 7], 136, 72),                # (columns in eights: the LDS variant's shapes)
    ([40, 1, 100, 32, 65], 264, 136),
    ([40, 1, 100, 0, 65], 136, 1096),     # nine column tiles: a run of eight and one
]


@pytest.fixture(params=["short", "auto", "tall", "wide"])
def variant(request):
    """"short" keeps bf16 / f16 on the f32 instruction too; otherwise shapes with columns in eights go through LDS
    to the 16-bit instructions, where a workgroup takes a run of column tiles: "tall" forces runs of one, "wide" of
    eight (otherwise chosen by the number of tiles)."""
    with cabi.tuning("MI355_GROUPED_IMPL", None if request.param == "auto" else request.param):
        yield request.param


def impl_of(p):
    d = p.desc()
    return cabi.load_kernels().mi355_grouped_matmul_impl(C.byref(d)).decode()


def test_dispatch_rules():
    p, _ = gc.case_2dx2d([5, 6], 8, 12, dt=BF16)
    assert impl_of(p) == "hip:mfma_grouped_k"
    p, _ = gc.case_2dx2d([5, 6], 8, 12, dt=F32, dtag="acb")
    assert impl_of(p) == "hip:mfma_grouped_k"
    p, _ = gc.case_2dx2d([5, 6], 6, 12, dt=F16)          # rows are read four at a time
    assert impl_of(p) == "hip:ref_grouped:any"
    p, _ = gc.case_2dx2d([5, 6], 8, 10, dt=F16)
    assert impl_of(p) == "hip:ref_grouped:any"
    with cabi.tuning("MI355_GROUPED_IMPL", "ref"):
        p, _ = gc.case_2dx2d([5, 6], 8, 12, dt=BF16)
        assert impl_of(p) == "hip:ref_grouped:any"


@pytest.mark.gpu
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"G{len(s[0])}x{sum(s[0])}x{s[1]}x{s[2]}")
@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("dtag", ["abc", "acb"])
def test_exact_data_matches_the_oracle(gpu, oracle, variant, shape, dt, dtag):
    from onednn_amd import grouped
    sizes, M, N = shape
    p, want = gc.case_2dx2d(sizes, M, N, dt=dt, dtag=dtag)
    assert impl_of(p) == "hip:mfma_grouped_k"
    st, ref = oracle.run_oracle_grouped(p)
    assert st == cabi.SUCCESS
    got = grouped.run_gpu(p)
    assert np.array_equal(got, ref), p.name
    if np.abs(want).max() <= {F32: 2.0 ** 24, BF16: 2.0 ** 8, F16: 2.0 ** 11}[dt]:   # (dst holds the sums exactly)
        assert np.array_equal(gc.logical_dst(p, got), want)


def random_case(sizes, M, N, dt, dtag, seed):
    rng = np.random.default_rng(seed)
    p, _ = gc.case_2dx2d(sizes, M, N, dt=dt, dtag=dtag)
    total = int(sum(sizes))
    S = decode(dt, encode(dt, rng.standard_normal((M, total))), M * total).reshape(M, total).astype(np.float64)
    W = decode(dt, encode(dt, rng.standard_normal((total, N))), total * N).reshape(total, N).astype(np.float64)
    p.src = encode(dt, np.ascontiguousarray(S.T))
    p.wei = encode(dt, W)
    want = np.zeros((len(sizes), M, N))
    tol = np.zeros_like(want)
    k0 = 0
    for g, kg in enumerate(sizes):
        s, w = S[:, k0:k0 + kg], W[k0:k0 + kg]
        want[g] = s @ w
        abs_sum = np.abs(s) @ np.abs(w)
        # f32 operands: the products round once each as well
        tol[g] = gemm_bound(max(kg, 1), abs_sum) + (U * abs_sum if dt == F32 else 0.0) \
            + HALF_ULP[dt] * (np.abs(want[g]) + gemm_bound(max(kg, 1), abs_sum)) \
            + (2.0 ** -25 if dt == F16 else 0.0)      # (half a step of f16's subnormals)
        k0 += kg
    return p, want, tol


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("dtag", ["abc", "acb"])
def test_random_data_within_the_derived_bound(gpu, variant, dt, dtag):
    from onednn_amd import grouped
    p, want, tol = random_case([33, 0, 5, 64, 17, 1, 90, 2, 300], 200, 264, dt, dtag, seed=31)
    assert impl_of(p) == "hip:mfma_grouped_k"
    got = gc.logical_dst(p, grouped.run_gpu(p))
    err = np.abs(got - want)
    assert np.all(err <= tol), f"worst {np.max(err / np.maximum(tol, 1e-30)):.3f} of the bound"
    # the bound is no formality: errors do occur
    assert err.max() > 0


@pytest.mark.gpu
def test_weights_gradient_shape_at_full_size_against_the_reference_order_kernel(gpu, variant):
    """32 experts, 2048 tokens routed unevenly, hidden 2048 x intermediate 1024 in bf16: every dst element of the
    tiles against the thread-per-element kernel within the bound."""
    from onednn_amd import grouped
    rng = np.random.default_rng(5)
    G, total, M, N = 32, 2048, 2048, 1024
    cuts = np.sort(rng.integers(0, total + 1, G - 1))
    sizes = np.diff(np.concatenate([[0], cuts, [total]])).tolist()
    p, want, tol = random_case(sizes, M, N, BF16, "abc", seed=6)
    assert impl_of(p) == "hip:mfma_grouped_k"
    got = gc.logical_dst(p, grouped.run_gpu(p))
    with cabi.tuning("MI355_GROUPED_IMPL", "ref"):
        assert impl_of(p) == "hip:ref_grouped:any"
        ref = gc.logical_dst(p, grouped.run_gpu(p))
    assert np.all(np.abs(ref - want) <= tol)
    assert np.all(np.abs(got - want) <= tol)
    assert np.all(np.abs(got - ref) <= 2 * tol)
