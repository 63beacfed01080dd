"""Pins, on the CPU, the oracle branches no benchmark configuration takes --
each against an expectation written independently in numpy (tests/tail_cases.py):

  * precomputed reductions, grouped src scales and zero points
    (ref_matmul_int8.cpp:146-155,213-238): per reduction group
    acc = sum (s - zs) w - pr * zw + G * zw * zs in int64, both with the real
    group sums (then the result must equal the plain zero-point form) and with
    arbitrary numbers in their place (then every term shows on its own);
  * prelu (primitive_attr_postops.cpp:218-241,362-389): sign test, masks, and
    the acb layout of the weights for three dims;
  * every eltwise algorithm of compute_eltwise_scalar_fwd (:49-87): exact
    float32 formulas where the reference's arithmetic is plain IEEE, float64
    libm within a few units in the last place where it calls libm;
  * every binary algorithm of compute_binary_scalar (:30-47) on integer-valued
    operands, exact.
"""
import numpy as np
import pytest

from onednn_amd import cabi
from tests import tail_cases as tc
from tests.helpers import logical

F = np.float32

PR_VARIANTS = [
    dict(),
    dict(true_sums=False),
    dict(with_src_zp=True),
    dict(with_src_zp=True, true_sums=False),
    dict(with_src_zp=True, src_zp_groups=True),
    dict(with_src_zp=True, src_zp_groups=True, true_sums=False),
    dict(src_dt="u8", with_src_zp=True, true_sums=False, g=32, gw=32),
    dict(with_scales=False, dst="s32", true_sums=False, with_src_zp=True),
    dict(g=16, gw=64, K=256, true_sums=False, with_src_zp=True, src_zp_groups=True),
]


@pytest.mark.parametrize("kw", PR_VARIANTS, ids=lambda kw: ",".join(f"{k}={v}" for k, v in kw.items()) or "plain")
def test_precomputed_reductions(oracle, kw):
    p, want = tc.pr_case(11, **kw)
    got = oracle.run_oracle(p).reshape(p.M, p.N)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_precomputed_reductions_terms_show_individually(oracle):
    # dropping `- pr * zw` or `+ G * zw * zs`, or flipping a sign, changes the expectation:
    # the four variants of the formula are pairwise different on this problem
    p, want = tc.pr_case(12, with_src_zp=True, true_sums=False, with_scales=False, dst="s32")
    got = oracle.run_oracle(p).reshape(p.M, p.N)
    assert np.array_equal(got, want)
    src, wei = p.src.astype(np.int64), p.wei.astype(np.int64)
    g, gw, zs = 16, 32, 5
    pr, wz = p.quant["src_pr"].data.astype(np.int64), p.quant["wei_zp"].data.astype(np.int64)
    variants = []
    for s_pr, s_x in ((-1, 1), (1, 1), (-1, -1), (-1, 0), (0, 1)):
        tot = np.zeros((p.M, p.N), np.int64)
        for gi in range(p.K // g):
            sl = slice(gi * g, (gi + 1) * g)
            zw = wz[gi * g // gw][None, :]
            tot += (src[:, sl] - zs) @ wei[sl] + s_pr * pr[:, gi][:, None] * zw + s_x * g * zw * zs
        variants.append(tot)
    assert np.array_equal(variants[0], want)
    for v in variants[1:]:
        assert not np.array_equal(v, want)


@pytest.mark.parametrize("mask_m,mask_n", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_prelu_two_dims(oracle, mask_m, mask_n):
    p, want, _ = tc.prelu_case(21, mask_m, mask_n)
    got = oracle.run_oracle(p).reshape(want.shape)
    assert (want < 0).any() and (want > 0).any()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("mask_b,mask_m,mask_n", [(0, 1, 1), (1, 0, 1), (1, 1, 0), (1, 1, 1), (1, 0, 0), (0, 0, 1)])
def test_prelu_three_dims_acb(oracle, mask_b, mask_m, mask_n):
    p, want, _ = tc.prelu_case(22, mask_m, mask_n, batch=3, mask_b=bool(mask_b))
    got = oracle.run_oracle(p).reshape(want.shape)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("name", sorted(tc.ELTWISE_TAIL))
def test_eltwise_algorithms(oracle, name):
    p, want, mode = tc.eltwise_case(name)
    got = logical(p, oracle.run_oracle(p)).reshape(p.M, p.N)
    if mode == "exact":
        assert np.array_equal(got.view(np.uint32), np.asarray(want, F).view(np.uint32))
    else:
        ok = tc.ulp_close(got, want, ulps=4, atol=mode[1])
        assert ok.all(), (name, got[~ok][:4], np.asarray(want)[~ok][:4])
    if name in ("soft_relu_big", "mish_big"):
        x = got if name == "soft_relu_big" else None
        # the overflow branch (in >= 88.72...: v = in) is reached
        _, alpha, _, _, scale, _ = tc.ELTWISE_TAIL[name]
        acc = p.src.astype(np.int64) @ p.wei.astype(np.int64)
        assert (acc * scale * (alpha if name == "soft_relu_big" else 1.0) > 89).any()


@pytest.mark.parametrize("name", tc.BINARY_TAIL)
@pytest.mark.parametrize("operand,odt", [("per_element", "f32"), ("per_n", "f32"), ("per_m", "s8"), ("scalar", "bf16")])
def test_binary_algorithms(oracle, name, operand, odt):
    p, want = tc.binary_case(name, operand, odt=odt)
    got = logical(p, oracle.run_oracle(p)).reshape(p.M, p.N)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_nstl_max_min_keep_the_second_operand_on_nan(oracle):
    # nstl::max(x, y) = x > y ? x : y and nstl::min = x < y ? x : y: a NaN in
    # either place selects y (unlike fmaxf)
    x = np.array([1, np.nan, 2, np.nan], F)
    y = np.array([np.nan, 5, -1, np.nan], F)
    mx = oracle.binary(cabi.BINARY["max"], x, y)
    mn = oracle.binary(cabi.BINARY["min"], x, y)
    assert np.isnan(mx[0]) and mx[1] == 5 and mx[2] == 2 and np.isnan(mx[3])
    assert np.isnan(mn[0]) and mn[1] == 5 and mn[2] == -1 and np.isnan(mn[3])
