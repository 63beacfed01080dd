"""Scaled dot-product attention, forward, on top of the matmul kernels:
    dst = softmax(scale * Q K + mask) V
-- the other caller the reference builds on its matmuls (src/common/sdpa_pd.hpp, sdpa_types.hpp; the reference
kernel src/gpu/intel/sdpa/ref.cl, causal masks as in micro.cl:864-878).  Here: two batched matmuls of this library
around a row-softmax kernel.

CPU part: the oracle's restatement of ref_sdpa is pinned against a float64 numpy softmax(QK + mask)V -- per-head and
shared keys / values, K given transposed in memory, broadcast masks, both causal masks, scale and inverted scale
(with a value where the reciprocal's rounding to the scale's type changes the result); the descriptor rules of
sdpa_desc_check (src/common/sdpa_utils.hpp:51-82) through the C API.

GPU part: execution against the oracle.  The device keeps the probabilities in the values' type between the two
matmuls (the reference kernel keeps f32) and sums in another order: outputs within
    bound = sum_k p_k |v_k| * (eps(type) + K-sum terms)
of the oracle's float64-accurate value, eps the type's relative half unit: 2^-8 for bf16, 2^-11 for f16, 2^-24 for
f32 (see `tolerance`)."""
import os

import numpy as np
import pytest

os.environ.setdefault("ONEDNN_AMD_ALLOW_NO_DEVICE", "1")

from onednn_amd import cabi, dnnl  # noqa: E402
from onednn_amd.problem import decode, storage_dtype  # noqa: E402
from tests.test_inner_product import encode  # noqa: E402

DT = cabi.DT_NAMES


@pytest.fixture(scope="module")
def eng():
    return dnnl.engine(dnnl.gpu, 0)


def values(dt, view):
    flat = np.ascontiguousarray(view).reshape(-1)
    return decode(DT[dt], flat, flat.size).astype(np.float64).reshape(view.shape)


def make(seed, b, h, hk, sq, sk, d, dv, dt, k_transposed=True, mag=1.0):
    """q [b][h][sq][d], k [b][hk][d][sk] (a view of [b][hk][sk][d] storage when k_transposed), v [b][hk][sk][dv]"""
    r = np.random.default_rng(seed)
    q = encode(mag * r.standard_normal((b, h, sq, d)).astype(np.float32), dt)
    if k_transposed:
        k = encode(mag * r.standard_normal((b, hk, sk, d)).astype(np.float32), dt).transpose(0, 1, 3, 2)
    else:
        k = encode(mag * r.standard_normal((b, hk, d, sk)).astype(np.float32), dt)
    v = encode(r.standard_normal((b, hk, sk, dv)).astype(np.float32), dt)
    return q, k, v


def ideal(q, k, v, dt, scale=None, invert=False, mask=None, mask_type=0):
    """float64 softmax(scale * QK + mask) V and sum_k p_k |v_k|"""
    Q, K, V = values(dt, q), values(dt, k), values(dt, v)
    s = np.matmul(Q, K)                                          # broadcasting over the first two dims
    if scale is not None:
        s = s * ((1.0 / scale) if invert else scale)
    if mask is not None:
        s = s + mask
    sq, sk = s.shape[2], s.shape[3]
    if mask_type in (2, 3):
        qi, ki = np.arange(sq)[:, None], np.arange(sk)[None, :]
        s = np.where(ki > qi + (sk - sq if mask_type == 3 else 0), -np.inf, s)
    with np.errstate(invalid="ignore"):
        e = np.exp(s - np.max(s, axis=-1, keepdims=True))
        p = e / e.sum(-1, keepdims=True)
    return np.matmul(p, V), np.matmul(p, np.abs(V))


# ------------------------------------------------------------------ the oracle, pinned
@pytest.mark.parametrize("hk", [4, 1])
@pytest.mark.parametrize("k_transposed", [True, False])
@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
def test_oracle_is_softmax_qk_v(oracle, hk, k_transposed, dt):
    q, k, v = make(1, 2, 4, hk, 7, 13, 16, 10, dt, k_transposed)
    sc = np.array([0.25], np.float32)
    got = oracle.run_oracle_sdpa(q, k, v, (dt, "f32", "f32", "f32"), scale=sc)
    want, _ = ideal(q, k, v, dt, scale=0.25)
    assert got.shape == want.shape
    assert np.allclose(got, want, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("mshape", [(2, 4, 7, 13), (1, 1, 7, 13), (2, 1, 1, 13), (1, 4, 7, 1)])
def test_oracle_mask_is_added_before_the_exponential(oracle, mshape):
    q, k, v = make(2, 2, 4, 4, 7, 13, 16, 10, "f32")
    mask = np.random.default_rng(3).standard_normal(mshape).astype(np.float32) * 3
    got = oracle.run_oracle_sdpa(q, k, v, ("f32",) * 4, mask=mask, mask_type=1)
    want, _ = ideal(q, k, v, "f32", mask=mask.astype(np.float64))
    assert np.allclose(got, want, rtol=2e-5, atol=2e-6)
    # (a mask that is constant along the keys leaves a softmax as it is; the others do not)
    plain, _ = ideal(q, k, v, "f32")
    assert np.allclose(got, plain, rtol=1e-3, atol=1e-4) == (mshape[3] == 1)


@pytest.mark.parametrize("mask_type,sq,sk", [(2, 9, 9), (2, 5, 12), (3, 5, 12), (3, 9, 9), (3, 1, 6)])
def test_oracle_causal_masks(oracle, mask_type, sq, sk):
    q, k, v = make(4, 1, 3, 3, sq, sk, 8, 6, "f32")
    got = oracle.run_oracle_sdpa(q, k, v, ("f32",) * 4, mask_type=mask_type)
    want, _ = ideal(q, k, v, "f32", mask_type=mask_type)
    assert np.allclose(got, want, rtol=2e-5, atol=2e-6)
    # the first query of a top-left mask sees the first key only: dst row 0 is the first value row
    if mask_type == 2:
        assert np.allclose(got[:, :, 0, :], values("f32", v)[:, :, 0, :], rtol=1e-6)
    # the last query of a bottom-right mask sees every key
    if mask_type == 3:
        full, _ = ideal(q, k, v, "f32")
        assert np.allclose(got[:, :, -1, :], full[:, :, -1, :], rtol=2e-5, atol=2e-6)


def test_oracle_inverted_scale_is_rounded_to_the_scales_type(oracle):
    """scale = 3 in f16: 1/3 rounds to 0.33325195; with scores of ~30 the difference to 1/3 in f32 moves the
    probabilities by more than the comparison's tolerance."""
    q, k, v = make(5, 1, 1, 1, 4, 6, 32, 4, "f32", mag=2.5)
    s16 = np.array([3.0], np.float16).view(np.uint16)
    got = oracle.run_oracle_sdpa(q, k, v, ("f32", "f32", "f16", "f32"), scale=s16, invert_scale=True)
    third16 = float(np.float16(np.float32(1.0) / np.float32(3.0)))
    want, _ = ideal(q, k, v, "f32", scale=third16)
    assert np.allclose(got, want, rtol=2e-5, atol=2e-6)
    other, _ = ideal(q, k, v, "f32", scale=1.0 / 3.0)
    assert np.abs(want - other).max() > 1e-4 and not np.allclose(got, other, rtol=2e-5, atol=2e-6)


# ------------------------------------------------------------------ descriptor rules (no GPU)
def md4(shape, dt, transposed=False):
    if transposed:                   # dims as given, the last two swapped in memory
        b, h, r, c = shape
        return dnnl.memory_desc(list(shape), DT[dt], strides=[h * r * c, r * c, 1, r])
    return dnnl.memory_desc(list(shape), DT[dt], tag=dnnl.tag_abcd)


def status_of(fn):
    try:
        fn()
        return dnnl.success
    except dnnl.error as e:
        return e.status


def sdpa_pd(eng, b=2, h=4, hk=4, sq=8, sk=16, d=32, dv=32, dt="bf16", ddt=None, **kw):
    return dnnl.sdpa_primitive_desc(eng, md4((b, h, sq, d), dt), md4((b, hk, d, sk), dt, transposed=True),
                                    md4((b, hk, sk, dv), dt), md4((b, h, sq, dv), ddt or dt), **kw)


def test_descriptor_rules(eng):
    pd = sdpa_pd(eng)
    assert pd.query_s32(dnnl.query_primitive_kind) == dnnl.kind_sdpa
    assert pd.impl_info_str().startswith("hip:sdpa(")
    inv, un = dnnl.invalid_arguments, dnnl.unimplemented
    q, k, v, d = md4((2, 4, 8, 32), "f16"), md4((2, 4, 32, 16), "f16"), md4((2, 4, 16, 24), "f16"), md4((2, 4, 8, 24), "f16")
    mk = lambda *a, **kw: status_of(lambda: dnnl.sdpa_primitive_desc(eng, *a, **kw))  # noqa: E731
    assert mk(q, k, v, d) == dnnl.success
    assert mk(q, md4((2, 4, 31, 16), "f16"), v, d) == inv                      # head size of q and k (sdpa_utils.hpp:64)
    assert mk(q, k, md4((2, 4, 15, 24), "f16"), d) == inv                      # keys of k and v (:67)
    assert mk(q, k, v, md4((2, 4, 9, 24), "f16")) == inv                       # queries of dst (:70)
    assert mk(q, k, v, md4((2, 4, 8, 25), "f16")) == inv                       # value head size of dst (:73)
    assert mk(q, k, v, d, attn_mask_type=7) == inv
    assert mk(q, k, v, d, prop=dnnl.forward_training) == un                    # no statistics for a backward pass
    assert mk(q, md4((2, 2, 32, 16), "f16"), md4((2, 2, 16, 24), "f16"), d) == un   # 1 < kv heads < heads
    assert mk(q, md4((2, 1, 32, 16), "f16"), md4((2, 1, 16, 24), "f16"), d) == dnnl.success
    assert mk(q, md4((2, 4, 32, 16), "bf16"), v, d) == un                      # one type for q, k, v
    a = dnnl.primitive_attr()
    a.set_scales_mask(dnnl.ARG_WEIGHTS, 0)
    assert mk(q, k, v, d, kq_attr=a) == un                                     # quantized keys
    mask = md4((1, 1, 8, 16), "f16")
    assert mk(q, k, v, d, mask_md=mask, attn_mask_type=dnnl.attn_mask_buffer) == dnnl.success
    assert mk(q, k, v, d, mask_md=md4((1, 1, 8, 15), "f16"), attn_mask_type=1) == inv
    sc = dnnl.memory_desc([1], DT["f16"], tag=dnnl.tag_a)
    assert mk(q, k, v, d, scale_md=sc, invert_scale=True) == dnnl.success
    assert mk(q, k, v, d, scale_md=dnnl.memory_desc([2], DT["f16"], tag=dnnl.tag_a)) == inv


def test_the_two_matmuls_run_on_the_matrix_cores(eng):
    pd = sdpa_pd(eng, b=1, h=16, hk=16, sq=512, sk=512, d=128, dv=128)
    assert pd.impl_info_str() == "hip:sdpa(hip:mfma_h16:gfx950,hip:mfma_h16:gfx950)"


# ------------------------------------------------------------------ execution on the device
def storage(view):
    order = np.argsort([-s for s in view.strides], kind="stable")
    return np.ascontiguousarray(view.transpose(order))


def run(q, k, v, dt, ddt, k_transposed, scale=None, sdt="f32", invert=False, mask=None, mdt="f32", mask_type=0,
        alg=dnnl.softmax_accurate):
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    b, h, sq, d = q.shape
    hk, sk, dv = k.shape[1], k.shape[3], v.shape[3]
    q_md, k_md = md4(q.shape, dt), md4(k.shape, dt, transposed=k_transposed)
    v_md, d_md = md4(v.shape, dt), md4((b, h, sq, dv), ddt)
    m_md = md4(mask.shape, mdt) if mask is not None else None
    s_md = dnnl.memory_desc([1], DT[sdt], tag=dnnl.tag_a) if scale is not None else None
    pd = dnnl.sdpa_primitive_desc(eng, q_md, k_md, v_md, d_md, mask_md=m_md, scale_md=s_md, invert_scale=invert,
                                  kv_head_number=hk, attn_mask_type=mask_type, softmax_alg=alg)
    prim = dnnl.sdpa(pd)
    dst = dnnl.memory(d_md, eng, np.full(b * h * sq * dv, 0x55, np.uint8).repeat(np.dtype(storage_dtype(DT[ddt])).itemsize))
    args = {dnnl.ARG_QUERIES: dnnl.memory(q_md, eng, storage(q)), dnnl.ARG_KEYS: dnnl.memory(k_md, eng, storage(k)),
            dnnl.ARG_VALUES: dnnl.memory(v_md, eng, storage(v)), dnnl.ARG_DST: dst}
    if mask is not None:
        args[dnnl.ARG_ATTN_MASK] = dnnl.memory(m_md, eng, mask)
    if scale is not None:
        args[dnnl.ARG_SCALE] = dnnl.memory(s_md, eng, scale)
    prim.execute(strm, args)
    strm.wait()
    return dst.read(storage_dtype(DT[ddt])).reshape(b, h, sq, dv), pd.impl_info_str()


def tolerance(dt, ddt, sk, pabs, want):
    """|device - exact| per dst element: the probabilities are rounded to the values' type before the second matmul
    (relative eps each), both sums run in f32 in the hardware's order (sqrt(sk) roundings of 2^-24 sum|terms| each,
    four standard deviations), the exponentials and their sum carry a few units of f32, dst rounds once."""
    half_ulp = {"f32": 2.0 ** -24, "bf16": 2.0 ** -8, "f16": 2.0 ** -11}    # relative, round to nearest
    before = pabs * (half_ulp[dt] + 4 * np.sqrt(sk) * 2.0 ** -24 + 2.0 ** -20)
    return before + (np.abs(want) + before) * half_ulp[ddt] + 1e-30


SHAPES = [  # b, h, hk, sq, sk, d, dv
    (2, 4, 4, 7, 13, 16, 10),
    (1, 8, 8, 128, 256, 64, 64),
    (2, 16, 1, 64, 384, 128, 128),        # one key / value head for all query heads
    (1, 4, 4, 1, 1000, 128, 128),         # decode: one query
    (1, 2, 2, 300, 77, 80, 48),
]


@pytest.mark.gpu
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dt,ddt", [("f32", "f32"), ("bf16", "bf16"), ("f16", "f16"), ("bf16", "f32")])
def test_gpu_against_the_oracle(gpu, oracle, shape, dt, ddt):
    b, h, hk, sq, sk, d, dv = shape
    q, k, v = make(11, b, h, hk, sq, sk, d, dv, dt)
    sc = np.array([1.0 / np.sqrt(d)], np.float32)
    mask = (np.random.default_rng(12).standard_normal((1, 1, sq, sk)) * 2).astype(np.float32)
    got, impl = run(q, k, v, dt, ddt, True, scale=sc, mask=mask, mask_type=1)
    want, pabs = ideal(q, k, v, dt, scale=float(sc[0]), mask=mask.astype(np.float64))
    ref = oracle.run_oracle_sdpa(q, k, v, (dt, "f32", "f32", "f32"), scale=sc, mask=mask, mask_type=1)
    assert np.allclose(ref, want, rtol=1e-4, atol=1e-5)                     # the oracle itself
    err = np.abs(values(ddt, got) - want)
    tol = tolerance(dt, ddt, sk, pabs, want)
    assert (err <= tol).all(), f"{impl}: worst {np.max(err / tol):.2f} of the bound"


@pytest.mark.gpu
@pytest.mark.parametrize("mask_type,sq,sk", [(2, 128, 128), (2, 40, 100), (3, 40, 100), (3, 1, 333)])
@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_gpu_causal_masks(gpu, oracle, mask_type, sq, sk, dt):
    q, k, v = make(13, 1, 4, 4, sq, sk, 64, 64, dt)
    sc = np.array([8.0], np.float32)
    got, impl = run(q, k, v, dt, dt, True, scale=sc, invert=True, mask_type=mask_type)
    want, pabs = ideal(q, k, v, dt, scale=8.0, invert=True, mask_type=mask_type)
    err = np.abs(values(dt, got) - want)
    assert (err <= tolerance(dt, dt, sk, pabs, want)).all(), impl
    if mask_type == 2:   # the first query sees the first key only
        assert np.array_equal(values(dt, got)[:, :, 0, :], values(dt, v)[:, :, 0, :])


@pytest.mark.gpu
def test_gpu_keys_in_either_memory_order_and_f16_scale(gpu, oracle):
    for k_transposed in (True, False):
        q, k, v = make(14, 2, 4, 4, 33, 65, 32, 32, "f16", k_transposed)
        s16 = np.array([6.0], np.float16).view(np.uint16)
        got, impl = run(q, k, v, "f16", "f16", k_transposed, scale=s16, sdt="f16", invert=True)
        want, pabs = ideal(q, k, v, "f16", scale=float(np.float16(np.float32(1) / np.float32(6))))
        err = np.abs(values("f16", got) - want)
        assert (err <= tolerance("f16", "f16", 65, pabs, want)).all(), impl


@pytest.mark.gpu
def test_gpu_a_row_of_minus_infinity(gpu):
    """An explicit mask that removes every key of some queries: NaN with softmax_accurate (0 / 0, as in the
    reference kernel), zeros with softmax_accurate_inf_as_zero."""
    q, k, v = make(15, 1, 2, 2, 6, 20, 16, 16, "f32")
    mask = np.zeros((1, 1, 6, 20), np.float32)
    mask[0, 0, 2, :] = -np.inf
    got, _ = run(q, k, v, "f32", "f32", True, mask=mask, mask_type=1)
    assert np.isnan(got[:, :, 2, :]).all() and np.isfinite(np.delete(got, 2, axis=2)).all()
    got0, _ = run(q, k, v, "f32", "f32", True, mask=mask, mask_type=1, alg=dnnl.softmax_accurate_inf_as_zero)
    assert not got0[:, :, 2, :].any()
    assert np.array_equal(np.delete(got0, 2, axis=2), np.delete(got, 2, axis=2))


@pytest.mark.gpu
def test_gpu_large_scores_do_not_overflow(gpu):
    """Scores of a few hundred: exp overflows f32 in the reference kernel's formula (inf / inf); relative to the
    row maximum it does not."""
    q, k, v = make(16, 1, 2, 2, 8, 64, 64, 16, "f32", mag=4.0)
    got, _ = run(q, k, v, "f32", "f32", True)
    want, pabs = ideal(q, k, v, "f32")
    assert np.isfinite(got).all()
    assert (np.abs(got - want) <= tolerance("f32", "f32", 64, pabs, want) + 1e-5 * np.abs(want)).all()
