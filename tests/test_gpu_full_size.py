"""The benchmark configurations at their full sizes (C3 8192^3 int8, C4
4096 x 8192 x 28672 fp8, C5 8192^3 MXFP4), through the C ABI, in the weights
layout the bench measures (what format_tag::any resolves to).

The oracle cannot finish these sizes in seconds, so it runs on a sample of dst
rows: a matmul row depends on its own src row (and its own per-row parameters
and post-op operands) only, so the sub-problem made of the sampled rows and all
of the weights has exactly those rows as its result.  Rows are drawn from every
256-row tile band, first and last rows included.  Bars as at the small sizes:
bit-exact for the s8 dst of the integer GEMM; the floating-point ones against
the oracle's float64 sums under the sqrt(K)-type bound of tests/helpers.py, with
an f32 dst as well as the configuration's bf16 so that the dst rounding does not
hide an error of the sum or the epilogue.
"""
import dataclasses

import numpy as np
import pytest

from onednn_amd import cabi, configs
from onednn_amd.problem import PostOp, QuantParam, run_gpu
from tests.helpers import assert_bit_exact, assert_gemm_close, fp8_mfma_bound

pytestmark = pytest.mark.gpu


def sample_rows(M, per_band, seed):
    r = np.random.default_rng(seed)
    rows = {0, M - 1}
    for band in range(0, M, 256):
        rows.update(int(x) for x in band + r.choice(256, size=per_band, replace=False))
    return np.array(sorted(rows))


def row_slice(p, rows):
    """The problem restricted to the given dst rows."""
    M, r = p.M, len(rows)

    def take(data):
        a = np.ascontiguousarray(data)
        return np.ascontiguousarray(a.reshape(M, -1)[rows])

    quant = {}
    for name, q in p.quant.items():
        per_row = name.startswith("src") and (q.mask & configs.MASK_ROW)
        quant[name] = QuantParam(q.dt, q.mask, take(q.data) if per_row else q.data, q.groups)
    post_ops = []
    for po in p.post_ops:
        if po.data is not None and po.stride[1] != 0:
            post_ops.append(dataclasses.replace(po, data=take(po.data), stride=(r * p.N, po.stride[1], po.stride[2])))
        else:
            post_ops.append(po)
    assert p.bias is None or p.bias_stride[1] == 0
    return dataclasses.replace(p, M=r, src=take(p.src), quant=quant, post_ops=post_ops, src_stride=None,
                               dst_stride=None, name=p.name + "-rows")


def rows_of(p, raw, rows):
    a = np.ascontiguousarray(raw)
    return np.ascontiguousarray(a.reshape(p.M, -1)[rows]).reshape(-1)


def test_config3_full_size_sampled_rows_are_bit_exact(gpu, oracle):
    p = configs.config3(wtag="ba")
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_i8")
    rows = sample_rows(p.M, 2, 3)
    sub = row_slice(p, rows)
    want = oracle.run_oracle(sub)
    assert_bit_exact(sub, rows_of(p, got, rows), want, name)
    # the dst is not trivially zero (ReLU) or saturated: a share of it rounds to interior values
    g = np.asarray(got).view(np.int8)
    assert np.mean((g > 0) & (g < 127)) > 0.05


@pytest.mark.parametrize("chain", ["gelu_tanh + residual", "swish x gate"])
@pytest.mark.parametrize("dst", ["bf16", "f32"])
def test_config4_full_size_sampled_rows(gpu, oracle, dst, chain):
    # against the oracle's float64 K-sums with bias, gelu_tanh and the residual in float64 on top:
    # bound = 4 standard deviations of the float32 summation error model (tests/helpers.py gemm_bound)
    # plus the matrix cores' fp8 alignment loss (fp8_mfma_bound), together about 0.1 on pre-activations
    # of standard deviation 90, carried through the chain; with the f32 dst nothing else is inside it,
    # the bf16 dst adds half a unit in its last place
    # (the second chain: the gated feed-forward layer on the same tensors, the other whole-row epilogue of the kernel)
    p = configs.config4(wtag="ba")
    p.dst_dt = cabi.DT_NAMES[dst]
    if chain == "swish x gate":
        elt, gate = p.post_ops
        elt.alg, elt.alpha = cabi.ELTWISE["swish"], 1.0
        gate.alg = cabi.BINARY["mul"]
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_f8")
    rows = sample_rows(p.M, 1, 4)
    sub = row_slice(p, rows)
    _, ideal, asum = oracle.run_oracle(sub, want_ideal=True)
    assert assert_gemm_close(sub, rows_of(p, got, rows), ideal, asum, what=name, hw=fp8_mfma_bound(sub)) < 1.0


@pytest.mark.parametrize("dst", ["bf16", "f32"])
def test_config5_full_size_sampled_rows(gpu, oracle, dst):
    p = configs.config5(wtag="ba")
    p.dst_dt = cabi.DT_NAMES[dst]
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_mxf4")
    rows = sample_rows(p.M, 1, 5)
    sub = row_slice(p, rows)
    _, ideal, asum = oracle.run_oracle(sub, want_ideal=True)
    assert assert_gemm_close(sub, rows_of(p, got, rows), ideal, asum, what=name) < 1.0


# ---------------------------------------------------------------- every element of dst at full size
# The sampled rows above anchor each kernel to the oracle; a fault tied to particular rows or columns of a tile is
# only seen when a sampled row lands on it.  The one-thread-per-element kernel would take minutes at these sizes, so
# the second opinion over all of dst is another tile geometry of the same family (other loop, other division of the
# tile among the wavefronts, other order of the tiles), itself anchored to the oracle on the same sampled rows, or --
# where the result is linear in the operands -- the row and column sums of dst against float64 products.

def test_config3_every_element_agrees_between_tile_geometries_and_weight_layouts(gpu, oracle):
    """C3 whole: the 256 x 256 LDS tiles (the dispatcher's choice), the 256 x 128 ones and the 32 x 32 tiles without LDS
    give the same 67 M bytes; so do row-major weights (the benchdnn line's --wtag=ab: the layout pre-pass runs inside
    the launch).  The small tiles are held to the oracle on the sampled rows like the large ones above."""
    p = configs.config3(wtag="ba")
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_i8")
    got = np.asarray(got).copy()
    rows = sample_rows(p.M, 2, 13)
    sub = row_slice(p, rows)
    want = oracle.run_oracle(sub)
    for tiles in ("small", "narrow"):
        with cabi.tuning("MI355_I8_TILES", tiles):
            other, oname = run_gpu(p, cabi.IMPL_I8_MFMA)
        other = np.asarray(other)
        assert_bit_exact(sub, rows_of(p, other, rows), want, f"{oname} {tiles}")
        assert np.array_equal(got, other), f"{tiles} tiles differ from the large ones in {np.count_nonzero(got != other)} bytes"
    pab = configs.config3(wtag="ab")
    ab, abname = run_gpu(pab)
    assert abname.startswith("hip:mfma_i8")
    assert np.array_equal(got, np.asarray(ab)), "row-major weights give other bytes than K-contiguous ones"


def test_config1_s32_accumulators_whole(gpu, oracle):
    """the configuration's own accumulator check (dst = s32, no scales), whole, through the dispatcher's choice and
    through both other tile geometries"""
    p = configs.config1(dst="s32")
    want = oracle.run_oracle(p)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_i8")
    assert_bit_exact(p, got, want, name)
    for tiles in ("wide", "narrow"):
        with cabi.tuning("MI355_I8_TILES", tiles):
            other, oname = run_gpu(p, cabi.IMPL_I8_MFMA)
        assert_bit_exact(p, other, want, f"{oname} {tiles}")


def test_config3_divide_against_reciprocal_dst_scale(gpu):
    """the reference's naive kernel divides by the dst scale, its JIT kernel multiplies by the reciprocal
    (src/cpu/x64/matmul/brgemm_matmul.cpp:703-709): how many of C3's 67 M outputs tell the two apart"""
    a, _ = run_gpu(configs.config3(wtag="ba", dst_scale_mode=cabi.DST_SCALE_DIVIDE))
    b, _ = run_gpu(configs.config3(wtag="ba", dst_scale_mode=cabi.DST_SCALE_RECIPROCAL))
    a, b = np.asarray(a).view(np.int8).astype(np.int16), np.asarray(b).view(np.int8).astype(np.int16)
    diff = np.abs(a - b)
    n = int(np.count_nonzero(diff))
    print(f"C3 divide vs reciprocal: {n} of {a.size} outputs differ ({n / a.size:.2e}), all by one unit")
    assert diff.max() <= 1            # a rounding tie decided the other way, never more
    assert n < a.size // 1000


def test_config4_every_element_agrees_between_tile_geometries(gpu, oracle):
    """C4 whole, bf16 dst with the full chain: 256 x 256 tiles of eight wavefronts against 256 x 128 tiles of four
    (another K loop, another tile order, two workgroups per compute unit): both add the products of a dst element in
    the same order, so every one of the 117 M elements must carry the same bits; the narrow tiles are held to the
    oracle's float64 sums on sampled rows like the wide ones above."""
    p = configs.config4(wtag="ba")
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_f8")
    got = np.asarray(got).copy()
    with cabi.tuning("MI355_F8_TILES", "narrow"):
        other, oname = run_gpu(p, cabi.IMPL_F8_MFMA)
    other = np.asarray(other)
    rows = sample_rows(p.M, 1, 14)
    sub = row_slice(p, rows)
    _, ideal, asum = oracle.run_oracle(sub, want_ideal=True)
    assert assert_gemm_close(sub, rows_of(p, other, rows), ideal, asum, what=oname + " narrow", hw=fp8_mfma_bound(sub)) < 1.0
    assert np.array_equal(got, other), f"{np.count_nonzero(got != other)} of {got.size} elements differ between the geometries"


def test_config5_every_element_row_and_column_sums(gpu):
    """C5 whole with an f32 dst: dst is linear in the operands, so its row sums are src . (weights . 1) and its column
    sums (1 . src) . weights, evaluated here in float64 from the decoded operands.  A sum of 8192 elements carries the
    rounding of its elements only: one element that is wrong by a hundredth of a typical value stands out."""
    from onednn_amd.problem import decode
    p = configs.config5(wtag="ba")
    p.dst_dt = cabi.DT_F32
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_mxf4")
    M, N, K = p.M, p.N, p.K
    D = np.asarray(got).view(np.float32).reshape(M, N).astype(np.float64)

    def operand(raw, scales, rows, k_major_scales):
        v = decode(cabi.DT_F4_E2M1, raw, rows * K).astype(np.float32).reshape(rows, K)
        s = decode(cabi.DT_E8M0, scales, rows * (K // 32)).astype(np.float32)
        s = s.reshape(K // 32, rows).T if k_major_scales else s.reshape(rows, K // 32)
        return (v.reshape(rows, K // 32, 32) * s[:, :, None]).reshape(rows, K)

    S = operand(p.src, p.quant["src_scale"].data, M, False)                 # [M][K]
    Wt = operand(p.wei, p.quant["wei_scale"].data, N, True)                 # [N][K]: weights are K-contiguous
    rs = S.astype(np.float64) @ Wt.astype(np.float64).sum(0)                # dst . 1
    cs = S.astype(np.float64).sum(0) @ Wt.astype(np.float64).T             # 1 . dst
    # Error model of a sum of dst elements.  An element is a float32 K-sum whose partial sums wander like
    # |src row|_2 |wei column|_2 / sqrt(K) (zero-mean data; sum|terms|, the worst case gemm_bound uses, is sqrt(K)
    # times that); each of the K additions rounds by at most half an ulp of the partial sum, independent and
    # uniform: standard deviation (2^-24 / sqrt 3) |src row|_2 |wei column|_2 per element, added in quadrature
    # over a row or column; eight standard deviations, plus the float64 sum's own rounding.
    sn = np.sqrt((S.astype(np.float64) ** 2).sum(1))
    wn = np.sqrt((Wt.astype(np.float64) ** 2).sum(1))
    per_elem = 8 * (2.0 ** -24 / np.sqrt(3.0))
    tol_r = per_elem * sn * np.sqrt((wn ** 2).sum()) + 2.0 ** -40 * np.abs(D).sum(1)
    tol_c = per_elem * wn * np.sqrt((sn ** 2).sum()) + 2.0 ** -40 * np.abs(D).sum(0)
    er, ec = np.abs(D.sum(1) - rs), np.abs(D.sum(0) - cs)
    assert (er <= tol_r).all(), f"row {er.argmax()}: sum off by {er.max()} (bound {tol_r[er.argmax()]})"
    assert (ec <= tol_c).all(), f"column {ec.argmax()}: sum off by {ec.max()} (bound {tol_c[ec.argmax()]})"
    # the check has teeth: one element moved by a hundredth of a typical value breaks its row's and column's bound,
    # and the measured deviations are rounding noise (a tenth of the bound), not a margin eaten up
    typical = np.abs(D).mean()
    assert 1e-2 * typical > tol_r.max() and 1e-2 * typical > tol_c.max()
    print(f"C5 row sums: worst {np.max(er / tol_r):.3f} of the bound, column sums {np.max(ec / tol_c):.3f}; "
          f"bound {tol_r.max():.3f} against a typical |dst| of {typical:.1f}")
