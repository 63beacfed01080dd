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


@pytest.mark.parametrize("dst", ["bf16", "f32"])
def test_config4_full_size_sampled_rows(gpu, oracle, dst):
    # against the oracle's float64 K-sums with bias, gelu_tanh and the residual in float64 on top:
    # bound = 4 standard deviations of the float32 summation error model (tests/helpers.py gemm_bound)
    # plus the matrix cores' fp8 alignment loss (fp8_mfma_bound), together about 0.1 on pre-activations
    # of standard deviation 90, carried through the chain; with the f32 dst nothing else is inside it,
    # the bf16 dst adds half a unit in its last place
    p = configs.config4(wtag="ba")
    p.dst_dt = cabi.DT_NAMES[dst]
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
