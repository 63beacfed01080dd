"""A K that is not whole 64-byte stages on the fp8 matrix-core tiles.

The reference's brgemm path blocks any K (src/cpu/x64/matmul/brgemm_matmul_utils.cpp:117-330); here the LDS-tile GEMM
core steps through K in stages of 64 bytes per row, and the rest of a K that is whole 16-byte chunks is multiplied by
one more, unpipelined step per tile (the stage's last 64 bytes with the chunks that were multiplied before zeroed).
Exact data (small integers: every product and partial sum is exact in f32, any order gives the same bits) must match
the oracle bit for bit, with K tails of one, two and three chunks, on both tile geometries and for every pair of fp8
formats; random data within the summation bound of tests/helpers.py.
"""
import numpy as np
import pytest

from onednn_amd import cabi, configs
from onednn_amd import dtypes as dtp
from onednn_amd.problem import MatmulProblem, PostOp, QuantParam, run_gpu, strides_for
from tests.helpers import assert_bit_exact, assert_gemm_close, fp8_mfma_bound

E4M3, E5M2 = cabi.DT_F8_E4M3, cabi.DT_F8_E5M2


def test_dispatch_rules():
    def impl(K, **kw):
        p = exact_problem(64, 64, K, **kw)
        st, i = cabi.query(p.desc())
        assert st == cabi.SUCCESS
        return cabi.impl_name(i)
    assert impl(4000).startswith("hip:mfma_f8")          # 62 stages and 32 bytes
    assert impl(80).startswith("hip:mfma_f8")            # one stage and one chunk
    assert impl(64).startswith("hip:mfma_f8")
    assert impl(48).startswith("hip:ref")                # less than a stage
    assert impl(72).startswith("hip:ref")                # not whole chunks


def to_e5m2(x):
    """exactly representable values -> e5m2 bytes (the top byte of their f16 encoding)"""
    return (np.asarray(x, np.float16).view(np.uint16) >> 8).astype(np.uint8)


def exact_problem(M, N, K, src_dt=E4M3, wei_dt=E4M3, dst_dt=cabi.DT_F32, wtag="ba", seed=3, batch=1, post=False):
    r = np.random.default_rng(seed + K)
    enc = {E4M3: lambda v: dtp.f32_to_e4m3(v.astype(np.float32).reshape(-1)), E5M2: lambda v: to_e5m2(v).reshape(-1)}
    S = r.integers(-3, 4, size=(batch, M, K))
    W = r.integers(-2, 3, size=(batch, N, K) if wtag == "ba" else (batch, K, N))
    bias = (r.integers(-64, 65, size=N) / 16.0).astype(np.float32)
    quant = {"src_scale": QuantParam(cabi.DT_F32, 0, np.array([0.5], np.float32)),
             "wei_scale": QuantParam(cabi.DT_F32, configs.MASK_COL, r.choice([0.25, 0.5, 1.0, 2.0], size=N).astype(np.float32))}
    po = [PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"])] if post else []
    return MatmulProblem(M=M, N=N, K=K, batch=batch, src_dt=src_dt, wei_dt=wei_dt, dst_dt=dst_dt, src=enc[src_dt](S),
                         wei=enc[wei_dt](W), wei_stride=strides_for(wtag, batch, K, N), bias_dt=cabi.DT_F32, bias=bias,
                         quant=quant, post_ops=po, name=f"f8-ktail-{K}")


@pytest.mark.gpu
@pytest.mark.parametrize("K", [80, 96, 112, 464, 4000])
@pytest.mark.parametrize("tiles", [None, "wide"])
def test_exact_data_bit_exact(gpu, oracle, K, tiles):
    p = exact_problem(300, 328, K, post=True)
    with cabi.tuning("MI355_F8_TILES", tiles):
        got, name = run_gpu(p)
    assert name.startswith("hip:mfma_f8"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), f"{name} {tiles}")


@pytest.mark.gpu
@pytest.mark.parametrize("src_dt,wei_dt", [(E4M3, E5M2), (E5M2, E4M3), (E5M2, E5M2)])
@pytest.mark.parametrize("wtag", ["ab", "ba"])
def test_format_pairs_layouts_and_batches(gpu, oracle, src_dt, wei_dt, wtag):
    p = exact_problem(70, 136, 208, src_dt=src_dt, wei_dt=wei_dt, dst_dt=cabi.DT_BF16, wtag=wtag, batch=2)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_f8"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
def test_a_nan_in_the_bytes_multiplied_twice_stays_in_its_row(gpu, oracle):
    """the tail step reloads bytes the last whole stage held; zeroed in both operands they add nothing, not even for a
    NaN: only the row (column) that holds one becomes NaN, as in the reference's sum"""
    p = exact_problem(64, 64, 96)
    src = np.asarray(p.src).copy().reshape(64, 96)
    src[5, 40] = 0x7f                     # e4m3 NaN, inside the reloaded 32 bytes
    p.src = src.reshape(-1)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_f8"), name
    g = np.asarray(got).view(np.float32).reshape(64, 64)
    assert np.isnan(g[5]).all() and not np.isnan(np.delete(g, 5, 0)).any()
    w = np.asarray(oracle.run_oracle(p)).view(np.float32).reshape(64, 64)
    assert np.array_equal(np.delete(g, 5, 0), np.delete(w, 5, 0))


@pytest.mark.gpu
@pytest.mark.parametrize("dst", ["f32", "bf16"])
def test_random_data_within_the_summation_bound(gpu, oracle, dst):
    """C4's data and chain at K = 4000: against the oracle's float64 sums"""
    p = configs.config4(M=384, N=640, K=4000, wtag="ba")
    p.dst_dt = cabi.DT_NAMES[dst]
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_f8"), name
    _, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    assert assert_gemm_close(p, got, ideal, asum, what=name, hw=fp8_mfma_bound(p)) < 1.0


# ---------------------------------------------------------------- MXFP4: K in whole blocks of 32, not whole stages of 128

def test_mxfp4_dispatch_rules():
    def impl(K):
        st, i = cabi.query(configs.config5(M=64, N=64, K=K).desc())
        assert st == cabi.SUCCESS
        return cabi.impl_name(i)
    assert impl(4064).startswith("hip:mfma_mxf4")        # 31 stages and three blocks
    assert impl(160).startswith("hip:mfma_mxf4")         # one stage and one block
    assert impl(96).startswith("hip:ref")                # less than a stage


@pytest.mark.gpu
@pytest.mark.parametrize("K", [160, 192, 224, 4064])
@pytest.mark.parametrize("wtag", ["ba", "ab"])
def test_mxfp4_tail_blocks(gpu, oracle, K, wtag):
    """C5's data at a K that ends one, two or three blocks into a stage: within the bound of the cross-block f32
    additions (block dots are exact, scales are powers of two), f32 and bf16 dst; and bit for bit when all scales are
    equal and the sums stay exactly representable"""
    p = configs.config5(M=300, N=328, K=K, wtag=wtag)
    _, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    for dst in (cabi.DT_F32, cabi.DT_BF16):
        p.dst_dt = dst
        got, name = run_gpu(p)
        assert name.startswith("hip:mfma_mxf4"), name
        assert_gemm_close(p, got, ideal, asum, what=f"{name} K={K}")
    if K < 1024:
        q = configs.config5(M=300, N=328, K=K, wtag=wtag)
        q.dst_dt = cabi.DT_F32
        q.quant["src_scale"].data[:] = 127
        q.quant["wei_scale"].data[:] = 126
        got, name = run_gpu(q)
        assert_bit_exact(q, got, oracle.run_oracle(q), name)


@pytest.mark.gpu
def test_mxfp4_tail_scales_belong_to_their_blocks(gpu, oracle):
    """one block of one row scaled up by 16: the result tells whether every block of the tail stage met its own
    scale (the tail stage's scales are the row's last four blocks, not the four after the last whole stage)"""
    K = 224
    p = configs.config5(M=64, N=64, K=K)
    p.dst_dt = cabi.DT_F32
    p.quant["src_scale"].data[:] = 127
    p.quant["wei_scale"].data[:] = 127
    want0 = np.asarray(oracle.run_oracle(p)).view(np.float32).reshape(64, 64).copy()
    for blk in range(K // 32):
        q = configs.config5(M=64, N=64, K=K)
        q.dst_dt = cabi.DT_F32
        q.quant["src_scale"].data[:] = 127
        q.quant["wei_scale"].data[:] = 127
        q.quant["src_scale"].data.reshape(64, K // 32)[7, blk] = 131     # x 16: every sum stays exactly representable
        got, name = run_gpu(q)
        assert name.startswith("hip:mfma_mxf4"), name
        assert_bit_exact(q, got, oracle.run_oracle(q), f"{name} block {blk}")
        g = np.asarray(got).view(np.float32).reshape(64, 64)
        assert np.array_equal(np.delete(g, 7, 0), np.delete(want0, 7, 0))
