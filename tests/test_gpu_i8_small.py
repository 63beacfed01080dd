"""hip:mfma_i8 on shapes its 256 x 256 tiles do not fit: a handful of tiles
(32 x 32 tiles that compute their own row / column sums) and a K that is not a
multiple of the 64-byte stage (steps beyond K filled with the operand's zero).
Integer accumulation and one rounding per written operation: bit for bit
against the oracle."""
import numpy as np
import pytest

from onednn_amd import cabi, configs
from onednn_amd.problem import MatmulProblem, PostOp, QuantParam, run_gpu, strides_for
from tests.helpers import assert_bit_exact

pytestmark = pytest.mark.gpu


def int8_problem(M, N, K, src_dt, wei_dt, dst_dt, wtag="ba", batch=1, src_zp=None, wei_zp=False, scales=True,
                 bias=False, post_ops=(), dst_scale=None, seed=31, wei_batch=True):
    r = np.random.default_rng(seed)
    lo = {cabi.DT_S8: -128, cabi.DT_U8: 0}
    np_dt = {cabi.DT_S8: np.int8, cabi.DT_U8: np.uint8}
    src = r.integers(lo[src_dt], lo[src_dt] + 256, size=(batch, M, K)).astype(np_dt[src_dt])
    wb = batch if wei_batch else 1
    wei = r.integers(lo[wei_dt], lo[wei_dt] + 256, size=(wb, K, N)).astype(np_dt[wei_dt])
    if wtag == "ba":
        wei = np.ascontiguousarray(np.swapaxes(wei, 1, 2))
    ws = list(strides_for(wtag, wb, K, N))
    if not wei_batch:
        ws[0] = 0
    quant = {}
    if src_zp is not None:
        quant["src_zp"] = QuantParam(cabi.DT_S32, configs.MASK_COMMON, np.array([src_zp], np.int32))
    if wei_zp:
        quant["wei_zp"] = QuantParam(cabi.DT_S8, configs.MASK_COL, r.integers(-20, 21, size=N).astype(np.int8))
    if scales:
        quant["src_scale"] = QuantParam(cabi.DT_F32, configs.MASK_COMMON, np.array([0.0173], np.float32))
        quant["wei_scale"] = QuantParam(cabi.DT_F32, configs.MASK_COL, r.uniform(1e-3, 1e-2, size=N).astype(np.float32))
    if dst_scale is not None:
        quant["dst_scale"] = QuantParam(cabi.DT_F32, configs.MASK_COMMON, np.array([dst_scale], np.float32))
    b = r.uniform(-1, 1, size=N).astype(np.float32) if bias else None
    return MatmulProblem(M=M, N=N, K=K, batch=batch, src_dt=src_dt, wei_dt=wei_dt, dst_dt=dst_dt, src=src, wei=wei,
                         wei_stride=tuple(ws), quant=quant, bias_dt=cabi.DT_F32 if bias else cabi.DT_UNDEF, bias=b,
                         post_ops=list(post_ops), name=f"i8 {M}x{K}x{N}")


def test_config1_runs_on_the_small_tiles_in_one_kernel(gpu, oracle):
    # the headline small configuration with the weights layout format_tag::any
    # resolves to: no scratch (no layout change, no sum kernels)
    p = configs.config1(wtag="ba")
    d = p.desc()
    st, impl = cabi.query(d, cabi.IMPL_AUTO)
    assert st == cabi.SUCCESS and cabi.impl_name(impl).startswith("hip:mfma_i8")
    assert cabi.scratch_bytes(d) == 0
    got, name = run_gpu(p)
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.parametrize("K", [16, 48, 80, 4000])
@pytest.mark.parametrize("src_dt,wei_dt", [(cabi.DT_U8, cabi.DT_S8), (cabi.DT_S8, cabi.DT_U8), (cabi.DT_S8, cabi.DT_S8),
                                           (cabi.DT_U8, cabi.DT_U8)])
def test_k_that_is_no_multiple_of_the_stage(gpu, oracle, K, src_dt, wei_dt):
    p = int8_problem(70, 130, K, src_dt, wei_dt, cabi.DT_F32, src_zp=3, wei_zp=True, bias=True)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_i8"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


def test_k_4000_at_a_size_the_large_tiles_would_take(gpu, oracle):
    # 32 tiles of 256 x 256 and batch 2: only K keeps it from the large tiles
    p = int8_problem(1024, 1024, 4000, cabi.DT_S8, cabi.DT_S8, cabi.DT_S8, batch=2,
                     post_ops=[PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"])], dst_scale=0.37)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_i8"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.parametrize("shape", [(1, 1, 64), (1, 33, 128), (31, 1, 192), (33, 65, 256), (256, 1024, 1024)])
@pytest.mark.parametrize("dst_dt", [cabi.DT_S32, cabi.DT_BF16, cabi.DT_U8])
def test_small_tiles_edges_and_dst_types(gpu, oracle, shape, dst_dt):
    M, N, K = shape
    scales = dst_dt != cabi.DT_S32
    p = int8_problem(M, N, K, cabi.DT_U8, cabi.DT_S8, dst_dt, src_zp=128, wei_zp=True, scales=scales, bias=scales,
                     dst_scale=3.1 if dst_dt == cabi.DT_U8 else None)
    with cabi.tuning("MI355_I8_TILES", "small"):
        got, name = run_gpu(p, cabi.IMPL_I8_MFMA)
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.parametrize("wtag", ["ab", "ba"])
@pytest.mark.parametrize("wei_batch", [True, False])
def test_small_tiles_batched_and_broadcast_weights(gpu, oracle, wtag, wei_batch):
    p = int8_problem(50, 72, 320, cabi.DT_U8, cabi.DT_S8, cabi.DT_F32, wtag=wtag, batch=3, src_zp=7, wei_zp=True,
                     wei_batch=wei_batch)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_i8"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.parametrize("src_dt,wei_dt", [(cabi.DT_U8, cabi.DT_U8), (cabi.DT_U8, cabi.DT_S8), (cabi.DT_S8, cabi.DT_U8)])
@pytest.mark.parametrize("dst_dt", [cabi.DT_S32, cabi.DT_S8])
def test_both_tile_geometries_against_the_oracle_with_re_biased_operands(gpu, oracle, src_dt, wei_dt, dst_dt):
    # rows 128 .. 255 of a large tile belong to the wavefronts whose first
    # iteration multiplies placeholder fragments: those must be the operand's
    # zero (0x80 for u8), or u8 x u8 gains 64 * 128 * 128 per element there
    raw = dst_dt == cabi.DT_S32
    p = int8_problem(300, 520, 512, src_dt, wei_dt, dst_dt, src_zp=100, wei_zp=True, scales=not raw,
                     dst_scale=None if raw else 60.0)
    want = oracle.run_oracle(p)
    if not raw:
        w = np.asarray(want).view(np.int8)
        assert np.mean(np.abs(w.astype(np.int32)) < 127) > 0.9      # not saturated away
    outs = []
    for tiles in ("large", "wide", "small"):
        with cabi.tuning("MI355_I8_TILES", tiles):
            got, name = run_gpu(p, cabi.IMPL_I8_MFMA)
        assert_bit_exact(p, got, want, f"{name} {tiles}")
        outs.append(np.asarray(got).copy())
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


@pytest.mark.gpu
@pytest.mark.parametrize("src_dt", [cabi.DT_S8, cabi.DT_U8])
def test_mid_size_problems_on_the_dispatchers_own_choice(gpu, oracle, src_dt):
    """30 large tiles (24 to 128 take the 256 x 128 LDS tiles by themselves), ragged in M and N: against the oracle, and
    the same bits from the 256 x 256 tiles"""
    cabi.tuning_set("MI355_I8_TILES", None)
    p = int8_problem(1500, 1100, 192, src_dt, cabi.DT_S8, cabi.DT_S8, src_zp=7 if src_dt == cabi.DT_U8 else None,
                     dst_scale=40.0, bias=True)
    want = oracle.run_oracle(p)
    got, name = run_gpu(p, cabi.IMPL_I8_MFMA)
    assert_bit_exact(p, got, want, name)
    with cabi.tuning("MI355_I8_TILES", "wide"):
        wide, name = run_gpu(p, cabi.IMPL_I8_MFMA)
    assert np.array_equal(np.asarray(got), np.asarray(wide))
