"""MXFP8 dense matmul on hip:mfma_f8: f8 x f8 with e8m0 scales per 32 k on both
operands (`src:per_ocic:e8m0:1x32 + wei:per_ocic:e8m0:32x1`, the reference's MX
tutorial examples/tutorials/matmul/mxfp_matmul.cpp), the scales applied by the
block-scaled matrix instruction.  ref_matmul_t with group_k = 32
(src/cpu/matmul/ref_matmul.cpp:168-236): a block's 32 products are summed, the
sum is multiplied by both scales, the blocks are added up.

On data whose block sums are exact (small integers; powers of two as scales)
every order of the additions gives the same f32, so the device must match the
oracle bit for bit -- with every block given its own scale, a lane that applies
a scale to the wrong block fails.  Random data: within the fp8 matrix-core bound
of tests/helpers.py around the oracle's float64 sum."""
import numpy as np
import pytest

from onednn_amd import cabi
from onednn_amd import dtypes as dtp
from onednn_amd.problem import MatmulProblem, PostOp, QuantParam, run_gpu, strides_for
from onednn_amd.problem import decode
from tests.helpers import assert_bit_exact, assert_gemm_close

MASK_ROW, MASK_COL = 2, 4


def e5m2(v):
    h = np.asarray(v, np.float32).astype(np.float16).view(np.uint16)
    assert not (h & 0xff).any()
    return (h >> 8).astype(np.uint8)


def problem(M, N, K, *, sdt="f8_e4m3", wdt="f8_e4m3", ddt="f32", wtag="ba", exact=True, seed=0, batch=1, bias=False,
            post_ops=None):
    r = np.random.default_rng(seed)
    if exact:
        sv = r.integers(-4, 5, size=(batch, M, K)).astype(np.float32)
        wv = r.integers(-4, 5, size=(batch, K, N)).astype(np.float32)
        ss = r.integers(122, 131, size=(batch, M, K // 32)).astype(np.uint8)
        ws = r.integers(122, 131, size=(batch, K // 32, N)).astype(np.uint8)
    else:
        sv = r.standard_normal((batch, M, K)).astype(np.float32)
        wv = r.standard_normal((batch, K, N)).astype(np.float32)
        ss = r.integers(120, 134, size=(batch, M, K // 32)).astype(np.uint8)
        ws = r.integers(120, 134, size=(batch, K // 32, N)).astype(np.uint8)
    enc = {"f8_e4m3": lambda v: dtp.f32_to_e4m3(v.reshape(-1)).reshape(v.shape), "f8_e5m2": e5m2}
    if not exact:
        enc["f8_e5m2"] = lambda v: (np.asarray(v, np.float32).astype(np.float16).view(np.uint16) >> 8).astype(np.uint8)
    src, wei = enc[sdt](sv), enc[wdt](wv)
    if wtag == "ba":
        wei = np.ascontiguousarray(wei.transpose(0, 2, 1))
    quant = {"src_scale": QuantParam(cabi.DT_E8M0, 1 | MASK_ROW | MASK_COL if batch > 1 else MASK_ROW | MASK_COL, ss, (1, 32)),
             "wei_scale": QuantParam(cabi.DT_E8M0, 1 | MASK_ROW | MASK_COL if batch > 1 else MASK_ROW | MASK_COL, ws, (32, 1))}
    b = r.integers(-8, 9, size=N).astype(np.float32) if bias else None
    return MatmulProblem(M=M, N=N, K=K, batch=batch, src_dt=cabi.DT_NAMES[sdt], wei_dt=cabi.DT_NAMES[wdt],
                         dst_dt=cabi.DT_NAMES[ddt], src=src, wei=wei, wei_stride=strides_for(wtag, batch, K, N),
                         quant=quant, bias_dt=cabi.DT_F32 if bias else cabi.DT_UNDEF, bias=b, post_ops=post_ops or [],
                         name=f"mxf8-{M}x{N}x{K}")


def test_dispatch_rules():
    st, impl = cabi.query(problem(64, 64, 128).desc())
    assert st == cabi.SUCCESS and impl == cabi.IMPL_F8_MFMA
    assert cabi.query(problem(64, 64, 192).desc())[1] == cabi.IMPL_F8_MFMA   # any whole number of 64-byte stages
    assert cabi.query(problem(64, 64, 160).desc())[1] == cabi.IMPL_F8_MFMA   # ... or of blocks: half a stage more
    assert cabi.query(problem(64, 64, 32).desc())[1] == cabi.IMPL_REF        # less than a stage
    p = problem(64, 64, 128)
    p.quant["wei_scale"] = QuantParam(cabi.DT_F32, MASK_COL, np.ones(64, np.float32))   # MX on one side only
    assert cabi.query(p.desc())[1] == cabi.IMPL_REF
    # the packed scales: 256 bytes per stage (two) for two blocks of 128 src rows and four blocks of 64 columns
    assert cabi.scratch_bytes(problem(64, 64, 128).desc()) == (2 + 4) * 2 * 256


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(256, 256, 128), (300, 200, 256), (1, 8, 128), (33, 515, 384), (512, 768, 1024),
                                   (300, 200, 192), (129, 65, 64)])
@pytest.mark.parametrize("sdt,wdt", [("f8_e4m3", "f8_e4m3"), ("f8_e5m2", "f8_e4m3"), ("f8_e4m3", "f8_e5m2"),
                                     ("f8_e5m2", "f8_e5m2")])
def test_exact_data_bit_exact(gpu, oracle, shape, sdt, wdt):
    M, N, K = shape
    p = problem(M, N, K, sdt=sdt, wdt=wdt, seed=M + K)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_f8"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
@pytest.mark.parametrize("wtag", ["ba", "ab"])
def test_exact_data_batched_with_bias_and_relu(gpu, oracle, wtag):
    post = [PostOp(cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"], alpha=0.5)]
    p = problem(100, 136, 256, seed=3, batch=2, bias=True, post_ops=post, wtag=wtag)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_f8"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
@pytest.mark.parametrize("K", [96, 160, 224, 1056])
@pytest.mark.parametrize("wtag", ["ba", "ab"])
def test_a_k_of_an_odd_number_of_blocks(gpu, oracle, K, wtag):
    """K = 64 s + 32: the last block is multiplied by one more step over the row's last 64 bytes, with the block
    before it (multiplied already) zeroed; every block has a scale of its own, so the tail's scale must be the last
    block's."""
    p = problem(300, 328, K, seed=K, wtag=wtag, batch=2 if K == 160 else 1, bias=True)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_f8"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
def test_a_long_k_of_an_odd_number_of_blocks_within_the_bound(gpu, oracle):
    """K = 4064 (63 stages and a block), random data: within the matrix-core bound around the float64 sum."""
    p = problem(320, 448, 4064, exact=False, seed=5)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_f8"), name
    _, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    assert_gemm_close(p, got, ideal, asum, what=name, hw=mx_mfma_bound(p))


@pytest.mark.gpu
def test_the_tail_ignores_the_scale_of_the_block_it_zeroes(gpu, oracle):
    """The block ahead of the tail block is read again and zeroed: a NaN scale (e8m0 0xff) of that block belongs to
    the step before; rows whose scales are finite stay finite."""
    p = problem(64, 96, 160, seed=9)
    ss = p.quant["src_scale"].data.reshape(1, 64, 5).copy()
    ss[0, 7, 3] = 0xff                    # block 3 = k 96 .. 127 of row 7: NaN, in its own step and nowhere else
    p.quant["src_scale"].data = ss
    got, name = run_gpu(p)
    want = oracle.run_oracle(p)
    g, w = np.asarray(got, np.float32).reshape(64, 96), np.asarray(want, np.float32).reshape(64, 96)
    assert np.isnan(g[7]).all() and np.isnan(w[7]).all()
    keep = np.arange(64) != 7
    assert np.array_equal(g[keep], w[keep]) and np.isfinite(g[keep]).all()


def mx_mfma_bound(p):
    """helpers.fp8_mfma_bound for block-scaled operands: the matrix core drops bits below 2^-13 of the largest
    product of a group of eight k; a group lies inside one block of 32, so the block's two scales multiply what is
    lost.  One standard deviation of the same model, over blocks of 32 of the scaled magnitudes, [M, N]."""
    M, N, K = p.M, p.N, p.K
    s = np.abs(decode(p.src_dt, p.src.reshape(-1), M * K).astype(np.float64)).reshape(M, K)
    w = np.abs(decode(p.wei_dt, p.wei.reshape(-1), N * K).astype(np.float64)).reshape(N, K)      # K-contiguous weights
    ss = 2.0 ** (p.quant["src_scale"].data.reshape(M, K // 32).astype(np.float64) - 127)
    ws = 2.0 ** (p.quant["wei_scale"].data.reshape(K // 32, N).astype(np.float64) - 127)
    S = s.reshape(M, K // 32, 32).max(2) * ss
    W = w.reshape(N, K // 32, 32).max(2).T * ws
    return np.sqrt(7.0 / 3.0 * 8.0 * ((S * S) @ (W * W))) * 2.0 ** -13


@pytest.mark.gpu
@pytest.mark.parametrize("ddt", ["f32", "bf16"])
def test_random_data_within_the_matrix_core_bound(gpu, oracle, ddt):
    p = problem(320, 448, 2048, exact=False, seed=4, ddt=ddt)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_f8"), name
    _, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    assert_gemm_close(p, got, ideal, asum, what=name, hw=mx_mfma_bound(p))


@pytest.mark.gpu
def test_block_scales_are_exact_powers_of_two_at_full_k(gpu):
    """A size-independent property at K = 8192 (256 blocks per row): raising every src scale byte by one doubles every
    dst value exactly, and raising the scales of a single block of weights doubles that block's contribution --
    checked through a problem whose other blocks are zero."""
    M, N, K = 512, 1024, 8192
    p1 = problem(M, N, K, exact=False, seed=31)
    p2 = problem(M, N, K, exact=False, seed=31)
    p2.quant["src_scale"].data = (p2.quant["src_scale"].data + 1).astype(np.uint8)
    g1, name = run_gpu(p1)
    g2, _ = run_gpu(p2)
    assert name.startswith("hip:mfma_f8"), name
    a, b = np.asarray(g1, np.float32), np.asarray(g2, np.float32)
    assert np.isfinite(a).all() and np.array_equal(b, a * np.float32(2))
    # one block of K alive: block 100 of the weights (k 3200 .. 3231); its scale raised by one doubles dst
    p3 = problem(M, N, K, exact=False, seed=31)
    w = p3.wei.reshape(1, N, K).copy()
    keep = w[:, :, 3200:3232].copy()
    w[:] = 0
    w[:, :, 3200:3232] = keep
    p3.wei = w
    g3, _ = run_gpu(p3)
    p3.quant["wei_scale"].data = p3.quant["wei_scale"].data.copy()
    p3.quant["wei_scale"].data.reshape(1, K // 32, N)[:, 100, :] += 1
    g4, _ = run_gpu(p3)
    a, b = np.asarray(g3, np.float32), np.asarray(g4, np.float32)
    assert np.abs(a).max() > 0 and np.array_equal(b, a * np.float32(2))
    # ... and the scales of any other block change nothing
    p3.quant["wei_scale"].data.reshape(1, K // 32, N)[:, 101, :] += 3
    g5, _ = run_gpu(p3)
    assert np.array_equal(np.asarray(g5, np.float32), b)
