"""Weight-only quantization beyond the decode kernels' 32 rows (prefill): bf16 src x
s4 / u4 / s8 / u8 weights with scales and zero points along K and N, fpmath
apply_to_int -- on hip:mfma_h16, whose weights copy is written by the reorder
with the weights' scales and zero points as its parameters ((w - zp) * scale
rounded to bf16: the flavour of the reference's JIT path,
brgemm_matmul_copy_utils.cpp:2870-2896, the oracle's FLAG_WEI_BF16) and the
16-bit tiles multiply.

Exact data (small integer src, power-of-two scales: every decompressed weight
and every partial sum is exact, in bf16 and in f32) must match the oracle bit for
bit in either flavour; random data are held to the f32 summation bound around
the oracle's float64 sum of the bf16-rounded weights."""
import numpy as np
import pytest

from onednn_amd import cabi, configs
from onednn_amd import dtypes as dtp
from onednn_amd.problem import run_gpu
from tests.helpers import assert_bit_exact, assert_gemm_close


def exact(p, seed=0):
    """small integer src; scales replaced by powers of two of the same type"""
    r = np.random.default_rng(seed)
    p.src = dtp.f32_to_bf16(r.integers(-4, 5, size=p.M * p.K).astype(np.float32)).reshape(p.M, p.K)
    if "wei_scale" in p.quant:
        q = p.quant["wei_scale"]
        v = (2.0 ** r.integers(-6, -1, size=np.asarray(q.data).size)).astype(np.float32)
        q.data = {cabi.DT_F32: v, cabi.DT_BF16: dtp.f32_to_bf16(v),
                  cabi.DT_F16: v.astype(np.float16).view(np.uint16)}[q.dt].reshape(np.asarray(q.data).shape)
    return p


def test_dispatch_rules():
    p = configs.woq_variant(64, 256, 256, 128)
    st, impl = cabi.query(p.desc())
    assert st == cabi.SUCCESS and impl == cabi.IMPL_H16_MFMA
    assert cabi.scratch_bytes(p.desc()) == 256 * 256 * 2                       # the decompressed weights, K-contiguous
    assert cabi.query(configs.woq_variant(32, 256, 256, 128).desc())[1] == cabi.IMPL_WOQ_GEMV   # decode sizes stay
    p = configs.woq_variant(64, 256, 256, 128)
    p.apply_to_int = False
    assert cabi.query(p.desc())[1] != cabi.IMPL_H16_MFMA


VARIANTS = [
    dict(),                                                       # u4, bf16 scales and u4 zero points per group of 128
    dict(wei_dt="s4", sc_dt="f32", zp_dt="s8"),
    dict(sc_dt="f16", zp_dt="s32", zp_kind="column"),
    dict(sc_kind="column", zp_kind="common", zp_dt="u8"),
    dict(zp_kind="none"),
    dict(sc_kind="none", zp_kind="none"),
    dict(dst_dt="f32", relu_bias=True),
]


@pytest.mark.gpu
@pytest.mark.parametrize("kw", VARIANTS, ids=[str(i) for i in range(len(VARIANTS))])
@pytest.mark.parametrize("shape", [(64, 256, 256, 128), (300, 192, 512, 64), (33, 130, 96, 32), (96, 512, 384, 64)])
def test_exact_data_bit_exact(gpu, oracle, kw, shape):
    """N in whole 256s with K in whole 64s takes the dedicated decompression kernel, everything else the reorder"""
    M, N, K, G = shape
    p = exact(configs.woq_variant(M, N, K, G, **kw), seed=M)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)
    assert_bit_exact(p, got, oracle.run_oracle(p, flags=oracle.FLAG_WEI_BF16), name)


@pytest.mark.gpu
@pytest.mark.parametrize("wtag", ["ab", "ba"])
def test_c2_shape_at_prefill_sizes(gpu, oracle, wtag):
    """the decode configuration's tensors at M = 256 (N and K reduced): random data against the float64 sum of the
    bf16-rounded weights"""
    p = configs.config2(M=256, N=1024, K=1024, wtag=wtag)
    p.dst_dt = cabi.DT_F32
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    _, ideal, asum = oracle.run_oracle(p, flags=oracle.FLAG_WEI_BF16, want_ideal=True)
    assert_gemm_close(p, got, ideal, asum, what=name)


@pytest.mark.gpu
@pytest.mark.parametrize("kw", VARIANTS, ids=[str(i) for i in range(len(VARIANTS))])
@pytest.mark.parametrize("shape", [(64, 72, 512, 64), (80, 300, 768, 256), (48, 96, 192, 64)])
def test_k_contiguous_weights(gpu, oracle, kw, shape):
    """two k per byte: K in whole 256s takes the dedicated kernel without the transposition, the last shape the reorder"""
    M, N, K, G = shape
    p = exact(configs.woq_variant(M, N, K, G, wtag="ba", **kw), seed=N)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)
    assert_bit_exact(p, got, oracle.run_oracle(p, flags=oracle.FLAG_WEI_BF16), name)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(64, 256, 256, 128), (40, 200, 96, 32)])
def test_f16_src(gpu, oracle, shape):
    """f16 src: the weights are decompressed to f16 (exact data, so the oracle's f32 weights are the same numbers)"""
    M, N, K, G = shape
    p = exact(configs.woq_variant(M, N, K, G, sc_dt="f16", zp_dt="s8", dst_dt="f32"), seed=3)
    p.src_dt = cabi.DT_F16
    p.src = dtp.bf16_to_f32(p.src).astype(np.float16).view(np.uint16).reshape(M, K)
    p.fpmath_mode = 2
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
def test_int8_weights(gpu, oracle):
    M, N, K = 128, 192, 256
    r = np.random.default_rng(5)
    p = configs.woq_variant(M, N, K, 128, sc_dt="f32", zp_dt="s8")
    p.wei_dt = cabi.DT_S8
    p.wei = r.integers(-128, 128, size=(K, N), dtype=np.int8)
    p = exact(p, seed=6)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
def test_decode_and_prefill_of_the_same_weights_differ_by_the_weight_rounding_only(gpu):
    """M <= 32 runs the decode kernels ((w - zp) * scale kept in f32, like ref_matmul_t), M > 32 the 16-bit tiles on
    weights decompressed and rounded to bf16 (the JIT flavour): the same src rows against the same weights differ by
    the bf16 rounding of each dequantized weight -- at most 2^-9 relative per weight -- plus the two f32 summations'
    own rounding.  Bounds the batch-size dependence INTEGRATION.md describes."""
    from tests.helpers import decode_terms, gemm_bound
    N, K = 512, 1024
    big = configs.config2(M=64, N=N, K=K)
    big.dst_dt = cabi.DT_F32
    small = configs.config2(M=32, N=N, K=K)
    small.dst_dt = cabi.DT_F32
    src = np.asarray(big.src).reshape(64, K)
    small.src = np.ascontiguousarray(src[:32]).reshape(np.asarray(small.src).shape)
    for name in ("wei", "quant"):
        setattr(small, name, getattr(big, name))        # the same weights, scales and zero points
    g_small, n_small = run_gpu(small)
    g_big, n_big = run_gpu(big)
    assert n_small.startswith("hip:woq") and n_big.startswith("hip:mfma_h16"), (n_small, n_big)
    a = np.asarray(g_small).view(np.float32).reshape(32, N).astype(np.float64)
    b = np.asarray(g_big).view(np.float32).reshape(64, N)[:32].astype(np.float64)
    s, wz, G, sc, _ = decode_terms(small)                                   # src [32, K], w - zp [K, N], scales [K/G, N]
    wdeq = np.abs(wz * np.repeat(sc, G, 0))                                 # |(w - zp) * scale|
    asum = np.abs(s) @ wdeq                                                 # sum |src| |dequantized weight|
    tol = 2.0 ** -9 * asum + 2 * gemm_bound(K, asum)
    err = np.abs(a - b)
    assert (err <= tol).all(), f"worst {np.max(err / tol):.2f} of the bound"
    assert err.max() > 0                                                    # the two flavours do differ


@pytest.mark.gpu
def test_the_decompressed_weights_themselves(gpu):
    """src = identity, so dst is the weights copy the launch wrote: (w - zp) * scale rounded to bf16 the way the
    reference rounds (nearest even; f32 subnormals flush to zero, bfloat16.cpp:29-49).  A third of the scale groups
    are f32 subnormals, so those wavefronts of the decompression kernel leave the hardware conversion for the
    software one; the others stay on it.  Every element against numpy."""
    M = N = K = 256
    p = configs.woq_variant(M, N, K, 64, sc_dt="f32", zp_dt="u8")
    p.src = dtp.f32_to_bf16(np.eye(M, dtype=np.float32).reshape(-1)).reshape(M, K)
    sc = np.asarray(p.quant["wei_scale"].data).copy().reshape(K // 64, N)
    sc[1] = np.float32(2.0 ** -140)                      # subnormal products (flushed by the conversion)
    sc[2, ::2] = np.float32(3.0e-39)                     # subnormal scales next to normal ones
    p.quant["wei_scale"].data = sc
    st, impl = cabi.query(p.desc())
    assert st == cabi.SUCCESS and impl == cabi.IMPL_H16_MFMA
    got = dtp.bf16_to_f32(np.asarray(run_gpu(p)[0]).view(np.uint16).reshape(-1)).reshape(M, N)
    codes = dtp.unpack_nibbles(np.asarray(p.wei).reshape(-1), K * N).reshape(K, N).astype(np.int32)
    zp = np.asarray(p.quant["wei_zp"].data).reshape(K // 64, N).astype(np.int32)
    w = ((codes - zp.repeat(64, axis=0)).astype(np.float32) * sc.repeat(64, axis=0)).astype(np.float32)
    want = dtp.bf16_to_f32(dtp.f32_to_bf16(w.reshape(-1))).reshape(K, N)
    assert np.array_equal(got, want)
    assert np.all(want[64:128] == 0) and np.any(want[:64] != 0)
