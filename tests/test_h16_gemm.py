"""hip:mfma_h16 -- bf16 x bf16, f16 x f16 and f32 x f32 matmul on the matrix-core tiles
(ref_matmul_t's f32 sum of exact products, src/cpu/matmul/ref_matmul.cpp:168-331).

Dispatch rules need no device.  On the device: data whose every partial sum is
exact in f32 (small integers, power-of-two scales) must match the oracle bit
for bit whatever the order of the sum -- that pins the operand layout, the
K-chunk pairing, ragged edges, batches and the epilogue; random data are held to
the forward error bound of an f32 K-sum (helpers.gemm_bound) around the
oracle's float64 sum; the full-size shape is checked against the generic
kernel."""
import numpy as np
import pytest

from onednn_amd import cabi
from onednn_amd import dtypes as dtp
from onednn_amd.problem import MatmulProblem, PostOp, QuantParam, run_gpu, strides_for
from tests.helpers import assert_bit_exact, assert_gemm_close

DT = cabi.DT_NAMES
MASK_COMMON, MASK_ROW, MASK_COL = 0, 2, 4


def enc(v, dt):
    v = np.asarray(v, np.float32)
    if dt == "f32":
        return v
    if dt == "bf16":
        return dtp.f32_to_bf16(v.reshape(-1)).reshape(v.shape)
    return v.astype(np.float16).view(np.uint16)


def problem(M, N, K, dt, ddt, *, batch=1, wtag="ba", exact=True, seed=0, bias=False, post_ops=None, quant=None,
            dst_init=None, wei_batch=True):
    r = np.random.default_rng(seed)
    if exact:
        sv = r.integers(-4, 5, size=(batch, M, K)).astype(np.float32)
        wv = r.integers(-4, 5, size=(batch if wei_batch else 1, K, N)).astype(np.float32)
    else:
        sv = r.standard_normal((batch, M, K)).astype(np.float32)
        wv = r.standard_normal((batch if wei_batch else 1, K, N)).astype(np.float32)
    src = enc(sv, dt)
    wei = enc(wv, dt)
    if wtag == "ba":
        wei = np.ascontiguousarray(wei.transpose(0, 2, 1))
    ws = list(strides_for(wtag, batch, K, N))
    if not wei_batch:
        ws[0] = 0
    b = None
    if bias:
        b = r.integers(-8, 9, size=N).astype(np.float32) if exact else r.uniform(-1, 1, size=N).astype(np.float32)
    return MatmulProblem(M=M, N=N, K=K, batch=batch, src_dt=DT[dt], wei_dt=DT[dt], dst_dt=DT[ddt], src=src, wei=wei,
                         wei_stride=tuple(ws), bias_dt=cabi.DT_F32 if bias else cabi.DT_UNDEF, bias=b,
                         post_ops=post_ops or [], quant=quant or {}, dst_init=dst_init, name=f"h16-{dt}-{ddt}-{M}x{N}x{K}")


# ------------------------------------------------------------------ dispatch (no device)
def test_dispatch_rules():
    q = lambda p: cabi.query(p.desc())  # noqa: E731
    st, impl = q(problem(64, 64, 64, "bf16", "f32"))
    assert st == cabi.SUCCESS and impl == cabi.IMPL_H16_MFMA
    assert cabi.impl_name(impl).startswith("hip:mfma_h16")
    assert q(problem(64, 64, 64, "f16", "f16"))[1] == cabi.IMPL_H16_MFMA
    assert q(problem(64, 64, 16, "f32", "f32"))[1] == cabi.IMPL_H16_MFMA           # f32: stages of 16 k
    assert q(problem(64, 64, 24, "f32", "f32"))[1] == cabi.IMPL_H16_MFMA          # ... 24 -> 32
    assert cabi.scratch_bytes(problem(64, 64, 24, "f32", "f32").desc()) == 2 * 64 * 32 * 4
    assert q(problem(1, 8, 32, "bf16", "bf16"))[1] == cabi.IMPL_H16_MFMA          # any M, N; K in stages of 32
    p = problem(64, 64, 48, "bf16", "f32")                                        # K not in whole stages: padded copies
    assert q(p)[1] == cabi.IMPL_H16_MFMA and cabi.scratch_bytes(p.desc()) == 2 * 64 * 64 * 2
    p = problem(64, 64, 64, "bf16", "f32", wtag="ab")                             # row-major weights: copied K-contiguous
    assert q(p)[1] == cabi.IMPL_H16_MFMA and cabi.scratch_bytes(p.desc()) == 64 * 64 * 2
    assert cabi.scratch_bytes(problem(64, 64, 64, "bf16", "f32").desc()) == 0
    p = problem(64, 64, 64, "bf16", "f32")
    p.wei_dt = cabi.DT_F16                                                       # mixed operand types
    assert q(p)[1] != cabi.IMPL_H16_MFMA
    p = problem(64, 64, 64, "bf16", "f32", quant={"src_zp": QuantParam(cabi.DT_S32, MASK_COMMON, np.array([1], np.int32))})
    assert q(p)[1] != cabi.IMPL_H16_MFMA
    p = problem(64, 64, 64, "bf16", "f32")
    p.impl = cabi.IMPL_H16_MFMA
    assert cabi.query(p.desc())[0] == cabi.SUCCESS
    p = problem(64, 64, 64, "bf16", "f32")
    p.wei_stride = (64 * 64 * 4, 2, 128)                                         # neither dim of the weights contiguous
    p.impl = cabi.IMPL_H16_MFMA
    assert cabi.query(p.desc())[0] == cabi.UNIMPLEMENTED


# ------------------------------------------------------------------ device
SHAPES = [(256, 256, 64), (300, 200, 96), (1, 8, 32), (33, 515, 160), (512, 768, 1024), (257, 255, 32)]


@pytest.mark.gpu
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dt,ddt", [("bf16", "f32"), ("bf16", "bf16"), ("f16", "f16"), ("f16", "f32"), ("f32", "f32"),
                                    ("f32", "bf16")])
def test_exact_data_bit_exact(gpu, oracle, shape, dt, ddt):
    M, N, K = shape
    # keep |sum| small enough for an exact 16-bit dst: |values| <= 4, K <= 1024 -> |sum| <= 16384 would not be,
    # so the 16-bit dst cases scale the sum down by a power of two
    post = [PostOp(cabi.PO_ELTWISE, alg=cabi.ELTWISE["linear"], alpha=2.0 ** -8, beta=0.0)] if ddt != "f32" else []
    p = problem(M, N, K, dt, ddt, seed=K + M, post_ops=post)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(300, 520, 256), (64, 256, 128), (257, 300, 64)])
@pytest.mark.parametrize("dt,ddt", [("bf16", "f32"), ("bf16", "bf16"), ("f16", "f16")])
def test_wide_tiles_on_small_problems(gpu, oracle, shape, dt, ddt):
    """problems of at most 128 large tiles take 256 x 128 tiles by themselves (every other test shape here but the
    f32 ones does); MI355_H16_TILES=wide puts them on the 256 x 256 tiles the large problems run on: the same bits"""
    M, N, K = shape
    post = [PostOp(cabi.PO_ELTWISE, alg=cabi.ELTWISE["linear"], alpha=2.0 ** -8, beta=0.0)] if ddt != "f32" else []
    p = problem(M, N, K, dt, ddt, seed=K + M, post_ops=post, bias=True)
    want = oracle.run_oracle(p)
    narrow, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, narrow, want, name)
    with cabi.tuning("MI355_H16_TILES", "wide"):
        wide, name = run_gpu(p)
    assert_bit_exact(p, wide, want, name + " wide")


@pytest.mark.gpu
@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
def test_exact_data_with_scales_bias_and_post_ops(gpu, oracle, dt):
    M, N, K = 130, 190, 128
    r = np.random.default_rng(5)
    quant = {"src_scale": QuantParam(cabi.DT_F32, MASK_COMMON, np.array([0.5], np.float32)),
             "wei_scale": QuantParam(cabi.DT_F32, MASK_COL, (2.0 ** r.integers(-3, 2, size=N)).astype(np.float32))}
    add = r.integers(-16, 17, size=(M, N)).astype(np.float32)
    post = [PostOp(cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"], alpha=0.25),
            PostOp(cabi.PO_BINARY, alg=cabi.BINARY["add"], dt=cabi.DT_F32, stride=(0, N, 1), data=add),
            PostOp(cabi.PO_SUM, scale=0.5)]
    init = r.integers(-32, 33, size=M * N).astype(np.float32)
    p = problem(M, N, K, dt, "f32", seed=6, bias=True, post_ops=post, quant=quant, dst_init=init)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(256, 256, 64), (300, 200, 96), (33, 520, 160), (512, 768, 1024)])
@pytest.mark.parametrize("chain", ["none", "bias", "residual", "bias+residual"])
def test_bf16_dst_with_bias_and_residual(gpu, oracle, shape, chain):
    """bf16 dst with a bias and / or a bf16 residual add (the transformer layer's chain): exact sums round to bf16
    the same way on both sides."""
    M, N, K = shape
    r = np.random.default_rng(12)
    post = []
    if "residual" in chain:
        res = dtp.f32_to_bf16(r.integers(-64, 65, size=M * N).astype(np.float32)).reshape(M, N)
        post = [PostOp(cabi.PO_BINARY, alg=cabi.BINARY["add"], dt=cabi.DT_BF16, stride=(0, N, 1), data=res)]
    p = problem(M, N, K, "bf16", "bf16", seed=13, bias="bias" in chain, post_ops=post)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("shape", [(300, 200, 96), (64, 130, 64), (512, 768, 1024)])
def test_row_major_weights_take_the_layout_pre_pass(gpu, oracle, dt, shape):
    M, N, K = shape
    p = problem(M, N, K, dt, "f32", seed=11, wtag="ab", bias=True)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
@pytest.mark.parametrize("wei_batch", [True, False])
@pytest.mark.parametrize("wtag", ["ba", "ab"])
def test_batched_exact(gpu, oracle, wei_batch, wtag):
    p = problem(100, 72, 64, "bf16", "f32", batch=3, seed=7, wei_batch=wei_batch, wtag=wtag)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
@pytest.mark.parametrize("dt,ddt", [("bf16", "f32"), ("bf16", "bf16"), ("f16", "f32"), ("f32", "f32")])
def test_random_data_within_the_f32_sum_bound(gpu, oracle, dt, ddt):
    p = problem(320, 448, 2048, dt, ddt, exact=False, seed=8, bias=True)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    _, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    # products of two f32 values round once each (2^-24 relative) before they are added; those of 16-bit values are exact
    hw = np.asarray(asum, np.float64).reshape(p.M, p.N) * 2.0 ** -24 if dt == "f32" else None
    assert_gemm_close(p, got, ideal, asum, what=name, hw=hw)


@pytest.mark.gpu
def test_matches_the_generic_kernel_on_a_large_shape(gpu):
    """2048 x 4096 x 4096 bf16 -> bf16, random data: against hip:ref:any (the reference's sequential f32 sum) within
    a few units of bf16 rounding of values of size sqrt(K)."""
    p = problem(2048, 4096, 4096, "bf16", "bf16", exact=False, seed=9)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    want, wname = run_gpu(p, cabi.IMPL_REF)
    assert wname.startswith("hip:ref")
    g = dtp.bf16_to_f32(got.reshape(-1)).astype(np.float64)
    w = dtp.bf16_to_f32(want.reshape(-1)).astype(np.float64)
    err = np.abs(g - w)
    tol = np.abs(w) * 2.0 ** -7 + 64 * 2.0 ** -7 * 0.05
    assert (err <= tol).all(), f"worst {err.max()} at {err.argmax()}"
    assert (err > 0).mean() < 0.2          # most elements round to the same bf16 value


# ------------------------------------------------------------------ f32 operands under fpmath_mode bf16 / f16 / any
FPMATH_BF16, FPMATH_F16, FPMATH_ANY = 1, 2, 3


def test_fpmath_dispatch_rules():
    p = problem(64, 96, 64, "f32", "f32", wtag="ab")
    p.fpmath_mode = FPMATH_BF16
    st, impl = cabi.query(p.desc())
    assert st == cabi.SUCCESS and impl == cabi.IMPL_H16_MFMA
    assert cabi.scratch_bytes(p.desc()) == 64 * 64 * 2 + 96 * 64 * 2             # both operands as 16-bit copies
    p.fpmath_mode = 0
    assert cabi.scratch_bytes(p.desc()) == 96 * 64 * 4                           # strict: only the f32 layout pre-pass
    p = problem(64, 96, 48, "f32", "f32")                                        # K = 48: bf16 copies padded to 64
    p.fpmath_mode = FPMATH_ANY
    assert cabi.query(p.desc())[1] == cabi.IMPL_H16_MFMA and cabi.scratch_bytes(p.desc()) == (64 + 96) * 64 * 2
    p.fpmath_mode = 0                                                            # strict: f32 stages of 16, read in place
    assert cabi.scratch_bytes(p.desc()) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("mode", [FPMATH_BF16, FPMATH_F16, FPMATH_ANY])
@pytest.mark.parametrize("wtag", ["ab", "ba"])
def test_fpmath_exact_data_bit_exact(gpu, oracle, mode, wtag):
    """values every 16-bit type holds exactly: the down-conversion changes nothing, the f32 oracle applies"""
    p = problem(300, 200, 96, "f32", "f32", seed=21, wtag=wtag, bias=True, batch=2)
    p.fpmath_mode = mode
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
def test_fpmath_bf16_is_the_bf16_matmul_of_the_rounded_operands(gpu):
    """random f32 operands under fpmath bf16 give the bits of the bf16 problem whose operands are the same values
    rounded to nearest even -- which pins the conversion and that nothing else changes"""
    M, N, K = 192, 320, 512
    r = np.random.default_rng(22)
    sv = r.standard_normal((1, M, K)).astype(np.float32)
    wv = r.standard_normal((1, K, N)).astype(np.float32)
    pf = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_F32, wei_dt=cabi.DT_F32, dst_dt=cabi.DT_F32, src=sv, wei=wv,
                       fpmath_mode=FPMATH_BF16, name="f32 under fpmath bf16")
    pb = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_BF16, wei_dt=cabi.DT_BF16, dst_dt=cabi.DT_F32,
                       src=enc(sv, "bf16"), wei=enc(wv, "bf16"), name="bf16")
    got_f, name_f = run_gpu(pf)
    got_b, name_b = run_gpu(pb)
    assert name_f.startswith("hip:mfma_h16") and name_b.startswith("hip:mfma_h16")
    assert np.array_equal(np.asarray(got_f).view(np.uint32), np.asarray(got_b).view(np.uint32))


# ------------------------------------------------------------------ any K, any plain layout: operand copies
@pytest.mark.gpu
@pytest.mark.parametrize("K", [1, 8, 33, 100, 1000])
@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("wtag", ["ab", "ba"])
def test_any_k_exact(gpu, oracle, K, dt, wtag):
    p = problem(130, 75, K, dt, "f32", seed=40 + K, wtag=wtag, bias=True)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
def test_column_major_src_and_batched_odd_k(gpu, oracle):
    M, N, K, B = 70, 90, 45, 3
    p = problem(M, N, K, "bf16", "bf16", seed=50, batch=B, wtag="ab")
    src = p.src.reshape(B, M, K)
    p.src = np.ascontiguousarray(src.transpose(0, 2, 1))          # [B][K][M]: M contiguous
    p.src_stride = (M * K, 1, M)
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.gpu
def test_fpmath_with_odd_k(gpu, oracle):
    p = problem(64, 48, 77, "f32", "f32", seed=51, wtag="ab")
    p.fpmath_mode = FPMATH_BF16
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_h16"), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)
