"""GPU parity for the branches outside the five benchmark configurations:
precomputed reductions with grouped src parameters, prelu, and every eltwise /
binary algorithm -- the problems of tests/tail_cases.py through the C ABI, on
the generic kernel and on whatever family the dispatcher picks, against the CPU
oracle (bit for bit where no libm function is involved) and against the
closed-form numpy expectation that pins the oracle itself."""
import numpy as np
import pytest

from onednn_amd import cabi, dnnl
from onednn_amd.problem import MatmulProblem, PostOp, QuantParam, run_gpu
from tests import tail_cases as tc
from tests.helpers import assert_bit_exact, logical
from tests.test_oracle_pins import PR_VARIANTS

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("i8_tiles")]
F = np.float32
IMPLS = [cabi.IMPL_REF, cabi.IMPL_AUTO]


@pytest.mark.parametrize("kw", PR_VARIANTS, ids=lambda kw: ",".join(f"{k}={v}" for k, v in kw.items()) or "plain")
def test_precomputed_reductions(gpu, oracle, kw):
    p, want = tc.pr_case(11, **kw)
    got, name = run_gpu(p)
    assert_bit_exact(p, got, oracle.run_oracle(p), name)
    assert np.array_equal(np.asarray(got).view(np.uint32).reshape(p.M, p.N), want.view(np.uint32))


def test_precomputed_reductions_larger_shape(gpu, oracle):
    # more rows / columns than a workgroup of the generic kernel covers, several groups
    p, want = tc.pr_case(13, with_src_zp=True, src_zp_groups=True, true_sums=False, M=70, N=130, K=512, g=32, gw=64)
    got, name = run_gpu(p)
    assert_bit_exact(p, got, oracle.run_oracle(p), name)
    assert np.array_equal(np.asarray(got).view(np.uint32).reshape(p.M, p.N), want.view(np.uint32))


def test_grouped_int8_src_scales_with_weights_zero_points(gpu, oracle):
    # the grouped int8 flow without reductions (ref_matmul_int8.cpp:184-258), on exact numpy arithmetic
    r = np.random.default_rng(5)
    M, N, K, g = 33, 96, 256, 64
    src = r.integers(-128, 128, size=(M, K)).astype(np.int8)
    wei = r.integers(-128, 128, size=(K, N)).astype(np.int8)
    ss = r.choice([0.0625, 0.125, 0.25], size=(M, K // g)).astype(F)
    ws = r.choice([0.0625, 0.125, 0.25], size=(K // g, N)).astype(F)
    wz = r.integers(-2, 3, size=(K // g, N)).astype(np.int8)
    p = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_S8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_F32, src=src, wei=wei,
                      quant={"src_scale": QuantParam(cabi.DT_F32, 6, ss, (1, g)),
                             "wei_scale": QuantParam(cabi.DT_F32, 6, ws, (g, 1)),
                             "wei_zp": QuantParam(cabi.DT_S8, 6, wz, (g, 1))}, name="grouped int8")
    want = np.zeros((M, N), F)
    for gi in range(K // g):
        sl = slice(gi * g, (gi + 1) * g)
        acc = src[:, sl].astype(np.int64) @ (wei[sl].astype(np.int64) - wz[gi][None, :].astype(np.int64))
        want = want + acc.astype(F) * ss[:, gi][:, None] * ws[gi][None, :]
    got, name = run_gpu(p)
    assert np.array_equal(np.asarray(got).view(np.uint32).reshape(M, N), want.view(np.uint32)), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.parametrize("mask_b,mask_m,mask_n", [(0, 0, 0), (0, 0, 1), (0, 1, 0), (0, 1, 1), (1, 0, 1), (1, 1, 0), (1, 1, 1)])
def test_prelu_generic_kernel(gpu, oracle, mask_b, mask_m, mask_n):
    batch = 3 if mask_b else 1
    p, want, _ = tc.prelu_case(22, mask_m, mask_n, batch=batch, mask_b=bool(mask_b), M=37, N=70)
    got, name = run_gpu(p)
    assert np.array_equal(np.asarray(got).reshape(want.shape), want), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("mask_m,mask_n", [(0, 1), (1, 0), (1, 1)])
def test_prelu_after_int8_gemm(gpu, oracle, impl, mask_m, mask_n):
    # the tile epilogue's interpreter of the MFMA families takes prelu too
    p, x = tc._int8_base(31, False, 0.37, M=96, N=320, K=128)
    r = np.random.default_rng(32)
    dm, dn = (p.M if mask_m else 1), (p.N if mask_n else 1)
    w = r.uniform(-2, 2, size=(dm, dn)).astype(F)
    p.post_ops = [PostOp(kind=cabi.PO_PRELU, dt=cabi.DT_F32, stride=(0, dn if mask_m else 0, 1 if mask_n else 0), data=w)]
    p.name = "prelu:int8"
    want = np.where(x >= 0, x, np.broadcast_to(w, x.shape) * x).astype(F)
    got, name = run_gpu(p, impl)
    if impl == cabi.IMPL_AUTO:
        assert name.startswith("hip:mfma_i8"), name
    assert np.array_equal(np.asarray(got).view(np.uint32).reshape(p.M, p.N), want.view(np.uint32)), name
    assert_bit_exact(p, got, oracle.run_oracle(p), name)


def test_prelu_three_dims_through_the_api(gpu):
    """dnnl_post_ops_append_prelu on a batched matmul: the weights memory is laid out acb."""
    r = np.random.default_rng(41)
    B, M, N, K = 3, 20, 24, 16
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    src = r.integers(-4, 5, size=(B, M, K)).astype(F)
    wei = r.integers(-4, 5, size=(B, K, N)).astype(F)
    v = np.einsum("bmk,bkn->bmn", src, wei).astype(F)
    f32 = cabi.DT_F32
    for mask in (0b111, 0b110, 0b101, 0b100, 0b011):
        db, dm, dn = (B if mask & 1 else 1), (M if mask & 2 else 1), (N if mask & 4 else 1)
        w = r.uniform(-2, 2, size=(db, dn, dm)).astype(F)
        po = dnnl.post_ops()
        po.append_prelu(mask)
        attr = dnnl.primitive_attr()
        attr.set_post_ops(po)
        mds = [dnnl.memory_desc([B, M, K], f32, tag=dnnl.tag_abc), dnnl.memory_desc([B, K, N], f32, tag=dnnl.tag_abc),
               dnnl.memory_desc([B, M, N], f32, tag=dnnl.tag_abc)]
        pd = dnnl.matmul_primitive_desc(eng, mds[0], mds[1], mds[2], attr=attr)
        dst = dnnl.memory(mds[2], eng)
        w_md = dnnl.memory_desc([db, dm, dn], f32, tag=dnnl.tag_acb)
        dnnl.matmul(pd).execute(strm, {
            dnnl.ARG_SRC: dnnl.memory(mds[0], eng, src), dnnl.ARG_WEIGHTS: dnnl.memory(mds[1], eng, wei), dnnl.ARG_DST: dst,
            dnnl.ARG_ATTR_MULTIPLE_POST_OP(0) | dnnl.ARG_WEIGHTS: dnnl.memory(w_md, eng, w)})
        strm.wait()
        want = np.where(v >= 0, v, np.broadcast_to(w.transpose(0, 2, 1), v.shape) * v)
        assert np.array_equal(dst.read(np.float32).reshape(B, M, N), want), bin(mask)


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("name", sorted(tc.ELTWISE_TAIL))
def test_eltwise_algorithms(gpu, oracle, name, impl):
    p, want, mode = tc.eltwise_case(name)
    got_raw, impl_name = run_gpu(p, impl)
    got = logical(p, got_raw).reshape(p.M, p.N)
    orc = logical(p, oracle.run_oracle(p)).reshape(p.M, p.N)
    if mode == "exact":
        assert np.array_equal(got.view(np.uint32), np.asarray(want, F).view(np.uint32)), impl_name
        assert np.array_equal(got.view(np.uint32), orc.view(np.uint32)), impl_name
    else:
        # the device's libm and the host's differ in the last places: 8 units against the float64 formula
        ok = tc.ulp_close(got, want, ulps=8, atol=mode[1])
        assert ok.all(), (name, impl_name, got[~ok][:4], np.asarray(want)[~ok][:4])
        ok = tc.ulp_close(got, orc.astype(np.float64), ulps=12, atol=2 * mode[1])
        assert ok.all(), (name, impl_name, got[~ok][:4], orc[~ok][:4])


@pytest.mark.parametrize("name,alpha", [("swish", 1.5), ("swish", -0.75), ("logistic", 0.0)])
def test_swish_and_logistic_on_full_tiles(gpu, oracle, name, alpha):
    # the tile kernels evaluate these two with the hardware exponential and reciprocal; where the argument is
    # negative the result is the exponential itself, so its accuracy shows: arguments out to +-25 (the result
    # down to 1e-16), every element against the float64 formula on the float32 product alpha * s the reference forms
    p, x = tc._int8_base(21, False, 0.11, M=256, N=256, K=64)
    p.post_ops = [PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE[name], alpha=alpha, beta=0.0, scale=1.0)]
    got_raw, impl_name = run_gpu(p)
    assert impl_name.startswith("hip:mfma_i8"), impl_name
    got = logical(p, got_raw).reshape(p.M, p.N)
    x64 = x.astype(np.float64)
    assert x64.min() < -18 and x64.max() > 18
    with np.errstate(over="ignore"):
        if name == "swish":
            want = x64 / (1.0 + np.exp(-(F(alpha) * x).astype(np.float64)))
        else:
            want = 1.0 / (1.0 + np.exp(-x64))
    ok = tc.ulp_close(got, want, ulps=8, atol=1e-37)
    assert ok.all(), (impl_name, x[~ok][:4], got[~ok][:4], want[~ok][:4])
    orc = logical(p, oracle.run_oracle(p)).reshape(p.M, p.N)
    ok = tc.ulp_close(got, orc.astype(np.float64), ulps=12, atol=2e-37)
    assert ok.all(), (impl_name, x[~ok][:4], got[~ok][:4], orc[~ok][:4])


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("name", tc.BINARY_TAIL)
@pytest.mark.parametrize("operand,odt", [("per_element", "f32"), ("per_n", "f32"), ("per_m", "s8"), ("scalar", "bf16")])
def test_binary_algorithms(gpu, oracle, name, operand, odt, impl):
    p, want = tc.binary_case(name, operand, odt=odt)
    got, impl_name = run_gpu(p, impl)
    assert np.array_equal(np.asarray(got).view(np.uint32).reshape(p.M, p.N), want.view(np.uint32)), impl_name
    assert_bit_exact(p, got, oracle.run_oracle(p), impl_name)
