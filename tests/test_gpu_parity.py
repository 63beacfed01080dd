"""GPU parity: HIP kernels (through the C ABI) against the CPU oracle on the
same seeded inputs, at sizes the oracle finishes in seconds."""
import numpy as np
import pytest

from onednn_amd import cabi, configs
from onednn_amd.problem import run_gpu
from tests.helpers import assert_bit_exact, assert_close, assert_decode_close, assert_gemm_close, fp8_mfma_bound

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("i8_tiles")]


@pytest.mark.parametrize("dst", ["s32", "f32"])
@pytest.mark.parametrize("impl", [cabi.IMPL_REF, cabi.IMPL_I8_MFMA])
def test_config1_small(gpu, oracle, dst, impl):
    p = configs.config1(M=96, N=320, K=256, dst=dst)
    got, name = run_gpu(p, impl)
    want = oracle.run_oracle(p)
    # integer accumulation is order-free and the epilogue has one rounding per
    # written operation: both kernels must reproduce the oracle bit for bit
    assert_bit_exact(p, got, want, name)


@pytest.mark.parametrize("impl", [cabi.IMPL_REF, cabi.IMPL_I8_MFMA])
@pytest.mark.parametrize("mode", [cabi.DST_SCALE_DIVIDE, cabi.DST_SCALE_RECIPROCAL])
def test_config3_small(gpu, oracle, impl, mode):
    p = configs.config3(M=160, N=288, K=512, dst_scale_mode=mode)
    got, name = run_gpu(p, impl)
    want = oracle.run_oracle(p)
    assert_bit_exact(p, got, want, name)


def test_config1_full_size(gpu, oracle):
    p = configs.config1()
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_i8")
    want = oracle.run_oracle(p)
    assert_bit_exact(p, got, want, name)


@pytest.mark.parametrize("impl", [cabi.IMPL_REF, cabi.IMPL_F8_MFMA])
@pytest.mark.parametrize("wtag", ["ab", "ba"])
def test_config4_small(gpu, oracle, impl, wtag):
    # fp8 x fp8 -> bf16 with bf16 bias, gelu_tanh and a bf16 residual add.
    # f32 accumulation order and the device tanhf differ from the oracle's:
    # against the oracle's float64 sum with the chain in float64 on top, under the
    # sqrt(K)-type bound of the float32 summation (tests/helpers.py gemm_bound),
    # for the configuration's bf16 dst and for an f32 dst
    for dst in (cabi.DT_BF16, cabi.DT_F32):
        p = configs.config4(M=192, N=320, K=512, wtag=wtag)
        p.dst_dt = dst
        got, name = run_gpu(p, impl)
        _, ideal, asum = oracle.run_oracle(p, want_ideal=True)
        assert_gemm_close(p, got, ideal, asum, what=name, hw=fp8_mfma_bound(p) if impl == cabi.IMPL_F8_MFMA else None)


@pytest.mark.parametrize("chain", ["swish", "swish*gate", "swish*gate, no bias", "gate alone", "gelu_tanh*gate",
                                   "gelu_tanh*gate, no bias"])
def test_config4_gated_feed_forward_chains(gpu, oracle, chain):
    # the gated feed-forward layer of the Llama family on C4's tensors: swish (SiLU) in place of gelu_tanh and a
    # multiplication by a bf16 tensor in place of the residual add (and gelu_tanh with that multiplication: GeGLU).
    # All of them run the fp8 tiles' whole-row epilogue; same bound as the configuration's own chain
    for dst, M, N, alpha in ((cabi.DT_BF16, 192, 320, 1.0), (cabi.DT_F32, 192, 320, 1.0), (cabi.DT_BF16, 300, 512, 1.702),
                             (cabi.DT_BF16, 256, 256, 0.5)):
        p = configs.config4(M=M, N=N, K=512)
        p.dst_dt = dst
        elt, gate = p.post_ops
        if "gelu" not in chain:
            elt.alg, elt.alpha = cabi.ELTWISE["swish"], alpha
        gate.alg = cabi.BINARY["mul"]
        p.post_ops = {"swish": [elt], "gate alone": [gate]}.get(chain, [elt, gate])
        if "no bias" in chain:
            p.bias, p.bias_dt = None, cabi.DT_UNDEF
        got, name = run_gpu(p, cabi.IMPL_F8_MFMA)
        _, ideal, asum = oracle.run_oracle(p, want_ideal=True)
        assert_gemm_close(p, got, ideal, asum, what=f"{name} {chain}", hw=fp8_mfma_bound(p))


def test_config4_no_postops_f32(gpu, oracle):
    # plain scaled fp8 GEMM into f32: only the summation order differs
    p = configs.config4(M=256, N=256, K=1024)
    p.post_ops = []
    p.bias, p.bias_dt = None, cabi.DT_UNDEF
    p.dst_dt = cabi.DT_F32
    got, name = run_gpu(p, cabi.IMPL_F8_MFMA)
    _, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    assert_gemm_close(p, got, ideal, asum, what=name, hw=fp8_mfma_bound(p))


@pytest.mark.parametrize("impl", [cabi.IMPL_REF, cabi.IMPL_MXF4_MFMA])
@pytest.mark.parametrize("wtag", ["ba", "ab"])
def test_config5_small(gpu, oracle, impl, wtag):
    # MXFP4: every 32-long block dot is exact in f32 and the e8m0 scales are
    # powers of two, so only the order of the K/32 cross-block additions can
    # differ: bounded by the forward error of that sum, then one bf16 rounding.
    p = configs.config5(M=160, N=288, K=512, wtag=wtag)
    got, name = run_gpu(p, impl)
    want, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    if impl == cabi.IMPL_REF:
        assert_bit_exact(p, got, want, name)   # same order as the reference
    else:
        assert_gemm_close(p, got, ideal, asum, what=name)
        q = configs.config5(M=160, N=288, K=512, wtag=wtag)
        q.dst_dt = cabi.DT_F32
        got, name = run_gpu(q, impl)
        assert_gemm_close(q, got, ideal, asum, what=name)


def test_config5_f32_dst_single_block_exact(gpu, oracle):
    # K = 128 is one MFMA: four blocks, f32 dst.  With all scales equal the
    # sum of four exactly representable block sums is exact in any order.
    p = configs.config5(M=256, N=256, K=128)
    p.dst_dt = cabi.DT_F32
    p.quant["src_scale"].data[:] = 127
    p.quant["wei_scale"].data[:] = 126
    got, name = run_gpu(p, cabi.IMPL_MXF4_MFMA)
    want = oracle.run_oracle(p)
    assert_bit_exact(p, got, want, name)


@pytest.mark.parametrize("M", [1, 8, 32])
def test_config2_small_ref_kernel(gpu, oracle, M):
    # weight-only int4 decode through the generic kernel: same operation order
    # as the reference's naive loop, no transcendental functions -> bit-exact
    p = configs.config2(M=M, N=512, K=1024)
    got, name = run_gpu(p, cabi.IMPL_REF)
    want = oracle.run_oracle(p)
    assert_bit_exact(p, got, want, name)


@pytest.mark.parametrize("M", [1, 8, 32])
def test_config2_small_woq_kernel(gpu, oracle, M):
    # the decode kernel evaluates the same real-valued expression with a
    # different rounding (group factor applied once per group, MFMA f32
    # accumulation): bf16 threshold plus the forward error bound of the K sum
    p = configs.config2(M=M, N=512, K=1024)
    got, name = run_gpu(p, cabi.IMPL_WOQ_GEMV)
    assert name.startswith("hip:woq_gemv")
    _, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    assert_decode_close(p, got, ideal, asum, what=name)


def test_woq_one_hot_rows_are_exact(gpu, oracle):
    # src = identity: every output is a single decompressed weight,
    # (w - zp) * scale with one rounding -> must equal the oracle bit for bit.
    # Exercises nibble order, group indexing and the K split / reduction.
    import numpy as np
    from onednn_amd import dtypes as dtp
    K = 32
    p = configs.config2(M=K, N=256, K=K, group=16)
    p.src = dtp.f32_to_bf16(np.eye(K, dtype=np.float32))
    p.dst_dt = cabi.DT_F32
    got, name = run_gpu(p, cabi.IMPL_WOQ_GEMV)
    want = oracle.run_oracle(p)
    assert_bit_exact(p, got, want, name)


WOQ_VARIANTS = [
    # M, N, K, group, weights, scales dt/kind, zero points dt/kind, dst, bias+relu
    (1, 512, 1024, 128, "u4", "f32", "grouped", "s8", "grouped", "bf16", False),
    (5, 272, 1040, 80, "u4", "f16", "column", "u8", "column", "f32", True),     # ragged N and K, per-column parameters
    (16, 512, 512, 64, "s4", "bf16", "grouped", "s4", "grouped", "bf16", False),
    (17, 256, 2048, 128, "s4", "bf16", "grouped", "s32", "common", "f32", False),
    (32, 1024, 512, 32, "u4", "f32", "grouped", "u4", "none", "bf16", True),
    (3, 4096, 256, 256, "u4", "bf16", "none", "u8", "grouped", "f32", False),    # no K split (wide N), no scales
    (8, 768, 4096, 128, "u4", "bf16", "grouped", "s32", "grouped", "bf16", False),
    # wide N: 512-column chunks, 16-byte weight loads
    (1, 2048, 1024, 128, "u4", "bf16", "grouped", "u4", "grouped", "bf16", False),
    (8, 2080, 528, 48, "s4", "f16", "grouped", "s8", "grouped", "f32", True),     # ragged last chunk, K not a multiple of the split
    (16, 4096, 1024, 128, "u4", "f32", "column", "u4", "common", "bf16", False),
    (2, 14336, 256, 128, "u4", "bf16", "grouped", "s4", "column", "f32", False),
]


@pytest.mark.parametrize("case", WOQ_VARIANTS, ids=lambda c: "-".join(str(x) for x in c))
def test_woq_attribute_variants(gpu, oracle, case):
    M, N, K, group, wdt, sdt, skind, zdt, zkind, ddt, relu_bias = case
    p = configs.woq_variant(M, N, K, group, wei_dt=wdt, sc_dt=sdt, sc_kind=skind, zp_dt=zdt, zp_kind=zkind,
                            dst_dt=ddt, relu_bias=relu_bias)
    got, name = run_gpu(p, cabi.IMPL_WOQ_GEMV)
    assert name.startswith("hip:woq_gemv")
    want, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    assert_decode_close(p, got, ideal, asum, what=name)
    # and the generic kernel follows the reference's operation order exactly
    got_ref, name_ref = run_gpu(p, cabi.IMPL_REF)
    assert_bit_exact(p, got_ref, want, name_ref)


def test_woq_back_to_back_launches_share_nothing(gpu, oracle):
    # the arrival counters return to zero after every launch: a second launch on
    # the same scratch, and a different problem right after, see a clean state
    from onednn_amd.problem import GpuRun
    a = configs.config2(M=4, N=512, K=2048)
    b = configs.config2(M=1, N=768, K=1024, seed=9)
    ra, rb = GpuRun(a, cabi.IMPL_WOQ_GEMV), GpuRun(b, cabi.IMPL_WOQ_GEMV)
    outs = []
    for r in (ra, ra, rb, ra, rb):
        r.reset_dst()
        r.launch()
        r.sync()
        outs.append(r.result())
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[3])
    assert np.array_equal(outs[2], outs[4])
    want, ideal, asum = oracle.run_oracle(b, want_ideal=True)
    assert_decode_close(b, outs[4], ideal, asum, what="second problem")
    ra.free()
    rb.free()


@pytest.mark.parametrize("scale", [1.0, 1.4e-45, 1e-43])
def test_bf16_dst_of_integer_gemm_is_bit_exact_including_flushed_subnormals(gpu, oracle, scale):
    """s8 x s8 -> bf16: integer accumulation, so the only rounding is the dst
    conversion.  The reference's bf16 conversion flushes f32 subnormals to a
    signed zero (src/common/bfloat16.cpp:29-49); the MFMA epilogue converts in
    hardware and must take its software path for those (scale 1.4e-45 makes every
    result subnormal, 1e-43 a mix of subnormal and normal values)."""
    from onednn_amd.problem import MatmulProblem, QuantParam
    r = np.random.default_rng(123)
    M, N, K = 256, 256, 128
    src = r.integers(-127, 128, size=(M, K), dtype=np.int8)
    wei = r.integers(-127, 128, size=(K, N), dtype=np.int8)
    p = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_S8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_BF16, src=src, wei=wei,
                      wei_stride=(K * N, N, 1),
                      quant={"src_scale": QuantParam(cabi.DT_F32, 0, np.array([scale], np.float32))})
    got, name = run_gpu(p, cabi.IMPL_I8_MFMA)
    want = oracle.run_oracle(p)
    assert_bit_exact(p, got, want, name)
    if scale == 1.4e-45:
        assert np.all((want.view(np.uint16) & 0x7fff) == 0)


@pytest.mark.parametrize("dst", ["f8_e4m3", "f8_e5m2"])
@pytest.mark.parametrize("with_nan", [False, True])
@pytest.mark.parametrize("dynamic", [False, True])
def test_fp8_dst_of_the_fp8_gemm_is_bit_exact_on_exact_sums(gpu, oracle, dst, with_nan, dynamic):
    # small-integer operands: every product and partial sum is exact in f32, so
    # the GEMM's summation order does not matter and the fp8 conversion of the
    # epilogue (hardware f32 -> f16 -> fp8 for wavefronts without NaNs, the
    # software one otherwise) must reproduce the oracle bit for bit, including
    # values beyond the range of the type (dst scale 4: |d| up to 576 > 448)
    import numpy as np
    from onednn_amd import dtypes as dtp
    from onednn_amd.problem import MatmulProblem, QuantParam
    M, N, K = 300, 320, 256
    r = np.random.default_rng(9)
    src = dtp.f32_to_e4m3(r.integers(-3, 4, size=(M, K)).astype(np.float32).reshape(-1))
    wei = dtp.f32_to_e4m3(r.integers(-3, 4, size=(N, K)).astype(np.float32).reshape(-1))   # K-contiguous (ba)
    bias = (r.integers(-64, 65, size=N) / 16.0).astype(np.float32)
    if with_nan:
        bias[5] = np.nan
    dst_dt = cabi.DT_F8_E4M3 if dst == "f8_e4m3" else cabi.DT_F8_E5M2
    p = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_F8_E4M3, wei_dt=cabi.DT_F8_E4M3, dst_dt=dst_dt, src=src, wei=wei,
                      wei_stride=(K * N, 1, K), bias_dt=cabi.DT_F32, bias=bias,
                      quant={"dst_scale": QuantParam(cabi.DT_F32, 0, np.array([4.0 if dst == "f8_e4m3" else 0.03125], np.float32))},
                      name=f"f8-exact-{dst}")
    if dynamic:
        # the same values through the dynamic (MX) quantization: exact sums give the
        # GEMM tile and the oracle the same group maxima, so scales and dst agree
        # bit for bit (a NaN does not enter the group maximum, as with the reference's
        # std::max, and converts to the NaN code of the type)
        from onednn_amd.problem import GpuRun
        from oracle import binding as orc
        p.quant["dst_scale"] = QuantParam(cabi.DT_E8M0, 6, np.zeros((1, M, N // 32), np.uint8), (1, 32))
        p.dst_dynamic = cabi.DST_DYNAMIC_MX
        run = GpuRun(p, cabi.IMPL_F8_MFMA)
        try:
            run.launch()
            got, sc = run.result(), run.dynamic_scales()
        finally:
            run.free()
        want, want_sc = orc.run_oracle_dynamic(p)
        assert np.array_equal(np.asarray(sc).reshape(-1), np.asarray(want_sc).reshape(-1))
        assert np.array_equal(np.asarray(got).view(np.uint8), np.asarray(want).view(np.uint8))
        return
    got, name = run_gpu(p, cabi.IMPL_F8_MFMA)
    want = oracle.run_oracle(p)
    assert_bit_exact(p, got, want, name)
    codes = np.asarray(got).view(np.uint8)
    assert len(np.unique(codes)) > 60           # the conversion is exercised over a large part of the code space


def test_hardware_fp8_conversions_match_the_software_ones_except_for_nans(gpu):
    # the calibration tool walks every f16 bit pattern through the hardware
    # f16 -> e4m3 / e5m2 conversions and 4 M f32 patterns through f32 -> f16 and
    # compares with the software conversions the oracle's restatement is pinned to
    import os
    import subprocess
    tool = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bin", "cvt_fp8_check")  # built by tests/Makefile
    assert os.path.exists(tool), "build tests/bin/cvt_fp8_check first (make -C tests, or __graft_entry__.build())"
    out = subprocess.run([tool], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    assert out.stdout.strip().splitlines()[-1] == "nan-only", out.stdout[-2000:]


@pytest.mark.parametrize("with_nan_inf", [False, True])
def test_f16_dst_of_integer_gemm_is_bit_exact(gpu, oracle, with_nan_inf):
    # integer accumulation is exact, so the f16 conversion of the batched tile
    # epilogue (hardware v_cvt_f16_f32) must equal the oracle's software
    # conversion bit for bit: normal values, f16 subnormals (tiny dst scale
    # inverse), overflow to infinity, and NaN / infinite inputs through the bias
    import numpy as np
    from onednn_amd.problem import QuantParam
    p = configs.config3(M=300, N=320, K=512, wtag="ba")
    p.dst_dt = cabi.DT_F16
    p.post_ops = []
    N = p.N
    # per-column scales spread over 40 binades: columns land in f16's subnormal, normal and overflow ranges
    sc = np.exp2(np.random.default_rng(3).uniform(-34, 6, size=N)).astype(np.float32)
    p.quant["wei_scale"] = QuantParam(cabi.DT_F32, configs.MASK_COL, sc)
    p.quant.pop("dst_scale")
    if with_nan_inf:
        bias = np.zeros(N, np.float32)
        bias[3], bias[40], bias[77] = np.nan, np.inf, -np.inf
        p.bias_dt, p.bias = cabi.DT_F32, bias
    got, name = run_gpu(p, cabi.IMPL_I8_MFMA)
    want = oracle.run_oracle(p)
    assert_bit_exact(p, got, want, name)
    h = np.asarray(got).view(np.uint16)
    e = (h >> 10) & 0x1f
    assert np.any((e == 0) & ((h & 0x3ff) != 0)) and np.any(e == 0x1f) and np.any((e > 0) & (e < 0x1f))
