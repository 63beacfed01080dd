"""Pins the oracle's matmul restatement (oracle/oracle_matmul.c) against what
the mathematics fixes, without running the reference:

  * s32 accumulators: integer arithmetic is exact and order-free, so a
    brute-force int64 numpy product must match bit for bit; closed forms
    (all-ones -> K, src == zero point -> 0, identity weights);
  * zero-point folding: sum (s-zs)(w-zw) == sum sw - zs sum w - zw sum s + K zs zw;
  * the epilogue order of ref_matmul_int8.cpp:241-306: re-evaluated with numpy
    float32 scalars, one rounding per operation;
  * int4 decode: one-hot src rows read single weights back (nibble order, group
    indexing of scales and zero points, ref_matmul.cpp:193-214);
  * fp paths: f64 evaluation with the forward error bound K * 2^-24 * sum|terms|;
  * MXFP4: 32-long e2m1 block dots are exact in f32 and e8m0 scales are powers
    of two, so a float64 evaluation is exact per block;
  * post-ops: textbook formulas, broadcast indexing, sum with zero point.
"""
import numpy as np
import pytest

from onednn_amd import cabi, configs
from onednn_amd import dtypes as dtp
from onednn_amd.problem import MatmulProblem, PostOp, QuantParam, decode, strides_for
from tests.helpers import logical

F = np.float32


def brute_acc(src, wei, zs=0, zw=0):
    return (src.astype(np.int64) - zs) @ (wei.astype(np.int64) - zw)


@pytest.mark.parametrize("src_dt,wei_dt", [("u8", "s8"), ("s8", "s8"), ("s8", "u8"), ("u8", "u8")])
def test_int8_accumulator_brute_force(oracle, src_dt, wei_dt):
    rng = np.random.default_rng(1)
    M, N, K = 17, 23, 301
    sd = np.uint8 if src_dt == "u8" else np.int8
    wd = np.uint8 if wei_dt == "u8" else np.int8
    src = rng.integers(np.iinfo(sd).min, np.iinfo(sd).max + 1, size=(M, K)).astype(sd)
    wei = rng.integers(np.iinfo(wd).min, np.iinfo(wd).max + 1, size=(K, N)).astype(wd)
    q = {"src_zp": QuantParam(cabi.DT_S32, 0, np.array([7], np.int32)),
         "wei_zp": QuantParam(cabi.DT_S32, 4, rng.integers(-5, 6, size=N).astype(np.int32))}
    p = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_NAMES[src_dt], wei_dt=cabi.DT_NAMES[wei_dt],
                      dst_dt=cabi.DT_S32, src=src, wei=wei, quant=q)
    acc = oracle.run_int8_acc(p).reshape(M, N)
    want = brute_acc(src, wei, 7, q["wei_zp"].data[None, :])
    assert np.array_equal(acc, want)
    # zero-point folding identity, all in exact integers
    zs, zw = 7, q["wei_zp"].data.astype(np.int64)
    s64, w64 = src.astype(np.int64), wei.astype(np.int64)
    folded = s64 @ w64 - zs * w64.sum(0)[None, :] - zw[None, :] * s64.sum(1)[:, None] + K * zs * zw[None, :]
    assert np.array_equal(folded, want)


def test_int8_closed_forms(oracle):
    M, N, K = 5, 7, 64
    ones = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_S8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_S32,
                         src=np.ones((M, K), np.int8), wei=np.ones((K, N), np.int8))
    assert (oracle.run_oracle(ones) == K).all()
    # src equal to its zero point -> 0
    z = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_U8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_S32,
                      src=np.full((M, K), 128, np.uint8),
                      wei=np.random.default_rng(0).integers(-127, 128, size=(K, N)).astype(np.int8),
                      quant={"src_zp": QuantParam(cabi.DT_S32, 0, np.array([128], np.int32))})
    assert (oracle.run_oracle(z) == 0).all()
    # identity weights copy src
    src = np.random.default_rng(2).integers(-128, 128, size=(M, K)).astype(np.int8)
    ident = MatmulProblem(M=M, N=K, K=K, src_dt=cabi.DT_S8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_S32,
                          src=src, wei=np.eye(K, dtype=np.int8))
    assert np.array_equal(oracle.run_oracle(ident).reshape(M, K), src.astype(np.int32))
    # transposed weights (tag ba) give the same numbers
    wei = np.random.default_rng(3).integers(-127, 128, size=(K, N)).astype(np.int8)
    a = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_S8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_S32, src=src, wei=wei)
    b = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_S8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_S32, src=src,
                      wei=np.ascontiguousarray(wei.T), wei_stride=strides_for("ba", 1, K, N))
    assert np.array_equal(oracle.run_oracle(a), oracle.run_oracle(b))


def test_config1_epilogue_order(oracle):
    # d = f32(acc) * src_scale; d *= wei_scale[n]; d += bias[n]   (two multiplies, then add)
    p = configs.config1(M=24, N=40, K=192)
    got = oracle.run_oracle(p).reshape(p.M, p.N)
    acc = brute_acc(p.src, p.wei, 128).astype(np.int32)
    d = acc.astype(F) * p.quant["src_scale"].data[0]
    d = d * p.quant["wei_scale"].data[None, :]
    d = d + p.bias[None, :]
    assert np.array_equal(got.view(np.uint32), d.astype(F).view(np.uint32))
    # the wrong order (scales multiplied together first) is detectably different
    alt = acc.astype(F) * (p.quant["src_scale"].data[0] * p.quant["wei_scale"].data[None, :]) + p.bias[None, :]
    assert not np.array_equal(alt.astype(F).view(np.uint32), got.view(np.uint32))


def test_config3_relu_dst_scale_saturate(oracle):
    p = configs.config3(M=32, N=48, K=256)
    got = oracle.run_oracle(p).reshape(p.M, p.N)
    acc = brute_acc(p.src, p.wei).astype(np.int32)
    d = acc.astype(F) * F(0.01)
    d = d * p.quant["wei_scale"].data[None, :]
    d = np.where(d > 0, d, d * F(0))
    d = d / F(0.05)
    want = np.rint(np.clip(d, F(-128), F(127))).astype(np.int8)
    assert np.array_equal(got, want)
    assert got.min() >= 0 and got.max() == 127            # relu floor, saturation reached
    # reciprocal flavour (brgemm_matmul.cpp:703-709): multiply by 1.f/0.05f
    pr = configs.config3(M=32, N=48, K=256, dst_scale_mode=cabi.DST_SCALE_RECIPROCAL)
    got_r = oracle.run_oracle(pr).reshape(p.M, p.N)
    d2 = acc.astype(F) * F(0.01)
    d2 = d2 * p.quant["wei_scale"].data[None, :]
    d2 = np.where(d2 > 0, d2, d2 * F(0)) * (F(1) / F(0.05))
    assert np.array_equal(got_r, np.rint(np.clip(d2, F(-128), F(127))).astype(np.int8))


def test_dst_zero_point_and_u8(oracle):
    rng = np.random.default_rng(4)
    M, N, K = 9, 16, 64
    src = rng.integers(-20, 20, size=(M, K)).astype(np.int8)
    wei = rng.integers(-20, 20, size=(K, N)).astype(np.int8)
    zp = rng.integers(0, 50, size=N).astype(np.int32)
    p = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_S8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_U8, src=src, wei=wei,
                      quant={"dst_scale": QuantParam(cabi.DT_F32, 0, np.array([8.0], F)),
                             "dst_zp": QuantParam(cabi.DT_S32, 4, zp)})
    got = oracle.run_oracle(p).reshape(M, N)
    d = brute_acc(src, wei).astype(F) / F(8.0) + zp[None, :].astype(F)
    assert np.array_equal(got, np.rint(np.clip(d, 0, 255)).astype(np.uint8))


def test_int8_grouped_scales_and_zero_points(oracle):
    # groups along K on both sides: per group s32 acc, scaled, then summed in f32
    rng = np.random.default_rng(5)
    M, N, K, g = 6, 10, 128, 32
    src = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    wei = rng.integers(-128, 128, size=(K, N)).astype(np.int8)
    ss = rng.choice([0.0625, 0.125, 0.25], size=(M, K // g)).astype(F)
    ws = rng.choice([0.0625, 0.125, 0.25], size=(K // g, N)).astype(F)
    wz = rng.integers(-2, 3, size=(K // g, N)).astype(np.int8)
    p = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_S8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_F32, src=src, wei=wei,
                      quant={"src_scale": QuantParam(cabi.DT_F32, 6, ss, (1, g)),
                             "wei_scale": QuantParam(cabi.DT_F32, 6, ws, (g, 1)),
                             "wei_zp": QuantParam(cabi.DT_S8, 6, wz, (g, 1))})
    got = oracle.run_oracle(p).reshape(M, N)
    want = np.zeros((M, N), F)
    for gi in range(K // g):
        sl = slice(gi * g, (gi + 1) * g)
        acc = src[:, sl].astype(np.int64) @ (wei[sl].astype(np.int64) - wz[gi][None, :].astype(np.int64))
        t = acc.astype(F) * ss[:, gi][:, None]
        t = t * ws[gi][None, :]
        want = want + t
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_int4_decode_one_hot_reads_weights_back(oracle):
    # M = K one-hot rows: dst[k, n] == (w[k, n] - zp[k/g, n]) * scale[k/g, n] exactly
    K, N, g = 256, 64, 128
    rng = np.random.default_rng(6)
    codes = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    zps = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    sc = rng.choice([0.25, 0.5, 2.0], size=(K // g, N)).astype(F)
    src = dtp.f32_to_bf16(np.eye(K, dtype=F))
    for wtag, packed in (("ab", dtp.pack_nibbles(codes)), ("ba", dtp.pack_nibbles(codes.T.copy()))):
        p = MatmulProblem(M=K, N=N, K=K, src_dt=cabi.DT_BF16, wei_dt=cabi.DT_U4, dst_dt=cabi.DT_F32,
                          src=src, wei=packed, wei_stride=strides_for(wtag, 1, K, N), apply_to_int=True,
                          quant={"wei_scale": QuantParam(cabi.DT_BF16, 6, dtp.f32_to_bf16(sc), (g, 1)),
                                 "wei_zp": QuantParam(cabi.DT_U4, 6, dtp.pack_nibbles(zps), (g, 1))})
        got = oracle.run_oracle(p).reshape(K, N)
        want = (codes.astype(F) - np.repeat(zps, g, 0).astype(F)) * np.repeat(sc, g, 0)
        assert np.array_equal(got, want), wtag
    # signed nibbles
    s_codes = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    p = MatmulProblem(M=K, N=N, K=K, src_dt=cabi.DT_BF16, wei_dt=cabi.DT_S4, dst_dt=cabi.DT_F32, src=src,
                      wei=dtp.pack_nibbles(s_codes), apply_to_int=True)
    got = oracle.run_oracle(p).reshape(K, N)
    assert np.array_equal(got, dtp.s4_codes_to_int(s_codes).astype(F))


def test_config2_against_f64(oracle):
    p = configs.config2(M=4, N=256, K=1024)
    got, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    w = dtp.unpack_nibbles(p.wei, p.K * p.N).reshape(p.K, p.N).astype(np.float64)
    zp = np.repeat(dtp.unpack_nibbles(p.quant["wei_zp"].data, p.K // 128 * p.N).reshape(-1, p.N), 128, 0)
    sc = np.repeat(dtp.bf16_to_f32(p.quant["wei_scale"].data).reshape(-1, p.N), 128, 0).astype(np.float64)
    wf = ((w - zp).astype(F) * sc.astype(F)).astype(np.float64)      # one f32 rounding, as the reference
    want = dtp.bf16_to_f32(p.src).reshape(p.M, p.K).astype(np.float64) @ wf
    assert np.allclose(ideal.reshape(p.M, p.N), want, rtol=1e-12, atol=1e-12)
    g = logical(p, got).reshape(p.M, p.N).astype(np.float64)
    bound = p.K * 2.0 ** -24 * asum.reshape(p.M, p.N) + 2.0 ** -8 * np.abs(want)
    assert (np.abs(g - want) <= bound).all()


def test_config4_against_f64_and_textbook_gelu(oracle):
    p = configs.config4(M=8, N=64, K=512)
    got, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    s = dtp.e4m3_to_f32(p.src).reshape(p.M, p.K).astype(np.float64)
    w = dtp.e4m3_to_f32(p.wei).reshape(p.K, p.N).astype(np.float64)
    ss, ws = float(p.quant["src_scale"].data[0]), float(p.quant["wei_scale"].data[0])
    pre = (s @ w) * ss * ws
    assert np.allclose(ideal.reshape(p.M, p.N), pre, rtol=1e-12)
    x = pre + dtp.bf16_to_f32(p.bias).astype(np.float64)[None, :]
    gelu = 0.5 * x * (1 + np.tanh(np.sqrt(2 / np.pi) * x * (1 + 0.044715 * x * x)))
    want = gelu + dtp.bf16_to_f32(p.post_ops[1].data).reshape(p.M, p.N).astype(np.float64)
    g = logical(p, got).reshape(p.M, p.N).astype(np.float64)
    tol = 1.2 * p.K * 2.0 ** -24 * asum.reshape(p.M, p.N) + 2.0 ** -8 * np.abs(want) + 1e-6
    assert (np.abs(g - want) <= tol).all()


def test_config5_blocks_are_exact(oracle):
    p = configs.config5(M=8, N=32, K=256)
    got, ideal, _ = oracle.run_oracle(p, want_ideal=True)
    s = dtp.E2M1_VALUES[dtp.unpack_nibbles(p.src, p.M * p.K)].reshape(p.M, p.K).astype(np.float64)
    w = dtp.E2M1_VALUES[dtp.unpack_nibbles(p.wei, p.N * p.K)].reshape(p.N, p.K).T.astype(np.float64)
    sa = dtp.e8m0_to_f32(p.quant["src_scale"].data).reshape(p.M, -1).astype(np.float64)
    sb = dtp.e8m0_to_f32(p.quant["wei_scale"].data).reshape(-1, p.N).astype(np.float64)
    want = np.zeros((p.M, p.N))
    seq = np.zeros((p.M, p.N), F)
    for g in range(p.K // 32):
        blk = s[:, 32 * g:32 * g + 32] @ w[32 * g:32 * g + 32]
        assert (np.abs(blk) <= 1152).all() and np.array_equal(blk, blk.astype(F))   # exact in f32
        term = blk * sa[:, g][:, None] * sb[g][None, :]
        want += term
        seq = seq + term.astype(F)          # the reference's sequential f32 sum over blocks
    assert np.allclose(ideal.reshape(p.M, p.N), want, rtol=1e-13)
    assert np.array_equal(got.reshape(p.M, p.N), dtp.f32_to_bf16(seq).reshape(p.M, p.N))


def test_mx_quantize_follows_the_stated_rule():
    rng = np.random.default_rng(8)
    x = rng.standard_normal((4, 64)).astype(F)
    codes, sb = configs.mx_quantize(x, axis=1)
    for r in range(4):
        for g in range(2):
            blk = x[r, 32 * g:32 * g + 32]
            e = int(np.floor(np.log2(np.abs(blk).max() / 6.0)))
            assert sb[r, g] == e + 127
            assert np.array_equal(codes[r, 32 * g:32 * g + 32], dtp.f32_to_e2m1_codes(blk / F(2.0) ** e))


def test_post_ops_chain_and_broadcast(oracle):
    rng = np.random.default_rng(9)
    M, N, K = 6, 8, 16
    src = rng.integers(-4, 5, size=(M, K)).astype(F)
    wei = rng.integers(-4, 5, size=(K, N)).astype(F)
    per_n = rng.standard_normal(N).astype(F)
    per_m = rng.standard_normal(M).astype(F)
    dst0 = rng.integers(-50, 50, size=(M, N)).astype(F)
    po = [
        PostOp(kind=cabi.PO_SUM, scale=0.5, zero_point=3),
        PostOp(kind=cabi.PO_BINARY, alg=cabi.BINARY["mul"], dt=cabi.DT_F32, stride=(0, 0, 1), data=per_n),
        PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["linear"], alpha=2.0, beta=-1.0, scale=1.0),
        PostOp(kind=cabi.PO_BINARY, alg=cabi.BINARY["max"], dt=cabi.DT_F32, stride=(0, 1, 0), data=per_m),
        PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["clip"], alpha=-30.0, beta=40.0, scale=1.0),
    ]
    p = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_F32, wei_dt=cabi.DT_F32, dst_dt=cabi.DT_F32, src=src,
                      wei=wei, post_ops=po, dst_init=dst0)
    got = oracle.run_oracle(p).reshape(M, N)
    v = (src @ wei).astype(F)                      # small integers: exact
    v = v + F(0.5) * (dst0 - F(3))
    v = v * per_n[None, :]
    v = F(2) * v + F(-1)
    v = np.maximum(v, per_m[:, None])
    v = np.clip(v, F(-30), F(40))
    assert np.array_equal(got, v)


def test_eltwise_formulas(oracle):
    x = np.linspace(-6, 6, 241).astype(F)
    E = cabi.ELTWISE
    assert np.array_equal(oracle.eltwise(E["relu"], x, 0.1), np.where(x > 0, x, x * F(0.1)))
    assert np.array_equal(oracle.eltwise(E["abs"], x), np.abs(x))
    assert np.array_equal(oracle.eltwise(E["square"], x), x * x)
    assert np.array_equal(oracle.eltwise(E["round"], x * F(0.5)), np.rint(x * F(0.5)))
    x64 = x.astype(np.float64)
    gelu = 0.5 * x64 * (1 + np.tanh(0.79788458347320556640625 * x64 * (1 + 0.044715 * x64 * x64)))
    assert np.allclose(oracle.eltwise(E["gelu_tanh"], x), gelu, rtol=3e-6, atol=1e-7)
    assert np.allclose(oracle.eltwise(E["tanh"], x), np.tanh(x64), rtol=2e-6)
    assert np.allclose(oracle.eltwise(E["logistic"], x), 1 / (1 + np.exp(-x64)), rtol=2e-6)
    assert np.allclose(oracle.eltwise(E["swish"], x, 1.5), x64 / (1 + np.exp(-1.5 * x64)), rtol=3e-6, atol=1e-7)
    assert np.allclose(oracle.eltwise(E["elu"], x, 0.7), np.where(x64 > 0, x64, 0.7 * np.expm1(x64)), rtol=2e-6)
    assert np.array_equal(oracle.eltwise(E["hardsigmoid"], x, 0.2, 0.5), np.clip(F(0.2) * x + F(0.5), 0, 1).astype(F))
    import math
    erf = np.array([math.erf(v / math.sqrt(2)) for v in x64])
    assert np.allclose(oracle.eltwise(E["gelu_erf"], x), 0.5 * x64 * (1 + erf), rtol=3e-6, atol=1e-7)


def test_zero_dims_leave_dst_untouched(oracle):
    # ref_matmul_int8.cpp:70-72: any zero dim (K included) returns before writing
    dst0 = np.full((3, 4), 9, np.int32)
    p = MatmulProblem(M=3, N=4, K=0, src_dt=cabi.DT_S8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_S32,
                      src=np.zeros((3, 0), np.int8), wei=np.zeros((0, 4), np.int8), dst_init=dst0)
    assert (oracle.run_oracle(p) == 9).all()


def test_batched_broadcast_weights(oracle):
    rng = np.random.default_rng(10)
    B, M, N, K = 3, 4, 5, 32
    src = rng.integers(-9, 10, size=(B, M, K)).astype(np.int8)
    wei = rng.integers(-9, 10, size=(K, N)).astype(np.int8)
    p = MatmulProblem(batch=B, M=M, N=N, K=K, src_dt=cabi.DT_S8, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_S32,
                      src=src, wei=wei, wei_stride=(0, N, 1))
    got = oracle.run_oracle(p).reshape(B, M, N)
    assert np.array_equal(got, np.einsum("bmk,kn->bmn", src.astype(np.int64), wei.astype(np.int64)))


def test_row_sampling_of_the_full_size_checks_is_consistent():
    """The full-size GPU checks compare sampled dst rows with the oracle run on
    the sub-problem made of those rows: here the same construction against the
    oracle's own full result, for the three GEMM configurations."""
    from oracle import binding as orc
    from tests.test_gpu_full_size import row_slice, rows_of, sample_rows
    for make in (lambda: configs.config3(M=512, N=128, K=256, wtag="ba"),
                 lambda: configs.config4(M=512, N=128, K=256, wtag="ba"),
                 lambda: configs.config5(M=512, N=128, K=256, wtag="ba")):
        p = make()
        full = orc.run_oracle(p)
        rows = sample_rows(p.M, 2, 1)
        want = orc.run_oracle(row_slice(p, rows))
        assert np.array_equal(np.asarray(rows_of(p, full, rows)).view(np.uint8),
                              np.asarray(want).view(np.uint8).reshape(-1)), p.name


def test_binary_select_keeps_the_value_where_the_condition_is_nonzero(oracle):
    # primitive_attr_postops.cpp:44,345-360: res = src2 ? res : src1, the condition loaded as an integer
    # (negative values are true); exact integer sums, numpy `where` is the check
    r = np.random.default_rng(21)
    for cdt, cnp in ((cabi.DT_S8, np.int8), (cabi.DT_U8, np.uint8), (cabi.DT_S32, np.int32)):
        p = configs.config1(M=24, N=40, K=64, dst="s32")
        acc = np.asarray(oracle.run_oracle(p)).view(np.int32).reshape(p.M, p.N)
        other = r.integers(-9, 10, size=(p.M, p.N)).astype(np.float32)
        cond = r.integers(0 if cnp is np.uint8 else -1, 2, size=(1, p.N)).astype(cnp)
        p.post_ops = [PostOp(kind=cabi.PO_BINARY, alg=cabi.BINARY["select"], dt=cabi.DT_F32, stride=(0, p.N, 1), data=other),
                      PostOp(kind=cabi.PO_SELECT_COND, dt=cdt, stride=(0, 0, 1), data=cond),
                      PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["linear"], alpha=3.0, beta=-1.0, scale=1.0)]
        got = np.asarray(oracle.run_oracle(p)).view(np.int32).reshape(p.M, p.N)
        assert np.array_equal(got, 3 * np.where(cond != 0, acc, other.astype(np.int32)) - 1)
