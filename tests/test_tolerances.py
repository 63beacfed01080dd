"""The bounds of tests/helpers.py that the floating-point GPU checks use are
derived from the kernels' summation; here they are shown, on the CPU and
against float64, to accept a float32 evaluation in the kernels' factoring and
to reject the mistakes they are meant to catch: a zero point of one K-group off
by one, a group scale off by one bf16 unit in the last place, an epilogue scale
off by one bf16 unit."""
import copy

import numpy as np

from onednn_amd import cabi, configs
from onednn_amd import dtypes as dtp
from tests import helpers as H

F = np.float32


def emulate_decode(p, chunk=32):
    """The decode kernels' arithmetic in numpy float32: per K-group S1 = sum
    src * (128 + w) and S0 = sum src accumulated chunk by chunk (a chunk's
    products are added exactly, the running sum rounds), t = S1 - (128 + zp) * S0,
    dst += scale * t."""
    src, wz, G, sc, _ = H.decode_terms(p)
    # recover w and zp separately: decode_terms returns w - zp; the offset form needs both
    M, K = src.shape
    q = p.quant["wei_zp"]
    zp = H.decode(q.dt, q.data, (K // G) * p.N).astype(np.float64).reshape(K // G, p.N)
    w = wz + np.repeat(zp, G, 0)
    out = np.zeros((M, p.N), F)
    for g in range(K // G):
        s1 = np.zeros((M, p.N), F)
        s0 = np.zeros((M, 1), F)
        for c in range(g * G, (g + 1) * G, chunk):
            s1 = (s1 + (src[:, c:c + chunk] @ (128.0 + w[c:c + chunk])).astype(F)).astype(F)
            s0 = (s0 + src[:, c:c + chunk].sum(1, keepdims=True).astype(F)).astype(F)
        t = (s1 - ((128.0 + zp[g]).astype(F)[None, :] * s0).astype(F)).astype(F)
        out = (out + (sc[g].astype(F)[None, :] * t).astype(F)).astype(F)
    return out


def as_f32_dst(p):
    p = copy.copy(p)
    p.dst_dt = cabi.DT_F32
    return p


def test_decode_bound_accepts_the_factored_f32_sum_and_rejects_wrong_parameters(oracle):
    p = as_f32_dst(configs.config2(M=8, N=512, K=4096))
    _, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    exact, tol = H.decode_bound(p)
    # the oracle's float64 sum uses the float32-rounded decompressed weights of the reference
    assert (np.abs(ideal.reshape(p.M, p.N) - exact) <= H.U * asum.reshape(p.M, p.N)).all()
    tol = tol + H.U * asum.reshape(p.M, p.N)
    good = emulate_decode(p)
    worst = H.assert_within_bound(p, good.view(np.uint32), ideal, tol)
    assert worst < 0.5                                    # typical error is far inside the bound
    # the former bound, 20 * K * 2^-24 * sum|terms|, was two orders of magnitude wider
    assert np.median(20 * p.K * H.U * asum.reshape(p.M, p.N) / tol) > 50

    # a zero point of one K-group off by one
    bad = copy.deepcopy(p)
    z = dtp.unpack_nibbles(bad.quant["wei_zp"].data, (p.K // 128) * p.N).reshape(-1, p.N)
    z[5] = (z[5] + 1) % 16
    bad.quant["wei_zp"].data = dtp.pack_nibbles(z)
    out = emulate_decode(bad)
    want, _, _ = H.finish_f64(p, ideal)
    frac = np.mean(np.abs(out - want) > tol + H.U * np.abs(want))
    assert frac > 0.95
    # under the former bound nearly all of them passed
    assert np.mean(np.abs(out - want) > 20 * p.K * H.U * asum.reshape(p.M, p.N) + 2.0 ** -8 * np.abs(want)) < 0.05

    # a scale of one K-group off by one bf16 unit in the last place
    bad = copy.deepcopy(p)
    s = np.asarray(bad.quant["wei_scale"].data).view(np.uint16).reshape(-1, p.N).copy()
    s[7] += 1
    bad.quant["wei_scale"].data = s
    out = emulate_decode(bad)
    frac = np.mean(np.abs(out - want) > tol + H.U * np.abs(want))
    assert frac > 0.3
    # ... and a single (group, column) entry still shows in that column
    bad = copy.deepcopy(p)
    s = np.asarray(bad.quant["wei_scale"].data).view(np.uint16).reshape(-1, p.N).copy()
    s[7, 100] += 1
    bad.quant["wei_scale"].data = s
    out = emulate_decode(bad)
    miss = np.abs(out - want) > tol + H.U * np.abs(want)
    assert miss[:, 100].any() and not np.delete(miss, 100, axis=1).any()


def test_gemm_bound_accepts_chunked_f32_sums_and_rejects_a_misscaled_epilogue(oracle):
    p = configs.config4(M=8, N=128, K=8192)
    p.dst_dt = cabi.DT_F32
    _, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    ideal, asum = ideal.reshape(p.M, p.N), asum.reshape(p.M, p.N)
    s = dtp.e4m3_to_f32(p.src).reshape(p.M, p.K).astype(np.float64)
    w = dtp.e4m3_to_f32(p.wei).reshape(p.K, p.N).astype(np.float64)
    ss, ws = F(p.quant["src_scale"].data[0]), F(p.quant["wei_scale"].data[0])
    acc = np.zeros((p.M, p.N), F)
    for c in range(0, p.K, 64):                           # a K step of the fp8 kernel: 64 products, one rounding
        acc = (acc + (s[:, c:c + 64] @ w[c:c + 64]).astype(F)).astype(F)
    pre = ((acc * ss).astype(F) * ws).astype(F)
    tol = H.gemm_bound(p.K, asum) + 2 * H.U * np.abs(ideal)
    want, lip, extra = H.finish_f64(p, ideal)

    def finish32(x):
        x = x.astype(np.float64)
        v, _, _ = H.finish_f64(p, x)                      # chain in f64 on the f32 sum, rounded once
        return v.astype(F)

    good = finish32(pre)
    assert H.assert_within_bound(p, good.view(np.uint32), ideal, tol) < 0.5
    # the worst-case bound K * 2^-24 * sum|terms| is sqrt(3 K) / 4 = 39 times wider
    assert np.allclose(p.K * H.U * asum / H.gemm_bound(p.K, asum), np.sqrt(3 * p.K) / 4)
    # weights scale off by one bf16 unit in the last place (2^-8 relative)
    bad = finish32(((acc * ss).astype(F) * F(ws * (1 + 2.0 ** -8))).astype(F))
    full_tol = lip * tol + extra + H.dst_rounding(p.dst_dt, want)
    # (gelu flattens the negative half of the pre-activations: the mistake shows in the other half)
    assert np.mean(np.abs(bad - want) > full_tol) > 0.3
    assert np.mean(np.abs(bad - want) > p.K * H.U * asum) < 0.01   # the worst-case bound saw nothing
