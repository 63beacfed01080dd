"""Comparison rules shared by the parity tests.

Integer dst (s32/s8/u8): bit-exact.  Floating-point dst: the relaxation ladder
of the reference's own checker (tests/benchdnn/utils/compare.cpp:345-513):
exact match, else |exp| <= 1e-5 and diff < eps_f32, else rel diff <= trh, with
trh = max(eps_dt, 1e-5) widened to the eltwise constants (diff <= max(eps_dt,
2e-5) or rdiff <= max(eps_dt, 8e-6)) when a transcendental post-op is present.
For results that depend on the summation order (f32 accumulation over K) the
accepted difference between two float32 evaluations is additionally bounded by
twice gemm_bound(): the sqrt(K)-type bound on one float32 K-sum against its
exact value, from the oracle's `abs_sum` = sum|terms|.  The checks at the
benchmark shapes do not use the ladder: they compare with the oracle's float64
sum under bounds derived from the kernels' summation (decode_bound, gemm_bound,
assert_within_bound below).
"""
import numpy as np

from onednn_amd import cabi
from onednn_amd.problem import decode

EPS = {cabi.DT_F32: 2.0 ** -23, cabi.DT_BF16: 2.0 ** -7, cabi.DT_F16: 2.0 ** -10,
       cabi.DT_F8_E4M3: 2.0 ** -3, cabi.DT_F8_E5M2: 2.0 ** -2}


def logical(prob, raw):
    """dst storage -> float32 [batch, M, N] honouring dst strides."""
    span = prob.dst_span()
    flat = decode(prob.dst_dt, raw, span)
    b, m, n = np.meshgrid(np.arange(prob.batch), np.arange(prob.M), np.arange(prob.N), indexing="ij")
    off = b * prob.dst_stride[0] + m * prob.dst_stride[1] + n * prob.dst_stride[2]
    return flat[off]


def assert_bit_exact(prob, got_raw, want_raw, what=""):
    got = np.ascontiguousarray(got_raw).view(np.uint8)
    want = np.ascontiguousarray(want_raw).view(np.uint8)
    assert got.shape == want.shape
    if not np.array_equal(got, want):
        g, w = logical(prob, got_raw), logical(prob, want_raw)
        bad = np.argwhere(g != w)
        first = tuple(bad[0]) if len(bad) else None
        raise AssertionError(
            f"{prob.name} {what}: {len(bad)} of {g.size} elements differ; first at {first}: "
            f"got {g[first] if first else '?'} want {w[first] if first else '?'}")


def compare(prob, got_raw, want_raw, *, abs_sum=None, transcendental=False, extra_rel=0.0):
    """The comparison ladder: returns (number of elements outside tolerance,
    description of the first one).  Integer dst types compare exactly."""
    g = logical(prob, got_raw).astype(np.float64)
    w = logical(prob, want_raw).astype(np.float64)
    if prob.dst_dt in (cabi.DT_S32, cabi.DT_S8, cabi.DT_U8):
        ok = g == w
    else:
        eps = EPS[prob.dst_dt]
        diff = np.abs(g - w)
        rdiff = diff / np.maximum(np.abs(w), 1e-30)
        ok = (g == w) | (np.isnan(g) & np.isnan(w))
        ok |= (np.abs(w) <= 1e-5) & (diff < 2.0 ** -23)
        trh = max(eps, 1e-5) + extra_rel
        ok |= rdiff <= trh
        if transcendental:
            ok |= (diff <= max(eps, 2e-5)) | (rdiff <= max(eps, 8e-6))
        if abs_sum is not None:
            # got and want are both float32 K-sums: each within gemm_bound of the exact value
            bound = 2.0 * gemm_bound(prob.K, np.asarray(abs_sum).reshape(g.shape))
            if prob.src_dt in (cabi.DT_F8_E4M3, cabi.DT_F8_E5M2):
                # the matrix cores' fp8 dot product drops bits below 2^-13 of the largest product of
                # a group of eight (see fp8_mfma_bound): 1e-5 * sum|terms| covers it at every K
                bound = bound + 1e-5 * np.asarray(abs_sum).reshape(g.shape)
            # one ulp of the dst type on top of the accumulation bound
            ok |= diff <= bound + eps * np.abs(w)
    if ok.all():
        return 0, ""
    bad = np.argwhere(~ok)
    i = tuple(bad[0])
    return len(bad), (f"{len(bad)} of {g.size} outside tolerance; first at {tuple(int(x) for x in i)}: "
                      f"got {g[i]} want {w[i]} diff {abs(g[i] - w[i]):.3e}")


def assert_close(prob, got_raw, want_raw, *, abs_sum=None, transcendental=False, what="",
                 extra_rel=0.0):
    nbad, msg = compare(prob, got_raw, want_raw, abs_sum=abs_sum, transcendental=transcendental,
                        extra_rel=extra_rel)
    if nbad:
        raise AssertionError(f"{prob.name} {what}: {msg}")


# --------------------------------------------------------------------------
# Bounds derived from the kernels' own summation, against a float64 evaluation
# --------------------------------------------------------------------------
U = 2.0 ** -24            # unit roundoff of float32


def _strided(flat, dims, strides):
    idx = np.zeros(dims, np.int64)
    for ax, (d, s) in enumerate(zip(dims, strides)):
        shape = [1] * len(dims)
        shape[ax] = d
        idx = idx + (np.arange(d, dtype=np.int64) * s).reshape(shape)
    return flat[idx]


def decode_terms(p):
    """float64 pieces of a weight-only decode problem: src [M, K], w - zp [K, N],
    the K-group size of the factored form and the per-group scales [K/G, N]."""
    assert p.batch == 1
    M, N, K = p.M, p.N, p.K
    src = decode(p.src_dt, p.src, M * K).astype(np.float64).reshape(M, K)
    span = (K - 1) * p.wei_stride[1] + (N - 1) * p.wei_stride[2] + 1
    w = _strided(decode(p.wei_dt, p.wei, span).astype(np.float64), (K, N), p.wei_stride[1:])

    def param(name, default):
        if name not in p.quant:
            return K, np.full((1, N), default, np.float64)
        q = p.quant[name]
        g = q.groups[0] if (q.mask & 2) else K
        rows = K // g
        cols = N if (q.mask & 4) else 1
        v = decode(q.dt, q.data, rows * cols).astype(np.float64).reshape(rows, cols)
        return g, np.broadcast_to(v, (rows, N))

    gs, sc = param("wei_scale", 1.0)
    gz, zp = param("wei_zp", 0.0)
    G = min(gs, gz)
    sc = np.repeat(sc, gs // G, 0)
    zp = np.repeat(zp, gz // G, 0)
    return src, w - np.repeat(zp, G, 0), G, sc, float(np.abs(zp).max())


def decode_bound(p, sf=3.0):
    """(exact, tol), both [M, N] float64, for the pre-bias sum of the decode
    kernels, which evaluate per K-group g of size G and column n

        t_g = S1 - (128 + zp) * S0,   S1 = sum_k src * (128 + w),  S0 = sum_k src
        dst = sum_g scale[g, n] * t_g

    in float32 on the matrix cores.  `exact` is that expression over the reals.
    Error model: every partial sum of S1 and S0 (times 128 + zp) is at most
    P_g = C * sum_{k in g} |src| in magnitude, C = 128 + 15 + max|zp| + 8, in
    whatever order the hardware adds; each of the at most 2G + 2 additions and
    multiplications of a group rounds with an error of at most U * P_g, taken as
    independent and uniform: standard deviation U / sqrt(3) * P_g each.  The bound
    is `sf` standard deviations of the total -- on normal data P_g is about ten
    times the typical partial sum, so sf = 3 leaves a wide margin -- plus worst-case
    terms for the cross-group additions and the scale multiplication,
    (K/G + 2) * U * sum_g |scale_g t_g|."""
    src, wz, G, sc, zmax = decode_terms(p)
    M, K = src.shape
    ng = K // G
    C = 128.0 + 15.0 + zmax + 8.0
    A = np.abs(src).reshape(M, ng, G).sum(-1)                       # [M, ng]
    exact = np.zeros((M, p.N))
    T = np.zeros((M, p.N))
    for g in range(ng):
        t = (src[:, g * G:(g + 1) * G] @ wz[g * G:(g + 1) * G]) * sc[g][None, :]
        exact += t
        T += np.abs(t)
    within = sf * (U / np.sqrt(3.0)) * np.sqrt(2.0 * G + 2.0) * C * np.sqrt((A * A) @ (sc * sc))
    return exact, within + (ng + 2) * U * T


def gemm_bound(K, abs_sum, sf=4.0):
    """Bound on the error of a float32 K-sum of exactly representable products
    against its float64 value: every partial sum is at most sum|terms| =
    `abs_sum` in magnitude, each of the K additions rounds by at most U times
    that, taken as independent and uniform (standard deviation U / sqrt(3) *
    abs_sum): `sf` standard deviations of the total, sqrt(K) instead of the
    worst case's K.  On zero-mean data the typical partial sum is a further
    sqrt(K) below abs_sum, which is the margin behind sf = 4."""
    return sf * (U / np.sqrt(3.0)) * np.sqrt(float(K)) * np.asarray(abs_sum, np.float64)


def finish_f64(p, pre):
    """bias and the post-op chain in float64 for the chains the configurations
    use (relu, gelu_tanh, swish, linear, binary add / mul, per element or per column).
    Returns (value, lip, extra): `lip` = how much an error of the pre-bias sum is
    amplified at most, `extra` = absolute error the float32 evaluation of the
    chain itself may add (a few units in the last place per step)."""
    M, N = p.M, p.N
    v = np.asarray(pre, np.float64).reshape(M, N).copy()
    lip = np.ones((M, N))
    extra = np.zeros((M, N))
    if p.bias is not None:
        b = decode(p.bias_dt, p.bias, np.asarray(p.bias).size).astype(np.float64)
        v = v + _strided(b, (M, N), p.bias_stride[1:])
        extra += U * np.abs(v)
    for po in p.post_ops:
        if po.kind == cabi.PO_ELTWISE and po.alg == cabi.ELTWISE["relu"] and po.alpha == 0:
            v = np.maximum(v, 0.0)
        elif po.kind == cabi.PO_ELTWISE and po.alg == cabi.ELTWISE["gelu_tanh"]:
            x = v
            v = 0.5 * x * (1 + np.tanh(0.79788458347320556640625 * x * (1 + 0.044715 * x * x)))
            lip = lip * 1.13                       # sup |gelu'| = 1.129
            extra = extra * 1.13 + 32 * U * np.maximum(np.abs(x), 1.0)
        elif po.kind == cabi.PO_ELTWISE and po.alg == cabi.ELTWISE["swish"]:
            x = v
            with np.errstate(over="ignore"):
                v = x / (1.0 + np.exp(-np.float64(np.float32(po.alpha)) * x))
            lip = lip * 1.1                        # sup |swish'| = 1.0998 whatever alpha
            extra = extra * 1.1 + 32 * U * np.maximum(np.abs(x), 1.0)
        elif po.kind == cabi.PO_ELTWISE and po.alg == cabi.ELTWISE["linear"]:
            v = po.alpha * v + po.beta
            lip, extra = lip * abs(po.alpha), extra * abs(po.alpha) + 2 * U * np.abs(v)
        elif po.kind == cabi.PO_BINARY and po.alg in (cabi.BINARY["add"], cabi.BINARY["mul"]):
            n_el = np.asarray(po.data).size * (2 if cabi.DT_BITS[po.dt] == 4 else 1)
            y = _strided(decode(po.dt, po.data, n_el).astype(np.float64), (M, N), po.stride[1:])
            if po.alg == cabi.BINARY["add"]:
                v = v + y
            else:
                v = v * y
                lip, extra = lip * np.abs(y), extra * np.abs(y)
            extra = extra + U * np.abs(v)
        else:
            raise NotImplementedError(f"finish_f64: post-op kind {po.kind} alg {po.alg:#x}")
        if po.kind == cabi.PO_ELTWISE and po.scale != 1.0:
            v, lip, extra = v * po.scale, lip * abs(po.scale), extra * abs(po.scale)
    assert "dst_scale" not in p.quant and "dst_zp" not in p.quant
    return v, lip, extra


def dst_rounding(dst_dt, v):
    """Half a unit in the last place of the dst type at |v| (zero for f32)."""
    if dst_dt == cabi.DT_F32:
        return U * np.abs(v)
    bits = {cabi.DT_BF16: 8, cabi.DT_F16: 11}[dst_dt]
    tiny = {cabi.DT_BF16: 2.0 ** -133, cabi.DT_F16: 2.0 ** -25}[dst_dt]
    return np.abs(v) * 2.0 ** -bits * (1 + 2.0 ** -10) + tiny


def assert_within_bound(p, got_raw, pre_exact, pre_tol, what=""):
    """dst against float64: |got - finish(pre_exact)| <= lip * pre_tol + chain
    rounding + half an ulp of the dst type."""
    want, lip, extra = finish_f64(p, pre_exact)
    got = logical(p, got_raw).astype(np.float64).reshape(p.M, p.N)
    tol = lip * np.asarray(pre_tol, np.float64).reshape(p.M, p.N) + extra + dst_rounding(p.dst_dt, want)
    bad = ~(np.abs(got - want) <= tol)
    if bad.any():
        i = tuple(int(x) for x in np.argwhere(bad)[0])
        raise AssertionError(f"{p.name} {what}: {int(bad.sum())} of {got.size} outside the bound; first at {i}: "
                             f"got {got[i]} want {want[i]} diff {abs(got[i] - want[i]):.3e} tol {tol[i]:.3e}; "
                             f"max diff/tol {float(np.nanmax(np.abs(got - want) / tol)):.2f}")
    return float(np.max(np.abs(got - want) / tol))


def assert_decode_close(p, got_raw, ideal, abs_sum, what="", bound=None):
    """A decode kernel's dst against the oracle's float64 sum `ideal` under
    decode_bound.  The oracle's sum uses the reference's float32-rounded
    decompressed weights, the kernels the unrounded (w - zp) * scale: they differ
    by at most U * sum|terms|, checked here and added to the bound."""
    exact, tol = bound if bound is not None else decode_bound(p)
    ideal = np.asarray(ideal, np.float64).reshape(p.M, p.N)
    asum = np.asarray(abs_sum, np.float64).reshape(p.M, p.N)
    assert (np.abs(ideal - exact) <= U * asum + 1e-300).all(), "oracle float64 sum vs numpy"
    return assert_within_bound(p, got_raw, ideal, tol + U * asum, what)


def fp8_mfma_bound(p):
    """What the matrix cores' fp8 dot product adds to gemm_bound, [M, N] float64.

    Measured on MI355X (v_mfma_f32_32x32x64_f8f6f4, one large product next to 63
    small ones): the products are added in groups of eight, aligned to the
    largest of the group, and bits below 2^-13 of it are dropped (toward zero);
    a small product is kept exactly down to 2^-13 of the large one and lost
    below, and only the seven that share the large one's group are affected.
    Model: each of the seven smaller products of a group loses up to
    q = 2^-13 max|product|, independent and uniform (variance q^2 / 3).  Which
    eight k share a group is not needed: max over a group <= max over its
    64-long K block <= max|src| * max|wei| of the block, so
        variance <= 7/3 * 8 * 2^-26 * sum_blocks (max|src| max|wei|)^2 * scales^2.
    One standard deviation of this model is returned: products near the group
    maximum lose nothing, which makes the model ten times wider than the
    measured error (rms 17 / 8.6 / 4.2 units of U * sum|terms| at K = 512 / 2048 /
    8192 on the configuration's data, maxima 101 / 39 / 18; this bound 530 / 270 /
    130)."""
    assert p.batch == 1
    M, N, K = p.M, p.N, p.K
    s = np.abs(decode(p.src_dt, p.src, M * K).astype(np.float64)).reshape(M, K)
    span = (K - 1) * p.wei_stride[1] + (N - 1) * p.wei_stride[2] + 1
    w = np.abs(_strided(decode(p.wei_dt, p.wei, span).astype(np.float64), (K, N), p.wei_stride[1:]))
    if K % 64:      # a K that ends inside a block: the block's other products are zeros
        pad = 64 - K % 64
        s = np.concatenate([s, np.zeros((M, pad))], 1)
        w = np.concatenate([w, np.zeros((pad, N))], 0)
        K += pad
    S = s.reshape(M, K // 64, 64).max(2)
    W = w.reshape(K // 64, 64, N).max(1)
    sc = 1.0
    for name in ("src_scale", "wei_scale"):
        if name in p.quant:
            q = p.quant[name]
            assert q.mask == 0
            sc *= float(decode(q.dt, q.data, 1)[0])
    return np.sqrt(7.0 / 3.0 * 8.0 * ((S * S) @ (W * W))) * 2.0 ** -13 * abs(sc)


def assert_gemm_close(p, got_raw, ideal, abs_sum, what="", sf=4.0, hw=None):
    """A GEMM kernel's dst against the oracle's float64 sum `ideal` (scales
    included) under gemm_bound, plus two roundings for the scale multiplications
    and, for the fp8 matrix-core kernel, `hw` = fp8_mfma_bound(p)."""
    ideal = np.asarray(ideal, np.float64).reshape(p.M, p.N)
    asum = np.asarray(abs_sum, np.float64).reshape(p.M, p.N)
    tol = gemm_bound(p.K, asum, sf) + 2 * U * np.abs(ideal)
    if hw is not None:
        tol = tol + hw
    return assert_within_bound(p, got_raw, ideal, tol, what)
