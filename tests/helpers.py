"""Comparison rules shared by the parity tests.

Integer dst (s32/s8/u8): bit-exact.  Floating-point dst: the relaxation ladder
of the reference's own checker (tests/benchdnn/utils/compare.cpp:345-513):
exact match, else |exp| <= 1e-5 and diff < eps_f32, else rel diff <= trh, with
trh = max(eps_dt, 1e-5) widened to the eltwise constants (diff <= max(eps_dt,
2e-5) or rdiff <= max(eps_dt, 8e-6)) when a transcendental post-op is present.
For results that depend on the summation order (f32 accumulation over K) the
accepted error is additionally bounded by the forward error of the sum:
K * 2^-24 * sum|terms| (see the oracle's `abs_sum`).
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
            bound = prob.K * 2.0 ** -24 * np.asarray(abs_sum).reshape(g.shape)
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
