"""Problems and closed-form expectations for the branches of the reference's
naive matmuls that the five benchmark configurations never take: precomputed
reductions with grouped src parameters (ref_matmul_int8.cpp:146-155,213-238),
the prelu post-op (primitive_attr_postops.cpp:218-241,362-389) and the eltwise
/ binary algorithms of compute_eltwise_scalar_fwd / compute_binary_scalar
(primitive_attr_postops.cpp:30-87).

Each builder returns the problem together with an expectation evaluated in
numpy from the written formula -- int64 for the integer part, float32 scalars
one rounding per operation where the reference's arithmetic is exact IEEE,
float64 where it calls libm.  tests/test_oracle_pins.py checks the oracle
against them on the CPU, tests/test_gpu_tail.py runs the same problems on the
device.  (Not a test module itself.)
"""
import numpy as np

from onednn_amd import cabi
from onednn_amd.problem import MatmulProblem, PostOp, QuantParam

F = np.float32
E, B = cabi.ELTWISE, cabi.BINARY


# ------------------------------------------------ precomputed reductions
def pr_case(seed, *, src_dt="s8", with_src_zp=False, src_zp_groups=False, true_sums=True, g=16, gw=32,
            with_scales=True, M=9, N=14, K=128, dst="f32"):
    """int8 matmul with DNNL_ARG_ATTR_PRECOMPUTED_REDUCTIONS | DNNL_ARG_SRC.

    Group sizes along K: reductions g (the smallest, matmul.cpp:585-600),
    weights zero points gw, src scales g, weights scales gw, src zero points gw
    (when grouped).  `true_sums=False` fills the reductions with random numbers
    instead of the group sums of src, so that the `- pr * zp_w` and the
    `+ G * zp_w * zp_s` terms show in the result on their own."""
    r = np.random.default_rng(seed)
    sd = np.uint8 if src_dt == "u8" else np.int8
    src = r.integers(np.iinfo(sd).min, np.iinfo(sd).max + 1, size=(M, K)).astype(sd)
    wei = r.integers(-128, 128, size=(K, N)).astype(np.int8)
    wz = r.integers(-7, 8, size=(K // gw, N)).astype(np.int8)
    q = {"wei_zp": QuantParam(cabi.DT_S8, 6, wz, (gw, 1))}
    if true_sums:
        pr = src.astype(np.int64).reshape(M, K // g, g).sum(-1).astype(np.int32)
    else:
        pr = r.integers(-3000, 3000, size=(M, K // g)).astype(np.int32)
    q["src_pr"] = QuantParam(cabi.DT_S32, 6, pr, (1, g))
    sz = None
    if with_src_zp:
        if src_zp_groups:
            sz = r.integers(-9, 10, size=(M, K // gw)).astype(np.int32)
            q["src_zp"] = QuantParam(cabi.DT_S32, 6, sz, (1, gw))
        else:
            sz = np.array([5], np.int32)
            q["src_zp"] = QuantParam(cabi.DT_S32, 0, sz)
    ss = ws = None
    if with_scales:
        ss = r.choice([0.0625, 0.125, 0.25, 0.5], size=(M, K // g)).astype(F)
        ws = r.uniform(0.001, 0.01, size=(K // gw, N)).astype(F)
        q["src_scale"] = QuantParam(cabi.DT_F32, 6, ss, (1, g))
        q["wei_scale"] = QuantParam(cabi.DT_F32, 6, ws, (gw, 1))
    p = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_NAMES[src_dt], wei_dt=cabi.DT_S8,
                      dst_dt=cabi.DT_NAMES[dst], src=src, wei=wei, quant=q, name=f"pr[{seed}]")

    # expectation: per reduction group, in exact integers
    #   acc_g = sum_k (s - zs) w  -  pr_g * zw  +  g * zw * zs
    # then f32(acc_g) * src_scale * wei_scale summed over groups in f32
    s64, w64 = src.astype(np.int64), wei.astype(np.int64)
    want = np.zeros((M, N), F)
    accs = []
    for gi in range(K // g):
        sl = slice(gi * g, (gi + 1) * g)
        zw = wz[gi * g // gw].astype(np.int64)[None, :]                 # [1, N]
        if sz is None:
            zs = np.zeros((M, 1), np.int64)
        elif src_zp_groups:
            zs = sz[:, gi * g // gw].astype(np.int64)[:, None]          # [M, 1]
        else:
            zs = np.full((M, 1), int(sz[0]), np.int64)
        acc = (s64[:, sl] - zs) @ w64[sl] - pr[:, gi].astype(np.int64)[:, None] * zw
        if sz is not None:
            acc = acc + g * zw * zs
        assert np.abs(acc).max() < 2 ** 31
        accs.append(acc)
        t = acc.astype(F)
        if with_scales:
            t = t * ss[:, gi][:, None]
            t = t * ws[gi * g // gw][None, :]
        want = want + t
    if true_sums:
        # with real group sums the whole expression is the plain zero-point form
        direct = sum(accs)
        zs_full = np.zeros((M, K), np.int64)
        if sz is not None:
            zs_full = np.repeat(sz.astype(np.int64), gw, 1) if src_zp_groups else np.full((M, K), int(sz[0]), np.int64)
        plain = np.zeros((M, N), np.int64)
        for gi in range(K // gw):
            sl = slice(gi * gw, (gi + 1) * gw)
            plain += (s64[:, sl] - zs_full[:, sl]) @ (w64[sl] - wz[gi].astype(np.int64)[None, :])
        assert np.array_equal(direct, plain)
    if dst == "s32":
        want = np.rint(want).astype(np.int32)
    return p, want


# ----------------------------------------------------------------- prelu
def prelu_case(seed, mask_m, mask_n, *, batch=1, mask_b=False, M=7, N=12, K=16):
    """f32 matmul on small integers (exact sums) followed by prelu.  The weights
    array is built in the reference's layout -- ab for two dims, acb for three
    (get_prelu_weights_format): dims under the mask, the M dim innermost when
    there is a batch dim -- and the strides handed to the kernels index it."""
    r = np.random.default_rng(seed)
    src = r.integers(-4, 5, size=(batch, M, K)).astype(F)
    wei = r.integers(-4, 5, size=(batch, K, N)).astype(F)
    db, dm, dn = (batch if mask_b else 1), (M if mask_m else 1), (N if mask_n else 1)
    if batch == 1:
        w = r.uniform(-2, 2, size=(dm, dn)).astype(F)               # tag ab
        stride = (0, dn if mask_m else 0, 1 if mask_n else 0)
        at = lambda b, m, n: w[m if mask_m else 0, n if mask_n else 0]
    else:
        w = r.uniform(-2, 2, size=(db, dn, dm)).astype(F)           # tag acb: memory order batch, N, M
        stride = (dn * dm if mask_b else 0, 1 if mask_m else 0, dm if mask_n else 0)
        at = lambda b, m, n: w[b if mask_b else 0, n if mask_n else 0, m if mask_m else 0]
    p = MatmulProblem(batch=batch, M=M, N=N, K=K, src_dt=cabi.DT_F32, wei_dt=cabi.DT_F32, dst_dt=cabi.DT_F32,
                      src=src, wei=wei, name=f"prelu[{seed}]",
                      post_ops=[PostOp(kind=cabi.PO_PRELU, dt=cabi.DT_F32, stride=stride, data=w)])
    v = np.einsum("bmk,bkn->bmn", src, wei).astype(F)
    want = v.copy()
    for b in range(batch):
        for m in range(M):
            for n in range(N):
                if not v[b, m, n] >= 0:
                    want[b, m, n] = at(b, m, n) * v[b, m, n]
    return p, want, w


# -------------------------------------------------- eltwise / binary tail
def _int8_base(seed, positive, scale, M=16, N=64, K=64, lim=4):
    r = np.random.default_rng(seed)
    if positive:
        src = r.integers(0, lim + 1, size=(M, K)).astype(np.uint8)
        sdt = cabi.DT_U8
    else:
        src = r.integers(-lim, lim + 1, size=(M, K)).astype(np.int8)
        sdt = cabi.DT_S8
    wei = (r.integers(0, lim + 1, size=(K, N)) if positive else r.integers(-lim, lim + 1, size=(K, N))).astype(np.int8)
    acc = src.astype(np.int64) @ wei.astype(np.int64)
    q = {}
    x = acc.astype(F)
    if scale is not None:
        q["src_scale"] = QuantParam(cabi.DT_F32, 0, np.array([scale], F))
        x = x * F(scale)
    p = MatmulProblem(M=M, N=N, K=K, src_dt=sdt, wei_dt=cabi.DT_S8, dst_dt=cabi.DT_F32, src=src, wei=wei, quant=q)
    return p, x


def _softrelu64(x, a):
    # the argument of exp is the float32 product the reference forms (`in = s * alpha`)
    t = (x.astype(F) * F(a)).astype(np.float64)
    return np.where(t < 88.72283172607421875, np.log1p(np.exp(np.minimum(t, 88.8))), t) / np.float64(F(a))


# name -> (alg, alpha, beta, positive inputs, src scale, f64 formula or None (exact float32 formula below))
ELTWISE_TAIL = {
    "sqrt": (E["sqrt"], 0.0, 0.0, True, 0.37, None),
    "exp": (E["exp"], 0.0, 0.0, False, 0.11, lambda x: np.exp(x)),
    "log": (E["log"], 0.0, 0.0, True, 0.37, lambda x: np.log(x)),
    "pow_sq": (E["pow"], 1.5, 2.0, False, 0.25, lambda x: 1.5 * x ** 2.0),
    "pow_sqrt": (E["pow"], 0.75, 0.5, True, 0.37, lambda x: 0.75 * x ** 0.5),
    "pow_inv": (E["pow"], 2.0, -1.0, True, 0.37, lambda x: 2.0 / x),
    "soft_relu": (E["soft_relu"], 0.7, 0.0, False, 0.9, lambda x: _softrelu64(x, 0.7)),
    "soft_relu_big": (E["soft_relu"], 2.0, 0.0, False, 1.5, lambda x: _softrelu64(x, 2.0)),
    "mish": (E["mish"], 0.0, 0.0, False, 0.21, lambda x: x * np.tanh(_softrelu64(x, 1.0))),
    "mish_big": (E["mish"], 0.0, 0.0, False, 1.5, lambda x: x * np.tanh(_softrelu64(x, 1.0))),
    "clip_v2": (E["clip_v2"], -3.25, 7.5, False, 0.37, None),
    "hardswish": (E["hardswish"], 1.0 / 6.0, 0.5, False, 0.09, None),
    "tanh": (E["tanh"], 0.0, 0.0, False, 0.05, lambda x: np.tanh(x)),
    "elu": (E["elu"], 0.7, 0.0, False, 0.11, lambda x: np.where(x > 0, x, np.float64(F(0.7)) * np.expm1(x))),
    "logistic": (E["logistic"], 0.0, 0.0, False, 0.11, lambda x: 1.0 / (1.0 + np.exp(-x))),
    "swish": (E["swish"], 1.5, 0.0, False, 0.11, lambda x: x / (1.0 + np.exp(-(F(1.5) * x.astype(F)).astype(np.float64)))),
    "gelu_erf": (E["gelu_erf"], 0.0, 0.0, False, 0.05, None),
    "abs": (E["abs"], 0.0, 0.0, False, 0.37, None),
    "square": (E["square"], 0.0, 0.0, False, 0.37, None),
    "round": (E["round"], 0.0, 0.0, False, 0.5, None),
    "hardsigmoid": (E["hardsigmoid"], 0.2, 0.5, False, 0.09, None),
    "linear": (E["linear"], 1.7, -0.3, False, 0.37, None),
    "relu_leaky": (E["relu"], 0.1, 0.0, False, 0.37, None),
    "clip": (E["clip"], -3.25, 7.5, False, 0.37, None),
}


def _exact_eltwise(name, x, alpha, beta):
    a, b = F(alpha), F(beta)
    if name == "sqrt":
        return np.sqrt(x)                        # correctly rounded in IEEE, as sqrtf
    if name in ("clip_v2", "clip"):
        return np.minimum(np.maximum(x, a), b)
    if name in ("hardswish", "hardsigmoid"):
        v = a * x + b
        h = np.where(v <= 0, F(0), np.where(v >= 1, F(1), v)).astype(F)
        return x * h if name == "hardswish" else h
    if name == "abs":
        return np.where(x > 0, x, -x)            # abs_fwd: a zero leaves as -0
    if name == "square":
        return x * x
    if name == "round":
        return np.rint(x)
    if name == "linear":
        return a * x + b
    if name == "relu_leaky":
        return np.where(x > 0, x, x * a)
    raise KeyError(name)


def eltwise_case(name, seed=3):
    alg, alpha, beta, positive, scale, f64 = ELTWISE_TAIL[name]
    p, x = _int8_base(seed, positive, scale)
    p.post_ops = [PostOp(kind=cabi.PO_ELTWISE, alg=alg, alpha=alpha, beta=beta, scale=1.0)]
    p.name = f"eltwise:{name}"
    if name == "gelu_erf":
        import math
        x64 = x.astype(np.float64)
        erf = np.vectorize(math.erf)((x * F(0.707106769084930419921875)).astype(np.float64))
        # `1.f + erff(v)` cancels for negative v: the float32 formula itself carries
        # an absolute error of an ulp of one times |s| / 2
        return p, 0.5 * x64 * (1 + erf), ("ulp", np.abs(x64) * 2.0 ** -23)
    if f64 is None:
        return p, _exact_eltwise(name, x, alpha, beta).astype(F), "exact"
    with np.errstate(over="ignore", divide="ignore", invalid="ignore"):
        return p, f64(x.astype(np.float64)), ("ulp", 1e-37)


BINARY_TAIL = ["div", "min", "sub", "ge", "gt", "le", "lt", "eq", "ne", "add", "mul", "max"]


def binary_case(name, operand="per_element", seed=4, odt="f32"):
    """x = integer-valued accumulators; y = small integers (non-zero for div),
    so that every comparison meets equal operands somewhere."""
    p, x = _int8_base(seed, False, None, K=16, lim=2)
    r = np.random.default_rng(seed + 100)
    shape = {"per_element": (p.M, p.N), "per_n": (1, p.N), "per_m": (p.M, 1), "scalar": (1, 1)}[operand]
    y = r.integers(-8, 9, size=shape)
    if name == "div":
        y = np.where(y == 0, 3, y)
    y = y.astype(F)
    stride = (0, shape[1] if shape[0] > 1 else 0, 1 if shape[1] > 1 else 0)
    if odt == "f32":
        data, dt = y, cabi.DT_F32
    elif odt == "s8":
        data, dt = y.astype(np.int8), cabi.DT_S8
    else:
        from onednn_amd import dtypes as dtp
        data, dt = dtp.f32_to_bf16(y), cabi.DT_BF16
    p.post_ops = [PostOp(kind=cabi.PO_BINARY, alg=B[name], dt=dt, stride=stride, data=data)]
    p.name = f"binary:{name}:{operand}:{odt}"
    yb = np.broadcast_to(y, (p.M, p.N))
    fn = {"div": lambda: x / yb, "min": lambda: np.minimum(x, yb), "sub": lambda: x - yb,
          "ge": lambda: x >= yb, "gt": lambda: x > yb, "le": lambda: x <= yb, "lt": lambda: x < yb,
          "eq": lambda: x == yb, "ne": lambda: x != yb, "add": lambda: x + yb, "mul": lambda: x * yb,
          "max": lambda: np.maximum(x, yb)}[name]
    want = fn().astype(F)
    if name in ("ge", "gt", "le", "lt", "eq", "ne"):
        assert 0 < want.sum() < want.size                              # both outcomes occur
    if name in ("ge", "le", "eq", "ne"):
        assert (x == yb).any()                                         # equal operands occur
    return p, want


def ulp_close(got, want64, ulps=4, atol=0.0):
    """|got - want| within `ulps` float32 units in the last place of want (plus atol)."""
    got = np.asarray(got, np.float64)
    w = np.asarray(want64, np.float64)
    with np.errstate(invalid="ignore", over="ignore"):
        w32 = w.astype(F)
        spacing = np.spacing(np.abs(w32)).astype(np.float64)
        ok = np.abs(got - w) <= ulps * spacing + atol
    ok |= np.isinf(w32) & (got == w32)            # overflow to the same infinity
    ok |= np.isnan(w) & np.isnan(got)
    return ok
