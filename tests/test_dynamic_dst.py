"""Dynamic (MX) quantization of dst: `quantization_mode::dynamic_mx` scales on
DNNL_ARG_DST are an output of the matmul (ref_matmul.cpp:268-423, rules
src/common/matmul.cpp:407-424).

What pins the oracle without running the reference: the group scale is a pure
function of the group's largest magnitude through exponent bytes
(float8.cpp:29-45: e8m0(x) keeps the exponent byte of x), so
  * constructed groups have known answers (amax 448 -> scale 1; amax 1 ->
    2^-8; amax just below 2 -> the scale of 1, and its largest values then
    saturate at the dst maximum; an all-zero group -> scale byte 0, zeros),
  * random problems are restated with numpy integer arithmetic on the f32 bit
    patterns of the pre-quantization values, which come from the oracle's own
    static path with an f32 dst (pinned elsewhere).
GPU: the generic kernel follows the same operations in the same order and
must reproduce dst and scales bit for bit; the GEMM tile kernels are checked
through the dequantized result.
"""
import numpy as np
import pytest

from onednn_amd import cabi, configs
from onednn_amd import dtypes as dtp
from onednn_amd.problem import GpuRun, MatmulProblem, PostOp, QuantParam
from oracle import binding as orc

DT_MAX = {cabi.DT_F8_E4M3: 448.0, cabi.DT_F8_E5M2: 57344.0}


def f32_problem(d, dst_dt):
    """dst = I x d: every pre-quantization value is exactly d[m, n]."""
    M, N = d.shape
    p = MatmulProblem(M=M, N=N, K=M, src_dt=cabi.DT_F32, wei_dt=cabi.DT_F32, dst_dt=dst_dt,
                      src=np.eye(M, dtype=np.float32), wei=np.ascontiguousarray(d, dtype=np.float32), name="dyn-f32")
    return dynamic(p)


def dynamic(p):
    p.quant["dst_scale"] = QuantParam(cabi.DT_E8M0, configs.MASK_ROW | configs.MASK_COL,
                                      np.zeros((p.batch, p.M, p.N // 32), np.uint8), (1, 32))
    p.dst_dynamic = cabi.DST_DYNAMIC_MX
    return p


def exponent_byte(x):
    return ((np.asarray(x, np.float32).view(np.uint32) >> 23) & 0xff).astype(np.uint8)


def from_exponent_byte(b):
    b = np.asarray(b, np.uint32)
    bits = np.where(b == 0, np.uint32(0x00400000), b << 23).astype(np.uint32)
    return bits.view(np.float32)


def numpy_dynamic(d, dst_dt):
    """The reference's steps on pre-quantization values d [rows, N]."""
    rows, N = d.shape
    g = d.reshape(rows, N // 32, 32)
    amax = np.abs(g).max(axis=2)
    dmax = np.float32(DT_MAX[dst_dt])
    ratio = from_exponent_byte(exponent_byte(amax)) / from_exponent_byte(exponent_byte(dmax))
    sbyte = exponent_byte(ratio.astype(np.float32))
    inv = np.float32(1.0) / from_exponent_byte(sbyte)
    x = np.clip(g * inv[:, :, None], -dmax, dmax).astype(np.float32).reshape(rows, N)
    to = dtp.f32_to_e4m3 if dst_dt == cabi.DT_F8_E4M3 else orc.f32_to_e5m2
    return to(x.reshape(-1)).reshape(rows, N), sbyte


# ------------------------------------------------------------------ CPU
def test_known_answers_of_the_group_scale():
    d = np.zeros((4, 64), np.float32)
    d[0, :32] = np.linspace(-448, 448, 32)            # amax 448 -> 256 / 256 = 1
    d[0, 32:] = 1.0                                   # amax 1 -> 1 / 256
    d[1, :32] = np.float32(1.9999999)                 # e8m0 rounds down to 1: x * 256 = 511.99 saturates at 448
    d[1, 0] = 0.5
    d[1, 32:] = 0.0                                   # all-zero group
    d[2, :32] = 3e-39                                 # subnormal amax: exponent byte 0 -> 2^-127 / 2^8 underflows to byte 0
    d[2, 32:] = 1e30                                  # 2^99 / 2^8 = 2^91
    d[3, :] = -np.arange(64, dtype=np.float32)
    p = f32_problem(d, cabi.DT_F8_E4M3)
    dst, sc = orc.run_oracle_dynamic(p)
    sc = sc.reshape(4, 2)
    val = dtp.e4m3_to_f32(dst).reshape(4, 64)
    assert sc[0, 0] == 127 and np.array_equal(val[0, :32], dtp.e4m3_to_f32(dtp.f32_to_e4m3(d[0, :32])))
    assert sc[0, 1] == 127 - 8 and np.all(val[0, 32:] == 256.0)
    assert sc[1, 0] == 127 - 8 and np.all(val[1, 1:32] == 448.0) and val[1, 0] == 128.0
    assert sc[1, 1] == 0 and np.all(val[1, 32:] == 0.0)
    assert sc[2, 0] == 0
    assert sc[2, 1] == 127 + 99 - 8
    # -63 .. -32: amax 63 -> 32 / 256 = 2^-3; -31 .. 0: 16 / 256 = 2^-4
    assert sc[3, 1] == 127 - 3 and sc[3, 0] == 127 - 4
    # 2^3 * 63 = 504 lies beyond the e4m3 range: saturated, not NaN
    assert np.array_equal(val[3, 32:], dtp.e4m3_to_f32(dtp.f32_to_e4m3(np.clip(d[3, 32:] * 8, -448, 448))))


@pytest.mark.parametrize("dst", ["f8_e4m3", "f8_e5m2"])
def test_oracle_follows_the_numpy_restatement(dst):
    dst_dt = cabi.DT_F8_E4M3 if dst == "f8_e4m3" else cabi.DT_F8_E5M2
    p = configs.config4(M=48, N=128, K=64)
    p.post_ops = [PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"], alpha=0.25, scale=3.0), p.post_ops[1]]
    # pre-quantization values: the static path with an f32 dst
    p.dst_dt = cabi.DT_F32
    pre = np.asarray(orc.run_oracle(p)).view(np.float32).reshape(p.M, p.N)
    p.dst_dt = dst_dt
    got, sc = orc.run_oracle_dynamic(dynamic(p))
    want, want_sc = numpy_dynamic(pre, dst_dt)
    assert np.array_equal(sc.reshape(p.M, p.N // 32), want_sc)
    assert np.array_equal(np.asarray(got).view(np.uint8).reshape(p.M, p.N), want)


def test_rules_of_the_descriptor():
    p = dynamic(configs.config4(M=32, N=64, K=64))
    p.dst_dt = cabi.DT_F8_E4M3
    # the generic kernel and the floating-point GEMM tiles
    assert cabi.query(p.desc(), cabi.IMPL_REF)[0] == cabi.SUCCESS
    big = dynamic(configs.config4(M=32, N=64, K=256))
    big.dst_dt = cabi.DT_F8_E4M3
    st, impl = cabi.query(big.desc())
    assert st == cabi.SUCCESS and cabi.impl_name(impl).startswith("hip:mfma_f8")
    for change in ("dt", "group", "mask", "dst", "n"):
        q = dynamic(configs.config4(M=32, N=64 if change != "n" else 80, K=64))
        q.dst_dt = cabi.DT_F8_E4M3 if change != "dst" else cabi.DT_BF16
        s = q.quant["dst_scale"]
        if change == "dt":
            s.dt = cabi.DT_F32
        if change == "group":
            s.groups = (1, 16)
        if change == "mask":
            s.mask = configs.MASK_COL
        assert cabi.query(q.desc())[0] == cabi.INVALID_ARGUMENTS, change
    # integer src: the reference's integer implementation has no dynamic quantization
    c = dynamic(configs.config1(M=32, N=64, K=64))
    c.dst_dt = cabi.DT_F8_E4M3
    assert cabi.query(c.desc())[0] == cabi.UNIMPLEMENTED


# ------------------------------------------------------------------ GPU
def run_gpu_dynamic(p, impl=None):
    run = GpuRun(p, impl)
    try:
        run.launch()
        return run.result(), run.dynamic_scales(), cabi.impl_name(run.impl)
    finally:
        run.free()


@pytest.mark.gpu
def test_gpu_known_answer_groups(gpu, oracle):
    r = np.random.default_rng(3)
    d = (r.standard_normal((16, 128)) * np.exp2(r.integers(-140, 120, size=(16, 4)).repeat(32, axis=1))).astype(np.float32)
    d[0, :32] = 0.0
    d[1, :32] = np.float32(1.9999999)
    for dst_dt in (cabi.DT_F8_E4M3, cabi.DT_F8_E5M2):
        p = f32_problem(d, dst_dt)
        got, sc, name = run_gpu_dynamic(p, cabi.IMPL_REF)
        want, want_sc = orc.run_oracle_dynamic(p)
        assert name == "hip:ref:any"
        assert np.array_equal(np.asarray(sc).reshape(-1), np.asarray(want_sc).reshape(-1))
        assert np.array_equal(np.asarray(got).view(np.uint8), np.asarray(want).view(np.uint8))


@pytest.mark.gpu
@pytest.mark.parametrize("dst", ["f8_e4m3", "f8_e5m2"])
def test_gpu_fp8_matmul_with_dynamic_dst_is_bit_exact(gpu, oracle, dst):
    # bias, leaky relu and a residual add before the quantization: no libm
    # function involved, so the generic kernel must match the oracle bit for bit
    p = configs.config4(M=80, N=192, K=128)
    p.post_ops = [PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"], alpha=0.25, scale=3.0), p.post_ops[1]]
    p.dst_dt = cabi.DT_F8_E4M3 if dst == "f8_e4m3" else cabi.DT_F8_E5M2
    p = dynamic(p)
    got, sc, name = run_gpu_dynamic(p, cabi.IMPL_REF)
    want, want_sc = orc.run_oracle_dynamic(p)
    assert name == "hip:ref:any"
    assert np.array_equal(np.asarray(sc).reshape(-1), np.asarray(want_sc).reshape(-1))
    assert np.array_equal(np.asarray(got).view(np.uint8), np.asarray(want).view(np.uint8))


@pytest.mark.gpu
@pytest.mark.parametrize("family", ["f8", "mxf4"])
def test_gpu_gemm_tiles_quantize_dst_dynamically(gpu, oracle, family):
    # The MFMA GEMM families round the K sum differently from the reference, so
    # a group's largest magnitude can fall on the other side of a power of two
    # and its scale differ by one step.  Checked instead: scale bytes within one
    # step of the oracle's (and equal nearly everywhere), and the dequantized
    # dst within the quantization error of the type at that scale.  Partial
    # tiles in both directions (M = 300, N = 320).
    if family == "f8":
        p = configs.config4(M=300, N=320, K=256)
        prefix = "hip:mfma_f8"
    else:
        p = configs.config5(M=300, N=320, K=256)
        prefix = "hip:mfma_mxf4"
    p.dst_dt = cabi.DT_F32
    pre = np.asarray(orc.run_oracle(p)).view(np.float32).reshape(p.M, p.N).astype(np.float64)
    p.dst_dt = cabi.DT_F8_E4M3
    p = dynamic(p)
    got, sc, name = run_gpu_dynamic(p)
    assert name.startswith(prefix)
    _, want_sc = orc.run_oracle_dynamic(p)
    sc = np.asarray(sc).reshape(p.M, p.N // 32).astype(np.int32)
    want_sc = np.asarray(want_sc).reshape(p.M, p.N // 32).astype(np.int32)
    assert np.all(np.abs(sc - want_sc) <= 1)
    assert np.mean(sc == want_sc) > 0.97
    deq = dtp.e4m3_to_f32(np.asarray(got).view(np.uint8).reshape(-1)).reshape(p.M, p.N).astype(np.float64)
    deq = deq * np.exp2(sc - 127.0).repeat(32, axis=1)
    amax = np.abs(pre).reshape(p.M, p.N // 32, 32).max(axis=2).repeat(32, axis=1)
    # e4m3 keeps 3 mantissa bits (half an ulp = 2^-4 of the value), the largest
    # values of a group saturate at 448 of at most 512 (12.5 %), subnormal steps
    # are 2^-9 of the scaled range
    tol = 0.14 * np.abs(pre) + amax * 2.0 ** -8 + 1e-6
    assert np.all(np.abs(deq - pre) <= tol), float(np.max(np.abs(deq - pre) / tol))


# ---- quantization_mode::dynamic_fp (NVFP4 flavour): f8_e4m3 scales per 16
# columns, f4_e2m1 or fp8 dst (ref_matmul.cpp:352-365, matmul.cpp:423-440)
E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], np.float64)
FP_MAX = {cabi.DT_F4_E2M1: 6.0, cabi.DT_F8_E4M3: 448.0, cabi.DT_F8_E5M2: 57344.0}


def dynamic_fp(p):
    p.quant["dst_scale"] = QuantParam(cabi.DT_F8_E4M3, configs.MASK_ROW | configs.MASK_COL,
                                      np.zeros((p.batch, p.M, p.N // 16), np.uint8), (1, 16))
    p.dst_dynamic = cabi.DST_DYNAMIC_FP
    return p


def nearest_even(x, grid):
    """Index of the value of the ascending `grid` nearest to each x >= 0; ties go to the even index
    (codes of e4m3 / e2m1 ascend with the value, and an even code has an even mantissa)."""
    x = np.asarray(x, np.float64)
    hi = np.clip(np.searchsorted(grid, x, side="left"), 1, len(grid) - 1)
    lo = hi - 1
    dl, dh = x - grid[lo], grid[hi] - x
    return np.where(dl < dh, lo, np.where(dh < dl, hi, np.where(lo % 2 == 0, lo, hi)))


def search_dynamic_fp(d, dst_dt):
    """The reference's steps, with every conversion done as a search for the nearest representable value."""
    rows, N = d.shape
    g = d.reshape(rows, N // 16, 16)
    amax = np.abs(g).max(axis=2)
    r = (amax / np.float32(FP_MAX[dst_dt])).astype(np.float32)
    r = np.maximum(np.minimum(r, np.float32(448.0)), np.float32(0.125))
    e4m3_pos = dtp.e4m3_to_f32(np.arange(0x7f, dtype=np.uint8)).astype(np.float64)     # codes 0 .. 0x7e, ascending
    # f32 -> e4m3 goes through f16 in the reference (float8.cpp:269-274): two roundings, the first one numpy's
    sbyte = nearest_even(r.astype(np.float16).astype(np.float64), e4m3_pos).astype(np.uint8)
    inv = (np.float32(1.0) / e4m3_pos[sbyte].astype(np.float32)).astype(np.float32)
    x = np.clip(g * inv[:, :, None], -FP_MAX[dst_dt], FP_MAX[dst_dt]).astype(np.float32).reshape(rows, N)
    if dst_dt == cabi.DT_F4_E2M1:
        codes = nearest_even(np.abs(x), E2M1).astype(np.uint8) | (np.signbit(x).astype(np.uint8) << 3)
    else:
        codes = nearest_even(np.abs(x).astype(np.float16).astype(np.float64), e4m3_pos).astype(np.uint8) \
            | (np.signbit(x).astype(np.uint8) << 7)
    return codes, sbyte


def unpack_dst(raw, dst_dt, M, N):
    raw = np.asarray(raw).view(np.uint8).reshape(-1)
    if dst_dt in (cabi.DT_F4_E2M1, cabi.DT_S4, cabi.DT_U4):
        return np.stack([raw & 0xf, raw >> 4], axis=1).reshape(M, N)
    return raw.reshape(M, N)


def test_dynamic_fp_known_answers():
    d = np.zeros((3, 32), np.float32)
    d[0, :16] = np.linspace(-6, 6, 16)                # amax 6 -> scale 1
    d[0, 16:] = 0.0                                   # zero group: the scale is clamped to 2^-3 from below
    d[1, :16] = 6 * 448 * 4                           # beyond the scale range: 448, and the values saturate at 6
    d[1, 16:] = 6 * 1.0625                            # 1.0625 lies halfway between the e4m3 values 1 and 1.125: even -> 1
    d[2, :16] = 6 * 1.1875                            # halfway between 1.125 (odd code) and 1.25 (even code) -> 1.25
    d[2, 16:] = [3.0, -1.5, 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.25, -5.0, 0.0, 6.0, -6.0, 0.1, 0.3]
    p = dynamic_fp(f32_problem_plain(d, cabi.DT_F4_E2M1))
    dst, sc = orc.run_oracle_dynamic(p)
    sc = dtp.e4m3_to_f32(np.asarray(sc).reshape(3, 2))
    codes = unpack_dst(dst, cabi.DT_F4_E2M1, 3, 32)
    val = E2M1[codes & 7] * np.where(codes & 8, -1.0, 1.0)
    assert sc[0, 0] == 1.0 and sc[0, 1] == 0.125 and np.all(val[0, 16:] == 0)
    assert sc[1, 0] == 448.0 and np.all(val[1, :16] == 6.0)
    assert sc[1, 1] == 1.0 and np.all(val[1, 16:] == 6.0)
    assert sc[2, 0] == 1.25
    # scale 1: halfway values go to the even code (0.25 -> 0, 0.75 -> 1, 1.25 -> 1, 1.75 -> 2, 2.5 -> 2, 3.5 -> 4, 5 -> 4)
    assert sc[2, 1] == 1.0
    assert np.array_equal(val[2, 16:], [3.0, -1.5, 0.0, 1.0, 1.0, 2.0, 2.0, 4.0, 4.0, -0.0, -4.0, 0.0, 6.0, -6.0, 0.0, 0.5])


def f32_problem_plain(d, dst_dt):
    M, N = d.shape
    return MatmulProblem(M=M, N=N, K=M, src_dt=cabi.DT_F32, wei_dt=cabi.DT_F32, dst_dt=dst_dt,
                         src=np.eye(M, dtype=np.float32), wei=np.ascontiguousarray(d, dtype=np.float32), name="dyn-fp")


@pytest.mark.parametrize("dst", ["f4_e2m1", "f8_e4m3"])
def test_dynamic_fp_oracle_follows_the_search_restatement(dst):
    dst_dt = cabi.DT_F4_E2M1 if dst == "f4_e2m1" else cabi.DT_F8_E4M3
    p = configs.config4(M=48, N=128, K=64)
    p.post_ops = [PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"], alpha=0.25, scale=3.0), p.post_ops[1]]
    p.dst_dt = cabi.DT_F32
    pre = np.asarray(orc.run_oracle(p)).view(np.float32).reshape(p.M, p.N)
    p.dst_dt = dst_dt
    got, sc = orc.run_oracle_dynamic(dynamic_fp(p))
    want, want_sc = search_dynamic_fp(pre, dst_dt)
    assert np.array_equal(np.asarray(sc).reshape(p.M, p.N // 16), want_sc)
    got = unpack_dst(got, dst_dt, p.M, p.N)
    # -0 and +0 are one value for the search
    zero = (want & (7 if dst_dt == cabi.DT_F4_E2M1 else 0x7f)) == 0
    assert np.array_equal(np.where(zero, got & (7 if dst_dt == cabi.DT_F4_E2M1 else 0x7f), got), np.where(zero, 0, want))


def test_dynamic_fp_rules_of_the_descriptor():
    p = dynamic_fp(configs.config4(M=32, N=64, K=256))
    p.dst_dt = cabi.DT_F4_E2M1
    st, impl = cabi.query(p.desc())
    assert st == cabi.SUCCESS and cabi.impl_name(impl).startswith("hip:mfma_f8")   # the GEMM tiles take it
    assert cabi.query(p.desc(), cabi.IMPL_REF)[0] == cabi.SUCCESS
    assert cabi.query(p.desc(), cabi.IMPL_H16_MFMA)[0] == cabi.UNIMPLEMENTED
    q = dynamic_fp(configs.config4(M=32, N=64, K=256))
    q.dst_dt = cabi.DT_F4_E2M1
    q.quant["dst_scale"].groups = (1, 32)
    assert cabi.query(q.desc())[0] == cabi.INVALID_ARGUMENTS
    q = dynamic_fp(configs.config4(M=32, N=64, K=256))
    q.dst_dt = cabi.DT_F4_E2M1
    q.quant["dst_scale"].dt = cabi.DT_E8M0
    assert cabi.query(q.desc())[0] == cabi.INVALID_ARGUMENTS
    # a 4-bit dst with a static scale: the tiles where groups of four columns are whole bytes, else the generic
    # kernel (whole bytes per row)
    s = configs.config4(M=32, N=64, K=256)
    s.dst_dt = cabi.DT_F4_E2M1
    st, impl = cabi.query(s.desc())
    assert st == cabi.SUCCESS and cabi.impl_name(impl).startswith("hip:mfma_f8")
    s = configs.config4(M=32, N=62, K=256)
    s.post_ops = []
    s.dst_dt = cabi.DT_F4_E2M1
    st, impl = cabi.query(s.desc())
    assert st == cabi.SUCCESS and cabi.impl_name(impl) == "hip:ref:any"
    s = configs.config4(M=32, N=63, K=256)
    s.post_ops = []
    s.dst_dt = cabi.DT_F4_E2M1
    assert cabi.query(s.desc())[0] == cabi.UNIMPLEMENTED
    # MX scales over a 4-bit dst (an MXFP4 output)
    m = dynamic(configs.config4(M=32, N=64, K=256))
    m.dst_dt = cabi.DT_F4_E2M1
    st, impl = cabi.query(m.desc())
    assert st == cabi.SUCCESS and cabi.impl_name(impl).startswith("hip:mfma_f8")


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["fp", "mx"])
@pytest.mark.parametrize("dst", ["f4_e2m1", "f8_e4m3", "f8_e5m2"])
def test_gpu_dynamic_fp_and_4bit_dst_are_bit_exact(gpu, oracle, dst, mode):
    if mode == "mx" and dst != "f4_e2m1":
        pytest.skip("covered above")
    dst_dt = {"f4_e2m1": cabi.DT_F4_E2M1, "f8_e4m3": cabi.DT_F8_E4M3, "f8_e5m2": cabi.DT_F8_E5M2}[dst]
    make = dynamic_fp if mode == "fp" else dynamic
    # constructed groups over many binades, zero groups, huge groups
    r = np.random.default_rng(5)
    d = (r.standard_normal((16, 128)) * np.exp2(r.integers(-20, 24, size=(16, 8)).repeat(16, axis=1))).astype(np.float32)
    d[0, :32] = 0.0
    d[1, :16] = 1e30
    p = make(f32_problem_plain(d, dst_dt))
    got, sc, name = run_gpu_dynamic(p, cabi.IMPL_REF)
    want, want_sc = orc.run_oracle_dynamic(p)
    assert name == "hip:ref:any"
    assert np.array_equal(np.asarray(sc).reshape(-1), np.asarray(want_sc).reshape(-1))
    assert np.array_equal(np.asarray(got).view(np.uint8), np.asarray(want).view(np.uint8))
    # a matmul with bias, leaky relu and a residual add before the quantization
    p = configs.config4(M=80, N=192, K=128)
    p.post_ops = [PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"], alpha=0.25, scale=3.0), p.post_ops[1]]
    p.dst_dt = dst_dt
    p = make(p)
    got, sc, name = run_gpu_dynamic(p, cabi.IMPL_REF)
    want, want_sc = orc.run_oracle_dynamic(p)
    assert name == "hip:ref:any"
    assert np.array_equal(np.asarray(sc).reshape(-1), np.asarray(want_sc).reshape(-1))
    assert np.array_equal(np.asarray(got).view(np.uint8), np.asarray(want).view(np.uint8))


def decode_dst(raw, dst_dt, M, N):
    codes = unpack_dst(raw, dst_dt, M, N)
    if dst_dt == cabi.DT_F4_E2M1:
        return np.where(codes & 8, -1.0, 1.0) * E2M1[codes & 7]
    if dst_dt == cabi.DT_S4:
        return ((codes.astype(np.int32) ^ 8) - 8).astype(np.float64)
    if dst_dt == cabi.DT_U4:
        return codes.astype(np.float64)
    f = dtp.e4m3_to_f32 if dst_dt == cabi.DT_F8_E4M3 else dtp.e5m2_to_f32
    return f(codes.reshape(-1)).reshape(M, N).astype(np.float64)


FAMILY = {"f8": (lambda **kw: configs.config4(**kw), "hip:mfma_f8"), "mxf4": (lambda **kw: configs.config5(**kw), "hip:mfma_mxf4"),
          "h16": (lambda **kw: configs.config_h16(dt="bf16", **kw), "hip:mfma_h16")}


@pytest.mark.gpu
@pytest.mark.parametrize("family", ["f8", "mxf4", "h16"])
@pytest.mark.parametrize("mode,dst", [("fp", "f4_e2m1"), ("fp", "f8_e4m3"), ("mx", "f4_e2m1"), ("mx", "f8_e4m3")])
def test_gpu_gemm_tiles_quantize_dst_in_groups_of_16_and_to_4_bits(gpu, oracle, family, mode, dst):
    """The NVFP4 flavour (f8_e4m3 scale per 16 columns) and 4-bit dst in the tiles' epilogue.  The tiles round the K
    sum differently from the reference, so scales and codes are checked through what they mean: a scale within one
    code of the oracle's (and equal nearly everywhere), and every element, times the scale the kernel wrote, within
    the spacing of the dst type around the f32 result.  Partial tiles in both directions."""
    dst_dt = {"f4_e2m1": cabi.DT_F4_E2M1, "f8_e4m3": cabi.DT_F8_E4M3}[dst]
    G = 16 if mode == "fp" else 32
    p = FAMILY[family][0](M=300, N=320, K=256)
    p.dst_dt = cabi.DT_F32
    pre = np.asarray(orc.run_oracle(p)).view(np.float32).reshape(p.M, p.N).astype(np.float64)
    p.dst_dt = dst_dt
    p = (dynamic_fp if mode == "fp" else dynamic)(p)
    got, sc, name = run_gpu_dynamic(p)
    assert name.startswith(FAMILY[family][1])
    _, want_sc = orc.run_oracle_dynamic(p)
    sc = np.asarray(sc).reshape(p.M, p.N // G).astype(np.int32)
    want_sc = np.asarray(want_sc).reshape(p.M, p.N // G).astype(np.int32)
    assert np.all(np.abs(sc - want_sc) <= 1)
    assert np.mean(sc == want_sc) > 0.97
    scale = (dtp.e4m3_to_f32(sc.astype(np.uint8).reshape(-1)).reshape(sc.shape).astype(np.float64) if mode == "fp"
             else np.exp2(sc - 127.0)).repeat(G, axis=1)
    x = np.clip(pre / scale, -FP_MAX[dst_dt], FP_MAX[dst_dt])
    q = decode_dst(got, dst_dt, p.M, p.N)
    # half the distance between neighbours of the dst type at |x| (e2m1: 0.25 up to 2, 0.5 up to 4, 1 up to 6; e4m3:
    # 2^-4 |x|, 2^-10 among the subnormals) + the tiles' own rounding of the sum, which may move x across a tie
    half = np.maximum(0.25, 0.25 * np.abs(x)) if dst_dt == cabi.DT_F4_E2M1 else np.abs(x) / 16 + 2.0 ** -10
    amax = np.abs(pre).reshape(p.M, p.N // G, G).max(axis=2).repeat(G, axis=1)
    tol = half + 2e-3 * amax / scale + 1e-6
    assert np.all(np.abs(q - x) <= tol), float(np.max(np.abs(q - x) / tol))
    assert len(np.unique(q)) >= (10 if dst_dt == cabi.DT_F4_E2M1 else 40)      # not a degenerate result


@pytest.mark.gpu
@pytest.mark.parametrize("family", ["f8", "mxf4", "h16"])
@pytest.mark.parametrize("dst", ["f4_e2m1", "s4", "u4"])
def test_gpu_gemm_tiles_store_a_4bit_dst_with_a_static_scale(gpu, oracle, family, dst):
    """Codes against the oracle's: equal nearly everywhere, never more than one step of the type apart (the tiles
    round the K sum differently).  Bias / post-ops as the configuration has them, a static dst scale."""
    dst_dt = {"f4_e2m1": cabi.DT_F4_E2M1, "s4": cabi.DT_S4, "u4": cabi.DT_U4}[dst]
    p = FAMILY[family][0](M=300, N=320, K=256)
    p.dst_dt = cabi.DT_F32
    pre = np.abs(np.asarray(orc.run_oracle(p)).view(np.float32).astype(np.float64))
    p.dst_dt = dst_dt
    p.quant["dst_scale"] = QuantParam(cabi.DT_F32, 0, np.array([np.percentile(pre, 90) / 5.0], np.float32))
    run = GpuRun(p, None)
    try:
        run.launch()
        got, name = run.result(), cabi.impl_name(run.impl)
    finally:
        run.free()
    assert name.startswith(FAMILY[family][1])
    want = orc.run_oracle(p)
    g, w = decode_dst(got, dst_dt, p.M, p.N), decode_dst(want, dst_dt, p.M, p.N)
    step = np.maximum(0.5, 0.5 * np.maximum(np.abs(g), np.abs(w))) if dst_dt == cabi.DT_F4_E2M1 else 1.0
    assert np.all(np.abs(g - w) <= step)
    assert np.mean(g == w) > 0.97
    assert len(np.unique(w)) >= 8


@pytest.mark.gpu
@pytest.mark.parametrize("dst", ["f4_e2m1", "s4", "u4"])
def test_gpu_4bit_dst_with_a_static_scale_is_bit_exact(gpu, oracle, dst):
    # two columns per byte, low nibble first; bias, leaky relu, residual add, then a static dst scale (and the old dst
    # through a sum post-op for f4): no libm function involved, the generic kernel matches the oracle bit for bit
    p = configs.config4(M=80, N=192, K=128)
    p.post_ops = [PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE["relu"], alpha=0.25, scale=3.0), p.post_ops[1]]
    if dst == "f4_e2m1":
        p.post_ops.append(PostOp(kind=cabi.PO_SUM, scale=0.5))
        p.dst_init = np.random.default_rng(9).integers(0, 256, size=p.M * p.N // 2).astype(np.uint8)
    p.dst_dt = {"f4_e2m1": cabi.DT_F4_E2M1, "s4": cabi.DT_S4, "u4": cabi.DT_U4}[dst]
    p.quant["dst_scale"] = QuantParam(cabi.DT_F32, 0, np.array([0.37], np.float32))
    run = GpuRun(p, cabi.IMPL_REF)
    try:
        run.launch()
        got, name = run.result(), cabi.impl_name(run.impl)
    finally:
        run.free()
    want = orc.run_oracle(p)
    assert name == "hip:ref:any"
    g, w = np.asarray(got).view(np.uint8), np.asarray(want).view(np.uint8)
    assert np.array_equal(g, w)
    assert len(np.unique(np.concatenate([w & 0xf, w >> 4]))) >= 8        # not a degenerate result


@pytest.mark.gpu
def test_gpu_the_tiles_convert_to_f4_like_the_reference(gpu, oracle):
    """dst = I x W in f32, so every dst code is the conversion of a chosen f32 value: every midpoint between two
    e2m1 values and its f32 neighbours (ties go to the even code), both signs, zero, subnormals, values beyond 6,
    infinities, and random values over many binades -- the tiles (hardware conversion) against the oracle's
    software conversion (float4 of the reference), code for code.  A NaN anywhere sends a wavefront to the software
    path; one column block holds NaNs to cover that too."""
    M = N = K = 256
    r = np.random.default_rng(3)
    mids = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0], np.float32)
    near = np.concatenate([mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(10))])
    special = np.array([0.0, 1e-45, 1e-38, 5.9999995, 6.0000005, 7.0, 448.0, 1e30, np.inf], np.float32)
    vals = np.concatenate([near, special])
    vals = np.concatenate([vals, -vals])
    W = (r.standard_normal((K, N)) * np.exp2(r.integers(-4, 4, size=(K, N)))).astype(np.float32)
    W.reshape(-1)[:vals.size] = vals
    W[:, 192:200] = r.choice([np.nan, 1.0, -2.5, 6.5], size=(K, 8)).astype(np.float32)
    p = MatmulProblem(M=M, N=N, K=K, src_dt=cabi.DT_F32, wei_dt=cabi.DT_F32, dst_dt=cabi.DT_F4_E2M1,
                      src=np.eye(M, dtype=np.float32), wei=W, name="f4-conversion")
    run = GpuRun(p, None)
    try:
        run.launch()
        got, name = run.result(), cabi.impl_name(run.impl)
    finally:
        run.free()
    assert name.startswith("hip:mfma_h16")
    want = orc.run_oracle(p)
    g, w = unpack_dst(got, cabi.DT_F4_E2M1, M, N), unpack_dst(want, cabi.DT_F4_E2M1, M, N)
    nan = np.isnan(W)
    # 0 x NaN spoils the whole column of a NaN; elsewhere the codes are the conversions of W (the sign of a zero aside)
    clean = ~nan.any(axis=0)
    same = (g == w) | ((g & 7) == 0) & ((w & 7) == 0)
    assert np.all(same[:, clean]), np.argwhere(~same[:, clean])[:5]
    assert np.all((g[:, ~clean] & 7) == (w[:, ~clean] & 7))
