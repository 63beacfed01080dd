"""Dropout and stochastic rounding of ref_matmul_t (src/cpu/matmul/ref_matmul.cpp:61-67,
283-331; ref_dropout src/cpu/primitive_attr_postops.cpp:296-310; stochastic_round_fwd
and the Philox generator src/common/math_utils.hpp:458-574).

The reference holds no known-answer vectors for them (benchdnn checks dropout
statistically), so the oracle's restatement is pinned from outside:
  * the Philox4x32-10 core against the known-answer vectors of the generator's
    authors (Random123, kat_vectors: zero, all-ones and pi-digits inputs) and
    against an independent implementation written here from the paper's round
    function with Python integers;
  * how idx / seed / offset become counter and key (math_utils.hpp:468-471,
    508-515) by what that construction implies: the four indices of a block
    are the four words of one output block, the 32-bit flavour does not depend
    on idx % 4, offset and seed reach the words they should;
  * dropout by its decision rule on values of p where it is decidable by hand
    (0, 1, a probability that is a power of two against the top bit of the random
    word), the 1 / (1 - p) scaling, and keep statistics;
  * stochastic rounding by what it must produce: a value of the dst type, one
    of the two neighbours of the input, the lower one when the low bits are
    zero, saturation / flush at the type's limits, and the carry probability
    its 8 (two-byte types) or 16 (one-byte types) random bits give.
GPU: the generic kernel against the oracle, bit for bit, values and masks."""
import ctypes as C
import os

import numpy as np
import pytest

os.environ.setdefault("ONEDNN_AMD_ALLOW_NO_DEVICE", "1")
from onednn_amd import cabi, dnnl  # noqa: E402
from onednn_amd import dtypes as dtp  # noqa: E402
from onednn_amd.problem import MatmulProblem, PostOp, decode  # noqa: E402

F32, BF16, F16, E4M3, E5M2 = cabi.DT_F32, cabi.DT_BF16, cabi.DT_F16, cabi.DT_F8_E4M3, cabi.DT_F8_E5M2
M32 = 0xffffffff


# ------------------------------------------------------------------ Philox
def philox_py(ctr, key):
    """Philox4x32-10 from the definition (Salmon, Moraes, Dror, Shaw, SC'11, section 3.3): ten
    rounds of two 32x32 -> 64 multiplications, key bumped by the Weyl constants between rounds."""
    c, k = list(ctr), list(key)
    for r in range(10):
        if r:
            k = [(k[0] + 0x9E3779B9) & M32, (k[1] + 0xBB67AE85) & M32]
        p0, p1 = 0xD2511F53 * c[0], 0xCD9E8D57 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & M32, (p0 >> 32) ^ c[3] ^ k[1], p0 & M32]
    return c


KAT = [  # Random123 kat_vectors, philox4x32 10 rounds: counter, key, expected
    ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((M32,) * 4, (M32,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
     (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


@pytest.mark.parametrize("ctr,key,want", KAT, ids=["zeros", "ones", "pi"])
def test_philox_known_answers(oracle, ctr, key, want):
    assert tuple(oracle.philox_block(ctr, key)) == want
    assert tuple(philox_py(ctr, key)) == want


def test_philox_block_against_the_independent_implementation(oracle):
    rng = np.random.default_rng(3)
    for _ in range(200):
        ctr = [int(x) for x in rng.integers(0, 2 ** 32, 4)]
        key = [int(x) for x in rng.integers(0, 2 ** 32, 2)]
        assert oracle.philox_block(ctr, key) == philox_py(ctr, key)


def test_counter_and_key_construction(oracle):
    """idx / 4 selects the block (counter words 2, 3), idx % 4 the word; the offset fills counter words 0, 1,
    the seed the key."""
    rng = np.random.default_rng(4)
    for _ in range(50):
        idx, seed, off = (int(x) for x in rng.integers(0, 2 ** 63, 3))
        base = idx & ~3
        block = philox_py((off & M32, off >> 32, base & M32, base >> 32), (seed & M32, seed >> 32))
        assert [oracle.philox(base + w, seed, off) for w in range(4)] == block
    # the 32-bit flavour packs (x, x + 1) into the offset and (x + 2, x + 3) into the index of the 64-bit one with
    # x = idx & ~3, the seed twice into the key: the 64-bit function then clears the two low bits of its index
    # (x + 2 -> x) and returns word (x + 2) % 4 = 2, so the counter is (x, x + 1, x, x + 3) and the value does
    # not depend on idx % 4
    for idx, seed in [(0, 0), (5, 77), (1023, 2 ** 31 + 5), (2 ** 32 - 1, 2 ** 32 - 1)]:
        x = idx & ~3
        want = philox_py((x, x + 1, x, x + 3), (seed, seed))[2]
        for w in range(4):
            assert oracle.philox_u32(x + w, seed) == want


# ------------------------------------------------------------------ dropout
def test_dropout_rule(oracle):
    for idx in range(64):
        assert oracle.dropout(3.5, idx, 0.0, 11, 0) == (3.5, 1) or oracle.philox_u32(idx, 11) == 0
        assert oracle.dropout(3.5, idx, 1.0, 11, 0) == (0.0, 0)              # never kept, 1 / (1 - p) not formed
        # p = 1/2: kept iff the random word exceeds (2^32 - 1) / 2, i.e. iff its top bit is set
        v, keep = oracle.dropout(3.0, idx, 0.5, 11, 0)
        assert keep == oracle.philox_u32(idx, 11) >> 31 and v == (6.0 if keep else 0.0)
        # a non-zero offset switches to the 64-bit generator
        v, keep = oracle.dropout(3.0, idx, 0.5, 11, 9)
        assert keep == oracle.philox(idx, 11, 9) >> 31 and v == (6.0 if keep else 0.0)
        # p outside [0, 1] is clamped for the decision after 1 / (1 - p) was formed from the given value
        v, keep = oracle.dropout(2.0, idx, -1.0, 11, 9)
        assert keep == (oracle.philox(idx, 11, 9) > 0) and (not keep or v == 1.0)
    # scaling by 1 / (1 - p) in float32
    v, keep = next((oracle.dropout(1.0, i, 0.3, 5, 1)) for i in range(100) if oracle.dropout(1.0, i, 0.3, 5, 1)[1])
    assert np.float32(v) == np.float32(1.0) * (np.float32(1.0) / (np.float32(1.0) - np.float32(0.3)))


@pytest.mark.parametrize("p", [0.1, 0.5, 0.8])
def test_dropout_keeps_about_one_minus_p(oracle, p):
    n = 20000
    kept = sum(oracle.dropout(1.0, i, p, 2024, 1)[1] for i in range(n))   # 64-bit flavour: independent per element
    sigma = np.sqrt(n * p * (1 - p))
    assert abs(kept - n * (1 - p)) < 5 * sigma


# ------------------------------------------------------- stochastic rounding
LIMITS = {BF16: (8, float.fromhex("0x1.fep127"), 2.0 ** -126), F16: (11, 65504.0, 2.0 ** -14),
          E5M2: (3, 57344.0, 2.0 ** -14), E4M3: (4, 448.0, 2.0 ** -6), F32: (24, float(np.finfo(np.float32).max), 2.0 ** -126)}


def bits(x):
    return int(np.float32(x).view(np.uint32))


@pytest.mark.parametrize("dt", [BF16, F16, E5M2, E4M3, F32], ids=["bf16", "f16", "e5m2", "e4m3", "f32"])
def test_stochastic_rounding_properties(oracle, dt):
    digits, hi, tiny = LIMITS[dt]
    drop = 24 - digits                                  # bits below the dst type's precision
    rng = np.random.default_rng(dt)
    xs = (rng.standard_normal(400) * np.exp(rng.uniform(-3, 3, 400))).astype(np.float32)
    for i, x in enumerate(xs):
        if not (tiny * 2 < abs(x) < hi / 2):
            continue
        r = oracle.stochastic_round(float(x), i, 99, dt)
        assert bits(r) & ((1 << drop) - 1) == 0          # a value of the dst type's precision
        lo = bits(x) & ~((1 << drop) - 1) & M32           # truncation toward zero ...
        assert bits(r) in (lo, lo + (1 << drop))          # ... or the next value away from zero
        # already representable: unchanged whatever the random bits
        assert oracle.stochastic_round(float(np.uint32(lo).view(np.float32)), i, 99, dt) == np.uint32(lo).view(np.float32)
    assert oracle.stochastic_round(float("inf"), 0, 1, dt) == np.float32(hi)       # saturation at the type's limits
    assert oracle.stochastic_round(float("-inf"), 0, 1, dt) == np.float32(-hi)
    if dt != F32:
        assert oracle.stochastic_round(hi * 1.5, 0, 1, dt) == np.float32(hi)
    assert oracle.stochastic_round(tiny / 4, 0, 1, dt) == 0.0                      # below the smallest normal: flushed
    assert oracle.stochastic_round(-tiny / 4, 0, 1, dt) == 0.0
    assert np.isnan(oracle.stochastic_round(float("nan"), 0, 1, dt))


@pytest.mark.parametrize("dt,rbits", [(BF16, 8), (F16, 8), (E5M2, 16), (E4M3, 16)], ids=["bf16", "f16", "e5m2", "e4m3"])
def test_stochastic_rounding_carry_probability(oracle, dt, rbits):
    """Two-byte types add 8 random bits, one-byte types 16, to the low end of the discarded bits: an input whose
    discarded bits are 2^drop - 2^(rbits - 1) is rounded up with probability one half, one whose discarded bits
    are below 2^drop - 2^rbits never."""
    digits, _, _ = LIMITS[dt]
    drop = 24 - digits
    base = bits(1.5) & ~((1 << drop) - 1)
    half = np.uint32(base + (1 << drop) - (1 << (rbits - 1))).view(np.float32)
    never = np.uint32(base + (1 << drop) - (1 << rbits) - 1).view(np.float32)
    n = 4000
    ups = sum(bits(oracle.stochastic_round(float(half), i, 5, dt)) != base for i in range(n))
    assert abs(ups - n / 2) < 5 * np.sqrt(n / 4)
    assert all(bits(oracle.stochastic_round(float(never), i, 5, dt)) == base for i in range(500))


# ------------------------------------------------------------- matmul level
def problem(dst_dt=F32, dropout=None, stochastic=False, batch=1, bias=False, relu=False, seed=1, M=12, N=20, K=16,
            exact=True):
    rng = np.random.default_rng(seed)
    if exact:
        src = rng.integers(-4, 5, (batch, M, K)).astype(np.float32)
        wei = rng.integers(-4, 5, (batch, K, N)).astype(np.float32)
    else:
        src = rng.standard_normal((batch, M, K)).astype(np.float32)
        wei = rng.standard_normal((batch, K, N)).astype(np.float32)
    p = MatmulProblem(M=M, N=N, K=K, batch=batch, src_dt=F32, wei_dt=F32, dst_dt=dst_dt, src=src, wei=wei,
                      dropout=dropout, dst_stochastic=stochastic, name="dropout / rounding")
    if bias:
        p.bias_dt, p.bias = F32, rng.integers(-8, 9, N).astype(np.float32)
    if relu:
        p.post_ops = [PostOp(cabi.PO_ELTWISE, cabi.ELTWISE["relu"])]
    return p


def test_oracle_matmul_applies_dropout_after_the_bias_and_before_the_post_ops(oracle):
    p = problem(dropout={"p": 0.5, "seed": 7, "mask": True}, bias=True, relu=True, batch=2)
    dst, mask = oracle.run_oracle_dropout(p)
    acc = np.einsum("bmk,bkn->bmn", p.src.astype(np.float64), p.wei.astype(np.float64)) + p.bias
    idx = np.arange(acc.size)
    keep = np.array([oracle.philox_u32(int(i), 7) >> 31 for i in idx]).reshape(acc.shape)   # p = 1/2: the top bit
    want = np.maximum(np.where(keep, acc * 2.0, 0.0), 0.0)
    assert np.array_equal(mask.reshape(acc.shape), keep)
    assert np.array_equal(dst.reshape(acc.shape), want.astype(np.float32))


def test_oracle_matmul_rounds_dst_with_the_dropout_seed(oracle):
    """ref_matmul.cpp:322-331: the element's dst offset and the dropout seed (0 without dropout), both cut to 32 bits."""
    for drop, seed in ((None, 0), ({"p": 0.0, "seed": 2 ** 40 + 17, "seed_s64": True}, 17)):
        p = problem(dst_dt=BF16, dropout=drop, stochastic=True, exact=False)
        dst = oracle.run_oracle(p)
        q = problem(dst_dt=F32, exact=False)
        plain = oracle.run_oracle(q).reshape(-1)
        want = np.array([oracle.stochastic_round(float(v), i, seed, BF16) for i, v in enumerate(plain)], np.float32)
        assert np.array_equal(decode(BF16, dst, want.size), want)


def test_rules_of_the_thin_c_abi():
    p = problem(dropout={"p": 0.5, "seed": 1})
    assert cabi.query(p.desc(), cabi.IMPL_AUTO) == (cabi.SUCCESS, cabi.IMPL_REF)
    p.src_dt = p.wei_dt = cabi.DT_S8                                     # ref_matmul_t only: floating-point src
    p.src, p.wei = p.src.astype(np.int8), p.wei.astype(np.int8)
    assert cabi.query(p.desc(), cabi.IMPL_AUTO)[0] == cabi.UNIMPLEMENTED
    p = problem(dropout={"p": 0.5, "seed": 1})
    p.dst_stride = (0, 1, p.M)                                           # dst must be plain row-major
    assert cabi.query(p.desc(), cabi.IMPL_AUTO)[0] == cabi.UNIMPLEMENTED
    p = problem(dst_dt=cabi.DT_S8, stochastic=True)                      # rounding of floating-point dst types only
    assert cabi.query(p.desc(), cabi.IMPL_AUTO)[0] == cabi.UNIMPLEMENTED
    p = problem(dst_dt=BF16, stochastic=True)
    assert cabi.query(p.desc(), cabi.IMPL_F8_MFMA)[0] == cabi.UNIMPLEMENTED   # generic kernel only


def test_attribute_rules():
    """primitive_attr_t::set_dropout (primitive_attr.cpp:423-438), rnd_mode_t::check (primitive_attr.hpp:251-258)"""
    def status(fn):
        try:
            fn()
        except dnnl.error as e:
            return e.status
        return dnnl.success

    a = dnnl.primitive_attr()
    assert a.get_dropout() == (0, 0, 0, 0) and a.get_rounding(dnnl.ARG_DST) == dnnl.rounding_environment
    a.set_dropout()
    assert a.get_dropout() == (0, cabi.DT_S32, 0, 0)
    a.set_dropout(dnnl.memory_desc([4, 8], cabi.DT_U8, tag=dnnl.tag_ab), dnnl.s64, True, True)
    assert a.get_dropout() == (cabi.DT_U8, dnnl.s64, 1, 1)
    assert status(lambda: a.set_dropout(dnnl.memory_desc([4, 8], F32, tag=dnnl.tag_ab))) == dnnl.invalid_arguments
    assert status(lambda: a.set_dropout(None, F32)) == dnnl.invalid_arguments            # the seed is s32 or s64
    a.set_rounding(dnnl.ARG_DST, dnnl.rounding_stochastic)
    assert a.get_rounding(dnnl.ARG_DST) == dnnl.rounding_stochastic
    assert status(lambda: a.set_rounding(dnnl.ARG_SRC, dnnl.rounding_stochastic)) == dnnl.invalid_arguments
    a.set_rounding(dnnl.ARG_SRC, dnnl.rounding_environment)                               # the default is always fine
    eng = dnnl.engine(dnnl.gpu, 0)

    def make(attr, ddt=BF16, sdt=F32, mask_dims=None):
        return status(lambda: dnnl.matmul_primitive_desc(
            eng, dnnl.memory_desc([4, 16], sdt, tag=dnnl.tag_ab), dnnl.memory_desc([16, 8], sdt, tag=dnnl.tag_ab),
            dnnl.memory_desc([4, 8], ddt, tag=dnnl.tag_ab), attr=attr))

    a = dnnl.primitive_attr()
    a.set_dropout(dnnl.memory_desc([4, 8], cabi.DT_U8, tag=dnnl.tag_any))
    a.set_rounding(dnnl.ARG_DST, dnnl.rounding_stochastic)
    assert make(a) == dnnl.success
    assert make(a, sdt=cabi.DT_S8, ddt=F32) == dnnl.unimplemented                        # integer src
    b = dnnl.primitive_attr()
    b.set_dropout(dnnl.memory_desc([4, 9], cabi.DT_U8, tag=dnnl.tag_ab))                  # the mask is laid out like dst
    assert make(b) == dnnl.unimplemented
    b = dnnl.primitive_attr()
    b.set_dropout(dnnl.memory_desc([4, 8], cabi.DT_U8, tag=dnnl.tag_ba))
    assert make(b) == dnnl.unimplemented
    b = dnnl.primitive_attr()
    b.set_rounding(dnnl.ARG_DIFF_SRC, dnnl.rounding_stochastic)                           # no such tensor in a matmul
    assert make(b) == dnnl.unimplemented


# --------------------------------------------------------------------- GPU
CASES = [
    ("dropout, mask, s32 seed", dict(dropout={"p": 0.3, "seed": 42, "mask": True})),
    ("dropout, no mask, bias + relu", dict(dropout={"p": 0.7, "seed": -5}, bias=True, relu=True)),
    ("dropout, s64 seed and offset", dict(dropout={"p": 0.25, "seed": 2 ** 45 + 3, "seed_s64": True, "offset": 2 ** 33 + 1,
                                                    "mask": True}, batch=3)),
    ("dropout, offset given as zero", dict(dropout={"p": 0.5, "seed": 9, "offset": 0, "mask": True})),
    ("dropout p = 0 and p = 1", dict(dropout={"p": 0.0, "seed": 1, "mask": True})),
    ("stochastic bf16", dict(dst_dt=BF16, stochastic=True, exact=False)),
    ("stochastic f16 with a dropout seed", dict(dst_dt=F16, stochastic=True, exact=False,
                                                dropout={"p": 0.4, "seed": 123456789, "mask": True})),
    ("stochastic e4m3", dict(dst_dt=E4M3, stochastic=True, exact=False)),
    ("stochastic e5m2, batch", dict(dst_dt=E5M2, stochastic=True, exact=False, batch=2)),
    ("stochastic f32 (flushes subnormals, nothing else)", dict(dst_dt=F32, stochastic=True, exact=False)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("label,kw", CASES, ids=[c[0] for c in CASES])
def test_gpu_matches_the_oracle(gpu, oracle, label, kw):
    from onednn_amd.problem import GpuRun
    p = problem(**kw)
    want, want_mask = oracle.run_oracle_dropout(p)
    run = GpuRun(p)
    try:
        assert cabi.impl_name(run.impl) == "hip:ref:any"
        run.launch()
        got = run.result()
        assert np.array_equal(np.asarray(got).view(np.uint8), np.asarray(want).view(np.uint8)), label
        if want_mask is not None:
            assert np.array_equal(run.dropout_mask(), want_mask)
    finally:
        run.free()
    if label.startswith("dropout p = 0"):
        p1 = problem(dropout={"p": 1.0, "seed": 1, "mask": True})
        run = GpuRun(p1)
        try:
            run.launch()
            assert not run.result().any() and not run.dropout_mask().any()
        finally:
            run.free()


@pytest.mark.gpu
@pytest.mark.parametrize("host_scalars", [False, True], ids=["device scalars", "host scalars"])
def test_gpu_through_the_dnnl_api(gpu, oracle, host_scalars):
    p = problem(dst_dt=BF16, stochastic=True, exact=False, bias=True,
                dropout={"p": 0.35, "seed": 2 ** 40 + 11, "seed_s64": True, "offset": 77, "mask": True})
    want, want_mask = oracle.run_oracle_dropout(p)
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    smd = dnnl.memory_desc([p.M, p.K], F32, tag=dnnl.tag_ab)
    wmd = dnnl.memory_desc([p.K, p.N], F32, tag=dnnl.tag_ab)
    dmd = dnnl.memory_desc([p.M, p.N], BF16, tag=dnnl.tag_ab)
    bmd = dnnl.memory_desc([1, p.N], F32, tag=dnnl.tag_ab)
    mmd = dnnl.memory_desc([p.M, p.N], cabi.DT_U8, tag=dnnl.tag_any)
    attr = dnnl.primitive_attr()
    attr.set_dropout(mmd, dnnl.s64, True, host_scalars)
    attr.set_rounding(dnnl.ARG_DST, dnnl.rounding_stochastic)
    pd = dnnl.matmul_primitive_desc(eng, smd, wmd, dmd, bias_md=bmd, attr=attr)
    assert pd.impl_info_str() == "hip:ref:any"
    prim = dnnl.matmul(pd)
    dst = dnnl.memory(dmd, eng, p.initial_dst())
    mask = dnnl.memory(dnnl.memory_desc([p.M, p.N], cabi.DT_U8, tag=dnnl.tag_ab), eng, np.full(p.M * p.N, 0xee, np.uint8))
    one = lambda dt, v, npdt: (dnnl.host_scalar(dt, npdt(v)) if host_scalars  # noqa: E731
                               else dnnl.memory(dnnl.memory_desc([1], dt, tag=dnnl.tag_a), eng, np.asarray([v], npdt)))
    args = {dnnl.ARG_SRC: dnnl.memory(smd, eng, p.src), dnnl.ARG_WEIGHTS: dnnl.memory(wmd, eng, p.wei),
            dnnl.ARG_BIAS: dnnl.memory(bmd, eng, p.bias), dnnl.ARG_DST: dst,
            dnnl.ARG_ATTR_DROPOUT_MASK: mask,
            dnnl.ARG_ATTR_DROPOUT_PROBABILITY: one(F32, 0.35, np.float32),
            dnnl.ARG_ATTR_DROPOUT_SEED: one(dnnl.s64, 2 ** 40 + 11, np.int64),
            dnnl.ARG_ATTR_DROPOUT_OFFSET: one(dnnl.s64, 77, np.int64)}
    prim.execute(strm, args)
    strm.wait()
    assert np.array_equal(dst.read(np.uint16), want)
    assert np.array_equal(mask.read(np.uint8), want_mask)
