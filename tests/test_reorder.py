"""Reorder: the oracle pinned against numpy (CPU), the HIP kernels against the
oracle (GPU, bit-exact: every output type is produced by one conversion from
one f32 value computed with the same operations in the same order).

What pins the oracle's reorder (src/cpu/reorder/simple_reorder.hpp:2579-2661,
:2168-2425) without running the reference:
  * index arithmetic: numpy's own transpose / reshape on tensors whose values
    are all distinct (a wrong stride, a swapped dim or a wrong group index
    moves some value);
  * arithmetic: numpy float32 operations are IEEE correctly rounded one at a
    time like the reference's scalar code, so `src_scale * (src - zp)`,
    `/ dst_scale`, `+ dst_zp` are restated with numpy operators and rint/clip;
    tie vectors (x.5) check round-half-even, out-of-range values saturation;
  * 4-bit packing: the nibble order known-answer test of the reference
    (tests/gtests/internals/test_nibble.cpp:36-88) is restated in
    test_oracle_dtypes.py for pack_nibbles/unpack_nibbles, which are used here.
"""
import os

import numpy as np
import pytest

from onednn_amd import cabi
from onednn_amd import dtypes as dtp
from onednn_amd.problem import QuantParam, decode
from onednn_amd.reorder import ReorderProblem, dense_strides, query, run_gpu
from oracle import binding as oracle


def rng(seed):
    return np.random.default_rng(1000 + seed)


# ------------------------------------------------------------- CPU: oracle pins
def test_permutation_matches_numpy_transpose():
    dims = (3, 5, 7)
    x = np.arange(np.prod(dims), dtype=np.float32).reshape(dims)
    for perm in [(0, 1, 2), (0, 2, 1), (2, 0, 1), (1, 2, 0), (2, 1, 0)]:
        p = ReorderProblem(dims=dims, src_dt=cabi.DT_F32, dst_dt=cabi.DT_F32, src=x,
                           dst_stride=dense_strides(dims, perm))
        got = oracle.reorder(p)
        want = np.ascontiguousarray(np.transpose(x, perm)).reshape(-1)
        assert np.array_equal(got, want), perm
    # strided (transposed) source as well
    xs = np.ascontiguousarray(np.transpose(x, (1, 0, 2)))  # memory order (5,3,7)
    p = ReorderProblem(dims=dims, src_dt=cabi.DT_F32, dst_dt=cabi.DT_F32, src=xs,
                       src_stride=dense_strides(dims, (1, 0, 2)))
    assert np.array_equal(oracle.reorder(p), x.reshape(-1))


def test_quantize_f32_to_s8_matches_numpy():
    M, N = 6, 8
    x = rng(1).uniform(-40, 40, size=(M, N)).astype(np.float32)
    x[0, :4] = [0.5, 1.5, 2.5, -0.5]          # ties
    x[1, :2] = [1e6, -1e6]                     # saturation
    ssc = rng(2).uniform(0.5, 2, size=N).astype(np.float32)      # per last dim
    dsc = np.array([0.25], np.float32)
    dzp = np.array([3], np.int32)
    p = ReorderProblem(dims=(M, N), src_dt=cabi.DT_F32, dst_dt=cabi.DT_S8, src=x,
                       quant={"src_scale": QuantParam(cabi.DT_F32, 2, ssc),
                              "dst_scale": QuantParam(cabi.DT_F32, 0, dsc),
                              "dst_zp": QuantParam(cabi.DT_S32, 0, dzp)})
    got = oracle.reorder(p).reshape(M, N)
    d = (ssc[None, :] * x).astype(np.float32)
    d = (d / dsc[0]).astype(np.float32) + np.float32(3)
    want = np.rint(np.clip(d, -128, 127)).astype(np.int8)
    assert np.array_equal(got, want)
    # unit scale and no zero point: plain saturating conversion with ties to even
    p2 = ReorderProblem(dims=(M, N), src_dt=cabi.DT_F32, dst_dt=cabi.DT_U8, src=x)
    assert np.array_equal(oracle.reorder(p2).reshape(M, N), np.rint(np.clip(x, 0, 255)).astype(np.uint8))


def test_dequantize_u4_grouped_matches_numpy_and_one_hot():
    K, N, G = 64, 10, 16
    codes = rng(3).integers(0, 16, size=(K, N)).astype(np.uint8)
    zp = rng(4).integers(0, 16, size=(K // G, N)).astype(np.uint8)
    sc = dtp.f32_to_bf16(rng(5).uniform(0.01, 0.1, size=(K // G, N)).astype(np.float32))
    p = ReorderProblem(dims=(K, N), src_dt=cabi.DT_U4, dst_dt=cabi.DT_F32, src=dtp.pack_nibbles(codes.reshape(-1)),
                       quant={"src_scale": QuantParam(cabi.DT_BF16, 3, sc, (G, 1)),
                              "src_zp": QuantParam(cabi.DT_U4, 3, dtp.pack_nibbles(zp.reshape(-1)), (G, 1))})
    got = oracle.reorder(p).reshape(K, N)
    scf = dtp.bf16_to_f32(sc).reshape(K // G, N)
    want = (np.repeat(scf, G, axis=0) * (codes.astype(np.float32) - np.repeat(zp, G, axis=0).astype(np.float32)))
    assert np.array_equal(got, want.astype(np.float32))
    # s4: sign extension
    s4 = rng(6).integers(-8, 8, size=(K, N))
    p = ReorderProblem(dims=(K, N), src_dt=cabi.DT_S4, dst_dt=cabi.DT_F32,
                       src=dtp.pack_nibbles((s4 & 0xf).astype(np.uint8).reshape(-1)))
    assert np.array_equal(oracle.reorder(p).reshape(K, N), s4.astype(np.float32))


def test_to_4bit_packs_along_the_dst_unit_stride_dim():
    K, N = 6, 8
    x = rng(7).uniform(-9, 17, size=(K, N)).astype(np.float32)
    x[0, :4] = [0.5, 1.5, 2.5, 14.5]
    for dt, lo, hi in ((cabi.DT_U4, 0, 15), (cabi.DT_S4, -8, 7)):
        codes = (np.rint(np.clip(x, lo, hi)).astype(np.int32) & 0xf).astype(np.uint8)
        p = ReorderProblem(dims=(K, N), src_dt=cabi.DT_F32, dst_dt=dt, src=x)
        assert np.array_equal(oracle.reorder(p), dtp.pack_nibbles(codes.reshape(-1)))
        # column-major dst ("ba"): pairs along K
        p = ReorderProblem(dims=(K, N), src_dt=cabi.DT_F32, dst_dt=dt, src=x, dst_stride=(1, K))
        assert np.array_equal(oracle.reorder(p), dtp.pack_nibbles(np.ascontiguousarray(codes.T).reshape(-1)))
    p = ReorderProblem(dims=(K, N), src_dt=cabi.DT_F32, dst_dt=cabi.DT_F4_E2M1, src=x)
    assert np.array_equal(oracle.reorder(p), dtp.pack_nibbles(dtp.f32_to_e2m1_codes(x.reshape(-1))))


def test_integer_sources_subtract_as_integers_and_sum_post_op():
    x = np.array([[2 ** 30 + 1, 2 ** 30 + 3, -5, 7]], dtype=np.int32)
    zp = np.array([2 ** 30], np.int32)
    p = ReorderProblem(dims=(1, 4), src_dt=cabi.DT_S32, dst_dt=cabi.DT_F32, src=x,
                       quant={"src_zp": QuantParam(cabi.DT_S32, 0, zp)})
    got = oracle.reorder(p)
    # a float subtraction would lose the +1 / +3 (2^30 + 1 is not a float)
    assert np.array_equal(got, (x.astype(np.int64) - 2 ** 30).astype(np.float32).reshape(-1))
    old = np.array([10, 20, 30, 40], np.float32)
    p = ReorderProblem(dims=(1, 4), src_dt=cabi.DT_S32, dst_dt=cabi.DT_F32, src=np.array([[1, 2, 3, 4]], np.int32),
                       beta=0.5, dst_init=old)
    assert np.array_equal(oracle.reorder(p), np.array([6, 12, 18, 24], np.float32))


def test_an_s32_copy_keeps_every_bit():
    """Same type, no attributes: the reference's copy implementations cast (simple_q10n.hpp:84-99); only its generic
    loop would round 2^24 + 1 to a float on the way.  With an attribute the value does go through f32."""
    x = np.array([[2 ** 24 + 1, -(2 ** 31), 2 ** 31 - 1, 2 ** 30 + 3, -7, 0]], dtype=np.int32)
    p = ReorderProblem(dims=(1, 6), src_dt=cabi.DT_S32, dst_dt=cabi.DT_S32, src=x)
    assert np.array_equal(oracle.reorder(p), x.reshape(-1))
    t = ReorderProblem(dims=(2, 3), src_dt=cabi.DT_S32, dst_dt=cabi.DT_S32, src=x.reshape(2, 3), dst_stride=(1, 2))
    assert np.array_equal(oracle.reorder(t), np.ascontiguousarray(x.reshape(2, 3).T).reshape(-1))
    q = ReorderProblem(dims=(1, 6), src_dt=cabi.DT_S32, dst_dt=cabi.DT_S32, src=x,
                       quant={"src_scale": QuantParam(cabi.DT_F32, 0, np.array([1.0], np.float32))})
    got = oracle.reorder(q)
    assert got[0] == 2 ** 24 and got[1] == -(2 ** 31) and got[4] == -7       # 2^24 + 1 is not a float


def test_conversions_between_the_float_types():
    x = rng(8).standard_normal(64).astype(np.float32) * 3
    for dt, enc in ((cabi.DT_BF16, dtp.f32_to_bf16), (cabi.DT_F16, dtp.f32_to_f16_bits),
                    (cabi.DT_F8_E4M3, dtp.f32_to_e4m3)):
        p = ReorderProblem(dims=(8, 8), src_dt=cabi.DT_F32, dst_dt=dt, src=x)
        assert np.array_equal(oracle.reorder(p), enc(x)), dt
        back = ReorderProblem(dims=(8, 8), src_dt=dt, dst_dt=cabi.DT_F32, src=enc(x))
        assert np.array_equal(oracle.reorder(back), decode(dt, enc(x), 64))
    e = np.array([0, 1, 126, 127, 128, 254], np.uint8)
    p = ReorderProblem(dims=(6,), src_dt=cabi.DT_E8M0, dst_dt=cabi.DT_F32, src=e)
    assert np.array_equal(oracle.reorder(p), dtp.e8m0_to_f32(e))


def test_query_rejects_what_the_kernels_do_not_compute():
    x = np.zeros((4, 6), np.float32)
    ok = ReorderProblem(dims=(4, 6), src_dt=cabi.DT_F32, dst_dt=cabi.DT_S8, src=x)
    assert query(ok) == cabi.SUCCESS
    # zero points need integer data (src/common/reorder.cpp:96-103)
    bad = ReorderProblem(dims=(4, 6), src_dt=cabi.DT_F32, dst_dt=cabi.DT_F32, src=x,
                         quant={"src_zp": QuantParam(cabi.DT_S32, 0, np.zeros(1, np.int32))})
    assert query(bad) == cabi.INVALID_ARGUMENTS
    # groups must divide the dims (:122-134)
    bad = ReorderProblem(dims=(4, 6), src_dt=cabi.DT_U8, dst_dt=cabi.DT_F32, src=x.astype(np.uint8),
                         quant={"src_scale": QuantParam(cabi.DT_F32, 3, np.ones(6, np.float32), (3, 1))})
    assert query(bad) == cabi.INVALID_ARGUMENTS
    # odd unit-stride dim of a 4-bit dst: nibble pairs would straddle rows
    odd = ReorderProblem(dims=(4, 5), src_dt=cabi.DT_F32, dst_dt=cabi.DT_U4, src=np.zeros((4, 5), np.float32))
    assert query(odd) == cabi.UNIMPLEMENTED


# ------------------------------------------------------------- GPU: parity
def _case(name, dims, src_dt, dst_dt, seed, src_perm=None, dst_perm=None, quant=None, beta=0.0):
    r = rng(seed)
    n = int(np.prod(dims))
    if src_dt == cabi.DT_F32:
        src = (r.standard_normal(n) * 20).astype(np.float32)
    elif src_dt == cabi.DT_BF16:
        src = dtp.f32_to_bf16((r.standard_normal(n) * 20).astype(np.float32))
    elif src_dt == cabi.DT_F16:
        src = (r.standard_normal(n) * 20).astype(np.float16).view(np.uint16)
    elif src_dt == cabi.DT_S8:
        src = r.integers(-128, 128, size=n).astype(np.int8)
    elif src_dt == cabi.DT_U8:
        src = r.integers(0, 256, size=n).astype(np.uint8)
    elif src_dt == cabi.DT_S32:
        src = r.integers(-2 ** 31, 2 ** 31, size=n).astype(np.int32)
    elif src_dt in (cabi.DT_U4, cabi.DT_S4, cabi.DT_F4_E2M1):
        src = dtp.pack_nibbles(r.integers(0, 16, size=n).astype(np.uint8))
    elif src_dt in (cabi.DT_F8_E4M3, cabi.DT_E8M0):
        src = r.integers(0, 255, size=n).astype(np.uint8)
        if src_dt == cabi.DT_F8_E4M3:
            src[(src & 0x7f) == 0x7f] = 0x3c  # no NaN codes
    else:
        raise ValueError(src_dt)
    kw = {}
    if src_perm is not None:
        kw["src_stride"] = dense_strides(dims, src_perm)
    if dst_perm is not None:
        kw["dst_stride"] = dense_strides(dims, dst_perm)
    p = ReorderProblem(dims=dims, src_dt=src_dt, dst_dt=dst_dt, src=src, quant=quant or {}, beta=beta, name=name,
                       **kw)
    if beta:
        p.dst_init = (r.standard_normal(p.dst_storage_elems()) * 4).astype(np.float32)
    return p


def _qp(seed, dt, mask, shape, groups=(1, 1), lo=0.05, hi=2.0):
    r = rng(seed)
    n = int(np.prod(shape))
    if dt == cabi.DT_F32:
        data = r.uniform(lo, hi, size=n).astype(np.float32)
    elif dt == cabi.DT_BF16:
        data = dtp.f32_to_bf16(r.uniform(lo, hi, size=n).astype(np.float32))
    elif dt == cabi.DT_S32:
        data = r.integers(-5, 6, size=n).astype(np.int32)
    elif dt == cabi.DT_U4:
        data = dtp.pack_nibbles(r.integers(0, 16, size=n).astype(np.uint8))
    elif dt == cabi.DT_S8:
        data = r.integers(-5, 6, size=n).astype(np.int8)
    else:
        raise ValueError(dt)
    return QuantParam(dt, mask, data, groups)


CASES = [
    # s32 over its whole range: a copy or a transposition keeps every bit (values beyond 2^24 included)
    lambda: _case("s32 copy", (19, 260), cabi.DT_S32, cabi.DT_S32, 38),
    lambda: _case("s32 transposition", (40, 1000), cabi.DT_S32, cabi.DT_S32, 39, dst_perm=(1, 0)),
    # direct kernel, 16 / 8 elements per lane: attribute-free (one base per unit) ...
    lambda: _case("s8 copy 16 per lane", (24, 512), cabi.DT_S8, cabi.DT_S8, 40),
    lambda: _case("u8->f32 16 per lane, rows strided", (3, 40, 64), cabi.DT_U8, cabi.DT_F32, 41, src_perm=(1, 0, 2)),
    lambda: _case("f32->bf16 8 per lane", (37, 72), cabi.DT_F32, cabi.DT_BF16, 42),
    lambda: _case("u4->s8 16 per lane", (20, 96), cabi.DT_U4, cabi.DT_S8, 43),
    lambda: _case("s8 copy, extent only a multiple of 8", (9, 40), cabi.DT_S8, cabi.DT_S8, 44),
    # ... and with parameters that are consecutive along the unit (vector loads) or constant along it
    lambda: _case("f32->s8 per-column scale, 8 per lane", (33, 128), cabi.DT_F32, cabi.DT_S8, 45,
                  quant={"dst_scale": _qp(60, cabi.DT_F32, 2, (128,))}),
    lambda: _case("s8->bf16 per-column bf16 scale + u4 zp", (17, 64), cabi.DT_S8, cabi.DT_BF16, 46,
                  quant={"src_scale": _qp(61, cabi.DT_BF16, 2, (64,)), "src_zp": _qp(62, cabi.DT_U4, 2, (64,))}),
    lambda: _case("s8->f32 per-row scale, per-column zp", (48, 64), cabi.DT_S8, cabi.DT_F32, 47,
                  quant={"src_scale": _qp(63, cabi.DT_F32, 1, (48,)), "src_zp": _qp(64, cabi.DT_S8, 2, (64,)),
                         "dst_scale": _qp(65, cabi.DT_F32, 3, (48, 64))}),
    lambda: _case("u8->s8 grouped along the unit (per-element offsets)", (16, 128), cabi.DT_U8, cabi.DT_S8, 48,
                  quant={"src_scale": _qp(66, cabi.DT_F32, 3, (16, 4), (1, 32))}),
    lambda: _case("f32->f32 per-column scale with sum (per-element offsets)", (12, 64), cabi.DT_F32, cabi.DT_F32, 49,
                  quant={"dst_scale": _qp(67, cabi.DT_F32, 2, (64,))}, beta=0.5),
    # 8-bit transposition in registers (whole 64 x 64 tiles) and its fallback for ragged extents
    lambda: _case("s8 ab->ba whole tiles", (128, 192), cabi.DT_S8, cabi.DT_S8, 50, dst_perm=(1, 0)),
    lambda: _case("u8 batched acb whole tiles", (3, 64, 128), cabi.DT_U8, cabi.DT_U8, 51, dst_perm=(0, 2, 1)),
    lambda: _case("e4m3 ba->ab whole tiles", (192, 64), cabi.DT_F8_E4M3, cabi.DT_F8_E4M3, 52, src_perm=(1, 0)),
    lambda: _case("s8 ab->ba ragged", (130, 192), cabi.DT_S8, cabi.DT_S8, 53, dst_perm=(1, 0)),
    # ... on 128 x 128 tiles (whole cache lines on both sides) where both extents are multiples of 128
    lambda: _case("s8 ab->ba whole 128-byte lines", (256, 384), cabi.DT_S8, cabi.DT_S8, 80, dst_perm=(1, 0)),
    lambda: _case("u8 batched acb whole 128-byte lines", (3, 128, 256), cabi.DT_U8, cabi.DT_U8, 81, dst_perm=(0, 2, 1)),
    lambda: _case("e4m3 ba->ab whole 128-byte lines", (384, 128), cabi.DT_F8_E4M3, cabi.DT_F8_E4M3, 82, src_perm=(1, 0)),
    # tiled kernel: attribute-free, parameters constant along / consecutive along the dst-contiguous dim, generic
    lambda: _case("bf16->f32 transposed", (96, 80), cabi.DT_BF16, cabi.DT_F32, 54, dst_perm=(1, 0)),
    lambda: _case("u4 transposed", (64, 96), cabi.DT_U4, cabi.DT_U4, 55, dst_perm=(1, 0)),
    lambda: _case("f32->s8 transposed, scale per src-contiguous dim", (72, 128), cabi.DT_F32, cabi.DT_S8, 56,
                  dst_perm=(1, 0), quant={"dst_scale": _qp(70, cabi.DT_F32, 2, (128,))}),
    lambda: _case("s8->f32 transposed, scale and zp per dst-contiguous dim", (64, 48), cabi.DT_S8, cabi.DT_F32, 57,
                  dst_perm=(1, 0), quant={"src_scale": _qp(71, cabi.DT_BF16, 1, (64,)), "src_zp": _qp(72, cabi.DT_S8, 1, (64,))}),
    lambda: _case("f32->s8 transposed, ragged dst-contiguous extent", (70, 64), cabi.DT_F32, cabi.DT_S8, 58,
                  dst_perm=(1, 0), quant={"dst_scale": _qp(73, cabi.DT_F32, 2, (64,))}),
    lambda: _case("u8->s8 transposed, groups on both dims", (64, 64), cabi.DT_U8, cabi.DT_S8, 59,
                  dst_perm=(1, 0), quant={"src_scale": _qp(74, cabi.DT_F32, 3, (2, 4), (32, 16))}),
    # direct kernel: same unit-stride dim on both sides
    lambda: _case("copy f32 ragged", (7, 33), cabi.DT_F32, cabi.DT_F32, 1),
    lambda: _case("f32->s8 packed stores", (64, 256), cabi.DT_F32, cabi.DT_S8, 2,
                  quant={"dst_scale": _qp(20, cabi.DT_F32, 0, (1,)), "dst_zp": _qp(21, cabi.DT_S32, 0, (1,))}),
    lambda: _case("f32->bf16 3-D", (3, 17, 40), cabi.DT_F32, cabi.DT_BF16, 3),
    lambda: _case("s8->f32 per-dim scales", (48, 36), cabi.DT_S8, cabi.DT_F32, 4,
                  quant={"src_scale": _qp(22, cabi.DT_F32, 2, (36,)), "src_zp": _qp(23, cabi.DT_S32, 0, (1,))}),
    lambda: _case("s32->s8 saturating", (16, 64), cabi.DT_S32, cabi.DT_S8, 5),
    lambda: _case("u4 grouped dequant", (128, 48), cabi.DT_U4, cabi.DT_BF16, 6,
                  quant={"src_scale": _qp(24, cabi.DT_BF16, 3, (4, 48), (32, 1), 0.01, 0.1),
                         "src_zp": _qp(25, cabi.DT_U4, 3, (4, 48), (32, 1))}),
    lambda: _case("f32->u4", (32, 64), cabi.DT_F32, cabi.DT_U4, 7),
    lambda: _case("f32->s4 odd rows", (5, 6), cabi.DT_F32, cabi.DT_S4, 8),
    lambda: _case("f32->f4_e2m1", (16, 32), cabi.DT_F32, cabi.DT_F4_E2M1, 9),
    lambda: _case("f32->e4m3", (16, 48), cabi.DT_F32, cabi.DT_F8_E4M3, 10),
    lambda: _case("e4m3->f32", (16, 48), cabi.DT_F8_E4M3, cabi.DT_F32, 11),
    lambda: _case("e8m0->f32", (8, 32), cabi.DT_E8M0, cabi.DT_F32, 12),
    lambda: _case("sum post-op", (12, 20), cabi.DT_S8, cabi.DT_F32, 13, beta=0.5),
    lambda: _case("strided both ways, no unit dim on dst", (9, 11), cabi.DT_F32, cabi.DT_F32, 14, dst_perm=(1, 0),
                  src_perm=(1, 0)),
    # tiled kernel: transpositions
    lambda: _case("s8 ab->ba", (256, 192), cabi.DT_S8, cabi.DT_S8, 15, dst_perm=(1, 0)),
    lambda: _case("s8 ab->ba ragged", (100, 70), cabi.DT_S8, cabi.DT_S8, 16, dst_perm=(1, 0)),
    lambda: _case("f32 ab -> s8 ba quantized", (130, 96), cabi.DT_F32, cabi.DT_S8, 17, dst_perm=(1, 0),
                  quant={"src_scale": _qp(26, cabi.DT_F32, 2, (96,)), "dst_scale": _qp(27, cabi.DT_F32, 0, (1,))}),
    lambda: _case("u4 ab -> u4 ba", (64, 96), cabi.DT_U4, cabi.DT_U4, 18, dst_perm=(1, 0)),
    lambda: _case("u4 ab -> u4 ba ragged", (38, 50), cabi.DT_U4, cabi.DT_U4, 19, dst_perm=(1, 0)),
    lambda: _case("bf16 batched transpose", (3, 40, 72), cabi.DT_BF16, cabi.DT_BF16, 30, dst_perm=(0, 2, 1)),
    lambda: _case("f32 batch-innermost src", (4, 33, 20), cabi.DT_F32, cabi.DT_F32, 31, src_perm=(1, 2, 0)),
    lambda: _case("f32 -> e4m3 transposed", (80, 64), cabi.DT_F32, cabi.DT_F8_E4M3, 32, dst_perm=(1, 0)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("make", CASES, ids=[f"r{i}" for i in range(len(CASES))])
def test_gpu_reorder_is_bit_exact(make):
    p = make()
    assert query(p) == cabi.SUCCESS, p.name
    want = oracle.reorder(p)
    got = run_gpu(p)
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, f"{p.name}: {bad.size} of {got.size} storage elements differ, first at {bad[:5]}"


# Row quantization kernel (float src -> 8-bit dst, scales per tensor or per column, at most one outer dim): ragged row
# counts, column counts that end inside a workgroup's 1024, every src / dst type it takes, and the values that leave
# its reciprocal-based division (scales outside 2^-20 .. 2^20, huge / infinite / tiny / signed-zero values)
ROW_CASES = [
    lambda: _case("f32->s8 src common, dst per column, dst zp", (37, 1100), cabi.DT_F32, cabi.DT_S8, 90,
                  quant={"src_scale": _qp(91, cabi.DT_F32, 0, (1,)), "dst_scale": _qp(92, cabi.DT_F32, 2, (1100,)),
                         "dst_zp": _qp(93, cabi.DT_S32, 0, (1,))}),
    lambda: _case("bf16->e4m3 common src scale", (5, 2052), cabi.DT_BF16, cabi.DT_F8_E4M3, 94,
                  quant={"src_scale": _qp(95, cabi.DT_F32, 0, (1,), lo=0.5, hi=4.0)}),
    lambda: _case("f16->u8 per-column src scale, dst zp", (18, 260), cabi.DT_F16, cabi.DT_U8, 96,
                  quant={"src_scale": _qp(97, cabi.DT_F32, 2, (260,)), "dst_zp": _qp(98, cabi.DT_S32, 0, (1,))}),
    lambda: _case("f32->e5m2 per-column dst scale", (7, 512), cabi.DT_F32, cabi.DT_F8_E5M2, 99,
                  quant={"dst_scale": _qp(100, cabi.DT_F32, 2, (512,))}),
    lambda: _case("f32->s8 one row", (4096,), cabi.DT_F32, cabi.DT_S8, 101,
                  quant={"dst_scale": _qp(102, cabi.DT_F32, 0, (1,))}),
    lambda: _case("bf16->s8 attribute-free", (9, 1024), cabi.DT_BF16, cabi.DT_S8, 103),
    lambda: _case("f16->e4m3 batched rows merge into one outer dim", (3, 5, 256), cabi.DT_F16, cabi.DT_F8_E4M3, 104,
                  quant={"dst_scale": _qp(105, cabi.DT_F32, 4, (256,))}),
]


@pytest.mark.gpu
@pytest.mark.parametrize("make", ROW_CASES, ids=[f"rows{i}" for i in range(len(ROW_CASES))])
def test_gpu_row_quantization_is_bit_exact(make):
    p = make()
    assert query(p) == cabi.SUCCESS, p.name
    want = oracle.reorder(p)
    got = run_gpu(p)
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, f"{p.name}: {bad.size} of {got.size} storage elements differ, first at {bad[:5]}"


@pytest.mark.gpu
@pytest.mark.parametrize("dst_dt", [cabi.DT_S8, cabi.DT_U8, cabi.DT_F8_E4M3])
def test_gpu_row_quantization_special_values(dst_dt):
    rows, cols = 12, 64
    r = rng(110)
    x = (r.standard_normal((rows, cols)) * 50).astype(np.float32)
    special = np.array([np.inf, -np.inf, 3e38, -3e38, 1e-40, -1e-40, 0.0, -0.0, 2.0 ** 100, -(2.0 ** 99), 127.5, -128.5,
                        0.5, 1.5, 2.5, -0.5, 1e-30, 448.0, 500.0, 57344.0], np.float32)
    x[0, :special.size] = special
    x[5, 3:3 + special.size] = special
    if dst_dt == cabi.DT_F8_E4M3:
        x[7, 9] = np.nan
    sc = r.uniform(0.05, 2.0, size=cols).astype(np.float32)
    sc[[1, 17, 40]] = [1e-8, 3e7, 2.0 ** -20]          # outside / at the edge of the reciprocal path's range
    sc[[2, 18]] = [-0.75, 2.0 ** 20]
    p = ReorderProblem(dims=(rows, cols), src_dt=cabi.DT_F32, dst_dt=dst_dt, src=x.reshape(-1),
                       quant={"dst_scale": QuantParam(cabi.DT_F32, 2, sc)}, name="special values")
    assert query(p) == cabi.SUCCESS
    want = oracle.reorder(p)
    got = run_gpu(p)
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, f"{bad.size} of {got.size} differ, first at {bad[:8]}: got {got[bad[:8]]} want {want[bad[:8]]}"


@pytest.mark.gpu
def test_gpu_generic_kernels_behind_the_dedicated_ones():
    """MI355_REORDER_GENERIC=1 (read once per process) keeps the row-quantization and whole-line transposition
    kernels out, so the same cases run on the direct / 64 x 64 kernels they would otherwise shadow."""
    import subprocess
    import sys
    env = dict(os.environ, MI355_REORDER_GENERIC="1")
    out = subprocess.run(
        [sys.executable, "-m", "pytest", os.path.abspath(__file__), "-q", "-m", "gpu", "-x", "-k",
         "test_gpu_reorder_is_bit_exact or test_gpu_row_quantization"],
        env=env, capture_output=True, text=True, timeout=600, cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-2000:]


@pytest.mark.gpu
def test_full_size_transposition_round_trips():
    """8192 x 8192 s8 (the weights of the int8 headline shape): ab -> ba -> ab
    returns the input, and the ba copy equals numpy's transpose."""
    N = 8192
    x = rng(40).integers(-128, 128, size=(N, N), dtype=np.int8)
    t = run_gpu(ReorderProblem(dims=(N, N), src_dt=cabi.DT_S8, dst_dt=cabi.DT_S8, src=x, dst_stride=(1, N)))
    assert np.array_equal(t.reshape(N, N), x.T)
    back = run_gpu(ReorderProblem(dims=(N, N), src_dt=cabi.DT_S8, dst_dt=cabi.DT_S8, src=t, src_stride=(1, N)))
    assert np.array_equal(back.reshape(N, N), x)


@pytest.mark.gpu
def test_full_size_quantization_matches_numpy():
    """f32 -> s8 with per-column scales at 4096 x 8192: numpy's float32
    arithmetic is the same sequence of correctly rounded operations."""
    M, N = 4096, 8192
    x = (rng(41).standard_normal((M, N)) * 30).astype(np.float32)
    ssc = rng(42).uniform(0.5, 2, size=N).astype(np.float32)
    p = ReorderProblem(dims=(M, N), src_dt=cabi.DT_F32, dst_dt=cabi.DT_S8, src=x,
                       quant={"src_scale": QuantParam(cabi.DT_F32, 2, ssc)})
    got = run_gpu(p).reshape(M, N)
    want = np.rint(np.clip(ssc[None, :] * x, -128, 127)).astype(np.int8)
    assert np.array_equal(got, want)
