"""Packed decode weights (MI355_WEI_PACK_WOQ64): the layout itself (CPU), and
the decode kernel that reads it against the CPU oracle, which always sees the
plain weights (GPU).

What pins the layout without a GPU: the nibble offset formula of the header is
evaluated element by element in plain Python, the numpy packer and the
six-dim reorder view (run by the oracle's reorder) must both reproduce it.
"""
import ctypes as C

import numpy as np
import pytest

from onednn_amd import cabi, configs
from onednn_amd import dtypes as dtp
from onednn_amd.problem import pack_woq64, run_gpu
from onednn_amd.reorder import ReorderProblem
from onednn_amd import reorder as reorder_host
from oracle import binding as oracle_binding
from tests.helpers import assert_bit_exact, assert_close, assert_decode_close, assert_gemm_close


def nibble_offset(k, n, K):
    return ((n // 64) * (K * 64) + (k // 8) * 512 + (n % 16) * 32 + ((n % 64) // 16) * 8
            + (k % 2) * 4 + (k % 8) // 2)


def random_u4(K, N, seed):
    r = np.random.default_rng(seed)
    nib = r.integers(0, 16, size=(K, N), dtype=np.uint8)
    return nib, dtp.pack_nibbles(nib.reshape(-1))


def woq64_view(K, N, stride_k, stride_n):
    d = cabi.ReorderDesc()
    lib = cabi.load_kernels()
    cabi.check(lib.mi355_wei_pack_reorder_dims(cabi.WEI_PACK_WOQ64, K, N, stride_k, stride_n, C.byref(d)))
    return (tuple(d.dims[i] for i in range(d.ndims)), tuple(d.src_stride[i] for i in range(d.ndims)),
            tuple(d.dst_stride[i] for i in range(d.ndims)))


# ------------------------------------------------------------------ CPU
@pytest.mark.parametrize("K,N", [(32, 64), (64, 128), (96, 192)])
def test_numpy_packer_follows_the_offset_formula(K, N):
    nib, raw = random_u4(K, N, 7)
    packed = dtp.unpack_nibbles(pack_woq64(raw, K, N), K * N)
    want = np.empty(K * N, np.uint8)
    for k in range(K):
        for n in range(N):
            want[nibble_offset(k, n, K)] = nib[k, n]
    assert np.array_equal(packed, want)
    # the formula is a bijection onto [0, K * N)
    offs = sorted(nibble_offset(k, n, K) for k in range(K) for n in range(N))
    assert offs == list(range(K * N))


@pytest.mark.parametrize("transposed", [False, True])
def test_reorder_view_packs_like_the_numpy_packer(transposed):
    K, N = 64, 128
    nib, raw = random_u4(K, N, 11)
    if transposed:  # weights stored [N][K]
        src = dtp.pack_nibbles(np.ascontiguousarray(nib.T).reshape(-1))
        sk, sn = 1, K
    else:
        src, sk, sn = raw, N, 1
    dims, ss, ds = woq64_view(K, N, sk, sn)
    assert int(np.prod(dims)) == K * N
    p = ReorderProblem(dims=dims, src_dt=cabi.DT_U4, dst_dt=cabi.DT_U4, src=src, src_stride=ss, dst_stride=ds)
    got = oracle_binding.reorder(p)
    assert np.array_equal(np.asarray(got).view(np.uint8).reshape(-1), pack_woq64(raw, K, N))
    assert np.array_equal(pack_woq64(src, K, N, sk, sn), pack_woq64(raw, K, N))


def test_packing_rules_of_the_matmul_descriptor():
    p = configs.config2(M=1, N=512, K=1024)
    p.wei_packing = cabi.WEI_PACK_WOQ64
    st, impl = cabi.query(p.desc())
    assert st == cabi.SUCCESS and cabi.impl_name(impl).startswith("hip:woq_packed")
    # the generic kernel reads the layout too, the plain decode kernel and the GEMM families do not
    assert cabi.query(p.desc(), cabi.IMPL_REF)[0] == cabi.SUCCESS
    assert cabi.query(p.desc(), cabi.IMPL_WOQ_GEMV)[0] == cabi.UNIMPLEMENTED
    # plain weights are not for the packed kernel
    q = configs.config2(M=1, N=512, K=1024)
    assert cabi.query(q.desc(), cabi.IMPL_WOQ_PACKED)[0] == cabi.UNIMPLEMENTED
    # shapes the layout does not tile, and other weight types, are invalid
    for M, N, K in [(1, 512 + 16, 1024), (1, 512, 1024 + 16)]:
        b = configs.config2(M=M, N=N, K=K, group=16)
        b.wei_packing = cabi.WEI_PACK_WOQ64
        assert cabi.query(b.desc())[0] == cabi.INVALID_ARGUMENTS
    c = configs.config1(M=32, N=64, K=64)
    c.wei_packing = cabi.WEI_PACK_WOQ64
    assert cabi.query(c.desc())[0] == cabi.INVALID_ARGUMENTS
    # group sizes the packed kernel does not cover fall to the generic kernel
    g = configs.config2(M=1, N=512, K=960, group=96)
    g.wei_packing = cabi.WEI_PACK_WOQ64
    st, impl = cabi.query(g.desc())
    assert st == cabi.SUCCESS and cabi.impl_name(impl).startswith("hip:ref")
    # more rows than the decode kernels take
    m = configs.config2(M=33, N=512, K=1024)
    m.wei_packing = cabi.WEI_PACK_WOQ64
    assert cabi.impl_name(cabi.query(m.desc())[1]).startswith("hip:ref")


# ------------------------------------------------------------------ GPU
def packed(p):
    p.wei_packing = cabi.WEI_PACK_WOQ64
    return p


@pytest.mark.gpu
@pytest.mark.parametrize("M", [1, 8, 32])
def test_config2_small_packed_kernel(gpu, oracle, M):
    # against the oracle's float64 sum, under the bound derived from the kernel's factoring
    p = packed(configs.config2(M=M, N=512, K=1024))
    got, name = run_gpu(p, cabi.IMPL_WOQ_PACKED)
    assert name.startswith("hip:woq_packed")
    want, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    assert_decode_close(p, got, ideal, asum, what=name)


@pytest.mark.gpu
@pytest.mark.parametrize("K,group", [(32, 32), (64, 32), (256, 64), (512, 128), (1024, 1024), (2080 - 32, 2048)])
def test_packed_one_hot_rows_are_exact(gpu, oracle, K, group):
    # src rows are unit vectors: every output is a single decompressed weight,
    # (w - zp) * scale with one rounding -> must equal the oracle bit for bit.
    # Exercises the nibble order, the k order of both MFMA operands, group
    # indexing and the split of K over wavefronts.
    M = 32
    p = packed(configs.config2(M=M, N=128, K=K, group=group))
    hot = np.zeros((M, K), np.float32)
    r = np.random.default_rng(K)
    hot[np.arange(M), r.choice(K, size=M, replace=K < M)] = 1.0
    p.src = dtp.f32_to_bf16(hot)
    p.dst_dt = cabi.DT_F32
    got, name = run_gpu(p, cabi.IMPL_WOQ_PACKED)
    want = oracle.run_oracle(p)
    assert_bit_exact(p, got, want, name)


PACKED_VARIANTS = [
    # M, N, K, group, weights, scales dt/kind, zero points dt/kind, dst, bias+relu
    (1, 512, 1024, 128, "u4", "f32", "grouped", "s8", "grouped", "bf16", False),
    (5, 320, 1056, 1056, "u4", "f16", "column", "u8", "column", "f32", True),   # per-column parameters, ragged K split
    (16, 512, 512, 64, "s4", "bf16", "grouped", "s4", "grouped", "bf16", False),
    (17, 256, 2048, 128, "s4", "bf16", "grouped", "s32", "common", "f32", False),
    (32, 1024, 512, 32, "u4", "f32", "grouped", "u4", "none", "bf16", True),
    (3, 4096, 256, 256, "u4", "bf16", "none", "u8", "grouped", "f32", False),
    (8, 768, 4096, 128, "u4", "bf16", "grouped", "s32", "grouped", "bf16", False),
    (8, 128, 4096, 512, "s4", "f16", "grouped", "s8", "grouped", "f32", True),   # a group holds several super-steps
    (24, 192, 3072, 1024, "u4", "bf16", "grouped", "u4", "grouped", "f32", False),
    (16, 4096, 1024, 128, "u4", "f32", "column", "u4", "common", "bf16", False),
    (2, 14336, 256, 128, "u4", "bf16", "grouped", "s4", "column", "f32", False),
    (20, 64, 96, 32, "u4", "bf16", "grouped", "u4", "grouped", "f32", False),    # fewer blocks than wavefronts
    (9, 64, 2304, 256, "u4", "bf16", "grouped", "u8", "grouped", "bf16", False), # uneven K ranges
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", PACKED_VARIANTS, ids=lambda c: "-".join(str(x) for x in c))
def test_packed_attribute_variants(gpu, oracle, case):
    M, N, K, group, wdt, sdt, skind, zdt, zkind, ddt, relu_bias = case
    p = packed(configs.woq_variant(M, N, K, group, wei_dt=wdt, sc_dt=sdt, sc_kind=skind, zp_dt=zdt, zp_kind=zkind,
                                   dst_dt=ddt, relu_bias=relu_bias))
    got, name = run_gpu(p, cabi.IMPL_AUTO)
    assert name.startswith("hip:woq_packed")
    want, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    assert_decode_close(p, got, ideal, asum, what=name)
    # and the generic kernel, reading the same packed weights, follows the
    # reference's operation order exactly
    got_ref, name_ref = run_gpu(p, cabi.IMPL_REF)
    assert_bit_exact(p, got_ref, want, name_ref)


@pytest.mark.gpu
@pytest.mark.parametrize("pad", [0, 2, 64])
@pytest.mark.parametrize("transposed", [False, True])
def test_gpu_reorder_writes_the_packed_layout(gpu, transposed, pad):
    # pad = 0 / 64: pitches the dedicated packing kernel takes (16-byte rows,
    # 4-byte columns); pad = 2: the generic strided kernels on the six-dim view
    K, N = 256, 192
    nib, raw = random_u4(K, N, 13)
    if transposed:
        wide = np.zeros((N, K + pad), np.uint8)
        wide[:, :K] = nib.T
        sk, sn = 1, K + pad
    else:
        wide = np.zeros((K, N + pad), np.uint8)
        wide[:, :N] = nib
        sk, sn = N + pad, 1
    src = dtp.pack_nibbles(wide.reshape(-1))
    dims, ss, ds = woq64_view(K, N, sk, sn)
    p = ReorderProblem(dims=dims, src_dt=cabi.DT_U4, dst_dt=cabi.DT_U4, src=src, src_stride=ss, dst_stride=ds)
    got = reorder_host.run_gpu(p)
    assert np.array_equal(np.asarray(got).view(np.uint8).reshape(-1), pack_woq64(raw, K, N))


@pytest.mark.gpu
@pytest.mark.parametrize("M", [1, 8, 32])
def test_config2_full_size_both_decode_kernels_f32_and_bf16_dst(gpu, oracle, M):
    """The full decode shape, every dst element, both kernels, against the
    oracle's float64 sums under the bound derived from the kernels' factoring
    (tests/helpers.py decode_bound: about 2e-3 absolute on outputs of standard
    deviation 5; a zero point of one group off by one moves an output by about
    0.14, a group scale off by one bf16 unit by about 4e-3 -- shown on the CPU in
    tests/test_tolerances.py).  With an f32 dst nothing but the kernel's own
    arithmetic is inside the bound; the bf16 dst adds half a unit in its last
    place."""
    import copy
    from tests.helpers import decode_bound
    p = configs.config2(M=M)
    _, ideal, asum = oracle.run_oracle(p, want_ideal=True)
    bound = decode_bound(p)
    for dst_dt in (cabi.DT_F32, cabi.DT_BF16):
        q = copy.copy(p)
        q.dst_dt = dst_dt
        plain, name_plain = run_gpu(q, cabi.IMPL_WOQ_GEMV)
        assert name_plain.startswith("hip:woq_gemv")
        assert_decode_close(q, plain, ideal, asum, what=name_plain, bound=bound)
        got, name = run_gpu(packed(copy.copy(q)), cabi.IMPL_WOQ_PACKED)
        assert name.startswith("hip:woq_packed")
        worst = assert_decode_close(q, got, ideal, asum, what=name, bound=bound)
        assert worst < 1.0
