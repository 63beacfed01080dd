"""A seeded random sweep over the reorder primitive: one to five dims, every
pair of the path's data types, random permutations of both layouts, scales and
zero points with random masks.  Whatever the query accepts runs on the GPU and
must equal the oracle (the reference's per-element formula,
simple_reorder.hpp:2579-2661) storage element by storage element."""
import random

import numpy as np
import pytest

from onednn_amd import cabi
from onednn_amd.reorder import query, run_gpu
from oracle import binding as oracle
from tests.test_reorder import _case, _qp

SRC = [cabi.DT_F32, cabi.DT_BF16, cabi.DT_F16, cabi.DT_S8, cabi.DT_U8, cabi.DT_S32, cabi.DT_U4, cabi.DT_S4,
       cabi.DT_F8_E4M3, cabi.DT_F4_E2M1]
DST = SRC + [cabi.DT_F8_E5M2]


def random_problem(rnd, i):
    nd = rnd.randint(1, 5)
    dims, budget = [], 100000
    for _ in range(nd):
        d = max(1, min(rnd.choice([1, 2, 3, 4, 7, 8, 16, 17, 32, 33, 64, 100, 128, 256, 1000]), budget))
        dims.append(d)
        budget //= d
    if rnd.random() < 0.5:          # (4-bit tensors need an even unit-stride dim)
        dims = [2 * ((d + 1) // 2) for d in dims]
    sp, dp = list(range(nd)), list(range(nd))
    if rnd.random() < 0.5:
        rnd.shuffle(sp)
    if rnd.random() < 0.5:
        rnd.shuffle(dp)

    def param(dt):
        mask = sum(1 << b for b in range(nd) if rnd.random() < 0.3)
        shape = tuple(dims[b] for b in range(nd) if mask >> b & 1) or (1,)
        return _qp(rnd.randint(0, 1 << 30), dt, mask, shape)

    quant = {}
    if rnd.random() < 0.4:
        quant["src_scale"] = param(rnd.choice([cabi.DT_F32, cabi.DT_BF16]))
    if rnd.random() < 0.4:
        quant["dst_scale"] = param(cabi.DT_F32)
    if rnd.random() < 0.3:
        quant["src_zp"] = param(cabi.DT_S32)
    if rnd.random() < 0.3:
        quant["dst_zp"] = _qp(rnd.randint(0, 1 << 30), cabi.DT_S32, 0, (1,))
    return _case(f"sweep {i}: {tuple(dims)} src order {sp} dst order {dp}", tuple(dims), rnd.choice(SRC), rnd.choice(DST),
                 rnd.randint(0, 1 << 30), src_perm=tuple(sp), dst_perm=tuple(dp), quant=quant)


def test_the_generator_is_deterministic():
    a = [random_problem(random.Random(3), i).name for i in range(20)]
    assert a == [random_problem(random.Random(3), i).name for i in range(20)]


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [1, 2])
def test_random_reorders_match_the_oracle(gpu, seed):
    rnd = random.Random(seed)
    ran = 0
    for i in range(400):
        p = random_problem(rnd, i)
        if query(p) != cabi.SUCCESS:
            continue
        ran += 1
        want, got = oracle.reorder(p), run_gpu(p)
        bad = np.flatnonzero(got != want)
        assert bad.size == 0, f"{p.name} {p.src_dt}->{p.dst_dt} {sorted(p.quant)}: {bad.size} of {got.size} differ"
    assert ran > 200
