"""A seeded random sweep over the matmul's knobs through the benchdnn-style
driver (tests/benchdnn_matmul.py), the way the reference's CI batches random
problem lists through benchdnn: data types of every kernel family, tags of
all three tensors (including `any`), bias, scales, zero points, chains of up
to three post-ops, and sizes that are mostly NOT multiples of any tile -- M, N
and K tails, single rows and columns, K below one step.  Every case runs
through the dnnl_* API on whatever implementation the library picks and is
compared with the CPU oracle by the driver's own criteria (bit-exact for
integer dst, the data-type thresholds otherwise)."""
import random

import pytest

from tests import benchdnn_matmul as bd

DTS = [("u8:s8:f32", "i8"), ("s8:s8:s8", "i8"), ("u8:s8:u8", "i8"), ("s8:s8:s32", "i8"), ("u8:u8:bf16", "i8"),
       ("f8_e4m3:f8_e4m3:bf16", "f8"), ("f8_e5m2:f8_e4m3:f32", "f8"), ("f8_e4m3:f8_e5m2:f8_e4m3", "f8"),
       ("bf16:bf16:bf16", "h"), ("f16:f16:f32", "h"), ("f32:f32:f32", "h"), ("bf16:bf16:f32", "h"),
       ("bf16:u4:bf16", "woq"), ("f16:s4:f16", "woq"), ("bf16:s8:bf16", "woq"),
       ("f8_e4m3:f8_e4m3:bf16", "mx"), ("f8_e5m2:f8_e4m3:f32", "mx"), ("f4_e2m1:f4_e2m1:bf16", "mx"),
       ("f4_e2m1:f4_e2m1:f32", "mx")]
POST_OPS = ["relu", "linear:2:1", "add:f32", "add:bf16:per_oc", "mul:f32:per_oc", "sum", "gelu_tanh", "clip:-1:2", "tanh",
            "max:f32", "sum:0.5", "swish:1", "abs"]


def random_case(rnd):
    def dim(kmax):
        c = rnd.random()
        if c < 0.25:
            return rnd.choice([16, 32, 64, 128, 256, 384, 512])
        if c < 0.5:
            return rnd.randint(1, 40)
        return rnd.randint(1, kmax)

    dt, fam = rnd.choice(DTS)
    src_dt, wei_dt, dst_dt = dt.split(":")
    M, N, K = dim(600), dim(600), dim(700)
    argv = ["--matmul", f"--dt={dt}", f"--stag={rnd.choice(['ab', 'ab', 'ba'])}", f"--wtag={rnd.choice(['ab', 'ba', 'any'])}"]
    if rnd.random() < 0.5:
        argv.append(f"--bia-dt={rnd.choice(['f32', 'bf16'])}")
    sc, zp, po = [], [], []
    if fam == "i8":
        if rnd.random() < 0.7:
            sc.append("src:common:0.25")
        if rnd.random() < 0.7:
            sc.append(rnd.choice(["wei:per_oc", "wei:common:0.5"]))
        if dst_dt in ("s8", "u8") and rnd.random() < 0.7:
            sc.append("dst:common:2")
        if rnd.random() < 0.5:
            zp.append(f"src:common:{rnd.choice([1, 3, 128])}")
        if dst_dt in ("s8", "u8") and rnd.random() < 0.4:
            zp.append("dst:common:2")
        if rnd.random() < 0.2:
            zp.append("wei:common:1")
    elif fam == "f8":
        if rnd.random() < 0.6:
            sc.append("src:common:0.5")
        if rnd.random() < 0.6:
            sc.append(rnd.choice(["wei:per_oc", "wei:common:2"]))
    elif fam == "mx":       # e8m0 scales per 32 k on both operands
        K = 32 * rnd.choice([1, 2, 3, 4, 5, 8, 9, 16, 17])
        N += N % 2
        sc.append("src:per_tensor:e8m0:1x32")
        sc.append("wei:per_tensor:e8m0:32x1")
    elif fam == "woq":
        G = rnd.choice([32, 64, 128])
        K = max(G, (K // G) * G)
        M = rnd.choice([1, 2, 5, 8, 16, 31, 32, 33, 100])
        if rnd.random() < 0.5:
            N = rnd.choice([64, 128, 512, 1024, 14336])
        argv.append(f"--attr-fpmath={'bf16' if src_dt == 'bf16' else 'f16'}:true")
        sc.append(f"wei:per_ocic:{src_dt}:{G}x1")
        if rnd.random() < 0.7:
            zp.append(f"wei:per_ocic:{rnd.choice(['u4', 'u8'] if wei_dt == 'u4' else ['u8', 's8'])}:{G}x1")
    for _ in range(rnd.choice([0, 0, 1, 1, 2, 3])):
        po.append(rnd.choice(POST_OPS))
    if sc:
        argv.append("--attr-scales=" + "+".join(sc))
    if zp:
        argv.append("--attr-zero-points=" + "+".join(zp))
    if po:
        argv.append("--attr-post-ops=" + "+".join(po))
    argv.append(f"{M}x{K}:{K}x{N}")
    return argv


def test_the_generator_is_deterministic_and_parses():
    a = [random_case(random.Random(11)) for _ in range(3)]
    b = [random_case(random.Random(11)) for _ in range(3)]
    assert a == b
    rnd = random.Random(5)
    for _ in range(200):
        _, specs = bd.parse(random_case(rnd))
        assert len(specs) == 1


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_problems_match_the_oracle(gpu, oracle, seed):
    rnd = random.Random(seed)
    failures, impls = [], {}
    for _ in range(250):
        argv = random_case(rnd)
        _, specs = bd.parse(argv)
        status, impl, details = bd.run_spec(specs[0])
        impls[impl.split(":gfx")[0]] = impls.get(impl.split(":gfx")[0], 0) + 1
        if status == "FAILED":
            failures.append((specs[0].repro(), impl, details if isinstance(details, str) else details.get("errors")))
    assert not failures, failures[:5]
    # the sweep reaches the tuned families, not only the generic kernel
    for family in ("hip:mfma_i8", "hip:mfma_f8", "hip:mfma_h16", "hip:mfma_mxf4", "hip:ref:any"):
        assert impls.get(family, 0) > 0, impls
