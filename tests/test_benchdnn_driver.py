"""The benchdnn-style driver: parsing and problem construction on the CPU, the
reference's own input lines (tests/benchdnn/inputs/matmul/*, adapted to the
supported knobs and shapes) on the GPU."""
import numpy as np
import pytest

from onednn_amd import cabi
from tests import benchdnn_matmul as bd


def test_comma_lists_expand_to_the_cartesian_product():
    mode, specs = bd.parse(["--matmul", "--mode=P", "--dt=u8:s8:s8,s8:s8:f32", "--wtag=ab,ba",
                            "--attr-scales=src:common:0.25+wei:per_oc", "10x30:30x20", "2x30:30x47"])
    assert mode == "P" and len(specs) == 8
    assert {s.dt for s in specs} == {"u8:s8:s8", "s8:s8:f32"} and {s.wtag for s in specs} == {"ab", "ba"}
    assert "--attr-scales=src:common:0.25+wei:per_oc" in specs[0].repro()


def test_problem_construction_follows_the_knobs():
    _, (sp,) = bd.parse(["--dt=bf16:u4:bf16", "--attr-scales=wei:per_ocic:bf16:32x1",
                         "--attr-zero-points=wei:per_ocic:u4:32x1", "--attr-fpmath=bf16:true", "6x96:96x64"])
    p = bd.build_problem(sp)
    assert (p.M, p.K, p.N) == (6, 96, 64) and p.apply_to_int and p.fpmath_mode == 1
    sc, zp = p.quant["wei_scale"], p.quant["wei_zp"]
    assert sc.dt == cabi.DT_BF16 and sc.mask == 6 and sc.groups == (32, 1) and sc.data.size == 3 * 64
    assert zp.dt == cabi.DT_U4 and zp.data.size == 3 * 64 // 2
    _, (sp,) = bd.parse(["--dt=u8:s8:f32", "--bia-dt=f32", "--attr-zero-points=src:common:1+wei:common:-1",
                         "--attr-post-ops=relu+add:f32:per_oc+sum:0.5", "10x30:30x20"])
    p = bd.build_problem(sp)
    assert p.quant["src_zp"].data.view(np.int32)[0] == 1 and p.quant["wei_zp"].data.view(np.int32)[0] == -1
    assert [o.kind for o in p.post_ops] == [cabi.PO_ELTWISE, cabi.PO_BINARY, cabi.PO_SUM]
    assert p.post_ops[1].stride == (0, 0, 1) and p.post_ops[2].scale == 0.5 and p.dst_init is not None


def test_fill_values_are_exact_in_every_type(oracle):
    # the driver's premise: data the types hold exactly, so the checks can be tight
    for name, dt in bd.DT.items():
        if name in ("e8m0", "s32"):
            continue
        lo, hi = bd.value_range(dt)
        vals = np.arange(lo, hi + 1, dtype=np.float32)
        back = oracle.load_float(dt, bd.encode(dt, vals), len(vals))
        assert np.array_equal(back, vals), name


# Adapted from tests/benchdnn/inputs/matmul/test_matmul_int8 (scales, zero
# points, post-ops, weights decompression, tags), option_set_fp8_mixed (int4
# decompression with 2-D grouped scales / zero points) and test_matmul_fp8.
LINES = [
    "--dt=u8:s8:s8,s8:s8:f32 --wtag=ab,ba --bia-dt=undef,f32 10x30:30x20 64x256:256x64",
    "--dt=u8:s8:s8,s8:s8:f32 --attr-scales=src:common:0.25+wei:common:0.5+dst:common:4 --attr-post-ops=sum 10x30:30x20",
    "--dt=u8:s8:s8 --wtag=ab,ba --attr-scales=src:common:0.25+wei:per_oc+dst:common:4 --attr-post-ops=relu "
    "10x30:30x20 300x128:128x260",
    "--dt=s8:s8:s32 --stag=ba --wtag=ab,ba --bia-dt=f32 --attr-scales=src:common:1.25,wei:per_oc,dst:common:0.5 "
    "--attr-post-ops=add:f32,sum+mul:s32:per_oc+linear:2:-1 10x30:30x20",
    "--dt=s8:s8:s8,s8:s8:s32,u8:s8:f32 --attr-zero-points=src:common:1+wei:common:-1+dst:common:2,"
    "src:common:-1+wei:common:1 10x30:30x20 256x192:192x256",
    "--dt=f32:s8:f32,bf16:s8:bf16 --attr-fpmath=bf16:true --attr-scales=wei:common:1.25:f32,wei:per_oc:bf16 "
    "--attr-zero-points=wei:common:-1:s8,wei:per_oc:u8 10x30:30x20",
    "--dt=u8:s8:s32,s8:s8:s32 --stag=ab,ba,any --wtag=ab,ba,any --dtag=ab,any 10x30:30x20 256x64:64x256",
    "--dt=bf16:s4:bf16,bf16:u4:bf16 --attr-scales=wei:per_ocic:bf16:32x1 --attr-zero-points=wei:per_ocic:s4:32x1 "
    "--attr-fpmath=bf16:true 6x96:96x64 1x4096:4096x512 8x1024:1024x768",
    "--dt=bf16:u4:f32 --attr-scales=wei:per_ocic:f32:128x1 --attr-zero-points=wei:per_ocic:u8:128x1,wei:common:2:s32 "
    "--attr-fpmath=bf16:true 32x2048:2048x512",
    "--dt=f8_e4m3:f8_e4m3:bf16,f8_e5m2:f8_e4m3:f32 --wtag=ab,ba --bia-dt=bf16 "
    "--attr-scales=src:common:0.5+wei:common:0.25 --attr-post-ops=,relu+add:bf16 48x128:128x80 256x512:512x256",
    "--dt=f4_e2m1:f4_e2m1:bf16 --wtag=ba --attr-scales=src:per_tensor:e8m0:1x32+wei:per_tensor:e8m0:32x1 "
    "64x256:256x96 256x512:512x256",
    # runtime dims: tests/benchdnn/inputs/matmul/test_matmul_all:4-25 and the int8 / decompression analogues
    "--dt=f32 --wtag=ab,ba --runtime_dims_masks=0,2:1,1:0,3:1 --bia-dt=undef,f32 "
    "--attr-scales=src:common:0.25+wei:per_oc+dst:common:4 --attr-post-ops=relu 10x30:30x20",
    "--dt=f32 --stag=ba --wtag=ab,ba --runtime_dims_masks=3:1,3:3 --bia-dt=f32 "
    "--attr-scales=src:common:0.25+wei:common:0.5+dst:common:4 --attr-post-ops=add:f32,sum+mul:s32:per_oc+linear:2:-1 "
    "10x30:30x20",
    "--dt=u8:s8:s8,s8:s8:f32 --wtag=ab,ba --runtime_dims_masks=1:0,3:3 --bia-dt=undef,f32 "
    "--attr-scales=src:common:0.25+wei:per_oc+dst:common:4 --attr-zero-points=,src:common:1+dst:common:2 "
    "10x30:30x20 300x128:128x260",
    "--dt=bf16:u4:bf16 --runtime_dims_masks=1:0 --attr-scales=wei:per_ocic:bf16:32x1 --attr-zero-points=wei:per_ocic:u4:32x1 "
    "--attr-fpmath=bf16:true 1x4096:4096x512 8x1024:1024x768",
    # dynamic dst quantization: harness_matmul_generated_ci:17,186,344,397 (2-D analogues)
    "--dt=f8_e5m2:f8_e5m2:f4_e2m1,f4_e2m1:f4_e2m1:f4_e2m1 --wtag=ab,ba "
    "--attr-scales=src:per_tensor:e8m0:1x32+wei:per_oc:f32+dst:dynamic_fp:f8_e4m3:1x16 --attr-post-ops=,clip:-0.25:1.0 "
    "76x288:288x352 1x64:64x2032",
    "--dt=f8_e4m3:f8_e4m3:f8_e4m3,f8_e4m3:f8_e4m3:f4_e2m1 --bia-dt=f32 "
    "--attr-scales=src:common:0.5+wei:common:0.25+dst:dynamic_mx:e8m0:1x32 --attr-post-ops=,relu 48x128:128x96",
    "--dt=f8_e4m3:f8_e4m3:bf16 --wtag=ba --runtime_dims_masks=3:3 --bia-dt=bf16 --attr-scales=src:common:0.5+wei:common:0.25 "
    "--attr-post-ops=relu+add:bf16 256x512:512x256",
]


@pytest.mark.gpu
@pytest.mark.parametrize("line", LINES, ids=[f"line{i}" for i in range(len(LINES))])
def test_reference_input_lines(gpu, oracle, line):
    mode, specs = bd.parse(line.split())
    assert specs
    ran = 0
    for sp in specs:
        status, impl, det = bd.run_spec(sp, "C")
        assert status != "FAILED", f"{sp.repro()} via {impl}: {det}"
        ran += status == "PASSED"
    assert ran, "every problem of the line was skipped"


@pytest.mark.gpu
def test_every_fast_family_is_reached_and_agrees_with_the_generic_kernel(gpu, oracle):
    # the same problems through the best implementation and through hip:ref:any
    seen = set()
    for line in ("--dt=u8:s8:s8 --wtag=ba --attr-scales=wei:per_oc --attr-post-ops=relu 256x128:128x256",
                 "--dt=f8_e4m3:f8_e4m3:bf16 --wtag=ba 256x128:128x256",
                 "--dt=bf16:u4:bf16 --attr-scales=wei:per_ocic:bf16:64x1 --attr-fpmath=bf16:true 4x512:512x256"):
        _, (sp,) = bd.parse(line.split())
        status, impl, det = bd.run_spec(sp, "C")
        assert status == "PASSED", (sp.repro(), det)
        seen.add(impl.split(":")[1])
        sp.impl = "ref"
        status, impl_ref, det = bd.run_spec(sp, "C")
        assert status == "PASSED" and impl_ref == "hip:ref:any", (sp.repro(), det)
    assert seen == {"mfma_i8", "mfma_f8", "woq_gemv"}
