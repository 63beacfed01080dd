"""The benchdnn-style driver: parsing and problem construction on the CPU, the
reference's own input lines (tests/benchdnn/inputs/matmul/*, adapted to the
supported knobs and shapes) on the GPU."""
import os

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
    # dropout: harness_matmul_smoke_ref:119, harness_matmul_generated_ci:302,335,417,484 (2-D analogues); stochastic
    # rounding of dst
    "--dt=f32 --bia-dt=undef,f32 --attr-post-ops=,relu --attr-dropout=0.5:12345678 10x30:30x20",
    "--dt=f32 --attr-scales=src:common:2:f32 --attr-dropout=0.25:275507:any:660341:false 1x64:64x484",
    "--dt=f32 --stag=ba --wtag=ba --attr-dropout=0.25:137415:undef:0:false,1:519230:any:0:false 1x921:921x1556",
    "--dt=f8_e5m2:f8_e5m2:bf16 --attr-scales=src:common:0.5+wei:per_oc --attr-post-ops=clip:-0.5:8 "
    "--attr-dropout=0.1:760263:undef:0:false 24x512:512x96",
    "--dt=f32:f32:bf16,bf16:bf16:f16,f32:f32:f8_e4m3 --attr-rounding-mode=dst:stochastic "
    "--attr-dropout=,0.5:77:any:5000000000 10x30:30x20",
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


# ---- buffers from files and the performance report (CPU: parsing, files, the oracle)
C1_LINE = ("--matmul --dt=u8:s8:f32 --stag=ab --wtag=ab --dtag=ab --bia-dt=f32 --bia_mask=2 "
           "--attr-scales=src:common:0.02+wei:per_oc --attr-zero-points=src:common:128 256x1024:1024x1024")


def test_buffer_prefix_round_trip_reproduces_dst(tmp_path, oracle):
    """--export-buffers writes PREFIX.<execution argument id>.bin for every filled
    buffer of the u8 x s8 -> f32 benchmark line (256x1024:1024x1024); --buffer-prefix on a problem generated from
    another seed brings back the same bytes and the same dst (fill.cpp:489-543)."""
    _, specs = bd.parse(C1_LINE.split())
    assert len(specs) == 1
    p = bd.build_problem(specs[0], seed=7)
    prefix = str(tmp_path / "bufs" / "cfg1")
    names = bd.export_buffers(p, prefix)
    # src, weights, bias, src scale, weights scale, src zero point
    assert sorted(int(n.split(".")[-2]) for n in names) == [1, 33, 41, 4097, 4129, 8193]
    sizes = {int(n.split(".")[-2]): os.path.getsize(n) for n in names}
    assert sizes == {1: 256 * 1024, 33: 1024 * 1024, 41: 4096, 4097: 4, 4129: 4096, 8193: 4}
    want = oracle.run_oracle(p)

    q = bd.build_problem(specs[0], seed=99)
    assert not np.array_equal(q.src, p.src) and not np.array_equal(q.wei, p.wei)
    done, err = bd.import_buffers(q, prefix)
    assert err is None and done == [1, 33, 41, 4097, 4129, 8193]
    for arg, (holder, attr) in bd.buffer_ids(q).items():
        h0, a0 = bd.buffer_ids(p)[arg]
        assert np.array_equal(np.asarray(getattr(holder, attr)).view(np.uint8).reshape(-1),
                              np.asarray(getattr(h0, a0)).view(np.uint8).reshape(-1)), arg
    got = oracle.run_oracle(q)
    assert np.array_equal(np.asarray(got).view(np.uint32), np.asarray(want).view(np.uint32))


def test_buffer_prefix_partial_and_mismatched_files(tmp_path):
    _, specs = bd.parse("--dt=s8:s8:s32 --attr-post-ops=add:f32+sum 10x30:30x20".split())
    p = bd.build_problem(specs[0])
    prefix = str(tmp_path / "x")
    names = bd.export_buffers(p, prefix)
    # src, weights, dst (the sum's input), the tensor of binary post-op 0
    assert sorted(int(n.split(".")[-2]) for n in names) == [1, 17, 33, 32770]
    # only src present: the rest keeps the generated data
    for n in names:
        if not n.endswith(".1.bin"):
            os.remove(n)
    q = bd.build_problem(specs[0], seed=3)
    wei_before = q.wei.copy()
    done, err = bd.import_buffers(q, prefix)
    assert err is None and done == [1]
    assert np.array_equal(q.src, p.src) and np.array_equal(q.wei, wei_before)
    # a file of the wrong size fails the case
    with open(f"{prefix}.33.bin", "wb") as f:
        f.write(b"\0" * 7)
    done, err = bd.import_buffers(bd.build_problem(specs[0]), prefix)
    assert err is not None and "differs in size" in err


def test_run_wide_knobs_do_not_multiply_the_problem_list():
    settings = dict(bd.SETTINGS)
    mode, specs = bd.parse(("--mode=P --perf-template=perf,%engine%,%impl%,%prb%,%-time% --buffer-prefix=/tmp/a/b "
                            "--max-ms-per-prb=50 --dt=u8:s8:f32,s8:s8:s32 10x30:30x20").split(), settings)
    assert mode == "P" and len(specs) == 2
    assert settings["buffer_prefix"] == "/tmp/a/b" and settings["max_ms_per_prb"] == "50"
    assert settings["perf_template"] == "perf,%engine%,%impl%,%prb%,%-time%"


def test_perf_template_fields_and_modifiers():
    """doc/knobs_perf_report.md: a custom template, the default one, time and unit modifiers."""
    _, specs = bd.parse(C1_LINE.split())
    sp = specs[0]
    det = {"min_ms": 0.5, "avg_ms": 1.0, "max_ms": 2.0, "ops": 2.0 * 256 * 1024 * 1024, "ibytes": 3e6, "obytes": 1e6,
           "cpd_ms": 1.5, "cp_ms": 2.5}
    T = "perf,%engine%,%impl%,%prb%,%-time%,%0time%,%-Gflops%,%0Gflops%,%-Gbw%"
    line = bd.perf_line(T, sp, "hip:mfma_i8:gfx950", det)
    f = line.split(",")
    assert f[:3] == ["perf", "gpu", "hip:mfma_i8:gfx950"]
    assert f[3] == sp.repro() and "256x1024:1024x1024" in f[3]
    assert [float(x) for x in f[4:]] == pytest.approx([0.5, 1.0, det["ops"] / 0.5e-3 / 1e9, det["ops"] / 1e-3 / 1e9,
                                                       4e6 / 0.5e-3 / 1e9], rel=1e-5)
    d = bd.perf_line("def", sp, "impl", det).split(",")
    assert d[0] == "perf" and d[3] == "" and float(d[5]) == pytest.approx(det["ops"] / 1e9, rel=1e-5)
    assert float(d[6]) == 4.0                                     # %+ctime%
    assert bd.perf_line("%+time%|%Kops%|%Miobytes%|%driver%|%idx%|%wtag%|%unknown%", sp, "i", det, idx=4) == \
        f"2|{det['ops'] / 1e3:g}|4|matmul|4|ab|%unknown%"


def test_cold_cache_knob_is_run_wide_and_checked():
    settings = dict(bd.SETTINGS)
    mode, specs = bd.parse("--mode=P --cold-cache=wei --dt=s8:s8:s32 10x30:30x20".split(), settings)
    assert len(specs) == 1 and settings["cold_cache"] == "wei"
    assert bd.cold_cache_sets({}, "none") == [{}]
    with pytest.raises(ValueError):
        bd.cold_cache_sets({}, "lukewarm")


@pytest.mark.gpu
@pytest.mark.parametrize("cc", ["wei", "all"])
def test_cold_cache_rotates_over_copies_and_leaves_the_result_alone(gpu, oracle, cc, capsys, monkeypatch):
    """tests/benchdnn/utils/cold_cache.hpp:28-45: the timed executions run on copies of the weights (or of every
    argument); the correctness pass and its verdict are those of the warm run."""
    monkeypatch.setattr(bd, "COLD_CACHE_BYTES", 8 << 20)          # a handful of copies is enough for the test
    line = "--matmul --dt=s8:s8:s8 --wtag=any --attr-scales=src:common:0.5+wei:per_oc 1024x1024:1024x1024"
    settings = dict(bd.SETTINGS, cold_cache=cc, max_ms_per_prb="50")
    _, specs = bd.parse(line.split())
    status, impl, det = bd.run_spec(specs[0], "CP", max_ms=50.0, settings=settings)
    assert status == "PASSED" and impl.startswith("hip:mfma_i8") and det["errors"] == 0
    assert det["cold_cache_buffers"] >= (8 if cc == "wei" else 2) and det["min_ms"] > 0
    assert bd.main(line.split() + ["--mode=P", f"--cold-cache={cc}", "--max-ms-per-prb=20"]) == 0
    assert any(ln.startswith("perf,") for ln in capsys.readouterr().out.splitlines())


@pytest.mark.gpu
def test_main_with_buffer_files_and_a_custom_perf_template(gpu, oracle, tmp_path, capsys):
    """The 256x1024:1024x1024 benchmark line end to end: export, then correctness + performance on
    the imported bytes with a custom report template."""
    prefix = str(tmp_path / "cfg1")
    assert bd.main(C1_LINE.split() + [f"--export-buffers={prefix}", "--mode=C"]) == 0
    capsys.readouterr()
    T = "--perf-template=perf,%engine%,%impl%,%prb%,%-time%,%0time%,%-Gflops%,%0Gflops%,%-Gbw%"
    assert bd.main(C1_LINE.split() + [f"--buffer-prefix={prefix}", "--mode=CP", "--max-ms-per-prb=50", T]) == 0
    out = capsys.readouterr().out.splitlines()
    perf = [ln for ln in out if ln.startswith("perf,")]
    assert len(perf) == 1
    f = perf[0].split(",")
    assert f[1] == "gpu" and f[2].startswith("hip:mfma_i8") and "256x1024:1024x1024" in f[3]
    tmin, tavg, gmin, gavg, bw = (float(x) for x in f[-5:])
    assert 0 < tmin <= tavg and gmin >= gavg > 0 and bw > 0
    # a file of the wrong size fails the case
    with open(f"{prefix}.1.bin", "ab") as fh:
        fh.write(b"\0")
    assert bd.main(C1_LINE.split() + [f"--buffer-prefix={prefix}", "--mode=C"]) == 1
    assert "differs in size" in capsys.readouterr().out
