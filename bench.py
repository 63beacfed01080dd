#!/usr/bin/env python3
"""Benchmark of the quantized matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2|c4|c5|c1]

A "step" is one launch of the matmul primitive (through the C ABI,
mi355_matmul_launch) on synthetic, seeded inputs that are resident in HBM
before the timed region starts.  The line printed at the end is one JSON
object: the headline metric of the chosen workload plus

  roofline      the dominant kernel of that workload against the MI355X peak
                that bounds it; the kernel duration is measured here with HIP
                events on the launch stream
  cpu_baseline  the CPU restatement of the reference algorithm (oracle/),
                timed on this machine's host cores on a bounded sample of the
                same workload
  others        the remaining benchmark configurations, measured the same way
                with fewer steps (informational)

Workloads (the benchmark configurations):
  c3  s8 x s8 -> s8, M=N=K=8192, scales + ReLU (MFMA int8 bound)      [default]
  c2  bf16 x u4 -> bf16 decode, K=4096 N=14336, M in {1,8,32} (HBM bound)
  c4  e4m3 x e4m3 -> bf16, 4096 x 8192 x 28672, bias+gelu+add (MFMA fp8 bound)
  c5  MXFP4, M=N=K=8192 (MFMA fp4 bound)
  m1  MXFP8 (e4m3, e8m0 scales per 32 k on both operands), M=N=K=8192 (MFMA fp8 bound)
  h1  bf16 x bf16 -> bf16, M=N=K=8192 (MFMA bf16 bound; the unquantized matmul on the same tiles)
  h2  f32 x f32 -> f32, M=N=K=8192 (MFMA f32 bound)
  c1  u8 x s8 -> f32, 256 x 1024 x 1024 (latency bound, no roofline claim)
Among the side workloads of a default run, p2 is C2's tensors at prefill sizes (M = 512 / 2048): the step includes
the decompression of the 4-bit weights into the bf16 copy the tiles read (MFMA bf16 bound).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

# `traffic` comes from the rocprofv3 summaries under profiles/ (two --pmc passes,
# FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for the
# plain copy kernel moving a known 256 MiB).  The counters sit behind the L2s:
# they count the bytes that miss them, whether the 256 MB memory-side cache or
# HBM then serves them.  Every summary carries the line "Bytes that miss the L2s
# per launch ...: N", which is read here, so that the figure in the JSON line can
# only be as old as the committed profile it names.
PROFILE_OF = {
    ("c3", "any"): "i8_gemm_kernel_c3_8192.md", ("c4", "any"): "f8_gemm_kernel_c4_4096x8192x28672.md",
    ("c5", "any"): "mxf4_gemm_kernel_c5_8192.md", ("c1", "any"): "i8_small_kernel_c1_256x1024x1024.md",
    ("h1", "any"): "f8_gemm_kernel_h1_bf16_8192.md", ("h2", "any"): "f8_gemm_kernel_h2_f32_8192.md",
    ("m1", "any"): "f8_gemm_kernel_m1_mxfp8_8192.md",
    ("c2", "any", 1): "woqp_kernel_c2_m1.md", ("c2", "any", 8): "woqp_kernel_c2_m8.md",
    ("c2", "any", 32): "woqp_kernel_c2_m32.md", ("c2", "ab", 1): "woq_gemv_kernel_c2_m1_plain_ab.md",
    ("c2", "ab", 8): "woq_gemv_kernel_c2_m8_plain_ab.md", ("c2", "ab", 32): "woq_gemv_kernel_c2_m32_plain_ab.md",
    ("r1", "any"): "reorder_rows_kernel_r1_f32_s8_8192.md", ("r2", "any"): "transpose8w_kernel_r2_s8_transpose_8192.md",
    ("r3", "any"): "pack_woq64_kernel_r3_u4_4096x14336.md",
    ("g1", "any"): "grouped_nsplit_kernel_g1_deepseek_v3_prefill.md",
    ("g2", "any"): "grouped_nsplit_kernel_g2_llama4_scout_prefill.md",
    ("g3", "any"): "grouped_tile_kernel_g3_deepseek_v3_decode.md",
    ("g4", "any"): "grouped_nsplit_kernel_g4_deepseek_v3_prefill_mxfp8.md",
    ("g5", "any"): "grouped_nsplit_kernel_g5_deepseek_v3_prefill_mxfp4.md",
    ("g6", "any"): "grouped_k_lds_kernel_g6_llama4_scout_weights_gradient.md",
}


def measured_traffic(name, wtag="any", M=None):
    """(bytes per launch, profile file) from the committed summary, or (None, None)."""
    import re
    key = (name, wtag, M) if name == "c2" else (name, "any")
    fn = PROFILE_OF.get(key)
    if not fn:
        return None, None
    path = os.path.join(ROOT, "profiles", fn)
    try:
        m = re.search(r"(?:Bytes that miss the L2s|HBM bytes) per launch[^:\n]*:\s*([0-9,]+)", open(path).read())
    except OSError:
        return None, None
    return (int(m.group(1).replace(",", "")), "profiles/" + fn) if m else (None, "profiles/" + fn)


# MI355X published peaks
PEAK_HBM_GBS = 8000.0
PEAK_I8_TOPS = 5000.0
PEAK_F8_TFLOPS = 5000.0
PEAK_F4_TFLOPS = 10100.0
PEAK_BF16_TFLOPS = 2500.0
PEAK_F32_TFLOPS = 157.3


# the MFMA instruction each compute-bound workload runs on (index into the calibration kernel's table)
CEILING_INSTR = {"c3": 1, "c1": 1, "c4": 2, "m1": 2, "c5": 5, "h1": 7, "h2": 8}


def measured_ceiling(lib, name):
    """What the workload's MFMA instruction sustains by itself on this box, now, with random operand bits
    (registers only: tests/calib/calib_kernels.hip), in the workload's unit; for the decode workload the rate of a
    read-only kernel with the decode kernel's access shape over the same 29.4 MB of weights.  None when the
    calibration library is not built."""
    from onednn_amd import cabi
    path = os.path.join(ROOT, "tests", "bin", "libmi355_calib.so")
    if not os.path.exists(path):
        return None
    cl = C.CDLL(path)
    vp = C.c_void_p
    timer = Timer(lib)
    if name == "c2":
        cl.mi355_calib_read_stream.argtypes = [vp, C.c_size_t, vp, vp]
        nbytes = 4096 * 14336 // 2
        bufs = [cabi.DeviceBuffer(nbytes) for _ in range(12)]
        sink = cabi.DeviceBuffer(4096)
        idx = [0]

        def step():
            cl.mi355_calib_read_stream(bufs[idx[0] % 12].ptr, C.c_size_t(nbytes), sink.ptr, None)
            idx[0] += 1

        timer.time_ms(step, 2000)
        ms = min(timer.time_ms(step, 200) for _ in range(3))
        for b in bufs:
            b.free()
        return {"value": nbytes / (ms * 1e-3) / 1e9, "unit": "GB/s",
                "what": "read-only kernel with the decode kernel's access shape over the same weights, per launch"}
    instr = CEILING_INSTR.get(name)
    if instr is None:
        return None
    cl.mi355_calib_mfma_rate.argtypes = [C.c_int, C.c_int, vp, vp, C.POINTER(C.c_double), vp]
    h = np.random.default_rng(1).integers(0, 2**32, size=4096, dtype=np.uint64).astype(np.uint32)
    if instr in (2, 3):
        h &= np.uint32(0x3f3f3f3f)
    elif instr in (6, 7):
        h &= np.uint32(0x3fff3fff)
    elif instr == 8:
        h &= np.uint32(0x3fffffff)
    bits, out = cabi.DeviceBuffer.from_numpy(h), cabi.DeviceBuffer(1 << 20)
    ops = C.c_double(0)

    def step():
        cl.mi355_calib_mfma_rate(instr, 20000, out.ptr, bits.ptr, C.byref(ops), None)

    step()
    cabi.check(lib.mi355_stream_sync(None))
    ms = min(timer.time_ms(step, 1) for _ in range(3))
    bits.free()
    out.free()
    return {"value": ops.value / (ms * 1e-3) / 1e12, "unit": "TFLOP/s",
            "what": "the kernel's MFMA instruction by itself, registers only, random operand bits"}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class Timer:
    """HIP events on the stream the kernels are launched on."""

    def __init__(self, lib, stream=None):
        self.lib, self.stream = lib, stream
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        from onednn_amd import cabi
        cabi.check(lib.mi355_event_create(C.byref(self.e0)))
        cabi.check(lib.mi355_event_create(C.byref(self.e1)))

    def time_ms(self, fn, iters):
        from onednn_amd import cabi
        cabi.check(self.lib.mi355_stream_sync(self.stream))
        cabi.check(self.lib.mi355_event_record(self.e0, self.stream))
        for _ in range(iters):
            fn()
        cabi.check(self.lib.mi355_event_record(self.e1, self.stream))
        cabi.check(self.lib.mi355_event_sync(self.e1))
        ms = C.c_float()
        cabi.check(self.lib.mi355_event_elapsed_ms(C.byref(ms), self.e0, self.e1))
        return ms.value / iters


def build_problem(name, M=None, wtag="any"):
    """`any` is what weights format_tag::any resolves to in the primitive
    descriptor: K-contiguous (ba) for the MFMA operand types, row-major (ab)
    for the int4 decode weights.  With an explicit `ab` the MFMA families run
    a layout pre-pass inside every launch, which then is part of the step."""
    from onednn_amd import cabi, configs
    if name == "c1":
        return configs.config1(wtag="ba" if wtag == "any" else wtag)
    if name == "c2":
        p = configs.config2(M=M or 1, wtag="ab" if wtag == "any" else wtag)
        if wtag == "any":  # what format_tag::any resolves to for decode weights
            p.wei_packing = cabi.WEI_PACK_WOQ64
        return p
    if name == "p2":  # C2's tensors at prefill size: the weights are decompressed into a bf16 copy inside every launch
        return configs.config2(M=M or 2048, wtag="ab" if wtag == "any" else wtag)
    mfma_tag = "ba" if wtag == "any" else wtag
    if name == "c3":
        return configs.config3(wtag=mfma_tag)
    if name == "c4":
        return configs.config4(wtag=mfma_tag)
    if name == "c4mx":
        # C4 with an MXFP8 dst: e4m3 values and e8m0 scales per 32 columns, computed and written by the matmul
        import numpy as np
        from onednn_amd.problem import QuantParam
        p = configs.config4(wtag=mfma_tag)
        p.dst_dt = cabi.DT_F8_E4M3
        p.quant["dst_scale"] = QuantParam(cabi.DT_E8M0, 6, np.zeros((1, p.M, p.N // 32), np.uint8), (1, 32))
        p.dst_dynamic = cabi.DST_DYNAMIC_MX
        p.name = "C4-dynamic-mx-dst"
        return p
    if name == "c4g":
        # C4's tensors as the gated feed-forward layer of the Llama family: swish in place of gelu_tanh, the bf16
        # tensor multiplied in place of the residual add
        p = configs.config4(wtag=mfma_tag)
        for po in p.post_ops:
            if po.kind == cabi.PO_ELTWISE:
                po.alg, po.alpha = cabi.ELTWISE["swish"], 1.0
            if po.kind == cabi.PO_BINARY:
                po.alg = cabi.BINARY["mul"]
        p.name = "C4-swish-gate"
        return p
    if name == "c5":
        return configs.config5(wtag=mfma_tag)
    if name == "h1":
        return configs.config_h16(wtag=mfma_tag)
    if name == "h2":
        return configs.config_h16(dt="f32", wtag=mfma_tag)
    if name == "m1":
        return configs.config_mxf8(wtag=mfma_tag)
    raise ValueError(name)


def algorithmic(name, p):
    """(work per launch, unit of the rate, roofline bound, peak)."""
    from onednn_amd import configs
    ops = 2.0 * p.batch * p.M * p.N * p.K
    if name == "c2":
        return configs.config2_bytes(p.M, p.N, p.K), "GB/s", "hbm", PEAK_HBM_GBS
    if name == "c3":
        return ops, "TOPS", "mfma", PEAK_I8_TOPS
    if name in ("c4", "c4mx", "c4g", "m1"):
        return ops, "TFLOP/s", "mfma", PEAK_F8_TFLOPS
    if name == "c5":
        return ops, "TFLOP/s", "mfma", PEAK_F4_TFLOPS
    if name in ("h1", "p2"):
        return ops, "TFLOP/s", "mfma", PEAK_BF16_TFLOPS
    if name == "h2":
        return ops, "TFLOP/s", "mfma", PEAK_F32_TFLOPS
    return ops, "TOPS", "mfma", PEAK_I8_TOPS


def rate(work, ms, unit):
    if unit == "GB/s":
        return work / (ms * 1e-3) / 1e9
    return work / (ms * 1e-3) / 1e12


GRAPH_REPLAY = True   # decode launches also timed as replays of a HIP graph (main() clears it under a profiler)


def run_gpu_workload(lib, name, steps, warmup, M=None, cold_copies=0, wtag="any", sustained_s=0.0):
    """Returns dict with ms_per_step, value, unit, impl.

    Before the warm-up steps the workload is launched back to back for about
    0.4 s, untimed: after an idle period the device needs a few hundred
    milliseconds of load before its clocks settle, and a timed region of a few
    milliseconds taken right after start-up measures that ramp rather than the
    kernel (the same launches measured 0.56 ms each in the first 10, 0.51 over
    30 and 0.46 over 300).  With sustained_s > 0 the workload is afterwards
    launched back to back for at least that many seconds, timed in chunks:
    `sustained` = average and best chunk."""
    from onednn_amd import cabi
    from onednn_amd.problem import GpuRun
    t0 = time.time()
    p = build_problem(name, M, wtag)
    log(f"[bench] {name}: generated {p.name} in {time.time() - t0:.1f}s")
    # decode runs on a created stream: its launches are also timed as replays of a HIP graph (below)
    stream = cabi.Stream() if name == "c2" else None
    sp = stream.ptr if stream else None
    runs = [GpuRun(p, stream=sp)]
    # decode is HBM-bound only if the weights are not already in the 256 MB
    # last-level cache: rotate over enough weight copies to exceed it
    for _ in range(cold_copies):
        runs.append(GpuRun(p, stream=sp))
    timer = Timer(lib, sp)
    idx = [0]

    def step():
        runs[idx[0] % len(runs)].launch()
        idx[0] += 1

    t_pre = time.time()
    while time.time() - t_pre < 0.4:     # settle the clocks (untimed)
        for _ in range(20):
            step()
        cabi.check(lib.mi355_stream_sync(sp))
    for _ in range(max(warmup, 1)):
        step()
    ms = timer.time_ms(step, steps)
    work, unit, bound, peak = algorithmic(name, p)
    graph = None
    if stream is not None and GRAPH_REPLAY:
        # The same `steps` launches (over the same rotation of weight copies) recorded once and replayed: what a
        # serving loop does with a step that is a few microseconds of kernel behind a few microseconds of launch.
        with cabi.Graph(stream) as g:
            for _ in range(steps):
                step()
        for _ in range(3):
            g.launch()
        reps = max(3, 2000 // steps)
        ms_g = timer.time_ms(g.launch, reps) / steps
        g.destroy()
        graph = {"ms_per_step": ms_g, "value": rate(work, ms_g, unit), "unit": unit, "launches_per_graph": steps,
                 "replays_timed": reps}
    sustained = None
    if sustained_s > 0:
        chunk = max(20, int(0.1 / max(ms * 1e-3, 1e-6)))      # ~0.1 s of launches per chunk
        chunks, t_s = [], time.time()
        while time.time() - t_s < sustained_s or len(chunks) < 3:
            chunks.append(timer.time_ms(step, chunk))
        sustained = {"seconds": round(time.time() - t_s, 2), "launches": chunk * len(chunks),
                     "ms_per_step_avg": sum(chunks) / len(chunks), "ms_per_step_min": min(chunks),
                     "value_avg": rate(work, sum(chunks) / len(chunks), unit), "value_best": rate(work, min(chunks), unit),
                     "unit": unit}
    out = {
        "workload": p.name, "impl": cabi.impl_name(runs[0].impl), "ms_per_step": ms,
        "value": rate(work, ms, unit), "unit": unit, "bound": bound, "peak": peak, "work": work,
        "shape": [p.M, p.K, p.N], "sustained": sustained, "graph": graph,
    }
    for r in runs:
        r.free()
    if stream is not None:
        stream.destroy()
    return out, p


def run_reorder_workloads(lib, steps, which=("r1", "r2", "r3")):
    """Informational: the reorder primitive on the tensors of the headline
    shape (HBM-bound; bytes = src + dst + parameter tensors)."""
    import numpy as np
    from onednn_amd import cabi
    from onednn_amd.problem import QuantParam
    from onednn_amd.reorder import GpuReorder, ReorderProblem
    N = 8192
    rng = np.random.default_rng(7)
    x8 = rng.integers(-128, 128, size=(N, N), dtype=np.int8)
    xf = rng.standard_normal((N, N)).astype(np.float32)
    sc = rng.uniform(0.5, 2, size=N).astype(np.float32)
    plan = {
        "r1": (ReorderProblem(dims=(N, N), src_dt=cabi.DT_F32, dst_dt=cabi.DT_S8, src=xf,
                              quant={"dst_scale": QuantParam(cabi.DT_F32, 2, sc)},
                              name="R1 f32->s8 8192x8192, per-column dst scales"), 5 * N * N + 4 * N),
        "r2": (ReorderProblem(dims=(N, N), src_dt=cabi.DT_S8, dst_dt=cabi.DT_S8, src=x8, dst_stride=(1, N),
                              name="R2 s8 8192x8192 ab->ba (weights into the layout format_tag::any resolves to)"),
               2 * N * N),
    }
    if "r3" in which:
        import ctypes as C
        K3, N3 = 4096, 14336
        d = cabi.ReorderDesc()
        cabi.check(lib.mi355_wei_pack_reorder_dims(cabi.WEI_PACK_WOQ64, K3, N3, N3, 1, C.byref(d)))
        w4 = rng.integers(0, 256, size=K3 * N3 // 2, dtype=np.uint8)
        plan["r3"] = (ReorderProblem(dims=tuple(d.dims[i] for i in range(6)), src_dt=cabi.DT_U4, dst_dt=cabi.DT_U4,
                                     src=w4, src_stride=tuple(d.src_stride[i] for i in range(6)),
                                     dst_stride=tuple(d.dst_stride[i] for i in range(6)),
                                     name="R3 u4 4096x14336 ab -> packed decode layout (what format_tag::any resolves to)"),
                      K3 * N3)
    out = []
    timer = Timer(lib)
    for key in which:
        p, nbytes = plan[key]
        r = GpuReorder(p)
        r.launch()
        ms = timer.time_ms(r.launch, steps)
        gbs = nbytes / (ms * 1e-3) / 1e9
        out.append({"workload": p.name, "impl": "hip:reorder:any", "ms_per_step": ms, "value": gbs, "unit": "GB/s",
                    "bound": "hbm", "peak": PEAK_HBM_GBS, "frac_of_peak": gbs / PEAK_HBM_GBS, "work": nbytes})
        log(f"[bench] {p.name}: {ms:.4f} ms -> {gbs:.1f} GB/s ({100 * gbs / PEAK_HBM_GBS:.1f}% of hbm peak) "
            "via hip:reorder:any")
        for b in r.bufs.values():
            b.free()
    return out


def run_grouped_workloads(lib, steps, which=("g1", "g2", "g3", "g4", "g5", "g6")):
    """The grouped (mixture-of-experts) matmul on shapes of the reference's
    shapes_grouped_moe files: fp8 e4m3 operands, a scale per src row and per
    group and column, bf16 dst.  HBM-bound: the weights of every group with
    rows are read once.  Two copies of every tensor alternate between launches
    so that the smaller shapes do not run out of the 256 MB last-level cache."""
    import numpy as np
    from onednn_amd import cabi, configs
    from onednn_amd.grouped import fill_args
    out = []
    timer = Timer(lib)
    for key in which:
        t0 = time.time()
        p = configs.grouped_k_config() if key == "g6" else configs.grouped_config(key)
        d = p.desc()
        cabi.check(lib.mi355_grouped_matmul_query(C.byref(d)))
        copies = 1 if p.wei.nbytes > (1 << 30) else 3
        sets, bufs = [], []
        for _ in range(copies):
            def place(arr):
                b = cabi.DeviceBuffer.from_numpy(np.ascontiguousarray(arr))
                bufs.append(b)
                return b.ptr
            a = fill_args(p, place)
            dst = cabi.DeviceBuffer(p.initial_dst().nbytes)
            bufs.append(dst)
            a.dst = dst.ptr
            sets.append(a)
        log(f"[bench] {key}: generated and uploaded {p.name} in {time.time() - t0:.1f}s")
        idx = [0]

        def step():
            cabi.check(lib.mi355_grouped_matmul_launch(C.byref(d), C.byref(sets[idx[0] % copies]), None))
            idx[0] += 1

        t_pre = time.time()
        while time.time() - t_pre < 0.4:     # settle the clocks (untimed), as for the other workloads
            for _ in range(20):
                step()
            cabi.check(lib.mi355_stream_sync(None))
        for _ in range(3):
            step()
        ms = timer.time_ms(step, steps)
        nbytes = configs.grouped_bytes(p)
        gbs = nbytes / (ms * 1e-3) / 1e9
        impl = lib.mi355_grouped_matmul_impl(C.byref(d)).decode()
        out.append({"workload": p.name, "impl": impl, "ms_per_step": ms, "value": gbs, "unit": "GB/s", "bound": "hbm",
                    "peak": PEAK_HBM_GBS, "frac_of_peak": gbs / PEAK_HBM_GBS, "work": nbytes,
                    "tflops": 2.0 * p.total * (p.M if key == "g6" else p.K) * p.N / (ms * 1e-3) / 1e12})
        log(f"[bench] {p.name}: {ms:.4f} ms -> {gbs:.1f} GB/s ({100 * gbs / PEAK_HBM_GBS:.1f}% of hbm peak) via {impl}")
        for b in bufs:
            b.free()
    return out


def grouped_cpu_baseline(name):
    """The oracle's restatement of ref_grouped_t on the first groups and columns of the workload."""
    from oracle import binding as oracle
    from onednn_amd import configs
    groups, N = {"g1": (16, 256), "g2": (2, 256), "g3": (64, 256), "g4": (16, 256), "g5": (16, 256), "g6": (2, 256)}[name]
    p = configs.grouped_k_config(groups=groups, M=1024, N=N) if name == "g6" else configs.grouped_config(name, groups=groups, N=N)
    oracle.load()
    reps, t0 = 0, time.time()
    while True:
        st, _ = oracle.run_oracle_grouped(p)
        assert st == 0
        reps += 1
        dt = time.time() - t0
        if dt >= 10.0 or reps >= 200:
            break
    from onednn_amd import configs as cf
    return {"value": cf.grouped_bytes(p) * reps / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"the first {groups} groups and {N} columns of the workload ({p.total} rows"
                      f"{' along K, 1024 rows of dst' if name == 'g6' else ''}); {reps} pass(es), "
                      f"{dt:.2f} s wall; oracle/liboracle.so, oracle_grouped_matmul (plain C restatement of "
                      "ref_grouped_t, one thread)"}


def cpu_baseline(name, M=None):
    """The oracle timed on a bounded sample of the same workload."""
    from oracle import binding as oracle
    from onednn_amd import configs
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    threads = min(threads, 16)
    os.environ["OMP_NUM_THREADS"] = str(threads)
    if name == "c3":
        p = configs.config3(M=512, N=1024, K=8192)
        sample = "M=512, N=1024, K=8192 slice of the 8192^3 problem shape"
    elif name == "c2":
        p = configs.config2(M=M or 1, N=14336, K=4096)
        sample = f"full problem M={p.M}, K=4096, N=14336"
    elif name == "c4":
        p = configs.config4(M=128, N=1024, K=8192)
        sample = "M=128, N=1024, K=8192 slice of the 4096x8192x28672 shape"
    elif name == "c5":
        p = configs.config5(M=128, N=1024, K=8192)
        sample = "M=128, N=1024, K=8192 slice of the 8192^3 shape"
    elif name == "m1":
        p = configs.config_mxf8(M=128, N=1024, K=8192)
        sample = "M=128, N=1024, K=8192 slice of the 8192^3 shape"
    elif name in ("h1", "h2"):
        p = configs.config_h16(M=128, N=1024, K=8192, dt="f32" if name == "h2" else "bf16")
        sample = "M=128, N=1024, K=8192 slice of the 8192^3 shape"
    else:
        p = configs.config1()
        sample = "full problem 256x1024x1024"
    oracle.load()
    # repeat the sample until about ten seconds of CPU work have been timed
    reps, t0 = 0, time.time()
    while True:
        oracle.run_oracle(p)
        reps += 1
        dt = time.time() - t0
        if dt >= 10.0 or reps >= 200:
            break
    work, unit, _, _ = algorithmic(name, p)
    # the reference's own optimized CPU path (brg_matmul, JIT) cannot be built on this machine; what it measured
    # where it could be built is quoted so that the port's number is not read as the reference's speed
    probe = {"c3": "4.97 TOPS (221 ms)", "c1": "6.37 TOPS (0.084 ms)",
             "c2": {1: "4.17 GB/s (7.05 ms)", 8: "4.64 GB/s (6.39 ms)", 32: "3.16 GB/s (9.67 ms)"}.get(M or 1),
             "c4": "no JIT implementation on that host (ref:any only)", "c5": "no CPU implementation (skipped)",
             "h1": "not measured", "h2": "not measured",
             "m1": "no CPU implementation (skipped)"}[name]
    return {"value": rate(work * reps, dt * 1e3, unit), "unit": unit, "cores": threads, "kind": "port",
            "reference_probe": {"what": "benchdnn --matmul --mode=P on the reference built with its own CMake, "
                                        "impl brg_matmul:avx10_1_512_amx, this configuration at full size",
                                "value": probe, "hardware": "8 vCPU Intel Xeon (Sapphire Rapids class, AMX), "
                                                            "OMP_NUM_THREADS=8; another machine, not this run"},
            "sample": sample + f"; {reps} pass(es), {dt:.2f} s wall; oracle/liboracle.so (plain C restatement of "
            "ref_matmul_t / ref_matmul_int8_t, OpenMP over dst rows; the reference itself needs CMake-generated "
            "headers and is not built here)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3", choices=["c1", "c2", "c3", "c4", "c5", "m1", "h1", "h2", "r1", "r2", "r3", "g1", "g2", "g3", "g4", "g5", "g6"],
                    help="c1..c5: the matmul configurations (c3 is the headline); r1..r3: the reorder "
                         "primitive on the headline shape's tensors; g1..g6: the grouped (mixture-of-experts) "
                         "matmul on shapes of the reference's shapes_grouped_moe files: fp8 with row / column scales "
                         "(g1..g3), MXFP8 (g4), MXFP4 (g5), and the variable-K pattern in bf16 (g6) (informational)")
    ap.add_argument("--decode-m", type=int, default=1, help="M of the c2 decode workload")
    ap.add_argument("--wtag", default="any", choices=["any", "ab", "ba"],
                    help="weights layout; any = what format_tag::any resolves to (default)")
    ap.add_argument("--sustained", type=float, default=1.5,
                    help="seconds of back-to-back launches of the headline workload after the timed steps "
                         "(reported as `sustained`; 0 = skip)")
    ap.add_argument("--no-others", action="store_true", help="skip the informational configs")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true",
                    help="skip the HIP-graph replay of the decode launches (skipped by itself under rocprofv3, whose "
                         "kernel tracing was seen to crash inside hipGraphLaunch)")
    ap.add_argument("--no-ceiling", action="store_true",
                    help="skip the measurement of the ceiling (the MFMA instruction / the weight stream by itself): "
                         "profiler runs, where its kernels would show up next to the workload's")
    ap.add_argument("--calib-read", action="store_true",
                    help="time a read-only kernel with the decode kernel's access shape over the C2 weights "
                         "(12 rotating copies, nothing cached) and exit: the floor of the weight stream")
    ap.add_argument("--calib-launch", action="store_true",
                    help="time empty launches of several grid shapes and the decode kernel's skeleton (read the C2 "
                         "weights, sum through LDS, store) and exit: what a launch and the stream cost by themselves")
    ap.add_argument("--calib-pattern", action="store_true",
                    help="time a read-only kernel that streams 256-row slabs the way the grouped matmul tiles do, with "
                         "64, 128, 256 and 1024 contiguous bytes per row and load instruction, over G1's weights "
                         "(3.76 GB) and exit: what the access shape costs by itself")
    ap.add_argument("--calib-mfma", action="store_true",
                    help="time the MFMA instructions of the GEMM kernels by themselves (registers only), with random "
                         "and with constant operand bits, and exit: the ceiling the power manager leaves")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also launch the plain copy kernel on 256 MiB three times: the known-size "
                         "dispatch that FETCH_SIZE / WRITE_SIZE counter passes are scaled by")
    args = ap.parse_args()
    global GRAPH_REPLAY
    if args.no_graph or any(k.startswith("ROCPROF") for k in os.environ):
        GRAPH_REPLAY = False
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU (one-GPU boxes only); "
                 "--gpus must be 1. How the path would shard is described in the design notes; it is not built.")

    from onednn_amd import cabi
    lib = cabi.load_kernels()  # raises if the HIP library is missing: no fallback
    n = C.c_int(0)
    cabi.check(lib.mi355_device_count(C.byref(n)))
    if n.value < 1:
        sys.exit("bench.py: no HIP device visible")
    cabi.check(lib.mi355_device_set(0))
    name = C.create_string_buffer(64)
    cus, khz = C.c_int(), C.c_int()
    hbm, l2 = C.c_int64(), C.c_int64()
    cabi.check(lib.mi355_device_info(0, name, 64, C.byref(cus), C.byref(khz), C.byref(hbm),
                                     C.byref(l2)))
    log(f"[bench] device {name.value.decode()} CUs={cus.value} clock={khz.value / 1e3:.0f} MHz "
        f"HBM={hbm.value / 2**30:.0f} GiB")

    main_name = args.workload

    def calib_lib():
        """the measurement kernels (tests/bin/libmi355_calib.so, built by tests/Makefile)"""
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests", "bin", "libmi355_calib.so")
        if not os.path.exists(path):
            sys.exit(f"bench.py: {path} is missing: build it with `make -C tests`")
        cl = C.CDLL(path)
        vp = C.c_void_p
        cl.mi355_calib_copy.argtypes = [vp, vp, C.c_size_t, vp]
        cl.mi355_calib_empty.argtypes = [C.c_int, C.c_int, vp]
        cl.mi355_calib_read_stream.argtypes = [vp, C.c_size_t, vp, vp]
        cl.mi355_calib_read_reduce.argtypes = [vp, C.c_size_t, vp, vp]
        cl.mi355_calib_read_pattern.argtypes = [vp, C.c_int64, C.c_int64, C.c_int, vp, vp]
        cl.mi355_calib_mfma_rate.argtypes = [C.c_int, C.c_int, vp, vp, C.POINTER(C.c_double), vp]
        return cl

    def ok(rc):
        if rc != 0:
            raise RuntimeError(f"calibration kernel refused its arguments or failed to launch ({rc})")

    if args.calib_launch:
        # what a launch costs by itself, and what the decode kernel's skeleton (read 128 KB per workgroup, meet in
        # LDS, store 64 values) costs over the C2 weights: back-to-back launches, HIP events around 200 of them
        cl = calib_lib()
        nbytes = 4096 * 14336 // 2
        bufs = [cabi.DeviceBuffer(nbytes) for _ in range(12)]
        out = cabi.DeviceBuffer(256 * (nbytes // (128 << 10)))
        timer, idx, rows = Timer(lib), [0], []

        def pre(step):
            t_pre = time.time()
            while time.time() - t_pre < 0.3:
                for _ in range(50):
                    step()
                cabi.check(lib.mi355_stream_sync(None))

        for label, blocks, threads in (("empty launch, 1 x 64", 1, 64), ("empty launch, 224 x 1024", 224, 1024),
                                       ("empty launch, 224 x 512", 224, 512), ("empty launch, 1024 x 256", 1024, 256)):
            def step():
                ok(cl.mi355_calib_empty(blocks, threads, None))
            pre(step)
            runs = [timer.time_ms(step, 200) for _ in range(5)]
            rows.append({"kernel": label, "us_avg": 1e3 * sum(runs) / 5, "us_best": 1e3 * min(runs)})
        for label, fn in (("read 29.4 MB, nothing kept", cl.mi355_calib_read_stream),
                          ("read 29.4 MB, sum through LDS, 64 stores per workgroup", cl.mi355_calib_read_reduce)):
            def step():
                ok(fn(bufs[idx[0] % 12].ptr, C.c_size_t(nbytes), out.ptr, None))
                idx[0] += 1
            pre(step)
            runs = [timer.time_ms(step, 200) for _ in range(5)]
            rows.append({"kernel": label, "us_avg": 1e3 * sum(runs) / 5, "us_best": 1e3 * min(runs)})
        for r in rows:
            log(f"[bench] {r['kernel']}: {r['us_avg']:.2f} us per launch (best of 5 x 200: {r['us_best']:.2f})")
        print(json.dumps({"metric": "launch and stream skeleton of the decode kernel", "unit": "us", "rows": rows}),
              flush=True)
        return
    if args.calib_pattern:
        cl = calib_lib()
        K, slabs = 7168, 2048
        buf, sink = cabi.DeviceBuffer(K * 256 * slabs), cabi.DeviceBuffer(4096)
        cabi.check(lib.mi355_mem_set(buf.ptr, 1, C.c_size_t(K * 256 * slabs), None))
        timer, rows = Timer(lib), []
        for run in (64, 128, 256, 1024):
            def step():
                ok(cl.mi355_calib_read_pattern(buf.ptr, slabs, K, run, sink.ptr, None))
            timer.time_ms(step, 20)
            ms = min(timer.time_ms(step, 10) for _ in range(3))
            gbs = K * 256 * slabs / (ms * 1e-3) / 1e9
            rows.append({"run_bytes": run, "rows_per_instruction": 1024 // run, "ms": ms, "GBps": gbs})
            log(f"[bench] {1024 // run:2d} rows x {run:4d} B per load instruction: {ms:.4f} ms -> {gbs:.0f} GB/s")
        print(json.dumps({"metric": "row streaming by access shape", "unit": "GB/s", "bytes": K * 256 * slabs,
                          "rows": rows}), flush=True)
        return
    if args.calib_read:
        cl = calib_lib()
        nbytes = 4096 * 14336 // 2
        bufs = [cabi.DeviceBuffer(nbytes) for _ in range(12)]
        sink = cabi.DeviceBuffer(4096)
        timer, idx = Timer(lib), [0]

        def step():
            ok(cl.mi355_calib_read_stream(bufs[idx[0] % 12].ptr, C.c_size_t(nbytes), sink.ptr, None))
            idx[0] += 1

        t_pre = time.time()
        while time.time() - t_pre < 0.4:
            for _ in range(50):
                step()
            cabi.check(lib.mi355_stream_sync(None))
        runs = [timer.time_ms(step, max(args.steps, 200)) for _ in range(5)]
        ms = sum(runs) / len(runs)
        log(f"[bench] read_stream_kernel over {nbytes} bytes (C2 weights), 12 rotating copies: "
            f"{ms * 1e3:.2f} us/launch avg of 5 x {max(args.steps, 200)}, best {min(runs) * 1e3:.2f} us -> "
            f"{nbytes / (ms * 1e-3) / 1e9:.0f} GB/s")
        print(json.dumps({"metric": "read floor of the C2 weight stream", "value": nbytes / (ms * 1e-3) / 1e9,
                          "unit": "GB/s", "us_per_launch": ms * 1e3, "us_best": min(runs) * 1e3, "bytes": nbytes}),
              flush=True)
        return

    if args.calib_mfma:
        cl = calib_lib()
        names = ["v_mfma_i32_32x32x32_i8", "v_mfma_i32_16x16x64_i8", "v_mfma_f32_32x32x64_f8f6f4 (fp8)",
                 "v_mfma_f32_16x16x128_f8f6f4 (fp8)", "v_mfma_scale_f32_32x32x64_f8f6f4 (fp4)",
                 "v_mfma_scale_f32_16x16x128_f8f6f4 (fp4)", "v_mfma_f32_32x32x16_bf16", "v_mfma_f32_16x16x32_bf16",
                 "v_mfma_f32_32x32x2_f32"]
        out = cabi.DeviceBuffer(1 << 20)
        rng = np.random.default_rng(1)
        rows = []
        for instr, name in enumerate(names):
            row = {"instruction": name}
            for kind in ("random", "constant"):
                h = rng.integers(0, 2**32, size=4096, dtype=np.uint64).astype(np.uint32) if kind == "random" \
                    else np.full(4096, 0x01010101, np.uint32)
                if "fp8" in name:     # finite, moderate values: clear sign and top exponent bit
                    h &= np.uint32(0x3f3f3f3f)
                elif "bf16" in name:
                    h &= np.uint32(0x3fff3fff)
                elif "_f32" in name and "x2_" in name:
                    h &= np.uint32(0x3fffffff)
                bits = cabi.DeviceBuffer.from_numpy(h)
                ops = C.c_double(0)
                timer = Timer(lib)

                def step():
                    ok(cl.mi355_calib_mfma_rate(instr, 20000, out.ptr, bits.ptr, C.byref(ops), None))

                step()
                cabi.check(lib.mi355_stream_sync(None))
                ms = min(timer.time_ms(step, 1) for _ in range(3))
                row[kind] = ops.value / (ms * 1e-3) / 1e12
                bits.free()
            rows.append(row)
            log(f"[bench] {name}: {row['random']:.0f} T(FL)OP/s with random operand bits, {row['constant']:.0f} with "
                "constant ones")
        print(json.dumps({"metric": "MFMA rate, registers only", "unit": "TOPS", "rows": rows}), flush=True)
        return

    def calib_copy():
        cl = calib_lib()
        nbytes = 256 << 20
        a, b = cabi.DeviceBuffer(nbytes), cabi.DeviceBuffer(nbytes)
        for _ in range(3):
            ok(cl.mi355_calib_copy(b.ptr, a.ptr, C.c_size_t(nbytes), None))
        cabi.check(lib.mi355_stream_sync(None))
        a.free()
        b.free()

    if main_name in ("r1", "r2", "r3"):
        r = run_reorder_workloads(lib, args.steps, (main_name,))[0]
        if args.calib_copy:
            calib_copy()
        print(json.dumps({
            "metric": "reorder GB/s", "value": r["value"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": {"r1": "f32", "r2": "s8", "r3": "u4"}[main_name], "data": "synthetic",
            "config": {"workload": r["workload"], "impl": r["impl"]},
            "roofline": {"bound": "hbm", "achieved": r["value"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": r["frac_of_peak"], "traffic": measured_traffic(main_name)[0],
                         "traffic_source": measured_traffic(main_name)[1], "algorithmic": r["work"],
                         "kernel": r["impl"], "kernel_ms": r["ms_per_step"]},
            "cpu_baseline": None, "others": []}), flush=True)
        return
    if main_name in ("g1", "g2", "g3", "g4", "g5", "g6"):
        r = run_grouped_workloads(lib, args.steps, (main_name,))[0]
        if args.calib_copy:
            calib_copy()
        cpu = None if args.no_cpu else grouped_cpu_baseline(main_name)
        print(json.dumps({
            "metric": "grouped %s matmul GB/s" % {"g4": "MXFP8", "g5": "MXFP4", "g6": "bf16 variable-K"}.get(main_name, "fp8"), "value": r["value"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": {"g5": "f4_e2m1", "g6": "bf16"}.get(main_name, "f8_e4m3"), "data": "synthetic",
            "config": {"workload": r["workload"], "impl": r["impl"], "tflops": r["tflops"]},
            "roofline": {"bound": "hbm", "achieved": r["value"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": r["frac_of_peak"], "traffic": measured_traffic(main_name)[0],
                         "traffic_source": measured_traffic(main_name)[1], "algorithmic": r["work"],
                         "kernel": r["impl"], "kernel_ms": r["ms_per_step"]},
            "cpu_baseline": cpu, "others": []}), flush=True)
        return
    cold = 11 if main_name == "c2" else 0
    res, prob = run_gpu_workload(lib, main_name, args.steps, args.warmup, args.decode_m, cold,
                                 args.wtag, sustained_s=args.sustained)
    log(f"[bench] {res['workload']}: {res['ms_per_step']:.4f} ms/step -> {res['value']:.1f} "
        f"{res['unit']} via {res['impl']}")
    if res.get("graph"):
        log(f"[bench] the same as a HIP graph of {res['graph']['launches_per_graph']} launches: "
            f"{res['graph']['ms_per_step']:.4f} ms/step -> {res['graph']['value']:.1f} {res['graph']['unit']}")

    if args.calib_copy:
        calib_copy()

    # The timed step is one launch whose time is dominated by one kernel (the
    # tile GEMM / the decode kernel); the small kernels of the same launch (the
    # split-K reduction of the decode path, column sums, the layout change of
    # `ab` weights when --wtag ab is forced) are part of the measured step and
    # therefore of `achieved`: it never flatters the dominant kernel.
    traffic, traffic_source = measured_traffic(main_name, "any" if args.wtag == "any" else "ab", prob.M)
    roofline = {
        "bound": res["bound"], "achieved": res["value"], "peak": res["peak"],
        "unit": "GB/s" if res["unit"] == "GB/s" else "TFLOP/s",
        "frac": res["value"] / res["peak"], "traffic": traffic, "traffic_source": traffic_source,
        "algorithmic": res["work"], "kernel": res["impl"], "kernel_ms": res["ms_per_step"],
    }
    # next to the published peak: what this box's matrix cores (or, for decode, its memory system) deliver to a
    # kernel that does nothing else -- `frac` stays priced against the published peak
    ceil = None if args.no_ceiling else measured_ceiling(lib, main_name)
    if ceil:
        roofline["ceiling"] = ceil["value"]
        roofline["ceiling_what"] = ceil["what"]
        roofline["frac_of_ceiling"] = res["value"] / ceil["value"]
        log(f"[bench] ceiling: {ceil['value']:.0f} {ceil['unit']} ({ceil['what']}) -> {100 * roofline['frac_of_ceiling']:.1f}% of it")

    others = []
    if not args.no_others:
        # (workload, M, weights tag); "ab" = row-major weights as in the reference's benchdnn line for C3: the
        # layout change then runs inside every launch
        plan = [("c2", 1, "any"), ("c2", 8, "any"), ("c2", 32, "any"), ("c2", 1, "ab"), ("c2", 8, "ab"), ("c2", 32, "ab"),
                ("c3", None, "any"), ("c3", None, "ab"),
                ("c4", None, "any"), ("c4mx", None, "any"), ("c4g", None, "any"), ("c5", None, "any"), ("c1", None, "any"),
                ("m1", None, "any"), ("h1", None, "any"), ("h2", None, "any"), ("p2", 512, "any"), ("p2", 2048, "any")]
        for nm, m, wt in plan:
            if nm == main_name and wt == args.wtag and (nm != "c2" or m == args.decode_m):
                continue
            try:
                r, _ = run_gpu_workload(lib, nm, max(5, args.steps // 2) if nm != "c2" else 200, 2, m,
                                        11 if nm == "c2" else 0, wt)
                r["frac_of_peak"] = r["value"] / r["peak"]
                if wt != "any":
                    r["workload"] += f" (weights tag {wt})"
                r["algorithmic"] = r["work"]
                # the layout pre-pass of row-major weights is not in the committed counter passes of the GEMMs
                r["traffic"], r["traffic_source"] = measured_traffic(nm, wt, m) if (nm == "c2" or wt == "any") else (None, None)
                others.append({k: r[k] for k in ("workload", "impl", "ms_per_step", "value", "unit",
                                                 "bound", "peak", "frac_of_peak", "algorithmic", "traffic",
                                                 "traffic_source")})
                if r.get("graph"):
                    others[-1]["graph_replay"] = r["graph"]
                log(f"[bench] {r['workload']}: {r['ms_per_step']:.4f} ms -> {r['value']:.1f} "
                    f"{r['unit']} ({100 * r['frac_of_peak']:.1f}% of {r['bound']} peak) via {r['impl']}"
                    + (f"; as a HIP graph of {r['graph']['launches_per_graph']} launches {r['graph']['ms_per_step']:.4f} ms"
                       if r.get("graph") else ""))
            except Exception as e:  # a failing side workload must not hide the headline
                others.append({"workload": f"{nm}-M{m}" if m else nm, "error": str(e)})
                log(f"[bench] {nm}: failed: {e}")

        try:
            others += run_reorder_workloads(lib, max(5, args.steps // 2))
        except Exception as e:
            others.append({"workload": "reorder", "error": str(e)})
            log(f"[bench] reorder: failed: {e}")
        try:
            others += run_grouped_workloads(lib, max(5, args.steps // 2))
        except Exception as e:
            others.append({"workload": "grouped", "error": str(e)})
            log(f"[bench] grouped: failed: {e}")

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(main_name, args.decode_m)
        log(f"[bench] cpu baseline: {cpu['value']:.4f} {cpu['unit']} on {cpu['cores']} threads")

    metric = {"c3": "int8 matmul TOPS @8192^3", "c2": "int4 weight-only decode GB/s",
              "c4": "fp8 matmul TFLOP/s @4096x8192x28672", "c5": "MXFP4 matmul TFLOP/s @8192^3",
              "c1": "int8 matmul TOPS @256x1024x1024", "h1": "bf16 matmul TFLOP/s @8192^3", "h2": "f32 matmul TFLOP/s @8192^3",
              "m1": "MXFP8 matmul TFLOP/s @8192^3"}[main_name]
    dtype = {"c3": "s8", "c2": "bf16", "c4": "f8_e4m3", "c5": "f4_e2m1", "c1": "u8", "h1": "bf16", "h2": "f32", "m1": "f8_e4m3"}[main_name]
    line = {
        "metric": metric, "value": res["value"], "unit": res["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": res["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype,
        "data": "synthetic",
        "config": {"workload": res["workload"], "shape_MKN": res["shape"], "impl": res["impl"],
                   "weights_layout": args.wtag},
        "roofline": roofline, "sustained": res["sustained"], "cpu_baseline": cpu, "others": others,
    }
    if res.get("graph"):
        line["graph_replay"] = res["graph"]
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
