#!/usr/bin/env python3
"""A matmul driver with benchdnn's command-line vocabulary.

    python tests/benchdnn_matmul.py --matmul [--mode=C|P|CP] --dt=u8:s8:f32 --wtag=ba \\
        --bia-dt=f32 --attr-scales=src:common:0.25+wei:per_oc --attr-zero-points=src:common:1 \\
        --attr-post-ops=relu+add:f32 256x1024:1024x1024

What it mirrors of the reference's harness (tests/benchdnn/matmul/matmul.cpp,
doc/knobs_attr.md): the knob syntax, comma lists expanding to the cartesian
product of problems, data filled with small integers and power-of-two scales
so that every product and partial sum is exact in f32 (fill_data :576-661,
fill.cpp:161-199), correctness against a naive reference (here the CPU oracle
under oracle/) and a perf mode that reports min / avg time of back-to-back
executions.  The library is driven through its dnnl_* C API exactly like a
user would: engine, memory descriptors, attributes, primitive descriptor,
primitive, execute.

Test infrastructure: the correctness mode needs the oracle, which the product
package never imports.

Buffers from files (tests/benchdnn/utils/fill.cpp:489-543, doc/knobs_common.md
"--buffer-prefix"): --buffer-prefix=PREFIX fills every buffer for which the
file PREFIX.<execution argument id>.bin exists with that file's bytes instead
of generated data (a file whose size differs from the buffer's fails the
case, as in the reference); --export-buffers=PREFIX writes the generated
buffers under those names, so that the reference's benchdnn can be run on the
bytes this driver ran on.  Ids: src 1, weights 33, bias 41, dst 17 (the sum
post-op's input), scales 4096 + arg, zero points 8192 + arg, the tensor of
binary post-op i 32768 * (i + 1) + 2.

Performance report (doc/knobs_perf_report.md): --perf-template=def | csv |
CUSTOM with the %engine% %impl% %name% %prb% %desc% %driver% %idx% %attr%
%stag% %wtag% %dtag% %bia_dt% fields and the measured %time% %ops% %flops%
%ibytes% %obytes% %iobytes% %bw% %ctime% %cpdtime% %cptime% (%clocks% and
%freq% print 0) with the time modifiers - 0 + and the unit modifiers K M G.

Supported knobs: --dt, --stag, --wtag, --dtag (ab | ba | any), --bia-dt,
--attr-scales, --attr-zero-points, --attr-post-ops, --attr-fpmath, --attr-dropout, --attr-rounding-mode, --impl,
--mode, --buffer-prefix, --export-buffers, --perf-template, --max-ms-per-prb, --cold-cache (none | wei | all),
and 2-D problem descriptors MxK:KxN.  Policies: common, per_oc,
per_ocic (with GxH groups), per_tensor (with GxH groups), per_dim_0, per_dim_1.
"""
import itertools
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

from onednn_amd import cabi, dnnl  # noqa: E402
from onednn_amd import dtypes as dtp  # noqa: E402
from onednn_amd.problem import MatmulProblem, PostOp, QuantParam, storage_dtype, strides_for  # noqa: E402

DT = {"f32": cabi.DT_F32, "bf16": cabi.DT_BF16, "f16": cabi.DT_F16, "s32": cabi.DT_S32, "s8": cabi.DT_S8,
      "u8": cabi.DT_U8, "s4": cabi.DT_S4, "u4": cabi.DT_U4, "f8_e4m3": cabi.DT_F8_E4M3,
      "f8_e5m2": cabi.DT_F8_E5M2, "f4_e2m1": cabi.DT_F4_E2M1, "e8m0": cabi.DT_E8M0}
MASK_ROW, MASK_COL = 2, 4  # bit 0 is the batch dimension of the thin C ABI


def encode(dt, values):
    """Logical values (small integers, exactly representable) -> raw storage of `dt`."""
    v = np.asarray(values, dtype=np.float32)
    if dt == cabi.DT_F32:
        return v
    if dt == cabi.DT_BF16:
        return dtp.f32_to_bf16(v)
    if dt == cabi.DT_F16:
        return v.astype(np.float16).view(np.uint16)
    if dt == cabi.DT_S32:
        return v.astype(np.int32)
    if dt == cabi.DT_S8:
        return v.astype(np.int8)
    if dt == cabi.DT_U8:
        return v.astype(np.uint8)
    if dt in (cabi.DT_S4, cabi.DT_U4):
        return dtp.pack_nibbles((v.astype(np.int32) & 0xF).astype(np.uint8))
    if dt == cabi.DT_F8_E4M3:
        return dtp.f32_to_e4m3(v)
    if dt == cabi.DT_F8_E5M2:
        # the fill values have at most two significant bits: e5m2 is the top byte of their f16 form
        return (v.astype(np.float16).view(np.uint16) >> 8).astype(np.uint8)
    if dt == cabi.DT_F4_E2M1:
        return dtp.pack_nibbles(dtp.f32_to_e2m1_codes(v))
    if dt == cabi.DT_E8M0:
        return dtp.f32_to_e8m0(v)
    raise ValueError(dt)


def value_range(dt):
    """Fill range per data type: small integers every type represents exactly."""
    if dt in (cabi.DT_U8, cabi.DT_U4):
        return 0, 8
    if dt == cabi.DT_F4_E2M1:
        return -2, 2
    return -4, 4


class Spec:
    """One fully specified problem (one element of the cartesian product)."""

    def __init__(self, **kw):
        self.__dict__.update(kw)

    def repro(self):
        parts = ["--matmul", f"--dt={self.dt}", f"--stag={self.stag}", f"--wtag={self.wtag}", f"--dtag={self.dtag}"]
        if self.bia_dt != "undef":
            parts.append(f"--bia-dt={self.bia_dt}")
        for knob in ("attr_scales", "attr_zero_points", "attr_post_ops", "attr_fpmath", "attr_dropout",
                     "attr_rounding_mode"):
            if getattr(self, knob):
                parts.append(f"--{knob.replace('_', '-')}={getattr(self, knob)}")
        if self.runtime_dims_masks:
            parts.append(f"--runtime_dims_masks={self.runtime_dims_masks}")
        if self.impl:
            parts.append(f"--impl={self.impl}")
        parts.append(self.desc)
        return " ".join(parts)


# settings of the run, not of a problem (they do not multiply the problem list)
SETTINGS = {"buffer_prefix": "", "export_buffers": "", "perf_template": "def", "max_ms_per_prb": "300",
            "cold_cache": "none"}
# --cold-cache (tests/benchdnn/utils/cold_cache.hpp:28-45, cold_cache.cpp:60-170): the timed executions rotate over
# copies of the weights (`wei`) or of every execution argument (`all`) so that no execution finds them in a cache;
# as many copies as it takes to exceed the caches (here: twice the 256 MB memory-side cache), at least two and at
# most COLD_CACHE_MAX_BUFFERS.
COLD_CACHE_BYTES = 512 << 20
COLD_CACHE_MAX_BUFFERS = 64


def cold_cache_sets(args, mode):
    """The argument dictionaries the timed executions rotate over: `args` itself plus copies of the cold arguments."""
    if mode == "none":
        return [args]
    if mode not in ("wei", "all"):
        raise ValueError(f"unknown --cold-cache mode {mode} (none, wei, all)")
    cold = [k for k in args if (mode == "all" or k == dnnl.ARG_WEIGHTS) and isinstance(args[k], dnnl.memory)]
    size = sum(args[k].md.get_size() for k in cold)
    if size == 0:
        return [args]
    n = max(2, min(COLD_CACHE_MAX_BUFFERS, -(-COLD_CACHE_BYTES // size)))
    sets = [args]
    for _ in range(n - 1):
        s = dict(args)
        for k in cold:
            m = args[k]
            nbytes = m.md.get_size()
            s[k] = dnnl.memory(m.md, m.engine, m.read(np.uint8)[:nbytes] if nbytes else None)
        sets.append(s)
    return sets


def parse(argv, settings=None):
    """benchdnn-style arguments -> (mode, [Spec, ...]); run-wide knobs go into
    `settings` (a dict like SETTINGS) when one is given."""
    knobs = {"dt": ["f32"], "stag": ["ab"], "wtag": ["ab"], "dtag": ["ab"], "bia_dt": ["undef"],
             "attr_scales": [""], "attr_zero_points": [""], "attr_post_ops": [""], "attr_fpmath": [""],
             "attr_dropout": [""], "attr_rounding_mode": [""], "runtime_dims_masks": [""], "impl": [""]}
    mode, specs = "C", []
    for a in argv:
        if a in ("--matmul", "--reset"):
            continue
        if a.startswith("--mode="):
            mode = a.split("=", 1)[1].upper()
            continue
        if a.startswith("--") and a[2:].partition("=")[0].replace("-", "_") in SETTINGS:
            k, _, v = a[2:].partition("=")
            if settings is not None:
                settings[k.replace("-", "_")] = v
            continue
        if a.startswith("--"):
            k, _, v = a[2:].partition("=")
            k = k.replace("-", "_")
            if k == "bia_mask":
                if v not in ("2", ""):
                    raise ValueError("only --bia_mask=2 (1 x N bias) is supported")
                continue
            if k not in knobs:
                raise ValueError(f"unknown knob --{k}")
            knobs[k] = v.split(",") if v else [""]
            continue
        for combo in itertools.product(*knobs.values()):
            specs.append(Spec(desc=a, **dict(zip(knobs.keys(), combo))))
    return mode, specs


def _tag_strides(tag, rows, cols):
    return strides_for("ab" if tag == "any" else tag, 1, rows, cols)


def build_problem(sp, seed=7):
    """Spec -> MatmulProblem with benchdnn-like data."""
    lhs, rhs = sp.desc.split(":")
    M, K = (int(x) for x in lhs.split("x"))
    K2, N = (int(x) for x in rhs.split("x"))
    if K != K2:
        raise ValueError(f"inconsistent K in {sp.desc}")
    dts = sp.dt.split(":")
    if len(dts) == 1:
        dts = dts * 3
    sdt, wdt, ddt = (DT[x] for x in dts)
    rng = np.random.default_rng(seed)

    def ints(dt, shape):
        lo, hi = value_range(dt)
        return rng.integers(lo, hi + 1, size=shape).astype(np.float32)

    wtag = sp.wtag
    if wtag == "any":  # what the primitive descriptor resolves `any` weights to
        mfma = (sdt in (cabi.DT_S8, cabi.DT_U8) and wdt in (cabi.DT_S8, cabi.DT_U8)) or (
            sdt in (cabi.DT_F8_E4M3, cabi.DT_F8_E5M2) and wdt in (cabi.DT_F8_E4M3, cabi.DT_F8_E5M2)) or (
            sdt == wdt == cabi.DT_F4_E2M1)
        wtag = "ba" if mfma else "ab"
    src_v, wei_v = ints(sdt, (M, K)), ints(wdt, (K, N))
    src = encode(sdt, src_v if sp.stag != "ba" else src_v.T.copy())
    wei = encode(wdt, wei_v if wtag != "ba" else wei_v.T.copy())
    kw = dict(src_stride=_tag_strides(sp.stag, M, K), wei_stride=strides_for(wtag, 1, K, N),
              dst_stride=_tag_strides(sp.dtag, M, N))
    if sp.bia_dt != "undef":
        kw["bias_dt"] = DT[sp.bia_dt]
        kw["bias"] = encode(DT[sp.bia_dt], rng.integers(-8, 9, size=N))
    dims = {"src": (M, K), "wei": (K, N), "dst": (M, N)}

    def quant_entry(arg, policy, rest, is_scale):
        value, dt, groups = None, (cabi.DT_F32 if is_scale else cabi.DT_S32), (1, 1)
        for tok in rest:
            if tok in DT:
                dt = DT[tok]
            elif "x" in tok and tok.replace("x", "").isdigit():
                groups = tuple(int(x) for x in tok.split("x"))
            elif tok:
                value = float(tok)
        r, c = dims[arg]
        if policy == "common":
            mask, shape = 0, (1,)
        elif policy in ("per_oc", "per_dim_1"):
            mask, shape = MASK_COL, (c,)
        elif policy == "per_dim_0":
            mask, shape = MASK_ROW, (r,)
        elif policy in ("per_ocic", "per_tensor", "per_dim_01"):
            mask, shape = MASK_ROW | MASK_COL, (r // groups[0], c // groups[1])
        elif policy in ("dynamic_mx", "dynamic_fp"):
            # dst:dynamic_fp:f8_e4m3:1x16 -- the scales are an output of the matmul
            if arg != "dst" or not is_scale:
                raise ValueError("dynamic quantization is a dst scale mode")
            kw["dst_dynamic"] = cabi.DST_DYNAMIC_MX if policy == "dynamic_mx" else cabi.DST_DYNAMIC_FP
            return QuantParam(dt, MASK_ROW | MASK_COL, np.zeros((r // groups[0], c // groups[1]), np.uint8), groups)
        else:
            raise ValueError(f"policy {policy}")
        if value is not None and policy == "common":
            vals = np.full(shape, value, np.float32)
        elif is_scale:
            vals = rng.choice(np.array([0.125, 0.25, 0.5], np.float32), size=shape)
        else:
            lo = 0 if dt in (cabi.DT_U8, cabi.DT_U4) else -2
            vals = rng.integers(lo, 3, size=shape).astype(np.float32)
        return QuantParam(dt, mask, encode(dt, vals), groups)

    quant = {}
    for knob, is_scale, suffix in ((sp.attr_scales, True, "scale"), (sp.attr_zero_points, False, "zp")):
        for ent in filter(None, knob.split("+")):
            arg, policy, *rest = ent.split(":")
            quant[f"{arg}_{suffix}"] = quant_entry(arg, policy, rest, is_scale)
    post_ops, dst_init = [], None
    for ent in filter(None, sp.attr_post_ops.split("+")):
        name, *rest = ent.split(":")
        if name in cabi.ELTWISE:
            alpha = float(rest[0]) if len(rest) > 0 else 0.0
            beta = float(rest[1]) if len(rest) > 1 else 0.0
            post_ops.append(PostOp(kind=cabi.PO_ELTWISE, alg=cabi.ELTWISE[name], alpha=alpha, beta=beta, scale=1.0))
        elif name in cabi.BINARY:
            bdt = DT[rest[0]] if rest else cabi.DT_F32
            policy = rest[1] if len(rest) > 1 else "per_tensor"
            shape, stride = {"per_tensor": ((M, N), (0, N, 1)), "per_oc": ((1, N), (0, 0, 1)),
                             "common": ((1, 1), (0, 0, 0))}[policy]
            post_ops.append(PostOp(kind=cabi.PO_BINARY, alg=cabi.BINARY[name], dt=bdt, stride=stride,
                                   data=encode(bdt, ints(bdt, shape))))
        elif name == "sum":
            post_ops.append(PostOp(kind=cabi.PO_SUM, scale=float(rest[0]) if rest else 1.0))
            dst_init = encode(ddt, ints(ddt, (M, N)))
        else:
            raise ValueError(f"post-op {name}")
    apply_to_int, fpmath = False, 0
    if sp.attr_fpmath:
        mode, _, flag = sp.attr_fpmath.partition(":")
        fpmath = {"strict": 0, "bf16": 1, "f16": 2, "any": 3}[mode]
        apply_to_int = flag == "true"
    impl = {"": cabi.IMPL_AUTO, "ref": cabi.IMPL_REF}.get(sp.impl, cabi.IMPL_AUTO)
    if sp.attr_dropout:
        # PROBABILITY[:SEED[:TAG[:OFFSET[:HOST_SCALARS]]]] (doc/knobs_attr.md "--attr-dropout"); the mask is laid
        # out like dst, so TAG only says whether there is one; host scalars are a property of the dnnl_* layer
        f = sp.attr_dropout.split(":") + [""] * 5
        seed = int(f[1] or 0)
        kw["dropout"] = {"p": float(f[0]), "seed": seed, "seed_s64": not -2 ** 31 <= seed < 2 ** 31,
                         "mask": f[2] != "undef", "offset": int(f[3]) if f[3] else None}
    if sp.attr_rounding_mode:
        # ARG:MODE[+...]; a matmul has dst only
        for item in sp.attr_rounding_mode.split("+"):
            arg, _, rmode = item.partition(":")
            if arg != "dst" or rmode not in ("environment", "stochastic"):
                raise ValueError(f"--attr-rounding-mode={item}")
            kw["dst_stochastic"] = rmode == "stochastic"
    return MatmulProblem(M=M, N=N, K=K, src_dt=sdt, wei_dt=wdt, dst_dt=ddt, src=src, wei=wei, quant=quant,
                         post_ops=post_ops, apply_to_int=apply_to_int, fpmath_mode=fpmath, dst_init=dst_init,
                         impl=impl, name=sp.desc, **kw)


def runtime_masks(text):
    """--runtime_dims_masks=[SRC][:WEI] -> (src, wei, dst) bit masks over (rows, cols);
    the dst mask follows: M from src, N from weights."""
    if not text:
        return 0, 0, 0
    a, _, b = text.partition(":")
    sm, wm = int(a or 0), int(b or 0)
    if (sm >> 1) & 1 != wm & 1:
        raise ValueError("K is a runtime dim in one of src / weights only")
    return sm, wm, (sm & 1) | (wm & 2)


def _pd_md(dims, dt, strides, mask):
    """The descriptor handed to the primitive descriptor: dims under `mask`
    are DNNL_RUNTIME_DIM_VAL, and so is every stride that is a product of one."""
    if not mask:
        return dnnl.memory_desc(list(dims), dt, strides=list(strides))
    R = dnnl.RUNTIME_DIM_VAL
    rt = [bool(mask >> i & 1) for i in range(len(dims))]
    st = [R if any(rt[j] and j != i and strides[j] < strides[i] for j in range(len(dims))) else strides[i]
          for i in range(len(dims))]
    return dnnl.memory_desc([R if rt[i] else dims[i] for i in range(len(dims))], dt, strides=st)


def api_objects(p, want_ref_impl=False, runtime_dims_masks=""):
    """MatmulProblem -> dnnl engine, primitive and execute arguments (2-D, dense)."""
    eng = dnnl.engine(dnnl.gpu, 0)
    strm = dnnl.stream(eng)
    smask, wmask, dmask = runtime_masks(runtime_dims_masks)
    src_md = dnnl.memory_desc([p.M, p.K], p.src_dt, strides=list(p.src_stride[1:]))
    wei_md = dnnl.memory_desc([p.K, p.N], p.wei_dt, strides=list(p.wei_stride[1:]))
    dst_md = dnnl.memory_desc([p.M, p.N], p.dst_dt, strides=list(p.dst_stride[1:]))
    bias_md = dnnl.memory_desc([1, p.N], p.bias_dt, tag=dnnl.tag_ab) if p.bias is not None else None
    attr = dnnl.primitive_attr()
    args = {}
    name_to = {"src": dnnl.ARG_SRC, "wei": dnnl.ARG_WEIGHTS, "dst": dnnl.ARG_DST}
    for qname, q in p.quant.items():
        which, kind = qname.split("_")
        arg, mask2d = name_to[which], q.mask >> 1
        groups = q.groups if q.groups != (1, 1) else ()
        dims = {"src": (p.M, p.K), "wei": (p.K, p.N), "dst": (p.M, p.N)}[which]
        qdims = [dims[0] // q.groups[0] if mask2d & 1 else 1, dims[1] // q.groups[1] if mask2d & 2 else 1]
        if kind == "scale" and which == "dst" and p.dst_dynamic:
            attr.set_scales(arg, mask2d, groups, q.dt, qmode={
                cabi.DST_DYNAMIC_MX: dnnl.quantization_mode_dynamic_mx,
                cabi.DST_DYNAMIC_FP: dnnl.quantization_mode_dynamic_fp}[p.dst_dynamic])
            flag = dnnl.ARG_ATTR_SCALES
        elif kind == "scale":
            attr.set_scales(arg, mask2d, groups, q.dt)
            flag = dnnl.ARG_ATTR_SCALES
        else:
            attr.set_zero_points(arg, mask2d, groups, q.dt)
            flag = dnnl.ARG_ATTR_ZERO_POINTS
        args[flag | arg] = dnnl.memory(dnnl.memory_desc(qdims, q.dt, tag=dnnl.tag_ab), eng, q.data)
    if p.fpmath_mode or p.apply_to_int:
        attr.set_fpmath_mode(p.fpmath_mode, p.apply_to_int)
    if p.dropout is not None:
        dr = p.dropout
        mask_md = dnnl.memory_desc([p.M, p.N], cabi.DT_U8, tag=dnnl.tag_any) if dr.get("mask") else None
        seed_dt, seed_np = (dnnl.s64, np.int64) if dr.get("seed_s64") else (cabi.DT_S32, np.int32)
        attr.set_dropout(mask_md, seed_dt, dr.get("offset") is not None, False)

        def one(dt, v, npdt):
            return dnnl.memory(dnnl.memory_desc([1], dt, tag=dnnl.tag_a), eng, np.asarray([v], npdt))
        args[dnnl.ARG_ATTR_DROPOUT_PROBABILITY] = one(cabi.DT_F32, dr["p"], np.float32)
        args[dnnl.ARG_ATTR_DROPOUT_SEED] = one(seed_dt, dr["seed"], seed_np)
        if dr.get("offset") is not None:
            args[dnnl.ARG_ATTR_DROPOUT_OFFSET] = one(dnnl.s64, dr["offset"], np.int64)
        if dr.get("mask"):
            args[dnnl.ARG_ATTR_DROPOUT_MASK] = dnnl.memory(dnnl.memory_desc([p.M, p.N], cabi.DT_U8, tag=dnnl.tag_ab), eng,
                                                           np.full(p.M * p.N, 0xee, np.uint8))
    if p.dst_stochastic:
        attr.set_rounding(dnnl.ARG_DST, dnnl.rounding_stochastic)
    po = dnnl.post_ops()
    for i, op in enumerate(p.post_ops):
        if op.kind == cabi.PO_ELTWISE:
            po.append_eltwise(op.alg, op.alpha, op.beta)
        elif op.kind == cabi.PO_BINARY:
            bmd = dnnl.memory_desc([p.M if op.stride[1] else 1, p.N if op.stride[2] else 1], op.dt, tag=dnnl.tag_ab)
            po.append_binary(op.alg, bmd)
            args[dnnl.ARG_ATTR_MULTIPLE_POST_OP(i) | dnnl.ARG_SRC_1] = dnnl.memory(bmd, eng, op.data)
        elif op.kind == cabi.PO_SUM:
            po.append_sum(op.scale, op.zero_point, op.dt)
    if p.post_ops:
        attr.set_post_ops(po)
    pd = dnnl.matmul_primitive_desc(
        eng, _pd_md([p.M, p.K], p.src_dt, p.src_stride[1:], smask), _pd_md([p.K, p.N], p.wei_dt, p.wei_stride[1:], wmask),
        _pd_md([p.M, p.N], p.dst_dt, p.dst_stride[1:], dmask),
        bias_md=_pd_md([1, p.N], p.bias_dt, (p.N, 1), dmask & 2) if bias_md else None, attr=attr)
    if want_ref_impl and not (smask or wmask):
        while pd.impl_info_str() != "hip:ref:any":
            if not pd.next_impl():
                raise RuntimeError("no hip:ref:any implementation in the list")
    prim = dnnl.matmul(pd)
    args[dnnl.ARG_SRC] = dnnl.memory(src_md, eng, p.src)
    args[dnnl.ARG_WEIGHTS] = dnnl.memory(wei_md, eng, p.wei)
    dst = dnnl.memory(dst_md, eng, p.initial_dst())
    args[dnnl.ARG_DST] = dst
    if p.bias is not None:
        args[dnnl.ARG_BIAS] = dnnl.memory(bias_md, eng, p.bias)
    return pd, prim, strm, args, dst


def buffer_ids(p):
    """{execution argument id: (holder object, attribute name)} of the buffers of a
    problem that benchdnn fills (dnnl_types.h: DNNL_ARG_*)."""
    ids = {dnnl.ARG_SRC: (p, "src"), dnnl.ARG_WEIGHTS: (p, "wei")}
    if p.bias is not None:
        ids[dnnl.ARG_BIAS] = (p, "bias")
    if p.dst_init is not None:
        ids[dnnl.ARG_DST] = (p, "dst_init")
    arg_of = {"src": dnnl.ARG_SRC, "wei": dnnl.ARG_WEIGHTS, "dst": dnnl.ARG_DST}
    for qname, q in p.quant.items():
        which, kind = qname.split("_")
        if which == "dst" and kind == "scale" and p.dst_dynamic:
            continue  # an output
        ids[(dnnl.ARG_ATTR_SCALES if kind == "scale" else dnnl.ARG_ATTR_ZERO_POINTS) | arg_of[which]] = (q, "data")
    for i, op in enumerate(p.post_ops):
        if op.kind == cabi.PO_BINARY:
            ids[dnnl.ARG_ATTR_MULTIPLE_POST_OP(i) | dnnl.ARG_SRC_1] = (op, "data")
    return ids


def export_buffers(p, prefix):
    """PREFIX.<id>.bin for every filled buffer, the bytes the library is handed."""
    names = []
    os.makedirs(os.path.dirname(os.path.abspath(prefix)), exist_ok=True)
    for arg, (holder, attr) in sorted(buffer_ids(p).items()):
        name = f"{prefix}.{arg}.bin"
        np.ascontiguousarray(getattr(holder, attr)).view(np.uint8).reshape(-1).tofile(name)
        names.append(name)
    return names


def import_buffers(p, prefix):
    """Fills the buffers whose files exist; returns (imported ids, error or None).
    A size mismatch is an error (fill.cpp:514-523)."""
    done = []
    for arg, (holder, attr) in sorted(buffer_ids(p).items()):
        name = f"{prefix}.{arg}.bin"
        if not os.path.exists(name):
            continue
        cur = np.ascontiguousarray(getattr(holder, attr))
        raw = np.fromfile(name, dtype=np.uint8)
        if raw.size != cur.nbytes:
            return done, (f"file '{name}' differs in size from the buffer's memory descriptor: "
                          f"actual {raw.size}, needed {cur.nbytes}")
        setattr(holder, attr, raw.view(cur.dtype).reshape(cur.shape))
        done.append(arg)
    return done, None


PERF_TEMPLATES = {
    "def": "perf,%engine%,%impl%,%name%,%prb%,%Gops%,%+ctime%,%-time%,%-Gflops%,%0time%,%0Gflops%",
    "csv": "perf,%engine%,%impl%,%name%,%driver%,%stag%,%wtag%,%dtag%,%bia_dt%,%attr%,%desc%,%Gops%,%+ctime%,"
           "%-time%,%-Gflops%,%0time%,%0Gflops%",
}


def perf_line(template, sp, impl, det, idx=0):
    """One report line: `template` with its %...% fields replaced
    (doc/knobs_perf_report.md; parser of tests/benchdnn/utils/perf_report.cpp)."""
    template = PERF_TEMPLATES.get(template, template)
    attr = " ".join(f"--{k.replace('_', '-')}={getattr(sp, k)}" for k in
                    ("attr_scales", "attr_zero_points", "attr_post_ops", "attr_fpmath") if getattr(sp, k))
    plain = {"engine": "gpu", "impl": impl, "name": "", "prb": sp.repro(), "desc": sp.desc, "driver": "matmul",
             "idx": str(idx), "attr": attr, "stag": sp.stag, "wtag": sp.wtag, "dtag": sp.dtag, "bia_dt": sp.bia_dt,
             "cfg": "", "dt": sp.dt, "dir": "", "mb": "0"}
    times = {"-": det["min_ms"], "0": det["avg_ms"], "+": det["max_ms"]}
    units = {"": 1.0, "K": 1e3, "M": 1e6, "G": 1e9}

    def field(m):
        tok = m.group(1)
        if tok in plain:
            return plain[tok]
        mm = re.fullmatch(r"([-0+]?)([KMG]?)(time|clocks|freq|ibytes|obytes|iobytes|bw|ops|flops|cpdtime|cptime|ctime)", tok)
        if not mm:
            return m.group(0)
        mod, unit, what = mm.groups()
        t_ms = times[mod or "-"]
        if what == "time":
            v = t_ms
        elif what in ("clocks", "freq"):
            v = 0.0
        elif what in ("ibytes", "obytes", "iobytes"):
            v = {"ibytes": det["ibytes"], "obytes": det["obytes"], "iobytes": det["ibytes"] + det["obytes"]}[what]
        elif what == "bw":
            v = (det["ibytes"] + det["obytes"]) / (t_ms * 1e-3)
        elif what == "ops":
            v = det["ops"]
        elif what == "flops":
            v = det["ops"] / (t_ms * 1e-3)
        else:  # creation times: one creation is measured, every modifier reports it
            v = {"cpdtime": det["cpd_ms"], "cptime": det["cp_ms"], "ctime": det["cpd_ms"] + det["cp_ms"]}[what]
        return f"{v / units[unit]:g}"

    return re.sub(r"%([^%]*)%", field, template)


def run_spec(sp, mode="C", min_times=5, max_ms=300.0, settings=None):
    """Returns (status, impl, details): status PASSED / FAILED / SKIPPED (unimplemented)."""
    settings = settings or SETTINGS
    p = build_problem(sp)
    if settings["export_buffers"]:
        export_buffers(p, settings["export_buffers"])
    if settings["buffer_prefix"]:
        _, err = import_buffers(p, settings["buffer_prefix"])
        if err:
            return "FAILED", "", err
    t_c0 = time.perf_counter()
    try:
        pd, prim, strm, args, dst = api_objects(p, want_ref_impl=sp.impl == "ref",
                                                runtime_dims_masks=sp.runtime_dims_masks)
    except dnnl.error as e:
        if e.status == dnnl.unimplemented:
            return "SKIPPED", "", "unimplemented"
        return "FAILED", "", f"primitive descriptor: {e}"
    impl = pd.impl_info_str()
    # (the primitive descriptor and the primitive are created in one helper: their sum is what is timed)
    details = {"cpd_ms": 0.0, "cp_ms": (time.perf_counter() - t_c0) * 1e3}
    if "C" in mode:
        from oracle import binding as oracle
        from tests.helpers import compare
        oracle.load()
        prim.execute(strm, args)
        strm.wait()
        got = dst.read(storage_dtype(p.dst_dt))
        if p.dst_dynamic:
            # exact fills: the K sums are exact, so dst and the scales the matmul wrote compare as bytes
            want, want_sc = oracle.run_oracle_dynamic(p)
            got_sc = args[dnnl.ARG_ATTR_SCALES | dnnl.ARG_DST].read(np.uint8)
            nbad = int(np.count_nonzero(got_sc.reshape(-1) != np.asarray(want_sc).reshape(-1)))
            nbad += int(np.count_nonzero(np.asarray(got).view(np.uint8).reshape(-1)
                                         != np.asarray(want).view(np.uint8).reshape(-1)))
            details["errors"] = nbad
            return ("FAILED", impl, f"{nbad} bytes of dst / dst scales differ") if nbad else ("PASSED", impl, details)
        want, _, asum = oracle.run_oracle(p, want_ideal=True)
        transcendental = any(op.kind == cabi.PO_ELTWISE and op.alg not in (
            cabi.ELTWISE["relu"], cabi.ELTWISE["linear"], cabi.ELTWISE["clip"]) for op in p.post_ops)
        nbad, msg = compare(p, got, want, abs_sum=asum, transcendental=transcendental)
        if not nbad and p.dropout is not None and p.dropout.get("mask"):
            got_mask = args[dnnl.ARG_ATTR_DROPOUT_MASK].read(np.uint8)
            nbad = int(np.count_nonzero(got_mask != p._oracle_mask))
            msg = f"{nbad} bytes of the dropout mask differ"
        details["errors"] = nbad
        if nbad:
            return "FAILED", impl, msg
    if "P" in mode:
        prim.execute(strm, args)
        strm.wait()
        sets = cold_cache_sets(args, settings["cold_cache"])
        details["cold_cache_buffers"] = len(sets)
        times, t_all, it = [], time.perf_counter(), 0
        while len(times) < min_times or (time.perf_counter() - t_all) * 1e3 < max_ms:
            t0 = time.perf_counter()
            for _ in range(10):
                prim.execute(strm, sets[it % len(sets)])
                it += 1
            strm.wait()
            times.append((time.perf_counter() - t0) * 1e3 / 10)
            if len(times) >= 1000:
                break
        details["min_ms"], details["avg_ms"], details["max_ms"] = min(times), sum(times) / len(times), max(times)
        details["ops"] = 2.0 * p.M * p.N * p.K
        details["gops"] = details["ops"] / (min(times) * 1e-3) / 1e9
        details["ibytes"] = float(sum(np.ascontiguousarray(getattr(h, a)).nbytes for h, a in buffer_ids(p).values()))
        details["obytes"] = float(p.M * p.N * cabi.DT_BITS[p.dst_dt] // 8)
    return "PASSED", impl, details


def main(argv):
    settings = dict(SETTINGS)
    mode, specs = parse(argv, settings)
    if (settings["buffer_prefix"] or settings["export_buffers"]) and len(specs) > 1:
        print("--buffer-prefix / --export-buffers work with one test case at a time")
        return 2
    failed = 0
    for i, sp in enumerate(specs):
        t0 = time.perf_counter()
        status, impl, det = run_spec(sp, mode, max_ms=float(settings["max_ms_per_prb"]), settings=settings)
        ms = (time.perf_counter() - t0) * 1e3
        if status == "FAILED":
            failed += 1
            print(f"{i}:FAILED ({det}) ({ms:.0f} ms) __REPRO: {sp.repro()}")
            continue
        print(f"{i}:{status} ({ms:.0f} ms) __REPRO: {sp.repro()}")
        if status == "PASSED" and "P" in mode:
            print(perf_line(settings["perf_template"], sp, impl, det, i))
    print(f"tests:{len(specs)} passed:{len(specs) - failed} failed:{failed}")
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
