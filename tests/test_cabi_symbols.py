"""The C-ABI library loads without a GPU and exports every function that
include/*.h declares (no compute calls here)."""
import ctypes as C
import glob
import os
import re

from onednn_amd import cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:mi355|dnnl)_[a-z0-9_]+)\s*\(", text)))


def test_kernel_library_exports_every_declared_symbol():
    lib = cabi.load_kernels()
    names = declared_functions(os.path.join(ROOT, "include", "mi355_matmul.h"))
    assert len(names) >= 20
    assert sorted(names) == sorted(cabi.KERNEL_SYMBOLS)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/mi355_matmul.h but not exported"


def test_struct_layout_matches_header_sizes():
    # sizes implied by the header's field lists (LP64): catches a drifting mirror
    assert C.sizeof(cabi.Quant) == 24
    assert C.sizeof(cabi.PostOp) == 56
    assert C.sizeof(cabi.MatmulDesc) == 32 + 16 + 4 * 24 + 7 * 24 + 16 + 32 * 56 + 16
    assert C.sizeof(cabi.MatmulArgs) == 8 * (11 + 32 + 4)     # + the four dropout pointers


def test_query_validates_without_a_device():
    d = cabi.MatmulDesc()
    st, _ = cabi.query(d)                      # all-zero descriptor: unknown data types
    assert st == cabi.INVALID_ARGUMENTS
    from onednn_amd import configs
    p = configs.config3(M=256, N=256, K=256)
    st, impl = cabi.query(p.desc())
    assert st == cabi.SUCCESS and cabi.impl_name(impl).startswith("hip:mfma_i8")
    dd = p.desc()
    dd.K = 200                                  # not a multiple of the K tile: generic kernel
    st, impl = cabi.query(dd)
    assert st == cabi.SUCCESS and cabi.impl_name(impl) == "hip:ref:any"
    st, _ = cabi.query(dd, cabi.IMPL_I8_MFMA)
    assert st == cabi.UNIMPLEMENTED
    p5 = configs.config5(M=128, N=128, K=256)
    st, impl = cabi.query(p5.desc())
    assert st == cabi.SUCCESS and cabi.impl_name(impl).startswith("hip:mfma_mxf4")
    p4 = configs.config4(M=128, N=128, K=256)
    st, impl = cabi.query(p4.desc())
    assert st == cabi.SUCCESS and cabi.impl_name(impl).startswith("hip:mfma_f8")
