"""The boundary through a compiler: small C programs that include only
include/dnnl_amd.h / include/mi355_matmul.h, built with gcc against the two
shared libraries and run on the device (u8 x s8 -> s32 matmuls and an inner product on
channels-last tensors, each checked against an integer loop inside the program; attention on f32 tensors against a
double-precision loop), and a C++ program over include/dnnl_amd.hpp written like the reference's int8 inference
tutorial, three more for its weight-only-quantization, MX and dynamic-quantization tutorials, and its inner-product example
with the two backward primitives added, its matmul and reorder examples.  Struct layouts, enum values and calling
conventions of the headers are what a compiled caller sees; the ctypes tests
only check names."""
import os
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")
LIB = os.path.join(ROOT, "onednn_amd", "lib")


def build(name, lib):
    """<name>.c with gcc as C11, or <name>.cpp (a caller of include/dnnl_amd.hpp) with g++ as C++11."""
    if shutil.which("gcc") is None or shutil.which("g++") is None:
        pytest.skip("no host compiler")
    d = tempfile.mkdtemp(prefix="cclient")
    exe = os.path.join(d, name)
    c_src = os.path.join(ROOT, "tests", "c_clients", name + ".c")
    cc = ["gcc", "-std=c11", c_src] if os.path.exists(c_src) else ["g++", "-std=c++11", "-O1", c_src + "pp"]
    subprocess.check_call(cc + ["-Wall", "-Wextra", "-Werror", "-I", INC, "-o", exe, "-L", LIB, "-l" + lib,
                                "-Wl,-rpath," + LIB, "-lm"])
    return d, exe


def test_headers_compile_as_c_and_link():
    # no device needed: the programs build against the headers and libraries
    for name, lib in (("dnnl_client", "dnnl_amd"), ("ip_client", "dnnl_amd"), ("sdpa_client", "dnnl_amd"),
                      ("mi355_client", "mi355_matmul"), ("dnnl_cpp_client", "dnnl_amd"), ("woq_cpp_client", "dnnl_amd"),
                      ("mxfp_cpp_client", "dnnl_amd"), ("quantization_cpp_client", "dnnl_amd"),
                      ("ip_cpp_client", "dnnl_amd"), ("primitives_cpp_client", "dnnl_amd")):
        d, exe = build(name, lib)
        assert os.path.exists(exe)
        shutil.rmtree(d, ignore_errors=True)


@pytest.mark.gpu
@pytest.mark.parametrize("name,lib,impl", [("dnnl_client", "dnnl_amd", "hip:mfma_i8"), ("ip_client", "dnnl_amd", "hip:mfma_i8"),
                                           ("sdpa_client", "dnnl_amd", "hip:sdpa("),
                                           ("dnnl_cpp_client", "dnnl_amd", "hip:mfma_i8"),
                                           ("woq_cpp_client", "dnnl_amd", "hip:"),
                                           ("mxfp_cpp_client", "dnnl_amd", "hip:"),
                                           ("quantization_cpp_client", "dnnl_amd", "hip:"),
                                           ("ip_cpp_client", "dnnl_amd", "hip:"),
                                           ("primitives_cpp_client", "dnnl_amd", "hip:"),
                                           ("mi355_client", "mi355_matmul", "hip:mfma_i8")])
def test_c_client_runs_on_the_device(gpu, name, lib, impl):
    d, exe = build(name, lib)
    try:
        out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
        assert out.returncode == 0 and out.stdout.startswith("ok " + impl), (out.stdout, out.stderr)
    finally:
        shutil.rmtree(d, ignore_errors=True)
