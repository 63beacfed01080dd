"""The MFMA epilogue divides by the dst scale with two fma corrections of
x * (1 / s) when dst is an integer type (tile_epilogue.hpp, div_by_fma).  The
same five operations on the host (tests/div_by_fma_check.c, IEEE fmaf) must
return the IEEE quotient bit for bit for 2^-90 <= |x| < 2^100 and a quotient
that vanishes in the integer rounding for smaller |x|: for the dst scale of the
int8 benchmark configuration (and a few others) over every float the device
path admits, and for random divisors (every mantissa pattern the correction is
sensitive to included) on random dividends."""
import os
import shutil
import subprocess
import tempfile

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def checker():
    if shutil.which("gcc") is None:
        pytest.skip("no host compiler")
    d = tempfile.mkdtemp(prefix="divfma")
    exe = os.path.join(d, "div_by_fma_check")
    subprocess.check_call(["gcc", "-O2", "-fopenmp", "-mfma", "-ffp-contract=off", "-o", exe,
                           os.path.join(HERE, "div_by_fma_check.c"), "-lm"])
    yield exe
    shutil.rmtree(d, ignore_errors=True)


@pytest.mark.parametrize("scale", [0.05, 3.0, 1.9999999])
def test_every_admitted_dividend(checker, scale):
    bits = int(np.float32(scale).view(np.uint32))
    out = subprocess.run([checker, "exhaustive", f"{bits:08x}"], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "0", (scale, out.stdout, out.stderr)


def test_random_divisors(checker):
    out = subprocess.run([checker, "sample", "20000", "20000"], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "0", (out.stdout, out.stderr)
