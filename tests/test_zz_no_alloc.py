"""mi355_matmul_launch_noalloc, the launch for callers that cannot allocate
device memory: its scratch is a static device array inside the library.  Two
calls in a row through the C ABI, the second on a smaller input, each bit for
bit equal to what mi355_matmul_launch writes with a caller-owned scratch buffer
(and to the oracle); a problem beyond the static buffer is refused."""
import ctypes as C

import numpy as np
import pytest

from onednn_amd import cabi, configs
from onednn_amd.problem import GpuRun

pytestmark = pytest.mark.gpu


def both_ways(p, impl=None):
    lib = cabi.load_kernels()
    run = GpuRun(p, impl)
    try:
        assert run.scratch is not None, "the case must use scratch memory"
        run.launch()
        want = np.array(run.result(), copy=True)
        run.reset_dst()
        cabi.check(lib.mi355_matmul_launch_noalloc(C.byref(run.desc), C.byref(run.args), run.stream))
        got = np.array(run.result(), copy=True)
        return got, want, cabi.impl_name(run.impl)
    finally:
        run.free()


def test_two_calls_in_a_row_second_smaller(gpu, oracle):
    # u8 src with a zero point and row-major weights: transposed weights + column sums live in scratch
    big = configs.config1(M=256, N=1024, K=1024)
    small = configs.config1(M=96, N=320, K=256)
    for p in (big, small):
        got, want, name = both_ways(p)
        assert name.startswith("hip:mfma_i8"), name
        assert np.array_equal(np.asarray(got).view(np.uint8), np.asarray(want).view(np.uint8)), p.M
        assert np.array_equal(np.asarray(got).view(np.uint8), np.asarray(oracle.run_oracle(p)).view(np.uint8))
    # split-K partial sums of the row-major decode kernel, larger then smaller
    for p in (configs.config2(M=8, N=2048, K=4096), configs.config2(M=1, N=512, K=1024)):
        got, want, name = both_ways(p, cabi.IMPL_WOQ_GEMV)
        assert name.startswith("hip:woq_gemv"), name
        assert np.array_equal(np.asarray(got).view(np.uint8), np.asarray(want).view(np.uint8)), p.M


def test_beyond_the_static_buffer_is_refused(gpu):
    lib = cabi.load_kernels()
    p = configs.config3(M=256, N=4096, K=4096)      # row-major weights: a 16 MiB transposed copy
    d = p.desc()
    need = cabi.scratch_bytes(d)
    assert need > cabi.NOALLOC_SCRATCH_BYTES
    a = cabi.MatmulArgs()
    st = lib.mi355_matmul_launch_noalloc(C.byref(d), C.byref(a), None)
    assert st == cabi.INVALID_ARGUMENTS
    msg = lib.mi355_last_error().decode()
    assert str(need) in msg and str(cabi.NOALLOC_SCRATCH_BYTES) in msg
