"""GPU parity: HIP kernels (through the C ABI) against the CPU oracle on the
same seeded inputs, at sizes the oracle finishes in seconds."""
import numpy as np
import pytest

from onednn_amd import cabi, configs
from onednn_amd.problem import run_gpu
from tests.helpers import assert_bit_exact, assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dst", ["s32", "f32"])
@pytest.mark.parametrize("impl", [cabi.IMPL_REF, cabi.IMPL_I8_MFMA])
def test_config1_small(gpu, oracle, dst, impl):
    p = configs.config1(M=96, N=320, K=256, dst=dst)
    got, name = run_gpu(p, impl)
    want = oracle.run_oracle(p)
    # integer accumulation is order-free and the epilogue has one rounding per
    # written operation: both kernels must reproduce the oracle bit for bit
    assert_bit_exact(p, got, want, name)


@pytest.mark.parametrize("impl", [cabi.IMPL_REF, cabi.IMPL_I8_MFMA])
@pytest.mark.parametrize("mode", [cabi.DST_SCALE_DIVIDE, cabi.DST_SCALE_RECIPROCAL])
def test_config3_small(gpu, oracle, impl, mode):
    p = configs.config3(M=160, N=288, K=512, dst_scale_mode=mode)
    got, name = run_gpu(p, impl)
    want = oracle.run_oracle(p)
    assert_bit_exact(p, got, want, name)


def test_config1_full_size(gpu, oracle):
    p = configs.config1()
    got, name = run_gpu(p)
    assert name.startswith("hip:mfma_i8")
    want = oracle.run_oracle(p)
    assert_bit_exact(p, got, want, name)
