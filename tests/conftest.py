import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import binding
    binding.load()
    return binding


@pytest.fixture(scope="session")
def gpu():
    """The C-ABI kernel library with a visible device; fails loudly, never
    falls back to a CPU path."""
    from onednn_amd import cabi
    lib = cabi.load_kernels()
    import ctypes as C
    n = C.c_int(0)
    cabi.check(lib.mi355_device_count(C.byref(n)))
    assert n.value > 0, "no HIP device visible"
    cabi.check(lib.mi355_device_set(0))
    return lib


@pytest.fixture(params=["large", "wide", "small"])
def i8_tiles(request):
    """Runs a test once per tile geometry of hip:mfma_i8 (the LDS tiles -- "large":
    256 x 128 when a problem has few tiles, as all test shapes do; "wide": 256 x 256
    -- and the 32 x 32 direct ones) wherever they can take the problem; by itself
    the dispatcher would give every small test shape to the small tiles."""
    from onednn_amd import cabi
    cabi.tuning_set("MI355_I8_TILES", request.param)
    if request.param == "wide":   # the fp8 family's switch between the same two LDS geometries
        cabi.tuning_set("MI355_F8_TILES", "wide")
    yield request.param
    cabi.tuning_set("MI355_I8_TILES", None)
    cabi.tuning_set("MI355_F8_TILES", None)
