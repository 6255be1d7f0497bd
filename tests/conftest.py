import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    import __graft_entry__ as ge
    return ge.load_package()


@pytest.fixture(scope="session")
def gpu(pkg):
    """The package with device 0 initialised; fails loudly when the HIP
    library or the device is missing (no CPU fallback exists)."""
    pkg.init(0)
    return pkg


def _roctx():
    """librocprofiler-sdk-roctx when LLM_TEST_ROCTX=1 (set for a `rocprofv3 --kernel-trace --marker-trace` run
    of the suite, which then shows which test launched which kernel); None otherwise."""
    if os.environ.get("LLM_TEST_ROCTX") != "1":
        return None
    if not hasattr(_roctx, "lib"):
        import ctypes
        _roctx.lib = ctypes.CDLL("librocprofiler-sdk-roctx.so")
        _roctx.lib.roctxRangePushA.argtypes = [ctypes.c_char_p]
    return _roctx.lib


@pytest.fixture(autouse=True)
def _test_as_marker_range(request):
    lib = _roctx()
    if lib:
        lib.roctxRangePushA(request.node.nodeid.encode())
    yield
    if lib:
        lib.roctxRangePop()
