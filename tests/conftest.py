import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "operators-rs_amd"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


# The CPU tier runs some of the GPU tests against a build of the library in which the kernels are compiled for the host
# and the HIP runtime is a stand-in (tests/cpu_sim, tests/test_cpu_sim_library.py): it starts pytest again with this
# variable naming that build.  Nothing else sets it; without it the tests load the product library.
if os.environ.get("OPHIP_CPU_SIM_LIBRARY"):
    import ophip

    ophip.LIB_PATH = os.environ["OPHIP_CPU_SIM_LIBRARY"]


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    import ophip

    if ophip.device_count() == 0:
        pytest.fail("GPU test selected but no HIP device is visible (the HIP backend has no CPU fallback)")
    g = ophip.Gpu(0)
    yield g


@pytest.fixture(scope="session")
def stream(gpu):
    s = gpu.stream()
    yield s
    s.synchronize()
