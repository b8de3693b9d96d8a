import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def oracle():
    """The CPU checker (oracle/), built on demand."""
    from oracle import oracle as orc
    orc.build()
    orc.lib()
    return orc


@pytest.fixture(scope="session")
def hip():
    """The HIP backend; GPU tests are skipped when no device is visible (cf. the reference's
    GTEST_SKIP in tests/CUDADeviceTest.cpp:89-92), but a missing library is an error."""
    import litenn_amd
    from litenn_amd import _lib
    _lib.load()  # raises if the extension was not built: never silently skipped
    if litenn_amd.HIPDeviceCount() == 0:
        pytest.skip("HIP device is not available")
    return litenn_amd


def rel_l2(a, b) -> float:
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))
