import os
import sys

import numpy as np
import pytest

# torch ships its own copy of the HIP runtime.  It has to be loaded before
# librsfk.so so that both use the same runtime inside this process (a process
# that initialises two HIP runtimes sees no GPU in the second one).
try:
    import torch  # noqa: F401
except Exception:  # pragma: no cover - torch is optional for everything but device buffers
    torch = None

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "gpu-rsfk_amd"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (runs the HIP library through its C ABI)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (test infrastructure)."""
    from oracle import rsfk_oracle
    rsfk_oracle.lib()
    return rsfk_oracle


@pytest.fixture(scope="session")
def capi():
    """ctypes view of librsfk.so.  Fails loudly if the library has not been built."""
    from gpu_rsfk import capi as c
    c.lib()
    return c


@pytest.fixture(scope="session")
def gpu(capi):
    """The HIP library on a machine that has a GPU."""
    n = capi.lib().rsfk_device_count()
    if n < 1:
        pytest.skip("no HIP device visible")
    return capi


@pytest.fixture
def rng():
    return np.random.default_rng(12345)
