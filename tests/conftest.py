import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


PKG = os.path.join(ROOT, "jetfire-int8training_amd")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    O.lib()
    lib = os.path.join(PKG, "libjetfire_hip.so")
    if os.path.exists(lib):                      # the checker draws its rounding noise with the library's round count
        import ctypes
        O.set_noise_rounds(ctypes.CDLL(lib).jf_philox_rounds())
    return O

PKG = os.path.join(ROOT, "jetfire-int8training_amd")
for p in (PKG, os.path.join(PKG, "Jetfire")):
    if p not in sys.path:
        sys.path.insert(0, p)


@pytest.fixture(scope="session")
def jf():
    """ctypes binding of the HIP library; a GPU test without the built library is an error, not a skip."""
    import jetfire_hip
    jetfire_hip.lib()
    return jetfire_hip
