import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "minfer-python_amd")
for p in (ROOT, PKG, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)
# the apps directory goes last: it holds a profile.py (the reference's name for that script), which must not
# shadow the standard library's `profile` module (cProfile, and through it torch.library.opcheck, imports it)
if os.path.join(PKG, "apps") not in sys.path:
    sys.path.append(os.path.join(PKG, "apps"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def kerns():
    # registers torch.ops.minfer.* the way the reference's test/conftest.py:1-2 does
    import minfer.kernels.torch_ext  # noqa: F401
    from minfer.kernels import KernelBackend
    return KernelBackend("torch_ext")
