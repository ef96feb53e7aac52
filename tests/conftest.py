import os
import sys

import pytest

# Bound every device-side wait in the test suite (about a minute of polling): a
# missing signal then ends in a failed assertion instead of a hung GPU.  Must be
# set before the kernel library is first used.
os.environ.setdefault("FO_WAIT_MAX_POLLS", "40000000")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU checker (oracle/), built on demand with its Makefile."""
    from oracle import oracle as o
    o.build()
    o.lib()
    return o


@pytest.fixture(scope="session")
def fo():
    """The product package with the HIP library loaded; GPU tests only."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import flashoverlap_amd
    from flashoverlap_amd import _capi
    _capi.lib()  # raises if libfo_kernels.so is missing: no silent fallback
    return flashoverlap_amd
