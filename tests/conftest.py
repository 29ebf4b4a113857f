import os
import sys

import pytest

# PyTorch ships its own copy of the HIP/HSA runtime.  A test that hands torch device pointers to the library needs
# both to share one runtime in the process, which is the case when torch is loaded first, whatever subset of the
# test files is collected.
try:
    import torch  # noqa: F401
except ImportError:
    pass

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as _oracle
    _oracle.build()
    return _oracle


@pytest.fixture(autouse=True)
def activations_start_as_nans(request, monkeypatch):
    """GPU tests create their instances with every activation byte 0xFF (binary16 NaN, DENOX_HIP_POISON=1): a dispatch
    that lets memory nobody wrote reach its result then fails its comparison instead of passing on whatever the
    allocation happened to hold."""
    if request.node.get_closest_marker("gpu") is not None:
        monkeypatch.setenv("DENOX_HIP_POISON", "1")
