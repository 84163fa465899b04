import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def rel_err(got, want):
    """max|got - want| / max|want| over a tensor: the metric of the 1e-10 / 1e-8 tolerances."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, "shape %r vs %r" % (got.shape, want.shape)
    if want.size == 0:
        return 0.0
    denom = np.max(np.abs(want))
    diff = np.max(np.abs(got - want))
    if denom == 0.0:
        return float(diff)
    return float(diff / denom)


@pytest.fixture(scope="session")
def engine():
    """The backend engine on GPU 0.  Fails (never skips) when the library or the GPU is missing,
    so a GPU run cannot pass on a silent fallback."""
    import rstorch_amd
    from rstorch_amd import _ffi
    assert os.path.exists(_ffi.library_path()), "librstorch_hip.so is not built: run __graft_entry__.build()"
    return rstorch_amd.default_engine()


@pytest.fixture(scope="session")
def oracle():
    import oracle as _oracle
    _oracle.lib()
    return _oracle
