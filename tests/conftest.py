import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_sessionstart(session):
    """A fresh checkout has no built library: build once (hipcc cross-compiles without a GPU).
    A tree that holds a built library is used as it is."""
    import __graft_entry__
    __graft_entry__.ensure_built()


def rel_err(x, y):
    """(max |x-y| / max(|y|, rms(y)),  max|x-y| / max|y|) -- both must pass a tolerance.

    Element-wise relative error is ill-defined where y crosses zero; the first
    figure floors the denominator at the RMS of the reference.
    """
    x = np.asarray(x, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    d = np.abs(x - y)
    rms = np.sqrt(np.mean(y * y))
    denom = np.maximum(np.abs(y), rms if rms > 0 else 1.0)
    amax = np.abs(y).max()
    return float((d / denom).max()), float(d.max() / (amax if amax > 0 else 1.0))


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.build()
    return o


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
