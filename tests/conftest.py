import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (C library under oracle/), built on first use."""
    from oracle import load
    return load()


@pytest.fixture(scope="session")
def isp():
    """inferspore_amd.ops on a GPU; the HIP library must already be built in-tree."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    from inferspore_amd import capi, ops
    capi.lib()  # raises if the HIP library is missing: GPU tests never fall back
    assert capi.lib().isp_init() == 0, "current device is not a gfx950"
    return ops


@pytest.fixture
def rng():
    return np.random.default_rng(0)
