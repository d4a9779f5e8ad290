"""Shared test configuration.

Markers: ``gpu`` tests need a MI355X and the built HIP library and go through
the C-ABI; everything else runs on CPU only (checker vs golden vectors, host
logic, symbol export).  As in the reference (tests/conftest.py:39-44) every
test is seeded from its own name.
"""
import os
import sys
from zlib import adler32

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "cnn-mellin_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

GPU_AVAIL = torch.cuda.is_available()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a MI355X and the built HIP library")
    config.addinivalue_line("markers", "slow: full-size property tests")


def pytest_runtest_setup(item):
    if any(mark.name == "gpu" for mark in item.iter_markers()) and not GPU_AVAIL:
        pytest.skip("no GPU visible")
    seed = abs(adler32(bytes(item.name, "utf-8")))
    torch.manual_seed(seed)
    np.random.seed(seed % (2 ** 32))


@pytest.fixture(autouse=True)
def _announce(request):
    # name the case before it touches the GPU so that a fault can be attributed
    print("\n[case] %s" % request.node.nodeid, flush=True)
    yield
