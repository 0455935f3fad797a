"""Shared fixtures.

``cpu``  the numpy oracle backend (oracle/nervanacpu.py) -- the checker.
``hip``  the MI355X backend; tests that use it carry the ``gpu`` marker and are
         skipped where no device is visible.
"""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run on the GPU box)")
    # the tests load the library the build left in the tree; build it only if
    # there is none
    import __graft_entry__
    __graft_entry__.ensure_built()


def _device_count():
    try:
        from neon_amd.backends.hip import runtime as hiprt
        return hiprt.device_count()
    except OSError:
        return 0


def pytest_collection_modifyitems(config, items):
    if _device_count() > 0:
        return
    skip = pytest.mark.skip(reason="no HIP device visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def cpu():
    from oracle import nervanacpu  # noqa: F401  registers 'cpu'
    from neon_amd.backends.backend import Backend
    be = Backend.allocate_backend("cpu", rng_seed=0)
    be.bsz = 128
    return be


@pytest.fixture(scope="session")
def hip():
    import neon_amd.backends  # noqa: F401  registers 'hip'
    from neon_amd.backends.backend import Backend
    be = Backend.allocate_backend("hip", rng_seed=0)
    be.bsz = 128
    yield be
    be.synchronize()


@pytest.fixture(scope="session")
def pair(cpu, hip):
    return cpu, hip
