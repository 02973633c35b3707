"""Test configuration: the ``gpu`` marker, import paths, shared helpers."""
import os
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parents[1]
for p in (ROOT, ROOT / "oracle"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) device")


@pytest.fixture(scope="session")
def lane():
    """The loaded lane; GPU tests fail loudly (not skip) when it is missing."""
    from tessera_amd import lane as _lane
    _lane.load()
    if not _lane.available():
        pytest.fail("gfx950 lane not available: GPU tests must run the HIP path")
    return _lane


def bf16(x):
    from tessera_amd import bf16 as _b
    return _b.from_float32(np.asarray(x, np.float32))
