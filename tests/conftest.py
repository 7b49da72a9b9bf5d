import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def lib():
    """libdeepracin.so; built in-tree beforehand (python -m deepracin_amd.build), only built here if absent."""
    import deepracin_amd as dr
    if not os.path.exists(dr.LIB_PATH):
        from deepracin_amd import build
        build.build(verbose=False)
    return dr.load_library()


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as orc
    orc.load()
    return orc


@pytest.fixture(scope="session")
def gpu(lib):
    """Initialised device; a GPU test without a device FAILS (no silent CPU fallback)."""
    import deepracin_amd as dr
    info = dr.DeviceInfo()
    rc = lib.drhip_init(0, info)
    assert rc == 0, "no usable gfx950 device: %s" % lib.drhip_last_error().decode()
    return info


def rel_err(a, b):
    """max |a-b| / max |b|: error relative to the layer's largest magnitude."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))
