import ctypes
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


class Dev:
    """Tiny RAII helper around drhip_malloc/upload/download for the tests."""

    def __init__(self, lib):
        self.lib = lib
        self.ptrs = []

    def put(self, arr):
        arr = np.ascontiguousarray(arr)
        p = ctypes.c_void_p()
        assert self.lib.drhip_malloc(ctypes.byref(p), max(arr.nbytes, 4)) == 0, self.lib.drhip_last_error()
        self.ptrs.append(p)
        if arr.nbytes:
            assert self.lib.drhip_upload(p, 0, arr.ctypes.data_as(ctypes.c_void_p), arr.nbytes, None) == 0
        return p

    def empty(self, n, dtype=np.float32):
        return self.put(np.full(n, -777, dtype))       # poison: unwritten outputs are visible

    def get(self, p, shape, dtype=np.float32):
        out = np.empty(shape, dtype)
        assert self.lib.drhip_download(out.ctypes.data_as(ctypes.c_void_p), p, 0, out.nbytes, None) == 0, self.lib.drhip_last_error()
        return out

    def close(self):
        for p in self.ptrs:
            self.lib.drhip_free(p)
        self.ptrs = []


@pytest.fixture
def dev(lib, gpu):
    d = Dev(lib)
    yield d
    d.close()


def rel_err(a, b, floor=1e-30):
    """max |a-b| / max |b|: error relative to the layer's largest magnitude (at least `floor`)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), floor))


RTOL, ATOL_OF_MAX = 1e-4, 1e-6


def atol_factor(terms):
    """The absolute part of the element-wise bound, 1e-6 * max|want|, is sized for sums of about a thousand
    products.  The rounding noise of an fp32 sum grows with the square root of its length whatever the order
    of summation (the oracle's sequential sum included), so longer sums get sqrt(terms / 1024) times the room
    (FC6 of VGG16, 25088 terms: 4.9e-6 * max)."""
    return max(1.0, (terms / 1024.0) ** 0.5)


def elem_err(a, b, terms=0, floor=1e-30):
    """Element-wise criterion: worst |a-b| / (1e-4*max(|b|, floor) + 1e-6*atol_factor(terms)*max|b|); <= 1 passes.  Unlike
    rel_err it does not let an element of small magnitude be far off just because the layer has large
    elements elsewhere.  Returns (ratio, flat index of the worst element)."""
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    if a.size == 0:
        return 0.0, -1
    bound = RTOL * np.maximum(np.abs(b), floor) + ATOL_OF_MAX * atol_factor(terms) * max(np.abs(b).max(), floor)
    r = np.abs(a - b) / bound
    k = int(np.argmax(r))
    return float(r[k]), k


def assert_close(got, want, what="tensor", tol=RTOL, terms=0, floor=1e-30):
    """Both gates of the per-layer parity bar: max|got-want| / max|want| <= tol (norm-wise) and, element by
    element, |got-want| <= 1e-4*|want| + 1e-6*max|want| (the absolute part widened for sums of more than
    1024 products, see atol_factor).  `floor`: a lower limit for max|want| -- the magnitude of the terms
    that were added up -- for tensors of one or a few elements, whose largest value can itself be the
    remainder of a cancellation (bias against the convolution sum).  The message names the worst element."""
    got, want = np.asarray(got), np.asarray(want)
    assert got.shape == want.shape, "%s: shape %s vs %s" % (what, got.shape, want.shape)
    e = rel_err(got, want, floor)
    r, k = elem_err(got, want, terms, floor)
    msg = "%s: norm-wise %.3g; worst element #%d got %.9g want %.9g (%.3g x its bound)" % (
        what, e, k, got.reshape(-1)[k] if k >= 0 else 0.0, want.reshape(-1)[k] if k >= 0 else 0.0, r)
    assert e <= tol and r <= 1.0, msg


def spec_terms(node):
    """Products summed per output element of a layer-list node (0 for nodes that do not accumulate)."""
    if node["op"] == "conv":
        w = node["w"]
        return int(w.shape[0] * w.shape[2] * w.shape[3])
    if node["op"] == "fc":
        return int(node["w"].shape[0])
    return 0
