"""drhip_fc_noalloc_f32 -- the fully-connected entry point that allocates nothing (its partial sums
live in an array inside the library's code object) -- against drhip_fc_f32 with a caller buffer,
through the C-ABI: bit for bit, on two calls in a row, the second with a smaller input, so that what
the first call left in the shared array would show if the second read any of it.
"""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _put(lib, arr):
    arr = np.ascontiguousarray(arr, np.float32)
    p = ctypes.c_void_p()
    assert lib.drhip_malloc(ctypes.byref(p), arr.nbytes) == 0, lib.drhip_last_error()
    assert lib.drhip_upload(p, 0, arr.ctypes.data_as(ctypes.c_void_p), arr.nbytes, None) == 0
    return p


def _get(lib, p, n):
    out = np.empty(n, np.float32)
    assert lib.drhip_download(out.ctypes.data_as(ctypes.c_void_p), p, 0, out.nbytes, None) == 0, lib.drhip_last_error()
    return out


def _free_device_bytes():
    """hipMemGetInfo of the runtime the library itself is linked against (already loaded into this process)."""
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def test_fc_noalloc_matches_fc_on_two_calls_in_a_row(lib, gpu, oracle):
    rng = np.random.default_rng(2024)
    held = []
    try:
        for K, N, relu in ((4096, 1000, 0), (1536, 520, 1)):         # the second call is the smaller one
            print("drhip_fc_noalloc_f32 K=%d N=%d relu=%d" % (K, N, relu), flush=True)
            nparts = lib.drhip_fc_scratch_floats(K, N)
            assert 0 < nparts <= lib.drhip_fc_noalloc_max_scratch_floats()     # split over row slices: the scratch is really used
            x = rng.standard_normal(K).astype(np.float32)
            Wt = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
            b = rng.standard_normal(N).astype(np.float32)
            xd, Wd, bd = _put(lib, x), _put(lib, Wt), _put(lib, b)
            parts = _put(lib, np.full(nparts, np.nan, np.float32))
            y_ref, y_new = _put(lib, np.full(N, -777.0)), _put(lib, np.full(N, -555.0))
            held += [xd, Wd, bd, parts, y_ref, y_new]
            assert lib.drhip_fc_f32(xd, Wd, bd, y_ref, parts, K, N, relu, None) == 0, lib.drhip_last_error()
            assert lib.drhip_stream_sync(None) == 0
            free_before = _free_device_bytes()
            assert lib.drhip_fc_noalloc_f32(xd, Wd, bd, y_new, K, N, relu, None) == 0, lib.drhip_last_error()
            assert lib.drhip_stream_sync(None) == 0
            assert _free_device_bytes() == free_before, "device memory was taken or given back during the call"
            want, got = _get(lib, y_ref, N), _get(lib, y_new, N)
            assert np.array_equal(want, got), "K=%d N=%d: %d of %d elements differ" % (K, N, int((want != got).sum()), N)
            # and the existing entry point itself is right (oracle, 1e-4 of the layer's largest magnitude)
            ref = oracle.fc(x.reshape(K, 1, 1), Wt, b, relu).reshape(-1)      # C = K, H = W = 1: rows in buffer order
            assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max()
        # an unsplit shape uses no scratch at all and must work too
        K, N = 64, 8
        assert lib.drhip_fc_scratch_floats(K, N) == 0
        x = rng.standard_normal(K).astype(np.float32)
        Wt = rng.standard_normal((K, N)).astype(np.float32)
        xd, Wd = _put(lib, x), _put(lib, Wt)
        y_ref, y_new = _put(lib, np.zeros(N)), _put(lib, np.ones(N))
        held += [xd, Wd, y_ref, y_new]
        assert lib.drhip_fc_f32(xd, Wd, None, y_ref, None, K, N, 0, None) == 0
        assert lib.drhip_fc_noalloc_f32(xd, Wd, None, y_new, K, N, 0, None) == 0, lib.drhip_last_error()
        assert np.array_equal(_get(lib, y_ref, N), _get(lib, y_new, N))
    finally:
        for p in held:
            lib.drhip_free(p)


def test_fc_noalloc_refuses_what_does_not_fit(lib, gpu):
    limit = lib.drhip_fc_noalloc_max_scratch_floats()
    assert limit == 64 * 1024
    K, N = 8192, 65280                                       # two row slices of 65280 columns
    assert lib.drhip_fc_scratch_floats(K, N) > limit
    fake = ctypes.c_void_p(256)                              # never dereferenced: the call must stop on the host
    rc = lib.drhip_fc_noalloc_f32(fake, fake, None, fake, K, N, 0, None)
    assert rc == -1 and b"built-in scratch" in lib.drhip_last_error()
    assert lib.drhip_fc_noalloc_f32(None, None, None, None, 8, 8, 0, None) == -1
