"""Helpers for the GPU parity tests: device buffers through the C ABI and error reporting."""
import ctypes as C

import numpy as np

from spy_amd import _lib as H

REL_TOL = 1e-3      # per-op float tolerance of the parity contract (max-abs error / max-abs value)


def dev(arr):
    return H.DeviceBuffer.from_numpy(np.ascontiguousarray(arr))


def dev_empty(nbytes, fill=None):
    b = H.DeviceBuffer(nbytes)
    if fill is not None:
        b.fill(fill)
    return b


def call(fn, *args):
    rc = fn(*args)
    if rc != 0:
        raise H.SpyHipError(rc, fn.__name__)


def rel_err(got, want):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    denom = max(float(np.abs(want).max()), 1e-30)
    return float(np.abs(got - want).max()) / denom


def assert_close(got, want, what, tol=REL_TOL):
    e = rel_err(got, want)
    print("%s: max-abs err %.3e (relative to max |ref| %.3e) = %.3e" % (what, float(np.abs(np.asarray(got, np.float64) - np.asarray(want, np.float64)).max()),
                                                                     float(np.abs(want).max()), e), flush=True)
    assert np.all(np.isfinite(got)), what
    assert e <= tol, "%s: relative error %.3e > %.1e" % (what, e, tol)
