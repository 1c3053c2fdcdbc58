"""Helpers for the GPU parity tests: device buffers through the C ABI and error reporting."""
import ctypes as C

import numpy as np

from spy_amd import _lib as H

REL_TOL = 1e-3      # per-op float tolerance of the parity contract (max-abs error / max-abs value)
# Across SEVERAL operators the reference's own rounding points re-amplify last-ulp differences:
# every MatMul re-quantizes its activations to Q8_0 (mat.cpp:95-128 in the Spy tree) and the softmax
# rounds its exp argument to fp16 (non-linear.cpp:170), so an input that differs by 1e-5 moves a
# few of those roundings to the neighbouring integer / fp16 value and the next operator's output
# by ~1e-3.  Any implementation whose fp32 summation order differs from the AVX host code sees
# this; whole-pass comparisons therefore use this looser bound, per-operator comparisons (same
# inputs on both sides) use REL_TOL.
E2E_TOL = 3e-2


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
