"""CPU-side checks of the drop-in boundary: the library loads and exports every symbol that
include/spy_hip.h declares; argument checks reject bad operands before any launch."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "spy_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(spy_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    from spy_amd import _lib
    L = _lib.load()
    names = declared_symbols()
    assert len(names) >= 30
    for n in names:
        assert hasattr(L, n), "libspy_hip.so does not export %s" % n
    # and the Python binding covers exactly the header
    assert sorted(_lib.SIGNATURES) == names


def test_error_strings():
    from spy_amd import _lib
    assert "not supported" in _lib.error_string(_lib.EUNSUPPORTED)
    assert "invalid" in _lib.error_string(_lib.EINVAL)
    assert _lib.error_string(0) == "success"


def test_argument_checks_without_gpu():
    """Shape / pointer validation happens on the host before any HIP call."""
    from spy_amd import _lib
    L = _lib.load()
    assert L.spy_hip_gemv_q8_0act(None, _lib.Q4_0, None, None, None, None, 8, 256, 1, 8) == _lib.EINVAL
    assert L.spy_hip_gemv_q8_0act(None, _lib.Q4_0, 16, 16, 16, None, 8, 250, 1, 8) == _lib.EINVAL      # K % 32
    assert L.spy_hip_gemv_q8_0act(None, _lib.F32, 16, 16, 16, None, 8, 256, 1, 8) == _lib.EUNSUPPORTED
    assert L.spy_hip_quantize_q8_0(None, 16, 1024, 16, 1, 100) == _lib.EINVAL
    t = _lib.Tensor()
    assert L.spy_hip_op_norm_rms(None, C.byref(t), C.byref(t), 1e-5) == _lib.EINVAL                  # null data


def test_missing_library_fails_loudly(monkeypatch):
    from spy_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", os.path.join(ROOT, "spy_amd", "no_such_lib.so"))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load()
