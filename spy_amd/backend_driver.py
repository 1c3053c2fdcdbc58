"""ctypes binding of libspy_backend.so: the C++ spy::Backend implementation driven through the
reference's operator API (one Backend::submit per graph node)."""
import ctypes as C
import os

import numpy as np

from . import _lib as H

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libspy_backend.so")
_lib = None


class HostTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("data", C.c_void_p), ("type", C.c_int32), ("rows", C.c_int64), ("cols", C.c_int64)]


SIGNATURES = {
    "spy_host_model_create": [C.POINTER(HostTensor), C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float,
                              C.c_char_p, C.POINTER(C.c_void_p)],
    "spy_host_model_forward": [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p],
    "spy_host_model_stats": [C.c_void_p, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64)],
    "spy_host_model_cache": [C.c_void_p, C.c_int, C.c_int, C.c_void_p],
    "spy_host_model_destroy": [C.c_void_p],
    "spy_host_unary_through_submit": [C.c_char_p, C.c_int, C.c_void_p, C.c_int64, C.c_int64, C.c_int, C.c_void_p, C.c_int64],
}


def load():
    global _lib
    if _lib is None:
        H.load()                                   # libspy_hip.so first: fails loudly when it is missing
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: build it with `make -C spy_amd/backend`" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = argtypes, C.c_int
        _lib = lib
    return _lib


class HostModel:
    """A LLaMA graph executed operator by operator through Backend::submit of the named backend."""

    def __init__(self, cfg, tensors, backend="hip:default"):
        self.L, self.cfg = load(), cfg
        shapes = cfg.tensor_shapes()
        self._keep = tensors
        arr = (HostTensor * len(shapes))()
        for i, (name, (t, rows, cols)) in enumerate(shapes.items()):
            arr[i] = HostTensor(name.encode(), tensors[name].ctypes.data, t, rows, cols)
        h = C.c_void_p()
        rc = self.L.spy_host_model_create(arr, len(shapes), cfg.n_layer, cfg.n_embd, cfg.n_head, cfg.n_ff, cfg.n_vocab, cfg.n_ctx,
                                          cfg.eps, cfg.rope_freq_base, backend.encode(), C.byref(h))
        if rc != 0:
            raise H.SpyHipError(rc, "spy_host_model_create") if rc > 0 else RuntimeError("spy_host_model_create: %d" % rc)
        self.handle = h

    def forward(self, tokens, n_past):
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        logits = np.empty((len(tokens), self.cfg.n_vocab), dtype=np.float32)
        rc = self.L.spy_host_model_forward(self.handle, tokens.ctypes.data, len(tokens), n_past, logits.ctypes.data)
        if rc != 0:
            raise H.SpyHipError(rc, "spy_host_model_forward") if rc > 0 else RuntimeError("spy_host_model_forward: %d" % rc)
        return logits

    def stats(self):
        v = [C.c_int64() for _ in range(4)]
        self.L.spy_host_model_stats(self.handle, *[C.byref(x) for x in v])
        return dict(zip(("n_ops", "n_submit", "n_alloc", "n_free"), [x.value for x in v]))

    def cache(self, layer, which):
        out = np.empty(self.cfg.n_ctx * self.cfg.n_embd, dtype=np.uint16)
        rc = self.L.spy_host_model_cache(self.handle, layer, which, out.ctypes.data)
        assert rc == 0, rc
        return out

    def close(self):
        if self.handle:
            self.L.spy_host_model_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def unary_through_submit(op, x, target_type=H.F32, backend="hip:default"):
    """One unary operator node (op: "relu", "silu", "quantize") on the rows of x (float32 [rows, cols]) through Backend::submit.
    Returns the result bytes as uint8 (quantize) or float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, cols = x.shape
    code = {"relu": 0, "silu": 1, "quantize": 2}[op]
    ttype = target_type if op == "quantize" else H.F32
    out = np.zeros(rows * H.row_size(ttype, cols), dtype=np.uint8)
    rc = load().spy_host_unary_through_submit(backend.encode(), code, x.ctypes.data, cols, rows, ttype, out.ctypes.data, out.nbytes)
    if rc != 0:
        raise H.SpyHipError(rc, "spy_host_unary_through_submit") if rc > 0 else RuntimeError("spy_host_unary_through_submit: %d" % rc)
    return out if op == "quantize" else out.view(np.float32).reshape(rows, cols)
