"""ctypes binding of oracle/libspy_oracle.so -- the CPU checker (test infrastructure only).

Only tests/, the smoke check and the cpu_baseline leg of bench.py may use this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "oracle", "libspy_oracle.so")

F32, F16, Q4_0, Q8_0, Q4_K, Q6_K, I32 = 0, 1, 2, 8, 12, 14, 26
TYPE_SIZE = {F32: 4, F16: 2, Q4_0: 18, Q8_0: 34, Q4_K: 144, Q6_K: 210, I32: 4}
BLOCK_SIZE = {F32: 1, F16: 1, Q4_0: 32, Q8_0: 32, Q4_K: 256, Q6_K: 256, I32: 1}
NP_DTYPE = {F32: np.float32, F16: np.uint16, I32: np.int32}


def row_size(t, n):
    return n * TYPE_SIZE[t] // BLOCK_SIZE[t]


class Tensor(C.Structure):
    _fields_ = [("type", C.c_int32), ("dim", C.c_int32), ("ne", C.c_int64 * 4), ("nb", C.c_int64 * 4),
                ("data", C.c_void_p)]


class RopeParam(C.Structure):
    _fields_ = [("mode", C.c_int32), ("num_past", C.c_int32), ("num_dim", C.c_int32), ("num_context", C.c_int32),
                ("num_origin_context", C.c_int32), ("freq_base", C.c_float), ("freq_scale", C.c_float),
                ("extend_factor", C.c_float), ("attention_factor", C.c_float), ("beta_fast", C.c_float),
                ("beta_slow", C.c_float), ("xpos_base", C.c_float), ("xpos_down", C.c_int32)]


class LlamaLayer(C.Structure):
    _fields_ = [("attn_norm", C.c_void_p), ("ffn_norm", C.c_void_p),
                ("wq", C.c_void_p), ("wk", C.c_void_p), ("wv", C.c_void_p), ("wo", C.c_void_p),
                ("w_gate", C.c_void_p), ("w_up", C.c_void_p), ("w_down", C.c_void_p),
                ("t_wq", C.c_int32), ("t_wk", C.c_int32), ("t_wv", C.c_int32), ("t_wo", C.c_int32),
                ("t_gate", C.c_int32), ("t_up", C.c_int32), ("t_down", C.c_int32)]


class Llama(C.Structure):
    _fields_ = [("n_layer", C.c_int32), ("n_embd", C.c_int32), ("n_head", C.c_int32), ("n_ff", C.c_int32),
                ("n_vocab", C.c_int32), ("n_ctx", C.c_int32), ("eps", C.c_float), ("rope_freq_base", C.c_float),
                ("nthread", C.c_int32), ("tok_embd", C.c_void_p), ("t_tok_embd", C.c_int32),
                ("out_norm", C.c_void_p), ("w_out", C.c_void_p), ("t_out", C.c_int32),
                ("layers", C.POINTER(LlamaLayer)), ("k_cache", C.POINTER(C.c_void_p)),
                ("v_cache", C.POINTER(C.c_void_p))]


def default_rope(num_dim, n_ctx, n_past=0, freq_base=10000.0):
    return RopeParam(0, n_past, num_dim, n_ctx, n_ctx, freq_base, 1.0, 0.0, 1.0, 32.0, 1.0, 0.0, 0)


def ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def tensor(arr, ttype, ne, nb=None, offset=0):
    """Describe memory held by numpy array `arr` as a Spy tensor (ne/nb in Spy order)."""
    t = Tensor()
    t.type, t.dim = ttype, len(ne)
    ne4 = list(ne) + [1] * (4 - len(ne))
    if nb is None:
        nb4 = [TYPE_SIZE[ttype], row_size(ttype, ne4[0]), 0, 0]
        nb4[2] = nb4[1] * ne4[1]
        nb4[3] = nb4[2] * ne4[2]
    else:
        nb4 = list(nb) + [ne4[len(nb) - 1] * nb[-1]] * (4 - len(nb))
    for i in range(4):
        t.ne[i], t.nb[i] = ne4[i], nb4[i]
    t.data = arr.ctypes.data + offset
    t._keep = arr
    return t


_lib = None


def build():
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "oracle")])


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB):
        build()
    _lib = _bind(C.CDLL(LIB))
    return _lib


LIB_FPFAST = os.path.join(ROOT, "oracle", "libspy_oracle_fpfast.so")
_lib_fpfast = None


def load_fpfast():
    """The same source compiled with -ffp-contract=fast -mfma (make -C oracle FPCONTRACT=fast): gcc may then fuse the scalar
    a * b + c expressions too, as a default GCC build of the reference would.  Only for the test that reports the difference."""
    global _lib_fpfast
    if _lib_fpfast is None:
        if not os.path.exists(LIB_FPFAST):
            subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "FPCONTRACT=fast"])
        _lib_fpfast = _bind(C.CDLL(LIB_FPFAST))
    return _lib_fpfast


def _bind(L):
    vp, i64, i32, f32 = C.c_void_p, C.c_int64, C.c_int32, C.c_float
    TP = C.POINTER(Tensor)
    sig = {
        "spy_o_f32_to_f16": (C.c_uint16, [f32]), "spy_o_f16_to_f32": (f32, [C.c_uint16]),
        "spy_o_f16_to_f32_ieee": (f32, [C.c_uint16]), "spy_o_silu_lut": (f32, [C.c_uint16]),
        "spy_o_exp_lut": (f32, [C.c_uint16]),
        "spy_o_type_size": (i64, [i32]), "spy_o_block_size": (i64, [i32]), "spy_o_row_size": (i64, [i32, i64]),
        "spy_o_quantize_q8_0": (None, [vp, vp, i64]), "spy_o_quantize_q4_0_ggml": (None, [vp, vp, i64]),
        "spy_o_quantize_q4_0_as_written": (None, [vp, vp, i64]), "spy_o_quantize_f16": (None, [vp, vp, i64]),
        "spy_o_quantize_q4_k": (None, [vp, vp, i64]), "spy_o_quantize_q6_k": (None, [vp, vp, i64]),
        "spy_o_dequantize_q4_0": (None, [vp, vp, i64]), "spy_o_dequantize_q8_0": (None, [vp, vp, i64]),
        "spy_o_dequantize_q4_k": (None, [vp, vp, i64]), "spy_o_dequantize_q6_k": (None, [vp, vp, i64]),
        "spy_o_dot_q4_0_q8_0": (f32, [vp, vp, i64]), "spy_o_dot_q8_0_q8_0": (f32, [vp, vp, i64]),
        "spy_o_dot_f16_f16": (f32, [vp, vp, i64]),
        "spy_o_dot_q4_0_q8_0_scalar": (f32, [vp, vp, i64]), "spy_o_dot_q8_0_q8_0_scalar": (f32, [vp, vp, i64]),
        "spy_o_dot_f16_f16_scalar": (f32, [vp, vp, i64]),
        "spy_o_dot_q4_k_q8_0": (f32, [vp, vp, i64]), "spy_o_dot_q6_k_q8_0": (f32, [vp, vp, i64]),
        "spy_o_block_dots": (i32, [i32, vp, vp, i64, vp]), "spy_o_have_avx2": (i32, []),
        "spy_o_matmul": (i32, [TP, TP, TP, i32]), "spy_o_norm_rms": (i32, [TP, TP, f32]),
        "spy_o_binary": (i32, [i32, TP, TP, TP]), "spy_o_silu": (i32, [TP, TP]), "spy_o_relu": (i32, [TP, TP]), "spy_o_quantize": (i32, [TP, TP]),
        "spy_o_softmax": (i32, [TP, TP, TP, f32]), "spy_o_rope": (i32, [TP, TP, TP, C.POINTER(RopeParam)]),
        "spy_o_dup": (i32, [TP, TP]), "spy_o_contiguous": (i32, [TP, TP]), "spy_o_get_row": (i32, [TP, TP, TP]),
        "spy_o_argmax": (i32, [vp, i64]),
        "spy_o_llama_forward": (i32, [C.POINTER(Llama), vp, i32, i32, vp]),
        "spy_o_llama_tap": (None, [C.c_char_p, i32, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    return L


# ---- numpy conveniences -------------------------------------------------------------------

def quantize(L, x, ttype):
    """x: float32 array whose last axis is a multiple of the block size -> uint8 block bytes."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    n = x.size
    out = np.zeros(row_size(ttype, n), dtype=np.uint8)
    fn = {Q8_0: L.spy_o_quantize_q8_0, Q4_0: L.spy_o_quantize_q4_0_ggml, Q4_K: L.spy_o_quantize_q4_k,
          Q6_K: L.spy_o_quantize_q6_k}[ttype]
    fn(ptr(x), ptr(out), n)
    return out


def dequantize(L, q, ttype, n):
    out = np.zeros(n, dtype=np.float32)
    fn = {Q8_0: L.spy_o_dequantize_q8_0, Q4_0: L.spy_o_dequantize_q4_0, Q4_K: L.spy_o_dequantize_q4_k,
          Q6_K: L.spy_o_dequantize_q6_k}[ttype]
    fn(ptr(q), ptr(out), n)
    return out


def f32_to_f16_bits(L, x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros(x.shape, dtype=np.uint16)
    L.spy_o_quantize_f16(ptr(x), ptr(out), x.size)
    return out


def matmul(L, w_bytes, wtype, M, K, x, nthread=1):
    """w: M rows of K elements (block bytes); x: float32 [T, K] -> float32 [T, M]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    T = x.shape[0]
    out = np.zeros((T, M), dtype=np.float32)
    tw = tensor(w_bytes, wtype, [K, M])
    tx = tensor(x, F32, [K, T])
    to = tensor(out, F32, [M, T])
    rc = L.spy_o_matmul(C.byref(tw), C.byref(tx), C.byref(to), nthread)
    assert rc == 0, rc
    return out
