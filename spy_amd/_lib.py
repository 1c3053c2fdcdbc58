"""ctypes binding of libspy_hip.so -- the gfx950 kernels behind the C ABI of include/spy_hip.h.

There is no CPU fallback: every call goes to the HIP library, and a missing library or a failing
HIP call raises.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("SPY_HIP_LIBRARY") or os.path.join(HERE, "libspy_hip.so")     # override: an alternative build of the same ABI

F32, F16, Q4_0, Q8_0, Q4_K, Q6_K, I32 = 0, 1, 2, 8, 12, 14, 26
TYPE_SIZE = {F32: 4, F16: 2, Q4_0: 18, Q8_0: 34, Q4_K: 144, Q6_K: 210, I32: 4}
BLOCK_SIZE = {F32: 1, F16: 1, Q4_0: 32, Q8_0: 32, Q4_K: 256, Q6_K: 256, I32: 1}

EUNSUPPORTED, EINVAL, ENOSPACE, ETIMEOUT = -1, -2, -3, -4


def row_size(t, n):
    return n * TYPE_SIZE[t] // BLOCK_SIZE[t]


class Tensor(C.Structure):
    """spy_hip_tensor: spy::Tensor flattened to POD."""
    _fields_ = [("type", C.c_int32), ("dim", C.c_int32), ("ne", C.c_int64 * 4), ("nb", C.c_int64 * 4),
                ("data", C.c_void_p)]


class RopeParam(C.Structure):
    _fields_ = [("mode", C.c_int32), ("num_past", C.c_int32), ("num_dim", C.c_int32), ("num_context", C.c_int32),
                ("num_origin_context", C.c_int32), ("freq_base", C.c_float), ("freq_scale", C.c_float),
                ("extend_factor", C.c_float), ("attention_factor", C.c_float), ("beta_fast", C.c_float),
                ("beta_slow", C.c_float), ("xpos_base", C.c_float), ("xpos_down", C.c_int32)]


class LlamaLayer(C.Structure):
    """spy_hip_llama_layer"""
    _fields_ = [(n, C.c_void_p) for n in ("attn_norm", "ffn_norm", "wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down")] + \
               [(n, C.c_int32) for n in ("t_wq", "t_wk", "t_wv", "t_wo", "t_gate", "t_up", "t_down")]


class LlamaDesc(C.Structure):
    """spy_hip_llama_desc"""
    _fields_ = [("n_layer", C.c_int32), ("n_embd", C.c_int32), ("n_head", C.c_int32), ("n_ff", C.c_int32),
                ("n_vocab", C.c_int32), ("n_ctx", C.c_int32), ("eps", C.c_float), ("rope_freq_base", C.c_float),
                ("wtype", C.c_int32), ("tok_embd", C.c_void_p), ("t_tok_embd", C.c_int32), ("out_norm", C.c_void_p),
                ("w_out", C.c_void_p), ("t_out", C.c_int32), ("layers", C.POINTER(LlamaLayer))]


class SpyHipError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        super().__init__("%s failed: %d (%s)" % (what, code, error_string(code)))


_lib = None
_vp, _i64, _i32, _f32, _sz = C.c_void_p, C.c_int64, C.c_int32, C.c_float, C.c_size_t
_TP = C.POINTER(Tensor)

# name -> (restype, argtypes); every symbol include/spy_hip.h declares
SIGNATURES = {
    "spy_hip_init": (_i32, [_i32]),
    "spy_hip_device_info": (_i32, [C.c_char_p, _i32, C.POINTER(_i32), C.POINTER(_sz), C.POINTER(_sz)]),
    "spy_hip_alloc": (_i32, [C.POINTER(_vp), _sz]),
    "spy_hip_free": (_i32, [_vp]),
    "spy_hip_upload": (_i32, [_vp, _vp, _sz, _vp]),
    "spy_hip_download": (_i32, [_vp, _vp, _sz, _vp]),
    "spy_hip_fill_u8": (_i32, [_vp, _i32, _sz, _vp]),
    "spy_hip_sync": (_i32, [_vp]),
    "spy_hip_stream_create": (_i32, [C.POINTER(_vp)]),
    "spy_hip_stream_destroy": (_i32, [_vp]),
    "spy_hip_event_create": (_i32, [C.POINTER(_vp)]),
    "spy_hip_event_record": (_i32, [_vp, _vp]),
    "spy_hip_event_elapsed_ms": (_i32, [_vp, _vp, C.POINTER(_f32)]),
    "spy_hip_event_destroy": (_i32, [_vp]),
    "spy_hip_capture_begin": (_i32, [_vp]),
    "spy_hip_capture_end": (_i32, [_vp, C.POINTER(_vp)]),
    "spy_hip_graph_launch": (_i32, [_vp, _vp]),
    "spy_hip_graph_destroy": (_i32, [_vp]),
    "spy_hip_error_string": (C.c_char_p, [_i32]),
    "spy_hip_op_matmul_scratch_size": (_sz, [_TP, _TP]),
    "spy_hip_op_matmul": (_i32, [_vp, _TP, _TP, _TP, _vp, _sz]),
    "spy_hip_op_matmul_noalloc_max_scratch": (_sz, []),
    "spy_hip_op_matmul_noalloc": (_i32, [_vp, _TP, _TP, _TP]),
    "spy_hip_op_norm_rms": (_i32, [_vp, _TP, _TP, _f32]),
    "spy_hip_op_binary": (_i32, [_vp, _i32, _TP, _TP, _TP]),
    "spy_hip_op_silu": (_i32, [_vp, _TP, _TP]),
    "spy_hip_op_relu": (_i32, [_vp, _TP, _TP]),
    "spy_hip_op_quantize": (_i32, [_vp, _TP, _TP]),
    "spy_hip_op_softmax": (_i32, [_vp, _TP, _TP, _TP, _f32]),
    "spy_hip_op_rope": (_i32, [_vp, _TP, _TP, _TP, C.POINTER(RopeParam)]),
    "spy_hip_rope_prepare": (_i32, [C.POINTER(RopeParam), _i64]),
    "spy_hip_op_dup": (_i32, [_vp, _TP, _TP]),
    "spy_hip_op_contiguous": (_i32, [_vp, _TP, _TP]),
    "spy_hip_op_get_row": (_i32, [_vp, _TP, _TP, _TP]),
    "spy_hip_take_error": (_i32, [C.POINTER(_i32)]),
    "spy_hip_set_exact_order": (_i32, [_i32]),
    "spy_hip_argmax": (_i32, [_vp, _vp, _i64, _vp]),
    "spy_hip_quantize_q8_0": (_i32, [_vp, _vp, _i64, _vp, _i64, _i64]),
    "spy_hip_quantize_f16": (_i32, [_vp, _vp, _i64, _vp, _i64, _i64]),
    "spy_hip_gemv_q8_0act": (_i32, [_vp, _i32, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64]),
    "spy_hip_gemm_q8_0act": (_i32, [_vp, _i32, _vp, _vp, _vp, _i64, _i64, _i64, _i64]),
    "spy_hip_prompt_attention": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i64, C.c_float]),
    "spy_hip_prompt_attention_exact_scratch_size": (_sz, [_i32, _i32, _i32]),
    "spy_hip_prompt_attention_exact": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i64, _i32, C.c_float, _vp, _sz]),
    "spy_hip_block_dots": (_i32, [_vp, _i32, _vp, _vp, _vp, _i64, _i64]),
    "spy_hip_rmsnorm_q8_0": (_i32, [_vp, _i32, _vp, _vp, _f32, _i64, _vp]),
    "spy_hip_rope_kvwrite": (_i32, [_vp, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _f32, _i32, _i32, _i32, _i64, _vp, _vp, _vp, _vp, _vp]),
    "spy_hip_attn_decode": (_i32, [_vp, _i32, _vp, _vp, _vp, _i32, _i32, _i64, _vp, _vp]),
    "spy_hip_gemv_fused": (_i32, [_vp, _i32, _i32, _vp, _vp, _vp, _f32, _vp, _vp, _i64, _i64, _vp]),
    "spy_hip_ffn_gate_up_silu": (_i32, [_vp, _i32, _i32, _vp, _vp, _vp, _vp, _f32, _vp, _i64, _i64, _vp]),
    "spy_hip_measure_mfma_i8": (_i32, [_vp, _i32, C.POINTER(_f32)]),
    "spy_hip_running_sum_f32": (_i32, [_vp, _vp, _i64, _i32, _vp]),
    "spy_hip_measure_mfma_i8_scaled": (_i32, [_vp, _i32, _i32, C.POINTER(_f32)]),
    "spy_hip_measure_hbm_read": (_i32, [_vp, _vp, _sz, _i32, C.POINTER(_f32)]),
    "spy_hip_llama_create": (_i32, [C.POINTER(LlamaDesc), C.POINTER(_vp)]),
    "spy_hip_llama_destroy": (_i32, [_vp]),
    "spy_hip_llama_forward": (_i32, [_vp, _vp, _vp, _i32, _i32, _vp]),
    "spy_hip_llama_forward_last": (_i32, [_vp, _vp, _vp, _i32, _i32, _vp]),
    "spy_hip_llama_decode_greedy": (_i32, [_vp, _vp, _i32, _i32, _i32, _vp, _i32]),
    "spy_hip_llama_set_order": (_i32, [_vp, _i32]),
    "spy_hip_llama_order": (_i32, [_vp]),
    "spy_hip_llama_set_spin_limit": (_i32, [_vp, C.c_uint32]),
    "spy_hip_llama_buffer": (_i32, [_vp, C.c_char_p, _i32, C.POINTER(_vp), C.POINTER(_sz)]),
    "spy_hip_llama_timing": (_i32, [_vp, C.POINTER(_f32), C.POINTER(_i32)]),
    "spy_hip_llama_single_kernel": (_i32, [_vp]),
    "spy_hip_llama_kernel_time": (_i32, [_vp, _vp, C.c_char_p, _i32, C.POINTER(_f32)]),
}


def load():
    """Load the in-tree HIP library. Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("%s is missing: build it with `make -C spy_amd/csrc` (or __graft_entry__.build()); "
                           "there is no CPU fallback" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(L, name)            # AttributeError here = header and library out of step
        fn.restype, fn.argtypes = res, args
    _lib = L
    return L


def error_string(code):
    return load().spy_hip_error_string(code).decode()


def check(code, what="spy_hip call"):
    if code != 0:
        raise SpyHipError(code, what)


_inited = False


def init(device_id=0):
    global _inited
    check(load().spy_hip_init(device_id), "spy_hip_init")
    _inited = True


def device_info():
    name = C.create_string_buffer(256)
    cu, tot, free = _i32(), _sz(), _sz()
    check(load().spy_hip_device_info(name, 256, C.byref(cu), C.byref(tot), C.byref(free)), "spy_hip_device_info")
    return {"name": name.value.decode(), "num_cu": cu.value, "total_mem": tot.value, "free_mem": free.value}


class DeviceBuffer:
    """Device memory obtained through spy_hip_alloc; freed with the object."""

    def __init__(self, nbytes):
        if not _inited:
            init(0)
        self.nbytes = int(nbytes)
        p = _vp()
        check(load().spy_hip_alloc(C.byref(p), max(self.nbytes, 1)), "spy_hip_alloc")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, arr):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        buf.upload(arr)
        return buf

    def upload(self, arr, offset=0):
        arr = np.ascontiguousarray(arr)
        assert offset + arr.nbytes <= self.nbytes
        check(load().spy_hip_upload(self.ptr + offset, arr.ctypes.data, arr.nbytes, None), "spy_hip_upload")

    def download(self, dtype, count=None, offset=0):
        dtype = np.dtype(dtype)
        if count is None:
            count = (self.nbytes - offset) // dtype.itemsize
        out = np.empty(count, dtype=dtype)
        assert offset + out.nbytes <= self.nbytes
        check(load().spy_hip_download(out.ctypes.data, self.ptr + offset, out.nbytes, None), "spy_hip_download")
        return out

    def fill(self, value=0):
        check(load().spy_hip_fill_u8(self.ptr, value, self.nbytes, None), "spy_hip_fill_u8")

    def free(self):
        if getattr(self, "ptr", None):
            load().spy_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def tensor(buf, ttype, ne, nb=None, offset=0):
    """Describe device memory (DeviceBuffer or raw pointer) as a spy_hip_tensor."""
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
    base = buf.ptr if isinstance(buf, DeviceBuffer) else int(buf)
    t.data = base + offset
    t._keep = buf
    return t


def sync(stream=None):
    check(load().spy_hip_sync(stream), "spy_hip_sync")
