"""Host side of the token loop: LLaMA-2 shaped models (synthetic, GGUF tensor names and native
block layouts), their upload to HBM, and the engine behind spy_hip_llama_*.

Mirrors what the reference spreads over LLAMAModel::build_graph (model/src/llm/model/llama.cpp in
the Spy tree), the simple loader and AutoModelGenerator::generate (app/cli/include/cli.h:60-129):
load tensors by name, run one prefill pass, then greedy single-token passes.
"""
import ctypes as C
import os

import numpy as np

from . import _lib as H

HERE = os.path.dirname(os.path.abspath(__file__))
SYNTH_PATH = os.path.join(HERE, "libspy_synth.so")


class Config:
    def __init__(self, n_layer=32, n_embd=4096, n_head=32, n_ff=11008, n_vocab=32000, n_ctx=4096, eps=1e-5,
                 rope_freq_base=10000.0, wtype=H.Q4_0, t_out=None, t_tok_embd=H.F32, tensor_types=None):
        self.n_layer, self.n_embd, self.n_head, self.n_ff = n_layer, n_embd, n_head, n_ff
        self.n_vocab, self.n_ctx, self.eps, self.rope_freq_base = n_vocab, n_ctx, eps, rope_freq_base
        self.wtype = wtype
        self.t_out = wtype if t_out is None else t_out
        self.t_tok_embd = t_tok_embd
        # per-tensor overrides of the layer-weight type, e.g. {"attn_v": Q6_K, "ffn_down": Q6_K} for a
        # Q4_K_M-style mix; only the operator-by-operator path takes mixed layers
        self.tensor_types = dict(tensor_types or {})

    @classmethod
    def llama2_7b(cls, n_ctx=4352, wtype=H.Q4_0, **kw):
        return cls(32, 4096, 32, 11008, 32000, n_ctx, 1e-5, 10000.0, wtype, **kw)

    def tensor_shapes(self):
        """name -> (type, rows, cols) in GGUF naming; cols is the contiguous dimension."""
        d, F, V = self.n_embd, self.n_ff, self.n_vocab
        out = {"token_embd.weight": (self.t_tok_embd, V, d), "output_norm.weight": (H.F32, 1, d),
               "output.weight": (self.t_out, V, d)}
        for i in range(self.n_layer):
            p = "blk.%d." % i
            out[p + "attn_norm.weight"] = (H.F32, 1, d)
            out[p + "ffn_norm.weight"] = (H.F32, 1, d)
            tt = lambda n: self.tensor_types.get(n, self.wtype)
            for n in ("attn_q", "attn_k", "attn_v", "attn_output"):
                out[p + n + ".weight"] = (tt(n), d, d)
            out[p + "ffn_gate.weight"] = (tt("ffn_gate"), F, d)
            out[p + "ffn_up.weight"] = (tt("ffn_up"), F, d)
            out[p + "ffn_down.weight"] = (tt("ffn_down"), d, F)
        return out

    def weight_bytes(self):
        """bytes of weights one single-token pass reads (the embedding table contributes one row)"""
        return sum(H.row_size(t, r * c) for n, (t, r, c) in self.tensor_shapes().items() if n != "token_embd.weight")


_synth = None


def synth_lib():
    global _synth
    if _synth is None:
        if not os.path.exists(SYNTH_PATH):
            raise RuntimeError("%s is missing: build it with `make -C spy_amd/csrc`" % SYNTH_PATH)
        L = C.CDLL(SYNTH_PATH)
        L.spy_synth_quantize.restype = C.c_size_t
        L.spy_synth_quantize.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p]
        L.spy_synth_f32.restype = None
        L.spy_synth_f32.argtypes = [C.c_uint64, C.c_int64, C.c_float, C.c_void_p]
        L.spy_synth_tensor.restype = C.c_size_t
        L.spy_synth_tensor.argtypes = [C.c_int, C.c_uint64, C.c_int64, C.c_float, C.c_int64, C.c_float, C.c_void_p]
        _synth = L
    return _synth


def _name_seed(seed, name):
    h = 1469598103934665603
    for ch in ("%d/%s" % (seed, name)).encode():
        h = ((h ^ ch) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


def synth_tensor(ttype, seed, name, n, std=0.02, outlier_every=0, outlier_mul=20.0, quantizer=None):
    """n elements of the named stream (~N(0, std), every outlier_every-th element x outlier_mul), stored as `ttype`
    blocks: F32, Q4_0, Q8_0 by the block rules the reference's host backend decodes, Q4_K / Q6_K by this package's own
    one-pass rule (the reference holds their layouts only).  `quantizer` (callable(float32 array, type) -> uint8 bytes)
    replaces the built-in rule where given."""
    S = synth_lib()
    s = _name_seed(seed, name)
    if quantizer is None or ttype in (H.F32, H.Q4_0, H.Q8_0):
        out = np.empty(H.row_size(ttype, n), dtype=np.uint8)
        got = S.spy_synth_tensor(ttype, s, n, std, outlier_every, outlier_mul, out.ctypes.data)
        assert got == out.nbytes, (ttype, n)
        return out
    x = np.empty(n, dtype=np.float32)
    S.spy_synth_tensor(H.F32, s, n, std, outlier_every, outlier_mul, x.ctypes.data)
    return quantizer(x, ttype)


def quantize(x, ttype):
    """float32 array -> block bytes of `ttype` (F32, Q4_0, Q8_0, Q4_K, Q6_K) by the package's own quantizers"""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(H.row_size(ttype, x.size), dtype=np.uint8)
    got = synth_lib().spy_synth_quantize(ttype, x.ctypes.data, x.size, out.ctypes.data)
    assert got == out.nbytes, (ttype, x.size)
    return out


def synth_model(cfg, seed=1234, std=0.02, outlier_every=0, quantizer=None, norm_jitter=0.1):
    """Random-init weights of the LLaMA-2 architecture: matrices ~N(0, std) (12-term integer
    approximation, bit-reproducible), norm weights 1 + N(0, norm_jitter), quantized with the GGUF
    block rules.  Returns {name: uint8 array}."""
    tensors = {}
    for name, (t, rows, cols) in cfg.tensor_shapes().items():
        if "norm" in name:
            w = np.frombuffer(synth_tensor(H.F32, seed, name, cols, norm_jitter).tobytes(), dtype=np.float32) + np.float32(1.0)
            tensors[name] = np.ascontiguousarray(w.astype(np.float32)).view(np.uint8)
        elif name == "token_embd.weight":
            tensors[name] = synth_tensor(t, seed, name, rows * cols, 1.0, 0, 20.0, quantizer)
        else:
            tensors[name] = synth_tensor(t, seed, name, rows * cols, std, outlier_every, 20.0, quantizer)
    return tensors


LlamaLayer, LlamaDesc = H.LlamaLayer, H.LlamaDesc

_LAYER_TYPES = [("t_wq", "attn_q"), ("t_wk", "attn_k"), ("t_wv", "attn_v"), ("t_wo", "attn_output"), ("t_gate", "ffn_gate"),
                ("t_up", "ffn_up"), ("t_down", "ffn_down")]
_LAYER_FIELDS = [("attn_norm", "attn_norm"), ("ffn_norm", "ffn_norm"), ("wq", "attn_q"), ("wk", "attn_k"), ("wv", "attn_v"),
                 ("wo", "attn_output"), ("w_gate", "ffn_gate"), ("w_up", "ffn_up"), ("w_down", "ffn_down")]


class Engine:
    """A model resident in HBM (native block layouts, uploaded once) and its token loop."""

    def __init__(self, cfg, tensors, device_id=0, order=None):
        """order: summation order of the fused single-token pass, 1 = the host backend's (bit-exact results), 0 = this
        backend's own, None = the library's default (1 where the kernels take the model)"""
        H.init(device_id)
        self.cfg = cfg
        self.L = H.load()
        self.dev = {}
        for name, (t, rows, cols) in cfg.tensor_shapes().items():
            arr = tensors[name]
            assert arr.nbytes == H.row_size(t, rows * cols), name
            self.dev[name] = H.DeviceBuffer.from_numpy(arr)
        self._layers = (LlamaLayer * cfg.n_layer)()
        for i in range(cfg.n_layer):
            for field, gname in _LAYER_FIELDS:
                setattr(self._layers[i], field, self.dev["blk.%d.%s.weight" % (i, gname)].ptr)
            for tfield, gname in _LAYER_TYPES:
                setattr(self._layers[i], tfield, cfg.tensor_types.get(gname, 0))
        d = LlamaDesc(cfg.n_layer, cfg.n_embd, cfg.n_head, cfg.n_ff, cfg.n_vocab, cfg.n_ctx, cfg.eps, cfg.rope_freq_base,
                      cfg.wtype, self.dev["token_embd.weight"].ptr, cfg.t_tok_embd, self.dev["output_norm.weight"].ptr,
                      self.dev["output.weight"].ptr, cfg.t_out, self._layers)
        self._desc = d
        h = C.c_void_p()
        H.check(self.L.spy_hip_llama_create(C.byref(d), C.byref(h)), "spy_hip_llama_create")
        self.handle = h
        if order is not None:
            self.set_order(order)

    def set_order(self, order):
        H.check(self.L.spy_hip_llama_set_order(self.handle, int(order)), "spy_hip_llama_set_order")

    def order(self):
        return self.L.spy_hip_llama_order(self.handle)

    def forward(self, tokens, n_past, want_logits=True):
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        logits = np.empty((len(tokens), self.cfg.n_vocab), dtype=np.float32) if want_logits else None
        H.check(self.L.spy_hip_llama_forward(self.handle, None, tokens.ctypes.data, len(tokens), n_past,
                                             logits.ctypes.data if want_logits else None), "spy_hip_llama_forward")
        return logits

    def forward_last(self, tokens, n_past):
        """The pass of forward() with the output head on the last token only: n_vocab logits."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        logits = np.empty(self.cfg.n_vocab, dtype=np.float32)
        H.check(self.L.spy_hip_llama_forward_last(self.handle, None, tokens.ctypes.data, len(tokens), n_past, logits.ctypes.data),
                "spy_hip_llama_forward_last")
        return logits

    def decode_greedy(self, first_token, n_past, n_steps, use_graph=True):
        out = np.empty(n_steps, dtype=np.int32)
        H.check(self.L.spy_hip_llama_decode_greedy(self.handle, None, int(first_token), int(n_past), int(n_steps),
                                                   out.ctypes.data, 1 if use_graph else 0), "spy_hip_llama_decode_greedy")
        return out

    def set_spin_limit(self, polls):
        """polls a bounded wait between workgroups may spend before the pass gives up (ETIMEOUT)"""
        H.check(self.L.spy_hip_llama_set_spin_limit(self.handle, int(polls)), "spy_hip_llama_set_spin_limit")

    def fuses_attention(self):
        """True when qkv, scores and softmax + KQV of a layer run as one launch"""
        return (self.L.spy_hip_llama_single_kernel(self.handle) & 2) == 2

    def timing(self):
        ms, n = C.c_float(), C.c_int32()
        H.check(self.L.spy_hip_llama_timing(self.handle, C.byref(ms), C.byref(n)), "spy_hip_llama_timing")
        return ms.value, n.value

    def kernel_time_us(self, which, reps=4):
        us = C.c_float()
        H.check(self.L.spy_hip_llama_kernel_time(self.handle, None, which.encode(), reps, C.byref(us)), "spy_hip_llama_kernel_time")
        return us.value

    def buffer(self, name, layer=0):
        p, n = C.c_void_p(), C.c_size_t()
        H.check(self.L.spy_hip_llama_buffer(self.handle, name.encode(), layer, C.byref(p), C.byref(n)), "spy_hip_llama_buffer")
        return p.value, n.value

    def read_buffer(self, name, layer=0, dtype=np.uint8):
        p, n = self.buffer(name, layer)
        out = np.empty(n // np.dtype(dtype).itemsize, dtype=dtype)
        H.check(self.L.spy_hip_download(out.ctypes.data, p, n, None), "spy_hip_download")
        return out

    def write_buffer(self, name, layer, arr):
        p, n = self.buffer(name, layer)
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= n
        H.check(self.L.spy_hip_upload(p, arr.ctypes.data, arr.nbytes, None), "spy_hip_upload")

    def generate(self, prompt_tokens, n_predict):
        """Prefill + greedy loop of AutoModelGenerator::generate (cli.h:60-129): returns the
        n_predict sampled tokens."""
        prompt = np.asarray(prompt_tokens, dtype=np.int32)
        logits = self.forward_last(prompt, 0)
        first = int(np.argmax(logits))              # np.argmax returns the first maximum, like greedy.h:20-25
        if n_predict == 1:
            return np.array([first], dtype=np.int32)
        rest = self.decode_greedy(first, len(prompt), n_predict - 1)
        return np.concatenate([[first], rest]).astype(np.int32)

    def close(self):
        if getattr(self, "handle", None):
            self.L.spy_hip_llama_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
