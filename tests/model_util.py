"""Runs the CPU oracle's LLaMA forward pass on the same tensors the HIP engine gets."""
import ctypes as C

import numpy as np

from tests import oracle_lib as O

_FIELDS = [("attn_norm", "attn_norm", None), ("ffn_norm", "ffn_norm", None), ("wq", "attn_q", "t_wq"), ("wk", "attn_k", "t_wk"),
           ("wv", "attn_v", "t_wv"), ("wo", "attn_output", "t_wo"), ("w_gate", "ffn_gate", "t_gate"), ("w_up", "ffn_up", "t_up"),
           ("w_down", "ffn_down", "t_down")]


class OracleModel:
    """The reference's token loop (cli.h:60-129 in the Spy tree) on the CPU oracle."""

    def __init__(self, cfg, tensors, nthread=8, lib=None):
        self.cfg, self.tensors, self.L = cfg, tensors, lib if lib is not None else O.load()
        self.layers = (O.LlamaLayer * cfg.n_layer)()
        for i in range(cfg.n_layer):
            for field, gname, tfield in _FIELDS:
                setattr(self.layers[i], field, tensors["blk.%d.%s.weight" % (i, gname)].ctypes.data)
                if tfield:
                    setattr(self.layers[i], tfield, cfg.tensor_types.get(gname, cfg.wtype))
        d, Cx = cfg.n_embd, cfg.n_ctx
        self.k_cache = [np.zeros(Cx * d, dtype=np.uint16) for _ in range(cfg.n_layer)]
        self.v_cache = [np.zeros(Cx * d, dtype=np.uint16) for _ in range(cfg.n_layer)]
        self._kp = (C.c_void_p * cfg.n_layer)(*[a.ctypes.data for a in self.k_cache])
        self._vp = (C.c_void_p * cfg.n_layer)(*[a.ctypes.data for a in self.v_cache])
        m = O.Llama()
        m.n_layer, m.n_embd, m.n_head, m.n_ff, m.n_vocab, m.n_ctx = cfg.n_layer, d, cfg.n_head, cfg.n_ff, cfg.n_vocab, Cx
        m.eps, m.rope_freq_base, m.nthread = cfg.eps, cfg.rope_freq_base, nthread
        m.tok_embd, m.t_tok_embd = tensors["token_embd.weight"].ctypes.data, cfg.t_tok_embd
        m.out_norm = tensors["output_norm.weight"].ctypes.data
        m.w_out, m.t_out = tensors["output.weight"].ctypes.data, cfg.t_out
        m.layers = self.layers
        m.k_cache = C.cast(self._kp, C.POINTER(C.c_void_p))
        m.v_cache = C.cast(self._vp, C.POINTER(C.c_void_p))
        self.m = m

    def forward(self, tokens, n_past):
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        logits = np.zeros((len(tokens), self.cfg.n_vocab), dtype=np.float32)
        rc = self.L.spy_o_llama_forward(C.byref(self.m), tokens.ctypes.data, len(tokens), n_past, logits.ctypes.data)
        assert rc == 0, rc
        return logits

    def tap(self, name, layer, n):
        buf = np.zeros(n, dtype=np.float32)
        self.L.spy_o_llama_tap(name.encode(), layer, buf.ctypes.data)
        self._taps = getattr(self, "_taps", []) + [buf, name]
        return buf

    def clear_taps(self):
        self.L.spy_o_llama_tap(None, 0, None)

    def generate(self, prompt, n_predict, margins=None):
        """prefill + greedy loop; optionally records the top-1/top-2 logit margin of every step"""
        prompt = np.asarray(prompt, dtype=np.int32)
        out = []
        logits = self.forward(prompt, 0)[-1]
        pos = len(prompt)
        for _ in range(n_predict):
            tok = int(self.L.spy_o_argmax(logits.ctypes.data, logits.size))
            if margins is not None:
                top2 = np.partition(logits, -2)[-2:]
                margins.append(float(top2[1] - top2[0]))
            out.append(tok)
            if len(out) == n_predict:
                break
            logits = self.forward(np.array([tok], dtype=np.int32), pos)[0]
            pos += 1
        return np.array(out, dtype=np.int32)


def k_quant_quantizer(x, ttype):
    """Q4_K / Q6_K blocks for synthetic models: the oracle's project-defined quantizers (the
    reference has none)."""
    return O.quantize(O.load(), x, ttype)
