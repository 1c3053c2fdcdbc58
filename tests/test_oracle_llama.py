"""Pins the oracle's LLaMA forward pass (operator sequence, residuals, cache layouts, mask) against
an independent dense fp64 implementation of the architecture, and the package's synthetic-model
generator against the oracle's quantizers."""
import numpy as np
import pytest

from tests import oracle_lib as O


def _dense_forward(cfg, tensors, L, tokens, kc, vc, n_past):
    """Textbook LLaMA in fp64 on the dequantised weights (no Q8_0 activations, no fp16 rounding);
    kc / vc: python lists of [n_ctx, d] arrays holding past K / V."""
    d, H, F = cfg.n_embd, cfg.n_head, cfg.n_ff
    hd = d // H

    def W(name, rows, cols, t):
        if t == O.F32:
            return tensors[name].view(np.float32).reshape(rows, cols).astype(np.float64)
        return O.dequantize(L, tensors[name], t, rows * cols).reshape(rows, cols).astype(np.float64)

    def norm(x, w):
        return x / np.sqrt((x ** 2).mean(axis=-1, keepdims=True) + cfg.eps) * w

    def rope(x, pos):                                   # x [T, H, hd], adjacent pairs
        k = np.arange(hd // 2)
        th = pos[:, None] * cfg.rope_freq_base ** (-2.0 * k / hd)[None, :]
        c, s = np.cos(th)[:, None, :], np.sin(th)[:, None, :]
        out = np.empty_like(x)
        out[..., 0::2] = x[..., 0::2] * c - x[..., 1::2] * s
        out[..., 1::2] = x[..., 0::2] * s + x[..., 1::2] * c
        return out

    T = len(tokens)
    pos = np.arange(n_past, n_past + T, dtype=np.float64)
    x = W("token_embd.weight", cfg.n_vocab, d, cfg.t_tok_embd)[tokens]
    for il in range(cfg.n_layer):
        p = "blk.%d." % il
        xn = norm(x, tensors[p + "attn_norm.weight"].view(np.float32).astype(np.float64))
        q = rope((xn @ W(p + "attn_q.weight", d, d, cfg.wtype).T).reshape(T, H, hd), pos)
        k = rope((xn @ W(p + "attn_k.weight", d, d, cfg.wtype).T).reshape(T, H, hd), pos)
        v = (xn @ W(p + "attn_v.weight", d, d, cfg.wtype).T)
        kc[il][n_past:n_past + T] = k.reshape(T, d)
        vc[il][n_past:n_past + T] = v
        n_kv = n_past + T
        K = kc[il][:n_kv].reshape(n_kv, H, hd)
        V = vc[il][:n_kv].reshape(n_kv, H, hd)
        s = np.einsum("thd,jhd->htj", q, K) / np.sqrt(hd)
        for i in range(T):
            s[:, i, n_past + i + 1:] = -np.inf
        pr = np.exp(s - s.max(axis=-1, keepdims=True))
        pr /= pr.sum(axis=-1, keepdims=True)
        o = np.einsum("htj,jhd->thd", pr, V).reshape(T, d)
        x1 = o @ W(p + "attn_output.weight", d, d, cfg.wtype).T + x
        xn = norm(x1, tensors[p + "ffn_norm.weight"].view(np.float32).astype(np.float64))
        g = xn @ W(p + "ffn_gate.weight", F, d, cfg.wtype).T
        u = xn @ W(p + "ffn_up.weight", F, d, cfg.wtype).T
        x = (u * (g / (1 + np.exp(-g)))) @ W(p + "ffn_down.weight", d, F, cfg.wtype).T + x1
    xn = norm(x, tensors["output_norm.weight"].view(np.float32).astype(np.float64))
    return xn @ W("output.weight", cfg.n_vocab, d, cfg.t_out).T


@pytest.mark.parametrize("wtype,t_emb", [(O.Q8_0, O.Q8_0), (O.Q4_0, O.F32)])
def test_oracle_forward_matches_dense_architecture(oracle, wtype, t_emb):
    from spy_amd import model as M
    from tests.model_util import OracleModel
    cfg = M.Config(n_layer=2, n_embd=128, n_head=2, n_ff=256, n_vocab=96, n_ctx=16, wtype=wtype, t_tok_embd=t_emb)
    tensors = M.synth_model(cfg, seed=3, std=0.08)
    ora = OracleModel(cfg, tensors, nthread=2)
    kc = [np.zeros((cfg.n_ctx, cfg.n_embd)) for _ in range(cfg.n_layer)]
    vc = [np.zeros((cfg.n_ctx, cfg.n_embd)) for _ in range(cfg.n_layer)]
    prompt = np.array([5, 17, 90, 3], dtype=np.int32)
    got = ora.forward(prompt, 0)
    want = _dense_forward(cfg, tensors, oracle, prompt, kc, vc, 0)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() < 0.03 * scale          # Q8_0 activations + fp16 rounding points
    assert np.corrcoef(got.ravel(), want.ravel())[0, 1] > 0.999
    # second pass: one token on top of the cache (n_past = 4)
    got1 = ora.forward(np.array([42], np.int32), 4)
    want1 = _dense_forward(cfg, tensors, oracle, np.array([42]), kc, vc, 4)
    assert np.abs(got1 - want1).max() < 0.03 * np.abs(want1).max()
    # cache layouts: K [token][head][hd] fp16, V transposed [d][n_ctx] fp16
    k0 = ora.k_cache[0].view(np.float16).astype(np.float64).reshape(cfg.n_ctx, cfg.n_embd)
    v0 = ora.v_cache[0].view(np.float16).astype(np.float64).reshape(cfg.n_embd, cfg.n_ctx)
    assert np.abs(k0[:5] - kc[0][:5]).max() < 0.03 * np.abs(kc[0][:5]).max()
    assert np.abs(v0[:, :5].T - vc[0][:5]).max() < 0.03 * np.abs(vc[0][:5]).max()
    assert not k0[5:].any() and not v0[:, 5:].any()
    # chunked prefill == one pass (each token only sees the cache before it)
    ora2 = OracleModel(cfg, tensors, nthread=1)
    a = ora2.forward(prompt[:3], 0); b = ora2.forward(prompt[3:], 3)
    assert np.array_equal(np.concatenate([a, b]), got)
    # context overflow is refused (llama.cpp:249)
    assert oracle.spy_o_llama_forward(ora.m, np.arange(20, dtype=np.int32).ctypes.data, 20, 0, np.zeros((20, 96), np.float32).ctypes.data) == 8


def test_synth_generator_is_reproducible_and_matches_oracle_quantizers(oracle):
    from spy_amd import model as M
    S = M.synth_lib()
    n = 32 * 4096
    x = np.empty(n, np.float32)
    S.spy_synth_f32(99, n, 0.02, x.ctypes.data)
    y = np.empty(n, np.float32)
    S.spy_synth_f32(99, n, 0.02, y.ctypes.data)
    assert np.array_equal(x, y)
    assert abs(float(x.std()) - 0.02) < 4e-4 and abs(float(x.mean())) < 3e-4
    assert abs(float(((x / 0.02) ** 4).mean()) - 2.9) < 0.15          # 12-term sum: kurtosis 3 - 0.1
    # the package's GGUF quantizers produce the oracle's bytes
    for t in (O.Q4_0, O.Q8_0):
        out = np.empty(O.row_size(t, n), np.uint8)
        assert S.spy_synth_quantize(t, x.ctypes.data, n, out.ctypes.data) == out.nbytes
        assert np.array_equal(out, O.quantize(oracle, x, t))
        # fused generate+quantize == generate then quantize
        out2 = np.empty_like(out)
        assert S.spy_synth_tensor(t, 99, n, 0.02, 0, 20.0, out2.ctypes.data) == out.nbytes
        assert np.array_equal(out, out2)
    # named streams differ, same name repeats
    a = M.synth_tensor(O.Q4_0, 1, "blk.0.attn_q.weight", 4096)
    assert np.array_equal(a, M.synth_tensor(O.Q4_0, 1, "blk.0.attn_q.weight", 4096))
    assert not np.array_equal(a, M.synth_tensor(O.Q4_0, 1, "blk.1.attn_q.weight", 4096))
    # byte accounting of the 7B Q4_0 model: 3 717 545 984 bytes streamed per token
    assert M.Config.llama2_7b().weight_bytes() == 3717545984
