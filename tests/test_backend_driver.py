"""The C++ host side: spy::hip::HIPBackend driven through Backend::submit, one call per graph node,
exactly as the reference's scheduler drives a backend (default_scheduler.h:46-229 in the Spy tree)."""
import os
import re

import numpy as np
import pytest

from tests import oracle_lib as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_driver_library_exports_header_symbols():
    from spy_amd import backend_driver as B
    text = open(os.path.join(ROOT, "include", "spy_backend_driver.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(spy_host_[a-z0-9_]+)\s*\(", text)))
    L = B.load()
    assert names == sorted(B.SIGNATURES)
    for n in names:
        assert hasattr(L, n)


def test_unknown_backend_name_is_rejected():
    """BackendFactory::init_backend returns no backend for a name nobody registered (backend.h:171-179);
    the lookup happens before any device call."""
    from spy_amd import backend_driver as B
    from spy_amd import model as M
    cfg = M.Config(n_layer=1, n_embd=64, n_head=2, n_ff=96, n_vocab=64, n_ctx=16, wtype=O.Q4_0)
    tensors = M.synth_model(cfg, seed=1)
    with pytest.raises(RuntimeError, match="-1"):
        B.HostModel(cfg, tensors, backend="cuda:default")


@pytest.mark.gpu
@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0])
def test_submit_path_matches_oracle_and_engine(wtype):
    from spy_amd import backend_driver as B
    from spy_amd import model as M
    from tests.gpu_util import assert_close
    from tests.model_util import OracleModel
    cfg = M.Config(n_layer=2, n_embd=256, n_head=2, n_ff=768, n_vocab=512, n_ctx=64, wtype=wtype)
    tensors = M.synth_model(cfg, seed=7)
    host, eng, ora = B.HostModel(cfg, tensors), M.Engine(cfg, tensors, order=0), OracleModel(cfg, tensors)
    prompt = np.random.default_rng(3).integers(0, cfg.n_vocab, 6).astype(np.int32)
    lg_h, lg_e, lg_o = host.forward(prompt, 0), eng.forward(prompt, 0), ora.forward(prompt, 0)
    assert_close(lg_h, lg_o, "submit-path prefill logits vs oracle")
    assert np.array_equal(lg_h, lg_e), "the submit path and the engine's prefill in its own order launch the same operator kernels"
    # the engine in the host's order (its default) issues the same operators in their exact forms: the oracle's bits
    eng1 = M.Engine(cfg, tensors)
    assert eng1.order() == 1
    assert np.array_equal(eng1.forward(prompt, 0).view(np.uint32), lg_o.view(np.uint32)), "prompt pass of an engine in order 1: the oracle's bits"
    eng1.close()
    st = host.stats()
    assert st["n_ops"] == 33 * cfg.n_layer + 4 and st["n_submit"] == st["n_ops"]      # 33 operators per layer + embedding + 3 head ops
    assert st["n_alloc"] == st["n_free"] > 0, st                                   # every Dynamic tensor went back to the pool (default_scheduler.h:186-228)
    for il in range(cfg.n_layer):
        for which, ref in ((0, ora.k_cache[il]), (1, ora.v_cache[il])):
            got = host.cache(il, which).view(np.float16).astype(np.float32)
            assert_close(got, ref.view(np.float16).astype(np.float32), "layer %d cache %d" % (il, which), 2e-3)
    # single-token steps on top of the cache, through submit again
    tok = int(np.argmax(lg_o[-1]))
    for step in range(3):
        t = np.array([tok], np.int32)
        lh, lo = host.forward(t, 6 + step)[0], ora.forward(t, 6 + step)[0]
        assert_close(lh, lo, "submit-path decode step %d" % step, 3e-3)
        tok = int(np.argmax(lo))
    st2 = host.stats()
    assert st2["n_alloc"] == st2["n_free"], st2
    host.close()
    eng.close()


@pytest.mark.gpu
@pytest.mark.parametrize("passes", [((0, 168), (168, 304), (304, 438)), ((0, 64),), ((0, 17), (17, 100), (100, 163)), ((0, 130), (130, 131), (131, 200))])
def test_engine_fused_prompt_attention_against_submit_path(passes):
    """Default prompt pass of the engine: scores, masked softmax and P.V^T of a layer in one kernel (no score matrix in
    memory).  Same arithmetic per element as the three operators of the submit path except for the order in which a
    row's exponentials are added: a probability now and then lands on the other side of an fp16 rounding boundary
    (tests/test_gpu_ops.py bounds that at the kernel), and the Q8_0 re-quantization of the following MatMuls turns such
    a difference into their rounding noise, as for any two implementations whose sums are not bit-identical.  Hence a
    bound at that noise level (5e-3 of the largest logit) and the same argmax on nearly every row.  Tile edges: passes
    that are not multiples of 64 tokens, caches that are not multiples of 64 positions, a single-token pass (the fused
    single-token kernels) in between."""
    from spy_amd import backend_driver as B
    from spy_amd import model as M
    from tests.gpu_util import rel_err
    cfg = M.Config(n_layer=2, n_embd=256, n_head=2, n_ff=768, n_vocab=512, n_ctx=448, wtype=O.Q4_0)
    tensors = M.synth_model(cfg, seed=11)
    host, eng = B.HostModel(cfg, tensors), M.Engine(cfg, tensors)
    prompt = np.random.default_rng(5).integers(0, cfg.n_vocab, passes[-1][1]).astype(np.int32)
    for start, stop in passes:
        print("pass", start, stop, flush=True)
        lg_h, lg_e = host.forward(prompt[start:stop], start), eng.forward(prompt[start:stop], start)
        assert np.isfinite(lg_e).all()
        err = rel_err(lg_e, lg_h)
        print("  max-abs err / max |logit| = %.2e" % err, flush=True)
        assert err < 5e-3, (start, stop, err)
        assert (np.argmax(lg_e, axis=1) == np.argmax(lg_h, axis=1)).mean() > 0.98
    host.close()


@pytest.mark.gpu
def test_engine_prompt_softmax_without_mask_tensor_matches_submit_path(monkeypatch):
    """The engine's prompt pass tells its softmax and its two attention products the causal shape as a number (no
    mask tensor read, tiles above the diagonal left out) and hands the probabilities over as fp16; the submit path
    runs MatMul / Softmax / MatMul with the graph's mask tensor (llama.cpp:248-263).  Same bits, also for passes on
    top of a filled cache."""
    monkeypatch.setenv("SPY_HIP_PROMPT_ATTN", "0")          # attention as MatMul -> Softmax -> MatMul, not the single kernel
    from spy_amd import backend_driver as B
    from spy_amd import model as M
    cfg = M.Config(n_layer=2, n_embd=256, n_head=2, n_ff=768, n_vocab=512, n_ctx=448, wtype=O.Q4_0)
    tensors = M.synth_model(cfg, seed=11)
    host, eng = B.HostModel(cfg, tensors), M.Engine(cfg, tensors, order=0)        # own order: the kernels the submit path launches by default
    prompt = np.random.default_rng(5).integers(0, cfg.n_vocab, 438).astype(np.int32)
    # passes of 168, 136 and 134 tokens: the attention products span several 128 x 128 tiles, some of them entirely
    # above the causal diagonal (left out by the engine); the last pass has rows of 438 positions (not a multiple of 8:
    # probabilities handed over as fp32)
    for start, stop in ((0, 168), (168, 304), (304, 438)):
        lg_h, lg_e = host.forward(prompt[start:stop], start), eng.forward(prompt[start:stop], start)
        assert np.isfinite(lg_e).all()
        assert np.array_equal(lg_h, lg_e), (start, stop)
    host.close()


@pytest.mark.gpu
def test_engine_prompt_pass_heads_of_64():
    """Heads the attention kernel does not take (it is built for 128-wide heads): the engine falls back to
    MatMul -> Softmax -> MatMul by itself, bit-identical to the submit path."""
    from spy_amd import backend_driver as B
    from spy_amd import model as M
    cfg = M.Config(n_layer=2, n_embd=256, n_head=4, n_ff=768, n_vocab=512, n_ctx=96, wtype=O.Q8_0)
    tensors = M.synth_model(cfg, seed=19)
    host, eng = B.HostModel(cfg, tensors), M.Engine(cfg, tensors)
    prompt = np.random.default_rng(6).integers(0, cfg.n_vocab, 90).astype(np.int32)
    for start, stop in ((0, 50), (50, 90)):
        lg_h, lg_e = host.forward(prompt[start:stop], start), eng.forward(prompt[start:stop], start)
        assert np.isfinite(lg_e).all() and np.array_equal(lg_h, lg_e), (start, stop)
    host.close(); eng.close()


@pytest.mark.gpu
def test_engine_prompt_pass_wide_layer_matches_submit_path(monkeypatch):
    """Layers wide enough (and passes long enough) for the 128 x 128 tile GEMM, where the engine runs gate and up as
    one grid: same bits as the submit path's separate MatMuls (attention as MatMul -> Softmax -> MatMul for this test)."""
    monkeypatch.setenv("SPY_HIP_PROMPT_ATTN", "0")
    from spy_amd import backend_driver as B
    from spy_amd import model as M
    for wtype, dims in ((O.Q4_0, (512, 4, 2816, 1024)), (O.Q8_0, (2048, 16, 2816, 1408)), (O.Q4_0, (2048, 16, 2816, 1408))):
        n_embd, n_head, n_ff, n_tok = dims       # the second: wq, wk, wv, wo and down wide enough for the tile kernel too
        cfg = M.Config(n_layer=1, n_embd=n_embd, n_head=n_head, n_ff=n_ff, n_vocab=512, n_ctx=n_tok + 16, wtype=wtype)
        tensors = M.synth_model(cfg, seed=3)
        host, eng = B.HostModel(cfg, tensors), M.Engine(cfg, tensors, order=0)
        prompt = np.random.default_rng(8).integers(0, cfg.n_vocab, n_tok).astype(np.int32)
        lg_h, lg_e = host.forward(prompt, 0), eng.forward(prompt, 0)
        assert np.isfinite(lg_e).all() and np.array_equal(lg_h, lg_e), dims
        host.close(); eng.close()


@pytest.mark.gpu
def test_submit_path_k_quant_mix_with_outliers():
    """The Q4_K_M-style mix (Q4_K for q, k, o, gate, up; Q6_K for v, down and the head; 0.1 % of the
    weights x20) through Backend::submit, against the oracle.  The reference has no K-quant arithmetic:
    both sides follow the public ggml block definitions (parity unpinned against the reference)."""
    from spy_amd import backend_driver as B
    from spy_amd import model as M
    from tests.gpu_util import assert_close
    from tests.model_util import OracleModel, k_quant_quantizer
    cfg = M.Config(n_layer=2, n_embd=512, n_head=4, n_ff=1024, n_vocab=768, n_ctx=48, wtype=O.Q4_K, t_out=O.Q6_K,
                   tensor_types={"attn_v": O.Q6_K, "ffn_down": O.Q6_K})
    tensors = M.synth_model(cfg, seed=21, outlier_every=1000, quantizer=k_quant_quantizer)
    host, ora = B.HostModel(cfg, tensors), OracleModel(cfg, tensors)
    prompt = np.random.default_rng(4).integers(0, cfg.n_vocab, 7).astype(np.int32)
    lo = ora.forward(prompt, 0)
    assert_close(host.forward(prompt, 0), lo, "K-quant mix prefill logits", 3e-3)
    tok = int(np.argmax(lo[-1]))
    for step in range(3):
        t = np.array([tok], np.int32)
        lh, l1 = host.forward(t, 7 + step)[0], ora.forward(t, 7 + step)[0]
        assert_close(lh, l1, "K-quant mix decode step %d" % step, 3e-3)
        tok = int(np.argmax(l1))
    host.close()


@pytest.mark.gpu
def test_relu_silu_quantize_nodes_through_submit(oracle):
    """The operators of the host backend's set that the LLaMA graph does not emit (Relu, Quantize; operator_impl.h:73,89 in
    the Spy tree), each as one node through Backend::submit with IO operands, against the oracle."""
    import ctypes as C
    from spy_amd import backend_driver as BD
    rng = np.random.default_rng(14)
    x = (rng.standard_normal((7, 128)) * 2).astype(np.float32)
    want = np.zeros_like(x)
    assert oracle.spy_o_relu(C.byref(O.tensor(x, O.F32, [128, 7])), C.byref(O.tensor(want, O.F32, [128, 7]))) == 0
    assert np.array_equal(BD.unary_through_submit("relu", x).view(np.uint32), want.view(np.uint32))
    for ttype in (O.Q8_0, O.F16):
        wq = np.zeros(7 * O.row_size(ttype, 128), np.uint8)
        assert oracle.spy_o_quantize(C.byref(O.tensor(x, O.F32, [128, 7])), C.byref(O.tensor(wq, ttype, [128, 7]))) == 0
        assert np.array_equal(BD.unary_through_submit("quantize", x, ttype), wq)
    with pytest.raises(RuntimeError):                                       # F32 -> Q4_0: OperatorStatus::Unsupport
        BD.unary_through_submit("quantize", x, O.Q4_0)
