"""The one-launch attention part of a layer against the three separate kernels and the CPU oracle."""
import numpy as np
import pytest

from tests import oracle_lib as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("wtype,n_layer,d,H,F,V,C", [
    (O.Q4_0, 3, 512, 4, 1024, 1024, 64),
    (O.Q8_0, 2, 1024, 8, 768, 640, 72),
    (O.Q4_0, 1, 4096, 32, 11008, 4096, 1024),    # real attention widths: 256 workgroups, one per compute unit
])
def test_fused_attention_launch_matches_split_kernels(wtype, n_layer, d, H, F, V, C, monkeypatch):
    """qkv + scores + softmax/KQV as one launch with head-local barriers against the three separate
    kernels and the oracle: logits of consecutive single-token passes and both KV caches."""
    from spy_amd import model as M
    from tests.gpu_util import assert_close, E2E_TOL
    from tests.model_util import OracleModel
    cfg = M.Config(n_layer=n_layer, n_embd=d, n_head=H, n_ff=F, n_vocab=V, n_ctx=C, wtype=wtype)
    tensors = M.synth_model(cfg, seed=13)
    monkeypatch.delenv("SPY_HIP_ATTN_SPLIT", raising=False)
    fused = M.Engine(cfg, tensors, order=0)              # the one-launch attention belongs to the backend's own summation order
    monkeypatch.setenv("SPY_HIP_ATTN_SPLIT", "1")
    split = M.Engine(cfg, tensors, order=0)
    ora = OracleModel(cfg, tensors)
    assert fused.fuses_attention() and not split.fuses_attention()
    rng = np.random.default_rng(17)
    n_prompt = C - 12
    for il in range(n_layer):                      # same cache contents everywhere
        k = (rng.standard_normal(n_prompt * d) * 1.2).astype(np.float16).view(np.uint16)
        v = np.zeros((d, C), np.float16)
        v[:, :n_prompt] = (rng.standard_normal((d, n_prompt)) * 1.2).astype(np.float16)
        for e in (fused, split):
            e.write_buffer("k_cache", il, np.concatenate([k, np.zeros((C - n_prompt) * d, np.uint16)]))
            e.write_buffer("v_cache", il, v.view(np.uint16))
        ora.k_cache[il][:n_prompt * d] = k
        ora.v_cache[il][:] = v.view(np.uint16).reshape(-1)
    tok = int(rng.integers(0, V))
    for step in range(6):
        t = np.array([tok], np.int32)
        lf, ls, lo = fused.forward(t, n_prompt + step)[0], split.forward(t, n_prompt + step)[0], ora.forward(t, n_prompt + step)[0]
        assert_close(lf, ls, "fused vs split logits, step %d" % step, E2E_TOL)
        assert_close(lf, lo, "fused vs oracle logits, step %d" % step, E2E_TOL)
        tok = int(np.argmax(lo))
    for il in range(n_layer):
        for name in ("k_cache", "v_cache"):
            a = fused.read_buffer(name, il, np.uint16).view(np.float16).astype(np.float32)
            b = split.read_buffer(name, il, np.uint16).view(np.float16).astype(np.float32)
            assert_close(a, b, "%s layer %d" % (name, il), 5e-3)
            assert np.array_equal(a == 0, b == 0)
    # graph replay of the greedy loop runs the same launches
    tf = fused.decode_greedy(tok, n_prompt + 6, 4, use_graph=True)
    assert len(tf) == 4
    fused.close()
    split.close()


def test_bounded_wait_gives_up_with_an_error_and_the_next_pass_is_clean(monkeypatch):
    """The give-up path of the waits between the workgroups of a head, forced from the host: with a poll budget of zero
    every wait that does not find its data at once raises the error word and the workgroup runs on to its end (no kernel
    hangs or traps).  The pass must report ETIMEOUT -- through spy_hip_llama_forward and through the greedy loop -- and,
    with the budget restored, the following passes must equal a fresh engine's: counters and exchange words were cleared."""
    from spy_amd import model as M
    from spy_amd import _lib as H
    cfg = M.Config(n_layer=2, n_embd=1024, n_head=8, n_ff=768, n_vocab=640, n_ctx=72, wtype=O.Q4_0)
    tensors = M.synth_model(cfg, seed=21)
    monkeypatch.delenv("SPY_HIP_ATTN_SPLIT", raising=False)
    eng, ref = M.Engine(cfg, tensors, order=0), M.Engine(cfg, tensors, order=0)
    assert eng.fuses_attention()
    rng = np.random.default_rng(3)
    prompt = rng.integers(0, cfg.n_vocab, 9).astype(np.int32)
    for e in (eng, ref):
        e.forward(prompt, 0)
    tok = np.array([int(rng.integers(0, cfg.n_vocab))], np.int32)
    want = ref.forward(tok, 9)[0]
    eng.set_spin_limit(0)
    codes = []
    for call in (lambda: eng.forward(tok, 9), lambda: eng.decode_greedy(int(tok[0]), 9, 2, use_graph=False),
                 lambda: eng.decode_greedy(int(tok[0]), 9, 2, use_graph=True)):
        try:
            call()
            codes.append(0)
        except H.SpyHipError as e:
            codes.append(e.code)
    print("codes with a poll budget of zero:", codes, flush=True)
    assert all(c in (0, H.ETIMEOUT) for c in codes) and H.ETIMEOUT in codes
    eng.set_spin_limit(400000)
    for rep in range(3):                           # launch numbers restart at 1 after the clean-up and climb again
        got = eng.forward(tok, 9)[0]
        assert np.array_equal(got, want), "pass %d after the forced give-up differs from a fresh engine's" % rep
    a, b = eng.decode_greedy(int(tok[0]), 9, 6, use_graph=True), ref.decode_greedy(int(tok[0]), 9, 6, use_graph=True)
    assert np.array_equal(a, b)
    eng.close()
    ref.close()
