"""GGUF file -> HBM -> token loop on the GPU: a model loaded from a file computes exactly what the same
model built from arrays computes, and agrees with the oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,kw", [
    ("q4_0, f32 embeddings", dict()),
    ("q8_0, q8_0 embeddings", dict(wtype=8, t_tok_embd=8)),
    ("q4_k body, q6_k wv / down / head", dict(wtype=12, t_out=14, tensor_types={"attn_v": 14, "ffn_down": 14})),
])
def test_loaded_model_equals_the_model_built_from_arrays(tmp_path, oracle, name, kw):
    from spy_amd import gguf as G, model as M
    from tests.gpu_util import E2E_TOL
    from tests.model_util import OracleModel, k_quant_quantizer
    kw = dict(kw)
    kw.setdefault("wtype", 2)
    cfg = M.Config(n_layer=2, n_embd=512, n_head=4, n_ff=1024, n_vocab=640, n_ctx=64, **kw)
    tensors = M.synth_model(cfg, seed=17, outlier_every=500, quantizer=k_quant_quantizer)
    path = G.write_llama(str(tmp_path / "m.gguf"), cfg, tensors, alignment=64)
    loaded = G.GGUFModel(path)
    assert loaded.weight_bytes == sum(t.nbytes for t in tensors.values())
    d = loaded.desc
    assert (d.n_layer, d.n_embd, d.n_head, d.n_ff, d.n_vocab, d.n_ctx) == (2, 512, 4, 1024, 640, 64)
    assert d.eps == np.float32(cfg.eps) and d.rope_freq_base == np.float32(cfg.rope_freq_base)
    assert loaded.file.get_arr_str("tokenizer.ggml.tokens", 5) == b"<t5>"
    direct = M.Engine(cfg, tensors)
    rng = np.random.default_rng(3)
    prompt = rng.integers(0, cfg.n_vocab, 7).astype(np.int32)
    a, b = loaded.engine.forward(prompt, 0), direct.forward(prompt, 0)
    assert np.array_equal(a, b), name
    ora = OracleModel(cfg, tensors)
    lo = ora.forward(prompt, 0)
    assert float(np.abs(a - lo).max() / np.abs(lo).max()) < E2E_TOL
    tok = int(np.argmax(a[-1]))
    ta, tb = loaded.engine.decode_greedy(tok, 7, 6), direct.decode_greedy(tok, 7, 6)
    assert np.array_equal(ta, tb), name
    assert np.array_equal(loaded.engine.generate(prompt, 5), direct.generate(prompt, 5))
    direct.close()
    loaded.close()


def test_context_argument_and_reload(tmp_path):
    """n_ctx = 0 takes the file's context length; another n_ctx sizes the KV caches (rounded up to 8)."""
    from spy_amd import gguf as G, model as M
    cfg = M.Config(n_layer=1, n_embd=256, n_head=2, n_ff=512, n_vocab=320, n_ctx=40, wtype=2)
    path = G.write_llama(str(tmp_path / "c.gguf"), cfg, M.synth_model(cfg, seed=2))
    m0 = G.GGUFModel(path)
    assert m0.desc.n_ctx == 40
    m1 = G.GGUFModel(path, n_ctx=21)
    assert m1.desc.n_ctx == 24
    t = np.array([3, 1, 4, 1, 5], np.int32)
    assert np.array_equal(m0.engine.forward(t, 0), m1.engine.forward(t, 0))
    m0.close(); m1.close()


def test_text_in_text_out(tmp_path, capsys):
    """Prompt text -> SentencePiece ids -> prompt pass + greedy loop -> text, and the command line around it."""
    from spy_amd import cli, gguf as G, model as M
    cfg = M.Config(n_layer=2, n_embd=256, n_head=2, n_ff=512, n_vocab=3 + 256 + 40, n_ctx=64, wtype=2)
    tensors = M.synth_model(cfg, seed=9)
    words = ["▁", "a", "b", "c", "d", "e", "t", "h", "▁t", "he", "▁the", "▁a", "at", "▁c", "▁cat", "ca", "▁s", "sa", "s"]
    toks = ["<unk>", "<s>", "</s>"] + ["<0x%02X>" % b for b in range(256)] + words + ["<pad%d>" % i for i in range(40 - len(words))]
    kv = G.llama_kv(cfg, toks) + [("tokenizer.ggml.scores", G.ARRAY, (G.F32, [0.0] * 259 + [-float(i) for i in range(40)])),
                                  ("tokenizer.ggml.token_type", G.ARRAY, (G.I32, [2, 3, 3] + [6] * 256 + [1] * 40))]
    infos = [(n, t, [c] if r == 1 else [c, r], tensors[n]) for n, (t, r, c) in cfg.tensor_shapes().items()]
    path = G.write_gguf(str(tmp_path / "t.gguf"), kv, infos)
    m = G.GGUFModel(path)
    ids = m.vocab.tokenize("the cat sat")
    assert ids[0] == 1 and m.vocab.detokenize(ids) == b" the cat sat"
    new, text = m.generate_text("the cat sat", 8)
    direct = M.Engine(cfg, tensors)
    want = direct.generate(np.asarray(ids, np.int32), 8)
    assert new == [int(t) for t in want] and text == m.vocab.detokenize(new)
    direct.close()
    from tests.model_util import OracleModel
    text_cpu = m.vocab.detokenize([int(t) for t in OracleModel(cfg, tensors).generate(np.asarray(ids, np.int32), 8)])
    m.close()
    cli.main([path, "-p", "the cat sat", "-n", "8"])
    out = capsys.readouterr()
    assert out.out == "the cat sat" + text.decode("utf-8", "replace") + "\n" and "generation: 8 tokens" in out.err
    # --exact: the same file through the exact-order operators gives the CPU oracle's tokens
    from spy_amd import _lib as H
    try:
        cli.main([path, "-p", "the cat sat", "-n", "8", "--exact"])
    finally:
        H.load().spy_hip_set_exact_order(0)
    out = capsys.readouterr()
    assert out.out == "the cat sat" + text_cpu.decode("utf-8", "replace") + "\n"
