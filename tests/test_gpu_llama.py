"""GPU parity of the token loop: prefill (operator by operator), the fused single-token pass, the
KV caches and the greedy tokens, against the CPU oracle on the same synthetic model."""
import numpy as np
import pytest

from tests import oracle_lib as O

pytestmark = pytest.mark.gpu


def _mk(cfg, seed=7, nthread=8, order=None):
    """order: summation order of the engine's fused single-token pass (1: the host backend's, 0: its own, None: default = 1)"""
    from spy_amd import model as M
    from tests.model_util import OracleModel, k_quant_quantizer
    tensors = M.synth_model(cfg, seed=seed, quantizer=k_quant_quantizer)
    return M.Engine(cfg, tensors, order=order), OracleModel(cfg, tensors, nthread=nthread), tensors


def _bits(got, want, what):
    got, want = np.ascontiguousarray(got, np.float32), np.ascontiguousarray(want, np.float32)
    n = int((got.view(np.uint32) != want.view(np.uint32)).sum())
    print("%s: %d of %d values differ from the oracle's bits" % (what, n, got.size), flush=True)
    assert n == 0, what


def _f16(a):
    return a.view(np.float16).astype(np.float32)


def _close(got, want, what, tol=1e-3):
    from tests.gpu_util import assert_close
    assert_close(got, want, what, tol)


@pytest.mark.parametrize("order", [1, 0])
@pytest.mark.parametrize("wtype,t_out,t_emb", [(O.Q4_0, O.Q4_0, O.F32), (O.Q8_0, O.Q8_0, O.Q8_0), (O.Q4_0, O.Q6_K, O.F32)])
def test_small_model_prefill_decode_and_tokens(wtype, t_out, t_emb, order):
    from spy_amd import model as M
    cfg = M.Config(n_layer=2, n_embd=256, n_head=2, n_ff=768, n_vocab=512, n_ctx=64, wtype=wtype, t_out=t_out, t_tok_embd=t_emb)
    eng, ora, _ = _mk(cfg, order=order)
    assert eng.order() == order
    rng = np.random.default_rng(3)
    prompt = rng.integers(0, cfg.n_vocab, 5).astype(np.int32)
    # prefill: logits of every prompt token, and the caches it leaves behind
    lg_g = eng.forward(prompt, 0)
    lg_o = ora.forward(prompt, 0)
    _close(lg_g, lg_o, "prefill logits (type %d)" % wtype)
    for il in range(cfg.n_layer):
        kg, ko = _f16(eng.read_buffer("k_cache", il, np.uint16)), _f16(ora.k_cache[il])
        vg, vo = _f16(eng.read_buffer("v_cache", il, np.uint16)), _f16(ora.v_cache[il])
        _close(kg, ko, "K cache layer %d" % il, 2e-3)       # fp16 storage: one ulp = 2^-11 relative
        _close(vg, vo, "V cache layer %d" % il, 2e-3)
        assert np.array_equal(kg == 0, ko == 0) and np.array_equal(vg == 0, vo == 0)     # same slots written
    # fused single-token pass on top of that cache
    tok = int(np.argmax(lg_o[-1]))
    lg1_g = eng.forward(np.array([tok], np.int32), 5)[0]
    lg1_o = ora.forward(np.array([tok], np.int32), 5)[0]
    _close(lg1_g, lg1_o, "fused decode logits (type %d)" % wtype)
    eng.close()


@pytest.mark.parametrize("name,kw", [
    ("Q4_0", dict(wtype=O.Q4_0)),
    ("Q8_0, Q8_0 embeddings", dict(wtype=O.Q8_0, t_tok_embd=O.Q8_0)),
    ("Q4_K_M mix", dict(wtype=O.Q4_K, t_out=O.Q6_K, tensor_types={"attn_v": O.Q6_K, "ffn_down": O.Q6_K})),
])
def test_prompt_passes_of_many_tokens_against_oracle(name, kw):
    """Passes of 16 tokens and more take the matrix-core GEMMs, the fused activation producers and the attention
    kernel: logits of every token and both caches against the CPU oracle, for a first pass and for one on top of
    a filled cache (head dimension 128, as the attention kernel requires)."""
    from spy_amd import model as M
    from tests.gpu_util import E2E_TOL
    cfg = M.Config(n_layer=2, n_embd=256, n_head=2, n_ff=768, n_vocab=512, n_ctx=96, **kw)
    eng, ora, _ = _mk(cfg, seed=13)
    prompt = np.random.default_rng(17).integers(0, cfg.n_vocab, 88).astype(np.int32)
    for start, stop in ((0, 48), (48, 88)):
        lg_g, lg_o = eng.forward(prompt[start:stop], start), ora.forward(prompt[start:stop], start)
        _close(lg_g, lg_o, "%s: logits of the pass over tokens %d..%d" % (name, start, stop), E2E_TOL)
        assert (np.argmax(lg_g, axis=1) == np.argmax(lg_o, axis=1)).mean() > 0.9
    for il in range(cfg.n_layer):
        kg, ko = _f16(eng.read_buffer("k_cache", il, np.uint16)), _f16(ora.k_cache[il])
        vg, vo = _f16(eng.read_buffer("v_cache", il, np.uint16)), _f16(ora.v_cache[il])
        _close(kg, ko, "K cache layer %d" % il, E2E_TOL if il else 2e-3)      # layer 0: one fp16 ulp; deeper layers carry the pass's noise
        _close(vg, vo, "V cache layer %d" % il, E2E_TOL if il else 2e-3)
        assert np.array_equal(kg == 0, ko == 0) and np.array_equal(vg == 0, vo == 0)
    eng.close()


def _comfortable_prompt(ora, cfg, n_prompt, n_predict, min_margin, tries=40):
    """A seeded random prompt whose greedy continuation on the CPU path has the widest top-1/top-2
    logit gaps (stops early once the smallest gap exceeds min_margin logit standard deviations):
    random-init models have nearly flat logits, and a near-tie is decided by the last ulp of either
    implementation."""
    best = None
    for seed in range(tries):
        prompt = np.random.default_rng(1000 + seed).integers(0, cfg.n_vocab, n_prompt).astype(np.int32)
        margins = []
        toks = ora.generate(prompt, n_predict, margins)
        sd = float(ora.forward(prompt, 0)[-1].std())
        if best is None or min(margins) / sd > best[2] / best[3]:
            best = (prompt, toks, min(margins), sd)
        if min(margins) > min_margin * sd:
            break
    return best


@pytest.mark.parametrize("n_prompt,chunk", [(6, None), (40, None), (72, "32")])
def test_forward_last_is_the_last_row_of_forward(n_prompt, chunk, monkeypatch):
    """spy_hip_llama_forward_last = the pass of spy_hip_llama_forward with the head on the last token only: same
    KV caches, and the logits of the last row (same kernels for a prompt below 16 tokens, the one-row head kernel
    against the matrix-core one above: 1e-3), also when the prompt goes through in chunks."""
    from spy_amd import model as M
    if chunk:
        monkeypatch.setenv("SPY_HIP_PREFILL_CHUNK", chunk)
    cfg = M.Config(n_layer=2, n_embd=256, n_head=2, n_ff=768, n_vocab=512, n_ctx=96, wtype=O.Q4_0)
    tensors = M.synth_model(cfg, seed=5)
    a, b = M.Engine(cfg, tensors), M.Engine(cfg, tensors)
    prompt = np.random.default_rng(9).integers(0, cfg.n_vocab, n_prompt).astype(np.int32)
    full = a.forward(prompt, 0)
    last = b.forward_last(prompt, 0)
    assert last.shape == (cfg.n_vocab,)
    if n_prompt < 16:
        assert np.array_equal(last, full[-1])
    else:
        _close(last, full[-1], "last-row logits")
        assert int(np.argmax(last)) == int(np.argmax(full[-1]))
    for il in range(cfg.n_layer):
        for name in ("k_cache", "v_cache"):
            assert np.array_equal(a.read_buffer(name, il), b.read_buffer(name, il)), (name, il)
    # a pass without any logits leaves the same caches too
    c = M.Engine(cfg, tensors)
    assert c.forward(prompt, 0, want_logits=False) is None
    assert np.array_equal(c.read_buffer("k_cache", 1), a.read_buffer("k_cache", 1))
    for e in (a, b, c):
        e.close()


@pytest.mark.parametrize("order", [1, 0])
def test_greedy_tokens_identical_small(order):
    """Single-token passes one by one against the oracle, then the free-running greedy loop.
    The reference's softmax rounds its exp argument to fp16 (non-linear.cpp:170 in the Spy tree), so a
    last-ulp difference in a score occasionally moves that argument to the neighbouring fp16 value
    (0.1-0.8 % on one probability).  With the handful of cached tokens of this test one probability
    carries a lot of weight, hence the end-to-end bound below is looser than the per-operator 1e-3
    (which the operator tests hold on identical inputs); the greedy tokens must still be identical."""
    from spy_amd import model as M
    from tests.gpu_util import rel_err
    cfg = M.Config(n_layer=3, n_embd=512, n_head=4, n_ff=1024, n_vocab=1024, n_ctx=64, wtype=O.Q4_0)
    eng, ora, _ = _mk(cfg, seed=11, order=order)
    prompt, want, margin, sd = _comfortable_prompt(ora, cfg, 8, 32, 0.05)
    print("prompt", prompt.tolist(), "min margin %.3e, logit std %.3e" % (margin, sd), flush=True)
    lg_o = ora.forward(prompt, 0)[-1]
    lg_g = eng.forward(prompt, 0)[-1]
    errs = []
    for step in range(32):
        errs.append(rel_err(lg_g, lg_o))
        print("step %2d n_kv %2d: logits max-abs err / max |logit| = %.2e" % (step, len(prompt) + step, errs[-1]), flush=True)
        assert int(np.argmax(lg_g)) == int(want[step])
        lg_o = ora.forward(want[step:step + 1], len(prompt) + step)[0]
        lg_g = eng.forward(want[step:step + 1], len(prompt) + step)[0]
    assert max(errs) < 3e-2
    # free-running greedy loop on the device: direct launches, then HIP-graph replay
    got_direct = eng.decode_greedy(int(want[0]), len(prompt), 31, use_graph=False)
    assert np.array_equal(got_direct, want[1:])
    got_graph = eng.decode_greedy(int(want[0]), len(prompt), 31, use_graph=True)
    assert np.array_equal(got_graph, want[1:])
    assert np.array_equal(eng.generate(prompt, 32), want)
    eng.close()


@pytest.mark.parametrize("order,n_ctx,positions", [(1, 1024, (700, 0, 1023)), (0, 1024, (700, 0, 1023)), (1, 4352, (4100, 4351, 4095)), (0, 4352, (4100, 4351))])
def test_fused_decode_real_widths_long_cache(order, n_ctx, positions):
    """d = 4096, F = 11008, 32 heads, one layer: the single-token pass over a cache filled up to the position
    (random fp16 K/V uploaded to both sides), also at the context of the named configuration (n_kv 4096 .. 4352).
    Order 1: attention output, layer output, logits and the cache slots written are the oracle's bits.  Order 0: the
    attention output (inputs identical on both sides up to fp16 flips of q) is held to the per-operator bound, the
    cache slots written to one fp16 ulp, the rest of the pass to the whole-pass bound."""
    from spy_amd import model as M
    from tests.gpu_util import E2E_TOL
    cfg = M.Config(n_layer=1, n_embd=4096, n_head=32, n_ff=11008, n_vocab=4096, n_ctx=n_ctx, wtype=O.Q4_0)
    eng, ora, _ = _mk(cfg, seed=21, nthread=16, order=order)
    rng = np.random.default_rng(9)
    for P in positions:
        k = (rng.standard_normal(cfg.n_ctx * cfg.n_embd) * 0.5).astype(np.float16).view(np.uint16)
        v = (rng.standard_normal(cfg.n_ctx * cfg.n_embd) * 0.5).astype(np.float16).view(np.uint16)
        ora.k_cache[0][:] = k; ora.v_cache[0][:] = v
        eng.write_buffer("k_cache", 0, k); eng.write_buffer("v_cache", 0, v)
        ora.clear_taps()
        kqv, layer_out = ora.tap("kqv", 0, cfg.n_embd), ora.tap("layer_out", 0, cfg.n_embd)
        tok = np.array([123], np.int32)
        lg_g = eng.forward(tok, P)[0]
        lg_o = ora.forward(tok, P)[0]
        ora.clear_taps()
        _close(eng.read_buffer("attn_out", 0, np.float32), kqv, "attention output, n_kv = %d" % (P + 1))
        _close(eng.read_buffer("x", 0, np.float32), layer_out, "layer output, n_kv = %d" % (P + 1), E2E_TOL)
        _close(lg_g, lg_o, "logits, n_kv = %d" % (P + 1), E2E_TOL)
        if order == 1:
            _bits(eng.read_buffer("attn_out", 0, np.float32), kqv, "attention output, n_kv = %d" % (P + 1))
            _bits(eng.read_buffer("x", 0, np.float32), layer_out, "layer output, n_kv = %d" % (P + 1))
            _bits(lg_g, lg_o, "logits, n_kv = %d" % (P + 1))
            assert np.array_equal(eng.read_buffer("k_cache", 0, np.uint16), ora.k_cache[0]) and np.array_equal(eng.read_buffer("v_cache", 0, np.uint16), ora.v_cache[0])
        kg = _f16(eng.read_buffer("k_cache", 0, np.uint16)).reshape(cfg.n_ctx, cfg.n_embd)
        ko = _f16(ora.k_cache[0]).reshape(cfg.n_ctx, cfg.n_embd)
        _close(kg[P], ko[P], "K row written at pos %d" % P, 2e-3)
        assert np.array_equal(np.delete(kg, P, axis=0), np.delete(ko, P, axis=0))           # every other slot untouched
        vg = _f16(eng.read_buffer("v_cache", 0, np.uint16)).reshape(cfg.n_embd, cfg.n_ctx)
        vo = _f16(ora.v_cache[0]).reshape(cfg.n_embd, cfg.n_ctx)
        _close(vg[:, P], vo[:, P], "V column written at pos %d" % P, 2e-3)
        assert np.array_equal(np.delete(vg, P, axis=1), np.delete(vo, P, axis=1))
    eng.close()


def test_model_wider_than_4096_takes_the_tiled_kernels():
    """n_embd = 5120 (the 13B width): the one-row-per-wave kernels stage 4096 activations per workgroup at most, so the fused
    single-token pass of such a model runs the 256-thread tiled kernels, in this backend's own summation order (the kernels of
    the host's order take n_embd <= 4096).  One layer against the oracle: per-pass bound, same greedy tokens both ways of
    running the loop."""
    from spy_amd import model as M
    from tests.gpu_util import E2E_TOL
    cfg = M.Config(n_layer=1, n_embd=5120, n_head=40, n_ff=13824, n_vocab=2048, n_ctx=64, wtype=O.Q4_0)
    eng, ora, _ = _mk(cfg, seed=41)
    assert eng.order() == 0
    prompt = np.random.default_rng(3).integers(0, cfg.n_vocab, 6).astype(np.int32)
    lg_g, lg_o = eng.forward(prompt, 0), ora.forward(prompt, 0)
    _close(lg_g, lg_o, "prompt logits, n_embd 5120", E2E_TOL)
    tok = int(np.argmax(lg_o[-1]))
    for step in range(3):
        t = np.array([tok], np.int32)
        lg, lo = eng.forward(t, 6 + step)[0], ora.forward(t, 6 + step)[0]
        _close(lg, lo, "single-token logits, n_embd 5120, step %d" % step, E2E_TOL)
        tok = int(np.argmax(lo))
    a = eng.decode_greedy(tok, 9, 4, use_graph=False)
    b = eng.decode_greedy(tok, 9, 4, use_graph=True)
    assert a.tolist() == b.tolist()
    eng.close()


@pytest.mark.parametrize("order", [1, 0])
def test_engine_with_a_smaller_context_does_not_lower_the_lds_limit_of_a_larger_one(order):
    """A kernel's dynamic-LDS limit belongs to the kernel for the whole process.  An engine with a long context raises it
    (softmax + P.V^T keeps a head's scores and V^T rows in LDS: about 140 KB at 4352 positions); an engine with a short
    context created afterwards, and the kernel-family entry points, must not lower it under the first engine's launches."""
    from spy_amd import model as M
    big = M.Config(n_layer=1, n_embd=4096, n_head=32, n_ff=11008, n_vocab=1024, n_ctx=4352, wtype=O.Q4_0)
    small = M.Config(n_layer=1, n_embd=4096, n_head=32, n_ff=11008, n_vocab=1024, n_ctx=64, wtype=O.Q4_0)
    tensors = M.synth_model(big, seed=3)
    a = M.Engine(big, tensors, order=order)
    rng = np.random.default_rng(2)
    a.write_buffer("k_cache", 0, (rng.standard_normal(big.n_ctx * big.n_embd) * 0.5).astype(np.float16).view(np.uint16))
    a.write_buffer("v_cache", 0, (rng.standard_normal(big.n_ctx * big.n_embd) * 0.5).astype(np.float16).view(np.uint16))
    tok = np.array([7], np.int32)
    first = a.forward(tok, 4300)[0]
    b = M.Engine(small, tensors, order=order)
    assert np.isfinite(b.forward(tok, 3)[0]).all()
    again = a.forward(tok, 4300)[0]                      # the same slot is rewritten with the same values
    assert np.array_equal(first.view(np.uint32), again.view(np.uint32))
    toks = a.decode_greedy(7, 4300, 4, use_graph=True)
    assert len(toks) == 4
    a.close(); b.close()


@pytest.mark.timeout(900)
def test_llama2_7b_q4_0_greedy_32_tokens():
    """The first named configuration on the engine the bench times: the 7B shape, Q4_0 body with the Q6_K output head, 8 random
    prompt tokens, 32 greedy steps, ctx 48.  The prompt goes through the exact-order operator kernels (library-wide switch on for that call only),
    the 32 steps through the engine's default single-token pass -- the fused launches in the host backend's summation
    order, replayed as a HIP graph.  All 32 tokens must be the CPU oracle's, and so must the bits of every pass's
    logits (teacher-forced single-token passes), no filter on near-ties."""
    import os
    from spy_amd import _lib as H
    from spy_amd import model as M
    cfg = M.Config.llama2_7b(n_ctx=48, wtype=O.Q4_0, t_out=O.Q6_K)
    eng, ora, _ = _mk(cfg, seed=1234, nthread=min(16, os.cpu_count() or 8))
    assert eng.order() == 1
    prompt = np.random.default_rng(5).integers(0, cfg.n_vocab, 8).astype(np.int32)
    margins = []
    want = ora.generate(prompt, 32, margins)
    print("7B Q4_0 + Q6_K head: prompt", prompt.tolist(), "\noracle tokens:", want.tolist(), "\nsmallest top-1/top-2 gap %.3e" % min(margins), flush=True)
    prev = H.load().spy_hip_set_exact_order(1)
    try:
        first = eng.forward_last(prompt, 0)
    finally:
        H.load().spy_hip_set_exact_order(prev)
    _bits(first, ora.forward(prompt, 0)[-1], "prompt pass, last row")
    assert int(np.argmax(first)) == int(want[0])
    got = np.concatenate([[want[0]], eng.decode_greedy(int(want[0]), len(prompt), 31, use_graph=True)])
    print("hip tokens:   ", got.tolist(), flush=True)
    assert got.tolist() == want.tolist()
    # the caches now hold the 8 + 31 tokens of both sides; teacher-forced passes over them again: same bits every time
    same = 0
    for step in range(31):
        lg_o = ora.forward(want[step:step + 1], len(prompt) + step)[0]
        lg_g = eng.forward(want[step:step + 1], len(prompt) + step)[0]
        same += int(np.array_equal(lg_o.view(np.uint32), lg_g.view(np.uint32)))
    print("%d of 31 single-token passes with bit-identical logits" % same, flush=True)
    assert same == 31
    eng.close()


def _full_size_case(cfg, seed, n_prompt, n_steps, n_forced, outlier_every=0):
    """A named configuration at its full size on the engine as it comes (summation order 1): the prompt in one call (tiled exact
    MatMul from packed operands, causal exact attention kernels, chunks of 2048 rows), n_steps greedy single-token passes (graph
    replay), n_forced teacher-forced passes.  Logits of every prompt row, every token and the logits of the forced passes must be
    the CPU oracle's bit for bit."""
    import os
    from spy_amd import model as M
    from tests.model_util import OracleModel
    tensors = M.synth_model(cfg, seed=seed, outlier_every=outlier_every)       # the package's own block quantizers, as in bench.py
    eng, ora = M.Engine(cfg, tensors), OracleModel(cfg, tensors, nthread=min(16, os.cpu_count() or 8))
    assert eng.order() == 1
    prompt = np.random.default_rng(seed + 1).integers(0, cfg.n_vocab, n_prompt).astype(np.int32)
    print("oracle prompt pass of %d tokens ..." % n_prompt, flush=True)
    import threading, time
    done = threading.Event()

    def heartbeat():                                 # a long CPU pass prints nothing by itself
        t0 = time.time()
        while not done.wait(60.0):
            print("  ... %d s" % (time.time() - t0), flush=True)
    threading.Thread(target=heartbeat, daemon=True).start()
    try:
        lg_o = ora.forward(prompt, 0)
    finally:
        done.set()
    lg_g = eng.forward(prompt, 0)
    _bits(lg_g, lg_o, "prompt pass of %d tokens, every row" % n_prompt)
    want, logits, pos = [], lg_o[-1], n_prompt
    del lg_o, lg_g
    for step in range(n_steps):
        want.append(int(np.argmax(logits)))
        if step + 1 < n_steps:
            logits = ora.forward(np.array([want[-1]], np.int32), pos)[0]
            pos += 1
        if step % 32 == 31:
            print("oracle step", step + 1, flush=True)
    got = [want[0]] + eng.decode_greedy(want[0], n_prompt, n_steps - 1, use_graph=True).tolist()
    print("oracle tokens:", want, "\nhip tokens:   ", got, flush=True)
    assert got == want
    same = 0
    for step in range(n_forced):
        lo = ora.forward(np.array([want[step]], np.int32), n_prompt + step)[0]
        lg = eng.forward(np.array([want[step]], np.int32), n_prompt + step)[0]
        same += int(np.array_equal(lo.view(np.uint32), lg.view(np.uint32)))
    print("%d of %d single-token passes with bit-identical logits" % (same, n_forced), flush=True)
    assert same == n_forced
    eng.close()


@pytest.mark.timeout(600)
def test_llama2_7b_q8_0_prompt_512_then_64_tokens():
    """The third named configuration: 7B shape in Q8_0 (32 layers), 512-token prompt, 64 greedy steps (n_kv 513 ... 576)."""
    from spy_amd import model as M
    _full_size_case(M.Config.llama2_7b(n_ctx=576, wtype=O.Q8_0), 4321, 512, 64, 16)


@pytest.mark.timeout(600)
def test_llama2_7b_width_4_layers_q4_0_prompt_4096_then_32_tokens():
    """The second named configuration (the one the bench times) with 4 of its 32 layers, so that the CPU oracle's pass fits the
    regular suite: Q4_0 body, Q6_K head, 4096-token prompt in two chunks of 2048 rows (the long-row grids of the exact prompt
    attention: 64 query tiles, key segments beyond one), 32 greedy steps at n_kv 4097 ... 4128 in a context of 4352, 4 forced passes."""
    from spy_amd import model as M
    cfg = M.Config.llama2_7b(n_ctx=4352, wtype=O.Q4_0, t_out=O.Q6_K)
    cfg.n_layer = 4
    _full_size_case(cfg, 4323, 4096, 32, 4)


@pytest.mark.timeout(600)
def test_llama2_7b_width_4_layers_q4_k_m_prompt_2048_then_32_tokens():
    """The fourth named configuration with 4 of its 32 layers: the Q4_K / Q6_K mix with 0.1 % of the weights x 20, 2048-token
    prompt, 32 greedy steps, 4 forced passes."""
    from spy_amd import model as M
    cfg = M.Config.llama2_7b(n_ctx=2560, wtype=O.Q4_K, t_out=O.Q6_K, tensor_types={"attn_v": O.Q6_K, "ffn_down": O.Q6_K})
    cfg.n_layer = 4
    _full_size_case(cfg, 4322, 2048, 32, 4, outlier_every=1000)


_slow = pytest.mark.skipif(not __import__("os").environ.get("SPY_FULL_SIZE_TESTS"), reason="many minutes of CPU oracle at the 7B size: set SPY_FULL_SIZE_TESTS=1")


@_slow
@pytest.mark.timeout(1150)
def test_llama2_7b_q4_k_m_prompt_2048_then_96_tokens():
    """The fourth named configuration: the Q4_K / Q6_K mix, 2048-token prompt; 96 of its 512 greedy steps (the oracle's K-quant
    prompt pass alone takes 16 minutes on 16 threads)."""
    from spy_amd import model as M
    cfg = M.Config.llama2_7b(n_ctx=2560, wtype=O.Q4_K, t_out=O.Q6_K, tensor_types={"attn_v": O.Q6_K, "ffn_down": O.Q6_K})
    _full_size_case(cfg, 4322, 2048, 96, 4, outlier_every=1000)            # 0.1 % of the weights x 20


@_slow
@pytest.mark.timeout(1150)
def test_llama2_7b_q4_0_prompt_4096_then_256_tokens():
    """The second named configuration (the one the bench times): Q4_0 with the Q6_K head, 4096-token prompt in two chunks, 256 greedy
    steps at n_kv 4097 ... 4352."""
    from spy_amd import model as M
    _full_size_case(M.Config.llama2_7b(n_ctx=4352, wtype=O.Q4_0, t_out=O.Q6_K), 4323, 4096, 256, 4)


@pytest.mark.timeout(900)
def test_llama2_7b_q4_0_own_order_stays_within_the_noise_bound():
    """The same configuration on the engine's own summation order (order 0), which is NOT the parity path.  Every MatMul of
    the reference re-quantizes its activations to Q8_0, so an implementation whose fp32 sums are not bit-identical
    decorrelates its Q8_0 rounding noise within a few layers: a few percent of the largest logit after 32 layers of a
    random-init model.  Fixed bounds: each pass's logits within 10 % of the largest logit; the same argmax at every
    teacher-forced step whose top-1/top-2 gap on the CPU path exceeds twice that bound."""
    import os
    from spy_amd import model as M
    from tests.gpu_util import rel_err
    BOUND = 0.10
    cfg = M.Config.llama2_7b(n_ctx=48, wtype=O.Q4_0)
    eng, ora, _ = _mk(cfg, seed=1234, nthread=min(16, os.cpu_count() or 8), order=0)
    prompt = np.random.default_rng(5).integers(0, cfg.n_vocab, 8).astype(np.int32)
    margins = []
    want = ora.generate(prompt, 32, margins)
    lg_o = ora.forward(prompt, 0)
    lg_g = eng.forward(prompt, 0)
    _close(lg_g, lg_o, "7B prefill logits (8 tokens)", BOUND)
    lg_o, lg_g = lg_o[-1], lg_g[-1]
    errs, same, decidable = [], [], []
    for step in range(32):
        errs.append(rel_err(lg_g, lg_o))
        same.append(int(np.argmax(lg_g)) == int(want[step]))
        decidable.append(margins[step] > 2 * BOUND * float(np.abs(lg_o).max()))
        lg_o = ora.forward(want[step:step + 1], len(prompt) + step)[0]
        lg_g = eng.forward(want[step:step + 1], len(prompt) + step)[0]
    print("own order: per-pass logits max-abs err / max |logit|: median %.2e max %.2e; %d of 32 teacher-forced argmax identical, %d steps decidable at the fixed bound"
          % (float(np.median(errs)), max(errs), sum(same), sum(decidable)), flush=True)
    assert max(errs) < BOUND
    assert all(s for s, d in zip(same, decidable) if d)
    eng.close()


@pytest.mark.timeout(600)
@pytest.mark.parametrize("name,kw", [
    ("Q4_0 body, Q6_K head", dict(wtype=O.Q4_0, t_out=O.Q6_K)),
    ("Q8_0", dict(wtype=O.Q8_0)),
    ("Q4_K_M mix", dict(wtype=O.Q4_K, t_out=O.Q6_K, tensor_types={"attn_v": O.Q6_K, "ffn_down": O.Q6_K})),
])
@pytest.mark.parametrize("order", [1, 0])
def test_llama2_7b_prompt_4096_properties(name, kw, order, monkeypatch):
    """The named configurations at full size (7B shape, 4096-token prompt), through properties that need no CPU pass.  (a) Chunking: the prompt in chunks of 2048 (default) and of 1024 tokens gives the same last-row logits
    bit for bit: every output of the matrix-core kernels (order 0) is accumulated in an order that does not depend on
    the tiling, and a query attends to the same cached positions in the same order whatever chunk it arrives in; the
    kernels of order 1 are told the length of the whole call, which is what the host's loops depend on.
    (b) Causality: the first 2048 tokens alone write the K cache rows (last layer) the full prompt writes.  In order 1
    this holds for the rows before position 2016 only, as in the reference: the host's fp16 dot adds the last 1..32
    positions of a pass one by one and the others in 32 accumulators, so the last 32 rows of a 2048-token pass round
    differently from the same rows inside a longer pass.
    (c) The token loop on top: decode_greedy and one-token forward passes emit the same tokens."""
    from spy_amd import model as M
    cfg = M.Config.llama2_7b(n_ctx=4096 + 32, **kw)
    tensors = M.synth_model(cfg, seed=1234, outlier_every=1000 if kw["wtype"] == O.Q4_K else 0)     # the mix as named: 0.1 % of the weights x 20
    prompt = np.random.default_rng(4096).integers(0, cfg.n_vocab, 4096).astype(np.int32)
    eng = M.Engine(cfg, tensors, order=order)
    assert eng.order() == order
    last_2048 = eng.forward_last(prompt, 0)
    assert np.isfinite(last_2048).all() and last_2048.std() > 0
    k_full = eng.read_buffer("k_cache", cfg.n_layer - 1, np.uint16).reshape(cfg.n_ctx, cfg.n_embd)[:2048].copy()
    first = int(np.argmax(last_2048))
    toks = eng.decode_greedy(first, 4096, 8)
    eng.close()
    eng2 = M.Engine(cfg, tensors, order=order)
    monkeypatch.setenv("SPY_HIP_PREFILL_CHUNK", "1024")
    last_1024 = eng2.forward_last(prompt, 0)
    monkeypatch.delenv("SPY_HIP_PREFILL_CHUNK")
    assert np.array_equal(last_1024, last_2048)
    tok, own = first, []
    for i in range(8):
        tok = int(np.argmax(eng2.forward(np.array([tok], np.int32), 4096 + i)[0]))
        own.append(tok)
    assert own == toks.tolist(), (own, toks.tolist())
    eng2.close()
    eng3 = M.Engine(cfg, tensors, order=order)
    eng3.forward(prompt[:2048], 0, want_logits=False)
    k_half = eng3.read_buffer("k_cache", cfg.n_layer - 1, np.uint16).reshape(cfg.n_ctx, cfg.n_embd)[:2048]
    rows = 2048 if order == 0 else 2016
    assert np.array_equal(k_half[:rows], k_full[:rows])
    eng3.close()


@pytest.mark.parametrize("name,kw", [
    ("Q4_0 body, Q6_K head", dict(wtype=O.Q4_0, t_out=O.Q6_K)),
    ("Q4_K + Q6_K head", dict(wtype=O.Q4_K, t_out=O.Q6_K)),
    ("Q6_K", dict(wtype=O.Q6_K)),
    ("Q4_K_M mix", dict(wtype=O.Q4_K, t_out=O.Q6_K, tensor_types={"attn_v": O.Q6_K, "ffn_down": O.Q6_K})),
    ("Q8_0 body, Q4_K gate|up", dict(wtype=O.Q8_0, tensor_types={"ffn_gate": O.Q4_K, "ffn_up": O.Q4_K})),
])
@pytest.mark.parametrize("dims", [(2, 512, 4, 1024, 768, 48), (1, 4096, 32, 11008, 2048, 1024)])
def test_k_quant_layers_in_the_fused_pass(name, kw, dims):
    """K-quant and mixed-type layers through the fused single-token kernels (and the prompt path) against
    the oracle.  The reference has no K-quant arithmetic: both sides follow the public ggml block layouts
    (parity unpinned against the reference itself)."""
    from spy_amd import model as M
    from tests.gpu_util import E2E_TOL          # whole passes: see the note on re-quantization there
    from tests.model_util import OracleModel, k_quant_quantizer
    n_layer, d, H_, F, V, C_ = dims
    cfg = M.Config(n_layer=n_layer, n_embd=d, n_head=H_, n_ff=F, n_vocab=V, n_ctx=C_, **kw)
    tensors = M.synth_model(cfg, seed=31, outlier_every=1000, quantizer=k_quant_quantizer)
    eng, ora = M.Engine(cfg, tensors), OracleModel(cfg, tensors)
    rng = np.random.default_rng(8)
    n_prompt = 9 if C_ < 512 else C_ - 10
    if C_ < 512:
        prompt = rng.integers(0, V, n_prompt).astype(np.int32)
        _close(eng.forward(prompt, 0), ora.forward(prompt, 0), "%s prefill logits" % name, E2E_TOL)
    else:
        for il in range(n_layer):
            k = (rng.standard_normal(n_prompt * d) * 1.2).astype(np.float16).view(np.uint16)
            v = np.zeros((d, C_), np.float16)
            v[:, :n_prompt] = (rng.standard_normal((d, n_prompt)) * 1.2).astype(np.float16)
            eng.write_buffer("k_cache", il, np.concatenate([k, np.zeros((C_ - n_prompt) * d, np.uint16)]))
            eng.write_buffer("v_cache", il, v.view(np.uint16))
            ora.k_cache[il][:n_prompt * d] = k
            ora.v_cache[il][:] = v.view(np.uint16).reshape(-1)
    tok = int(rng.integers(0, V))
    for step in range(3):
        t = np.array([tok], np.int32)
        lg, lo = eng.forward(t, n_prompt + step)[0], ora.forward(t, n_prompt + step)[0]
        _close(lg, lo, "%s single-token logits, step %d" % (name, step), E2E_TOL)
        tok = int(np.argmax(lo))
    toks = eng.decode_greedy(tok, n_prompt + 3, 3, use_graph=True)
    assert len(toks) == 3
    eng.close()
