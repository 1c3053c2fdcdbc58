"""The smoke check: a small pass of the hot path on the GPU compared with the CPU oracle."""
import ctypes as C


def run_smoke(H, O, np):
    H.init(0)
    L, oracle = H.load(), O.load()
    rng = np.random.default_rng(0)
    M, K, T = 256, 4096, 2
    w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.02).astype(np.float32), O.Q4_0)
    x = rng.standard_normal((T, K)).astype(np.float32)
    want = O.matmul(oracle, w, O.Q4_0, M, K, x, nthread=2)
    dw, dx = H.DeviceBuffer.from_numpy(w), H.DeviceBuffer.from_numpy(x)
    dd = H.DeviceBuffer(T * M * 4)
    tw, tx, td = H.tensor(dw, H.Q4_0, [K, M]), H.tensor(dx, H.F32, [K, T]), H.tensor(dd, H.F32, [M, T])
    need = L.spy_hip_op_matmul_scratch_size(C.byref(tw), C.byref(tx))
    sc = H.DeviceBuffer(need)
    H.check(L.spy_hip_op_matmul(None, C.byref(tw), C.byref(tx), C.byref(td), sc.ptr, need), "spy_hip_op_matmul")
    H.sync()
    got = dd.download(np.float32).reshape(T, M)
    err = float(np.abs(got - want).max() / np.abs(want).max())
    assert np.array_equal(sc.download(np.uint8), O.quantize(oracle, x, O.Q8_0)), "Q8_0 activations differ from the oracle"
    assert err < 1e-3, err
    print("smoke ok: Q4_0 matmul %dx%d T=%d, max relative error %.2e on %s" % (M, K, T, err, H.device_info()["name"]))
    # the token loop itself: prompt pass, fused single-token passes and the on-device greedy loop of a small model
    from spy_amd import model as M_
    from tests.model_util import OracleModel
    cfg = M_.Config(n_layer=2, n_embd=512, n_head=4, n_ff=1024, n_vocab=1024, n_ctx=64, wtype=H.Q4_0)
    tensors = M_.synth_model(cfg, seed=3)
    eng, ora = M_.Engine(cfg, tensors), OracleModel(cfg, tensors, nthread=2)
    prompt = rng.integers(0, cfg.n_vocab, 6).astype(np.int32)
    lg, lo = eng.forward(prompt, 0), ora.forward(prompt, 0)
    e1 = float(np.abs(lg - lo).max() / np.abs(lo).max())
    tok = int(np.argmax(lo[-1]))
    lg1, lo1 = eng.forward(np.array([tok], np.int32), 6)[0], ora.forward(np.array([tok], np.int32), 6)[0]
    e2 = float(np.abs(lg1 - lo1).max() / np.abs(lo1).max())
    assert e1 < 3e-2 and e2 < 3e-2, (e1, e2)
    toks = eng.decode_greedy(int(np.argmax(lo1)), 7, 4, use_graph=True)
    assert len(toks) == 4 and all(0 <= int(t) < cfg.n_vocab for t in toks)
    # exact-order mode: the same passes with every sum in the host backend's order -- the oracle's bits and tokens
    prev = L.spy_hip_set_exact_order(1)
    try:
        eng2, ora2 = M_.Engine(cfg, tensors), OracleModel(cfg, tensors, nthread=2)
        assert np.array_equal(eng2.forward(prompt, 0).view(np.uint32), lo.view(np.uint32)), "exact order: prompt logits differ from the oracle's bits"
        assert eng2.generate(prompt, 8).tolist() == ora2.generate(prompt, 8).tolist(), "exact order: greedy tokens differ from the oracle's"
        eng2.close()
    finally:
        L.spy_hip_set_exact_order(prev)
    eng.close()
    print("smoke ok: 2-layer token loop, prompt logits err %.2e, single-token logits err %.2e, greedy tokens %s; exact-order mode: logits bit-identical, 8 greedy tokens identical" % (e1, e2, list(map(int, toks))))
