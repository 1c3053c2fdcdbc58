"""The isolated operator sweep (configuration C5) as assertions: every kernel family at the full 7B shapes against the
CPU oracle, through the C ABI.  GEMV: all four weight types x all four matrix shapes at batch 1, every output row for the
three layer shapes and 2048 sampled rows for the 32000-row head; GEMM: batches 16, 128, 512 on all four shapes,
sampled (row, token) pairs; decode attention at KV length 512 and 4096 is in test_gpu_fused_ops.py.
Weights ~N(0, 0.02) quantized by the oracle's quantizers, activations ~N(0, 1) quantized by Quantizator<FP32,Q8_0>."""
import numpy as np
import pytest

from tests import oracle_lib as O

pytestmark = pytest.mark.gpu
TYPES = [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K]
DOT = {O.Q4_0: "spy_o_dot_q4_0_q8_0", O.Q8_0: "spy_o_dot_q8_0_q8_0", O.Q4_K: "spy_o_dot_q4_k_q8_0", O.Q6_K: "spy_o_dot_q6_k_q8_0"}
_cache = {}


def _weights(oracle, wtype, M, K):
    key = (wtype, M, K)
    if key not in _cache:
        _cache.clear()                                   # one matrix at a time (the head is 0.5 GB as floats)
        rng = np.random.default_rng(M * 7 + K + wtype)
        _cache[key] = O.quantize(oracle, (rng.standard_normal((M, K), dtype=np.float32) * np.float32(0.02)), wtype)
    return _cache[key]


@pytest.mark.parametrize("wtype", TYPES)
@pytest.mark.parametrize("M,K", [(4096, 4096), (11008, 4096), (4096, 11008), (32000, 4096)])
def test_gemv_batch_1_all_shapes_all_types(hip, oracle, wtype, M, K):
    from tests.gpu_util import dev, dev_empty, call, assert_close
    if wtype in (O.Q4_K, O.Q6_K) and K % 256:
        pytest.skip("K-quant rows are whole super-blocks of 256 elements")
    w = _weights(oracle, wtype, M, K)
    x = np.random.default_rng(K).standard_normal((1, K)).astype(np.float32)
    xq = O.quantize(oracle, x, O.Q8_0)
    dw, dxq, dout = dev(w), dev(xq), dev_empty(M * 4, 0xFF)
    call(hip.load().spy_hip_gemv_q8_0act, None, wtype, dw.ptr, dxq.ptr, dout.ptr, None, M, K, 1, M)
    got = dout.download(np.float32)
    rows = np.arange(M) if M <= 11008 else np.random.default_rng(1).choice(M, 2048, replace=False)
    rb = O.row_size(wtype, K)
    fn = getattr(oracle, DOT[wtype])
    want = np.array([fn(w.ctypes.data + int(r) * rb, O.ptr(xq), K) for r in rows], np.float32)
    assert_close(got[rows], want, "gemv %dx%d type %d (%d rows checked)" % (M, K, wtype, len(rows)))
    assert np.all(np.isfinite(got))


@pytest.mark.parametrize("T", [16, 128, 512])            # the top decorator varies fastest: one weight matrix serves its three batches
@pytest.mark.parametrize("wtype", TYPES)
@pytest.mark.parametrize("M,K", [(4096, 4096), (11008, 4096), (4096, 11008), (32000, 4096)])
def test_gemm_batches_all_types(hip, oracle, wtype, M, K, T):
    from tests.gpu_util import dev, dev_empty, call, assert_close
    if wtype in (O.Q4_K, O.Q6_K) and K % 256:
        pytest.skip("K-quant rows are whole super-blocks of 256 elements")
    w = _weights(oracle, wtype, M, K)
    x = np.random.default_rng(T * 131 + K).standard_normal((T, K)).astype(np.float32)
    xq = O.quantize(oracle, x, O.Q8_0).reshape(T, -1)
    dw, dxq, dout = dev(w), dev(xq), dev_empty(T * M * 4, 0xFF)
    call(hip.load().spy_hip_gemm_q8_0act, None, wtype, dw.ptr, dxq.ptr, dout.ptr, M, K, T, M)
    got = dout.download(np.float32).reshape(T, M)
    rng = np.random.default_rng(T + M)
    rows, toks = rng.choice(M, 192, replace=False), rng.integers(0, T, 192)
    rows[:4] = [0, M - 1, 127, 128]; toks[:4] = [0, T - 1, T - 1, 0]          # tile corners
    rb = O.row_size(wtype, K)
    fn = getattr(oracle, DOT[wtype])
    want = np.array([fn(w.ctypes.data + int(r) * rb, xq[t].ctypes.data, K) for r, t in zip(rows, toks)], np.float32)
    assert_close(got[toks, rows], want, "gemm %dx%d type %d T=%d (192 outputs checked)" % (M, K, wtype, T))
    assert np.all(np.isfinite(got))
