"""GPU parity: the HIP kernels behind the C ABI against the CPU oracle on the same seeded inputs.
Integer / byte results are compared bit for bit; float results to 1e-3 relative."""
import ctypes as C

import numpy as np
import pytest

from tests import oracle_lib as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from spy_amd import _lib as H
    H.init(0)
    print("device:", H.device_info(), flush=True)
    return H


def _weights(oracle, rng, M, K, wtype, outliers=False):
    wf = (rng.standard_normal((M, K)) * 0.02).astype(np.float32)
    if outliers:
        idx = rng.integers(0, wf.size, max(1, wf.size // 1000))
        wf.reshape(-1)[idx] *= 20
    return O.quantize(oracle, wf, wtype)


# ---- A3: Q8_0 activation quantizer, bit-exact -------------------------------------------------
@pytest.mark.parametrize("nrow,K", [(1, 32), (1, 4096), (3, 11008), (8, 4096), (512, 256)])
def test_quantize_q8_0_bit_exact(hip, oracle, nrow, K):
    from tests.gpu_util import dev, dev_empty, call
    rng = np.random.default_rng(nrow * 131 + K)
    x = (rng.standard_normal((nrow, K)) * rng.uniform(1e-3, 30, (nrow, 1))).astype(np.float32)
    # adversarial blocks: zeros, ties at .5, a single outlier, denormal scale, negative max
    x[0, :32] = 0.0
    if K >= 128:
        x[0, 32:64] = np.concatenate([[127.0], np.arange(31) + 0.5]).astype(np.float32)
        x[0, 64:96] = 1e-3; x[0, 70] = 1e4
        x[0, 96:128] = (rng.standard_normal(32) * 1e-7).astype(np.float32)
    want = O.quantize(oracle, x, O.Q8_0)
    dx, dy = dev(x), dev_empty(want.nbytes, 0xAA)
    call(hip.load().spy_hip_quantize_q8_0, None, dx.ptr, K * 4, dy.ptr, nrow, K)
    got = dy.download(np.uint8)
    assert np.array_equal(got, want)


def test_quantize_q8_0_strided_rows(hip, oracle):
    from tests.gpu_util import dev, dev_empty, call
    rng = np.random.default_rng(77)
    x = rng.standard_normal((5, 512)).astype(np.float32)
    dx, dy = dev(x), dev_empty(5 * 8 * 34, 0)
    call(hip.load().spy_hip_quantize_q8_0, None, dx.ptr, 512 * 4, dy.ptr, 5, 256)   # first 256 of each 512-float row
    want = O.quantize(oracle, x[:, :256], O.Q8_0)
    assert np.array_equal(dy.download(np.uint8), want)


# ---- A4/A5/A15: int32 block dots, bit-exact, from the GEMV kernels themselves ----------------------
@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K])
@pytest.mark.parametrize("M,K", [(5, 256), (37, 4096), (9, 11008), (6, 96), (3, 32)])
def test_block_dots_bit_exact(hip, oracle, wtype, M, K):
    from tests.gpu_util import dev, dev_empty, call
    if wtype in (O.Q4_K, O.Q6_K) and K % 256:
        pytest.skip("super-blocks need K % 256 == 0")
    rng = np.random.default_rng(wtype * 1000 + M + K)
    w = _weights(oracle, rng, M, K, wtype, outliers=True)
    xq = O.quantize(oracle, rng.standard_normal(K).astype(np.float32), O.Q8_0)
    nsub = K // 16 if wtype == O.Q6_K else K // 32
    want = np.zeros((M, nsub), dtype=np.int32)
    rs = O.row_size(wtype, K)
    for m in range(M):
        assert oracle.spy_o_block_dots(wtype, w.ctypes.data + m * rs, O.ptr(xq), K, want[m].ctypes.data) == 0
    dw, dxq, dout = dev(w), dev(xq), dev_empty((M * nsub + M) * 4, 0xCD)
    call(hip.load().spy_hip_block_dots, None, wtype, dw.ptr, dxq.ptr, dout.ptr, M, K)
    got = dout.download(np.int32, M * nsub).reshape(M, nsub)
    assert np.array_equal(got, want)


# ---- A4/A5/A7/A15: GEMV float results --------------------------------------------------------------
@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K])
@pytest.mark.parametrize("M,K,T", [(64, 4096, 1), (129, 4096, 3), (40, 11008, 1), (33, 11008, 11), (16, 256, 8), (7, 64, 2)])
def test_gemv_matches_oracle(hip, oracle, wtype, M, K, T):
    from tests.gpu_util import dev, dev_empty, call, assert_close
    if wtype in (O.Q4_K, O.Q6_K) and K % 256:
        pytest.skip("super-blocks need K % 256 == 0")
    rng = np.random.default_rng(wtype * 7919 + M * 31 + K + T)
    w = _weights(oracle, rng, M, K, wtype)
    x = rng.standard_normal((T, K)).astype(np.float32)
    want = O.matmul(oracle, w, wtype, M, K, x, nthread=4)                 # [T, M]
    xq = O.quantize(oracle, x, O.Q8_0)
    res = rng.standard_normal((T, M)).astype(np.float32)
    dw, dxq, dres = dev(w), dev(xq), dev(res)
    dout = dev_empty(T * M * 4, 0xFF)
    L = hip.load()
    call(L.spy_hip_gemv_q8_0act, None, wtype, dw.ptr, dxq.ptr, dout.ptr, None, M, K, T, M)
    assert_close(dout.download(np.float32).reshape(T, M), want, "gemv type %d %dx%d T=%d" % (wtype, M, K, T))
    call(L.spy_hip_gemv_q8_0act, None, wtype, dw.ptr, dxq.ptr, dout.ptr, dres.ptr, M, K, T, M)
    assert_close(dout.download(np.float32).reshape(T, M), want + res, "gemv+residual type %d" % wtype)


def test_gemv_zero_scale_and_single_block(hip, oracle):
    from tests.gpu_util import dev, dev_empty, call
    w = np.zeros((4, 18), np.uint8); w[:, 2:] = 0x5A                      # d = 0: every dot is exactly 0
    xq = O.quantize(oracle, np.linspace(-1, 1, 32).astype(np.float32), O.Q8_0)
    dw, dxq, dout = dev(w), dev(xq), dev_empty(16, 0xFF)          # keep the buffers alive across the launch
    call(hip.load().spy_hip_gemv_q8_0act, None, O.Q4_0, dw.ptr, dxq.ptr, dout.ptr, None, 4, 32, 1, 4)
    assert np.array_equal(dout.download(np.float32), np.zeros(4, np.float32))


def test_gemv_full_shapes_linearity(hip, oracle):
    """Full 7B shapes, checked through a size-independent property instead of the oracle:
    W.(a) + W.(b) with exact-integer activations equals the oracle on 64 sampled rows."""
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(2024)
    for M, K in [(4096, 4096), (11008, 4096), (4096, 11008)]:
        w = rng.integers(0, 256, (M, K // 32, 18), dtype=np.uint8)
        w[:, :, :2] = (rng.uniform(0.5, 2, (M, K // 32)) * 0.0025).astype(np.float16).view(np.uint8).reshape(M, K // 32, 2)
        x = rng.standard_normal((1, K)).astype(np.float32)
        xq = O.quantize(oracle, x, O.Q8_0)
        dw, dxq, dout = dev(w), dev(xq), dev_empty(M * 4, 0xFF)
        call(hip.load().spy_hip_gemv_q8_0act, None, O.Q4_0, dw.ptr, dxq.ptr, dout.ptr, None, M, K, 1, M)
        got = dout.download(np.float32)
        rows = rng.choice(M, 64, replace=False)
        want = np.array([oracle.spy_o_dot_q4_0_q8_0(w[r].ctypes.data, O.ptr(xq), K) for r in rows], np.float32)
        scale = float(np.abs(want).max())
        assert float(np.abs(got[rows] - want).max()) <= 1e-3 * scale
        assert np.all(np.isfinite(got))


@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0])
@pytest.mark.parametrize("M,K,T", [(20011, 256, 1), (9003, 6400, 2), (5000, 12800, 1)])
def test_gemv_many_row_tiles(hip, oracle, wtype, M, K, T):
    """More row tiles than resident workgroups: every workgroup walks several tiles (both weight
    register buffers in use), for each lanes-per-row configuration."""
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(M + K)
    nblk = K // 32
    bs = O.TYPE_SIZE[wtype]
    w = rng.integers(0, 256, (M, nblk, bs), dtype=np.uint8)
    w[:, :, :2] = (rng.uniform(0.5, 2, (M, nblk)) * 0.0025).astype(np.float16).view(np.uint8).reshape(M, nblk, 2)
    if wtype == O.Q8_0:
        w[:, :, 2:][w[:, :, 2:] == 0x80] = 0x81                         # keep quants in [-127, 127]
    x = rng.standard_normal((T, K)).astype(np.float32)
    want = O.matmul(oracle, w, wtype, M, K, x, nthread=8)
    xq = O.quantize(oracle, x, O.Q8_0)
    dw, dxq, dout = dev(w), dev(xq), dev_empty(T * M * 4, 0xFF)
    call(hip.load().spy_hip_gemv_q8_0act, None, wtype, dw.ptr, dxq.ptr, dout.ptr, None, M, K, T, M)
    assert_close(dout.download(np.float32).reshape(T, M), want, "gemv type %d %dx%d T=%d" % (wtype, M, K, T))
