"""Prompt-sized products on the matrix cores: the int8-MFMA quantized GEMM and the fp16-MFMA
attention GEMM behind the MatMul operator, against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

from tests import oracle_lib as O

pytestmark = pytest.mark.gpu
B = C.byref


@pytest.fixture(scope="module")
def hip():
    from spy_amd import _lib
    _lib.init(0)
    return _lib


@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0])
@pytest.mark.parametrize("M,K,T", [(128, 4096, 128), (256, 256, 16), (200, 11008, 77), (130, 64, 129), (4096, 4096, 256),
                                   (96, 4096, 33), (70, 1024, 64), (33, 64, 17), (1000, 2048, 31)])
def test_gemm_q8_0act_matches_oracle(hip, oracle, wtype, M, K, T):
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(wtype * 131 + M + K + T)
    w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.02).astype(np.float32), wtype)
    x = rng.standard_normal((T, K)).astype(np.float32)
    x[:, : K // 2] *= 3.0                                   # blocks with different scales
    want = O.matmul(oracle, w, wtype, M, K, x, nthread=8)   # [T, M]
    xq = O.quantize(oracle, x, O.Q8_0)
    dw, dxq, dout = dev(w), dev(xq), dev_empty(T * M * 4, 0xFF)
    call(hip.load().spy_hip_gemm_q8_0act, None, wtype, dw.ptr, dxq.ptr, dout.ptr, M, K, T, M)
    assert_close(dout.download(np.float32).reshape(T, M), want, "gemm type %d %dx%d T=%d" % (wtype, M, K, T))


@pytest.mark.parametrize("tiling", ["tile", "tile64", None])
@pytest.mark.parametrize("wtype", [O.Q4_K, O.Q6_K])
@pytest.mark.parametrize("M,K,T", [(128, 4096, 128), (256, 256, 16), (200, 11008, 77), (130, 512, 129), (4096, 4096, 256)])
def test_gemm_k_quants_match_oracle(hip, oracle, wtype, M, K, T, tiling, monkeypatch):
    """Super-block weights: every sub-block scale / minimum (Q4_K) and both 16-element groups of a
    32-element MFMA block (Q6_K) take part; weights with offsets and outliers so that minima and the
    6-bit scale fields above index 3 are not trivial.  Each shape with the 128 x 128 tiling, the 64 x 64
    tiling and whatever the library picks for it."""
    from tests.gpu_util import dev, dev_empty, call, assert_close
    if tiling: monkeypatch.setenv("SPY_HIP_GEMM", tiling)
    else: monkeypatch.delenv("SPY_HIP_GEMM", raising=False)
    rng = np.random.default_rng(wtype * 977 + M + K + T)
    wf = (rng.standard_normal((M, K)) * 0.02).astype(np.float32)
    wf += (rng.standard_normal((M, K // 32, 1)) * 0.03).astype(np.float32).repeat(32, 2).reshape(M, K)
    wf[rng.random((M, K)) < 0.01] *= 8.0
    w = O.quantize(oracle, wf, wtype)
    x = rng.standard_normal((T, K)).astype(np.float32)
    x[:, : K // 2] *= 3.0
    want = O.matmul(oracle, w, wtype, M, K, x, nthread=8)
    xq = O.quantize(oracle, x, O.Q8_0)
    dw, dxq, dout = dev(w), dev(xq), dev_empty(T * M * 4, 0xFF)
    call(hip.load().spy_hip_gemm_q8_0act, None, wtype, dw.ptr, dxq.ptr, dout.ptr, M, K, T, M)
    assert_close(dout.download(np.float32).reshape(T, M), want, "gemm type %d %dx%d T=%d" % (wtype, M, K, T))


@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K])
def test_gemm_random_shapes_strided_destination_and_untouched_padding(hip, oracle, wtype):
    """Seeded ragged shapes on both sides of every kernel choice (row kernels, 32-row kernel, 64 x 64 and 128 x 128 tiles),
    written through a destination stride larger than M: the results equal the oracle's and no byte outside the T x M
    region is written (columns M .. stride-1 of every row, and a guard row behind the last one)."""
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(4000 + wtype)
    kq = wtype in (O.Q4_K, O.Q6_K)
    for case in range(6):
        M = int(rng.integers(1, 400))
        K = int(rng.integers(1, 5)) * 256 if (kq or case % 2 == 0) else int(rng.integers(1, 12)) * 64
        T = int(rng.choice([1, 2, 15, 16, 17, 31, 33, 63, 64, 65, 127, 129, 200, 257]))
        pad = int(rng.integers(1, 9))
        stride = M + pad
        w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.05).astype(np.float32), wtype)
        x = (rng.standard_normal((T, K)) * rng.choice([0.1, 1.0, 10.0])).astype(np.float32)
        want = O.matmul(oracle, w, wtype, M, K, x, nthread=8)
        xq = O.quantize(oracle, x, O.Q8_0)
        dw, dxq, dout = dev(w), dev(xq), dev_empty((T + 1) * stride * 4, 0xFF)
        call(hip.load().spy_hip_gemm_q8_0act, None, wtype, dw.ptr, dxq.ptr, dout.ptr, M, K, T, stride)
        raw = dout.download(np.uint32).reshape(T + 1, stride)
        assert np.all(raw[:T, M:] == 0xFFFFFFFF) and np.all(raw[T] == 0xFFFFFFFF), "type %d %dx%d T=%d stride %d: wrote outside the result" % (wtype, M, K, T, stride)
        assert_close(raw[:T, :M].view(np.float32), want, "gemm type %d %dx%d T=%d stride %d" % (wtype, M, K, T, stride))


def test_gemm_integer_scales_is_exact(hip, oracle):
    """With power-of-two scales and small integers every product and sum is exact in fp32: the GEMM
    must then equal the integer matrix product bit for bit (pins the MFMA operand / result layout)."""
    from tests.gpu_util import dev, dev_empty, call
    rng = np.random.default_rng(5)
    M, K, T = 160, 128, 96
    n = rng.integers(0, 16, (M, K))                                          # nibbles
    w = np.zeros((M, K // 32, 18), np.uint8)
    w[:, :, :2] = np.array([1.0], np.float16).view(np.uint8)                 # d = 1
    nb = n.reshape(M, K // 32, 32)
    w[:, :, 2:] = (nb[:, :, :16] | (nb[:, :, 16:] << 4)).astype(np.uint8)
    q = rng.integers(-127, 128, (T, K)).astype(np.int8)
    xq = np.zeros((T, K // 32, 34), np.uint8)
    xq[:, :, :2] = np.array([0.5], np.float16).view(np.uint8)                # d = 0.5
    xq[:, :, 2:] = q.reshape(T, K // 32, 32).view(np.uint8)
    dw, dxq, dout = dev(w), dev(xq), dev_empty(T * M * 4, 0xFF)
    call(hip.load().spy_hip_gemm_q8_0act, None, O.Q4_0, dw.ptr, dxq.ptr, dout.ptr, M, K, T, M)
    want = 0.5 * (q.astype(np.int64) @ (n.astype(np.int64) - 8).T)
    assert np.array_equal(dout.download(np.float32).reshape(T, M), want.astype(np.float32))


def test_op_matmul_prompt_sizes(hip, oracle):
    """MatMul operator with many activation rows: the quantized weights route to the int8 GEMM, the
    attention views (strided K cache / transposed V cache) to the fp16 GEMM."""
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(21)
    L = hip.load()
    # quantized weights
    M, K, T = 384, 512, 48
    w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.05).astype(np.float32), O.Q4_0)
    x = rng.standard_normal((T, K)).astype(np.float32)
    want = O.matmul(oracle, w, O.Q4_0, M, K, x, nthread=8)
    dw, dx, dd = dev(w), dev(x), dev_empty(T * M * 4, 0xFF)
    tw, tx, td = hip.tensor(dw, hip.Q4_0, [K, M]), hip.tensor(dx, hip.F32, [K, T]), hip.tensor(dd, hip.F32, [M, T])
    need = L.spy_hip_op_matmul_scratch_size(B(tw), B(tx))
    sc = dev_empty(need, 0)
    call(L.spy_hip_op_matmul, None, B(tw), B(tx), B(td), sc.ptr, need)
    assert_close(dd.download(np.float32).reshape(T, M), want, "op_matmul Q4_0 T=48")
    # attention products
    hd, H_, T, n_kv, Cx = 128, 4, 40, 72, 96
    d = hd * H_
    kc = rng.standard_normal((Cx, H_, hd)).astype(np.float16)
    vc = rng.standard_normal((d, Cx)).astype(np.float16)
    q = rng.standard_normal((T, H_, hd)).astype(np.float32)
    P = rng.random((H_, T, n_kv)).astype(np.float32)
    S_want = np.zeros((H_, T, n_kv), np.float32)
    O_want = np.zeros((H_, T, hd), np.float32)
    assert oracle.spy_o_matmul(B(O.tensor(kc.view(np.uint16), O.F16, [hd, n_kv, H_], nb=[2, 2 * d, 2 * hd])),
                               B(O.tensor(q, O.F32, [hd, T, H_], nb=[4, 4 * d, 4 * hd])), B(O.tensor(S_want, O.F32, [n_kv, T, H_])), 4) == 0
    assert oracle.spy_o_matmul(B(O.tensor(vc.view(np.uint16), O.F16, [n_kv, hd, H_], nb=[2, 2 * Cx, 2 * Cx * hd])),
                               B(O.tensor(P, O.F32, [n_kv, T, H_])), B(O.tensor(O_want, O.F32, [hd, T, H_])), 4) == 0
    dkc, dvc, dq, dP = dev(kc.view(np.uint16)), dev(vc.view(np.uint16)), dev(q), dev(P)
    dS, dO = dev_empty(S_want.nbytes, 0xFF), dev_empty(O_want.nbytes, 0xFF)
    tk = hip.tensor(dkc, hip.F16, [hd, n_kv, H_], nb=[2, 2 * d, 2 * hd])
    tq = hip.tensor(dq, hip.F32, [hd, T, H_], nb=[4, 4 * d, 4 * hd])
    tS = hip.tensor(dS, hip.F32, [n_kv, T, H_])
    need = L.spy_hip_op_matmul_scratch_size(B(tk), B(tq))
    sc = dev_empty(need, 0)
    call(L.spy_hip_op_matmul, None, B(tk), B(tq), B(tS), sc.ptr, need)
    assert_close(dS.download(np.float32).reshape(S_want.shape), S_want, "attn_score T=40", tol=1e-5)
    tv = hip.tensor(dvc, hip.F16, [n_kv, hd, H_], nb=[2, 2 * Cx, 2 * Cx * hd])
    tP = hip.tensor(dP, hip.F32, [n_kv, T, H_])
    tO = hip.tensor(dO, hip.F32, [hd, T, H_])
    need = L.spy_hip_op_matmul_scratch_size(B(tv), B(tP))
    sc2 = dev_empty(need, 0)
    call(L.spy_hip_op_matmul, None, B(tv), B(tP), B(tO), sc2.ptr, need)
    assert_close(dO.download(np.float32).reshape(O_want.shape), O_want, "KQV T=40", tol=1e-5)
