"""Exact-order mode of the operator entry points (spy_hip_set_exact_order): every float sum in the order
of the host backend's loops (vec_dot.h:42-146, vec_util.h:75-81, non-linear.cpp:129-223 in the Spy tree),
exp / silu / cos / sin from the host's libm.  The bar here is equality of the BITS with the CPU oracle:
per operator, for a whole model through Backend::submit, and for the greedy tokens of the 7B shape."""
import ctypes as C
import os

import numpy as np
import pytest

from tests import oracle_lib as O

pytestmark = pytest.mark.gpu


@pytest.fixture()
def hip():
    from spy_amd import _lib as H
    H.init(0)
    prev = H.load().spy_hip_set_exact_order(1)
    yield H
    H.load().spy_hip_set_exact_order(prev)


def B(t):
    return C.byref(t)


def _same_bits(got, want, what):
    got, want = np.ascontiguousarray(got, np.float32), np.ascontiguousarray(want, np.float32)
    bad = got.view(np.uint32) != want.view(np.uint32)
    assert not bad.any(), "%s: %d of %d outputs differ in their bits, largest difference %.3e" % (
        what, int(bad.sum()), bad.size, float(np.abs(got.astype(np.float64) - want.astype(np.float64))[bad].max()))


@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K])
@pytest.mark.parametrize("M,K,T", [(96, 4096, 5), (40, 11008, 1), (33, 256, 3)])
@pytest.mark.parametrize("serial", [False, True])
def test_quantized_matmul_bits(hip, oracle, wtype, M, K, T, serial, monkeypatch):
    """serial: one thread per output element (the plain restatement); otherwise the eight accumulators of an
    output element in eight lanes (Q4_0 / Q8_0).  Both must give the oracle's bits."""
    from tests.gpu_util import dev, dev_empty, call
    if serial:
        monkeypatch.setenv("SPY_HIP_EXACT_SERIAL", "1")
    if K % 256 and wtype in (O.Q4_K, O.Q6_K):
        pytest.skip("K-quant rows are whole super-blocks")
    rng = np.random.default_rng(100 * wtype + K + T)
    w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.02).astype(np.float32), wtype)
    x = (rng.standard_normal((T, K)) * rng.uniform(0.1, 30.0, (T, 1))).astype(np.float32)
    want = O.matmul(oracle, w, wtype, M, K, x, nthread=4)
    dw, dx, dd = dev(w), dev(x), dev_empty(T * M * 4, 0xFF)
    tw, tx, td = hip.tensor(dw, wtype, [K, M]), hip.tensor(dx, hip.F32, [K, T]), hip.tensor(dd, hip.F32, [M, T])
    L = hip.load()
    need = L.spy_hip_op_matmul_scratch_size(B(tw), B(tx))
    scratch = dev_empty(need, 0)
    call(L.spy_hip_op_matmul, None, B(tw), B(tx), B(td), scratch.ptr, need)
    _same_bits(dd.download(np.float32).reshape(T, M), want, "matmul type %d %dx%d T %d" % (wtype, M, K, T))


@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K])
@pytest.mark.parametrize("M,K", [(100, 4096), (4096, 4096), (37, 128), (33, 256), (50, 8192), (21, 11008), (19, 16384)])
def test_single_row_matmul_takes_the_two_phase_kernel(hip, oracle, wtype, M, K, monkeypatch):
    """One f32 activation row against a quantized matrix (every MatMul of a single-token pass through Backend::submit) runs as ONE
    launch of the fused pass's two-phase kernel, which quantizes the row itself: the oracle's bits, and the bits of the lane
    kernels behind SPY_HIP_EXACT_TILED=0, for row counts that are no multiple of the 16 rows of a workgroup and for one to
    four slabs of K."""
    from tests.gpu_util import dev, dev_empty, call
    kq = wtype in (O.Q4_K, O.Q6_K)
    if kq and (K % 256 or K > 12288):
        pytest.skip("K-quant rows: whole super-blocks, at most three slabs")
    rng = np.random.default_rng(31 * wtype + M + K)
    w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.02).astype(np.float32), wtype)
    x = (rng.standard_normal((1, K)) * 3.0).astype(np.float32)
    x[0, 5] = 0.0
    x[0, 64:96] = 0.0                                                   # a block of zeros: scale 0
    want = O.matmul(oracle, w, wtype, M, K, x, nthread=4)
    dw, dx = dev(w), dev(x)
    tw, tx = hip.tensor(dw, wtype, [K, M]), hip.tensor(dx, hip.F32, [K, 1])
    L = hip.load()
    need = L.spy_hip_op_matmul_scratch_size(B(tw), B(tx))
    scratch = dev_empty(need, 0xEE)
    for tiled in ("1", "0"):
        monkeypatch.setenv("SPY_HIP_EXACT_TILED", tiled)
        dd = dev_empty(M * 4 + 64, 0xFF)
        call(L.spy_hip_op_matmul, None, B(tw), B(tx), B(hip.tensor(dd, hip.F32, [M, 1])), scratch.ptr, need)
        got = dd.download(np.float32)
        _same_bits(got[:M].reshape(1, M), want, "single-row matmul type %d %dx%d, SPY_HIP_EXACT_TILED=%s" % (wtype, M, K, tiled))
        assert (got[M:].view(np.uint32) == 0xFFFFFFFF).all(), "nothing is written beyond the M outputs"
        if tiled == "1":
            # the one-launch route leaves the scratch buffer alone (the row is quantized in LDS)
            assert (scratch.download(np.uint8) == 0xEE).all(), "the single-row route does not use the scratch buffer"


@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K])
@pytest.mark.parametrize("M,K,T", [(96, 4096, 16), (200, 512, 70), (64, 128, 64), (64, 256, 64), (132, 11008, 33), (4096, 4096, 130)])
def test_tiled_matmul_bits(hip, oracle, wtype, M, K, T, monkeypatch):
    """Sixteen activation rows and more take the tiled kernel (64 x 64 outputs per workgroup, the eight accumulators
    of every output in registers): the oracle's bits, with whole and partial tiles along both sides, and the same
    bits as the row kernels give (SPY_HIP_EXACT_TILED=0)."""
    from tests.gpu_util import dev, dev_empty, call
    if K % 256 and wtype in (O.Q4_K, O.Q6_K):
        pytest.skip("K-quant rows are whole super-blocks")
    rng = np.random.default_rng(7 * wtype + M + K + T)
    w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.02).astype(np.float32), wtype)
    x = (rng.standard_normal((T, K)) * rng.uniform(0.1, 30.0, (T, 1))).astype(np.float32)
    want = O.matmul(oracle, w, wtype, M, K, x, nthread=8)
    dw, dx = dev(w), dev(x)
    tw, tx = hip.tensor(dw, wtype, [K, M]), hip.tensor(dx, hip.F32, [K, T])
    L = hip.load()
    need = L.spy_hip_op_matmul_scratch_size(B(tw), B(tx))
    scratch = dev_empty(need, 0)
    for tiled in ("1", "u", "0"):          # tiled kernel from packed operands, unpacking per tile, row kernels
        monkeypatch.setenv("SPY_HIP_EXACT_TILED", tiled)
        dd = dev_empty(T * M * 4, 0xFF)
        td = hip.tensor(dd, hip.F32, [M, T])
        call(L.spy_hip_op_matmul, None, B(tw), B(tx), B(td), scratch.ptr, need)
        _same_bits(dd.download(np.float32).reshape(T, M), want, "matmul type %d %dx%d T %d tiled %s" % (wtype, M, K, T, tiled))
    # a scratch buffer that holds the converted activations and nothing else: no room for packed operands, same bits
    monkeypatch.setenv("SPY_HIP_EXACT_TILED", "1")
    act = T * (K // 32) * 34
    assert act <= need
    small = dev_empty(act, 0)
    dd = dev_empty(T * M * 4, 0xFF)
    call(L.spy_hip_op_matmul, None, B(tw), B(tx), B(hip.tensor(dd, hip.F32, [M, T])), small.ptr, act)
    _same_bits(dd.download(np.float32).reshape(T, M), want, "matmul type %d %dx%d T %d, activations-only scratch" % (wtype, M, K, T))
    if wtype in (O.Q4_0, O.Q8_0) and T >= 16 and (K // 32) % 2 == 0:
        assert need > act + 2 * (M + T) * K, "the scratch size of the exact order covers the packed operands"


@pytest.mark.parametrize("T", [1, 2, 40])
def test_q8_0_weights_of_any_byte(hip, oracle, T):
    """Weight bytes a quantizer never writes (-128): the host backend's sign / maddubs sequence
    (vec_util.h:101-110) gives 128 * -128 for (-128) * (-128); the exact mode follows it.  T = 2: the row kernel;
    T = 40: the tiled kernel, whose plain signed products are the same numbers because the activation bytes,
    quantized inside the call, never reach -128."""
    from tests.gpu_util import dev, dev_empty, call
    rng = np.random.default_rng(77)
    M, K = 16, 512
    w = O.quantize(oracle, rng.standard_normal((M, K)).astype(np.float32), O.Q8_0).copy()
    blocks = w.reshape(M * K // 32, 34)
    blocks[:, 2:] = rng.integers(0, 256, (blocks.shape[0], 32), dtype=np.uint8)
    blocks[::3, 2:6] = 0x80
    x = rng.standard_normal((T, K)).astype(np.float32)
    want = O.matmul(oracle, w, O.Q8_0, M, K, x, nthread=1)
    dw, dx, dd = dev(w), dev(x), dev_empty(T * M * 4, 0xFF)
    tw, tx, td = hip.tensor(dw, O.Q8_0, [K, M]), hip.tensor(dx, hip.F32, [K, T]), hip.tensor(dd, hip.F32, [M, T])
    L = hip.load()
    need = L.spy_hip_op_matmul_scratch_size(B(tw), B(tx))
    scratch = dev_empty(need, 0)
    call(L.spy_hip_op_matmul, None, B(tw), B(tx), B(td), scratch.ptr, need)
    _same_bits(dd.download(np.float32).reshape(T, M), want, "Q8_0 with arbitrary weight bytes")


@pytest.mark.parametrize("n_kv", [1, 31, 32, 33, 64, 65, 300, 4241])
@pytest.mark.parametrize("serial", [False, True])
def test_attention_products_bits(hip, oracle, n_kv, serial, monkeypatch):
    """attn_score (contraction over 128) and KQV (contraction over n_kv: the strict `i + 32 < n` loop bound
    and the scalar tail of Dot<FP16,FP16>, vec_dot.h:124-145) through the cache views."""
    from tests.gpu_util import dev, dev_empty, call
    if serial:
        monkeypatch.setenv("SPY_HIP_EXACT_SERIAL", "1")
    rng = np.random.default_rng(9 + n_kv)
    hd, H_, T = 128, 4, 2
    Cx = n_kv + 11
    d = hd * H_
    kc = rng.standard_normal((Cx, H_, hd)).astype(np.float16)
    vc = rng.standard_normal((d, Cx)).astype(np.float16)
    q = rng.standard_normal((T, H_, hd)).astype(np.float32)
    P = rng.random((H_, T, n_kv)).astype(np.float32)
    S_want, O_want = np.zeros((H_, T, n_kv), np.float32), np.zeros((H_, T, hd), np.float32)
    assert oracle.spy_o_matmul(B(O.tensor(kc.view(np.uint16), O.F16, [hd, n_kv, H_], nb=[2, 2 * d, 2 * hd])),
                               B(O.tensor(q, O.F32, [hd, T, H_], nb=[4, 4 * d, 4 * hd])), B(O.tensor(S_want, O.F32, [n_kv, T, H_])), 2) == 0
    assert oracle.spy_o_matmul(B(O.tensor(vc.view(np.uint16), O.F16, [n_kv, hd, H_], nb=[2, 2 * Cx, 2 * Cx * hd])),
                               B(O.tensor(P, O.F32, [n_kv, T, H_])), B(O.tensor(O_want, O.F32, [hd, T, H_])), 2) == 0
    L = hip.load()
    dkc, dvc, dq, dP = dev(kc.view(np.uint16)), dev(vc.view(np.uint16)), dev(q), dev(P)
    dS, dO = dev_empty(S_want.nbytes, 0xFF), dev_empty(O_want.nbytes, 0xFF)
    tk = hip.tensor(dkc, hip.F16, [hd, n_kv, H_], nb=[2, 2 * d, 2 * hd])
    tq = hip.tensor(dq, hip.F32, [hd, T, H_], nb=[4, 4 * d, 4 * hd])
    tS = hip.tensor(dS, hip.F32, [n_kv, T, H_])
    tv = hip.tensor(dvc, hip.F16, [n_kv, hd, H_], nb=[2, 2 * Cx, 2 * Cx * hd])
    tP, tO = hip.tensor(dP, hip.F32, [n_kv, T, H_]), hip.tensor(dO, hip.F32, [hd, T, H_])
    need = max(L.spy_hip_op_matmul_scratch_size(B(tk), B(tq)), L.spy_hip_op_matmul_scratch_size(B(tv), B(tP)), 256)
    sc = dev_empty(need, 0)
    call(L.spy_hip_op_matmul, None, B(tk), B(tq), B(tS), sc.ptr, need)
    _same_bits(dS.download(np.float32).reshape(S_want.shape), S_want, "attn_score n_kv %d" % n_kv)
    call(L.spy_hip_op_matmul, None, B(tv), B(tP), B(tO), sc.ptr, need)
    _same_bits(dO.download(np.float32).reshape(O_want.shape), O_want, "KQV n_kv %d" % n_kv)


@pytest.mark.parametrize("H_,past,T,n_ctx,cuts", [
    (32, 0, 40, 64, (0, 40)),                 # all 32 heads, a pass shorter than two chunks of 32
    (4, 168, 136, 448, (0, 136)),             # on top of cached tokens
    (2, 57, 200, 320, (0, 37, 101, 200)),     # the same pass in three pieces: row length 257 (tail of one, remainder of one)
    (2, 0, 230, 256, (0, 64, 230)),           # row length 230: 6 elements in the scalar tail, 2 in the softmax remainder
    (1, 4000, 95, 4096, (0, 32, 95)),         # long rows: row length 4095, tail of 31, remainder of 3
    (3, 31, 1, 64, (0, 1)),                   # one query row
])
def test_exact_prompt_attention_bits(hip, oracle, H_, past, T, n_ctx, cuts):
    """spy_hip_prompt_attention_exact against the oracle's MatMul(K view, q) -> Softmax(causal mask, scale) ->
    MatMul(V^T view, P) over the whole pass: equal bits, also when the pass is handed over in pieces (each piece is told
    the row length of the whole pass)."""
    from tests.gpu_util import dev, dev_empty, call
    hd, n_kv = 128, past + T
    d = H_ * hd
    rng = np.random.default_rng(17 * T + past)
    scale = float(1.0 / np.sqrt(hd))
    q = (rng.standard_normal((T, H_, hd)) * 1.5).astype(np.float32)
    kc = np.zeros((n_ctx, d), np.float16); kc[:n_kv] = rng.standard_normal((n_kv, d)).astype(np.float16)
    vc = np.full((d, n_ctx), np.nan, np.float16); vc[:, :n_kv] = rng.standard_normal((d, n_kv)).astype(np.float16)   # NaN where nothing is cached yet
    mask = np.where(np.arange(n_ctx)[None, :] <= (np.arange(T)[:, None] + past), 0.0, -np.inf).astype(np.float32)
    S_o, P_o = np.zeros((H_, T, n_kv), np.float32), np.zeros((H_, T, n_kv), np.float32)
    O_o = np.zeros((H_, T, hd), np.float32)
    assert oracle.spy_o_matmul(B(O.tensor(kc.view(np.uint16), O.F16, [hd, n_kv, H_], nb=[2, 2 * d, 2 * hd])),
                               B(O.tensor(q, O.F32, [hd, T, H_], nb=[4, 4 * d, 4 * hd])), B(O.tensor(S_o, O.F32, [n_kv, T, H_])), 4) == 0
    assert oracle.spy_o_softmax(B(O.tensor(S_o, O.F32, [n_kv, T, H_])), B(O.tensor(mask, O.I32, [n_ctx, T])), B(O.tensor(P_o, O.F32, [n_kv, T, H_])), scale) == 0
    vc_o = np.where(np.isnan(vc), np.float16(0), vc)          # the oracle multiplies the masked zeros with what the cache holds
    assert oracle.spy_o_matmul(B(O.tensor(vc_o.view(np.uint16), O.F16, [n_kv, hd, H_], nb=[2, 2 * n_ctx, 2 * n_ctx * hd])),
                               B(O.tensor(P_o, O.F32, [n_kv, T, H_])), B(O.tensor(O_o, O.F32, [hd, T, H_])), 4) == 0
    want = np.ascontiguousarray(O_o.transpose(1, 0, 2)).reshape(T, d)
    L = hip.load()
    dq, dk, dv = dev(q), dev(kc.view(np.uint16)), dev(vc.view(np.uint16))
    out = dev_empty(T * d * 4, 0xFF)
    for a, b in zip(cuts[:-1], cuts[1:]):
        need = L.spy_hip_prompt_attention_exact_scratch_size(b - a, H_, past + a)
        sc = dev_empty(need, 0xFF)
        call(L.spy_hip_prompt_attention_exact, None, dq.ptr + a * d * 4, dk.ptr, dv.ptr, out.ptr + a * d * 4, b - a, H_, hd, past + a, n_ctx, n_kv, scale, sc.ptr, need)
    _same_bits(out.download(np.float32).reshape(T, d), want, "attention H %d past %d T %d in %d pieces" % (H_, past, T, len(cuts) - 1))
    assert L.spy_hip_prompt_attention_exact(None, dq.ptr, dk.ptr, dv.ptr, out.ptr, T, H_, 64, past, n_ctx, n_kv, scale, sc.ptr, need) == hip.EUNSUPPORTED
    assert L.spy_hip_prompt_attention_exact(None, dq.ptr, dk.ptr, dv.ptr, out.ptr, T, H_, hd, past, n_ctx, n_kv, scale, sc.ptr, 1024) == hip.ENOSPACE


def test_norm_softmax_silu_rope_bits(hip, oracle):
    from tests.gpu_util import dev, dev_empty, call
    L = hip.load()
    rng = np.random.default_rng(21)
    # NormRMS: rows of whole groups of four, with a remainder, longer than one LDS pass
    for T, d in [(1, 4096), (7, 4096), (2, 103), (3, 11008), (2, 4099), (1, 3)]:
        x = (rng.standard_normal((T, d)) * 2.5).astype(np.float32)
        want = np.zeros_like(x)
        assert oracle.spy_o_norm_rms(B(O.tensor(x, O.F32, [d, T])), B(O.tensor(want, O.F32, [d, T])), 1e-5) == 0
        dx, dy = dev(x), dev_empty(x.nbytes, 0xFF)
        call(L.spy_hip_op_norm_rms, None, B(hip.tensor(dx, hip.F32, [d, T])), B(hip.tensor(dy, hip.F32, [d, T])), 1e-5)
        _same_bits(dy.download(np.float32).reshape(T, d), want, "norm_rms %dx%d" % (T, d))
    # Silu: every fp16 bit pattern that is a finite number, and fp32 values between them
    bits = np.arange(0, 0x10000, dtype=np.uint16)
    finite = (bits & 0x7C00) != 0x7C00
    x = np.concatenate([bits[finite].view(np.float16).astype(np.float32), rng.standard_normal(4096).astype(np.float32) * 4])
    want = np.zeros_like(x)
    assert oracle.spy_o_silu(B(O.tensor(x, O.F32, [x.size])), B(O.tensor(want, O.F32, [x.size]))) == 0
    dx, dy = dev(x), dev_empty(x.nbytes, 0xFF)
    call(L.spy_hip_op_silu, None, B(hip.tensor(dx, hip.F32, [x.size])), B(hip.tensor(dy, hip.F32, [x.size])))
    _same_bits(dy.download(np.float32), want, "silu")
    # Softmax: causal mask, no mask, rows shorter and longer than one LDS pass
    scale = float(1.0 / np.sqrt(128.0))
    for (H_, T, n_kv, Cx, P) in [(32, 1, 300, 512, 299), (4, 5, 9, 16, 4), (2, 3, 1030, 1100, 1027), (2, 2, 4243, 4352, 4241), (1, 1, 1, 8, 0)]:
        s = (rng.standard_normal((H_, T, n_kv)) * 12).astype(np.float32)
        mask = np.where(np.arange(Cx)[None, :] <= (np.arange(T)[:, None] + P), 0.0, -np.inf).astype(np.float32)
        ds, dm, dd = dev(s), dev(mask), dev_empty(s.nbytes, 0xFF)
        for use_mask in (True, False):
            want = np.zeros_like(s)
            assert oracle.spy_o_softmax(B(O.tensor(s, O.F32, [n_kv, T, H_])), B(O.tensor(mask, O.I32, [Cx, T])) if use_mask else None,
                                        B(O.tensor(want, O.F32, [n_kv, T, H_])), scale) == 0
            call(L.spy_hip_op_softmax, None, B(hip.tensor(ds, hip.F32, [n_kv, T, H_])), B(hip.tensor(dm, hip.I32, [Cx, T])) if use_mask else None,
                 B(hip.tensor(dd, hip.F32, [n_kv, T, H_])), scale)
            _same_bits(dd.download(np.float32).reshape(s.shape), want, "softmax H%d T%d n_kv%d mask %d" % (H_, T, n_kv, use_mask))
    # Rope
    hd, H_, T = 128, 32, 7
    pos = np.array([0, 1, 7, 100, 2047, 4095, 4351], dtype=np.int32)
    x = rng.standard_normal((T, H_, hd)).astype(np.float32)
    want = np.zeros_like(x)
    rp = O.default_rope(hd, 4352)
    assert oracle.spy_o_rope(B(O.tensor(x, O.F32, [hd, H_, T])), B(O.tensor(pos, O.I32, [T])), B(O.tensor(want, O.F32, [hd, H_, T])), B(rp)) == 0
    dx, dp, dy = dev(x), dev(pos), dev_empty(x.nbytes, 0xFF)
    # with a context length: one table of all positions kept on the device; without: the positions read back per call
    for n_ctx in (4352, 0):
        hp = hip.RopeParam(0, 0, hd, n_ctx, 4352, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, 0.0, 0)
        dy = dev_empty(x.nbytes, 0xFF)
        call(L.spy_hip_op_rope, None, B(hip.tensor(dx, hip.F32, [hd, H_, T])), B(hip.tensor(dp, hip.I32, [T])), B(hip.tensor(dy, hip.F32, [hd, H_, T])), B(hp))
        _same_bits(dy.download(np.float32).reshape(x.shape), want, "rope, context %d" % n_ctx)
    # YaRN magnitude and xpos: tables of this call's tokens from the host, zeta beside cos / sin
    for kw in (dict(freq_scale=0.25, extend_factor=1.0, attention_factor=1.1), dict(xpos_base=512.0, xpos_down=0),
               dict(freq_scale=0.5, extend_factor=0.7, xpos_base=300.0, xpos_down=1)):
        rp2 = O.default_rope(hd, 4352)
        hp = hip.RopeParam(0, 0, hd, 4352, 4352, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, 0.0, 0)
        for k, v in kw.items():
            setattr(rp2, k, v); setattr(hp, k, v)
        want2 = np.zeros_like(x)
        assert oracle.spy_o_rope(B(O.tensor(x, O.F32, [hd, H_, T])), B(O.tensor(pos, O.I32, [T])), B(O.tensor(want2, O.F32, [hd, H_, T])), B(rp2)) == 0
        dy = dev_empty(x.nbytes, 0xFF)
        call(L.spy_hip_op_rope, None, B(hip.tensor(dx, hip.F32, [hd, H_, T])), B(hip.tensor(dp, hip.I32, [T])), B(hip.tensor(dy, hip.F32, [hd, H_, T])), B(hp))
        _same_bits(dy.download(np.float32).reshape(x.shape), want2, "rope %s" % kw)
    flag = C.c_int32(-1)
    call(L.spy_hip_take_error, C.byref(flag)); assert flag.value == 0
    hp = hip.RopeParam(0, 0, hd, 4096, 4096, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, 0.0, 0)       # position 4351 lies beyond this context
    call(L.spy_hip_op_rope, None, B(hip.tensor(dx, hip.F32, [hd, H_, T])), B(hip.tensor(dp, hip.I32, [T])), B(hip.tensor(dy, hip.F32, [hd, H_, T])), B(hp))
    call(L.spy_hip_take_error, C.byref(flag)); assert flag.value == 1


def test_exact_order_operators_under_stream_capture(hip, oracle):
    """The exact-order Silu, Softmax and Rope recorded under HIP stream capture and replayed: the operator entry points
    allocate nothing and wait for nothing once spy_hip_init has built the device's tables (and spy_hip_rope_prepare the
    table of the Rope parameters), so the recording succeeds, and every replay -- with eager calls of the same operators on
    other data in between -- leaves the oracle's bits.  An exact-order Rope whose table was not prepared is refused under
    capture (it would have to allocate) and the capture survives the refusal."""
    from tests.gpu_util import dev, dev_empty, call
    L = hip.load()
    rng = np.random.default_rng(33)
    hd, H_, T, n_kv, Cx = 128, 4, 3, 700, 768
    scale = float(1.0 / np.sqrt(128.0))
    g = (rng.standard_normal(2048) * 3).astype(np.float32)
    s = (rng.standard_normal((H_, T, n_kv)) * 9).astype(np.float32)
    mask = np.where(np.arange(Cx)[None, :] <= (np.arange(T)[:, None] + n_kv - T), 0.0, -np.inf).astype(np.float32)
    xr = rng.standard_normal((T, H_, hd)).astype(np.float32)
    pos = np.array([5, 400, 767], np.int32)
    w_silu, w_soft, w_rope = np.zeros_like(g), np.zeros_like(s), np.zeros_like(xr)
    assert oracle.spy_o_silu(B(O.tensor(g, O.F32, [g.size])), B(O.tensor(w_silu, O.F32, [g.size]))) == 0
    assert oracle.spy_o_softmax(B(O.tensor(s, O.F32, [n_kv, T, H_])), B(O.tensor(mask, O.I32, [Cx, T])), B(O.tensor(w_soft, O.F32, [n_kv, T, H_])), scale) == 0
    rp = O.default_rope(hd, Cx)
    assert oracle.spy_o_rope(B(O.tensor(xr, O.F32, [hd, H_, T])), B(O.tensor(pos, O.I32, [T])), B(O.tensor(w_rope, O.F32, [hd, H_, T])), B(rp)) == 0
    dg, ds, dm, dx, dp = dev(g), dev(s), dev(mask), dev(xr), dev(pos)
    o_silu, o_soft, o_rope = dev_empty(g.nbytes, 0xFF), dev_empty(s.nbytes, 0xFF), dev_empty(xr.nbytes, 0xFF)
    hp = hip.RopeParam(0, 0, hd, Cx, Cx, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, 0.0, 0)
    hp_new = hip.RopeParam(0, 0, hd, Cx, Cx, 5000.0, 1.0, 0.0, 1.0, 32.0, 1.0, 0.0, 0)       # a parameter set nobody prepared
    call(L.spy_hip_rope_prepare, B(hp), hd)
    st = C.c_void_p()
    call(L.spy_hip_stream_create, C.byref(st))
    t_g, t_os = hip.tensor(dg, hip.F32, [g.size]), hip.tensor(o_silu, hip.F32, [g.size])
    t_s, t_m, t_o = hip.tensor(ds, hip.F32, [n_kv, T, H_]), hip.tensor(dm, hip.I32, [Cx, T]), hip.tensor(o_soft, hip.F32, [n_kv, T, H_])
    t_x, t_p, t_r = hip.tensor(dx, hip.F32, [hd, H_, T]), hip.tensor(dp, hip.I32, [T]), hip.tensor(o_rope, hip.F32, [hd, H_, T])
    # a single-row MatMul with 8192-wide Q8_0 rows: its launch needs 86 KB of LDS, a limit that spy_hip_init has raised already
    Mm, Km = 64, 8192
    wm = O.quantize(oracle, (rng.standard_normal((Mm, Km)) * 0.02).astype(np.float32), O.Q8_0)
    xm = rng.standard_normal((1, Km)).astype(np.float32)
    w_mm = O.matmul(oracle, wm, O.Q8_0, Mm, Km, xm, nthread=2)
    dwm, dxm, o_mm = dev(wm), dev(xm), dev_empty(Mm * 4, 0xFF)
    t_wm, t_xm, t_om = hip.tensor(dwm, hip.Q8_0, [Km, Mm]), hip.tensor(dxm, hip.F32, [Km, 1]), hip.tensor(o_mm, hip.F32, [Mm, 1])
    mm_need = L.spy_hip_op_matmul_scratch_size(B(t_wm), B(t_xm))
    mm_scratch = dev_empty(mm_need, 0)
    print("capture: exact-order silu, softmax, rope, single-row matmul", flush=True)
    call(L.spy_hip_capture_begin, st)
    rcs = [L.spy_hip_op_silu(st, B(t_g), B(t_os)), L.spy_hip_op_softmax(st, B(t_s), B(t_m), B(t_o), scale), L.spy_hip_op_rope(st, B(t_x), B(t_p), B(t_r), B(hp))]
    rc_mm = L.spy_hip_op_matmul(st, B(t_wm), B(t_xm), B(t_om), mm_scratch.ptr, mm_need)
    rc_unprepared = L.spy_hip_op_rope(st, B(t_x), B(t_p), B(t_r), B(hp_new))
    gexec = C.c_void_p()
    rc_end = L.spy_hip_capture_end(st, C.byref(gexec))
    assert rcs == [0, 0, 0] and rc_mm == 0 and rc_end == 0 and gexec.value, (rcs, rc_mm, rc_end)
    assert rc_unprepared == hip.EUNSUPPORTED
    # other data for the eager calls between the replays
    g2, s2 = dev((rng.standard_normal(2048) * 3).astype(np.float32)), dev((rng.standard_normal((H_, T, n_kv)) * 9).astype(np.float32))
    e_silu, e_soft = dev_empty(g.nbytes, 0), dev_empty(s.nbytes, 0)
    for replay in range(3):
        for b in (o_silu, o_soft, o_rope, o_mm):
            b.fill(0xFF)
        hip.sync()                                       # the fills ran on the null stream; the graph's stream does not wait for them by itself
        call(L.spy_hip_graph_launch, gexec, st)
        hip.sync(st)
        _same_bits(o_silu.download(np.float32), w_silu, "silu, replay %d" % replay)
        _same_bits(o_soft.download(np.float32).reshape(s.shape), w_soft, "softmax, replay %d" % replay)
        _same_bits(o_rope.download(np.float32).reshape(xr.shape), w_rope, "rope, replay %d" % replay)
        _same_bits(o_mm.download(np.float32).reshape(1, Mm), w_mm, "single-row matmul, replay %d" % replay)
        call(L.spy_hip_op_silu, None, B(hip.tensor(g2, hip.F32, [g.size])), B(hip.tensor(e_silu, hip.F32, [g.size])))
        call(L.spy_hip_op_softmax, None, B(hip.tensor(s2, hip.F32, [n_kv, T, H_])), B(t_m), B(hip.tensor(e_soft, hip.F32, [n_kv, T, H_])), scale)
        hip.sync()
    call(L.spy_hip_graph_destroy, gexec)
    # outside capture the unprepared parameter set builds its table on first use
    call(L.spy_hip_op_rope, None, B(t_x), B(t_p), B(t_r), B(hp_new))
    hip.sync()
    call(L.spy_hip_stream_destroy, st)


def test_switch_returns_previous_setting_and_default_is_off():
    from spy_amd import _lib as H
    L = H.load()
    if os.environ.get("SPY_HIP_EXACT", "0") not in ("", "0"):
        pytest.skip("exact order switched on by the environment")
    assert L.spy_hip_set_exact_order(1) == 0
    assert L.spy_hip_set_exact_order(0) == 1
    assert L.spy_hip_set_exact_order(0) == 0


@pytest.mark.parametrize("name,kw", [
    ("Q4_0", dict(wtype=O.Q4_0)),
    ("Q8_0", dict(wtype=O.Q8_0)),
    ("Q4_K/Q6_K mix", dict(wtype=O.Q4_K, t_out=O.Q6_K, tensor_types={"attn_v": O.Q6_K, "ffn_down": O.Q6_K})),
])
def test_whole_model_through_submit_has_the_oracle_bits(hip, name, kw):
    """33 operators per layer through Backend::submit: the logits of a prompt pass and of single-token passes on
    top of it, and both caches, equal the CPU oracle's bit for bit."""
    from spy_amd import backend_driver as BD
    from spy_amd import model as M
    from tests.model_util import OracleModel, k_quant_quantizer
    cfg = M.Config(n_layer=3, n_embd=256, n_head=2, n_ff=768, n_vocab=512, n_ctx=64, **kw)
    tensors = M.synth_model(cfg, seed=11, quantizer=k_quant_quantizer)
    host, ora = BD.HostModel(cfg, tensors), OracleModel(cfg, tensors)
    prompt = np.random.default_rng(3).integers(0, cfg.n_vocab, 9).astype(np.int32)
    _same_bits(host.forward(prompt, 0), ora.forward(prompt, 0), name + ": prompt logits")
    for il in range(cfg.n_layer):
        for which, ref in ((0, ora.k_cache[il]), (1, ora.v_cache[il])):
            assert np.array_equal(host.cache(il, which).view(np.uint16), ref.view(np.uint16)), (name, il, which)
    toks = ora.generate(prompt, 12)
    ora2 = OracleModel(cfg, tensors)
    lg = ora2.forward(prompt, 0)[-1]
    for step in range(12):
        assert int(np.argmax(lg)) == int(toks[step])
        t = toks[step:step + 1]
        lh, lg = host.forward(t, 9 + step)[0], ora2.forward(t, 9 + step)[0]
        _same_bits(lh, lg, "%s: single-token pass %d" % (name, step))
    host.close()


@pytest.mark.parametrize("n_prompt", [5, 21])
def test_engine_follows_the_switch(hip, n_prompt):
    """spy_hip_llama_forward / _forward_last / _decode_greedy in exact order: prompt passes below and above the 16
    tokens from which the default path fuses operators, single-token passes, and the greedy loop."""
    from spy_amd import model as M
    from tests.model_util import OracleModel
    cfg = M.Config(n_layer=2, n_embd=256, n_head=2, n_ff=768, n_vocab=512, n_ctx=64, wtype=O.Q4_0)
    tensors = M.synth_model(cfg, seed=5)
    eng, ora = M.Engine(cfg, tensors), OracleModel(cfg, tensors)
    prompt = np.random.default_rng(n_prompt).integers(0, cfg.n_vocab, n_prompt).astype(np.int32)
    lg = ora.forward(prompt, 0)
    _same_bits(eng.forward(prompt, 0), lg, "engine prompt pass of %d tokens" % n_prompt)
    _same_bits(eng.forward_last(prompt, 0), lg[-1], "engine prompt pass, last row only")
    t = np.array([int(np.argmax(lg[-1]))], np.int32)
    _same_bits(eng.forward(t, n_prompt)[0], ora.forward(t, n_prompt)[0], "engine single-token pass")
    want = OracleModel(cfg, tensors).generate(prompt, 20)
    assert eng.generate(prompt, 20).tolist() == want.tolist()
    eng.close()


@pytest.mark.parametrize("n_prompt,n_first,chunk", [(100, 0, 0), (130, 70, 0), (97, 0, 32), (200, 33, 64), (256, 0, 0), (65, 64, 0)])
def test_engine_prompt_attention_kernels_have_the_oracle_bits(hip, n_prompt, n_first, chunk, monkeypatch):
    """Prompt passes of the engine in exact order with heads of 128: scores, softmax and the product with V^T come from the
    three kernels that leave out the masked part.  One pass, a pass on top of cached tokens, and calls cut into chunks of
    32 or 64 query rows (the row length the host's loops depend on is that of the whole call): the oracle's bits, and
    the bits of the operator-by-operator path (SPY_HIP_EXACT_PROMPT_ATTN=0)."""
    from spy_amd import model as M
    from tests.model_util import OracleModel
    cfg = M.Config(n_layer=2, n_embd=256, n_head=2, n_ff=768, n_vocab=512, n_ctx=256, wtype=O.Q4_0)
    tensors = M.synth_model(cfg, seed=6)
    prompt = np.random.default_rng(n_prompt).integers(0, cfg.n_vocab, n_prompt).astype(np.int32)
    ora = OracleModel(cfg, tensors)
    want_first = ora.forward(prompt[:n_first], 0) if n_first else None
    want = ora.forward(prompt[n_first:], n_first)
    if chunk:
        monkeypatch.setenv("SPY_HIP_PREFILL_CHUNK", str(chunk))
    for kernels in ("1", "0"):
        monkeypatch.setenv("SPY_HIP_EXACT_PROMPT_ATTN", kernels)
        eng = M.Engine(cfg, tensors)
        if n_first:
            _same_bits(eng.forward(prompt[:n_first], 0), want_first, "first %d tokens, kernels %s" % (n_first, kernels))
        _same_bits(eng.forward(prompt[n_first:], n_first), want, "%d tokens after %d, chunk %d, kernels %s" % (n_prompt - n_first, n_first, chunk, kernels))
        eng.close()


def test_prompt_attention_kernels_at_the_7b_width(hip, monkeypatch):
    """One layer of the 7B shape, 700 tokens on top of 300: the attention kernels against the operator path, bit for bit."""
    from spy_amd import model as M
    cfg = M.Config.llama2_7b(n_ctx=1024, wtype=O.Q4_0)
    cfg.n_layer = 1
    tensors = M.synth_model(cfg, seed=8)
    prompt = np.random.default_rng(1).integers(0, cfg.n_vocab, 1000).astype(np.int32)
    got = {}
    for kernels in ("1", "0"):
        monkeypatch.setenv("SPY_HIP_EXACT_PROMPT_ATTN", kernels)
        eng = M.Engine(cfg, tensors)
        eng.forward(prompt[:300], 0, want_logits=False)
        got[kernels] = eng.forward_last(prompt[300:], 300)
        eng.close()
    _same_bits(got["1"], got["0"], "7B width, 700 tokens after 300")


@pytest.mark.timeout(600)
@pytest.mark.parametrize("name,kw", [
    ("Q4_0 body, Q6_K head", dict(wtype=O.Q4_0, t_out=O.Q6_K)),
    ("Q8_0", dict(wtype=O.Q8_0)),
    ("Q4_K_M mix", dict(wtype=O.Q4_K, t_out=O.Q6_K, tensor_types={"attn_v": O.Q6_K, "ffn_down": O.Q6_K})),
])
def test_default_engine_at_7b_width_prompt_and_tokens_have_the_oracle_bits(name, kw):
    """The engine as it comes (order 1, no switch set), two layers of the 7B width: a 70-token prompt (tiled exact MatMul of the
    layer's weight types, the three causal attention kernels), a second prompt pass of 33 tokens on top of it, then 6 greedy
    steps through the fused single-token kernels.  Logits of both prompt passes and every generated token equal the CPU
    oracle's, bit for bit."""
    from spy_amd import _lib as H
    from spy_amd import model as M
    from tests.model_util import OracleModel, k_quant_quantizer
    H.init(0)
    cfg = M.Config.llama2_7b(n_ctx=128, **kw)
    cfg.n_layer = 2
    tensors = M.synth_model(cfg, seed=77, quantizer=k_quant_quantizer)
    eng, ora = M.Engine(cfg, tensors), OracleModel(cfg, tensors, nthread=min(16, os.cpu_count() or 8))
    assert eng.order() == 1
    prompt = np.random.default_rng(12).integers(0, cfg.n_vocab, 103).astype(np.int32)
    _same_bits(eng.forward_last(prompt[:70], 0), ora.forward(prompt[:70], 0)[-1], name + ": last row of a 70-token prompt")
    lg = ora.forward(prompt[70:], 70)
    _same_bits(eng.forward(prompt[70:], 70), lg, name + ": 33 tokens on top of 70")
    first = int(np.argmax(lg[-1]))
    want = [first]
    for i in range(6):
        want.append(int(np.argmax(ora.forward(np.array([want[-1]], np.int32), 103 + i)[0])))
    got = eng.decode_greedy(first, 103, 6)
    assert [int(t) for t in got] == want[1:], (name, got, want)
    eng.close()


@pytest.mark.timeout(900)
@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0])
def test_llama2_7b_greedy_32_tokens_identical(wtype):
    """The 7B shape, Q4_0 or Q8_0, 8 random prompt tokens, 32 greedy steps through Backend::submit in exact order:
    the 32 tokens are the CPU oracle's, and so are the bits of every pass's logits."""
    from spy_amd import _lib as H
    from spy_amd import backend_driver as BD
    from spy_amd import model as M
    from tests.model_util import OracleModel
    H.init(0)
    cfg = M.Config.llama2_7b(n_ctx=48, wtype=wtype)
    tensors = M.synth_model(cfg, seed=1234)
    ora = OracleModel(cfg, tensors, nthread=min(16, os.cpu_count() or 8))
    prompt = np.random.default_rng(5).integers(0, cfg.n_vocab, 8).astype(np.int32)
    prev = H.load().spy_hip_set_exact_order(1)
    try:
        host = BD.HostModel(cfg, tensors)
        lg_o, lg_h = ora.forward(prompt, 0)[-1], host.forward(prompt, 0)[-1]
        want, got, equal_bits = [], [], 0
        for step in range(32):
            equal_bits += int(np.array_equal(lg_o.view(np.uint32), lg_h.view(np.uint32)))
            want.append(int(ora.L.spy_o_argmax(lg_o.ctypes.data, lg_o.size)))
            got.append(int(np.argmax(lg_h)))                       # numpy's argmax is the first maximum too
            if step == 31:
                break
            lg_o = ora.forward(np.array([want[-1]], np.int32), 8 + step)[0]
            lg_h = host.forward(np.array([got[-1]], np.int32), 8 + step)[0]
        print("oracle tokens:", want, "\nhip tokens:   ", got, "\n%d of 32 passes with bit-identical logits" % equal_bits, flush=True)
        assert got == want
        assert equal_bits == 32
        host.close()
        # the token loop of the engine (prompt pass, then its greedy loop) follows the switch: same 32 tokens
        eng = M.Engine(cfg, tensors)
        got_eng = eng.generate(prompt, 32).tolist()
        print("engine tokens:", got_eng, flush=True)
        assert got_eng == want
        eng.close()
    finally:
        H.load().spy_hip_set_exact_order(prev)
