"""The kernel families of the fused single-token pass, each driven alone through the C ABI on identical inputs against
the CPU oracle's operator sequence, at the widths of the 7B shape (d = 4096, F = 11008, 32 heads x 128, vocab 32000).

order 1 (the host backend's summation order) must give the oracle's bits: Q8_0 bytes of the prologue, every float of
the epilogues, the fp16 values written to q and to both caches.  order 0 (this backend's own order) is held to the
per-operator tolerance of 1e-3 (max-abs error / max-abs value); its prologue bytes may differ from the oracle's in the
few places where a last-ulp difference of the RMS scale moves a rounding to the neighbouring integer.
"""
import ctypes as C

import numpy as np
import pytest

from tests import oracle_lib as O

pytestmark = pytest.mark.gpu
B = C.byref
TYPES = [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K]
EPS = 1e-5


def _norm_mul(oracle, x, w, eps=EPS):
    """NormRMS then Mul by the norm weight, as the graph's two nodes (attention.cpp:274-282)"""
    x = np.ascontiguousarray(x, np.float32)
    y = np.zeros_like(x)
    assert oracle.spy_o_norm_rms(B(O.tensor(x, O.F32, [x.size, 1])), B(O.tensor(y, O.F32, [x.size, 1])), eps) == 0
    out = np.zeros_like(x)
    assert oracle.spy_o_binary(2, B(O.tensor(y, O.F32, [x.size, 1])), B(O.tensor(w, O.F32, [x.size, 1])), B(O.tensor(out, O.F32, [x.size, 1]))) == 0
    return out


def _check(got, want, what, order, tol=1e-3):
    from tests.gpu_util import rel_err
    got, want = np.asarray(got), np.asarray(want)
    e = rel_err(got, want)
    same = float((got.view(np.uint32) == want.view(np.uint32)).mean()) if got.dtype == np.float32 else float((got == want).mean())
    print("%s, order %d: max-abs err / max |ref| = %.3e, %.2f %% bit-identical" % (what, order, e, 100 * same), flush=True)
    assert np.all(np.isfinite(got.astype(np.float64)))
    if order == 1:
        assert same == 1.0, "%s: %d of %d values differ from the oracle's bits" % (what, int(round((1 - same) * got.size)), got.size)
    else:
        assert e <= tol, "%s: relative error %.3e > %.1e" % (what, e, tol)


def _check_q8(got, want, what, order):
    """native Q8_0 blocks: order 1 identical; order 0: scales identical, quants off by at most one step in at most 0.5 %"""
    got, want = got.reshape(-1, 34), want.reshape(-1, 34)
    diff = np.abs(got[:, 2:].view(np.int8).astype(np.int32) - want[:, 2:].view(np.int8).astype(np.int32))
    print("%s, order %d: %d of %d quants differ, largest step %d, scales equal: %s" % (what, order, int((diff != 0).sum()), diff.size, int(diff.max()),
                                                                                    bool(np.array_equal(got[:, :2], want[:, :2]))), flush=True)
    if order == 1:
        assert np.array_equal(got, want), what
    else:
        assert diff.max() <= 1 and (diff != 0).mean() <= 5e-3, what
        assert (got[:, :2] != want[:, :2]).any(axis=1).mean() <= 5e-3, what


@pytest.mark.parametrize("order", [1, 0])
@pytest.mark.parametrize("K,norm", [(4096, True), (4096, False), (11008, False), (512, True), (1024, True), (8192, True), (5120, True), (11008, True)])
def test_rmsnorm_q8_0_prologue(hip, oracle, order, K, norm):
    from tests.gpu_util import dev, dev_empty, call
    rng = np.random.default_rng(K + norm)
    x = (rng.standard_normal(K) * rng.uniform(0.2, 3.0)).astype(np.float32)
    x[5:9] = 0.0
    x[K // 2] *= 40.0                                       # an outlier block
    x[32:64] = 0.0                                          # a block of zeros: scale 0, quants 0
    w = (1.0 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    want = O.quantize(oracle, _norm_mul(oracle, x, w) if norm else x, O.Q8_0)
    dx, dw, dy = dev(x), dev(w), dev_empty(K // 32 * 34, 0xEE)
    call(hip.load().spy_hip_rmsnorm_q8_0, None, order, dx.ptr, dw.ptr if norm else None, EPS, K, dy.ptr)
    _check_q8(dy.download(np.uint8), want, "RMSNorm -> Q8_0, K %d norm %s" % (K, norm), order)


@pytest.mark.parametrize("order", [1, 0])
@pytest.mark.parametrize("wtype", TYPES)
@pytest.mark.parametrize("M,K", [(4096, 4096), (4096, 11008)])
def test_gemv_with_residual(hip, oracle, order, wtype, M, K):
    """KQV_linear + Add (K = 4096) and ffn_down + Add (K = 11008): Q8_0(x) -> Dot<W,Q8_0> per row -> + residual"""
    from tests.gpu_util import dev, dev_empty, call
    if wtype in (O.Q4_K, O.Q6_K) and K % 256:
        pytest.skip("K-quant rows are whole super-blocks of 256 elements")
    rng = np.random.default_rng(wtype * 7 + K)
    w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.02).astype(np.float32), wtype)
    x = rng.standard_normal(K).astype(np.float32)
    resid = rng.standard_normal(M).astype(np.float32)
    want = O.matmul(oracle, w, wtype, M, K, x[None, :], nthread=8)[0] + resid
    dw, dx, dr, do, dq = dev(w), dev(x), dev(resid), dev_empty(M * 4, 0xEE), dev_empty(K // 32 * 34, 0xEE)
    call(hip.load().spy_hip_gemv_fused, None, order, wtype, dw.ptr, dx.ptr, None, 0.0, dr.ptr, do.ptr, M, K, dq.ptr)
    _check_q8(dq.download(np.uint8), O.quantize(oracle, x, O.Q8_0), "staged activations", 1)       # no norm: the bytes are exact in both orders
    _check(do.download(np.float32), want, "%dx%d type %d + residual" % (M, K, wtype), order)


@pytest.mark.parametrize("order", [1, 0])
@pytest.mark.parametrize("wtype", [O.Q6_K, O.Q4_0, O.Q8_0, O.Q4_K])
def test_output_head(hip, oracle, order, wtype):
    """result_norm, result_linear, output at 32000 x 4096 (the named configuration's head is Q6_K)"""
    from tests.gpu_util import dev, dev_empty, call
    M, K = 32000, 4096
    rng = np.random.default_rng(wtype + 99)
    w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.02).astype(np.float32), wtype)
    x = (rng.standard_normal(K) * 1.7).astype(np.float32)
    nw = (1.0 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    xn = _norm_mul(oracle, x, nw)
    want = O.matmul(oracle, w, wtype, M, K, xn[None, :], nthread=8)[0]
    dw, dx, dn, do, dq = dev(w), dev(x), dev(nw), dev_empty(M * 4, 0xEE), dev_empty(K // 32 * 34, 0xEE)
    call(hip.load().spy_hip_gemv_fused, None, order, wtype, dw.ptr, dx.ptr, dn.ptr, EPS, None, do.ptr, M, K, dq.ptr)
    _check_q8(dq.download(np.uint8), O.quantize(oracle, xn, O.Q8_0), "head prologue", order)
    _check(do.download(np.float32), want, "head 32000x4096 type %d" % wtype, order)


@pytest.mark.parametrize("order", [1, 0])
@pytest.mark.parametrize("wtype", TYPES)
def test_ffn_gate_up_silu(hip, oracle, order, wtype):
    """ffn_norm, ffn_gate, ffn_up, Silu, Mul at F = 11008, d = 4096"""
    from tests.gpu_util import dev, dev_empty, call
    F, K = 11008, 4096
    rng = np.random.default_rng(wtype + 5)
    wg = O.quantize(oracle, (rng.standard_normal((F, K)) * 0.02).astype(np.float32), wtype)
    wu = O.quantize(oracle, (rng.standard_normal((F, K)) * 0.02).astype(np.float32), wtype)
    x = (rng.standard_normal(K) * 2.0).astype(np.float32)
    nw = (1.0 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    xn = _norm_mul(oracle, x, nw)
    g = O.matmul(oracle, wg, wtype, F, K, xn[None, :], nthread=8)[0]
    u = O.matmul(oracle, wu, wtype, F, K, xn[None, :], nthread=8)[0]
    sg = np.zeros_like(g)
    assert oracle.spy_o_silu(B(O.tensor(g, O.F32, [F, 1])), B(O.tensor(sg, O.F32, [F, 1]))) == 0
    want = u * sg
    dg, du, dx, dn, do, dq = dev(wg), dev(wu), dev(x), dev(nw), dev_empty(F * 4, 0xEE), dev_empty(K // 32 * 34, 0xEE)
    call(hip.load().spy_hip_ffn_gate_up_silu, None, order, wtype, dg.ptr, du.ptr, dx.ptr, dn.ptr, EPS, do.ptr, F, K, dq.ptr)
    _check_q8(dq.download(np.uint8), O.quantize(oracle, xn, O.Q8_0), "gate|up prologue", order)
    _check(do.download(np.float32), want, "up * silu(gate), type %d" % wtype, order)


def _rope_table(oracle, pos, hd, n_ctx):
    """cos, sin per pair of position pos, through the oracle's Rope on unit vectors (1, 0): the host libm's values"""
    unit = np.zeros(hd, np.float32); unit[0::2] = 1.0
    out = np.zeros(hd, np.float32)
    p = np.array([pos], np.int32)
    rp = O.default_rope(hd, n_ctx, pos)
    assert oracle.spy_o_rope(B(O.tensor(unit, O.F32, [hd, 1, 1])), B(O.tensor(p, O.I32, [1])), B(O.tensor(out, O.F32, [hd, 1, 1])), B(rp)) == 0
    return out


@pytest.mark.parametrize("order", [1, 0])
@pytest.mark.parametrize("wtype,wtype_v,pos", [(O.Q4_0, 0, 0), (O.Q4_0, 0, 4100), (O.Q8_0, 0, 517), (O.Q4_K, O.Q6_K, 33), (O.Q6_K, 0, 1000)])
def test_rope_kvwrite(hip, oracle, order, wtype, wtype_v, pos):
    """attn_norm, Q/K/V_project, Rope, fp16 Q, KV-cache copies of one token at d = 4096, 32 heads"""
    from tests.gpu_util import dev, dev_empty, call
    d, H_, hd, n_ctx = 4096, 32, 128, 4352
    tv = wtype_v or wtype
    rng = np.random.default_rng(wtype * 3 + pos)
    ws = [O.quantize(oracle, (rng.standard_normal((d, d)) * 0.02).astype(np.float32), t) for t in (wtype, wtype, tv)]
    x = (rng.standard_normal(d) * 1.3).astype(np.float32)
    nw = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    xn = _norm_mul(oracle, x, nw)
    q, k, v = (O.matmul(oracle, ws[i], t, d, d, xn[None, :], nthread=8)[0] for i, t in enumerate((wtype, wtype, tv)))
    p = np.array([pos], np.int32)
    rp = O.default_rope(hd, n_ctx, pos)
    for a in (q, k):
        assert oracle.spy_o_rope(B(O.tensor(a, O.F32, [hd, H_, 1])), B(O.tensor(p, O.I32, [1])), B(O.tensor(a, O.F32, [hd, H_, 1])), B(rp)) == 0
    want_q, want_k, want_v = (O.f32_to_f16_bits(oracle, a) for a in (q, k, v))
    table = _rope_table(oracle, pos, hd, n_ctx)
    dws = [dev(w) for w in ws]
    dx, dn, dt = dev(x), dev(nw), dev(table)
    dq16, dk, dv, dxq = dev_empty(d * 2, 0xEE), dev_empty(n_ctx * d * 2, 0), dev_empty(d * n_ctx * 2, 0), dev_empty(d // 32 * 34, 0xEE)
    call(hip.load().spy_hip_rope_kvwrite, None, order, wtype, wtype_v, dws[0].ptr, dws[1].ptr, dws[2].ptr, dx.ptr, dn.ptr, EPS, d, H_, pos, n_ctx, dt.ptr,
         dq16.ptr, dk.ptr, dv.ptr, dxq.ptr)
    _check_q8(dxq.download(np.uint8), O.quantize(oracle, xn, O.Q8_0), "qkv prologue", order)
    got_q = dq16.download(np.uint16)
    kc, vc = dk.download(np.uint16).reshape(n_ctx, d), dv.download(np.uint16).reshape(d, n_ctx)
    f = lambda a: a.view(np.float16).astype(np.float32)
    for name, got, want in (("q (fp16)", got_q, want_q), ("K cache row", kc[pos], want_k), ("V^T cache column", vc[:, pos], want_v)):
        if order == 1:
            assert np.array_equal(got, want), "%s: %d of %d fp16 values differ" % (name, int((got != want).sum()), got.size)
        else:
            _check(f(got), f(want), name, 0, tol=2e-3)               # one fp16 step at the largest value is 1e-3
    # nothing else in the caches was touched
    kc[pos] = 0; vc[:, pos] = 0
    assert not kc.any() and not vc.any()


@pytest.mark.parametrize("order", [1, 0])
@pytest.mark.parametrize("n_kv", [1, 31, 32, 33, 512, 1025, 4096, 4351])
def test_attn_decode(hip, oracle, order, n_kv):
    """attn_score -> Softmax -> KQV of one token over n_kv cached tokens, 32 heads x 128, caches as the graph lays them out;
    n_kv = 32 k, 32 k + 1: the chunks of 32 of the KQV dot end exactly at / one past the strict bound of its SIMD loop"""
    from tests.gpu_util import dev, dev_empty, call
    H_, hd, n_ctx = 32, 128, 4352
    d = H_ * hd
    rng = np.random.default_rng(n_kv)
    q16 = (rng.standard_normal(d) * 1.5).astype(np.float16)
    kc = np.zeros((n_ctx, d), np.float16); kc[:n_kv] = rng.standard_normal((n_kv, d)).astype(np.float16)
    vc = (rng.standard_normal((d, n_ctx)) * 100).astype(np.float16)                 # slots beyond n_kv hold junk that must not be read into the sums
    vc[:, :n_kv] = rng.standard_normal((d, n_kv)).astype(np.float16)
    kc[n_kv:] = np.float16(300.0)
    # the oracle's three operators on the same bits (q is already fp16: the MatMul's rounding of it is the identity)
    qf = q16.astype(np.float32)
    S = np.zeros((H_, 1, n_kv), np.float32)
    P = np.zeros_like(S)
    out = np.zeros((H_, 1, hd), np.float32)
    assert oracle.spy_o_matmul(B(O.tensor(kc.view(np.uint16), O.F16, [hd, n_kv, H_], nb=[2, 2 * d, 2 * hd])),
                               B(O.tensor(qf, O.F32, [hd, 1, H_], nb=[4, 4 * d, 4 * hd])), B(O.tensor(S, O.F32, [n_kv, 1, H_])), 8) == 0
    mask = np.zeros((1, n_ctx), np.float32)
    scale = np.float32(1.0) / np.sqrt(np.float32(hd))               # SoftmaxParam::scale = 1.0f / sqrtf(hd) (attention.cpp:113), in fp32
    assert oracle.spy_o_softmax(B(O.tensor(S, O.F32, [n_kv, 1, H_])), B(O.tensor(mask, O.F32, [n_ctx, 1])), B(O.tensor(P, O.F32, [n_kv, 1, H_])),
                                float(scale)) == 0
    assert oracle.spy_o_matmul(B(O.tensor(vc.view(np.uint16), O.F16, [n_kv, hd, H_], nb=[2, 2 * n_ctx, 2 * n_ctx * hd])),
                               B(O.tensor(P, O.F32, [n_kv, 1, H_])), B(O.tensor(out, O.F32, [hd, 1, H_])), 8) == 0
    dq, dk, dv = dev(q16.view(np.uint16)), dev(kc.view(np.uint16)), dev(vc.view(np.uint16))
    ds, do = dev_empty(H_ * n_ctx * 4, 0xEE), dev_empty(d * 4, 0xEE)
    call(hip.load().spy_hip_attn_decode, None, order, dq.ptr, dk.ptr, dv.ptr, H_, n_kv, n_ctx, ds.ptr, do.ptr)
    got_s = ds.download(np.float32).reshape(H_, n_ctx)[:, :n_kv]
    want_t = (S[:, 0, :] * scale).astype(np.float32)
    _check(np.ascontiguousarray(got_s), np.ascontiguousarray(want_t), "scores * scale, n_kv %d" % n_kv, order)
    _check(do.download(np.float32), out.reshape(-1), "attention output, n_kv %d" % n_kv, order)


@pytest.mark.parametrize("grid,n_kv", [(64, 4351), (7, 300), (100, 1900)])
def test_attn_scores_in_several_rounds(hip, grid, n_kv, monkeypatch):
    """The score kernel of order 1 deals the cached tokens out over its workgroups and takes a workgroup's share in rounds of 18
    tokens, the next round's keys requested while the current round is multiplied.  With one workgroup per compute unit of this
    part a share never exceeds one round at the supported cache lengths; SPY_HIP_SCORES_GRID forces fewer workgroups, so that the
    rounds (full ones, a short last one, workgroups without tokens) are exercised: same bits as the one-round launch."""
    from tests.gpu_util import dev, dev_empty, call
    H_, hd, n_ctx = 32, 128, 4352
    d = H_ * hd
    rng = np.random.default_rng(grid * 10000 + n_kv)
    q16 = (rng.standard_normal(d) * 1.5).astype(np.float16)
    kc = np.zeros((n_ctx, d), np.float16); kc[:n_kv] = rng.standard_normal((n_kv, d)).astype(np.float16)
    vc = np.zeros((d, n_ctx), np.float16); vc[:, :n_kv] = rng.standard_normal((d, n_kv)).astype(np.float16)
    dq, dk, dv = dev(q16.view(np.uint16)), dev(kc.view(np.uint16)), dev(vc.view(np.uint16))
    res = []
    for g in (None, grid):
        if g is None:
            monkeypatch.delenv("SPY_HIP_SCORES_GRID", raising=False)
        else:
            monkeypatch.setenv("SPY_HIP_SCORES_GRID", str(g))
        ds, do = dev_empty(H_ * n_ctx * 4, 0xEE), dev_empty(d * 4, 0xEE)
        call(hip.load().spy_hip_attn_decode, None, 1, dq.ptr, dk.ptr, dv.ptr, H_, n_kv, n_ctx, ds.ptr, do.ptr)
        hip.sync()
        res.append((ds.download(np.uint32).reshape(H_, n_ctx)[:, :n_kv].copy(), do.download(np.uint32).copy()))
    assert np.array_equal(res[0][0], res[1][0]), "scores differ between one round and %d workgroups" % grid
    assert np.array_equal(res[0][1], res[1][1])


def _running_sum_ref(t):
    """libstdc++'s reduce for random-access ranges on floats: (t0 + t1) + (t2 + t3) per group of four, groups added to one
    running sum in order (every operation rounded to fp32)."""
    t = t.astype(np.float32)
    g = ((t[0::4] + t[1::4]).astype(np.float32) + (t[2::4] + t[3::4]).astype(np.float32)).astype(np.float32)
    s = np.float32(0.0)
    for x in g:
        s = np.float32(s + x)
    return s


def _running_sum_cases():
    rng = np.random.default_rng(77)
    cases = {}
    for n in (4, 8, 252, 256, 260, 4096, 4100, 4352, 8192):
        cases["squares of normals, n=%d" % n] = (rng.standard_normal(n) ** 2).astype(np.float32)
    e = np.exp(-np.abs(rng.standard_normal(4352)) * 6).astype(np.float32); e[1234] = 1.0
    cases["softmax-like exponentials"] = e
    # ties: the running sum sits at 1 (ulp 2^-23) and every group adds exactly half an ulp; even and odd starting mantissa
    t = np.zeros(4096, np.float32); t[0] = 1.0; t[4::4] = 2.0 ** -24
    cases["half-ulp ties from an even sum"] = t
    t = np.zeros(4096, np.float32); t[0] = 1.0; t[1] = 2.0 ** -23; t[4::4] = 2.0 ** -24
    cases["half-ulp ties from an odd sum"] = t
    t = np.zeros(4096, np.float32); t[0] = 1.0; t[4::8] = 2.0 ** -24; t[8::8] = 3 * 2.0 ** -24; t[2000] = 2.0 ** -23
    cases["mixed half and one-and-a-half ulps"] = t
    # sums that land exactly on powers of two, and growth by doubling (a crossing in almost every chunk)
    cases["ones"] = np.ones(8192, np.float32)
    cases["quarters"] = np.full(4096, 0.25, np.float32)
    t = np.zeros(512, np.float32); t[0::4] = (2.0 ** (np.arange(128) / 2.0)).astype(np.float32)
    cases["geometric growth"] = t
    # a term far above the running sum, huge dynamic range, denormals, zeros
    t = (rng.standard_normal(4096) ** 2).astype(np.float32) * 1e-20; t[1000] = 3e18; t[3000] = 7.5e30
    cases["outliers 1e38 apart"] = t
    t = np.zeros(4096, np.float32); t[5::7] = 1e-42; t[4000] = 1e-38
    cases["denormals"] = t
    cases["zeros"] = np.zeros(1024, np.float32)
    t = (rng.standard_normal(8192) ** 2).astype(np.float32); t[::3] *= 2.0 ** -12; t = (t * 2.0 ** 12).round() / np.float32(2.0 ** 12)
    cases["coarse grid (many exact ties)"] = t.astype(np.float32)
    return cases


@pytest.mark.parametrize("chunked", [0, 1])
def test_running_sum_in_the_host_order_bit_for_bit(hip, chunked):
    """spy_hip_running_sum_f32 against the definition, walked in numpy: the plain chain and the chunked form (integer increments
    inside a binade, ties by the parity of the running mantissa, the chain where the sum crosses a power of two) must both give
    the bits of the one-by-one sum.  The cases aim at what the chunked form could get wrong: exact ties from even and odd sums,
    sums that land on powers of two, a crossing in every chunk, terms above the running sum, denormals."""
    from tests.gpu_util import dev, dev_empty, call
    L = hip.load()
    bad = []
    for name, t in _running_sum_cases().items():
        want = _running_sum_ref(t)
        dt, do = dev(t), dev_empty(4, 0xFF)
        call(L.spy_hip_running_sum_f32, None, dt.ptr, t.size, chunked, do.ptr)
        hip.sync()
        got = do.download(np.float32)[0]
        if got.view(np.uint32) != want.view(np.uint32):
            bad.append("%s: got %r (0x%08x), want %r (0x%08x)" % (name, got, got.view(np.uint32), want, want.view(np.uint32)))
    assert not bad, "\n".join(bad)
