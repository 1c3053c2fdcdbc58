"""Pins the oracle's operators against fp64 closed forms, invariants and layout known-answers."""
import ctypes as C

import numpy as np
import pytest

from tests import oracle_lib as O


def h2f(a):
    return a.view(np.float16).astype(np.float64)


def f2h_round(a):
    with np.errstate(over="ignore"):
        return np.asarray(a, dtype=np.float32).astype(np.float16)


@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K])
@pytest.mark.parametrize("T", [1, 3])
def test_matmul_vs_dense(oracle, wtype, T):
    rng = np.random.default_rng(100 + wtype + T)
    M, K = 48, 512
    wf = (rng.standard_normal((M, K)) * 0.02).astype(np.float32)
    w = O.quantize(oracle, wf, wtype)
    x = rng.standard_normal((T, K)).astype(np.float32)
    got = O.matmul(oracle, w, wtype, M, K, x, nthread=3)
    wd = O.dequantize(oracle, w, wtype, M * K).reshape(M, K).astype(np.float64)
    xd = O.dequantize(oracle, O.quantize(oracle, x, O.Q8_0), O.Q8_0, T * K).reshape(T, K).astype(np.float64)
    want = xd @ wd.T
    assert np.allclose(got, want, rtol=1e-4, atol=1e-5 * np.abs(want).max())
    # threads do not change the result
    assert np.array_equal(got, O.matmul(oracle, w, wtype, M, K, x, nthread=1))


def test_matmul_f16_strided_views(oracle):
    """attn_score / KQV operand views (attention.cpp:207-223,248-262): K [hd, n_kv, H] with strides
    (2, 2d, 2hd) over a [token][head][hd] cache; Q permuted [hd, T, H]."""
    rng = np.random.default_rng(5)
    hd, H, T, n_kv, Cx = 16, 3, 2, 7, 12
    d = hd * H
    kc = rng.standard_normal((Cx, H, hd)).astype(np.float16)
    q = rng.standard_normal((T, H, hd)).astype(np.float32)            # [hd, H, T] contiguous
    tk = O.tensor(kc.view(np.uint16), O.F16, [hd, n_kv, H], nb=[2, 2 * d, 2 * hd])
    tq = O.tensor(q, O.F32, [hd, T, H], nb=[4, 4 * d, 4 * hd])
    S = np.zeros((H, T, n_kv), dtype=np.float32)
    ts = O.tensor(S, O.F32, [n_kv, T, H])
    assert oracle.spy_o_matmul(C.byref(tk), C.byref(tq), C.byref(ts), 2) == 0
    q16 = f2h_round(q).astype(np.float64)
    want = np.einsum("thd,jhd->htj", q16, kc[:n_kv].astype(np.float64))
    assert np.allclose(S, want, rtol=2e-6, atol=1e-5)
    # V^T cache [d][C]: V view [n_kv, hd, H] strides (2, 2C, 2C*hd); P [n_kv, T, H] -> O [hd, T, H]
    vc = rng.standard_normal((d, Cx)).astype(np.float16)
    P = rng.random((H, T, n_kv)).astype(np.float32)
    tv = O.tensor(vc.view(np.uint16), O.F16, [n_kv, hd, H], nb=[2, 2 * Cx, 2 * Cx * hd])
    tp = O.tensor(P, O.F32, [n_kv, T, H])
    Oo = np.zeros((H, T, hd), dtype=np.float32)
    to = O.tensor(Oo, O.F32, [hd, T, H])
    assert oracle.spy_o_matmul(C.byref(tv), C.byref(tp), C.byref(to), 1) == 0
    want = np.einsum("htj,hdj->htd", f2h_round(P).astype(np.float64), vc.reshape(H, hd, Cx)[:, :, :n_kv].astype(np.float64))
    assert np.allclose(Oo, want, rtol=2e-6, atol=1e-5)


def test_matmul_unsupported(oracle):
    a = np.zeros((4, 32), np.float32)
    ta, tb = O.tensor(a, O.F32, [32, 4]), O.tensor(a.view(np.int32), O.I32, [32, 4])
    out = np.zeros((4, 4), np.float32)
    assert oracle.spy_o_matmul(C.byref(tb), C.byref(ta), C.byref(O.tensor(out, O.F32, [4, 4])), 1) == 1


def test_norm_rms(oracle):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((3, 4096)) * 3).astype(np.float32)
    y = np.zeros_like(x)
    assert oracle.spy_o_norm_rms(C.byref(O.tensor(x, O.F32, [4096, 3])), C.byref(O.tensor(y, O.F32, [4096, 3])), 1e-5) == 0
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-5)
    assert np.allclose(y, want, rtol=3e-6)
    assert np.allclose((y.astype(np.float64) ** 2).mean(axis=1), 1.0, rtol=1e-4)


def test_binary_broadcast(oracle):
    rng = np.random.default_rng(3)
    a = rng.standard_normal((5, 64)).astype(np.float32)
    w = rng.standard_normal(64).astype(np.float32)
    for op, f in [(0, np.add), (1, np.subtract), (2, np.multiply), (3, np.divide)]:
        out = np.zeros_like(a)
        assert oracle.spy_o_binary(op, C.byref(O.tensor(a, O.F32, [64, 5])), C.byref(O.tensor(w, O.F32, [64])),
                                   C.byref(O.tensor(out, O.F32, [64, 5]))) == 0
        assert np.array_equal(out, f(a, w[None, :]))
    b = rng.standard_normal((5, 64)).astype(np.float32)
    out = np.zeros_like(a)
    oracle.spy_o_binary(0, C.byref(O.tensor(a, O.F32, [64, 5])), C.byref(O.tensor(b, O.F32, [64, 5])), C.byref(O.tensor(out, O.F32, [64, 5])))
    assert np.array_equal(out, a + b)


def test_silu_exhaustive_over_fp16(oracle):
    bits = np.arange(0, 0x10000, dtype=np.uint16)
    finite = (bits & 0x7C00) != 0x7C00
    x = bits[finite].view(np.float16).astype(np.float32)
    y = np.zeros_like(x)
    assert oracle.spy_o_silu(C.byref(O.tensor(x, O.F32, [x.size])), C.byref(O.tensor(y, O.F32, [x.size]))) == 0
    v = x.astype(np.float64)
    with np.errstate(over="ignore"):
        e = np.exp(-v)
    e[e > np.finfo(np.float32).max] = np.inf        # expf overflows in fp32: the table holds v/inf = -0
    want = v / (1.0 + e)
    assert np.allclose(y, want, rtol=4e-7, atol=1e-44)  # fp32 denormal floor
    # the argument is rounded to fp16 first (non-linear.cpp:13)
    xs = np.array([1.0004, -2.3001, 0.33337], np.float32)
    ys = np.zeros_like(xs)
    oracle.spy_o_silu(C.byref(O.tensor(xs, O.F32, [3])), C.byref(O.tensor(ys, O.F32, [3])))
    v = f2h_round(xs).astype(np.float64)
    assert np.allclose(ys, v / (1 + np.exp(-v)), rtol=4e-7)


def _softmax_closed_form(s, mask, scale):
    t = ((s + mask).astype(np.float32) * np.float32(scale)).astype(np.float32)
    m = t.max(axis=-1, keepdims=True)
    with np.errstate(invalid="ignore"):
        arg = f2h_round((t - m).astype(np.float32)).astype(np.float64)
    e = np.where(np.isneginf(mask), 0.0, np.exp(arg))
    return e / e.sum(axis=-1, keepdims=True)


def test_masked_softmax(oracle):
    rng = np.random.default_rng(8)
    H, T, n_kv, Cx, P = 4, 5, 9, 16, 4
    s = (rng.standard_normal((H, T, n_kv)) * 20).astype(np.float32)
    mask = np.full((T, Cx), -np.inf, dtype=np.float32)
    for i in range(T):
        mask[i, :i + P + 1] = 0.0
    out = np.zeros_like(s)
    scale = 1.0 / np.sqrt(128.0)
    rc = oracle.spy_o_softmax(C.byref(O.tensor(s, O.F32, [n_kv, T, H])), C.byref(O.tensor(mask, O.F32, [Cx, T])),
                              C.byref(O.tensor(out, O.F32, [n_kv, T, H])), scale)
    assert rc == 0
    want = _softmax_closed_form(s, mask[None, :, :n_kv], scale)
    assert np.allclose(out, want, rtol=2e-6, atol=1e-30)
    assert np.allclose(out.sum(axis=-1), 1.0, rtol=1e-5)
    for i in range(T):
        assert not out[:, i, i + P + 1:].any()                      # masked entries are exactly 0
    # the fp16 rounding of the exp argument is visible: compare with the unrounded softmax
    t = s.astype(np.float64) * scale + mask[None, :, :n_kv]
    plain = np.exp(t - t.max(axis=-1, keepdims=True)); plain /= plain.sum(axis=-1, keepdims=True)
    assert np.abs(out - plain).max() > 1e-5
    # unmasked variant (non-linear.cpp:86-127)
    out2 = np.zeros_like(s)
    assert oracle.spy_o_softmax(C.byref(O.tensor(s, O.F32, [n_kv, T, H])), None, C.byref(O.tensor(out2, O.F32, [n_kv, T, H])), scale) == 0
    assert np.allclose(out2, _softmax_closed_form(s, np.zeros((1, 1, n_kv), np.float32), scale), rtol=2e-6)


def test_rope(oracle):
    rng = np.random.default_rng(6)
    hd, H, T = 128, 4, 6
    pos = np.array([0, 1, 7, 100, 2047, 4351], dtype=np.int32)
    x = rng.standard_normal((T, H, hd)).astype(np.float32)
    y = np.zeros_like(x)
    rp = O.default_rope(hd, 4352)
    assert oracle.spy_o_rope(C.byref(O.tensor(x, O.F32, [hd, H, T])), C.byref(O.tensor(pos, O.I32, [T])),
                             C.byref(O.tensor(y, O.F32, [hd, H, T])), C.byref(rp)) == 0
    k = np.arange(hd // 2, dtype=np.float64)
    theta = pos[:, None].astype(np.float64) * 10000.0 ** (-2.0 * k / hd)[None, :]
    c, s = np.cos(theta)[:, None, :], np.sin(theta)[:, None, :]
    x0, x1 = x[..., 0::2].astype(np.float64), x[..., 1::2].astype(np.float64)
    want = np.empty(x.shape, dtype=np.float64)
    want[..., 0::2] = x0 * c - x1 * s
    want[..., 1::2] = x0 * s + x1 * c
    # theta is built by repeated fp32 multiplication (non-linear.cpp:304-309): drift is bounded by
    # ~64 ulp of theta, i.e. an absolute angle error of pos * 64 * 2^-24
    tol = 4352 * 64 * 2.0 ** -24 * np.abs(x).max() * 2
    assert np.abs(y - want).max() < tol
    assert np.allclose(y[:3], want[:3], atol=2e-5)
    assert np.array_equal(y[0], x[0])                                        # position 0 is the identity
    n_in = x0 ** 2 + x1 ** 2
    n_out = y[..., 0::2].astype(np.float64) ** 2 + y[..., 1::2].astype(np.float64) ** 2
    assert np.allclose(n_in, n_out, rtol=1e-5)                               # rotations preserve pair norms
    assert oracle.spy_o_rope(C.byref(O.tensor(x, O.F32, [hd, H, T])), C.byref(O.tensor(pos, O.I32, [T])),
                             C.byref(O.tensor(y, O.F32, [hd, H, T])), C.byref(O.RopeParam(2, 0, hd, 64, 64, 1e4, 1, 0, 1, 32, 1, 0, 0))) == 1


def test_rope_glm_closed_form(oracle):
    """Mode GLM (non-linear.cpp:315-343 in the Spy tree) against its definition in float64: for i0 < ne0 / 4 the elements
    (i0, i0 + nd / 2) turn by min(p, C - 2) * base^(-2 i0 / nd) and the elements (i0 + nd, i0 + 3 nd / 2) by
    max(p - (C - 2), 0) * base^(-2 i0 / nd); pair norms are kept, position 0 is the identity, and below C - 2 the second
    pair does not move."""
    rng = np.random.default_rng(26)
    nd, H, T, Cx = 64, 3, 6, 100
    ne0 = 2 * nd
    pos = np.array([0, 1, 50, 98, 99, 140], dtype=np.int32)
    x = rng.standard_normal((T, H, ne0)).astype(np.float32)
    y = np.zeros_like(x)
    rp = O.default_rope(nd, Cx); rp.mode = 4
    assert oracle.spy_o_rope(C.byref(O.tensor(x, O.F32, [ne0, H, T])), C.byref(O.tensor(pos, O.I32, [T])),
                             C.byref(O.tensor(y, O.F32, [ne0, H, T])), C.byref(rp)) == 0
    i0 = np.arange(ne0 // 4, dtype=np.float64)
    sc = 10000.0 ** (-2.0 * i0 / nd)
    ta = np.minimum(pos, Cx - 2)[:, None].astype(np.float64) * sc[None, :]
    tb = np.maximum(pos - (Cx - 2), 0)[:, None].astype(np.float64) * sc[None, :]
    xd = x.astype(np.float64)
    want = xd.copy()
    q = ne0 // 4
    for (a, b, th) in ((0, nd // 2, ta), (nd, nd // 2 + nd, tb)):
        c, s_ = np.cos(th)[:, None, :], np.sin(th)[:, None, :]
        xa, xb = xd[..., a:a + q], xd[..., b:b + q]
        want[..., a:a + q] = xa * c - xb * s_
        want[..., b:b + q] = xa * s_ + xb * c
    assert np.abs(y - want).max() < 140 * 64 * 2.0 ** -24 * np.abs(x).max() * 2 + 1e-6
    assert np.array_equal(y[0], x[0])
    assert np.array_equal(y[2][:, nd:], x[2][:, nd:])                        # p = 50 < C - 2: the second angle is 0
    n_in = xd[..., :q] ** 2 + xd[..., nd // 2:nd // 2 + q] ** 2
    n_out = y[..., :q].astype(np.float64) ** 2 + y[..., nd // 2:nd // 2 + q].astype(np.float64) ** 2
    assert np.allclose(n_in, n_out, rtol=1e-5)


def test_relu_and_quantize_operators(oracle):
    rng = np.random.default_rng(27)
    x = (rng.standard_normal((2, 3, 64)) * 2).astype(np.float32)
    y = np.zeros_like(x)
    assert oracle.spy_o_relu(C.byref(O.tensor(x, O.F32, [64, 3, 2])), C.byref(O.tensor(y, O.F32, [64, 3, 2]))) == 0
    assert np.array_equal(y, np.maximum(x, 0))
    q = np.zeros(6 * 68, np.uint8)
    assert oracle.spy_o_quantize(C.byref(O.tensor(x, O.F32, [64, 3, 2])), C.byref(O.tensor(q, O.Q8_0, [64, 3, 2]))) == 0
    assert np.array_equal(q, O.quantize(oracle, x, O.Q8_0))                   # the operator = the row quantizer, row after row
    h = np.zeros(6 * 128, np.uint8)
    assert oracle.spy_o_quantize(C.byref(O.tensor(x, O.F32, [64, 3, 2])), C.byref(O.tensor(h, O.F16, [64, 3, 2]))) == 0
    assert np.array_equal(h.view(np.float16), x.astype(np.float16).reshape(-1))
    assert oracle.spy_o_quantize(C.byref(O.tensor(x, O.F32, [64, 3, 2])), C.byref(O.tensor(q, O.Q4_0, [64, 3, 2]))) == 1


def test_rope_yarn_and_xpos_reduce_to_known_forms(oracle):
    """Pins for the two extensions of the default Rope branch.  (1) extend_factor != 0 (rope_yarn, non-linear.cpp:247-260): the
    ramp is 1 - std::clamp(0.0F, 1.0F, y), which clamps the value 0 into [1, y] and so is 0, leaving only
    mscale *= 1 + 0.1 ln(1 / freq_scale): the result must equal, bit for bit, a plain Rope whose attention_factor is
    that product -- for any extend_factor and any beta_fast / beta_slow.  (2) xpos (:353-354): every product is
    multiplied by zeta = ((i0 + 0.4 ne0) / (1.4 ne0)) ^ (pos / xpos_base), or its inverse: out / zeta must be the plain
    rotation, pair norms scale by zeta^2, position 0 has zeta = 1, and up * down restores the plain rotation's norm."""
    rng = np.random.default_rng(16)
    hd, H, T = 64, 3, 5
    pos = np.array([0, 2, 31, 500, 3000], dtype=np.int32)
    x = rng.standard_normal((T, H, hd)).astype(np.float32)

    def run(rp):
        y = np.zeros_like(x)
        assert oracle.spy_o_rope(C.byref(O.tensor(x, O.F32, [hd, H, T])), C.byref(O.tensor(pos, O.I32, [T])),
                                 C.byref(O.tensor(y, O.F32, [hd, H, T])), C.byref(rp)) == 0
        return y

    # (1)
    for ext, fs, af, bf, bs in ((1.0, 0.25, 1.0, 32.0, 1.0), (0.3, 0.5, 1.3, 8.0, 2.0), (-2.0, 2.0, 0.7, 32.0, 1.0)):
        yarn = O.RopeParam(0, 0, hd, 4096, 2048, 1e4, fs, ext, af, bf, bs, 0, 0)
        m = np.float32(af) * (np.float32(1.0) + np.float32(0.1) * np.log(np.float32(1.0) / np.float32(fs)).astype(np.float32))
        plain = O.RopeParam(0, 0, hd, 4096, 2048, 1e4, fs, 0.0, float(np.float32(m)), bf, bs, 0, 0)
        a, b = run(yarn), run(plain)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (ext, fs)
    # (2)
    plain = run(O.default_rope(hd, 4096))
    i0 = np.arange(0, hd, 2, dtype=np.float64)
    for base in (512.0, 77.0):
        # base and exponent rounded to fp32 as the reference forms them (a rounding of the base grows with the exponent), the power in fp64
        f = np.float32
        b32 = ((i0.astype(f) + f(0.4) * f(hd)) / (f(1.4) * f(hd))).astype(np.float64)
        e32 = (pos.astype(f) / f(base)).astype(np.float64)
        zeta = b32[None, :] ** e32[:, None]                                                       # [T, hd / 2]
        up = run(O.RopeParam(0, 0, hd, 4096, 4096, 1e4, 1, 0, 1, 32, 1, base, 0))
        down = run(O.RopeParam(0, 0, hd, 4096, 4096, 1e4, 1, 0, 1, 32, 1, base, 1))
        z = np.repeat(zeta, 2, axis=1)[:, None, :]
        # the two products of an output cancel, so the bound is relative to their size: a few fp32 roundings of (|x0| + |x1|) * zeta
        mag = np.repeat(np.abs(x[..., 0::2]) + np.abs(x[..., 1::2]), 2, axis=-1).astype(np.float64)
        assert (np.abs(up - plain * z) <= 8 * 2.0 ** -24 * mag * z).all()
        assert (np.abs(down - plain / z) <= 8 * 2.0 ** -24 * mag / z).all()
        assert np.array_equal(up[0], plain[0]) and np.array_equal(down[0], plain[0])         # position 0: zeta = 1
        assert (np.abs(up.astype(np.float64) * down - plain.astype(np.float64) ** 2) <= 32 * 2.0 ** -24 * mag ** 2).all()


def test_kv_cache_writes(oracle):
    """KCache_cpy / VCache_cpy (attention.cpp:188-246): K lands at [token][head][hd], V lands
    transposed at [d][C] column P+t; every other cache byte is untouched."""
    rng = np.random.default_rng(13)
    hd, H, T, Cx, P = 8, 3, 2, 10, 5
    d = hd * H
    k = rng.standard_normal((T, H, hd)).astype(np.float32)
    v = rng.standard_normal((T, d)).astype(np.float32)                      # V [d, T] contiguous
    kc = np.full((Cx, H, hd), 0x7777, dtype=np.uint16)
    vc = np.full((d, Cx), 0x7777, dtype=np.uint16)
    tk = O.tensor(k, O.F32, [hd, H, T])
    tkc = O.tensor(kc, O.F16, [T * d], offset=2 * d * P)
    assert oracle.spy_o_dup(C.byref(tk), C.byref(tkc)) == 0
    want = np.full_like(kc, 0x7777)
    want[P:P + T] = f2h_round(k).view(np.uint16)
    assert np.array_equal(kc, want)
    tvt = O.tensor(v, O.F32, [T, d], nb=[4 * d, 4])                         # Transpose view of V
    tvc = O.tensor(vc, O.F16, [T, d], nb=[2, 2 * Cx], offset=2 * P)
    assert oracle.spy_o_dup(C.byref(tvt), C.byref(tvc)) == 0
    wantv = np.full_like(vc, 0x7777)
    wantv[:, P:P + T] = f2h_round(v).view(np.uint16).T
    assert np.array_equal(vc, wantv)


def test_contiguous_of_permuted(oracle):
    rng = np.random.default_rng(14)
    hd, T, H = 8, 3, 4
    o = rng.standard_normal((H, T, hd)).astype(np.float32)                  # [hd, T, H]
    out = np.zeros((T, H, hd), dtype=np.float32)                            # [hd, H, T]
    src = O.tensor(o, O.F32, [hd, H, T], nb=[4, 4 * hd * T, 4 * hd, 4 * hd * T * H])
    assert oracle.spy_o_contiguous(C.byref(src), C.byref(O.tensor(out, O.F32, [hd, H, T]))) == 0
    assert np.array_equal(out, o.transpose(1, 0, 2))


def test_get_row_and_argmax(oracle):
    rng = np.random.default_rng(15)
    V, d = 50, 64
    emb = rng.standard_normal((V, d)).astype(np.float32)
    ids = np.array([3, 49, 0, 3], dtype=np.int32)
    out = np.zeros((4, d), np.float32)
    assert oracle.spy_o_get_row(C.byref(O.tensor(emb, O.F32, [d, V])), C.byref(O.tensor(ids, O.I32, [4])), C.byref(O.tensor(out, O.F32, [d, 4]))) == 0
    assert np.array_equal(out, emb[ids])
    q = O.quantize(oracle, emb, O.Q8_0)
    assert oracle.spy_o_get_row(C.byref(O.tensor(q, O.Q8_0, [d, V])), C.byref(O.tensor(ids, O.I32, [4])), C.byref(O.tensor(out, O.F32, [d, 4]))) == 0
    assert np.array_equal(out, O.dequantize(oracle, q, O.Q8_0, V * d).reshape(V, d)[ids])
    bad = np.array([50], dtype=np.int32)
    assert oracle.spy_o_get_row(C.byref(O.tensor(emb, O.F32, [d, V])), C.byref(O.tensor(bad, O.I32, [1])), C.byref(O.tensor(out, O.F32, [d, 1]))) == 7
    q4 = O.quantize(oracle, emb, O.Q4_0)                                     # view.cpp:74-75: anything else aborts
    assert oracle.spy_o_get_row(C.byref(O.tensor(q4, O.Q4_0, [d, V])), C.byref(O.tensor(ids, O.I32, [4])), C.byref(O.tensor(out, O.F32, [d, 4]))) == 1
    lg = np.array([0.1, 3.0, -1.0, 3.0, 2.0], np.float32)
    assert oracle.spy_o_argmax(O.ptr(lg), 5) == 1                            # first maximum (greedy.h:21)
