"""GPU parity of the per-operator entry points (spy_hip_op_*) against the CPU oracle, through the
same strided tensor views the LLaMA graph hands to a backend."""
import ctypes as C

import numpy as np
import pytest

from tests import oracle_lib as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from spy_amd import _lib as H
    H.init(0)
    return H


def B(t):
    return C.byref(t)


def test_norm_rms(hip, oracle):
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(1)
    for T, d in [(1, 4096), (7, 4096), (2, 100)]:
        x = (rng.standard_normal((T, d)) * 2.5).astype(np.float32)
        want = np.zeros_like(x)
        assert oracle.spy_o_norm_rms(B(O.tensor(x, O.F32, [d, T])), B(O.tensor(want, O.F32, [d, T])), 1e-5) == 0
        dx, dy = dev(x), dev_empty(x.nbytes, 0xFF)
        call(hip.load().spy_hip_op_norm_rms, None, B(hip.tensor(dx, hip.F32, [d, T])), B(hip.tensor(dy, hip.F32, [d, T])), 1e-5)
        assert_close(dy.download(np.float32).reshape(T, d), want, "norm_rms %dx%d" % (T, d), tol=1e-5)


def test_binary_ops_exact(hip, oracle):
    from tests.gpu_util import dev, dev_empty, call
    rng = np.random.default_rng(2)
    a = rng.standard_normal((6, 4096)).astype(np.float32)
    w = rng.standard_normal(4096).astype(np.float32)
    b = rng.standard_normal((6, 4096)).astype(np.float32)
    da, dw, db = dev(a), dev(w), dev(b)
    for op in range(4):
        for (hb, ob, ne_b) in [(dw, w, [4096]), (db, b, [4096, 6])]:
            want = np.zeros_like(a)
            assert oracle.spy_o_binary(op, B(O.tensor(a, O.F32, [4096, 6])), B(O.tensor(ob, O.F32, ne_b)), B(O.tensor(want, O.F32, [4096, 6]))) == 0
            dd = dev_empty(a.nbytes, 0xFF)
            call(hip.load().spy_hip_op_binary, None, op, B(hip.tensor(da, hip.F32, [4096, 6])), B(hip.tensor(hb, hip.F32, ne_b)),
                 B(hip.tensor(dd, hip.F32, [4096, 6])))
            assert np.array_equal(dd.download(np.float32).reshape(6, 4096).view(np.uint32), want.view(np.uint32))   # IEEE single ops: exact


def test_silu_all_fp16_inputs(hip, oracle):
    from tests.gpu_util import dev, dev_empty, call
    bits = np.arange(0, 0x10000, dtype=np.uint16)
    finite = (bits & 0x7C00) != 0x7C00
    x = np.concatenate([bits[finite].view(np.float16).astype(np.float32),
                        np.random.default_rng(3).standard_normal(4096).astype(np.float32) * 4])
    want = np.zeros_like(x)
    assert oracle.spy_o_silu(B(O.tensor(x, O.F32, [x.size])), B(O.tensor(want, O.F32, [x.size]))) == 0
    dx, dy = dev(x), dev_empty(x.nbytes, 0xFF)
    call(hip.load().spy_hip_op_silu, None, B(hip.tensor(dx, hip.F32, [x.size])), B(hip.tensor(dy, hip.F32, [x.size])))
    got = dy.download(np.float32)
    big = np.abs(want) > 1e-30
    rel = np.abs(got[big] - want[big]) / np.abs(want[big])
    print("silu: max elementwise relative error %.3e over %d fp16 inputs" % (rel.max(), big.sum()), flush=True)
    assert rel.max() < 1e-5 and np.abs(got[~big] - want[~big]).max() < 1e-30


def test_masked_softmax(hip, oracle):
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(4)
    for (H_, T, n_kv, Cx, P) in [(32, 1, 300, 512, 299), (4, 5, 9, 16, 4), (2, 3, 1030, 1100, 1027)]:
        s = (rng.standard_normal((H_, T, n_kv)) * 12).astype(np.float32)
        mask = np.full((T, Cx), -np.inf, dtype=np.float32)
        for i in range(T):
            mask[i, :i + P + 1] = 0.0
        scale = float(1.0 / np.sqrt(128.0))
        want = np.zeros_like(s)
        assert oracle.spy_o_softmax(B(O.tensor(s, O.F32, [n_kv, T, H_])), B(O.tensor(mask, O.I32, [Cx, T])), B(O.tensor(want, O.F32, [n_kv, T, H_])), scale) == 0
        ds, dm, dd = dev(s), dev(mask), dev_empty(s.nbytes, 0xFF)
        call(hip.load().spy_hip_op_softmax, None, B(hip.tensor(ds, hip.F32, [n_kv, T, H_])), B(hip.tensor(dm, hip.I32, [Cx, T])),
             B(hip.tensor(dd, hip.F32, [n_kv, T, H_])), scale)
        got = dd.download(np.float32).reshape(s.shape)
        assert_close(got, want, "softmax H%d T%d n_kv%d" % (H_, T, n_kv), tol=1e-5)
        assert np.array_equal(got == 0, want == 0)                          # masked entries exactly zero
    # unmasked form
    want = np.zeros_like(s)
    assert oracle.spy_o_softmax(B(O.tensor(s, O.F32, [n_kv, T, H_])), None, B(O.tensor(want, O.F32, [n_kv, T, H_])), scale) == 0
    call(hip.load().spy_hip_op_softmax, None, B(hip.tensor(ds, hip.F32, [n_kv, T, H_])), None, B(hip.tensor(dd, hip.F32, [n_kv, T, H_])), scale)
    assert_close(dd.download(np.float32).reshape(s.shape), want, "softmax unmasked", tol=1e-5)


def test_softmax_row_kernel_and_fp16_output(hip, oracle):
    """Rows of up to 16384 elements take the kernel that keeps a row in LDS, longer rows the three-pass kernel; both against
    the oracle, with and without a causal mask.  The fp16 output of the row kernel is its fp32 output rounded to nearest even,
    which is what the KQV product does to it first (mat.cpp:37 in the Spy tree)."""
    from tests.gpu_util import dev, dev_empty, call
    rng = np.random.default_rng(12)
    scale = 0.0883883461356163
    L = hip.load()
    for (H_, T, n_kv, Cx, P) in [(4, 24, 40, 64, 16), (2, 5, 1000, 1024, 995), (1, 3, 4104, 4352, 4101), (1, 2, 16500, 16512, 16498)]:
        s = (rng.standard_normal((H_, T, n_kv)) * 4).astype(np.float32)
        mask = np.where(np.arange(Cx)[None, :] <= (np.arange(T)[:, None] + P), 0.0, -np.inf).astype(np.float32)
        ds, dm = dev(s), dev(mask.view(np.int32))
        for name, use_mask in (("masked", True), ("plain", False)):
            tm = B(hip.tensor(dm, hip.I32, [Cx, T])) if use_mask else None
            dr = dev_empty(s.nbytes, 0xFF)
            call(L.spy_hip_op_softmax, None, B(hip.tensor(ds, hip.F32, [n_kv, T, H_])), tm, B(hip.tensor(dr, hip.F32, [n_kv, T, H_])), scale)
            row = dr.download(np.float32)
            if n_kv <= 16384:
                dh = dev_empty(s.nbytes // 2, 0xFF)
                call(L.spy_hip_op_softmax, None, B(hip.tensor(ds, hip.F32, [n_kv, T, H_])), tm, B(hip.tensor(dh, hip.F16, [n_kv, T, H_])), scale)
                assert np.array_equal(dh.download(np.float16).view(np.uint16), row.astype(np.float16).view(np.uint16)), (name, H_, T, n_kv)
            else:       # the fp16 output is the row kernel's alone
                dh = dev_empty(s.nbytes // 2, 0xFF)
                assert L.spy_hip_op_softmax(None, B(hip.tensor(ds, hip.F32, [n_kv, T, H_])), tm, B(hip.tensor(dh, hip.F16, [n_kv, T, H_])), scale) == hip.EUNSUPPORTED
            want = np.zeros_like(s)
            om = B(O.tensor(mask.view(np.int32), O.I32, [Cx, T])) if use_mask else None
            assert oracle.spy_o_softmax(B(O.tensor(s, O.F32, [n_kv, T, H_])), om, B(O.tensor(want, O.F32, [n_kv, T, H_])), scale) == 0
            assert float(np.abs(row.reshape(want.shape) - want).max()) < 1e-5, (name, H_, T, n_kv)
            assert np.array_equal(row.reshape(want.shape) == 0, want == 0)


def test_rope(hip, oracle):
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(5)
    hd, H_, T = 128, 32, 6
    pos = np.array([0, 1, 7, 100, 2047, 4351], dtype=np.int32)
    x = rng.standard_normal((T, H_, hd)).astype(np.float32)
    want = np.zeros_like(x)
    rp = O.default_rope(hd, 4352)
    assert oracle.spy_o_rope(B(O.tensor(x, O.F32, [hd, H_, T])), B(O.tensor(pos, O.I32, [T])), B(O.tensor(want, O.F32, [hd, H_, T])), B(rp)) == 0
    dx, dp, dy = dev(x), dev(pos), dev_empty(x.nbytes, 0xFF)
    hp = hip.RopeParam(0, 0, hd, 4352, 4352, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, 0.0, 0)
    call(hip.load().spy_hip_op_rope, None, B(hip.tensor(dx, hip.F32, [hd, H_, T])), B(hip.tensor(dp, hip.I32, [T])),
         B(hip.tensor(dy, hip.F32, [hd, H_, T])), B(hp))
    got = dy.download(np.float32).reshape(x.shape)
    assert_close(got, want, "rope", tol=1e-5)
    assert np.array_equal(got[0], x[0])                                     # position 0 = identity
    hp.mode = 2
    assert hip.load().spy_hip_op_rope(None, B(hip.tensor(dx, hip.F32, [hd, H_, T])), B(hip.tensor(dp, hip.I32, [T])),
                                      B(hip.tensor(dy, hip.F32, [hd, H_, T])), B(hp)) == hip.EUNSUPPORTED


def test_rope_glm(hip, oracle):
    """Mode GLM (non-linear.cpp:315-343 in the Spy tree) as written: rows of 2 * num_dim elements, positions on both sides of
    num_context - 2 (the second angle is 0 before it); in place as well; rows the four indices would leave are refused."""
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(6)
    nd, H_, T, C_ = 64, 8, 6, 100
    ne0 = 2 * nd
    pos = np.array([0, 1, 50, 98, 99, 140], dtype=np.int32)
    x = rng.standard_normal((T, H_, ne0)).astype(np.float32)
    want = np.zeros_like(x)
    rp = O.default_rope(nd, C_); rp.mode = 4
    assert oracle.spy_o_rope(B(O.tensor(x, O.F32, [ne0, H_, T])), B(O.tensor(pos, O.I32, [T])), B(O.tensor(want, O.F32, [ne0, H_, T])), B(rp)) == 0
    dx, dp, dy = dev(x), dev(pos), dev_empty(x.nbytes, 0xFF)
    hp = hip.RopeParam(4, 0, nd, C_, C_, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, 0.0, 0)
    L = hip.load()
    call(L.spy_hip_op_rope, None, B(hip.tensor(dx, hip.F32, [ne0, H_, T])), B(hip.tensor(dp, hip.I32, [T])), B(hip.tensor(dy, hip.F32, [ne0, H_, T])), B(hp))
    got = dy.download(np.float32).reshape(x.shape)
    assert_close(got, want, "rope GLM", tol=1e-5)
    assert np.array_equal(got[0], x[0])                                     # position 0: both angles 0
    call(L.spy_hip_op_rope, None, B(hip.tensor(dx, hip.F32, [ne0, H_, T])), B(hip.tensor(dp, hip.I32, [T])), B(hip.tensor(dx, hip.F32, [ne0, H_, T])), B(hp))   # in place
    assert np.array_equal(dx.download(np.float32).reshape(x.shape).view(np.uint32), got.view(np.uint32))
    hp.num_dim = ne0                                                        # i0 + 3 num_dim / 2 would leave the row
    assert L.spy_hip_op_rope(None, B(hip.tensor(dx, hip.F32, [ne0, H_, T])), B(hip.tensor(dp, hip.I32, [T])), B(hip.tensor(dy, hip.F32, [ne0, H_, T])), B(hp)) == hip.EINVAL


def test_relu_and_quantize_operators(hip, oracle):
    """Relu (non-linear.cpp:16-50) and Quantize (backend/host/operator/quantize.cpp:18-41) of the host backend's operator
    set: exact results; the conversions the reference cannot do right are refused."""
    from tests.gpu_util import dev, dev_empty, call
    rng = np.random.default_rng(8)
    L = hip.load()
    x = (rng.standard_normal((3, 5, 256)) * 3).astype(np.float32)
    x[0, 0, :4] = [0.0, -0.0, np.inf, -np.inf]
    dx, dy = dev(x), dev_empty(x.nbytes, 0xFF)
    call(L.spy_hip_op_relu, None, B(hip.tensor(dx, hip.F32, [256, 5, 3])), B(hip.tensor(dy, hip.F32, [256, 5, 3])))
    want = np.zeros_like(x)
    assert oracle.spy_o_relu(B(O.tensor(x, O.F32, [256, 5, 3])), B(O.tensor(want, O.F32, [256, 5, 3]))) == 0
    assert np.array_equal(dy.download(np.float32).view(np.uint32), want.reshape(-1).view(np.uint32))
    assert np.array_equal(want, np.where(x < 0, np.float32(0), x))
    x[0, 0, 2:4] = [7.5, -7.5]                                              # finite values for the quantizers (an infinite block scale has no defined quants)
    dx = dev(x)
    for ttype in (O.Q8_0, O.F16):
        nbytes = 15 * O.row_size(ttype, 256)
        dq = dev_empty(nbytes, 0xFF)
        call(L.spy_hip_op_quantize, None, B(hip.tensor(dx, hip.F32, [256, 5, 3])), B(hip.tensor(dq, ttype, [256, 5, 3])))
        wq = np.zeros(nbytes, np.uint8)
        assert oracle.spy_o_quantize(B(O.tensor(x, O.F32, [256, 5, 3])), B(O.tensor(wq, ttype, [256, 5, 3]))) == 0
        assert np.array_equal(dq.download(np.uint8), wq), ttype
    dq = dev_empty(15 * O.row_size(O.Q4_0, 256), 0)
    assert L.spy_hip_op_quantize(None, B(hip.tensor(dx, hip.F32, [256, 5, 3])), B(hip.tensor(dq, hip.Q4_0, [256, 5, 3]))) == hip.EUNSUPPORTED


@pytest.mark.parametrize("name,kw", [
    ("YaRN magnitude (extend_factor 1, freq_scale 0.25)", dict(freq_scale=0.25, extend_factor=1.0, attention_factor=1.1)),
    ("xpos up", dict(xpos_base=512.0, xpos_down=0)),
    ("xpos down with YaRN", dict(freq_scale=0.5, extend_factor=0.7, xpos_base=300.0, xpos_down=1)),
])
def test_rope_yarn_and_xpos(hip, oracle, name, kw):
    """The two Rope extensions the reference plumbs through its default branch (non-linear.cpp:242-260, 349-364):
    extend_factor != 0 changes the magnitude only (the ramp is 1 - std::clamp(0.0F, 1.0F, y) = 0 as written), xpos
    multiplies every product by zeta.  Against the oracle to 1e-5 here, to the bit in exact order (test_gpu_exact_order.py)."""
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(51)
    hd, H_, T = 128, 4, 5
    pos = np.array([0, 3, 100, 2047, 4351], dtype=np.int32)
    x = rng.standard_normal((T, H_, hd)).astype(np.float32)
    want = np.zeros_like(x)
    rp = O.default_rope(hd, 4352)
    hp = hip.RopeParam(0, 0, hd, 4352, 4352, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, 0.0, 0)
    for k, v in kw.items():
        setattr(rp, k, v); setattr(hp, k, v)
    assert oracle.spy_o_rope(B(O.tensor(x, O.F32, [hd, H_, T])), B(O.tensor(pos, O.I32, [T])), B(O.tensor(want, O.F32, [hd, H_, T])), B(rp)) == 0
    dx, dp, dy = dev(x), dev(pos), dev_empty(x.nbytes, 0xFF)
    call(hip.load().spy_hip_op_rope, None, B(hip.tensor(dx, hip.F32, [hd, H_, T])), B(hip.tensor(dp, hip.I32, [T])),
         B(hip.tensor(dy, hip.F32, [hd, H_, T])), B(hp))
    assert_close(dy.download(np.float32).reshape(x.shape), want, "rope, " + name, tol=1e-5)


def test_kv_cache_copy_bit_exact(hip, oracle):
    """KCache_cpy / VCache_cpy (attention.cpp:188-246 in the Spy tree) through the Copy operator."""
    from tests.gpu_util import dev, call
    rng = np.random.default_rng(6)
    hd, H_, T, Cx, P = 128, 32, 3, 40, 17
    d = hd * H_
    k = rng.standard_normal((T, H_, hd)).astype(np.float32)
    v = rng.standard_normal((T, d)).astype(np.float32)
    kc = np.full((Cx, H_, hd), 0x7777, dtype=np.uint16)
    vc = np.full((d, Cx), 0x7777, dtype=np.uint16)
    want_k, want_v = kc.copy(), vc.copy()
    assert oracle.spy_o_dup(B(O.tensor(k, O.F32, [hd, H_, T])), B(O.tensor(want_k, O.F16, [T * d], offset=2 * d * P))) == 0
    assert oracle.spy_o_dup(B(O.tensor(v, O.F32, [T, d], nb=[4 * d, 4])), B(O.tensor(want_v, O.F16, [T, d], nb=[2, 2 * Cx], offset=2 * P))) == 0
    dk, dv, dkc, dvc = dev(k), dev(v), dev(kc), dev(vc)
    L = hip.load()
    call(L.spy_hip_op_dup, None, B(hip.tensor(dk, hip.F32, [hd, H_, T])), B(hip.tensor(dkc, hip.F16, [T * d], offset=2 * d * P)))
    call(L.spy_hip_op_dup, None, B(hip.tensor(dv, hip.F32, [T, d], nb=[4 * d, 4])), B(hip.tensor(dvc, hip.F16, [T, d], nb=[2, 2 * Cx], offset=2 * P)))
    assert np.array_equal(dkc.download(np.uint16).reshape(kc.shape), want_k)
    assert np.array_equal(dvc.download(np.uint16).reshape(vc.shape), want_v)


def test_contiguous_and_get_row_and_argmax(hip, oracle):
    from tests.gpu_util import dev, dev_empty, call
    rng = np.random.default_rng(7)
    hd, T, H_ = 128, 3, 32
    o = rng.standard_normal((H_, T, hd)).astype(np.float32)
    do, dd = dev(o), dev_empty(o.nbytes, 0xFF)
    L = hip.load()
    call(L.spy_hip_op_contiguous, None, B(hip.tensor(do, hip.F32, [hd, H_, T], nb=[4, 4 * hd * T, 4 * hd, 4 * hd * T * H_])), B(hip.tensor(dd, hip.F32, [hd, H_, T])))
    assert np.array_equal(dd.download(np.float32).reshape(T, H_, hd), o.transpose(1, 0, 2))
    # GetRow: F32 and Q8_0 tables
    V, d = 1000, 4096
    emb = rng.standard_normal((V, d)).astype(np.float32)
    ids = np.array([3, 999, 0, 3, 512], dtype=np.int32)
    q = O.quantize(oracle, emb, O.Q8_0)
    for tab, tt in [(emb, O.F32), (q, O.Q8_0)]:
        want = np.zeros((5, d), np.float32)
        assert oracle.spy_o_get_row(B(O.tensor(tab, tt, [d, V])), B(O.tensor(ids, O.I32, [5])), B(O.tensor(want, O.F32, [d, 5]))) == 0
        dt, di, dout = dev(tab), dev(ids), dev_empty(want.nbytes, 0xFF)
        call(L.spy_hip_op_get_row, None, B(hip.tensor(dt, tt, [d, V])), B(hip.tensor(di, hip.I32, [5])), B(hip.tensor(dout, hip.F32, [d, 5])))
        assert np.array_equal(dout.download(np.float32).reshape(5, d).view(np.uint32), want.view(np.uint32))
    flag = C.c_int32(-1)
    call(L.spy_hip_take_error, C.byref(flag)); assert flag.value == 0
    bad = np.array([1000], dtype=np.int32)
    dbad = dev(bad)
    call(L.spy_hip_op_get_row, None, B(hip.tensor(dt, tt, [d, V])), B(hip.tensor(dbad, hip.I32, [1])), B(hip.tensor(dout, hip.F32, [d, 1])))
    call(L.spy_hip_take_error, C.byref(flag)); assert flag.value == 1       # the reference asserts here (view.cpp:61)
    q4 = O.quantize(oracle, emb[:4], O.Q4_0)
    dq4 = dev(q4)
    assert L.spy_hip_op_get_row(None, B(hip.tensor(dq4, hip.Q4_0, [d, 4])), B(hip.tensor(di, hip.I32, [5])), B(hip.tensor(dout, hip.F32, [d, 5]))) == hip.EUNSUPPORTED
    # argmax: first maximum
    lg = rng.standard_normal(32000).astype(np.float32)
    lg[[77, 31999, 4000]] = lg.max() + 1.0
    dl, di32 = dev(lg), dev_empty(4, 0)
    call(L.spy_hip_argmax, None, dl.ptr, 32000, di32.ptr)
    assert di32.download(np.int32)[0] == oracle.spy_o_argmax(O.ptr(lg), 32000) == 77


@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K])
def test_op_matmul_quantized(hip, oracle, wtype):
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(8 + wtype)
    M, K, T = 96, 4096, 5
    w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.02).astype(np.float32), wtype)
    x = rng.standard_normal((T, K)).astype(np.float32)
    want = O.matmul(oracle, w, wtype, M, K, x, nthread=4)
    dw, dx, dd = dev(w), dev(x), dev_empty(T * M * 4, 0xFF)
    tw, tx, td = hip.tensor(dw, wtype, [K, M]), hip.tensor(dx, hip.F32, [K, T]), hip.tensor(dd, hip.F32, [M, T])
    L = hip.load()
    need = L.spy_hip_op_matmul_scratch_size(B(tw), B(tx))
    assert need == T * (K // 32) * 34
    assert L.spy_hip_op_matmul(None, B(tw), B(tx), B(td), None, 0) == hip.ENOSPACE
    scratch = dev_empty(need, 0)
    call(L.spy_hip_op_matmul, None, B(tw), B(tx), B(td), scratch.ptr, need)
    assert_close(dd.download(np.float32).reshape(T, M), want, "op_matmul type %d" % wtype)
    # activations: identical Q8_0 bytes to the oracle's
    assert np.array_equal(scratch.download(np.uint8), O.quantize(oracle, x, O.Q8_0))


@pytest.mark.parametrize("wtype", [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K])
@pytest.mark.parametrize("M,K", [(100, 4096), (4096, 4096), (37, 64), (33, 256), (21, 11008), (6000, 4096), (50, 16384), (16000, 512)])
def test_op_matmul_single_row(hip, oracle, wtype, M, K):
    """One f32 activation row (the weight products of a single-token pass through Backend::submit): one launch of the
    one-row-per-wave kernel, which quantizes the row in LDS and leaves the scratch buffer alone; one row per wave up to 5120
    rows, three above, the two-launch way beyond 15360 rows or where the row length does not fit."""
    from tests.gpu_util import dev, dev_empty, call, assert_close
    kq = wtype in (O.Q4_K, O.Q6_K)
    if kq and K % 256:
        pytest.skip("K-quant rows are whole super-blocks")
    rng = np.random.default_rng(5 * wtype + M + K)
    w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.02).astype(np.float32), wtype)
    x = rng.standard_normal((1, K)).astype(np.float32)
    x[0, :32] = 0.0
    want = O.matmul(oracle, w, wtype, M, K, x, nthread=8)
    dw, dx, dd = dev(w), dev(x), dev_empty(M * 4 + 64, 0xFF)
    tw, tx, td = hip.tensor(dw, wtype, [K, M]), hip.tensor(dx, hip.F32, [K, 1]), hip.tensor(dd, hip.F32, [M, 1])
    L = hip.load()
    need = L.spy_hip_op_matmul_scratch_size(B(tw), B(tx))
    scratch = dev_empty(need, 0xEE)
    call(L.spy_hip_op_matmul, None, B(tw), B(tx), B(td), scratch.ptr, need)
    got = dd.download(np.float32)
    assert_close(got[:M].reshape(1, M), want, "single-row op_matmul type %d %dx%d" % (wtype, M, K))
    assert (got[M:].view(np.uint32) == 0xFFFFFFFF).all(), "nothing is written beyond the M outputs"
    one_launch = M <= 15360 and not (kq and K > 12288) and (M <= 5120 or K <= 4096)
    assert (scratch.download(np.uint8) == 0xEE).all() == one_launch, "which route ran (the one-launch route does not touch the scratch buffer)"


def test_op_matmul_attention_views(hip, oracle):
    """attn_score and KQV through the strided K / V^T cache views and the permuted Q."""
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(9)
    hd, H_, T, n_kv, Cx = 128, 32, 2, 37, 64
    d = hd * H_
    kc = rng.standard_normal((Cx, H_, hd)).astype(np.float16)
    vc = rng.standard_normal((d, Cx)).astype(np.float16)
    q = rng.standard_normal((T, H_, hd)).astype(np.float32)
    P = rng.random((H_, T, n_kv)).astype(np.float32)
    S_want = np.zeros((H_, T, n_kv), np.float32)
    O_want = np.zeros((H_, T, hd), np.float32)
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
    need = L.spy_hip_op_matmul_scratch_size(B(tk), B(tq))
    assert need == hd * T * H_ * 2
    sc = dev_empty(need, 0)
    call(L.spy_hip_op_matmul, None, B(tk), B(tq), B(tS), sc.ptr, need)
    assert_close(dS.download(np.float32).reshape(S_want.shape), S_want, "attn_score", tol=1e-5)
    tv = hip.tensor(dvc, hip.F16, [n_kv, hd, H_], nb=[2, 2 * Cx, 2 * Cx * hd])
    tP = hip.tensor(dP, hip.F32, [n_kv, T, H_])
    tO = hip.tensor(dO, hip.F32, [hd, T, H_])
    need = L.spy_hip_op_matmul_scratch_size(B(tv), B(tP))
    sc = dev_empty(need, 0)
    call(L.spy_hip_op_matmul, None, B(tv), B(tP), B(tO), sc.ptr, need)
    assert_close(dO.download(np.float32).reshape(O_want.shape), O_want, "KQV", tol=1e-5)
    # F32 x F32 has no hip implementation: reported, not aborted
    assert L.spy_hip_op_matmul(None, B(tq), B(tq), B(tS), None, 0) == hip.EUNSUPPORTED


@pytest.mark.parametrize("H_,T,past,n_ctx", [(2, 40, 0, 64), (3, 136, 168, 448), (2, 200, 57, 320), (1, 64, 4032, 4096), (2, 1, 77, 128), (1, 130, 0, 136)])
def test_prompt_attention_kernel_against_operator_sequence(hip, H_, T, past, n_ctx):
    """spy_hip_prompt_attention = MatMul(K view, q) -> Softmax(causal mask, scale) -> MatMul(V^T view, P) of the
    operator ABI on the same fp16 inputs.  The products accumulate in the same order and the maximum is exact, so the
    only difference is the order in which a row's exponentials are added: the results agree to a few fp32 ulps except
    where that moves a probability across an fp16 rounding boundary (2^-11 of that probability)."""
    from tests.gpu_util import dev, dev_empty, call, rel_err
    hd, n_kv = 128, past + T
    d = H_ * hd
    rng = np.random.default_rng(1000 * T + past)
    scale = 1.0 / np.sqrt(hd)
    q = rng.standard_normal((H_, T, hd)).astype(np.float16)
    kc = np.zeros((n_ctx, d), np.float16); kc[:n_kv] = rng.standard_normal((n_kv, d)).astype(np.float16)
    vc = np.zeros((d, n_ctx), np.float16); vc[:, :n_kv] = rng.standard_normal((d, n_kv)).astype(np.float16)
    dq, dk, dv = dev(q), dev(kc), dev(vc)
    L = hip.load()
    fused = dev_empty(T * d * 4, 0xFF)
    call(L.spy_hip_prompt_attention, None, dq.ptr, dk.ptr, dv.ptr, fused.ptr, T, H_, hd, past, n_ctx, scale)
    # the operator sequence, tensors as the LLaMA graph views them
    mask = np.where(np.arange(n_ctx)[None, :] <= (np.arange(T)[:, None] + past), 0.0, -np.inf).astype(np.float32)
    dm = dev(mask.view(np.int32))
    tk = hip.tensor(dk, hip.F16, [hd, n_kv, H_], nb=[2, 2 * d, 2 * hd])
    tq = hip.tensor(dq, hip.F16, [hd, T, H_])
    dS, dP, ref = dev_empty(n_kv * T * H_ * 4, 0xFF), dev_empty(n_kv * T * H_ * 4, 0xFF), dev_empty(T * d * 4, 0xFF)
    tS, tP = hip.tensor(dS, hip.F32, [n_kv, T, H_]), hip.tensor(dP, hip.F32, [n_kv, T, H_])
    tv = hip.tensor(dv, hip.F16, [n_kv, hd, H_], nb=[2, 2 * n_ctx, 2 * n_ctx * hd])
    tO = hip.tensor(ref, hip.F32, [hd, T, H_], nb=[4, 4 * d, 4 * hd])
    need = max(L.spy_hip_op_matmul_scratch_size(B(tk), B(tq)), L.spy_hip_op_matmul_scratch_size(B(tv), B(tP)), 256)
    sc = dev_empty(need)
    call(L.spy_hip_op_matmul, None, B(tk), B(tq), B(tS), sc.ptr, need)
    call(L.spy_hip_op_softmax, None, B(tS), B(hip.tensor(dm, hip.I32, [n_ctx, T])), B(tP), scale)
    call(L.spy_hip_op_matmul, None, B(tv), B(tP), B(tO), sc.ptr, need)
    hip.sync()
    got, want = fused.download(np.float32).reshape(T, d), ref.download(np.float32).reshape(T, d)
    assert np.isfinite(got).all()
    err = rel_err(got, want)
    frac_equal = float((got.view(np.uint32) == want.view(np.uint32)).mean())
    print("H %d T %d past %d: max-abs err / max |out| = %.2e, %.1f %% of the outputs bit-identical" % (H_, T, past, err, 100 * frac_equal), flush=True)
    assert err < 2e-4
    # and against the definition in float64 on the same fp16 inputs
    for h in range(H_):
        qf, kf, vf = q[h].astype(np.float64), kc[:n_kv, h * hd:(h + 1) * hd].astype(np.float64), vc[h * hd:(h + 1) * hd, :n_kv].astype(np.float64)
        t = (qf @ kf.T) * scale
        t[np.arange(n_kv)[None, :] > (np.arange(T)[:, None] + past)] = -np.inf
        e = np.exp((t - t.max(axis=1, keepdims=True)).astype(np.float16).astype(np.float64))
        p = (e / e.sum(axis=1, keepdims=True)).astype(np.float16).astype(np.float64)
        assert rel_err(got[:, h * hd:(h + 1) * hd], p @ vf.T) < 1e-3


def test_prompt_attention_score_far_below_the_row_maximum(hip):
    """A key whose score lies more than 65504 below its row's maximum: the softmax argument rounds to -inf in fp16, its
    exponential is 0 (as expf gives in the operator sequence) and the row stays finite.  Also: a scale that is not positive
    is refused (the kernel takes the row maximum over the raw dot products)."""
    from tests.gpu_util import dev, dev_empty, call, rel_err
    H_, T, past, n_ctx, hd = 2, 72, 9, 128, 128
    d, n_kv = H_ * hd, past + T
    rng = np.random.default_rng(5)
    scale = 1.0 / np.sqrt(hd)
    q = rng.standard_normal((H_, T, hd)).astype(np.float16)
    q[:, 5::7, :] = np.float16(200.0)                                 # some queries point one way ...
    kc = np.zeros((n_ctx, d), np.float16); kc[:n_kv] = rng.standard_normal((n_kv, d)).astype(np.float16)
    kc[3] = np.float16(-200.0)                                        # ... and one visible key the opposite way: q.k = -5.1e6
    vc = np.zeros((d, n_ctx), np.float16); vc[:, :n_kv] = rng.standard_normal((d, n_kv)).astype(np.float16)
    dq, dk, dv = dev(q), dev(kc), dev(vc)
    L = hip.load()
    fused = dev_empty(T * d * 4, 0xFF)
    call(L.spy_hip_prompt_attention, None, dq.ptr, dk.ptr, dv.ptr, fused.ptr, T, H_, hd, past, n_ctx, scale)
    hip.sync()
    got = fused.download(np.float32).reshape(T, d)
    assert np.isfinite(got).all()
    for h in range(H_):
        qf, kf, vf = q[h].astype(np.float64), kc[:n_kv, h * hd:(h + 1) * hd].astype(np.float64), vc[h * hd:(h + 1) * hd, :n_kv].astype(np.float64)
        t = ((qf @ kf.T).astype(np.float32) * np.float32(scale)).astype(np.float64)
        t[np.arange(n_kv)[None, :] > (np.arange(T)[:, None] + past)] = -np.inf
        with np.errstate(over="ignore"):
            arg = (t - t.max(axis=1, keepdims=True)).astype(np.float32).astype(np.float16)
        assert np.isneginf(arg[5, 3])                                  # the case is there: a visible key at -inf
        e = np.exp(arg.astype(np.float64))
        p = (e / e.sum(axis=1, keepdims=True)).astype(np.float16).astype(np.float64)
        assert rel_err(got[:, h * hd:(h + 1) * hd], p @ vf.T) < 1e-3
    assert L.spy_hip_prompt_attention(None, dq.ptr, dk.ptr, dv.ptr, fused.ptr, T, H_, hd, past, n_ctx, 0.0) == hip.EINVAL
    assert L.spy_hip_prompt_attention(None, dq.ptr, dk.ptr, dv.ptr, fused.ptr, T, H_, hd, past, n_ctx, -scale) == hip.EINVAL


def test_measured_ceilings_are_plausible(hip):
    """The measurement entry points behind the denominators of the operator sweep: the bare int8 MFMA loop, the same loop with
    the per-block scaling of the quantized GEMM in both epilogue forms, and the read scan.  Sanity bounds only: below the
    published peaks, the scaled loops below the bare one, the biased-accumulator form not slower than the conversion form."""
    import ctypes as C
    L = hip.load()
    bare, cvt, biased, gbps = C.c_float(), C.c_float(), C.c_float(), C.c_float()
    assert L.spy_hip_measure_mfma_i8(None, 2000, C.byref(bare)) == 0
    assert L.spy_hip_measure_mfma_i8_scaled(None, 2000, 0, C.byref(cvt)) == 0
    assert L.spy_hip_measure_mfma_i8_scaled(None, 2000, 1, C.byref(biased)) == 0
    assert L.spy_hip_measure_mfma_i8_scaled(None, 2000, 2, C.byref(biased)) == hip.EINVAL
    buf = hip.DeviceBuffer(256 << 20)
    buf.fill(1)
    assert L.spy_hip_measure_hbm_read(None, buf.ptr, buf.nbytes, 3, C.byref(gbps)) == 0
    buf.free()
    print("int8 MFMA %.0f TOP/s, block-scaled inner loop %.0f (conversion) / %.0f (biased accumulator) TOP/s, read scan %.0f GB/s"
          % (bare.value, cvt.value, biased.value, gbps.value), flush=True)
    assert 1000 < bare.value < 5000
    assert 300 < cvt.value < bare.value and 300 < biased.value < bare.value
    assert biased.value > 0.95 * cvt.value
    assert 1000 < gbps.value < 8000
