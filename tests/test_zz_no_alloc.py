"""The allocation-free MatMul entry point against spy_hip_op_matmul, through the C ABI: same bits, on two calls in a
row, the second with a smaller input (it finds the first call's bytes in the shared fixed array), then the size limit."""
import ctypes as C

import numpy as np
import pytest

from tests import oracle_lib as O

pytestmark = pytest.mark.gpu
B = C.byref


def _both(hip, oracle, wtype, M, K, T, seed):
    from tests.gpu_util import dev, dev_empty, call, assert_close
    rng = np.random.default_rng(seed)
    w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.02).astype(np.float32), wtype)
    x = rng.standard_normal((T, K)).astype(np.float32)
    dw, dx = dev(w), dev(x)
    d_ref, d_new = dev_empty(T * M * 4, 0xFF), dev_empty(T * M * 4, 0xEE)
    tw, tx = hip.tensor(dw, wtype, [K, M]), hip.tensor(dx, hip.F32, [K, T])
    L = hip.load()
    need = L.spy_hip_op_matmul_scratch_size(B(tw), B(tx))
    assert 0 < need <= L.spy_hip_op_matmul_noalloc_max_scratch()
    scratch = dev_empty(need, 0)
    call(L.spy_hip_op_matmul, None, B(tw), B(tx), B(hip.tensor(d_ref, hip.F32, [M, T])), scratch.ptr, need)
    call(L.spy_hip_op_matmul_noalloc, None, B(tw), B(tx), B(hip.tensor(d_new, hip.F32, [M, T])))
    hip.sync()
    ref, new = d_ref.download(np.float32), d_new.download(np.float32)
    assert np.array_equal(ref.view(np.uint32), new.view(np.uint32)), "no-alloc MatMul differs from spy_hip_op_matmul (type %d, T %d)" % (wtype, T)
    if T <= 8:
        assert_close(ref.reshape(T, M), O.matmul(oracle, w, wtype, M, K, x, nthread=4), "op_matmul vs oracle, type %d" % wtype)


def test_noalloc_matmul_equals_matmul_on_two_calls_in_a_row(hip, oracle):
    print("no-alloc MatMul: Q4_0 160x4096 T=40 (matrix cores), then Q8_0 96x2048 T=3 (row kernels), then fp16 x f32", flush=True)
    _both(hip, oracle, O.Q4_0, 160, 4096, 40, 1)        # 174 080 bytes of Q8_0 activations in the fixed array
    _both(hip, oracle, O.Q8_0, 96, 2048, 3, 2)          # a smaller input right after: 6 528 bytes, the rest of the array holds the first call's
    _both(hip, oracle, O.Q4_0, 160, 4096, 40, 1)        # and the first again


def test_noalloc_matmul_fp16_weights_and_limit(hip, oracle):
    """fp16 left operand (the attention products' type pair): f32 activations are rounded to fp16 in the fixed array;
    a request beyond the array is refused with ENOSPACE and nothing is launched."""
    from tests.gpu_util import dev, dev_empty, call
    rng = np.random.default_rng(5)
    M, K, T = 64, 256, 7
    w16 = rng.standard_normal((M, K)).astype(np.float16)
    x = rng.standard_normal((T, K)).astype(np.float32)
    dw, dx = dev(w16.view(np.uint16)), dev(x)
    d_ref, d_new = dev_empty(T * M * 4, 0xFF), dev_empty(T * M * 4, 0xEE)
    tw, tx = hip.tensor(dw, hip.F16, [K, M]), hip.tensor(dx, hip.F32, [K, T])
    L = hip.load()
    need = L.spy_hip_op_matmul_scratch_size(B(tw), B(tx))
    scratch = dev_empty(need, 0)
    call(L.spy_hip_op_matmul, None, B(tw), B(tx), B(hip.tensor(d_ref, hip.F32, [M, T])), scratch.ptr, need)
    call(L.spy_hip_op_matmul_noalloc, None, B(tw), B(tx), B(hip.tensor(d_new, hip.F32, [M, T])))
    hip.sync()
    assert np.array_equal(d_ref.download(np.uint32), d_new.download(np.uint32))
    # beyond the limit: 8 MiB / (4096 / 32 * 34) = 1927 rows fit, 2000 do not.  Only shapes are read before the refusal.
    big_T = 2000
    tw4 = hip.tensor(dw, hip.Q4_0, [4096, 8])
    txb = hip.tensor(dx, hip.F32, [4096, big_T])
    assert L.spy_hip_op_matmul_scratch_size(B(tw4), B(txb)) > L.spy_hip_op_matmul_noalloc_max_scratch()
    assert L.spy_hip_op_matmul_noalloc(None, B(tw4), B(txb), B(hip.tensor(d_new, hip.F32, [8, big_T]))) == hip.ENOSPACE


def test_noalloc_matmul_in_the_host_summation_order(hip, oracle):
    """With the host backend's summation order on and 16 activation rows or more, the tiled exact MatMul runs from fp16 copies
    of both operands placed behind the activations when the workspace has room.  Small shape: the copies fit the fixed array
    (the packed kernel inside it); 7B-width shape: spy_hip_op_matmul_scratch_size exceeds the array while the activations
    alone fit, and the call still succeeds (the kernel that unpacks per tile).  Both: the CPU oracle's bits."""
    from tests.gpu_util import dev, dev_empty, call
    L = hip.load()
    prev = L.spy_hip_set_exact_order(1)
    try:
        for (M, K, T, fits) in ((160, 4096, 40, True), (4096, 4096, 64, False)):
            rng = np.random.default_rng(M + T)
            w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.02).astype(np.float32), O.Q4_0)
            x = rng.standard_normal((T, K)).astype(np.float32)
            dw, dx, dout = dev(w), dev(x), dev_empty(T * M * 4, 0xEE)
            tw, tx = hip.tensor(dw, hip.Q4_0, [K, M]), hip.tensor(dx, hip.F32, [K, T])
            need = L.spy_hip_op_matmul_scratch_size(B(tw), B(tx))
            assert (need <= L.spy_hip_op_matmul_noalloc_max_scratch()) == fits, (need, fits)
            print("no-alloc exact MatMul %dx%d T=%d: full workspace %d bytes, fixed array %d" % (M, K, T, need, L.spy_hip_op_matmul_noalloc_max_scratch()), flush=True)
            call(L.spy_hip_op_matmul_noalloc, None, B(tw), B(tx), B(hip.tensor(dout, hip.F32, [M, T])))
            hip.sync()
            got = dout.download(np.float32).reshape(T, M)
            want = O.matmul(oracle, w, O.Q4_0, M, K, x, nthread=8)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "no-alloc exact MatMul %dx%d T=%d differs from the oracle's bits" % (M, K, T)
    finally:
        L.spy_hip_set_exact_order(prev)


def test_noalloc_matmul_captured_and_replayed(hip, oracle):
    """The use the entry point exists for: one call recorded under HIP stream capture and replayed three times, with an
    eager call on other operands between the replays (it overwrites the shared fixed array; the replayed call converts its
    own activations again, so every replay gives the first result).  A replayed graph counts as a call like any other: it
    must not overlap with another call on the same device."""
    from tests.gpu_util import dev, dev_empty, call
    L = hip.load()
    rng = np.random.default_rng(77)
    M, K, T = 160, 4096, 40
    w = O.quantize(oracle, (rng.standard_normal((M, K)) * 0.02).astype(np.float32), O.Q4_0)
    x, x2 = rng.standard_normal((T, K)).astype(np.float32), rng.standard_normal((T, K)).astype(np.float32)
    dw, dx, dx2 = dev(w), dev(x), dev(x2)
    d_ref, d_cap, d_other = dev_empty(T * M * 4, 0xFF), dev_empty(T * M * 4, 0xEE), dev_empty(T * M * 4, 0xDD)
    tw, tx, tx2 = hip.tensor(dw, hip.Q4_0, [K, M]), hip.tensor(dx, hip.F32, [K, T]), hip.tensor(dx2, hip.F32, [K, T])
    call(L.spy_hip_op_matmul_noalloc, None, B(tw), B(tx), B(hip.tensor(d_ref, hip.F32, [M, T])))        # eager: the result to match
    hip.sync()
    ref = d_ref.download(np.uint32)
    st = C.c_void_p()
    call(L.spy_hip_stream_create, C.byref(st))
    print("capture: no-alloc MatMul Q4_0 160x4096 T=40", flush=True)
    call(L.spy_hip_capture_begin, st)
    rc = L.spy_hip_op_matmul_noalloc(st, B(tw), B(tx), B(hip.tensor(d_cap, hip.F32, [M, T])))
    gexec = C.c_void_p()
    rc_end = L.spy_hip_capture_end(st, C.byref(gexec))
    assert rc == 0 and rc_end == 0 and gexec.value, (rc, rc_end)
    for replay in range(3):
        d_cap.fill(0xEE)
        hip.sync()                                       # the fill ran on the null stream; the graph's stream does not wait for it by itself
        call(L.spy_hip_graph_launch, gexec, st)
        hip.sync(st)
        assert np.array_equal(d_cap.download(np.uint32), ref), "replay %d differs from the eager call" % replay
        call(L.spy_hip_op_matmul_noalloc, None, B(tw), B(tx2), B(hip.tensor(d_other, hip.F32, [M, T])))
        hip.sync()
    call(L.spy_hip_graph_destroy, gexec)
    call(L.spy_hip_stream_destroy, st)
