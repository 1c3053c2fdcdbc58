"""Pins the oracle's dot products: int32 block dots by brute force (order-independent, so
bit-exact by construction), float results against fp64 sums of the dequantised operands, and
the lane / tail structure through cases whose exact fp32 answer is computable by hand."""
import numpy as np
import pytest

from tests import oracle_lib as O


def _rand_q4_0(rng, nblk, scale=0.02):
    b = np.zeros((nblk, 18), dtype=np.uint8)
    b[:, :2] = (rng.uniform(0.5, 2.0, nblk) * scale / 8).astype(np.float16).view(np.uint8).reshape(nblk, 2)
    b[:, 2:] = rng.integers(0, 256, (nblk, 16), dtype=np.uint8)
    return b.reshape(-1)


def _rand_q8_0(rng, nblk, full_range=False):
    b = np.zeros((nblk, 34), dtype=np.uint8)
    b[:, :2] = (rng.uniform(0.5, 2.0, nblk) / 127).astype(np.float16).view(np.uint8).reshape(nblk, 2)
    lo = -128 if full_range else -127
    b[:, 2:] = rng.integers(lo, 128, (nblk, 32)).astype(np.int8).view(np.uint8)
    return b.reshape(-1)


def _unpack_q4_0(b):
    b = b.reshape(-1, 18)
    d = b[:, :2].copy().view(np.float16).astype(np.float64).reshape(-1)
    q = np.concatenate([(b[:, 2:] & 0xF).astype(np.int32) - 8, (b[:, 2:] >> 4).astype(np.int32) - 8], axis=1)
    return d, q


def _unpack_q8_0(b):
    b = b.reshape(-1, 34)
    return b[:, :2].copy().view(np.float16).astype(np.float64).reshape(-1), b[:, 2:].copy().view(np.int8).astype(np.int32)


@pytest.mark.parametrize("n", [32, 64, 4096, 11008])
def test_q4_0_q8_0(oracle, n):
    rng = np.random.default_rng(n)
    w, x = _rand_q4_0(rng, n // 32), _rand_q8_0(rng, n // 32)
    dw, qw = _unpack_q4_0(w)
    dx, qx = _unpack_q8_0(x)
    ib = (qw * qx).sum(axis=1)
    got_ib = np.zeros(n // 32, dtype=np.int32)
    assert oracle.spy_o_block_dots(O.Q4_0, O.ptr(w), O.ptr(x), n, O.ptr(got_ib)) == 0
    assert np.array_equal(got_ib, ib)
    want = float((dw * dx * ib).sum())
    scale = float(np.abs(dw * dx * ib).sum()) + 1e-30
    got = oracle.spy_o_dot_q4_0_q8_0(O.ptr(w), O.ptr(x), n)
    assert abs(got - want) <= 2e-6 * scale
    assert got == oracle.spy_o_dot_q4_0_q8_0_scalar(O.ptr(w), O.ptr(x), n)   # AVX2 == scalar, bit for bit


@pytest.mark.parametrize("n", [32, 96, 4096, 11008])
def test_q8_0_q8_0(oracle, n):
    rng = np.random.default_rng(n + 1)
    w, x = _rand_q8_0(rng, n // 32), _rand_q8_0(rng, n // 32)
    dw, qw = _unpack_q8_0(w)
    dx, qx = _unpack_q8_0(x)
    ib = (qw * qx).sum(axis=1)
    got_ib = np.zeros(n // 32, dtype=np.int32)
    assert oracle.spy_o_block_dots(O.Q8_0, O.ptr(w), O.ptr(x), n, O.ptr(got_ib)) == 0
    assert np.array_equal(got_ib, ib)
    want = float((dw * dx * ib).sum())
    scale = float(np.abs(dw * dx * ib).sum()) + 1e-30
    got = oracle.spy_o_dot_q8_0_q8_0(O.ptr(w), O.ptr(x), n)
    assert abs(got - want) <= 2e-6 * scale
    assert got == oracle.spy_o_dot_q8_0_q8_0_scalar(O.ptr(w), O.ptr(x), n)


def test_q4_0_lane_structure_exact(oracle):
    """One block, d = 1: the result is hsum of 8 integer lane partials -- exact in fp32, equal to
    the integer block dot whatever the lane order; with two blocks whose scales differ by 2^20 a
    dropped or double-counted lane shows up as an integer error."""
    rng = np.random.default_rng(9)
    w, x = _rand_q4_0(rng, 2), _rand_q8_0(rng, 2)
    w = w.reshape(2, 18); x = x.reshape(2, 34)
    w[0, :2] = np.array([1.0], np.float16).view(np.uint8); w[1, :2] = np.array([2.0 ** -10], np.float16).view(np.uint8)
    x[0, :2] = np.array([1.0], np.float16).view(np.uint8); x[1, :2] = np.array([2.0 ** -10], np.float16).view(np.uint8)
    _, qw = _unpack_q4_0(w.reshape(-1)); _, qx = _unpack_q8_0(x.reshape(-1))
    ib = (qw * qx).sum(axis=1)
    want = float(ib[0]) + float(ib[1]) * 2.0 ** -20           # exact in fp32 (|ib| < 2^15, 35 bits needed? no: lanes are separate)
    got = oracle.spy_o_dot_q4_0_q8_0(O.ptr(w.reshape(-1)), O.ptr(x.reshape(-1)), 64)
    assert abs(got - want) <= abs(want) * 2 ** -22


def test_q8_0_signed_extremes(oracle):
    # sign trick of mul_sum_i8_pairs (vec_util.h:101-110): x = -127/127 against y = +-127
    w = np.zeros(34, np.uint8); x = np.zeros(34, np.uint8)
    w[:2] = x[:2] = np.array([1.0], np.float16).view(np.uint8)
    w[2:] = np.array([-127, 127] * 16, np.int8).view(np.uint8)
    x[2:] = np.array([127, 127, -127, -127] * 8, np.int8).view(np.uint8)
    assert oracle.spy_o_dot_q8_0_q8_0(O.ptr(w), O.ptr(x), 32) == 0.0
    x[2:] = np.array([-127, 127] * 16, np.int8).view(np.uint8)
    assert oracle.spy_o_dot_q8_0_q8_0(O.ptr(w), O.ptr(x), 32) == 32 * 127 * 127
    # x == 0 lanes contribute nothing (sign_epi8 zeroes them)
    w[2:] = 0
    assert oracle.spy_o_dot_q8_0_q8_0(O.ptr(w), O.ptr(x), 32) == 0.0


@pytest.mark.parametrize("n", [1, 31, 32, 33, 64, 65, 128, 512, 4097])
def test_f16_dot_vs_fp64(oracle, n):
    rng = np.random.default_rng(n)
    a = rng.standard_normal(n).astype(np.float16)
    b = rng.standard_normal(n).astype(np.float16)
    want = float((a.astype(np.float64) * b.astype(np.float64)).sum())
    scale = float(np.abs(a.astype(np.float64) * b.astype(np.float64)).sum())
    got = oracle.spy_o_dot_f16_f16(O.ptr(a.view(np.uint16)), O.ptr(b.view(np.uint16)), n)
    assert abs(got - want) <= 4e-6 * scale
    assert got == oracle.spy_o_dot_f16_f16_scalar(O.ptr(a.view(np.uint16)), O.ptr(b.view(np.uint16)), n)


def test_f16_dot_strict_tail(oracle):
    """vec_dot.h:132 loops while i + 32 < n (strict): n = 32 goes entirely through the sequential
    scalar tail, so the result is the left-to-right fp32 sum of fp32 products; n = 64 sends only the
    first 32 elements through the 8-lane accumulators."""
    rng = np.random.default_rng(4)
    a = rng.standard_normal(64).astype(np.float16)
    b = rng.standard_normal(64).astype(np.float16)
    prod = (a.astype(np.float32) * b.astype(np.float32)).astype(np.float32)

    def seq(p):
        s = np.float32(0)
        for v in p:
            s = np.float32(s + v)
        return s

    got32 = oracle.spy_o_dot_f16_f16(O.ptr(a.view(np.uint16)), O.ptr(b.view(np.uint16)), 32)
    assert np.float32(got32) == seq(prod[:32])
    # n = 64: lanes l of the four accumulators hold single products (exact), reduced as
    # ((s0+s2)+(s1+s3)) per lane, then (l + l+4), then pairwise; tail = sequential over 32..63
    p = prod[:32].reshape(4, 8)
    lane = ((p[0] + p[2]).astype(np.float32) + (p[1] + p[3]).astype(np.float32)).astype(np.float32)
    t = (lane[:4] + lane[4:]).astype(np.float32)
    simd = np.float32(np.float32(t[0] + t[1]) + np.float32(t[2] + t[3]))
    want64 = np.float32(seq(prod[32:]) + simd)
    got64 = oracle.spy_o_dot_f16_f16(O.ptr(a.view(np.uint16)), O.ptr(b.view(np.uint16)), 64)
    assert np.float32(got64) == want64


@pytest.mark.parametrize("ttype,fn", [(O.Q4_K, "spy_o_dot_q4_k_q8_0"), (O.Q6_K, "spy_o_dot_q6_k_q8_0")])
def test_k_quant_dots_equal_dense(oracle, ttype, fn):
    """PARITY UNPINNED by the reference.  The project-defined K-quant x Q8_0 dot must equal the
    fp64 dot of the two dequantised vectors."""
    rng = np.random.default_rng(21)
    n = 4096
    wf = (rng.standard_normal(n) * 0.02).astype(np.float32)
    wf[rng.integers(0, n, 4)] *= 20
    w = O.quantize(oracle, wf, ttype)
    x = O.quantize(oracle, rng.standard_normal(n).astype(np.float32), O.Q8_0)
    wd = O.dequantize(oracle, w, ttype, n).astype(np.float64)
    xd = O.dequantize(oracle, x, O.Q8_0, n).astype(np.float64)
    want = float((wd * xd).sum())
    got = getattr(oracle, fn)(O.ptr(w), O.ptr(x), n)
    assert abs(got - want) <= 3e-6 * float(np.abs(wd * xd).sum())
    # integer sub-block dots by brute force from the dequantised integers
    nsub = n // (32 if ttype == O.Q4_K else 16)
    ib = np.zeros(nsub, np.int32)
    assert oracle.spy_o_block_dots(ttype, O.ptr(w), O.ptr(x), n, O.ptr(ib)) == 0
    _, qx = _unpack_q8_0(x)
    if ttype == O.Q4_K:
        qs = w.reshape(-1, 144)[:, 16:]
        q = np.stack([np.concatenate([(qs[:, 32 * i:32 * i + 32] & 0xF), (qs[:, 32 * i:32 * i + 32] >> 4)], axis=1) for i in range(4)], axis=1)
        q = q.reshape(-1, 32).astype(np.int32)
        assert np.array_equal(ib, (q * qx).sum(axis=1))
    else:
        assert ib.shape[0] == n // 16
