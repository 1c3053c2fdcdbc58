"""Pins the oracle's number system and quantizers against IEEE definitions, closed forms and
hand-packed blocks (the reference ships no golden vectors for this path)."""
import ctypes as C

import numpy as np
import pytest

from tests import oracle_lib as O


def test_block_sizes(oracle):
    # quant.h:25-28,139-142 and k-quant.h:101-111,177-182 -> 18 / 34 / 144 / 210 bytes
    for t, size, blk in [(O.Q4_0, 18, 32), (O.Q8_0, 34, 32), (O.Q4_K, 144, 256), (O.Q6_K, 210, 256),
                         (O.F32, 4, 1), (O.F16, 2, 1), (O.I32, 4, 1)]:
        assert oracle.spy_o_type_size(t) == size
        assert oracle.spy_o_block_size(t) == blk
    assert oracle.spy_o_row_size(O.Q4_0, 4096) == 2304
    assert oracle.spy_o_row_size(O.Q8_0, 11008) == 11696
    assert oracle.spy_o_row_size(O.Q6_K, 4096) == 3360


def test_f16_to_f32_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.spy_o_f16_to_f32_ieee(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    # the reference's table never fills its last entry (conversion.h:39-41): 0xFFFF -> 0
    assert oracle.spy_o_f16_to_f32(0xFFFF) == 0.0
    assert oracle.spy_o_f16_to_f32(0x3C00) == 1.0
    assert oracle.spy_o_exp_lut(0xFFFF) == 0.0 and oracle.spy_o_silu_lut(0xFFFF) == 0.0


def test_f32_to_f16_rne(oracle):
    rng = np.random.default_rng(1)
    # every fp16 value, its neighbours in fp32 and the exact midpoints between fp16 neighbours
    h = np.arange(0, 0x7C00, dtype=np.uint16)
    v = h.view(np.float16).astype(np.float64)
    nxt = (h + 1).view(np.float16).astype(np.float64)
    mid = ((v + nxt) / 2).astype(np.float32)            # exactly representable in fp32
    cands = [v.astype(np.float32), mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))]
    cands.append(rng.standard_normal(200000).astype(np.float32) * np.float32(10.0))
    cands.append((rng.standard_normal(50000) * 1e-6).astype(np.float32))
    cands.append(np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 65536.0, 1e9, np.inf, -np.inf, 2.0 ** -24,
                           2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 5.96e-8, 1e-10],
                          dtype=np.float32))
    x = np.concatenate(cands)
    x = np.concatenate([x, -x])
    got = O.f32_to_f16_bits(oracle, x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)     # numpy: IEEE round-to-nearest-even
    assert np.array_equal(got, want)


def test_lut_functions(oracle):
    # silu / exp tables are evaluated in fp32 on the fp16-rounded argument (non-linear.h:44-45,136-137)
    for h in [0x0000, 0x3C00, 0xBC00, 0x4500, 0xC500, 0x7BFF, 0xFBFF, 0x0001]:
        v = np.array([h], dtype=np.uint16).view(np.float16).astype(np.float64)[0]
        with np.errstate(over="ignore"):
            e, s = np.exp(v), v / (1.0 + np.exp(-v))
        assert oracle.spy_o_exp_lut(h) == pytest.approx(e, rel=2e-7) or np.isinf(e)
        assert oracle.spy_o_silu_lut(h) == pytest.approx(s, rel=4e-7, abs=1e-30)
    assert oracle.spy_o_silu_lut(0x3C00) == pytest.approx(0.7310586, rel=1e-6)
    assert oracle.spy_o_exp_lut(0xBC00) == pytest.approx(0.36787945, rel=1e-6)


def _q8_unpack(b):
    b = b.reshape(-1, 34)
    d = b[:, :2].copy().view(np.uint16).reshape(-1).view(np.float16).astype(np.float32)
    q = b[:, 2:].copy().view(np.int8)
    return d, q


def test_quantize_q8_0_known_answers(oracle):
    # amax = 127 -> id = 1 exactly, so q_j = rint(x_j): element order, ties-to-even, saturation.
    x = np.zeros(32, dtype=np.float32)
    x[0] = 127.0
    x[1:32] = np.arange(1, 32)
    d, q = _q8_unpack(O.quantize(oracle, x, O.Q8_0))
    assert d[0] == 1.0
    assert np.array_equal(q[0], x.astype(np.int8))          # identity element order (vec_convert.h:255-256)
    x2 = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.49, 3.51] + [0.0] * 23, dtype=np.float32)
    _, q2 = _q8_unpack(O.quantize(oracle, x2, O.Q8_0))
    assert list(q2[0][:9]) == [127, 0, 2, 2, 0, -2, -2, 3, 4]   # round half to even (:235-238)
    # all-zero block: id = 0 (:225) -> zeros, scale 0
    d0, q0 = _q8_unpack(O.quantize(oracle, np.zeros(32, np.float32), O.Q8_0))
    assert d0[0] == 0.0 and not q0.any()
    # negative maximum maps to -127
    x3 = np.full(32, 0.25, np.float32); x3[7] = -3.0
    d3, q3 = _q8_unpack(O.quantize(oracle, x3, O.Q8_0))
    assert q3[0][7] == -127 and d3[0] == np.float32(np.float16(np.float32(3.0) / np.float32(127.0)))


def test_quantize_q8_0_closed_form_and_bound(oracle):
    rng = np.random.default_rng(7)
    x = (rng.standard_normal((512, 32)) * rng.uniform(1e-4, 50, (512, 1))).astype(np.float32)
    x[5, 3] = 1e4                       # single outlier
    x[6] *= 1e-7                        # denormal fp16 scale
    d, q = _q8_unpack(O.quantize(oracle, x, O.Q8_0))
    amax = np.abs(x).max(axis=1)
    idv = (np.float32(127.0) / amax).astype(np.float32)
    want_q = np.rint((x * idv[:, None]).astype(np.float32)).astype(np.int32)
    assert np.array_equal(q.astype(np.int32), want_q)
    assert np.array_equal(d, (amax / np.float32(127.0)).astype(np.float32).astype(np.float16).astype(np.float32))
    assert np.abs(q).max() == 127
    # reconstruction with the exact fp32 step is within half a step
    step = amax / 127.0
    assert np.all(np.abs(q * step[:, None] - x) <= 0.5001 * step[:, None] + 1e-30)


def test_q4_0_ggml_rule_and_dequant(oracle):
    # hand-packed block: d = 0.5, nibbles n_j = j % 16 -> element j = low nibble of qs[j], j+16 = high
    blk = np.zeros(18, dtype=np.uint8)
    blk[:2] = np.array([0.5], dtype=np.float16).view(np.uint8)
    lo = np.arange(16) % 16
    hi = (np.arange(16) * 3 + 1) % 16
    blk[2:] = lo | (hi << 4)
    y = O.dequantize(oracle, blk, O.Q4_0, 32)
    assert np.array_equal(y[:16], (lo - 8) * 0.5)
    assert np.array_equal(y[16:], (hi - 8) * 0.5)
    # quantizer: max magnitude element maps to nibble 0 (value -8*d = max); round trip error <= |d|/2 (+ clip at +7)
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((256, 32)) * 0.02).astype(np.float32)
    q = O.quantize(oracle, x, O.Q4_0)
    y = O.dequantize(oracle, q, O.Q4_0, x.size).reshape(x.shape)
    imax = np.abs(x).argmax(axis=1)
    mx = x[np.arange(256), imax]
    d = (mx / np.float32(-8.0)).astype(np.float32)
    d16 = d.astype(np.float16).astype(np.float32)
    assert np.array_equal(q.reshape(-1, 18)[:, :2].copy().view(np.uint16).reshape(-1), d.astype(np.float16).view(np.uint16))
    assert np.allclose(y[np.arange(256), imax], -8 * d16)
    # closed form of every nibble
    idv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
    nib = np.minimum(15, ((x * idv[:, None]).astype(np.float32) + np.float32(8.5)).astype(np.int8))
    qs = q.reshape(-1, 18)[:, 2:]
    assert np.array_equal(qs & 0x0F, nib[:, :16])
    assert np.array_equal(qs >> 4, nib[:, 16:])
    err = np.abs(y - x)
    assert np.all(err <= np.abs(d16)[:, None] * 1.0001 + 1e-9)      # <= one step (the +8.5 rule clips the top bin)
    assert np.median(err / np.abs(d16)[:, None]) < 0.3


def test_q4_0_as_written_is_known_bad(oracle):
    # vec_convert.h:83-117: 16 floats per emitted block, inverse scale 0 -> every written nibble is 8
    rng = np.random.default_rng(0)
    x = rng.standard_normal(64).astype(np.float32)
    out = np.zeros(4 * 18, dtype=np.uint8)
    oracle.spy_o_quantize_q4_0_as_written(O.ptr(x), O.ptr(out), 64)
    blocks = out.reshape(4, 18)
    assert np.all(blocks[:, 2:10] == 0x88)        # only 8 of the 16 quant bytes are written
    assert np.all(blocks[:, 10:] == 0)
    assert np.all(O.dequantize(oracle, out, O.Q4_0, 128).reshape(4, 32)[:, :8] == 0)


def _pack_q4k_scales(sc, m):
    s = np.zeros(12, dtype=np.uint8)
    for j in range(4):
        s[j] = sc[j] | ((sc[j + 4] >> 4) << 6)
        s[j + 4] = m[j] | ((m[j + 4] >> 4) << 6)
        s[j + 8] = (sc[j + 4] & 0xF) | ((m[j + 4] & 0xF) << 4)
    return s


def test_q4_k_unpack_hand_packed(oracle):
    """PARITY UNPINNED by the reference (layout only, k-quant.h:101-111); pinned to the public ggml
    format by an independent numpy packer."""
    rng = np.random.default_rng(11)
    sc = rng.integers(0, 64, 8).astype(np.uint8)
    m = rng.integers(0, 64, 8).astype(np.uint8)
    q = rng.integers(0, 16, 256).astype(np.uint8)
    blk = np.zeros(144, dtype=np.uint8)
    blk[0:2] = np.array([0.25], np.float16).view(np.uint8)
    blk[2:4] = np.array([0.125], np.float16).view(np.uint8)
    blk[4:16] = _pack_q4k_scales(sc, m)
    for i in range(4):                       # sub-blocks 2i (low nibbles) and 2i+1 (high nibbles) share 32 bytes
        blk[16 + 32 * i:16 + 32 * i + 32] = q[64 * i:64 * i + 32] | (q[64 * i + 32:64 * i + 64] << 4)
    y = O.dequantize(oracle, blk, O.Q4_K, 256)
    want = (0.25 * np.repeat(sc, 32) * q - 0.125 * np.repeat(m, 32)).astype(np.float32)
    assert np.array_equal(y, want)


def test_q6_k_unpack_hand_packed(oracle):
    """PARITY UNPINNED by the reference (layout only, k-quant.h:177-182)."""
    rng = np.random.default_rng(12)
    q = rng.integers(0, 64, 256)
    sc = rng.integers(-128, 128, 16).astype(np.int8)
    blk = np.zeros(210, dtype=np.uint8)
    for half in range(2):
        for l in range(32):
            e = [q[128 * half + l + 32 * g] for g in range(4)]
            blk[64 * half + l] = (e[0] & 0xF) | ((e[2] & 0xF) << 4)
            blk[64 * half + l + 32] = (e[1] & 0xF) | ((e[3] & 0xF) << 4)
            blk[128 + 32 * half + l] = (e[0] >> 4) | ((e[1] >> 4) << 2) | ((e[2] >> 4) << 4) | ((e[3] >> 4) << 6)
    blk[192:208] = sc.view(np.uint8)
    blk[208:210] = np.array([0.5], np.float16).view(np.uint8)
    y = O.dequantize(oracle, blk, O.Q6_K, 256)
    want = (0.5 * np.repeat(sc.astype(np.float32), 16) * (q - 32)).astype(np.float32)
    assert np.array_equal(y, want)


@pytest.mark.parametrize("ttype,tol", [(O.Q4_K, 0.12), (O.Q6_K, 0.03)])
def test_k_quant_roundtrip_bounds(oracle, ttype, tol):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(256 * 64) * 0.02).astype(np.float32)
    x[rng.integers(0, x.size, 16)] *= 20            # outliers as in the Q4_K_M configuration
    y = O.dequantize(oracle, O.quantize(oracle, x, ttype), ttype, x.size)
    blk = 32 if ttype == O.Q4_K else 16
    rng_blk = np.abs(x.reshape(-1, blk)).max(axis=1, keepdims=True) + 1e-12
    assert np.max(np.abs(y - x).reshape(-1, blk) / rng_blk) < tol * 2.5
    assert np.sqrt(np.mean((y - x) ** 2)) / np.sqrt(np.mean(x ** 2)) < tol
    # zeros stay zeros
    z = O.dequantize(oracle, O.quantize(oracle, np.zeros(256, np.float32), ttype), ttype, 256)
    assert not z.any()


@pytest.mark.parametrize("ttype", [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K])
def test_package_quantizers_write_the_oracles_bytes(oracle, ttype):
    """The block quantizers of the package (spy_amd/csrc/host/synth.c: synthetic models for the bench and the full-size GPU
    tests) against the oracle's, written independently from the same rules: identical bytes on normal weights, weights
    with 0.1 % outliers x 20, an all-zero super-block, a constant block and a block with a single non-zero element."""
    from spy_amd import model as M
    rng = np.random.default_rng(ttype)
    x = (rng.standard_normal(256 * 64) * 0.02).astype(np.float32)
    x[::1000] *= 20.0
    x[256:512] = 0.0
    x[512:768] = 0.013
    x[768:1024] = 0.0
    x[800] = -0.4
    assert np.array_equal(M.quantize(x, ttype), O.quantize(oracle, x, ttype))
    # the named stream, quantized on the fly, equals quantizing its float form
    n = 256 * 8
    xs = np.frombuffer(M.synth_tensor(O.F32, 3, "t", n, 0.02, 100, 20.0).tobytes(), np.float32)
    assert np.array_equal(M.synth_tensor(ttype, 3, "t", n, 0.02, 100, 20.0), O.quantize(oracle, xs, ttype))
