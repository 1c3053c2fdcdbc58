"""GGUF ingest on the CPU: the writer and the C reader agree byte for byte, the reader accepts what
GGUFAdapter::init_from_file accepts (storage/src/adapter/gguf_adapter.cpp:90-190) and rejects broken files
with a message, and the loader refuses models this backend does not run before touching the GPU."""
import os
import re
import struct

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def G():
    from spy_amd import gguf
    gguf.load()
    return gguf


def small_model(G, **kw):
    from spy_amd import _lib as H, model as M
    cfg = M.Config(n_layer=2, n_embd=256, n_head=2, n_ff=512, n_vocab=96, n_ctx=32, wtype=H.Q4_0, **kw)
    return cfg, M.synth_model(cfg, seed=5)


def test_header_symbols_are_exported(G):
    text = open(os.path.join(ROOT, "include", "spy_gguf.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(spy_gguf_[a-z0-9_]+)\s*\(", text)))
    assert len(names) >= 18
    L = G.load()
    for n in names:
        assert hasattr(L, n), "libspy_backend.so does not export %s" % n
    assert sorted(G.SIGNATURES) == names


@pytest.mark.parametrize("alignment", [32, 64, 4096])
def test_round_trip_of_every_value_type(G, tmp_path, alignment):
    from spy_amd import _lib as H
    rng = np.random.default_rng(alignment)
    kv = [("general.architecture", G.STRING, "llama"), ("a.u8", G.U8, 200), ("a.i8", G.I8, -100), ("a.u16", G.U16, 60000),
          ("a.i16", G.I16, -30000), ("a.u32", G.U32, 4000000000), ("a.i32", G.I32, -2000000000), ("a.f32", G.F32, 1e-5),
          ("a.bool", G.BOOL, True), ("a.u64", G.U64, 1 << 40), ("a.i64", G.I64, -(1 << 40)), ("a.f64", G.F64, 2.5),
          ("a.empty", G.STRING, ""), ("tokenizer.ggml.tokens", G.ARRAY, (G.STRING, ["<unk>", "", "▁he", "\xe9"])),
          ("tokenizer.ggml.scores", G.ARRAY, (G.F32, [0.0, -1.5, -2.0, 3.25])), ("tokenizer.ggml.token_type", G.ARRAY, (G.I32, [2, 3, 1, 1]))]
    tensors = [("t.f32", H.F32, [7], rng.integers(0, 256, 28, dtype=np.uint8)),
               ("t.q4_0", H.Q4_0, [64, 3], rng.integers(0, 256, 3 * 36, dtype=np.uint8)),
               ("t.q8_0", H.Q8_0, [32, 5], rng.integers(0, 256, 5 * 34, dtype=np.uint8)),
               ("t.q4_k", H.Q4_K, [256, 2], rng.integers(0, 256, 2 * 144, dtype=np.uint8)),
               ("t.q6_k", H.Q6_K, [512], rng.integers(0, 256, 2 * 210, dtype=np.uint8)),
               ("t.f16", H.F16, [3, 2, 2], rng.integers(0, 256, 24, dtype=np.uint8))]
    path = G.write_gguf(str(tmp_path / "x.gguf"), kv, tensors, alignment=alignment)
    f = G.GGUFFile(path)
    hd = f.header()
    n_kv = len(kv) + (1 if alignment != 32 else 0)
    assert (hd["version"], hd["n_tensors"], hd["n_kv"], hd["alignment"]) == (3, 6, n_kv, alignment)
    assert hd["data_offset"] % alignment == 0
    assert hd["data_bytes"] == sum(-(-t[3].nbytes // alignment) * alignment for t in tensors)
    assert os.path.getsize(path) == hd["data_offset"] + hd["data_bytes"]
    assert f.get_str("general.architecture") == "llama" and f.get_str("a.empty") == ""
    assert f.get_u32("a.u32") == 4000000000
    assert f.get_f32("a.f32") == np.float32(1e-5)
    for key, want in (("a.u8", G.U8), ("a.i8", G.I8), ("a.u16", G.U16), ("a.i16", G.I16), ("a.i32", G.I32), ("a.bool", G.BOOL),
                      ("a.u64", G.U64), ("a.i64", G.I64), ("a.f64", G.F64)):
        assert f.kv_type(key)[0] == want
    assert f.kv_type("tokenizer.ggml.tokens") == (G.ARRAY, G.STRING, 4)
    assert [f.get_arr_str("tokenizer.ggml.tokens", i) for i in range(4)] == ["<unk>".encode(), b"", "▁he".encode(), "\xe9".encode()]
    assert np.array_equal(f.get_arr("tokenizer.ggml.scores", np.float32), np.array([0.0, -1.5, -2.0, 3.25], np.float32))
    assert np.array_equal(f.get_arr("tokenizer.ggml.token_type", np.int32), [2, 3, 1, 1])
    offset = 0
    for i, (name, t, ne, data) in enumerate(tensors):
        info = f.tensor_info(i)
        assert info["name"] == name and info["type"] == t and info["n_dim"] == len(ne)
        assert info["ne"] == list(ne) + [1] * (4 - len(ne)) and info["nbytes"] == data.nbytes and info["offset"] == offset
        assert f.find_tensor(name) == i
        assert np.array_equal(f.tensor_data(i), data)
        offset += -(-data.nbytes // alignment) * alignment
    assert f.find_tensor("nope") == -1
    # strict getters, like the reference's std::get<>: a value stored with another type is refused
    with pytest.raises(G.GGUFError) as e:
        f.get_u32("a.u64")
    assert e.value.code == G.EKEY and "a.u64" in str(e.value)
    with pytest.raises(G.GGUFError) as e:
        f.get_u32("absent.key")
    assert e.value.code == G.EKEY
    f.close()


def test_writer_layout_independently(G, tmp_path):
    """The first bytes of a written file, decoded by hand."""
    from spy_amd import _lib as H
    path = G.write_gguf(str(tmp_path / "y.gguf"), [("k", G.U32, 7)], [("w", H.F32, [2], np.arange(8, dtype=np.uint8))])
    raw = open(path, "rb").read()
    assert raw[:4] == b"GGUF" and struct.unpack_from("<IQQ", raw, 4) == (3, 1, 1)
    pos = 24
    klen, = struct.unpack_from("<Q", raw, pos)
    assert raw[pos + 8:pos + 8 + klen] == b"k"
    pos += 8 + klen
    assert struct.unpack_from("<II", raw, pos) == (G.U32, 7)
    pos += 8
    nlen, = struct.unpack_from("<Q", raw, pos)
    assert raw[pos + 8:pos + 8 + nlen] == b"w"
    pos += 8 + nlen
    assert struct.unpack_from("<IQIQ", raw, pos) == (1, 2, H.F32, 0)
    pos += 24
    data_at = -(-pos // 32) * 32
    assert raw[data_at:data_at + 8] == bytes(range(8)) and len(raw) == data_at + 32


def test_broken_files_are_rejected_with_a_message(G, tmp_path):
    from spy_amd import _lib as H
    good = G.write_gguf(str(tmp_path / "good.gguf"), [("general.architecture", G.STRING, "llama")],
                        [("w", H.Q4_0, [64], np.zeros(36, np.uint8))])
    raw = open(good, "rb").read()

    def expect(name, blob, code, word):
        p = str(tmp_path / name)
        open(p, "wb").write(blob)
        with pytest.raises(G.GGUFError) as e:
            G.GGUFFile(p)
        assert e.value.code == code and word in str(e.value), str(e.value)

    expect("magic.gguf", b"GGML" + raw[4:], G.EFORMAT, "magic")
    expect("version.gguf", raw[:4] + struct.pack("<I", 1) + raw[8:], G.EFORMAT, "version")
    expect("short.gguf", raw[:40], G.EFORMAT, "truncated")
    expect("nodata.gguf", raw[:-30], G.EFORMAT, "beyond the file")
    with pytest.raises(G.GGUFError) as e:
        G.GGUFFile(str(tmp_path / "missing.gguf"))
    assert e.value.code == G.EIO
    # 48 elements are not a whole number of Q4_0 blocks
    bad = G.write_gguf(str(tmp_path / "blocks.gguf"), [], [("w", H.F32, [4], np.zeros(16, np.uint8))])
    blob = bytearray(open(bad, "rb").read())
    i = blob.index(b"w") + 1
    struct.pack_into("<IQIQ", blob, i, 1, 48, H.Q4_0, 0)
    expect("blocks2.gguf", bytes(blob), G.EFORMAT, "multiple of the block size")
    # an offset that is not aligned
    struct.pack_into("<IQIQ", blob, i, 1, 4, H.F32, 8)
    expect("offset.gguf", bytes(blob), G.EFORMAT, "not aligned")
    # a tensor type this backend does not store (Q5_0 = 6)
    struct.pack_into("<IQIQ", blob, i, 1, 32, 6, 0)
    expect("type.gguf", bytes(blob), G.EUNSUPPORTED, "type 6")
    # crafted sizes that wrap 64-bit arithmetic must not pass the bounds checks: an offset near 2^64 (aligned), an element
    # count whose byte size wraps, and a two-dimensional shape whose product wraps to a small number
    struct.pack_into("<IQIQ", blob, i, 1, 4, H.F32, 2 ** 64 - 32)
    expect("wrap_offset.gguf", bytes(blob), G.EFORMAT, "beyond the file")
    struct.pack_into("<IQIQ", blob, i, 1, 2 ** 62, H.F32, 0)
    expect("wrap_bytes.gguf", bytes(blob), G.EFORMAT, "overflows")
    two = G.write_gguf(str(tmp_path / "two.gguf"), [], [("w", H.F32, [2, 2], np.zeros(16, np.uint8))])
    blob2 = bytearray(open(two, "rb").read())
    j = blob2.index(b"w") + 1
    struct.pack_into("<IQQIQ", blob2, j, 2, 2 ** 33, 2 ** 31 + 1, H.F32, 0)      # product = 2^64 + 2^33: wraps to 2^33
    expect("wrap_shape.gguf", bytes(blob2), G.EFORMAT, "overflows")


def test_loader_refuses_models_it_does_not_run(G, tmp_path):
    """These checks come before the first device call, so they run without a GPU."""
    cfg, tensors = small_model(G)

    def refuse(name, code, word, **kw):
        p = G.write_llama(str(tmp_path / name), cfg, tensors, **kw)
        h = G._vp()
        rc = G.load().spy_gguf_model_load(p.encode(), 0, h)
        msg = G.load().spy_gguf_last_error().decode()
        assert rc == code and word in msg and not h.value, (rc, msg)

    refuse("arch.gguf", G.EUNSUPPORTED, "architecture gpt2", arch="gpt2")
    refuse("gqa.gguf", G.EUNSUPPORTED, "grouped-query", head_count_kv=1)
    # context_length stored as UInt64: the reference's strict getter refuses it, so does this one
    kv = [(k, G.U64 if k == "llama.context_length" else t, v) for k, t, v in G.llama_kv(cfg)]
    infos = [(n, t, [c] if r == 1 else [c, r], tensors[n]) for n, (t, r, c) in cfg.tensor_shapes().items()]
    p = G.write_gguf(str(tmp_path / "u64.gguf"), kv, infos)
    h = G._vp()
    assert G.load().spy_gguf_model_load(p.encode(), 0, h) == G.EKEY and "llama.context_length" in G.load().spy_gguf_last_error().decode()
    # 64-wide heads (256 / 4): not the 128-wide heads the attention kernels are built for
    from spy_amd import model as M, _lib as H
    cfg2 = M.Config(n_layer=1, n_embd=256, n_head=4, n_ff=512, n_vocab=96, n_ctx=32, wtype=H.Q4_0)
    p = G.write_llama(str(tmp_path / "heads.gguf"), cfg2, M.synth_model(cfg2, seed=6))
    assert G.load().spy_gguf_model_load(p.encode(), 0, h) == G.EUNSUPPORTED and "128" in G.load().spy_gguf_last_error().decode()
