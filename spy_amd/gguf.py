"""GGUF files: a writer (the reference has a reader only; tests and synthetic models need files) and the
ctypes binding of the C reader / loader in libspy_backend.so (include/spy_gguf.h).

File layout as spy::GGUFAdapter::init_from_file reads it (storage/src/adapter/gguf_adapter.cpp:90-190):
magic "GGUF", u32 version, u64 tensor count, u64 key/value count, key/value pairs, tensor infos
{string name, u32 n_dim, u64 ne[n_dim], u32 type, u64 offset}, padding to `general.alignment`, tensor data
each padded to the alignment."""
import ctypes as C
import os
import struct

import numpy as np

from . import _lib as H
from . import backend_driver as B

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_SCALAR_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<?", U64: "<Q", I64: "<q", F64: "<d"}

EIO, EFORMAT, EKEY, EUNSUPPORTED, EINVAL = -1, -2, -3, -4, -5


def _string(s):
    b = s if isinstance(s, bytes) else s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _value(vtype, v):
    if vtype == STRING:
        return _string(v)
    if vtype == ARRAY:
        etype, items = v
        out = [struct.pack("<IQ", etype, len(items))]
        if etype == STRING:
            out += [_string(x) for x in items]
        else:
            out.append(np.asarray(items, dtype=np.dtype(_SCALAR_FMT[etype][1:]).newbyteorder("<")).tobytes())
        return b"".join(out)
    return struct.pack(_SCALAR_FMT[vtype], v)


def write_gguf(path, kv, tensors, alignment=32, version=3):
    """kv: list of (key, type, value) (arrays: value = (element type, sequence)); tensors: list of
    (name, type, ne, data) with ne[0] the contiguous dimension and data a uint8 array in the type's block
    layout.  `general.alignment` is written when it differs from the default 32."""
    kv = list(kv)
    if alignment != 32 and not any(k == "general.alignment" for k, _, _ in kv):
        kv.append(("general.alignment", U32, alignment))
    head = [b"GGUF", struct.pack("<IQQ", version, len(tensors), len(kv))]
    for key, vtype, v in kv:
        head.append(_string(key) + struct.pack("<I", vtype) + _value(vtype, v))
    offset = 0
    for name, ttype, ne, data in tensors:
        nbytes = H.row_size(ttype, int(np.prod(ne)))
        assert data.nbytes == nbytes, (name, data.nbytes, nbytes)
        head.append(_string(name) + struct.pack("<I", len(ne)) + struct.pack("<%dQ" % len(ne), *ne) + struct.pack("<IQ", ttype, offset))
        offset += -(-nbytes // alignment) * alignment
    blob = b"".join(head)
    with open(path, "wb") as f:
        f.write(blob)
        f.write(b"\0" * (-len(blob) % alignment))
        for name, ttype, ne, data in tensors:
            f.write(np.ascontiguousarray(data).view(np.uint8).tobytes())
            f.write(b"\0" * (-data.nbytes % alignment))
    return path


def llama_kv(cfg, tokens=None, arch="llama", head_count_kv=None):
    """The metadata the reference's HyperParam / LLAMAModel read (model/include/llm/model/abstract_model.h:72-144,
    llama.h:55-62), stored with the types its strict getters demand; a dummy vocabulary unless given."""
    if tokens is None:
        tokens = ["<t%d>" % i for i in range(cfg.n_vocab)]
    return [
        ("general.architecture", STRING, arch),
        ("general.name", STRING, "synthetic"),
        (arch + ".context_length", U32, cfg.n_ctx),
        (arch + ".embedding_length", U32, cfg.n_embd),
        (arch + ".feed_forward_length", U32, cfg.n_ff),
        (arch + ".attention.head_count", U32, cfg.n_head),
        (arch + ".attention.head_count_kv", U32, cfg.n_head if head_count_kv is None else head_count_kv),
        (arch + ".block_count", U32, cfg.n_layer),
        (arch + ".attention.layer_norm_rms_epsilon", F32, cfg.eps),
        (arch + ".rope.freq_base", F32, cfg.rope_freq_base),
        (arch + ".rope.dimension_count", U32, cfg.n_embd // cfg.n_head),
        ("tokenizer.ggml.model", STRING, "llama"),
        ("tokenizer.ggml.tokens", ARRAY, (STRING, tokens)),
    ]


def write_llama(path, cfg, tensors, tokens=None, alignment=32, **kw):
    """A model of spy_amd.model.Config / synth_model as a GGUF file."""
    infos = []
    for name, (t, rows, cols) in cfg.tensor_shapes().items():
        ne = [cols] if rows == 1 and "norm" in name else [cols, rows]
        infos.append((name, t, ne, tensors[name]))
    return write_gguf(path, llama_kv(cfg, tokens, **kw), infos, alignment)


# ---- the C reader / loader --------------------------------------------------------------------------
_vp, _u32, _u64, _i32, _i64 = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int32, C.c_int64
_P = C.POINTER
SIGNATURES = {
    "spy_gguf_last_error": (C.c_char_p, []),
    "spy_gguf_open": (C.c_int, [C.c_char_p, _P(_vp)]),
    "spy_gguf_close": (None, [_vp]),
    "spy_gguf_header": (C.c_int, [_vp, _P(_u32), _P(_u64), _P(_u64), _P(_u32), _P(_u64), _P(_u64)]),
    "spy_gguf_kv_type": (C.c_int, [_vp, C.c_char_p, _P(_i32), _P(_i32), _P(_u64)]),
    "spy_gguf_get_u32": (C.c_int, [_vp, C.c_char_p, _P(_u32)]),
    "spy_gguf_get_f32": (C.c_int, [_vp, C.c_char_p, _P(C.c_float)]),
    "spy_gguf_get_str": (C.c_int, [_vp, C.c_char_p, _P(_vp), _P(_u64)]),
    "spy_gguf_get_arr_str": (C.c_int, [_vp, C.c_char_p, _u64, _P(_vp), _P(_u64)]),
    "spy_gguf_get_arr_data": (C.c_int, [_vp, C.c_char_p, _P(_vp), _P(_u64)]),
    "spy_gguf_tensor_info": (C.c_int, [_vp, _u64, _P(C.c_char_p), _P(_i32), _P(_i32), _P(_i64 * 4), _P(_u64), _P(_u64)]),
    "spy_gguf_find_tensor": (_i64, [_vp, C.c_char_p]),
    "spy_gguf_tensor_data": (C.c_int, [_vp, _u64, _P(_vp)]),
    "spy_gguf_model_load": (C.c_int, [C.c_char_p, _i32, _P(_vp)]),
    "spy_gguf_model_engine": (_vp, [_vp]),
    "spy_gguf_model_file": (_vp, [_vp]),
    "spy_gguf_model_info": (C.c_int, [_vp, _P(H.LlamaDesc), _P(_u64), _P(C.c_double), _P(C.c_double), _P(C.c_double)]),
    "spy_gguf_model_free": (None, [_vp]),
}
_lib = None


def load():
    global _lib
    if _lib is None:
        lib = C.CDLL(B.LIB_PATH) if os.path.exists(B.LIB_PATH) else None
        if lib is None:
            raise RuntimeError("%s is missing: build it with `make -C spy_amd/backend`" % B.LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


class GGUFError(RuntimeError):
    def __init__(self, code, what):
        super().__init__("%s: %s (code %d)" % (what, load().spy_gguf_last_error().decode("utf-8", "replace"), code))
        self.code = code


def _check(rc, what):
    if rc != 0:
        raise GGUFError(rc, what)


class GGUFFile:
    """A parsed, memory-mapped GGUF file (spy_gguf_open)."""

    def __init__(self, path=None, handle=None):
        self.L = load()
        self._own = handle is None
        if handle is None:
            h = _vp()
            _check(self.L.spy_gguf_open(os.fsencode(path), C.byref(h)), "spy_gguf_open(%s)" % path)
            handle = h.value
        self.h = handle

    def close(self):
        if self.h and self._own:
            self.L.spy_gguf_close(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def header(self):
        v, nt, nk, al, off, nb = _u32(), _u64(), _u64(), _u32(), _u64(), _u64()
        _check(self.L.spy_gguf_header(self.h, v, nt, nk, al, off, nb), "spy_gguf_header")
        return {"version": v.value, "n_tensors": nt.value, "n_kv": nk.value, "alignment": al.value, "data_offset": off.value, "data_bytes": nb.value}

    def kv_type(self, key):
        t, e, n = _i32(), _i32(), _u64()
        _check(self.L.spy_gguf_kv_type(self.h, key.encode(), t, e, n), "spy_gguf_kv_type(%s)" % key)
        return t.value, e.value, n.value

    def get_u32(self, key):
        v = _u32()
        _check(self.L.spy_gguf_get_u32(self.h, key.encode(), v), "spy_gguf_get_u32(%s)" % key)
        return v.value

    def get_f32(self, key):
        v = C.c_float()
        _check(self.L.spy_gguf_get_f32(self.h, key.encode(), v), "spy_gguf_get_f32(%s)" % key)
        return v.value

    def get_str(self, key):
        p, n = _vp(), _u64()
        _check(self.L.spy_gguf_get_str(self.h, key.encode(), p, n), "spy_gguf_get_str(%s)" % key)
        return C.string_at(p.value, n.value).decode("utf-8")

    def get_arr_str(self, key, i):
        p, n = _vp(), _u64()
        _check(self.L.spy_gguf_get_arr_str(self.h, key.encode(), i, p, n), "spy_gguf_get_arr_str(%s, %d)" % (key, i))
        return C.string_at(p.value, n.value)

    def get_arr(self, key, dtype):
        p, n = _vp(), _u64()
        _check(self.L.spy_gguf_get_arr_data(self.h, key.encode(), p, n), "spy_gguf_get_arr_data(%s)" % key)
        return np.frombuffer(C.string_at(p.value, n.value * np.dtype(dtype).itemsize), dtype=dtype)

    def tensor_info(self, i):
        name, t, nd, ne, off, nb = C.c_char_p(), _i32(), _i32(), (_i64 * 4)(), _u64(), _u64()
        _check(self.L.spy_gguf_tensor_info(self.h, i, name, t, nd, ne, off, nb), "spy_gguf_tensor_info(%d)" % i)
        return {"name": name.value.decode(), "type": t.value, "n_dim": nd.value, "ne": list(ne), "offset": off.value, "nbytes": nb.value}

    def find_tensor(self, name):
        return self.L.spy_gguf_find_tensor(self.h, name.encode())

    def tensor_data(self, i):
        p = _vp()
        _check(self.L.spy_gguf_tensor_data(self.h, i, p), "spy_gguf_tensor_data(%d)" % i)
        return np.frombuffer(C.string_at(p.value, self.tensor_info(i)["nbytes"]), dtype=np.uint8)


class GGUFModel:
    """File -> HBM -> token loop (spy_gguf_model_load).  `engine` is a spy_amd.model.Engine over the loaded
    model: forward / decode_greedy / generate as for a model built from arrays."""

    def __init__(self, path, n_ctx=0, device_id=0):
        from . import model as M
        H.init(device_id)
        self.L = load()
        h = _vp()
        _check(self.L.spy_gguf_model_load(os.fsencode(path), n_ctx, C.byref(h)), "spy_gguf_model_load(%s)" % path)
        self.h = h.value
        desc, nb, p_ms, u_ms, c_ms = H.LlamaDesc(), _u64(), C.c_double(), C.c_double(), C.c_double()
        _check(self.L.spy_gguf_model_info(self.h, desc, nb, p_ms, u_ms, c_ms), "spy_gguf_model_info")
        self.desc = desc
        self.weight_bytes, self.parse_ms, self.upload_ms, self.create_ms = nb.value, p_ms.value, u_ms.value, c_ms.value
        self.file = GGUFFile(handle=self.L.spy_gguf_model_file(self.h))
        cfg = M.Config(desc.n_layer, desc.n_embd, desc.n_head, desc.n_ff, desc.n_vocab, desc.n_ctx, desc.eps, desc.rope_freq_base,
                       desc.wtype, desc.t_out, desc.t_tok_embd)
        eng = M.Engine.__new__(M.Engine)
        eng.cfg, eng.L, eng.dev, eng.handle = cfg, H.load(), {}, C.c_void_p(self.L.spy_gguf_model_engine(self.h))
        eng.close = lambda: None                                 # the loaded model owns the token loop
        self.engine = eng

    @property
    def vocab(self):
        """SentencePiece vocabulary of the file (built on first use)."""
        if getattr(self, "_vocab", None) is None:
            if not getattr(self, "h", None):
                raise RuntimeError("the model has been closed")
            self._vocab = Vocab(self.file)
        return self._vocab

    def generate_text(self, prompt, n_predict):
        """What AutoModelGenerator::generate does with a prompt (app/cli/include/cli.h:60-129 in the Spy tree):
        tokenize(prompt, bos = true, special = false), prompt pass, greedy loop; returns (ids, text of the new tokens)."""
        ids = self.vocab.tokenize(prompt, add_bos=True, special=False)
        new = self.engine.generate(np.asarray(ids, dtype=np.int32), n_predict)
        return [int(t) for t in new], self.vocab.detokenize([int(t) for t in new])

    def close(self):
        if getattr(self, "_vocab", None) is not None:
            self._vocab.close()
            self._vocab = None
        if getattr(self, "h", None):
            self.engine.handle = None
            self.L.spy_gguf_model_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


# ---- SentencePiece vocabulary (include/spy_vocab.h) --------------------------------------------------
VOCAB_SIGNATURES = {
    "spy_vocab_from_gguf": (C.c_int, [_vp, _P(_vp)]),
    "spy_vocab_free": (None, [_vp]),
    "spy_vocab_size": (_i32, [_vp]),
    "spy_vocab_special_ids": (C.c_int, [_vp, _P(_i32), _P(_i32), _P(_i32), _P(_i32), _P(_i32), _P(_i32)]),
    "spy_vocab_token": (C.c_int, [_vp, _i32, _P(_vp), _P(_u64), _P(C.c_float), _P(_i32)]),
    "spy_vocab_tokenize": (_i64, [_vp, C.c_char_p, _u64, _i32, _i32, _P(_i32), _u64]),
    "spy_vocab_token_to_piece": (_i64, [_vp, _i32, C.c_char_p, _u64]),
    "spy_vocab_detokenize": (_i64, [_vp, _P(_i32), _u64, C.c_char_p, _u64]),
}


class Vocab:
    """SentencePiece vocabulary of a GGUF file: tokenize / detokenize as spy::SentencePieceVocab does."""

    def __init__(self, gguf_file):
        self.L = load()
        for name, (res, args) in VOCAB_SIGNATURES.items():
            fn = getattr(self.L, name)
            fn.restype, fn.argtypes = res, args
        h = _vp()
        _check(self.L.spy_vocab_from_gguf(gguf_file.h, C.byref(h)), "spy_vocab_from_gguf")
        self.h = h.value

    def close(self):
        if getattr(self, "h", None):
            self.L.spy_vocab_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __len__(self):
        return self.L.spy_vocab_size(self.h)

    def special_ids(self):
        v = [_i32() for _ in range(6)]
        _check(self.L.spy_vocab_special_ids(self.h, *v), "spy_vocab_special_ids")
        return dict(zip(("bos", "eos", "unk", "sep", "pad", "linefeed"), (x.value for x in v)))

    def token(self, i):
        p, n, s, t = _vp(), _u64(), C.c_float(), _i32()
        _check(self.L.spy_vocab_token(self.h, i, p, n, s, t), "spy_vocab_token(%d)" % i)
        return C.string_at(p.value, n.value), s.value, t.value

    def tokenize(self, text, add_bos=True, special=False):
        raw = text if isinstance(text, bytes) else text.encode("utf-8")
        cap = 3 * len(raw) + 8
        ids = (_i32 * cap)()
        n = self.L.spy_vocab_tokenize(self.h, raw, len(raw), int(add_bos), int(special), ids, cap)
        if n < 0:
            raise GGUFError(int(n), "spy_vocab_tokenize")
        return list(ids[:n])

    def piece(self, i):
        buf = C.create_string_buffer(256)
        n = self.L.spy_vocab_token_to_piece(self.h, i, buf, 256)
        return buf.raw[:n]

    def detokenize(self, ids):
        arr = (_i32 * max(len(ids), 1))(*ids)
        cap = 64 + 16 * len(ids)
        while True:
            buf = C.create_string_buffer(cap)
            n = self.L.spy_vocab_detokenize(self.h, arr, len(ids), buf, cap)
            if n < 0:
                raise GGUFError(int(n), "spy_vocab_detokenize")
            if n <= cap:
                return buf.raw[:n]
            cap = int(n)
