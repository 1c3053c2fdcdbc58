"""SentencePiece tokenizer (include/spy_vocab.h) on the CPU.

Checked against (1) cases worked out by hand from the merge rule, (2) a plain-Python restatement of
spy::SentencePieceVocab::tokenize_inner / try_add_bigram / resegment (model/include/llm/vocab/
sentence_piece_vocab.h:99-211 in the Spy tree) on random vocabularies and texts, (3) the round trip through
token_to_piece.  The reference's tests hold no tokenizer vectors: parity with its compiled code is unpinned."""
import heapq
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ESC = "▁".encode("utf-8")
NORMAL, UNKNOWN, CONTROL, USER, UNUSED, BYTE = 1, 2, 3, 4, 5, 6


@pytest.fixture(scope="module")
def G():
    from spy_amd import gguf
    gguf.load()
    return gguf


def make_vocab(G, tmp_path, name, pieces, with_bytes=True, extra_kv=()):
    """pieces: list of (bytes, score); ids 0..2 are <unk>, <s>, </s>, then (optionally) the 256 byte tokens."""
    toks = [(b"<unk>", 0.0, UNKNOWN), (b"<s>", 0.0, CONTROL), (b"</s>", 0.0, CONTROL)]
    if with_bytes:
        toks += [(b"<0x%02X>" % b, 0.0, BYTE) for b in range(256)]
    toks += [(p, s, NORMAL) for p, s in pieces]
    kv = [("general.architecture", G.STRING, "llama"), ("tokenizer.ggml.model", G.STRING, "llama"),
          ("tokenizer.ggml.tokens", G.ARRAY, (G.STRING, [t[0] for t in toks])),
          ("tokenizer.ggml.scores", G.ARRAY, (G.F32, [t[1] for t in toks])),
          ("tokenizer.ggml.token_type", G.ARRAY, (G.I32, [t[2] for t in toks]))] + list(extra_kv)
    path = G.write_gguf(str(tmp_path / name), kv, [])
    f = G.GGUFFile(path)
    v = G.Vocab(f)
    f.close()                                  # the vocabulary keeps its own copy
    return v, toks


def utf8_len(b):
    return [1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, 2, 3, 4][b >> 4]


def tokenize_restated(toks, text, add_bos=True):
    """The reference's algorithm, statement by statement, with fresh state."""
    table = {}
    for i, t in enumerate(toks):
        table[t[0]] = i
    out = [1] if add_bos else []
    if not text:
        return out
    s = ESC + text.replace(b" ", ESC)
    syms, offs = [], 0
    while offs < len(s):
        n = min(utf8_len(s[offs]), len(s) - offs)
        syms.append([len(syms) - 1, -1 if offs + n == len(s) else len(syms) + 1, offs, n])     # prev, next, start, n
        offs += n
    heap, rev = [], {}

    def add(l, r):
        if l == -1 or r == -1:
            return
        t = s[syms[l][2]:syms[l][2] + syms[l][3] + syms[r][3]]
        if t in table:
            heapq.heappush(heap, (-toks[table[t]][1], l, r, len(t)))
            rev[t] = (l, r)
    for i in range(1, len(syms)):
        add(i - 1, i)
    while heap:
        _, l, r, size = heapq.heappop(heap)
        L, R = syms[l], syms[r]
        if L[3] == 0 or R[3] == 0 or L[3] + R[3] != size:
            continue
        L[3] += R[3]
        R[3] = 0
        L[1] = R[1]
        if R[1] >= 0:
            syms[R[1]][0] = l
        add(L[0], l)
        add(l, L[1])

    def reseg(sym):
        t = s[sym[2]:sym[2] + sym[3]]
        if t in table:
            out.append(table[t])
        elif t in rev:
            reseg(syms[rev[t][0]])
            reseg(syms[rev[t][1]])
        else:
            for b in t:
                out.append(table[b"<0x%02X>" % b])
    i = 0
    while i != -1:
        reseg(syms[i])
        i = syms[i][1]
    return out


def test_header_symbols_are_exported(G):
    text = open(os.path.join(ROOT, "include", "spy_vocab.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(spy_vocab_[a-z0-9_]+)\s*\(", text)))
    assert sorted(G.VOCAB_SIGNATURES) == names and len(names) == 8
    for n in names:
        assert hasattr(G.load(), n)


def test_cases_worked_out_by_hand(G, tmp_path):
    e = lambda s: s.replace(" ", "▁").encode("utf-8")
    pieces = [(e(" "), -1.0), (b"h", -2), (b"e", -2), (b"l", -2), (b"o", -2), (b"w", -2), (b"r", -2), (b"d", -2), (b"a", -2),
              (b"he", -0.5), (b"ll", -0.6), (b"llo", -0.4), (b"hello", -0.1), (e(" hello"), -0.05),
              (b"or", -0.7), (b"ld", -0.8), (b"world", -0.2), (e(" world"), -0.15), (e(" w"), -0.9), (b"aa", -0.3)]
    v, toks = make_vocab(G, tmp_path, "hand.gguf", pieces)
    idx = {t[0]: i for i, t in enumerate(toks)}
    assert len(v) == len(toks) and v.special_ids() == {"bos": 1, "eos": 2, "unk": 0, "sep": -1, "pad": -1, "linefeed": idx[b"<0x0A>"]}
    # "hello world" -> "▁hello▁world".  he, ll, llo, hello, ▁hello are all tokens, so the first word merges completely;
    # "world" has no token for any of its halves (wo, wor, orld, rld): or, ld and ▁w merge and nothing larger can form
    assert v.tokenize("hello world") == [1, idx[e(" hello")], idx[e(" w")], idx[b"or"], idx[b"ld"]]
    assert v.tokenize("hello world", add_bos=False) == [idx[e(" hello")], idx[e(" w")], idx[b"or"], idx[b"ld"]]
    assert v.tokenize("", add_bos=True) == [1] and v.tokenize("", add_bos=False) == []
    # equal scores: the leftmost pair merges first -> "▁" "aa" "a", not "▁" "a" "aa"
    assert v.tokenize("aaa", add_bos=False) == [idx[e(" ")], idx[b"aa"], idx[b"a"]]
    assert v.tokenize("aaaa", add_bos=False) == [idx[e(" ")], idx[b"aa"], idx[b"aa"]]
    # "held": he + l + d (no "hel", no "eld", "ld" has a lower score than "he" but both merge: h e l d -> he l d -> he ld)
    assert v.tokenize("held", add_bos=False) == [idx[e(" ")], idx[b"he"], idx[b"ld"]]
    # characters without a token are spelled as bytes; é = C3 A9, € = E2 82 AC; "x" is ASCII without a token
    assert v.tokenize("hé", add_bos=False) == [idx[e(" ")], idx[b"h"], idx[b"<0xC3>"], idx[b"<0xA9>"]]
    assert v.tokenize("€x", add_bos=False) == [idx[e(" ")], idx[b"<0xE2>"], idx[b"<0x82>"], idx[b"<0xAC>"], idx[b"<0x78>"]]
    # special = true changes nothing (the reference never fills its table of special tokens)
    assert v.tokenize("<s>hello", add_bos=False, special=True) == v.tokenize("<s>hello", add_bos=False, special=False)
    # pieces: escaped spaces back to spaces, byte tokens to their byte, control tokens to nothing, unknown to U+2585
    assert v.piece(idx[e(" hello")]) == b" hello" and v.piece(idx[b"<0xC3>"]) == b"\xc3" and v.piece(1) == b"" and v.piece(0) == "▅".encode()
    for text in ("hello world", "héllo  w€rld", "a", " leading and trailing ", "tab\tnew\nline"):
        assert v.detokenize(v.tokenize(text, add_bos=True)) == (" " + text).encode("utf-8")


def test_against_the_restated_algorithm_on_random_vocabularies(G, tmp_path):
    rng = np.random.default_rng(7)
    alphabet = [b"a", b"b", b"c", b"d", " ".replace(" ", "▁").encode(), "é".encode(), "中".encode(), "\U0001f600".encode()]
    for trial in range(6):
        pieces = {}
        for a in alphabet[:6 + trial % 3]:
            pieces[a] = float(-10 - rng.integers(0, 3))
        while len(pieces) < 60:
            n = int(rng.integers(2, 5))
            p = b"".join(alphabet[int(i)] for i in rng.integers(0, len(alphabet), n))
            pieces[p] = float(np.round(-rng.random() * 4, 1))               # coarse scores: many ties
        v, toks = make_vocab(G, tmp_path, "rand%d.gguf" % trial, sorted(pieces.items()))
        for _ in range(200):
            n = int(rng.integers(1, 24))
            chars = [alphabet[int(i)] if i < len(alphabet) else b" " for i in rng.integers(0, len(alphabet) + 2, n)]
            text = b"".join(chars).replace(alphabet[4], b" ")
            if rng.random() < 0.1:
                text += bytes([int(rng.integers(128, 256))])                  # a stray byte (truncated UTF-8)
            want = tokenize_restated(toks, text)
            assert v.tokenize(text) == want, (trial, text)
            assert v.detokenize(want) == b" " + text


def test_vocabulary_without_byte_tokens_and_special_ids(G, tmp_path):
    v, toks = make_vocab(G, tmp_path, "nobytes.gguf", [("▁".encode(), -1.0), (b"a", -1.0), (b"\n", -1.0)], with_bytes=False,
                         extra_kv=[("tokenizer.ggml.bos_token_id", G.U32, 2), ("tokenizer.ggml.eos_token_id", G.U32, 1),
                                   ("tokenizer.ggml.padding_token_id", G.U32, 999)])         # 999 is out of range: default kept
    ids = v.special_ids()
    assert ids["bos"] == 2 and ids["eos"] == 1 and ids["pad"] == -1 and ids["linefeed"] == 5      # "\n" itself is the fallback token
    assert v.tokenize("a\na") == [2, 3, 4, 5, 4]
    with pytest.raises(G.GGUFError) as e:
        v.tokenize("ab")                        # b has no token and there are no byte tokens: the reference throws here
    assert e.value.code == G.EKEY
    assert v.token(4) == (b"a", -1.0, NORMAL)
