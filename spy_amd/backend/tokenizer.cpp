// SentencePiece tokenizer over the vocabulary of a GGUF file (see include/spy_vocab.h for what it follows).
#include "../../include/spy_vocab.h"

#include <cstring>
#include <queue>
#include <string>
#include <string_view>
#include <unordered_map>
#include <vector>

int spy_gguf_fail(int code, const char *fmt, ...);        // gguf_loader.cpp: sets the thread's error text

namespace {

struct Token { std::string text; float score = 0.0f; int32_t type = SPY_TOKEN_NORMAL; };

const char ESC[] = "\xe2\x96\x81";                        // U+2581, the escaped space

size_t utf8_len(char c) {
    static const size_t lookup[16] = {1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, 2, 3, 4};
    return lookup[(uint8_t)c >> 4];
}

}  // namespace

struct spy_vocab {
    std::vector<Token> tokens;
    std::unordered_map<std::string_view, int32_t> ids;    // views into tokens[i].text (the vector never changes after construction)
    int32_t bos = 1, eos = 2, unk = 0, sep = -1, pad = -1, linefeed = 13;
    bool add_space_prefix = true;

    int32_t find(std::string_view s) const { auto it = ids.find(s); return it == ids.end() ? -1 : it->second; }
    // <0xXX>, else the byte itself as a one-character token, else -1 (sentence_piece_vocab.h:213-223)
    int32_t byte_token(uint8_t ch) const {
        static const char HEX[] = "0123456789ABCDEF";
        const char buf[6] = {'<', '0', 'x', HEX[ch >> 4], HEX[ch & 15], '>'};
        const int32_t id = find(std::string_view(buf, 6));
        if (id >= 0) return id;
        const char c = (char)ch;
        return find(std::string_view(&c, 1));
    }
};

namespace {

struct Symbol { int prev, next; const char *text; size_t n; };
struct Bigram { int left, right; float score; size_t size; };
struct BigramLess {                                       // priority: higher score first, then the leftmost pair (:27-30)
    bool operator()(const Bigram &a, const Bigram &b) const { return a.score < b.score || (a.score == b.score && a.left > b.left); }
};

struct Session {
    const spy_vocab &v;
    std::vector<Symbol> symbols;
    std::priority_queue<Bigram, std::vector<Bigram>, BigramLess> queue;
    std::unordered_map<std::string, std::pair<int, int>> rev_merge;
    bool failed = false;

    void try_add_bigram(int left, int right) {
        if (left == -1 || right == -1) return;
        const std::string_view text(symbols[left].text, symbols[left].n + symbols[right].n);
        const int32_t id = v.find(text);
        if (id < 0) return;
        queue.push(Bigram{left, right, v.tokens[id].score, text.size()});
        rev_merge[std::string(text)] = {left, right};
    }
    void resegment(const Symbol &s, std::vector<int32_t> &out) {
        const std::string_view text(s.text, s.n);
        const int32_t id = v.find(text);
        if (id >= 0) { out.push_back(id); return; }
        const auto p = rev_merge.find(std::string(text));
        if (p == rev_merge.end()) {                       // no token and no merge: spell the bytes
            for (size_t j = 0; j < s.n; j++) {
                const int32_t b = v.byte_token((uint8_t)s.text[j]);
                if (b < 0) { failed = true; return; }
                out.push_back(b);
            }
            return;
        }
        resegment(symbols[p->second.first], out);
        resegment(symbols[p->second.second], out);
    }
    void run(const std::string &text, std::vector<int32_t> &out) {
        int index = 0;
        size_t offs = 0;
        while (offs < text.size()) {                      // one symbol per UTF-8 character
            Symbol s;
            s.text = text.data() + offs;
            s.n = std::min(utf8_len(text[offs]), text.size() - offs);
            offs += s.n;
            s.prev = index - 1;
            s.next = offs == text.size() ? -1 : index + 1;
            index++;
            symbols.push_back(s);
        }
        for (size_t i = 1; i < symbols.size(); i++) try_add_bigram((int)i - 1, (int)i);
        while (!queue.empty()) {
            const Bigram b = queue.top();
            queue.pop();
            Symbol &l = symbols[b.left], &r = symbols[b.right];
            if (l.n == 0 || r.n == 0 || l.n + r.n != b.size) continue;     // one of them was merged meanwhile
            l.n += r.n;
            r.n = 0;
            l.next = r.next;
            if (r.next >= 0) symbols[r.next].prev = b.left;
            try_add_bigram(l.prev, b.left);
            try_add_bigram(b.left, l.next);
        }
        if (symbols.empty()) return;
        for (int i = 0; i != -1; i = symbols[i].next) resegment(symbols[i], out);
    }
};

int get_id(const spy_gguf *g, const char *key, int32_t n_vocab, int32_t &id) {
    int32_t type;
    if (spy_gguf_kv_type(g, key, &type, nullptr, nullptr) != 0) return 0;           // absent: keep the default
    uint32_t v;
    const int rc = spy_gguf_get_u32(g, key, &v);
    if (rc) return rc;
    if (v < (uint32_t)n_vocab) id = (int32_t)v;                                     // bad ids keep the default (abstract_vocab.h:104-111)
    return 0;
}

}  // namespace

extern "C" int spy_vocab_from_gguf(const spy_gguf *g, spy_vocab **out) {
    if (!g || !out) return spy_gguf_fail(SPY_GGUF_EINVAL, "null argument");
    *out = nullptr;
    int32_t type, et;
    uint64_t n;
    int rc = spy_gguf_kv_type(g, "tokenizer.ggml.tokens", &type, &et, &n);
    if (rc) return rc;
    if (type != SPY_GGUF_ARRAY || et != SPY_GGUF_STRING) return spy_gguf_fail(SPY_GGUF_EKEY, "tokenizer.ggml.tokens is not an array of strings");
    spy_vocab *v = new spy_vocab;
    v->tokens.resize(n);
    for (uint64_t i = 0; i < n; i++) {
        const char *s; uint64_t len;
        if ((rc = spy_gguf_get_arr_str(g, "tokenizer.ggml.tokens", i, &s, &len))) { delete v; return rc; }
        v->tokens[i].text.assign(s, len);
    }
    for (uint64_t i = 0; i < n; i++) v->ids[std::string_view(v->tokens[i].text)] = (int32_t)i;   // a repeated text keeps its last id (insert_or_assign, :78)
    const void *p; uint64_t m;
    if (spy_gguf_kv_type(g, "tokenizer.ggml.scores", &type, &et, &m) == 0) {
        if (type != SPY_GGUF_ARRAY || et != SPY_GGUF_F32 || m < n) { delete v; return spy_gguf_fail(SPY_GGUF_EKEY, "tokenizer.ggml.scores is not an array of %llu Float32", (unsigned long long)n); }
        spy_gguf_get_arr_data(g, "tokenizer.ggml.scores", &p, &m);
        for (uint64_t i = 0; i < n; i++) memcpy(&v->tokens[i].score, (const uint8_t *)p + 4 * i, 4);
    }
    if (spy_gguf_kv_type(g, "tokenizer.ggml.token_type", &type, &et, &m) == 0) {
        if (type != SPY_GGUF_ARRAY || et != SPY_GGUF_I32 || m < n) { delete v; return spy_gguf_fail(SPY_GGUF_EKEY, "tokenizer.ggml.token_type is not an array of %llu Int32", (unsigned long long)n); }
        spy_gguf_get_arr_data(g, "tokenizer.ggml.token_type", &p, &m);
        for (uint64_t i = 0; i < n; i++) memcpy(&v->tokens[i].type, (const uint8_t *)p + 4 * i, 4);
    }
    const int32_t nv = (int32_t)n;
    if ((rc = get_id(g, "tokenizer.ggml.bos_token_id", nv, v->bos)) || (rc = get_id(g, "tokenizer.ggml.eos_token_id", nv, v->eos)) ||
        (rc = get_id(g, "tokenizer.ggml.unknown_token_id", nv, v->unk)) || (rc = get_id(g, "tokenizer.ggml.seperator_token_id", nv, v->sep)) ||
        (rc = get_id(g, "tokenizer.ggml.padding_token_id", nv, v->pad))) { delete v; return rc; }
    const int32_t lf = v->byte_token('\n');
    if (lf >= 0) v->linefeed = lf;
    *out = v;
    return 0;
}

extern "C" void spy_vocab_free(spy_vocab *v) { delete v; }
extern "C" int32_t spy_vocab_size(const spy_vocab *v) { return v ? (int32_t)v->tokens.size() : 0; }

extern "C" int spy_vocab_special_ids(const spy_vocab *v, int32_t *bos, int32_t *eos, int32_t *unk, int32_t *sep, int32_t *pad, int32_t *linefeed) {
    if (!v) return spy_gguf_fail(SPY_GGUF_EINVAL, "null argument");
    if (bos) *bos = v->bos;
    if (eos) *eos = v->eos;
    if (unk) *unk = v->unk;
    if (sep) *sep = v->sep;
    if (pad) *pad = v->pad;
    if (linefeed) *linefeed = v->linefeed;
    return 0;
}

extern "C" int spy_vocab_token(const spy_vocab *v, int32_t id, const char **text, uint64_t *len, float *score, int32_t *type) {
    if (!v || id < 0 || id >= (int32_t)v->tokens.size()) return spy_gguf_fail(SPY_GGUF_EINVAL, "token id %d of %d", id, v ? (int)v->tokens.size() : 0);
    const Token &t = v->tokens[id];
    if (text) *text = t.text.data();
    if (len) *len = t.text.size();
    if (score) *score = t.score;
    if (type) *type = t.type;
    return 0;
}

extern "C" int64_t spy_vocab_tokenize(const spy_vocab *v, const char *text, uint64_t len, int32_t add_bos, int32_t special, int32_t *ids, uint64_t cap) {
    if (!v || (!text && len) || (!ids && cap)) return spy_gguf_fail(SPY_GGUF_EINVAL, "null argument");
    (void)special;                                        // the reference's table of special tokens is empty: no partition
    std::vector<int32_t> out;
    if (add_bos && v->bos != -1) out.push_back(v->bos);
    if (len) {
        std::string s;
        s.reserve(len * 3 + 3);
        if (v->add_space_prefix) s += ESC;
        for (uint64_t i = 0; i < len; i++) { if (text[i] == ' ') s += ESC; else s += text[i]; }
        Session session{*v, {}, {}, {}, false};
        session.run(s, out);
        if (session.failed) return spy_gguf_fail(SPY_GGUF_EKEY, "a character of the text has neither a token nor a byte token in this vocabulary");
    }
    for (uint64_t i = 0; i < out.size() && i < cap; i++) ids[i] = out[i];
    return (int64_t)out.size();
}

namespace {
void piece(const spy_vocab *v, int32_t id, std::string &out) {
    if (id < 0 || id >= (int32_t)v->tokens.size()) return;
    const Token &t = v->tokens[id];
    switch (t.type) {
    case SPY_TOKEN_NORMAL: {
        size_t pos = 0;
        for (;;) {
            const size_t at = t.text.find(ESC, pos);
            if (at == std::string::npos) { out.append(t.text, pos, std::string::npos); break; }
            out.append(t.text, pos, at - pos);
            out += ' ';
            pos = at + 3;
        }
        break;
    }
    case SPY_TOKEN_BYTE: {                                // "<0xXX>" (sentence_piece_vocab.h:225-230)
        auto hex = [](char c) { return c >= '0' && c <= '9' ? c - '0' : c >= 'A' && c <= 'F' ? c - 'A' + 10 : c >= 'a' && c <= 'f' ? c - 'a' + 10 : 0; };
        if (t.text.size() >= 5) out += (char)(hex(t.text[3]) * 16 + hex(t.text[4]));
        break;
    }
    case SPY_TOKEN_USER_DEFINED: out += t.text; break;
    case SPY_TOKEN_UNKNOWN: out += "\xe2\x96\x85"; break;
    default: break;                                       // control: nothing (undefined / unused abort in the reference)
    }
}
}  // namespace

extern "C" int64_t spy_vocab_token_to_piece(const spy_vocab *v, int32_t id, char *buf, uint64_t cap) {
    if (!v || (!buf && cap)) return spy_gguf_fail(SPY_GGUF_EINVAL, "null argument");
    std::string s;
    piece(v, id, s);
    memcpy(buf, s.data(), s.size() < cap ? s.size() : cap);
    return (int64_t)s.size();
}

extern "C" int64_t spy_vocab_detokenize(const spy_vocab *v, const int32_t *ids, uint64_t n, char *buf, uint64_t cap) {
    if (!v || (!ids && n) || (!buf && cap)) return spy_gguf_fail(SPY_GGUF_EINVAL, "null argument");
    std::string s;
    for (uint64_t i = 0; i < n; i++) piece(v, ids[i], s);
    memcpy(buf, s.data(), s.size() < cap ? s.size() : cap);
    return (int64_t)s.size();
}
