// SentencePiece tokenizer over the vocabulary of a GGUF file (see include/spy_vocab.h for what it follows).
#include "../../include/spy_vocab.h"

#include <algorithm>
#include <cstring>
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

// Greedy pair merging over the characters of one text (the SentencePiece scheme of sentence_piece_vocab.h:120-211): the text is
// a chain of pieces, at first one per UTF-8 character; the best-scoring adjacent pair that is a vocabulary entry is joined, and
// so on until no adjacent pair is an entry.  Pieces are kept as parallel arrays indexed by their position in the first chain;
// a piece of length 0 has been absorbed by its left neighbour.
struct Candidate { float score; int lhs, rhs; size_t joined; };   // joined: byte length of the pair when it was proposed
// heap order: the higher score wins, among equal scores the pair further left (:27-30)
inline bool worse(const Candidate &a, const Candidate &b) { return a.score < b.score || (a.score == b.score && a.lhs > b.lhs); }

class Merger {
public:
    explicit Merger(const spy_vocab &vocab) : v_(vocab) {}
    bool failed() const { return failed_; }

    void tokenize(const std::string &text, std::vector<int32_t> &out) {
        split_characters(text);
        const int n = (int)len_.size();
        if (n == 0) return;
        for (int i = 0; i + 1 < n; i++) propose(i, i + 1);
        while (!heap_.empty()) {
            std::pop_heap(heap_.begin(), heap_.end(), worse);
            const Candidate c = heap_.back();
            heap_.pop_back();
            // stale when either side was absorbed or grew since the proposal
            if (len_[c.lhs] == 0 || len_[c.rhs] == 0 || len_[c.lhs] + len_[c.rhs] != c.joined) continue;
            len_[c.lhs] = c.joined;
            len_[c.rhs] = 0;
            const int after = after_[c.rhs];
            after_[c.lhs] = after;
            if (after >= 0) before_[after] = c.lhs;
            propose(before_[c.lhs], c.lhs);
            propose(c.lhs, after);
        }
        for (int i = 0; i >= 0; i = after_[i]) emit(i, out);
    }

private:
    const spy_vocab &v_;
    std::vector<const char *> at_;
    std::vector<size_t> len_;
    std::vector<int> before_, after_;
    std::vector<Candidate> heap_;
    // every pair ever proposed, by its joined text: how a piece that is no entry itself is taken apart again (:181-211)
    std::unordered_map<std::string, std::pair<int, int>> halves_;
    bool failed_ = false;

    void split_characters(const std::string &text) {
        for (size_t o = 0; o < text.size();) {
            const size_t n = std::min(utf8_len(text[o]), text.size() - o);
            at_.push_back(text.data() + o);
            len_.push_back(n);
            before_.push_back((int)len_.size() - 2);
            o += n;
            after_.push_back(o < text.size() ? (int)len_.size() : -1);
        }
    }
    void propose(int lhs, int rhs) {
        if (lhs < 0 || rhs < 0) return;
        const std::string_view joined(at_[lhs], len_[lhs] + len_[rhs]);
        const int32_t id = v_.find(joined);
        if (id < 0) return;
        heap_.push_back(Candidate{v_.tokens[id].score, lhs, rhs, joined.size()});
        std::push_heap(heap_.begin(), heap_.end(), worse);
        halves_[std::string(joined)] = {lhs, rhs};
    }
    // a piece's ids: its own entry, else the ids of the two pieces it was joined from, else its bytes (explicit stack, right half pushed first)
    void emit(int piece, std::vector<int32_t> &out) {
        std::vector<int> todo(1, piece);
        while (!todo.empty()) {
            const int p = todo.back();
            todo.pop_back();
            const std::string_view text(at_[p], len_[p]);
            const int32_t id = v_.find(text);
            if (id >= 0) { out.push_back(id); continue; }
            const auto h = halves_.find(std::string(text));
            if (h != halves_.end()) { todo.push_back(h->second.second); todo.push_back(h->second.first); continue; }
            for (const char ch : text) {
                const int32_t b = v_.byte_token((uint8_t)ch);
                if (b < 0) { failed_ = true; return; }
                out.push_back(b);
            }
        }
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
        Merger merger(*v);
        merger.tokenize(s, out);
        if (merger.failed()) return spy_gguf_fail(SPY_GGUF_EKEY, "a character of the text has neither a token nor a byte token in this vocabulary");
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
