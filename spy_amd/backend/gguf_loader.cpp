// GGUF ingest: parse the memory-mapped file, upload every tensor once to HBM in its own block layout,
// create the token loop.  Follows what GGUFAdapter::init_from_file accepts
// (storage/src/adapter/gguf_adapter.cpp:90-190 in the Spy tree) and what HyperParam / LLAMAModel read from
// the metadata (model/include/llm/model/abstract_model.h:72-144, model/include/llm/model/llama.h:55-62).
#include "../../include/spy_gguf.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

namespace {

thread_local std::string g_error;

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

// bytes per block and elements per block of the tensor types this backend stores (NumberType codes)
bool type_layout(int32_t type, uint64_t &block_bytes, uint64_t &block_elems) {
    switch (type) {
    case SPY_HIP_F32:  block_bytes = 4;   block_elems = 1;   return true;
    case SPY_HIP_F16:  block_bytes = 2;   block_elems = 1;   return true;
    case SPY_HIP_Q4_0: block_bytes = 18;  block_elems = 32;  return true;
    case SPY_HIP_Q8_0: block_bytes = 34;  block_elems = 32;  return true;
    case SPY_HIP_Q4_K: block_bytes = 144; block_elems = 256; return true;
    case SPY_HIP_Q6_K: block_bytes = 210; block_elems = 256; return true;
    case SPY_HIP_I32:  block_bytes = 4;   block_elems = 1;   return true;
    default: return false;
    }
}

const uint64_t SCALAR_SIZE[13] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};

struct KV {
    int32_t type = -1, elem_type = -1;
    const uint8_t *data = nullptr;          // scalar: the value; string: its bytes; numeric array: packed elements
    uint64_t n = 0;                         // string length / array length
    std::vector<std::pair<const char *, uint64_t>> strings;   // string arrays
};

struct TensorInfo {
    std::string name;
    int32_t type = 0, n_dim = 0;
    int64_t ne[4] = {1, 1, 1, 1};
    uint64_t offset = 0, nbytes = 0;
};

}  // namespace

// the same for the other sources of this library (tokenizer.cpp)
int spy_gguf_fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

struct spy_gguf {
    int fd = -1;
    const uint8_t *base = nullptr;
    uint64_t size = 0;
    uint32_t version = 0, alignment = 32;
    uint64_t n_tensors = 0, n_kv = 0, data_offset = 0, data_bytes = 0;
    std::map<std::string, KV> kv;
    std::vector<TensorInfo> tensors;
    std::map<std::string, uint64_t> by_name;
};

namespace {

struct Cursor {
    const uint8_t *p, *end;
    bool ok = true;
    template <class T> T get() {
        T v{};
        if ((uint64_t)(end - p) < sizeof(T)) { ok = false; return v; }
        memcpy(&v, p, sizeof(T));
        p += sizeof(T);
        return v;
    }
    bool skip(uint64_t n) {
        if ((uint64_t)(end - p) < n) { ok = false; return false; }
        p += n;
        return true;
    }
    bool str(const char *&s, uint64_t &len) {
        len = get<uint64_t>();
        s = (const char *)p;
        return ok && skip(len);
    }
};

int parse(spy_gguf *g) {
    Cursor c{g->base, g->base + g->size};
    if (g->size < 24 || memcmp(g->base, "GGUF", 4) != 0) return fail(SPY_GGUF_EFORMAT, "invalid magic characters (expect: GGUF)");
    c.skip(4);
    g->version = c.get<uint32_t>();
    g->n_tensors = c.get<uint64_t>();
    g->n_kv = c.get<uint64_t>();
    if (g->version < 2 || g->version > 3) return fail(SPY_GGUF_EFORMAT, "GGUF version %u is not supported (2 and 3 are: 64-bit counts)", g->version);
    if (g->n_tensors > g->size || g->n_kv > g->size) return fail(SPY_GGUF_EFORMAT, "implausible header counts");
    for (uint64_t i = 0; i < g->n_kv; i++) {
        const char *ks; uint64_t klen;
        if (!c.str(ks, klen)) return fail(SPY_GGUF_EFORMAT, "truncated key/value section");
        KV v;
        v.type = (int32_t)c.get<uint32_t>();
        if (!c.ok || v.type < 0 || v.type > SPY_GGUF_F64) return fail(SPY_GGUF_EFORMAT, "unknown gguf data type %d of key %.*s", v.type, (int)klen, ks);
        if (v.type == SPY_GGUF_STRING) {
            const char *s; uint64_t n;
            if (!c.str(s, n)) return fail(SPY_GGUF_EFORMAT, "truncated string value");
            v.data = (const uint8_t *)s; v.n = n;
        } else if (v.type == SPY_GGUF_ARRAY) {
            v.elem_type = (int32_t)c.get<uint32_t>();
            v.n = c.get<uint64_t>();
            if (!c.ok || v.elem_type < 0 || v.elem_type > SPY_GGUF_F64 || v.elem_type == SPY_GGUF_ARRAY)
                return fail(SPY_GGUF_EFORMAT, "unknown gguf data type in array %.*s", (int)klen, ks);
            if (v.elem_type == SPY_GGUF_STRING) {
                if (v.n > g->size) return fail(SPY_GGUF_EFORMAT, "implausible array length");
                v.strings.reserve(v.n);
                for (uint64_t j = 0; j < v.n; j++) {
                    const char *s; uint64_t n;
                    if (!c.str(s, n)) return fail(SPY_GGUF_EFORMAT, "truncated string array %.*s", (int)klen, ks);
                    v.strings.emplace_back(s, n);
                }
            } else {
                v.data = c.p;
                if (v.n > g->size || !c.skip(v.n * SCALAR_SIZE[v.elem_type])) return fail(SPY_GGUF_EFORMAT, "truncated array %.*s", (int)klen, ks);
            }
        } else {
            v.data = c.p;
            if (!c.skip(SCALAR_SIZE[v.type])) return fail(SPY_GGUF_EFORMAT, "truncated value");
        }
        g->kv[std::string(ks, klen)] = std::move(v);
    }
    g->tensors.resize(g->n_tensors);
    for (uint64_t i = 0; i < g->n_tensors; i++) {
        TensorInfo &t = g->tensors[i];
        const char *s; uint64_t n;
        if (!c.str(s, n)) return fail(SPY_GGUF_EFORMAT, "truncated tensor infos");
        t.name.assign(s, n);
        t.n_dim = (int32_t)c.get<uint32_t>();
        if (!c.ok || t.n_dim < 1 || t.n_dim > 4) return fail(SPY_GGUF_EFORMAT, "tensor %s: %d dimensions", t.name.c_str(), t.n_dim);
        uint64_t elems = 1;
        bool overflow = false;
        for (int d = 0; d < t.n_dim; d++) {
            const uint64_t e = c.get<uint64_t>();
            t.ne[d] = (int64_t)e;
            if (e > (uint64_t)INT64_MAX || (e != 0 && elems > UINT64_MAX / e)) overflow = true;       // a crafted shape must not wrap the product
            else elems *= e;
        }
        if (overflow) return fail(SPY_GGUF_EFORMAT, "tensor %s: shape overflows 64 bits", t.name.c_str());
        t.type = (int32_t)c.get<uint32_t>();
        t.offset = c.get<uint64_t>();
        if (!c.ok) return fail(SPY_GGUF_EFORMAT, "truncated tensor infos");
        uint64_t bb, be;
        if (!type_layout(t.type, bb, be)) return fail(SPY_GGUF_EUNSUPPORTED, "tensor %s: type %d is not one this backend stores", t.name.c_str(), t.type);
        if (elems % be != 0) return fail(SPY_GGUF_EFORMAT, "tensor %s: number of elements (%llu) is not a multiple of the block size (%llu)",
                                         t.name.c_str(), (unsigned long long)elems, (unsigned long long)be);
        if (elems / be > UINT64_MAX / bb) return fail(SPY_GGUF_EFORMAT, "tensor %s: size overflows 64 bits", t.name.c_str());
        t.nbytes = elems / be * bb;
        g->by_name[t.name] = i;
    }
    auto al = g->kv.find("general.alignment");
    if (al != g->kv.end()) {
        if (al->second.type != SPY_GGUF_U32) return fail(SPY_GGUF_EKEY, "general.alignment is not stored as UInt32");
        memcpy(&g->alignment, al->second.data, 4);
        if (g->alignment == 0 || (g->alignment & (g->alignment - 1))) return fail(SPY_GGUF_EFORMAT, "alignment %u is not a power of two", g->alignment);
    }
    const uint64_t pos = (uint64_t)(c.p - g->base);
    g->data_offset = (pos + g->alignment - 1) / g->alignment * g->alignment;
    if (g->data_offset > g->size) return fail(SPY_GGUF_EFORMAT, "the tensor data would start beyond the file");
    const uint64_t room = g->size - g->data_offset;                  // bytes of the data section
    for (const TensorInfo &t : g->tensors) {
        if (t.offset % g->alignment != 0) return fail(SPY_GGUF_EFORMAT, "tensor %s: offset %llu is not aligned to %u", t.name.c_str(), (unsigned long long)t.offset, g->alignment);
        // subtraction form: none of these can wrap, whatever the file says
        if (t.offset > room || t.nbytes > room - t.offset)
            return fail(SPY_GGUF_EFORMAT, "tensor %s: data (%llu bytes at %llu) ends beyond the file", t.name.c_str(), (unsigned long long)t.nbytes,
                        (unsigned long long)t.offset);
        g->data_bytes += (t.nbytes + g->alignment - 1) / g->alignment * g->alignment;
    }
    return 0;
}

const KV *find(const spy_gguf *g, const char *key, int32_t type, int &rc) {
    auto it = g->kv.find(key);
    if (it == g->kv.end()) { rc = fail(SPY_GGUF_EKEY, "key %s is absent", key); return nullptr; }
    if (type >= 0 && it->second.type != type) { rc = fail(SPY_GGUF_EKEY, "key %s is stored as type %d, not %d", key, it->second.type, type); return nullptr; }
    rc = 0;
    return &it->second;
}

double ms_since(std::chrono::steady_clock::time_point t0) {
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
}

}  // namespace

extern "C" const char *spy_gguf_last_error(void) { return g_error.c_str(); }

extern "C" int spy_gguf_open(const char *path, spy_gguf **out) {
    if (!path || !out) return fail(SPY_GGUF_EINVAL, "null argument");
    *out = nullptr;
    const int fd = open(path, O_RDONLY);
    if (fd < 0) return fail(SPY_GGUF_EIO, "cannot open file: %s", path);
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) { close(fd); return fail(SPY_GGUF_EIO, "cannot stat file: %s", path); }
    void *base = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    if (base == MAP_FAILED) { close(fd); return fail(SPY_GGUF_EIO, "cannot map file: %s", path); }
    spy_gguf *g = new spy_gguf;
    g->fd = fd; g->base = (const uint8_t *)base; g->size = (uint64_t)st.st_size;
    const int rc = parse(g);
    if (rc) { spy_gguf_close(g); return rc; }
    *out = g;
    return 0;
}

extern "C" void spy_gguf_close(spy_gguf *g) {
    if (!g) return;
    if (g->base) munmap((void *)g->base, g->size);
    if (g->fd >= 0) close(g->fd);
    delete g;
}

extern "C" int spy_gguf_header(const spy_gguf *g, uint32_t *version, uint64_t *n_tensors, uint64_t *n_kv, uint32_t *alignment,
                               uint64_t *data_offset, uint64_t *data_bytes) {
    if (!g) return fail(SPY_GGUF_EINVAL, "null argument");
    if (version) *version = g->version;
    if (n_tensors) *n_tensors = g->n_tensors;
    if (n_kv) *n_kv = g->n_kv;
    if (alignment) *alignment = g->alignment;
    if (data_offset) *data_offset = g->data_offset;
    if (data_bytes) *data_bytes = g->data_bytes;
    return 0;
}

extern "C" int spy_gguf_kv_type(const spy_gguf *g, const char *key, int32_t *type, int32_t *elem_type, uint64_t *n) {
    if (!g || !key) return fail(SPY_GGUF_EINVAL, "null argument");
    int rc;
    const KV *v = find(g, key, -1, rc);
    if (!v) return rc;
    if (type) *type = v->type;
    if (elem_type) *elem_type = v->elem_type;
    if (n) *n = v->n;
    return 0;
}

extern "C" int spy_gguf_get_u32(const spy_gguf *g, const char *key, uint32_t *out) {
    if (!g || !key || !out) return fail(SPY_GGUF_EINVAL, "null argument");
    int rc;
    const KV *v = find(g, key, SPY_GGUF_U32, rc);
    if (!v) return rc;
    memcpy(out, v->data, 4);
    return 0;
}

extern "C" int spy_gguf_get_f32(const spy_gguf *g, const char *key, float *out) {
    if (!g || !key || !out) return fail(SPY_GGUF_EINVAL, "null argument");
    int rc;
    const KV *v = find(g, key, SPY_GGUF_F32, rc);
    if (!v) return rc;
    memcpy(out, v->data, 4);
    return 0;
}

extern "C" int spy_gguf_get_str(const spy_gguf *g, const char *key, const char **ptr, uint64_t *len) {
    if (!g || !key || !ptr || !len) return fail(SPY_GGUF_EINVAL, "null argument");
    int rc;
    const KV *v = find(g, key, SPY_GGUF_STRING, rc);
    if (!v) return rc;
    *ptr = (const char *)v->data; *len = v->n;
    return 0;
}

extern "C" int spy_gguf_get_arr_str(const spy_gguf *g, const char *key, uint64_t i, const char **ptr, uint64_t *len) {
    if (!g || !key || !ptr || !len) return fail(SPY_GGUF_EINVAL, "null argument");
    int rc;
    const KV *v = find(g, key, SPY_GGUF_ARRAY, rc);
    if (!v) return rc;
    if (v->elem_type != SPY_GGUF_STRING) return fail(SPY_GGUF_EKEY, "key %s is not an array of strings", key);
    if (i >= v->n) return fail(SPY_GGUF_EINVAL, "index %llu beyond the %llu entries of %s", (unsigned long long)i, (unsigned long long)v->n, key);
    *ptr = v->strings[i].first; *len = v->strings[i].second;
    return 0;
}

extern "C" int spy_gguf_get_arr_data(const spy_gguf *g, const char *key, const void **ptr, uint64_t *n) {
    if (!g || !key || !ptr || !n) return fail(SPY_GGUF_EINVAL, "null argument");
    int rc;
    const KV *v = find(g, key, SPY_GGUF_ARRAY, rc);
    if (!v) return rc;
    if (v->elem_type == SPY_GGUF_STRING) return fail(SPY_GGUF_EKEY, "key %s is an array of strings", key);
    *ptr = v->data; *n = v->n;
    return 0;
}

extern "C" int spy_gguf_tensor_info(const spy_gguf *g, uint64_t index, const char **name, int32_t *type, int32_t *n_dim, int64_t ne[4],
                                    uint64_t *offset, uint64_t *nbytes) {
    if (!g) return fail(SPY_GGUF_EINVAL, "null argument");
    if (index >= g->tensors.size()) return fail(SPY_GGUF_EINVAL, "tensor index %llu of %zu", (unsigned long long)index, g->tensors.size());
    const TensorInfo &t = g->tensors[index];
    if (name) *name = t.name.c_str();
    if (type) *type = t.type;
    if (n_dim) *n_dim = t.n_dim;
    if (ne) memcpy(ne, t.ne, sizeof(t.ne));
    if (offset) *offset = t.offset;
    if (nbytes) *nbytes = t.nbytes;
    return 0;
}

extern "C" int64_t spy_gguf_find_tensor(const spy_gguf *g, const char *name) {
    if (!g || !name) return -1;
    auto it = g->by_name.find(name);
    return it == g->by_name.end() ? -1 : (int64_t)it->second;
}

extern "C" int spy_gguf_tensor_data(const spy_gguf *g, uint64_t index, const void **ptr) {
    if (!g || !ptr) return fail(SPY_GGUF_EINVAL, "null argument");
    if (index >= g->tensors.size()) return fail(SPY_GGUF_EINVAL, "tensor index %llu of %zu", (unsigned long long)index, g->tensors.size());
    *ptr = g->base + g->data_offset + g->tensors[index].offset;
    return 0;
}

// ---- file -> HBM -> token loop ----------------------------------------------------------------------

struct spy_gguf_model {
    spy_gguf *file = nullptr;
    std::vector<void *> device;                 // one allocation per tensor, freed with the model
    std::vector<spy_hip_llama_layer> layers;
    spy_hip_llama_desc desc{};
    spy_hip_llama *engine = nullptr;
    uint64_t weight_bytes = 0;
    double parse_ms = 0, upload_ms = 0, create_ms = 0;
};

namespace {

bool is_matrix_type(int32_t t) { return t == SPY_HIP_Q4_0 || t == SPY_HIP_Q8_0 || t == SPY_HIP_Q4_K || t == SPY_HIP_Q6_K; }

// uploads tensor `name` after checking its type and shape (ne0 = contiguous dimension)
int upload(spy_gguf_model *m, const std::string &name, int64_t ne0, int64_t ne1, bool matrix, bool embedding, const void **dev, int32_t *type) {
    const spy_gguf *g = m->file;
    const int64_t idx = spy_gguf_find_tensor(g, name.c_str());
    if (idx < 0) return fail(SPY_GGUF_EFORMAT, "tensor %s is missing", name.c_str());
    const TensorInfo &t = g->tensors[(size_t)idx];
    if (t.ne[0] != ne0 || t.ne[1] != ne1 || t.ne[2] != 1 || t.ne[3] != 1)
        return fail(SPY_GGUF_EFORMAT, "tensor %s: shape [%lld, %lld, %lld, %lld], expected [%lld, %lld]", name.c_str(), (long long)t.ne[0], (long long)t.ne[1],
                    (long long)t.ne[2], (long long)t.ne[3], (long long)ne0, (long long)ne1);
    const bool ok = embedding ? (t.type == SPY_HIP_F32 || t.type == SPY_HIP_Q8_0) : matrix ? is_matrix_type(t.type) : t.type == SPY_HIP_F32;
    if (!ok) return fail(SPY_GGUF_EUNSUPPORTED, "tensor %s: type %d (%s)", name.c_str(), t.type,
                         embedding ? "token embeddings must be F32 or Q8_0" : matrix ? "matrices must be Q4_0, Q8_0, Q4_K or Q6_K" : "norm weights must be F32");
    void *p = nullptr;
    int rc = spy_hip_alloc(&p, t.nbytes);
    if (rc) return fail(rc, "tensor %s: device allocation of %llu bytes failed: %s", name.c_str(), (unsigned long long)t.nbytes, spy_hip_error_string(rc));
    m->device.push_back(p);
    rc = spy_hip_upload(p, g->base + g->data_offset + t.offset, t.nbytes, nullptr);
    if (rc) return fail(rc, "tensor %s: upload failed: %s", name.c_str(), spy_hip_error_string(rc));
    m->weight_bytes += t.nbytes;
    *dev = p;
    if (type) *type = t.type;
    return 0;
}

int build(spy_gguf_model *m, int32_t n_ctx) {
    const spy_gguf *g = m->file;
    const char *as; uint64_t alen;
    int rc = spy_gguf_get_str(g, "general.architecture", &as, &alen);
    if (rc) return rc;
    const std::string arch(as, alen);
    if (arch != "llama") return fail(SPY_GGUF_EUNSUPPORTED, "architecture %s (this backend runs llama)", arch.c_str());
    uint32_t ctx = 0, d = 0, ff = 0, heads = 0, heads_kv = 0, blocks = 0;
    float eps = 0.0f, freq_base = 10000.0f;
    if ((rc = spy_gguf_get_u32(g, (arch + ".context_length").c_str(), &ctx))) return rc;
    if ((rc = spy_gguf_get_u32(g, (arch + ".embedding_length").c_str(), &d))) return rc;
    if ((rc = spy_gguf_get_u32(g, (arch + ".feed_forward_length").c_str(), &ff))) return rc;
    if ((rc = spy_gguf_get_u32(g, (arch + ".attention.head_count").c_str(), &heads))) return rc;
    if ((rc = spy_gguf_get_u32(g, (arch + ".block_count").c_str(), &blocks))) return rc;
    if ((rc = spy_gguf_get_f32(g, (arch + ".attention.layer_norm_rms_epsilon").c_str(), &eps))) return rc;
    // absent head_count_kv: the reference ends up with a zero-sized KV cache (abstract_model.h:89,96-97); ggml's rule (= head_count) is used here
    heads_kv = heads;
    if (g->kv.count(arch + ".attention.head_count_kv") && (rc = spy_gguf_get_u32(g, (arch + ".attention.head_count_kv").c_str(), &heads_kv))) return rc;
    if (g->kv.count(arch + ".rope.freq_base") && (rc = spy_gguf_get_f32(g, (arch + ".rope.freq_base").c_str(), &freq_base))) return rc;
    if (g->kv.count(arch + ".rope.dimension_count")) {
        uint32_t rd = 0;
        if ((rc = spy_gguf_get_u32(g, (arch + ".rope.dimension_count").c_str(), &rd))) return rc;
        if (rd != 128) return fail(SPY_GGUF_EUNSUPPORTED, "rope.dimension_count %u (llama.h:60-61 of the reference requires 128)", rd);
    }
    if (!g->kv.count("tokenizer.ggml.tokens")) return fail(SPY_GGUF_EKEY, "key tokenizer.ggml.tokens is absent");
    uint64_t n_vocab = g->kv.at("tokenizer.ggml.tokens").n;
    if (g->kv.count(arch + ".vocab_size")) {
        uint32_t v = 0;
        if ((rc = spy_gguf_get_u32(g, (arch + ".vocab_size").c_str(), &v))) return rc;
        n_vocab = v;
    }
    if (heads == 0 || d % heads != 0 || d / heads != 128) return fail(SPY_GGUF_EUNSUPPORTED, "embedding %u over %u heads: this backend runs 128-wide heads", d, heads);
    if (heads_kv != heads) return fail(SPY_GGUF_EUNSUPPORTED, "grouped-query attention (head_count_kv %u of %u heads) is not built", heads_kv, heads);
    if (n_ctx <= 0) n_ctx = (int32_t)ctx;
    n_ctx = (n_ctx + 7) & ~7;

    spy_hip_llama_desc &D = m->desc;
    D.n_layer = (int32_t)blocks; D.n_embd = (int32_t)d; D.n_head = (int32_t)heads; D.n_ff = (int32_t)ff; D.n_vocab = (int32_t)n_vocab; D.n_ctx = n_ctx;
    D.eps = eps; D.rope_freq_base = freq_base;
    const void *p = nullptr;
    if ((rc = upload(m, "token_embd.weight", d, (int64_t)n_vocab, false, true, &D.tok_embd, &D.t_tok_embd))) return rc;
    if ((rc = upload(m, "output_norm.weight", d, 1, false, false, &p, nullptr))) return rc;
    D.out_norm = (const float *)p;
    if ((rc = upload(m, "output.weight", d, (int64_t)n_vocab, true, false, &D.w_out, &D.t_out))) return rc;
    m->layers.resize(blocks);
    for (uint32_t i = 0; i < blocks; i++) {
        spy_hip_llama_layer &L = m->layers[i];
        memset(&L, 0, sizeof(L));
        const std::string b = "blk." + std::to_string(i) + ".";
        if ((rc = upload(m, b + "attn_norm.weight", d, 1, false, false, &p, nullptr))) return rc;
        L.attn_norm = (const float *)p;
        if ((rc = upload(m, b + "ffn_norm.weight", d, 1, false, false, &p, nullptr))) return rc;
        L.ffn_norm = (const float *)p;
        if ((rc = upload(m, b + "attn_q.weight", d, d, true, false, &L.wq, &L.t_wq))) return rc;
        if ((rc = upload(m, b + "attn_k.weight", d, d, true, false, &L.wk, &L.t_wk))) return rc;
        if ((rc = upload(m, b + "attn_v.weight", d, d, true, false, &L.wv, &L.t_wv))) return rc;
        if ((rc = upload(m, b + "attn_output.weight", d, d, true, false, &L.wo, &L.t_wo))) return rc;
        if ((rc = upload(m, b + "ffn_gate.weight", d, ff, true, false, &L.w_gate, &L.t_gate))) return rc;
        if ((rc = upload(m, b + "ffn_up.weight", d, ff, true, false, &L.w_up, &L.t_up))) return rc;
        if ((rc = upload(m, b + "ffn_down.weight", ff, d, true, false, &L.w_down, &L.t_down))) return rc;
    }
    D.wtype = blocks ? m->layers[0].t_wq : D.t_out;       // main type: the per-tensor fields carry the rest
    D.layers = m->layers.data();
    return 0;
}

}  // namespace

extern "C" int spy_gguf_model_load(const char *path, int32_t n_ctx, spy_gguf_model **out) {
    if (!path || !out || n_ctx < 0) return fail(SPY_GGUF_EINVAL, "bad argument");
    *out = nullptr;
    spy_gguf_model *m = new spy_gguf_model;
    auto t0 = std::chrono::steady_clock::now();
    int rc = spy_gguf_open(path, &m->file);
    m->parse_ms = ms_since(t0);
    if (!rc) {
        t0 = std::chrono::steady_clock::now();
        rc = build(m, n_ctx);
        if (!rc && (rc = spy_hip_sync(nullptr))) fail(rc, "upload failed: %s", spy_hip_error_string(rc));
        m->upload_ms = ms_since(t0);
    }
    if (!rc) {
        t0 = std::chrono::steady_clock::now();
        rc = spy_hip_llama_create(&m->desc, &m->engine);
        if (rc) fail(rc > 0 ? rc : SPY_GGUF_EUNSUPPORTED, "spy_hip_llama_create failed: %s", spy_hip_error_string(rc));
        m->create_ms = ms_since(t0);
    }
    if (rc) { spy_gguf_model_free(m); return rc; }
    *out = m;
    return 0;
}

extern "C" spy_hip_llama *spy_gguf_model_engine(spy_gguf_model *m) { return m ? m->engine : nullptr; }
extern "C" const spy_gguf *spy_gguf_model_file(const spy_gguf_model *m) { return m ? m->file : nullptr; }

extern "C" int spy_gguf_model_info(const spy_gguf_model *m, spy_hip_llama_desc *desc, uint64_t *weight_bytes, double *parse_ms, double *upload_ms,
                                   double *create_ms) {
    if (!m) return fail(SPY_GGUF_EINVAL, "null argument");
    if (desc) *desc = m->desc;
    if (weight_bytes) *weight_bytes = m->weight_bytes;
    if (parse_ms) *parse_ms = m->parse_ms;
    if (upload_ms) *upload_ms = m->upload_ms;
    if (create_ms) *create_ms = m->create_ms;
    return 0;
}

extern "C" void spy_gguf_model_free(spy_gguf_model *m) {
    if (!m) return;
    if (m->engine) spy_hip_llama_destroy(m->engine);
    for (void *p : m->device) spy_hip_free(p);
    spy_gguf_close(m->file);
    delete m;
}
