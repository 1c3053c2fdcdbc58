// A minimal driver for backend/hip: the LLaMA compute graph the reference builds
// (model/src/llm/model/llama.cpp:86-313, model/src/llm/plugin/{attention,ffn,inout}.cpp in the Spy
// tree), executed with the greedy scheduler's discipline (backend/distributor/include/scheduler/
// default_scheduler.h:46-229: constants fetched by name, outputs allocated through the backend before
// submit, inputs released from the completion callback) against any spy::Backend.  It exists so
// that the backend can be exercised through the reference's own operator API; it is not a
// re-implementation of Spy's model / orchestration / storage layers.
#include <cmath>
#include <cstring>
#include <deque>
#include <limits>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "hip_backend.h"
#include "../../include/spy_hip.h"

namespace spy {

// ---- shape propagation of the operator definitions (operator/*.h, propagate()) --------------------
static void same_as_input(OperatorNode *op) {
    DataNode *o = op->output_data(0);
    o->view_src = nullptr;
    o->tensor.shape = op->input_data(0)->tensor.shape;
}
void OperatorDefinition<OperatorType::Input>::propagate() {}
void OperatorDefinition<OperatorType::Nop>::propagate() { same_as_input(this); output_data(0)->view_src = input_data(0); }
void OperatorDefinition<OperatorType::Dup>::propagate() { same_as_input(this); }
void OperatorDefinition<OperatorType::Silu>::propagate() { same_as_input(this); }
void OperatorDefinition<OperatorType::Relu>::propagate() { same_as_input(this); }
void OperatorDefinition<OperatorType::Quantize>::propagate() {                      // operator/quantize.h: the operand's elements in the target type
    const Shape &s = input_data(0)->tensor.shape;
    DataNode *o = output_data(0);
    o->view_src = nullptr;
    o->tensor.shape = Shape({s.elements[0], s.elements[1], s.elements[2], s.elements[3]}, params.get_val().target_type);
    o->tensor.shape.dim = s.dim;
}
void OperatorDefinition<OperatorType::Softmax>::propagate() { same_as_input(this); }
void OperatorDefinition<OperatorType::NormRMS>::propagate() { same_as_input(this); }
void OperatorDefinition<OperatorType::Rope>::propagate() { same_as_input(this); }
void OperatorDefinition<OperatorType::Add>::propagate() { same_as_input(this); }
void OperatorDefinition<OperatorType::Sub>::propagate() { same_as_input(this); }
void OperatorDefinition<OperatorType::Mul>::propagate() { same_as_input(this); }
void OperatorDefinition<OperatorType::Div>::propagate() { same_as_input(this); }
void OperatorDefinition<OperatorType::Copy>::propagate() { same_as_input(this); output_data(0)->view_src = input_data(0); }   // view.h (Copy): out = src shape
void OperatorDefinition<OperatorType::MatMul>::propagate() {                        // operator/mat.h:46-66
    const Shape &a = input_data(0)->tensor.shape, &b = input_data(1)->tensor.shape;
    DataNode *o = output_data(0);
    o->view_src = nullptr;
    o->tensor.shape = Shape({a.elements[1], b.elements[1], b.elements[2], b.elements[3]}, NumberType::FP32);
}
void OperatorDefinition<OperatorType::GetRow>::propagate() {                        // operator/view.h (GetRow)
    const Shape &t = input_data(0)->tensor.shape, &ids = input_data(1)->tensor.shape;
    DataNode *o = output_data(0);
    o->view_src = nullptr;
    o->tensor.shape = Shape({t.elements[0], ids.elements[0]}, NumberType::FP32);
}
void OperatorDefinition<OperatorType::Contiguous>::propagate() {
    const Shape &s = input_data(0)->tensor.shape;
    DataNode *o = output_data(0);
    o->view_src = nullptr;
    o->tensor.shape = Shape({s.elements[0], s.elements[1], s.elements[2], s.elements[3]}, s.number_type);
    o->tensor.shape.dim = s.dim;
}
void OperatorDefinition<OperatorType::Reshape>::propagate() { output_data(0)->view_src = input_data(0); output_data(0)->tensor.shape = params.get_val().new_shape; }
void OperatorDefinition<OperatorType::View>::propagate() { output_data(0)->view_src = input_data(0); output_data(0)->tensor.shape = params.get_val().new_shape; }
void OperatorDefinition<OperatorType::Transpose>::propagate() {
    Shape s = input_data(0)->tensor.shape;
    std::swap(s.elements[0], s.elements[1]);
    std::swap(s.bytes[0], s.bytes[1]);
    output_data(0)->view_src = nullptr;
    output_data(0)->tensor.shape = s;
}
void OperatorDefinition<OperatorType::Permute>::propagate() {
    const Shape &in = input_data(0)->tensor.shape;
    Shape s = in;
    const auto &axis = params.get_val().axis;
    for (uint32_t i = 0; i < MAX_DIM; ++i) { s.elements[i] = in.elements[axis[i]]; s.bytes[i] = in.bytes[axis[i]]; }
    s.dim = 4;
    output_data(0)->view_src = nullptr;
    output_data(0)->tensor.shape = s;
}

}  // namespace spy

using namespace spy;

namespace {

struct HostTensor { const void *data; NumberType type; int64_t rows, cols; };

struct Model {
    int n_layer, n_embd, n_head, n_ff, n_vocab, n_ctx;
    float eps, rope_freq_base;
    std::unordered_map<std::string, HostTensor> loader;              // ModelLoader::load(name) (loader.h:11-38)
    std::unique_ptr<Backend> backend;
    std::vector<void *> k_cache, v_cache;                            // Cache nodes: allocated once through the backend
    // one pass
    std::deque<DataNode> data;
    std::vector<std::unique_ptr<OperatorNode>> ops;
    std::unordered_map<const DataNode *, int> pending;                // consumers still to run (GraphControlHeader::data_output)
    std::vector<float> kq_mask;
    std::vector<int32_t> ids, pos;
    std::vector<float> logits;
    int64_t n_submit = 0, n_alloc = 0, n_free = 0;
};

DataNode *new_data(Model &m, const std::string &name, DataNodeType type, int layer) {
    m.data.emplace_back();
    DataNode *n = &m.data.back();
    n->name = name; n->node_prop.node_type = type; n->node_prop.layer_id = layer; n->id = (uint32_t)m.data.size() - 1;
    return n;
}

DataNode *constant(Model &m, const std::string &name, int layer) {
    const HostTensor &t = m.loader.at(name);
    DataNode *n = new_data(m, name, DataNodeType::Constant, layer);
    n->tensor.shape = t.rows > 1 ? Shape({t.cols, t.rows}, t.type) : Shape({t.cols}, t.type);
    return n;
}

template <OperatorType OP, class... Args>
DataNode *emit(Model &m, const std::string &name, DataNodeProperty prop, std::initializer_list<DataNode *> inputs, Args &&...args) {
    auto op = std::make_unique<OperatorDefinition<OP>>(std::forward<Args>(args)...);
    op->name = name;
    for (DataNode *in : inputs) op->add_input(in);
    DataNode *out = new_data(m, name + "-out", prop.node_type, prop.layer_id);
    op->add_output(out);
    op->propagate();
    m.ops.push_back(std::move(op));
    return out;
}

// LLAMAModel::build_graph for T new tokens after P cached ones
DataNode *build(Model &m, int T, int P) {
    const int64_t d = m.n_embd, H = m.n_head, hd = d / H, C = m.n_ctx, n_kv = (int64_t)P + T;
    m.data.clear(); m.ops.clear(); m.pending.clear();
    const DataNodeProperty io{DataNodeType::IO, -1, -1};
    DataNode *ids = new_data(m, "input_token_id", DataNodeType::IO, -1);
    ids->tensor = Tensor(Shape({T}, NumberType::INT32), m.ids.data());
    DataNode *pos = new_data(m, "input_position", DataNodeType::IO, -1);
    pos->tensor = Tensor(Shape({T}, NumberType::INT32), m.pos.data());
    DataNode *mask = new_data(m, "KQ_mask", DataNodeType::IO, -1);
    mask->tensor = Tensor(Shape({C, T}, NumberType::INT32), m.kq_mask.data());       // typed INT32, read as float (inout.cpp:43-47)

    DataNodeProperty dyn{DataNodeType::Dynamic, -1, -1};
    DataNode *x = emit<OperatorType::GetRow>(m, "input_embedding", dyn, {constant(m, "token_embd.weight", -1), ids});
    const RopeParam rope{RopeType::Norm, P, (int32_t)hd, (int32_t)C, (int32_t)C, m.rope_freq_base, 1.0f, 0.0f, 1.0f, 32.0f, 1.0f, 0.0f, false};
    for (int il = 0; il < m.n_layer; ++il) {
        dyn.layer_id = il;
        const std::string p = "blk." + std::to_string(il) + ".";
        DataNode *n1 = emit<OperatorType::NormRMS>(m, "attn_norm", dyn, {x}, NormRMSParam{m.eps});
        DataNode *xn = emit<OperatorType::Mul>(m, "attn_norm_linear", dyn, {n1, constant(m, p + "attn_norm.weight", il)});
        DataNode *q = emit<OperatorType::MatMul>(m, "Q_project", dyn, {constant(m, p + "attn_q.weight", il), xn});
        DataNode *k = emit<OperatorType::MatMul>(m, "K_project", dyn, {constant(m, p + "attn_k.weight", il), xn});
        DataNode *v = emit<OperatorType::MatMul>(m, "V_project", dyn, {constant(m, p + "attn_v.weight", il), xn});
        DataNode *q3 = emit<OperatorType::Reshape>(m, "Q_project", dyn, {q}, ReshapeParam{Shape({hd, H, T}, NumberType::FP32)});
        DataNode *k3 = emit<OperatorType::Reshape>(m, "K_project", dyn, {k}, ReshapeParam{Shape({hd, H, T}, NumberType::FP32)});
        DataNode *qr = emit<OperatorType::Rope>(m, "Q_rope", dyn, {q3, pos}, rope);
        DataNode *kr = emit<OperatorType::Rope>(m, "K_rope", dyn, {k3, pos}, rope);
        DataNode *qo = emit<OperatorType::Permute>(m, "Q_out", dyn, {qr}, PermuteParam{{0, 2, 1, 3}});
        DataNode *vt = emit<OperatorType::Transpose>(m, "V_t", dyn, {v});
        // KV cache (attention.cpp:180-265)
        DataNode *kc = new_data(m, "KCache", DataNodeType::Cache, il);
        kc->tensor = Tensor(Shape({d * C}, NumberType::FP16), m.k_cache[il]);
        DataNode *vc = new_data(m, "VCache", DataNodeType::Cache, il);
        vc->tensor = Tensor(Shape({d * C}, NumberType::FP16), m.v_cache[il]);
        const int64_t k_off = get_row_size(NumberType::FP16, d) * P, v_off = get_type_size(NumberType::FP16) * P;
        DataNode *kview = emit<OperatorType::View>(m, "KCache_view", dyn, {kc}, ViewParam{k_off, Shape({T * d}, {2}, NumberType::FP16)});
        DataNode *ksync = emit<OperatorType::Copy>(m, "KCache_cpy", dyn, {kr, kview});
        DataNode *kall = emit<OperatorType::View>(m, "KCache_total", dyn, {ksync}, ViewParam{-k_off, Shape({hd, n_kv, H}, {2, 2 * d, 2 * hd}, NumberType::FP16)});
        DataNode *vview = emit<OperatorType::View>(m, "VCache_view", dyn, {vc}, ViewParam{v_off, Shape({T, d}, {2, 2 * C}, NumberType::FP16)});
        DataNode *vsync = emit<OperatorType::Copy>(m, "VCache_cpy", dyn, {vt, vview});
        DataNode *vall = emit<OperatorType::View>(m, "VCache_total", dyn, {vsync}, ViewParam{-v_off, Shape({n_kv, hd, H}, {2, 2 * C, 2 * C * hd}, NumberType::FP16)});
        // attention_projection (attention.cpp:104-144)
        DataNode *s = emit<OperatorType::MatMul>(m, "attn_score", dyn, {kall, qo});
        DataNode *pr = emit<OperatorType::Softmax>(m, "attn_score_softmax", dyn, {s, mask}, SoftmaxParam{1.0f / std::sqrt((float)hd)});
        DataNode *kqv = emit<OperatorType::MatMul>(m, "KQV", dyn, {vall, pr});
        DataNode *kqv_p = emit<OperatorType::Permute>(m, "KQV", dyn, {kqv}, PermuteParam{{0, 2, 1, 3}});
        DataNode *kqv_c = emit<OperatorType::Contiguous>(m, "KQV", dyn, {kqv_p});
        DataNode *kqv_r = emit<OperatorType::Reshape>(m, "KQV", dyn, {kqv_c}, ReshapeParam{Shape({d, T}, NumberType::FP32)});
        DataNode *attn = emit<OperatorType::MatMul>(m, "KQV_linear", dyn, {constant(m, p + "attn_output.weight", il), kqv_r});
        DataNode *ffn_inp = emit<OperatorType::Add>(m, "ffn_input", dyn, {attn, x});
        // FFN (ffn.cpp:5-42)
        DataNode *n2 = emit<OperatorType::NormRMS>(m, "ffn_norm", dyn, {ffn_inp}, NormRMSParam{m.eps});
        DataNode *xn2 = emit<OperatorType::Mul>(m, "ffn_norm_linear", dyn, {n2, constant(m, p + "ffn_norm.weight", il)});
        DataNode *up = emit<OperatorType::MatMul>(m, "ffn_up", dyn, {constant(m, p + "ffn_up.weight", il), xn2});
        DataNode *gate = emit<OperatorType::MatMul>(m, "ffn_gate", dyn, {constant(m, p + "ffn_gate.weight", il), xn2});
        DataNode *act = emit<OperatorType::Silu>(m, "ffn_gate_activate", dyn, {gate});
        DataNode *par = emit<OperatorType::Mul>(m, "ffn_par", dyn, {up, act});
        DataNode *down = emit<OperatorType::MatMul>(m, "ffn_down", dyn, {constant(m, p + "ffn_down.weight", il), par});
        x = emit<OperatorType::Add>(m, "logit_output", dyn, {ffn_inp, down});
    }
    dyn.layer_id = -1;
    DataNode *rn = emit<OperatorType::NormRMS>(m, "result_norm", dyn, {x}, NormRMSParam{m.eps});
    DataNode *rw = emit<OperatorType::Mul>(m, "result_linear", dyn, {rn, constant(m, "output_norm.weight", -1)});
    DataNode *out = emit<OperatorType::MatMul>(m, "output", io, {constant(m, "output.weight", -1), rw});
    m.logits.resize((size_t)out->tensor.total_element());
    out->tensor.set_data_ptr(m.logits.data());
    return out;
}

// DefaultGraphScheduler::execute, sequentially in topological (= construction) order
int execute(Model &m) {
    Backend *be = m.backend.get();
    for (DataNode &n : m.data) m.pending[&n] = (int)n.num_output();
    for (auto &op_ptr : m.ops) {
        OperatorNode *op = op_ptr.get();
        if (!be->is_support(op->op_type)) return -1;
        for (size_t i = 0; i < op->num_input(); ++i) {               // try_fetch_inputs (default_scheduler.h:141-165)
            DataNode *n = op->input_data(i);
            if (n->node_prop.node_type == DataNodeType::Constant) n->tensor.set_data_ptr(const_cast<void *>(m.loader.at(n->name).data));
        }
        DataNode *out = op->output_data(0);
        if (!is_view(op->op_type)) {                                  // try_allocate_outputs (:167-184)
            if (out->tensor.get() == nullptr) { out->tensor.set_data_ptr(be->alloc_memory((size_t)out->tensor.total_size())); ++m.n_alloc; }
        } else {
            DataNode *in0 = op->input_data(0);
            DataNode *src = in0->view_src ? in0->view_src : in0;
            out->view_src = src;
            ++m.pending[src];
        }
        ++m.n_submit;
        be->submit(op, [&m, op, be]() {                               // try_deallocate_inputs (:186-228)
            for (size_t i = 0; i < op->num_input(); ++i) {
                DataNode *n = op->input_data(i);
                DataNode *owner = n->is_view() ? n->view_src : n;
                const DataNodeType t = owner->node_prop.node_type;
                const int left = --m.pending[owner];
                if (left == 0 && t == DataNodeType::Dynamic && owner->tensor.get() != nullptr) {
                    be->dealloc_memory(owner->tensor.get(), (size_t)owner->tensor.total_size());
                    owner->tensor.set_data_ptr(nullptr);
                    ++m.n_free;
                }
            }
        });
    }
    return 0;
}

}  // namespace

// ---- C ABI for the tests ------------------------------------------------------------------------------
extern "C" {

struct spy_host_tensor { const char *name; const void *data; int32_t type; int64_t rows, cols; };

struct spy_host_model { Model m; };

int spy_host_model_create(const spy_host_tensor *tensors, int n_tensors, int n_layer, int n_embd, int n_head, int n_ff, int n_vocab,
                          int n_ctx, float eps, float rope_freq_base, const char *backend_name, spy_host_model **out) {
    if (!tensors || !out || !backend_name) return -2;
    auto h = std::make_unique<spy_host_model>();
    Model &m = h->m;
    m.n_layer = n_layer; m.n_embd = n_embd; m.n_head = n_head; m.n_ff = n_ff; m.n_vocab = n_vocab; m.n_ctx = n_ctx;
    m.eps = eps; m.rope_freq_base = rope_freq_base;
    for (int i = 0; i < n_tensors; ++i)
        m.loader[tensors[i].name] = HostTensor{tensors[i].data, static_cast<NumberType>(tensors[i].type), tensors[i].rows, tensors[i].cols};
    BackendFactory factory;                                           // registers "hip:default" (backend.h:142-155)
    ConfigTable config;
    config.set("device_id", "0");
    m.backend = factory.init_backend(backend_name, config);
    if (!m.backend) return -1;
    const size_t cache_bytes = (size_t)n_ctx * n_embd * 2;
    for (int il = 0; il < n_layer; ++il) {                            // Cache nodes: backend memory, never freed (default_scheduler.h:157-163)
        m.k_cache.push_back(m.backend->alloc_memory(cache_bytes));
        m.v_cache.push_back(m.backend->alloc_memory(cache_bytes));
        if (!m.k_cache.back() || !m.v_cache.back()) return 2;
        spy_hip_fill_u8(m.k_cache.back(), 0, cache_bytes, nullptr);   // unwritten slots read as +0 (they are masked, but must not hold NaN bit patterns)
        spy_hip_fill_u8(m.v_cache.back(), 0, cache_bytes, nullptr);
    }
    spy_hip_sync(nullptr);
    *out = h.release();
    return 0;
}

int spy_host_model_forward(spy_host_model *h, const int32_t *tokens, int n_token, int n_past, float *logits) {
    if (!h || !tokens || n_token <= 0 || n_past < 0) return -2;
    Model &m = h->m;
    if ((int64_t)n_past + n_token > m.n_ctx) return -2;               // llama.cpp:249
    m.ids.assign(tokens, tokens + n_token);
    m.pos.resize(n_token);
    for (int i = 0; i < n_token; ++i) m.pos[i] = n_past + i;
    m.kq_mask.assign((size_t)n_token * m.n_ctx, -std::numeric_limits<float>::infinity());   // llama.cpp:248-257
    for (int64_t i = 0; i < n_token; ++i)
        for (int64_t j = 0; j <= i + n_past; ++j) m.kq_mask[(size_t)m.n_ctx * i + j] = 0.0f;
    build(m, n_token, n_past);
    const int rc = execute(m);
    if (rc) return rc;
    auto *hb = dynamic_cast<spy::hip::HIPBackend *>(m.backend.get());
    if (hb) {
        hb->sync();
        if (hb->last_status() != OperatorStatus::Success) return hb->last_status() == OperatorStatus::Unsupport ? -1 : (hb->last_error() ? hb->last_error() : 1);
    }
    if (logits) std::memcpy(logits, m.logits.data(), m.logits.size() * sizeof(float));
    return 0;
}

int spy_host_model_stats(spy_host_model *h, int64_t *n_ops, int64_t *n_submit, int64_t *n_alloc, int64_t *n_free) {
    if (!h) return -2;
    if (n_ops) *n_ops = (int64_t)h->m.ops.size();
    if (n_submit) *n_submit = h->m.n_submit;
    if (n_alloc) *n_alloc = h->m.n_alloc;
    if (n_free) *n_free = h->m.n_free;
    return 0;
}

int spy_host_model_cache(spy_host_model *h, int layer, int which, void *dst_host) {   // which: 0 K, 1 V
    if (!h || layer < 0 || layer >= h->m.n_layer || !dst_host) return -2;
    auto *hb = dynamic_cast<spy::hip::HIPBackend *>(h->m.backend.get());
    if (hb) hb->sync();
    return spy_hip_download(dst_host, which ? h->m.v_cache[layer] : h->m.k_cache[layer], (size_t)h->m.n_ctx * h->m.n_embd * 2, nullptr);
}

int spy_host_model_destroy(spy_host_model *h) { delete h; return 0; }

// One unary operator node through Backend::submit on host data: x = f32 [ne1][ne0] (IO node, uploaded by the backend), the
// result an IO node as well (host-visible when submit's callback has run).  op: 0 Relu, 1 Silu, 2 Quantize to target_type
// (NumberType code).  Returns 0, -1 unsupported by the backend, -2 bad arguments, else the backend's error.
int spy_host_unary_through_submit(const char *backend_name, int op, const float *x, int64_t ne0, int64_t ne1, int target_type, void *out, int64_t out_bytes) {
    if (!backend_name || !x || !out || ne0 <= 0 || ne1 <= 0) return -2;
    BackendFactory factory;
    ConfigTable config;
    config.set("device_id", "0");
    std::unique_ptr<Backend> be = factory.init_backend(backend_name, config);
    if (!be) return -1;
    DataNode in, res;
    in.name = "x"; in.node_prop.node_type = DataNodeType::IO; in.id = 0;
    in.tensor = Tensor(Shape({ne0, ne1}, NumberType::FP32), const_cast<float *>(x));
    res.name = "y"; res.node_prop.node_type = DataNodeType::IO; res.id = 1;
    std::unique_ptr<OperatorNode> node;
    if (op == 0) node = std::make_unique<OperatorDefinition<OperatorType::Relu>>();
    else if (op == 1) node = std::make_unique<OperatorDefinition<OperatorType::Silu>>();
    else if (op == 2) node = std::make_unique<OperatorDefinition<OperatorType::Quantize>>(QuantizeParam{static_cast<NumberType>(target_type)});
    else return -2;
    node->add_input(&in);
    node->add_output(&res);
    node->propagate();
    if ((int64_t)res.tensor.total_size() != out_bytes) return -2;
    res.tensor.set_data_ptr(out);
    if (!be->is_support(node->op_type)) return -1;
    bool called = false;
    be->submit(node.get(), [&called]() { called = true; });
    if (!called) return 1;
    auto *hb = dynamic_cast<spy::hip::HIPBackend *>(be.get());
    if (hb) {
        hb->sync();
        if (hb->last_status() != OperatorStatus::Success) return hb->last_status() == OperatorStatus::Unsupport ? -1 : (hb->last_error() ? hb->last_error() : 1);
    }
    return 0;
}

}  // extern "C"
