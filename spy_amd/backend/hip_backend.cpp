// See hip_backend.h.  Operator dispatch mirrors CPUBackend::get_execute_func
// (backend/host/backend/cpu_backend.cpp:71-94 in the Spy tree): one case per OperatorType, each
// forwarding the node's tensors to the matching spy_hip_op_* entry point.
#include "hip_backend.h"

#include <cstring>

#include <rocprofiler-sdk-roctx/roctx.h>

#include "../../include/spy_hip.h"

namespace spy::hip {

// Name of the marker range around one operator: "hip-<Op>", the counterpart of the "cpu-<Op>" ranges the host
// backend opens around every operator (backend/host/include/operator_impl.h:57-63).
static const char *range_name(OperatorType t) {
    switch (t) {
    case OperatorType::Input: return "hip-Input";
    case OperatorType::Nop: return "hip-Nop";
    case OperatorType::Dup: return "hip-Dup";
    case OperatorType::Copy: return "hip-Copy";
    case OperatorType::View: return "hip-View";
    case OperatorType::Reshape: return "hip-Reshape";
    case OperatorType::MaskedCopy: return "hip-MaskedCopy";
    case OperatorType::MaskedSelect: return "hip-MaskedSelect";
    case OperatorType::GetRow: return "hip-GetRow";
    case OperatorType::Transpose: return "hip-Transpose";
    case OperatorType::Permute: return "hip-Permute";
    case OperatorType::Contiguous: return "hip-Contiguous";
    case OperatorType::Relu: return "hip-Relu";
    case OperatorType::Silu: return "hip-Silu";
    case OperatorType::Gelu: return "hip-Gelu";
    case OperatorType::Max: return "hip-Max";
    case OperatorType::Min: return "hip-Min";
    case OperatorType::Softmax: return "hip-Softmax";
    case OperatorType::Add: return "hip-Add";
    case OperatorType::Sub: return "hip-Sub";
    case OperatorType::Mul: return "hip-Mul";
    case OperatorType::Div: return "hip-Div";
    case OperatorType::Mod: return "hip-Mod";
    case OperatorType::MatMul: return "hip-MatMul";
    case OperatorType::Sum: return "hip-Sum";
    case OperatorType::Norm: return "hip-Norm";
    case OperatorType::NormRMS: return "hip-NormRMS";
    case OperatorType::Rope: return "hip-Rope";
    case OperatorType::Quantize: return "hip-Quantize";
    }
    return "hip-Unknown";
}

namespace {
struct MarkerRange {                    // closed on every return path of run()
    explicit MarkerRange(const char *name) { roctxRangePushA(name); }
    ~MarkerRange() { roctxRangePop(); }
    MarkerRange(const MarkerRange &) = delete;
    MarkerRange &operator=(const MarkerRange &) = delete;
};
}  // namespace

static spy_hip_tensor flat(const Tensor &t, const void *data) {
    spy_hip_tensor o;
    o.type = static_cast<int32_t>(t.shape.number_type);
    o.dim = static_cast<int32_t>(t.shape.dim);
    for (int i = 0; i < 4; ++i) { o.ne[i] = t.shape.elements[i]; o.nb[i] = t.shape.bytes[i]; }
    o.data = const_cast<void *>(data);
    return o;
}

HIPBackend::HIPBackend(const BackendFactory::BackendConfiguration &config) : Backend(BackendType::Device) {
    device_id_ = config.parse_or("device_id", 0);           // same key as the CUDA stub (backend/cuda/include/default_backend.h:38-40)
    last_error_ = spy_hip_init(device_id_);
    if (last_error_ == 0) last_error_ = spy_hip_stream_create(&stream_);
    if (last_error_ != 0) last_status_ = OperatorStatus::Fail;
}

HIPBackend::~HIPBackend() noexcept {
    spy_hip_sync(nullptr);
    for (auto &kv : pool_) for (void *p : kv.second) spy_hip_free(p);
    for (auto &kv : constants_) spy_hip_free(kv.second);
    for (auto &kv : io_) spy_hip_free(kv.second.dev);
    if (stream_) spy_hip_stream_destroy(stream_);
}

size_t HIPBackend::get_max_memory_capacity() const {
    size_t total = 0;
    spy_hip_device_info(nullptr, 0, nullptr, &total, nullptr);
    return total;
}

size_t HIPBackend::get_avail_memory_capacity() const {
    size_t free_mem = 0;
    spy_hip_device_info(nullptr, 0, nullptr, nullptr, &free_mem);
    return free_mem;
}

static size_t bucket(size_t size) {                           // next power of two, at least 256 bytes
    size_t b = 256;
    while (b < size) b <<= 1;
    return b;
}

void *HIPBackend::alloc_memory(size_t size) {
    std::lock_guard<std::mutex> lock(mutex_);
    const size_t b = bucket(size);
    auto &free_list = pool_[b];
    void *p = nullptr;
    if (!free_list.empty()) { p = free_list.back(); free_list.pop_back(); }
    else if (spy_hip_alloc(&p, b) != 0) return nullptr;
    bucket_of_[p] = b;
    return p;
}

void HIPBackend::dealloc_memory(void *ptr, size_t) {
    if (!ptr) return;
    std::lock_guard<std::mutex> lock(mutex_);
    const auto it = bucket_of_.find(ptr);
    if (it == bucket_of_.end()) return;                        // not ours: undefined in the interface, ignored here
    pool_[it->second].push_back(ptr);
}

bool HIPBackend::is_support(OperatorType t) const {
    switch (t) {
    case OperatorType::Nop: case OperatorType::Dup: case OperatorType::Copy: case OperatorType::View: case OperatorType::Reshape:
    case OperatorType::GetRow: case OperatorType::Transpose: case OperatorType::Permute: case OperatorType::Contiguous:
    case OperatorType::Silu: case OperatorType::Softmax: case OperatorType::Add: case OperatorType::Sub: case OperatorType::Mul:
    case OperatorType::Div: case OperatorType::MatMul: case OperatorType::NormRMS: case OperatorType::Rope:
    case OperatorType::Relu: case OperatorType::Quantize:
        return true;
    default:
        return false;
    }
}

void HIPBackend::sync() { spy_hip_sync(stream_); }

// Device address of a node's data.  Dynamic / Cache tensors already hold device pointers (they
// were handed out by alloc_memory and view arithmetic keeps them on the device).
const void *HIPBackend::device_view(DataNode *node, bool is_output) {
    Tensor &t = node->tensor;
    const DataNodeType nt = node->node_prop.node_type;
    if (nt == DataNodeType::Constant) {
        const auto it = constants_.find(t.data_ptr);
        if (it != constants_.end()) return it->second;
        void *dev = nullptr;
        const size_t bytes = static_cast<size_t>(t.total_size());
        if (spy_hip_alloc(&dev, bytes) != 0 || spy_hip_upload(dev, t.data_ptr, bytes, stream_) != 0) return nullptr;
        constants_[t.data_ptr] = dev;
        return dev;
    }
    if (nt == DataNodeType::IO) {
        Staged &s = io_[node];
        const size_t bytes = static_cast<size_t>(t.total_size());
        if (s.bytes < bytes) {
            if (s.dev) { spy_hip_sync(stream_); spy_hip_free(s.dev); }
            s.dev = nullptr; s.bytes = 0; s.uploaded_valid = false;
            if (spy_hip_alloc(&s.dev, bytes) != 0) return nullptr;
            s.bytes = bytes;
        }
        if (is_output) { s.uploaded_valid = false; return s.dev; }                                   // the device copy is about to change
        // host vectors change from pass to pass, not within one: a tensor of up to 8 MiB whose bytes are those of the last upload stays
        constexpr size_t kCompareLimit = 8u << 20;                                                   // the mask of a 1024-token prompt is 4 MiB: comparing costs a third of uploading
        if (bytes <= kCompareLimit && s.uploaded_valid && s.uploaded.size() == bytes && std::memcmp(s.uploaded.data(), t.data_ptr, bytes) == 0) return s.dev;
        if (spy_hip_upload(s.dev, t.data_ptr, bytes, stream_) != 0) return nullptr;
        s.uploaded_valid = bytes <= kCompareLimit;
        if (s.uploaded_valid) s.uploaded.assign(static_cast<const uint8_t *>(t.data_ptr), static_cast<const uint8_t *>(t.data_ptr) + bytes);
        return s.dev;
    }
    return t.data_ptr;
}

OperatorStatus HIPBackend::run(OperatorNode *op) {
    const OperatorType type = op->op_type;
    const MarkerRange range(range_name(type));
    // zero-copy operators only move the data pointer (view.cpp:219-276): no launch
    switch (type) {
    case OperatorType::Nop: return OperatorStatus::Success;
    case OperatorType::Reshape: case OperatorType::Transpose: case OperatorType::Permute:
        op->output_data(0)->tensor.set_data_ptr(op->input_data(0)->tensor.get());
        return OperatorStatus::Success;
    case OperatorType::View: {
        const int64_t offset = static_cast<OperatorDefinition<OperatorType::View> *>(op)->params.get_val().offset;
        op->output_data(0)->tensor.set_data_ptr(op->input_data(0)->tensor.get<uint8_t>() + offset);
        return OperatorStatus::Success;
    }
    default: break;
    }
    if (!is_support(type)) return OperatorStatus::Unsupport;

    spy_hip_tensor in[3];
    const size_t nin = op->num_input();
    if (nin > 3 || op->num_output() < 1) return OperatorStatus::Fail;
    for (size_t i = 0; i < nin; ++i) {
        DataNode *n = op->input_data(i);
        // Copy writes INTO its second operand (view.cpp:219-227): that one is an output for staging purposes
        const void *p = device_view(n, type == OperatorType::Copy && i == 1);
        if (!p) return OperatorStatus::Fail;
        in[i] = flat(n->tensor, p);
    }
    DataNode *out_node = op->output_data(0);
    const bool out_io = out_node->node_prop.node_type == DataNodeType::IO;
    spy_hip_tensor out;
    if (type != OperatorType::Copy) {
        const void *p = device_view(out_node, true);
        if (!p) return OperatorStatus::Fail;
        out = flat(out_node->tensor, p);
    }

    int rc = 0;
    switch (type) {
    case OperatorType::MatMul: {
        const size_t need = spy_hip_op_matmul_scratch_size(&in[0], &in[1]);
        void *scratch = need ? alloc_memory(need) : nullptr;
        if (need && !scratch) return OperatorStatus::Fail;
        rc = spy_hip_op_matmul(stream_, &in[0], &in[1], &out, scratch, need);
        if (scratch) dealloc_memory(scratch, need);              // stream order keeps it alive until the kernels are done
        break;
    }
    case OperatorType::NormRMS:
        rc = spy_hip_op_norm_rms(stream_, &in[0], &out, static_cast<OperatorDefinition<OperatorType::NormRMS> *>(op)->params.get_val().eps);
        break;
    case OperatorType::Add: rc = spy_hip_op_binary(stream_, 0, &in[0], &in[1], &out); break;
    case OperatorType::Sub: rc = spy_hip_op_binary(stream_, 1, &in[0], &in[1], &out); break;
    case OperatorType::Mul: rc = spy_hip_op_binary(stream_, 2, &in[0], &in[1], &out); break;
    case OperatorType::Div: rc = spy_hip_op_binary(stream_, 3, &in[0], &in[1], &out); break;
    case OperatorType::Silu: rc = spy_hip_op_silu(stream_, &in[0], &out); break;
    case OperatorType::Relu: rc = spy_hip_op_relu(stream_, &in[0], &out); break;
    case OperatorType::Quantize: rc = spy_hip_op_quantize(stream_, &in[0], &out); break;
    case OperatorType::Softmax:
        rc = spy_hip_op_softmax(stream_, &in[0], nin > 1 ? &in[1] : nullptr, &out,
                                static_cast<OperatorDefinition<OperatorType::Softmax> *>(op)->params.get_val().scale);
        break;
    case OperatorType::Rope: {
        const RopeParam &p = static_cast<OperatorDefinition<OperatorType::Rope> *>(op)->params.get_val();
        spy_hip_rope_param hp;
        hp.mode = static_cast<int32_t>(p.mode); hp.num_past = p.num_past; hp.num_dim = p.num_dim; hp.num_context = p.num_context;
        hp.num_origin_context = p.num_origin_context; hp.freq_base = p.freq_base; hp.freq_scale = p.freq_scale;
        hp.extend_factor = p.extend_factor; hp.attention_factor = p.attention_factor; hp.beta_fast = p.beta_fast; hp.beta_slow = p.beta_slow;
        hp.xpos_base = p.xpos_base; hp.xpos_down = p.xpos_down ? 1 : 0;
        rc = spy_hip_op_rope(stream_, &in[0], &in[1], &out, &hp);
        break;
    }
    case OperatorType::Dup: rc = spy_hip_op_dup(stream_, &in[0], &out); break;
    case OperatorType::Copy:
        rc = spy_hip_op_dup(stream_, &in[0], &in[1]);
        if (rc == 0) out_node->tensor.set_data_ptr(op->input_data(1)->tensor.get());     // view.cpp:224-226
        break;
    case OperatorType::Contiguous: rc = spy_hip_op_contiguous(stream_, &in[0], &out); break;
    case OperatorType::GetRow: rc = spy_hip_op_get_row(stream_, &in[0], &in[1], &out); break;
    default: return OperatorStatus::Unsupport;
    }
    if (rc == SPY_HIP_EUNSUPPORTED) return OperatorStatus::Unsupport;
    if (rc != 0) { last_error_ = rc; return OperatorStatus::Fail; }
    if (out_io && type != OperatorType::Copy) {                  // e.g. the logits: host-visible before the callback
        rc = spy_hip_download(out_node->tensor.data_ptr, out.data, static_cast<size_t>(out_node->tensor.total_size()), stream_);
        if (rc != 0) { last_error_ = rc; return OperatorStatus::Fail; }
        // the pass's device-side error flag (a GetRow index outside its table: the reference asserts, view.cpp:61)
        int flag = 0;
        rc = spy_hip_take_error(&flag);
        if (rc != 0 || flag != 0) { last_error_ = rc != 0 ? rc : SPY_HIP_EINVAL; return OperatorStatus::Fail; }
    }
    return OperatorStatus::Success;
}

void HIPBackend::submit(OperatorNode *op_node_ptr, std::function<void()> &&callback) {
    {
        // one operator at a time: run() touches the constant and staging maps and the one stream.  The callback runs
        // outside the lock (it frees inputs through dealloc_memory and may submit successors).
        std::lock_guard<std::mutex> lock(submit_mutex_);
        const OperatorStatus st = run(op_node_ptr);
        if (st != OperatorStatus::Success) last_status_ = st;    // the CPU backend asserts here (default_backend.h:175-176)
    }
    if (callback) callback();
}

static std::unique_ptr<Backend> make_default(const BackendFactory::BackendConfiguration &config) { return std::make_unique<HIPBackend>(config); }

void init_backend(BackendFactory &factory) { factory.add_backend_map(BackendFactory::make_backend_name("hip", "default"), make_default); }

}  // namespace spy::hip
