// backend/hip: the MI355X backend behind Spy's operator API.
// Counterpart of DefaultCPUBackend (backend/host/include/default_backend.h:106-200 in the Spy tree):
// same Backend interface, registered as "hip:default"; every operator goes to the gfx950 kernels
// through the C ABI of include/spy_hip.h on one in-order HIP stream.
#pragma once

#include <cstdint>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "spy/backend.h"

namespace spy::hip {

class HIPBackend final : public Backend {
public:
    explicit HIPBackend(const BackendFactory::BackendConfiguration &config);
    ~HIPBackend() noexcept override;

    size_t get_max_memory_capacity() const override;
    size_t get_avail_memory_capacity() const override;
    // Device memory.  Blocks come from a size-bucketed pool; because every kernel runs on the one
    // in-order stream a freed block may be handed out again at once (the scheduler frees inputs from
    // the completion callback, default_scheduler.h:186-228, while later kernels are still queued).
    void *alloc_memory(size_t size) override;
    void dealloc_memory(void *ptr, size_t size) override;
    size_t get_max_concurrency() const override { return 1; }
    size_t get_avail_concurrency() const override { return 1; }
    bool is_support(OperatorType op_type) const override;
    // Runs the operator and then the callback, exactly once.  Constant inputs arrive as host
    // pointers into the loader's mapping (default_scheduler.h:146-151) and are uploaded to HBM the
    // first time they are seen, in their native block layout; IO tensors (token ids, positions, KQ
    // mask, logits) are host vectors and are staged per pass; the callback of an operator whose output
    // is an IO node runs only after the result has reached the host.
    void submit(OperatorNode *op_node_ptr, std::function<void()> &&callback = nullptr) override;

    OperatorStatus last_status() const { return last_status_; }
    int last_error() const { return last_error_; }
    void sync();

private:
    const void *device_view(DataNode *node, bool is_output);
    OperatorStatus run(OperatorNode *op);

    int device_id_ = 0;
    void *stream_ = nullptr;
    std::mutex mutex_;                                            // the memory pool
    std::mutex submit_mutex_;                                     // run(): maps, staging buffers, stream order
    std::map<size_t, std::vector<void *>> pool_;                  // bucket size -> free blocks
    std::unordered_map<void *, size_t> bucket_of_;
    std::unordered_map<const void *, void *> constants_;          // host pointer -> device copy
    // device copy of an IO tensor, and (up to 8 MiB) the host bytes it was last uploaded from: the positions and the mask of a
    // pass are read by one operator per layer, and uploading them again for each costs more than comparing them
    struct Staged { void *dev = nullptr; size_t bytes = 0; std::vector<uint8_t> uploaded; bool uploaded_valid = false; };
    std::unordered_map<const DataNode *, Staged> io_;             // IO node -> staging buffer
    OperatorStatus last_status_ = OperatorStatus::Success;
    int last_error_ = 0;
};

void init_backend(BackendFactory &factory);

}  // namespace spy::hip
