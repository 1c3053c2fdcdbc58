// The backend interface: restates backend/interface/include/backend/backend.h:22-130 and
// backend/type.h:5-19 of the Spy tree (same class and method names and meanings).
#pragma once

#include <cstddef>
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <string_view>
#include <unordered_map>

#include "spy/graph.h"

namespace spy {

enum class BackendType { Host, Share, Device, Unknown };

enum class OperatorStatus { Success, Fail, Unsupport };

// util/include/util/wrapper/config_table.h:49-71: string -> string with typed lookup
class ConfigTable {
    std::map<std::string, std::string> table_;
public:
    void set(const std::string &k, const std::string &v) { table_[k] = v; }
    int parse_or(const std::string &k, int fallback) const {
        const auto it = table_.find(k);
        return it == table_.end() ? fallback : std::stoi(it->second);
    }
};

class Backend {
    BackendType backend_type_;
public:
    explicit Backend(BackendType t) : backend_type_(t) {}
    virtual ~Backend() = default;
    BackendType type() const { return backend_type_; }

    virtual size_t get_max_memory_capacity() const = 0;
    virtual size_t get_avail_memory_capacity() const = 0;
    virtual void *alloc_memory(size_t size) = 0;
    virtual void dealloc_memory(void *ptr, size_t size) = 0;
    virtual size_t get_max_concurrency() const = 0;
    virtual size_t get_avail_concurrency() const = 0;
    virtual bool is_support(OperatorType op_type) const = 0;
    virtual void submit(OperatorNode *op_node_ptr, std::function<void()> &&callback = nullptr) = 0;
};

class BackendFactory {
public:
    using BackendConfiguration = ConfigTable;
    using BackendGeneratorFunc = std::unique_ptr<Backend> (*)(const BackendConfiguration &);
private:
    std::unordered_map<std::string, BackendGeneratorFunc> generator_map_;
public:
    BackendFactory();
    std::unique_ptr<Backend> init_backend(const std::string &name, const BackendConfiguration &config) {
        const auto it = generator_map_.find(name);
        return it == generator_map_.end() ? nullptr : it->second(config);
    }
    void add_backend_map(const std::string &name, BackendGeneratorFunc f) { generator_map_.insert_or_assign(name, f); }
    static std::string make_backend_name(std::string_view device, std::string_view policy) { return std::string(device) + ":" + std::string(policy); }
};

namespace hip { void init_backend(BackendFactory &); }   // registers "hip:default" (next to cpu::init_backend, backend.h:142-155)

inline BackendFactory::BackendFactory() { hip::init_backend(*this); }

}  // namespace spy
