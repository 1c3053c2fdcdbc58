// Graph nodes and operator definitions of the token loop: restates, with the same names, the parts
// of orchestration/include/graph/{basic_node,data_node,op_node}.h and
// orchestration/include/operator/{type,parameter,mat,non-linear,view,basic,input}.h (Spy tree) that a
// backend reads when an OperatorNode is submitted to it.
#pragma once

#include <array>
#include <cstdint>
#include <optional>
#include <string>
#include <vector>

#include "spy/tensor.h"

namespace spy {

enum class OperatorType : int32_t {            // operator/type.h:38-52
    Input,
    Nop, Dup, Copy, View, Reshape, MaskedCopy, MaskedSelect, GetRow, Transpose, Permute, Contiguous,
    Relu, Silu, Gelu, Max, Min, Softmax,
    Add, Sub, Mul, Div, Mod, MatMul,
    Sum,
    Norm, NormRMS, Rope,
    Quantize
};

inline constexpr bool is_view(OperatorType t) {  // operator/type.h:115-126
    switch (t) {
    case OperatorType::View: case OperatorType::Reshape: case OperatorType::Transpose: case OperatorType::Permute: case OperatorType::Copy: return true;
    default: return false;
    }
}

struct BasicNode {                               // graph/basic_node.h:22-129
    uint32_t id = 0xFFFFFFFFu;
    std::string name = "Unknown";
    bool active = true;
    std::vector<BasicNode *> input_list, output_list;
    virtual ~BasicNode() = default;

    void add_input(BasicNode *n) { input_list.push_back(n); n->output_list.push_back(this); }
    void add_output(BasicNode *n) { output_list.push_back(n); n->input_list.push_back(this); }
    size_t num_input() const { return input_list.size(); }
    size_t num_output() const { return output_list.size(); }
    template <class T = BasicNode> T *input(size_t i) const { return static_cast<T *>(input_list[i]); }
    template <class T = BasicNode> T *output(size_t i) const { return static_cast<T *>(output_list[i]); }
};

enum class DataNodeType : int {                  // graph/data_node.h:12-34
    Constant = 0, IO = 1, Cache = 2, Static = 3, ShapeDynamic = 4, DataDynamic = 5, Dynamic = 6, Default = Dynamic
};

struct DataNodeProperty {
    DataNodeType node_type = DataNodeType::Default;
    int layer_id = -1;
    int expert_id = -1;
};

struct DataNode final : BasicNode {              // graph/data_node.h:42-73
    DataNode *view_src = nullptr;
    Tensor tensor;
    DataNodeProperty node_prop;
    bool is_view() const { return view_src != nullptr; }
};

struct OperatorNode : BasicNode {                // graph/op_node.h:11-62
    OperatorType op_type = OperatorType::Nop;
    OperatorNode() = default;
    explicit OperatorNode(OperatorType t) : op_type(t) {}
    DataNode *input_data(size_t i) const { return input<DataNode>(i); }
    DataNode *output_data(size_t i) const { return output<DataNode>(i); }
    virtual void propagate() = 0;
};

template <class T> class OperatorParameter {      // operator/parameter.h:9-79
    std::optional<T> val_;
    const T *ref_ptr_ = nullptr;
public:
    OperatorParameter() = default;
    OperatorParameter(const T &v) : val_(v) {}
    void set_val(const T &v) { ref_ptr_ = nullptr; val_ = v; }
    const T &get_val() const { return val_.value(); }
    bool is_val() const { return val_.has_value(); }
};

template <OperatorType T_op_type> struct OperatorDefinition {};

// operators without parameters: output shape rules as in operator/common.h and view.h
#define SPY_SIMPLE_OP(OP)                                                      \
    template <> struct OperatorDefinition<OperatorType::OP> final : OperatorNode { \
        OperatorDefinition() : OperatorNode(OperatorType::OP) {}               \
        void propagate() override;                                             \
    };
SPY_SIMPLE_OP(Input) SPY_SIMPLE_OP(Nop) SPY_SIMPLE_OP(Dup) SPY_SIMPLE_OP(Copy) SPY_SIMPLE_OP(GetRow) SPY_SIMPLE_OP(Transpose)
SPY_SIMPLE_OP(Contiguous) SPY_SIMPLE_OP(Silu) SPY_SIMPLE_OP(Relu) SPY_SIMPLE_OP(Add) SPY_SIMPLE_OP(Sub) SPY_SIMPLE_OP(Mul) SPY_SIMPLE_OP(Div) SPY_SIMPLE_OP(MatMul)
#undef SPY_SIMPLE_OP

#define SPY_PARAM_OP(OP, ...)                                                  \
    template <> struct OperatorDefinition<OperatorType::OP> final : OperatorNode { \
        __VA_ARGS__                                                            \
        OperatorParameter<Param> params;                                       \
        OperatorDefinition() : OperatorNode(OperatorType::OP) {}               \
        explicit OperatorDefinition(const Param &p) : OperatorNode(OperatorType::OP), params(p) {} \
        void propagate() override;                                             \
    };
SPY_PARAM_OP(Softmax, struct Param { float scale; };)                               // non-linear.h:45
SPY_PARAM_OP(NormRMS, struct Param { float eps; };)                                 // non-linear.h:117
SPY_PARAM_OP(Reshape, struct Param { Shape new_shape; };)                           // view.h (Reshape)
SPY_PARAM_OP(View, struct Param { int64_t offset; Shape new_shape; };)              // view.h (View)
SPY_PARAM_OP(Permute, struct Param { std::array<int64_t, MAX_DIM> axis; };)         // view.h (Permute)
SPY_PARAM_OP(Quantize, struct Param { NumberType target_type; };)                   // operator/quantize.h:19
enum class RopeType : int { None = -1, Norm = 0, Neox = 2, GLM = 4 };              // non-linear.h:184-189
SPY_PARAM_OP(Rope, struct Param {                                                   // non-linear.h:191-207
    RopeType mode; int32_t num_past, num_dim, num_context, num_origin_context;
    float freq_base, freq_scale, extend_factor, attention_factor, beta_fast, beta_slow, xpos_base; bool xpos_down; };)
#undef SPY_PARAM_OP

using SoftmaxParam = OperatorDefinition<OperatorType::Softmax>::Param;
using NormRMSParam = OperatorDefinition<OperatorType::NormRMS>::Param;
using ReshapeParam = OperatorDefinition<OperatorType::Reshape>::Param;
using ViewParam    = OperatorDefinition<OperatorType::View>::Param;
using PermuteParam = OperatorDefinition<OperatorType::Permute>::Param;
using RopeParam    = OperatorDefinition<OperatorType::Rope>::Param;
using QuantizeParam = OperatorDefinition<OperatorType::Quantize>::Param;

}  // namespace spy
