// Shape / Tensor: restates the members of orchestration/include/number/tensor.h:23-263 (Spy tree)
// that operators read -- number_type, dim, elements[4], bytes[4] (byte strides, bytes[0] = block
// size), data_ptr -- with the same names and semantics.
#pragma once

#include <array>
#include <cstdint>
#include <initializer_list>

#include "spy/number.h"

namespace spy {

constexpr uint32_t MAX_DIM = 4;

struct Shape {
    using DimensionArray = std::array<int64_t, MAX_DIM>;

    NumberType     number_type = NumberType::FP32;
    uint32_t       dim = 0;
    DimensionArray elements{0, 0, 0, 0};
    DimensionArray bytes{0, 0, 0, 0};

    Shape() = default;

    // contiguous layout (tensor.h:44-80)
    Shape(std::initializer_list<int64_t> ne, NumberType type) : number_type(type), dim((uint32_t)ne.size()) {
        uint32_t i = 0;
        for (int64_t e : ne) elements[i++] = e;
        for (; i < MAX_DIM; ++i) elements[i] = 1;
        bytes[0] = get_type_size(type);
        int64_t acc = get_row_size(type, elements[0]);
        for (uint32_t k = 1; k < MAX_DIM; ++k) { bytes[k] = acc; acc *= elements[k]; }
    }

    // explicit strides (tensor.h:92-104): trailing dimensions get 1 element and the total size
    Shape(std::initializer_list<int64_t> ne, std::initializer_list<int64_t> nb, NumberType type) : number_type(type), dim((uint32_t)ne.size()) {
        uint32_t i = 0;
        for (int64_t e : ne) elements[i++] = e;
        i = 0;
        for (int64_t b : nb) bytes[i++] = b;
        const int64_t total = elements[dim - 1] * bytes[dim - 1];
        for (uint32_t k = dim; k < MAX_DIM; ++k) { elements[k] = 1; bytes[k] = total; }
    }

    bool operator==(const Shape &o) const { return number_type == o.number_type && dim == o.dim && elements == o.elements && bytes == o.bytes; }

    int64_t total_size() const {                     // tensor.h:131-137
        int64_t size = bytes[0] * elements[0] / get_block_size(number_type);
        for (uint32_t i = 1; i < dim; ++i) size += bytes[i] * (elements[i] - 1);
        return size;
    }
    int64_t total_element() const { return elements[0] * elements[1] * elements[2] * elements[3]; }
    int64_t num_row() const { return elements[1] * elements[2] * elements[3]; }
    int64_t row_size() const { return get_type_size(number_type) * elements[0] / get_block_size(number_type); }
};

struct Tensor {
    Shape shape;
    void *data_ptr = nullptr;

    Tensor() = default;
    Tensor(const Shape &s, void *p) : shape(s), data_ptr(p) {}

    template <class T = void> T *get() const { return static_cast<T *>(data_ptr); }
    void set_data_ptr(void *p) { data_ptr = p; }
    const Shape &get_shape() const { return shape; }
    NumberType type() const { return shape.number_type; }
    int64_t total_size() const { return shape.total_size(); }
    int64_t total_element() const { return shape.total_element(); }
};

}  // namespace spy
