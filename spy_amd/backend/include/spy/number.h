// Number types and block sizes as the backend sees them.
// Restates orchestration/include/number/number_impl/type.h:12-45 and number.h:33-63 of the Spy tree
// (same enumerator names and values = ggml type ids) so that backend/hip compiles unchanged
// against a real Spy checkout; only the members the token loop touches are present.
#pragma once

#include <cstdint>

namespace spy {

enum class NumberType : int {
    FP32 = 0, FP16 = 1, Q4_0 = 2, Q4_1 = 3, Q5_0 = 6, Q5_1 = 7, Q8_0 = 8, Q8_1 = 9,
    Q2_K = 10, Q3_K = 11, Q4_K = 12, Q5_K = 13, Q6_K = 14, Q8_K = 15,
    INT8 = 24, INT16 = 25, INT32 = 26, INT64 = 27, FP64 = 28
};

inline constexpr int64_t get_type_size(NumberType t) {
    switch (t) {
    case NumberType::FP32: case NumberType::INT32: return 4;
    case NumberType::FP16: case NumberType::INT16: return 2;
    case NumberType::INT8: return 1;
    case NumberType::INT64: case NumberType::FP64: return 8;
    case NumberType::Q4_0: return 18;
    case NumberType::Q8_0: return 34;
    case NumberType::Q4_K: return 144;
    case NumberType::Q6_K: return 210;
    default: return 0;
    }
}

inline constexpr int64_t get_block_size(NumberType t) {
    switch (t) {
    case NumberType::Q4_0: case NumberType::Q8_0: return 32;
    case NumberType::Q4_K: case NumberType::Q6_K: return 256;
    default: return 1;
    }
}

inline constexpr int64_t get_row_size(NumberType t, int64_t n) { return n * get_type_size(t) / get_block_size(t); }

}  // namespace spy
