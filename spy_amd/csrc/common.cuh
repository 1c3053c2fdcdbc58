// Shared device/host helpers for the gfx950 kernels: block layouts, fp16 conversion,
// wavefront reductions, argument checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/spy_hip.h"

#define SPY_WAVE 64

// Block layouts (orchestration/include/number/number_impl/quant.h:25-28,139-142 and
// k-quant.h:101-111,177-182 in the Spy tree). Weights stay in these native layouts in HBM.
struct __attribute__((packed)) blk_q4_0 { uint16_t d; uint8_t qs[16]; };
struct __attribute__((packed)) blk_q8_0 { uint16_t d; int8_t qs[32]; };
struct __attribute__((packed)) blk_q4_k { uint16_t d, dmin; uint8_t scales[12]; uint8_t qs[128]; };
struct __attribute__((packed)) blk_q6_k { uint8_t ql[128]; uint8_t qh[64]; int8_t scales[16]; uint16_t d; };
static_assert(sizeof(blk_q4_0) == 18 && sizeof(blk_q8_0) == 34 && sizeof(blk_q4_k) == 144 && sizeof(blk_q6_k) == 210, "block sizes");

static inline __host__ __device__ int64_t spy_type_size(int t) {
    switch (t) {
    case SPY_HIP_F32: case SPY_HIP_I32: return 4;
    case SPY_HIP_F16: return 2;
    case SPY_HIP_Q4_0: return 18;
    case SPY_HIP_Q8_0: return 34;
    case SPY_HIP_Q4_K: return 144;
    case SPY_HIP_Q6_K: return 210;
    }
    return 0;
}
static inline __host__ __device__ int64_t spy_block_size(int t) {
    switch (t) {
    case SPY_HIP_F32: case SPY_HIP_I32: case SPY_HIP_F16: return 1;
    case SPY_HIP_Q4_0: case SPY_HIP_Q8_0: return 32;
    case SPY_HIP_Q4_K: case SPY_HIP_Q6_K: return 256;
    }
    return 0;
}
static inline __host__ __device__ int64_t spy_row_size(int t, int64_t n) { return n * spy_type_size(t) / spy_block_size(t); }

// fp16 <-> fp32: IEEE round-to-nearest-even narrowing (v_cvt_f16_f32) and exact widening.
static __device__ __forceinline__ float h2f(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
// The empty asm keeps the operand a finished fp32 value: without it the compiler folds a preceding multiply or add
// into v_fma_mixlo_f16, which rounds once (straight to fp16) where the reference rounds twice (fp32, then fp16) --
// a different result whenever the fp32 rounding lands on an fp16 tie.
static __device__ __forceinline__ uint16_t f2h(float f) { asm("" : "+v"(f)); return __builtin_bit_cast(uint16_t, (_Float16)f); }

static __device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, SPY_WAVE);
    return v;
}
static __device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, SPY_WAVE));
    return v;
}
static __device__ __forceinline__ int wave_sum_i32(int v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, SPY_WAVE);
    return v;
}

// raises the dynamic-LDS limit of `kern` on the current device to at least `lds` bytes (runtime.hip: one record per device and
// kernel for the whole process, only ever raised)
int spy_raise_lds_limit(const void *kern, size_t lds);

#define SPY_CHECK_ARG(cond) do { if (!(cond)) return SPY_HIP_EINVAL; } while (0)
#define SPY_LAUNCH_RC() ((int)hipGetLastError())

static inline bool spy_t_contiguous(const spy_hip_tensor *t) {
    return t->nb[0] == spy_type_size(t->type) && t->nb[1] == t->nb[0] * t->ne[0] / spy_block_size(t->type) &&
           t->nb[2] == t->nb[1] * t->ne[1] && t->nb[3] == t->nb[2] * t->ne[2];
}
static inline int64_t spy_t_nrow(const spy_hip_tensor *t) { return t->ne[1] * t->ne[2] * t->ne[3]; }
static inline int64_t spy_t_nelem(const spy_hip_tensor *t) { return t->ne[0] * t->ne[1] * t->ne[2] * t->ne[3]; }
