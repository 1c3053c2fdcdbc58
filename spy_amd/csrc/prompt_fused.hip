// Fused activation producers of the prompt pass: the elementwise operators that sit between two
// MatMuls of the LLaMA graph, ending in the Q8_0 blocks the next MatMul's int8 GEMM reads, so that the
// fp32 intermediates never go to memory and activations shared by several MatMuls are quantized once.
//
//   norm_mul_q8:  NormRMS (non-linear.cpp:194-223) -> Mul by the norm weights (basic.cpp:15-50) ->
//                 Quantizator<FP32,Q8_0> (vec_convert.h:178-261); feeds wq|wk|wv or gate|up
//   silu_mul_q8:  Silu (non-linear.cpp:11-14,57-77) -> Mul (up x silu(gate)) -> Q8_0; feeds down
//
// Each step is the arithmetic of the operator kernel it replaces, in the same order and with the same
// roundings (the sum of squares is accumulated by the same thread pattern as norm_rms_kernel), so the
// blocks are the bytes spy_hip_op_norm_rms / _binary / _silu followed by spy_hip_quantize_q8_0 produce.
#include "common.cuh"

// 32 consecutive elements held 4 per lane by 8 adjacent lanes -> one Q8_0 block {fp16 d, int8 q[32]}
static __device__ __forceinline__ void store_q8_block(const float4 v, uint8_t *blk, int sub) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, __shfl_xor(amax, 1, SPY_WAVE));
    amax = fmaxf(amax, __shfl_xor(amax, 2, SPY_WAVE));
    amax = fmaxf(amax, __shfl_xor(amax, 4, SPY_WAVE));
    const float d = amax / 127.0f;
    const float id = (amax != 0.0f) ? 127.0f / amax : 0.0f;
    int q[4] = {(int)rintf(v.x * id), (int)rintf(v.y * id), (int)rintf(v.z * id), (int)rintf(v.w * id)};
#pragma unroll
    for (int i = 0; i < 4; i++) q[i] = q[i] < -128 ? -128 : (q[i] > 127 ? 127 : q[i]);
    uint16_t *out = (uint16_t *)(blk + 2 + sub * 4);       // 34-byte blocks: 2-byte alignment only
    out[0] = (uint16_t)((q[0] & 0xFF) | ((q[1] & 0xFF) << 8));
    out[1] = (uint16_t)((q[2] & 0xFF) | ((q[3] & 0xFF) << 8));
    if (sub == 0) *(uint16_t *)blk = f2h(d);
}

// one workgroup per token row of K floats (K % 32 == 0, rows 16-byte aligned)
__global__ __launch_bounds__(256) void norm_mul_q8_kernel(const float *__restrict__ x, int64_t x_stride, const float *__restrict__ w, float eps,
                                                          uint8_t *__restrict__ y, int K) {
    __shared__ float s_part[4];
    const float *s = (const float *)((const uint8_t *)x + (size_t)blockIdx.x * x_stride);
    float acc = 0.0f;
    for (int i = threadIdx.x; i < K; i += 256) { const float v = s[i]; acc = fmaf(v, v, acc); }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = acc;
    __syncthreads();
    const float sum = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
    const float mean = sum / (float)K;
    const float scale = 1.0f / sqrtf(mean + eps);
    uint8_t *yr = y + (size_t)blockIdx.x * (K / 32) * 34;
    const int sub = threadIdx.x & 7;
    for (int g = threadIdx.x; g < K / 4; g += 256) {        // K / 4 is a multiple of 8: whole 8-lane groups stay together
        const float4 v = ((const float4 *)s)[g], ww = ((const float4 *)w)[g];
        const float4 z = make_float4((v.x * scale) * ww.x, (v.y * scale) * ww.y, (v.z * scale) * ww.z, (v.w * scale) * ww.w);
        store_q8_block(z, yr + (size_t)(g >> 3) * 34, sub);
    }
}

static __device__ __forceinline__ float silu_ref(float x) {     // the reference's table entry for fp16(x)
    const float v = h2f(f2h(x));
    return v / (1.0f + expf(-v));
}
// flat over nrow x F elements, 4 per thread; F % 32 == 0
__global__ __launch_bounds__(256) void silu_mul_q8_kernel(const float4 *__restrict__ gate, const float4 *__restrict__ up, uint8_t *__restrict__ y, int64_t total4) {
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= total4) return;                                  // total4 is a multiple of 8: whole 8-lane groups leave together
    const float4 a = gate[g], u = up[g];
    const float4 z = make_float4(u.x * silu_ref(a.x), u.y * silu_ref(a.y), u.z * silu_ref(a.z), u.w * silu_ref(a.w));
    store_q8_block(z, y + (size_t)(g >> 3) * 34, threadIdx.x & 7);
}

int spy_norm_mul_q8_launch(hipStream_t st, const float *x, int64_t x_stride, const float *w, float eps, void *y, int64_t nrow, int64_t K) {
    SPY_CHECK_ARG(x && w && y && nrow > 0 && nrow < (1ll << 31) && K > 0 && K % 32 == 0 && K < (1ll << 31));
    SPY_CHECK_ARG(x_stride % 16 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0 && ((uintptr_t)y % 2) == 0);
    norm_mul_q8_kernel<<<dim3((unsigned)nrow), dim3(256), 0, st>>>(x, x_stride, w, eps, (uint8_t *)y, (int)K);
    return SPY_LAUNCH_RC();
}

int spy_silu_mul_q8_launch(hipStream_t st, const float *gate, const float *up, void *y, int64_t nrow, int64_t F) {
    SPY_CHECK_ARG(gate && up && y && nrow > 0 && F > 0 && F % 32 == 0);
    SPY_CHECK_ARG(((uintptr_t)gate % 16) == 0 && ((uintptr_t)up % 16) == 0 && ((uintptr_t)y % 2) == 0);
    const int64_t total4 = nrow * F / 4;
    SPY_CHECK_ARG((total4 + 255) / 256 < (1ll << 31));
    silu_mul_q8_kernel<<<dim3((unsigned)((total4 + 255) / 256)), dim3(256), 0, st>>>((const float4 *)gate, (const float4 *)up, (uint8_t *)y, total4);
    return SPY_LAUNCH_RC();
}
