// Activation converters: FP32 -> Q8_0 and FP32 -> FP16.
// Replace Quantizator<FP32,Q8_0>::transform and Quantizator<FP32,FP16>::transform
// (backend/host/include/simd/vec_convert.h:178-261 and :39-65 in the Spy tree), which
// OperatorMatMulImpl::execute runs on every activation row (backend/host/operator/mat.cpp:95-128).
#include "common.cuh"

// One 32-element block per 8 lanes (4 floats = one 128-bit load per lane); 32 blocks per
// 256-thread workgroup.  amax is reduced inside the 8-lane group.
// Bit-exactness: d = amax/127 and id = 127/amax are IEEE divisions, q = rint(x*id) is
// round-half-even (v_rndne_f32), exactly the AVX sequence of the reference.
__global__ __launch_bounds__(256) void quantize_q8_0_kernel(const float *__restrict__ x, int64_t x_stride,
                                                            uint8_t *__restrict__ y, int64_t nrow, int64_t nblk) {
    const int64_t gblk = (int64_t)blockIdx.x * 32 + (threadIdx.x >> 3);
    const int sub = threadIdx.x & 7;
    if (gblk >= nrow * nblk) return;      // whole 8-lane groups leave together
    const int64_t row = gblk / nblk, b = gblk % nblk;
    const float4 v = *(const float4 *)((const uint8_t *)x + row * x_stride + (b * 32 + sub * 4) * 4);
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, __shfl_xor(amax, 1, SPY_WAVE));
    amax = fmaxf(amax, __shfl_xor(amax, 2, SPY_WAVE));
    amax = fmaxf(amax, __shfl_xor(amax, 4, SPY_WAVE));
    const float d  = amax / 127.0f;
    const float id = (amax != 0.0f) ? 127.0f / amax : 0.0f;
    int q[4] = {(int)rintf(v.x * id), (int)rintf(v.y * id), (int)rintf(v.z * id), (int)rintf(v.w * id)};
#pragma unroll
    for (int i = 0; i < 4; i++) q[i] = q[i] < -128 ? -128 : (q[i] > 127 ? 127 : q[i]);
    uint8_t *blk = y + (row * nblk + b) * 34;          // 34-byte blocks: 2-byte alignment only
    uint16_t *out = (uint16_t *)(blk + 2 + sub * 4);
    out[0] = (uint16_t)((q[0] & 0xFF) | ((q[1] & 0xFF) << 8));
    out[1] = (uint16_t)((q[2] & 0xFF) | ((q[3] & 0xFF) << 8));
    if (sub == 0) *(uint16_t *)blk = f2h(d);
}

__global__ __launch_bounds__(256) void quantize_f16_kernel(const float *__restrict__ x, int64_t x_stride,
                                                           uint16_t *__restrict__ y, int64_t nrow, int64_t K) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nrow * K) return;
    const int64_t row = i / K, c = i % K;
    y[i] = f2h(*(const float *)((const uint8_t *)x + row * x_stride + c * 4));
}

extern "C" int spy_hip_quantize_q8_0(void *stream, const float *x, int64_t x_stride, void *y, int64_t nrow, int64_t K) {
    SPY_CHECK_ARG(x && y && nrow > 0 && K > 0 && K % 32 == 0);
    SPY_CHECK_ARG(x_stride % 16 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)y % 2) == 0);
    const int64_t nblk = K / 32, total = nrow * nblk;
    SPY_CHECK_ARG((total + 31) / 32 < (1ll << 31));
    quantize_q8_0_kernel<<<dim3((unsigned)((total + 31) / 32)), dim3(256), 0, (hipStream_t)stream>>>(x, x_stride, (uint8_t *)y, nrow, nblk);
    return SPY_LAUNCH_RC();
}

extern "C" int spy_hip_quantize_f16(void *stream, const float *x, int64_t x_stride, void *y, int64_t nrow, int64_t K) {
    SPY_CHECK_ARG(x && y && nrow > 0 && K > 0 && x_stride % 4 == 0);
    const int64_t total = nrow * K;
    SPY_CHECK_ARG((total + 255) / 256 < (1ll << 31));
    quantize_f16_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(x, x_stride, (uint16_t *)y, nrow, K);
    return SPY_LAUNCH_RC();
}
