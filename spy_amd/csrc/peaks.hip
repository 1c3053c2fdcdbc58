// Measured ceilings of the part, next to the published peaks the rooflines divide by:
//   * int8 matrix cores: waves that do nothing but v_mfma_i32_32x32x32_i8 on register operands;
//   * HBM read: every lane streams 16-byte pieces of a large buffer, nothing else.
//   * the same MFMA with the per-block scaling that the quantized GEMM needs per output (spy_hip_measure_mfma_i8_scaled).
// They back the denominators printed by the operator sweep; no product path calls them.
#include "common.cuh"

#define HIP_TRY(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) return (int)e_; } while (0)

typedef int v4i_p __attribute__((ext_vector_type(4)));
typedef int v16i_p __attribute__((ext_vector_type(16)));

#define PEAK_MFMA_CHAINS 4
__global__ __launch_bounds__(256) void peak_mfma_i8_kernel(int iters, int *sink) {
    v4i_p a = {(int)threadIdx.x, 0x01010101, 0x02020202, (int)blockIdx.x}, b = {0x01010101, (int)threadIdx.x, 0x03030303, 0x01010101};
    v16i_p acc[PEAK_MFMA_CHAINS];
#pragma unroll
    for (int c = 0; c < PEAK_MFMA_CHAINS; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[c][r] = c + r;
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int c = 0; c < PEAK_MFMA_CHAINS; c++) acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[c], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int c = 0; c < PEAK_MFMA_CHAINS; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) s ^= acc[c][r];
    if (s == 0x7fffffff) sink[0] = s;                       // keeps the chains alive, practically never taken
}

// Achieved int8 MFMA rate in TOP/s (2 operations per multiply-accumulate), `iters` x 4 MFMAs per wave,
// 8 workgroups of 4 waves per compute unit.
extern "C" int spy_hip_measure_mfma_i8(void *stream, int32_t iters, float *tops) {
    SPY_CHECK_ARG(iters > 0 && iters <= (1 << 22) && tops);
    hipStream_t st = (hipStream_t)stream;
    hipDeviceProp_t prop;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    HIP_TRY(hipGetDeviceProperties(&prop, dev));
    int *sink = nullptr;
    HIP_TRY(hipMalloc(&sink, 64));
    hipEvent_t e0, e1;
    HIP_TRY(hipEventCreate(&e0)); HIP_TRY(hipEventCreate(&e1));
    const int grid = prop.multiProcessorCount * 8;
    peak_mfma_i8_kernel<<<grid, 256, 0, st>>>(16, sink);    // warm-up
    HIP_TRY(hipEventRecord(e0, st));
    peak_mfma_i8_kernel<<<grid, 256, 0, st>>>(iters, sink);
    HIP_TRY(hipEventRecord(e1, st));
    HIP_TRY(hipEventSynchronize(e1));
    float ms = 0.0f;
    HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
    const double ops = (double)grid * 4.0 * (double)iters * PEAK_MFMA_CHAINS * 2.0 * 32.0 * 32.0 * 32.0;
    *tops = (float)(ops / ((double)ms * 1e-3) / 1e12);
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
    HIP_TRY(hipFree(sink));
    return SPY_LAUNCH_RC();
}

// The block-scaled int8 GEMM's inner work on register operands only: per quantization block and 32 x 32 output tile one
// v_mfma_i32_32x32x32_i8 (the block dots), one v_mfma_f32_32x32x8_f16 (the outer product of the two scale vectors) and
// the 32 vector instructions that bring the dots to fp32 and accumulate them, dot * scale, per lane; a wave owns 2 x 2
// tiles as in the GEMM kernel, three workgroups per compute unit.  MODE 0: v_cvt_f32_i32 + v_fma_f32 per output.
// MODE 1: the MFMA accumulates onto the integer 0x4B400000, whose float value is 12582912 + dot, and a v_sub_f32
// takes the 12582912 off again (exact below 2^22) before the fma.  No LDS, no global loads: the ceiling that the
// epilogue leaves to the int8 matrix cores.
typedef _Float16 v4h_p __attribute__((ext_vector_type(4)));
typedef float v16f_p __attribute__((ext_vector_type(16)));
template <int MODE>
__global__ __launch_bounds__(256, 3) void peak_mfma_i8_scaled_kernel(int iters, float *sink) {
    v4i_p a[2] = {{(int)threadIdx.x, 0x01010101, 0x02020202, (int)blockIdx.x}, {0x01020304, (int)threadIdx.x, 0x02020202, 0x05050505}};
    v4i_p b[2] = {{0x01010101, (int)threadIdx.x, 0x03030303, 0x01010101}, {0x01010101, 0x7f7f7f7f, (int)blockIdx.x, 0x01010101}};
    v4h_p ha[2] = {{(_Float16)0.5f, 0, 0, 0}, {(_Float16)0.25f, 0, 0, 0}}, hb[2] = {{(_Float16)(threadIdx.x & 31 ? 0.125f : 0.5f), 0, 0, 0}, {(_Float16)1.0f, 0, 0, 0}};
    float acc[2][2][16];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
    v16i_p cinit;
#pragma unroll
    for (int r = 0; r < 16; r++) cinit[r] = MODE == 1 ? 0x4B400000 : 0;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) {
                v16f_p zf = {0};
                const v16i_p I = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], cinit, 0, 0, 0);
                const v16f_p S = __builtin_amdgcn_mfma_f32_32x32x8f16(ha[i], hb[j], zf, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float f = MODE == 1 ? __int_as_float(I[r]) - 12582912.0f : (float)I[r];
                    acc[i][j][r] = fmaf(S[r], f, acc[i][j][r]);
                }
            }
        a[0].x += 1; b[1].z ^= it;                         // the operands change from block to block
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) s += acc[i][j][r];
    if (s == 1.2345e-30f) sink[0] = s;
}

// Achieved rate, in TOP/s of int8 multiply-accumulates (2 operations each), of the block-scaled inner loop above:
// mode 0 = conversion + fma per output, mode 1 = biased accumulator + subtraction + fma.
extern "C" int spy_hip_measure_mfma_i8_scaled(void *stream, int32_t iters, int32_t mode, float *tops) {
    SPY_CHECK_ARG(iters > 0 && iters <= (1 << 22) && tops && (mode == 0 || mode == 1));
    hipStream_t st = (hipStream_t)stream;
    hipDeviceProp_t prop;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    HIP_TRY(hipGetDeviceProperties(&prop, dev));
    float *sink = nullptr;
    HIP_TRY(hipMalloc(&sink, 64));
    hipEvent_t e0, e1;
    HIP_TRY(hipEventCreate(&e0)); HIP_TRY(hipEventCreate(&e1));
    const int grid = prop.multiProcessorCount * 3;
    auto launch = [&](int n) {
        if (mode == 0) peak_mfma_i8_scaled_kernel<0><<<grid, 256, 0, st>>>(n, sink);
        else peak_mfma_i8_scaled_kernel<1><<<grid, 256, 0, st>>>(n, sink);
    };
    launch(16);                                             // warm-up
    HIP_TRY(hipEventRecord(e0, st));
    launch(iters);
    HIP_TRY(hipEventRecord(e1, st));
    HIP_TRY(hipEventSynchronize(e1));
    float ms = 0.0f;
    HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
    const double ops = (double)grid * 4.0 * (double)iters * 4.0 * 2.0 * 32.0 * 32.0 * 32.0;
    *tops = (float)(ops / ((double)ms * 1e-3) / 1e12);
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
    HIP_TRY(hipFree(sink));
    return SPY_LAUNCH_RC();
}

#define PEAK_READ_UNROLL 8
__global__ __launch_bounds__(256) void peak_read_kernel(const uint4 *__restrict__ p, size_t n16, uint32_t *sink) {
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    uint32_t x = 0;
    for (; i + (PEAK_READ_UNROLL - 1) * stride < n16; i += PEAK_READ_UNROLL * stride) {
        uint4 v[PEAK_READ_UNROLL];
#pragma unroll
        for (int u = 0; u < PEAK_READ_UNROLL; u++) v[u] = p[i + u * stride];
#pragma unroll
        for (int u = 0; u < PEAK_READ_UNROLL; u++) x ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < n16; i += stride) { const uint4 v = p[i]; x ^= v.x ^ v.y ^ v.z ^ v.w; }
    if (x == 0x12345679u) sink[0] = x;
}

// Achieved read rate in GB/s over `bytes` of device memory at `buf` (contents irrelevant; 16-byte aligned),
// averaged over `reps` passes.  Use a buffer far larger than the caches (>= 1 GiB).
extern "C" int spy_hip_measure_hbm_read(void *stream, const void *buf, size_t bytes, int32_t reps, float *gbps) {
    SPY_CHECK_ARG(buf && bytes >= (1u << 20) && (((uintptr_t)buf) & 15) == 0 && reps > 0 && gbps);
    hipStream_t st = (hipStream_t)stream;
    hipDeviceProp_t prop;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    HIP_TRY(hipGetDeviceProperties(&prop, dev));
    uint32_t *sink = nullptr;
    HIP_TRY(hipMalloc(&sink, 64));
    hipEvent_t e0, e1;
    HIP_TRY(hipEventCreate(&e0)); HIP_TRY(hipEventCreate(&e1));
    const int grid = prop.multiProcessorCount * 8;
    const size_t n16 = bytes / 16;
    peak_read_kernel<<<grid, 256, 0, st>>>((const uint4 *)buf, n16, sink);
    HIP_TRY(hipEventRecord(e0, st));
    for (int r = 0; r < reps; r++) peak_read_kernel<<<grid, 256, 0, st>>>((const uint4 *)buf, n16, sink);
    HIP_TRY(hipEventRecord(e1, st));
    HIP_TRY(hipEventSynchronize(e1));
    float ms = 0.0f;
    HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
    *gbps = (float)((double)n16 * 16.0 * reps / ((double)ms * 1e-3) / 1e9);
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
    HIP_TRY(hipFree(sink));
    return SPY_LAUNCH_RC();
}
