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

// ---- RoPE + cache writes of a prompt pass -----------------------------------------------------------
// Rope (non-linear.cpp:270-371, default branch) rotates q and k of every layer by angles that depend on
// the position and the pair index only: they are computed once per pass into a table, with the
// arithmetic of the operator kernel (theta built by k successive fp32 multiplications, :304-309; cosf /
// sinf of theta * freq_scale, times the attention factor).  Per layer one kernel then rotates q and k
// and stores them where the next operators read them: q as fp16 [head][token][hd] (the conversion the
// score product applies to its right operand, mat.cpp:37) and k as fp16 into the K cache rows of the
// pass (the Copy of view.cpp:83-227); a second kernel transposes v into the V^T cache.
__global__ __launch_bounds__(64) void rope_table_kernel(float2 *__restrict__ table, int past, int npair, float theta_scale, float freq_scale, float mscale) {
    const int t = blockIdx.x;
    const float p = (float)(past + t);
    for (int k = threadIdx.x; k < npair; k += 64) {
        float theta = p;
        for (int j = 0; j < k; j++) theta *= theta_scale;
        const float ang = freq_scale * theta;
        table[(size_t)t * npair + k] = make_float2(cosf(ang) * mscale, sinf(ang) * mscale);
    }
}

// grid (T, H); q, k: f32 [T][H * hd]; q16: fp16 [H][T][hd]; kc: K cache row of the pass's first token, fp16 [T][H * hd]
__global__ __launch_bounds__(64) void rope_store_kernel(const float *__restrict__ q, const float *__restrict__ k, const float2 *__restrict__ table,
                                                        uint16_t *__restrict__ q16, uint16_t *__restrict__ kc, int T, int H, int hd) {
    const int t = blockIdx.x, h = blockIdx.y, npair = hd / 2;
    const size_t row = ((size_t)t * H + h) * hd;
    for (int p = threadIdx.x; p < npair; p += 64) {
        const float2 cs = table[(size_t)t * npair + p];
        const float2 a = *(const float2 *)(q + row + 2 * p), b = *(const float2 *)(k + row + 2 * p);
        const float q0 = a.x * cs.x - a.y * cs.y, q1 = a.x * cs.y + a.y * cs.x;
        const float k0 = b.x * cs.x - b.y * cs.y, k1 = b.x * cs.y + b.y * cs.x;
        *(uint32_t *)(q16 + ((size_t)h * T + t) * hd + 2 * p) = (uint32_t)f2h(q0) | ((uint32_t)f2h(q1) << 16);
        *(uint32_t *)(kc + row + 2 * p) = (uint32_t)f2h(k0) | ((uint32_t)f2h(k1) << 16);
    }
}

// v: f32 [T][d] -> V^T cache: fp16 vc[col * n_ctx + t] for t < T (vc points at the pass's first position); 64 x 64 tiles through LDS
__global__ __launch_bounds__(256) void vt_store_kernel(const float *__restrict__ v, uint16_t *__restrict__ vc, int T, int d, int64_t n_ctx) {
    __shared__ uint16_t tile[64][66];
    const int t0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int tt = i >> 6, cc = i & 63;
        tile[tt][cc] = (t0 + tt < T && c0 + cc < d) ? f2h(v[(size_t)(t0 + tt) * d + c0 + cc]) : (uint16_t)0;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int cc = i >> 6, tt = i & 63;
        if (t0 + tt < T && c0 + cc < d) vc[(size_t)(c0 + cc) * n_ctx + t0 + tt] = tile[tt][cc];
    }
}

int spy_rope_table_launch(hipStream_t st, float *table, int past, int T, int hd, float freq_base, float freq_scale, float mscale) {
    SPY_CHECK_ARG(table && past >= 0 && T > 0 && hd > 0 && hd % 2 == 0);
    const float theta_scale = powf(freq_base, -2.0f / (float)hd);             // host libm, as the reference (:282)
    rope_table_kernel<<<dim3((unsigned)T), dim3(64), 0, st>>>((float2 *)table, past, hd / 2, theta_scale, freq_scale, mscale);
    return SPY_LAUNCH_RC();
}

int spy_rope_store_launch(hipStream_t st, const float *q, const float *k, const float *table, uint16_t *q16, uint16_t *kc, int T, int H, int hd) {
    SPY_CHECK_ARG(q && k && table && q16 && kc && T > 0 && H > 0 && H < 65536 && hd > 0 && hd % 2 == 0);
    SPY_CHECK_ARG(((uintptr_t)q % 8) == 0 && ((uintptr_t)k % 8) == 0 && ((uintptr_t)table % 8) == 0 && ((uintptr_t)q16 % 4) == 0 && ((uintptr_t)kc % 4) == 0);
    rope_store_kernel<<<dim3((unsigned)T, (unsigned)H), dim3(64), 0, st>>>(q, k, (const float2 *)table, q16, kc, T, H, hd);
    return SPY_LAUNCH_RC();
}

int spy_vt_store_launch(hipStream_t st, const float *v, uint16_t *vc, int T, int d, int64_t n_ctx) {
    SPY_CHECK_ARG(v && vc && T > 0 && d > 0 && n_ctx >= T && (d + 63) / 64 < 65536);
    vt_store_kernel<<<dim3((unsigned)((T + 63) / 64), (unsigned)((d + 63) / 64)), dim3(256), 0, st>>>(v, vc, T, d, n_ctx);
    return SPY_LAUNCH_RC();
}
