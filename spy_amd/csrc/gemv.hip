// Quantized matrix x vector(s): every weight row dotted with 1..8 Q8_0 activation rows.
// Replaces the Dot<Q4_0,Q8_0> / Dot<Q8_0,Q8_0> loops of OperatorMatMulImpl::execute
// (backend/host/include/simd/vec_dot.h:42-115, backend/host/operator/mat.cpp:130-143 in the Spy
// tree) and adds Q4_K / Q6_K weights, which the reference only declares.
//
// HBM-bound: each weight byte is read once.  Weights stay in their native GGUF block layout
// (18-byte Q4_0 / 34-byte Q8_0 blocks, 2-byte aligned), so a workgroup streams a contiguous
// span of whole rows with 128-bit coalesced loads into LDS and the lanes then pick their
// 4-byte-aligned block PAIRS (36 / 68 bytes, an odd number of dwords -> conflict-free LDS
// reads) out of LDS.  Activations are staged once per workgroup as aligned int8 plus
// {scale, sum(q)} per block; sum(q) turns sum((n-8)*q) into sum(n*q) - 8*sum(q), so the nibbles
// feed v_dot4_i32_i8 without a per-byte subtract.  The int32 block dot is exact; only the
// fp32 accumulation order differs from the reference's 8-lane AVX accumulators.
#include "common.cuh"

#define GEMV_THREADS 256
#define GEMV_WAVES 4
#define GEMV_MAX_ROUNDS 12                 // 128-bit loads per thread per tile (<= 48 KiB tile)
#define GEMV_TILE_TARGET 28672

template <int WT> struct wt_traits;
template <> struct wt_traits<SPY_HIP_Q4_0> { static constexpr int BLK = 18; };
template <> struct wt_traits<SPY_HIP_Q8_0> { static constexpr int BLK = 34; };

// Stage T rows of native Q8_0 activations into LDS: qs -> s_q[(t*nblk+b)*32 ..], and
// s_meta[t*nblk+b] = {bits(float scale), sum of the 32 quants}.
static __device__ __forceinline__ void stage_activations(const uint8_t *__restrict__ xq, int8_t *s_q, int2 *s_meta, int total_blk) {
    const uint16_t *src = (const uint16_t *)xq;
    const int total_h = total_blk * 17;
    for (int h = threadIdx.x; h < total_h; h += GEMV_THREADS) {
        const int b = h / 17, w = h - b * 17;
        const uint16_t v = src[h];
        if (w == 0) s_meta[b].x = __float_as_int(h2f(v));
        else ((uint16_t *)s_q)[b * 16 + (w - 1)] = v;
    }
    __syncthreads();
    for (int b = threadIdx.x; b < total_blk; b += GEMV_THREADS) {
        const int4 *q = (const int4 *)(s_q + b * 32);
        const int4 q0 = q[0], q1 = q[1];
        int s = 0;
        s = __builtin_amdgcn_sdot4(q0.x, 0x01010101, s, false); s = __builtin_amdgcn_sdot4(q0.y, 0x01010101, s, false);
        s = __builtin_amdgcn_sdot4(q0.z, 0x01010101, s, false); s = __builtin_amdgcn_sdot4(q0.w, 0x01010101, s, false);
        s = __builtin_amdgcn_sdot4(q1.x, 0x01010101, s, false); s = __builtin_amdgcn_sdot4(q1.y, 0x01010101, s, false);
        s = __builtin_amdgcn_sdot4(q1.z, 0x01010101, s, false); s = __builtin_amdgcn_sdot4(q1.w, 0x01010101, s, false);
        s_meta[b].y = s;
    }
}

// int32 dot of one Q4_0 block (4 dwords of packed nibbles) with 32 int8 activations
static __device__ __forceinline__ int dot_q4_block(const uint32_t n[4], const int4 x0, const int4 x1, int sumq) {
    const int xl[4] = {x0.x, x0.y, x0.z, x0.w}, xh[4] = {x1.x, x1.y, x1.z, x1.w};
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        s = __builtin_amdgcn_sdot4((int)(n[i] & 0x0F0F0F0Fu), xl[i], s, false);          // elements 4i..4i+3
        s = __builtin_amdgcn_sdot4((int)((n[i] >> 4) & 0x0F0F0F0Fu), xh[i], s, false);   // elements 16+4i..
    }
    return s - 8 * sumq;
}

static __device__ __forceinline__ int dot_q8_block(const uint32_t n[8], const int4 x0, const int4 x1) {
    int s = 0;
    s = __builtin_amdgcn_sdot4((int)n[0], x0.x, s, false); s = __builtin_amdgcn_sdot4((int)n[1], x0.y, s, false);
    s = __builtin_amdgcn_sdot4((int)n[2], x0.z, s, false); s = __builtin_amdgcn_sdot4((int)n[3], x0.w, s, false);
    s = __builtin_amdgcn_sdot4((int)n[4], x1.x, s, false); s = __builtin_amdgcn_sdot4((int)n[5], x1.y, s, false);
    s = __builtin_amdgcn_sdot4((int)n[6], x1.z, s, false); s = __builtin_amdgcn_sdot4((int)n[7], x1.w, s, false);
    return s;
}

// grid.x = number of row tiles; R rows per tile; requires K % 256 == 0 (rows 16-byte aligned,
// even block count).  LDS: [tile R*RB][s_q T*K][s_meta T*nblk*8].
template <int WT, int NT, bool DUMP>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_tile_kernel(const uint8_t *__restrict__ W, const uint8_t *__restrict__ xq,
                                                                 float *__restrict__ dst, const float *__restrict__ residual,
                                                                 int32_t *__restrict__ dump, int M, int K, int R, int64_t dst_stride) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int BLK = wt_traits<WT>::BLK;
    const int nblk = K / 32, npair = nblk / 2;
    const int RB = nblk * BLK;
    const int r0 = blockIdx.x * R;
    const int nrow = min(R, M - r0);
    const int tile_bytes = nrow * RB;
    uint8_t *s_tile = smem;
    int8_t *s_q = (int8_t *)(smem + (((size_t)R * RB + 15) & ~(size_t)15));
    int2 *s_meta = (int2 *)(s_q + (size_t)NT * K);

    // 1. put the whole weight tile in flight (registers), 2. stage activations, 3. tile -> LDS
    const uint8_t *src = W + (size_t)r0 * RB;
    uint4 regs[GEMV_MAX_ROUNDS];
#pragma unroll
    for (int i = 0; i < GEMV_MAX_ROUNDS; i++) {
        const int off = (i * GEMV_THREADS + threadIdx.x) * 16;
        if (off < tile_bytes) regs[i] = *(const uint4 *)(src + off);
    }
    stage_activations(xq, s_q, s_meta, NT * nblk);
#pragma unroll
    for (int i = 0; i < GEMV_MAX_ROUNDS; i++) {
        const int off = (i * GEMV_THREADS + threadIdx.x) * 16;
        if (off < tile_bytes) *(uint4 *)(s_tile + off) = regs[i];
    }
    __syncthreads();

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int r = wave; r < nrow; r += GEMV_WAVES) {
        const uint32_t *rowp = (const uint32_t *)(s_tile + (size_t)r * RB);
        float acc[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) acc[t] = 0.0f;
        for (int p = lane; p < npair; p += SPY_WAVE) {
            if constexpr (WT == SPY_HIP_Q4_0) {
                const uint32_t *wp = rowp + p * 9;
                uint32_t w[9];
#pragma unroll
                for (int i = 0; i < 9; i++) w[i] = wp[i];
                const float dA = h2f((uint16_t)(w[0] & 0xFFFFu)), dB = h2f((uint16_t)(w[4] >> 16));
                uint32_t a[4];
#pragma unroll
                for (int i = 0; i < 4; i++) a[i] = __builtin_amdgcn_alignbit(w[i + 1], w[i], 16);
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const int bA = t * nblk + 2 * p;
                    const int4 *xa = (const int4 *)(s_q + (size_t)bA * 32);
                    const int2 mA = s_meta[bA], mB = s_meta[bA + 1];
                    const int iA = dot_q4_block(a, xa[0], xa[1], mA.y);
                    const int iB = dot_q4_block(&w[5], xa[2], xa[3], mB.y);
                    if constexpr (DUMP) { dump[(size_t)(r0 + r) * nblk + 2 * p] = iA; dump[(size_t)(r0 + r) * nblk + 2 * p + 1] = iB; }
                    acc[t] = fmaf(dA * __int_as_float(mA.x), (float)iA, acc[t]);
                    acc[t] = fmaf(dB * __int_as_float(mB.x), (float)iB, acc[t]);
                }
            } else {
                const uint32_t *wp = rowp + p * 17;
                uint32_t w[17];
#pragma unroll
                for (int i = 0; i < 17; i++) w[i] = wp[i];
                const float dA = h2f((uint16_t)(w[0] & 0xFFFFu)), dB = h2f((uint16_t)(w[8] >> 16));
                uint32_t a[8];
#pragma unroll
                for (int i = 0; i < 8; i++) a[i] = __builtin_amdgcn_alignbit(w[i + 1], w[i], 16);
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const int bA = t * nblk + 2 * p;
                    const int4 *xa = (const int4 *)(s_q + (size_t)bA * 32);
                    const int2 mA = s_meta[bA], mB = s_meta[bA + 1];
                    const int iA = dot_q8_block(a, xa[0], xa[1]);
                    const int iB = dot_q8_block(&w[9], xa[2], xa[3]);
                    if constexpr (DUMP) { dump[(size_t)(r0 + r) * nblk + 2 * p] = iA; dump[(size_t)(r0 + r) * nblk + 2 * p + 1] = iB; }
                    acc[t] = fmaf(dA * __int_as_float(mA.x), (float)iA, acc[t]);
                    acc[t] = fmaf(dB * __int_as_float(mB.x), (float)iB, acc[t]);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const float s = wave_sum(acc[t]);
            if (lane == 0) {
                const size_t o = (size_t)t * dst_stride + (r0 + r);
                dst[o] = residual ? s + residual[o] : s;
            }
        }
    }
}

// ---- generic path: any K % 32 == 0 (Q4_0 / Q8_0) or K % 256 == 0 (Q4_K / Q6_K); one wave per
// row, lanes stride over Q8_0 activation blocks and read weights from global memory bytewise.
// Used for shapes the tiled kernel does not take and for the K-quants.
static __device__ __forceinline__ void q4k_scale_min(int j, const uint8_t *s, int &sc, int &m) {
    if (j < 4) { sc = s[j] & 63; m = s[j + 4] & 63; }
    else { sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4); m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4); }
}

template <int WT, bool DUMP>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_generic_kernel(const uint8_t *__restrict__ W, const uint8_t *__restrict__ xq,
                                                                    float *__restrict__ dst, const float *__restrict__ residual,
                                                                    int32_t *__restrict__ dump, int M, int K, int T, int64_t dst_stride) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int m = blockIdx.x * GEMV_WAVES + wave;
    if (m >= M) return;
    const int nblk = K / 32;                               // Q8_0 activation blocks per row
    const uint8_t *wrow = W + (size_t)m * spy_row_size(WT, K);
    for (int t = 0; t < T; t++) {
        const blk_q8_0 *x = (const blk_q8_0 *)(xq + (size_t)t * nblk * 34);
        float acc = 0.0f;
        for (int b = lane; b < nblk; b += SPY_WAVE) {
            const float dx = h2f(x[b].d);
            const int8_t *q = x[b].qs;
            if constexpr (WT == SPY_HIP_Q4_0) {
                const blk_q4_0 *w = (const blk_q4_0 *)wrow + b;
                int s = 0;
                for (int j = 0; j < 16; j++) s += ((w->qs[j] & 0x0F) - 8) * q[j] + ((w->qs[j] >> 4) - 8) * q[j + 16];
                if constexpr (DUMP) dump[(size_t)m * nblk + b] = s;
                acc = fmaf(h2f(w->d) * dx, (float)s, acc);
            } else if constexpr (WT == SPY_HIP_Q8_0) {
                const blk_q8_0 *w = (const blk_q8_0 *)wrow + b;
                int s = 0;
                for (int j = 0; j < 32; j++) s += (int)w->qs[j] * q[j];
                if constexpr (DUMP) dump[(size_t)m * nblk + b] = s;
                acc = fmaf(h2f(w->d) * dx, (float)s, acc);
            } else if constexpr (WT == SPY_HIP_Q4_K) {
                // sub-block j = b % 8 of super-block b / 8: value = d*sc*q - dmin*m
                const blk_q4_k *w = (const blk_q4_k *)wrow + (b >> 3);
                const int j = b & 7;
                int sc, mn; q4k_scale_min(j, w->scales, sc, mn);
                const uint8_t *qs = w->qs + 32 * (j >> 1);
                int isum = 0, bsum = 0;
                for (int l = 0; l < 32; l++) { const int v = (j & 1) ? (qs[l] >> 4) : (qs[l] & 0x0F); isum += v * q[l]; bsum += q[l]; }
                if constexpr (DUMP) dump[(size_t)m * nblk + b] = isum;
                acc = fmaf(dx, h2f(w->d) * (float)(sc * isum) - h2f(w->dmin) * (float)(mn * bsum), acc);
            } else {
                // Q6_K: activation block t8 = b % 8 covers 16-element sub-blocks 2*t8, 2*t8+1
                const blk_q6_k *w = (const blk_q6_k *)wrow + (b >> 3);
                const int t8 = b & 7, half = t8 >> 2, grp = t8 & 3;
                const uint8_t *ql = w->ql + 64 * half + 32 * (grp & 1), *qh = w->qh + 32 * half;
                int s = 0;
                for (int hh = 0; hh < 2; hh++) {
                    int isum = 0;
                    for (int l = 16 * hh; l < 16 * hh + 16; l++) {
                        const int lo = (grp < 2) ? (ql[l] & 0x0F) : (ql[l] >> 4);
                        const int hi = (qh[l] >> (2 * grp)) & 3;
                        isum += ((lo | (hi << 4)) - 32) * q[l];
                    }
                    if constexpr (DUMP) dump[(size_t)m * (nblk * 2) + 2 * b + hh] = isum;
                    s += (int)w->scales[2 * t8 + hh] * isum;
                }
                acc = fmaf(dx * h2f(w->d), (float)s, acc);
            }
        }
        acc = wave_sum(acc);
        if (lane == 0) {
            const size_t o = (size_t)t * dst_stride + m;
            dst[o] = residual ? acc + residual[o] : acc;
        }
    }
}

static int tile_rows(int wtype, int64_t K) {
    const int64_t RB = spy_row_size(wtype, K);
    int64_t g = GEMV_TILE_TARGET / (GEMV_WAVES * RB);
    if (g < 1) g = 1;
    return (int)(GEMV_WAVES * g);
}

template <int WT, int NT, bool DUMP>
static int launch_tile(hipStream_t st, const void *w, const void *xq, float *dst, const float *residual, int32_t *dump,
                       int64_t M, int64_t K, int64_t dst_stride) {
    const int R = tile_rows(WT, K);
    const int64_t RB = spy_row_size(WT, K);
    if (R * RB > (int64_t)GEMV_MAX_ROUNDS * GEMV_THREADS * 16) return SPY_HIP_EUNSUPPORTED;
    const size_t lds = (((size_t)R * RB + 15) & ~(size_t)15) + (size_t)NT * K + (size_t)NT * (K / 32) * 8;
    if (lds > 160 * 1024) return SPY_HIP_EUNSUPPORTED;
    auto kern = gemv_tile_kernel<WT, NT, DUMP>;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
    }
    const unsigned grid = (unsigned)((M + R - 1) / R);
    kern<<<dim3(grid), dim3(GEMV_THREADS), lds, st>>>((const uint8_t *)w, (const uint8_t *)xq, dst, residual, dump, (int)M, (int)K, R, dst_stride);
    return SPY_LAUNCH_RC();
}

template <int WT, bool DUMP>
static int launch_generic(hipStream_t st, const void *w, const void *xq, float *dst, const float *residual, int32_t *dump,
                          int64_t M, int64_t K, int64_t T, int64_t dst_stride) {
    const unsigned grid = (unsigned)((M + GEMV_WAVES - 1) / GEMV_WAVES);
    gemv_generic_kernel<WT, DUMP><<<dim3(grid), dim3(GEMV_THREADS), 0, st>>>((const uint8_t *)w, (const uint8_t *)xq, dst, residual, dump,
                                                                              (int)M, (int)K, (int)T, dst_stride);
    return SPY_LAUNCH_RC();
}

template <int WT>
static int gemv_tiled_cols(hipStream_t st, const void *w, const uint8_t *xq, float *dst, const float *residual,
                           int64_t M, int64_t K, int64_t T, int64_t dst_stride) {
    // weights are re-read once per group of up to 8 activation rows
    const int64_t xrow = (K / 32) * 34;
    int64_t t = 0;
    while (t < T) {
        const int64_t left = T - t;
        int rc;
        const float *res = residual ? residual + t * dst_stride : nullptr;
        float *d = dst + t * dst_stride;
        const uint8_t *x = xq + t * xrow;
        if (left >= 8)      { rc = launch_tile<WT, 8, false>(st, w, x, d, res, nullptr, M, K, dst_stride); t += 8; }
        else if (left >= 4) { rc = launch_tile<WT, 4, false>(st, w, x, d, res, nullptr, M, K, dst_stride); t += 4; }
        else if (left >= 2) { rc = launch_tile<WT, 2, false>(st, w, x, d, res, nullptr, M, K, dst_stride); t += 2; }
        else                { rc = launch_tile<WT, 1, false>(st, w, x, d, res, nullptr, M, K, dst_stride); t += 1; }
        if (rc) return rc;
    }
    return 0;
}

static int check_gemv_args(int wtype, const void *w, const void *xq, const void *dst, int64_t M, int64_t K, int64_t T) {
    SPY_CHECK_ARG(w && xq && dst && M > 0 && K > 0 && T > 0);
    SPY_CHECK_ARG(M < (1ll << 30) && K < (1ll << 24) && T < (1ll << 24));
    SPY_CHECK_ARG(((uintptr_t)w % 16) == 0 && ((uintptr_t)xq % 2) == 0 && ((uintptr_t)dst % 4) == 0);
    switch (wtype) {
    case SPY_HIP_Q4_0: case SPY_HIP_Q8_0: SPY_CHECK_ARG(K % 32 == 0); break;
    case SPY_HIP_Q4_K: case SPY_HIP_Q6_K: SPY_CHECK_ARG(K % 256 == 0); break;
    default: return SPY_HIP_EUNSUPPORTED;
    }
    return 0;
}

extern "C" int spy_hip_gemv_q8_0act(void *stream, int wtype, const void *w, const void *xq, float *dst, const float *residual,
                                    int64_t M, int64_t K, int64_t T, int64_t dst_stride) {
    int rc = check_gemv_args(wtype, w, xq, dst, M, K, T);
    if (rc) return rc;
    SPY_CHECK_ARG(dst_stride >= M);
    hipStream_t st = (hipStream_t)stream;
    const bool tiled = (K % 256 == 0);
    switch (wtype) {
    case SPY_HIP_Q4_0:
        return tiled ? gemv_tiled_cols<SPY_HIP_Q4_0>(st, w, (const uint8_t *)xq, dst, residual, M, K, T, dst_stride)
                     : launch_generic<SPY_HIP_Q4_0, false>(st, w, xq, dst, residual, nullptr, M, K, T, dst_stride);
    case SPY_HIP_Q8_0:
        return tiled ? gemv_tiled_cols<SPY_HIP_Q8_0>(st, w, (const uint8_t *)xq, dst, residual, M, K, T, dst_stride)
                     : launch_generic<SPY_HIP_Q8_0, false>(st, w, xq, dst, residual, nullptr, M, K, T, dst_stride);
    case SPY_HIP_Q4_K: return launch_generic<SPY_HIP_Q4_K, false>(st, w, xq, dst, residual, nullptr, M, K, T, dst_stride);
    case SPY_HIP_Q6_K: return launch_generic<SPY_HIP_Q6_K, false>(st, w, xq, dst, residual, nullptr, M, K, T, dst_stride);
    }
    return SPY_HIP_EUNSUPPORTED;
}

// Same kernels with the DUMP switch on: every lane also stores the int32 dot of each block it
// computes, so the parity test sees the integers the GEMV itself accumulates.
extern "C" int spy_hip_block_dots(void *stream, int wtype, const void *w, const void *xq, int32_t *out, int64_t M, int64_t K) {
    int rc = check_gemv_args(wtype, w, xq, out, M, K, 1);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    // the float result goes to a throw-away slot behind the dump: out must hold M*nsub + M ints
    const int64_t nsub = (wtype == SPY_HIP_Q6_K) ? K / 16 : K / 32;
    float *sink = (float *)(out + M * nsub);
    const bool tiled = (K % 256 == 0);
    switch (wtype) {
    case SPY_HIP_Q4_0:
        return tiled ? launch_tile<SPY_HIP_Q4_0, 1, true>(st, w, xq, sink, nullptr, out, M, K, M)
                     : launch_generic<SPY_HIP_Q4_0, true>(st, w, xq, sink, nullptr, out, M, K, 1, M);
    case SPY_HIP_Q8_0:
        return tiled ? launch_tile<SPY_HIP_Q8_0, 1, true>(st, w, xq, sink, nullptr, out, M, K, M)
                     : launch_generic<SPY_HIP_Q8_0, true>(st, w, xq, sink, nullptr, out, M, K, 1, M);
    case SPY_HIP_Q4_K: return launch_generic<SPY_HIP_Q4_K, true>(st, w, xq, sink, nullptr, out, M, K, 1, M);
    case SPY_HIP_Q6_K: return launch_generic<SPY_HIP_Q6_K, true>(st, w, xq, sink, nullptr, out, M, K, 1, M);
    }
    return SPY_HIP_EUNSUPPORTED;
}
