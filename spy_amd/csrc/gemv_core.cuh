// Device-side building blocks of the quantized matrix x vector kernels (Q4_0 / Q8_0 weights,
// Q8_0 activations).  Shared by the stand-alone GEMV launchers and the fused token-loop kernels.
//
// Work split: LPR (16, 32 or 64) lanes share one weight row, a wave covers 64/LPR rows at once
// and a 256-thread workgroup 4x that.  A lane owns block PAIRS p = it*LPR + l of its row (a pair
// of native blocks is 36 / 68 bytes: 4-byte aligned, loaded straight from HBM as dwords, no LDS
// staging of weights).  All of a tile's weight loads are issued before anything else so the HBM
// latency overlaps the activation staging; the reduction over the LPR lanes runs on DPP.
//
// Activations live in LDS in a "staged" form: int8 q[K] (16-byte aligned) followed by one
// {float scale, int32 sum(q)} per 32-element block; sum(q) folds the -8 offset of the Q4_0
// nibbles: sum((n-8)*q) = sum(n*q) - 8*sum(q), keeping the int32 block dot exact.
#pragma once

#include "common.cuh"

#ifndef GEMV_THREADS
#define GEMV_THREADS 256
#endif
#define GEMV_WAVES (GEMV_THREADS / 64)
// float4 of input per thread that cover K elements in the staging prologues
#define GEMV_SIT_FOR(K) (((K) + 4 * GEMV_THREADS - 1) / (4 * GEMV_THREADS))

// agent-scope accesses: coherent between compute units and XCDs
static __device__ __forceinline__ float ldc(const float *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
static __device__ __forceinline__ uint32_t ldc(const uint32_t *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
static __device__ __forceinline__ void stc(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
static __device__ __forceinline__ void stc(uint32_t *p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
static __device__ __forceinline__ void stc(uint16_t *p, uint16_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
static __device__ __forceinline__ float4 ldc4(const float *p) { return make_float4(ldc(p), ldc(p + 1), ldc(p + 2), ldc(p + 3)); }

template <int WT> struct wt_traits;
template <> struct wt_traits<SPY_HIP_Q4_0> { static constexpr int BLK = 18, PAIR_DW = 9; };
template <> struct wt_traits<SPY_HIP_Q8_0> { static constexpr int BLK = 34, PAIR_DW = 17; };
// K-quants (64 lanes per row only): a lane's unit is a quarter super-block = 64 elements, the same
// span as a block pair.  Q4_K: the 16-byte header {d, dmin, scales[12]} + the 32 nibble bytes of sub-blocks
// 2j, 2j+1.  Q6_K (super-blocks only 2-byte aligned; the hardware takes unaligned vector loads): three
// 16-byte chunks (ql, ql + 32, qh), 8 scale bytes and d.
template <> struct wt_traits<SPY_HIP_Q4_K> { static constexpr int PAIR_DW = 12; };
template <> struct wt_traits<SPY_HIP_Q6_K> { static constexpr int PAIR_DW = 15; };
#define GEMV_NIT_MAX 4        // block pairs per lane per row tile: 1..4 (exact value is a template parameter)

template <int CTRL> static __device__ __forceinline__ float dpp_add(float v) {
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL> static __device__ __forceinline__ float dpp_max(float v) {
    return fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true)));
}
template <int CTRL> static __device__ __forceinline__ int dpp_add_i(int v) {
    return v + __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
// Sum over each aligned group of LPR lanes; every lane of the group receives the total.
template <int LPR> static __device__ __forceinline__ float group_sum(float v) {
    v = dpp_add<0xB1>(v);    // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);    // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);   // row_half_mirror
    v = dpp_add<0x140>(v);   // row_mirror: all 16 lanes of a DPP row now hold the row total
    if constexpr (LPR >= 32) v += __shfl_xor(v, 16, SPY_WAVE);
    if constexpr (LPR >= 64) v += __shfl_xor(v, 32, SPY_WAVE);
    return v;
}
// Sum over the whole wave for ONE reader: after the in-row steps every lane of a 16-lane DPP row holds
// its row total R0..R3; row_bcast15 adds R0 into row 1 and R2 into row 3, row_bcast31 adds R0+R1 into
// rows 2, 3: lanes 48..63 end up with (R2+R3)+(R0+R1), the same additions as group_sum<64>, without
// the two LDS permutes.  Only lane 63 (any of 48..63) may use the result.
static __device__ __forceinline__ float wave_total_lane63(float v) {
    v = dpp_add<0xB1>(v); v = dpp_add<0x4E>(v); v = dpp_add<0x141>(v); v = dpp_add<0x140>(v);
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, false));   // row_bcast15 -> rows 1, 3
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xC, 0xF, false));   // row_bcast31 -> rows 2, 3
    return v;
}
// max / sum over aligned groups of 8 lanes (one Q8_0 block = 8 lanes x 4 floats)
static __device__ __forceinline__ float oct_max(float v) {
    v = dpp_max<0xB1>(v); v = dpp_max<0x4E>(v); v = dpp_max<0x141>(v);
    return v;
}
static __device__ __forceinline__ int oct_sum_i(int v) {
    v = dpp_add_i<0xB1>(v); v = dpp_add_i<0x4E>(v); v = dpp_add_i<0x141>(v);
    return v;
}

// One staged activation column in LDS.  The 64 int8 of block pair p are kept as four 16-byte parts,
// part j at byte (j * (npair + 1) + p) * 16: consecutive lanes own consecutive pairs, so each
// 128-bit LDS read of a wave touches consecutive words (no bank conflicts), and the +1 skews the
// four parts over different banks for the staging writes.
struct staged_act {
    const int8_t *q;         // K + 64 bytes, swizzled as above
    const int2 *meta;        // K/32 x {bits(float scale), sum(q)}
};
static __host__ __device__ inline size_t staged_q_bytes(int64_t K) { return (size_t)K + 64; }
static __host__ __device__ inline size_t staged_bytes(int64_t K) { return staged_q_bytes(K) + (size_t)(K / 32) * 8; }
// dword index in LDS of natural dword i (= element index / 4) of the activation vector
static __device__ __forceinline__ int act_dw(int i, int npair) { return (((((i >> 2) & 3) * (npair + 1)) + (i >> 4)) << 2) + (i & 3); }
static __device__ __forceinline__ const int4 *act_part(const int8_t *q, int p, int j, int npair) {
    return (const int4 *)(q + (size_t)(j * (npair + 1) + p) * 16);
}

// ---- activation staging --------------------------------------------------------------------

// native Q8_0 blocks (34 bytes, 2-byte aligned) -> staged LDS form. Ends with __syncthreads().
template <int THREADS = GEMV_THREADS>
static __device__ __forceinline__ void stage_native_q8(const uint8_t *__restrict__ xq, int8_t *s_q, int2 *s_meta, int nblk) {
    const uint16_t *src = (const uint16_t *)xq;
    const int total_h = nblk * 17;
    for (int h = threadIdx.x; h < total_h; h += THREADS) {
        const int b = h / 17, w = h - b * 17;
        const uint16_t v = src[h];
        if (w == 0) s_meta[b].x = __float_as_int(h2f(v));
        else { const int hw = b * 16 + (w - 1); ((uint16_t *)s_q)[2 * act_dw(hw >> 1, nblk >> 1) + (hw & 1)] = v; }
    }
    __syncthreads();
    for (int b = threadIdx.x; b < nblk; b += THREADS) {
        const int4 q0 = *act_part(s_q, b >> 1, 2 * (b & 1), nblk >> 1), q1 = *act_part(s_q, b >> 1, 2 * (b & 1) + 1, nblk >> 1);
        int s = 0;
        s = __builtin_amdgcn_sdot4(q0.x, 0x01010101, s, false); s = __builtin_amdgcn_sdot4(q0.y, 0x01010101, s, false);
        s = __builtin_amdgcn_sdot4(q0.z, 0x01010101, s, false); s = __builtin_amdgcn_sdot4(q0.w, 0x01010101, s, false);
        s = __builtin_amdgcn_sdot4(q1.x, 0x01010101, s, false); s = __builtin_amdgcn_sdot4(q1.y, 0x01010101, s, false);
        s = __builtin_amdgcn_sdot4(q1.z, 0x01010101, s, false); s = __builtin_amdgcn_sdot4(q1.w, 0x01010101, s, false);
        s_meta[b].y = s;
    }
    __syncthreads();
}

// The same in two steps, so that the activation loads can be requested BEFORE the first weight rows (the
// compute unit serves its memory requests in order: activations requested behind the rows arrive behind
// them) and turned into the staged form afterwards.  The row must be 4-byte aligned (nblk even); a thread
// holds NDW dwords, NDW * THREADS >= nblk * 17 / 2.
template <int THREADS, int NDW>
static __device__ __forceinline__ void stage_native_q8_load(const uint8_t *__restrict__ xq, int nblk, uint32_t (&r)[NDW]) {
    const uint32_t *src = (const uint32_t *)xq;
    const int total = (nblk * 17) >> 1;
#pragma unroll
    for (int i = 0; i < NDW; i++) r[i] = src[min((int)threadIdx.x + i * THREADS, total - 1)];
}
template <int THREADS, int NDW>
static __device__ __forceinline__ void stage_native_q8_finish(const uint32_t (&r)[NDW], int8_t *s_q, int2 *s_meta, int nblk) {
    const int total = (nblk * 17) >> 1;
#pragma unroll
    for (int i = 0; i < NDW; i++) {
        const int dw = (int)threadIdx.x + i * THREADS;
        if (dw < total) {
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const int h = 2 * dw + e, b = h / 17, w = h - b * 17;
                const uint16_t v = (uint16_t)(e ? r[i] >> 16 : r[i] & 0xFFFFu);
                if (w == 0) s_meta[b].x = __float_as_int(h2f(v));
                else { const int hw = b * 16 + (w - 1); ((uint16_t *)s_q)[2 * act_dw(hw >> 1, nblk >> 1) + (hw & 1)] = v; }
            }
        }
    }
    __syncthreads();
    for (int b = threadIdx.x; b < nblk; b += THREADS) {
        const int4 q0 = *act_part(s_q, b >> 1, 2 * (b & 1), nblk >> 1), q1 = *act_part(s_q, b >> 1, 2 * (b & 1) + 1, nblk >> 1);
        int s = 0;
        s = __builtin_amdgcn_sdot4(q0.x, 0x01010101, s, false); s = __builtin_amdgcn_sdot4(q0.y, 0x01010101, s, false);
        s = __builtin_amdgcn_sdot4(q0.z, 0x01010101, s, false); s = __builtin_amdgcn_sdot4(q0.w, 0x01010101, s, false);
        s = __builtin_amdgcn_sdot4(q1.x, 0x01010101, s, false); s = __builtin_amdgcn_sdot4(q1.y, 0x01010101, s, false);
        s = __builtin_amdgcn_sdot4(q1.z, 0x01010101, s, false); s = __builtin_amdgcn_sdot4(q1.w, 0x01010101, s, false);
        s_meta[b].y = s;
    }
    __syncthreads();
}

// Quantize 4 consecutive floats held by each of 8 consecutive lanes (one 32-element block) the
// way Quantizator<FP32,Q8_0>::transform does (vec_convert.h:197-260 in the Spy tree): amax,
// d = amax/127 (stored as fp16), id = 127/amax, q = rint(x*id) saturated to int8.
// Returns the 4 quants packed in a dword; lane 0 of the octet also gets {scale bits, sum q}.
static __device__ __forceinline__ uint32_t quantize_oct(const float4 v, int2 &meta) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = oct_max(amax);
    const float d  = amax / 127.0f;
    const float id = (amax != 0.0f) ? 127.0f / amax : 0.0f;
    int q0 = (int)rintf(v.x * id), q1 = (int)rintf(v.y * id), q2 = (int)rintf(v.z * id), q3 = (int)rintf(v.w * id);
    q0 = min(127, max(-128, q0)); q1 = min(127, max(-128, q1)); q2 = min(127, max(-128, q2)); q3 = min(127, max(-128, q3));
    const int s = oct_sum_i(q0 + q1 + q2 + q3);
    meta.x = __float_as_int(h2f(f2h(d)));
    meta.y = s;
    return (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) | ((uint32_t)(q2 & 0xFF) << 16) | ((uint32_t)(q3 & 0xFF) << 24);
}

// f32 vector -> staged LDS form, one pass (no normalisation).  K % 32 == 0, x 16-byte aligned.
// Ends with __syncthreads().
static __device__ __forceinline__ void stage_f32_plain(const float *__restrict__ x, int8_t *s_q, int2 *s_meta, int K) {
    // 8 consecutive lanes hold one 32-element block; the trip count is uniform per octet
    for (int i = threadIdx.x; i < K / 4; i += GEMV_THREADS) {
        int2 meta;
        const uint32_t q = quantize_oct(((const float4 *)x)[i], meta);
        ((uint32_t *)s_q)[act_dw(i, K >> 6)] = q;
        if ((threadIdx.x & 7) == 0) s_meta[i >> 3] = meta;
    }
    __syncthreads();
}

// The same with the global loads split off, so that a kernel can issue them BEFORE its weight-tile
// loads: the memory counter retires loads in order, and a prologue whose loads were issued after the
// tiles' would wait for the tiles as well.  SIT float4 per thread: K <= 1024*SIT.
template <int SIT> struct plain_regs { float4 x[SIT]; };

template <int SIT>
static __device__ __forceinline__ void stage_plain_load(plain_regs<SIT> &r, const float *__restrict__ x, int K) {
#pragma unroll
    for (int j = 0; j < SIT; j++) {
        const int i = min((int)threadIdx.x + j * GEMV_THREADS, K / 4 - 1);      // unconditional (see load_tile)
        r.x[j] = ((const float4 *)x)[i];
    }
}

template <int SIT>
static __device__ __forceinline__ void stage_plain_finish(const plain_regs<SIT> &r, int8_t *s_q, int2 *s_meta, int K) {
#pragma unroll
    for (int j = 0; j < SIT; j++) {
        const int i = threadIdx.x + j * GEMV_THREADS;
        if (i < K / 4) {
            int2 meta;
            const uint32_t q = quantize_oct(r.x[j], meta);
            ((uint32_t *)s_q)[act_dw(i, K >> 6)] = q;
            if ((threadIdx.x & 7) == 0) s_meta[i >> 3] = meta;
        }
    }
    __syncthreads();
}

// RMS-normalised, weighted f32 vector -> staged LDS form.  NormRMS as the reference:
// scale = 1/sqrt(sum(x^2)/K + eps), y = (x*scale)*w (non-linear.cpp:216-219 and the separate Mul
// node, attention.cpp:274-282 in the Spy tree).  Split in two so that a kernel can put the global
// loads in flight first (load), do other work, and finish later; x and w stay in registers
// (SIT float4 each per thread: K <= 1024*SIT).  finish ends with __syncthreads().
template <int SIT> struct stage_regs { float4 x[SIT]; float4 w[SIT]; };

template <int SIT>
static __device__ __forceinline__ void stage_norm_load(stage_regs<SIT> &r, const float *__restrict__ x, const float *__restrict__ normw, int K) {
#pragma unroll
    for (int j = 0; j < SIT; j++) {
        const int i = min((int)threadIdx.x + j * GEMV_THREADS, K / 4 - 1);      // unconditional (see load_tile)
        r.x[j] = ((const float4 *)x)[i]; r.w[j] = ((const float4 *)normw)[i];
    }
}

template <int SIT>
static __device__ __forceinline__ void stage_norm_finish(stage_regs<SIT> &r, float eps, int8_t *s_q, int2 *s_meta, int K, float *s_red) {
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < SIT; j++) {
        if (threadIdx.x + j * GEMV_THREADS < K / 4) {
            const float4 v = r.x[j];
            acc = fmaf(v.x, v.x, acc); acc = fmaf(v.y, v.y, acc); acc = fmaf(v.z, v.z, acc); acc = fmaf(v.w, v.w, acc);
        }
    }
    acc = group_sum<64>(acc);
    if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = acc;
    __syncthreads();
    float sum = 0.0f;
#pragma unroll
    for (int w = 0; w < GEMV_WAVES; w += 4) sum += (s_red[w] + s_red[w + 1]) + (s_red[w + 2] + s_red[w + 3]);
    const float scale = 1.0f / sqrtf(sum / (float)K + eps);
#pragma unroll
    for (int j = 0; j < SIT; j++) {
        const int i = threadIdx.x + j * GEMV_THREADS;
        if (i < K / 4) {
            float4 v = r.x[j];
            const float4 w = r.w[j];
            v.x = (v.x * scale) * w.x; v.y = (v.y * scale) * w.y; v.z = (v.z * scale) * w.z; v.w = (v.w * scale) * w.w;
            int2 meta;
            const uint32_t q = quantize_oct(v, meta);
            ((uint32_t *)s_q)[act_dw(i, K >> 6)] = q;
            if ((threadIdx.x & 7) == 0) s_meta[i >> 3] = meta;
        }
    }
    __syncthreads();
}

// ---- weight tiles --------------------------------------------------------------------------

template <int WT, int NIT> struct wtile { uint32_t w[NIT][wt_traits<WT>::PAIR_DW]; };

// Branch-free on purpose: the memory counter retires loads in order, and the compiler can only
// wait for "all but the N youngest" loads when those N are issued unconditionally.  Lanes whose
// pair index lies beyond the row re-read the last pair (a cache hit that dot_tile ignores).
template <int WT, int LPR, int NIT>
static __device__ __forceinline__ void load_tile(wtile<WT, NIT> &t, const uint8_t *__restrict__ rowp, int npair, int l) {
    constexpr int DW = wt_traits<WT>::PAIR_DW;
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int p = min(it * LPR + l, npair - 1);
        if constexpr (WT == SPY_HIP_Q4_K) {
            static_assert(WT != SPY_HIP_Q4_K || LPR == 64, "K-quant tiles use 64 lanes per row");
            const uint8_t *sb = rowp + (size_t)(p >> 2) * 144;
            const uint4 hdr = *(const uint4 *)sb, q0 = *(const uint4 *)(sb + 16 + 32 * (p & 3)), q1 = *(const uint4 *)(sb + 32 + 32 * (p & 3));
            t.w[it][0] = hdr.x; t.w[it][1] = hdr.y; t.w[it][2] = hdr.z; t.w[it][3] = hdr.w;
            t.w[it][4] = q0.x; t.w[it][5] = q0.y; t.w[it][6] = q0.z; t.w[it][7] = q0.w;
            t.w[it][8] = q1.x; t.w[it][9] = q1.y; t.w[it][10] = q1.z; t.w[it][11] = q1.w;
        } else if constexpr (WT == SPY_HIP_Q6_K) {
            static_assert(WT != SPY_HIP_Q6_K || LPR == 64, "K-quant tiles use 64 lanes per row");
            // lane (n = half of the super-block, e = 16-element slice): ql[64n + 16e ..], ql[64n + 32 + 16e ..], qh[32n + 16e ..], scales[8n ..]
            const int j = p & 3, n = j >> 1, e = j & 1;
            const uint8_t *sb = rowp + (size_t)(p >> 2) * 210;
            uint4 ca, cb, ch; uint2 cs;
            __builtin_memcpy(&ca, __builtin_assume_aligned(sb + 64 * n + 16 * e, 2), 16);
            __builtin_memcpy(&cb, __builtin_assume_aligned(sb + 64 * n + 32 + 16 * e, 2), 16);
            __builtin_memcpy(&ch, __builtin_assume_aligned(sb + 128 + 32 * n + 16 * e, 2), 16);
            __builtin_memcpy(&cs, __builtin_assume_aligned(sb + 192 + 8 * n, 2), 8);
            t.w[it][0] = ca.x; t.w[it][1] = ca.y; t.w[it][2] = ca.z; t.w[it][3] = ca.w;
            t.w[it][4] = cb.x; t.w[it][5] = cb.y; t.w[it][6] = cb.z; t.w[it][7] = cb.w;
            t.w[it][8] = ch.x; t.w[it][9] = ch.y; t.w[it][10] = ch.z; t.w[it][11] = ch.w;
            t.w[it][12] = cs.x; t.w[it][13] = cs.y;
            t.w[it][14] = *(const uint16_t *)(sb + 208);
        } else {
            const uint32_t *wp = (const uint32_t *)rowp + (size_t)p * DW;
#pragma unroll
            for (int i = 0; i < DW; i++) t.w[it][i] = wp[i];
        }
    }
}

static __device__ __forceinline__ int dot_q4_dwords(const uint32_t n0, const uint32_t n1, const uint32_t n2, const uint32_t n3,
                                                    const int4 xl, const int4 xh) {
    int s = 0;
    s = __builtin_amdgcn_sdot4((int)(n0 & 0x0F0F0F0Fu), xl.x, s, false); s = __builtin_amdgcn_sdot4((int)((n0 >> 4) & 0x0F0F0F0Fu), xh.x, s, false);
    s = __builtin_amdgcn_sdot4((int)(n1 & 0x0F0F0F0Fu), xl.y, s, false); s = __builtin_amdgcn_sdot4((int)((n1 >> 4) & 0x0F0F0F0Fu), xh.y, s, false);
    s = __builtin_amdgcn_sdot4((int)(n2 & 0x0F0F0F0Fu), xl.z, s, false); s = __builtin_amdgcn_sdot4((int)((n2 >> 4) & 0x0F0F0F0Fu), xh.z, s, false);
    s = __builtin_amdgcn_sdot4((int)(n3 & 0x0F0F0F0Fu), xl.w, s, false); s = __builtin_amdgcn_sdot4((int)((n3 >> 4) & 0x0F0F0F0Fu), xh.w, s, false);
    return s;
}
static __device__ __forceinline__ int dot_q8_dwords(const uint32_t *n, const int4 x0, const int4 x1) {
    int s = 0;
    s = __builtin_amdgcn_sdot4((int)n[0], x0.x, s, false); s = __builtin_amdgcn_sdot4((int)n[1], x0.y, s, false);
    s = __builtin_amdgcn_sdot4((int)n[2], x0.z, s, false); s = __builtin_amdgcn_sdot4((int)n[3], x0.w, s, false);
    s = __builtin_amdgcn_sdot4((int)n[4], x1.x, s, false); s = __builtin_amdgcn_sdot4((int)n[5], x1.y, s, false);
    s = __builtin_amdgcn_sdot4((int)n[6], x1.z, s, false); s = __builtin_amdgcn_sdot4((int)n[7], x1.w, s, false);
    return s;
}

// Partial dot of the lane's pairs of one weight row with NT staged activation columns.
// dump (optional): int32 dot of every block, row-major [nblk] for activation column 0.
// One block pair of a weight row (w: its PAIR_DW dwords) with the matching 64 int8 activations
// (x0..x3: 16 bytes each) and their meta {scale bits, sum q} x 2: the two exact int32 block dots
// (optionally dumped), scaled and accumulated like the reference's fma (vec_dot.h:76-79).
// byte k (0..11) of three dwords
static __device__ __forceinline__ uint32_t byte_of3(uint32_t a, uint32_t b, uint32_t c, int k) {
    const uint32_t w = k < 4 ? a : (k < 8 ? b : c);
    return (w >> (8 * (k & 3))) & 0xFFu;
}
// 4 packed 6-bit values (0..63 per byte) -> 4 int8 of (v - 32)
static __device__ __forceinline__ uint32_t q6_m32(uint32_t v) { return (v + 0x60606060u) ^ 0x80808080u; }

template <int WT>
static __device__ __forceinline__ float dot_pair(const uint32_t *w, const int4 x0, const int4 x1, const int4 x2, const int4 x3, const int4 mm, const int4 mm2,
                                                 int p, float acc, int32_t *dump2) {
    if constexpr (WT == SPY_HIP_Q4_K) {
        // sub-blocks a = 2j (low nibbles) and a + 1 (high nibbles) of the super-block; 6-bit scale / min pairs
        // from scales[12]; value = d*sc*q - dmin*m (k-quant.h:101-111 holds the layout only)
        const int j = p & 3, a = 2 * j;
        const float d = h2f((uint16_t)(w[0] & 0xFFFFu)), dmin = h2f((uint16_t)(w[0] >> 16));
        int scA, mA, scB, mB;
        if (j < 2) {
            scA = byte_of3(w[1], w[2], w[3], a) & 63;     mA = byte_of3(w[1], w[2], w[3], a + 4) & 63;
            scB = byte_of3(w[1], w[2], w[3], a + 1) & 63; mB = byte_of3(w[1], w[2], w[3], a + 5) & 63;
        } else {
            const uint32_t hA = byte_of3(w[1], w[2], w[3], a + 4), hB = byte_of3(w[1], w[2], w[3], a + 5);
            scA = (hA & 0x0F) | ((byte_of3(w[1], w[2], w[3], a - 4) >> 6) << 4); mA = (hA >> 4) | ((byte_of3(w[1], w[2], w[3], a) >> 6) << 4);
            scB = (hB & 0x0F) | ((byte_of3(w[1], w[2], w[3], a - 3) >> 6) << 4); mB = (hB >> 4) | ((byte_of3(w[1], w[2], w[3], a + 1) >> 6) << 4);
        }
        int iA = 0, iB = 0;
        const int xa[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w}, xb[8] = {x2.x, x2.y, x2.z, x2.w, x3.x, x3.y, x3.z, x3.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            iA = __builtin_amdgcn_sdot4((int)(w[4 + i] & 0x0F0F0F0Fu), xa[i], iA, false);
            iB = __builtin_amdgcn_sdot4((int)((w[4 + i] >> 4) & 0x0F0F0F0Fu), xb[i], iB, false);
        }
        if (dump2) { dump2[0] = iA; dump2[1] = iB; }
        // 24-bit multiplies (full rate): |i| <= 32 * 15 * 127, |sum q_x| <= 32 * 127, scales below 64
        acc = fmaf(__int_as_float(mm.x), d * (float)__mul24(scA, iA) - dmin * (float)__mul24(mA, mm.y), acc);
        acc = fmaf(__int_as_float(mm.z), d * (float)__mul24(scB, iB) - dmin * (float)__mul24(mB, mm.w), acc);
        return acc;
    } else if constexpr (WT == SPY_HIP_Q6_K) {
        // lane (n, e): elements l + 32 m, l in [16e, 16e + 16), m = 0..3 of half n: 6-bit quants from the low /
        // high nibbles of ql / ql + 32 and bit pairs 2m of qh, minus 32; scale = d * scales[8n + e + 2m]
        const uint32_t *qa = w, *qb = w + 4, *qh = w + 8;
        const uint32_t s0 = w[12], s1 = w[13];
        const int e = p & 1;
        const float d = h2f((uint16_t)(w[14] & 0xFFFFu));
        int isum[4] = {0, 0, 0, 0};
        const int xm[4][4] = {{x0.x, x0.y, x0.z, x0.w}, {x1.x, x1.y, x1.z, x1.w}, {x2.x, x2.y, x2.z, x2.w}, {x3.x, x3.y, x3.z, x3.w}};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t h = qh[i];
            isum[0] = __builtin_amdgcn_sdot4((int)q6_m32((qa[i] & 0x0F0F0F0Fu) | ((h & 0x03030303u) << 4)), xm[0][i], isum[0], false);
            isum[1] = __builtin_amdgcn_sdot4((int)q6_m32((qb[i] & 0x0F0F0F0Fu) | ((h & 0x0C0C0C0Cu) << 2)), xm[1][i], isum[1], false);
            isum[2] = __builtin_amdgcn_sdot4((int)q6_m32(((qa[i] >> 4) & 0x0F0F0F0Fu) | (h & 0x30303030u)), xm[2][i], isum[2], false);
            isum[3] = __builtin_amdgcn_sdot4((int)q6_m32(((qb[i] >> 4) & 0x0F0F0F0Fu) | ((h >> 2) & 0x30303030u)), xm[3][i], isum[3], false);
        }
        const float dx[4] = {__int_as_float(mm.x), __int_as_float(mm.z), __int_as_float(mm2.x), __int_as_float(mm2.z)};
#pragma unroll
        for (int m = 0; m < 4; m++) {
            const int k = e + 2 * m;                                     // scale byte of the half (0..7)
            const int sc = (int)(int8_t)(((k < 4 ? s0 : s1) >> (8 * (k & 3))) & 0xFFu);
            acc = fmaf(dx[m] * d, (float)__mul24(sc, isum[m]), acc);               // |isum| <= 16 * 32 * 127: 24-bit multiply (full rate)
        }
        return acc;
    } else {
    int iA, iB;
    float dA, dB;
    if constexpr (WT == SPY_HIP_Q4_0) {
        dA = h2f((uint16_t)(w[0] & 0xFFFFu)); dB = h2f((uint16_t)(w[4] >> 16));
        const uint32_t a0 = __builtin_amdgcn_alignbit(w[1], w[0], 16), a1 = __builtin_amdgcn_alignbit(w[2], w[1], 16);
        const uint32_t a2 = __builtin_amdgcn_alignbit(w[3], w[2], 16), a3 = __builtin_amdgcn_alignbit(w[4], w[3], 16);
        iA = dot_q4_dwords(a0, a1, a2, a3, x0, x1) - 8 * mm.y;
        iB = dot_q4_dwords(w[5], w[6], w[7], w[8], x2, x3) - 8 * mm.w;
    } else {
        dA = h2f((uint16_t)(w[0] & 0xFFFFu)); dB = h2f((uint16_t)(w[8] >> 16));
        uint32_t a[8];
#pragma unroll
        for (int i = 0; i < 8; i++) a[i] = __builtin_amdgcn_alignbit(w[i + 1], w[i], 16);
        iA = dot_q8_dwords(a, x0, x1);
        iB = dot_q8_dwords(&w[9], x2, x3);
    }
    if (dump2) { dump2[0] = iA; dump2[1] = iB; }
    acc = fmaf(dA * __int_as_float(mm.x), (float)iA, acc);
    acc = fmaf(dB * __int_as_float(mm.z), (float)iB, acc);
    return acc;
    }
}

template <int WT, int LPR, int NIT, int NT>
static __device__ __forceinline__ void dot_tile(const wtile<WT, NIT> &t, const staged_act *act, int npair, int l,
                                                float acc[NT], int32_t *dump) {
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int p = it * LPR + l;
        if (p < npair) {
#pragma unroll
            for (int c = 0; c < NT; c++) {
                const int8_t *xq = act[c].q;
                const int4 mm = *(const int4 *)(act[c].meta + 2 * p);
                acc[c] = dot_pair<WT>(t.w[it], *act_part(xq, p, 0, npair), *act_part(xq, p, 1, npair), *act_part(xq, p, 2, npair), *act_part(xq, p, 3, npair),
                                      mm, mm, p, acc[c], (dump && c == 0) ? dump + 2 * p : nullptr);
            }
        }
    }
}

// The activations one lane needs when it owns the same block pairs of every row (64 lanes per row):
// read from LDS once, reused for all rows of the wave.
template <int NIT> struct act_frag { int4 x[NIT][4]; int4 mm[NIT]; int4 mm2[NIT]; };
template <int WT, int NIT>
static __device__ __forceinline__ void load_act_frag(act_frag<NIT> &f, const staged_act &act, int npair, int lane) {
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int p = min(it * 64 + lane, npair - 1);
        if constexpr (WT == SPY_HIP_Q6_K) {
            // 16-element slices e and 2 + e of the two pairs (= four 32-element blocks) of the lane's half
            const int pa = p & ~1, pb = p | 1, e = p & 1;
            f.x[it][0] = *act_part(act.q, pa, e, npair); f.x[it][1] = *act_part(act.q, pa, 2 + e, npair);
            f.x[it][2] = *act_part(act.q, pb, e, npair); f.x[it][3] = *act_part(act.q, pb, 2 + e, npair);
            f.mm[it] = *(const int4 *)(act.meta + 2 * pa);
            f.mm2[it] = *(const int4 *)(act.meta + 2 * pb);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) f.x[it][j] = *act_part(act.q, p, j, npair);
            f.mm[it] = *(const int4 *)(act.meta + 2 * p);
            f.mm2[it] = f.mm[it];
        }
    }
}
template <int WT, int NIT>
static __device__ __forceinline__ float dot_row_frag(const wtile<WT, NIT> &t, const act_frag<NIT> &f, int npair, int lane) {
    float acc = 0.0f;
#pragma unroll
    for (int it = 0; it < NIT; it++)
        if (it * 64 + lane < npair) acc = dot_pair<WT>(t.w[it], f.x[it][0], f.x[it][1], f.x[it][2], f.x[it][3], f.mm[it], f.mm2[it], it * 64 + lane, acc, nullptr);
    return acc;
}

// The same dot with the activations read from LDS unit by unit (single-row waves with several units per
// lane: keeps the register footprint to one unit's activations).
template <int WT, int NIT>
static __device__ __forceinline__ float dot_row_lds(const wtile<WT, NIT> &t, const staged_act &act, int npair, int lane) {
    float acc = 0.0f;
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int p = it * 64 + lane;
        if (p < npair) {
            act_frag<1> f;
            load_act_frag<WT, 1>(f, act, npair, p);
            acc = dot_pair<WT>(t.w[it], f.x[0][0], f.x[0][1], f.x[0][2], f.x[0][3], f.mm[0], f.mm2[0], p, acc, nullptr);
        }
    }
    return acc;
}

// (lanes per row, block pairs per lane) for K elements: the smallest lane count whose pairs-per-lane
// fits GEMV_NIT_MAX; lpr = 0 when nothing fits (K must be a multiple of 64 so that every row is a
// whole number of 4-byte aligned block pairs).
struct gemv_cfg { int lpr, nit; };
static inline gemv_cfg pick_cfg(int64_t K, int max_lpr = 64) {
    gemv_cfg c = {0, 0};
    if (K % 64 != 0 || K <= 0) return c;
    const int64_t npair = K / 64;
    for (int lpr = 16; lpr <= max_lpr; lpr *= 2) {
        const int64_t nit = (npair + lpr - 1) / lpr;
        if (nit <= GEMV_NIT_MAX) { c.lpr = lpr; c.nit = (int)nit; return c; }
    }
    return c;
}

// dispatch a callable templated on <LPR, NIT> from run-time values
#define GEMV_DISPATCH_CFG(cfg, CALL)                                                       \
    switch ((cfg).lpr * 8 + (cfg).nit) {                                                   \
    case 16 * 8 + 1: CALL(16, 1); break; case 16 * 8 + 2: CALL(16, 2); break;              \
    case 16 * 8 + 3: CALL(16, 3); break; case 16 * 8 + 4: CALL(16, 4); break;              \
    case 32 * 8 + 3: CALL(32, 3); break; case 32 * 8 + 4: CALL(32, 4); break;              \
    case 64 * 8 + 3: CALL(64, 3); break; case 64 * 8 + 4: CALL(64, 4); break;              \
    default: break;                                                                        \
    }
