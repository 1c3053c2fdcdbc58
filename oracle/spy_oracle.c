/*
 * spy_oracle.c -- CPU restatement of the BL-GS/Spy host backend for the LLaMA-2 token loop.
 *
 * TEST INFRASTRUCTURE ONLY (see spy_oracle.h).  Plain C, no dependency on the reference
 * tree, written from a reading of the reference sources cited at each function.
 *
 * Conventions restated from the reference build (CMakeArch.cmake:8-17: AVX2+FMA+F16C on):
 *   - every float operation is a single IEEE binary32 operation; the only fused operations
 *     are the explicit fmaf() calls that stand for _mm256_fmadd_ps in the reference;
 *     this file is compiled with -ffp-contract=off so nothing else fuses.  Whether gcc
 *     fused the reference's scalar tails (vec_dot.h:142, non-linear.cpp:362-363) is not
 *     knowable without its build: those sites are "pinned to tolerance only".
 *   - SIMD lane structure is written out as arrays of 8 floats / ints.
 *
 * PARITY UNPINNED: all Q4_K / Q6_K functions.  The reference defines only the block
 * layouts (orchestration/include/number/number_impl/k-quant.h:79-117,162-188); its generic
 * Dot<> aborts (vec_dot.h:29-40) and its generic quantizer throws (vec_convert.h:30-36).
 * They restate the public ggml block format and are checked against invariants only.
 */
#define _GNU_SOURCE
#include "spy_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <stdio.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#if defined(__x86_64__)
#include <immintrin.h>
#endif

/* ============================================================================================
 * Number system
 * ========================================================================================== */

#define QK 32     /* Q4_0 / Q8_0 block length (quant.h:16,131) */
#define QK_K 256  /* super-block length (type.h:58) */

typedef struct { uint16_t d; uint8_t qs[16]; } blk_q4_0;                 /* quant.h:25-28   */
typedef struct { uint16_t d; int8_t  qs[32]; } blk_q8_0;                 /* quant.h:139-142 */
typedef struct { uint16_t d, dmin; uint8_t scales[12]; uint8_t qs[128]; } blk_q4_k; /* k-quant.h:101-111 */
typedef struct { uint8_t ql[128]; uint8_t qh[64]; int8_t scales[16]; uint16_t d; } blk_q6_k; /* k-quant.h:177-182 (scales read as int8, ggml) */

_Static_assert(sizeof(blk_q4_0) == 18, "q4_0");
_Static_assert(sizeof(blk_q8_0) == 34, "q8_0");
_Static_assert(sizeof(blk_q4_k) == 144, "q4_k");
_Static_assert(sizeof(blk_q6_k) == 210, "q6_k");

int64_t spy_o_type_size(int type) {
    switch (type) {
    case SPY_O_F32: return 4;  case SPY_O_F16: return 2;  case SPY_O_I32: return 4;
    case SPY_O_Q4_0: return 18; case SPY_O_Q8_0: return 34;
    case SPY_O_Q4_K: return 144; case SPY_O_Q6_K: return 210;
    }
    return 0;
}

int64_t spy_o_block_size(int type) {
    switch (type) {
    case SPY_O_F32: case SPY_O_F16: case SPY_O_I32: return 1;
    case SPY_O_Q4_0: case SPY_O_Q8_0: return QK;
    case SPY_O_Q4_K: case SPY_O_Q6_K: return QK_K;
    }
    return 0;
}

int64_t spy_o_row_size(int type, int64_t n) { return n * spy_o_type_size(type) / spy_o_block_size(type); }

/* IEEE binary32 -> binary16, round to nearest even.  The reference calls
 * simde_float16_from_float32 (lookup_table.h:54); simde is not vendored, its contract is
 * IEEE RNE (hardware vcvtps2ph on the reference's build flags). */
uint16_t spy_o_f32_to_f16(float f) {
    uint32_t x; memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t ax   = x & 0x7fffffffu;
    if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu)); /* NaN, quieted */
    if (ax >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);                         /* >= 65536 or inf */
    const uint32_t exp = ax >> 23;
    if (exp < 113) {                       /* below the smallest normal half 2^-14: subnormal or zero */
        const uint32_t shift = 126 - exp;  /* exp 112 -> 14 */
        if (shift > 24) return (uint16_t)sign;
        const uint32_t mant = (ax & 0x7fffffu) | 0x800000u;
        uint32_t h = mant >> shift;
        const uint32_t rem  = mant & ((1u << shift) - 1u);
        const uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((exp - 112) << 10) | ((ax >> 13) & 0x3ffu);
    const uint32_t rem = ax & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;   /* may carry into the exponent, up to inf */
    return (uint16_t)(sign | h);
}

float spy_o_f16_to_f32_ieee(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t exp  = (h >> 10) & 0x1fu;
    uint32_t mant = h & 0x3ffu;
    uint32_t x;
    if (exp == 0) {
        if (mant == 0) x = sign;
        else {
            int e = -1;
            do { e++; mant <<= 1; } while (!(mant & 0x400u));
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | ((mant & 0x3ffu) << 13);
        }
    } else if (exp == 31) x = sign | 0x7f800000u | (mant << 13);
    else x = sign | ((exp + 112) << 23) | (mant << 13);
    float f; memcpy(&f, &x, 4);
    return f;
}

/* The reference converts through a 65 536-entry table whose constructor loop is
 * `for (Key k = 0; k < MAX_KEY; ++k)` (conversion.h:39-41): entry 0xFFFF is never written and
 * stays 0 (static storage). Same loop bound for the silu / exp tables (non-linear.h:42-47,134-139). */
float spy_o_f16_to_f32(uint16_t h) { return h == 0xFFFFu ? 0.0f : spy_o_f16_to_f32_ieee(h); }

float spy_o_silu_lut(uint16_t h) {
    if (h == 0xFFFFu) return 0.0f;
    const float v = spy_o_f16_to_f32_ieee(h);
    return v / (1.0f + expf(-v));          /* non-linear.h:44-45 (std::exp(float) == expf) */
}

float spy_o_exp_lut(uint16_t h) {
    if (h == 0xFFFFu) return 0.0f;
    return expf(spy_o_f16_to_f32_ieee(h)); /* non-linear.h:136-137 */
}

/* Shape(dim, elements, type): contiguous strides (tensor.h:44-58) */
void spy_o_tensor_contiguous(spy_o_tensor *t, int type, int dim, const int64_t *ne, void *data) {
    t->type = type; t->dim = dim; t->data = data;
    for (int i = 0; i < 4; i++) t->ne[i] = i < dim ? ne[i] : 1;
    t->nb[0] = spy_o_type_size(type);
    int64_t acc = spy_o_row_size(type, t->ne[0]);
    for (int i = 1; i < 4; i++) { t->nb[i] = acc; acc *= t->ne[i]; }
}

/* Tensor::get(index_array) (tensor.h:225-236): index 0 is divided by the block size */
static inline void *tget(const spy_o_tensor *t, int64_t i0, int64_t i1, int64_t i2, int64_t i3) {
    i0 /= spy_o_block_size(t->type);
    return (uint8_t *)t->data + i0 * t->nb[0] + i1 * t->nb[1] + i2 * t->nb[2] + i3 * t->nb[3];
}

static inline int64_t t_nrow(const spy_o_tensor *t) { return t->ne[1] * t->ne[2] * t->ne[3]; }
static inline int64_t t_nelem(const spy_o_tensor *t) { return t->ne[0] * t->ne[1] * t->ne[2] * t->ne[3]; }
static inline int64_t t_row_size(const spy_o_tensor *t) { return spy_o_type_size(t->type) * t->ne[0] / spy_o_block_size(t->type); }

/* Shape::is_continuous (tensor.h:167-173) */
static int t_is_contiguous(const spy_o_tensor *t) {
    return t->nb[0] == spy_o_type_size(t->type)
        && t->nb[1] == t->nb[0] * t->ne[0] / spy_o_block_size(t->type)
        && t->nb[2] == t->nb[1] * t->ne[1]
        && t->nb[3] == t->nb[2] * t->ne[2];
}

static int t_same_shape(const spy_o_tensor *a, const spy_o_tensor *b) {  /* Shape::operator== (tensor.h:106-109) */
    if (a->type != b->type || a->dim != b->dim) return 0;
    for (int i = 0; i < 4; i++) if (a->ne[i] != b->ne[i] || a->nb[i] != b->nb[i]) return 0;
    return 1;
}

/* ============================================================================================
 * Quantizers
 * ========================================================================================== */

static inline int8_t sat_i8(int32_t v) { return (int8_t)(v < -128 ? -128 : v > 127 ? 127 : v); }

/* Quantizator<FP32,Q8_0>::transform (vec_convert.h:197-260).
 * amax over 32 floats; d = amax/127 stored as fp16; id = amax ? 127/amax : 0; each element is
 * x*id rounded to nearest even (_mm256_round_ps NEAREST, :235-238), converted to int32 and
 * narrowed with signed saturation (:247-250); the final permute restores element order (:255-256). */
void spy_o_quantize_q8_0(const float *x, void *vy, int64_t n) {
    blk_q8_0 *y = (blk_q8_0 *)vy;
    const int64_t nb = n / QK;
    for (int64_t i = 0; i < nb; i++) {
        float amax = 0.0f;
        for (int j = 0; j < QK; j++) { const float a = fabsf(x[i * QK + j]); if (a > amax) amax = a; }
        const float d  = amax / 127.0f;
        const float id = (amax != 0.0f) ? 127.0f / amax : 0.0f;
        y[i].d = spy_o_f32_to_f16(d);
        for (int j = 0; j < QK; j++) {
            const float v = x[i * QK + j] * id;
            y[i].qs[j] = sat_i8((int32_t)rintf(v));
        }
    }
}

/* The Q4_0 rule that Dot<Q4_0,Q8_0> decodes (vec_dot.h:62-75: element j = low nibble of
 * quants[j], element j+16 = high nibble, value (nibble-8)*delta): d = max/-8 where max is the
 * signed value of largest magnitude, id = d ? 1/d : 0, q = min(15, (int8)(x*id + 8.5)).
 * This is what vec_convert.h:86-120 evidently intends; as written that function is not usable
 * (see spy_o_quantize_q4_0_as_written). */
void spy_o_quantize_q4_0_ggml(const float *x, void *vy, int64_t n) {
    blk_q4_0 *y = (blk_q4_0 *)vy;
    const int64_t nb = n / QK;
    for (int64_t i = 0; i < nb; i++) {
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < QK; j++) {
            const float v = x[i * QK + j];
            if (amax < fabsf(v)) { amax = fabsf(v); max = v; }
        }
        const float d  = max / -8.0f;
        const float id = (d != 0.0f) ? 1.0f / d : 0.0f;
        y[i].d = spy_o_f32_to_f16(d);
        for (int j = 0; j < QK / 2; j++) {
            const float x0 = x[i * QK + j] * id;
            const float x1 = x[i * QK + QK / 2 + j] * id;
            int q0 = (int8_t)(x0 + 8.5f); if (q0 > 15) q0 = 15;
            int q1 = (int8_t)(x1 + 8.5f); if (q1 > 15) q1 = 15;
            y[i].qs[j] = (uint8_t)(q0 | (q1 << 4));
        }
    }
}

/* Quantizator<FP32,Q4_0>::transform exactly as written (vec_convert.h:86-120): it consumes
 * NUM_FROM_UNIT = K/R = 16 floats per emitted block (:83,:87), writes only quants[0..7] (:108),
 * and its inverse scale is `(max == 0) ? 1/delta : 0` (:104), i.e. 0 for every non-zero block,
 * so every written nibble is (int8)(0 + 8.5) = 8.  Kept as a documented known-bad case: the
 * hot path never calls it (mat.cpp:32-42 only produces Q8_0 / FP16 activations).
 * `y` must hold n_from/16 blocks and is expected to be zero-filled by the caller. */
void spy_o_quantize_q4_0_as_written(const float *x, void *vy, int64_t n_from) {
    blk_q4_0 *y = (blk_q4_0 *)vy;
    const int U = 16;
    const int64_t nb = n_from / U;
    for (int64_t i = 0; i < nb; i++) {
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < U; j++) {
            const float v = x[i * U + j];
            if (amax < fabsf(v)) { amax = fabsf(v); max = v; }
        }
        const float d  = max / -8.0f;
        const float id = (max == 0.0f) ? (1.0f / d) : 0.0f;
        y[i].d = spy_o_f32_to_f16(d);
        for (int j = 0; j < U / 2; j++) {
            const float x0 = x[i * U + j] * id;
            const float x1 = x[i * U + U / 2 + j] * id;
            /* 0 * inf = NaN when max == 0; (int8)NaN is implementation-defined: the all-zero
             * block is excluded from the tests of this function. */
            int q0 = (int8_t)(x0 + 8.5f); if (q0 > 15) q0 = 15;
            int q1 = (int8_t)(x1 + 8.5f); if (q1 > 15) q1 = 15;
            y[i].qs[j] = (uint8_t)((uint8_t)q0 | ((uint8_t)q1 << 4));
        }
    }
}

/* Quantizator<FP32,FP16>::transform (vec_convert.h:56-64): RNE per element */
void spy_o_quantize_f16(const float *x, uint16_t *y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = spy_o_f32_to_f16(x[i]);
}

/* value = (nibble - 8) * fp16(d); element j low nibble, j+16 high nibble (vec_dot.h:62-75).
 * NOT the reference's Quantizator<Q4_0,FP32> (vec_convert.h:369-377), which writes the high
 * nibbles at +32 instead of +16 and overruns; that function is off the hot path. */
void spy_o_dequantize_q4_0(const void *vx, float *y, int64_t n) {
    const blk_q4_0 *x = (const blk_q4_0 *)vx;
    for (int64_t i = 0; i < n / QK; i++) {
        const float d = spy_o_f16_to_f32(x[i].d);
        for (int j = 0; j < 16; j++) {
            y[i * QK + j]      = (float)((x[i].qs[j] & 0x0F) - 8) * d;
            y[i * QK + j + 16] = (float)((x[i].qs[j] >> 4) - 8) * d;
        }
    }
}

/* Quantizator<Q8_0,FP32>::transform (vec_convert.h:436-442) */
void spy_o_dequantize_q8_0(const void *vx, float *y, int64_t n) {
    const blk_q8_0 *x = (const blk_q8_0 *)vx;
    for (int64_t i = 0; i < n / QK; i++) {
        const float d = spy_o_f16_to_f32(x[i].d);
        for (int j = 0; j < QK; j++) y[i * QK + j] = (float)x[i].qs[j] * d;
    }
}

/* ---- K-quants: PARITY UNPINNED (public ggml block format, restated) ---------------------- */

/* 6-bit (scale, min) pair j of a Q4_K super-block from scales[12] */
static inline void q4k_scale_min(int j, const uint8_t *s, uint8_t *sc, uint8_t *m) {
    if (j < 4) { *sc = s[j] & 63; *m = s[j + 4] & 63; }
    else {
        *sc = (uint8_t)((s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4));
        *m  = (uint8_t)((s[j + 4] >> 4)   | ((s[j]     >> 6) << 4));
    }
}

static inline void q4k_pack_scale_min(int j, uint8_t *s, uint8_t sc, uint8_t m) {
    if (j < 4) { s[j] = (uint8_t)((s[j] & 0xC0) | sc); s[j + 4] = (uint8_t)((s[j + 4] & 0xC0) | m); }
    else {
        s[j + 4] = (uint8_t)((sc & 0x0F) | ((m & 0x0F) << 4));
        s[j - 4] = (uint8_t)((s[j - 4] & 0x3F) | ((sc >> 4) << 6));
        s[j]     = (uint8_t)((s[j]     & 0x3F) | ((m  >> 4) << 6));
    }
}

/* element l of sub-blocks 2i / 2i+1 = low / high nibble of qs[32 i + l];
 * value = d*sc*q - dmin*m */
void spy_o_dequantize_q4_k(const void *vx, float *y, int64_t n) {
    const blk_q4_k *x = (const blk_q4_k *)vx;
    for (int64_t b = 0; b < n / QK_K; b++) {
        const float d = spy_o_f16_to_f32(x[b].d), dmin = spy_o_f16_to_f32(x[b].dmin);
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m; q4k_scale_min(j, x[b].scales, &sc, &m);
            const float d1 = d * (float)sc, m1 = dmin * (float)m;
            for (int l = 0; l < 32; l++) {
                const uint8_t byte = x[b].qs[32 * (j / 2) + l];
                const int q = (j & 1) ? (byte >> 4) : (byte & 0x0F);
                y[b * QK_K + 32 * j + l] = d1 * (float)q - m1;
            }
        }
    }
}

/* 6-bit quant (value - 32) of element e (0..255) of a Q6_K super-block */
static inline int q6k_get(const blk_q6_k *x, int e) {
    const int half = e / 128, r = e % 128, grp = r / 32, l = r % 32;
    const uint8_t *ql = x->ql + 64 * half, *qh = x->qh + 32 * half;
    int lo;
    switch (grp) {
    case 0:  lo = ql[l] & 0x0F;      break;
    case 1:  lo = ql[l + 32] & 0x0F; break;
    case 2:  lo = ql[l] >> 4;        break;
    default: lo = ql[l + 32] >> 4;   break;
    }
    const int hi = (qh[l] >> (2 * grp)) & 3;
    return (lo | (hi << 4)) - 32;
}

void spy_o_dequantize_q6_k(const void *vx, float *y, int64_t n) {
    const blk_q6_k *x = (const blk_q6_k *)vx;
    for (int64_t b = 0; b < n / QK_K; b++) {
        const float d = spy_o_f16_to_f32(x[b].d);
        for (int e = 0; e < QK_K; e++)
            y[b * QK_K + e] = d * (float)x[b].scales[e / 16] * (float)q6k_get(&x[b], e);
    }
}

/* Project-defined Q4_K quantizer (NOT ggml's iterative make_qkx2_quants search): per 32-element
 * sub-block an affine grid [min(0,lo), hi] with 15 steps; the 8 steps and 8 (negated) minima
 * are themselves quantized to 6 bits against the super-block maxima. */
void spy_o_quantize_q4_k(const float *x, void *vy, int64_t n) {
    blk_q4_k *y = (blk_q4_k *)vy;
    for (int64_t b = 0; b < n / QK_K; b++) {
        float scales[8], mins[8], max_scale = 0.0f, max_min = 0.0f;
        const float *xb = x + b * QK_K;
        for (int j = 0; j < 8; j++) {
            float lo = 0.0f, hi = 0.0f;
            for (int l = 0; l < 32; l++) { const float v = xb[32 * j + l]; if (v < lo) lo = v; if (v > hi) hi = v; }
            scales[j] = (hi - lo) / 15.0f; mins[j] = -lo;
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        const float d = max_scale / 63.0f, dmin = max_min / 63.0f;
        y[b].d = spy_o_f32_to_f16(d); y[b].dmin = spy_o_f32_to_f16(dmin);
        const float df = spy_o_f16_to_f32(y[b].d), dminf = spy_o_f16_to_f32(y[b].dmin);
        memset(y[b].scales, 0, 12);
        for (int j = 0; j < 8; j++) {
            int sc = df    > 0.0f ? (int)rintf(scales[j] / df)  : 0; if (sc > 63) sc = 63;
            int m  = dminf > 0.0f ? (int)rintf(mins[j] / dminf) : 0; if (m > 63) m = 63;
            q4k_pack_scale_min(j, y[b].scales, (uint8_t)sc, (uint8_t)m);
        }
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m; q4k_scale_min(j, y[b].scales, &sc, &m);
            const float d1 = df * (float)sc, m1 = dminf * (float)m;
            for (int l = 0; l < 32; l++) {
                int q = d1 > 0.0f ? (int)rintf((xb[32 * j + l] + m1) / d1) : 0;
                q = q < 0 ? 0 : q > 15 ? 15 : q;
                uint8_t *p = &y[b].qs[32 * (j / 2) + l];
                if (j & 1) *p = (uint8_t)((*p & 0x0F) | (q << 4)); else *p = (uint8_t)q;
            }
        }
    }
}

/* Project-defined Q6_K quantizer (NOT ggml's make_qx_quants search): per 16-element sub-block a
 * symmetric step amax/31, the 16 steps quantized to int8 against the super-block maximum. */
void spy_o_quantize_q6_k(const float *x, void *vy, int64_t n) {
    blk_q6_k *y = (blk_q6_k *)vy;
    for (int64_t b = 0; b < n / QK_K; b++) {
        const float *xb = x + b * QK_K;
        float steps[16], max_step = 0.0f;
        for (int j = 0; j < 16; j++) {
            float amax = 0.0f;
            for (int l = 0; l < 16; l++) { const float a = fabsf(xb[16 * j + l]); if (a > amax) amax = a; }
            steps[j] = amax / 31.0f;
            if (steps[j] > max_step) max_step = steps[j];
        }
        const float d = max_step / 127.0f;
        y[b].d = spy_o_f32_to_f16(d);
        const float df = spy_o_f16_to_f32(y[b].d);
        memset(y[b].ql, 0, 128); memset(y[b].qh, 0, 64);
        for (int j = 0; j < 16; j++) {
            int sc = df > 0.0f ? (int)ceilf(steps[j] / df) : 0; if (sc > 127) sc = 127;
            y[b].scales[j] = (int8_t)sc;
        }
        for (int e = 0; e < QK_K; e++) {
            const float step = df * (float)y[b].scales[e / 16];
            int q = step > 0.0f ? (int)rintf(xb[e] / step) : 0;
            q = (q < -32 ? -32 : q > 31 ? 31 : q) + 32;
            const int half = e / 128, r = e % 128, grp = r / 32, l = r % 32;
            uint8_t *ql = y[b].ql + 64 * half, *qh = y[b].qh + 32 * half;
            const int lo = q & 0x0F, hi = q >> 4;
            switch (grp) {
            case 0:  ql[l]      |= (uint8_t)lo;        break;
            case 1:  ql[l + 32] |= (uint8_t)lo;        break;
            case 2:  ql[l]      |= (uint8_t)(lo << 4); break;
            default: ql[l + 32] |= (uint8_t)(lo << 4); break;
            }
            qh[l] |= (uint8_t)(hi << (2 * grp));
        }
    }
}

/* ============================================================================================
 * Dot products
 * ========================================================================================== */

/* hsum_float_8 (vec_util.h:75-81): ((a0+a4)+(a2+a6)) + ((a1+a5)+(a3+a7)) */
static inline float hsum8(const float a[8]) {
    const float r0 = a[4] + a[0], r1 = a[5] + a[1], r2 = a[6] + a[2], r3 = a[7] + a[3];
    const float s0 = r0 + r2, s1 = r1 + r3;
    return s0 + s1;
}

static inline int16_t sat_i16(int32_t v) { return (int16_t)(v < -32768 ? -32768 : v > 32767 ? 32767 : v); }

/* mul_sum_i8_pairs (vec_util.h:101-110) on one group of 4 int8 pairs:
 * ax = |x| as uint8, sy = y with the sign of x (0 when x == 0), maddubs = saturating int16 sum of
 * adjacent products, madd with ones = sum of adjacent int16 -> int32. */
static inline int32_t mul_sum4(const int8_t *x, const int8_t *y) {
    int32_t pair[2];
    for (int p = 0; p < 2; p++) {
        int32_t s = 0;
        for (int k = 0; k < 2; k++) {
            const int8_t xv = x[2 * p + k], yv = y[2 * p + k];
            const uint8_t ax = (uint8_t)(xv < 0 ? -xv : xv);                          /* sign_epi8(x, x) */
            const int8_t  sy = xv < 0 ? (int8_t)(-yv) : (xv == 0 ? 0 : yv);           /* sign_epi8(y, x) */
            s += (int32_t)ax * (int32_t)sy;
        }
        pair[p] = sat_i16(s);
    }
    return pair[0] + pair[1];
}

/* Dot<Q4_0,Q8_0>::exec (vec_dot.h:49-85): per block, lanes 4..7 hold the low-nibble half
 * (elements 0..15, four products per lane), lanes 0..3 the high-nibble half (elements 16..31)
 * because of _mm256_set_m128i(i32_0, i32_1) (:78); acc = fma(d, p, acc) per lane (:81). */
static float dot_q4_0_q8_0_scalar(const blk_q4_0 *w, const blk_q8_0 *x, int64_t n) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int64_t i = 0; i < n / QK; i++) {
        const float d = spy_o_f16_to_f32(w[i].d) * spy_o_f16_to_f32(x[i].d);
        int8_t lo[16], hi[16];
        for (int j = 0; j < 16; j++) { lo[j] = (int8_t)((w[i].qs[j] & 0x0F) - 8); hi[j] = (int8_t)((w[i].qs[j] >> 4) - 8); }
        int32_t p[8];
        for (int k = 0; k < 4; k++) {
            p[4 + k] = mul_sum4(lo + 4 * k, x[i].qs + 4 * k);
            p[k]     = mul_sum4(hi + 4 * k, x[i].qs + 16 + 4 * k);
        }
        for (int l = 0; l < 8; l++) acc[l] = fmaf(d, (float)p[l], acc[l]);
    }
    return hsum8(acc);
}

/* Dot<Q8_0,Q8_0>::exec (vec_dot.h:95-114): lane l = elements 4l..4l+3 (vec_util.h:126-132) */
static float dot_q8_0_q8_0_scalar(const blk_q8_0 *w, const blk_q8_0 *x, int64_t n) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int64_t i = 0; i < n / QK; i++) {
        const float d = spy_o_f16_to_f32(w[i].d) * spy_o_f16_to_f32(x[i].d);
        for (int l = 0; l < 8; l++) acc[l] = fmaf(d, (float)mul_sum4(w[i].qs + 4 * l, x[i].qs + 4 * l), acc[l]);
    }
    return hsum8(acc);
}

/* Dot<FP16,FP16>::exec (vec_dot.h:124-145): four 8-lane fma accumulators over chunks of 32 while
 * `i + 32 < n` (strict), FP16::block_reduce (vec_util.h:61-71), then a scalar tail over the
 * remaining 1..32 elements through the conversion table; returns tail + simd. */
static float dot_f16_f16_scalar(const uint16_t *a, const uint16_t *b, int64_t n) {
    float sum[4][8];
    memset(sum, 0, sizeof(sum));
    int64_t i = 0;
    for (; i + 32 < n; i += 32)
        for (int j = 0; j < 4; j++)
            for (int l = 0; l < 8; l++)
                sum[j][l] = fmaf(spy_o_f16_to_f32_ieee(a[i + 8 * j + l]), spy_o_f16_to_f32_ieee(b[i + 8 * j + l]), sum[j][l]);
    for (int l = 0; l < 8; l++) { sum[0][l] += sum[2][l]; sum[1][l] += sum[3][l]; }
    for (int l = 0; l < 8; l++) sum[0][l] += sum[1][l];
    float t0[4];
    for (int l = 0; l < 4; l++) t0[l] = sum[0][l] + sum[0][l + 4];
    const float simd_res = (t0[0] + t0[1]) + (t0[2] + t0[3]);
    float tail = 0.0f;
    for (; i < n; i++) tail += spy_o_f16_to_f32(a[i]) * spy_o_f16_to_f32(b[i]);
    return tail + simd_res;
}

#if defined(__x86_64__)
/* AVX2 forms of the same three dots, for the timed CPU baseline.  Same lane structure and the
 * same per-lane fma sequence, hence bit-identical to the scalar forms (checked in the tests). */
__attribute__((target("avx2,fma,f16c")))
static inline float hsum8_avx(__m256 v) {
    float a[8]; _mm256_storeu_ps(a, v); return hsum8(a);
}

__attribute__((target("avx2,fma,f16c")))
static float dot_q4_0_q8_0_avx2(const blk_q4_0 *w, const blk_q8_0 *x, int64_t n) {
    __m256 acc = _mm256_setzero_ps();
    const __m256i m4 = _mm256_set1_epi8(0x0F), off = _mm256_set1_epi8(8), ones = _mm256_set1_epi16(1);
    for (int64_t i = 0; i < n / QK; i++) {
        const float d = spy_o_f16_to_f32(w[i].d) * spy_o_f16_to_f32(x[i].d);
        const __m128i raw = _mm_loadu_si128((const __m128i *)w[i].qs);
        /* low 128 bits: high nibbles (elements 16..31), high 128 bits: low nibbles (0..15) */
        __m256i q = _mm256_set_m128i(raw, _mm_srli_epi16(raw, 4));
        q = _mm256_sub_epi8(_mm256_and_si256(q, m4), off);
        const __m256i yv = _mm256_set_m128i(_mm_loadu_si128((const __m128i *)x[i].qs),
                                            _mm_loadu_si128((const __m128i *)(x[i].qs + 16)));
        const __m256i aq = _mm256_sign_epi8(q, q), sy = _mm256_sign_epi8(yv, q);
        const __m256i p  = _mm256_madd_epi16(ones, _mm256_maddubs_epi16(aq, sy));
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(p), acc);
    }
    return hsum8_avx(acc);
}

__attribute__((target("avx2,fma,f16c")))
static float dot_q8_0_q8_0_avx2(const blk_q8_0 *w, const blk_q8_0 *x, int64_t n) {
    __m256 acc = _mm256_setzero_ps();
    const __m256i ones = _mm256_set1_epi16(1);
    for (int64_t i = 0; i < n / QK; i++) {
        const float d = spy_o_f16_to_f32(w[i].d) * spy_o_f16_to_f32(x[i].d);
        const __m256i a = _mm256_loadu_si256((const __m256i *)w[i].qs);
        const __m256i b = _mm256_loadu_si256((const __m256i *)x[i].qs);
        const __m256i p = _mm256_madd_epi16(ones, _mm256_maddubs_epi16(_mm256_sign_epi8(a, a), _mm256_sign_epi8(b, a)));
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(p), acc);
    }
    return hsum8_avx(acc);
}

__attribute__((target("avx2,fma,f16c")))
static float dot_f16_f16_avx2(const uint16_t *a, const uint16_t *b, int64_t n) {
    __m256 s[4] = {_mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps()};
    int64_t i = 0;
    for (; i + 32 < n; i += 32)
        for (int j = 0; j < 4; j++) {
            const __m256 av = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(a + i + 8 * j)));
            const __m256 bv = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(b + i + 8 * j)));
            s[j] = _mm256_fmadd_ps(av, bv, s[j]);
        }
    s[0] = _mm256_add_ps(s[0], s[2]); s[1] = _mm256_add_ps(s[1], s[3]);
    s[0] = _mm256_add_ps(s[0], s[1]);
    float v[8]; _mm256_storeu_ps(v, s[0]);
    const float t0 = v[0] + v[4], t1 = v[1] + v[5], t2 = v[2] + v[6], t3 = v[3] + v[7];
    const float simd_res = (t0 + t1) + (t2 + t3);
    float tail = 0.0f;
    for (; i < n; i++) tail += spy_o_f16_to_f32(a[i]) * spy_o_f16_to_f32(b[i]);
    return tail + simd_res;
}
#endif

static int g_avx2 = -1;
int spy_o_have_avx2(void) {
    if (g_avx2 < 0) {
#if defined(__x86_64__)
        g_avx2 = __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma") && __builtin_cpu_supports("f16c");
        if (getenv("SPY_ORACLE_SCALAR")) g_avx2 = 0;
#else
        g_avx2 = 0;
#endif
    }
    return g_avx2;
}

float spy_o_dot_q4_0_q8_0(const void *w, const void *x, int64_t n) {
#if defined(__x86_64__)
    if (spy_o_have_avx2()) return dot_q4_0_q8_0_avx2((const blk_q4_0 *)w, (const blk_q8_0 *)x, n);
#endif
    return dot_q4_0_q8_0_scalar((const blk_q4_0 *)w, (const blk_q8_0 *)x, n);
}
float spy_o_dot_q8_0_q8_0(const void *w, const void *x, int64_t n) {
#if defined(__x86_64__)
    if (spy_o_have_avx2()) return dot_q8_0_q8_0_avx2((const blk_q8_0 *)w, (const blk_q8_0 *)x, n);
#endif
    return dot_q8_0_q8_0_scalar((const blk_q8_0 *)w, (const blk_q8_0 *)x, n);
}
float spy_o_dot_f16_f16(const uint16_t *a, const uint16_t *b, int64_t n) {
#if defined(__x86_64__)
    if (spy_o_have_avx2()) return dot_f16_f16_avx2(a, b, n);
#endif
    return dot_f16_f16_scalar(a, b, n);
}
/* scalar forms exported for the AVX2-vs-scalar identity test */
float spy_o_dot_q4_0_q8_0_scalar(const void *w, const void *x, int64_t n) { return dot_q4_0_q8_0_scalar((const blk_q4_0 *)w, (const blk_q8_0 *)x, n); }
float spy_o_dot_q8_0_q8_0_scalar(const void *w, const void *x, int64_t n) { return dot_q8_0_q8_0_scalar((const blk_q8_0 *)w, (const blk_q8_0 *)x, n); }
float spy_o_dot_f16_f16_scalar(const uint16_t *a, const uint16_t *b, int64_t n) { return dot_f16_f16_scalar(a, b, n); }

/* ---- K-quant dots against Q8_0 activations: PARITY UNPINNED (project-defined) ------------
 * Q4_K: sub-block j (32 elements) lines up with Q8_0 block j of the super-block:
 *   acc += dx_j * ( d*(float)(sc_j*isum_j) - dmin*(float)(m_j*bsum_j) ),
 *   isum_j = sum q*q8 (q in 0..15), bsum_j = sum q8.
 * Q6_K: Q8_0 block t covers 16-element sub-blocks 2t, 2t+1:
 *   acc += dx_t * d * (float)(sc_2t*isum_2t + sc_2t+1*isum_2t+1), isum over (q6-32)*q8. */
float spy_o_dot_q4_k_q8_0(const void *vw, const void *vx, int64_t n) {
    const blk_q4_k *w = (const blk_q4_k *)vw; const blk_q8_0 *x = (const blk_q8_0 *)vx;
    float acc = 0.0f;
    for (int64_t b = 0; b < n / QK_K; b++) {
        const float d = spy_o_f16_to_f32(w[b].d), dmin = spy_o_f16_to_f32(w[b].dmin);
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m; q4k_scale_min(j, w[b].scales, &sc, &m);
            const blk_q8_0 *xb = &x[b * 8 + j];
            int32_t isum = 0, bsum = 0;
            for (int l = 0; l < 32; l++) {
                const uint8_t byte = w[b].qs[32 * (j / 2) + l];
                const int q = (j & 1) ? (byte >> 4) : (byte & 0x0F);
                isum += q * xb->qs[l]; bsum += xb->qs[l];
            }
            const float dx = spy_o_f16_to_f32(xb->d);
            acc = fmaf(dx, d * (float)((int32_t)sc * isum) - dmin * (float)((int32_t)m * bsum), acc);
        }
    }
    return acc;
}

float spy_o_dot_q6_k_q8_0(const void *vw, const void *vx, int64_t n) {
    const blk_q6_k *w = (const blk_q6_k *)vw; const blk_q8_0 *x = (const blk_q8_0 *)vx;
    float acc = 0.0f;
    for (int64_t b = 0; b < n / QK_K; b++) {
        const float d = spy_o_f16_to_f32(w[b].d);
        for (int t = 0; t < 8; t++) {
            const blk_q8_0 *xb = &x[b * 8 + t];
            int32_t s = 0;
            for (int h = 0; h < 2; h++) {
                int32_t isum = 0;
                for (int l = 0; l < 16; l++) isum += q6k_get(&w[b], 32 * t + 16 * h + l) * xb->qs[16 * h + l];
                s += (int32_t)w[b].scales[2 * t + h] * isum;
            }
            acc = fmaf(spy_o_f16_to_f32(xb->d) * d, (float)s, acc);
        }
    }
    return acc;
}

/* int32 dot of every block (Q4_0, Q8_0: n/32 values; Q4_K: n/32 values of sum q*q8 with q in
 * 0..15; Q6_K: n/16 values of sum (q6-32)*q8).  Plain integer sums: order-independent. */
int spy_o_block_dots(int wtype, const void *vw, const void *vx, int64_t n, int32_t *out) {
    const blk_q8_0 *x = (const blk_q8_0 *)vx;
    if (wtype == SPY_O_Q4_0) {
        const blk_q4_0 *w = (const blk_q4_0 *)vw;
        for (int64_t i = 0; i < n / QK; i++) {
            int32_t s = 0;
            for (int j = 0; j < 16; j++)
                s += ((w[i].qs[j] & 0x0F) - 8) * x[i].qs[j] + ((w[i].qs[j] >> 4) - 8) * x[i].qs[j + 16];
            out[i] = s;
        }
        return 0;
    }
    if (wtype == SPY_O_Q8_0) {
        const blk_q8_0 *w = (const blk_q8_0 *)vw;
        for (int64_t i = 0; i < n / QK; i++) {
            int32_t s = 0;
            for (int j = 0; j < QK; j++) s += (int32_t)w[i].qs[j] * x[i].qs[j];
            out[i] = s;
        }
        return 0;
    }
    if (wtype == SPY_O_Q4_K) {
        const blk_q4_k *w = (const blk_q4_k *)vw;
        for (int64_t b = 0; b < n / QK_K; b++)
            for (int j = 0; j < 8; j++) {
                int32_t s = 0;
                for (int l = 0; l < 32; l++) {
                    const uint8_t byte = w[b].qs[32 * (j / 2) + l];
                    s += ((j & 1) ? (byte >> 4) : (byte & 0x0F)) * x[b * 8 + j].qs[l];
                }
                out[b * 8 + j] = s;
            }
        return 0;
    }
    if (wtype == SPY_O_Q6_K) {
        const blk_q6_k *w = (const blk_q6_k *)vw;
        for (int64_t b = 0; b < n / QK_K; b++)
            for (int j = 0; j < 16; j++) {
                int32_t s = 0;
                for (int l = 0; l < 16; l++) s += q6k_get(&w[b], 16 * j + l) * x[b * 8 + j / 2].qs[16 * (j & 1) + l];
                out[b * 16 + j] = s;
            }
        return 0;
    }
    return 1;
}

/* ============================================================================================
 * Operators
 * ========================================================================================== */

/* target_buffer_type (mat.cpp:32-42) */
static int target_buffer_type(int t0, int t1) {
    if (t0 == t1) return t0;
    if (t0 == SPY_O_F16 && t1 == SPY_O_F32) return SPY_O_F16;
    if (t0 == SPY_O_Q4_0 && t1 == SPY_O_F32) return SPY_O_Q8_0;
    if (t0 == SPY_O_Q8_0 && t1 == SPY_O_F32) return SPY_O_Q8_0;
    return t0;
}

typedef float (*dot_fn)(const void *, const void *, int64_t);
static float dot_f16_v(const void *a, const void *b, int64_t n) { return spy_o_dot_f16_f16((const uint16_t *)a, (const uint16_t *)b, n); }

/* OperatorMatMulImpl::execute (mat.cpp:71-146).  Activation rows are converted to the
 * "mid" type into a contiguous scratch (:95-128), then dst[i01,i11,i02,i03] =
 * dot(w_row(i01,i02,i03), x_row(i11,i02,i03), ne00) with the output index running fastest along
 * the weight rows (:131-143).  Threads take 16-output blocks round-robin (:130-131).
 * Extension beyond the reference: (Q4_K|Q6_K, F32) -> Q8_0 activations (the reference falls
 * through to `return type_0` and then aborts in the generic Dot<>). */
int spy_o_matmul(const spy_o_tensor *w, const spy_o_tensor *x, spy_o_tensor *dst, int nthread) {
    const int t0 = w->type, t1 = x->type;
    int tmid = target_buffer_type(t0, t1);
    if ((t0 == SPY_O_Q4_K || t0 == SPY_O_Q6_K) && t1 == SPY_O_F32) tmid = SPY_O_Q8_0;
    dot_fn dot = NULL;
    if (t0 == SPY_O_Q4_0 && tmid == SPY_O_Q8_0) dot = spy_o_dot_q4_0_q8_0;
    else if (t0 == SPY_O_Q8_0 && tmid == SPY_O_Q8_0) dot = spy_o_dot_q8_0_q8_0;
    else if (t0 == SPY_O_F16 && tmid == SPY_O_F16) dot = dot_f16_v;
    else if (t0 == SPY_O_Q4_K && tmid == SPY_O_Q8_0) dot = spy_o_dot_q4_k_q8_0;
    else if (t0 == SPY_O_Q6_K && tmid == SPY_O_Q8_0) dot = spy_o_dot_q6_k_q8_0;
    else return 1;
    if (t1 != SPY_O_F32 && t1 != tmid) return 1;

    const int64_t ne00 = w->ne[0], ne01 = w->ne[1], ne02 = w->ne[2];
    const int64_t ne10 = x->ne[0], ne11 = x->ne[1], ne12 = x->ne[2], ne13 = x->ne[3];
    if (ne00 != ne10 || w->ne[2] != ne12 || w->ne[3] != ne13) return 2;   /* operator/mat.h:56-59 */
    const int64_t num_dst = t_nelem(dst);

    spy_o_tensor xq = *x;
    uint8_t *scratch = NULL;
    if (t1 != tmid) {
        const int64_t nrow = t_nrow(x), rsz = spy_o_row_size(tmid, ne10);
        scratch = (uint8_t *)malloc((size_t)(nrow * rsz) + 64);
        if (!scratch) return 3;
        #pragma omp parallel for num_threads(nthread > 0 ? nthread : 1) schedule(static)
        for (int64_t r = 0; r < nrow; r++) {
            const int64_t i13 = r / (ne12 * ne11), i12 = r % (ne12 * ne11) / ne11, i11 = r % ne11;
            const float *src = (const float *)tget(x, 0, i11, i12, i13);
            if (tmid == SPY_O_Q8_0) spy_o_quantize_q8_0(src, scratch + r * rsz, ne10);
            else spy_o_quantize_f16(src, (uint16_t *)(scratch + r * rsz), ne10);
        }
        const int64_t ne[4] = {ne10, ne11, ne12, ne13};
        spy_o_tensor_contiguous(&xq, tmid, 4, ne, scratch);
    }

    const int64_t nblk = (num_dst + 15) / 16;
    #pragma omp parallel for num_threads(nthread > 0 ? nthread : 1) schedule(static, 1)
    for (int64_t blk = 0; blk < nblk; blk++) {
        const int64_t end = (blk * 16 + 16 < num_dst) ? blk * 16 + 16 : num_dst;
        for (int64_t c = blk * 16; c < end; c++) {
            const int64_t i03 = c / (ne01 * ne11) / ne02;
            const int64_t i02 = c / (ne01 * ne11) % ne02;
            const int64_t i11 = c % (ne01 * ne11) / ne01;
            const int64_t i01 = c % (ne01 * ne11) % ne01;
            const void *xr = tget(&xq, 0, i11, i02, i03);
            const void *wr = tget(w, 0, i01, i02, i03);
            *(float *)tget(dst, i01, i11, i02, i03) = dot(wr, xr, ne00);
        }
    }
    free(scratch);
    return 0;
}

/* libstdc++ std::reduce / std::transform_reduce on random-access iterators: groups of four as
 * init = init + ((a0 + a1) + (a2 + a3)), then a sequential tail (bits/stl_numeric / <numeric>
 * __is_random_access_iter branch).  The reference is built with libstdc++ (gcc). */
static float reduce4(const float *p, int64_t n, int square) {
    float init = 0.0f;
    int64_t i = 0;
    for (; n - i >= 4; i += 4) {
        const float a0 = square ? p[i] * p[i] : p[i],         a1 = square ? p[i + 1] * p[i + 1] : p[i + 1];
        const float a2 = square ? p[i + 2] * p[i + 2] : p[i + 2], a3 = square ? p[i + 3] * p[i + 3] : p[i + 3];
        const float v1 = a0 + a1, v2 = a2 + a3, v3 = v1 + v2;
        init = init + v3;
    }
    for (; i < n; i++) init = init + (square ? p[i] * p[i] : p[i]);
    return init;
}

/* OperatorNormRMSImpl::execute (non-linear.cpp:194-223) */
int spy_o_norm_rms(const spy_o_tensor *x, spy_o_tensor *dst, float eps) {
    if (x->type != SPY_O_F32 || dst->type != SPY_O_F32) return 1;
    const int64_t ne0 = dst->ne[0], ne1 = dst->ne[1], ne2 = dst->ne[2], nrow = t_nrow(dst);
    for (int64_t r = 0; r < nrow; r++) {
        const int64_t i3 = r / (ne1 * ne2), i2 = r % (ne1 * ne2) / ne1, i1 = r % ne1;
        const float *s = (const float *)tget(x, 0, i1, i2, i3);
        float *d = (float *)tget(dst, 0, i1, i2, i3);
        const float sum   = reduce4(s, ne0, 1);
        const float mean  = sum / (float)ne0;
        const float scale = 1.0f / sqrtf(mean + eps);
        for (int64_t i = 0; i < ne0; i++) d[i] = s[i] * scale;
    }
    return 0;
}

/* binary_execution<Op> (basic.cpp:15-50), index arithmetic exactly as written (:30-36): correct
 * for operands of at most two dimensions, which is all the LLaMA graph produces. */
int spy_o_binary(int op, const spy_o_tensor *a, const spy_o_tensor *b, spy_o_tensor *dst) {
    if (a->type != SPY_O_F32 || b->type != SPY_O_F32 || dst->type != SPY_O_F32) return 1;
    const int64_t ne00 = a->ne[0], ne01 = a->ne[1], ne02 = a->ne[2], ne03 = a->ne[3];
    const int64_t ne10 = b->ne[0], ne11 = b->ne[1], ne12 = b->ne[2], ne13 = b->ne[3];
    const int64_t nrow = ne03 * ne02 * ne01;
    for (int64_t r = 0; r < nrow; r++) {
        const int64_t i03 = r / (ne01 * ne02);
        const int64_t i02 = (r - i03 * ne03) / ne01;
        const int64_t i01 = r - i03 * ne03 - i02 * ne02;
        const int64_t i13 = i03 % ne13, i12 = i02 % ne12, i11 = i01 % ne11;
        for (int64_t rep = 0; rep < ne00 / ne10; rep++) {
            const int64_t i00 = rep * ne00;
            const float *pa = (const float *)tget(a, i00, i01, i02, i03);
            const float *pb = (const float *)tget(b, 0, i11, i12, i13);
            float *pd = (float *)tget(dst, i00, i01, i02, i03);
            for (int64_t i = 0; i < ne10; i++) {
                switch (op) {
                case 0: pd[i] = pa[i] + pb[i]; break;
                case 1: pd[i] = pa[i] - pb[i]; break;
                case 2: pd[i] = pa[i] * pb[i]; break;
                default: pd[i] = pa[i] / pb[i]; break;
                }
            }
        }
    }
    return 0;
}

/* OperatorSiluImpl::execute (non-linear.cpp:57-77) with Silu<T> (:11-14): LUT on fp16(x) */
int spy_o_silu(const spy_o_tensor *x, spy_o_tensor *dst) {
    const int64_t ne00 = x->ne[0], ne01 = x->ne[1], ne02 = x->ne[2], nrow = t_nrow(x);
    for (int64_t r = 0; r < nrow; r++) {
        const int64_t i03 = r / (ne01 * ne02), i02 = r % (ne01 * ne02) / ne01, i01 = r % ne01;
        const float *s = (const float *)tget(x, 0, i01, i02, i03);
        float *d = (float *)tget(dst, 0, i01, i02, i03);
        for (int64_t i = 0; i < ne00; i++) d[i] = spy_o_silu_lut(spy_o_f32_to_f16(s[i]));
    }
    return 0;
}

/* OperatorReluImpl::execute (non-linear.cpp:28-50) with Relu<T> (:16-19): std::max(val, 0) */
int spy_o_relu(const spy_o_tensor *x, spy_o_tensor *dst) {
    const int64_t ne00 = x->ne[0], ne01 = x->ne[1], ne02 = x->ne[2], nrow = t_nrow(x);
    for (int64_t r = 0; r < nrow; r++) {
        const int64_t i03 = r / (ne01 * ne02), i02 = r % (ne01 * ne02) / ne01, i01 = r % ne01;
        const float *s = (const float *)tget(x, 0, i01, i02, i03);
        float *d = (float *)tget(dst, 0, i01, i02, i03);
        for (int64_t i = 0; i < ne00; i++) d[i] = (s[i] < 0.0f) ? 0.0f : s[i];      /* std::max(a, b) = (a < b) ? b : a */
    }
    return 0;
}

/* OperatorQuantizeImpl::execute (backend/host/operator/quantize.cpp:18-41): rows through auto_quantize_inner
 * (vec_convert.h:463-468); F32 -> Q8_0 and F32 -> F16 (the reference's F32 -> Q4_0 is the known-bad *_as_written) */
int spy_o_quantize(const spy_o_tensor *x, spy_o_tensor *dst) {
    if (x->type != SPY_O_F32 || (dst->type != SPY_O_Q8_0 && dst->type != SPY_O_F16)) return 1;
    const int64_t ne00 = x->ne[0], ne01 = x->ne[1], ne02 = x->ne[2], nrow = t_nrow(x);
    for (int64_t r = 0; r < nrow; r++) {
        const int64_t i03 = r / (ne01 * ne02), i02 = r % (ne01 * ne02) / ne01, i01 = r % ne01;
        const float *s = (const float *)tget(x, 0, i01, i02, i03);
        void *d = tget(dst, 0, i01, i02, i03);
        if (dst->type == SPY_O_Q8_0) spy_o_quantize_q8_0(s, d, ne00); else spy_o_quantize_f16(s, (uint16_t *)d, ne00);
    }
    return 0;
}

/* operator_softmax_execute (non-linear.cpp:86-127) when mask == NULL, else
 * operator_masked_softmax_execute (:129-180): t = (s + mask) * scale; m = max t; t -= m;
 * e = mask == -inf ? 0 : exp_lut(fp16(t)); sum = std::reduce(e); e *= 1/sum. */
int spy_o_softmax(const spy_o_tensor *x, const spy_o_tensor *mask, spy_o_tensor *dst, float scale) {
    const int64_t ne0 = dst->ne[0], ne1 = dst->ne[1], ne2 = dst->ne[2], nrow = t_nrow(dst);
    for (int64_t r = 0; r < nrow; r++) {
        const int64_t i3 = r / (ne1 * ne2), i2 = r % (ne1 * ne2) / ne1, i1 = r % ne1;
        const float *s = (const float *)tget(x, 0, i1, i2, i3);
        const float *mk = mask ? (const float *)tget(mask, 0, i1, 0, 0) : NULL;
        float *d = (float *)tget(dst, 0, i1, i2, i3);
        if (mk) { for (int64_t i = 0; i < ne0; i++) d[i] = s[i] + mk[i];
                  for (int64_t i = 0; i < ne0; i++) d[i] *= scale; }
        else    { for (int64_t i = 0; i < ne0; i++) d[i] = s[i] * scale; }
        float mx = d[0];
        for (int64_t i = 1; i < ne0; i++) if (mx < d[i]) mx = d[i];       /* std::max_element */
        if (isnan(mx)) return 4;
        for (int64_t i = 0; i < ne0; i++) d[i] -= mx;
        for (int64_t i = 0; i < ne0; i++) {
            if (mk && mk[i] == -INFINITY) d[i] = 0.0f;
            else d[i] = spy_o_exp_lut(spy_o_f32_to_f16(d[i]));
        }
        const float sum = reduce4(d, ne0, 0);
        if (!(sum > 0.0f)) return 5;
        const float inv = 1.0f / sum;
        for (int64_t i = 0; i < ne0; i++) d[i] *= inv;
    }
    return 0;
}

/* rope_yarn_corr_dim(s) (non-linear.cpp:226-240).  `2 * std::numbers::pi` makes the inner
 * expression double (:228). */
static float yarn_corr_dim(int32_t n_dim, int32_t n_orig, float n_rot, float base) {
    return (float)((double)(float)n_dim * log((double)n_orig / ((double)(n_rot * 2) * 3.141592653589793238462643383279502884)) / (double)(2 * logf(base)));
}

/* rope_yarn (non-linear.cpp:247-260) including rope_yarn_ramp (:242-245) as written:
 * std::clamp(0.0F, 1.0F, y) clamps the VALUE 0 into [1, y] and so returns 1 whenever y >= 1 is
 * a valid upper bound, making the ramp 0; with ext_factor == 0 (the default) it is not evaluated. */
static void rope_yarn(float theta_extrap, float freq_scale, const float corr[2], int64_t i0, float ext_factor,
                      float mscale, float *cos_theta, float *sin_theta) {
    const float theta_interp = freq_scale * theta_extrap;
    float theta = theta_interp;
    if (ext_factor != 0.0f) {
        const float hi = fmaxf(0.001f, corr[1] - corr[0]);
        const float y  = ((float)(i0 / 2) - corr[0]) / hi;
        const float lo_b = 1.0f, v = 0.0f;
        const float clamped = (v < lo_b) ? lo_b : ((y < v) ? y : v);
        const float ramp_mix = (1.0f - clamped) * ext_factor;
        theta = theta_interp * (1 - ramp_mix) + theta_extrap * ramp_mix;
        mscale *= 1.0f + 0.1f * logf(1.0f / freq_scale);
    }
    *cos_theta = cosf(theta) * mscale;
    *sin_theta = sinf(theta) * mscale;
}

/* OperatorRopeImpl::execute (non-linear.cpp:270-371), default branch (mode Norm / None):
 * theta starts at pos[i2] and is multiplied by theta_scale = powf(freq_base, -2/num_dim) once
 * per pair (:304-309); adjacent pairs are rotated (:349-364).  GLM / Neox: unsupported here
 * (Neox aborts in the reference too, :344-346). */
int spy_o_rope(const spy_o_tensor *x, const spy_o_tensor *pos, spy_o_tensor *dst, const spy_o_rope_param *p) {
    if (p->mode == 2) return 1;
    const float theta_scale = powf(p->freq_base, -2.0f / (float)p->num_dim);
    if (p->mode == 4) {
        /* GLM (non-linear.cpp:315-343), as written; the caller keeps the four indices of every i0 inside the row */
        const int64_t ne0 = dst->ne[0], ne1 = dst->ne[1], ne2 = dst->ne[2], ne3 = dst->ne[3];
        const int nd = p->num_dim;
        for (int64_t mi = 0; mi < ne2 * ne3; mi++) {
            const int64_t i3 = mi / ne2, i2 = mi % ne2;
            const int32_t pp = ((const int32_t *)pos->data)[i2];
            for (int64_t i1 = 0; i1 < ne1; i1++) {
                float theta_base = (float)(pp < p->num_context - 2 ? pp : p->num_context - 2);
                float block_theta = (float)(pp - (p->num_context - 2) > 0 ? pp - (p->num_context - 2) : 0);
                for (int64_t i0 = 0; i0 < ne0 / 4; i0++) {
                    const float c = cosf(theta_base), s = sinf(theta_base), cb = cosf(block_theta), sb = sinf(block_theta);
                    theta_base *= theta_scale;
                    block_theta *= theta_scale;
                    const float *sp = (const float *)tget(x, i0, i1, i2, i3);
                    float *dp = (float *)tget(dst, i0, i1, i2, i3);
                    const float x0 = sp[0], x1 = sp[nd / 2], x2 = sp[nd], x3 = sp[nd / 2 + nd];
                    dp[0] = x0 * c - x1 * s;
                    dp[nd / 2] = x0 * s + x1 * c;
                    dp[nd] = x2 * cb - x3 * sb;
                    dp[nd / 2 + nd] = x2 * sb + x3 * cb;
                }
            }
        }
        return 0;
    }
    float corr[2];
    {
        const float start = floorf(yarn_corr_dim(p->num_dim, p->num_origin_context, p->beta_fast, p->freq_base));
        const float end   = ceilf(yarn_corr_dim(p->num_dim, p->num_origin_context, p->beta_slow, p->freq_base));
        corr[0] = fmaxf(0.0f, start);
        corr[1] = fminf((float)(p->num_dim - 1), end);
    }
    const int64_t ne0 = dst->ne[0], ne1 = dst->ne[1], ne2 = dst->ne[2], ne3 = dst->ne[3];
    float *cache = (float *)malloc(sizeof(float) * (size_t)ne0);
    for (int64_t mi = 0; mi < ne2 * ne3; mi++) {
        const int64_t i3 = mi / ne2, i2 = mi % ne2;
        const int32_t pp = ((const int32_t *)pos->data)[i2];
        float theta = (float)*(const int32_t *)tget(pos, i2, 0, 0, 0);
        for (int64_t i0 = 0; i0 < ne0; i0 += 2) {
            rope_yarn(theta, p->freq_scale, corr, i0, p->extend_factor, p->attention_factor, &cache[i0], &cache[i0 + 1]);
            theta *= theta_scale;
        }
        for (int64_t i1 = 0; i1 < ne1; i1++) {
            for (int64_t i0 = 0; i0 < ne0; i0 += 2) {
                const float c = cache[i0], s = cache[i0 + 1];
                float zeta = (p->xpos_base != 0.0f) ? powf(((float)i0 + 0.4f * (float)ne0) / (1.4f * (float)ne0), (float)pp / p->xpos_base) : 1.0f;
                if (p->xpos_down) zeta = 1.0f / zeta;
                const float *sp = (const float *)tget(x, i0, i1, i2, i3);
                float *dp = (float *)tget(dst, i0, i1, i2, i3);
                const float x0 = sp[0], x1 = sp[1];
                dp[0] = x0 * c * zeta - x1 * s * zeta;
                dp[1] = x0 * s * zeta + x1 * c * zeta;
            }
        }
    }
    free(cache);
    return 0;
}

/* dup_execute (view.cpp:83-195): contiguous source -> same-shape destination row by row, or a
 * contiguous destination filled row after row (:132-159, used by the K-cache write); otherwise
 * element by element through the destination's strides with the flat element counter unravelled
 * in the DESTINATION's dimensions (:164-190, used by the transposed V-cache write). */
int spy_o_dup(const spy_o_tensor *src, spy_o_tensor *dst) {
    const int64_t ne0 = dst->ne[0], ne1 = dst->ne[1], ne2 = dst->ne[2];
    const int64_t ne00 = src->ne[0], ne01 = src->ne[1], ne02 = src->ne[2];
    const int64_t nrow = t_nrow(src), src_row_size = t_row_size(src);
    const int ts = src->type, td = dst->type;
    for (int64_t r = 0; r < nrow; r++) {
        const int64_t i03 = r / (ne01 * ne02), i02 = r % (ne01 * ne02) / ne01, i01 = r % ne01;
        const void *sp = tget(src, 0, i01, i02, i03);
        if (t_is_contiguous(src)) {
            void *dp;
            if (t_same_shape(src, dst)) dp = tget(dst, 0, i01, i02, i03);
            else if (t_is_contiguous(dst)) dp = (uint8_t *)dst->data + spy_o_row_size(td, ne00) * r;
            else return 6;
            if (ts == td) memcpy(dp, sp, (size_t)src_row_size);
            else if (ts == SPY_O_F32 && td == SPY_O_F16) { for (int64_t i = 0; i < ne00; i++) ((uint16_t *)dp)[i] = spy_o_f32_to_f16(((const float *)sp)[i]); }
            else if (ts == SPY_O_F16 && td == SPY_O_F32) { for (int64_t i = 0; i < ne00; i++) ((float *)dp)[i] = spy_o_f16_to_f32(((const uint16_t *)sp)[i]); }
            else return 1;
        } else {
            for (int64_t i00 = 0; i00 < ne00; i00++) {
                const int64_t g = i00 + ne00 * r;
                const int64_t i0 = g % ne0, i1 = g / ne0 % ne1, i2 = g % (ne2 * ne1 * ne0) / (ne1 * ne0), i3 = g / (ne2 * ne1 * ne0);
                const float *s1 = (const float *)tget(src, i00, i01, i02, i03);
                if (ts == SPY_O_F32 && td == SPY_O_F32) *(float *)tget(dst, i0, i1, i2, i3) = *s1;
                else if (ts == SPY_O_F32 && td == SPY_O_F16) *(uint16_t *)tget(dst, i0, i1, i2, i3) = spy_o_f32_to_f16(*s1);
                else return 1;
            }
        }
    }
    return 0;
}

/* OperatorContiguousImpl::execute (view.cpp:285-321) */
int spy_o_contiguous(const spy_o_tensor *src, spy_o_tensor *dst) {
    const int64_t ne00 = src->ne[0], ne01 = src->ne[1], ne02 = src->ne[2];
    const int64_t nrow = t_nrow(src), rsz = t_row_size(src);
    const int transposed = src->nb[0] > src->nb[1];                       /* tensor.h:178 */
    for (int64_t r = 0; r < nrow; r++) {
        const int64_t i03 = r / (ne01 * ne02), i02 = r % (ne01 * ne02) / ne01, i01 = r % ne01;
        if (!transposed) memcpy((uint8_t *)dst->data + r * rsz, tget(src, 0, i01, i02, i03), (size_t)rsz);
        else for (int64_t i00 = 0; i00 < ne00; i00++)
            *(float *)tget(dst, i00, i01, i02, i03) = *(const float *)tget(src, i00, i01, i02, i03);
    }
    return 0;
}

/* OperatorGetRowImpl::execute (view.cpp:33-81): same-type memcpy or Q8_0 -> F32 */
int spy_o_get_row(const spy_o_tensor *table, const spy_o_tensor *ids, spy_o_tensor *dst) {
    const int64_t ne00 = table->ne[0];
    const int64_t ne10 = ids->ne[0], ne11 = ids->ne[1], ne12 = ids->ne[2];
    const int64_t n = ne10 * ne11 * ne12, nrow0 = t_nrow(table);
    const int64_t srs = t_row_size(table), drs = t_row_size(dst);
    const int32_t *idp = (const int32_t *)ids->data;
    for (int64_t r = 0; r < n; r++) {
        const int64_t i12 = r / (ne10 * ne11), i11 = r % (ne10 * ne11) / ne10;
        const int64_t row = idp[r];
        if (row >= nrow0 || row < 0) return 7;                           /* view.cpp:61 (assert) */
        const void *sp = tget(table, 0, row, i11, i12);
        if (table->type == dst->type) memcpy((uint8_t *)dst->data + srs * r, sp, (size_t)srs);
        else if (table->type == SPY_O_Q8_0 && dst->type == SPY_O_F32) spy_o_dequantize_q8_0(sp, (float *)((uint8_t *)dst->data + drs * r), ne00);
        else return 1;
    }
    return 0;
}

/* SamplerImpl<Greedy>::sample (greedy.h:20-25): std::max_element -> first maximum */
int32_t spy_o_argmax(const float *logits, int64_t n) {
    int64_t best = 0;
    for (int64_t i = 1; i < n; i++) if (logits[best] < logits[i]) best = i;
    return (int32_t)best;
}

/* ============================================================================================
 * The LLaMA forward pass: the operator sequence LLAMAModel::build_graph wires up
 * (llama.cpp:86-264, attention.cpp:25-302, ffn.cpp:5-42, inout.cpp:5-78), executed in
 * topological order with the host operators above.
 * ========================================================================================== */

static struct { char name[24]; int layer; float *out; } g_tap[16];
static int g_ntap = 0;

void spy_o_llama_tap(const char *name, int layer, float *out) {
    if (!name) { g_ntap = 0; return; }
    if (g_ntap < 16) { strncpy(g_tap[g_ntap].name, name, 23); g_tap[g_ntap].name[23] = 0; g_tap[g_ntap].layer = layer; g_tap[g_ntap].out = out; g_ntap++; }
}

static void tap(const char *name, int layer, const float *src, int64_t n) {
    for (int i = 0; i < g_ntap; i++)
        if (g_tap[i].layer == layer && strcmp(g_tap[i].name, name) == 0) memcpy(g_tap[i].out, src, sizeof(float) * (size_t)n);
}

static void view3(spy_o_tensor *t, int type, void *data, int64_t e0, int64_t e1, int64_t e2, int64_t b0, int64_t b1, int64_t b2) {
    /* Shape(elements, bytes, type) (tensor.h:92-104): trailing dims get ne 1, nb = total */
    t->type = type; t->dim = 3; t->data = data;
    t->ne[0] = e0; t->ne[1] = e1; t->ne[2] = e2; t->ne[3] = 1;
    t->nb[0] = b0; t->nb[1] = b1; t->nb[2] = b2; t->nb[3] = e2 * b2;
}

#define CHK(e) do { int rc_ = (e); if (rc_) { fprintf(stderr, "spy_oracle: %s failed (%d) at line %d\n", #e, rc_, __LINE__); free(buf); return rc_; } } while (0)

int spy_o_llama_forward(const spy_o_llama *m, const int32_t *tokens, int T, int P, float *logits) {
    const int64_t d = m->n_embd, H = m->n_head, hd = d / H, F = m->n_ff, V = m->n_vocab, C = m->n_ctx;
    const int64_t n_kv = (int64_t)P + T;
    const int nt = m->nthread > 0 ? m->nthread : 1;
    if (n_kv > C) return 8;                                                /* llama.cpp:249 */

    /* f32 work buffers */
    const int64_t n_f = 8 * d * T + 3 * F * T + 2 * n_kv * T * H + C * T;
    float *buf = (float *)malloc(sizeof(float) * (size_t)n_f + sizeof(int32_t) * (size_t)T);
    if (!buf) return 3;
    float *x = buf, *xn = x + d * T, *q = xn + d * T, *k = q + d * T, *v = k + d * T, *o = v + d * T,
          *o2 = o + d * T, *t1 = o2 + d * T, *up = t1 + d * T, *gate = up + F * T, *par = gate + F * T,
          *S = par + F * T, *Pm = S + n_kv * T * H, *mask = Pm + n_kv * T * H;
    int32_t *pos = (int32_t *)(mask + C * T);
    for (int i = 0; i < T; i++) pos[i] = P + i;                            /* cli.h:64-66,121-123 */

    /* KQ mask (llama.cpp:248-257): -inf except 0 for j <= i + P; row length n_ctx */
    for (int64_t i = 0; i < T; i++)
        for (int64_t j = 0; j < C; j++) mask[C * i + j] = (j <= i + P) ? 0.0f : -INFINITY;

    spy_o_tensor t_ids, t_pos, t_mask, t_x, t_xn;
    { const int64_t ne[1] = {T}; spy_o_tensor_contiguous(&t_ids, SPY_O_I32, 1, ne, (void *)tokens);
      spy_o_tensor_contiguous(&t_pos, SPY_O_I32, 1, ne, pos); }
    { const int64_t ne[2] = {C, T}; spy_o_tensor_contiguous(&t_mask, SPY_O_I32, 2, ne, mask); }  /* inout.cpp:43-47: typed INT32, read as float */
    { const int64_t ne[2] = {d, T}; spy_o_tensor_contiguous(&t_x, SPY_O_F32, 2, ne, x); spy_o_tensor_contiguous(&t_xn, SPY_O_F32, 2, ne, xn); }

    /* GetRow input_embedding (inout.cpp:26-29) */
    { spy_o_tensor te; const int64_t ne[2] = {d, V}; spy_o_tensor_contiguous(&te, m->t_tok_embd, 2, ne, (void *)m->tok_embd);
      CHK(spy_o_get_row(&te, &t_ids, &t_x)); }

    spy_o_rope_param rp;
    memset(&rp, 0, sizeof(rp));
    rp.mode = 0; rp.num_past = P; rp.num_dim = (int32_t)hd; rp.num_context = (int32_t)C; rp.num_origin_context = (int32_t)C;
    rp.freq_base = m->rope_freq_base; rp.freq_scale = 1.0f; rp.extend_factor = 0.0f; rp.attention_factor = 1.0f;
    rp.beta_fast = 32.0f; rp.beta_slow = 1.0f; rp.xpos_base = 0.0f; rp.xpos_down = 0;

    for (int il = 0; il < m->n_layer; il++) {
        const spy_o_llama_layer *L = &m->layers[il];
        spy_o_tensor t_w, t_nw, t_q, t_k, t_v, t_o, t_o2, t_t1;
        const int64_t ne_dT[2] = {d, T}, ne_d[1] = {d}, ne_dd[2] = {d, d};
        spy_o_tensor_contiguous(&t_q, SPY_O_F32, 2, ne_dT, q); spy_o_tensor_contiguous(&t_k, SPY_O_F32, 2, ne_dT, k);
        spy_o_tensor_contiguous(&t_v, SPY_O_F32, 2, ne_dT, v); spy_o_tensor_contiguous(&t_o, SPY_O_F32, 2, ne_dT, o);
        spy_o_tensor_contiguous(&t_o2, SPY_O_F32, 2, ne_dT, o2); spy_o_tensor_contiguous(&t_t1, SPY_O_F32, 2, ne_dT, t1);

        /* attn_norm + attn_norm_linear (attention.cpp:274-282) */
        CHK(spy_o_norm_rms(&t_x, &t_xn, m->eps));
        spy_o_tensor_contiguous(&t_nw, SPY_O_F32, 1, ne_d, (void *)L->attn_norm);
        CHK(spy_o_binary(2, &t_xn, &t_nw, &t_xn));
        tap("attn_norm", il, xn, d * T);

        /* Q/K/V_project (attention.cpp:28-39) */
        spy_o_tensor_contiguous(&t_w, L->t_wq, 2, ne_dd, (void *)L->wq); CHK(spy_o_matmul(&t_w, &t_xn, &t_q, nt));
        spy_o_tensor_contiguous(&t_w, L->t_wk, 2, ne_dd, (void *)L->wk); CHK(spy_o_matmul(&t_w, &t_xn, &t_k, nt));
        spy_o_tensor_contiguous(&t_w, L->t_wv, 2, ne_dd, (void *)L->wv); CHK(spy_o_matmul(&t_w, &t_xn, &t_v, nt));
        tap("v", il, v, d * T);

        /* Reshape to [hd, H, T] + Rope (attention.cpp:65-101) */
        spy_o_tensor t_q3, t_k3;
        { const int64_t ne[3] = {hd, H, T}; spy_o_tensor_contiguous(&t_q3, SPY_O_F32, 3, ne, q); spy_o_tensor_contiguous(&t_k3, SPY_O_F32, 3, ne, k); }
        CHK(spy_o_rope(&t_q3, &t_pos, &t_q3, &rp));
        CHK(spy_o_rope(&t_k3, &t_pos, &t_k3, &rp));
        tap("q_rope", il, q, d * T); tap("k_rope", il, k, d * T);

        /* Q_out = Permute {0,2,1,3}: [hd, T, H] view (attention.cpp:287-290) */
        spy_o_tensor t_qp = t_q3;
        t_qp.dim = 4; t_qp.ne[1] = t_q3.ne[2]; t_qp.ne[2] = t_q3.ne[1]; t_qp.nb[1] = t_q3.nb[2]; t_qp.nb[2] = t_q3.nb[1];
        /* V_t = Transpose: [T, d] view (attention.cpp:292-295) */
        spy_o_tensor t_vt = t_v; t_vt.ne[0] = t_v.ne[1]; t_vt.ne[1] = t_v.ne[0]; t_vt.nb[0] = t_v.nb[1]; t_vt.nb[1] = t_v.nb[0];

        /* KCache_view + KCache_cpy (attention.cpp:188-205): 1-D f16 view of T*d elements at byte
         * offset row_size(f16, d) * P; then KCache_total: [hd, n_kv, H] strides (2, 2d, 2hd) */
        spy_o_tensor t_kc, t_kall, t_vc, t_vall;
        { const int64_t ne[1] = {T * d}; spy_o_tensor_contiguous(&t_kc, SPY_O_F16, 1, ne, (uint8_t *)m->k_cache[il] + 2 * d * P); }
        CHK(spy_o_dup(&t_k3, &t_kc));
        view3(&t_kall, SPY_O_F16, m->k_cache[il], hd, n_kv, H, 2, 2 * d, 2 * hd);
        /* VCache_view + VCache_cpy (attention.cpp:228-246): [T, d] strides (2, 2C) at byte offset 2P;
         * VCache_total: [n_kv, hd, H] strides (2, 2C, 2C*hd) */
        t_vc.type = SPY_O_F16; t_vc.dim = 2; t_vc.data = (uint8_t *)m->v_cache[il] + 2 * P;
        t_vc.ne[0] = T; t_vc.ne[1] = d; t_vc.ne[2] = 1; t_vc.ne[3] = 1;
        t_vc.nb[0] = 2; t_vc.nb[1] = 2 * C; t_vc.nb[2] = d * 2 * C; t_vc.nb[3] = d * 2 * C;
        CHK(spy_o_dup(&t_vt, &t_vc));
        view3(&t_vall, SPY_O_F16, m->v_cache[il], n_kv, hd, H, 2, 2 * C, 2 * C * hd);

        /* attn_score, softmax, KQV (attention.cpp:108-121) */
        spy_o_tensor t_S, t_P, t_O;
        { const int64_t ne[3] = {n_kv, T, H}; spy_o_tensor_contiguous(&t_S, SPY_O_F32, 3, ne, S); spy_o_tensor_contiguous(&t_P, SPY_O_F32, 3, ne, Pm); }
        CHK(spy_o_matmul(&t_kall, &t_qp, &t_S, nt));
        CHK(spy_o_softmax(&t_S, &t_mask, &t_P, 1.0f / sqrtf((float)hd)));
        { const int64_t ne[3] = {hd, T, H}; spy_o_tensor_contiguous(&t_O, SPY_O_F32, 3, ne, o); }
        CHK(spy_o_matmul(&t_vall, &t_P, &t_O, nt));
        /* Permute {0,2,1,3} + Contiguous + Reshape [d, T] (attention.cpp:122-135) */
        spy_o_tensor t_Op = t_O;
        t_Op.dim = 4; t_Op.ne[1] = t_O.ne[2]; t_Op.ne[2] = t_O.ne[1]; t_Op.nb[1] = t_O.nb[2]; t_Op.nb[2] = t_O.nb[1];
        CHK(spy_o_contiguous(&t_Op, &t_o2));
        tap("kqv", il, o2, d * T);
        /* KQV_linear (attention.cpp:136-139) */
        spy_o_tensor_contiguous(&t_w, L->t_wo, 2, ne_dd, (void *)L->wo); CHK(spy_o_matmul(&t_w, &t_o2, &t_t1, nt));
        tap("attn_out", il, t1, d * T);
        /* ffn_input = attn_out + x (llama.cpp:194-197) */
        CHK(spy_o_binary(0, &t_t1, &t_x, &t_t1));
        tap("ffn_inp", il, t1, d * T);

        /* FFN (ffn.cpp:12-39) */
        CHK(spy_o_norm_rms(&t_t1, &t_xn, m->eps));
        spy_o_tensor_contiguous(&t_nw, SPY_O_F32, 1, ne_d, (void *)L->ffn_norm);
        CHK(spy_o_binary(2, &t_xn, &t_nw, &t_xn));
        spy_o_tensor t_up, t_gate, t_par;
        { const int64_t ne[2] = {F, T}; spy_o_tensor_contiguous(&t_up, SPY_O_F32, 2, ne, up); spy_o_tensor_contiguous(&t_gate, SPY_O_F32, 2, ne, gate);
          spy_o_tensor_contiguous(&t_par, SPY_O_F32, 2, ne, par); }
        { const int64_t ne[2] = {d, F}; spy_o_tensor_contiguous(&t_w, L->t_up, 2, ne, (void *)L->w_up); CHK(spy_o_matmul(&t_w, &t_xn, &t_up, nt));
          spy_o_tensor_contiguous(&t_w, L->t_gate, 2, ne, (void *)L->w_gate); CHK(spy_o_matmul(&t_w, &t_xn, &t_gate, nt)); }
        CHK(spy_o_silu(&t_gate, &t_gate));
        CHK(spy_o_binary(2, &t_up, &t_gate, &t_par));
        tap("ffn_par", il, par, F * T);
        { const int64_t ne[2] = {F, d}; spy_o_tensor_contiguous(&t_w, L->t_down, 2, ne, (void *)L->w_down); CHK(spy_o_matmul(&t_w, &t_par, &t_o, nt)); }
        { spy_o_tensor t_od; spy_o_tensor_contiguous(&t_od, SPY_O_F32, 2, ne_dT, o);
          /* logit_output = ffn_inp + ffn_out (llama.cpp:207-210) -> next layer's input */
          CHK(spy_o_binary(0, &t_t1, &t_od, &t_x)); }
        tap("layer_out", il, x, d * T);
    }

    /* result_norm, result_linear, output (inout.cpp:59-75) */
    CHK(spy_o_norm_rms(&t_x, &t_xn, m->eps));
    { spy_o_tensor t_nw; const int64_t ne[1] = {d}; spy_o_tensor_contiguous(&t_nw, SPY_O_F32, 1, ne, (void *)m->out_norm);
      CHK(spy_o_binary(2, &t_xn, &t_nw, &t_xn)); }
    { spy_o_tensor t_w, t_l; const int64_t ne[2] = {d, V}, nel[2] = {V, T};
      spy_o_tensor_contiguous(&t_w, m->t_out, 2, ne, (void *)m->w_out);
      spy_o_tensor_contiguous(&t_l, SPY_O_F32, 2, nel, logits);
      CHK(spy_o_matmul(&t_w, &t_xn, &t_l, nt)); }
    free(buf);
    return 0;
}
