/*
 * Synthetic model tensors for the LLaMA-2 shapes: a counter-based generator that yields the same
 * bytes on every machine, and the GGUF block quantizers used to store them.
 *
 * The reference ships no model and no usable FP32->Q4_0 quantizer (its
 * Quantizator<FP32,Q4_0>, backend/host/include/simd/vec_convert.h:86-120 in the Spy tree, consumes
 * 16 floats per 32-element block and zeroes its inverse scale), so tensors are quantized with the
 * rule its Dot<Q4_0,Q8_0> decodes (vec_dot.h:62-75): d = max/-8, q = min(15, (int8)(x/d + 8.5)),
 * element j in the low nibble of qs[j], element j+16 in the high nibble.  Q8_0 follows
 * Quantizator<FP32,Q8_0> (vec_convert.h:178-261).  Q4_K and Q6_K have layouts only in the reference
 * (number_impl/k-quant.h:101-111,177-182) and no quantizer anywhere; the rule here is this project's
 * own, one pass per super-block (no iterative search): Q4_K an affine 16-level grid per 32 elements
 * whose 8 steps and 8 minima are held in 6 bits against the super-block maxima, Q6_K a symmetric
 * 64-level grid per 16 elements whose 16 steps are held as int8 against the super-block maximum.
 *
 * Values: x = (sum of 12 uniform 16-bit integers - 6*65535) * c.  The integer sum is exact, the
 * conversion to float is exact (< 2^24) and the single multiplication rounds identically
 * everywhere, so the stream is bit-reproducible; with c = std / sqrt(65536^2 - 1) it is the classic
 * 12-term approximation of N(0, std) (lighter tails than a true normal beyond ~3 sigma).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

/* element `idx` of stream `seed`: depends on (seed, idx) only */
static inline float synth_value(uint64_t seed, uint64_t idx, float c) {
    const uint64_t base = splitmix64(seed) ^ (idx * 3ull);
    int32_t s = 0;
    for (int k = 0; k < 3; k++) {
        const uint64_t r = splitmix64(base + (uint64_t)k);
        s += (int32_t)(r & 0xFFFF) + (int32_t)((r >> 16) & 0xFFFF) + (int32_t)((r >> 32) & 0xFFFF) + (int32_t)((r >> 48) & 0xFFFF);
    }
    return (float)(s - 6 * 65535) * c;
}

/* std of the integer sum: sqrt(12 * (65536^2 - 1) / 12) */
static inline float synth_scale(float std) { return (float)((double)std / sqrt(65536.0 * 65536.0 - 1.0)); }

static uint16_t f32_to_f16(float f) {          /* IEEE round-to-nearest-even */
    uint32_t x; memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u, ax = x & 0x7fffffffu;
    if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (ax >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);
    const uint32_t e = ax >> 23;
    if (e < 113) {
        const uint32_t shift = 126 - e;
        if (shift > 24) return (uint16_t)sign;
        const uint32_t mant = (ax & 0x7fffffu) | 0x800000u;
        uint32_t h = mant >> shift;
        const uint32_t rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((e - 112) << 10) | ((ax >> 13) & 0x3ffu);
    const uint32_t rem = ax & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

static void quant_q4_0_block(const float *x, uint8_t *out) {
    float amax = 0.0f, max = 0.0f;
    for (int j = 0; j < 32; j++) if (amax < fabsf(x[j])) { amax = fabsf(x[j]); max = x[j]; }
    const float d = max / -8.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
    const uint16_t dh = f32_to_f16(d);
    memcpy(out, &dh, 2);
    for (int j = 0; j < 16; j++) {
        int q0 = (int8_t)(x[j] * id + 8.5f), q1 = (int8_t)(x[j + 16] * id + 8.5f);
        if (q0 > 15) q0 = 15;
        if (q1 > 15) q1 = 15;
        out[2 + j] = (uint8_t)(q0 | (q1 << 4));
    }
}

static void quant_q8_0_block(const float *x, uint8_t *out) {
    float amax = 0.0f;
    for (int j = 0; j < 32; j++) if (fabsf(x[j]) > amax) amax = fabsf(x[j]);
    const float d = amax / 127.0f, id = amax != 0.0f ? 127.0f / amax : 0.0f;
    const uint16_t dh = f32_to_f16(d);
    memcpy(out, &dh, 2);
    for (int j = 0; j < 32; j++) {
        int q = (int)rintf(x[j] * id);
        q = q < -128 ? -128 : q > 127 ? 127 : q;
        out[2 + j] = (uint8_t)(int8_t)q;
    }
}

static float f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1F, m = h & 0x3FFu, x;
    if (e == 0) {
        if (m == 0) x = sign;
        else { int k = -1; do { m <<= 1; k++; } while (!(m & 0x400u)); x = sign | ((uint32_t)(112 - k) << 23) | ((m & 0x3FFu) << 13); }
    } else if (e == 31) x = sign | 0x7F800000u | (m << 13);
    else x = sign | ((e + 112) << 23) | (m << 13);
    float f; memcpy(&f, &x, 4); return f;
}

/* Q4_K super-block (144 bytes: d, dmin, scales[12], qs[128]) from 256 floats.  Sub-block j (32 elements): grid
 * [min(0, lo), hi] in 15 steps; step and -min rounded to 6 bits against d = max step / 63, dmin = max(-min) / 63;
 * (scale, min) pair j lives in scales[] as ggml packs it: j < 4: low 6 bits of bytes j and j + 4; j >= 4: low / high
 * nibble of byte j + 4 plus the top two bits of bytes j - 4 and j.  Element l of sub-blocks 2i / 2i+1 is the low /
 * high nibble of qs[32 i + l]. */
static void quant_q4_k_block(const float *x, uint8_t *out) {
    float step[8], neg_min[8], top_step = 0.0f, top_min = 0.0f;
    for (int j = 0; j < 8; j++) {
        float lo = 0.0f, hi = 0.0f;
        for (int l = 0; l < 32; l++) { const float v = x[32 * j + l]; if (v < lo) lo = v; if (v > hi) hi = v; }
        step[j] = (hi - lo) / 15.0f; neg_min[j] = -lo;
        if (step[j] > top_step) top_step = step[j];
        if (neg_min[j] > top_min) top_min = neg_min[j];
    }
    const uint16_t dh = f32_to_f16(top_step / 63.0f), mh = f32_to_f16(top_min / 63.0f);
    const float d = f16_to_f32(dh), dmin = f16_to_f32(mh);
    memcpy(out, &dh, 2); memcpy(out + 2, &mh, 2);
    uint8_t *sc6 = out + 4, *qs = out + 16;
    memset(sc6, 0, 12);
    int sc[8], mn[8];
    for (int j = 0; j < 8; j++) {
        sc[j] = d > 0.0f ? (int)rintf(step[j] / d) : 0;       if (sc[j] > 63) sc[j] = 63;
        mn[j] = dmin > 0.0f ? (int)rintf(neg_min[j] / dmin) : 0; if (mn[j] > 63) mn[j] = 63;
        if (j < 4) { sc6[j] |= (uint8_t)sc[j]; sc6[j + 4] |= (uint8_t)mn[j]; }
        else {
            sc6[j + 4] = (uint8_t)((sc[j] & 0x0F) | ((mn[j] & 0x0F) << 4));
            sc6[j - 4] |= (uint8_t)((sc[j] >> 4) << 6);
            sc6[j]     |= (uint8_t)((mn[j] >> 4) << 6);
        }
    }
    for (int j = 0; j < 8; j++) {
        const float d1 = d * (float)sc[j], m1 = dmin * (float)mn[j];
        for (int l = 0; l < 32; l++) {
            int q = d1 > 0.0f ? (int)rintf((x[32 * j + l] + m1) / d1) : 0;
            q = q < 0 ? 0 : q > 15 ? 15 : q;
            uint8_t *p = &qs[32 * (j / 2) + l];
            *p = (j & 1) ? (uint8_t)((*p & 0x0F) | (q << 4)) : (uint8_t)q;
        }
    }
}

/* Q6_K super-block (210 bytes: ql[128], qh[64], scales[16] int8, d) from 256 floats.  Sub-block j (16 elements): step
 * amax / 31, held as int8 scale = ceil(step / d) against d = max step / 127; q = round(x / (d * scale)) in -32..31,
 * stored + 32 as 6 bits: for half n (128 elements), group g (32 elements), l < 32: low 4 bits in the low (g < 2) or
 * high nibble of ql[64 n + l + 32 (g & 1)], top 2 bits at bit 2 g of qh[32 n + l]. */
static void quant_q6_k_block(const float *x, uint8_t *out) {
    float step[16], top = 0.0f;
    for (int j = 0; j < 16; j++) {
        float amax = 0.0f;
        for (int l = 0; l < 16; l++) { const float a = fabsf(x[16 * j + l]); if (a > amax) amax = a; }
        step[j] = amax / 31.0f;
        if (step[j] > top) top = step[j];
    }
    const uint16_t dh = f32_to_f16(top / 127.0f);
    const float d = f16_to_f32(dh);
    uint8_t *ql = out, *qh = out + 128;
    int8_t *scales = (int8_t *)(out + 192);
    memset(out, 0, 192);
    memcpy(out + 208, &dh, 2);
    for (int j = 0; j < 16; j++) {
        int sc = d > 0.0f ? (int)ceilf(step[j] / d) : 0;
        scales[j] = (int8_t)(sc > 127 ? 127 : sc);
    }
    for (int e = 0; e < 256; e++) {
        const float st = d * (float)scales[e / 16];
        int q = st > 0.0f ? (int)rintf(x[e] / st) : 0;
        q = (q < -32 ? -32 : q > 31 ? 31 : q) + 32;
        const int n = e >> 7, g = (e >> 5) & 3, l = e & 31;
        uint8_t *lo = &ql[64 * n + l + 32 * (g & 1)];
        *lo |= (uint8_t)((q & 0x0F) << (g < 2 ? 0 : 4));
        qh[32 * n + l] |= (uint8_t)((q >> 4) << (2 * g));
    }
}

/* type ids as GGUF: 0 F32, 2 Q4_0, 8 Q8_0, 12 Q4_K, 14 Q6_K.  Returns bytes written, 0 for an unsupported type. */
size_t spy_synth_quantize(int type, const float *x, int64_t n, void *out) {
    uint8_t *o = (uint8_t *)out;
    if (type == 0) { memcpy(out, x, (size_t)n * 4); return (size_t)n * 4; }
    if (n % 32) return 0;
    const int64_t nb = n / 32;
    if (type == 2) {
        #pragma omp parallel for schedule(static)
        for (int64_t b = 0; b < nb; b++) quant_q4_0_block(x + b * 32, o + b * 18);
        return (size_t)nb * 18;
    }
    if (type == 8) {
        #pragma omp parallel for schedule(static)
        for (int64_t b = 0; b < nb; b++) quant_q8_0_block(x + b * 32, o + b * 34);
        return (size_t)nb * 34;
    }
    if ((type == 12 || type == 14) && n % 256 == 0) {
        const int64_t nsb = n / 256;
        const int sb = type == 12 ? 144 : 210;
        #pragma omp parallel for schedule(static)
        for (int64_t b = 0; b < nsb; b++) { if (type == 12) quant_q4_k_block(x + b * 256, o + b * sb); else quant_q6_k_block(x + b * 256, o + b * sb); }
        return (size_t)nsb * sb;
    }
    return 0;
}

void spy_synth_f32(uint64_t seed, int64_t n, float std, float *out) {
    const float c = synth_scale(std);
    #pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) out[i] = synth_value(seed, (uint64_t)i, c);
}

/* n elements of stream `seed`, scaled to `std`, every `outlier_every`-th element (0 = none)
 * multiplied by outlier_mul, quantized to `type` straight into `out` (no float copy kept). */
size_t spy_synth_tensor(int type, uint64_t seed, int64_t n, float std, int64_t outlier_every, float outlier_mul, void *out) {
    const float c = synth_scale(std);
    if (type == 0) {
        float *o = (float *)out;
        #pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < n; i++) {
            float v = synth_value(seed, (uint64_t)i, c);
            if (outlier_every > 0 && i % outlier_every == outlier_every - 1) v *= outlier_mul;
            o[i] = v;
        }
        return (size_t)n * 4;
    }
    if (type == 12 || type == 14) {              /* K-quants: whole super-blocks of 256 elements */
        if (n % 256) return 0;
        const int64_t nsb = n / 256;
        const int sb = type == 12 ? 144 : 210;
        uint8_t *o = (uint8_t *)out;
        #pragma omp parallel for schedule(static)
        for (int64_t b = 0; b < nsb; b++) {
            float x[256];
            for (int j = 0; j < 256; j++) {
                const int64_t i = b * 256 + j;
                float v = synth_value(seed, (uint64_t)i, c);
                if (outlier_every > 0 && i % outlier_every == outlier_every - 1) v *= outlier_mul;
                x[j] = v;
            }
            if (type == 12) quant_q4_k_block(x, o + b * sb); else quant_q6_k_block(x, o + b * sb);
        }
        return (size_t)nsb * sb;
    }
    if ((type != 2 && type != 8) || n % 32) return 0;
    const int64_t nb = n / 32;
    const int bs = type == 2 ? 18 : 34;
    uint8_t *o = (uint8_t *)out;
    #pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < nb; b++) {
        float x[32];
        for (int j = 0; j < 32; j++) {
            const int64_t i = b * 32 + j;
            float v = synth_value(seed, (uint64_t)i, c);
            if (outlier_every > 0 && i % outlier_every == outlier_every - 1) v *= outlier_mul;
            x[j] = v;
        }
        if (type == 2) quant_q4_0_block(x, o + b * bs); else quant_q8_0_block(x, o + b * bs);
    }
    return (size_t)nb * bs;
}
