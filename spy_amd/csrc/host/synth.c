/*
 * Synthetic model tensors for the LLaMA-2 shapes: a counter-based generator that yields the same
 * bytes on every machine, and the GGUF block quantizers used to store them.
 *
 * The reference ships no model and no usable FP32->Q4_0 quantizer (its
 * Quantizator<FP32,Q4_0>, backend/host/include/simd/vec_convert.h:86-120 in the Spy tree, consumes
 * 16 floats per 32-element block and zeroes its inverse scale), so tensors are quantized with the
 * rule its Dot<Q4_0,Q8_0> decodes (vec_dot.h:62-75): d = max/-8, q = min(15, (int8)(x/d + 8.5)),
 * element j in the low nibble of qs[j], element j+16 in the high nibble.  Q8_0 follows
 * Quantizator<FP32,Q8_0> (vec_convert.h:178-261).
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

/* type ids as GGUF: 0 F32, 2 Q4_0, 8 Q8_0.  Returns bytes written, 0 for an unsupported type. */
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
