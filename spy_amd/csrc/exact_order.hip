// Exact-order forms of the operators whose fp32 results depend on the ORDER of their additions or on
// the host's libm: the quantized and fp16 dots of MatMul, NormRMS, Softmax, Silu and Rope.
//
// The fast kernels add a row's terms in whatever order suits 64 lanes; Spy's host backend adds them in
// the order of its 8-lane AVX accumulators and of libstdc++'s four-way reduce, and looks exp / silu up
// in tables that glibc filled.  The results agree to about 1e-7, but every MatMul re-quantizes its
// activations to Q8_0 (mat.cpp:95-128) and the softmax rounds its exp argument to fp16
// (non-linear.cpp:170), so a last-ulp difference moves a rounding now and then and the greedy tokens of
// a model with near-tied logits can differ.  With spy_hip_set_exact_order(1) (or SPY_HIP_EXACT=1) the
// spy_hip_op_* entry points launch the kernels below instead: every accumulator of the host loops has
// one lane (or one thread) that walks its sum in the host backend's order, the tables and the rotation
// angles come from the host's libm, and the outputs are the host backend's bit for bit.  The token loop
// issues the prompt passes of a model in the host's order through these kernels as well (a thread-local
// scope, spy_exact_thread_scope); its single-token passes have fused kernels of their own.
#include "common.cuh"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <vector>

namespace {

struct xdesc {
    uint8_t *p;
    int64_t ne[4], nb[4];
};
xdesc mkx(const spy_hip_tensor *t) {
    xdesc d;
    d.p = (uint8_t *)t->data;
    for (int i = 0; i < 4; i++) { d.ne[i] = t->ne[i]; d.nb[i] = t->nb[i]; }
    return d;
}
__device__ __forceinline__ uint8_t *xat(const xdesc &t, int64_t i0, int64_t i1, int64_t i2, int64_t i3) {
    return t.p + i0 * t.nb[0] + i1 * t.nb[1] + i2 * t.nb[2] + i3 * t.nb[3];
}

int g_exact = -1;          // -1: not decided yet (environment), 0 / 1
// Per-device state, set up once per device and kept until the process ends (never freed, never replaced: a stream of
// another thread may still read it), guarded by one mutex:
//   lut    exp table [65536], then silu table [65536]; built by spy_exact_device_setup, which spy_hip_init calls
//   rope   the Rope tables (cos / sin of every position of a context) by parameter set; built by spy_hip_rope_prepare, or by
//          the first exact-order Rope call with a new parameter set where that call is allowed to allocate (not under capture)
#define XO_MAX_DEVICES 64
#define XO_MAX_ROPE_TABLES 16
struct rope_key { int64_t npos, ne0; float freq_base, freq_scale, factor; int32_t num_dim; };
struct rope_entry { rope_key k; float *dev; };
struct device_state { float *lut = nullptr; std::vector<rope_entry> rope; };
device_state g_dev[XO_MAX_DEVICES];
std::mutex g_mu;
int current_device() { int dev = -1; return (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < XO_MAX_DEVICES) ? dev : -1; }

// IEEE binary16 -> binary32 on the host
float host_h2f(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1F, mant = h & 0x3FFu, x;
    if (exp == 0) {
        if (mant == 0) x = sign;
        else {
            int e = -1;
            do { mant <<= 1; e++; } while (!(mant & 0x400u));
            x = sign | ((uint32_t)(112 - e) << 23) | ((mant & 0x3FFu) << 13);
        }
    } else if (exp == 31) x = sign | 0x7F800000u | (mant << 13);
    else x = sign | ((exp + 112) << 23) | (mant << 13);
    float f;
    memcpy(&f, &x, 4);
    return f;
}

// The reference's tables (lookup_table_impl/non-linear.h:39-47,131-139): entry k holds the function of
// float(half k), evaluated by the host's libm in fp32; the loop stops before k = 0xFFFF, which stays 0.
int device_luts(const float **lut) {
    const int dev = current_device();
    if (dev < 0) return SPY_HIP_EINVAL;
    std::lock_guard<std::mutex> lock(g_mu);
    if (g_dev[dev].lut) { *lut = g_dev[dev].lut; return 0; }
    std::vector<float> h(2 * 65536, 0.0f);
    for (uint32_t k = 0; k < 0xFFFFu; k++) {
        const float v = host_h2f((uint16_t)k);
        h[k] = expf(v);
        h[65536 + k] = v / (1.0f + expf(-v));
    }
    float *d = nullptr;
    hipError_t e = hipMalloc((void **)&d, h.size() * sizeof(float));
    if (e != hipSuccess) return (int)e;
    e = hipMemcpy(d, h.data(), h.size() * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) { (void)hipFree(d); return (int)e; }
    g_dev[dev].lut = d;
    *lut = d;
    return 0;
}

// conversion.h:39-41: the fp16 -> fp32 table has no entry for 0xFFFF either
__device__ __forceinline__ float h2f_tab(uint16_t h) { return h == 0xFFFFu ? 0.0f : h2f(h); }

// libstdc++'s std::reduce / std::transform_reduce over a random-access range: groups of four as
// init = init + ((a0 + a1) + (a2 + a3)), then the remaining elements one by one.  The 256 threads of the
// workgroup prepare the group sums of up to 4096 elements in LDS, thread 0 adds them in order.
template <bool SQUARE>
__device__ float reduce4_block(const float *p, int64_t n, float *s_grp, float *s_out) {
    const int64_t ngrp = n / 4;
    float init = 0.0f;
    for (int64_t g0 = 0; g0 < ngrp; g0 += 1024) {
        const int cnt = (int)min((int64_t)1024, ngrp - g0);
        for (int g = threadIdx.x; g < cnt; g += 256) {
            const float *q = p + (g0 + g) * 4;
            float a0 = q[0], a1 = q[1], a2 = q[2], a3 = q[3];
            if (SQUARE) { a0 = a0 * a0; a1 = a1 * a1; a2 = a2 * a2; a3 = a3 * a3; }
            const float v1 = a0 + a1, v2 = a2 + a3;
            s_grp[g] = v1 + v2;
        }
        __syncthreads();
        if (threadIdx.x == 0)
            for (int g = 0; g < cnt; g++) init = init + s_grp[g];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        for (int64_t i = ngrp * 4; i < n; i++) { const float a = p[i]; init = init + (SQUARE ? a * a : a); }
        *s_out = init;
    }
    __syncthreads();
    return *s_out;
}

// NormRMS (non-linear.cpp:194-223): one workgroup per row
__global__ __launch_bounds__(256) void exact_norm_rms_kernel(xdesc x, xdesc y, float eps) {
    __shared__ float s_grp[1024];
    __shared__ float s_out;
    const int64_t r = blockIdx.x;
    const int64_t ne0 = y.ne[0], ne1 = y.ne[1], ne2 = y.ne[2];
    const int64_t i3 = r / (ne1 * ne2), i2 = r % (ne1 * ne2) / ne1, i1 = r % ne1;
    const float *s = (const float *)xat(x, 0, i1, i2, i3);
    float *d = (float *)xat(y, 0, i1, i2, i3);
    const float sum = reduce4_block<true>(s, ne0, s_grp, &s_out);
    const float mean = sum / (float)ne0;
    const float scale = 1.0f / sqrtf(mean + eps);
    for (int64_t i = threadIdx.x; i < ne0; i += 256) d[i] = s[i] * scale;
}

// Silu (non-linear.cpp:11-14,57-77): table look-up on fp16(x)
__global__ __launch_bounds__(256) void exact_silu_kernel(xdesc x, xdesc d, const float *__restrict__ lut, int64_t total) {
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= total) return;
    const int64_t i0 = g % x.ne[0], r = g / x.ne[0];
    const int64_t i1 = r % x.ne[1], i2 = r / x.ne[1] % x.ne[2], i3 = r / (x.ne[1] * x.ne[2]);
    *(float *)xat(d, i0, i1, i2, i3) = lut[65536 + f2h(*(const float *)xat(x, i0, i1, i2, i3))];
}

// Softmax (non-linear.cpp:86-180), the row kept in dst between the steps as the reference keeps it
__global__ __launch_bounds__(256) void exact_softmax_kernel(xdesc x, xdesc mask, bool has_mask, xdesc y, float scale, const float *__restrict__ lut) {
    __shared__ float s_grp[1024];
    __shared__ float s_out;
    __shared__ float s_part[4];
    const int64_t r = blockIdx.x;
    const int64_t ne0 = y.ne[0], ne1 = y.ne[1], ne2 = y.ne[2];
    const int64_t i3 = r / (ne1 * ne2), i2 = r % (ne1 * ne2) / ne1, i1 = r % ne1;
    const float *s = (const float *)xat(x, 0, i1, i2, i3);
    const float *mk_ = has_mask ? (const float *)xat(mask, 0, i1, 0, 0) : nullptr;
    float *d = (float *)xat(y, 0, i1, i2, i3);
    float mx = -INFINITY;
    for (int64_t i = threadIdx.x; i < ne0; i += 256) {
        float t;
        if (has_mask) { t = s[i] + mk_[i]; t = t * scale; }
        else t = s[i] * scale;
        d[i] = t;
        mx = fmaxf(mx, t);
    }
    mx = wave_max(mx);
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(s_part[0], s_part[1]), fmaxf(s_part[2], s_part[3]));
    for (int64_t i = threadIdx.x; i < ne0; i += 256) {
        const float t = d[i] - mx;
        d[i] = (has_mask && mk_[i] == -INFINITY) ? 0.0f : lut[f2h(t)];
    }
    __syncthreads();
    const float sum = reduce4_block<false>(d, ne0, s_grp, &s_out);
    const float inv = 1.0f / sum;
    for (int64_t i = threadIdx.x; i < ne0; i += 256) d[i] *= inv;
}

// Rope (non-linear.cpp:270-371), default branch; tab = cos, sin per pair, from the host: one row per token of
// this call (pos == nullptr) or one row per position 0 .. npos-1, the token's position read here.  zeta: the xpos
// factors of the call's tokens (one per pair, after the cos / sin of a row: rows of ne0 + ne0 / 2 floats), or none.
__global__ __launch_bounds__(64) void exact_rope_kernel(xdesc x, xdesc y, const float *__restrict__ tab, const uint8_t *__restrict__ pos, int64_t pos_stride,
                                                        int64_t npos, int *err, int zeta) {
    const int64_t i1 = blockIdx.x, i2 = blockIdx.y, i3 = blockIdx.z;
    const int64_t ne0 = y.ne[0];
    const int64_t tab_row = zeta ? ne0 + ne0 / 2 : ne0;
    int64_t row = i2;
    if (pos) {
        row = *(const int32_t *)(pos + i2 * pos_stride);
        if (row < 0 || row >= npos) { if (threadIdx.x == 0) *err = 1; return; }      // beyond the context the table was built for
    }
    for (int64_t i0 = 2 * threadIdx.x; i0 < ne0; i0 += 128) {
        const float c = tab[row * tab_row + i0], s = tab[row * tab_row + i0 + 1];
        const float *sp = (const float *)xat(x, i0, i1, i2, i3);
        float *dp = (float *)xat(y, i0, i1, i2, i3);
        const float x0 = sp[0], x1 = sp[1];
        float a = x0 * c, b = x1 * s, e = x0 * s, f = x1 * c;
        if (zeta) {
            const float z = tab[row * tab_row + ne0 + i0 / 2];
            a = a * z; b = b * z; e = e * z; f = f * z;
        }
        dp[0] = a - b;
        dp[1] = e + f;
    }
}

// mul_sum_i8_pairs (vec_util.h:101-110) on four int8 pairs: |x| as uint8 times y with the sign of x,
// adjacent products added with int16 saturation (maddubs), the two sums added as int32 (madd with ones)
__device__ __forceinline__ int32_t mul_sum4(const int8_t *x, const int8_t *y) {
    int32_t pair[2];
#pragma unroll
    for (int p = 0; p < 2; p++) {
        int32_t s = 0;
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const int8_t xv = x[2 * p + k], yv = y[2 * p + k];
            const int32_t ax = (uint8_t)(xv < 0 ? -xv : xv);
            const int32_t sy = xv < 0 ? (int32_t)(int8_t)(-yv) : (xv == 0 ? 0 : (int32_t)yv);
            s += ax * sy;
        }
        pair[p] = s < -32768 ? -32768 : (s > 32767 ? 32767 : s);
    }
    return pair[0] + pair[1];
}

// hsum_float_8 (vec_util.h:75-81)
__device__ __forceinline__ float hsum8(const float *a) {
    const float r0 = a[4] + a[0], r1 = a[5] + a[1], r2 = a[6] + a[2], r3 = a[7] + a[3];
    const float s0 = r0 + r2, s1 = r1 + r3;
    return s0 + s1;
}

// Dot<Q4_0,Q8_0>::exec (vec_dot.h:42-86): accumulators 4..7 take the low-nibble half (elements 0..15),
// 0..3 the high-nibble half, four products each; acc = fma(d_w * d_x, float(part), acc) block after block
__device__ float dot_q4_0(const uint8_t *wv, const uint8_t *xv, int64_t n) {
    const blk_q4_0 *w = (const blk_q4_0 *)wv;
    const blk_q8_0 *x = (const blk_q8_0 *)xv;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int64_t i = 0; i < n / 32; i++) {
        const float d = h2f_tab(w[i].d) * h2f_tab(x[i].d);
        int8_t lo[16], hi[16], q[32];
#pragma unroll
        for (int j = 0; j < 16; j++) { const uint8_t b = w[i].qs[j]; lo[j] = (int8_t)((b & 0x0F) - 8); hi[j] = (int8_t)((b >> 4) - 8); }
#pragma unroll
        for (int j = 0; j < 32; j++) q[j] = x[i].qs[j];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            acc[4 + k] = fmaf(d, (float)mul_sum4(lo + 4 * k, q + 4 * k), acc[4 + k]);
            acc[k] = fmaf(d, (float)mul_sum4(hi + 4 * k, q + 16 + 4 * k), acc[k]);
        }
    }
    return hsum8(acc);
}

// Dot<Q8_0,Q8_0>::exec (vec_dot.h:88-115): accumulator l takes elements 4l..4l+3
__device__ float dot_q8_0(const uint8_t *wv, const uint8_t *xv, int64_t n) {
    const blk_q8_0 *w = (const blk_q8_0 *)wv, *x = (const blk_q8_0 *)xv;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int64_t i = 0; i < n / 32; i++) {
        const float d = h2f_tab(w[i].d) * h2f_tab(x[i].d);
        int8_t a[32], b[32];
#pragma unroll
        for (int j = 0; j < 32; j++) { a[j] = w[i].qs[j]; b[j] = x[i].qs[j]; }
#pragma unroll
        for (int l = 0; l < 8; l++) acc[l] = fmaf(d, (float)mul_sum4(a + 4 * l, b + 4 * l), acc[l]);
    }
    return hsum8(acc);
}

// Dot<FP16,FP16>::exec (vec_dot.h:117-146): four 8-lane fma accumulators over chunks of 32 while
// i + 32 < n, FP16::block_reduce (vec_util.h:61-71), the last 1..32 elements as a scalar sum of products
// through the conversion table, result = tail + simd
__device__ float dot_f16(const uint8_t *av, const uint8_t *bv, int64_t n) {
    const uint16_t *a = (const uint16_t *)av, *b = (const uint16_t *)bv;
    float sum[32];
#pragma unroll
    for (int l = 0; l < 32; l++) sum[l] = 0.0f;
    int64_t i = 0;
    for (; i + 32 < n; i += 32) {
#pragma unroll
        for (int l = 0; l < 32; l++) sum[l] = fmaf(h2f(a[i + l]), h2f(b[i + l]), sum[l]);
    }
#pragma unroll
    for (int l = 0; l < 8; l++) { sum[l] += sum[16 + l]; sum[8 + l] += sum[24 + l]; }
#pragma unroll
    for (int l = 0; l < 8; l++) sum[l] += sum[8 + l];
    const float t0 = sum[0] + sum[4], t1 = sum[1] + sum[5], t2 = sum[2] + sum[6], t3 = sum[3] + sum[7];
    const float u0 = t0 + t1, u1 = t2 + t3;
    const float simd = u0 + u1;
    float tail = 0.0f;
    for (; i < n; i++) { const float pr = h2f_tab(a[i]) * h2f_tab(b[i]); tail += pr; }
    return tail + simd;
}

// K-quant rows against Q8_0 activations.  The reference has no K-quant arithmetic; the order is the one
// this project defines: one accumulator, sub-block after sub-block.
__device__ float dot_q4_k(const uint8_t *wv, const uint8_t *xv, int64_t n) {
    const blk_q4_k *w = (const blk_q4_k *)wv;
    const blk_q8_0 *x = (const blk_q8_0 *)xv;
    float acc = 0.0f;
    for (int64_t b = 0; b < n / 256; b++) {
        const float d = h2f_tab(w[b].d), dmin = h2f_tab(w[b].dmin);
        const uint8_t *s = w[b].scales;
        for (int j = 0; j < 8; j++) {
            int32_t sc, m;
            if (j < 4) { sc = s[j] & 63; m = s[j + 4] & 63; }
            else { sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4); m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4); }
            const blk_q8_0 *xb = &x[b * 8 + j];
            int32_t isum = 0, bsum = 0;
            for (int l = 0; l < 32; l++) {
                const uint8_t byte = w[b].qs[32 * (j / 2) + l];
                const int32_t q = (j & 1) ? (byte >> 4) : (byte & 0x0F);
                const int32_t xq = xb->qs[l];
                isum += q * xq;
                bsum += xq;
            }
            const float dx = h2f_tab(xb->d);
            const float pos = d * (float)(sc * isum), neg = dmin * (float)(m * bsum);
            acc = fmaf(dx, pos - neg, acc);
        }
    }
    return acc;
}

__device__ __forceinline__ int32_t q6k_get(const blk_q6_k *x, int e) {
    const int half = e / 128, r = e % 128, grp = r / 32, l = r % 32;
    const uint8_t *ql = x->ql + 64 * half, *qh = x->qh + 32 * half;
    int32_t lo;
    switch (grp) {
    case 0: lo = ql[l] & 0x0F; break;
    case 1: lo = ql[l + 32] & 0x0F; break;
    case 2: lo = ql[l] >> 4; break;
    default: lo = ql[l + 32] >> 4; break;
    }
    const int32_t hi = (qh[l] >> (2 * grp)) & 3;
    return (lo | (hi << 4)) - 32;
}

__device__ float dot_q6_k(const uint8_t *wv, const uint8_t *xv, int64_t n) {
    const blk_q6_k *w = (const blk_q6_k *)wv;
    const blk_q8_0 *x = (const blk_q8_0 *)xv;
    float acc = 0.0f;
    for (int64_t b = 0; b < n / 256; b++) {
        const float d = h2f_tab(w[b].d);
        for (int t = 0; t < 8; t++) {
            const blk_q8_0 *xb = &x[b * 8 + t];
            int32_t s = 0;
            for (int h = 0; h < 2; h++) {
                int32_t isum = 0;
                for (int l = 0; l < 16; l++) isum += q6k_get(&w[b], 32 * t + 16 * h + l) * (int32_t)xb->qs[16 * h + l];
                s += (int32_t)w[b].scales[2 * t + h] * isum;
            }
            const float dd = h2f_tab(xb->d) * d;
            acc = fmaf(dd, (float)s, acc);
        }
    }
    return acc;
}

// MatMul (mat.cpp:130-143): one thread per output element, the output index running fastest along the
// weight rows; xm = the activations in the intermediate type, contiguous [ne00, ne11, ne02, ne03]
template <int WT>
__global__ __launch_bounds__(64) void exact_dots_kernel(xdesc w, const uint8_t *__restrict__ xm, int64_t x_row, xdesc d, int64_t ne11, int64_t total) {
    const int64_t o = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (o >= total) return;
    const int64_t ne00 = w.ne[0], ne01 = w.ne[1], ne02 = w.ne[2];
    const int64_t i01 = o % ne01, i11 = o / ne01 % ne11, i02 = o / (ne01 * ne11) % ne02, i03 = o / (ne01 * ne11 * ne02);
    const uint8_t *wr = xat(w, 0, i01, i02, i03);
    const uint8_t *xr = xm + ((i03 * ne02 + i02) * ne11 + i11) * x_row;
    float v;
    if (WT == SPY_HIP_Q4_0) v = dot_q4_0(wr, xr, ne00);
    else if (WT == SPY_HIP_Q8_0) v = dot_q8_0(wr, xr, ne00);
    else if (WT == SPY_HIP_Q4_K) v = dot_q4_k(wr, xr, ne00);
    else if (WT == SPY_HIP_Q6_K) v = dot_q6_k(wr, xr, ne00);
    else v = dot_f16(wr, xr, ne00);
    *(float *)xat(d, i01, i11, i02, i03) = v;
}

// The same Q4_0 / Q8_0 dots with the eight accumulators of an output element spread over eight lanes: lane l keeps
// accumulator l (its four products per block), the blocks follow one another in each lane exactly as in the host loop,
// and hsum_float_8 becomes three exchanges (l ^ 4, l ^ 2, l ^ 1 -- the additions of the tree, whose operands commute).
// A workgroup computes 32 consecutive output elements; where they all belong to one activation row of at most
// DOTS8_LDS_BLOCKS blocks, the row is unpacked into LDS once (scale as fp32, quants as aligned words).
#define DOTS8_LDS_BLOCKS 1024
__device__ __forceinline__ uint32_t ld_u32_a2(const uint8_t *p) {      // four bytes from a 2-byte-aligned address
    return (uint32_t)*(const uint16_t *)p | ((uint32_t)*(const uint16_t *)(p + 2) << 16);
}
__device__ __forceinline__ int32_t mul_sum4_packed(uint32_t a, uint32_t b) {
    int8_t x[4], y[4];
#pragma unroll
    for (int k = 0; k < 4; k++) { x[k] = (int8_t)(a >> (8 * k)); y[k] = (int8_t)(b >> (8 * k)); }
    return mul_sum4(x, y);
}
template <int WT>
__global__ __launch_bounds__(256) void exact_dots8_kernel(xdesc w, const uint8_t *__restrict__ xm, int64_t x_row, xdesc d, int64_t ne11, int64_t total) {
    __shared__ float s_d[DOTS8_LDS_BLOCKS];
    __shared__ uint32_t s_q[DOTS8_LDS_BLOCKS * 8];
    const int64_t ne00 = w.ne[0], ne01 = w.ne[1], ne02 = w.ne[2];
    const int64_t nb = ne00 / 32;
    const int64_t o_first = (int64_t)blockIdx.x * 32, o_last = min(o_first + 31, total - 1);
    const bool staged = nb <= DOTS8_LDS_BLOCKS && o_first / ne01 == o_last / ne01;      // one (i11, i02, i03) for the workgroup
    if (staged) {
        const int64_t xr = o_first / ne01;                                              // = (i03 * ne02 + i02) * ne11 + i11
        const uint8_t *xb = xm + xr * x_row;
        for (int64_t i = threadIdx.x; i < nb; i += 256) {
            const uint8_t *b = xb + i * 34;
            s_d[i] = h2f_tab(*(const uint16_t *)b);
#pragma unroll
            for (int j = 0; j < 8; j++) s_q[i * 8 + j] = ld_u32_a2(b + 2 + 4 * j);
        }
        __syncthreads();
    }
    const int64_t o = o_first + (threadIdx.x >> 3);
    if (o >= total) return;                       // whole groups of eight lanes leave together, after the barrier
    const int l = threadIdx.x & 7;
    const int64_t i01 = o % ne01, i11 = o / ne01 % ne11, i02 = o / (ne01 * ne11) % ne02, i03 = o / (ne01 * ne11 * ne02);
    const uint8_t *wr = xat(w, 0, i01, i02, i03);
    const uint8_t *xr = xm + ((i03 * ne02 + i02) * ne11 + i11) * x_row;
    // Q4_0: lanes 0..3 take the high nibbles against elements 16..31, lanes 4..7 the low nibbles against 0..15;
    // Q8_0: lane l takes elements 4l..4l+3
    const int wo = WT == SPY_HIP_Q4_0 ? 2 + 4 * (l & 3) : 2 + 4 * l;
    const int xg = WT == SPY_HIP_Q4_0 ? (l < 4 ? 4 : 0) + (l & 3) : l;
    const int wsz = WT == SPY_HIP_Q4_0 ? 18 : 34;
    // The row is walked 16 blocks at a time with the next 16 blocks' loads in flight: an output element has only its
    // eight lanes, so the latency of the weight loads has to be covered by each lane's own requests.  Loads beyond the
    // row are clamped to its last block (and not used), which keeps them unconditional.
    constexpr int U = 16;
    float acc = 0.0f;
    uint32_t a_cur[U], a_nxt[U];
    uint16_t d_cur[U], d_nxt[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint8_t *wb = wr + min((int64_t)u, nb - 1) * wsz;
        d_cur[u] = *(const uint16_t *)wb;
        a_cur[u] = ld_u32_a2(wb + wo);
    }
    for (int64_t i0 = 0; i0 < nb; i0 += U) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint8_t *wb = wr + min(i0 + U + u, nb - 1) * wsz;
            d_nxt[u] = *(const uint16_t *)wb;
            a_nxt[u] = ld_u32_a2(wb + wo);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int64_t i = i0 + u;
            if (i < nb) {
                const float dw = h2f_tab(d_cur[u]);
                uint32_t a = a_cur[u];
                if (WT == SPY_HIP_Q4_0) {
                    a = (l < 4 ? (a >> 4) : a) & 0x0F0F0F0Fu;
                    a = (a | 0x80808080u) - 0x08080808u;          // per byte n - 8 without a borrow across bytes ...
                    a ^= 0x80808080u;                             // ... (n + 128 - 8) with the top bit flipped back = n - 8 mod 256
                }
                float dx;
                uint32_t b;
                if (staged) { dx = s_d[i]; b = s_q[i * 8 + xg]; }
                else { const uint8_t *xb = xr + i * 34; dx = h2f_tab(*(const uint16_t *)xb); b = ld_u32_a2(xb + 2 + 4 * xg); }
                acc = fmaf(dw * dx, (float)mul_sum4_packed(a, b), acc);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) { a_cur[u] = a_nxt[u]; d_cur[u] = d_nxt[u]; }
    }
    acc += __shfl_xor(acc, 4, SPY_WAVE);          // r_l = a_l + a_(l+4)
    acc += __shfl_xor(acc, 2, SPY_WAVE);          // s_0 = r_0 + r_2, s_1 = r_1 + r_3
    acc += __shfl_xor(acc, 1, SPY_WAVE);          // s_0 + s_1
    if (l == 0) *(float *)xat(d, i01, i11, i02, i03) = acc;
}

// The Q4_0 / Q8_0 dots for many activation rows at once (prompts): a workgroup computes a tile of 64 weight rows by 64 activation
// rows, a wave 16 x 64 of it, a lane 16 output elements with the eight accumulators of each in registers.  Every accumulator still
// receives its block terms in block order, fma(d_w * d_x, float(integer sum of its four products), acc), and the eight are added in
// hsum_float_8's tree at the end, so the results are those of exact_dots8_kernel bit for bit; what changes is that a weight block
// and an activation block are unpacked once per tile (into LDS, as words in element order: the low nibbles of a Q4_0 block first,
// then the high ones) instead of once per output, and that the integer sums come from the matrix cores.
// v_mfma_*_16x16x4_4b_* computes four 16 x 16 products over four elements each, lane l supplying row l % 16 of A and column l % 16 of
// B for product l / 16: with the A-matrix broadcast (cbsz:2 abid:q: all four products take the A operand of lane block q) one
// instruction multiplies a wave's 16 weight rows by its 64 activation rows over one element word -- exactly one accumulator's share
// of a block, nothing wasted -- and the four lane blocks can hold the words of four different element words: one LDS read per lane
// feeds four instructions.  Output register 4b + v of lane (blk, r): weight row 16 * wave + 4 * blk + v, activation row 16b + r.
// The scale products d_w * d_x of a block come the same way from v_mfma_f32_16x16x1_4b_f32 (one product per output, rounded once:
// the bits of the vector multiply).
// The hardware multiplies the signed values as they are, which equals the host's abs / sign / saturating pair sum
// (vec_util.h:101-110) as long as no ACTIVATION byte is -128; the launcher takes this kernel only for activations that this
// library quantized itself (|q| <= 127).
#define XGB_TILE 64
#define XGB_KB 4          // blocks per stage of the K-quant kernel
typedef int xgb_v4i __attribute__((ext_vector_type(4)));
typedef float xgb_v4f __attribute__((ext_vector_type(4)));
typedef int xgb_v16i __attribute__((ext_vector_type(16)));
typedef float xgb_v16f __attribute__((ext_vector_type(16)));
// v_mfma_i32_16x16x4_4b_i8 with the A operand of lane block abid for all four products (abid has to be an immediate)
__device__ __forceinline__ xgb_v16i xgb_mfma16(uint32_t w, uint32_t x, const xgb_v16i &c, int abid) {
    switch (abid) {
    case 0: return __builtin_amdgcn_mfma_i32_16x16x4i8((int)w, (int)x, c, 2, 0, 0);
    case 1: return __builtin_amdgcn_mfma_i32_16x16x4i8((int)w, (int)x, c, 2, 1, 0);
    case 2: return __builtin_amdgcn_mfma_i32_16x16x4i8((int)w, (int)x, c, 2, 2, 0);
    default: return __builtin_amdgcn_mfma_i32_16x16x4i8((int)w, (int)x, c, 2, 3, 0);
    }
}
// The integer sums are delivered as floats: the quants are converted to fp16 once, when a tile is staged (every int8 is an fp16
// exactly), and v_mfma_f32_16x16x4_4b_f16 adds the four products of an accumulator's share in fp32 -- integers below 2^16, so the
// sum is exact whatever order the hardware adds them in.  The vector units are left with ONE instruction per term, the fma onto
// the accumulator (with the int8 form of the instruction and a biased accumulator they need a subtraction as well: 0.88 ms per
// GEMM of a 2048-row chunk against 0.75).  A stage is two blocks (the fp16 operands take twice the LDS).
typedef _Float16 xgf_h2 __attribute__((ext_vector_type(2)));
typedef _Float16 xgf_h4 __attribute__((ext_vector_type(4)));
// bytes v0..v3 (already biased to 0..255 resp. 0..15) -> fp16 pairs (v0 - sub, v1 - sub), (v2 - sub, v3 - sub): 0x6400 | v is the fp16
// 1024 + v, and the subtraction of 1024 + bias is exact
__device__ __forceinline__ uint2 xgf_bytes_to_h4(uint32_t v, float sub) {
    const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u), hi = __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u);
    const xgf_h2 c = {(_Float16)sub, (_Float16)sub};
    const xgf_h2 l2 = __builtin_bit_cast(xgf_h2, lo) - c, h2 = __builtin_bit_cast(xgf_h2, hi) - c;
    return make_uint2(__builtin_bit_cast(uint32_t, l2), __builtin_bit_cast(uint32_t, h2));
}
__device__ __forceinline__ xgb_v16f xgf_mfma16(const uint2 &w, const uint2 &x, int abid) {
    const xgf_h4 a = __builtin_bit_cast(xgf_h4, w), b = __builtin_bit_cast(xgf_h4, x);
    const xgb_v16f c = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    switch (abid) {
    case 0: return __builtin_amdgcn_mfma_f32_16x16x4f16(a, b, c, 2, 0, 0);
    case 1: return __builtin_amdgcn_mfma_f32_16x16x4f16(a, b, c, 2, 1, 0);
    case 2: return __builtin_amdgcn_mfma_f32_16x16x4f16(a, b, c, 2, 2, 0);
    default: return __builtin_amdgcn_mfma_f32_16x16x4f16(a, b, c, 2, 3, 0);
    }
}
#define XGF_KB 2
template <int WT>
__global__ __launch_bounds__(256, 2) void exact_gemm8f_kernel(const uint8_t *__restrict__ w, int64_t w_row, int64_t ne01, int64_t nb,
                                                               const uint8_t *__restrict__ xm, int64_t x_row, int64_t ne11,
                                                               float *__restrict__ dst, int64_t d_row) {
    constexpr int WPL = XGB_TILE + 8;
    __shared__ __align__(16) uint2 s_wq[2][XGF_KB][8][WPL];        // [buffer][block][element word][weight row]: four fp16
    __shared__ __align__(16) uint2 s_xq[2][XGF_KB][8][XGB_TILE];
    __shared__ __align__(16) float s_wd[2][XGF_KB][XGB_TILE];
    __shared__ __align__(16) float s_xd[2][XGF_KB][XGB_TILE];
    const int tid = threadIdx.x;
    const int wv = tid >> 6, bj = tid & 63, blk = bj >> 4, r = bj & 15;
    const int64_t m0 = (int64_t)blockIdx.x * XGB_TILE, t0 = (int64_t)blockIdx.y * XGB_TILE;

    // loaders: a thread takes ONE block of one row per stage -- waves 0, 1: weight rows, blocks 0 / 1 of the stage; waves 2, 3: activation
    // rows.  Two neighbouring blocks are 36 (Q4_0) or 68 bytes (Q8_0), whole aligned words; the second block starts in the middle of a word.
    const bool ld_w = tid < 128;
    const int ld_row = tid & 63, ld_blk = (tid >> 6) & 1;
    constexpr int NWQ = WT == SPY_HIP_Q4_0 ? 9 : 17;               // words per pair of weight blocks
    const uint32_t *ld_src;
    if (ld_w) ld_src = (const uint32_t *)(w + min(m0 + ld_row, ne01 - 1) * w_row) + (WT == SPY_HIP_Q4_0 ? 4 : 8) * ld_blk;
    else ld_src = (const uint32_t *)(xm + min(t0 + ld_row, ne11 - 1) * x_row) + 8 * ld_blk;
    uint32_t g[9];
    auto fetch = [&](int64_t stage) {
        const uint32_t *p = ld_src + stage * (ld_w ? NWQ : 17);
        if (ld_w && WT == SPY_HIP_Q4_0) {
#pragma unroll
            for (int i = 0; i < 5; i++) g[i] = p[i];
        } else {
#pragma unroll
            for (int i = 0; i < 9; i++) g[i] = p[i];
        }
    };
    auto put = [&](int buf) {
        if (ld_w && WT == SPY_HIP_Q4_0) {
            // block 0 of the pair: scale in the low half of g[0], quant bytes from byte 2; block 1: scale in the high half of g[0] (= word 4
            // of the pair), quants g[1..4]
            s_wd[buf][ld_blk][ld_row] = h2f_tab((uint16_t)(ld_blk ? g[0] >> 16 : g[0] & 0xFFFFu));
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t q = ld_blk ? g[1 + k] : __builtin_amdgcn_alignbit(g[k + 1], g[k], 16);
                s_wq[buf][ld_blk][k][ld_row] = xgf_bytes_to_h4(q & 0x0F0F0F0Fu, 1032.0f);              // low nibbles: elements 4k .. 4k + 3, n - 8
                s_wq[buf][ld_blk][4 + k][ld_row] = xgf_bytes_to_h4((q >> 4) & 0x0F0F0F0Fu, 1032.0f);   // high nibbles: elements 16 + 4k ..
            }
        } else {
            // Q8_0: block 0 = scale in the low half of g[0], quants from byte 2; block 1 = scale in the high half of g[0] (word 8 of the pair), quants g[1..8]
            const float d = h2f_tab((uint16_t)(ld_blk ? g[0] >> 16 : g[0] & 0xFFFFu));
            if (ld_w) s_wd[buf][ld_blk][ld_row] = d; else s_xd[buf][ld_blk][ld_row] = d;
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const uint32_t q = ld_blk ? g[1 + k] : __builtin_amdgcn_alignbit(g[k + 1], g[k], 16);
                const uint2 h = xgf_bytes_to_h4(q ^ 0x80808080u, 1152.0f);                               // signed bytes: b + 128, then - 128
                if (ld_w) s_wq[buf][ld_blk][k][ld_row] = h; else s_xq[buf][ld_blk][k][ld_row] = h;
            }
        }
    };

    float acc[4][4][8];
#pragma unroll
    for (int b = 0; b < 4; b++)
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int a = 0; a < 8; a++) acc[b][c][a] = 0.0f;
    const xgb_v16f zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};

    const int64_t nstage = nb / XGF_KB;
    fetch(0);
    put(0);
    __syncthreads();
    for (int64_t s = 0; s < nstage; s++) {
        const int buf = (int)(s & 1);
        if (s + 1 < nstage) fetch(s + 1);
        // output register 4b + v of lane (blk, r): weight row 16 * wave + 4 * blk + v, activation row 16b + r
#pragma unroll 1
        for (int kb = 0; kb < XGF_KB; kb++) {
            const float wdreg = s_wd[buf][kb][16 * wv + r], xdl = s_xd[buf][kb][bj];
            const uint2 w0 = s_wq[buf][kb][blk][16 * wv + r], w1 = s_wq[buf][kb][4 + blk][16 * wv + r];      // lane block q holds words q and 4 + q
            uint2 xql[8];
#pragma unroll
            for (int e = 0; e < 8; e++) xql[e] = s_xq[buf][kb][e][bj];
            const xgb_v16f D = __builtin_amdgcn_mfma_f32_16x16x1f32(wdreg, xdl, zero16, 2, 0, 0);
            // the matrix instruction of word e + 1 is issued before the vector work on the results of word e
            xgb_v16f p[2];
            p[0] = xgf_mfma16(w0, xql[0], 0);
#pragma unroll
            for (int e = 0; e < 8; e++) {
                if (e + 1 < 8) p[(e + 1) & 1] = xgf_mfma16(e + 1 < 4 ? w0 : w1, xql[e + 1], (e + 1) & 3);
                __builtin_amdgcn_sched_barrier(0);      // keeps the matrix instruction ahead of the fmas below (else the compiler issues it after them and waits for it)
                const int a = WT == SPY_HIP_Q4_0 ? ((e + 4) & 7) : e;
#pragma unroll
                for (int n = 0; n < 16; n++) acc[n >> 2][n & 3][a] = fmaf(D[n], p[e & 1][n], acc[n >> 2][n & 3][a]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (s + 1 < nstage) put(buf ^ 1);
        __syncthreads();
    }
    const int64_t row = m0 + 16 * wv + 4 * blk;
#pragma unroll
    for (int b = 0; b < 4; b++) {
        const int64_t tok = t0 + 16 * b + r;
        if (tok < ne11 && row < ne01)
            *(float4 *)(dst + tok * d_row + row) = make_float4(hsum8(acc[b][0]), hsum8(acc[b][1]), hsum8(acc[b][2]), hsum8(acc[b][3]));
    }
}

// The same tile from operands that were staged as fp16 ONCE per MatMul instead of once per tile (a weight tile is used by every
// tile of activation rows and the other way round: 32 and 64 to 172 times for a 2048-row chunk of a 7B prompt).  The packing kernel
// writes the words in the order the tile kernel's LDS holds them -- [tile of 64 rows][block][element word][row], four fp16 per
// entry, and the block scales as floats, [tile][block][row] -- so staging is a plain copy of 16-byte pieces, and the vector units
// of the tile kernel issue little but the fma per term.  Rows past the end of the matrix are packed as zeros (never stored).
// Weight words are rotated by 16 rows in the odd element words, which spreads the four lane blocks of a wave's read (four
// different element words, the same 16 rows) over all LDS banks.
#define XGP_KB 2
#define XGP_WPOS(row, e) (((row) + 16 * ((e) & 1)) & 63)
template <int WT>        // type of the source blocks: Q4_0 (weights) or Q8_0 (weights, activations)
__global__ __launch_bounds__(256) void xgp_pack_kernel(const uint8_t *__restrict__ src, int64_t row_bytes, int64_t nrows, int64_t nb,
                                                       uint2 *__restrict__ q, float *__restrict__ d, int rotate) {
    const int row_in = threadIdx.x & 63;
    const int64_t tile = blockIdx.y, ib = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6), row = tile * XGB_TILE + row_in;
    if (ib >= nb) return;
    uint2 *qo = q + (tile * nb + ib) * (8 * XGB_TILE);
    float *dout = d + (tile * nb + ib) * XGB_TILE + row_in;
    if (row >= nrows) {
#pragma unroll
        for (int e = 0; e < 8; e++) qo[e * XGB_TILE + (rotate ? XGP_WPOS(row_in, e) : row_in)] = make_uint2(0u, 0u);
        *dout = 0.0f;
        return;
    }
    // blocks are 2-byte aligned: scale, then 16 (Q4_0) or 32 (Q8_0) quant bytes
    const uint16_t *p = (const uint16_t *)(src + row * row_bytes + ib * (WT == SPY_HIP_Q4_0 ? 18 : 34));
    *dout = h2f_tab(p[0]);
    if (WT == SPY_HIP_Q4_0) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t v = (uint32_t)p[1 + 2 * k] | ((uint32_t)p[2 + 2 * k] << 16);
            qo[k * XGB_TILE + (rotate ? XGP_WPOS(row_in, k) : row_in)] = xgf_bytes_to_h4(v & 0x0F0F0F0Fu, 1032.0f);                  // elements 4k .. 4k + 3
            qo[(4 + k) * XGB_TILE + (rotate ? XGP_WPOS(row_in, 4 + k) : row_in)] = xgf_bytes_to_h4((v >> 4) & 0x0F0F0F0Fu, 1032.0f); // elements 16 + 4k ..
        }
    } else {
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const uint32_t v = (uint32_t)p[1 + 2 * k] | ((uint32_t)p[2 + 2 * k] << 16);
            qo[k * XGB_TILE + (rotate ? XGP_WPOS(row_in, k) : row_in)] = xgf_bytes_to_h4(v ^ 0x80808080u, 1152.0f);
        }
    }
}
template <int WT>        // weight type: decides which accumulator a word belongs to
__global__ __launch_bounds__(256, 2) void exact_gemm8p_kernel(const uint2 *__restrict__ wq, const float *__restrict__ wd, const uint2 *__restrict__ xq,
                                                               const float *__restrict__ xd, int64_t nb, int64_t ne01, int64_t ne11,
                                                               float *__restrict__ dst, int64_t d_row) {
    __shared__ __align__(16) uint2 s_wq[2][XGP_KB][8][XGB_TILE];
    __shared__ __align__(16) uint2 s_xq[2][XGP_KB][8][XGB_TILE];
    __shared__ __align__(16) float s_wd[2][XGP_KB * XGB_TILE];
    __shared__ __align__(16) float s_xd[2][XGP_KB * XGB_TILE];
    static_assert(XGP_KB == 2, "the copy below moves two 16-byte pieces per operand and one scale per thread and stage");
    const int tid = threadIdx.x;
    const int wv = tid >> 6, bj = tid & 63, blk = bj >> 4, r = bj & 15;
    const int64_t m0 = (int64_t)blockIdx.x * XGB_TILE, t0 = (int64_t)blockIdx.y * XGB_TILE;
    // a stage of an operand: XGP_KB blocks x 8 words x 64 rows x 8 bytes = 512 pieces of 16 bytes, two per thread
    const uint4 *gw = (const uint4 *)(wq + (int64_t)blockIdx.x * nb * (8 * XGB_TILE)) + tid;
    const uint4 *gx = (const uint4 *)(xq + (int64_t)blockIdx.y * nb * (8 * XGB_TILE)) + tid;
    const float *gd = tid < 128 ? wd + (int64_t)blockIdx.x * nb * XGB_TILE + tid : xd + (int64_t)blockIdx.y * nb * XGB_TILE + (tid - 128);
    uint4 g0, g1, g2, g3;
    float gs;
#define XGP_FETCH(stage) { g0 = gw[(stage) * 512]; g1 = gw[(stage) * 512 + 256]; g2 = gx[(stage) * 512]; g3 = gx[(stage) * 512 + 256]; \
                           gs = gd[(stage) * (XGP_KB * XGB_TILE)]; }
#define XGP_PUT(buf) { uint4 *lw = (uint4 *)&s_wq[buf][0][0][0] + tid, *lx = (uint4 *)&s_xq[buf][0][0][0] + tid; \
                       lw[0] = g0; lw[256] = g1; lx[0] = g2; lx[256] = g3; \
                       if (tid < 128) s_wd[buf][tid] = gs; else s_xd[buf][tid - 128] = gs; }

    float acc[4][4][8];
#pragma unroll
    for (int b = 0; b < 4; b++)
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int a = 0; a < 8; a++) acc[b][c][a] = 0.0f;
    const xgb_v16f zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    const int wpos = XGP_WPOS(16 * wv + r, blk);      // words blk and 4 + blk have the same parity

    const int64_t nstage = nb / XGP_KB;
    XGP_FETCH(0)
    XGP_PUT(0)
    __syncthreads();
    for (int64_t s = 0; s < nstage; s++) {
        const int buf = (int)(s & 1);
        if (s + 1 < nstage) XGP_FETCH(s + 1)
#pragma unroll 1
        for (int kb = 0; kb < XGP_KB; kb++) {
            const float wdreg = s_wd[buf][kb * XGB_TILE + 16 * wv + r], xdl = s_xd[buf][kb * XGB_TILE + bj];
            const uint2 w0 = s_wq[buf][kb][blk][wpos], w1 = s_wq[buf][kb][4 + blk][wpos];
            uint2 xql[8];
#pragma unroll
            for (int e = 0; e < 8; e++) xql[e] = s_xq[buf][kb][e][bj];
            const xgb_v16f D = __builtin_amdgcn_mfma_f32_16x16x1f32(wdreg, xdl, zero16, 2, 0, 0);
            xgb_v16f p[2];
            p[0] = xgf_mfma16(w0, xql[0], 0);
#pragma unroll
            for (int e = 0; e < 8; e++) {
                if (e + 1 < 8) p[(e + 1) & 1] = xgf_mfma16(e + 1 < 4 ? w0 : w1, xql[e + 1], (e + 1) & 3);
                __builtin_amdgcn_sched_barrier(0);      // the matrix instruction of word e + 1 stays ahead of the fmas on word e
                const int a = WT == SPY_HIP_Q4_0 ? ((e + 4) & 7) : e;
#pragma unroll
                for (int n = 0; n < 16; n++) acc[n >> 2][n & 3][a] = fmaf(D[n], p[e & 1][n], acc[n >> 2][n & 3][a]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (s + 1 < nstage) XGP_PUT(buf ^ 1)
        __syncthreads();
    }
    const int64_t row = m0 + 16 * wv + 4 * blk;
#pragma unroll
    for (int b = 0; b < 4; b++) {
        const int64_t tok = t0 + 16 * b + r;
        if (tok < ne11 && row < ne01)
            *(float4 *)(dst + tok * d_row + row) = make_float4(hsum8(acc[b][0]), hsum8(acc[b][1]), hsum8(acc[b][2]), hsum8(acc[b][3]));
    }
}

// The K-quant dots for many activation rows at once, tiled like exact_gemm8f_kernel (64 x 64 outputs per workgroup, a
// wave 16 weight rows x 64 activation rows per v_mfma_i32_16x16x4_4b_i8, weight words through its A-matrix broadcast).  These dots keep ONE accumulator per output and add a term per sub-block of 32 elements, in order:
//   Q4_K:  acc = fma(d_x, d * float(sc * isum) - dmin * float(m * bsum), acc)       isum = sum q * x, bsum = sum x over the sub-block
//   Q6_K:  acc = fma(d_x * d, float(sc0 * isum0 + sc1 * isum1), acc)                 isum0 / isum1 over the two halves of 16 elements
// The integer sums are chains of matrix instructions over the element words of a sub-block (exact: integers); a stage is half a
// super-block (four sub-blocks).  The bits are those of exact_dotsk_kernel and of the oracle.
template <int WT>
__global__ __launch_bounds__(256, 3) void exact_gemmk_kernel(const uint8_t *__restrict__ w, int64_t w_row, int64_t ne01, int64_t nsb,
                                                              const uint8_t *__restrict__ xm, int64_t x_row, int64_t ne11,
                                                              float *__restrict__ dst, int64_t d_row) {
    constexpr bool K4 = WT == SPY_HIP_Q4_K;
    constexpr int WPL = XGB_TILE + 16;                             // four weight planes are read at once: the padding puts them on different banks
    __shared__ __align__(16) uint32_t s_wq[2][XGB_KB][8][WPL];     // element words of the weights
    __shared__ __align__(16) uint32_t s_xq[2][XGB_KB][8][XGB_TILE];
    __shared__ __align__(16) int32_t s_ws0[2][XGB_KB][XGB_TILE];   // Q4_K: sc          Q6_K: scale of elements 0..15
    __shared__ __align__(16) int32_t s_ws1[2][XGB_KB][XGB_TILE];   // Q4_K: m           Q6_K: scale of elements 16..31
    __shared__ __align__(16) float s_wd[2][2][XGB_TILE];           // d, dmin of the super-block (Q6_K: d)
    __shared__ __align__(16) float s_xd[2][XGB_KB][XGB_TILE];
    __shared__ __align__(16) int32_t s_xb[2][XGB_KB][XGB_TILE];    // Q4_K: sum of the activation quants of the block
    const int tid = threadIdx.x;
    const int wv = tid >> 6, bj = tid & 63, blk = bj >> 4, r = bj & 15;
    const int64_t m0 = (int64_t)blockIdx.x * XGB_TILE, t0 = (int64_t)blockIdx.y * XGB_TILE;

    // loaders: waves 0 and 1 bring weights (a thread: one row, two of the stage's four sub-blocks), waves 2 and 3 activation blocks
    const bool ld_w = tid < 128;
    const int ld_row = tid & 63, ld_pair = (tid >> 6) & 1;
    const int ld_slot = ld_row;
    const uint8_t *ld_wrow = w + min(m0 + ld_row, ne01 - 1) * w_row;
    const uint32_t *ld_xsrc = (const uint32_t *)(xm + min(t0 + ld_row, ne11 - 1) * x_row) + ld_pair * 17;
    uint32_t g[17];                                                // activations: two Q8_0 blocks; weights: quant words and scale bytes
    auto fetch = [&](int64_t stage) {
        if (!ld_w) {
            const uint32_t *p = ld_xsrc + stage * 34;
#pragma unroll
            for (int i = 0; i < 17; i++) g[i] = p[i];
        } else if (K4) {
            // super-block of 144 bytes: d, dmin, scales[12], qs[128]; sub-blocks 2k and 2k + 1 are the low and high nibbles of qs[32k .. 32k + 31]
            const uint8_t *sb = ld_wrow + (stage >> 1) * 144;
            const uint4 *q = (const uint4 *)(sb + 16 + 64 * (stage & 1) + 32 * ld_pair);
            const uint4 a = q[0], b = q[1];
            g[0] = a.x; g[1] = a.y; g[2] = a.z; g[3] = a.w; g[4] = b.x; g[5] = b.y; g[6] = b.z; g[7] = b.w;
            const uint32_t *h = (const uint32_t *)sb;
            g[8] = h[0]; g[9] = h[1]; g[10] = h[2]; g[11] = h[3];
        } else {
            // super-block of 210 bytes (2-byte aligned): ql[128], qh[64], scales[16], d.  Half h of it = sub-blocks 4h .. 4h + 3; this thread
            // takes sub-blocks 4h + p and 4h + p + 2: the low and high nibbles of ql[64h + 32p ..], with bits 2(p), 2(p + 2) of qh[32h ..]
            const uint8_t *sb = ld_wrow + (stage >> 1) * 210;
            const int h = (int)(stage & 1);
#pragma unroll
            for (int i = 0; i < 8; i++) g[i] = ld_u32_a2(sb + 64 * h + 32 * ld_pair + 4 * i);
#pragma unroll
            for (int i = 0; i < 8; i++) g[8 + i] = ld_u32_a2(sb + 128 + 32 * h + 4 * i);
            g[16] = (uint32_t)*(const uint16_t *)(sb + 192 + 2 * (4 * h + ld_pair)) | ((uint32_t)*(const uint16_t *)(sb + 192 + 2 * (4 * h + ld_pair + 2)) << 16);
        }
    };
    auto put = [&](int buf, int64_t stage) {
        if (!ld_w) {
            const int k0 = 2 * ld_pair;
            s_xd[buf][k0][ld_row] = h2f_tab((uint16_t)(g[0] & 0xFFFFu));
            s_xd[buf][k0 + 1][ld_row] = h2f_tab((uint16_t)(g[8] >> 16));
            int32_t b0 = 0, b1 = 0;
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const uint32_t q0 = __builtin_amdgcn_alignbit(g[k + 1], g[k], 16), q1 = g[9 + k];
                s_xq[buf][k0][k][ld_row] = q0; s_xq[buf][k0 + 1][k][ld_row] = q1;
                if (K4) { b0 = __builtin_amdgcn_sdot4((int)q0, 0x01010101, b0, false); b1 = __builtin_amdgcn_sdot4((int)q1, 0x01010101, b1, false); }
            }
            if (K4) { s_xb[buf][k0][ld_row] = b0; s_xb[buf][k0 + 1][ld_row] = b1; }
        } else if (K4) {
            const int k0 = 2 * ld_pair;                            // sub-blocks k0 (low nibbles) and k0 + 1 (high nibbles) of the stage
#pragma unroll
            for (int k = 0; k < 8; k++) {
                s_wq[buf][k0][k][ld_slot] = g[k] & 0x0F0F0F0Fu;
                s_wq[buf][k0 + 1][k][ld_slot] = (g[k] >> 4) & 0x0F0F0F0Fu;
            }
            // get_scale_min_k4 for sub-blocks j and j + 1 of the super-block, j = 4 * (stage & 1) + k0
            const uint8_t sbytes[12] = {(uint8_t)(g[9]), (uint8_t)(g[9] >> 8), (uint8_t)(g[9] >> 16), (uint8_t)(g[9] >> 24), (uint8_t)(g[10]), (uint8_t)(g[10] >> 8),
                                        (uint8_t)(g[10] >> 16), (uint8_t)(g[10] >> 24), (uint8_t)(g[11]), (uint8_t)(g[11] >> 8), (uint8_t)(g[11] >> 16), (uint8_t)(g[11] >> 24)};
#pragma unroll
            for (int u = 0; u < 2; u++) {
                int32_t sc, m;
                if ((stage & 1) == 0) { const int j = k0 + u; sc = sbytes[j] & 63; m = sbytes[j + 4] & 63; }
                else { const int j = 4 + k0 + u; sc = (sbytes[j + 4] & 0x0F) | ((sbytes[j - 4] >> 6) << 4); m = (sbytes[j + 4] >> 4) | ((sbytes[j] >> 6) << 4); }
                s_ws0[buf][k0 + u][ld_slot] = sc;
                s_ws1[buf][k0 + u][ld_slot] = m;
            }
            if (ld_pair == 0) {
                s_wd[buf][0][ld_slot] = h2f_tab((uint16_t)(g[8] & 0xFFFFu));
                s_wd[buf][1][ld_slot] = h2f_tab((uint16_t)(g[8] >> 16));
            }
        } else {
            const uint8_t *sb = ld_wrow + (stage >> 1) * 210;
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int gq = ld_pair + 2 * u;                    // sub-block of the stage: 0 / 2 for pair 0, 1 / 3 for pair 1
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    const uint32_t lo = (u ? (g[k] >> 4) : g[k]) & 0x0F0F0F0Fu, hi = (g[8 + k] >> (2 * gq)) & 0x03030303u;
                    const uint32_t q = lo | (hi << 4);
                    s_wq[buf][gq][k][ld_slot] = ((q | 0x80808080u) - 0x20202020u) ^ 0x80808080u;      // per byte q - 32
                }
                const uint32_t sc2 = u ? (g[16] >> 16) : (g[16] & 0xFFFFu);
                s_ws0[buf][gq][ld_slot] = (int32_t)(int8_t)(sc2 & 0xFFu);
                s_ws1[buf][gq][ld_slot] = (int32_t)(int8_t)(sc2 >> 8);
            }
            if (ld_pair == 0) s_wd[buf][0][ld_slot] = h2f_tab(*(const uint16_t *)(sb + 208));
        }
    };

    float acc[4][4];                                               // [b][v]: activation row 16b + r, weight row 16 * wave + 4 * blk + v
#pragma unroll
    for (int b = 0; b < 4; b++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[b][c] = 0.0f;
    xgb_v16i zero16i;
#pragma unroll
    for (int n = 0; n < 16; n++) zero16i[n] = 0;

    const int64_t nstage = 2 * nsb;
    fetch(0);
    put(0, 0);
    __syncthreads();
    for (int64_t s = 0; s < nstage; s++) {
        const int buf = (int)(s & 1);
        if (s + 1 < nstage) fetch(s + 1);
        // this lane's four weight rows 16 * wave + 4 * blk + v: d, dmin of the super-block
        const xgb_v4f dw = *(const xgb_v4f *)&s_wd[buf][0][16 * wv + 4 * blk];
        xgb_v4f dmn = dw;
        if (K4) dmn = *(const xgb_v4f *)&s_wd[buf][1][16 * wv + 4 * blk];
#pragma unroll 1
        for (int half = 0; half < XGB_KB / 2; half++) {
            uint32_t wreg[4];                                      // lane block q, read i: word (4i + q) & 7 of sub-block 2 * half + (4i + q) / 8, row 16 * wave + r
#pragma unroll
            for (int i = 0; i < 4; i++) wreg[i] = s_wq[buf][2 * half + (i >> 1)][4 * (i & 1) + blk][16 * wv + r];
#pragma unroll
            for (int kb2 = 0; kb2 < 2; kb2++) {
                const int kb = 2 * half + kb2;
                uint32_t xq[8];
#pragma unroll
                for (int e = 0; e < 8; e++) xq[e] = s_xq[buf][kb][e][bj];
                const xgb_v4i s0 = *(const xgb_v4i *)&s_ws0[buf][kb][16 * wv + 4 * blk], s1 = *(const xgb_v4i *)&s_ws1[buf][kb][16 * wv + 4 * blk];
                // integer sums of the sub-block, register 4b + v: isum (Q4_K) or the two halves lo, hi (Q6_K)
                xgb_v16i lo = zero16i, hi = zero16i;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    if (K4 || e < 4) lo = xgb_mfma16(wreg[2 * kb2 + (e >> 2)], xq[e], lo, e & 3);
                    else hi = xgb_mfma16(wreg[2 * kb2 + (e >> 2)], xq[e], hi, e & 3);
                }
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const float xd = s_xd[buf][kb][16 * b + r];
                    if (K4) {
                        const int32_t xb = s_xb[buf][kb][16 * b + r];
#pragma unroll
                        for (int v = 0; v < 4; v++) {
                            const float pos = dw[v] * (float)__mul24(s0[v], lo[4 * b + v]);
                            const float neg = dmn[v] * (float)__mul24(s1[v], xb);
                            acc[b][v] = fmaf(xd, pos - neg, acc[b][v]);
                        }
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; v++) {
                            const int32_t sv = __mul24(s0[v], lo[4 * b + v]) + __mul24(s1[v], hi[4 * b + v]);
                            const float dd = xd * dw[v];
                            acc[b][v] = fmaf(dd, (float)sv, acc[b][v]);
                        }
                    }
                }
            }
        }
        if (s + 1 < nstage) put(buf ^ 1, s + 1);
        __syncthreads();
    }
    const int64_t row = m0 + 16 * wv + 4 * blk;
#pragma unroll
    for (int b = 0; b < 4; b++) {
        const int64_t tok = t0 + 16 * b + r;
        if (tok < ne11 && row < ne01) *(float4 *)(dst + tok * d_row + row) = make_float4(acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
    }
}

// K-quant rows with the eight sub-blocks (Q4_K) or Q8_0 blocks (Q6_K) of a super-block in eight lanes: lane j forms
// the integer sums and the fp32 term of its part, then every lane walks the ONE accumulator of the project's order
// through the eight terms in turn (terms broadcast from their lanes), so all eight lanes hold the same sum.
template <int WT>
__global__ __launch_bounds__(256) void exact_dotsk_kernel(xdesc w, const uint8_t *__restrict__ xm, int64_t x_row, xdesc d, int64_t ne11, int64_t total) {
    const int64_t o = (int64_t)blockIdx.x * 32 + (threadIdx.x >> 3);
    if (o >= total) return;                       // whole groups of eight lanes leave together
    const int j = threadIdx.x & 7;
    const int64_t ne00 = w.ne[0], ne01 = w.ne[1], ne02 = w.ne[2];
    const int64_t i01 = o % ne01, i11 = o / ne01 % ne11, i02 = o / (ne01 * ne11) % ne02, i03 = o / (ne01 * ne11 * ne02);
    const uint8_t *wr = xat(w, 0, i01, i02, i03);
    const blk_q8_0 *x = (const blk_q8_0 *)(xm + ((i03 * ne02 + i02) * ne11 + i11) * x_row);
    float acc = 0.0f;
    for (int64_t b = 0; b < ne00 / 256; b++) {
        const blk_q8_0 *xb = &x[b * 8 + j];
        float scale, term;                        // acc = fma(scale, term, acc), part after part
        if (WT == SPY_HIP_Q4_K) {
            const blk_q4_k *wb = (const blk_q4_k *)wr + b;
            const float dw = h2f_tab(wb->d), dmin = h2f_tab(wb->dmin);
            const uint8_t *s = wb->scales;
            int32_t sc, m;
            if (j < 4) { sc = s[j] & 63; m = s[j + 4] & 63; }
            else { sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4); m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4); }
            int32_t isum = 0, bsum = 0;
#pragma unroll 8
            for (int l = 0; l < 32; l++) {
                const uint8_t byte = wb->qs[32 * (j / 2) + l];
                const int32_t q = (j & 1) ? (byte >> 4) : (byte & 0x0F);
                const int32_t xq = xb->qs[l];
                isum += q * xq;
                bsum += xq;
            }
            const float pos = dw * (float)(sc * isum), neg = dmin * (float)(m * bsum);
            scale = h2f_tab(xb->d);
            term = pos - neg;
        } else {
            const blk_q6_k *wb = (const blk_q6_k *)wr + b;
            int32_t sv = 0;
            for (int h = 0; h < 2; h++) {
                int32_t isum = 0;
#pragma unroll 8
                for (int l = 0; l < 16; l++) isum += q6k_get(wb, 32 * j + 16 * h + l) * (int32_t)xb->qs[16 * h + l];
                sv += (int32_t)wb->scales[2 * j + h] * isum;
            }
            scale = h2f_tab(xb->d) * h2f_tab(wb->d);
            term = (float)sv;
        }
#pragma unroll
        for (int t = 0; t < 8; t++) {
            const float sc_t = __shfl(scale, (threadIdx.x & 56) | t, SPY_WAVE), te_t = __shfl(term, (threadIdx.x & 56) | t, SPY_WAVE);
            acc = fmaf(sc_t, te_t, acc);
        }
    }
    if (j == 0) *(float *)xat(d, i01, i11, i02, i03) = acc;
}

// Dot<FP16,FP16> with its 4 x 8 accumulators in 32 lanes: lane 8j + l keeps accumulator l of vector j.
__global__ __launch_bounds__(256) void exact_dots32_kernel(xdesc w, const uint8_t *__restrict__ xm, int64_t x_row, xdesc d, int64_t ne11, int64_t total) {
    const int64_t o = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);
    if (o >= total) return;                       // whole groups of 32 lanes leave together
    const int l = threadIdx.x & 31;
    const int64_t n = w.ne[0], ne01 = w.ne[1], ne02 = w.ne[2];
    const int64_t i01 = o % ne01, i11 = o / ne01 % ne11, i02 = o / (ne01 * ne11) % ne02, i03 = o / (ne01 * ne11 * ne02);
    const uint16_t *a = (const uint16_t *)xat(w, 0, i01, i02, i03);
    const uint16_t *b = (const uint16_t *)(xm + ((i03 * ne02 + i02) * ne11 + i11) * x_row);
    float acc = 0.0f;
    int64_t i = 0;
#pragma unroll 4
    for (; i + 32 < n; i += 32) acc = fmaf(h2f(a[i + l]), h2f(b[i + l]), acc);
    acc += __shfl_xor(acc, 16, SPY_WAVE);         // sum[0] += sum[2], sum[1] += sum[3]
    acc += __shfl_xor(acc, 8, SPY_WAVE);          // sum[0] += sum[1]
    acc += __shfl_xor(acc, 4, SPY_WAVE);          // t_l = sum[0][l] + sum[0][l + 4]
    acc += __shfl_xor(acc, 1, SPY_WAVE);          // t_0 + t_1, t_2 + t_3
    acc += __shfl_xor(acc, 2, SPY_WAVE);          // (t_0 + t_1) + (t_2 + t_3)
    if (l == 0) {
        float tail = 0.0f;
        for (; i < n; i++) { const float pr = h2f_tab(a[i]) * h2f_tab(b[i]); tail += pr; }
        *(float *)xat(d, i01, i11, i02, i03) = tail + acc;
    }
}

}   // namespace

// the two tables on the current device: exp [65536], then silu [65536]
int spy_exact_luts(const float **lut) { return device_luts(lut); }
// spy_hip_init: the tables exist before the first operator call, which then has nothing to allocate
int spy_exact_matvec_prepare_q4_0();      // engine_q*.hip: LDS limits of the single-row MatMul launches
int spy_exact_matvec_prepare_q8_0();
int spy_exact_matvec_prepare_q4_k();
int spy_exact_matvec_prepare_q6_k();
int spy_exact_device_setup() {
    const float *lut = nullptr;
    int rc = device_luts(&lut);
    if (!rc) rc = spy_exact_matvec_prepare_q4_0();
    if (!rc) rc = spy_exact_matvec_prepare_q8_0();
    if (!rc) rc = spy_exact_matvec_prepare_q4_k();
    if (!rc) rc = spy_exact_matvec_prepare_q6_k();
    return rc;
}

// A caller may switch the exact order on for the calls its own thread makes (a model whose passes run in the host's order
// issues its prompt operators that way) without touching what other threads see.
static thread_local int t_exact = -1;
int spy_exact_thread_scope(int on) {      // on: 1, 0, or -1 for "as the library-wide switch says"; returns the previous value
    const int prev = t_exact;
    t_exact = on;
    return prev;
}

int spy_exact_on() {
    if (t_exact >= 0) return t_exact;
    if (g_exact < 0) {
        const char *e = getenv("SPY_HIP_EXACT");
        g_exact = (e && *e && *e != '0') ? 1 : 0;
    }
    return g_exact;
}

extern "C" int spy_hip_set_exact_order(int on) {
    const int prev = spy_exact_on();
    g_exact = on ? 1 : 0;
    return prev;
}

// The callers (the spy_hip_op_* entry points) have validated types, shapes and strides.
int spy_exact_norm_rms(hipStream_t st, const spy_hip_tensor *x, const spy_hip_tensor *dst, float eps) {
    exact_norm_rms_kernel<<<dim3((unsigned)spy_t_nrow(dst)), dim3(256), 0, st>>>(mkx(x), mkx(dst), eps);
    return SPY_LAUNCH_RC();
}

int spy_exact_silu(hipStream_t st, const spy_hip_tensor *x, const spy_hip_tensor *dst) {
    const float *lut = nullptr;
    int rc = device_luts(&lut);
    if (rc) return rc;
    const int64_t total = spy_t_nelem(x);
    exact_silu_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st>>>(mkx(x), mkx(dst), lut, total);
    return SPY_LAUNCH_RC();
}

int spy_exact_softmax(hipStream_t st, const spy_hip_tensor *x, const spy_hip_tensor *mask, const spy_hip_tensor *dst, float scale) {
    if (dst->type != SPY_HIP_F32) return SPY_HIP_EUNSUPPORTED;      // the fp16 output is a shortcut of the fast path
    const float *lut = nullptr;
    int rc = device_luts(&lut);
    if (rc) return rc;
    exact_softmax_kernel<<<dim3((unsigned)spy_t_nrow(dst)), dim3(256), 0, st>>>(mkx(x), mkx(mask ? mask : x), mask != nullptr, mkx(dst), scale, lut);
    return SPY_LAUNCH_RC();
}

// cos / sin of one token: theta starts at the position and is multiplied by theta_scale once per pair
// (non-linear.cpp:304-309), cosf / sinf from the host's libm as in the reference.  extend_factor != 0 (rope_yarn,
// :247-260): the ramp is 1 - std::clamp(0.0F, 1.0F, y), which clamps the VALUE 0 into [1, y] and is therefore 0; the mix
// and the magnitude correction are evaluated as written.  zeta (xpos, :353-354), when asked for, follows the pairs.
static void rope_row(float *row, int32_t position, int64_t ne0, float theta_scale, const spy_hip_rope_param *p, bool zeta) {
    float theta = (float)position;
    for (int64_t i0 = 0; i0 < ne0; i0 += 2) {
        const float theta_interp = p->freq_scale * theta;
        float ang = theta_interp, mscale = p->attention_factor;
        if (p->extend_factor != 0.0f) {
            const float ramp_mix = (1.0f - 1.0f) * p->extend_factor;
            ang = theta_interp * (1 - ramp_mix) + theta * ramp_mix;
            mscale *= 1.0f + 0.1f * logf(1.0f / p->freq_scale);
        }
        row[i0] = cosf(ang) * mscale;
        row[i0 + 1] = sinf(ang) * mscale;
        theta *= theta_scale;
        if (zeta) {
            float z = powf(((float)i0 + 0.4f * (float)ne0) / (1.4f * (float)ne0), (float)position / p->xpos_base);
            if (p->xpos_down) z = 1.0f / z;
            row[ne0 + i0 / 2] = z;
        }
    }
}

int *spy_hip_err_flag_ptr();      // runtime.hip

// The table of a parameter set on the current device: cos / sin of every position of the context, from the host's libm.
// build: make it if it is missing (allocates and copies: not under stream capture).  *tab stays nullptr when it is missing and
// was not built.
static bool rope_table_applies(const spy_hip_rope_param *p, int64_t ne0) {
    return p->num_context > 0 && (int64_t)p->num_context * ne0 * 4 <= (64ll << 20) && p->xpos_base == 0.0f && p->extend_factor == 0.0f;
}
static int rope_table(const spy_hip_rope_param *p, int64_t ne0, bool build, const float **tab) {
    *tab = nullptr;
    const int dev = current_device();
    if (dev < 0) return SPY_HIP_EINVAL;
    const rope_key k = {p->num_context, ne0, p->freq_base, p->freq_scale, p->attention_factor, p->num_dim};
    std::lock_guard<std::mutex> lock(g_mu);
    for (const rope_entry &e : g_dev[dev].rope)
        if (e.k.npos == k.npos && e.k.ne0 == k.ne0 && e.k.freq_base == k.freq_base && e.k.freq_scale == k.freq_scale && e.k.factor == k.factor && e.k.num_dim == k.num_dim) {
            *tab = e.dev;
            return 0;
        }
    if (!build || g_dev[dev].rope.size() >= XO_MAX_ROPE_TABLES) return 0;
    const float theta_scale = powf(p->freq_base, -2.0f / (float)p->num_dim);
    std::vector<float> h((size_t)(k.npos * ne0));
    for (int64_t q = 0; q < k.npos; q++) rope_row(&h[(size_t)(q * ne0)], (int32_t)q, ne0, theta_scale, p, false);
    float *d = nullptr;
    hipError_t e = hipMalloc((void **)&d, h.size() * sizeof(float));
    if (e != hipSuccess) return (int)e;
    e = hipMemcpy(d, h.data(), h.size() * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) { (void)hipFree(d); return (int)e; }
    g_dev[dev].rope.push_back({k, d});
    *tab = d;
    return 0;
}

// Builds the exact-order Rope table of a parameter set ahead of time (ne0: the rotated row length, dst->ne[0] of the Rope
// calls to come), so that those calls neither allocate nor synchronise and can be captured into a HIP graph.
extern "C" int spy_hip_rope_prepare(const spy_hip_rope_param *p, int64_t ne0) {
    SPY_CHECK_ARG(p && ne0 > 0 && ne0 % 2 == 0 && p->num_dim > 0);
    if (!rope_table_applies(p, ne0)) return SPY_HIP_EUNSUPPORTED;
    const float *tab = nullptr;
    const int rc = rope_table(p, ne0, true, &tab);
    if (rc) return rc;
    return tab ? 0 : SPY_HIP_ENOSPACE;                     // XO_MAX_ROPE_TABLES parameter sets per device
}

int spy_exact_rope(hipStream_t st, const spy_hip_tensor *x, const spy_hip_tensor *pos, const spy_hip_tensor *dst, const spy_hip_rope_param *p) {
    const int64_t ne0 = dst->ne[0], ne2 = dst->ne[2];
    const float theta_scale = powf(p->freq_base, -2.0f / (float)p->num_dim);
    const dim3 grid((unsigned)dst->ne[1], (unsigned)dst->ne[2], (unsigned)dst->ne[3]);
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (st && hipStreamIsCapturing(st, &cap) != hipSuccess) cap = hipStreamCaptureStatusNone;
    const bool capturing = cap != hipStreamCaptureStatusNone;
    const bool zeta = p->xpos_base != 0.0f;
    // The rotations of every position of the context, built once per parameter set and kept on the device: the kernel
    // then looks its token's position up itself and the call needs no allocation, no copy and no wait.
    if (rope_table_applies(p, ne0) && spy_hip_err_flag_ptr()) {
        const float *tab = nullptr;
        const int rc = rope_table(p, ne0, !capturing, &tab);
        if (rc) return rc;
        if (tab) {
            exact_rope_kernel<<<grid, dim3(64), 0, st>>>(mkx(x), mkx(dst), tab, (const uint8_t *)pos->data, pos->nb[0], p->num_context, spy_hip_err_flag_ptr(), 0);
            return SPY_LAUNCH_RC();
        }
    }
    // No table (no context length, xpos or the YaRN extension, more parameter sets than are kept): wait for the stream, read the
    // positions back and upload the rows of this call's tokens.  Allocates and synchronises: not available under capture.
    if (capturing) return SPY_HIP_EUNSUPPORTED;
    hipError_t e = hipStreamSynchronize(st);
    if (e != hipSuccess) return (int)e;
    std::vector<int32_t> hp((size_t)ne2);
    if (pos->nb[0] == 4) e = hipMemcpy(hp.data(), pos->data, (size_t)ne2 * 4, hipMemcpyDeviceToHost);
    else e = hipMemcpy2D(hp.data(), 4, pos->data, (size_t)pos->nb[0], 4, (size_t)ne2, hipMemcpyDeviceToHost);
    if (e != hipSuccess) return (int)e;
    const int64_t tab_row = zeta ? ne0 + ne0 / 2 : ne0;
    std::vector<float> tab((size_t)(ne2 * tab_row));
    for (int64_t i2 = 0; i2 < ne2; i2++) rope_row(&tab[(size_t)(i2 * tab_row)], hp[(size_t)i2], ne0, theta_scale, p, zeta);
    const size_t need = tab.size() * sizeof(float);
    float *d = nullptr;                                     // this call's own rows: nothing shared with other threads
    e = hipMalloc((void **)&d, need);
    if (e != hipSuccess) return (int)e;
    e = hipMemcpy(d, tab.data(), need, hipMemcpyHostToDevice);
    if (e == hipSuccess) {
        exact_rope_kernel<<<grid, dim3(64), 0, st>>>(mkx(x), mkx(dst), d, nullptr, 0, 0, nullptr, zeta ? 1 : 0);
        e = hipGetLastError();
        if (e == hipSuccess) e = hipStreamSynchronize(st);
    }
    (void)hipFree(d);
    return e == hipSuccess ? 0 : (int)e;
}

// x_own_quants: the Q8_0 activations were quantized by this library (no byte is -128)
// bytes of workspace with which a MatMul of ne01 weight rows of ne00 elements by ne11 activation rows runs from packed fp16 operands
// (0: that kernel does not apply to the shape)
size_t spy_exact_pack_bytes(int64_t ne01, int64_t ne00, int64_t ne11) {
    const int64_t nb = ne00 / 32;
    if (ne11 < 16 || ne00 % 32 != 0 || nb <= 0 || nb % XGP_KB != 0) return 0;
    const int64_t tiles = (ne01 + XGB_TILE - 1) / XGB_TILE + (ne11 + XGB_TILE - 1) / XGB_TILE;
    return (size_t)(tiles * nb * (8 * XGB_TILE * 8 + XGB_TILE * 4));       // quants and scales: multiples of 256 bytes each
}
// MatMul of one f32 activation row with a quantized matrix: the two-phase kernel of the fused single-token pass (exact_decode.cuh),
// which quantizes the row in LDS and walks every row's accumulators in the host's order -- one launch instead of a quantization
// and one of the lane kernels below, at the bandwidth of the fused pass.  SPY_HIP_EUNSUPPORTED where it does not apply (lengths,
// alignment, or the test switches that select the lane / serial kernels): the caller then takes the general way.
int spy_exact_matvec_q4_0(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
int spy_exact_matvec_q8_0(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
int spy_exact_matvec_q4_k(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
int spy_exact_matvec_q6_k(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
int spy_exact_matvec(hipStream_t st, int t0, const void *w, const float *x, float *out, int64_t M, int64_t K) {
    if (getenv("SPY_HIP_EXACT_SERIAL")) return SPY_HIP_EUNSUPPORTED;
    const char *env_tiled = getenv("SPY_HIP_EXACT_TILED");
    if (env_tiled && *env_tiled == '0') return SPY_HIP_EUNSUPPORTED;
    if (M <= 0 || M >= (1ll << 30) || K <= 0 || K > 16384 || ((uintptr_t)w & 3) != 0 || ((uintptr_t)x & 15) != 0 || ((uintptr_t)out & 3) != 0) return SPY_HIP_EUNSUPPORTED;
    switch (t0) {
    case SPY_HIP_Q4_0: return spy_exact_matvec_q4_0(st, w, x, out, (int)M, (int)K);
    case SPY_HIP_Q8_0: return spy_exact_matvec_q8_0(st, w, x, out, (int)M, (int)K);
    case SPY_HIP_Q4_K: return ((uintptr_t)w & 15) == 0 ? spy_exact_matvec_q4_k(st, w, x, out, (int)M, (int)K) : SPY_HIP_EUNSUPPORTED;
    case SPY_HIP_Q6_K: return spy_exact_matvec_q6_k(st, w, x, out, (int)M, (int)K);
    default: return SPY_HIP_EUNSUPPORTED;
    }
}
// pack, pack_bytes: workspace for the packed operands (may be null / short: the tile kernel then unpacks per tile)
int spy_exact_dots(hipStream_t st, int t0, const spy_hip_tensor *w, const uint8_t *xm, int64_t x_row, int64_t ne11, const spy_hip_tensor *dst, int x_own_quants,
                   void *pack, size_t pack_bytes) {
    const int64_t total = w->ne[1] * ne11 * w->ne[2] * w->ne[3];
    if (total <= 0 || (total + 7) / 8 >= (1ll << 31)) return SPY_HIP_EINVAL;
    // many activation rows of a plain matrix: the tiled kernel (SPY_HIP_EXACT_TILED=0 keeps the row kernels, for the tests
    // that compare the two)
    if ((t0 == SPY_HIP_Q4_0 || t0 == SPY_HIP_Q8_0) && x_own_quants && ne11 >= 16 && w->ne[2] == 1 && w->ne[3] == 1) {
        const char *env_tiled = getenv("SPY_HIP_EXACT_TILED");
        const bool tiled = !(env_tiled && *env_tiled == '0');
        const int64_t nb = w->ne[0] / 32, ne01 = w->ne[1];
        const bool fits = nb > 0 && nb % XGF_KB == 0 && ne01 % 4 == 0 && w->nb[1] % 4 == 0 && x_row % 4 == 0 && ((uintptr_t)w->data & 3) == 0 &&
                          ((uintptr_t)xm & 3) == 0 && dst->nb[0] == 4 && dst->nb[1] % 16 == 0 && ((uintptr_t)dst->data & 15) == 0 &&
                          (ne11 + XGB_TILE - 1) / XGB_TILE <= 65535 && !getenv("SPY_HIP_EXACT_SERIAL");
        if (tiled && fits) {
            const dim3 grid((unsigned)((ne01 + XGB_TILE - 1) / XGB_TILE), (unsigned)((ne11 + XGB_TILE - 1) / XGB_TILE));
            const size_t pk = spy_exact_pack_bytes(ne01, w->ne[0], ne11);
            // SPY_HIP_EXACT_TILED=u: operands unpacked per tile even where the workspace would do
            if (pk && pack && pack_bytes >= pk && ((uintptr_t)pack & 15) == 0 && grid.x <= 65535 && !(env_tiled && *env_tiled == 'u')) {
                const int64_t mt = grid.x, tt = grid.y;
                uint2 *wq = (uint2 *)pack, *xq = wq + mt * nb * (8 * XGB_TILE);
                float *wd = (float *)(xq + tt * nb * (8 * XGB_TILE)), *xd = wd + mt * nb * XGB_TILE;
                const dim3 gw((unsigned)((nb + 3) / 4), (unsigned)mt), gx((unsigned)((nb + 3) / 4), (unsigned)tt);
                if (t0 == SPY_HIP_Q4_0) xgp_pack_kernel<SPY_HIP_Q4_0><<<gw, dim3(256), 0, st>>>((const uint8_t *)w->data, w->nb[1], ne01, nb, wq, wd, 1);
                else xgp_pack_kernel<SPY_HIP_Q8_0><<<gw, dim3(256), 0, st>>>((const uint8_t *)w->data, w->nb[1], ne01, nb, wq, wd, 1);
                xgp_pack_kernel<SPY_HIP_Q8_0><<<gx, dim3(256), 0, st>>>(xm, x_row, ne11, nb, xq, xd, 0);
                if (hipGetLastError() != hipSuccess) return SPY_HIP_EINVAL;
                if (t0 == SPY_HIP_Q4_0)
                    exact_gemm8p_kernel<SPY_HIP_Q4_0><<<grid, dim3(256), 0, st>>>(wq, wd, xq, xd, nb, ne01, ne11, (float *)dst->data, dst->nb[1] / 4);
                else
                    exact_gemm8p_kernel<SPY_HIP_Q8_0><<<grid, dim3(256), 0, st>>>(wq, wd, xq, xd, nb, ne01, ne11, (float *)dst->data, dst->nb[1] / 4);
                return SPY_LAUNCH_RC();
            }
            if (t0 == SPY_HIP_Q4_0)
                exact_gemm8f_kernel<SPY_HIP_Q4_0><<<grid, dim3(256), 0, st>>>((const uint8_t *)w->data, w->nb[1], ne01, nb, xm, x_row, ne11, (float *)dst->data, dst->nb[1] / 4);
            else
                exact_gemm8f_kernel<SPY_HIP_Q8_0><<<grid, dim3(256), 0, st>>>((const uint8_t *)w->data, w->nb[1], ne01, nb, xm, x_row, ne11, (float *)dst->data, dst->nb[1] / 4);
            return SPY_LAUNCH_RC();
        }
    }
    const dim3 grid((unsigned)((total + 63) / 64)), block(64);
    // SPY_HIP_EXACT_SERIAL=1: one thread per output element for every type (the plain restatement the lane forms are tested against)
    if ((t0 == SPY_HIP_Q4_K || t0 == SPY_HIP_Q6_K) && ne11 >= 16 && w->ne[2] == 1 && w->ne[3] == 1) {
        const char *env_tiled = getenv("SPY_HIP_EXACT_TILED");
        const int64_t nsb = w->ne[0] / 256, ne01 = w->ne[1];
        const bool fits = nsb > 0 && w->ne[0] % 256 == 0 && ne01 % 4 == 0 && x_row % 4 == 0 && ((uintptr_t)xm & 3) == 0 && dst->nb[0] == 4 && dst->nb[1] % 16 == 0 &&
                          ((uintptr_t)dst->data & 15) == 0 && (ne11 + XGB_TILE - 1) / XGB_TILE <= 65535 && !getenv("SPY_HIP_EXACT_SERIAL") &&
                          (t0 == SPY_HIP_Q4_K ? (((uintptr_t)w->data & 15) == 0 && w->nb[1] % 16 == 0) : (((uintptr_t)w->data & 1) == 0 && w->nb[1] % 2 == 0));
        if (fits && !(env_tiled && *env_tiled == '0')) {
            const dim3 grid((unsigned)((ne01 + XGB_TILE - 1) / XGB_TILE), (unsigned)((ne11 + XGB_TILE - 1) / XGB_TILE));
            if (t0 == SPY_HIP_Q4_K)
                exact_gemmk_kernel<SPY_HIP_Q4_K><<<grid, dim3(256), 0, st>>>((const uint8_t *)w->data, w->nb[1], ne01, nsb, xm, x_row, ne11, (float *)dst->data, dst->nb[1] / 4);
            else
                exact_gemmk_kernel<SPY_HIP_Q6_K><<<grid, dim3(256), 0, st>>>((const uint8_t *)w->data, w->nb[1], ne01, nsb, xm, x_row, ne11, (float *)dst->data, dst->nb[1] / 4);
            return SPY_LAUNCH_RC();
        }
    }
    const bool serial = getenv("SPY_HIP_EXACT_SERIAL") != nullptr;
    const dim3 grid8((unsigned)((total + 31) / 32)), grid32((unsigned)((total + 7) / 8));
    if (!serial && t0 == SPY_HIP_Q4_0) { exact_dots8_kernel<SPY_HIP_Q4_0><<<grid8, dim3(256), 0, st>>>(mkx(w), xm, x_row, mkx(dst), ne11, total); return SPY_LAUNCH_RC(); }
    if (!serial && t0 == SPY_HIP_Q8_0) { exact_dots8_kernel<SPY_HIP_Q8_0><<<grid8, dim3(256), 0, st>>>(mkx(w), xm, x_row, mkx(dst), ne11, total); return SPY_LAUNCH_RC(); }
    if (!serial && t0 == SPY_HIP_Q4_K) { exact_dotsk_kernel<SPY_HIP_Q4_K><<<grid8, dim3(256), 0, st>>>(mkx(w), xm, x_row, mkx(dst), ne11, total); return SPY_LAUNCH_RC(); }
    if (!serial && t0 == SPY_HIP_Q6_K) { exact_dotsk_kernel<SPY_HIP_Q6_K><<<grid8, dim3(256), 0, st>>>(mkx(w), xm, x_row, mkx(dst), ne11, total); return SPY_LAUNCH_RC(); }
    if (!serial && t0 == SPY_HIP_F16) { exact_dots32_kernel<<<grid32, dim3(256), 0, st>>>(mkx(w), xm, x_row, mkx(dst), ne11, total); return SPY_LAUNCH_RC(); }
    switch (t0) {
    case SPY_HIP_Q4_0: exact_dots_kernel<SPY_HIP_Q4_0><<<grid, block, 0, st>>>(mkx(w), xm, x_row, mkx(dst), ne11, total); break;
    case SPY_HIP_Q8_0: exact_dots_kernel<SPY_HIP_Q8_0><<<grid, block, 0, st>>>(mkx(w), xm, x_row, mkx(dst), ne11, total); break;
    case SPY_HIP_Q4_K: exact_dots_kernel<SPY_HIP_Q4_K><<<grid, block, 0, st>>>(mkx(w), xm, x_row, mkx(dst), ne11, total); break;
    case SPY_HIP_Q6_K: exact_dots_kernel<SPY_HIP_Q6_K><<<grid, block, 0, st>>>(mkx(w), xm, x_row, mkx(dst), ne11, total); break;
    case SPY_HIP_F16: exact_dots_kernel<SPY_HIP_F16><<<grid, block, 0, st>>>(mkx(w), xm, x_row, mkx(dst), ne11, total); break;
    default: return SPY_HIP_EUNSUPPORTED;
    }
    return SPY_LAUNCH_RC();
}
