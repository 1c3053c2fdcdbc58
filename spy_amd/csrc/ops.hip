// One entry point per operator of Spy's host backend (backend/host/operator/*.cpp in the Spy
// tree), taking the operator's tensors with their byte strides.  These are the general,
// stride-honouring forms that a per-operator submit() uses; the fused token loop has its own
// specialised kernels.
#include "common.cuh"
#include <stdlib.h>

#include <math.h>

int *spy_hip_err_flag_ptr();

// exact_order.hip: the same operators with every sum in the host backend's order (spy_hip_set_exact_order)
int spy_exact_on();
int spy_exact_norm_rms(hipStream_t st, const spy_hip_tensor *x, const spy_hip_tensor *dst, float eps);
int spy_exact_silu(hipStream_t st, const spy_hip_tensor *x, const spy_hip_tensor *dst);
int spy_exact_softmax(hipStream_t st, const spy_hip_tensor *x, const spy_hip_tensor *mask, const spy_hip_tensor *dst, float scale);
int spy_exact_rope(hipStream_t st, const spy_hip_tensor *x, const spy_hip_tensor *pos, const spy_hip_tensor *dst, const spy_hip_rope_param *p);
int spy_exact_matvec(hipStream_t st, int t0, const void *w, const float *x, float *out, int64_t M, int64_t K);
int spy_exact_dots(hipStream_t st, int t0, const spy_hip_tensor *w, const uint8_t *xm, int64_t x_row, int64_t ne11, const spy_hip_tensor *dst, int x_own_quants,
                   void *pack, size_t pack_bytes);
size_t spy_exact_pack_bytes(int64_t ne01, int64_t ne00, int64_t ne11);

struct tdesc {              // a tensor as the kernels see it
    uint8_t *p;
    int64_t ne[4], nb[4];
};
static tdesc mk(const spy_hip_tensor *t) {
    tdesc d;
    d.p = (uint8_t *)t->data;
    for (int i = 0; i < 4; i++) { d.ne[i] = t->ne[i]; d.nb[i] = t->nb[i]; }
    return d;
}
static __device__ __forceinline__ uint8_t *at(const tdesc &t, int64_t i0, int64_t i1, int64_t i2, int64_t i3) {
    return t.p + i0 * t.nb[0] + i1 * t.nb[1] + i2 * t.nb[2] + i3 * t.nb[3];
}
static bool same_ne(const spy_hip_tensor *a, const spy_hip_tensor *b) {
    for (int i = 0; i < 4; i++) if (a->ne[i] != b->ne[i]) return false;
    return true;
}
static bool same_shape(const spy_hip_tensor *a, const spy_hip_tensor *b) {      // Shape::operator== (tensor.h:106-109)
    if (a->type != b->type || a->dim != b->dim) return false;
    for (int i = 0; i < 4; i++) if (a->ne[i] != b->ne[i] || a->nb[i] != b->nb[i]) return false;
    return true;
}
static unsigned grid_for(int64_t n, int per) { return (unsigned)((n + per - 1) / per); }
#define CHECK_GRID(n, per) SPY_CHECK_ARG((n) > 0 && ((n) + (per) - 1) / (per) < (1ll << 31))

// ---------------------------------------------------------------------------------------------
// NormRMS (non-linear.cpp:194-223): y = x * (1 / sqrt(sum(x^2)/n + eps)); one workgroup per row.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void norm_rms_kernel(tdesc x, tdesc y, float eps) {
    __shared__ float s_part[4];
    const int64_t r = blockIdx.x;
    const int64_t ne0 = y.ne[0], ne1 = y.ne[1], ne2 = y.ne[2];
    const int64_t i3 = r / (ne1 * ne2), i2 = r % (ne1 * ne2) / ne1, i1 = r % ne1;
    const float *s = (const float *)at(x, 0, i1, i2, i3);
    float *d = (float *)at(y, 0, i1, i2, i3);
    float acc = 0.0f;
    for (int64_t i = threadIdx.x; i < ne0; i += 256) { const float v = s[i]; acc = fmaf(v, v, acc); }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = acc;
    __syncthreads();
    const float sum = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
    const float mean = sum / (float)ne0;
    const float scale = 1.0f / sqrtf(mean + eps);
    for (int64_t i = threadIdx.x; i < ne0; i += 256) d[i] = s[i] * scale;
}

extern "C" int spy_hip_op_norm_rms(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *dst, float eps) {
    SPY_CHECK_ARG(x && dst && x->data && dst->data);
    if (x->type != SPY_HIP_F32 || dst->type != SPY_HIP_F32) return SPY_HIP_EUNSUPPORTED;   // spy_assert (non-linear.cpp:199-200)
    SPY_CHECK_ARG(same_ne(x, dst) && x->nb[0] == 4 && dst->nb[0] == 4);
    const int64_t nrow = spy_t_nrow(dst);
    CHECK_GRID(nrow, 1);
    if (spy_exact_on()) return spy_exact_norm_rms((hipStream_t)stream, x, dst, eps);
    norm_rms_kernel<<<dim3((unsigned)nrow), dim3(256), 0, (hipStream_t)stream>>>(mk(x), mk(dst), eps);
    return SPY_LAUNCH_RC();
}

// ---------------------------------------------------------------------------------------------
// Add / Sub / Mul / Div (basic.cpp:15-50): dst = a (op) b, b broadcast over rows by i % ne1x and
// repeated along dim 0 when ne00 is a multiple of ne10.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void binary_kernel(int op, tdesc a, tdesc b, tdesc d, int64_t total) {
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= total) return;
    const int64_t i0 = g % a.ne[0], r = g / a.ne[0];
    const int64_t i1 = r % a.ne[1], i2 = r / a.ne[1] % a.ne[2], i3 = r / (a.ne[1] * a.ne[2]);
    const float va = *(const float *)at(a, i0, i1, i2, i3);
    const float vb = *(const float *)at(b, i0 % b.ne[0], i1 % b.ne[1], i2 % b.ne[2], i3 % b.ne[3]);
    float v;
    switch (op) {
    case 0: v = va + vb; break;
    case 1: v = va - vb; break;
    case 2: v = va * vb; break;
    default: v = va / vb; break;
    }
    *(float *)at(d, i0, i1, i2, i3) = v;
}

// The shapes the LLaMA graph uses -- contiguous a and dst, b either of the same shape or one contiguous row repeated over
// the rows (a norm weight) -- four elements per thread, no index arithmetic beyond one remainder.
__global__ __launch_bounds__(256) void binary_rows_kernel(int op, const float4 *a, const float4 *b, float4 *d,      /* dst may be a or b */
                                                          int64_t total4, int64_t b4) {
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= total4) return;
    const float4 va = a[g], vb = b[b4 == total4 ? g : g % b4];
    float4 v;
    switch (op) {
    case 0: v = make_float4(va.x + vb.x, va.y + vb.y, va.z + vb.z, va.w + vb.w); break;
    case 1: v = make_float4(va.x - vb.x, va.y - vb.y, va.z - vb.z, va.w - vb.w); break;
    case 2: v = make_float4(va.x * vb.x, va.y * vb.y, va.z * vb.z, va.w * vb.w); break;
    default: v = make_float4(va.x / vb.x, va.y / vb.y, va.z / vb.z, va.w / vb.w); break;
    }
    d[g] = v;
}

extern "C" int spy_hip_op_binary(void *stream, int op, const spy_hip_tensor *a, const spy_hip_tensor *b, const spy_hip_tensor *dst) {
    SPY_CHECK_ARG(a && b && dst && a->data && b->data && dst->data && op >= 0 && op <= 3);
    if (a->type != SPY_HIP_F32 || b->type != SPY_HIP_F32 || dst->type != SPY_HIP_F32) return SPY_HIP_EUNSUPPORTED;
    SPY_CHECK_ARG(same_ne(a, dst));
    for (int i = 0; i < 4; i++) SPY_CHECK_ARG(b->ne[i] > 0 && a->ne[i] % b->ne[i] == 0);   // Shape::can_repeat (tensor.h:186-190)
    const int64_t total = spy_t_nelem(a);
    CHECK_GRID(total, 256);
    const int64_t nb_ = spy_t_nelem(b);
    const bool b_row = b->ne[1] == 1 && b->ne[2] == 1 && b->ne[3] == 1 && b->nb[0] == 4;          // one row, repeated
    const bool b_same = nb_ == total && same_ne(a, b) && spy_t_contiguous(b);
    if (spy_t_contiguous(a) && spy_t_contiguous(dst) && (b_row || b_same) && a->ne[0] % 4 == 0 && b->ne[0] % 4 == 0 && (b_same || a->ne[0] == b->ne[0]) &&
        (((uintptr_t)a->data | (uintptr_t)b->data | (uintptr_t)dst->data) & 15) == 0) {
        binary_rows_kernel<<<dim3(grid_for(total / 4, 256)), dim3(256), 0, (hipStream_t)stream>>>(op, (const float4 *)a->data, (const float4 *)b->data,
                                                                                                (float4 *)dst->data, total / 4, (b_same ? total : b->ne[0]) / 4);
        return SPY_LAUNCH_RC();
    }
    binary_kernel<<<dim3(grid_for(total, 256)), dim3(256), 0, (hipStream_t)stream>>>(op, mk(a), mk(b), mk(dst), total);
    return SPY_LAUNCH_RC();
}

// ---------------------------------------------------------------------------------------------
// Silu (non-linear.cpp:11-14,57-77): the reference looks silu up in a table indexed by fp16(x),
// whose entries are v / (1 + expf(-v)) evaluated in fp32 on v = float(fp16(x)).
// ---------------------------------------------------------------------------------------------
static __device__ __forceinline__ float silu_ref(float x) {
    const float v = h2f(f2h(x));
    return v / (1.0f + expf(-v));
}

__global__ __launch_bounds__(256) void silu_kernel(tdesc x, tdesc d, int64_t total) {
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= total) return;
    const int64_t i0 = g % x.ne[0], r = g / x.ne[0];
    const int64_t i1 = r % x.ne[1], i2 = r / x.ne[1] % x.ne[2], i3 = r / (x.ne[1] * x.ne[2]);
    *(float *)at(d, i0, i1, i2, i3) = silu_ref(*(const float *)at(x, i0, i1, i2, i3));
}

__global__ __launch_bounds__(256) void silu_flat_kernel(const float4 *x, float4 *d, int64_t total4)      /* in place allowed */ {
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= total4) return;
    const float4 v = x[g];
    d[g] = make_float4(silu_ref(v.x), silu_ref(v.y), silu_ref(v.z), silu_ref(v.w));
}

extern "C" int spy_hip_op_silu(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *dst) {
    SPY_CHECK_ARG(x && dst && x->data && dst->data);
    if (x->type != SPY_HIP_F32 || dst->type != SPY_HIP_F32) return SPY_HIP_EUNSUPPORTED;
    SPY_CHECK_ARG(same_ne(x, dst));
    const int64_t total = spy_t_nelem(x);
    CHECK_GRID(total, 256);
    if (spy_exact_on()) return spy_exact_silu((hipStream_t)stream, x, dst);
    if (spy_t_contiguous(x) && spy_t_contiguous(dst) && total % 4 == 0 && (((uintptr_t)x->data | (uintptr_t)dst->data) & 15) == 0) {
        silu_flat_kernel<<<dim3(grid_for(total / 4, 256)), dim3(256), 0, (hipStream_t)stream>>>((const float4 *)x->data, (float4 *)dst->data, total / 4);
        return SPY_LAUNCH_RC();
    }
    silu_kernel<<<dim3(grid_for(total, 256)), dim3(256), 0, (hipStream_t)stream>>>(mk(x), mk(dst), total);
    return SPY_LAUNCH_RC();
}

// ---------------------------------------------------------------------------------------------
// Relu (non-linear.cpp:16-19,28-50): std::max(x, 0) element by element (a NaN stays a NaN: std::max returns its first
// argument unless it is smaller than the second).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void relu_kernel(tdesc x, tdesc d, int64_t total) {
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= total) return;
    const int64_t i0 = g % x.ne[0], r = g / x.ne[0];
    const int64_t i1 = r % x.ne[1], i2 = r / x.ne[1] % x.ne[2], i3 = r / (x.ne[1] * x.ne[2]);
    const float v = *(const float *)at(x, i0, i1, i2, i3);
    *(float *)at(d, i0, i1, i2, i3) = v < 0.0f ? 0.0f : v;
}

extern "C" int spy_hip_op_relu(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *dst) {
    SPY_CHECK_ARG(x && dst && x->data && dst->data);
    if (x->type != SPY_HIP_F32 || dst->type != SPY_HIP_F32) return SPY_HIP_EUNSUPPORTED;
    SPY_CHECK_ARG(same_ne(x, dst) && x->nb[0] == 4 && dst->nb[0] == 4);
    const int64_t total = spy_t_nelem(x);
    CHECK_GRID(total, 256);
    relu_kernel<<<dim3(grid_for(total, 256)), dim3(256), 0, (hipStream_t)stream>>>(mk(x), mk(dst), total);
    return SPY_LAUNCH_RC();
}

// ---------------------------------------------------------------------------------------------
// Quantize (backend/host/operator/quantize.cpp:18-41): row by row through auto_quantize_inner (vec_convert.h:463-468).
// F32 -> Q8_0 (Quantizator<FP32,Q8_0>, :178-261) and F32 -> F16 (:39-65) are the conversions of the reference that work;
// its F32 -> Q4_0 fills half of every block and inverts the scale (:83-117) and is refused here, like the K-quants
// (no quantizer in the reference at all).
// ---------------------------------------------------------------------------------------------
extern "C" int spy_hip_op_quantize(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *dst) {
    SPY_CHECK_ARG(x && dst && x->data && dst->data);
    if (x->type != SPY_HIP_F32 || (dst->type != SPY_HIP_Q8_0 && dst->type != SPY_HIP_F16)) return SPY_HIP_EUNSUPPORTED;
    SPY_CHECK_ARG(same_ne(x, dst) && x->nb[0] == 4 && dst->nb[0] == spy_type_size(dst->type) && x->ne[0] > 0 && spy_t_nrow(x) > 0);
    if (dst->type == SPY_HIP_Q8_0) SPY_CHECK_ARG(x->ne[0] % 32 == 0);
    // rows of a matrix in one launch where both sides step evenly from row to row; otherwise one launch per matrix
    const int64_t K = x->ne[0], drow = spy_row_size(dst->type, K);
    const bool dst_rows_packed = dst->nb[1] == drow && dst->nb[2] == drow * dst->ne[1] && dst->nb[3] == dst->nb[2] * dst->ne[2];
    SPY_CHECK_ARG(dst_rows_packed);                                     // the quantizing kernels write rows back to back
    for (int64_t i3 = 0; i3 < x->ne[3]; i3++)
        for (int64_t i2 = 0; i2 < x->ne[2]; i2++) {
            const float *src = (const float *)((const uint8_t *)x->data + i2 * x->nb[2] + i3 * x->nb[3]);
            uint8_t *out = (uint8_t *)dst->data + i2 * dst->nb[2] + i3 * dst->nb[3];
            const int rc = dst->type == SPY_HIP_Q8_0 ? spy_hip_quantize_q8_0(stream, src, x->nb[1], out, x->ne[1], K)
                                                     : spy_hip_quantize_f16(stream, src, x->nb[1], out, x->ne[1], K);
            if (rc) return rc;
        }
    return 0;
}

// ---------------------------------------------------------------------------------------------
// Softmax (non-linear.cpp:86-180): t = (s + mask) * scale; m = max t; e = mask == -inf ? 0 :
// expf(float(fp16(t - m))); p = e * (1 / sum e).  One workgroup per row; dst doubles as the
// row scratch exactly as in the reference.
// ---------------------------------------------------------------------------------------------
static __device__ __forceinline__ float block_reduce_256(float v, bool is_max, float *s_part) {
    v = is_max ? wave_max(v) : wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = v;
    __syncthreads();
    return is_max ? fmaxf(fmaxf(s_part[0], s_part[1]), fmaxf(s_part[2], s_part[3])) : (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
}

__global__ __launch_bounds__(256) void softmax_kernel(tdesc x, tdesc mask, bool has_mask, tdesc y, float scale) {
    __shared__ float s_part[4];
    const int64_t r = blockIdx.x;
    const int64_t ne0 = y.ne[0], ne1 = y.ne[1], ne2 = y.ne[2];
    const int64_t i3 = r / (ne1 * ne2), i2 = r % (ne1 * ne2) / ne1, i1 = r % ne1;
    const float *s = (const float *)at(x, 0, i1, i2, i3);
    const float *mk_ = has_mask ? (const float *)at(mask, 0, i1, 0, 0) : nullptr;
    float *d = (float *)at(y, 0, i1, i2, i3);
    float mx = -INFINITY;
    for (int64_t i = threadIdx.x; i < ne0; i += 256) {
        const float t = has_mask ? (s[i] + mk_[i]) * scale : s[i] * scale;
        d[i] = t;
        mx = fmaxf(mx, t);
    }
    mx = block_reduce_256(mx, true, s_part);
    float sum = 0.0f;
    for (int64_t i = threadIdx.x; i < ne0; i += 256) {
        float e;
        if (has_mask && mk_[i] == -INFINITY) e = 0.0f;
        else e = expf(h2f(f2h(d[i] - mx)));
        d[i] = e;
        sum += e;
    }
    sum = block_reduce_256(sum, false, s_part);
    const float inv = 1.0f / sum;
    for (int64_t i = threadIdx.x; i < ne0; i += 256) d[i] *= inv;
}

// The same arithmetic with the row kept in LDS between the passes (one read of the scores, one write of the
// probabilities) for rows of up to SOFTMAX_LDS_ROW elements; the additions of the sum happen in the same order
// as above (thread stride 256, then the same tree), so both kernels give the same bits.  Masked elements
// (mask = -inf, scale > 0) are not read: (s - inf) * scale = -inf whatever the finite score.  F16OUT stores the
// probabilities rounded to fp16, which is what the KQV product does to them first anyway (mat.cpp:37).
#define SOFTMAX_LDS_ROW 16384
template <bool F16OUT>
__global__ __launch_bounds__(256) void softmax_row_kernel(tdesc x, tdesc mask, bool has_mask, tdesc y, float scale, int causal_past) {
    extern __shared__ __attribute__((aligned(16))) float s_row[];
    __shared__ float s_part[4];
    const int64_t r = blockIdx.x;
    const int ne0 = (int)y.ne[0];
    const int64_t ne1 = y.ne[1], ne2 = y.ne[2];
    const int64_t i3 = r / (ne1 * ne2), i2 = r % (ne1 * ne2) / ne1, i1 = r % ne1;
    const float *s = (const float *)at(x, 0, i1, i2, i3);
    // causal_past >= 0: the mask is known to be the causal one of a pass that starts at position causal_past (row i1 sees
    // the first causal_past + i1 + 1 elements) and is not read; the elements beyond contribute -inf to the maximum and 0
    // to the sum, i.e. nothing, so the bits are those of the masked path
    const int nv = causal_past >= 0 ? (int)min((int64_t)ne0, causal_past + i1 + 1) : ne0;
    const float *mk_ = (has_mask && causal_past < 0) ? (const float *)at(mask, 0, i1, 0, 0) : nullptr;
    float mx = -INFINITY;
    for (int i = threadIdx.x; i < nv; i += 256) {
        float t;
        if (mk_) { const float mv = mk_[i]; t = (mv == -INFINITY) ? -INFINITY : (s[i] + mv) * scale; }
        else t = s[i] * scale;
        s_row[i] = t;
        mx = fmaxf(mx, t);
    }
    mx = block_reduce_256(mx, true, s_part);
    float sum = 0.0f;
    for (int i = threadIdx.x; i < nv; i += 256) {
        const float t = s_row[i];
        const float e = (mk_ && t == -INFINITY) ? 0.0f : expf(h2f(f2h(t - mx)));
        s_row[i] = e;
        sum += e;
    }
    sum = block_reduce_256(sum, false, s_part);
    const float inv = 1.0f / sum;
    if constexpr (F16OUT) {
        uint16_t *d = (uint16_t *)at(y, 0, i1, i2, i3);
        for (int i = threadIdx.x; i < ne0; i += 256) d[i] = i < nv ? f2h(s_row[i] * inv) : (uint16_t)0;
    } else {
        float *d = (float *)at(y, 0, i1, i2, i3);
        for (int i = threadIdx.x; i < ne0; i += 256) d[i] = i < nv ? s_row[i] * inv : 0.0f;
    }
}

static int softmax_launch(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *mask, const spy_hip_tensor *dst, float scale, int causal_past);
// Softmax under the causal mask of a pass that starts at position n_past, without reading a mask tensor (the token
// loop fills its masks itself and knows their shape).  Same bits as spy_hip_op_softmax with that mask.
int spy_softmax_row_ok(int64_t ne0) { return ne0 <= SOFTMAX_LDS_ROW; }   // rows of ne0 elements take the row kernel
int spy_softmax_causal_launch(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *dst, float scale, int n_past) {
    SPY_CHECK_ARG(n_past >= 0 && dst && scale > 0.0f && spy_softmax_row_ok(dst->ne[0]));
    return softmax_launch(stream, x, nullptr, dst, scale, n_past);
}

extern "C" int spy_hip_op_softmax(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *mask, const spy_hip_tensor *dst, float scale) {
    return softmax_launch(stream, x, mask, dst, scale, -1);
}

static int softmax_launch(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *mask, const spy_hip_tensor *dst, float scale, int causal_past) {
    SPY_CHECK_ARG(x && dst && x->data && dst->data);
    if (x->type != SPY_HIP_F32 || (dst->type != SPY_HIP_F32 && dst->type != SPY_HIP_F16)) return SPY_HIP_EUNSUPPORTED;
    SPY_CHECK_ARG(same_ne(x, dst) && x->nb[0] == 4 && dst->nb[0] == (dst->type == SPY_HIP_F16 ? 2 : 4));
    tdesc m = mk(x);
    if (mask) {
        // the mask is typed INT32 by the graph (inout.cpp:43-47) but read as float (non-linear.cpp:147)
        SPY_CHECK_ARG(mask->data && mask->nb[0] == 4 && mask->ne[0] >= dst->ne[0] && mask->ne[1] >= dst->ne[1]);
        m = mk(mask);
    }
    const int64_t nrow = spy_t_nrow(dst);
    CHECK_GRID(nrow, 1);
    if (causal_past < 0 && dst->type == SPY_HIP_F32 && spy_exact_on()) return spy_exact_softmax((hipStream_t)stream, x, mask, dst, scale);
    // a masked element of the generic kernel reads as (s + mask) * scale: the row kernel's shortcut needs scale > 0 and a
    // mask that really is 0 / -inf, which is what the graph builds (llama.cpp:248-263)
    const bool row_ok = spy_softmax_row_ok(dst->ne[0]) && scale > 0.0f;
    if (dst->type == SPY_HIP_F16 && !row_ok) return SPY_HIP_EUNSUPPORTED;
    if (row_ok) {
        const size_t lds = (size_t)dst->ne[0] * 4;
        if (lds > 48 * 1024) {
            int rc_ = spy_raise_lds_limit((const void *)softmax_row_kernel<false>, SOFTMAX_LDS_ROW * 4);
            if (!rc_) rc_ = spy_raise_lds_limit((const void *)softmax_row_kernel<true>, SOFTMAX_LDS_ROW * 4);
            if (rc_) return rc_;
        }
        if (dst->type == SPY_HIP_F16) softmax_row_kernel<true><<<dim3((unsigned)nrow), dim3(256), lds, (hipStream_t)stream>>>(mk(x), m, mask != nullptr, mk(dst), scale, causal_past);
        else softmax_row_kernel<false><<<dim3((unsigned)nrow), dim3(256), lds, (hipStream_t)stream>>>(mk(x), m, mask != nullptr, mk(dst), scale, causal_past);
        return SPY_LAUNCH_RC();
    }
    if (causal_past >= 0) return SPY_HIP_EINVAL;
    softmax_kernel<<<dim3((unsigned)nrow), dim3(256), 0, (hipStream_t)stream>>>(mk(x), m, mask != nullptr, mk(dst), scale);
    return SPY_LAUNCH_RC();
}

// ---------------------------------------------------------------------------------------------
// Rope (non-linear.cpp:270-371), default branch: pair k of token i2 is rotated by
// theta_k = pos[i2] * theta_scale^k where the power is built by k successive fp32
// multiplications (:304-309); cos/sin of theta*freq_scale, times attention_factor.
// ---------------------------------------------------------------------------------------------
// ramp_on: extend_factor != 0 (YaRN, rope_yarn :247-260).  As written, rope_yarn_ramp (:242-245) clamps the VALUE 0 into
// [1, y] -- std::clamp(0.0F, 1.0F, y) -- and so returns 1 - 1 = 0: ramp_mix = 0 * extend_factor, the angle stays the
// interpolated one (the mix is still evaluated as written) and only the magnitude changes (mscale, folded in by the caller).
// xpos (:353-354): zeta = pow((i0 + 0.4 ne0) / (1.4 ne0), position / xpos_base), inverted for xpos_down, times every product.
__global__ __launch_bounds__(64) void rope_kernel(tdesc x, const int32_t *pos, int64_t pos_stride, tdesc y, float theta_scale,
                                                  float freq_scale, float mscale, int ramp_on, float ramp_mix, float xpos_base, int xpos_down) {
    const int64_t i1 = blockIdx.x, i2 = blockIdx.y, i3 = blockIdx.z;
    const int32_t pi = *(const int32_t *)((const uint8_t *)pos + i2 * pos_stride);
    const float p = (float)pi;
    const int64_t npair = y.ne[0] / 2;
    const float ne0f = (float)y.ne[0];
    for (int64_t k = threadIdx.x; k < npair; k += 64) {
        float theta = p;
        for (int64_t j = 0; j < k; j++) theta *= theta_scale;
        float ang = freq_scale * theta;
        if (ramp_on) ang = ang * (1 - ramp_mix) + theta * ramp_mix;
        const float c = cosf(ang) * mscale, s = sinf(ang) * mscale;
        const float *sp = (const float *)at(x, 2 * k, i1, i2, i3);
        float *dp = (float *)at(y, 2 * k, i1, i2, i3);
        const float x0 = sp[0], x1 = sp[1];
        if (xpos_base != 0.0f) {
            float zeta = powf(((float)(2 * k) + 0.4f * ne0f) / (1.4f * ne0f), p / xpos_base);
            if (xpos_down) zeta = 1.0f / zeta;
            dp[0] = x0 * c * zeta - x1 * s * zeta;
            dp[1] = x0 * s * zeta + x1 * c * zeta;
        } else {
            dp[0] = x0 * c - x1 * s;
            dp[1] = x0 * s + x1 * c;
        }
    }
}

// Mode GLM (non-linear.cpp:315-343), as written: per row (i1, i2, i3) and i0 < ne0 / 4, with p = pos[i2]:
// theta_base = min(p, num_context - 2), block_theta = max(p - (num_context - 2), 0), both multiplied by theta_scale once per
// i0; elements i0 and i0 + num_dim / 2 are rotated by theta_base, elements i0 + num_dim and i0 + num_dim / 2 + num_dim by
// block_theta.  cosf / sinf on the device (within the per-operator tolerance of the host's).
__global__ __launch_bounds__(64) void rope_glm_kernel(tdesc x, const int32_t *pos, int64_t pos_stride, tdesc y, float theta_scale, int num_context, int num_dim) {
    const int64_t i1 = blockIdx.x, i2 = blockIdx.y, i3 = blockIdx.z;
    const int32_t p = *(const int32_t *)((const uint8_t *)pos + i2 * pos_stride);
    const int nd = num_dim;
    for (int64_t i0 = threadIdx.x; i0 < y.ne[0] / 4; i0 += 64) {
        float theta_base = (float)min(p, num_context - 2), block_theta = (float)max(p - (num_context - 2), 0);
        for (int64_t j = 0; j < i0; j++) { theta_base *= theta_scale; block_theta *= theta_scale; }
        const float c = cosf(theta_base), s = sinf(theta_base), cb = cosf(block_theta), sb = sinf(block_theta);
        const float *sp = (const float *)at(x, i0, i1, i2, i3);
        float *dp = (float *)at(y, i0, i1, i2, i3);
        const float x0 = sp[0], x1 = sp[nd / 2], x2 = sp[nd], x3 = sp[nd / 2 + nd];
        dp[0] = x0 * c - x1 * s;
        dp[nd / 2] = x0 * s + x1 * c;
        dp[nd] = x2 * cb - x3 * sb;
        dp[nd / 2 + nd] = x2 * sb + x3 * cb;
    }
}

extern "C" int spy_hip_op_rope(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *pos, const spy_hip_tensor *dst, const spy_hip_rope_param *p) {
    SPY_CHECK_ARG(x && pos && dst && p && x->data && pos->data && dst->data);
    if (x->type != SPY_HIP_F32 || dst->type != SPY_HIP_F32 || pos->type != SPY_HIP_I32) return SPY_HIP_EUNSUPPORTED;
    if (p->mode == 4) {                                                       // GLM
        if (spy_exact_on()) return SPY_HIP_EUNSUPPORTED;                      // no host-libm table for this mode
        SPY_CHECK_ARG(same_ne(x, dst) && x->nb[0] == 4 && dst->nb[0] == 4 && p->num_dim > 0 && p->num_dim % 2 == 0 && dst->ne[0] >= 4);
        SPY_CHECK_ARG(pos->ne[0] >= dst->ne[2] && dst->ne[1] < 65536 && dst->ne[2] < 65536 && dst->ne[3] < 65536 && dst->ne[1] > 0 && dst->ne[2] > 0 && dst->ne[3] > 0);
        // the four elements of the last i0 must lie inside the row (the reference does not check: it would read the next row); and an
        // in-place call must not have one i0 write what another reads: true when the four index ranges do not overlap
        SPY_CHECK_ARG(dst->ne[0] / 4 - 1 + p->num_dim / 2 + p->num_dim < dst->ne[0] && p->num_dim / 2 >= dst->ne[0] / 4);
        const float ts = powf(p->freq_base, -2.0f / (float)p->num_dim);
        rope_glm_kernel<<<dim3((unsigned)dst->ne[1], (unsigned)dst->ne[2], (unsigned)dst->ne[3]), dim3(64), 0, (hipStream_t)stream>>>(
            mk(x), (const int32_t *)pos->data, pos->nb[0], mk(dst), ts, p->num_context, p->num_dim);
        return SPY_LAUNCH_RC();
    }
    if (p->mode != 0 && p->mode != -1) return SPY_HIP_EUNSUPPORTED;          // Neox (aborts in the reference too)
    SPY_CHECK_ARG(same_ne(x, dst) && x->nb[0] == 4 && dst->nb[0] == 4 && dst->ne[0] % 2 == 0 && p->num_dim > 0);
    SPY_CHECK_ARG(pos->ne[0] >= dst->ne[2] && dst->ne[1] < 65536 && dst->ne[2] < (1ll << 31) && dst->ne[3] < 65536);
    SPY_CHECK_ARG(dst->ne[1] > 0 && dst->ne[2] > 0 && dst->ne[3] > 0);
    const float theta_scale = powf(p->freq_base, -2.0f / (float)p->num_dim);   // host libm, as the reference (:282)
    // CUDA-style grids cap y/z at 65535: put the token index on x when it is the large one
    const dim3 grid((unsigned)dst->ne[1], (unsigned)dst->ne[2], (unsigned)dst->ne[3]);
    SPY_CHECK_ARG(dst->ne[2] < 65536);
    if (spy_exact_on()) return spy_exact_rope((hipStream_t)stream, x, pos, dst, p);
    float mscale = p->attention_factor;
    const int ramp_on = p->extend_factor != 0.0f;
    if (ramp_on) mscale *= 1.0f + 0.1f * logf(1.0f / p->freq_scale);          // :257, host libm as the reference
    rope_kernel<<<grid, dim3(64), 0, (hipStream_t)stream>>>(mk(x), (const int32_t *)pos->data, pos->nb[0], mk(dst), theta_scale,
                                                           p->freq_scale, mscale, ramp_on, (1.0f - 1.0f) * p->extend_factor, p->xpos_base, p->xpos_down);
    return SPY_LAUNCH_RC();
}

// ---------------------------------------------------------------------------------------------
// Dup / Copy (view.cpp:83-195).  mode 0: same shape, element (i0..i3) -> element (i0..i3);
// mode 1: contiguous src -> contiguous dst of another shape = flat copy; mode 2: strided src,
// flat source counter unravelled in the destination's dimensions (:164-171).
// conv: 0 raw 4-byte copy, 1 f32 -> f16, 2 f16 -> f32, 3 raw 2-byte copy.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dup_kernel(tdesc s, tdesc d, int mode, int conv, int64_t total) {
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= total) return;
    const int64_t i00 = g % s.ne[0], r = g / s.ne[0];
    const int64_t i01 = r % s.ne[1], i02 = r / s.ne[1] % s.ne[2], i03 = r / (s.ne[1] * s.ne[2]);
    const uint8_t *sp = at(s, i00, i01, i02, i03);
    uint8_t *dp;
    if (mode == 0) dp = at(d, i00, i01, i02, i03);
    else if (mode == 1) dp = d.p + g * d.nb[0];
    else {
        const int64_t i0 = g % d.ne[0], i1 = g / d.ne[0] % d.ne[1];
        const int64_t i2 = g % (d.ne[2] * d.ne[1] * d.ne[0]) / (d.ne[1] * d.ne[0]), i3 = g / (d.ne[2] * d.ne[1] * d.ne[0]);
        dp = at(d, i0, i1, i2, i3);
    }
    switch (conv) {
    case 0: *(uint32_t *)dp = *(const uint32_t *)sp; break;
    case 1: *(uint16_t *)dp = f2h(*(const float *)sp); break;
    case 2: *(float *)dp = h2f(*(const uint16_t *)sp); break;
    default: *(uint16_t *)dp = *(const uint16_t *)sp; break;
    }
}

static int conv_code(int ts, int td) {
    if (ts == td && (ts == SPY_HIP_F32 || ts == SPY_HIP_I32)) return 0;
    if (ts == SPY_HIP_F32 && td == SPY_HIP_F16) return 1;
    if (ts == SPY_HIP_F16 && td == SPY_HIP_F32) return 2;
    if (ts == SPY_HIP_F16 && td == SPY_HIP_F16) return 3;
    return -1;
}

extern "C" int spy_hip_op_dup(void *stream, const spy_hip_tensor *src, const spy_hip_tensor *dst) {
    SPY_CHECK_ARG(src && dst && src->data && dst->data);
    const int conv = conv_code(src->type, dst->type);
    if (conv < 0) return SPY_HIP_EUNSUPPORTED;
    SPY_CHECK_ARG(spy_t_nelem(src) == spy_t_nelem(dst));                     // operator/view.h Copy::propagate
    int mode;
    if (spy_t_contiguous(src)) {
        if (same_shape(src, dst)) mode = 0;                                  // row-by-row memcpy (view.cpp:106-109)
        else if (spy_t_contiguous(dst)) mode = 1;                            // rows appended to a contiguous destination (:132-159)
        else return SPY_HIP_EUNSUPPORTED;                                    // spy_assert(false) (:160-162)
    } else {
        if (conv == 2 || conv == 3) return SPY_HIP_EUNSUPPORTED;             // only F32 sources (:173-188)
        mode = 2;
    }
    const int64_t total = spy_t_nelem(src);
    CHECK_GRID(total, 256);
    dup_kernel<<<dim3(grid_for(total, 256)), dim3(256), 0, (hipStream_t)stream>>>(mk(src), mk(dst), mode, conv, total);
    return SPY_LAUNCH_RC();
}

// Contiguous (view.cpp:285-321): dst (contiguous, src's dims) [i0..i3] = src[i0..i3]
__global__ __launch_bounds__(256) void contiguous_kernel(tdesc s, float *d, int64_t total) {
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= total) return;
    const int64_t i0 = g % s.ne[0], r = g / s.ne[0];
    const int64_t i1 = r % s.ne[1], i2 = r / s.ne[1] % s.ne[2], i3 = r / (s.ne[1] * s.ne[2]);
    d[g] = *(const float *)at(s, i0, i1, i2, i3);
}

extern "C" int spy_hip_op_contiguous(void *stream, const spy_hip_tensor *src, const spy_hip_tensor *dst) {
    SPY_CHECK_ARG(src && dst && src->data && dst->data);
    if (src->type != SPY_HIP_F32 || dst->type != SPY_HIP_F32) return SPY_HIP_EUNSUPPORTED;
    SPY_CHECK_ARG(same_ne(src, dst) && spy_t_contiguous(dst));
    const int64_t total = spy_t_nelem(src);
    CHECK_GRID(total, 256);
    contiguous_kernel<<<dim3(grid_for(total, 256)), dim3(256), 0, (hipStream_t)stream>>>(mk(src), (float *)dst->data, total);
    return SPY_LAUNCH_RC();
}

// ---------------------------------------------------------------------------------------------
// GetRow (view.cpp:33-81): one workgroup per requested row; F32 copy or Q8_0 -> F32
// (q * fp16 scale, vec_convert.h:436-442).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void get_row_kernel(tdesc table, bool q8, const int32_t *ids, int64_t ne10, int64_t ne11,
                                                      float *dst, int64_t dst_row_elems, int64_t nrow_table, int *err) {
    const int64_t r = blockIdx.x;
    const int64_t i12 = r / (ne10 * ne11), i11 = r % (ne10 * ne11) / ne10;
    const int64_t row = ids[r];
    if (row < 0 || row >= nrow_table) { if (threadIdx.x == 0 && err) atomicExch(err, 1); return; }
    const uint8_t *sp = table.p + row * table.nb[1] + i11 * table.nb[2] + i12 * table.nb[3];
    float *dp = dst + r * dst_row_elems;
    const int64_t ne00 = table.ne[0];
    if (!q8) { for (int64_t i = threadIdx.x; i < ne00; i += 256) dp[i] = ((const float *)sp)[i]; }
    else {
        for (int64_t i = threadIdx.x; i < ne00; i += 256) {
            const blk_q8_0 *b = (const blk_q8_0 *)sp + (i >> 5);
            dp[i] = (float)b->qs[i & 31] * h2f(b->d);
        }
    }
}

extern "C" int spy_hip_op_get_row(void *stream, const spy_hip_tensor *table, const spy_hip_tensor *ids, const spy_hip_tensor *dst) {
    SPY_CHECK_ARG(table && ids && dst && table->data && ids->data && dst->data);
    if (ids->type != SPY_HIP_I32 || dst->type != SPY_HIP_F32) return SPY_HIP_EUNSUPPORTED;
    if (table->type != SPY_HIP_F32 && table->type != SPY_HIP_Q8_0) return SPY_HIP_EUNSUPPORTED;   // spy_abort (view.cpp:74-75)
    SPY_CHECK_ARG(spy_t_contiguous(ids) && spy_t_contiguous(dst) && dst->ne[0] == table->ne[0]);
    SPY_CHECK_ARG(table->nb[0] == spy_type_size(table->type));
    const int64_t n = ids->ne[0] * ids->ne[1] * ids->ne[2];
    SPY_CHECK_ARG(spy_t_nrow(dst) >= n);
    CHECK_GRID(n, 1);
    get_row_kernel<<<dim3((unsigned)n), dim3(256), 0, (hipStream_t)stream>>>(mk(table), table->type == SPY_HIP_Q8_0, (const int32_t *)ids->data,
                                                                             ids->ne[0], ids->ne[1], (float *)dst->data, dst->ne[0],
                                                                             spy_t_nrow(table), spy_hip_err_flag_ptr());
    return SPY_LAUNCH_RC();
}

// ---------------------------------------------------------------------------------------------
// Greedy argmax (greedy.h:20-25): std::max_element keeps the FIRST maximum.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void argmax_kernel(const float *__restrict__ x, int64_t n, int32_t *out) {
    __shared__ float s_v[16];
    __shared__ int s_i[16];
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int64_t i = threadIdx.x; i < n; i += 1024) {
        const float v = x[i];
        if (v > best || (bi == 0x7fffffff && !(v < best))) { best = v; bi = (int)i; }   // strided scan keeps the lowest index per thread
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, SPY_WAVE);
        const int oi = __shfl_xor(bi, o, SPY_WAVE);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if ((threadIdx.x & 63) == 0) { s_v[threadIdx.x >> 6] = best; s_i[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; w++) if (s_v[w] > best || (s_v[w] == best && s_i[w] < bi)) { best = s_v[w]; bi = s_i[w]; }
        *out = bi == 0x7fffffff ? 0 : bi;
    }
}

extern "C" int spy_hip_argmax(void *stream, const float *logits, int64_t n, int32_t *out_index) {
    SPY_CHECK_ARG(logits && out_index && n > 0 && n < (1ll << 31));
    argmax_kernel<<<dim3(1), dim3(1024), 0, (hipStream_t)stream>>>(logits, n, out_index);
    return SPY_LAUNCH_RC();
}

// ---------------------------------------------------------------------------------------------
// MatMul (mat.cpp:32-146)
// ---------------------------------------------------------------------------------------------
// fp16 weight rows x fp16 activation rows (Dot<FP16,FP16>, vec_dot.h:117-146): one wave per
// output element, lanes stride along the contraction.  w and dst strided, xh contiguous.
__global__ __launch_bounds__(256) void matmul_f16_kernel(tdesc w, const uint16_t *__restrict__ xh, tdesc d, int64_t ne11, int64_t total) {
    const int64_t o = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (o >= total) return;
    const int lane = threadIdx.x & 63;
    const int64_t ne00 = w.ne[0], ne01 = w.ne[1], ne02 = w.ne[2];
    const int64_t i01 = o % ne01, i11 = o / ne01 % ne11, i02 = o / (ne01 * ne11) % ne02, i03 = o / (ne01 * ne11 * ne02);
    const uint16_t *wr = (const uint16_t *)at(w, 0, i01, i02, i03);
    const uint16_t *xr = xh + ((i03 * ne02 + i02) * ne11 + i11) * ne00;
    float acc = 0.0f;
    for (int64_t k = lane; k < ne00; k += 64) acc = fmaf(h2f(wr[k]), h2f(xr[k]), acc);
    acc = wave_sum(acc);
    if (lane == 0) *(float *)at(d, i01, i11, i02, i03) = acc;
}

int spy_gemm_f16_launch(hipStream_t st, const void *A, int64_t a_nb1, int64_t a_nb2, const uint16_t *B, void *dst, int64_t d_nb1, int64_t d_nb2,
                        int64_t M, int64_t N, int64_t K, int64_t nbatch, int skip_past, int klimit_past);      // gemm.hip

static int mid_type(int t0, int t1) {                                        // target_buffer_type (mat.cpp:32-42) + K-quants
    if (t0 == t1) return t0;
    if (t0 == SPY_HIP_F16 && t1 == SPY_HIP_F32) return SPY_HIP_F16;
    if ((t0 == SPY_HIP_Q4_0 || t0 == SPY_HIP_Q8_0 || t0 == SPY_HIP_Q4_K || t0 == SPY_HIP_Q6_K) && t1 == SPY_HIP_F32) return SPY_HIP_Q8_0;
    return t0;
}

// f32 [ne10, ne11, batches] with byte strides -> contiguous fp16, 4 elements per thread; blockIdx.y = batch
__global__ __launch_bounds__(256) void to_f16_batched_kernel(const uint8_t *__restrict__ x, int64_t nb1, int64_t nb2, int64_t nb3,
                                                              uint16_t *__restrict__ y, int64_t ne10, int64_t ne11, int64_t ne12) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x, q = ne10 / 4;
    if (i >= q * ne11) return;
    const int64_t row = i / q, c = i - row * q, b = blockIdx.y, i12 = b % ne12, i13 = b / ne12;
    const float4 v = *(const float4 *)(x + i13 * nb3 + i12 * nb2 + row * nb1 + c * 16);
    uint2 o;
    o.x = (uint32_t)f2h(v.x) | ((uint32_t)f2h(v.y) << 16);
    o.y = (uint32_t)f2h(v.z) | ((uint32_t)f2h(v.w) << 16);
    *(uint2 *)(y + (b * ne11 + row) * ne10 + c * 4) = o;
}

// the same for any row length and alignment (4-byte aligned floats): one element per thread
__global__ __launch_bounds__(256) void to_f16_batched_scalar_kernel(const uint8_t *__restrict__ x, int64_t nb1, int64_t nb2, int64_t nb3,
                                                                     uint16_t *__restrict__ y, int64_t ne10, int64_t ne11, int64_t ne12) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= ne10 * ne11) return;
    const int64_t row = i / ne10, c = i - row * ne10, b = blockIdx.y, i12 = b % ne12, i13 = b / ne12;
    y[(b * ne11 + row) * ne10 + c] = f2h(*(const float *)(x + i13 * nb3 + i12 * nb2 + row * nb1 + c * 4));
}

// bytes of the converted activations: the part of the scratch buffer that MatMul cannot do without
static size_t matmul_act_bytes(const spy_hip_tensor *w, const spy_hip_tensor *x) {
    if (!w || !x) return 0;
    const int tm = mid_type(w->type, x->type);
    if (tm == x->type) return 0;
    if (tm != SPY_HIP_Q8_0 && tm != SPY_HIP_F16) return 0;
    if (x->ne[0] % spy_block_size(tm) != 0) return 0;
    return (size_t)(spy_t_nrow(x) * spy_row_size(tm, x->ne[0]));
}
// ... plus, while the exact summation order is on, room for the fp16 copies of both operands that its prompt-sized Q4_0 / Q8_0
// MatMul runs from (a call with less than this, but the activations' part, runs the kernel that unpacks per tile: same results)
extern "C" size_t spy_hip_op_matmul_scratch_size(const spy_hip_tensor *w, const spy_hip_tensor *x) {
    const size_t act = matmul_act_bytes(w, x);
    if (!act || !spy_exact_on() || x->type != SPY_HIP_F32 || (w->type != SPY_HIP_Q4_0 && w->type != SPY_HIP_Q8_0) || w->ne[2] != 1 || w->ne[3] != 1) return act;
    const size_t pk = spy_exact_pack_bytes(w->ne[1], w->ne[0], x->ne[1]);
    return pk ? ((act + 255) & ~(size_t)255) + pk : act;
}

int spy_own_matvec_q4_0(hipStream_t st, const void *w, const float *x, float *out, int M, int K);      // engine_q*.hip: the one-row-per-wave kernel without a residual
int spy_own_matvec_q8_0(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
int spy_own_matvec_q4_k(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
int spy_own_matvec_q6_k(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
static int own_matvec(hipStream_t st, int t0, const void *w, const float *x, float *out, int64_t M, int64_t K) {
    if (M <= 0 || M >= (1ll << 30) || K <= 0 || K > 16384 || ((uintptr_t)w & 3) != 0 || ((uintptr_t)x & 15) != 0 || ((uintptr_t)out & 3) != 0) return SPY_HIP_EUNSUPPORTED;
    switch (t0) {
    case SPY_HIP_Q4_0: return spy_own_matvec_q4_0(st, w, x, out, (int)M, (int)K);
    case SPY_HIP_Q8_0: return spy_own_matvec_q8_0(st, w, x, out, (int)M, (int)K);
    case SPY_HIP_Q4_K: return ((uintptr_t)w & 15) == 0 ? spy_own_matvec_q4_k(st, w, x, out, (int)M, (int)K) : SPY_HIP_EUNSUPPORTED;
    case SPY_HIP_Q6_K: return spy_own_matvec_q6_k(st, w, x, out, (int)M, (int)K);
    default: return SPY_HIP_EUNSUPPORTED;
    }
}
static int matmul_impl(void *stream, const spy_hip_tensor *w, const spy_hip_tensor *x, const spy_hip_tensor *dst, void *scratch, size_t scratch_bytes,
                       int skip_past, int klimit_past);
extern "C" int spy_hip_op_matmul(void *stream, const spy_hip_tensor *w, const spy_hip_tensor *x, const spy_hip_tensor *dst,
                                 void *scratch, size_t scratch_bytes) {
    return matmul_impl(stream, w, x, dst, scratch, scratch_bytes, -1, -1);
}
// The two attention products of a prompt pass that starts at position `past`, told about the causal structure so that
// the fp16 GEMM leaves out what the mask removes anyway: which = 0: scores (rows of w = cache positions; tiles the
// softmax will never read are not computed), which = 1: probabilities x V^T (the contraction stops where the
// probabilities of a tile are all zero).  Other shapes / types run as the plain operator.
int spy_matmul_causal(void *stream, const spy_hip_tensor *w, const spy_hip_tensor *x, const spy_hip_tensor *dst, void *scratch, size_t scratch_bytes,
                      int which, int past) {
    SPY_CHECK_ARG(past >= 0 && (which == 0 || which == 1));
    return matmul_impl(stream, w, x, dst, scratch, scratch_bytes, which == 0 ? past : -1, which == 1 ? past : -1);
}
static int matmul_impl(void *stream, const spy_hip_tensor *w, const spy_hip_tensor *x, const spy_hip_tensor *dst, void *scratch, size_t scratch_bytes,
                       int skip_past, int klimit_past) {
    SPY_CHECK_ARG(w && x && dst && w->data && x->data && dst->data);
    const int t0 = w->type, t1 = x->type, tm = mid_type(t0, t1);
    if (dst->type != SPY_HIP_F32) return SPY_HIP_EUNSUPPORTED;
    const bool quant = (t0 == SPY_HIP_Q4_0 || t0 == SPY_HIP_Q8_0 || t0 == SPY_HIP_Q4_K || t0 == SPY_HIP_Q6_K) && tm == SPY_HIP_Q8_0;
    const bool half = (t0 == SPY_HIP_F16 && tm == SPY_HIP_F16);
    if (!quant && !half) return SPY_HIP_EUNSUPPORTED;                        // generic Dot<> aborts (vec_dot.h:29-40)
    if (t1 != SPY_HIP_F32 && t1 != tm) return SPY_HIP_EUNSUPPORTED;
    const int64_t ne00 = w->ne[0], ne01 = w->ne[1], ne02 = w->ne[2], ne03 = w->ne[3];
    const int64_t ne10 = x->ne[0], ne11 = x->ne[1], ne12 = x->ne[2], ne13 = x->ne[3];
    SPY_CHECK_ARG(ne00 == ne10 && ne02 == ne12 && ne03 == ne13);             // operator/mat.h:56-59
    SPY_CHECK_ARG(dst->ne[0] == ne01 && dst->ne[1] == ne11 && dst->ne[2] == ne12 && dst->ne[3] == ne13 && dst->nb[0] == 4);
    SPY_CHECK_ARG(ne00 % spy_block_size(t0) == 0 && ne00 % spy_block_size(tm) == 0);
    hipStream_t st = (hipStream_t)stream;

    // a single f32 row against a quantized matrix (every weight product of a single-token pass): one launch that quantizes the row
    // itself in LDS, in the host's summation order or this backend's own
    if (quant && t1 == SPY_HIP_F32 && ne11 == 1 && ne12 == 1 && ne13 == 1 && skip_past < 0 && klimit_past < 0 && x->nb[0] == 4 &&
        w->nb[0] == spy_type_size(t0) && w->nb[1] == spy_row_size(t0, ne00)) {
        const int rc = spy_exact_on() ? spy_exact_matvec(st, t0, w->data, (const float *)x->data, (float *)dst->data, ne01, ne00)
                                      : own_matvec(st, t0, w->data, (const float *)x->data, (float *)dst->data, ne01, ne00);
        if (rc != SPY_HIP_EUNSUPPORTED) return rc;
    }
    // the host's order with 2 .. 15 rows (a short prompt): the same launch once per row -- the lane kernels below take 44 us per row
    // of a 4096 x 4096 matrix, this one 5; from 16 rows on the tiled kernel
    if (quant && t1 == SPY_HIP_F32 && ne11 >= 2 && ne11 <= 15 && ne12 == 1 && ne13 == 1 && skip_past < 0 && klimit_past < 0 && spy_exact_on() &&
        x->nb[0] == 4 && x->nb[1] % 16 == 0 && dst->nb[1] % 4 == 0 && w->nb[0] == spy_type_size(t0) && w->nb[1] == spy_row_size(t0, ne00)) {
        int rc = 0;
        for (int64_t i = 0; i < ne11 && rc == 0; i++) {
            rc = spy_exact_matvec(st, t0, w->data, (const float *)((const uint8_t *)x->data + i * x->nb[1]), (float *)((uint8_t *)dst->data + i * dst->nb[1]), ne01, ne00);
            if (rc == SPY_HIP_EUNSUPPORTED && i == 0) break;             // nothing launched yet: the general way
        }
        if (rc != SPY_HIP_EUNSUPPORTED) return rc;
    }

    // 1. activations -> mid type, contiguous [ne10, ne11, ne12, ne13] in scratch (mat.cpp:95-128)
    const uint8_t *xm = (const uint8_t *)x->data;
    const int64_t mid_row = spy_row_size(tm, ne10);
    if (t1 != tm) {
        const size_t need = (size_t)(spy_t_nrow(x) * mid_row);
        if (!scratch || scratch_bytes < need) return SPY_HIP_ENOSPACE;
        SPY_CHECK_ARG(x->nb[0] == 4);
        if (tm == SPY_HIP_F16 && ne12 * ne13 > 1 && ne12 * ne13 <= 65535 && ne10 % 4 == 0 && x->nb[1] % 16 == 0 && x->nb[2] % 16 == 0 &&
            x->nb[3] % 16 == 0 && ((uintptr_t)x->data & 15) == 0 && ne10 * ne11 / 4 < (1ll << 31) * 256) {
            // all batches (heads) in one launch
            to_f16_batched_kernel<<<dim3((unsigned)((ne10 / 4 * ne11 + 255) / 256), (unsigned)(ne12 * ne13)), dim3(256), 0, st>>>(
                (const uint8_t *)x->data, x->nb[1], x->nb[2], x->nb[3], (uint16_t *)scratch, ne10, ne11, ne12);
            if (hipGetLastError() != hipSuccess) return SPY_HIP_EINVAL;
        } else if (tm == SPY_HIP_F16 && ne12 * ne13 > 1 && ne12 * ne13 <= 65535 && x->nb[1] % 4 == 0 && x->nb[2] % 4 == 0 && x->nb[3] % 4 == 0 &&
                   ((uintptr_t)x->data & 3) == 0 && (ne10 * ne11 + 255) / 256 < (1ll << 31)) {
            // all batches in one launch, element by element (a single token's probabilities: n_kv is a multiple of 4 one time in four)
            to_f16_batched_scalar_kernel<<<dim3((unsigned)((ne10 * ne11 + 255) / 256), (unsigned)(ne12 * ne13)), dim3(256), 0, st>>>(
                (const uint8_t *)x->data, x->nb[1], x->nb[2], x->nb[3], (uint16_t *)scratch, ne10, ne11, ne12);
            if (hipGetLastError() != hipSuccess) return SPY_HIP_EINVAL;
        } else
        for (int64_t i13 = 0; i13 < ne13; i13++)
            for (int64_t i12 = 0; i12 < ne12; i12++) {
                const float *src = (const float *)((const uint8_t *)x->data + i12 * x->nb[2] + i13 * x->nb[3]);
                uint8_t *out = (uint8_t *)scratch + ((i13 * ne12 + i12) * ne11) * mid_row;
                int rc = (tm == SPY_HIP_Q8_0) ? spy_hip_quantize_q8_0(stream, src, x->nb[1], out, ne11, ne10)
                                              : spy_hip_quantize_f16(stream, src, x->nb[1], out, ne11, ne10);
                if (rc) return rc;
            }
        xm = (const uint8_t *)scratch;
    } else {
        SPY_CHECK_ARG(spy_t_contiguous(x));
    }

    // 2. dots
    if (quant) {
        SPY_CHECK_ARG(w->nb[0] == spy_type_size(t0) && w->nb[1] == spy_row_size(t0, ne00));   // whole contiguous rows
        SPY_CHECK_ARG(dst->nb[1] % 4 == 0);
        if (skip_past < 0 && klimit_past < 0 && spy_exact_on()) {
            // what the activations leave of the scratch buffer: workspace for packed operands
            const size_t used = t1 != tm ? ((size_t)(spy_t_nrow(x) * mid_row) + 255) & ~(size_t)255 : 0;
            const bool room = scratch && scratch_bytes > used && ((uintptr_t)scratch & 15) == 0;
            return spy_exact_dots(st, t0, w, xm, mid_row, ne11, dst, t1 != tm, room ? (uint8_t *)scratch + used : nullptr, room ? scratch_bytes - used : 0);
        }
        for (int64_t i3 = 0; i3 < ne03; i3++)
            for (int64_t i2 = 0; i2 < ne02; i2++) {
                const uint8_t *wp = (const uint8_t *)w->data + i2 * w->nb[2] + i3 * w->nb[3];
                const uint8_t *xp = xm + ((i3 * ne12 + i2) * ne11) * mid_row;
                float *dp = (float *)((uint8_t *)dst->data + i2 * dst->nb[2] + i3 * dst->nb[3]);
                // many activation rows: matrix cores; few: the bandwidth-bound row kernels
                const bool mfma = ne11 >= 16 && ne00 % 64 == 0;
                int rc = mfma ? spy_hip_gemm_q8_0act(stream, t0, wp, xp, dp, ne01, ne00, ne11, dst->nb[1] / 4)
                              : spy_hip_gemv_q8_0act(stream, t0, wp, xp, dp, nullptr, ne01, ne00, ne11, dst->nb[1] / 4);
                if (rc) return rc;
            }
        return 0;
    }
    SPY_CHECK_ARG(w->nb[0] == 2);
    if (skip_past < 0 && klimit_past < 0 && spy_exact_on()) return spy_exact_dots(st, t0, w, xm, mid_row, ne11, dst, 0, nullptr, 0);
    if (ne11 >= 16 && ne01 >= 16 && ne00 % 8 == 0 && w->nb[1] % 16 == 0 && w->nb[2] % 16 == 0 && w->nb[3] % 16 == 0 &&
        ((uintptr_t)w->data & 15) == 0 && ((uintptr_t)xm & 15) == 0 && dst->nb[1] % 4 == 0 && dst->nb[2] % 4 == 0 && ne02 <= 65535) {
        for (int64_t i3 = 0; i3 < ne03; i3++) {            // prompt-sized attention products: fp16 MFMA
            int rc = spy_gemm_f16_launch(st, (const uint8_t *)w->data + i3 * w->nb[3], w->nb[1], w->nb[2], (const uint16_t *)xm + i3 * ne12 * ne11 * ne00,
                                         (uint8_t *)dst->data + i3 * dst->nb[3], dst->nb[1], dst->nb[2], ne01, ne11, ne00, ne02, skip_past, klimit_past);
            if (rc) return rc;
        }
        return 0;
    }
    const int64_t total = ne01 * ne11 * ne02 * ne03;
    CHECK_GRID(total, 4);
    matmul_f16_kernel<<<dim3(grid_for(total, 4)), dim3(256), 0, st>>>(mk(w), (const uint16_t *)xm, mk(dst), ne11, total);
    return SPY_LAUNCH_RC();
}

// ---- MatMul for callers that cannot allocate ---------------------------------------------------------
// spy_hip_op_matmul takes the buffer for the converted activations (Q8_0 blocks or fp16 rows) from its caller, who has to
// size and allocate it.  Code under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc cannot:
// for them the same operator runs with that buffer in a fixed array in device memory.  Each device that loads the library
// holds its own copy of the array until the process ends; every call on a device shares it, so calls that overlap on one
// device race, and a call sees the bytes the previous call left (the conversion kernels overwrite every byte the dots read).
#define SPY_STATIC_SCRATCH_BYTES (8u << 20)      // 8 MiB: 512 activation rows of 11008 elements as Q8_0 blocks (5.6 MiB) fit
#define SPY_STATIC_SCRATCH_MAX_DEVICES 64
static __device__ __align__(256) uint8_t scratch[SPY_STATIC_SCRATCH_BYTES];
static void *g_scratch_ptr[SPY_STATIC_SCRATCH_MAX_DEVICES];     // the array's device address, per device

// Called by spy_hip_init with the device current (and by the entry point's first call on a device that never went through
// it): the array's name is only a host-side handle, its address on the current device comes from the runtime.
int spy_static_scratch_setup(int device) {
    if (device < 0 || device >= SPY_STATIC_SCRATCH_MAX_DEVICES) return SPY_HIP_EINVAL;
    if (g_scratch_ptr[device]) return 0;
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return SPY_HIP_EINVAL;
    g_scratch_ptr[device] = p;
    return 0;
}

extern "C" size_t spy_hip_op_matmul_noalloc_max_scratch(void) { return SPY_STATIC_SCRATCH_BYTES; }

extern "C" int spy_hip_op_matmul_noalloc(void *stream, const spy_hip_tensor *w, const spy_hip_tensor *x, const spy_hip_tensor *dst) {
    SPY_CHECK_ARG(w && x && dst);
    int dev = -1;
    const hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    const int rc = spy_static_scratch_setup(dev);
    if (rc) return rc;
    const size_t need = matmul_act_bytes(w, x);
    if (need > SPY_STATIC_SCRATCH_BYTES) return SPY_HIP_ENOSPACE;     // the converted activations do not fit the fixed array
    return matmul_impl(stream, w, x, dst, g_scratch_ptr[dev], SPY_STATIC_SCRATCH_BYTES, -1, -1);
}
