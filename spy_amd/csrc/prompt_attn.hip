// Causal attention of a prompt pass in one kernel: scores, masked softmax and the product with V^T
// for a tile of 64 queries of one head, without writing the score or probability matrices to memory.
//
// Replaces, for passes over many tokens, the operator sequence MatMul(K, q) -> Softmax(mask, scale) ->
// MatMul(V^T, P) of the LLaMA graph (attention.cpp:25-302; mat.cpp:32-146 with Dot<FP16,FP16>,
// vec_dot.h:117-146; non-linear.cpp:129-180 in the Spy tree).  The arithmetic per element is that of
// those operators: fp16 x fp16 products accumulated in fp32 over the head dimension in ascending order;
// t = s * scale; m = max t over the row; e = expf(float(fp16(t - m))); p = e * (1 / sum e), rounded to
// fp16 as the second MatMul rounds its right operand (mat.cpp:37); fp32 accumulation over the cached
// positions in ascending order.  The softmax needs the row maximum before any exponential and the row
// sum before any probability, so the scores of a tile are computed three times (cheap on the matrix
// cores) instead of being kept: pass 1 maximum, pass 2 sum, pass 3 probabilities and the product.
// (Two passes would need either the scores of a query tile against the whole cache kept somewhere,
// 64 x n_kv floats, or probabilities rounded to fp16 before the sum is known, which is a different
// rounding from the operators'.)  The kernel is bound by the vector instructions of the softmax, not
// by the matrix cores: tiles below the diagonal run without mask compares, the maximum is taken over
// the raw dot products (rounding is monotonic) and the exponential is seven instructions.
// Only the order in which a row's exponentials are added, and the last bit of an exponential, differ
// from softmax_row_kernel.
//
// 256 threads = 2 x 2 waves; a score tile is 64 cached positions x 64 queries, one 32 x 32 MFMA tile per
// wave (positions along the accumulator registers, queries along the lanes, so a lane owns one query);
// the output tile is 128 head dimensions x 64 queries, two 32 x 32 tiles per wave.
#include "common.cuh"

#include <type_traits>

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

#define PA_KROW 272     // LDS bytes per K row: 128 halfs + 16 pad
#define PA_VROW 144     // LDS bytes per V^T / P row: 64 halfs + 16 pad

// e^x for an argument that is a value of fp16 and not above 0 (a score minus its row maximum, rounded as Softmax rounds it).
// log2(e) = LH + LL with 13 significant bits in LH: x * LH is exact in fp32 for an 11-bit x, so is its distance f to the
// nearest integer n; e^x = 2^n * 2^(f + x * LL), with v_exp_f32 on an argument within [-0.5, 0.5] and one rounding (an fma)
// before it: within an ulp or so of expf.  Results below the normal range come out of ldexp as expf returns them.
// A score more than 65504 below its row maximum rounds to -inf in fp16 (expf gives 0 there, the decomposition inf - inf): the
// argument is held at the lowest finite fp16 value, whose exponential is 0 as well.
static __device__ __forceinline__ float pa_exp(_Float16 xh) {
    const float LH = 5909.0f / 4096.0f, LL = 6.80877639634e-05f;
    xh = xh > (_Float16)(-65504.0f) ? xh : (_Float16)(-65504.0f);
    const float ph = fmaf((float)xh, LH, 0.0f), n = rintf(ph);     // the fp16 operand goes into the fma as it is
    const float g = fmaf((float)xh, LL, ph - n);
    return ldexpf(__builtin_amdgcn_exp2f(g), (int)n);
}

struct pattn_args {
    const uint16_t *q16;   // [H][T][128] fp16 (rotated queries)
    const uint16_t *kc;    // K cache, fp16 [n_ctx][H * 128]
    const uint16_t *vc;    // V^T cache, fp16 [H * 128][n_ctx]
    float *out;            // f32 [T][H * 128]
    int T, H, past, n_ctx;
    float scale;
};

// LDS: K tile 0 | K tile 1 or the V^T tile | P tile = 45 KiB, three workgroups per compute unit.  Passes 1 and 2 alternate
// between the two K tiles (one barrier per tile); pass 3 has a second barrier per tile anyway (between the scores and the
// product), which also separates a tile's K reads from the next tile's K store: it keeps K in tile 0 and V^T in the other.
__global__ __launch_bounds__(256, 3) void prompt_attn_kernel(pattn_args a) {
    __shared__ __attribute__((aligned(16))) uint8_t sKV[64 * PA_KROW + 128 * PA_VROW];
    __shared__ __attribute__((aligned(16))) uint8_t sP[64 * PA_VROW];
    static_assert(128 * PA_VROW >= 64 * PA_KROW, "the V^T tile covers the second K tile");
    uint8_t *const sK0 = sKV, *const sK1 = sKV + 64 * PA_KROW, *const sV = sK1;
    __shared__ float s_stat[2][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const int T = a.T, H = a.H, NQ = (T + 63) / 64;
    // Workgroup b runs on XCD b % 8, each with its own L2: all query tiles of a head go to one XCD, so that the head's K and
    // V^T rows (read by every tile, three times) stay in that L2.  Head counts that are not a multiple of 8 use the plain order.
    int h, qt;
    if (H % 8 == 0) { const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3; h = (slot / NQ) * 8 + xcd; qt = slot % NQ; }
    else { h = blockIdx.x / NQ; qt = blockIdx.x % NQ; }
    const int q0 = (NQ - 1 - qt) * 64;                              // late queries (most cached positions) first
    const size_t d = (size_t)H * 128;
    const int n_kv = a.past + T;
    const int ql = wn * 32 + (lane & 31), t = q0 + ql, tq = min(t, T - 1);
    const int limit = a.past + tq;                                  // last cached position this lane's query sees
    const int kv_end = a.past + min(q0 + 63, T - 1) + 1;            // positions any query of the tile sees (<= n_kv)
    const int ntile = (kv_end + 63) / 64;
    const float scale = a.scale;

    v8h fq[8];                                                      // this lane's query: B operand of the score MFMAs
#pragma unroll
    for (int ks = 0; ks < 8; ks++) fq[ks] = *(const v8h *)(a.q16 + ((size_t)h * T + tq) * 128 + ks * 16 + (lane >> 5) * 8);

    // K rows j*64 .. +63 of the head -> registers -> LDS (rows past the cache end re-read its last row: masked below).
    // The loads of tile j + 1 are issued before tile j is multiplied, so that their latency is covered.
    struct quad { uint4 a, b, c, d; };
    quad rk, rv;
    const uint16_t *kbase = a.kc + (size_t)h * 128 + (tid & 15) * 8;         // thread's 16-byte piece of rows (tid >> 4) + 16 i
    const uint16_t *vbase = a.vc + ((size_t)h * 128 + (tid >> 3)) * a.n_ctx;   // thread's piece (tid & 7) of rows (tid >> 3) + 32 i
    // A tile whose 64 rows all lie inside the cache takes its addresses from the tile index alone; the last tile clamps (rows
    // past the cache end re-read its last row: masked below).
    const uint16_t *kthread = kbase + (size_t)(tid >> 4) * d;
    const size_t k16 = (size_t)16 * d;
    auto gload_k = [&](int j) -> quad {
        if (j * 64 + 64 <= n_kv) {
            const uint16_t *p = kthread + (size_t)j * 64 * d;
            return quad{*(const uint4 *)p, *(const uint4 *)(p + k16), *(const uint4 *)(p + 2 * k16), *(const uint4 *)(p + 3 * k16)};
        }
        auto krow = [&](int i) { return (const uint4 *)(kbase + (size_t)min(j * 64 + (tid >> 4) + 16 * i, n_kv - 1) * d); };
        return quad{*krow(0), *krow(1), *krow(2), *krow(3)};
    };
    auto store_k = [&](int b, const quad &r) {
        uint8_t *p = (b ? sK1 : sK0) + (tid >> 4) * PA_KROW + (tid & 15) * 16;
        *(uint4 *)p = r.a; *(uint4 *)(p + 16 * PA_KROW) = r.b; *(uint4 *)(p + 32 * PA_KROW) = r.c; *(uint4 *)(p + 48 * PA_KROW) = r.d;
    };
    auto gload_v = [&](int j) -> quad {                             // V^T tile: 128 rows x 64 positions
        const int col = min(j * 64 + (tid & 7) * 8, a.n_ctx - 8);   // groups of 8 past the cache end carry zero probabilities
        const uint16_t *p = vbase + col;
        const size_t rs = (size_t)32 * a.n_ctx;
        return quad{*(const uint4 *)p, *(const uint4 *)(p + rs), *(const uint4 *)(p + 2 * rs), *(const uint4 *)(p + 3 * rs)};
    };
    auto store_v = [&](const quad &r) {
        uint8_t *p = sV + (tid >> 3) * PA_VROW + (tid & 7) * 16;
        *(uint4 *)p = r.a; *(uint4 *)(p + 32 * PA_VROW) = r.b; *(uint4 *)(p + 64 * PA_VROW) = r.c; *(uint4 *)(p + 96 * PA_VROW) = r.d;
    };
    auto scores = [&](int b) {
        v16f acc = {0};
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            const v8h fa = *(const v8h *)((b ? sK1 : sK0) + (wm * 32 + (lane & 31)) * PA_KROW + ks * 32 + (lane >> 5) * 16);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fq[ks], acc, 0, 0, 0);
        }
        return acc;
    };
    // accumulator register r of tile j holds position j*64 + wm*32 + (r/4)*8 + (lane>>5)*4 + (r&3)
    const int pos0 = wm * 32 + (lane >> 5) * 4;
    // Tiles 0 .. nfree-1 lie below the diagonal for every query of the workgroup (their last position is visible to query q0):
    // no masking there.  The remaining one or two tiles compare positions against the lane's limit.
    const int nfree = min(ntile, max(0, (a.past + q0 + 1) / 64));
    using free_t = std::integral_constant<bool, false>;
    using diag_t = std::integral_constant<bool, true>;

    // pass 1: row maximum of t = s * scale.  Rounding is monotonic, so max(s * scale) = max(s) * scale: one product per row.
    float smax = -INFINITY;
    rk = gload_k(0);
    auto pass1 = [&](int j, auto masked) {
        store_k(j & 1, rk);
        rk = gload_k(min(j + 1, ntile - 1));                        // unconditional: the last tile re-reads itself
        __syncthreads();
        const v16f s = scores(j & 1);
        if constexpr (decltype(masked)::value) {
            const int room = limit - (j * 64 + pos0);               // register r is visible to this lane's query iff (r/4)*8 + (r&3) <= room
#pragma unroll
            for (int r = 0; r < 16; r++) smax = fmaxf(smax, ((r >> 2) * 8 + (r & 3) <= room) ? s[r] : -INFINITY);
        } else {
#pragma unroll
            for (int r = 0; r < 16; r++) smax = fmaxf(smax, s[r]);
        }
    };
    for (int j = 0; j < nfree; j++) pass1(j, free_t{});
    for (int j = nfree; j < ntile; j++) pass1(j, diag_t{});
    float m = smax * scale;
    m = fmaxf(m, __shfl_xor(m, 32, SPY_WAVE));
    if (lane < 32) s_stat[wm][ql] = m;
    __syncthreads();
    m = fmaxf(s_stat[0][ql], s_stat[1][ql]);
    __syncthreads();

    // pass 2: row sum of e = exp(fp16(t - m))
    float sum = 0.0f;
    rk = gload_k(0);
    auto pass2 = [&](int j, auto masked) {
        store_k(j & 1, rk);
        rk = gload_k(min(j + 1, ntile - 1));
        __syncthreads();
        const v16f s = scores(j & 1);
        // every exponential is evaluated (no divergent branches: the 16 evaluations interleave) and the masked ones are
        // replaced by 0 afterwards; adding those zeros changes nothing
        float e[16];
#pragma unroll
        for (int r = 0; r < 16; r++) e[r] = pa_exp((_Float16)(s[r] * scale - m));
        if constexpr (decltype(masked)::value) {
            const int room = limit - (j * 64 + pos0);
#pragma unroll
            for (int r = 0; r < 16; r++) sum += ((r >> 2) * 8 + (r & 3) <= room) ? e[r] : 0.0f;
        } else {
#pragma unroll
            for (int r = 0; r < 16; r++) sum += e[r];
        }
    };
    for (int j = 0; j < nfree; j++) pass2(j, free_t{});
    for (int j = nfree; j < ntile; j++) pass2(j, diag_t{});
    sum += __shfl_xor(sum, 32, SPY_WAVE);
    if (lane < 32) s_stat[wm][ql] = sum;
    __syncthreads();
    const float inv = 1.0f / (s_stat[0][ql] + s_stat[1][ql]);

    // pass 3: probabilities (fp16) through LDS, times V^T
    v16f oacc[2] = {{0}, {0}};
    rk = gload_k(0);
    auto pass3 = [&](int j, auto masked) {
        store_k(0, rk);                                             // every wave passed the previous tile's second barrier: its K reads are done
        rk = gload_k(min(j + 1, ntile - 1));
        rv = gload_v(j);                                            // needed after the scores of this tile
        __syncthreads();                                            // K tile stored; every wave is done with the previous tile's sP / sV
        const v16f s = scores(0);
        const int room = limit - (j * 64 + pos0);
        float e[16];
#pragma unroll
        for (int r = 0; r < 16; r++) e[r] = pa_exp((_Float16)(s[r] * scale - m));
#pragma unroll
        for (int g = 0; g < 4; g++) {
            uint32_t p[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                if constexpr (decltype(masked)::value) p[k] = f2h((g * 8 + k <= room) ? e[4 * g + k] * inv : 0.0f);
                else p[k] = f2h(e[4 * g + k] * inv);
            }
            *(uint2 *)(sP + ql * PA_VROW + (pos0 + g * 8) * 2) = make_uint2(p[0] | (p[1] << 16), p[2] | (p[3] << 16));
        }
        store_v(rv);
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const v8h fa = *(const v8h *)(sV + (wm * 64 + i * 32 + (lane & 31)) * PA_VROW + ks * 32 + (lane >> 5) * 16);
                const v8h fb = *(const v8h *)(sP + ql * PA_VROW + ks * 32 + (lane >> 5) * 16);
                oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb, oacc[i], 0, 0, 0);
            }
    };
    for (int j = 0; j < nfree; j++) pass3(j, free_t{});
    for (int j = nfree; j < ntile; j++) pass3(j, diag_t{});
    if (t < T) {
        float *o = a.out + ((size_t)t * H + h) * 128;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int dd = wm * 64 + i * 32 + g * 8 + (lane >> 5) * 4;
                *(float4 *)(o + dd) = make_float4(oacc[i][4 * g], oacc[i][4 * g + 1], oacc[i][4 * g + 2], oacc[i][4 * g + 3]);
            }
    }
}

// q16: rotated queries as fp16 [H][T][128]; k_cache / v_cache: the layer's caches with the pass's rows already stored;
// out: f32 [T][H * 128] (the layout of the attention output after Permute + Contiguous)
int spy_prompt_attn_launch(hipStream_t st, const uint16_t *q16, const uint16_t *k_cache, const uint16_t *v_cache, float *out,
                           int T, int H, int hd, int past, int64_t n_ctx, float scale) {
    SPY_CHECK_ARG(q16 && k_cache && v_cache && out && T > 0 && H > 0 && H < 65536 && past >= 0 && (int64_t)((T + 63) / 64) * H < (1ll << 31));
    if (hd != 128 || n_ctx % 8 != 0 || n_ctx < 64 || n_ctx >= (1ll << 31)) return SPY_HIP_EUNSUPPORTED;
    SPY_CHECK_ARG(scale > 0.0f);          // the row maximum is taken over the raw dot products and scaled afterwards
    SPY_CHECK_ARG((int64_t)past + T <= n_ctx && ((uintptr_t)q16 % 16) == 0 && ((uintptr_t)k_cache % 16) == 0 && ((uintptr_t)v_cache % 16) == 0 && ((uintptr_t)out % 16) == 0);
    pattn_args a;
    a.q16 = q16; a.kc = k_cache; a.vc = v_cache; a.out = out; a.T = T; a.H = H; a.past = past; a.n_ctx = (int)n_ctx; a.scale = scale;
    prompt_attn_kernel<<<dim3((unsigned)(((T + 63) / 64) * H)), dim3(256), 0, st>>>(a);
    return SPY_LAUNCH_RC();
}

extern "C" int spy_hip_prompt_attention(void *stream, const void *q16, const void *k_cache, const void *v_cache, float *out,
                                        int32_t T, int32_t H, int32_t hd, int32_t past, int64_t n_ctx, float scale) {
    return spy_prompt_attn_launch((hipStream_t)stream, (const uint16_t *)q16, (const uint16_t *)k_cache, (const uint16_t *)v_cache, out, T, H, hd, past, n_ctx, scale);
}
