// Quantized matrix x vector(s): every weight row dotted with 1..8 Q8_0 activation rows.
// Replaces the Dot<Q4_0,Q8_0> / Dot<Q8_0,Q8_0> loops of OperatorMatMulImpl::execute
// (backend/host/include/simd/vec_dot.h:42-115, backend/host/operator/mat.cpp:130-143 in the Spy
// tree) and adds Q4_K / Q6_K weights, which the reference only declares.
//
// HBM-bound: each weight byte is read once, straight from the native GGUF block layout.  The
// int32 block dot is exact; only the fp32 accumulation order differs from the reference's 8-lane
// AVX accumulators.  See gemv_core.cuh for the work split.
#include "gemv_core.cuh"

struct gemv_args {
    const uint8_t *W;        // M rows of K elements, native blocks, contiguous
    const uint8_t *xq;       // NT rows of native Q8_0 blocks, contiguous
    float *dst;              // dst[c*dst_stride + m]
    const float *residual;   // optional, same indexing as dst
    int32_t *dump;           // optional: int32 block dots of column 0, [M][K/32]
    int M, K;
    int64_t dst_stride;
};

// Persistent workgroups: each strides over row tiles, always with two tiles' weights in flight
// (two register buffers).
template <int WT, int LPR, int NIT, int NT, bool DUMP>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_kernel(gemv_args a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int RPW = SPY_WAVE / LPR, RPT = GEMV_WAVES * RPW;
    const int K = a.K, nblk = K / 32, npair = K / 64;
    const size_t RB = (size_t)nblk * wt_traits<WT>::BLK;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l = lane % LPR, g = lane / LPR;
    const int ntiles = (a.M + RPT - 1) / RPT, G = gridDim.x;
    const int rofs = wave * RPW + g;

    wtile<WT, NIT> A, B;
    int tile = blockIdx.x;
    auto fetch = [&](wtile<WT, NIT> &t, int tl) {             // unconditional: beyond the matrix re-reads the last row
        const int r = tl * RPT + rofs;
        load_tile<WT, LPR, NIT>(t, a.W + (size_t)(tl < ntiles && r < a.M ? r : a.M - 1) * RB, npair, l);
    };
    fetch(A, tile);
    fetch(B, tile + G);

    staged_act act[NT];
#pragma unroll
    for (int c = 0; c < NT; c++) {
        int8_t *q = (int8_t *)(smem + (size_t)c * staged_bytes(K));
        int2 *meta = (int2 *)(q + staged_q_bytes(K));
        stage_native_q8(a.xq + (size_t)c * nblk * 34, q, meta, nblk);
        act[c].q = q; act[c].meta = meta;
    }

    auto finish = [&](const wtile<WT, NIT> &t, int tl) {
        const int r = tl * RPT + rofs;
        float acc[NT];
#pragma unroll
        for (int c = 0; c < NT; c++) acc[c] = 0.0f;
        if (r < a.M) dot_tile<WT, LPR, NIT, NT>(t, act, npair, l, acc, DUMP ? a.dump + (size_t)r * nblk : nullptr);
#pragma unroll
        for (int c = 0; c < NT; c++) {
            const float s = group_sum<LPR>(acc[c]);
            if (l == 0 && r < a.M) {
                const size_t o = (size_t)c * a.dst_stride + r;
                a.dst[o] = a.residual ? s + a.residual[o] : s;
            }
        }
    };

    while (tile < ntiles) {
        finish(A, tile);
        fetch(A, tile + 2 * G);
        tile += G;
        if (tile >= ntiles) break;
        finish(B, tile);
        fetch(B, tile + 2 * G);
        tile += G;
    }
}

// ---- one weight row per wave, 1024-thread workgroups (all four weight types; K <= 4096 * NITK) ------
// The standalone form of the single-token kernels: native Q8_0 activation row(s) staged into LDS by
// the whole workgroup, every wave owns rows r = gw + k*NW with 64 lanes x NITK 64-element units each,
// WROW_DEPTH rows requested ahead of their use.  T activation rows are handled one after the other
// against the same row registers (the weights are read once per launch for up to WROW_T rows).
#define WROW_THREADS 1024
#define WROW_DEPTH 3
#define WROW_T 4
template <int WT, int NITK, int NR>
__global__ __launch_bounds__(WROW_THREADS) void wave_row_kernel(gemv_args a, int T) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int NW = (int)gridDim.x * (WROW_THREADS / 64), gw = (int)blockIdx.x * (WROW_THREADS / 64) + wave;
    const int K = a.K, nblk = K / 32, npair = K / 64;
    const size_t RB = (size_t)spy_row_size(WT, K);
    // ring of row registers: row k lives in t[k % RING] and is requested RING - 1 rows ahead of its use
    constexpr int RING = NR < (NITK == 1 ? 4 : 2) ? NR : (NITK == 1 ? 4 : 2);
    constexpr int DEPTH = RING > 1 ? RING - 1 : 1;
    wtile<WT, NITK> t[RING];
    auto issue = [&](int k) {
        const int u = gw + k * NW, r = u < a.M ? u : gw % a.M;
        load_tile<WT, 64, NITK>(t[k % RING], a.W + (size_t)r * RB, npair, lane);
    };
    // activation row 0 is requested first, the first weight rows behind it
    uint32_t xr[NITK + 1];
    stage_native_q8_load<WROW_THREADS, NITK + 1>(a.xq, nblk, xr);
    __builtin_amdgcn_s_barrier();          // every wave's activation request is queued before any wave's first row (issue order, not data)
#pragma unroll
    for (int k = 0; k < NR; k++) if (k < DEPTH) issue(k);
    auto act_of = [&](int c) {                              // staged activation row c (computed, not kept: no private array)
        staged_act s;
        int8_t *q = (int8_t *)(smem + (size_t)c * staged_bytes(K));
        s.q = q; s.meta = (const int2 *)(q + staged_q_bytes(K));
        return s;
    };
    stage_native_q8_finish<WROW_THREADS, NITK + 1>(xr, (int8_t *)smem, (int2 *)(smem + staged_q_bytes(K)), nblk);
    for (int c = 1; c < T; c++) {
        int8_t *q = (int8_t *)(smem + (size_t)c * staged_bytes(K));
        stage_native_q8<WROW_THREADS>(a.xq + (size_t)c * nblk * 34, q, (int2 *)(q + staged_q_bytes(K)), nblk);
    }
    const staged_act act0 = act_of(0);
    constexpr bool HOIST = NR > 1 && NITK == 1;             // keep the lane's activations in registers across rows
    act_frag<HOIST ? NITK : 1> af;
    if constexpr (HOIST) load_act_frag<WT, NITK>(af, act0, npair, lane);
#pragma unroll
    for (int k = 0; k < NR; k++) {
        if (RING > 1 && k + DEPTH < NR) issue(k + DEPTH);
        const int r = gw + k * NW;
        float s;
        if constexpr (HOIST) s = wave_total_lane63(dot_row_frag<WT, NITK>(t[k % RING], af, npair, lane));
        else s = wave_total_lane63(dot_row_lds<WT, NITK>(t[k % RING], act0, npair, lane));
        if (lane == 63 && r < a.M) a.dst[r] = a.residual ? s + a.residual[r] : s;
        for (int c = 1; c < T; c++) {                       // further activation rows against the same weight registers
            s = wave_total_lane63(dot_row_lds<WT, NITK>(t[k % RING], act_of(c), npair, lane));
            const size_t o = (size_t)c * a.dst_stride + r;
            if (lane == 63 && r < a.M) a.dst[o] = a.residual ? s + a.residual[o] : s;
        }
    }
}

template <int WT, int NITK, int NR>
static int launch_wave_row_nr(hipStream_t st, const gemv_args &a, int T, size_t lds, int grid) {
    auto kern = wave_row_kernel<WT, NITK, NR>;
    { const int rc_ = spy_raise_lds_limit((const void *)kern, lds); if (rc_) return rc_; }
    kern<<<dim3((unsigned)grid), dim3(WROW_THREADS), lds, st>>>(a, T);
    return SPY_LAUNCH_RC();
}

// Rows per wave: the fewest of {1, 2, 3, 4, 6, 8} that covers M with at most one workgroup per compute
// unit (an even spread; more workgroups than compute units would leave some of them with twice the work);
// matrices beyond 8 rows per wave take more workgroups.
template <int WT, int NITK>
static int launch_wave_row_nitk(hipStream_t st, const gemv_args &a, int T) {
    static int num_cu = 0;
    if (!num_cu) { int dev = 0; hipDeviceProp_t prop; num_cu = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) ? prop.multiProcessorCount : 256; }
    const size_t lds = (size_t)T * staged_bytes(a.K);
    const int waves = WROW_THREADS / 64;
    const int64_t need = ((int64_t)a.M + (int64_t)num_cu * waves - 1) / ((int64_t)num_cu * waves);
    // rows of more than 4096 elements take one row per wave (several 64-element units per lane: the registers
    // go to the row itself); Q6_K rows (15 dwords per unit) at most 4
    constexpr int NRMAX = NITK > 1 ? 1 : (WT == SPY_HIP_Q6_K ? 4 : 8);
    int nr = need <= 1 ? 1 : need <= 2 ? 2 : need <= 3 ? 3 : need <= 4 ? 4 : need <= 6 ? 6 : 8;
    if (nr > NRMAX) nr = NRMAX;
    const int grid = (int)(((int64_t)a.M + (int64_t)waves * nr - 1) / ((int64_t)waves * nr));
    if constexpr (NRMAX >= 4) {
        switch (nr) {
        case 2: return launch_wave_row_nr<WT, NITK, 2>(st, a, T, lds, grid);
        case 3: return launch_wave_row_nr<WT, NITK, 3>(st, a, T, lds, grid);
        case 4: return launch_wave_row_nr<WT, NITK, 4>(st, a, T, lds, grid);
        default: break;
        }
    }
    if constexpr (NRMAX >= 8) {
        if (nr == 6) return launch_wave_row_nr<WT, NITK, 6>(st, a, T, lds, grid);
        if (nr == 8) return launch_wave_row_nr<WT, NITK, 8>(st, a, T, lds, grid);
    }
    return launch_wave_row_nr<WT, NITK, 1>(st, a, T, lds, grid);
}

// the one-row-per-wave kernels take K % 64 == 0, K <= 12288 and 4-byte aligned activation rows
static bool wave_rows_ok(int64_t K, const void *xq) { return K % 64 == 0 && K <= 12288 && (((uintptr_t)xq) & 3) == 0; }

// K % 64 == 0 (Q4_0 / Q8_0) or K % 256 == 0 (K-quants), K <= 12288
template <int WT>
static int launch_wave_rows(hipStream_t st, const void *w, const uint8_t *xq, float *dst, const float *residual, int64_t M, int64_t K, int64_t T, int64_t dst_stride) {
    const int64_t xrow = (K / 32) * 34;
    for (int64_t t = 0; t < T; t += WROW_T) {
        gemv_args a;
        a.W = (const uint8_t *)w; a.xq = xq + t * xrow; a.dst = dst + t * dst_stride;
        a.residual = residual ? residual + t * dst_stride : nullptr; a.dump = nullptr;
        a.M = (int)M; a.K = (int)K; a.dst_stride = dst_stride;
        const int tc = (int)(T - t < WROW_T ? T - t : WROW_T);
        int rc;
        switch ((K + 4095) / 4096) {
        case 1: rc = launch_wave_row_nitk<WT, 1>(st, a, tc); break;
        case 2: rc = launch_wave_row_nitk<WT, 2>(st, a, tc); break;
        case 3: rc = launch_wave_row_nitk<WT, 3>(st, a, tc); break;
        default: return SPY_HIP_EUNSUPPORTED;
        }
        if (rc) return rc;
    }
    return 0;
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


static int g_num_cu = 0;
static int num_cu() {
    if (!g_num_cu) {
        int dev = 0; hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) g_num_cu = prop.multiProcessorCount;
        if (g_num_cu <= 0) g_num_cu = 256;
    }
    return g_num_cu;
}

// workgroups of `kern` that fit on the device at once (persistent kernels launch exactly that many)
template <class Kern>
static int resident_blocks(Kern kern, size_t lds) {
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, GEMV_THREADS, lds) != hipSuccess || per_cu < 1) per_cu = 1;
    return per_cu * num_cu();
}

template <int WT, int LPR, int NIT, int NT, bool DUMP>
static int launch_fast(hipStream_t st, const gemv_args &a) {
    constexpr int RPT = GEMV_WAVES * (SPY_WAVE / LPR);
    const size_t lds = (size_t)NT * staged_bytes(a.K);
    if (lds > 160 * 1024) return SPY_HIP_EUNSUPPORTED;
    auto kern = gemv_kernel<WT, LPR, NIT, NT, DUMP>;
    { const int rc_ = spy_raise_lds_limit((const void *)kern, lds); if (rc_) return rc_; }
    const int ntiles = (a.M + RPT - 1) / RPT;
    const int cap = resident_blocks(kern, lds);
    kern<<<dim3((unsigned)(ntiles < cap ? ntiles : cap)), dim3(GEMV_THREADS), lds, st>>>(a);
    return SPY_LAUNCH_RC();
}

template <int WT, int NT, bool DUMP>
static int launch_fast_lpr(hipStream_t st, const gemv_args &a) {
    const gemv_cfg cfg = pick_cfg(a.K);
    int rc = SPY_HIP_EUNSUPPORTED;
#define CALL(LPR, NIT) rc = launch_fast<WT, LPR, NIT, NT, DUMP>(st, a)
    GEMV_DISPATCH_CFG(cfg, CALL)
#undef CALL
    return rc;
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
static int gemv_fast_cols(hipStream_t st, const void *w, const uint8_t *xq, float *dst, const float *residual,
                          int64_t M, int64_t K, int64_t T, int64_t dst_stride) {
    // weights are re-read once per group of up to 8 activation rows
    const int64_t xrow = (K / 32) * 34;
    int64_t t = 0;
    while (t < T) {
        const int64_t left = T - t;
        gemv_args a;
        a.W = (const uint8_t *)w; a.xq = xq + t * xrow; a.dst = dst + t * dst_stride;
        a.residual = residual ? residual + t * dst_stride : nullptr; a.dump = nullptr;
        a.M = (int)M; a.K = (int)K; a.dst_stride = dst_stride;
        int rc;
        if (left >= 8)      { rc = launch_fast_lpr<WT, 8, false>(st, a); t += 8; }
        else if (left >= 4) { rc = launch_fast_lpr<WT, 4, false>(st, a); t += 4; }
        else if (left >= 2) { rc = launch_fast_lpr<WT, 2, false>(st, a); t += 2; }
        else                { rc = launch_fast_lpr<WT, 1, false>(st, a); t += 1; }
        if (rc) return rc;
    }
    return 0;
}

static int check_gemv_args(int wtype, const void *w, const void *xq, const void *dst, int64_t M, int64_t K, int64_t T) {
    SPY_CHECK_ARG(w && xq && dst && M > 0 && K > 0 && T > 0);
    SPY_CHECK_ARG(M < (1ll << 30) && K < (1ll << 24) && T < (1ll << 24));
    SPY_CHECK_ARG(((uintptr_t)w % 4) == 0 && ((uintptr_t)xq % 2) == 0 && ((uintptr_t)dst % 4) == 0);
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
    switch (wtype) {
    case SPY_HIP_Q4_0:
        if (wave_rows_ok(K, xq)) return launch_wave_rows<SPY_HIP_Q4_0>(st, w, (const uint8_t *)xq, dst, residual, M, K, T, dst_stride);
        return pick_cfg(K).lpr ? gemv_fast_cols<SPY_HIP_Q4_0>(st, w, (const uint8_t *)xq, dst, residual, M, K, T, dst_stride)
                                         : launch_generic<SPY_HIP_Q4_0, false>(st, w, xq, dst, residual, nullptr, M, K, T, dst_stride);
    case SPY_HIP_Q8_0:
        if (wave_rows_ok(K, xq)) return launch_wave_rows<SPY_HIP_Q8_0>(st, w, (const uint8_t *)xq, dst, residual, M, K, T, dst_stride);
        return pick_cfg(K).lpr ? gemv_fast_cols<SPY_HIP_Q8_0>(st, w, (const uint8_t *)xq, dst, residual, M, K, T, dst_stride)
                                         : launch_generic<SPY_HIP_Q8_0, false>(st, w, xq, dst, residual, nullptr, M, K, T, dst_stride);
    case SPY_HIP_Q4_K:
        return wave_rows_ok(K, xq) ? launch_wave_rows<SPY_HIP_Q4_K>(st, w, (const uint8_t *)xq, dst, residual, M, K, T, dst_stride)
                          : launch_generic<SPY_HIP_Q4_K, false>(st, w, xq, dst, residual, nullptr, M, K, T, dst_stride);
    case SPY_HIP_Q6_K:
        return wave_rows_ok(K, xq) ? launch_wave_rows<SPY_HIP_Q6_K>(st, w, (const uint8_t *)xq, dst, residual, M, K, T, dst_stride)
                          : launch_generic<SPY_HIP_Q6_K, false>(st, w, xq, dst, residual, nullptr, M, K, T, dst_stride);
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
    gemv_args a;
    a.W = (const uint8_t *)w; a.xq = (const uint8_t *)xq; a.dst = sink; a.residual = nullptr; a.dump = out;
    a.M = (int)M; a.K = (int)K; a.dst_stride = M;
    switch (wtype) {
    case SPY_HIP_Q4_0:
        return pick_cfg(K).lpr ? launch_fast_lpr<SPY_HIP_Q4_0, 1, true>(st, a)
                                         : launch_generic<SPY_HIP_Q4_0, true>(st, w, xq, sink, nullptr, out, M, K, 1, M);
    case SPY_HIP_Q8_0:
        return pick_cfg(K).lpr ? launch_fast_lpr<SPY_HIP_Q8_0, 1, true>(st, a)
                                         : launch_generic<SPY_HIP_Q8_0, true>(st, w, xq, sink, nullptr, out, M, K, 1, M);
    case SPY_HIP_Q4_K: return launch_generic<SPY_HIP_Q4_K, true>(st, w, xq, sink, nullptr, out, M, K, 1, M);
    case SPY_HIP_Q6_K: return launch_generic<SPY_HIP_Q6_K, true>(st, w, xq, sink, nullptr, out, M, K, 1, M);
    }
    return SPY_HIP_EUNSUPPORTED;
}
