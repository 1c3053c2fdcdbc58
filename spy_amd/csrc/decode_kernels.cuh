// Kernels of the fused single-token pass (decode).  Six launches per layer:
//   qkv      : RMSNorm*w -> Q8_0 (in LDS) -> wq|wk|wv GEMV -> RoPE -> q (fp16), K cache, V^T cache
//   scores   : s[h][j] = (K[j,h] . fp16(q[h])) * scale            (split over tokens)
//   pv       : softmax with the reference's fp16 rounding points, then P.V (split over head dims)
//   wo       : Q8_0(attn) -> wo GEMV -> + residual
//   gate_up  : RMSNorm*w -> Q8_0 -> gate|up GEMV -> up * silu(gate)
//   down     : Q8_0(h) -> down GEMV -> + residual
// Every rounding point of the operator-by-operator graph is kept (see the comments at each step);
// only fp32 summation orders differ.
#pragma once

#include "gemv_core.cuh"

struct dev_state {           // lives in device memory so that a captured graph can be replayed
    int32_t token;           // token consumed by this pass
    int32_t pos;             // its position = number of tokens already in the KV cache
    int32_t step;            // passes done since the loop was armed
    int32_t err;
};

// ---- persistent GEMV over row tiles with two tiles' weights always in flight ---------------------
// SIDE: one float per row (the residual) travels with the row's tile, so that the epilogue does not
// issue a load of its own (which would have to wait for every older load, i.e. the next tile).
template <int WT, int LPR, int NIT, bool SIDE = false> struct gemv_stream {
    static constexpr int RPW = SPY_WAVE / LPR, RPT = GEMV_WAVES * RPW;
    wtile<WT, NIT> A, B;
    float sideA, sideB;
    const float *side;
    int tile, ntiles, G, npair, l, g, rofs, M;

    // unconditional: a tile index beyond the matrix re-reads the last row (never used)
    template <class RowPtr> __device__ __forceinline__ void fetch(wtile<WT, NIT> &t, float &sd, int tl, RowPtr rowptr) {
        int r = tl * RPT + rofs;
        r = (tl < ntiles && r < M) ? r : M - 1;
        load_tile<WT, LPR, NIT>(t, rowptr(r), npair, l);
        if constexpr (SIDE) sd = side[r];
    }
    template <class RowPtr> __device__ __forceinline__ void begin(int M_, int K, RowPtr rowptr, const float *side_ = nullptr) {
        M = M_; side = side_;
        npair = K / 64;
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
        l = lane % LPR; g = lane / LPR; rofs = wave * RPW + g;
        ntiles = (M + RPT - 1) / RPT; G = gridDim.x; tile = blockIdx.x;
        fetch(A, sideA, tile, rowptr);
        fetch(B, sideB, tile + G, rowptr);
    }
    // epi(r, total, side, valid): called by every lane; `total` is the row's dot, present in all LPR lanes
    template <class RowPtr, class Epi> __device__ __forceinline__ void run(const staged_act &act, RowPtr rowptr, Epi epi) {
        auto finish = [&](const wtile<WT, NIT> &t, float sd, int tl) {
            const int r = tl * RPT + rofs;
            float acc[1] = {0.0f};
            if (r < M) dot_tile<WT, LPR, NIT, 1>(t, &act, npair, l, acc, nullptr);
            epi(r, group_sum<LPR>(acc[0]), sd, r < M);
        };
        while (tile < ntiles) {
            finish(A, sideA, tile);
            fetch(A, sideA, tile + 2 * G, rowptr);
            tile += G;
            if (tile >= ntiles) break;
            finish(B, sideB, tile);
            fetch(B, sideB, tile + 2 * G, rowptr);
            tile += G;
        }
    }
};

// silu as the reference's table: v = float(fp16(x)); v / (1 + expf(-v))  (non-linear.cpp:11-14)
static __device__ __forceinline__ float silu_lut(float x) {
    const float v = h2f(f2h(x));
    return v / (1.0f + expf(-v));
}

// ---- fused GEMVs ----------------------------------------------------------------------------------
struct fused_args {
    const uint8_t *W0, *W1, *W2;
    int M, K;                      // total rows over all matrices, contraction length
    const float *x_in;             // f32[K] prologue input
    const float *normw; float eps; // RMSNorm weight (NORM prologue)
    const float *resid; float *out;
    const dev_state *st; const float *rope_cs; uint16_t *q16; uint16_t *kc; uint16_t *vc;
    int n_ctx, d, hd;
    int pos_imm;                   // st == nullptr: the position as a number (kernel-family entry points)
    uint8_t *q8_dump;              // tests: workgroup 0 of a one-row-per-wave launch writes its staged activations here as native Q8_0 blocks
};

enum { EPI_QKV = 0, EPI_RESID = 1, EPI_GATEUP = 2, EPI_STORE = 3 };

// Prologue: EPI_RESID stages the plain f32 input, every other epilogue the RMS-normalised, weighted
// one; either way SIT float4 of x per thread (K <= 1024*SIT) are requested before the weight tiles.
template <int WT, int LPR, int NIT, int SIT, int EPI>
__global__ __launch_bounds__(GEMV_THREADS) void fused_gemv_kernel(fused_args a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[GEMV_WAVES];
    constexpr bool NORM = (EPI != EPI_RESID);
    const size_t RB = (size_t)spy_row_size(WT, a.K);
    // the matrix bases are selected by arithmetic on wave-uniform differences: a select between
    // the kernel arguments themselves becomes a per-lane load from the argument block
    const ptrdiff_t dW1 = a.W1 - a.W0, dW2 = a.W2 - a.W0;
    auto rowptr = [&](int r) -> const uint8_t * {
        if constexpr (EPI == EPI_QKV) {
            const int m = (r >= a.d) + (r >= 2 * a.d);
            return a.W0 + (m == 0 ? (ptrdiff_t)0 : (m == 1 ? dW1 : dW2)) + (ptrdiff_t)(r - m * a.d) * (ptrdiff_t)RB;
        } else if constexpr (EPI == EPI_GATEUP) return a.W0 + ((r & 1) ? dW1 : (ptrdiff_t)0) + (ptrdiff_t)(r >> 1) * (ptrdiff_t)RB;
        else return a.W0 + (size_t)r * RB;
    };
    stage_regs<NORM ? SIT : 1> sr;
    plain_regs<NORM ? 1 : SIT> pr;
    if constexpr (NORM) stage_norm_load<SIT>(sr, a.x_in, a.normw, a.K);
    else stage_plain_load<SIT>(pr, a.x_in, a.K);
    float rope_v = 0.0f;
    if constexpr (EPI == EPI_QKV) rope_v = a.rope_cs[min((int)threadIdx.x, a.hd - 1)];   // cos/sin table of this position -> LDS
    gemv_stream<WT, LPR, NIT, EPI == EPI_RESID> gs;
    gs.begin(a.M, a.K, rowptr, a.resid);             // the first two tiles' weights are in flight from here on

    int8_t *s_q = (int8_t *)smem;
    int2 *s_meta = (int2 *)(smem + staged_q_bytes(a.K));
    float *s_rope = (float *)(smem + staged_bytes(a.K));
    if constexpr (EPI == EPI_QKV) { if ((int)threadIdx.x < a.hd) s_rope[threadIdx.x] = rope_v; }
    if constexpr (NORM) stage_norm_finish<SIT>(sr, a.eps, s_q, s_meta, a.K, s_red);
    else stage_plain_finish<SIT>(pr, s_q, s_meta, a.K);
    staged_act act; act.q = s_q; act.meta = s_meta;

    const int l = gs.l;
    const int pos = (EPI == EPI_QKV) ? a.st->pos : 0;
    auto epi = [&](int r, float s, float side, bool valid) {
        if constexpr (EPI == EPI_RESID) { if (valid && l == 0) a.out[r] = s + side; }
        else if constexpr (EPI == EPI_STORE) { if (valid && l == 0) a.out[r] = s; }
        else if constexpr (EPI == EPI_GATEUP) {
            // rows 2i (gate) and 2i+1 (up) sit in neighbouring lane groups
            const float other = __shfl_xor(s, LPR, SPY_WAVE);
            if (valid && l == 0 && (r & 1) == 0) a.out[r >> 1] = other * silu_lut(s);   // Mul(ffn_up, silu(ffn_gate)) (ffn.cpp:24-35)
        } else {
            const float other = __shfl_xor(s, LPR, SPY_WAVE);
            if (valid && l == 0) {
                const int m = (r >= a.d) + (r >= 2 * a.d), row = r - m * a.d;
                if (m == 2) a.vc[(size_t)row * a.n_ctx + pos] = f2h(s);                    // VCache_cpy: [d][C] column pos
                else {
                    const int k = (row % a.hd) >> 1;
                    const float c = s_rope[2 * k], sn = s_rope[2 * k + 1];
                    // (x0, x1) -> (x0*c - x1*s, x0*s + x1*c) on adjacent rows (non-linear.cpp:359-363)
                    const float v = (row & 1) ? (other * sn + s * c) : (s * c - other * sn);
                    if (m == 0) a.q16[row] = f2h(v);                                       // attn_score rounds Q to fp16 (mat.cpp:37)
                    else a.kc[(size_t)pos * a.d + row] = f2h(v);                           // KCache_cpy: [token][head][hd]
                }
            }
        }
    };
    gs.run(act, rowptr, epi);
}

// ---- one weight row per wave ------------------------------------------------------------------------
// 1024-thread workgroups, one per compute unit: every wave owns whole rows (64 lanes x NITK block
// pairs), all of them requested at kernel start right after the activation vector, which the 1024
// threads then stage together (one float4 each for K = 4096).  Compared with fused_gemv_kernel this
// quarters the redundant activation reads and the staging work per thread; it is used where a row
// fits 64 lanes x NITK pairs (K <= 4096 * NITK).
//   EPI_QKV   : wave j -> rows 2j, 2j+1 of [W0; W1] (a RoPE pair) and row j of W2          (grid covers d waves)
//   EPI_GATEUP: wave   -> NR pairs (W0 row i, W1 row i), i = gw + k*NW
//   EPI_RESID / EPI_STORE: wave -> NR rows r = gw + k*NW of W0
#define WGV_THREADS 1024
#define WGV_WAVES 16
// Activations of a one-row-per-wave kernel: (RMSNorm * weight ->) Q8_0 in the staged LDS form, by all 1024 threads (float4
// tid + j * 1024 each).  NormRMS (non-linear.cpp:216-219 and the separate Mul node): sums of squares per wave on DPP, the 16
// wave sums as a tree.  Ends with __syncthreads().
template <int NITK, bool NORM>
static __device__ __forceinline__ void wgv_stage(const float4 (&xv)[NITK], const float4 (&wv)[NORM ? NITK : 1], int K, float eps,
                                                 int8_t *s_q, int2 *s_meta, float *s_red) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float scale = 1.0f;
    if constexpr (NORM) {
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < NITK; j++) {
            if (tid + j * WGV_THREADS < K / 4) { const float4 v = xv[j]; acc = fmaf(v.x, v.x, acc); acc = fmaf(v.y, v.y, acc); acc = fmaf(v.z, v.z, acc); acc = fmaf(v.w, v.w, acc); }
        }
        acc = group_sum<64>(acc);
        if (lane == 0) s_red[wave] = acc;
        __syncthreads();
        const float sum = (((s_red[0] + s_red[1]) + (s_red[2] + s_red[3])) + ((s_red[4] + s_red[5]) + (s_red[6] + s_red[7]))) +
                          (((s_red[8] + s_red[9]) + (s_red[10] + s_red[11])) + ((s_red[12] + s_red[13]) + (s_red[14] + s_red[15])));
        scale = 1.0f / sqrtf(sum / (float)K + eps);
    }
#pragma unroll
    for (int j = 0; j < NITK; j++) {
        const int i = tid + j * WGV_THREADS;
        if (i < K / 4) {
            float4 v = xv[j];
            if constexpr (NORM) { const float4 w = wv[j]; v.x = (v.x * scale) * w.x; v.y = (v.y * scale) * w.y; v.z = (v.z * scale) * w.z; v.w = (v.w * scale) * w.w; }
            int2 meta;
            const uint32_t q = quantize_oct(v, meta);
            ((uint32_t *)s_q)[act_dw(i, K >> 6)] = q;
            if ((tid & 7) == 0) s_meta[i >> 3] = meta;
        }
    }
    __syncthreads();
}

#ifndef WGV_DEPTH_QKV
#define WGV_DEPTH_QKV 2
#endif
#ifndef WGV_DEPTH
#define WGV_DEPTH 3             // rows per wave requested ahead of their use
#endif
template <int WT, int NITK, int NR, int EPI, int WTV = WT>      // WTV: type of W2 (the v rows of EPI_QKV)
__global__ __launch_bounds__(WGV_THREADS) void wave_gemv_kernel(fused_args a) {
    constexpr bool NORM = (EPI != EPI_RESID);
    constexpr int NB = EPI == EPI_QKV ? 3 : (EPI == EPI_GATEUP ? 2 * NR : NR);
    constexpr int DEPTH = EPI == EPI_QKV ? WGV_DEPTH_QKV : WGV_DEPTH;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[WGV_WAVES];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int NW = (int)gridDim.x * WGV_WAVES, gw = (int)blockIdx.x * WGV_WAVES + wave;
    const int K = a.K, npair = K / 64;
    const size_t RB = (size_t)spy_row_size(WT, K);

    // 1. the activation vector (and what the epilogue needs), 2. the rows: all unconditional, in this order
    float4 xv[NITK], wv[NORM ? NITK : 1];
#pragma unroll
    for (int j = 0; j < NITK; j++) {
        const int i = min(tid + j * WGV_THREADS, K / 4 - 1);
        xv[j] = ((const float4 *)a.x_in)[i];
        if constexpr (NORM) wv[j] = ((const float4 *)a.normw)[i];
    }
    float rope_v = 0.0f, side[EPI == EPI_RESID ? NR : 1];
    if constexpr (EPI == EPI_QKV) rope_v = a.rope_cs[min(tid, a.hd - 1)];
    // Row k of this wave.  Only WGV_DEPTH rows per wave are requested ahead of their use: the compute
    // unit's vector-memory queue is finite, and a wave that tries to put all its rows in flight at
    // once sits in the issue stage until the queue drains (most of the kernel), holding up the staging
    // barriers of everybody else.
    // Row k lives in slot k % RING: the slot is free again by the time row k + RING is requested (rows up to k + RING - DEPTH - 1
    // have been multiplied by then), so the registers hold DEPTH + 1 rows whatever the number of rows per wave.
    constexpr int RING = NB < DEPTH + 1 ? NB : DEPTH + 1;
    wtile<WT, NITK> t[RING];
    wtile<WTV, NITK> tv;
    auto issue = [&](int k) {
        if constexpr (EPI == EPI_QKV) {
            const int j = gw % a.d;
            const uint8_t *p0 = 2 * j < a.d ? a.W0 + (size_t)(2 * j) * RB : a.W1 + (size_t)(2 * j - a.d) * RB;
            if (k == 2) load_tile<WTV, 64, NITK>(tv, a.W2 + (size_t)j * spy_row_size(WTV, K), npair, lane);
            else load_tile<WT, 64, NITK>(t[k % RING], p0 + (size_t)k * RB, npair, lane);
        } else if constexpr (EPI == EPI_GATEUP) {
            const int F = a.M / 2, u = gw + (k >> 1) * NW, i = u < F ? u : gw % F;
            load_tile<WT, 64, NITK>(t[k % RING], ((k & 1) ? a.W1 : a.W0) + (size_t)i * RB, npair, lane);
        } else {
            const int u = gw + k * NW, r = u < a.M ? u : gw % a.M;
            load_tile<WT, 64, NITK>(t[k % RING], a.W0 + (size_t)r * RB, npair, lane);
            if constexpr (EPI == EPI_RESID) side[k] = a.resid ? a.resid[r] : 0.0f;
        }
    };
    // The compute unit serves its memory requests in order: every wave's activation request goes into the queue before any
    // wave's first row (the barrier waits for the requests to be issued, not for the data).  Without it the last waves' x arrives
    // behind 15 waves' worth of rows, and the staging barrier with it.
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int k = 0; k < NB; k++) if (k < DEPTH) issue(k);

    // 3. stage the activations: RMSNorm * weight (non-linear.cpp:216-219 and the separate Mul node) or plain, then Q8_0
    int8_t *s_q = (int8_t *)smem;
    int2 *s_meta = (int2 *)(smem + staged_q_bytes(K));
    float *s_rope = (float *)(smem + staged_bytes(K));
    if constexpr (EPI == EPI_QKV) { if (tid < a.hd) s_rope[tid] = rope_v; }
    wgv_stage<NITK, NORM>(xv, wv, K, a.eps, s_q, s_meta, s_red);
    if (a.q8_dump && blockIdx.x == 0) {
        for (int b = tid; b < K / 32; b += WGV_THREADS) {
            uint16_t *dst = (uint16_t *)(a.q8_dump + (size_t)b * 34);
            dst[0] = f2h(__int_as_float(s_meta[b].x));
            for (int i = 0; i < 8; i++) {
                const uint32_t q = ((const uint32_t *)s_q)[act_dw(b * 8 + i, K >> 6)];
                dst[1 + 2 * i] = (uint16_t)(q & 0xFFFFu); dst[2 + 2 * i] = (uint16_t)(q >> 16);
            }
        }
    }
    staged_act act; act.q = s_q; act.meta = s_meta;
    act_frag<NITK> af;                                    // this lane's activations: the same for every row
    load_act_frag<WT, NITK>(af, act, npair, lane);
    // partial dots of all rows (requesting the row WGV_DEPTH ahead before each), then their wave reductions
    // (independent chains); totals land in lane 63
    float s[NB];
#pragma unroll
    for (int k = 0; k < NB; k++) {
        if constexpr (NB > DEPTH + 1) __builtin_amdgcn_sched_barrier(0);     // keep the requests where they are: hoisted, they would need more than the ring
        if (k + DEPTH < NB) issue(k + DEPTH);
        if (EPI == EPI_QKV && k == 2) {
            if constexpr (WTV == WT) s[k] = dot_row_frag<WTV, NITK>(tv, af, npair, lane);
            else { act_frag<NITK> av; load_act_frag<WTV, NITK>(av, act, npair, lane); s[k] = dot_row_frag<WTV, NITK>(tv, av, npair, lane); }
        } else s[k] = dot_row_frag<WT, NITK>(t[k % RING], af, npair, lane);
    }
#pragma unroll
    for (int k = 0; k < NB; k++) s[k] = wave_total_lane63(s[k]);

    // 4. epilogues (lane 63 holds the totals)
    if constexpr (EPI == EPI_QKV) {
        if (lane == 63 && gw < a.d) {
            const int j = gw, row = (2 * j) % a.d, k = (row % a.hd) >> 1, pos = a.st ? a.st->pos : a.pos_imm;
            const float c = s_rope[2 * k], sn = s_rope[2 * k + 1];
            // (x0, x1) -> (x0*c - x1*s, x0*s + x1*c) on adjacent rows (non-linear.cpp:359-363)
            const uint32_t pr = (uint32_t)f2h(s[0] * c - s[1] * sn) | ((uint32_t)f2h(s[0] * sn + s[1] * c) << 16);
            if (2 * j < a.d) ((uint32_t *)a.q16)[j] = pr;                                        // attn_score rounds Q to fp16 (mat.cpp:37)
            else ((uint32_t *)(a.kc + (size_t)pos * a.d))[j - a.d / 2] = pr;                      // KCache_cpy: [token][head][hd]
            a.vc[(size_t)j * a.n_ctx + pos] = f2h(s[2]);                                         // VCache_cpy: [d][C] column pos
        }
    } else if constexpr (EPI == EPI_GATEUP) {
        const int F = a.M / 2;
#pragma unroll
        for (int k = 0; k < NR; k++) {
            const int i = gw + k * NW;
            if (lane == 63 && i < F) a.out[i] = s[2 * k + 1] * silu_lut(s[2 * k]);                 // Mul(ffn_up, silu(ffn_gate)) (ffn.cpp:24-35)
        }
    } else {
#pragma unroll
        for (int k = 0; k < NR; k++) {
            const int r = gw + k * NW;
            if (lane == 63 && r < a.M) { if constexpr (EPI == EPI_RESID) a.out[r] = a.resid ? s[k] + side[k] : s[k]; else a.out[r] = s[k]; }     // no resid: the MatMul alone
        }
    }
}

// ---- the attention part of a layer in one kernel -----------------------------------------------------
// qkv, scores and softmax + KQV of a layer only depend on each other head by head: head h's scores need
// rows h*128.. of wq / wk (and the cached keys of head h), its KQV needs those scores and rows of wv.
// One launch therefore runs all three steps with the 8 workgroups of a head (8 x 16 waves = 128 waves)
// synchronising among themselves instead of returning to the host queue twice:
//   A  wave w of the head: RoPE pair w of q (w < 64) or k (w >= 64) and row w of v   (as wave_gemv_kernel<EPI_QKV>)
//   B  wave w: keys 4u..4u+3, u = w + 128 k, of head h: 64 lanes x 128 bit = 4 keys per load   (as attn_scores_kernel)
//   C  workgroup g: softmax of the head's scores, then V^T rows h*128 + 16 g + wave             (as attn_pv_kernel)
// What one step hands to the next crosses workgroups (and XCDs): it is written with agent-scope atomic
// stores by wave 0 of each workgroup (results pass through LDS), which waits for their completion before
// thread 0 arrives at the head's counter, and read with agent-scope atomic loads after it.  The counters
// only ever count up: the target of barrier i is 8 * (launches of this layer so far + 1), the launch count
// is kept next to them and bumped by workgroup 0 of the head after the last barrier.  Polls are bounded:
// on expiry the error flag of the device state is raised and the workgroup leaves.
// All of a launch's workgroups must be resident (grid <= compute units, one 1024-thread workgroup each).
#ifndef ATL_WAVES
#define ATL_WAVES 16              // waves per workgroup: 16 (one workgroup per compute unit) or 8 (two; measured 8 % slower, also with the second one started late)
#endif
#define ATL_THREADS (ATL_WAVES * 64)
#define ATL_GPH (128 / ATL_WAVES)  // workgroups per head
#define ATL_NX (1024 / ATL_THREADS)
#define ATL_NS (5120 / ATL_THREADS) // scores per thread of the softmax step (n_ctx <= 5120)
#define ATL_RS 10                 // groups of 4 keys per wave (n_ctx <= 128 * 4 * ATL_RS)
#define ATL_RV 10                 // 128-bit pieces per lane of a V^T row (n_ctx <= 512 * ATL_RV)
#ifndef ATL_DEPTH_K
#define ATL_DEPTH_K 3               // key groups / V^T pieces per wave requested ahead of their use
#endif
#ifndef ATL_DEPTH_V
#define ATL_DEPTH_V 3
#endif
struct attn_layer_args {
    const uint8_t *wq, *wk, *wv;
    const float *x_in, *normw; float eps;
    dev_state *st; const float *rope_cs;
    uint16_t *q16, *kc, *vc;
    float *scores, *attn_out;
    uint32_t *sync;               // per head 3 x 32 words: arrivals of barrier 1, of barrier 2, launches so far
    int d, n_head, n_ctx;
    float scale; uint32_t spin_limit;
#ifdef ATL_STAMPS
    long long *dbg;               // measurement builds only: wall-clock stamps (10 ns units) of workgroups 0 and 100
#endif
};
#ifdef ATL_STAMPS
#define ATL_STAMP(i) do { if (a.dbg && tid == 0) { if (blockIdx.x == 0 || blockIdx.x == 100) a.dbg[(blockIdx.x ? 64 : 0) + (i)] = wall_clock64(); \
                                                    if ((i) == 0 || (i) == 3 || (i) == 5 || (i) == 8) a.dbg[128 + blockIdx.x * 8 + ((i) == 0 ? 0 : (i) == 3 ? 1 : (i) == 5 ? 2 : 3)] = wall_clock64(); \
                                                    if ((i) == 0) { a.dbg[128 + blockIdx.x * 8 + 4] = __builtin_amdgcn_s_getreg((31 << 11) | 4); a.dbg[128 + blockIdx.x * 8 + 5] = __builtin_amdgcn_s_getreg((31 << 11) | 20); } } } while (0)
#else
#define ATL_STAMP(i) do { } while (0)
#endif

template <int WT, int WTV>        // types of wq / wk and of wv
__global__ __launch_bounds__(ATL_THREADS, 4) void attn_layer_kernel(attn_layer_args a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[16];
    __shared__ int s_ok;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = blockIdx.x / ATL_GPH, g = blockIdx.x % ATL_GPH, w = g * ATL_WAVES + wave;      // w: wave of the head, 0..127
    const int d = a.d, npair = d / 64, n_ctx = a.n_ctx;
    const size_t RB = (size_t)spy_row_size(WT, d);
    const int pos = a.st->pos, n_kv = pos + 1;
    uint32_t *sync = a.sync + (size_t)h * 96;
    // the launch count was written by the previous launch: an ordinary (scalar) load sees it, and stays out of
    // the vector-memory queue in which the first activation loads would otherwise wait behind it
    const uint32_t epoch = sync[64] + 1u;                            // number of this launch (per head), never 0
    const uint32_t target = (uint32_t)ATL_GPH * epoch;
    // q and the new K row of the head travel from the workgroups that compute them to those that use them as 64-bit words
    // {value, epoch}, written and read with single atomic accesses: the value is valid exactly when its epoch is this
    // launch's, so the consumers poll the data itself and no barrier (wait for the stores, counter, poll) sits between
    // the projections and the scores.  128 words per head behind the barrier counters: 0..63 q, 64..127 k (fp16 pairs).
    uint64_t *xch = (uint64_t *)(a.sync + (size_t)a.n_head * 96) + (size_t)h * 128;
    ATL_STAMP(0);

    int8_t *s_q = (int8_t *)smem;
    int2 *s_meta = (int2 *)(smem + staged_q_bytes(d));
    float *s_rope = (float *)(smem + staged_bytes(d));               // 128
    float *s_out = s_rope + 128;                                     // [ATL_WAVES][4 * ATL_RS]
    float *s_t = s_out + ATL_WAVES * 4 * ATL_RS;                     // n_ctx
    uint16_t *s_p = (uint16_t *)(s_t + n_ctx);                       // n_ctx + 8

    // wave 0 writes the workgroup's results, waits for the stores, thread 0 goes through the head's barrier
    auto publish_and_sync = [&](uint32_t *counter, auto writer) -> bool {
        __syncthreads();
        if (wave == 0) {
            writer();
            __builtin_amdgcn_s_waitcnt(0);
            if (lane == 0) {
                __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                uint32_t spins = 0;
                int ok = 1;
                while ((int32_t)(__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - target) < 0) {
                    if (++spins > a.spin_limit) { __hip_atomic_store(&a.st->err, 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); ok = 0; break; }
                    __builtin_amdgcn_s_sleep(1);
                }
                s_ok = ok;
            }
        }
        __syncthreads();
        return s_ok != 0;
    };

    // ================= A: attn_norm, Q/K/V_project of head h, rope, KV-cache copies =================
    // the 1024 float4 of x (d <= 4096) are spread over the workgroup's threads: ATL_NX each, float4 tid + j * ATL_THREADS
    float4 xv[ATL_NX], wv[ATL_NX];
#pragma unroll
    for (int j = 0; j < ATL_NX; j++) {
        const int i4 = min(tid + j * ATL_THREADS, d / 4 - 1);
        xv[j] = ((const float4 *)a.x_in)[i4]; wv[j] = ((const float4 *)a.normw)[i4];
    }
    const float rope_v = a.rope_cs[min(tid, 127)];
    wtile<WT, 1> t[2];
    wtile<WTV, 1> tv;
    const int wp = w & 63;                                           // RoPE pair of the head
    const uint8_t *p0 = (w < 64 ? a.wq : a.wk) + (size_t)(h * 128 + 2 * wp) * RB;
    __builtin_amdgcn_s_barrier();            // x of every wave ahead of every wave's rows in the compute unit's memory queue
    load_tile<WT, 64, 1>(t[0], p0, npair, lane);
    load_tile<WT, 64, 1>(t[1], p0 + RB, npair, lane);
    if (tid < 128) s_rope[tid] = rope_v;
    {
        // sums of squares per 64 float4 (one entry of s_red each), added in the same order whatever the workgroup size
#pragma unroll
        for (int j = 0; j < ATL_NX; j++) {
            float acc = 0.0f;
            if (tid + j * ATL_THREADS < d / 4) { const float4 v = xv[j]; acc = fmaf(v.x, v.x, acc); acc = fmaf(v.y, v.y, acc); acc = fmaf(v.z, v.z, acc); acc = fmaf(v.w, v.w, acc); }
            acc = group_sum<64>(acc);
            if (lane == 0) s_red[wave + j * ATL_WAVES] = acc;
        }
        ATL_STAMP(9);
        __syncthreads();
        ATL_STAMP(10);
        const float sum = (((s_red[0] + s_red[1]) + (s_red[2] + s_red[3])) + ((s_red[4] + s_red[5]) + (s_red[6] + s_red[7]))) +
                          (((s_red[8] + s_red[9]) + (s_red[10] + s_red[11])) + ((s_red[12] + s_red[13]) + (s_red[14] + s_red[15])));
        const float scale = 1.0f / sqrtf(sum / (float)d + a.eps);
#pragma unroll
        for (int j = 0; j < ATL_NX; j++) {
            const int i = tid + j * ATL_THREADS;
            if (i < d / 4) {
                float4 v = xv[j];
                v.x = (v.x * scale) * wv[j].x; v.y = (v.y * scale) * wv[j].y; v.z = (v.z * scale) * wv[j].z; v.w = (v.w * scale) * wv[j].w;
                int2 meta;
                const uint32_t q = quantize_oct(v, meta);
                ((uint32_t *)s_q)[act_dw(i, d >> 6)] = q;
                if ((i & 7) == 0) s_meta[i >> 3] = meta;
            }
        }
        __syncthreads();
    }
    ATL_STAMP(1);
    uint4 kb[ATL_RS];
    auto fetch_k = [&](int k) {                                      // keys 4u..4u+3 of head h, u = w + 128 k
        const int tok = min(4 * (w + 128 * k) + (lane >> 4), n_kv - 1);
        kb[k] = *(const uint4 *)(a.kc + (size_t)tok * d + h * 128 + (lane & 15) * 8);
    };
    {
        staged_act act; act.q = s_q; act.meta = s_meta;
        act_frag<1> af;
        load_act_frag<WT, 1>(af, act, npair, lane);
        float s0 = dot_row_frag<WT, 1>(t[0], af, npair, lane);
        load_tile<WTV, 64, 1>(tv, a.wv + (size_t)(h * 128 + w) * spy_row_size(WTV, d), npair, lane);
        float s1 = dot_row_frag<WT, 1>(t[1], af, npair, lane);
        float s2;
        if constexpr (WTV == WT) s2 = dot_row_frag<WTV, 1>(tv, af, npair, lane);
        else { act_frag<1> av; load_act_frag<WTV, 1>(av, act, npair, lane); s2 = dot_row_frag<WTV, 1>(tv, av, npair, lane); }
        s0 = wave_total_lane63(s0); s1 = wave_total_lane63(s1); s2 = wave_total_lane63(s2);
        if (lane == 63) {
            const float c = s_rope[2 * wp], sn = s_rope[2 * wp + 1];
            // (x0, x1) -> (x0*c - x1*s, x0*s + x1*c) on adjacent rows (non-linear.cpp:359-363)
            s_out[wave * 2] = __uint_as_float((uint32_t)f2h(s0 * c - s1 * sn) | ((uint32_t)f2h(s0 * sn + s1 * c) << 16));
            s_out[wave * 2 + 1] = __uint_as_float((uint32_t)f2h(s2));
        }
        if (wave != 0) {                     // (requesting the keys only after the barrier, behind q, measured 1 us slower)
#pragma unroll
            for (int k = 0; k < ATL_DEPTH_K; k++) fetch_k(k);
        }
    }
    ATL_STAMP(2);
    __syncthreads();
    if (wave == 0 && lane < ATL_WAVES) {
        const int ww = g * ATL_WAVES + lane, pp = ww & 63;
        const uint32_t pr = __float_as_uint(s_out[lane * 2]);
        __hip_atomic_store(xch + ww, ((uint64_t)epoch << 32) | pr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // attn_score rounds Q to fp16 (mat.cpp:37)
        if (ww >= 64) stc((uint32_t *)(a.kc + (size_t)pos * d) + h * 64 + pp, pr);                          // KCache_cpy: [token][head][hd] (for the passes to come)
        stc(a.vc + (size_t)(h * 128 + ww) * n_ctx + pos, (uint16_t)__float_as_uint(s_out[lane * 2 + 1]));   // VCache_cpy: [d][C] column pos (read after the barrier below)
    }
    __syncthreads();                                                 // s_out is written again below
    ATL_STAMP(3);

    // ================= B: t = (K.q) * scale for head h ================================================
    const uint16_t *vrow = a.vc + (size_t)(h * 128 + w) * n_ctx;
    uint4 vb[ATL_RV];
    // pieces past the last cached token re-read the last piece (same cache line: no memory traffic for the unused part of the row)
    auto fetch_v = [&](int i) { vb[i] = *(const uint4 *)(vrow + (size_t)min(i * 64 + lane, (n_kv - 1) >> 3) * 8); };
    {
        // four words of q per lane, polled until all four carry this launch's epoch (bounded: the error flag is set and the
        // pass goes on with what is there)
        uint32_t qw[4];
        {
            const uint64_t *qs = xch + (lane & 15) * 4;
            uint32_t spins = 0;
            for (;;) {
                bool ok = true;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint64_t v = __hip_atomic_load(qs + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    qw[j] = (uint32_t)v; ok = ok && (uint32_t)(v >> 32) == epoch;
                }
                if (__all(ok)) break;
                if (++spins > a.spin_limit) { if (lane == 0) __hip_atomic_store(&a.st->err, 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); break; }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        if (wave == 0) {
#pragma unroll
            for (int k = 0; k < ATL_DEPTH_K; k++) fetch_k(k);
        }
        float qf[8];
#pragma unroll
        for (int j = 0; j < 4; j++) { qf[2 * j] = h2f((uint16_t)(qw[j] & 0xFFFFu)); qf[2 * j + 1] = h2f((uint16_t)(qw[j] >> 16)); }
#pragma unroll
        for (int k = 0; k < ATL_RS; k++) {
            if (k + ATL_DEPTH_K < ATL_RS) fetch_k(k + ATL_DEPTH_K);
            const int tok = 4 * (w + 128 * k) + (lane >> 4);
            uint4 kv = kb[k];
            if (tok == pos) {                                        // computed in step A by another workgroup: taken from the exchange words
                const uint64_t *ks = xch + 64 + (lane & 15) * 4;
                uint32_t kw4[4], spins = 0;
                for (;;) {
                    bool ok = true;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const uint64_t v = __hip_atomic_load(ks + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        kw4[j] = (uint32_t)v; ok = ok && (uint32_t)(v >> 32) == epoch;
                    }
                    if (ok) break;
                    if (++spins > a.spin_limit) { __hip_atomic_store(&a.st->err, 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); break; }
                    __builtin_amdgcn_s_sleep(1);
                }
                kv = make_uint4(kw4[0], kw4[1], kw4[2], kw4[3]);
            }
            const uint32_t kw[4] = {kv.x, kv.y, kv.z, kv.w};
            float s = 0.0f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                s = fmaf(h2f((uint16_t)(kw[j] & 0xFFFFu)), qf[2 * j], s);
                s = fmaf(h2f((uint16_t)(kw[j] >> 16)), qf[2 * j + 1], s);
            }
            s = group_sum<16>(s);
            if ((lane & 15) == 0) s_out[wave * (4 * ATL_RS) + k * 4 + (lane >> 4)] = s * a.scale;
        }
    }
    ATL_STAMP(4);
    if (!publish_and_sync(sync + 32, [&]() {
            for (int idx = lane; idx < ATL_WAVES * 4 * ATL_RS; idx += 64) {
                const int wv_ = idx / (4 * ATL_RS), r = idx - wv_ * (4 * ATL_RS);
                const int tok = 4 * (g * ATL_WAVES + wv_ + 128 * (r >> 2)) + (r & 3);
                if (tok < n_kv) stc(a.scores + (size_t)h * n_ctx + tok, s_out[idx]);
            }
        })) return;
    ATL_STAMP(5);
    if (g == 0 && tid == 0) sync[64] = target / (uint32_t)ATL_GPH;                  // every workgroup of the head has read the old count

    // ================= C: softmax of the head's scores, KQV rows 16 g .. 16 g + 15 ====================
    // m = max t; e = expf(float(fp16(t - m))); p = e * (1/sum e) (non-linear.cpp:158-176); P is rounded
    // to fp16 for the KQV product (mat.cpp:37, vec_dot.h:117-146)
    {
        const float *srow = a.scores + (size_t)h * n_ctx;
        const int n_pad = (n_kv + 7) & ~7;
        float mx = -INFINITY;
        // the head's scores first, for every wave (they are what the softmax waits for), the first V^T pieces behind them; no
        // V^T request before the barrier above: its stores, atomics and polls would wait behind them in the memory queue
        float sreg[ATL_NS];
#pragma unroll
        for (int u = 0; u < ATL_NS; u++) sreg[u] = ldc(srow + min(tid + u * ATL_THREADS, n_ctx - 1));
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int i = 0; i < ATL_DEPTH_V; i++) fetch_v(i);
#pragma unroll
        for (int u = 0; u < ATL_NS; u++) { const int j = tid + u * ATL_THREADS; if (j < n_kv) { s_t[j] = sreg[u]; mx = fmaxf(mx, sreg[u]); } }
        mx = wave_max(mx);
        if (lane == 0) s_red[wave] = mx;
        __syncthreads();
        ATL_STAMP(6);
        mx = s_red[0];
#pragma unroll
        for (int i = 1; i < ATL_WAVES; i++) mx = fmaxf(mx, s_red[i]);
        __syncthreads();
        // partial sums per residue class j mod 1024 (thread tid + c * ATL_THREADS of a 1024-thread workgroup), one entry of
        // s_red per 64 classes: the same additions in the same order whatever the workgroup size
#pragma unroll
        for (int c = 0; c < ATL_NX; c++) {
            float sum = 0.0f;
            for (int j = tid + c * ATL_THREADS; j < n_kv; j += 1024) { const float e = expf(h2f(f2h(s_t[j] - mx))); s_t[j] = e; sum += e; }
            sum = group_sum<64>(sum);
            if (lane == 0) s_red[wave + c * ATL_WAVES] = sum;
        }
        __syncthreads();
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) sum += s_red[i];
        const float inv = 1.0f / sum;
        for (int j = tid; j < n_pad; j += ATL_THREADS) s_p[j] = j < n_kv ? f2h(s_t[j] * inv) : (uint16_t)0;
        __syncthreads();
        ATL_STAMP(7);
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < ATL_RV; i++) {
            if (i + ATL_DEPTH_V < ATL_RV) fetch_v(i + ATL_DEPTH_V);
            const int pc = i * 64 + lane;
            if (pc * 8 < n_kv) {
                const uint4 pp = *(const uint4 *)(s_p + pc * 8);
                const uint32_t vw[4] = {vb[i].x, vb[i].y, vb[i].z, vb[i].w}, pw[4] = {pp.x, pp.y, pp.z, pp.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    // cache slots past n_kv hold whatever was there before: never multiply them in
                    if (pc * 8 + 2 * j < n_kv) acc = fmaf(h2f((uint16_t)(vw[j] & 0xFFFFu)), h2f((uint16_t)(pw[j] & 0xFFFFu)), acc);
                    if (pc * 8 + 2 * j + 1 < n_kv) acc = fmaf(h2f((uint16_t)(vw[j] >> 16)), h2f((uint16_t)(pw[j] >> 16)), acc);
                }
            }
        }
        acc = wave_total_lane63(acc);
        if (lane == 63) a.attn_out[h * 128 + w] = acc;
        ATL_STAMP(8);
    }
}

#ifdef SPY_DECODE_COMMON_KERNELS   // type-independent kernels: compiled by one translation unit only

// ---- token embedding + RoPE table ---------------------------------------------------------------
// GetRow (view.cpp:33-81): F32 copy or Q8_0 dequant.  The cos/sin table of this position follows
// the reference's recurrence: theta_0 = pos, theta_{k+1} = theta_k * theta_scale in fp32
// (non-linear.cpp:304-309), cosf / sinf of it.
__global__ __launch_bounds__(256) void embed_kernel(dev_state *st, const uint8_t *__restrict__ table, int q8, int d, int n_vocab,
                                                    float *__restrict__ x, float *__restrict__ rope_cs, float theta_scale, int hd) {
    int tok = st->token;
    if (tok < 0 || tok >= n_vocab) { if (threadIdx.x == 0) st->err = 1; tok = 0; }
    if (!q8) {
        const float *row = (const float *)table + (size_t)tok * d;
        for (int i = threadIdx.x; i < d; i += 256) x[i] = row[i];
    } else {
        const blk_q8_0 *row = (const blk_q8_0 *)(table + (size_t)tok * (d / 32) * 34);
        for (int i = threadIdx.x; i < d; i += 256) x[i] = (float)row[i >> 5].qs[i & 31] * h2f(row[i >> 5].d);
    }
    for (int k = threadIdx.x; k < hd / 2; k += 256) {
        float theta = (float)st->pos;
        for (int j = 0; j < k; j++) theta *= theta_scale;
        rope_cs[2 * k] = cosf(theta);
        rope_cs[2 * k + 1] = sinf(theta);
    }
}

// ---- attention scores ---------------------------------------------------------------------------
// One workgroup per chunk of ATT_TCH cached tokens, all heads: a (token, head) key is 256 bytes
// = 16 lanes x 128-bit; a thread covers two heads (h and h+16) so that 2*ATT_TCH loads are in
// flight per thread.  t = (K.q + mask) * scale with mask = 0 for every cached token of a
// single-token pass (llama.cpp:248-257), i.e. t = dot * scale.
#define ATT_TCH 8
#ifndef ATT_DEPTH
#define ATT_DEPTH 3             // key loads per thread requested ahead of their use
#endif
__global__ __launch_bounds__(256) void attn_scores_kernel(const dev_state *st, int pos_imm, const uint16_t *__restrict__ q16, const uint16_t *__restrict__ kc,
                                                          float *__restrict__ scores, int n_head, int n_ctx, float scale) {
    const int n_kv = (st ? st->pos : pos_imm) + 1;
    const int t0 = blockIdx.x * ATT_TCH;
    if (t0 >= n_kv) return;
    const int d = n_head * 128;
    const int piece = threadIdx.x & 15, hsel = threadIdx.x >> 4;     // 2 x 16 heads per pass over the workgroup
    for (int h0 = 0; h0 < n_head; h0 += 32) {
        // q first, then the keys with ATT_DEPTH loads per thread ahead of their use; every load
        // unconditional (heads / tokens beyond the range re-read the last one, results not stored)
        uint4 qv[2], kv[2 * ATT_TCH];
#pragma unroll
        for (int hh = 0; hh < 2; hh++) qv[hh] = *(const uint4 *)(q16 + min(h0 + hsel + 16 * hh, n_head - 1) * 128 + piece * 8);
        auto fetch = [&](int idx) {
            const int head = min(h0 + hsel + 16 * (idx / ATT_TCH), n_head - 1), tok = min(t0 + idx % ATT_TCH, n_kv - 1);
            kv[idx] = *(const uint4 *)(kc + (size_t)tok * d + head * 128 + piece * 8);
        };
#pragma unroll
        for (int idx = 0; idx < ATT_DEPTH; idx++) fetch(idx);
        float qf[2][8];
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
            const uint32_t qw[4] = {qv[hh].x, qv[hh].y, qv[hh].z, qv[hh].w};
#pragma unroll
            for (int j = 0; j < 4; j++) { qf[hh][2 * j] = h2f((uint16_t)(qw[j] & 0xFFFFu)); qf[hh][2 * j + 1] = h2f((uint16_t)(qw[j] >> 16)); }
        }
#pragma unroll
        for (int idx = 0; idx < 2 * ATT_TCH; idx++) {
            if (idx + ATT_DEPTH < 2 * ATT_TCH) fetch(idx + ATT_DEPTH);
            const int hh = idx / ATT_TCH, tt = idx % ATT_TCH, head = h0 + hsel + 16 * hh;
            const uint32_t kw[4] = {kv[idx].x, kv[idx].y, kv[idx].z, kv[idx].w};
            float s = 0.0f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                s = fmaf(h2f((uint16_t)(kw[j] & 0xFFFFu)), qf[hh][2 * j], s);
                s = fmaf(h2f((uint16_t)(kw[j] >> 16)), qf[hh][2 * j + 1], s);
            }
            s = group_sum<16>(s);
            if (head < n_head && piece == 0 && t0 + tt < n_kv) scores[(size_t)head * n_ctx + t0 + tt] = s * scale;
        }
    }
}

// ---- softmax + P.V ------------------------------------------------------------------------------
// One 1024-thread workgroup per (head, 16 head dims): wave w owns V^T row head*128 + dgrp*16 + w,
// contiguous along tokens, 64 lanes x 128-bit per step; the first PV_PIECES steps of the row are
// put in flight before the softmax so that the HBM latency hides behind it.  The softmax of the
// head's row is recomputed by each of the 8 workgroups of a head: m = max t;
// e = expf(float(fp16(t - m))); p = e * (1/sum e) (non-linear.cpp:158-176); P is rounded to fp16 for the
// KQV product (mat.cpp:37, vec_dot.h:117-146).
#define PV_THREADS 1024
#define PV_PIECES 10            // 128-bit pieces per lane per chunk: 10*64*8 = 5120 tokens per chunk
#ifndef PV_DEPTH
#define PV_DEPTH 3              // pieces per wave requested ahead of their use
#endif
#define PV_NS 5                 // scores per thread kept in registers (5 * 1024 = 5120 tokens; more are read in a loop)
__global__ __launch_bounds__(PV_THREADS) void attn_pv_kernel(const dev_state *st, int pos_imm, const float *__restrict__ scores, const uint16_t *__restrict__ vc,
                                                             float *__restrict__ attn_out, int n_ctx) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_part[16];
    const int n_kv = (st ? st->pos : pos_imm) + 1;
    const int head = blockIdx.x >> 3, dgrp = blockIdx.x & 7;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int row = head * 128 + dgrp * 16 + wave;
    const uint16_t *vrow = vc + (size_t)row * n_ctx;
    const int n_pad = (n_kv + 7) & ~7, npiece = n_pad >> 3;
    // Loads in the order they are needed and all unconditional (indices clamped into the row): the
    // head's scores first, then the first PV_PIECES steps of the V^T row, so that the softmax below
    // only waits for the scores while the row streams in.
    const float *srow = scores + (size_t)head * n_ctx;
    float sreg[PV_NS];
#pragma unroll
    for (int u = 0; u < PV_NS; u++) sreg[u] = srow[min((int)threadIdx.x + u * PV_THREADS, n_ctx - 1)];
    // only PV_DEPTH pieces per wave ahead of their use (the vector-memory queue of the compute unit is
    // finite: a wave that asks for everything at once sits in the issue stage and delays the barriers below)
    uint4 vv[PV_PIECES];
    auto fetch = [&](int pc0, int u) { vv[u] = *(const uint4 *)(vrow + (size_t)min(pc0 + u * 64 + lane, npiece - 1) * 8); };   // past the last token: the last piece again (no traffic)
#pragma unroll
    for (int u = 0; u < PV_DEPTH; u++) fetch(0, u);

    float *s_t = (float *)smem;                               // n_ctx floats
    uint16_t *s_p = (uint16_t *)(smem + (size_t)n_ctx * 4);    // n_ctx halfs (+ pad)
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < PV_NS; u++) { const int j = threadIdx.x + u * PV_THREADS; if (j < n_kv) { s_t[j] = sreg[u]; mx = fmaxf(mx, sreg[u]); } }
    for (int j = threadIdx.x + PV_NS * PV_THREADS; j < n_kv; j += PV_THREADS) { const float t = srow[j]; s_t[j] = t; mx = fmaxf(mx, t); }
    mx = wave_max(mx);
    if (lane == 0) s_part[wave] = mx;
    __syncthreads();
    mx = s_part[0];
#pragma unroll
    for (int w = 1; w < 16; w++) mx = fmaxf(mx, s_part[w]);
    __syncthreads();
    float sum = 0.0f;
    for (int j = threadIdx.x; j < n_kv; j += PV_THREADS) { const float e = expf(h2f(f2h(s_t[j] - mx))); s_t[j] = e; sum += e; }
    sum = group_sum<64>(sum);
    if (lane == 0) s_part[wave] = sum;
    __syncthreads();
    sum = 0.0f;
#pragma unroll
    for (int w = 0; w < 16; w++) sum += s_part[w];
    const float inv = 1.0f / sum;
    for (int j = threadIdx.x; j < n_pad; j += PV_THREADS) s_p[j] = j < n_kv ? f2h(s_t[j] * inv) : (uint16_t)0;
    __syncthreads();

    float acc = 0.0f;
    auto consume = [&](int pc0) {
#pragma unroll
        for (int u = 0; u < PV_PIECES; u++) {
            if (u + PV_DEPTH < PV_PIECES) fetch(pc0, u + PV_DEPTH);
            const int pc = pc0 + u * 64 + lane;
            if (pc < npiece) {
                const uint4 pp = *(const uint4 *)(s_p + pc * 8);
                const uint32_t vw[4] = {vv[u].x, vv[u].y, vv[u].z, vv[u].w}, pw[4] = {pp.x, pp.y, pp.z, pp.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    // cache slots past n_kv hold whatever was there before: never multiply them in
                    if (pc * 8 + 2 * j < n_kv) acc = fmaf(h2f((uint16_t)(vw[j] & 0xFFFFu)), h2f((uint16_t)(pw[j] & 0xFFFFu)), acc);
                    if (pc * 8 + 2 * j + 1 < n_kv) acc = fmaf(h2f((uint16_t)(vw[j] >> 16)), h2f((uint16_t)(pw[j] >> 16)), acc);
                }
            }
        }
    };
    consume(0);                                                // the pieces requested at the top
    for (int pc0 = PV_PIECES * 64; pc0 < npiece; pc0 += PV_PIECES * 64) {
#pragma unroll
        for (int u = 0; u < PV_DEPTH; u++) fetch(pc0, u);
        consume(pc0);
    }
    acc = group_sum<64>(acc);
    if (lane == 0) attn_out[row] = acc;
}

// ---- greedy sampling + loop advance -------------------------------------------------------------
// argmax with std::max_element's first-maximum rule (greedy.h:20-25), then the loop step of
// AutoModelGenerator::generate (cli.h:121-123): the sampled token becomes the next input at pos+1.
// With `table` != nullptr the kernel goes on to what the next pass starts with: the embedding row of the sampled
// token and the RoPE table of the next position (embed_kernel's work), so that a greedy step is one launch shorter.
__global__ __launch_bounds__(1024) void sample_advance_kernel(dev_state *st, const float *__restrict__ logits, int n, int32_t *__restrict__ tokens_out,
                                                              int max_out, const uint8_t *__restrict__ table, int q8, int d, float *__restrict__ x,
                                                              float *__restrict__ rope_cs, float theta_scale, int hd) {
    __shared__ float s_v[16];
    __shared__ int s_i[16];
    __shared__ int s_next[1];
    float best = -INFINITY;
    int bi = 0x7fffffff;
    const int step = st->step, pos = st->pos + 1;
    // 16 logits per thread requested together (one at a time, the loop is 32 memory round trips long)
    for (int base = 0; base < n; base += 16 * 1024) {
        float v[16];
#pragma unroll
        for (int u = 0; u < 16; u++) v[u] = logits[min(base + (int)threadIdx.x + u * 1024, n - 1)];
#pragma unroll
        for (int u = 0; u < 16; u++) {
            const int i = base + (int)threadIdx.x + u * 1024;
            if (i < n && (v[u] > best || (bi == 0x7fffffff && !(v[u] < best)))) { best = v[u]; bi = i; }
        }
    }
    if (table != nullptr) {
        // the RoPE table of the next position does not depend on the token: computed while the maximum is being reduced
        for (int k = threadIdx.x; k < hd / 2; k += 1024) {
            float theta = (float)pos;
            for (int j = 0; j < k; j++) theta *= theta_scale;
            rope_cs[2 * k] = cosf(theta);
            rope_cs[2 * k + 1] = sinf(theta);
        }
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
        if (bi == 0x7fffffff) bi = 0;
        if (step < max_out) tokens_out[step] = bi;
        st->token = bi;
        st->pos = pos;
        st->step = step + 1;
        s_next[0] = bi;
    }
    if (table == nullptr) return;
    __syncthreads();
    const int tok = s_next[0];                 // an index of the logits: always a valid row
    if (!q8) {
        const float *row = (const float *)table + (size_t)tok * d;
        for (int i = threadIdx.x; i < d; i += 1024) x[i] = row[i];
    } else {
        const blk_q8_0 *row = (const blk_q8_0 *)(table + (size_t)tok * (d / 32) * 34);
        for (int i = threadIdx.x; i < d; i += 1024) x[i] = (float)row[i >> 5].qs[i & 31] * h2f(row[i >> 5].d);
    }
}

#endif  // SPY_DECODE_COMMON_KERNELS
