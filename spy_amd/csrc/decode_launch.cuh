// Launchers of the fused single-token-pass kernels, templated on the layer-weight type; included by
// one translation unit per type.
#pragma once

#include "engine_types.cuh"

#include <math.h>
#include <string.h>

template <int WT, int LPR, int NIT, int SIT, int EPI>
static int launch_fused(spy_hip_llama *m, hipStream_t st, const fused_args &a) {
    constexpr int RPT = GEMV_WAVES * (SPY_WAVE / LPR);
    const size_t lds = staged_bytes(a.K) + (EPI == EPI_QKV ? 4 * (size_t)a.hd : 0);      // + the RoPE cos|sin table
    auto kern = fused_gemv_kernel<WT, LPR, NIT, SIT, EPI>;
    int &cap = m->grid_cap[(const void *)kern];           // workgroups resident at once (persistent grid)
    if (!cap) {
        RC_TRY(spy_ensure_lds(m, (const void *)kern, lds));
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, GEMV_THREADS, lds) != hipSuccess || per_cu < 1) per_cu = 1;
        cap = per_cu * m->num_cu;
    }
    if (m->dry) return 0;
    const int ntiles = (a.M + RPT - 1) / RPT;
    kern<<<dim3((unsigned)(ntiles < cap ? ntiles : cap)), dim3(GEMV_THREADS), lds, st>>>(a);
    return SPY_LAUNCH_RC();
}

// RMSNorm-prologue kernels (K = n_embd): x and the norm weight stay in registers, 4 or 8 float4 each
template <int WT, int EPI>
static int launch_fused_norm(spy_hip_llama *m, hipStream_t st, gemv_cfg cfg, const fused_args &a) {
    int rc = SPY_HIP_EUNSUPPORTED;
    const bool big = a.K > 4096;
    if (a.K > 8192) return rc;
#define CALL(LPR, NIT) rc = big ? launch_fused<WT, LPR, NIT, GEMV_SIT_FOR(8192), EPI>(m, st, a) : launch_fused<WT, LPR, NIT, GEMV_SIT_FOR(4096), EPI>(m, st, a)
    switch (cfg.lpr * 8 + cfg.nit) {
    case 16 * 8 + 1: CALL(16, 1); break; case 16 * 8 + 2: CALL(16, 2); break;
    case 16 * 8 + 3: CALL(16, 3); break; case 16 * 8 + 4: CALL(16, 4); break;
    case 32 * 8 + 3: CALL(32, 3); break; case 32 * 8 + 4: CALL(32, 4); break;
    default: break;
    }
#undef CALL
    return rc;
}

template <int WT>
static int launch_fused_resid(spy_hip_llama *m, hipStream_t st, gemv_cfg cfg, const fused_args &a) {
    int rc = SPY_HIP_EUNSUPPORTED;
    // input registers per thread follow the tile shape: K <= 64 * LPR * NIT
#define CALL(LPR, NIT) rc = launch_fused<WT, LPR, NIT, GEMV_SIT_FOR(64 * LPR * NIT), EPI_RESID>(m, st, a)
    GEMV_DISPATCH_CFG(cfg, CALL)
#undef CALL
    return rc;
}


// ---- one-row-per-wave kernels (K <= 4096 * NITK) ---------------------------------------------------
template <int WT, int NITK, int NR, int EPI, int WTV = WT>
static int launch_wave(spy_hip_llama *m, hipStream_t st, const fused_args &a) {
    const size_t lds = staged_bytes(a.K) + (EPI == EPI_QKV ? 4 * (size_t)a.hd : 0);
    auto kern = wave_gemv_kernel<WT, NITK, NR, EPI, WTV>;
    RC_TRY(spy_ensure_lds(m, (const void *)kern, lds));
    if (m->dry) return 0;
    const int units = EPI == EPI_QKV ? a.d : (EPI == EPI_GATEUP ? a.M / 2 : a.M);       // one per wave and step
    const int grid = (units + WGV_WAVES * NR - 1) / (WGV_WAVES * NR);
    kern<<<dim3((unsigned)grid), dim3(WGV_THREADS), lds, st>>>(a);
    return SPY_LAUNCH_RC();
}
// rows (head) and row pairs (gate|up) per wave.  The kernel keeps a ring of DEPTH + 1 rows in registers; 8 rows per wave give
// 250 workgroups for 32000 rows, one per compute unit.  The wide rows of Q8_0 / Q6_K (17 / 15 dwords per lane) stay at 4:
// with 8 the kernel spills a dozen registers and measured 24.3 instead of 21.5 us (Q6_K), 27.3 instead of 20.8 us (Q8_0).
// gate|up: 3 pairs per wave for every type = 230 workgroups for 11008 pairs, one round over the compute units (2 pairs gave
// 344 workgroups, a second round a third full: Q8_0 22.1 -> 18.7 us).  Dealing the 11008 pairs out over 256 workgroups
// (2 or 3 per wave; the third re-reading a row, skipped, or left out by a second instantiation of the loop) was slower: 682 -> 664 / 620 / 669 tok/s.
// The 230 workgroups already draw what the memory system delivers.
template <int WT> struct wave_rows {
    static constexpr int HEAD = (WT == SPY_HIP_Q4_0 || WT == SPY_HIP_Q4_K) ? 8 : 4;
    static constexpr int GATEUP = 3;
};
static inline int layer_type(const spy_hip_llama *m, int t) { return t ? t : m->desc.wtype; }

template <int WT>
static int launch_wave_resid(spy_hip_llama *m, hipStream_t st, const fused_args &a) {
    switch ((a.K + 4095) / 4096) {
    case 1: return launch_wave<WT, 1, 1, EPI_RESID>(m, st, a);
    case 2: return launch_wave<WT, 2, 1, EPI_RESID>(m, st, a);
    case 3: return launch_wave<WT, 3, 1, EPI_RESID>(m, st, a);
    case 4: if constexpr (WT == SPY_HIP_Q4_0 || WT == SPY_HIP_Q8_0) return launch_wave<WT, 4, 1, EPI_RESID>(m, st, a); else return SPY_HIP_EUNSUPPORTED;
    default: return SPY_HIP_EUNSUPPORTED;
    }
}

// MatMul of ONE f32 activation row (the operator path's single-token products) through the one-row-per-wave kernel: the row is
// quantized to Q8_0 in LDS by the launch itself, nothing is added to the dots.  No engine behind the call.  One row per wave
// up to about one workgroup per compute unit (4096 rows), three rows per wave above (11008 rows: 230 workgroups); matrices
// with more rows than that are left to the caller's two-launch way (SPY_HIP_EUNSUPPORTED).
template <int WT, int NITK, int NR>
static int launch_wave_plain(hipStream_t st, const fused_args &a) {
    const size_t lds = staged_bytes(a.K);
    auto kern = wave_gemv_kernel<WT, NITK, NR, EPI_RESID, WT>;
    RC_TRY(spy_raise_lds_limit((const void *)kern, lds));
    kern<<<dim3((unsigned)((a.M + WGV_WAVES * NR - 1) / (WGV_WAVES * NR))), dim3(WGV_THREADS), lds, st>>>(a);
    return SPY_LAUNCH_RC();
}
template <int WT>
static int wave_plain(hipStream_t st, const void *w, const float *x, float *out, int M, int K) {
    constexpr bool KQ = WT == SPY_HIP_Q4_K || WT == SPY_HIP_Q6_K;
    if (M <= 0 || K <= 0 || K % (KQ ? 256 : 64) != 0) return SPY_HIP_EUNSUPPORTED;
    fused_args a;
    memset(&a, 0, sizeof(a));
    a.W0 = (const uint8_t *)w; a.M = M; a.K = K; a.x_in = x; a.out = out;
    const int nitk = (K + 4095) / 4096;
    if (M <= 320 * WGV_WAVES) {
        switch (nitk) {
        case 1: return launch_wave_plain<WT, 1, 1>(st, a);
        case 2: return launch_wave_plain<WT, 2, 1>(st, a);
        case 3: return launch_wave_plain<WT, 3, 1>(st, a);
        case 4: if constexpr (!KQ) return launch_wave_plain<WT, 4, 1>(st, a); else return SPY_HIP_EUNSUPPORTED;
        default: return SPY_HIP_EUNSUPPORTED;
        }
    }
    if (nitk == 1 && M <= 320 * WGV_WAVES * 3) return launch_wave_plain<WT, 1, 3>(st, a);
    return SPY_HIP_EUNSUPPORTED;
}

// qkv + scores + softmax/KQV of one layer in one launch (head-local barriers)
template <int WT, int WTV>
static int launch_attn_layer_tv(spy_hip_llama *m, hipStream_t st, int il, bool probe) {
    const spy_hip_llama_desc &c = m->desc;
    const spy_hip_llama_layer &L = m->layers[il];
    const size_t lds = staged_bytes(c.n_embd) + 512 + (size_t)ATL_WAVES * 4 * ATL_RS * 4 + (size_t)c.n_ctx * 6 + 16;
    auto kern = attn_layer_kernel<WT, WTV>;
    if (probe || lds > m->lds_set[(const void *)kern]) {
        RC_TRY(spy_ensure_lds(m, (const void *)kern, lds));
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, ATL_THREADS, lds) != hipSuccess) per_cu = 0;
        if (per_cu * m->num_cu < c.n_head * ATL_GPH) return SPY_HIP_EUNSUPPORTED;        // the head barriers need every workgroup resident
    }
    if (probe || m->dry) return 0;
    attn_layer_args a;
    memset(&a, 0, sizeof(a));
    a.wq = (const uint8_t *)L.wq; a.wk = (const uint8_t *)L.wk; a.wv = (const uint8_t *)L.wv;
    a.x_in = m->x; a.normw = (const float *)L.attn_norm; a.eps = c.eps;
    a.st = m->st; a.rope_cs = m->rope_cs; a.q16 = m->q16; a.kc = m->k_cache[il]; a.vc = m->v_cache[il];
    a.scores = m->scores; a.attn_out = m->attn_out; a.sync = m->attn_sync;
    a.d = c.n_embd; a.n_head = c.n_head; a.n_ctx = c.n_ctx;
    a.scale = 1.0f / sqrtf((float)m->hd);                   // SoftmaxParam::scale (attention.cpp:113)
    a.spin_limit = m->spin_limit;
#ifdef ATL_STAMPS
    a.dbg = m->stamp_dbg;
#endif
    kern<<<dim3((unsigned)(c.n_head * ATL_GPH)), dim3(ATL_THREADS), lds, st>>>(a);
    return SPY_LAUNCH_RC();
}

// wq / wk of type WT; wv of the same type or, next to Q4_K, Q6_K
template <int WT>
static int launch_attn_layer(spy_hip_llama *m, hipStream_t st, int il, bool probe) {
    const int tv = layer_type(m, m->layers[il].t_wv);
    if (tv == WT) return launch_attn_layer_tv<WT, WT>(m, st, il, probe);
    if constexpr (WT == SPY_HIP_Q4_K) { if (tv == SPY_HIP_Q6_K) return launch_attn_layer_tv<SPY_HIP_Q4_K, SPY_HIP_Q6_K>(m, st, il, probe); }
    return SPY_HIP_EUNSUPPORTED;
}
template <int WT>
static int launch_wave_qkv(spy_hip_llama *m, hipStream_t st, int il, const fused_args &a) {
    const int tv = layer_type(m, m->layers[il].t_wv);
    if (tv == WT) return launch_wave<WT, 1, 1, EPI_QKV>(m, st, a);
    if constexpr (WT == SPY_HIP_Q4_K) { if (tv == SPY_HIP_Q6_K) return launch_wave<SPY_HIP_Q4_K, 1, 1, EPI_QKV, SPY_HIP_Q6_K>(m, st, a); }
    return SPY_HIP_EUNSUPPORTED;
}

// one kernel of layer il of the single-token pass; WT is the type of the kernel's (first) matrix
template <int WT>
static int enqueue_kernel(spy_hip_llama *m, hipStream_t st, int which, int il) {
    const spy_hip_llama_desc &c = m->desc;
    const int d = c.n_embd, F = c.n_ff, C = c.n_ctx;
    const spy_hip_llama_layer &L = m->layers[il];
    fused_args a;
    memset(&a, 0, sizeof(a));
    a.st = m->st; a.rope_cs = m->rope_cs; a.q16 = m->q16; a.kc = m->k_cache[il]; a.vc = m->v_cache[il];
    a.n_ctx = C; a.d = d; a.hd = m->hd; a.eps = c.eps; a.pos_imm = m->pos_imm; a.q8_dump = m->q8_dump;
    switch (which) {
    case K_QKV:      // attn_norm, attn_norm_linear, Q/K/V_project, rope, KV-cache copies
        a.W0 = (const uint8_t *)L.wq; a.W1 = (const uint8_t *)L.wk; a.W2 = (const uint8_t *)L.wv;
        a.M = 3 * d; a.K = d; a.x_in = m->x; a.normw = L.attn_norm;
        if (m->attn_fused) return launch_attn_layer<WT>(m, st, il, false);
        if (m->wave) return launch_wave_qkv<WT>(m, st, il, a);
        if constexpr (WT == SPY_HIP_Q4_0 || WT == SPY_HIP_Q8_0) return launch_fused_norm<WT, EPI_QKV>(m, st, m->cfg_d, a);
        return SPY_HIP_EUNSUPPORTED;
    case K_WO:       // KQV_linear + ffn_input
        a.W0 = (const uint8_t *)L.wo; a.M = d; a.K = d; a.x_in = m->attn_out; a.resid = m->x; a.out = m->x1;
        if (m->wave) return launch_wave_resid<WT>(m, st, a);
        if constexpr (WT == SPY_HIP_Q4_0 || WT == SPY_HIP_Q8_0) return launch_fused_resid<WT>(m, st, m->cfg_d, a);
        return SPY_HIP_EUNSUPPORTED;
    case K_GATEUP:   // ffn_norm, ffn_up, ffn_gate, silu, ffn_par
        a.W0 = (const uint8_t *)L.w_gate; a.W1 = (const uint8_t *)L.w_up; a.M = 2 * F; a.K = d; a.x_in = m->x1; a.normw = L.ffn_norm; a.out = m->hbuf;
        if (m->wave) return launch_wave<WT, 1, wave_rows<WT>::GATEUP, EPI_GATEUP>(m, st, a);
        if constexpr (WT == SPY_HIP_Q4_0 || WT == SPY_HIP_Q8_0) return launch_fused_norm<WT, EPI_GATEUP>(m, st, m->cfg_d, a);
        return SPY_HIP_EUNSUPPORTED;
    case K_DOWN:     // ffn_down + logit_output (the next layer's input)
        a.W0 = (const uint8_t *)L.w_down; a.M = d; a.K = F; a.x_in = m->hbuf; a.resid = m->x1; a.out = m->x;
        if (m->wave) return launch_wave_resid<WT>(m, st, a);
        if constexpr (WT == SPY_HIP_Q4_0 || WT == SPY_HIP_Q8_0) return launch_fused_resid<WT>(m, st, m->cfg_ff, a);
        return SPY_HIP_EUNSUPPORTED;
    }
    return SPY_HIP_EINVAL;
}

// result_norm, result_linear, output; WT is the type of the output matrix
template <int WT>
static int enqueue_head(spy_hip_llama *m, hipStream_t st) {
    const spy_hip_llama_desc &c = m->desc;
    const int d = c.n_embd;
    fused_args a;
    memset(&a, 0, sizeof(a));
    a.W0 = (const uint8_t *)c.w_out; a.M = c.n_vocab; a.K = d; a.x_in = m->x; a.normw = c.out_norm; a.eps = c.eps; a.out = m->logits; a.q8_dump = m->q8_dump;
    if (m->wave) return launch_wave<WT, 1, wave_rows<WT>::HEAD, EPI_STORE>(m, st, a);
    if constexpr (WT == SPY_HIP_Q4_0 || WT == SPY_HIP_Q8_0) return launch_fused_norm<WT, EPI_STORE>(m, st, m->cfg_d, a);
    // no row kernel for this shape: norm + weight + Q8_0 through the operator kernels
    if (m->dry) return 0;
    spy_hip_tensor tx, tw, txn;
    memset(&tx, 0, sizeof(tx));
    tx.type = SPY_HIP_F32; tx.dim = 1; tx.ne[0] = d; tx.ne[1] = tx.ne[2] = tx.ne[3] = 1; tx.nb[0] = 4; tx.nb[1] = tx.nb[2] = tx.nb[3] = 4 * d;
    tw = tx; txn = tx;
    tx.data = m->x; tw.data = (void *)c.out_norm; txn.data = m->x1;
    RC_TRY(spy_hip_op_norm_rms(st, &tx, &txn, c.eps));
    RC_TRY(spy_hip_op_binary(st, 2, &txn, &tw, &txn));
    RC_TRY(spy_hip_quantize_q8_0(st, m->x1, 4 * d, m->xq_head, 1, d));
    return spy_hip_gemv_q8_0act(st, c.t_out, c.w_out, m->xq_head, m->logits, nullptr, c.n_vocab, d, 1, c.n_vocab);
}

template <int WT>
static int enqueue_any(spy_hip_llama *m, hipStream_t st, int which, int il) {
    return which == K_HEAD ? enqueue_head<WT>(m, st) : enqueue_kernel<WT>(m, st, which, il);
}
