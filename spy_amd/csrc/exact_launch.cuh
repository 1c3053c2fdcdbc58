// Launchers of the exact-order single-token-pass kernels (exact_decode.cuh), templated on the layer-weight type;
// included by one translation unit per type next to decode_launch.cuh.
#pragma once

#include "exact_decode.cuh"
#include "engine_types.cuh"

#include <string.h>

template <int WT, int NITK, int RPS, int NSTEP, int EPI, int WTV = WT>
static int launch_xg(spy_hip_llama *m, hipStream_t st, const xg_args &a, int units) {
    constexpr int NCH = xg_traits<WT>::NCH, NCHV = xg_traits<WTV>::NCH;
    constexpr int rows_max = EPI == EPI_QKV ? 2 : RPS;
    const size_t lds = ((staged_bytes(a.K) + 15) & ~(size_t)15) + (size_t)XG_WAVES * rows_max * xg_slot_floats(NCH > NCHV ? NCH : NCHV) * 4;
    if (lds > 160 * 1024) return SPY_HIP_EUNSUPPORTED;
    auto kern = xgemv_kernel<WT, NITK, RPS, NSTEP, EPI, WTV>;
    RC_TRY(spy_ensure_lds(m, (const void *)kern, lds));
    if (m->dry) return 0;
    const int per_wg = XG_WAVES * (EPI == EPI_QKV ? 1 : (EPI == EPI_GATEUP ? NSTEP : RPS * NSTEP));     // units (QKV: waves, GATEUP: pairs, else rows) per workgroup
    kern<<<dim3((unsigned)((units + per_wg - 1) / per_wg)), dim3(XG_THREADS), lds, st>>>(a);
    return SPY_LAUNCH_RC();
}

// rows per wave of the output head and pairs per wave of gate|up, as wave_rows in decode_launch.cuh
// Q4_0 / Q8_0: 2 rows per wave and step (32 row slots of 4.6 KB fill LDS); K-quant rows have one accumulator and small slots: 4
template <int WT> struct xg_rows {
    static constexpr bool KQ = WT == SPY_HIP_Q4_K || WT == SPY_HIP_Q6_K;
    static constexpr int HEAD_RPS = KQ ? 4 : 2;
    static constexpr int HEAD_STEPS = WT == SPY_HIP_Q4_0 ? 4 : 2;                               // 8 rows per wave (Q8_0: 4: its rows are twice as wide)
    static constexpr int GATEUP_STEPS = 3;
};

template <int WT>
static int xg_resid(spy_hip_llama *m, hipStream_t st, const xg_args &a) {
    switch ((a.K + 4095) / 4096) {
    case 1: return launch_xg<WT, 1, 1, 1, EPI_RESID>(m, st, a, a.M);
    case 2: return launch_xg<WT, 2, 1, 1, EPI_RESID>(m, st, a, a.M);
    case 3: return launch_xg<WT, 3, 1, 1, EPI_RESID>(m, st, a, a.M);
    case 4: if constexpr (WT == SPY_HIP_Q4_0 || WT == SPY_HIP_Q8_0) return launch_xg<WT, 4, 1, 1, EPI_RESID>(m, st, a, a.M); else return SPY_HIP_EUNSUPPORTED;
    default: return SPY_HIP_EUNSUPPORTED;
    }
}

// MatMul of ONE f32 activation row (the operator path's single-token products) through the same two-phase kernel: the row is
// quantized to Q8_0 in LDS as Quantizator<FP32,Q8_0> does, the dots are Dot<W,Q8_0>::exec per row, nothing is added to them.
// No engine behind the call: the LDS limit goes straight to the process-wide record.
template <int WT, int NITK>
static int launch_xg_plain(hipStream_t st, const xg_args &a) {
    constexpr int NCH = xg_traits<WT>::NCH;
    const size_t lds = ((staged_bytes(a.K) + 15) & ~(size_t)15) + (size_t)XG_WAVES * xg_slot_floats(NCH) * 4;
    if (lds > 160 * 1024) return SPY_HIP_EUNSUPPORTED;
    auto kern = xgemv_kernel<WT, NITK, 1, 1, EPI_RESID, WT>;
    RC_TRY(spy_raise_lds_limit((const void *)kern, lds));
    kern<<<dim3((unsigned)((a.M + XG_WAVES - 1) / XG_WAVES)), dim3(XG_THREADS), lds, st>>>(a);
    return SPY_LAUNCH_RC();
}
// the LDS limits of these launches for every row length they take, raised ahead (spy_hip_init): an operator call then finds them
// in the process-wide record and sets no kernel attribute, whatever it runs under
template <int WT, int NITK>
static int xg_plain_prepare_one() {
    constexpr int NCH = xg_traits<WT>::NCH;
    const size_t lds = ((staged_bytes(4096 * NITK) + 15) & ~(size_t)15) + (size_t)XG_WAVES * xg_slot_floats(NCH) * 4;
    return lds > 160 * 1024 ? 0 : spy_raise_lds_limit((const void *)xgemv_kernel<WT, NITK, 1, 1, EPI_RESID, WT>, lds);
}
template <int WT>
static int xg_plain_prepare() {
    RC_TRY((xg_plain_prepare_one<WT, 1>()));
    RC_TRY((xg_plain_prepare_one<WT, 2>()));
    RC_TRY((xg_plain_prepare_one<WT, 3>()));
    if constexpr (WT == SPY_HIP_Q4_0 || WT == SPY_HIP_Q8_0) RC_TRY((xg_plain_prepare_one<WT, 4>()));
    return 0;
}
template <int WT>
static int xg_plain(hipStream_t st, const void *w, const float *x, float *out, int M, int K) {
    constexpr bool KQ = WT == SPY_HIP_Q4_K || WT == SPY_HIP_Q6_K;
    if (M <= 0 || K <= 0 || K % (KQ ? 256 : 128) != 0) return SPY_HIP_EUNSUPPORTED;
    xg_args a;
    memset(&a, 0, sizeof(a));
    a.W0 = (const uint8_t *)w; a.M = M; a.K = K; a.x_in = x; a.out = out;
    switch ((K + 4095) / 4096) {
    case 1: return launch_xg_plain<WT, 1>(st, a);
    case 2: return launch_xg_plain<WT, 2>(st, a);
    case 3: return launch_xg_plain<WT, 3>(st, a);
    case 4: if constexpr (!KQ) return launch_xg_plain<WT, 4>(st, a); else return SPY_HIP_EUNSUPPORTED;
    default: return SPY_HIP_EUNSUPPORTED;
    }
}

// one exact-order kernel of layer il (which: K_QKV, K_WO, K_GATEUP, K_DOWN) or the head (K_HEAD); WT = type of the kernel's (first) matrix
template <int WT>
static int enqueue_exact(spy_hip_llama *m, hipStream_t st, int which, int il) {
    const spy_hip_llama_desc &c = m->desc;
    const int d = c.n_embd, F = c.n_ff;
    xg_args a;
    memset(&a, 0, sizeof(a));
    a.st = m->st; a.rope_tab = m->rope_tab; a.q16 = m->q16; a.lut = m->lut;
    a.n_ctx = c.n_ctx; a.d = d; a.hd = m->hd; a.eps = c.eps; a.q8_dump = m->q8_dump; a.pos_imm = m->pos_imm; a.rope_row0 = m->rope_row0; a.dbg = m->stamp_dbg;
    if (which == K_HEAD) {
        a.W0 = (const uint8_t *)c.w_out; a.M = c.n_vocab; a.K = d; a.x_in = m->x; a.normw = c.out_norm; a.out = m->logits;
        return launch_xg<WT, 1, xg_rows<WT>::HEAD_RPS, xg_rows<WT>::HEAD_STEPS, EPI_STORE>(m, st, a, a.M);
    }
    const spy_hip_llama_layer &L = m->layers[il];
    a.kc = m->k_cache[il]; a.vc = m->v_cache[il];
    switch (which) {
    case K_QKV: {
        a.W0 = (const uint8_t *)L.wq; a.W1 = (const uint8_t *)L.wk; a.W2 = (const uint8_t *)L.wv;
        a.M = d; a.K = d; a.x_in = m->x; a.normw = L.attn_norm;
        const int tv = layer_type(m, L.t_wv);
        if (tv == WT) return launch_xg<WT, 1, 2, 1, EPI_QKV>(m, st, a, d);
        if constexpr (WT == SPY_HIP_Q4_K) { if (tv == SPY_HIP_Q6_K) return launch_xg<SPY_HIP_Q4_K, 1, 2, 1, EPI_QKV, SPY_HIP_Q6_K>(m, st, a, d); }
        return SPY_HIP_EUNSUPPORTED;
    }
    case K_WO:
        a.W0 = (const uint8_t *)L.wo; a.M = d; a.K = d; a.x_in = m->attn_out; a.resid = m->x; a.out = m->x1;
        return xg_resid<WT>(m, st, a);
    case K_GATEUP:
        a.W0 = (const uint8_t *)L.w_gate; a.W1 = (const uint8_t *)L.w_up; a.M = F; a.K = d; a.x_in = m->x1; a.normw = L.ffn_norm; a.out = m->hbuf;
        return launch_xg<WT, 1, 2, xg_rows<WT>::GATEUP_STEPS, EPI_GATEUP>(m, st, a, F);
    case K_DOWN:
        a.W0 = (const uint8_t *)L.w_down; a.M = d; a.K = F; a.x_in = m->hbuf; a.resid = m->x1; a.out = m->x;
        return xg_resid<WT>(m, st, a);
    }
    return SPY_HIP_EINVAL;
}
