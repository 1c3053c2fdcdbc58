// The token loop on the device: one forward pass of the LLaMA graph
// (model/src/llm/model/llama.cpp:86-264 and plugins in the Spy tree) for a single new token as
// six fused kernels per layer, greedy sampling on the device (greedy.h:20-25, cli.h:88-128), the
// whole pass captured once as a HIP graph and replayed per token.  Passes over several tokens
// (prompts) run operator by operator through the spy_hip_op_* entry points, exactly as the graph
// lists them.
#define SPY_DECODE_COMMON_KERNELS
#include "engine_types.cuh"
#include "exact_decode.cuh"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <vector>


static bool fused_ok(const spy_hip_llama *m);
static int probe_attn(spy_hip_llama *m, int il) {
    switch (m->layers[il].t_wq) {
    case SPY_HIP_Q4_0: return spy_probe_attn_layer_q4_0(m, il);
    case SPY_HIP_Q8_0: return spy_probe_attn_layer_q8_0(m, il);
    case SPY_HIP_Q4_K: return spy_probe_attn_layer_q4_k(m, il);
    case SPY_HIP_Q6_K: return spy_probe_attn_layer_q6_k(m, il);
    }
    return SPY_HIP_EUNSUPPORTED;
}
enum { PASS_LOGITS = 0, PASS_GREEDY = 1 };
int spy_exact_on();                              // exact_order.hip
int spy_exact_thread_scope(int on);              // exact_order.hip
int spy_exact_luts(const float **lut);           // exact_order.hip
// summation order of the next single-token pass: the host backend's when the engine is set to it or the library-wide
// exact-order switch is on (and the exact kernels take the model), else this backend's own
static int pass_order(const spy_hip_llama *m) { return (m->exact_ok && (m->order == 1 || spy_exact_on())) ? 1 : 0; }
static int enqueue_pass_any(spy_hip_llama *m, hipStream_t st, int mode);

static int dalloc(spy_hip_llama *m, void **p, size_t bytes, bool zero) {
    HIP_TRY(hipMalloc(p, bytes));
    m->owned.push_back(*p);
    if (zero) HIP_TRY(hipMemset(*p, 0, bytes));
    return 0;
}

extern "C" int spy_hip_llama_destroy(spy_hip_llama *m) {
    if (!m) return 0;
    (void)hipDeviceSynchronize();
    if (m->graph_exec) (void)hipGraphExecDestroy(m->graph_exec);
    if (m->graph_n_exec) (void)hipGraphExecDestroy(m->graph_n_exec);
    if (m->graph_n) (void)hipGraphDestroy(m->graph_n);
    if (m->graph) (void)hipGraphDestroy(m->graph);
    if (m->own_stream) (void)hipStreamDestroy(m->own_stream);
    if (m->ev0) (void)hipEventDestroy(m->ev0);
    if (m->ev1) (void)hipEventDestroy(m->ev1);
    for (void *p : m->owned) (void)hipFree(p);
    if (m->ops_buf) (void)hipFree(m->ops_buf);
    delete m;
    return 0;
}

extern "C" int spy_hip_llama_create(const spy_hip_llama_desc *desc, spy_hip_llama **out) {
    SPY_CHECK_ARG(desc && out && desc->layers);
    *out = nullptr;
    const spy_hip_llama_desc &c = *desc;
    SPY_CHECK_ARG(c.n_layer > 0 && c.n_embd > 0 && c.n_head > 0 && c.n_ff > 0 && c.n_vocab > 0 && c.n_ctx > 0);
    SPY_CHECK_ARG(c.n_embd % c.n_head == 0 && c.n_ctx % 8 == 0 && c.n_embd % 64 == 0 && c.n_ff % 64 == 0);
    SPY_CHECK_ARG(c.tok_embd && c.out_norm && c.w_out);
    auto is_wt = [](int t) { return t == SPY_HIP_Q4_0 || t == SPY_HIP_Q8_0 || t == SPY_HIP_Q4_K || t == SPY_HIP_Q6_K; };
    auto is_kq = [](int t) { return t == SPY_HIP_Q4_K || t == SPY_HIP_Q6_K; };
    if (!is_wt(c.wtype)) return SPY_HIP_EUNSUPPORTED;
    if (c.t_tok_embd != SPY_HIP_F32 && c.t_tok_embd != SPY_HIP_Q8_0) return SPY_HIP_EUNSUPPORTED;     // GetRow (view.cpp:65-77)
    if (c.t_out != SPY_HIP_Q4_0 && c.t_out != SPY_HIP_Q8_0 && c.t_out != SPY_HIP_Q4_K && c.t_out != SPY_HIP_Q6_K) return SPY_HIP_EUNSUPPORTED;
    if ((c.t_out == SPY_HIP_Q4_K || c.t_out == SPY_HIP_Q6_K) && c.n_embd % 256 != 0) return SPY_HIP_EINVAL;
    spy_hip_llama *m = new spy_hip_llama();
    m->desc = c;
    m->layers.assign(c.layers, c.layers + c.n_layer);
    m->desc.layers = m->layers.data();
    m->hd = c.n_embd / c.n_head;
    m->uniform = (c.wtype == SPY_HIP_Q4_0 || c.wtype == SPY_HIP_Q8_0) && c.t_out == c.wtype;
    for (int i = 0; i < c.n_layer; i++) {
        spy_hip_llama_layer &L = m->layers[i];
        if (!L.attn_norm || !L.ffn_norm || !L.wq || !L.wk || !L.wv || !L.wo || !L.w_gate || !L.w_up || !L.w_down) { delete m; return SPY_HIP_EINVAL; }
        int32_t *tt[7] = {&L.t_wq, &L.t_wk, &L.t_wv, &L.t_wo, &L.t_gate, &L.t_up, &L.t_down};
        for (int k = 0; k < 7; k++) {
            if (*tt[k] == 0) *tt[k] = c.wtype;
            if (!is_wt(*tt[k])) { delete m; return SPY_HIP_EUNSUPPORTED; }
            if (is_kq(*tt[k]) && (c.n_embd % 256 != 0 || c.n_ff % 256 != 0)) { delete m; return SPY_HIP_EINVAL; }
            if (*tt[k] != c.wtype) m->uniform = false;
        }
    }
    m->cfg_d  = pick_cfg(c.n_embd, 32);
    m->cfg_ff = pick_cfg(c.n_ff);
    m->wave = wave_ok(m);                   // n_embd > 4096 (uniform Q4_0 / Q8_0 models): the 256-thread tiled kernels
    {
        int dev = 0; hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0) m->num_cu = prop.multiProcessorCount;
    }
    m->theta_scale = powf(c.rope_freq_base, -2.0f / (float)m->hd);      // non-linear.cpp:282, host libm like the reference
    const size_t d = c.n_embd, C = c.n_ctx;
    int rc = 0;
    m->k_cache.resize(c.n_layer); m->v_cache.resize(c.n_layer);
    for (int i = 0; i < c.n_layer && !rc; i++) {
        rc = dalloc(m, (void **)&m->k_cache[i], C * d * 2, true);
        if (!rc) rc = dalloc(m, (void **)&m->v_cache[i], C * d * 2, true);
    }
    if (!rc) rc = dalloc(m, (void **)&m->x, d * 4, true);
    if (!rc) rc = dalloc(m, (void **)&m->x1, d * 4, true);
    if (!rc) rc = dalloc(m, (void **)&m->attn_out, d * 4, true);
    if (!rc) rc = dalloc(m, (void **)&m->hbuf, (size_t)c.n_ff * 4, true);
    if (!rc) rc = dalloc(m, (void **)&m->scores, (size_t)c.n_head * C * 4, true);
    if (!rc) rc = dalloc(m, (void **)&m->logits, (size_t)c.n_vocab * 4, true);
    if (!rc) rc = dalloc(m, (void **)&m->rope_cs, (size_t)m->hd * 4, true);
    if (!rc) rc = dalloc(m, (void **)&m->q16, d * 2, true);
    if (!rc) rc = dalloc(m, (void **)&m->xq_head, (d / 32) * 34, true);
    if (!rc) rc = dalloc(m, (void **)&m->st, sizeof(dev_state), true);
    m->max_out = 1 << 16;
    if (!rc) rc = dalloc(m, (void **)&m->tokens_out, (size_t)m->max_out * 4, true);
    if (!rc) rc = (int)hipEventCreate(&m->ev0);
    if (!rc) rc = (int)hipEventCreate(&m->ev1);
    if (!rc) rc = (int)hipStreamCreateWithFlags(&m->own_stream, hipStreamNonBlocking);
    {   // softmax + P.V keeps one head's scores (f32) and probabilities (f16) in LDS
        const size_t pv_lds = C * 4 + C * 2 + 16;
        if (!rc && pv_lds > 160 * 1024) rc = SPY_HIP_EUNSUPPORTED;
        if (!rc) rc = spy_raise_lds_limit((const void *)attn_pv_kernel, pv_lds);
    }
    if (!rc && fused_ok(m) && m->wave) {   // one launch for the attention part of a layer where its workgroups are all resident (SPY_HIP_ATTN_SPLIT=1: three launches)
        const char *env = getenv("SPY_HIP_ATTN_SPLIT");
        rc = dalloc(m, (void **)&m->attn_sync, (size_t)c.n_head * 96 * 4 + (size_t)c.n_head * 128 * 8, true);   // barrier counters + per head 128 {value, epoch} exchange words
        if (!rc && !(env && env[0] == '1') && m->hd == 128 && c.n_head * 8 <= m->num_cu && c.n_ctx <= 128 * 4 * ATL_RS && c.n_ctx <= 512 * ATL_RV)
        {
            bool ok = true;
            for (int il = 0; il < c.n_layer && ok; il++) ok = probe_attn(m, il) == 0;
            m->attn_fused = ok;
        }
    }
    if (!rc && fused_ok(m)) { m->dry = true; rc = enqueue_pass_any(m, m->own_stream, PASS_GREEDY); m->dry = false; }   // sizes the persistent grids
    // the host backend's summation order: cos / sin of every position from the host's libm (theta_0 = pos, theta_{k+1} =
    // theta_k * theta_scale in fp32, non-linear.cpp:304-309), the exp / silu tables, shapes the kernels take
    if (!rc && fused_ok(m) && m->wave && m->hd == 128 && c.n_embd % 128 == 0 && c.n_ff % 128 == 0 && c.n_ff <= 16384 &&
        c.n_ctx <= 512 * XP_NP && xattn_pv_lds(c.n_ctx) <= 160 * 1024 - 256 && xattn_scores_lds(c.n_head) <= 160 * 1024) {
        std::vector<float> tab((size_t)c.n_ctx * m->hd);
        for (int pos = 0; pos < c.n_ctx; pos++) {
            float theta = (float)pos;
            for (int i0 = 0; i0 < m->hd; i0 += 2) {
                tab[(size_t)pos * m->hd + i0] = cosf(theta);
                tab[(size_t)pos * m->hd + i0 + 1] = sinf(theta);
                theta *= m->theta_scale;
            }
        }
        rc = dalloc(m, (void **)&m->rope_tab, tab.size() * 4, false);
        if (!rc) rc = (int)hipMemcpy(m->rope_tab, tab.data(), tab.size() * 4, hipMemcpyHostToDevice);
        if (!rc) rc = spy_exact_luts(&m->lut);
        if (!rc) rc = spy_ensure_lds(m, (const void *)xattn_pv_kernel<0>, xattn_pv_lds(c.n_ctx));
        if (!rc) rc = spy_ensure_lds(m, (const void *)xattn_scores_kernel<0>, xattn_scores_lds(c.n_head));
        if (!rc) {
            m->exact_ok = true;
            m->order = 1;
            m->dry = true; rc = enqueue_pass_any(m, m->own_stream, PASS_GREEDY); m->dry = false;
            if (rc == SPY_HIP_EUNSUPPORTED) { rc = 0; m->exact_ok = false; m->order = 0; }
            const char *env = getenv("SPY_HIP_ORDER");                       // "own": this backend's own summation order by default
            if (env && env[0] == 'o') m->order = 0;
        }
    }
#if defined(ATL_STAMPS) || defined(XDBG_STAMPS)
    if (!rc && getenv("SPY_HIP_STAMPS")) rc = dalloc(m, (void **)&m->stamp_dbg, (128 + 512 * 8) * sizeof(long long), true);
#endif
    if (rc) { spy_hip_llama_destroy(m); return rc; }
    *out = m;
    return 0;
}

extern "C" int spy_hip_llama_buffer(spy_hip_llama *m, const char *name, int32_t layer, void **ptr, size_t *bytes) {
    SPY_CHECK_ARG(m && name && ptr);
    const size_t d = m->desc.n_embd, C = m->desc.n_ctx;
    void *p = nullptr; size_t n = 0;
    if (!strcmp(name, "k_cache") || !strcmp(name, "v_cache")) {
        SPY_CHECK_ARG(layer >= 0 && layer < m->desc.n_layer);
        p = name[0] == 'k' ? (void *)m->k_cache[layer] : (void *)m->v_cache[layer]; n = C * d * 2;
    } else if (!strcmp(name, "x")) { p = m->x; n = d * 4; }
    else if (!strcmp(name, "logits")) { p = m->logits; n = (size_t)m->desc.n_vocab * 4; }
    else if (!strcmp(name, "scores")) { p = m->scores; n = (size_t)m->desc.n_head * C * 4; }
    else if (!strcmp(name, "attn_out")) { p = m->attn_out; n = d * 4; }
    else if (!strcmp(name, "phase_stamps") && m->stamp_dbg) { p = m->stamp_dbg; n = (128 + 512 * 8) * sizeof(long long); }
    else return SPY_HIP_EINVAL;
    *ptr = p;
    if (bytes) *bytes = n;
    return 0;
}

extern "C" int spy_hip_llama_single_kernel(spy_hip_llama *m) { return m ? ((m->attn_fused && pass_order(m) == 0) ? 2 : 0) : SPY_HIP_EINVAL; }

extern "C" int spy_hip_llama_set_order(spy_hip_llama *m, int32_t order) {
    SPY_CHECK_ARG(m && (order == 0 || order == 1));
    if (order == 1 && !m->exact_ok) return SPY_HIP_EUNSUPPORTED;
    m->order = order;
    return 0;
}
extern "C" int spy_hip_llama_order(spy_hip_llama *m) { return m ? pass_order(m) : SPY_HIP_EINVAL; }

extern "C" int spy_hip_llama_timing(spy_hip_llama *m, float *ms_per_pass, int32_t *n_pass) {
    SPY_CHECK_ARG(m);
    if (ms_per_pass) *ms_per_pass = m->timed_pass ? (float)(m->timed_ms / m->timed_pass) : 0.0f;
    if (n_pass) *n_pass = m->timed_pass;
    m->timed_ms = 0.0; m->timed_pass = 0;
    return 0;
}

static bool fused_ok(const spy_hip_llama *m) {
    // the fused kernels assume 128-wide heads (one key = 16 lanes x 128 bit), row pairs that share a
    // wave in the qkv / gate-up epilogues (<= 32 lanes per row) and n_embd <= 8192
    if (!(m->hd == 128 && (m->cfg_d.lpr == 16 || m->cfg_d.lpr == 32) && m->cfg_ff.lpr != 0 && m->desc.n_embd % 4 == 0 && m->desc.n_embd <= 8192)) return false;
    if (m->uniform) return true;
    // mixed / K-quant layers: only the one-row-per-wave kernels, and the matrices one kernel reads share a type
    if (!m->wave || m->desc.n_ff > 12288) return false;
    for (const spy_hip_llama_layer &L : m->layers) {
        if (L.t_wq != L.t_wk || L.t_gate != L.t_up) return false;
        if (L.t_wv != L.t_wq && !(L.t_wq == SPY_HIP_Q4_K && L.t_wv == SPY_HIP_Q6_K)) return false;
    }
    return true;
}

static int enqueue_one(spy_hip_llama *m, hipStream_t st, int which, int il) {
    const spy_hip_llama_desc &c = m->desc;
    if (pass_order(m) == 1 || (m->dry && m->order == 1)) {      // the host backend's summation order: six launches per layer
        if (which == K_SCORES) {
            if (m->dry) return 0;
            // one workgroup per compute unit; SPY_HIP_SCORES_GRID (tests) forces fewer, so that a workgroup's share of the tokens
            // takes several rounds of XS_TOK, as it would on a part with fewer compute units or a longer cache
            int sgrid = m->num_cu;
            if (const char *e = getenv("SPY_HIP_SCORES_GRID")) { const int v = atoi(e); if (v >= 1 && v <= m->num_cu) sgrid = v; }
            xattn_scores_kernel<0><<<dim3((unsigned)sgrid), dim3(XS_THREADS), xattn_scores_lds(c.n_head), st>>>(
                m->st, m->pos_imm, m->q16, m->k_cache[il], m->scores, c.n_head, c.n_ctx, 1.0f / sqrtf((float)m->hd));   // SoftmaxParam::scale (attention.cpp:113)
            return SPY_LAUNCH_RC();
        }
        if (which == K_PV) {
            if (m->dry) return 0;
            xattn_pv_kernel<0><<<dim3((unsigned)(c.n_head * 8)), dim3(XP_THREADS), xattn_pv_lds(c.n_ctx), st>>>(m->st, m->pos_imm, m->scores, m->v_cache[il], m->attn_out, m->lut, c.n_ctx, m->stamp_dbg);
            return SPY_LAUNCH_RC();
        }
        const spy_hip_llama_layer &Lx = m->layers[which == K_HEAD ? 0 : il];
        const int tx = which == K_QKV ? Lx.t_wq : which == K_WO ? Lx.t_wo : which == K_GATEUP ? Lx.t_gate : which == K_DOWN ? Lx.t_down : c.t_out;
        switch (tx) {
        case SPY_HIP_Q4_0: return spy_enqueue_exact_q4_0(m, st, which, il);
        case SPY_HIP_Q8_0: return spy_enqueue_exact_q8_0(m, st, which, il);
        case SPY_HIP_Q4_K: return spy_enqueue_exact_q4_k(m, st, which, il);
        case SPY_HIP_Q6_K: return spy_enqueue_exact_q6_k(m, st, which, il);
        }
        return SPY_HIP_EUNSUPPORTED;
    }
    if ((which == K_SCORES || which == K_PV) && m->attn_fused) return 0;     // part of the K_QKV launch
    if (which == K_SCORES) {            // attn_score
        if (m->dry) return 0;
        const float scale = 1.0f / sqrtf((float)m->hd);                     // SoftmaxParam::scale (attention.cpp:113)
        attn_scores_kernel<<<dim3((unsigned)((c.n_ctx + ATT_TCH - 1) / ATT_TCH)), dim3(256), 0, st>>>(m->st, m->pos_imm, m->q16, m->k_cache[il], m->scores,
                                                                                                      c.n_head, c.n_ctx, scale);
        return SPY_LAUNCH_RC();
    }
    if (which == K_PV) {                // softmax, KQV (+ permute/contiguous: attn_out is already [hd, H] contiguous)
        if (m->dry) return 0;
        const size_t pv_lds = (size_t)c.n_ctx * 4 + (size_t)c.n_ctx * 2 + 16;
        attn_pv_kernel<<<dim3((unsigned)(c.n_head * 8)), dim3(PV_THREADS), pv_lds, st>>>(m->st, m->pos_imm, m->scores, m->v_cache[il], m->attn_out, c.n_ctx);
        return SPY_LAUNCH_RC();
    }
    // dispatch on the type of the kernel's (first) matrix
    const spy_hip_llama_layer &L = m->layers[which == K_HEAD ? 0 : il];
    const int t = which == K_QKV ? L.t_wq : which == K_WO ? L.t_wo : which == K_GATEUP ? L.t_gate : which == K_DOWN ? L.t_down : c.t_out;
    switch (t) {
    case SPY_HIP_Q4_0: return spy_enqueue_kernel_q4_0(m, st, which, il);
    case SPY_HIP_Q8_0: return spy_enqueue_kernel_q8_0(m, st, which, il);
    case SPY_HIP_Q4_K: return spy_enqueue_kernel_q4_k(m, st, which, il);
    case SPY_HIP_Q6_K: return spy_enqueue_kernel_q6_k(m, st, which, il);
    }
    return SPY_HIP_EUNSUPPORTED;
}

// After a pass: the device state's error word.  1 = a token id outside the vocabulary; 2, 3 = a bounded wait between
// workgroups expired, the pass went on with what was there and its results are void.  The head barriers' arrival counters
// and exchange words are then in an unknown state: they are cleared (fill kernel, stream order) so that the next pass starts
// from launch number 1 with no stale word carrying a valid-looking number.
__global__ __launch_bounds__(256) void fill_words_kernel(uint32_t *p, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0u;
}
static int check_pass_error(spy_hip_llama *m, hipStream_t st) {
    dev_state back;
    HIP_TRY(hipMemcpyAsync(&back, m->st, sizeof(back), hipMemcpyDeviceToHost, st));
    HIP_TRY(hipStreamSynchronize(st));
    if (!back.err) return 0;
    if (back.err != 1 && m->attn_sync) {
        const size_t words = ((size_t)m->desc.n_head * 96 * 4 + (size_t)m->desc.n_head * 128 * 8) / 4;
        fill_words_kernel<<<dim3((unsigned)((words + 255) / 256)), dim3(256), 0, st>>>(m->attn_sync, words);
        HIP_TRY(hipGetLastError());
        HIP_TRY(hipStreamSynchronize(st));
    }
    return back.err == 1 ? SPY_HIP_EINVAL : SPY_HIP_ETIMEOUT;
}

extern "C" int spy_hip_llama_set_spin_limit(spy_hip_llama *m, uint32_t polls) {
    SPY_CHECK_ARG(m);
    m->spin_limit = polls;
    // captured graphs carry the old limit in their kernel arguments
    if (m->graph_exec) { (void)hipGraphExecDestroy(m->graph_exec); m->graph_exec = nullptr; }
    if (m->graph_n_exec) { (void)hipGraphExecDestroy(m->graph_n_exec); m->graph_n_exec = nullptr; }
    return 0;
}

static int enqueue_embed(spy_hip_llama *m, hipStream_t st) {
    const spy_hip_llama_desc &c = m->desc;
    embed_kernel<<<dim3(1), dim3(256), 0, st>>>(m->st, (const uint8_t *)c.tok_embd, c.t_tok_embd == SPY_HIP_Q8_0, c.n_embd, c.n_vocab, m->x,
                                                m->rope_cs, m->theta_scale, m->hd);
    return SPY_LAUNCH_RC();
}

// One single-token pass.  PASS_LOGITS: embedding, layers, head (spy_hip_llama_forward).  PASS_GREEDY: layers, head, and one
// launch that samples, advances the position and prepares the next pass's embedding and RoPE table -- the first pass of a
// greedy run is preceded by enqueue_embed.
static int enqueue_pass_any(spy_hip_llama *m, hipStream_t st, int mode) {
    const spy_hip_llama_desc &c = m->desc;
    auto sample = [&](bool embed_next) {
        sample_advance_kernel<<<dim3(1), dim3(1024), 0, st>>>(m->st, m->logits, c.n_vocab, m->tokens_out, m->max_out,
                                                              embed_next ? (const uint8_t *)c.tok_embd : nullptr, c.t_tok_embd == SPY_HIP_Q8_0, c.n_embd,
                                                              m->x, m->rope_cs, m->theta_scale, m->hd);
        return SPY_LAUNCH_RC();
    };
    if (mode == PASS_LOGITS && !m->dry) RC_TRY(enqueue_embed(m, st));
    for (int il = 0; il < c.n_layer; il++)
        for (int k = K_QKV; k <= K_DOWN; k++) RC_TRY(enqueue_one(m, st, k, il));
    RC_TRY(enqueue_one(m, st, K_HEAD, 0));
    if (mode == PASS_GREEDY && !m->dry) RC_TRY(sample(true));
    return 0;
}

// ---- passes over several tokens: operator by operator --------------------------------------------
static spy_hip_tensor T2(int type, void *p, int64_t e0, int64_t e1) {
    spy_hip_tensor t;
    t.type = type; t.dim = 2; t.data = p;
    t.ne[0] = e0; t.ne[1] = e1; t.ne[2] = 1; t.ne[3] = 1;
    t.nb[0] = spy_type_size(type); t.nb[1] = spy_row_size(type, e0); t.nb[2] = t.nb[1] * e1; t.nb[3] = t.nb[2];
    return t;
}
static spy_hip_tensor T3s(int type, void *p, int64_t e0, int64_t e1, int64_t e2, int64_t b0, int64_t b1, int64_t b2) {
    spy_hip_tensor t;
    t.type = type; t.dim = 3; t.data = p;
    t.ne[0] = e0; t.ne[1] = e1; t.ne[2] = e2; t.ne[3] = 1;
    t.nb[0] = b0; t.nb[1] = b1; t.nb[2] = b2; t.nb[3] = e2 * b2;
    return t;
}

int spy_matmul_causal(void *stream, const spy_hip_tensor *w, const spy_hip_tensor *x, const spy_hip_tensor *dst, void *scratch, size_t scratch_bytes,
                      int which, int past);                                                                                  // ops.hip
int spy_norm_mul_q8_launch(hipStream_t st, const float *x, int64_t x_stride, const float *w, float eps, void *y, int64_t nrow, int64_t K);   // prompt_fused.hip
int spy_silu_mul_q8_launch(hipStream_t st, const float *gate, const float *up, void *y, int64_t nrow, int64_t F);                           // prompt_fused.hip
int spy_rope_table_launch(hipStream_t st, float *table, int past, int T, int hd, float freq_base, float freq_scale, float mscale);       // prompt_fused.hip
int spy_rope_store_launch(hipStream_t st, const float *q, const float *k, const float *table, uint16_t *q16, uint16_t *kc, int T, int H, int hd);
int spy_vt_store_launch(hipStream_t st, const float *v, uint16_t *vc, int T, int d, int64_t n_ctx);
int spy_prompt_attn_launch(hipStream_t st, const uint16_t *q16, const uint16_t *k_cache, const uint16_t *v_cache, float *out,
                           int T, int H, int hd, int past, int64_t n_ctx, float scale);                                       // prompt_attn.hip
int spy_gemm_q8act_pair(hipStream_t st, int wtype, const void *w1, const void *w2, const void *xq, float *dst1, float *dst2,
                        int64_t M, int64_t K, int64_t T, int64_t dst_stride);                                                  // gemm.hip
int spy_softmax_causal_launch(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *dst, float scale, int n_past);   // ops.hip
int spy_exact_on();                                                                                                          // exact_order.hip
int spy_softmax_row_ok(int64_t ne0);                                                                                         // ops.hip
int64_t spy_exact_prompt_attn_row(int64_t n_kv);                                                                             // exact_prompt.hip
size_t spy_exact_pack_bytes(int64_t ne01, int64_t ne00, int64_t ne11);                                                           // exact_order.hip
int spy_exact_prompt_attn(hipStream_t st, const float *q, const uint16_t *kc, const uint16_t *vt, float *S, uint16_t *P16, float *out, const float *lut,
                          int T, int H, int P, int64_t C, int n_total, float scale);                                        // exact_prompt.hip

// KQ mask of a pass over tokens P .. P + T - 1 (llama.cpp:248-263): row i allows the cached positions j <= P + i
__global__ __launch_bounds__(256) void causal_mask_kernel(float *__restrict__ mask, int C, int P) {
    const int j = blockIdx.x * 256 + threadIdx.x, i = blockIdx.y;
    if (j < C) mask[(size_t)i * C + j] = (j <= i + P) ? 0.0f : -INFINITY;
}

#ifndef SPY_PREFILL_CHUNK
#define SPY_PREFILL_CHUNK 2048        // tokens per operator-by-operator pass of a long prompt (4096-token prompt: 0.33 s with 512, 0.27 with 1024, 0.24 with 2048, 0.25 with 4096)
#endif
enum { HEAD_ALL = 0, HEAD_NONE = 1, HEAD_LAST = 2 };     // output head of a pass: every token's logits (the reference's graph), none, the last token's
// n_total: the cached positions after the whole call this pass belongs to (= P + T unless the call is cut into chunks)
static bool exact_attn_ok(const spy_hip_llama *m) {
    const char *e = getenv("SPY_HIP_EXACT_PROMPT_ATTN");
    return m->hd == 128 && m->desc.n_ctx % 32 == 0 && m->desc.n_ctx <= 8192 && m->lut && !(e && e[0] == '0');
}
static int forward_ops(spy_hip_llama *m, hipStream_t st, const int32_t *tokens_host, int T, int P, float *logits_host, int head, int n_total) {
    const spy_hip_llama_desc &c = m->desc;
    const int64_t d = c.n_embd, F = c.n_ff, C = c.n_ctx, H = c.n_head, hd = m->hd, V = c.n_vocab, n_kv = (int64_t)P + T;
    // Passes over many tokens (every MatMul on the matrix cores): the elementwise operators between two MatMuls write the
    // next MatMul's Q8_0 activations directly (same bytes as the separate operators: prompt_fused.hip)
    // exact-order mode (spy_hip_set_exact_order): the plain operators only, each in its exact form
    const bool exact = spy_exact_on() != 0;
    const bool fuse_act = !exact && T >= 16 && d % 64 == 0 && F % 64 == 0;
    // ... and the attention of a layer is one kernel (prompt_attn.hip) where its shape conditions hold;
    // SPY_HIP_PROMPT_ATTN=0: attention as MatMul -> Softmax -> MatMul (bit-identical to the operator path)
    const char *pa_env = getenv("SPY_HIP_PROMPT_ATTN");
    const bool fuse_attn = fuse_act && hd == 128 && C % 8 == 0 && C >= 64 && !(pa_env && pa_env[0] == '0');
    // scratch layout (bytes); the score / probability matrices and the mask exist only without the attention kernel,
    // the logits of every row only when they were asked for
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += (bytes + 255) & ~(size_t)255; return o; };
    // exact order with heads of 128: the three attention kernels of exact_prompt.hip (same bits as the operators, masked part left out)
    const bool xattn = exact && exact_attn_ok(m);
    const size_t sp_bytes = fuse_attn ? 0 : xattn ? (size_t)spy_exact_prompt_attn_row(n_kv) * T * H * 4 : (size_t)n_kv * T * H * 4;
    const size_t o_x = take(d * T * 4), o_xn = take(d * T * 4), o_q = take(d * T * 4), o_k = take(d * T * 4), o_v = take(d * T * 4),
                 o_o = take(d * T * 4), o_o2 = take(d * T * 4), o_t1 = take(d * T * 4), o_up = take(F * T * 4), o_gate = take(F * T * 4),
                 o_par = take(F * T * 4), o_S = take(sp_bytes), o_P = take(sp_bytes), o_mask = take(fuse_attn || xattn ? 0 : C * T * 4),
                 o_ids = take(T * 4), o_pos = take(T * 4), o_logits = take(head == HEAD_ALL ? V * T * 4 : V * 4), o_rt = take(T * hd * 4);
    const size_t act_q8 = (size_t)T * ((F > d ? F : d) / 32) * 34;
    const size_t act_f16 = sp_bytes / 2 > (size_t)d * T * 2 ? sp_bytes / 2 : (size_t)d * T * 2;
    // exact order: room behind the activations for the packed fp16 operands of the largest MatMul (spy_exact_pack_bytes)
    size_t pack = 0;
    if (exact && T >= 16) {
        const int64_t shapes[3][2] = {{d, d}, {F, d}, {d, F}};
        for (auto &sh : shapes) { const size_t b = spy_exact_pack_bytes(sh[0], sh[1], T); pack = b > pack ? b : pack; }
    }
    const size_t o_scr = take((act_q8 > act_f16 ? act_q8 : act_f16) + 256 + pack);
    const size_t scr_bytes = off - o_scr;
    if (off > m->ops_bytes) {
        if (m->ops_buf) { HIP_TRY(hipStreamSynchronize(st)); HIP_TRY(hipFree(m->ops_buf)); m->ops_buf = nullptr; m->ops_bytes = 0; }
        HIP_TRY(hipMalloc((void **)&m->ops_buf, off));
        m->ops_bytes = off;
    }
    uint8_t *B = m->ops_buf;
    float *x = (float *)(B + o_x), *xn = (float *)(B + o_xn), *q = (float *)(B + o_q), *k = (float *)(B + o_k), *v = (float *)(B + o_v),
          *o = (float *)(B + o_o), *o2 = (float *)(B + o_o2), *t1 = (float *)(B + o_t1), *up = (float *)(B + o_up), *gate = (float *)(B + o_gate),
          *par = (float *)(B + o_par), *S = (float *)(B + o_S), *Pm = (float *)(B + o_P), *mask = (float *)(B + o_mask), *lg = (float *)(B + o_logits);
    int32_t *ids = (int32_t *)(B + o_ids), *pos = (int32_t *)(B + o_pos);
    void *scr = B + o_scr;

    // IO tensors: ids, positions, KQ mask (llama.cpp:248-263)
    {
        std::vector<int32_t> hp(T);
        for (int i = 0; i < T; i++) hp[i] = P + i;
        HIP_TRY(hipMemcpyAsync(ids, tokens_host, (size_t)T * 4, hipMemcpyHostToDevice, st));
        HIP_TRY(hipMemcpyAsync(pos, hp.data(), (size_t)T * 4, hipMemcpyHostToDevice, st));
        if (!fuse_attn && !xattn) {
            causal_mask_kernel<<<dim3((unsigned)((C + 255) / 256), (unsigned)T), dim3(256), 0, st>>>(mask, (int)C, P);   // filled on the device: 35 MB per 2048-token chunk
            HIP_TRY(hipGetLastError());
        }
        HIP_TRY(hipStreamSynchronize(st));
    }
    spy_hip_tensor t_ids = T2(SPY_HIP_I32, ids, T, 1), t_pos = t_ids, t_mask = T2(SPY_HIP_I32, mask, C, T);
    t_ids.dim = 1; t_pos.dim = 1; t_pos.data = pos;
    spy_hip_tensor t_x = T2(SPY_HIP_F32, x, d, T), t_xn = T2(SPY_HIP_F32, xn, d, T), t_q = T2(SPY_HIP_F32, q, d, T), t_k = T2(SPY_HIP_F32, k, d, T),
                   t_v = T2(SPY_HIP_F32, v, d, T), t_o2 = T2(SPY_HIP_F32, o2, d, T), t_t1 = T2(SPY_HIP_F32, t1, d, T), t_od = T2(SPY_HIP_F32, o, d, T);
    spy_hip_tensor t_up = T2(SPY_HIP_F32, up, F, T), t_gate = T2(SPY_HIP_F32, gate, F, T), t_par = T2(SPY_HIP_F32, par, F, T);
    { spy_hip_tensor te = T2(c.t_tok_embd, (void *)c.tok_embd, d, V); RC_TRY(spy_hip_op_get_row(st, &te, &t_ids, &t_x)); }
    spy_hip_rope_param rp;
    memset(&rp, 0, sizeof(rp));
    rp.mode = 0; rp.num_past = P; rp.num_dim = (int32_t)hd; rp.num_context = (int32_t)C; rp.num_origin_context = (int32_t)C;
    rp.freq_base = c.rope_freq_base; rp.freq_scale = 1.0f; rp.attention_factor = 1.0f; rp.beta_fast = 32.0f; rp.beta_slow = 1.0f;
    const float scale = 1.0f / sqrtf((float)hd);
    auto mm = [&](const void *w, int wt, int64_t K, int64_t M, spy_hip_tensor *xin, spy_hip_tensor *out) {
        spy_hip_tensor tw = T2(wt, (void *)w, K, M);
        return spy_hip_op_matmul(st, &tw, xin, out, scr, scr_bytes);
    };
    float *rope_tab = (float *)(B + o_rt);
    if (fuse_act) RC_TRY(spy_rope_table_launch(st, rope_tab, P, T, (int)hd, rp.freq_base, rp.freq_scale, rp.attention_factor));
    for (int il = 0; il < c.n_layer; il++) {
        const spy_hip_llama_layer &L = m->layers[il];
        spy_hip_tensor t_nw = T2(SPY_HIP_F32, (void *)L.attn_norm, d, 1); t_nw.dim = 1;
        if (fuse_act) {           // NormRMS -> Mul -> Q8_0 in one kernel, quantized once for the three MatMuls
            RC_TRY(spy_norm_mul_q8_launch(st, x, 4 * d, (const float *)L.attn_norm, c.eps, scr, T, d));
            RC_TRY(spy_hip_gemm_q8_0act(st, L.t_wq, L.wq, scr, q, d, d, T, d));
            RC_TRY(spy_hip_gemm_q8_0act(st, L.t_wk, L.wk, scr, k, d, d, T, d));
            RC_TRY(spy_hip_gemm_q8_0act(st, L.t_wv, L.wv, scr, v, d, d, T, d));
        } else {
            RC_TRY(spy_hip_op_norm_rms(st, &t_x, &t_xn, c.eps));
            RC_TRY(spy_hip_op_binary(st, 2, &t_xn, &t_nw, &t_xn));
            RC_TRY(mm(L.wq, L.t_wq, d, d, &t_xn, &t_q));
            RC_TRY(mm(L.wk, L.t_wk, d, d, &t_xn, &t_k));
            RC_TRY(mm(L.wv, L.t_wv, d, d, &t_xn, &t_v));
        }
        spy_hip_tensor t_qp;
        if (fuse_act) {           // Rope(q), Rope(k), the fp16 conversion of q and both cache writes in two kernels (prompt_fused.hip)
            RC_TRY(spy_rope_store_launch(st, q, k, rope_tab, (uint16_t *)xn, (uint16_t *)m->k_cache[il] + d * P, T, (int)H, (int)hd));
            RC_TRY(spy_vt_store_launch(st, v, (uint16_t *)m->v_cache[il] + P, T, (int)d, C));
            t_qp = T3s(SPY_HIP_F16, xn, hd, T, H, 2, 2 * hd, 2 * hd * T);
        } else {
            spy_hip_tensor t_q3 = T3s(SPY_HIP_F32, q, hd, H, T, 4, 4 * hd, 4 * d), t_k3 = T3s(SPY_HIP_F32, k, hd, H, T, 4, 4 * hd, 4 * d);
            RC_TRY(spy_hip_op_rope(st, &t_q3, &t_pos, &t_q3, &rp));
            RC_TRY(spy_hip_op_rope(st, &t_k3, &t_pos, &t_k3, &rp));
            t_qp = T3s(SPY_HIP_F32, q, hd, T, H, 4, 4 * d, 4 * hd);                                        // Permute {0,2,1,3}
            spy_hip_tensor t_vt = T2(SPY_HIP_F32, v, T, d); t_vt.nb[0] = 4 * d; t_vt.nb[1] = 4; t_vt.nb[2] = t_vt.nb[3] = 4 * d * T;   // Transpose
            spy_hip_tensor t_kc = T2(SPY_HIP_F16, (uint8_t *)m->k_cache[il] + 2 * d * P, (int64_t)T * d, 1); t_kc.dim = 1;
            RC_TRY(spy_hip_op_dup(st, &t_k3, &t_kc));
            spy_hip_tensor t_vc = T2(SPY_HIP_F16, (uint8_t *)m->v_cache[il] + 2 * (int64_t)P, T, d);
            t_vc.nb[0] = 2; t_vc.nb[1] = 2 * C; t_vc.nb[2] = t_vc.nb[3] = d * 2 * C;
            RC_TRY(spy_hip_op_dup(st, &t_vt, &t_vc));
        }
        if (fuse_attn) {          // scores, masked softmax and the product with V^T in one kernel: no score / probability matrix in memory
            RC_TRY(spy_prompt_attn_launch(st, (const uint16_t *)xn, (const uint16_t *)m->k_cache[il], (const uint16_t *)m->v_cache[il], o2,
                                          T, (int)H, (int)hd, P, C, scale));
        } else if (xattn) {
            RC_TRY(spy_exact_prompt_attn(st, q, (const uint16_t *)m->k_cache[il], (const uint16_t *)m->v_cache[il], S, (uint16_t *)Pm, o2, m->lut,
                                         T, (int)H, P, C, n_total, scale));
        } else {
        spy_hip_tensor t_kall = T3s(SPY_HIP_F16, m->k_cache[il], hd, n_kv, H, 2, 2 * d, 2 * hd);
        spy_hip_tensor t_vall = T3s(SPY_HIP_F16, m->v_cache[il], n_kv, hd, H, 2, 2 * C, 2 * C * hd);
        // causal_ok: the softmax below takes the row kernel, which reads no score beyond a row's causal length and writes
        // zeros there: the two products may then leave out what the mask removes
        const bool causal_ok = !exact && spy_softmax_row_ok(n_kv) != 0;
        // the probabilities go to the KQV product as fp16 (its first step, mat.cpp:37): the softmax writes them that way
        // directly where the fp16 GEMM takes them (rows of a multiple of 8 elements)
        const bool p16 = n_kv % 8 == 0 && causal_ok && T >= 16;
        spy_hip_tensor t_S = T3s(SPY_HIP_F32, S, n_kv, T, H, 4, 4 * n_kv, 4 * n_kv * T);
        spy_hip_tensor t_P = p16 ? T3s(SPY_HIP_F16, Pm, n_kv, T, H, 2, 2 * n_kv, 2 * n_kv * T) : T3s(SPY_HIP_F32, Pm, n_kv, T, H, 4, 4 * n_kv, 4 * n_kv * T);
        RC_TRY(causal_ok ? spy_matmul_causal(st, &t_kall, &t_qp, &t_S, scr, scr_bytes, 0, P) : spy_hip_op_matmul(st, &t_kall, &t_qp, &t_S, scr, scr_bytes));
        // the mask of this pass is the causal one filled above: the row kernel takes its shape as a number
        RC_TRY(causal_ok ? spy_softmax_causal_launch(st, &t_S, &t_P, scale, P) : spy_hip_op_softmax(st, &t_S, &t_mask, &t_P, scale));
        // fused: the product writes [hd, T, H] through the strides of the permuted view, i.e. straight into the contiguous
        // [hd, H, T] buffer the next MatMul reads (Permute {0,2,1,3} + Contiguous without a copy)
        spy_hip_tensor t_O = fuse_act ? T3s(SPY_HIP_F32, o2, hd, T, H, 4, 4 * d, 4 * hd) : T3s(SPY_HIP_F32, o, hd, T, H, 4, 4 * hd, 4 * hd * T);
        RC_TRY(causal_ok ? spy_matmul_causal(st, &t_vall, &t_P, &t_O, scr, scr_bytes, 1, P) : spy_hip_op_matmul(st, &t_vall, &t_P, &t_O, scr, scr_bytes));
        if (!fuse_act) {
            spy_hip_tensor t_Op = T3s(SPY_HIP_F32, o, hd, H, T, 4, 4 * hd * T, 4 * hd);                // Permute {0,2,1,3}
            spy_hip_tensor t_o2c = T3s(SPY_HIP_F32, o2, hd, H, T, 4, 4 * hd, 4 * d);
            RC_TRY(spy_hip_op_contiguous(st, &t_Op, &t_o2c));
        }
        }
        RC_TRY(mm(L.wo, L.t_wo, d, d, &t_o2, &t_t1));
        RC_TRY(spy_hip_op_binary(st, 0, &t_t1, &t_x, &t_t1));
        t_nw.data = (void *)L.ffn_norm;
        if (fuse_act) {
            RC_TRY(spy_norm_mul_q8_launch(st, t1, 4 * d, (const float *)L.ffn_norm, c.eps, scr, T, d));
            if (L.t_up == L.t_gate) RC_TRY(spy_gemm_q8act_pair(st, L.t_up, L.w_up, L.w_gate, scr, up, gate, F, d, T, F));   // one grid for both
            else {
                RC_TRY(spy_hip_gemm_q8_0act(st, L.t_up, L.w_up, scr, up, F, d, T, F));
                RC_TRY(spy_hip_gemm_q8_0act(st, L.t_gate, L.w_gate, scr, gate, F, d, T, F));
            }
            RC_TRY(spy_silu_mul_q8_launch(st, gate, up, scr, T, F));        // Silu -> Mul -> Q8_0
            RC_TRY(spy_hip_gemm_q8_0act(st, L.t_down, L.w_down, scr, o, d, F, T, d));
        } else {
            RC_TRY(spy_hip_op_norm_rms(st, &t_t1, &t_xn, c.eps));
            RC_TRY(spy_hip_op_binary(st, 2, &t_xn, &t_nw, &t_xn));
            RC_TRY(mm(L.w_up, L.t_up, d, F, &t_xn, &t_up));
            RC_TRY(mm(L.w_gate, L.t_gate, d, F, &t_xn, &t_gate));
            RC_TRY(spy_hip_op_silu(st, &t_gate, &t_gate));
            RC_TRY(spy_hip_op_binary(st, 2, &t_up, &t_gate, &t_par));
            RC_TRY(mm(L.w_down, L.t_down, F, d, &t_par, &t_od));
        }
        RC_TRY(spy_hip_op_binary(st, 0, &t_t1, &t_od, &t_x));
    }
    if (head == HEAD_ALL) {
        spy_hip_tensor t_nw = T2(SPY_HIP_F32, (void *)c.out_norm, d, 1); t_nw.dim = 1;
        spy_hip_tensor t_l = T2(SPY_HIP_F32, lg, V, T);
        if (fuse_act) {
            RC_TRY(spy_norm_mul_q8_launch(st, x, 4 * d, (const float *)c.out_norm, c.eps, scr, T, d));
            RC_TRY(spy_hip_gemm_q8_0act(st, c.t_out, c.w_out, scr, lg, V, d, T, V));
        } else {
            RC_TRY(spy_hip_op_norm_rms(st, &t_x, &t_xn, c.eps));
            RC_TRY(spy_hip_op_binary(st, 2, &t_xn, &t_nw, &t_xn));
            RC_TRY(mm(c.w_out, c.t_out, d, V, &t_xn, &t_l));
        }
    } else if (head == HEAD_LAST) {         // the three head operators on the last token's row only
        spy_hip_tensor t_nw = T2(SPY_HIP_F32, (void *)c.out_norm, d, 1); t_nw.dim = 1;
        spy_hip_tensor t_x1 = T2(SPY_HIP_F32, x + (size_t)(T - 1) * d, d, 1), t_xn1 = T2(SPY_HIP_F32, xn, d, 1), t_l1 = T2(SPY_HIP_F32, lg, V, 1);
        RC_TRY(spy_hip_op_norm_rms(st, &t_x1, &t_xn1, c.eps));
        RC_TRY(spy_hip_op_binary(st, 2, &t_xn1, &t_nw, &t_xn1));
        RC_TRY(mm(c.w_out, c.t_out, d, V, &t_xn1, &t_l1));
        if (logits_host) HIP_TRY(hipMemcpyAsync(logits_host, lg, (size_t)V * 4, hipMemcpyDeviceToHost, st));
    }
    if (head == HEAD_ALL && logits_host) HIP_TRY(hipMemcpyAsync(logits_host, lg, (size_t)V * T * 4, hipMemcpyDeviceToHost, st));
    HIP_TRY(hipStreamSynchronize(st));
    return 0;
}

static int forward_any(spy_hip_llama *m, void *stream, const int32_t *tokens_host, int32_t n_token, int32_t n_past, float *logits_host, bool last_only) {
    SPY_CHECK_ARG(m && tokens_host && n_token > 0 && n_past >= 0);
    SPY_CHECK_ARG((int64_t)n_past + n_token <= m->desc.n_ctx);                  // llama.cpp:249
    hipStream_t st = stream ? (hipStream_t)stream : m->own_stream;
    for (int i = 0; i < n_token; i++) SPY_CHECK_ARG(tokens_host[i] >= 0 && tokens_host[i] < m->desc.n_vocab);   // view.cpp:61
    // A model in order 1 runs its prompt passes in the host's order as well (SPY_HIP_PROMPT_ORDER=0: prompts on the matrix cores in
    // this backend's own order, single-token passes still in order 1)
    struct scope_t { int prev; bool on; ~scope_t() { if (on) spy_exact_thread_scope(prev); } } scope = {-1, false};
    if (n_token > 1 && !spy_exact_on() && pass_order(m) == 1) {
        const char *e = getenv("SPY_HIP_PROMPT_ORDER");
        if (!(e && e[0] == '0')) { scope.prev = spy_exact_thread_scope(1); scope.on = true; }
    }
    const bool exact = spy_exact_on() != 0;
    // single tokens: the fused pass, in the order pass_order() names (with the library-wide exact-order switch on and a
    // model the exact kernels do not take, operator by operator instead)
    if (n_token == 1 && fused_ok(m) && (!exact || m->exact_ok)) {
        dev_state h = {tokens_host[0], n_past, 0, 0};
        HIP_TRY(hipMemcpyAsync(m->st, &h, sizeof(h), hipMemcpyHostToDevice, st));
        RC_TRY(enqueue_pass_any(m, st, PASS_LOGITS));
        if (logits_host) HIP_TRY(hipMemcpyAsync(logits_host, m->logits, (size_t)m->desc.n_vocab * 4, hipMemcpyDeviceToHost, st));
        return check_pass_error(m, st);
    }
    // longer passes in chunks: each chunk attends to everything before it, so the result per token
    // is that of one pass over the whole prompt
    // (the scores of a chunk take n_kv * chunk * n_head * 6 bytes of scratch; larger chunks fill the matrix-core grids better)
    const char *ch_env = getenv("SPY_HIP_PREFILL_CHUNK");
    const int ch_req = ch_env ? atoi(ch_env) : 0;
    // exact order: one pass over the whole prompt, as the reference runs it (a chunk boundary moves elements between
    // the 8-lane part and the scalar tail of the KQV dots and between the groups of four of the softmax sum)
    // ... unless the attention kernels that take the length of the whole row as a number are in use
    const int CH = exact && !exact_attn_ok(m) ? n_token : ch_req >= 16 ? ch_req : SPY_PREFILL_CHUNK;
    for (int t0 = 0; t0 < n_token; t0 += CH) {
        const int tc = n_token - t0 < CH ? n_token - t0 : CH;
        // logits nobody asked for are not computed: no buffer -> no head; last_only -> the head runs on the last row of the last chunk
        const int head = !logits_host ? HEAD_NONE : !last_only ? HEAD_ALL : (t0 + tc == n_token ? HEAD_LAST : HEAD_NONE);
        float *dst = !logits_host ? nullptr : last_only ? logits_host : logits_host + (size_t)t0 * m->desc.n_vocab;
        RC_TRY(forward_ops(m, st, tokens_host + t0, tc, n_past + t0, dst, head, n_past + n_token));
    }
    return 0;
}

extern "C" int spy_hip_llama_forward(spy_hip_llama *m, void *stream, const int32_t *tokens_host, int32_t n_token, int32_t n_past,
                                     float *logits_host) {
    return forward_any(m, stream, tokens_host, n_token, n_past, logits_host, false);
}

extern "C" int spy_hip_llama_forward_last(spy_hip_llama *m, void *stream, const int32_t *tokens_host, int32_t n_token, int32_t n_past,
                                          float *logits_last_host) {
    return forward_any(m, stream, tokens_host, n_token, n_past, logits_last_host, true);
}

#ifndef SPY_GRAPH_STEPS
#define SPY_GRAPH_STEPS 8   // passes per replayed graph of the greedy loop (the remainder runs the one-pass graph)
#endif
extern "C" int spy_hip_llama_decode_greedy(spy_hip_llama *m, void *stream, int32_t first_token, int32_t n_past, int32_t n_steps,
                                           int32_t *tokens_host, int32_t use_graph) {
    SPY_CHECK_ARG(m && n_steps > 0 && n_past >= 0 && first_token >= 0 && first_token < m->desc.n_vocab);
    SPY_CHECK_ARG((int64_t)n_past + n_steps <= m->desc.n_ctx && n_steps <= m->max_out);
    if (spy_exact_on() && !m->exact_ok) {
        // exact order for a model the fused exact kernels do not take: the reference's loop as it stands (cli.h:88-128) -- one operator-by-operator pass per token,
        // the first maximum of its logits (greedy.h:20-25) taken on the host
        std::vector<float> lg((size_t)m->desc.n_vocab);
        int32_t tok = first_token;
        for (int i = 0; i < n_steps; i++) {
            RC_TRY(forward_any(m, stream, &tok, 1, n_past + i, lg.data(), false));
            tok = (int32_t)(std::max_element(lg.begin(), lg.end()) - lg.begin());
            if (tokens_host) tokens_host[i] = tok;
        }
        return 0;
    }
    if (!fused_ok(m)) return SPY_HIP_EUNSUPPORTED;
    hipStream_t st = stream ? (hipStream_t)stream : m->own_stream;
    dev_state h = {first_token, n_past, 0, 0};
    HIP_TRY(hipMemcpyAsync(m->st, &h, sizeof(h), hipMemcpyHostToDevice, st));
    HIP_TRY(hipStreamSynchronize(st));
    if (use_graph && (!m->graph_exec || !m->graph_n_exec || m->graph_stream != st || m->graph_order != pass_order(m))) {
        m->graph_order = pass_order(m);
        if (m->graph_exec) { (void)hipGraphExecDestroy(m->graph_exec); m->graph_exec = nullptr; }
        if (m->graph) { (void)hipGraphDestroy(m->graph); m->graph = nullptr; }
        HIP_TRY(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        const int rc = enqueue_pass_any(m, st, PASS_GREEDY);
        hipError_t e = hipStreamEndCapture(st, &m->graph);
        if (rc) return rc;
        if (e != hipSuccess) return (int)e;
        HIP_TRY(hipGraphInstantiate(&m->graph_exec, m->graph, nullptr, nullptr, 0));
        m->graph_stream = st;
        // several passes as one graph: nothing in a pass depends on the host (token, position and step count live on the device)
        if (m->graph_n_exec) { (void)hipGraphExecDestroy(m->graph_n_exec); m->graph_n_exec = nullptr; }
        if (m->graph_n) { (void)hipGraphDestroy(m->graph_n); m->graph_n = nullptr; }
        HIP_TRY(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        int rcn = 0;
        for (int i = 0; i < SPY_GRAPH_STEPS && !rcn; i++) rcn = enqueue_pass_any(m, st, PASS_GREEDY);
        e = hipStreamEndCapture(st, &m->graph_n);
        if (rcn) return rcn;
        if (e != hipSuccess) return (int)e;
        HIP_TRY(hipGraphInstantiate(&m->graph_n_exec, m->graph_n, nullptr, nullptr, 0));
    }
    RC_TRY(enqueue_embed(m, st));              // embedding of the first token; every step prepares the next one's
    HIP_TRY(hipEventRecord(m->ev0, st));
    for (int i = 0; i < n_steps;) {
        if (use_graph && n_steps - i >= SPY_GRAPH_STEPS) { HIP_TRY(hipGraphLaunch(m->graph_n_exec, st)); i += SPY_GRAPH_STEPS; continue; }
        if (use_graph) HIP_TRY(hipGraphLaunch(m->graph_exec, st));
        else RC_TRY(enqueue_pass_any(m, st, PASS_GREEDY));
        i++;
    }
    HIP_TRY(hipEventRecord(m->ev1, st));
    HIP_TRY(hipEventSynchronize(m->ev1));
    float ms = 0.0f;
    HIP_TRY(hipEventElapsedTime(&ms, m->ev0, m->ev1));
    m->timed_ms += ms; m->timed_pass += n_steps;
    RC_TRY(check_pass_error(m, st));
    if (tokens_host) HIP_TRY(hipMemcpy(tokens_host, m->tokens_out, (size_t)n_steps * 4, hipMemcpyDeviceToHost));
    return 0;
}

// Average duration of ONE kernel of the single-token pass, measured with HIP events on the stream it
// is launched on: the kernel is launched for layer 0, 1, .. n_layer-1 (different weights and
// caches every launch, so nothing is served from a cache that the token loop would not have),
// `reps` times over.  The position used is the one left by the last pass.  which: "qkv", "scores",
// "pv", "wo", "gate_up", "down", "head".
extern "C" int spy_hip_llama_kernel_time(spy_hip_llama *m, void *stream, const char *which, int32_t reps, float *us_per_launch) {
    SPY_CHECK_ARG(m && which && reps > 0 && us_per_launch);
    if (!fused_ok(m)) return SPY_HIP_EUNSUPPORTED;
    static const char *names[K_COUNT] = {"qkv", "scores", "pv", "wo", "gate_up", "down", "head"};
    int k = -1;
    for (int i = 0; i < K_COUNT; i++) if (!strcmp(which, names[i])) k = i;
    SPY_CHECK_ARG(k >= 0);
    hipStream_t st = stream ? (hipStream_t)stream : m->own_stream;
    auto once = [&](int il) { return enqueue_one(m, st, k, il); };
    for (int il = 0; il < m->desc.n_layer; il++) RC_TRY(once(il));           // warm-up
    HIP_TRY(hipEventRecord(m->ev0, st));
    for (int r = 0; r < reps; r++)
        for (int il = 0; il < m->desc.n_layer; il++) RC_TRY(once(il));
    HIP_TRY(hipEventRecord(m->ev1, st));
    HIP_TRY(hipEventSynchronize(m->ev1));
    float ms = 0.0f;
    HIP_TRY(hipEventElapsedTime(&ms, m->ev0, m->ev1));
    *us_per_launch = ms * 1000.0f / (float)(reps * m->desc.n_layer);
    return 0;
}

// ---- the kernel families of the fused single-token pass, one at a time ---------------------------------------------------
// Each entry point launches exactly what the token loop launches for that part of a layer (same templates, same grids),
// on the caller's buffers and without a device state: a bare engine description is filled with the caller's pointers and
// handed to the same enqueue functions.  order: 1 = the host backend's summation order, 0 = this backend's own.
namespace {

template <int ORDER, int NITK, bool NORM>
__global__ __launch_bounds__(1024) void stage_dump_kernel(const float *__restrict__ x, const float *__restrict__ normw, float eps, int K, uint8_t *__restrict__ out) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[16];
    __shared__ float s_sum;
    const int tid = threadIdx.x;
    float4 xv[NITK], wv[NORM ? NITK : 1];
#pragma unroll
    for (int j = 0; j < NITK; j++) {
        const int i = min(tid + j * 1024, K / 4 - 1);
        xv[j] = ((const float4 *)x)[i];
        if constexpr (NORM) wv[j] = ((const float4 *)normw)[i];
    }
    int8_t *s_q = (int8_t *)smem;
    int2 *s_meta = (int2 *)(smem + staged_q_bytes(K));
    float *s_grp = (float *)(smem + ((staged_bytes(K) + 15) & ~(size_t)15));
    if constexpr (ORDER == 1) xg_stage<NITK, NORM, true>(xv, wv, K, eps, s_q, s_meta, s_grp, &s_sum, []() {});     // the chunked sum where it applies (K <= 8192): what gate|up runs
    else wgv_stage<NITK, NORM>(xv, wv, K, eps, s_q, s_meta, s_red);
    xg_dump_q8(s_q, s_meta, K, out);
}

template <int ORDER, bool NORM>
int stage_dump(hipStream_t st, const float *x, const float *normw, float eps, int64_t K, void *yq) {
    const size_t lds = ((staged_bytes(K) + 15) & ~(size_t)15) + (size_t)K + 1280;   // + K / 4 group sums, what the serial sum reads ahead, the records of the chunked sum
    switch ((K + 4095) / 4096) {
    case 1: stage_dump_kernel<ORDER, 1, NORM><<<dim3(1), dim3(1024), lds, st>>>(x, normw, eps, (int)K, (uint8_t *)yq); break;
    case 2: stage_dump_kernel<ORDER, 2, NORM><<<dim3(1), dim3(1024), lds, st>>>(x, normw, eps, (int)K, (uint8_t *)yq); break;
    case 3: stage_dump_kernel<ORDER, 3, NORM><<<dim3(1), dim3(1024), lds, st>>>(x, normw, eps, (int)K, (uint8_t *)yq); break;
    default: return SPY_HIP_EUNSUPPORTED;
    }
    return SPY_LAUNCH_RC();
}

// a bare engine: one layer, the caller's buffers, nothing owned
struct family_ctx {
    spy_hip_llama m;
    int init(int order, int n_embd, int n_head, int n_ff, int n_vocab, int64_t n_ctx, int wtype) {
        if (order != 0 && order != 1) return SPY_HIP_EINVAL;
        if (n_embd <= 0 || n_head <= 0 || n_embd % n_head != 0 || n_ctx <= 0 || n_ctx > (1 << 24)) return SPY_HIP_EINVAL;
        spy_hip_llama_desc &c = m.desc;
        memset(&c, 0, sizeof(c));
        c.n_layer = 1; c.n_embd = n_embd; c.n_head = n_head; c.n_ff = n_ff; c.n_vocab = n_vocab; c.n_ctx = (int32_t)n_ctx;
        c.eps = 0.0f; c.rope_freq_base = 10000.0f; c.wtype = wtype; c.t_out = wtype;
        m.layers.resize(1);
        memset(&m.layers[0], 0, sizeof(spy_hip_llama_layer));
        int32_t *tt[7] = {&m.layers[0].t_wq, &m.layers[0].t_wk, &m.layers[0].t_wv, &m.layers[0].t_wo, &m.layers[0].t_gate, &m.layers[0].t_up, &m.layers[0].t_down};
        for (int k = 0; k < 7; k++) *tt[k] = wtype;
        m.desc.layers = m.layers.data();
        m.hd = n_embd / n_head;
        m.k_cache.assign(1, nullptr); m.v_cache.assign(1, nullptr);
        m.wave = wave_ok(&m);
        if (!m.wave) return SPY_HIP_EUNSUPPORTED;
        const bool kq = wtype == SPY_HIP_Q4_K || wtype == SPY_HIP_Q6_K;
        if (wtype != SPY_HIP_Q4_0 && wtype != SPY_HIP_Q8_0 && !kq) return SPY_HIP_EUNSUPPORTED;
        if (kq && (n_embd % 256 != 0 || n_ff % 256 != 0)) return SPY_HIP_EINVAL;
        int dev = 0; hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0) m.num_cu = prop.multiProcessorCount;
        if (order == 1) {
            if (n_embd % 128 != 0 || n_ff % 128 != 0) return SPY_HIP_EUNSUPPORTED;
            RC_TRY(spy_exact_luts(&m.lut));
            m.exact_ok = true; m.order = 1;
        }
        return 0;
    }
};

}   // namespace

// libstdc++'s 4-way running sum of n non-negative terms (n % 4 == 0, n <= 8192): groups (t0 + t1) + (t2 + t3) added to one
// running sum, by one chain of additions (chunked == 0) or through xg_exact_sum (chunked == 1)
template <int NG>
__global__ __launch_bounds__(1024) void running_sum_kernel(const float *__restrict__ terms, int n, int chunked, float *__restrict__ out) {
    __shared__ __attribute__((aligned(16))) float s_g[2048 + 64];
    __shared__ xg_psum_lds s_l;
    const int tid = threadIdx.x, ng = n / 4;
    float grp[NG];
#pragma unroll
    for (int j = 0; j < NG; j++) {
        const int i = tid + j * 1024;
        grp[j] = 0.0f;
        if (i < ng) {
            const float4 v = ((const float4 *)terms)[i];
            const float v1 = v.x + v.y, v2 = v.z + v.w;
            grp[j] = v1 + v2;
            s_g[i] = grp[j];
        }
    }
    float tot;
    if (chunked) tot = xg_exact_sum<NG>(grp, ng, s_g, &s_l, 0.0f, []() {});
    else { __syncthreads(); tot = tid < 64 ? xg_serial_sum(s_g, ng, 0.0f) : 0.0f; }
    if (tid == 0) *out = tot;
}

extern "C" int spy_hip_running_sum_f32(void *stream, const float *terms, int64_t n, int32_t chunked, float *out) {
    SPY_CHECK_ARG(terms && out && n > 0 && n % 4 == 0 && n <= 8192 && (chunked == 0 || chunked == 1) && (((uintptr_t)terms) & 15) == 0);
    if (n <= 4096) running_sum_kernel<1><<<dim3(1), dim3(1024), 0, (hipStream_t)stream>>>(terms, (int)n, chunked, out);
    else running_sum_kernel<2><<<dim3(1), dim3(1024), 0, (hipStream_t)stream>>>(terms, (int)n, chunked, out);
    return SPY_LAUNCH_RC();
}

extern "C" int spy_hip_rmsnorm_q8_0(void *stream, int32_t order, const float *x, const float *normw, float eps, int64_t K, void *yq) {
    SPY_CHECK_ARG(x && yq && K > 0 && K % 64 == 0 && (order == 0 || order == 1));
    if (order == 1 && K % 128 != 0) return SPY_HIP_EUNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (order == 1) return normw ? stage_dump<1, true>(st, x, normw, eps, K, yq) : stage_dump<1, false>(st, x, normw, eps, K, yq);
    return normw ? stage_dump<0, true>(st, x, normw, eps, K, yq) : stage_dump<0, false>(st, x, normw, eps, K, yq);
}

extern "C" int spy_hip_gemv_fused(void *stream, int32_t order, int32_t wtype, const void *w, const float *x, const float *normw, float eps,
                                  const float *resid, float *out, int64_t M, int64_t K, void *xq_dump) {
    SPY_CHECK_ARG(w && x && out && M > 0 && K > 0 && M < (1ll << 30) && K < (1ll << 20));
    family_ctx f;
    if (normw && !resid) {                       // result_norm, result_linear, output: RMSNorm * weight -> Q8_0 -> rows of w
        RC_TRY(f.init(order, (int)K, (int)(K / 128), (int)K, (int)M, 8, wtype));
        f.m.desc.w_out = w; f.m.desc.out_norm = normw; f.m.desc.eps = eps;
        f.m.x = (float *)x; f.m.logits = out; f.m.q8_dump = (uint8_t *)xq_dump;
        return enqueue_one(&f.m, (hipStream_t)stream, K_HEAD, 0);
    }
    if (!normw && resid) {                       // KQV_linear + Add, ffn_down + Add: Q8_0(x) -> rows of w -> + resid
        SPY_CHECK_ARG(M % 128 == 0);
        RC_TRY(f.init(order, (int)M, (int)(M / 128), (int)K, 1, 8, wtype));
        f.m.layers[0].w_down = w;
        f.m.hbuf = (float *)x; f.m.x1 = (float *)resid; f.m.x = out; f.m.q8_dump = (uint8_t *)xq_dump;
        return enqueue_one(&f.m, (hipStream_t)stream, K_DOWN, 0);
    }
    return SPY_HIP_EUNSUPPORTED;
}

extern "C" int spy_hip_ffn_gate_up_silu(void *stream, int32_t order, int32_t wtype, const void *w_gate, const void *w_up, const float *x, const float *normw,
                                        float eps, float *out, int64_t F, int64_t K, void *xq_dump) {
    SPY_CHECK_ARG(w_gate && w_up && x && normw && out && F > 0 && K > 0 && K % 128 == 0 && F < (1ll << 24) && K < (1ll << 20));
    family_ctx f;
    RC_TRY(f.init(order, (int)K, (int)(K / 128), (int)F, 1, 8, wtype));
    f.m.layers[0].w_gate = w_gate; f.m.layers[0].w_up = w_up; f.m.layers[0].ffn_norm = normw; f.m.desc.eps = eps;
    f.m.x1 = (float *)x; f.m.hbuf = out; f.m.q8_dump = (uint8_t *)xq_dump;
    return enqueue_one(&f.m, (hipStream_t)stream, K_GATEUP, 0);
}

extern "C" int spy_hip_rope_kvwrite(void *stream, int32_t order, int32_t wtype, int32_t wtype_v, const void *wq, const void *wk, const void *wv, const float *x,
                                    const float *normw, float eps, int32_t n_embd, int32_t n_head, int32_t pos, int64_t n_ctx, const float *rope_cs,
                                    void *q16, void *k_cache, void *v_cache, void *xq_dump) {
    SPY_CHECK_ARG(wq && wk && wv && x && normw && rope_cs && q16 && k_cache && v_cache && pos >= 0 && pos < n_ctx && n_embd % 128 == 0);
    family_ctx f;
    RC_TRY(f.init(order, n_embd, n_head, n_embd, 1, n_ctx, wtype));
    if (f.m.hd != 128) return SPY_HIP_EUNSUPPORTED;
    spy_hip_llama_layer &L = f.m.layers[0];
    L.wq = wq; L.wk = wk; L.wv = wv; L.attn_norm = normw; L.t_wv = wtype_v ? wtype_v : wtype;
    f.m.desc.eps = eps;
    f.m.x = (float *)x; f.m.q16 = (uint16_t *)q16; f.m.k_cache[0] = (uint16_t *)k_cache; f.m.v_cache[0] = (uint16_t *)v_cache;
    f.m.rope_cs = (float *)rope_cs; f.m.rope_tab = (float *)rope_cs; f.m.rope_row0 = pos; f.m.pos_imm = pos; f.m.q8_dump = (uint8_t *)xq_dump;
    return enqueue_one(&f.m, (hipStream_t)stream, K_QKV, 0);
}

extern "C" int spy_hip_attn_decode(void *stream, int32_t order, const void *q16, const void *k_cache, const void *v_cache, int32_t n_head, int32_t n_kv,
                                   int64_t n_ctx, float *scores, float *out) {
    SPY_CHECK_ARG(q16 && k_cache && v_cache && scores && out && n_head > 0 && n_kv > 0 && n_kv <= n_ctx && n_ctx % 8 == 0);
    family_ctx f;
    RC_TRY(f.init(order, n_head * 128, n_head, n_head * 128, 1, n_ctx, SPY_HIP_Q4_0));
    const size_t pv_lds = (size_t)n_ctx * 6 + 16;
    if (order == 1) {
        if (n_ctx > 512 * XP_NP || xattn_pv_lds((int)n_ctx) > 160 * 1024 - 256 || xattn_scores_lds(n_head) > 160 * 1024) return SPY_HIP_EUNSUPPORTED;
        RC_TRY(spy_ensure_lds(&f.m, (const void *)xattn_pv_kernel<0>, xattn_pv_lds((int)n_ctx)));
        RC_TRY(spy_ensure_lds(&f.m, (const void *)xattn_scores_kernel<0>, xattn_scores_lds(n_head)));
    } else {
        if (pv_lds > 160 * 1024) return SPY_HIP_EUNSUPPORTED;
        RC_TRY(spy_ensure_lds(&f.m, (const void *)attn_pv_kernel, pv_lds));
    }
    f.m.q16 = (uint16_t *)q16; f.m.k_cache[0] = (uint16_t *)k_cache; f.m.v_cache[0] = (uint16_t *)v_cache;
    f.m.scores = scores; f.m.attn_out = out; f.m.pos_imm = n_kv - 1;
    RC_TRY(enqueue_one(&f.m, (hipStream_t)stream, K_SCORES, 0));
    return enqueue_one(&f.m, (hipStream_t)stream, K_PV, 0);
}
