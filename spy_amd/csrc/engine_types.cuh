// Shared declarations of the token-loop engine (state, per-kernel launch entry points).
#pragma once

#include "decode_kernels.cuh"

#include <unordered_map>
#include <vector>

#define HIP_TRY(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) return (int)e_; } while (0)
#define RC_TRY(x) do { int rc_ = (x); if (rc_) return rc_; } while (0)

struct spy_hip_llama {
    spy_hip_llama_desc desc;
    std::vector<spy_hip_llama_layer> layers;
    int hd = 0;
    gemv_cfg cfg_d = {0, 0}, cfg_ff = {0, 0};   // lanes-per-row / pairs-per-lane for K = n_embd and K = n_ff
    bool dry = false;
    bool attn_fused = false;                    // qkv + scores + softmax/KQV of a layer in one launch
    uint32_t *attn_sync = nullptr;
    bool uniform = true;                        // every layer matrix and the head in desc.wtype, Q4_0 or Q8_0
    bool wave = false;                          // one-row-per-wave kernels (1024-thread workgroups) instead of the tiled ones
    std::vector<uint16_t *> k_cache, v_cache;
    float *x = nullptr, *x1 = nullptr, *attn_out = nullptr, *hbuf = nullptr, *scores = nullptr, *logits = nullptr, *rope_cs = nullptr;
    uint16_t *q16 = nullptr;
    uint8_t *xq_head = nullptr;          // native Q8_0 activations for a K-quant output head
    dev_state *st = nullptr;
    int32_t *tokens_out = nullptr;
    int max_out = 0;
    int num_cu = 256;
    float theta_scale = 0.0f;
    // op-by-op path scratch (sized lazily for the largest chunk seen)
    uint8_t *ops_buf = nullptr; size_t ops_bytes = 0;
    // graph of one single-token pass
    hipGraph_t graph = nullptr; hipGraphExec_t graph_exec = nullptr; hipStream_t graph_stream = nullptr;
    hipGraph_t graph_n = nullptr; hipGraphExec_t graph_n_exec = nullptr;   // SPY_GRAPH_STEPS passes in one graph
    int graph_order = -1;                                                  // summation order the graphs were captured with
    hipStream_t own_stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    double timed_ms = 0.0; int timed_pass = 0;
    // Summation order of the fused single-token pass: 1 = the host backend's (exact_decode.cuh: every output equal to the CPU
    // backend's bit for bit), 0 = this backend's own (decode_kernels.cuh: faster, equal to about 1e-7 per operator)
    int order = 0;
    bool exact_ok = false;                      // the exact-order kernels take this model's shapes
    float *rope_tab = nullptr;                  // [n_ctx][hd]: cos, sin of every position's angles, from the host's libm (non-linear.cpp:304-309)
    const float *lut = nullptr;                 // exp table [65536], silu table [65536], filled by the host's libm
    uint8_t *q8_dump = nullptr;                 // tests: where workgroup 0 of a launch leaves its staged Q8_0 activations
    int pos_imm = 0, rope_row0 = 0;             // kernel-family entry points (no device state): the position; first position of rope_tab
    long long *stamp_dbg = nullptr;             // measurement builds (-DATL_STAMPS) only
    uint32_t spin_limit = 400000;               // polls of a bounded inter-workgroup wait before a pass gives up (~0.5 s)
    // per engine launcher state: the largest dynamic-LDS size this engine has asked for per kernel (the limit itself is kept
    // per device and kernel for the whole process and only ever raised: spy_raise_lds_limit), resident workgroups of a persistent grid
    std::unordered_map<const void *, size_t> lds_set;
    std::unordered_map<const void *, int> grid_cap;
    std::vector<void *> owned;
};


// a kernel's dynamic-LDS limit covers this engine's launches: the limit belongs to the kernel function for the whole process,
// so it is raised through the process-wide record and never lowered by an engine with a smaller context
static inline int spy_ensure_lds(spy_hip_llama *m, const void *kern, size_t lds) {
    size_t &have = m->lds_set[kern];
    if (lds > have) {
        RC_TRY(spy_raise_lds_limit(kern, lds));
        have = lds;
    }
    return 0;
}

// shapes the one-row-per-wave kernels take
static inline bool wave_ok(const spy_hip_llama *m) {
    const spy_hip_llama_desc &c = m->desc;
    return c.n_embd % 64 == 0 && c.n_embd <= 4096 && c.n_ff % 64 == 0 && c.n_ff <= 16384 && m->hd <= WGV_THREADS && m->hd % 2 == 0 && c.n_embd % 2 == 0;
}

enum { K_QKV = 0, K_SCORES, K_PV, K_WO, K_GATEUP, K_DOWN, K_HEAD, K_COUNT };

// One kernel of layer il of the single-token pass (K_HEAD: il ignored), for each layer-weight type.
// With m->dry set nothing is launched: the call only sizes the persistent grids.
int spy_enqueue_kernel_q4_0(spy_hip_llama *m, hipStream_t st, int which, int il);
int spy_enqueue_kernel_q8_0(spy_hip_llama *m, hipStream_t st, int which, int il);
int spy_enqueue_kernel_q4_k(spy_hip_llama *m, hipStream_t st, int which, int il);
int spy_enqueue_kernel_q6_k(spy_hip_llama *m, hipStream_t st, int which, int il);
// the same in the host backend's summation order (exact_launch.cuh)
int spy_enqueue_exact_q4_0(spy_hip_llama *m, hipStream_t st, int which, int il);
int spy_enqueue_exact_q8_0(spy_hip_llama *m, hipStream_t st, int which, int il);
int spy_enqueue_exact_q4_k(spy_hip_llama *m, hipStream_t st, int which, int il);
int spy_enqueue_exact_q6_k(spy_hip_llama *m, hipStream_t st, int which, int il);
// out[0..M) = rows of w (M x K, type of the name) . x (K floats, 16-byte aligned) in the host backend's order, one launch, no engine:
// SPY_HIP_EUNSUPPORTED for lengths the kernel does not take (K % 128, K-quants K % 256; K <= 16384, K-quants 12288)
int spy_exact_matvec_q4_0(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
int spy_exact_matvec_q8_0(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
int spy_exact_matvec_q4_k(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
int spy_exact_matvec_q6_k(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
// the same in this backend's own summation order (one-row-per-wave kernel; K % 64, K-quants K % 256; matrices of up to 15360 rows)
int spy_own_matvec_q4_0(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
int spy_own_matvec_q8_0(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
int spy_own_matvec_q4_k(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
int spy_own_matvec_q6_k(hipStream_t st, const void *w, const float *x, float *out, int M, int K);
// probe: only check that the fused attention launch for this layer's types exists and that all its workgroups are resident
int spy_probe_attn_layer_q4_0(spy_hip_llama *m, int il);
int spy_probe_attn_layer_q8_0(spy_hip_llama *m, int il);
int spy_probe_attn_layer_q4_k(spy_hip_llama *m, int il);
int spy_probe_attn_layer_q6_k(spy_hip_llama *m, int il);
