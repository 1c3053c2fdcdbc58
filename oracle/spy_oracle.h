/*
 * spy_oracle.h -- CPU restatement of the BL-GS/Spy host backend for the LLaMA-2 token loop.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker that the HIP path is compared
 * against (tests/, the smoke check and the cpu_baseline leg of the benchmark).  Nothing in
 * the shipped package may include, link, load or call it.
 *
 * Every function cites the reference file:line it restates (paths are relative to the
 * root of the BL-GS/Spy tree).  The reference cannot be compiled in this image: all of its
 * hot-path headers include simde / spdlog / magic_enum, none of which is vendored, so the
 * restatement is pinned by the closed forms, invariants and brute-force checks in
 * tests/test_oracle_*.py rather than by running the reference.
 *
 * Parity status per function (see the .c file for details):
 *   pinned by mathematics / IEEE definitions : fp16 conversions, Q8_0 quantizer, all int32
 *       block dots, dequantizers, layouts, masks, argmax, KV-cache placement.
 *   pinned to tolerance only (float summation ORDER restated from reading, not executed):
 *       dot_q4_0_q8_0 / dot_q8_0_q8_0 / dot_f16_f16 float results, norm_rms, softmax, rope.
 *   PARITY UNPINNED (no implementation exists in the reference): every Q4_K / Q6_K function.
 */
#ifndef SPY_ORACLE_H
#define SPY_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* NumberType ids: orchestration/include/number/number_impl/type.h:12-45 (= ggml type ids) */
enum {
    SPY_O_F32  = 0,
    SPY_O_F16  = 1,
    SPY_O_Q4_0 = 2,
    SPY_O_Q8_0 = 8,
    SPY_O_Q4_K = 12,
    SPY_O_Q6_K = 14,
    SPY_O_I32  = 26
};

/* Tensor = Shape{number_type, dim, elements[4], bytes[4]} + data_ptr
 * (orchestration/include/number/tensor.h:23-36,209-222). nb[] are BYTE strides; nb[0] is the
 * size of one block (tensor.h:50-57). */
typedef struct spy_o_tensor {
    int32_t type;
    int32_t dim;
    int64_t ne[4];
    int64_t nb[4];
    void   *data;
} spy_o_tensor;

/* ---- number system ------------------------------------------------------------------- */
int64_t  spy_o_type_size(int type);                 /* number.h:33-39  */
int64_t  spy_o_block_size(int type);                /* number.h:47-53  */
int64_t  spy_o_row_size(int type, int64_t n);       /* number.h:61-63  */
uint16_t spy_o_f32_to_f16(float x);                 /* lookup_table.h:54 (IEEE RNE) */
float    spy_o_f16_to_f32(uint16_t h);              /* lookup_table.h:52 + conversion.h:36-41 */
float    spy_o_f16_to_f32_ieee(uint16_t h);         /* exact widening, no table quirk */
float    spy_o_silu_lut(uint16_t h);                /* lookup_table_impl/non-linear.h:39-47 */
float    spy_o_exp_lut(uint16_t h);                 /* lookup_table_impl/non-linear.h:131-139 */
void     spy_o_tensor_contiguous(spy_o_tensor *t, int type, int dim, const int64_t *ne, void *data); /* tensor.h:44-58 */

/* ---- quantizers / dequantizers ------------------------------------------------------- */
void spy_o_quantize_q8_0(const float *x, void *y, int64_t n);        /* vec_convert.h:178-261 */
void spy_o_quantize_q4_0_ggml(const float *x, void *y, int64_t n);   /* intended rule (see .c) */
void spy_o_quantize_q4_0_as_written(const float *x, void *y, int64_t n_from); /* vec_convert.h:86-120, known-bad */
void spy_o_quantize_f16(const float *x, uint16_t *y, int64_t n);     /* vec_convert.h:56-64   */
void spy_o_quantize_q4_k(const float *x, void *y, int64_t n);        /* PARITY UNPINNED */
void spy_o_quantize_q6_k(const float *x, void *y, int64_t n);        /* PARITY UNPINNED */
void spy_o_dequantize_q4_0(const void *x, float *y, int64_t n);      /* closed form (n-8)*d; vec_dot.h:62-75 */
void spy_o_dequantize_q8_0(const void *x, float *y, int64_t n);      /* vec_convert.h:436-442 */
void spy_o_dequantize_q4_k(const void *x, float *y, int64_t n);      /* PARITY UNPINNED */
void spy_o_dequantize_q6_k(const void *x, float *y, int64_t n);      /* PARITY UNPINNED */

/* ---- dot products -------------------------------------------------------------------- */
float spy_o_dot_q4_0_q8_0(const void *w, const void *x, int64_t n);  /* vec_dot.h:42-86   */
float spy_o_dot_q8_0_q8_0(const void *w, const void *x, int64_t n);  /* vec_dot.h:88-115  */
float spy_o_dot_f16_f16(const uint16_t *a, const uint16_t *b, int64_t n); /* vec_dot.h:117-146 */
float spy_o_dot_q4_k_q8_0(const void *w, const void *x, int64_t n);  /* PARITY UNPINNED */
float spy_o_dot_q6_k_q8_0(const void *w, const void *x, int64_t n);  /* PARITY UNPINNED */
/* int32 dot of every 32-element block (Q4_0/Q8_0) or sub-block (Q4_K: 32, Q6_K: 16) */
int   spy_o_block_dots(int wtype, const void *w, const void *x, int64_t n, int32_t *out);
/* AVX2 build of the same three reference dots (bit-identical to the scalar ones; used for
 * the timed CPU baseline).  Returns 0 when the host lacks AVX2/FMA/F16C. */
int   spy_o_have_avx2(void);

/* ---- operators (backend/host/operator/ sources) --------------------------------------- */
/* all return 0 on success, 1 for an unsupported type combination (the reference aborts) */
int spy_o_matmul(const spy_o_tensor *w, const spy_o_tensor *x, spy_o_tensor *dst, int nthread);       /* mat.cpp:32-146 */
int spy_o_norm_rms(const spy_o_tensor *x, spy_o_tensor *dst, float eps);                              /* non-linear.cpp:194-223 */
int spy_o_binary(int op, const spy_o_tensor *a, const spy_o_tensor *b, spy_o_tensor *dst);            /* basic.cpp:15-50; op 0 add 1 sub 2 mul 3 div */
int spy_o_silu(const spy_o_tensor *x, spy_o_tensor *dst);                                             /* non-linear.cpp:57-77 */
int spy_o_relu(const spy_o_tensor *x, spy_o_tensor *dst);                                             /* non-linear.cpp:16-50 */
int spy_o_quantize(const spy_o_tensor *x, spy_o_tensor *dst);                                         /* quantize.cpp:18-41; F32 -> Q8_0 / F16 */
int spy_o_softmax(const spy_o_tensor *x, const spy_o_tensor *mask, spy_o_tensor *dst, float scale);   /* non-linear.cpp:86-180 */
typedef struct spy_o_rope_param {  /* operator/non-linear.h:191-207 */
    int32_t mode, num_past, num_dim, num_context, num_origin_context;
    float   freq_base, freq_scale, extend_factor, attention_factor, beta_fast, beta_slow, xpos_base;
    int32_t xpos_down;
} spy_o_rope_param;
int spy_o_rope(const spy_o_tensor *x, const spy_o_tensor *pos, spy_o_tensor *dst, const spy_o_rope_param *p); /* non-linear.cpp:270-371 */
int spy_o_dup(const spy_o_tensor *src, spy_o_tensor *dst);                                            /* view.cpp:83-195 */
int spy_o_contiguous(const spy_o_tensor *src, spy_o_tensor *dst);                                     /* view.cpp:285-321 */
int spy_o_get_row(const spy_o_tensor *table, const spy_o_tensor *ids, spy_o_tensor *dst);             /* view.cpp:33-81 */
int32_t spy_o_argmax(const float *logits, int64_t n);                                                 /* greedy.h:20-25 */

/* ---- the LLaMA token loop (model/src/llm/model/llama.cpp:86-313 and plugins) ---------- */
typedef struct spy_o_llama_layer {
    const float *attn_norm, *ffn_norm;                      /* f32[d]                        */
    const void  *wq, *wk, *wv, *wo, *w_gate, *w_up, *w_down;
    int32_t      t_wq, t_wk, t_wv, t_wo, t_gate, t_up, t_down; /* NumberType of each weight  */
} spy_o_llama_layer;

typedef struct spy_o_llama {
    int32_t n_layer, n_embd, n_head, n_ff, n_vocab, n_ctx;
    float   eps, rope_freq_base;
    int32_t nthread;
    const void  *tok_embd;   int32_t t_tok_embd;   /* F32 or Q8_0 (view.cpp:65-77)          */
    const float *out_norm;
    const void  *w_out;      int32_t t_out;
    const spy_o_llama_layer *layers;
    uint16_t **k_cache;      /* per layer: f16 [n_ctx][n_head][hd]   (attention.cpp:188-205)  */
    uint16_t **v_cache;      /* per layer: f16 [n_embd][n_ctx]       (attention.cpp:228-246)  */
} spy_o_llama;

/* One forward pass over n_token new tokens at positions n_past .. n_past+n_token-1.
 * logits: f32[n_vocab * n_token] (all tokens, llama.cpp:229-232). Returns 0 on success. */
int spy_o_llama_forward(const spy_o_llama *m, const int32_t *tokens, int n_token, int n_past, float *logits);
/* Hook for per-op comparisons: when non-NULL, the forward pass copies the named
 * intermediate of layer `layer` into `out` (f32).  Names: "attn_norm", "q_rope", "k_rope",
 * "v", "kqv", "attn_out", "ffn_inp", "ffn_par", "layer_out". */
void spy_o_llama_tap(const char *name, int layer, float *out);

#ifdef __cplusplus
}
#endif
#endif
