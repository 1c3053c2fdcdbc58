/*
 * spy_hip.h -- C ABI of the MI355X (gfx950) backend for Spy's LLaMA-2 token loop.
 *
 * This is the drop-in boundary.  Spy has no C ABI of its own: its backends are C++ classes
 * derived from spy::Backend (backend/interface/include/backend/backend.h:31-95) whose
 * submit(OperatorNode*, callback) dispatches on OperatorType to one OperatorImpl<Op>::execute
 * per operator (backend/host/include/operator_impl.h:17-89, backend/host/backend/cpu_backend.cpp:71-94).
 * Each spy_hip_op_* entry point below replaces one of those execute() bodies and takes the same
 * operands: the operator's input/output `Tensor`s (orchestration/include/number/tensor.h:209-222)
 * flattened to POD, and the operator's Param struct flattened to scalars.
 *
 * Conventions
 *   - every function returns 0 on success, a positive hipError_t, or a negative SPY_HIP_E* code;
 *     nothing throws and nothing aborts (the reference asserts/aborts instead,
 *     backend/host/include/default_backend.h:72-78);
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); launches are
 *     asynchronous, the caller synchronises;
 *   - all tensor memory is device memory owned by the caller; the spy_hip_op_* entry points never allocate, free or
 *     synchronise once spy_hip_init has run on the device (it builds the tables the exact-order operators look values
 *     up in), so they can be recorded under HIP stream capture.  The one exception is exact-order Rope, whose table of
 *     host-libm angles depends on the call's parameters: spy_hip_rope_prepare builds it ahead of time; without that the
 *     first call with a new parameter set builds it (allocating) where it may, and under capture returns
 *     SPY_HIP_EUNSUPPORTED instead;
 *   - shapes use Spy's order: ne[0] is the contiguous dimension, nb[] are BYTE strides and nb[0]
 *     is the size of one block (tensor.h:50-57).
 */
#ifndef SPY_HIP_H
#define SPY_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SPY_HIP_EUNSUPPORTED (-1) /* OperatorStatus::Unsupport (backend.h:22-29) */
#define SPY_HIP_EINVAL       (-2) /* shape / argument check failed (spy_assert in the reference) */
#define SPY_HIP_ENOSPACE     (-3) /* caller-provided scratch too small */
#define SPY_HIP_ETIMEOUT     (-4) /* a bounded wait between workgroups of a fused launch expired: the pass's results are void */

/* NumberType ids (orchestration/include/number/number_impl/type.h:12-45) */
enum spy_hip_type {
    SPY_HIP_F32 = 0, SPY_HIP_F16 = 1, SPY_HIP_Q4_0 = 2, SPY_HIP_Q8_0 = 8,
    SPY_HIP_Q4_K = 12, SPY_HIP_Q6_K = 14, SPY_HIP_I32 = 26
};

/* spy::Tensor flattened (tensor.h:23-36, 209-222) */
typedef struct spy_hip_tensor {
    int32_t type;
    int32_t dim;
    int64_t ne[4];
    int64_t nb[4];
    void   *data;
} spy_hip_tensor;

/* ---- runtime: replaces DefaultCPUBackend's constructor / alloc_memory / dealloc_memory
 *      (backend/host/include/default_backend.h:121-156) and the capacity queries of
 *      spy::Backend (backend.h:44-51) ------------------------------------------------------- */
int spy_hip_init(int device_id);
int spy_hip_device_info(char *name, int name_len, int *num_cu, size_t *total_mem, size_t *free_mem);
int spy_hip_alloc(void **ptr, size_t bytes);
int spy_hip_free(void *ptr);
int spy_hip_upload(void *dst_dev, const void *src_host, size_t bytes, void *stream);
int spy_hip_download(void *dst_host, const void *src_dev, size_t bytes, void *stream);
int spy_hip_fill_u8(void *dst_dev, int value, size_t bytes, void *stream);   /* fill kernel, graph-safe */
int spy_hip_sync(void *stream);                      /* NULL: whole device */
int spy_hip_stream_create(void **stream);
int spy_hip_stream_destroy(void *stream);
int spy_hip_event_create(void **event);
int spy_hip_event_record(void *event, void *stream);
int spy_hip_event_elapsed_ms(void *start, void *stop, float *ms);   /* synchronises on `stop` */
int spy_hip_event_destroy(void *event);
/* Stream capture for callers without the HIP headers: every call made on `stream` between begin and end is recorded
 * instead of run; end instantiates the recording as an executable graph (*graph_exec), which graph_launch replays on a
 * stream.  No counterpart in the reference (its scheduler re-dispatches every operator every pass,
 * default_scheduler.h:46-111). */
int spy_hip_capture_begin(void *stream);
int spy_hip_capture_end(void *stream, void **graph_exec);
int spy_hip_graph_launch(void *graph_exec, void *stream);
int spy_hip_graph_destroy(void *graph_exec);
const char *spy_hip_error_string(int code);

/* ---- operators: one per OperatorImpl<Op>::execute of the host backend ---------------------- */

/* MatMul -- OperatorMatMulImpl::execute (backend/host/operator/mat.cpp:71-146).
 * dst[i01,i11,i2,i3] = dot(w[:,i01,i2,i3], x[:,i11,i2,i3]).  Type routing as
 * target_buffer_type (mat.cpp:32-42): (Q4_0|Q8_0, F32) quantizes x to Q8_0, (F16, F32) rounds x
 * to fp16; additionally (Q4_K|Q6_K, F32) -> Q8_0 activations, which the reference lacks.
 * `scratch` holds the converted activations (the reference allocates it in get_control_header,
 * mat.cpp:61-68); query its size with spy_hip_op_matmul_scratch_size.  While the host's summation
 * order is on (spy_hip_set_exact_order) that size also covers fp16 copies of both operands, from which
 * the prompt-sized Q4_0 / Q8_0 MatMul of that order runs fastest; a buffer that holds only the
 * activations (rows * row size of the converted type) is accepted too and gives the same results.
 * One contiguous f32 row against a plain quantized matrix (the weight products of a single-token pass) is
 * quantized inside the launch that multiplies it and leaves `scratch` untouched, in either summation order. */
size_t spy_hip_op_matmul_scratch_size(const spy_hip_tensor *w, const spy_hip_tensor *x);
int spy_hip_op_matmul(void *stream, const spy_hip_tensor *w, const spy_hip_tensor *x, const spy_hip_tensor *dst,
                      void *scratch, size_t scratch_bytes);
/* MatMul with no allocation anywhere -- no counterpart in the reference, whose MatMul allocates its activation buffer
 * per node (mat.cpp:61-68).  For callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  Same operator and same results as spy_hip_op_matmul; the converted activations go
 * to a fixed array in device memory (spy_hip_op_matmul_noalloc_max_scratch() bytes, 8 MiB, held by every device the
 * library runs on until the process ends) instead of a caller buffer.  Returns SPY_HIP_ENOSPACE when the converted
 * activations (rows * row size of the converted type) exceed that.  All calls on a device share the array: calls that overlap on one
 * device (different streams or threads) race, and a replay of a graph that recorded such a call counts as a call.  While
 * the host's summation order is on, the fp16 operand copies of spy_hip_op_matmul_scratch_size go into the array as well
 * when they fit behind the activations, and are left out (same results) when they do not. */
size_t spy_hip_op_matmul_noalloc_max_scratch(void);
int spy_hip_op_matmul_noalloc(void *stream, const spy_hip_tensor *w, const spy_hip_tensor *x, const spy_hip_tensor *dst);
/* NormRMS -- OperatorNormRMSImpl::execute (non-linear.cpp:194-223); eps = NormRMSParam::eps */
int spy_hip_op_norm_rms(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *dst, float eps);
/* Add/Sub/Mul/Div -- binary_execution<Op> (basic.cpp:15-50); op: 0 add, 1 sub, 2 mul, 3 div */
int spy_hip_op_binary(void *stream, int op, const spy_hip_tensor *a, const spy_hip_tensor *b, const spy_hip_tensor *dst);
/* Silu -- OperatorSiluImpl::execute (non-linear.cpp:57-77) */
int spy_hip_op_silu(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *dst);
/* Relu -- OperatorReluImpl::execute (non-linear.cpp:16-50): max(x, 0), f32 */
int spy_hip_op_relu(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *dst);
/* Quantize -- OperatorQuantizeImpl::execute (backend/host/operator/quantize.cpp:18-41): rows of x converted to dst's type by
 * auto_quantize_inner (vec_convert.h:463-468).  F32 -> Q8_0 and F32 -> F16; dst rows back to back.  F32 -> Q4_0 is
 * SPY_HIP_EUNSUPPORTED: the reference's own (vec_convert.h:83-117) fills half of every block and inverts the scale. */
int spy_hip_op_quantize(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *dst);
/* Softmax -- OperatorSoftmaxImpl::execute (non-linear.cpp:86-185); mask may be NULL;
 * scale = SoftmaxParam::scale.  dst may also be FP16 (rows of up to 16384 elements, scale > 0): the
 * probabilities rounded the way the KQV MatMul rounds its right operand first (mat.cpp:37), so that the
 * product can take them without a conversion pass */
int spy_hip_op_softmax(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *mask, const spy_hip_tensor *dst, float scale);
/* Rope -- OperatorRopeImpl::execute (non-linear.cpp:270-371); fields of RopeParam
 * (orchestration/include/operator/non-linear.h:191-207).  Supported: mode None/Norm (-1/0), including
 * extend_factor != 0 (rope_yarn, :242-260: as written its ramp is 0, so the angle stays the interpolated one and the
 * magnitude is multiplied by 1 + 0.1 ln(1 / freq_scale)) and xpos_base != 0 (zeta, :353-354), and mode GLM (4; :315-343,
 * as written: elements i0, i0 + num_dim / 2 rotated by min(p, num_context - 2) * theta_scale^i0 and elements i0 + num_dim,
 * i0 + 3 num_dim / 2 by max(p - (num_context - 2), 0) * theta_scale^i0 for i0 < ne0 / 4; rows in which those indices would
 * leave the row are refused with EINVAL where the reference reads past it; not in the exact-order mode).  Neox (2) aborts in
 * the reference and is EUNSUPPORTED here. */
typedef struct spy_hip_rope_param {
    int32_t mode, num_past, num_dim, num_context, num_origin_context;
    float   freq_base, freq_scale, extend_factor, attention_factor, beta_fast, beta_slow, xpos_base;
    int32_t xpos_down;
} spy_hip_rope_param;
int spy_hip_op_rope(void *stream, const spy_hip_tensor *x, const spy_hip_tensor *pos, const spy_hip_tensor *dst, const spy_hip_rope_param *p);
/* Exact-order Rope takes cosf / sinf of every position's angles from the host's libm, as the reference does
 * (non-linear.cpp:304-309): a table per parameter set {num_context, ne0, freq_base, freq_scale, attention_factor, num_dim},
 * kept on the device until the process ends (at most 16 per device).  This call builds it ahead of time (ne0 = the rotated
 * row length, dst->ne[0] of the calls to come), after which exact-order spy_hip_op_rope with these parameters neither
 * allocates nor synchronises.  SPY_HIP_EUNSUPPORTED where no table applies (no context length, xpos, YaRN extension:
 * those calls read the positions back and synchronise). */
int spy_hip_rope_prepare(const spy_hip_rope_param *p, int64_t ne0);
/* Dup / Copy -- dup_execute (view.cpp:83-195): F32->F32, F32->F16, F16->F32 through strides */
int spy_hip_op_dup(void *stream, const spy_hip_tensor *src, const spy_hip_tensor *dst);
/* Contiguous -- OperatorContiguousImpl::execute (view.cpp:285-321) */
int spy_hip_op_contiguous(void *stream, const spy_hip_tensor *src, const spy_hip_tensor *dst);
/* GetRow -- OperatorGetRowImpl::execute (view.cpp:33-81): F32 or Q8_0 table -> F32 rows.
 * Row ids outside the table leave the output row untouched and raise the device-side error flag
 * returned by spy_hip_take_error (the reference asserts, view.cpp:61). */
int spy_hip_op_get_row(void *stream, const spy_hip_tensor *table, const spy_hip_tensor *ids, const spy_hip_tensor *dst);
int spy_hip_take_error(int *flag);   /* reads and clears the device error flag (synchronises) */
/* Exact-order mode of the spy_hip_op_* entry points (on != 0; returns the previous setting; the environment
 * variable SPY_HIP_EXACT=1 is its initial value).  MatMul, NormRMS, Softmax, Silu and Rope then add their terms
 * in the order of the host backend's own loops -- the 8-lane accumulators and hsum_float_8 of Dot<Q4_0,Q8_0>,
 * Dot<Q8_0,Q8_0> and Dot<FP16,FP16> (vec_dot.h:42-146, vec_util.h:75-81), libstdc++'s four-way std::reduce in
 * NormRMS and Softmax (non-linear.cpp:129-223) -- and take exp / silu from tables and the Rope angles from the
 * host's libm (lookup_table_impl/non-linear.h:39-47,131-139, non-linear.cpp:270-371), so that every operator
 * output equals the host backend's bit for bit.  A checking mode, about 12 x slower than the fused token
 * loop.  spy_hip_llama_forward / _forward_last / _decode_greedy follow it: every pass runs operator by operator
 * (the prompt as one pass, the greedy loop with the argmax on the host).  With RopeParam::num_context > 0 the
 * rotations of all positions are kept in a device table and a position outside it raises the error flag of
 * spy_hip_take_error; with num_context == 0 Rope reads the positions back and synchronises the stream. */
int spy_hip_set_exact_order(int on);
/* Greedy sampling -- SamplerImpl<Greedy>::sample (model/include/llm/sampler/greedy.h:20-25):
 * index of the FIRST maximum of n logits, written to *out_index (device int32) */
int spy_hip_argmax(void *stream, const float *logits, int64_t n, int32_t *out_index);

/* ---- kernel families used by the operators above and by the fused token loop --------------- */

/* Quantizator<FP32,Q8_0>::transform (backend/host/include/simd/vec_convert.h:178-261):
 * nrow rows of K floats (row stride x_stride BYTES) -> nrow rows of K/32 native Q8_0 blocks */
int spy_hip_quantize_q8_0(void *stream, const float *x, int64_t x_stride, void *y, int64_t nrow, int64_t K);
/* Quantizator<FP32,FP16>::transform (vec_convert.h:39-65) */
int spy_hip_quantize_f16(void *stream, const float *x, int64_t x_stride, void *y, int64_t nrow, int64_t K);
/* Dot<W,Q8_0>::exec over every weight row (vec_dot.h:42-115): dst[t*dst_stride + m] =
 * dot(w row m, xq row t) (+ residual[t*dst_stride + m] when residual != NULL).
 * w: M rows of K elements in native block layout, contiguous; xq: T rows of K/32 native Q8_0
 * blocks, contiguous; strides in ELEMENTS. */
int spy_hip_gemv_q8_0act(void *stream, int wtype, const void *w, const void *xq, float *dst, const float *residual,
                         int64_t M, int64_t K, int64_t T, int64_t dst_stride);
/* The same dots for many activation rows at once (prompt passes) on the matrix cores: int8 MFMA,
 * one 32-element block per instruction, exact int32 block dots scaled by h2f(d_w)*h2f(d_x) and
 * accumulated in fp32 (K-quants: per sub-block / 16-element group).  K % 64 == 0 (K-quants: K % 256 == 0);
 * operands as for spy_hip_gemv_q8_0act. */
int spy_hip_gemm_q8_0act(void *stream, int wtype, const void *w, const void *xq, float *dst,
                         int64_t M, int64_t K, int64_t T, int64_t dst_stride);
/* Causal attention of a pass over T tokens at positions past .. past+T-1, all heads, in one kernel: the
 * operator sequence MatMul(K cache view, q) -> Softmax(causal mask, scale) -> MatMul(V^T cache view, P) of
 * the LLaMA graph (attention.cpp:25-302; mat.cpp:32-146; non-linear.cpp:129-180) without the score and
 * probability matrices in memory.  q16: rotated queries as fp16 [H][T][hd]; k_cache: fp16 [n_ctx][H*hd];
 * v_cache: fp16 [H*hd][n_ctx], both already holding the pass's own rows; out: f32 [T][H*hd].
 * hd must be 128 and n_ctx a multiple of 8 (else SPY_HIP_EUNSUPPORTED). */
int spy_hip_prompt_attention(void *stream, const void *q16, const void *k_cache, const void *v_cache, float *out,
                             int32_t T, int32_t H, int32_t hd, int32_t past, int64_t n_ctx, float scale);
/* The same three operators in the host backend's summation order, bit for bit (Dot<FP16,FP16> with its 32 accumulators,
 * tree and scalar tail, vec_dot.h:117-146; Softmax with the table exp and libstdc++'s groups of four,
 * non-linear.cpp:86-180), as three kernels that leave out what the causal mask removes.  q: rotated queries as f32
 * [T][H*hd] (converted to fp16 inside, as MatMul does, mat.cpp:37); caches and out as above.  n_total: the cached
 * positions after the whole pass this call is a part of (past + T when the pass is not cut into chunks): the host's
 * dot adds the last 1..32 of them one by one and its softmax sum the last n_total % 4 terms.  scratch: device memory
 * of spy_hip_prompt_attention_exact_scratch_size bytes, 256-byte aligned (scores and probabilities of this call).
 * hd must be 128, n_ctx a multiple of 32 and past + T at most 8192 (else SPY_HIP_EUNSUPPORTED). */
size_t spy_hip_prompt_attention_exact_scratch_size(int32_t T, int32_t H, int32_t past);
int spy_hip_prompt_attention_exact(void *stream, const float *q, const void *k_cache, const void *v_cache, float *out,
                                   int32_t T, int32_t H, int32_t hd, int32_t past, int64_t n_ctx, int32_t n_total, float scale,
                                   void *scratch, size_t scratch_bytes);
/* the int32 dot of every 32-element block (Q4_0, Q8_0, Q4_K sub-blocks) or 16-element
 * sub-block (Q6_K) of every weight row with activation row 0: out[m*nsub + b], written by the
 * GEMV kernels themselves (same code path, dump switch on).  `out` must hold M*nsub + M int32:
 * the last M slots receive the float results and are scratch. */
int spy_hip_block_dots(void *stream, int wtype, const void *w, const void *xq, int32_t *out, int64_t M, int64_t K);

/* ---- the kernel families of the fused single-token pass, one launch at a time.  Each runs exactly the launch the token
 *      loop below uses for that part of a layer (same kernel, same grid), on the caller's buffers; order = 1: the host
 *      backend's summation order (results equal, bit for bit, to the host backend's compiled without fp contraction), 0: this backend's own.  K (and F) must be
 *      multiples of 128 for order 1, rows at most 4096 elements wide for the norm prologue (16384 for the plain one). ------- */
/* The running sum that NormRMS and Softmax of the host backend take over their terms: libstdc++'s std::reduce /
 * std::transform_reduce for random-access ranges (non-linear.cpp:165-168, 205-208) adds groups of four,
 * (t0 + t1) + (t2 + t3), to ONE running sum in order.  n non-negative floats (n % 4 == 0, n <= 8192, 16-byte aligned)
 * -> *out, bit for bit; chunked = 0: one chain of additions, 1: the chunked form the gate|up kernel of order 1 uses
 * (integer increments per 64-term chunk inside a binade, the chain only where the sum crosses a power of two). */
int spy_hip_running_sum_f32(void *stream, const float *terms, int64_t n, int32_t chunked, float *out);
/* RMSNorm * weight -> Q8_0: OperatorNormRMSImpl::execute + the Mul node + Quantizator<FP32,Q8_0>::transform
 * (non-linear.cpp:194-223, basic.cpp:15-50, vec_convert.h:178-261) as the fused kernels stage their activations;
 * normw == NULL: the quantization alone.  yq: K/32 native Q8_0 blocks. */
int spy_hip_rmsnorm_q8_0(void *stream, int32_t order, const float *x, const float *normw, float eps, int64_t K, void *yq);
/* attn_norm, Q/K/V_project, 2 x Rope, the fp16 rounding of Q and both KV-cache copies of one token at position pos
 * (attention.cpp:25-265; mat.cpp:71-146; non-linear.cpp:270-371; view.cpp:83-227): q16 = fp16[n_embd], row pos of
 * k_cache (fp16 [n_ctx][n_embd]) and column pos of v_cache (fp16 [n_embd][n_ctx]).  rope_cs: cos, sin per pair of the
 * position's angles (hd floats; theta_0 = pos, theta_{k+1} = theta_k * powf(base, -2/hd) in fp32).  wtype_v: type of wv
 * (0 = wtype; Q6_K next to Q4_K).  xq_dump: NULL or K/32 Q8_0 blocks that receive the staged activations. */
int spy_hip_rope_kvwrite(void *stream, int32_t order, int32_t wtype, int32_t wtype_v, const void *wq, const void *wk, const void *wv, const float *x,
                         const float *normw, float eps, int32_t n_embd, int32_t n_head, int32_t pos, int64_t n_ctx, const float *rope_cs,
                         void *q16, void *k_cache, void *v_cache, void *xq_dump);
/* attn_score, Softmax, KQV of one token over n_kv cached tokens, all heads (MatMul(K view, q) -> Softmax(mask 0, scale
 * 1/sqrt(128)) -> MatMul(V^T view, P); mat.cpp:71-146, vec_dot.h:117-146, non-linear.cpp:129-180): two launches (scores;
 * softmax + P.V^T).  scores: scratch f32 [n_head][n_ctx]; out: f32 [n_head * 128]. */
int spy_hip_attn_decode(void *stream, int32_t order, const void *q16, const void *k_cache, const void *v_cache, int32_t n_head, int32_t n_kv,
                        int64_t n_ctx, float *scores, float *out);
/* One matrix x vector launch with its prologue and epilogue: normw != NULL, resid == NULL: RMSNorm * weight -> Q8_0 -> M rows
 * of w (result_norm .. output); normw == NULL, resid != NULL: Q8_0(x) -> rows of w -> + resid (KQV_linear + Add, ffn_down
 * + Add; M % 128 == 0).  Dot<W,Q8_0>::exec per row (vec_dot.h:42-115). */
int spy_hip_gemv_fused(void *stream, int32_t order, int32_t wtype, const void *w, const float *x, const float *normw, float eps,
                       const float *resid, float *out, int64_t M, int64_t K, void *xq_dump);
/* ffn_norm, ffn_gate, ffn_up, Silu, Mul (ffn.cpp:5-42; non-linear.cpp:11-14,57-77): out[i] = up_i * silu(gate_i), F values */
int spy_hip_ffn_gate_up_silu(void *stream, int32_t order, int32_t wtype, const void *w_gate, const void *w_up, const float *x, const float *normw,
                             float eps, float *out, int64_t F, int64_t K, void *xq_dump);

/* ---- measured ceilings of the part (no counterpart in the reference; they back the roofline denominators
 *      printed by the operator sweep and are called by nothing else) ---- */
/* int8 matrix-core rate in TOP/s (2 operations per multiply-accumulate): waves issuing only
 * v_mfma_i32_32x32x32_i8 on register operands, iters x 4 per wave */
int spy_hip_measure_mfma_i8(void *stream, int32_t iters, float *tops);
/* The same matrix instruction with what a block-scaled GEMM adds per quantization block and 32 x 32 tile, on register
 * operands only: the fp16 outer product of the scales and the 32 vector instructions per lane that scale and
 * accumulate the block dots (mode 0: conversion + fma; mode 1: biased integer accumulator, subtraction + fma, as
 * spy_hip_gemm_q8_0act does it).  The ceiling that this epilogue leaves to the int8 matrix cores; TOP/s of int8
 * operations.  No counterpart in the reference. */
int spy_hip_measure_mfma_i8_scaled(void *stream, int32_t iters, int32_t mode, float *tops);
/* read rate in GB/s over `bytes` of device memory (16-byte aligned, >= 1 MiB; use >= 1 GiB), reps passes */
int spy_hip_measure_hbm_read(void *stream, const void *buf, size_t bytes, int32_t reps, float *gbps);

/* ---- the token loop: replaces the per-operator dispatch of one forward pass
 *      (DefaultGraphScheduler::execute, backend/distributor/include/scheduler/default_scheduler.h:46-111,
 *      over the graph LLAMAModel::build_graph wires, model/src/llm/model/llama.cpp:86-264) and the
 *      greedy loop of AutoModelGenerator::generate (app/cli/include/cli.h:88-128) for single-token
 *      passes.  Same operators, same rounding points, same KV-cache layouts
 *      (K: f16 [n_ctx][n_head][hd], V: f16 [n_embd][n_ctx]; model/src/llm/plugin/attention.cpp:188-262);
 *      fused into four kernels per layer and replayed as a HIP graph. ----------------------------- */
typedef struct spy_hip_llama_layer {
    const float *attn_norm, *ffn_norm;                         /* f32[n_embd], device          */
    const void  *wq, *wk, *wv, *wo, *w_gate, *w_up, *w_down;   /* native GGUF blocks, device   */
    /* type of each matrix: Q4_0, Q8_0, Q4_K or Q6_K; 0 = the description's wtype.  Within a layer wq and
     * wk share a type and so do w_gate and w_up (they are read by the same kernel); wv may be Q6_K next
     * to Q4_K wq / wk (the Q4_K_M mix). */
    int32_t t_wq, t_wk, t_wv, t_wo, t_gate, t_up, t_down;
} spy_hip_llama_layer;

typedef struct spy_hip_llama_desc {
    int32_t n_layer, n_embd, n_head, n_ff, n_vocab, n_ctx;     /* n_ctx % 8 == 0               */
    float   eps, rope_freq_base;
    int32_t wtype;                                             /* default type of the layer matrices: Q4_0, Q8_0, Q4_K, Q6_K */
    const void  *tok_embd;  int32_t t_tok_embd;                /* F32 or Q8_0 (GetRow, view.cpp:65-77) */
    const float *out_norm;
    const void  *w_out;     int32_t t_out;                     /* Q4_0, Q8_0, Q4_K or Q6_K     */
    const spy_hip_llama_layer *layers;                         /* host array of n_layer entries */
} spy_hip_llama_desc;

typedef struct spy_hip_llama spy_hip_llama;

/* Allocates the KV caches (zero-filled) and the activation scratch on the current device --
 * the Cache / Dynamic tensors the scheduler would request through alloc_memory
 * (default_scheduler.h:157-175).  Weights stay where the caller uploaded them. */
int spy_hip_llama_create(const spy_hip_llama_desc *desc, spy_hip_llama **out);
int spy_hip_llama_destroy(spy_hip_llama *m);
/* One forward pass over n_token tokens at positions n_past.. (any n_token >= 1; passes of more
 * than one token run the operator kernels one after the other below 16 tokens and, from 16 tokens, the
 * matrix-core GEMMs with fused activation producers and the attention kernel; long prompts go through in
 * chunks of 2048 tokens).  logits_host: NULL (no output head is computed) or n_vocab*n_token floats. */
int spy_hip_llama_forward(spy_hip_llama *m, void *stream, const int32_t *tokens_host, int32_t n_token, int32_t n_past,
                          float *logits_host);
/* The same pass with the output head applied to the last token only: logits_last_host receives
 * n_vocab floats (NULL: no head at all).  What a token loop needs from a prompt: the reference's graph
 * computes the logits of every prompt token (llama.cpp:86-313) and the loop then samples from the last
 * row (cli.h:88-100); the other rows, n_vocab*(n_token-1) floats, are neither computed nor copied here. */
int spy_hip_llama_forward_last(spy_hip_llama *m, void *stream, const int32_t *tokens_host, int32_t n_token, int32_t n_past,
                               float *logits_last_host);
/* n_steps single-token passes with greedy sampling on the device: step i consumes the token
 * sampled by step i-1 (the first consumes first_token at position n_past) and tokens_host[i]
 * receives the token sampled by step i.  use_graph: replay a captured HIP graph. */
int spy_hip_llama_decode_greedy(spy_hip_llama *m, void *stream, int32_t first_token, int32_t n_past, int32_t n_steps,
                                int32_t *tokens_host, int32_t use_graph);
/* Summation order of the model's passes: of the fused single-token pass, and of prompt passes (in order 1 they run
 * operator by operator through the exact-order kernels, in order 0 on the matrix cores).  1 (the default wherever the kernels take the model: 128-wide heads,
 * n_embd and n_ff multiples of 128): the host backend's -- the eight accumulators and hsum_float_8 of its quantized dots,
 * the 4 x 8 accumulators, tree and scalar tail of its fp16 dots (vec_dot.h:42-146), libstdc++'s four-way reduce in
 * NormRMS and Softmax (non-linear.cpp:129-223), exp / silu from the fp16-indexed tables and the RoPE angles from the
 * host's libm -- so that logits and greedy tokens equal, bit for bit, those of the host backend compiled without fp contraction (a
 * build with -ffp-contract=fast fuses x * x + y in NormRMS and differs in last bits).  0: this backend's own order
 * (lane-parallel sums; per-operator results equal to about 1e-7, greedy tokens of a model with near-tied logits may
 * differ).  The environment variable SPY_HIP_ORDER=own at creation selects 0.  spy_hip_set_exact_order(1) forces 1 for
 * every engine while it is on.  spy_hip_llama_order returns the order the next single-token pass will use. */
int spy_hip_llama_set_order(spy_hip_llama *m, int32_t order);
int spy_hip_llama_order(spy_hip_llama *m);
/* Polls a bounded wait between the workgroups of a fused launch may spend before it gives up (default 400000, about
 * half a second).  On expiry every workgroup still runs to its end, the pass returns SPY_HIP_ETIMEOUT and the hand-over
 * words are cleared, so the next pass is a clean one.  Captured graphs are dropped (they carry the old limit). */
int spy_hip_llama_set_spin_limit(spy_hip_llama *m, uint32_t polls);
/* device pointers of the engine's buffers, for tests and profiling: name one of "k_cache",
 * "v_cache" (layer 0..n_layer-1), "x", "logits", "scores", "attn_out" (layer ignored) */
int spy_hip_llama_buffer(spy_hip_llama *m, const char *name, int32_t layer, void **ptr, size_t *bytes);
/* average duration (ms) of the HIP-event-timed single-token passes since the last call, and their
 * count; timing is recorded around every pass of spy_hip_llama_decode_greedy */
int spy_hip_llama_timing(spy_hip_llama *m, float *ms_per_pass, int32_t *n_pass);
/* average duration (microseconds) of one kernel of the single-token pass, HIP events around
 * reps x n_layer launches that walk the layers (fresh weights / caches every launch); which:
 * "qkv", "scores", "pv", "wo", "gate_up", "down", "head".  Uses the position of the last pass. */
int spy_hip_llama_kernel_time(spy_hip_llama *m, void *stream, const char *which, int32_t reps, float *us_per_launch);
/* How single-token passes are launched, as a bit mask (negative: error).
 * bit 1 (value 2): the attention part of a layer (qkv, scores, softmax + KQV) is ONE launch whose
 *   workgroups synchronise head by head; used where all its workgroups are resident (128-wide heads,
 *   8 * n_head <= compute units, n_ctx <= 5120) unless SPY_HIP_ATTN_SPLIT=1 was set at creation.
 * bit 0 is reserved (always 0). */
int spy_hip_llama_single_kernel(spy_hip_llama *m);

#ifdef __cplusplus
}
#endif
#endif
