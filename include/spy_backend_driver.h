/*
 * Test driver of the C++ host side (spy::hip::HIPBackend behind the spy::Backend interface).
 *
 * These entry points have no counterpart in the Spy tree: they wrap what its CLI does with a backend
 * -- build the LLaMA graph (model/src/llm/model/llama.cpp:86-313), execute it operator by operator
 * through Backend::submit (backend/distributor/include/scheduler/default_scheduler.h:46-229) -- so
 * that the parity tests can drive the C++ class from Python.  POD only, host pointers in, host
 * logits out.  Library: spy_amd/libspy_backend.so (needs spy_amd/libspy_hip.so next to it).
 */
#ifndef SPY_BACKEND_DRIVER_H
#define SPY_BACKEND_DRIVER_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One GGUF-named weight tensor in HOST memory, native block layout; `type` uses the NumberType
 * codes (0 FP32, 1 FP16, 2 Q4_0, 8 Q8_0, 12 Q4_K, 14 Q6_K); cols is the contiguous dimension. */
typedef struct spy_host_tensor {
    const char *name;
    const void *data;
    int32_t type;
    int64_t rows, cols;
} spy_host_tensor;

typedef struct spy_host_model spy_host_model;

/* backend_name is a BackendFactory key ("hip:default").  Returns 0, -1 if the factory has no such
 * backend, -2 on bad arguments, 2 if device memory for the KV caches could not be allocated. */
int spy_host_model_create(const spy_host_tensor *tensors, int n_tensors, int n_layer, int n_embd, int n_head, int n_ff, int n_vocab,
                          int n_ctx, float eps, float rope_freq_base, const char *backend_name, spy_host_model **out);
/* One pass over n_token tokens after n_past cached ones; logits (may be NULL) gets n_token * n_vocab floats. */
int spy_host_model_forward(spy_host_model *m, const int32_t *tokens, int n_token, int n_past, float *logits);
/* Counters of the last pass / since creation: operator nodes in the graph, submits, backend allocations and releases. */
int spy_host_model_stats(spy_host_model *m, int64_t *n_ops, int64_t *n_submit, int64_t *n_alloc, int64_t *n_free);
/* Copies one layer's K (which = 0) or V (1) cache, n_ctx * n_embd fp16 values, to host memory. */
int spy_host_model_cache(spy_host_model *m, int layer, int which, void *dst_host);
int spy_host_model_destroy(spy_host_model *m);

/* One unary operator node through Backend::submit: x = f32 [ne1][ne0] in host memory (an IO node), the result in host memory
 * too.  op: 0 Relu, 1 Silu, 2 Quantize to target_type (NumberType code; out_bytes = the result's size in that type).
 * Returns 0, -1 if the backend does not take the operator or conversion, -2 on bad arguments, else the backend's error. */
int spy_host_unary_through_submit(const char *backend_name, int op, const float *x, int64_t ne0, int64_t ne1, int target_type, void *out, int64_t out_bytes);

#ifdef __cplusplus
}
#endif
#endif
