// Single-token-pass kernels instantiated for Q4_K matrices.
#include "decode_launch.cuh"
#include "exact_launch.cuh"

int spy_enqueue_kernel_q4_k(spy_hip_llama *m, hipStream_t st, int which, int il) { return enqueue_any<SPY_HIP_Q4_K>(m, st, which, il); }
int spy_probe_attn_layer_q4_k(spy_hip_llama *m, int il) { return launch_attn_layer<SPY_HIP_Q4_K>(m, nullptr, il, true); }
int spy_enqueue_exact_q4_k(spy_hip_llama *m, hipStream_t st, int which, int il) { return enqueue_exact<SPY_HIP_Q4_K>(m, st, which, il); }
int spy_exact_matvec_q4_k(hipStream_t st, const void *w, const float *x, float *out, int M, int K) { return xg_plain<SPY_HIP_Q4_K>(st, w, x, out, M, K); }
int spy_own_matvec_q4_k(hipStream_t st, const void *w, const float *x, float *out, int M, int K) { return wave_plain<SPY_HIP_Q4_K>(st, w, x, out, M, K); }
int spy_exact_matvec_prepare_q4_k() { return xg_plain_prepare<SPY_HIP_Q4_K>(); }
