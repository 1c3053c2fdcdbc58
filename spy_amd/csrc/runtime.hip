// Runtime entry points of the C ABI: device selection, memory, streams, events.
// Counterpart of DefaultCPUBackend's constructor and alloc/dealloc
// (backend/host/include/default_backend.h:121-156 in the Spy tree).
#include "common.cuh"

#include <stdio.h>
#include <string.h>

static int g_device = -1;
static int *g_err_flag = nullptr;   // device int, raised by kernels that detect bad operands

int *spy_hip_err_flag_ptr() { return g_err_flag; }
int spy_static_scratch_setup(int device);    // ops.hip: address of the fixed scratch array on the current device

extern "C" int spy_hip_init(int device_id) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) return (int)e;
    if (device_id < 0 || device_id >= n) return SPY_HIP_EINVAL;
    e = hipSetDevice(device_id);
    if (e != hipSuccess) return (int)e;
    if (g_device != device_id || !g_err_flag) {
        if (g_err_flag) { (void)hipFree(g_err_flag); g_err_flag = nullptr; }
        e = hipMalloc((void **)&g_err_flag, sizeof(int));
        if (e != hipSuccess) return (int)e;
        e = hipMemset(g_err_flag, 0, sizeof(int));
        if (e != hipSuccess) return (int)e;
    }
    g_device = device_id;
    return spy_static_scratch_setup(device_id);
}

extern "C" int spy_hip_device_info(char *name, int name_len, int *num_cu, size_t *total_mem, size_t *free_mem) {
    if (g_device < 0) return SPY_HIP_EINVAL;
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, g_device);
    if (e != hipSuccess) return (int)e;
    if (name && name_len > 0) { snprintf(name, (size_t)name_len, "%s (%s)", prop.name, prop.gcnArchName); }
    if (num_cu) *num_cu = prop.multiProcessorCount;
    size_t f = 0, t = 0;
    e = hipMemGetInfo(&f, &t);
    if (e != hipSuccess) return (int)e;
    if (total_mem) *total_mem = t;
    if (free_mem) *free_mem = f;
    return 0;
}

extern "C" int spy_hip_alloc(void **ptr, size_t bytes) {
    if (!ptr) return SPY_HIP_EINVAL;
    *ptr = nullptr;
    if (bytes == 0) return 0;
    return (int)hipMalloc(ptr, bytes);
}

extern "C" int spy_hip_free(void *ptr) { return ptr ? (int)hipFree(ptr) : 0; }

extern "C" int spy_hip_upload(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return 0;
    if (!dst || !src) return SPY_HIP_EINVAL;
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream);
    if (e != hipSuccess) return (int)e;
    return (int)hipStreamSynchronize((hipStream_t)stream);   // the host buffer may be pageable
}

extern "C" int spy_hip_download(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return 0;
    if (!dst || !src) return SPY_HIP_EINVAL;
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e != hipSuccess) return (int)e;
    return (int)hipStreamSynchronize((hipStream_t)stream);
}

__global__ void fill_u8_kernel(uint8_t *p, uint8_t v, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

// A fill kernel rather than hipMemsetAsync so that callers may capture it into a HIP graph.
extern "C" int spy_hip_fill_u8(void *dst, int value, size_t bytes, void *stream) {
    if (bytes == 0) return 0;
    if (!dst) return SPY_HIP_EINVAL;
    size_t blocks = (bytes + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    fill_u8_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>((uint8_t *)dst, (uint8_t)value, bytes);
    return SPY_LAUNCH_RC();
}

extern "C" int spy_hip_sync(void *stream) {
    return stream ? (int)hipStreamSynchronize((hipStream_t)stream) : (int)hipDeviceSynchronize();
}

extern "C" int spy_hip_stream_create(void **stream) {
    if (!stream) return SPY_HIP_EINVAL;
    hipStream_t s;
    hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);   // default priority
    *stream = (e == hipSuccess) ? (void *)s : nullptr;
    return (int)e;
}
extern "C" int spy_hip_stream_destroy(void *stream) { return stream ? (int)hipStreamDestroy((hipStream_t)stream) : 0; }

extern "C" int spy_hip_event_create(void **event) {
    if (!event) return SPY_HIP_EINVAL;
    hipEvent_t ev;
    hipError_t e = hipEventCreate(&ev);
    *event = (e == hipSuccess) ? (void *)ev : nullptr;
    return (int)e;
}
extern "C" int spy_hip_event_record(void *event, void *stream) { return (int)hipEventRecord((hipEvent_t)event, (hipStream_t)stream); }
extern "C" int spy_hip_event_elapsed_ms(void *start, void *stop, float *ms) {
    hipError_t e = hipEventSynchronize((hipEvent_t)stop);
    if (e != hipSuccess) return (int)e;
    return (int)hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop);
}
extern "C" int spy_hip_event_destroy(void *event) { return event ? (int)hipEventDestroy((hipEvent_t)event) : 0; }

extern "C" int spy_hip_take_error(int *flag) {
    if (!flag || !g_err_flag) return SPY_HIP_EINVAL;
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return (int)e;
    e = hipMemcpy(flag, g_err_flag, sizeof(int), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return (int)e;
    return (int)hipMemset(g_err_flag, 0, sizeof(int));
}

extern "C" const char *spy_hip_error_string(int code) {
    switch (code) {
    case 0: return "success";
    case SPY_HIP_EUNSUPPORTED: return "operator or type combination not supported by the hip backend";
    case SPY_HIP_EINVAL: return "invalid argument or shape";
    case SPY_HIP_ENOSPACE: return "scratch buffer too small";
    case SPY_HIP_ETIMEOUT: return "a bounded wait between workgroups expired; the pass's results are void";
    }
    return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
}
