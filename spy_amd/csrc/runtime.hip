// Runtime entry points of the C ABI: device selection, memory, streams, events.
// Counterpart of DefaultCPUBackend's constructor and alloc/dealloc
// (backend/host/include/default_backend.h:121-156 in the Spy tree).
#include "common.cuh"

#include <stdio.h>
#include <string.h>

#include <map>
#include <mutex>
#include <utility>

// Per-device state of the library.  Everything an operator call needs beyond its operands is set up by spy_hip_init, once per
// device and kept until the process ends, so that the spy_hip_op_* entry points neither allocate nor synchronise:
//   err_flag   device int raised by kernels that detect bad operands
//   (the exp / silu tables of the exact-order operators and their Rope tables live in exact_order.hip, same discipline)
#define SPY_MAX_DEVICES 64
static int g_device = -1;
static int *g_err_flag[SPY_MAX_DEVICES];
static std::mutex g_runtime_mu;

int *spy_hip_err_flag_ptr() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SPY_MAX_DEVICES) return nullptr;
    return g_err_flag[dev];
}
int spy_static_scratch_setup(int device);    // ops.hip: address of the fixed scratch array on the current device
int spy_exact_device_setup();                // exact_order.hip: the exp / silu tables of the current device

// A kernel's dynamic-LDS limit (hipFuncAttributeMaxDynamicSharedMemorySize) belongs to the kernel function on a device for the
// whole process, whoever launches it: it is kept here per (device, kernel) and only ever raised, so that an engine or operator
// call with a smaller need never lowers it under a launch that was sized for more.
int spy_raise_lds_limit(const void *kern, size_t lds) {
    if (lds <= 48 * 1024) return 0;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    static std::map<std::pair<int, const void *>, size_t> limit;
    std::lock_guard<std::mutex> lock(g_runtime_mu);
    size_t &have = limit[std::make_pair(dev, kern)];
    if (lds > have) {
        e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        have = lds;
    }
    return 0;
}

extern "C" int spy_hip_init(int device_id) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) return (int)e;
    if (device_id < 0 || device_id >= n || device_id >= SPY_MAX_DEVICES) return SPY_HIP_EINVAL;
    e = hipSetDevice(device_id);
    if (e != hipSuccess) return (int)e;
    {
        std::lock_guard<std::mutex> lock(g_runtime_mu);
        if (!g_err_flag[device_id]) {
            int *p = nullptr;
            e = hipMalloc((void **)&p, sizeof(int));
            if (e != hipSuccess) return (int)e;
            e = hipMemset(p, 0, sizeof(int));
            if (e != hipSuccess) { (void)hipFree(p); return (int)e; }
            g_err_flag[device_id] = p;
        }
        g_device = device_id;
    }
    const int rc = spy_exact_device_setup();
    if (rc) return rc;
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
    int *dflag = spy_hip_err_flag_ptr();
    if (!flag || !dflag) return SPY_HIP_EINVAL;
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return (int)e;
    e = hipMemcpy(flag, dflag, sizeof(int), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return (int)e;
    return (int)hipMemset(dflag, 0, sizeof(int));
}

// ---- stream capture: a sequence of calls on `stream` recorded once and replayed --------------------------------------------
// Thin wrappers so that a caller without the HIP headers (a binding in another language, the tests) can put operator calls
// under capture.  Between begin and end every call on the stream is recorded instead of run; calls that would allocate or
// synchronise fail there, which is what the operator entry points are built to avoid.
extern "C" int spy_hip_capture_begin(void *stream) {
    if (!stream) return SPY_HIP_EINVAL;                         // the null stream cannot be captured
    return (int)hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal);
}
extern "C" int spy_hip_capture_end(void *stream, void **graph_exec) {
    if (!stream || !graph_exec) return SPY_HIP_EINVAL;
    *graph_exec = nullptr;
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture((hipStream_t)stream, &g);
    if (e != hipSuccess) return (int)e;
    hipGraphExec_t x = nullptr;
    e = hipGraphInstantiate(&x, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) return (int)e;
    *graph_exec = (void *)x;
    return 0;
}
extern "C" int spy_hip_graph_launch(void *graph_exec, void *stream) {
    if (!graph_exec) return SPY_HIP_EINVAL;
    return (int)hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream);
}
extern "C" int spy_hip_graph_destroy(void *graph_exec) { return graph_exec ? (int)hipGraphExecDestroy((hipGraphExec_t)graph_exec) : 0; }

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
