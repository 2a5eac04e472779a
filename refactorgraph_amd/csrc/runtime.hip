// Device and memory entry points of the C ABI: the HIP calls a hardware::Device /
// hardware::Memory backend needs (the reference's CUDA equivalents live in
// src/02hardware/src/devices/nvidia/{device.cc,memory.cc}).
#include "common.hpp"

extern "C" {

int rg_hip_device_count(int *count) {
    if (!count) return RG_HIP_E_ARGUMENT;
    return static_cast<int>(hipGetDeviceCount(count));
}

int rg_hip_set_device(int card) { return static_cast<int>(hipSetDevice(card)); }

int rg_hip_mem_info(size_t *free_bytes, size_t *total_bytes) {
    if (!free_bytes || !total_bytes) return RG_HIP_E_ARGUMENT;
    return static_cast<int>(hipMemGetInfo(free_bytes, total_bytes));
}

int rg_hip_device_name(char *buf, size_t len) {
    if (!buf || len == 0) return RG_HIP_E_ARGUMENT;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return static_cast<int>(e);
    size_t i = 0;
    for (; i + 1 < len && prop.gcnArchName[i]; ++i) buf[i] = prop.gcnArchName[i];
    buf[i] = '\0';
    return 0;
}

int rg_hip_malloc(void **ptr, size_t bytes) {
    if (!ptr) return RG_HIP_E_ARGUMENT;
    return static_cast<int>(hipMalloc(ptr, bytes));
}

int rg_hip_free(void *ptr) { return static_cast<int>(hipFree(ptr)); }

int rg_hip_memcpy_h2d(void *dst, const void *src, size_t bytes) {
    return static_cast<int>(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
}

int rg_hip_memcpy_d2h(void *dst, const void *src, size_t bytes) {
    return static_cast<int>(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
}

int rg_hip_memcpy_d2d(void *dst, const void *src, size_t bytes) {
    return static_cast<int>(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice));
}

int rg_hip_memcpy_d2d_async(void *dst, const void *src, size_t bytes, void *stream) {
    return static_cast<int>(
        hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, rg::as_stream(stream)));
}

int rg_hip_sync(void) { return static_cast<int>(hipDeviceSynchronize()); }

int rg_hip_stream_create(void **stream) {
    if (!stream) return RG_HIP_E_ARGUMENT;
    hipStream_t s = nullptr;
    const hipError_t rc = hipStreamCreate(&s);
    *stream = s;
    return static_cast<int>(rc);
}
int rg_hip_stream_destroy(void *stream) { return static_cast<int>(hipStreamDestroy(rg::as_stream(stream))); }
int rg_hip_stream_sync(void *stream) { return static_cast<int>(hipStreamSynchronize(rg::as_stream(stream))); }

int rg_hip_graph_begin(void *stream) {
    if (!stream) return RG_HIP_E_ARGUMENT;  // the default stream cannot record
    return static_cast<int>(hipStreamBeginCapture(rg::as_stream(stream), hipStreamCaptureModeRelaxed));
}
int rg_hip_graph_end(void *stream, void **graph_exec) {
    if (!stream || !graph_exec) return RG_HIP_E_ARGUMENT;
    *graph_exec = nullptr;
    hipGraph_t graph = nullptr;
    hipError_t rc = hipStreamEndCapture(rg::as_stream(stream), &graph);
    if (rc != hipSuccess) return static_cast<int>(rc);
    hipGraphExec_t exec = nullptr;
    rc = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void) hipGraphDestroy(graph);
    if (rc != hipSuccess) return static_cast<int>(rc);
    *graph_exec = exec;
    return 0;
}
int rg_hip_graph_launch(void *graph_exec, void *stream) {
    if (!graph_exec) return RG_HIP_E_ARGUMENT;
    return static_cast<int>(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), rg::as_stream(stream)));
}
int rg_hip_graph_destroy(void *graph_exec) {
    if (!graph_exec) return 0;
    return static_cast<int>(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
}

const char *rg_hip_error_string(int status) {
    switch (status) {
        case RG_HIP_E_UNSUPPORTED: return "rg_hip: no kernel for this dtype/shape";
        case RG_HIP_E_ARGUMENT: return "rg_hip: invalid argument";
        case RG_HIP_E_WORKSPACE: return "rg_hip: workspace too small";
        default: return hipGetErrorString(static_cast<hipError_t>(status));
    }
}

}  // extern "C"
