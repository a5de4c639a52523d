// Library/device helpers of the C ABI: memory, streams, events, fills, error strings.
#include <cstdio>
#include <cstring>
#include "host_util.hpp"

namespace {
__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, size_t n) {
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}
}  // namespace

using namespace glide;

extern "C" {

const char* glide_hip_version(void) { return "glide-hip 0.1 (gfx950)"; }

const char* glide_hip_error_string(int code) {
    switch (code) {
        case GLIDE_OK: return "success";
        case GLIDE_ERR_UNSUPPORTED: return "size outside the supported range";
        case GLIDE_ERR_BAD_ARGUMENT: return "bad argument";
        case GLIDE_ERR_NO_DEVICE: return "no HIP device";
        default: return code > 0 ? hipGetErrorString(static_cast<hipError_t>(code)) : "unknown error";
    }
}

int glide_hip_set_device(int device) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n == 0) return GLIDE_ERR_NO_DEVICE;
    GLIDE_HIP_TRY(hipSetDevice(device));
    return GLIDE_OK;
}

int glide_hip_device_info(char* name, size_t name_len, int* compute_units, size_t* total_mem) {
    int dev = 0;
    GLIDE_HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    GLIDE_HIP_TRY(hipGetDeviceProperties(&prop, dev));
    if (name && name_len) {
        std::snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (total_mem) *total_mem = prop.totalGlobalMem;
    return GLIDE_OK;
}

int glide_hip_mem_info(size_t* free_bytes, size_t* total_bytes) {
    size_t f = 0, t = 0;
    GLIDE_HIP_TRY(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return GLIDE_OK;
}

int glide_hip_malloc(void** ptr, size_t bytes) {
    if (!ptr) return GLIDE_ERR_BAD_ARGUMENT;
    GLIDE_HIP_TRY(hipMalloc(ptr, bytes ? bytes : 1));
    return GLIDE_OK;
}
int glide_hip_free(void* ptr) {
    GLIDE_HIP_TRY(hipFree(ptr));
    return GLIDE_OK;
}
int glide_hip_host_alloc_pinned(void** ptr, size_t bytes) {
    if (!ptr) return GLIDE_ERR_BAD_ARGUMENT;
    GLIDE_HIP_TRY(hipHostMalloc(ptr, bytes ? bytes : 1, hipHostMallocDefault));
    return GLIDE_OK;
}
int glide_hip_host_free_pinned(void* ptr) {
    GLIDE_HIP_TRY(hipHostFree(ptr));
    return GLIDE_OK;
}
int glide_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
    GLIDE_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    GLIDE_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return GLIDE_OK;
}
int glide_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
    GLIDE_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    GLIDE_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return GLIDE_OK;
}
int glide_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream) {
    GLIDE_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return GLIDE_OK;
}
int glide_hip_memcpy_h2d_async(void* dst, const void* src, size_t bytes, void* stream) {
    GLIDE_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    return GLIDE_OK;
}
int glide_hip_memcpy_d2h_async(void* dst, const void* src, size_t bytes, void* stream) {
    GLIDE_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    return GLIDE_OK;
}
int glide_hip_stream_wait_event(void* stream, void* event) {
    GLIDE_HIP_TRY(hipStreamWaitEvent(as_stream(stream), static_cast<hipEvent_t>(event), 0));
    return GLIDE_OK;
}
int glide_hip_fill_u32(uint32_t* ptr, uint32_t value, size_t count, void* stream) {
    if (!ptr) return GLIDE_ERR_BAD_ARGUMENT;
    if (count == 0) return GLIDE_OK;
    const unsigned blocks = static_cast<unsigned>(count / 256 + 1 > 4096 ? 4096 : count / 256 + 1);
    hipLaunchKernelGGL(fill_u32_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), ptr, value, count);
    return launch_status();
}
int glide_hip_stream_create(void** stream) {
    if (!stream) return GLIDE_ERR_BAD_ARGUMENT;
    hipStream_t s;
    GLIDE_HIP_TRY(hipStreamCreate(&s));  // default priority
    *stream = s;
    return GLIDE_OK;
}
int glide_hip_stream_destroy(void* stream) {
    GLIDE_HIP_TRY(hipStreamDestroy(as_stream(stream)));
    return GLIDE_OK;
}
int glide_hip_stream_synchronize(void* stream) {
    GLIDE_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return GLIDE_OK;
}
int glide_hip_event_create(void** event) {
    if (!event) return GLIDE_ERR_BAD_ARGUMENT;
    hipEvent_t e;
    GLIDE_HIP_TRY(hipEventCreate(&e));
    *event = e;
    return GLIDE_OK;
}
int glide_hip_event_destroy(void* event) {
    GLIDE_HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return GLIDE_OK;
}
int glide_hip_event_record(void* event, void* stream) {
    GLIDE_HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)));
    return GLIDE_OK;
}
int glide_hip_event_elapsed_ms(void* start, void* stop, float* ms) {
    if (!ms) return GLIDE_ERR_BAD_ARGUMENT;
    GLIDE_HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
    GLIDE_HIP_TRY(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return GLIDE_OK;
}

}  // extern "C"
