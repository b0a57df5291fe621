// Device, memory, stream and event entry points of libiomx: the only
// translation units that touch the HIP runtime are the ones in this directory.
#include "iomx_common.hpp"

#include <cstdio>

namespace iomx {

namespace {
thread_local iomx_launch_info g_last_launch = {};
}

void record_launch(const char* kernel, uint32_t grid, uint32_t block, uint64_t work) {
    std::snprintf(g_last_launch.kernel, sizeof(g_last_launch.kernel), "%s", kernel);
    g_last_launch.grid = grid;
    g_last_launch.block = block;
    g_last_launch.work_items = work;
}

// IOMX_OK when [ptr, ptr + bytes) lies inside one device allocation.
int device_range(const void* ptr, size_t bytes) {
    hipDeviceptr_t base = nullptr;
    size_t size = 0;
    if (hipMemGetAddressRange(&base, &size, const_cast<void*>(ptr)) != hipSuccess) {
        (void)hipGetLastError();
        return IOMX_ERR_INVALID;
    }
    const uintptr_t b = reinterpret_cast<uintptr_t>(base), p = reinterpret_cast<uintptr_t>(ptr);
    if (p < b || bytes > size || p - b > size - bytes) return IOMX_ERR_INVALID;
    return IOMX_OK;
}

__global__ void fill_kernel(u32x4* __restrict__ dst, uint64_t chunks, uint32_t word) {
    const u32x4 v = {word, word, word, word};
    for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < chunks;
         i += (uint64_t)gridDim.x * blockDim.x)
        dst[i] = v;
}

// One lane stores a word for the host to see: stream order puts it behind everything
// submitted before, the system-scope release behind their writes.
__global__ void write_word_kernel(uint32_t* word, uint32_t value) {
    __hip_atomic_store(word, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

__global__ void fill_bytes_kernel(uint8_t* __restrict__ dst, uint64_t bytes, uint8_t value) {
    for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < bytes;
         i += (uint64_t)gridDim.x * blockDim.x)
        dst[i] = value;
}

}  // namespace iomx

using namespace iomx;

extern "C" {

const char* iomx_error_string(int status) {
    switch (status) {
        case IOMX_OK: return "ok";
        case IOMX_ERR_INVALID: return "iomx: invalid request";
        case IOMX_ERR_UNSUPPORTED: return "iomx: unsupported leaf or shape";
        case IOMX_ERR_OVERFLOW: return "iomx: address arithmetic overflows";
        case IOMX_ERR_EXHAUSTED: return "iomx: request exceeds the fixed scratch array";
        default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "iomx: unknown status";
}

int iomx_device_count(int* count) {
    if (!count) return IOMX_ERR_INVALID;
    *count = 0;
    IOMX_HIP(hipGetDeviceCount(count));
    return IOMX_OK;
}

int iomx_set_device(int ordinal) {
    IOMX_HIP(hipSetDevice(ordinal));
    return IOMX_OK;
}

int iomx_get_device(int* ordinal) {
    if (!ordinal) return IOMX_ERR_INVALID;
    IOMX_HIP(hipGetDevice(ordinal));
    return IOMX_OK;
}

int iomx_get_device_props(int ordinal, iomx_device_props* props) {
    if (!props) return IOMX_ERR_INVALID;
    hipDeviceProp_t p;
    IOMX_HIP(hipGetDeviceProperties(&p, ordinal));
    std::memset(props, 0, sizeof(*props));
    std::snprintf(props->name, sizeof(props->name), "%s", p.gcnArchName);
    props->compute_units = p.multiProcessorCount;
    props->wavefront_size = p.warpSize;
    props->lds_bytes_per_cu = static_cast<int>(p.sharedMemPerBlock);
    props->global_bytes = p.totalGlobalMem;
    return IOMX_OK;
}

int iomx_device_synchronize(void) {
    IOMX_HIP(hipDeviceSynchronize());
    return IOMX_OK;
}

int iomx_malloc(void** ptr, size_t bytes) {
    if (!ptr) return IOMX_ERR_INVALID;
    *ptr = nullptr;
    IOMX_HIP(hipMalloc(ptr, bytes));
    return IOMX_OK;
}

int iomx_free(void* ptr) {
    IOMX_HIP(hipFree(ptr));
    return IOMX_OK;
}

int iomx_host_alloc(void** ptr, size_t bytes) {
    if (!ptr) return IOMX_ERR_INVALID;
    *ptr = nullptr;
    IOMX_HIP(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
    return IOMX_OK;
}

int iomx_host_free(void* ptr) {
    IOMX_HIP(hipHostFree(ptr));
    return IOMX_OK;
}

int iomx_pointer_device(const void* ptr, int* ordinal) {
    if (!ptr || !ordinal) return IOMX_ERR_INVALID;
    hipPointerAttribute_t attr;
    const hipError_t e = hipPointerGetAttributes(&attr, ptr);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return (int)e;
    }
    if (attr.type != hipMemoryTypeDevice) return IOMX_ERR_INVALID;
    *ordinal = attr.device;
    return IOMX_OK;
}

// A fill kernel rather than hipMemsetAsync, so that a caller may capture it
// into a HIP graph.
int iomx_fill_async(void* ptr, uint8_t value, size_t bytes, iomx_stream_t stream) {
    if (bytes == 0) return IOMX_OK;
    if (!ptr) return IOMX_ERR_INVALID;
    const uint32_t word = 0x01010101u * value;
    if ((reinterpret_cast<uintptr_t>(ptr) & 15u) == 0 && (bytes & 15u) == 0) {
        const uint64_t chunks = bytes / 16;
        const uint32_t grid = (uint32_t)((chunks + 255) / 256 > 65536 ? 65536 : (chunks + 255) / 256);
        hipLaunchKernelGGL(fill_kernel, dim3(grid), dim3(256), 0, native(stream),
                           static_cast<u32x4*>(ptr), chunks, word);
    } else {
        const uint32_t grid = (uint32_t)((bytes + 255) / 256 > 65536 ? 65536 : (bytes + 255) / 256);
        hipLaunchKernelGGL(fill_bytes_kernel, dim3(grid), dim3(256), 0, native(stream),
                           static_cast<uint8_t*>(ptr), (uint64_t)bytes, value);
    }
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}

// The blocking copies check the device side of the request against the allocation it
// points into before the runtime sees it: a range that runs past its allocation comes back
// as IOMX_ERR_INVALID instead of as a fault inside a staging copy.
int iomx_memcpy_h2d(void* dst, const void* src, size_t bytes) {
    if (bytes == 0) return IOMX_OK;
    if (!dst || !src) return IOMX_ERR_INVALID;
    IOMX_TRY(device_range(dst, bytes));
    IOMX_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return IOMX_OK;
}

int iomx_memcpy_d2h(void* dst, const void* src, size_t bytes) {
    if (bytes == 0) return IOMX_OK;
    if (!dst || !src) return IOMX_ERR_INVALID;
    IOMX_TRY(device_range(src, bytes));
    IOMX_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return IOMX_OK;
}

int iomx_memcpy_h2d_async(void* dst, const void* src, size_t bytes, iomx_stream_t stream) {
    IOMX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, native(stream)));
    return IOMX_OK;
}

int iomx_memcpy_d2h_async(void* dst, const void* src, size_t bytes, iomx_stream_t stream) {
    IOMX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, native(stream)));
    return IOMX_OK;
}

int iomx_memcpy_d2d_async(void* dst, const void* src, size_t bytes, iomx_stream_t stream) {
    IOMX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, native(stream)));
    return IOMX_OK;
}

int iomx_stream_create(iomx_stream_t* stream) {
    if (!stream) return IOMX_ERR_INVALID;
    hipStream_t s = nullptr;
    IOMX_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = reinterpret_cast<iomx_stream_t>(s);
    return IOMX_OK;
}

int iomx_stream_destroy(iomx_stream_t stream) {
    IOMX_HIP(hipStreamDestroy(native(stream)));
    return IOMX_OK;
}

int iomx_stream_synchronize(iomx_stream_t stream) {
    IOMX_HIP(hipStreamSynchronize(native(stream)));
    return IOMX_OK;
}

int iomx_stream_begin_capture(iomx_stream_t stream) {
    if (!stream) return IOMX_ERR_INVALID;          // the null stream cannot be captured
    IOMX_HIP(hipStreamBeginCapture(native(stream), hipStreamCaptureModeThreadLocal));
    return IOMX_OK;
}

int iomx_stream_end_capture(iomx_stream_t stream, iomx_graph_t* graph) {
    if (!stream || !graph) return IOMX_ERR_INVALID;
    hipGraph_t recorded = nullptr;
    IOMX_HIP(hipStreamEndCapture(native(stream), &recorded));
    hipGraphExec_t exec = nullptr;
    const hipError_t status = hipGraphInstantiate(&exec, recorded, nullptr, nullptr, 0);
    (void)hipGraphDestroy(recorded);
    IOMX_HIP(status);
    *graph = reinterpret_cast<iomx_graph_t>(exec);
    return IOMX_OK;
}

int iomx_graph_launch(iomx_graph_t graph, iomx_stream_t stream) {
    if (!graph) return IOMX_ERR_INVALID;
    IOMX_HIP(hipGraphLaunch(reinterpret_cast<hipGraphExec_t>(graph), native(stream)));
    return IOMX_OK;
}

int iomx_graph_destroy(iomx_graph_t graph) {
    if (graph) IOMX_HIP(hipGraphExecDestroy(reinterpret_cast<hipGraphExec_t>(graph)));
    return IOMX_OK;
}

int iomx_event_create(iomx_event_t* event, int enable_timing) {
    if (!event) return IOMX_ERR_INVALID;
    hipEvent_t e = nullptr;
    IOMX_HIP(hipEventCreateWithFlags(&e, enable_timing ? hipEventDefault : hipEventDisableTiming));
    *event = reinterpret_cast<iomx_event_t>(e);
    return IOMX_OK;
}

int iomx_event_destroy(iomx_event_t event) {
    IOMX_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
    return IOMX_OK;
}

int iomx_event_record(iomx_event_t event, iomx_stream_t stream) {
    IOMX_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), native(stream)));
    return IOMX_OK;
}

int iomx_event_synchronize(iomx_event_t event) {
    IOMX_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
    return IOMX_OK;
}

int iomx_event_query(iomx_event_t event, int* done) {
    if (!done) return IOMX_ERR_INVALID;
    const hipError_t e = hipEventQuery(reinterpret_cast<hipEvent_t>(event));
    if (e == hipSuccess) { *done = 1; return IOMX_OK; }
    if (e == hipErrorNotReady) { (void)hipGetLastError(); *done = 0; return IOMX_OK; }
    return (int)e;
}

int iomx_host_device_address(void* host, void** device) {
    if (!host || !device) return IOMX_ERR_INVALID;
    *device = nullptr;
    IOMX_HIP(hipHostGetDevicePointer(device, host, 0));
    return IOMX_OK;
}

int iomx_stream_write_word(iomx_stream_t stream, void* device_word, uint32_t value) {
    if (!device_word || (reinterpret_cast<uintptr_t>(device_word) & 3u)) return IOMX_ERR_INVALID;
    hipLaunchKernelGGL(write_word_kernel, dim3(1), dim3(1), 0, native(stream),
                       static_cast<uint32_t*>(device_word), value);
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}

int iomx_event_elapsed_ms(iomx_event_t start, iomx_event_t stop, float* ms) {
    if (!ms) return IOMX_ERR_INVALID;
    IOMX_HIP(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start),
                                 reinterpret_cast<hipEvent_t>(stop)));
    return IOMX_OK;
}

int iomx_last_launch(iomx_launch_info* info) {
    if (!info) return IOMX_ERR_INVALID;
    *info = g_last_launch;
    return IOMX_OK;
}

}  // extern "C"
