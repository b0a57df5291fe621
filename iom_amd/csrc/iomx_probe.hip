// Bandwidth probes: the bare streams that the operation kernels are judged against.
// One 128-bit chunk per lane, one-shot grid, nontemporal access -- the launch shape of
// elementwise_stream_kernel without any of its address arithmetic or operations.
#include "iomx_common.hpp"

namespace iomx {

// The read-only and write-only streams use 256-lane workgroups: a wave that only loads (or
// only stores) 1 KiB ends so quickly that 64-lane workgroups are bound by the rate at which
// the dispatcher starts them (4.6 TB/s against 6.6 TB/s measured).
__global__ __launch_bounds__(256) void probe_read_kernel(const u32x4* __restrict__ a, u32x4* __restrict__ sink) {
    const u32x4 v = __builtin_nontemporal_load(a + (size_t)blockIdx.x * 256 + threadIdx.x);
    // never true for the probe's fill pattern; keeps the load alive
    if (v.x == 0x12345678u && v.y == 0x9ABCDEF0u && v.z == 0x0F1E2D3Cu) sink[threadIdx.x] = v;
}

__global__ __launch_bounds__(256) void probe_write_kernel(u32x4* __restrict__ out) {
    const u32x4 v = {blockIdx.x, threadIdx.x, 0u, 0u};
    __builtin_nontemporal_store(v, out + (size_t)blockIdx.x * 256 + threadIdx.x);
}

__global__ __launch_bounds__(64) void probe_copy_kernel(const u32x4* __restrict__ a, u32x4* __restrict__ out) {
    const size_t c = (size_t)blockIdx.x * 64 + threadIdx.x;
    __builtin_nontemporal_store(__builtin_nontemporal_load(a + c), out + c);
}

__global__ __launch_bounds__(64) void probe_add_kernel(const u32x4* __restrict__ a, const u32x4* __restrict__ b,
                                                       u32x4* __restrict__ out) {
    const size_t c = (size_t)blockIdx.x * 64 + threadIdx.x;
    u32x4 v = __builtin_nontemporal_load(a + c);
    const u32x4 w = __builtin_nontemporal_load(b + c);
    v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
    __builtin_nontemporal_store(v, out + c);
}

// The memory side of the resident RMSNorm kernel and nothing else: a 1024-lane workgroup loads
// four chunks per lane (64 KiB, one BF16 band of 2048 features), meets at a barrier and stores.
__global__ __launch_bounds__(1024) void probe_held_copy_kernel(const u32x4* __restrict__ a, u32x4* __restrict__ out) {
    const size_t base = (size_t)blockIdx.x * 4096 + threadIdx.x;
    u32x4 held[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) held[k] = __builtin_nontemporal_load(a + base + k * 1024);
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; ++k) __builtin_nontemporal_store(held[k], out + base + k * 1024);
}

}  // namespace iomx

using namespace iomx;

extern "C" int iomx_probe_stream(int mode, const void* a, const void* b, void* out, uint64_t bytes,
                                 iomx_stream_t stream) {
    if (bytes == 0 || bytes % 4096 != 0 || bytes / 4096 > 0x7FFFFFFFull / 4) return IOMX_ERR_INVALID;
    const uintptr_t align = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)
                          | reinterpret_cast<uintptr_t>(out);
    if ((align & 15u) != 0 || !out) return IOMX_ERR_INVALID;
    const hipStream_t s = native(stream);
    const uint64_t chunks = bytes / 16;
    const u32x4* pa = static_cast<const u32x4*>(a);
    const u32x4* pb = static_cast<const u32x4*>(b);
    u32x4* po = static_cast<u32x4*>(out);
    switch (mode) {
        case IOMX_PROBE_READ:
            if (!a) return IOMX_ERR_INVALID;
            hipLaunchKernelGGL(probe_read_kernel, dim3((uint32_t)(chunks / 256)), dim3(256), 0, s, pa, po);
            record_launch("probe_read", (uint32_t)(chunks / 256), 256, chunks);
            break;
        case IOMX_PROBE_WRITE:
            hipLaunchKernelGGL(probe_write_kernel, dim3((uint32_t)(chunks / 256)), dim3(256), 0, s, po);
            record_launch("probe_write", (uint32_t)(chunks / 256), 256, chunks);
            break;
        case IOMX_PROBE_COPY:
            if (!a) return IOMX_ERR_INVALID;
            hipLaunchKernelGGL(probe_copy_kernel, dim3((uint32_t)(chunks / 64)), dim3(64), 0, s, pa, po);
            record_launch("probe_copy", (uint32_t)(chunks / 64), 64, chunks);
            break;
        case IOMX_PROBE_ADD:
            if (!a || !b) return IOMX_ERR_INVALID;
            hipLaunchKernelGGL(probe_add_kernel, dim3((uint32_t)(chunks / 64)), dim3(64), 0, s, pa, pb, po);
            record_launch("probe_add", (uint32_t)(chunks / 64), 64, chunks);
            break;
        case IOMX_PROBE_HELD_COPY:
            if (!a || bytes % 65536 != 0) return IOMX_ERR_INVALID;
            hipLaunchKernelGGL(probe_held_copy_kernel, dim3((uint32_t)(chunks / 4096)), dim3(1024), 0, s, pa, po);
            record_launch("probe_held_copy", (uint32_t)(chunks / 4096), 1024, chunks);
            break;
        default:
            return IOMX_ERR_INVALID;
    }
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}
