// Calibration kernels of the measurement harness (include/hogwild_bench.h): a plain streaming read, the achievable
// HBM rate the attention kernel is compared with, and a plain copy of known size that scales the FETCH_SIZE /
// WRITE_SIZE hardware counters.  Built into libhogwild_bench.so, separate from the product library.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/hogwild_bench.h"
#include "../../include/hogwild_hip.h"

namespace {

typedef unsigned int u32;
typedef u32 u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void stream_read_chunked_kernel(const u32x4* src, size_t n16, u32* sink) {
    // A workgroup takes 32 KB of consecutive memory per round, eight independent 16-byte loads per thread (a wave has
    // 8 KB in flight), so that a launch with one workgroup per compute unit is bound by memory and not by one load's
    // latency per round.  (Eight loads a whole grid stride apart, each in another 2 MB page, cost a quarter of the rate.)
    constexpr int UN = 8;
    u32x4 acc = {0, 0, 0, 0};
    const size_t chunk = (size_t)UN * blockDim.x;                       // 16-byte pieces per workgroup and round
    const size_t rounds = n16 / chunk;
    for (size_t r = blockIdx.x; r < rounds; r += gridDim.x) {
        const u32x4* p = src + r * chunk + threadIdx.x;
        u32x4 x[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) x[u] = __builtin_nontemporal_load(p + u * blockDim.x);
#pragma unroll
        for (int u = 0; u < UN; ++u) acc ^= x[u];
    }
    for (size_t i = rounds * chunk + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
        acc ^= __builtin_nontemporal_load(src + i);
    u32 r = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (r == 0x9e3779b9u) sink[threadIdx.x] = r;   // practically never: keeps the loads alive without a store stream
}

// one 16-byte load per thread and round: with eight workgroups per compute unit (what hw_stream_read launches) this is
// the fastest plain read found on this device
__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4* src, size_t n16, u32* sink) {
    u32x4 acc = {0, 0, 0, 0};
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) {
        u32x4 x = __builtin_nontemporal_load(src + i);
        acc ^= x;
    }
    u32 r = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (r == 0x9e3779b9u) sink[threadIdx.x] = r;   // practically never: keeps the loads alive without a store stream
}

__global__ __launch_bounds__(256) void stream_copy_kernel(u32x4* dst, const u32x4* src, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

extern "C" {

int hw_stream_read(const void* src, size_t bytes, uint32_t* sink, void* stream) {
    if (src == nullptr || sink == nullptr) return HW_ERR_NULL;
    if (bytes % 16 != 0 || !aligned16(src)) return HW_ERR_ALIGN;
    hipLaunchKernelGGL(stream_read_kernel, dim3(2048), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       reinterpret_cast<const u32x4*>(src), bytes / 16, sink);
    return (int)hipGetLastError();
}

int hw_stream_read_shaped(const void* src, size_t bytes, uint32_t* sink, int workgroups, void* stream) {
    if (src == nullptr || sink == nullptr) return HW_ERR_NULL;
    if (bytes % 16 != 0 || !aligned16(src)) return HW_ERR_ALIGN;
    if (workgroups < 1 || workgroups > 65536) return HW_ERR_SHAPE;
    hipLaunchKernelGGL(stream_read_chunked_kernel, dim3(workgroups), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       reinterpret_cast<const u32x4*>(src), bytes / 16, sink);
    return (int)hipGetLastError();
}

int hw_stream_copy(void* dst, const void* src, size_t bytes, void* stream) {
    if (src == nullptr || dst == nullptr) return HW_ERR_NULL;
    if (bytes % 16 != 0 || !aligned16(src) || !aligned16(dst)) return HW_ERR_ALIGN;
    hipLaunchKernelGGL(stream_copy_kernel, dim3(2048), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       reinterpret_cast<u32x4*>(dst), reinterpret_cast<const u32x4*>(src), bytes / 16);
    return (int)hipGetLastError();
}

}  // extern "C"
