// A pure read stream over device memory: the yardstick for "what does this GPU deliver to a kernel
// that only reads".  Not one of the reference's operators; the benchmark times it next to the
// attention kernels so that their fraction of the 8 TB/s HBM peak can be read against the
// fraction a kernel with no arithmetic and no stores reaches.
#include "l3_device.hpp"
#include "l3_host.hpp"

namespace l3 {

namespace {

constexpr int kStreamThreads = 512;
constexpr int kStreamUnroll = 8;   // 16-byte loads a lane has in flight: 64 KiB per workgroup and trip

// Trip i of workgroup w covers the 64 KiB block i * gridDim.x + w: at any moment the workgroups
// together read one contiguous stretch of gridDim.x * 64 KiB, which spreads over every memory
// channel whatever the buffer's size.
__global__ void __launch_bounds__(kStreamThreads)
hbm_read_stream_kernel(const uint4* __restrict__ src, int64_t n16, uint32_t* __restrict__ sink) {
    constexpr int64_t kBlock = int64_t(kStreamThreads) * kStreamUnroll;
    uint32_t acc = 0;
    for (int64_t base = int64_t(blockIdx.x) * kBlock; base < n16; base += int64_t(gridDim.x) * kBlock) {
        uint4 v[kStreamUnroll];
#pragma unroll
        for (int u = 0; u < kStreamUnroll; ++u) {
            const int64_t i = base + u * kStreamThreads + threadIdx.x;
            v[u] = (i < n16) ? load16_stream(reinterpret_cast<const uint16_t*>(src + i)) : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int u = 0; u < kStreamUnroll; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x9e3779b9u) *sink = acc;   // keeps the loads; practically never taken
}

// The same sweep with every 16 bytes read written once to `dst`: what a row-wise operator (one read
// and one write per element, no arithmetic to speak of) can reach.  Stores are plain, as in the operators.
template <int UNROLL>
__global__ void __launch_bounds__(kStreamThreads)
hbm_rw_stream_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, int64_t n16) {
    constexpr int64_t kBlock = int64_t(kStreamThreads) * UNROLL;
    for (int64_t base = int64_t(blockIdx.x) * kBlock; base < n16; base += int64_t(gridDim.x) * kBlock) {
        uint4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int64_t i = base + u * kStreamThreads + threadIdx.x;
            v[u] = (i < n16) ? load16_stream(reinterpret_cast<const uint16_t*>(src + i)) : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int64_t i = base + u * kStreamThreads + threadIdx.x;
            if (i < n16) dst[i] = v[u];
        }
    }
}

}  // namespace

int launch_hbm_rw_stream(const void* src, void* dst, size_t bytes, int workgroups, int block_kib, hipStream_t stream) {
    const dim3 g{unsigned(workgroups)}, b{kStreamThreads};
    const uint4* s4 = static_cast<const uint4*>(src);
    uint4* d4 = static_cast<uint4*>(dst);
    const int64_t n16 = int64_t(bytes / 16);
    // a workgroup's trip moves kStreamThreads * 16 bytes per load in flight: 8, 16, 32 or 64 KiB
    if (block_kib == 8) hipLaunchKernelGGL(hbm_rw_stream_kernel<1>, g, b, 0, stream, s4, d4, n16);
    else if (block_kib == 16) hipLaunchKernelGGL(hbm_rw_stream_kernel<2>, g, b, 0, stream, s4, d4, n16);
    else if (block_kib == 32) hipLaunchKernelGGL(hbm_rw_stream_kernel<4>, g, b, 0, stream, s4, d4, n16);
    else hipLaunchKernelGGL(hbm_rw_stream_kernel<8>, g, b, 0, stream, s4, d4, n16);
    return int(hipGetLastError());
}

int launch_hbm_read_stream(const void* src, size_t bytes, void* sink, int workgroups, hipStream_t stream) {
    hipLaunchKernelGGL(hbm_read_stream_kernel, dim3(unsigned(workgroups)), dim3(kStreamThreads), 0, stream,
                       static_cast<const uint4*>(src), int64_t(bytes / 16), static_cast<uint32_t*>(sink));
    return int(hipGetLastError());
}

}  // namespace l3
