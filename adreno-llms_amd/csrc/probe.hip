// Streaming-read probe: what the memory system gives a kernel that only reads, with the access
// pattern of the GEMV kernels (a wavefront reads contiguous kilobytes with 16-byte loads per
// lane, wavefronts stride through the buffer, 3 blocks of 4 wavefronts per CU).  The practical
// ceiling the GEMV figures are compared with, as the reference's gemv_stream_buf is for its
// GEMVs (QW/kernels/gemv_m1.cl:105-131, host QW/src/main.cpp:27-154).
#include "../../include/mi_linear.h"
#include "common.h"

namespace mi {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kProbeUnroll = 8;          // 16-byte loads in flight per lane: 8 KB per wavefront and step

__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4* __restrict__ src, size_t pieces,
                                                          uint32_t* __restrict__ sink) {
    const size_t wave = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) >> 6;
    const size_t waves = (static_cast<size_t>(gridDim.x) * blockDim.x) >> 6;
    const int lane = threadIdx.x & 63;
    u32x4 acc = {0, 0, 0, 0};
    const size_t step = 64 * kProbeUnroll;
    size_t base = wave * step;
    for (; base + step <= pieces; base += waves * step) {
        u32x4 v[kProbeUnroll];
        #pragma unroll
        for (int u = 0; u < kProbeUnroll; ++u) v[u] = __builtin_nontemporal_load(src + base + u * 64 + lane);
        #pragma unroll
        for (int u = 0; u < kProbeUnroll; ++u) acc ^= v[u];
    }
    // the tail (less than one step) goes to the wavefront whose turn it would have been
    if (base < pieces)
        for (size_t i = base + lane; i < pieces; i += 64) acc ^= __builtin_nontemporal_load(src + i);
    // never true for the probe's data (the sink's only purpose is to keep the loads alive)
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9E3779B9u && sink) sink[0] = acc.x;
}

}  // namespace
}  // namespace mi

extern "C" int mi_stream_read_probe(void* stream, const void* src, size_t bytes, void* sink) {
    using namespace mi;
    if (!ensure_init()) return 0;
    if (!src || bytes < 16 || reinterpret_cast<uintptr_t>(src) % 16) {
        MI_ERROR_FMT("mi_stream_read_probe: bad argument (src=%p bytes=%zu)", src, bytes);
        return 0;
    }
    const int blocks = 3 * (device_info().cus > 0 ? device_info().cus : 256);
    hipLaunchKernelGGL(stream_read_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const u32x4*>(src), bytes / 16, static_cast<uint32_t*>(sink));
    return MI_HIP_OK(hipGetLastError()) ? 1 : 0;
}
