// Measurement aid: a plain streaming read of a device buffer, the fastest way this GPU delivers bytes from HBM to
// the compute units.  Benchmarks time it beside the attention kernels so that their achieved bandwidth can be read
// against what the memory system gives a kernel that does nothing else (measurably below the nominal peak).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/decoding_attn_hip.h"

namespace {

// Each work-group reads one contiguous slab with 16-byte loads, eight in flight per lane.
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* __restrict__ p, size_t per_block, uint32_t* sink) {
    constexpr int U = 8;
    const uint4* b = p + (size_t)blockIdx.x * per_block;
    uint32_t acc = 0;
    for (size_t i = threadIdx.x; i + (size_t)(U - 1) * 256 < per_block; i += (size_t)256 * U) {
        uint4 a[U];
#pragma unroll
        for (int u = 0; u < U; ++u) a[u] = b[i + (size_t)u * 256];
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= a[u].x ^ a[u].y ^ a[u].z ^ a[u].w;
    }
    if (acc == 0x9e3779b9u && sink) sink[0] = acc;  // keeps the loads alive; practically never taken
}

}  // namespace

extern "C" int da_probe_stream_read(const void* buf, size_t bytes, void* sink, void* hip_stream) {
    if (!buf || (reinterpret_cast<uintptr_t>(buf) & 15u) != 0) return DA_ERR_INVALID_ARGUMENT;
    constexpr size_t kBlocks = 4096, kGrain = (size_t)256 * 8;  // 16-byte elements one work-group reads per trip
    const size_t per_block = bytes / 16 / kBlocks / kGrain * kGrain;
    if (per_block == 0) return DA_ERR_INVALID_ARGUMENT;  // needs at least 128 MiB
    hipLaunchKernelGGL(stream_read_kernel, dim3(kBlocks), dim3(256), 0, reinterpret_cast<hipStream_t>(hip_stream),
                       reinterpret_cast<const uint4*>(buf), per_block, reinterpret_cast<uint32_t*>(sink));
    return hipGetLastError() == hipSuccess ? DA_OK : DA_ERR_HIP;
}

extern "C" size_t da_probe_stream_read_bytes(size_t bytes) {
    constexpr size_t kBlocks = 4096, kGrain = (size_t)256 * 8;
    return bytes / 16 / kBlocks / kGrain * kGrain * kBlocks * 16;
}
