// Measurement aid: a plain streaming read of a device buffer, the fastest way this GPU delivers bytes from HBM to
// the compute units.  Benchmarks time it beside the attention kernels so that their achieved bandwidth can be read
// against what the memory system gives a kernel that does nothing else (measurably below the nominal peak).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/decoding_attn_hip.h"
#include "decoding_attn_probe.h"

namespace {

// Each work-group reads one contiguous slab with 16-byte loads, eight in flight per lane, marked non-temporal as the
// attention kernels' K/V loads are (6.2-6.3 TB/s with ordinary loads, 7.0-7.1 TB/s with the hint, on this GPU).
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4* __restrict__ p, size_t per_block, uint32_t* sink) {
    constexpr int U = 8;
    const u32x4* b = p + (size_t)blockIdx.x * per_block;
    uint32_t acc = 0;
    for (size_t i = threadIdx.x; i + (size_t)(U - 1) * 256 < per_block; i += (size_t)256 * U) {
        u32x4 a[U];
#pragma unroll
        for (int u = 0; u < U; ++u) a[u] = __builtin_nontemporal_load(&b[i + (size_t)u * 256]);
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= a[u].x ^ a[u].y ^ a[u].z ^ a[u].w;
    }
    if (acc == 0x9e3779b9u && sink) sink[0] = acc;  // keeps the loads alive; practically never taken
}

// One wave per SIMD on every CU issuing v_mfma_f32_32x32x16_f16 back to back, each fed by one ds_read_b128 of the
// caller's operand values (a matrix instruction's power depends on its operands: zeros run at nearly the nominal clock,
// N(0,1) values far below it), nothing else.  What this sustains is the matrix-pipe rate the chip's power limit
// leaves a kernel, the practical ceiling for the latent (MLA) kernel's matrix work.
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
constexpr int kMfmaBlocks = 256, kMfmaPerTrip = 32;
__global__ __launch_bounds__(256) void mfma_rate_kernel(const half8* __restrict__ operands, int iters, float* sink) {
    __shared__ __attribute__((aligned(16))) half8 lds[2048];  // 32 KiB of operand values
    const int lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < 2048; i += 256) lds[i] = operands[i];
    __syncthreads();
    half8 a[8], b[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        a[j] = operands[lane + 64 * j];
        b[j] = operands[lane + 64 * (8 + j)];
    }
    float16v c[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) c[i][r] = 0.0f;
    const uint32_t la = (uint32_t)(uintptr_t)lds + lane * 16;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < kMfmaPerTrip; ++u) {
            // operand u % 8 was requested eight steps ago; seven younger reads may be outstanding
            asm volatile("s_waitcnt lgkmcnt(7)" : "+v"(a[u & 7]));
            asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c[u % 16]) : "v"(a[u & 7]), "v"(b[u & 7]));
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(a[u & 7]) : "v"(la), "n"((u & 31) * 1024));
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += c[i][r];
#pragma unroll
    for (int j = 0; j < 8; ++j) s += (float)a[j][0];
    sink[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace

extern "C" int da_probe_mfma_rate(const void* operands, int iters, void* sink, void* hip_stream) {
    if (!operands || !sink || iters <= 0 || (reinterpret_cast<uintptr_t>(operands) & 15u) != 0) return DA_ERR_INVALID_ARGUMENT;
    hipLaunchKernelGGL(mfma_rate_kernel, dim3(kMfmaBlocks), dim3(256), 0, reinterpret_cast<hipStream_t>(hip_stream),
                       reinterpret_cast<const half8*>(operands), iters, reinterpret_cast<float*>(sink));
    return hipGetLastError() == hipSuccess ? DA_OK : DA_ERR_HIP;
}

extern "C" double da_probe_mfma_rate_flops(int iters) {
    // work-groups x waves x trips x matrix instructions x (2 x 32 x 32 x 16 flops)
    return (double)kMfmaBlocks * 4.0 * (double)iters * kMfmaPerTrip * 32768.0;
}

extern "C" int da_probe_stream_read(const void* buf, size_t bytes, void* sink, void* hip_stream) {
    if (!buf || (reinterpret_cast<uintptr_t>(buf) & 15u) != 0) return DA_ERR_INVALID_ARGUMENT;
    constexpr size_t kBlocks = 4096, kGrain = (size_t)256 * 8;  // 16-byte elements one work-group reads per trip
    const size_t per_block = bytes / 16 / kBlocks / kGrain * kGrain;
    if (per_block == 0) return DA_ERR_INVALID_ARGUMENT;  // needs at least 128 MiB
    hipLaunchKernelGGL(stream_read_kernel, dim3(kBlocks), dim3(256), 0, reinterpret_cast<hipStream_t>(hip_stream),
                       reinterpret_cast<const u32x4*>(buf), per_block, reinterpret_cast<uint32_t*>(sink));
    return hipGetLastError() == hipSuccess ? DA_OK : DA_ERR_HIP;
}

extern "C" size_t da_probe_stream_read_bytes(size_t bytes) {
    constexpr size_t kBlocks = 4096, kGrain = (size_t)256 * 8;
    return bytes / 16 / kBlocks / kGrain * kGrain * kBlocks * 16;
}
