// Sweep-kernel instantiations for the latent (576, 512) head, the split-merge kernel and the prefix kernel of the
// balanced grid.
#include "da_sweep_launch.h"
namespace da {
hipError_t launch_sweep_d576(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream) {
    return launch_sweep_dim<576, 512, 2>(p, is_bf16, rt, grid, stream);
}
hipError_t launch_reduce(const ReduceParams& p, bool is_bf16, int blocks, hipStream_t stream) {
    // `blocks` counts (sequence, head) rows; one thread per four output columns
    const long long threads = (long long)blocks * (p.dim_v / 4);
    const dim3 grid((unsigned)((threads + 255) / 256));
    if (is_bf16)
        hipLaunchKernelGGL((reduce_kernel<bf16_tag>), grid, dim3(256), 0, stream, p, blocks);
    else
        hipLaunchKernelGGL((reduce_kernel<f16_tag>), grid, dim3(256), 0, stream, p, blocks);
    return hipGetLastError();
}
namespace {
// Positions of paged sequences on the balanced grid's line: out[b] = sum over b' < b of ceil(len[b'] / 2^shift),
// out[batch] the total.  One work-group of 1024 threads walks the lengths 1024 at a time.
__global__ __launch_bounds__(1024) void flat_prefix_kernel(const int32_t* __restrict__ seq_lens, int batch, int shift,
                                                            int32_t* __restrict__ out) {
    __shared__ int wave_sum[16];
    __shared__ int carry_s;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) {
        carry_s = 0;
        out[0] = 0;
    }
    __syncthreads();
    for (int base = 0; base < batch; base += 1024) {
        const int i = base + tid;
        const int v = i < batch ? (max(seq_lens[i], 0) + (1 << shift) - 1) >> shift : 0;
        int incl = v;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
        if (lane == 63) wave_sum[wave] = incl;
        __syncthreads();
        int before = carry_s;
        for (int w = 0; w < wave; ++w) before += wave_sum[w];
        if (i < batch) out[i + 1] = before + incl;
        __syncthreads();
        if (tid == 1023) carry_s = before + incl;
        __syncthreads();
    }
}

}  // namespace

hipError_t launch_flat_prefix(const int32_t* seq_lens, int batch, int shift, int32_t* out, hipStream_t stream) {
    hipLaunchKernelGGL(flat_prefix_kernel, dim3(1), dim3(1024), 0, stream, seq_lens, batch, shift, out);
    return hipGetLastError();
}
}  // namespace da
