// Sweep-kernel instantiations for the latent (576, 512) head, and the split-merge kernel.
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
}  // namespace da
