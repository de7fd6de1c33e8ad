// Sweep-kernel instantiations for the latent (576, 512) head, and the split-merge kernel.
#include "da_sweep_launch.h"
namespace da {
hipError_t launch_sweep_d576(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream) {
    return launch_sweep_dim<576, 512, 2>(p, is_bf16, rt, grid, stream);
}
hipError_t launch_reduce(const ReduceParams& p, bool is_bf16, int blocks, hipStream_t stream) {
    if (is_bf16)
        hipLaunchKernelGGL((reduce_kernel<bf16_tag>), dim3(blocks), dim3(128), 0, stream, p);
    else
        hipLaunchKernelGGL((reduce_kernel<f16_tag>), dim3(blocks), dim3(128), 0, stream, p);
    return hipGetLastError();
}
}  // namespace da
