// Sweep-kernel instantiations for head dimension 64.
#include "da_sweep_launch.h"
namespace da {
hipError_t launch_sweep_d64(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream) {
    return launch_sweep_dim<64, 64, 4>(p, is_bf16, rt, grid, stream);
}
}  // namespace da
