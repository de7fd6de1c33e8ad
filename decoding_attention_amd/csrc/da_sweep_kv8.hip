// Sweep-kernel instantiations for an FP8 (e4m3) K/V cache, all head dimensions.
#include "da_sweep_launch.h"
namespace da {
hipError_t launch_sweep_kv8(const SweepParams& p, bool is_bf16, int dim, int rt, dim3 grid, hipStream_t stream) {
    switch (dim) {
        case 64: return launch_sweep_dim<64, 64, 4, true>(p, is_bf16, rt, grid, stream);
        case 96: return launch_sweep_dim<96, 96, 4, true>(p, is_bf16, rt, grid, stream);
        case 128: return launch_sweep_dim<128, 128, 4, true>(p, is_bf16, rt, grid, stream);
        case 256: return launch_sweep_dim<256, 256, 4, true>(p, is_bf16, rt, grid, stream);
        case 576: return launch_sweep_dim<576, 512, 2, true>(p, is_bf16, rt, grid, stream);
        default: return hipErrorInvalidValue;
    }
}
}  // namespace da
