// Sweep-kernel instantiations for an 8-bit or 4-bit K/V cache (FP8 e4m3, int8, int4), all head dimensions.
#include "da_sweep_launch.h"
namespace da {
namespace {
template <int FMT>
hipError_t launch_fmt(const SweepParams& p, bool is_bf16, int dim, int rt, dim3 grid, hipStream_t stream) {
    switch (dim) {
        case 64: return launch_sweep_dim<64, 64, 4, FMT>(p, is_bf16, rt, grid, stream);
        case 96: return launch_sweep_dim<96, 96, 4, FMT>(p, is_bf16, rt, grid, stream);
        case 128: return launch_sweep_dim<128, 128, 4, FMT>(p, is_bf16, rt, grid, stream);
        case 256: return launch_sweep_dim<256, 256, 4, FMT>(p, is_bf16, rt, grid, stream);
        case 576: return launch_sweep_dim<576, 512, 2, FMT>(p, is_bf16, rt, grid, stream);
        default: return hipErrorInvalidValue;
    }
}
}  // namespace

hipError_t launch_sweep_kv8(const SweepParams& p, int fmt, bool is_bf16, int dim, int rt, dim3 grid,
                            hipStream_t stream) {
    if (fmt == kKvInt4) return launch_fmt<kKvInt4>(p, is_bf16, dim, rt, grid, stream);
    return fmt == kKvInt8 ? launch_fmt<kKvInt8>(p, is_bf16, dim, rt, grid, stream)
                          : launch_fmt<kKvFp8>(p, is_bf16, dim, rt, grid, stream);
}
}  // namespace da
