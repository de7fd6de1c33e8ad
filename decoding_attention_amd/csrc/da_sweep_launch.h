// Instantiation helper: each da_sweep_d*.hip translation unit defines one launcher for its
// (dim, dim_v) pair so the pairs compile in parallel.
#pragma once
#include "da_sweep.h"

namespace da {

// Tile shape per head dimension: G lanes per row, U rows in flight per row slot.
template <int D> struct SweepTile;
template <> struct SweepTile<64>  { static constexpr int G = 8,  U = 8; };
template <> struct SweepTile<96>  { static constexpr int G = 4,  U = 2; };
template <> struct SweepTile<128> { static constexpr int G = 8,  U = 4; };
template <> struct SweepTile<256> { static constexpr int G = 16, U = 4; };
template <> struct SweepTile<576> { static constexpr int G = 8,  U = 1; };

template <typename Tag, int D, int DV, int RT, int KV8 = 0>
inline hipError_t launch_sweep_rt(const SweepParams& p, dim3 grid, hipStream_t stream) {
    constexpr int G = SweepTile<D>::G, U = SweepTile<D>::U;
    hipLaunchKernelGGL((sweep_kernel<Tag, D, DV, G, RT, U, KV8>), grid, dim3(256), 0, stream, p);
    return hipGetLastError();
}

template <int D, int DV, int MAXRT, int KV8 = 0>
inline hipError_t launch_sweep_dim(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream) {
    if (is_bf16) {
        if (rt == 1) return launch_sweep_rt<bf16_tag, D, DV, 1, KV8>(p, grid, stream);
        if (rt == 2) return launch_sweep_rt<bf16_tag, D, DV, 2, KV8>(p, grid, stream);
        if constexpr (MAXRT >= 4) {
            if (rt == 4) return launch_sweep_rt<bf16_tag, D, DV, 4, KV8>(p, grid, stream);
        }
    } else {
        if (rt == 1) return launch_sweep_rt<f16_tag, D, DV, 1, KV8>(p, grid, stream);
        if (rt == 2) return launch_sweep_rt<f16_tag, D, DV, 2, KV8>(p, grid, stream);
        if constexpr (MAXRT >= 4) {
            if (rt == 4) return launch_sweep_rt<f16_tag, D, DV, 4, KV8>(p, grid, stream);
        }
    }
    return hipErrorInvalidValue;
}

// rows of K one work-group consumes per loop trip (4 waves)
template <int D> constexpr int sweep_rows_per_trip() { return 4 * (kWave / SweepTile<D>::G) * SweepTile<D>::U; }

hipError_t launch_sweep_d64(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream);
hipError_t launch_sweep_d96(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream);
hipError_t launch_sweep_d128(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream);
hipError_t launch_sweep_d256(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream);
hipError_t launch_sweep_d576(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream);
// the VALU sweep over an FP8 (e4m3) K/V cache, any supported (dim, dim_v)
// 8-bit K/V of format fmt (kKvFp8 or kKvInt8)
hipError_t launch_sweep_kv8(const SweepParams& p, int fmt, bool is_bf16, int dim, int rt, dim3 grid,
                            hipStream_t stream);
hipError_t launch_reduce(const ReduceParams& p, bool is_bf16, int blocks, hipStream_t stream);
// out[0 .. batch] = running sum of ceil(seq_lens / 2^shift) (positions of paged sequences on the balanced grid's line)
hipError_t launch_flat_prefix(const int32_t* seq_lens, int batch, int shift, int32_t* out, hipStream_t stream);

}  // namespace da
