// MFMA kernel for grouped query heads over one KV head (latent MLA form): launcher interface.
#pragma once
#include "da_common.h"

namespace da {
bool mla_supported(size_t dim, size_t dim_v, int ratio);
int mla_heads_per_group(int ratio);
int mla_rows_per_trip();
hipError_t launch_mla(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream);
// the same over an 8-bit K cache of format fmt (kKvFp8 or kKvInt8)
hipError_t launch_mla_kv8(const SweepParams& p, int fmt, bool is_bf16, int rt, dim3 grid, hipStream_t stream);
}  // namespace da
