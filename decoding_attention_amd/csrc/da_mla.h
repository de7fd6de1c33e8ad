// MFMA kernel for grouped query heads over one KV head (latent MLA form): launcher interface.
#pragma once
#include "da_common.h"

namespace da {
bool mla_supported(size_t dim, size_t dim_v, int ratio);
int mla_heads_per_group(int ratio);
int mla_rows_per_trip();
// work-groups of one or two waves run two to a CU (two tile buffers instead of three) when the grid has more
// work-groups than this (DA_MLA_TWO_PER_CU_FROM, default 256)
int mla_two_per_cu_from();
hipError_t launch_mla(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream);
// Whether a latent-kernel launch with rt heads per work-group (rt / 32 waves) leaves its split partials as normalised
// 16-bit block records (ReduceParams::half_partials, nat_block in da_common.h): whenever the records of whole blocks
// of 32 heads fit the workspace area sized for fp32 partials of head_q rows, i.e. from 17 heads per KV head up.
inline bool mla_half_partials(bool latent_kernel, int rt, size_t head_q, size_t head_k, int groups) {
    return latent_kernel && rt % 32 == 0 &&
           nat_split_bytes(nat_blocks((int)head_k, groups, rt / 32)) <= head_q * 512 * sizeof(float);
}
// the software-pipelined kernel for work-groups of 128 heads over 16-bit K (da_mla_pipe.hip); launch_mla routes to it
hipError_t launch_mla_pipe(const SweepParams& p, bool is_bf16, dim3 grid, hipStream_t stream);
// its form over an 8-bit K cache of format fmt (kKvFp8 or kKvInt8), for the layouts mla_pipe_kv8_supported names
bool mla_pipe_kv8_supported(const SweepParams& p);
bool mla_pipe_kv8_off();  // DA_MLA_PIPE_KV8=0: 8-bit K stays on the compiler-scheduled kernel (measurements)
hipError_t launch_mla_pipe_kv8(const SweepParams& p, int fmt, bool is_bf16, dim3 grid, hipStream_t stream);
// the (576, 512) shape with V in a buffer of its own (16-bit K/V; packed, or pages of 16 tokens and more)
hipError_t launch_mla_vd(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream);
// the same over an 8-bit K cache of format fmt (kKvFp8 or kKvInt8)
hipError_t launch_mla_kv8(const SweepParams& p, int fmt, bool is_bf16, int rt, dim3 grid, hipStream_t stream);
}  // namespace da
