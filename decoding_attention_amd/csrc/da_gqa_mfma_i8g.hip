// Instantiations and launcher of the grouped-head MFMA sweep over an int8 K/V cache with a (scale, zero) pair per
// run of 64 elements of every (token, KV head) row.
#include "da_gqa_mfma_launch.h"

namespace da {

hipError_t launch_gqa_mfma_i8g(const SweepParams& p, bool is_bf16, int dim, int heads_per_group, bool wave_per_head,
                               dim3 grid, hipStream_t stream) {
    constexpr int kFormat = kKvInt8 | kKvPerToken | kKvGroup64;
    if (p.k_tok == nullptr || p.v_tok == nullptr || (dim != 128 && dim != 256)) return hipErrorInvalidValue;
    return is_bf16 ? gqa_launch::launch_tag<bf16_tag, kFormat>(p, dim, heads_per_group, wave_per_head, grid, stream)
                   : gqa_launch::launch_tag<f16_tag, kFormat>(p, dim, heads_per_group, wave_per_head, grid, stream);
}

}  // namespace da
