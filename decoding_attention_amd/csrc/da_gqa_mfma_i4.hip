// Instantiations and launcher of the grouped-head MFMA sweep over an int4 K/V cache.
#include "da_gqa_mfma_launch.h"

namespace da {

hipError_t launch_gqa_mfma_i4(const SweepParams& p, bool is_bf16, int dim, int heads_per_group, bool wave_per_head,
                              dim3 grid, hipStream_t stream) {
    return is_bf16 ? gqa_launch::launch_tag<bf16_tag, kKvInt4>(p, dim, heads_per_group, wave_per_head, grid, stream)
                   : gqa_launch::launch_tag<f16_tag, kKvInt4>(p, dim, heads_per_group, wave_per_head, grid, stream);
}

}  // namespace da
