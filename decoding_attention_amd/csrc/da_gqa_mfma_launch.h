// Launch helpers of the grouped-head MFMA sweep, shared by the translation units that instantiate it (16-bit
// K/V in da_gqa_mfma.hip, FP8 in da_gqa_mfma_kv8.hip, int8 in da_gqa_mfma_i8.hip, int4 in da_gqa_mfma_i4.hip, the per-token forms in da_gqa_mfma_i4t.hip and da_gqa_mfma_i8t.hip, int4 and int8 with a pair per 64 elements in
// da_gqa_mfma_i4g.hip and da_gqa_mfma_i8g.hip; separate units so that the sets compile in parallel).
#pragma once
#include "da_gqa_mfma.h"


namespace da {

namespace gqa_launch {

template <typename Tag, int D, int NT, bool WH, int KV8, int PGM>
hipError_t launch_form(const SweepParams& p, dim3 grid, hipStream_t stream) {
    constexpr int DV = D == 576 ? 512 : D;  // (576, 512): the latent form, V inside the K rows
    // the next tile's loads issued as soon as this tile's registers are free, not after its last matrix instruction
    // (d = 256 with 32 heads a group: the longer live ranges do not fit 512 registers, 41 to 78 of them spilled)
    constexpr bool kPrefetch = D <= 128 || D == 576 || (D == 256 && NT == 1);
    constexpr int kMinWaves = (D <= 128 && (NT == 1 || D <= 64)) ? 2 : 1;
    auto kern = gqa_mfma_kernel<Tag, D, DV, NT, kPrefetch, WH, kMinWaves, KV8, PGM>;
    const size_t lds = gqa_lds_bytes<DV>(NT, (KV8 & kKvPerToken) == 0 ? 0 : ((KV8 & kKvGroup64) != 0 ? D / 64 : 1));
    if (lds > 48 * 1024) {
        static std::atomic<uint64_t> devices_done{0};
        const hipError_t attr_err = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds, devices_done);
        if (attr_err != hipSuccess) return attr_err;
    }
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, p);
    return hipGetLastError();
}

// 16-token pages of paged K/V take the form that fetches a tile as two runs, smaller pages the form with a lookup
// per row (instantiations of their own: the extra addresses cost registers the other layouts should not pay for)
template <typename Tag, int D, int NT, bool WH, int KV8>
hipError_t launch_one(const SweepParams& p, dim3 grid, hipStream_t stream) {
    if (p.block_table != nullptr && p.page_shift < 4) return launch_form<Tag, D, NT, WH, KV8, 2>(p, grid, stream);
    if (p.block_table != nullptr && p.page_shift == 4) return launch_form<Tag, D, NT, WH, KV8, 1>(p, grid, stream);
    return launch_form<Tag, D, NT, WH, KV8, 0>(p, grid, stream);
}

template <typename Tag, int D, int KV8>
hipError_t launch_dim(const SweepParams& p, int heads_per_group, bool wh, dim3 grid, hipStream_t stream) {
    if (heads_per_group == 16)
        return wh ? launch_one<Tag, D, 1, true, KV8>(p, grid, stream) : launch_one<Tag, D, 1, false, KV8>(p, grid, stream);
    // (a pair per 64 elements at d = 256: four sets of factors and 32 heads do not fit a wave's registers)
    if constexpr (!((KV8 & kKvGroup64) != 0 && D == 256))
        if (heads_per_group == 32)
            return wh ? launch_one<Tag, D, 2, true, KV8>(p, grid, stream)
                      : launch_one<Tag, D, 2, false, KV8>(p, grid, stream);
    return hipErrorInvalidValue;
}

template <typename Tag, int KV8>
hipError_t launch_tag(const SweepParams& p, int dim, int heads_per_group, bool wh, dim3 grid, hipStream_t stream) {
    switch (dim) {
        case 64:  // (one pair per 64 elements is one pair per row here: the per-token instantiation serves it)
            if constexpr ((KV8 & kKvGroup64) == 0) return launch_dim<Tag, 64, KV8>(p, heads_per_group, wh, grid, stream);
            return hipErrorInvalidValue;
        case 96:
            if constexpr (!KV8) return launch_dim<Tag, 96, 0>(p, heads_per_group, wh, grid, stream);
            return hipErrorInvalidValue;  // 8-bit loads pair up k-steps: head dims that are multiples of 64 only
        case 128: return launch_dim<Tag, 128, KV8>(p, heads_per_group, wh, grid, stream);
        case 256: return launch_dim<Tag, 256, KV8>(p, heads_per_group, wh, grid, stream);
        case 576:  // the latent form with up to 16 query heads: one KV head, its tokens shared by the four waves
            if constexpr ((KV8 & kKvPerToken) == 0)
                if (heads_per_group == 16 && !wh) return launch_one<Tag, 576, 1, false, KV8>(p, grid, stream);
            return hipErrorInvalidValue;
        default: return hipErrorInvalidValue;
    }
}

}  // namespace gqa_launch

}  // namespace da
