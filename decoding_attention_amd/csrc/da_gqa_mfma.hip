// Instantiations and launcher of the grouped-head MFMA sweep.
#include "da_gqa_mfma.h"

#include <mutex>

namespace da {

namespace {

template <typename Tag, int D, int NT, bool WH>
hipError_t launch_one(const SweepParams& p, dim3 grid, hipStream_t stream) {
    constexpr bool kPrefetch = D <= 128;
    constexpr int kMinWaves = (D <= 128 && (NT == 1 || D <= 64)) ? 2 : 1;
    auto kern = gqa_mfma_kernel<Tag, D, D, NT, kPrefetch, WH, kMinWaves>;
    const size_t lds = gqa_lds_bytes<D>(NT);
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        if (lds > 48 * 1024)
            attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    });
    if (attr_err != hipSuccess) return attr_err;
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, p);
    return hipGetLastError();
}

template <typename Tag, int D>
hipError_t launch_dim(const SweepParams& p, int heads_per_group, bool wh, dim3 grid, hipStream_t stream) {
    if (heads_per_group == 16)
        return wh ? launch_one<Tag, D, 1, true>(p, grid, stream) : launch_one<Tag, D, 1, false>(p, grid, stream);
    if (heads_per_group == 32)
        return wh ? launch_one<Tag, D, 2, true>(p, grid, stream) : launch_one<Tag, D, 2, false>(p, grid, stream);
    return hipErrorInvalidValue;
}

template <typename Tag>
hipError_t launch_tag(const SweepParams& p, int dim, int heads_per_group, bool wh, dim3 grid, hipStream_t stream) {
    switch (dim) {
        case 64: return launch_dim<Tag, 64>(p, heads_per_group, wh, grid, stream);
        case 96: return launch_dim<Tag, 96>(p, heads_per_group, wh, grid, stream);
        case 128: return launch_dim<Tag, 128>(p, heads_per_group, wh, grid, stream);
        case 256: return launch_dim<Tag, 256>(p, heads_per_group, wh, grid, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

hipError_t launch_gqa_mfma(const SweepParams& p, bool is_bf16, int dim, int heads_per_group, bool wave_per_head,
                           dim3 grid, hipStream_t stream) {
    return is_bf16 ? launch_tag<bf16_tag>(p, dim, heads_per_group, wave_per_head, grid, stream)
                   : launch_tag<f16_tag>(p, dim, heads_per_group, wave_per_head, grid, stream);
}

}  // namespace da
