// Sweep-kernel instantiations for the latent (576, 512) head, the split-merge kernel and the prefix kernel of the
// balanced grid.
#include "da_sweep_launch.h"
namespace da {
hipError_t launch_sweep_d576(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream) {
    return launch_sweep_dim<576, 512, 2>(p, is_bf16, rt, grid, stream);
}
template <typename Tag, int SG>
static void launch_reduce_sg(const ReduceParams& p, int blocks, hipStream_t stream) {
    const long long nc4 = p.dim_v / 4;
    if constexpr (SG > 1) {
        if (p.half_partials) {
            // SG lanes per (row of a block, four columns), dead rows of the blocks included
            const long long lanes = (long long)(blocks / p.head_q) * p.nat_blocks * 32 * nc4 * SG;
            hipLaunchKernelGGL((reduce_kernel<Tag, SG, true>), dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, stream, p,
                               blocks);
            return;
        }
    }
    // SG = 1: one thread per (row, four columns); SG > 1: one wave per (row, 64 / SG column groups), four waves a block
    const long long units = SG == 1 ? (long long)blocks * nc4 : (long long)blocks * (nc4 / (64 / SG)) * 64;
    const dim3 grid((unsigned)((units + 255) / 256));
    hipLaunchKernelGGL((reduce_kernel<Tag, SG, false>), grid, dim3(256), 0, stream, p, blocks);
}

hipError_t launch_reduce(const ReduceParams& p, bool is_bf16, int blocks, hipStream_t stream) {
    // `blocks` counts (sequence, head) rows.  Many splits of few rows (one long sequence): several lanes share the
    // splits of one output element, so that the merge is not one long chain of dependent loads per thread.
    const long long threads = (long long)blocks * (p.dim_v / 4);
    int sg = 1;
    while (sg < 8 && p.nsplit >= 8 * sg && threads * sg < (1ll << 18)) sg *= 2;
    while (sg > 1 && (p.dim_v / 4) % (64 / sg) != 0) sg /= 2;
    // The 16-byte-a-lane merge of the 16-bit records is the faster one as soon as it has a few work-groups a CU: the
    // several-lanes-a-value form only where there are too few rows for that (measured, 128 heads over one latent head:
    // batch 8 x 4096 tokens, 16 splits, 30.6 -> 24.4 us a call; batch 4 x 2048, 16 splits, 23.9 -> 19.9; batch 8 x
    // 1024, 8 splits, 21.6 -> 16.7; batch 2 x 4096 a tie; batch 1 x 4096, 32 splits, loses 19.5 -> 20.6)
    if (p.half_partials && threads >= (1ll << 15)) sg = 1;
    // normalised 16-bit partials (the pipelined latent kernel's: dim_v = 512, never the balanced grid), one lane per
    // element: eight columns a thread, dead rows of the blocks included
    if (p.half_partials && (p.dim_v != 512 || p.flat_wgs != 0 || p.nat_blocks <= 0 || p.head_q <= 0))
        return hipErrorInvalidValue;
    if (p.half_partials && sg == 1) {
        const int per_kv = p.groups * p.nat_waves, head_k = p.nat_blocks / per_kv;
        constexpr int ny = 8 / kReduce16Runs;  // work-groups per block of 32 heads
        if (ny * per_kv > 65535 || head_k > 65535) return hipErrorInvalidValue;
        const dim3 grid((unsigned)(blocks / p.head_q), (unsigned)(ny * per_kv), (unsigned)head_k);
        if (is_bf16)
            hipLaunchKernelGGL((reduce16_kernel<bf16_tag>), grid, dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL((reduce16_kernel<f16_tag>), grid, dim3(256), 0, stream, p);
        return hipGetLastError();
    }
    switch (sg) {
        case 8: is_bf16 ? launch_reduce_sg<bf16_tag, 8>(p, blocks, stream) : launch_reduce_sg<f16_tag, 8>(p, blocks, stream); break;
        case 4: is_bf16 ? launch_reduce_sg<bf16_tag, 4>(p, blocks, stream) : launch_reduce_sg<f16_tag, 4>(p, blocks, stream); break;
        case 2: is_bf16 ? launch_reduce_sg<bf16_tag, 2>(p, blocks, stream) : launch_reduce_sg<f16_tag, 2>(p, blocks, stream); break;
        default: is_bf16 ? launch_reduce_sg<bf16_tag, 1>(p, blocks, stream) : launch_reduce_sg<f16_tag, 1>(p, blocks, stream); break;
    }
    return hipGetLastError();
}
namespace {
// Positions of paged sequences on the balanced grid's line: out[b] = sum over b' < b of ceil(len[b'] / 2^shift),
// out[batch] the total.  One work-group of 1024 threads walks the lengths 1024 at a time.
__global__ __launch_bounds__(1024) void flat_prefix_kernel(const int32_t* __restrict__ seq_lens, int batch, int shift,
                                                            int32_t* __restrict__ out) {
    __shared__ int wave_sum[16];
    __shared__ int carry_s;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) {
        carry_s = 0;
        out[0] = 0;
    }
    __syncthreads();
    for (int base = 0; base < batch; base += 1024) {
        const int i = base + tid;
        const int v = i < batch ? (max(seq_lens[i], 0) + (1 << shift) - 1) >> shift : 0;
        int incl = v;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
        if (lane == 63) wave_sum[wave] = incl;
        __syncthreads();
        int before = carry_s;
        for (int w = 0; w < wave; ++w) before += wave_sum[w];
        if (i < batch) out[i + 1] = before + incl;
        __syncthreads();
        if (tid == 1023) carry_s = before + incl;
        __syncthreads();
    }
}

}  // namespace

hipError_t launch_flat_prefix(const int32_t* seq_lens, int batch, int shift, int32_t* out, hipStream_t stream) {
    hipLaunchKernelGGL(flat_prefix_kernel, dim3(1), dim3(1024), 0, stream, seq_lens, batch, shift, out);
    return hipGetLastError();
}
}  // namespace da
