// Device helpers shared by the latent (MLA) MFMA kernels: matrix-instruction wrappers, direct-to-LDS loads,
// LDS reads and waits issued from assembly, and the swizzles of the LDS tile layout.
//
// LDS tile layout (both kernels).  A tile of 32 tokens has two regions: the 512 value columns of the 32 rows (1 KiB per
// row) and the remaining 64 key columns (128 B per row).  One direct-to-LDS load instruction fills exactly one row of
// the first region (or eight rows of the second), so its source is a wave-uniform row address plus a per-lane chunk
// offset.  Inside a row the 16-byte chunks are XOR-swizzled with the row index --
//   first region:  chunk c of row r at c ^ ((r & 3) << 2 | (r >> 2) & 3)
//   second region: chunk c of row r at c ^ ((r >> 1) & 7)
// -- which makes both read patterns (16 rows x one chunk for K, 4 rows x 64 bytes for V^T) conflict-free, and because
// XOR commutes with the per-step chunk offsets every read address is one per-lane base XOR a constant.
#pragma once
#include "da_common.h"

namespace da {
namespace mla {

constexpr int kTile = 32;  // tokens per LDS tile
constexpr int kNBuf = 3;   // LDS tile buffers (two tiles in flight behind the one being read)
constexpr float kLazy = 8.0f;  // the running maximum moves only when exceeded by this much (log2 units)
constexpr int kKPD = 8;  // K fragments read from LDS ahead of the MFMA that uses them
constexpr int kVPD = 6;  // V^T fragment pairs read ahead

typedef short s16x4 __attribute__((__vector_size__(4 * sizeof(short))));

template <typename Tag>
struct Mma;
template <>
struct Mma<f16_tag> {
    typedef f16x8 vec8;
    static __device__ __forceinline__ f32x16 mma(vec8 a, vec8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    // same product with the accumulator pinned to ordinary VGPRs (the score tile: the accumulation
    // registers are all taken by the output tiles)
    static __device__ __forceinline__ void mma_v(vec8 a, vec8 b, f32x16& c) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void mma_v0(vec8 a, vec8 b, f32x16& c) {  // c = a.b
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=v"(c) : "v"(a), "v"(b));
    }
    // the same from assembly with the accumulator in accumulation registers (a fixed place in an instruction
    // sequence written by hand)
    static __device__ __forceinline__ void mma_a(vec8 a, vec8 b, f32x16& c) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
    // two fp32 values -> one register of two 16-bit values, round to nearest even (as an instruction with a fixed place)
    static __device__ __forceinline__ void pack2(uint32_t& dst, float lo, float hi) {
        asm volatile("s_nop 0\n\tv_cvt_pk_f16_f32 %0, %1, %2" : "=v"(dst) : "v"(lo), "v"(hi));
    }
    static __device__ __forceinline__ vec8 pack8(const float* x) {
        vec8 v;
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (_Float16)x[j];
        return v;
    }
};
template <>
struct Mma<bf16_tag> {
    typedef bf16x8 vec8;
    static __device__ __forceinline__ f32x16 mma(vec8 a, vec8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void mma_v(vec8 a, vec8 b, f32x16& c) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void mma_v0(vec8 a, vec8 b, f32x16& c) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=v"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void mma_a(vec8 a, vec8 b, f32x16& c) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void pack2(uint32_t& dst, float lo, float hi) {
        // (s_nop: a result of the transcendental unit needs one wait state before an ordinary vector instruction
        // reads it, and this may directly follow the exp2 of `hi`)
        asm volatile("s_nop 0\n\tv_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(dst) : "v"(lo), "v"(hi));
    }
    static __device__ __forceinline__ vec8 pack8(const float* x) {
        vec8 v;
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (__bf16)x[j];
        return v;
    }
};

// 16 bytes per lane from global memory straight into LDS at lds_off + lane * 16 (lds_off is
// wave-uniform).  Issued from assembly so that the wait for it is placed by hand: the
// compiler would otherwise drain every outstanding load before the next LDS read.
// The source address is a wave-uniform 64-bit base plus a 32-bit per-lane byte offset.
// STREAM: the load is marked non-temporal (the K/V tiles, read once per call: this GPU's HBM streams 12 % faster that
// way; not Q, which the splits of a sequence share through the L2).
template <bool STREAM = false>
__device__ __forceinline__ void lds_dma16(const void* gbase, uint32_t lane_off, uint32_t lds_off) {
    const uint32_t off = __builtin_amdgcn_readfirstlane(lds_off);
    const uintptr_t b = reinterpret_cast<uintptr_t>(gbase);
    // readfirstlane returns a signed int: go through uint32_t so that the low word is not sign-extended
    const uint64_t base = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b) |
                          ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32)) << 32);
    if constexpr (STREAM)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt" ::"v"(lane_off), "s"(base), "s"(off)
                     : "memory");
    else
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(off)
                     : "memory");
}

// The same with a full per-lane address (rows of different pages in one load).
template <bool STREAM = false>
__device__ __forceinline__ void lds_dma16_v(const void* lane_addr, uint32_t lds_off) {
    const uint32_t off = __builtin_amdgcn_readfirstlane(lds_off);
    if constexpr (STREAM)
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" ::"v"(lane_addr), "s"(off) : "memory");
    else
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(lane_addr), "s"(off) : "memory");
}

// x *= alpha for an MFMA accumulator element that lives in an accumulation register.  Written as
// assembly on the AGPR so that the (rare) rescale path does not pull the 256 accumulators of a
// wave into ordinary VGPRs around the whole loop.
__device__ __forceinline__ void scale_acc(float& x, float alpha) {
    float tmp;
    asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 %0, %1"
                 : "+a"(x), "=&v"(tmp)
                 : "v"(alpha));
}

// LDS reads issued from assembly, in program order and with hand-placed waits.  Left to itself the compiler
// sinks these reads next to their use to save registers (the kernel sits at the register limit), which leaves
// one or two reads in flight; a single wavefront per SIMD then stalls on LDS latency before every MFMA.
template <int OFF, typename V>
__device__ __forceinline__ void lds_read_b128(V& dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void lds_read_tr16_b64(s16x4& dst, uint32_t addr) {
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
// Wait until at most N LDS reads are outstanding; the operands pass through so that no consumer of them can
// be scheduled ahead of the wait.
template <int N, typename V>
__device__ __forceinline__ void wait_lgkm(V& x) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x) : "n"(N));
}
template <int N, typename V>
__device__ __forceinline__ void wait_lgkm(V& x, V& y) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(x), "+v"(y) : "n"(N));
}

// Chunk swizzles of the two tile regions (see the header comment).
__device__ __forceinline__ int swz_a(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }
__device__ __forceinline__ int swz_b(int r) { return (r >> 1) & 7; }

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

}  // namespace mla
}  // namespace da
