// Single-query attention for a group of query heads that share one KV head (GQA / MQA), with
// both contractions on the matrix cores so that the sweep stays bandwidth-bound for any group
// size (wave64, gfx950).
//
// One work-group of four wavefronts serves one (sequence, KV head, group of up to 16*NT query
// heads, sequence split).  Wavefronts do not share data while streaming: each takes every
// fourth 32-token tile of the split and keeps its own online-softmax state; the four states
// are merged through LDS at the end.  Per tile and wavefront:
//
//   K rows go from global memory straight into MFMA A-operand layout (16-byte loads: lane
//   (n, g) takes bytes [(ks*4+g)*16, +16) of row n, so one instruction reads 64 contiguous
//   bytes of 16 rows), and  S^T[16 tok x 16 heads] = K . Q^T  accumulates over D/32 k-steps
//   of v_mfma_f32_16x16x32 with the Q rows held in registers as B-operands.
//
//   The score tile leaves the MFMA with one head per lane (column n) and 4 tokens per lane, so
//   the online softmax is lane-local except for the maximum across the four 16-lane groups,
//   and two score tiles (32 tokens) are exactly one B-operand of the second product.
//
//   V rows are loaded coalesced, parked in a wave-private LDS tile, and read back transposed
//   (ds_read_b64_tr_b16: 8 tokens of one column per lane) as the A-operand of
//   O^T[DV x 16 heads] += V^T . P^T.
//
// The latent form with up to 16 query heads (D = 576, DV = 512, V the first 512 columns of each K row: a
// tensor-parallel shard of an MLA model) runs here too: the rows are loaded once, as K, and their value columns are
// parked in the LDS tile from the K registers.
//
// Mathematics as in the reference kernel (csrc/kernel/decoding_attn/decoding_fwd_kernel.h:50-235,
// head mapping block_info.h:14-30); the reference streams K and V once per query head on CUDA
// cores and keeps the whole score row in shared memory.
#pragma once
#include "da_common.h"

namespace da {

typedef short s16x4_t __attribute__((__vector_size__(4 * sizeof(short))));
typedef short s16x8_t __attribute__((__vector_size__(8 * sizeof(short))));

template <typename Tag>
struct Mma16;
template <>
struct Mma16<f16_tag> {
    typedef f16x8 vec8;
    static __device__ __forceinline__ f32x4 mma(vec8 a, vec8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    // the same product with the second operand held in accumulation registers (frees ordinary ones where a kernel
    // is short of them); issued from assembly, so the caller pads the result hazard itself (settle)
    // (the wait states in front cover an operand that a vector instruction has just written)
    static __device__ __forceinline__ void mma_bacc(vec8 a, const vec8& b, f32x4& c) {
        asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
    }
    static __device__ __forceinline__ void mma_bacc0(vec8 a, const vec8& b, f32x4& c) {  // c = a.b
        asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=v"(c) : "v"(a), "a"(b));
    }
    static __device__ __forceinline__ vec8 pack8(const float* x) {
        vec8 v;
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (_Float16)x[j];
        return v;
    }
};
template <>
struct Mma16<bf16_tag> {
    typedef bf16x8 vec8;
    static __device__ __forceinline__ f32x4 mma(vec8 a, vec8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void mma_bacc(vec8 a, const vec8& b, f32x4& c) {
        asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
    }
    static __device__ __forceinline__ void mma_bacc0(vec8 a, const vec8& b, f32x4& c) {
        asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=v"(c) : "v"(a), "a"(b));
    }
    static __device__ __forceinline__ vec8 pack8(const float* x) {
        vec8 v;
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (__bf16)x[j];
        return v;
    }
};

// x rounded to the 16-bit compute type and widened again
template <typename Tag>
__device__ __forceinline__ float round16(float x) {
    if constexpr (std::is_same<Tag, bf16_tag>::value)
        return (float)(__bf16)x;
    else
        return (float)(_Float16)x;
}

// Wait states between the last matrix instruction issued from assembly and the first ordinary read of its result
// (the compiler cannot see into the assembly to place them).
__device__ __forceinline__ void settle(f32x4& c) { asm volatile("s_nop 15\n\ts_nop 3" : "+v"(c)); }

constexpr int kGqaTile = 32;  // tokens per wave iteration

template <int DV>
constexpr int gqa_v_pitch() { return DV * 2 + 32; }  // LDS row pitch of the V tile: conflict-free transposed reads

template <int DV>
constexpr int gqa_merge_pitch() { return DV + 4; }  // floats per row of the merge area: conflict-free row writes

constexpr int kGqaTokBytes = 512;  // per wave and pair of a row: the (scale, zero) pairs of a tile's tokens, K and V

template <int DV>
constexpr size_t gqa_lds_bytes(int nt, int tok_pairs = 0) {
    // V tiles of the four waves (and, behind them, their tiles' per-token pairs), reused for the final merge
    // ([4][heads][pitch] floats + (m, l))
    const size_t vt = 4 * (size_t)kGqaTile * gqa_v_pitch<DV>() + (size_t)tok_pairs * 4 * kGqaTokBytes;
    const size_t mg = 4 * (size_t)(16 * nt) * (gqa_merge_pitch<DV>() + 2) * sizeof(float);
    return vt > mg ? vt : mg;
}

// WH (wave per head): the four wavefronts of a work-group take four consecutive KV heads over the same
// tokens, so together they read whole [token][4 heads][D] rows (1 KiB contiguous for D = 128) at about the
// same time, which HBM serves measurably faster than four streams of 256-byte pieces; no merge is needed.
// Otherwise (head_k not a multiple of 4) the wavefronts split the tokens of one KV head and merge at the end.
// MINW: wavefronts per SIMD the register allocation must leave room for (2 caps the kernel at 256 registers
// and keeps the accumulators in ordinary VGPRs, so the rescale needs no accumulation-register copies).
// KV8: K and V hold 8-bit elements (1 = FP8 e4m3, 2 = int8; 0 = 16-bit K/V).  Loads stay 16 bytes per lane
// (sixteen elements: the k indices of two consecutive k-steps, so the Q fragments are gathered with the matching
// index order) and the elements are converted exactly to the compute type on their way into the matrix instruction
// (K) or the LDS tile (V).
// One segment of work: tokens [c0, c1) of sequence b (first row `start`, `len` tokens) for the KV heads and head
// group `by` selects (blockIdx.y, or its renumbered stand-in).  `direct`: the segment is the whole sequence, so the result goes to o; otherwise the
// un-normalised partial of head h goes to workspace row part0 + h * part_stride.
// PGM: how paged K/V is addressed.  0: one page lookup per tile (pages hold a multiple of 32 tokens; also the packed
// layout); 1: 16-token pages, a tile is fetched as two runs of 16 tokens, each from one page; 2: smaller pages, every
// lane looks up the page of the row it loads.
template <typename Tag, int D, int DV, int NT, bool PREFETCH, bool WH, int KV8, int PGM>
__device__ __forceinline__ void gqa_segment(const SweepParams& p, uint8_t* const smem, const int by, const int b,
                                            const int start, const int len, const int c0, const int c1,
                                            const size_t part0, const int part_stride, const bool direct) {
    using MM = Mma16<Tag>;
    using vec8 = typename MM::vec8;
    using EL = Elem<Tag>;
    constexpr int KS = D / 32;      // k-steps of Q K^T
    constexpr int CT = DV / 16;     // 16-column tiles of the output
    constexpr int CPR = DV / 8;     // 16-byte chunks per V row
    constexpr int VP = gqa_v_pitch<DV>();
    constexpr int NW = WH ? 1 : 4;  // wavefronts that share the tokens of one KV head
    constexpr int HG = 16 * NT;     // query heads per KV head and work-group
    constexpr float kLazy = 8.0f;   // the running maximum moves only when exceeded by this much (log2 units)
    constexpr int FMT = KV8 & 7;                    // element format (kKvFp8, kKvInt8, kKvInt4; 0 = 16-bit)
    // TOK: every (token, KV head) row has its own (scale, zero) pair (p.k_tok, p.v_tok): with integers n,
    // K[t][c] = a_k[t] (n[t][c] - z_k[t]), so q . K[t] = a_k[t] (q . n[t] - z_k[t] sum_c q[c]): the matrix
    // instruction works on the integers, and the score tile takes one multiply-add per element with the sum of the
    // head's q row.  V[t][c] = a_v[t] (n[t][c] - z_v[t]) likewise: the probabilities are multiplied by a_v[t] on
    // their way into the second product, and sum_t p'[t] z_v[t], one number per head, comes off every column at the end.
    constexpr bool TOK = (KV8 & kKvPerToken) != 0;
    // NG: pairs per row.  With kKvGroup64 every run of 64 elements of a row has its own pair: a run is what two
    // consecutive k-steps of the score product cover (8-bit layouts) and what four 16-column tiles of the output
    // cover, so the score tile is summed per run before the factors go on, and the second product takes a
    // probability operand per run.
    constexpr int NG = (TOK && (KV8 & kKvGroup64) != 0) ? D / 64 : 1;
    static_assert(NG == 1 || (D == DV && D % 64 == 0), "one pair per 64 elements");
    // B4: an int4 cache.  Its nibbles reach the matrix instructions as kInt4Bias + n (int4x8_biased), the eight
    // elements of a word in the order 0, 4, 1, 5, 2, 6, 3, 7: Q is gathered in that order, the bias leaves the scores
    // through the sum of the head's q row and the outputs through the sum of the rounded probabilities, and the
    // output columns, which come out in that order within every run of eight, are put right after the last tile.
    constexpr bool B4 = FMT == kKvInt4;
    const uint32_t b4_one = B4 ? int4_biased_one<Tag>() : 0u;
    auto convert8 = [&](uint2 w) __attribute__((always_inline)) {
        if constexpr (B4)
            return int4x8_biased<Tag>(w.x, b4_one);
        else if constexpr (FMT != 0)
            return kv8x8_to_16<Tag, FMT>(w);
        else
            return make_uint4(w.x, w.y, 0u, 0u);  // (16-bit K/V: never called)
    };
    constexpr int KB = KV8 ? 1 : 2;                 // bytes per K/V element
    constexpr int KSR = KV8 ? KS / 2 : KS;          // K registers (16 bytes) per 16-token tile
    constexpr int CPRL = KV8 ? DV / 16 : CPR;       // 16-byte chunks per V row as loaded
    // VK: V is the first DV columns of each K row (the latent form, D = 576 and DV = 512).  The rows are loaded once,
    // as K, and their value columns go to the LDS tile from the K registers after the score products.
    constexpr bool VK = D != DV;
    constexpr int NVR = VK ? 1 : kGqaTile * CPRL / 64;  // V registers (16 bytes) per tile
    static_assert(!VK || (DV < D && DV % 64 == 0), "value columns inside the key rows");
    static_assert(D % 32 == 0 && DV % 16 == 0 && (kGqaTile * CPR) % 64 == 0, "shape");
    static_assert(!KV8 || (D % 64 == 0 && (kGqaTile * CPRL) % 64 == 0), "8-bit K/V: two k-steps per 16-byte load");
    static_assert(!TOK || (!VK && (FMT == kKvInt8 || FMT == kKvInt4)), "per-token factors: integer K/V, V of its own");

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 15;
    const int g = lane >> 4;

    const int hk = WH ? (by / p.groups) * 4 + wave : by / p.groups;
    const int grp = by % p.groups;
    const int tw = WH ? 0 : wave;  // this wave's position among the waves that share the tokens

    const int h_base = hk * p.ratio + grp * HG;
    const int nh = min(HG, p.ratio - grp * HG);  // live heads of this group
    uint16_t* const o16 = reinterpret_cast<uint16_t*>(p.o);

    if (c0 >= c1) {
        // every wave of the work-group sees the same (sequence, split), so they all leave together; the
        // work-group covers NR runs of nh heads, one per KV head
        constexpr int NR = WH ? 4 : 1;
        const int wg_h_first = (WH ? (by / p.groups) * 4 : hk) * p.ratio + grp * HG;
        if (direct) zero_rows<DV>(p, b, wg_h_first, nh, NR, p.ratio);
        return;
    }

    // Q rows as B-operands: lane (n, g) holds Q[head nt*16+n][(ks*4+g)*8 .. +8)
    vec8 qf[NT][KS];
    float slope[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int h = h_base + min(nt * 16 + n, nh - 1);
        const uint16_t* qrow = reinterpret_cast<const uint16_t*>(p.q) + ((size_t)b * p.head_q + h) * D;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            // k indices this lane contributes to k-step ks: those of the K fragment it will hold
            const int at = KV8 ? (ks >> 1) * 64 + g * 16 + (ks & 1) * 8 : ks * 32 + g * 8;
            qf[nt][ks] = __builtin_bit_cast(vec8, *reinterpret_cast<const uint4*>(qrow + at));
            if constexpr (B4) qf[nt][ks] = __builtin_shufflevector(qf[nt][ks], qf[nt][ks], 0, 4, 1, 5, 2, 6, 3, 7);
        }
        slope[nt] = p.is_alibi ? alibi_slope_log2(p.slopes, h, p.head_q) : 0.0f;
    }
    // (TOK, B4) sum of each head's q row: the four 16-lane groups hold different elements of the same rows
    float qsum[NT][NG];  // (per run of the row when the pairs are)
    if constexpr (TOK || B4) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int qg = 0; qg < NG; ++qg) {
                // (a dot product with ones: one instruction per pair of elements)
                constexpr uint32_t kOnes = std::is_same<Tag, f16_tag>::value ? 0x3C003C00u : 0x3F803F80u;
                float acc_q = 0.0f;
#pragma unroll
                for (int ks = qg * (KS / NG); ks < (qg + 1) * (KS / NG); ++ks) {
                    const uint4 w = __builtin_bit_cast(uint4, qf[nt][ks]);
                    acc_q = EL::dot2(w.x, kOnes, acc_q);
                    acc_q = EL::dot2(w.y, kOnes, acc_q);
                    acc_q = EL::dot2(w.z, kOnes, acc_q);
                    acc_q = EL::dot2(w.w, kOnes, acc_q);
                }
                acc_q += __shfl_xor(acc_q, 16);
                acc_q += __shfl_xor(acc_q, 32);
                qsum[nt][qg] = acc_q;
            }
    }

    f32x4 acc[NT][CT];
    float m[NT], l[NT];
    float corr[NT][NG];  // (TOK) sum over tokens of p'[t] z_v[t], in the accumulators' units
    // (bf16, NG > 1) the denominators under the other runs' V scales: a probability rounded to eight bits for one run
    // is not the one rounded for another, and each run's columns are divided by the sum of what they were multiplied
    // by (the columns are brought to l's units after the last tile)
    constexpr bool LQ = NG > 1 && std::is_same<Tag, bf16_tag>::value;
    float lq[NT][NG];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        m[nt] = kNegBig;
        l[nt] = 0.0f;
#pragma unroll
        for (int qg = 0; qg < NG; ++qg) corr[nt][qg] = lq[nt][qg] = 0.0f;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc[nt][ct] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }

    // wave-uniform byte bases (scalar registers) and 32-bit per-lane byte offsets
    // (a tile of kGqaTile tokens starts at a multiple of kGqaTile within the sequence; pages of paged K/V hold a
    // multiple of kGqaTile tokens, so one row_ref per tile locates it, or, with HP, 16 tokens: one per half)
    const uint8_t* const kbytes = reinterpret_cast<const uint8_t*>(p.k) + (size_t)hk * D * KB;
    const uint8_t* const vbytes = reinterpret_cast<const uint8_t*>(p.v) + (size_t)hk * p.v_head * KB;
    const uint32_t k_row_b = (uint32_t)p.k_row * KB, v_row_b = (uint32_t)p.v_row * KB;
    // (an int4 cache's elements come out of the conversion times a power of two, divided out here)
    const float sl = p.scale_log2 * head_scale(p.k_scale, hk);  // score scale, log2 units
    const float vs = head_scale(p.v_scale, hk);
    // (B4, per-head factors) the bias' share of every score of head nt, in log2 units
    float bias_q[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) bias_q[nt] = (B4 && !TOK) ? kInt4Bias * sl * qsum[nt][0] : 0.0f;

    // wave-private V tile in LDS
    uint8_t* const vt = smem + wave * (kGqaTile * VP);
    // transposed-read address of this lane: 16-lane group g reads rows g*4 .. g*4+3 (and +16), 16 columns
    const uint8_t* const v_rd = vt + (g * 4 + (n >> 2)) * VP + (n & 3) * 8;
    typedef __attribute__((address_space(3))) s16x4_t* lds_s4;

    // One tile in registers: K in A-operand layout [16-token tile][k-step], V row-major chunks.  There is a
    // single register set: the loads of the next tile are issued as soon as this tile's registers are free
    // (V once it is parked in LDS, K once the score MFMAs have read it), so they fly during the rest of the
    // tile's work without doubling the register footprint.
    struct TileRegs {
        uint4 k[2][KSR];
        uint4 v[NVR];
        float2 tokp[NG];  // (TOK) lanes 0 .. 31: the K pairs of the tile's token `lane`; 32 .. 63: the V pairs of lane - 32
    };
    TileRegs tr;

    // Rows past the end re-read the last valid row (in whichever run of 16 that is, with 16-token pages) and are
    // masked.  The choice between the two runs is wave-uniform: an M-tile of K is one run, and a V load instruction
    // covers a power-of-two number of rows inside one run, except for d = 96 (12 chunks per row), which chooses
    // per lane.
    constexpr bool HP = PGM == 1;
    // per-lane address of row `row` of the tile at tok0 (PGM == 2): its page from the block table, then the row in it
    auto lane_row = [&](int tok0, int row, const uint8_t* bytes, int64_t page_stride, uint32_t row_bytes) {
        const int tok = tok0 + row;
        const int page = p.block_table[(int64_t)b * p.max_blocks + (tok >> p.page_shift)];
        return bytes + ((int64_t)page * page_stride * KB + (int64_t)(tok & ((1 << p.page_shift) - 1)) * row_bytes);
    };
    // K/V rows are read once per call: non-temporal loads (see stream_load16).  Not in the latent form, whose rows
    // serve several head groups from the caches and which measured slower with the hint (16 heads, batch 64 x 4096
    // tokens: 63.8 -> 67.2 us), and not where a head's row is no whole number of 128-byte lines (d = 96: 192 bytes;
    // 8-bit K/V at d = 64): the line two neighbouring heads share would be dropped after the first one's read and
    // fetched again for the second (32/8 heads d 96, batch 256 x 4096 tokens: 594.5 us with the hint, 544.6 without;
    // batch 16 x 4096: 39.9 and 32.9).
    auto kv_load16 = [](const uint8_t* ptr) __attribute__((always_inline)) {
        if constexpr (FMT == kKvInt4)
            return kv4_load16(ptr);  // (eight bytes from half the address, widened to sixteen int8 elements)
        else if constexpr (VK || (D * KB) % 128 != 0)
            return *reinterpret_cast<const uint4*>(ptr);
        else
            return stream_load16(ptr);
    };
    auto load_k = [&](int tok0, TileRegs& r) __attribute__((always_inline)) {
        const int last = c1 - 1 - tok0;
        if constexpr (PGM == 2) {
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
                const uint8_t* const row = lane_row(tok0, min(mt * 16 + n, last), kbytes, p.k_page, k_row_b) + g * 16;
#pragma unroll
                for (int ks = 0; ks < KSR; ++ks) r.k[mt][ks] = kv_load16(row + ks * 64);
            }
            return;
        }
        const uint8_t* const base0 = kbytes + row_ref(p, b, start, tok0).k * KB;
        const uint8_t* base1 = base0;
        if constexpr (HP)
            if (last >= 16) base1 = kbytes + row_ref(p, b, start, tok0 + 16).k * KB;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            const bool second = HP && mt == 1 && last >= 16;
            const uint8_t* const base = second ? base1 : base0;
            const uint32_t off = (uint32_t)(min(mt * 16 + n, last) - (second ? 16 : 0)) * k_row_b + g * 16;
#pragma unroll
            for (int ks = 0; ks < KSR; ++ks) r.k[mt][ks] = kv_load16(base + off + ks * 64);
        }
    };
    // (TOK) one pair per lane and tile, rows past the end as the last valid one; the wave passes them through its
    // corner of LDS (tokbuf: K scales, K zeros, V scales, V zeros, 32 floats each per run of the row) to the lanes
    // that need them
    float* const tokbuf = reinterpret_cast<float*>(smem + 4 * kGqaTile * VP + wave * (NG * kGqaTokBytes));
    auto load_tok = [&](int tok0, TileRegs& r) __attribute__((always_inline)) {
        if constexpr (TOK) {
            const int row = min(lane & 31, c1 - 1 - tok0);
            int64_t at;  // the row's number in the pools' row numbering (a page holds 2^page_shift rows)
            if (p.block_table == nullptr) {
                at = (int64_t)start + tok0 + row;
            } else if constexpr (PGM == 0) {
                at = ((int64_t)page_of(p, b, tok0) << p.page_shift) + ((tok0 & ((1 << p.page_shift) - 1)) + row);
            } else {
                const int tok = tok0 + row;
                at = ((int64_t)p.block_table[(int64_t)b * p.max_blocks + (tok >> p.page_shift)] << p.page_shift) +
                     (tok & ((1 << p.page_shift) - 1));
            }
            const float2* const pool = reinterpret_cast<const float2*>(lane < 32 ? p.k_tok : p.v_tok);
#pragma unroll
            for (int qg = 0; qg < NG; ++qg) r.tokp[qg] = pool[(at * p.head_k + hk) * NG + qg];
        }
    };
    auto load_v = [&](int tok0, TileRegs& r) __attribute__((always_inline)) {
        const int last = c1 - 1 - tok0;
        if constexpr (PGM == 2) {
#pragma unroll
            for (int i = 0; i < NVR; ++i) {
                const int slot = i * 64 + lane;
                const int row = slot / CPRL, ch = slot % CPRL;
                r.v[i] = kv_load16(lane_row(tok0, min(row, last), vbytes, p.v_page, v_row_b) + ch * 16);
            }
            return;
        }
        const uint8_t* const base0 = vbytes + row_ref(p, b, start, tok0).v * KB;
        const uint8_t* base1 = base0;
        if constexpr (HP)
            if (last >= 16) base1 = vbytes + row_ref(p, b, start, tok0 + 16).v * KB;
        constexpr bool kUniform = 64 % CPRL == 0 && 16 % (64 / CPRL) == 0;
#pragma unroll
        for (int i = 0; i < NVR; ++i) {
            const int slot = i * 64 + lane;
            const int row = slot / CPRL, ch = slot % CPRL;
            const bool second = HP && (kUniform ? i * (64 / CPRL) >= 16 : row >= 16) && last >= 16;
            const uint8_t* const base = second ? base1 : base0;
            const uint32_t off = (uint32_t)(min(row, last) - (second ? 16 : 0)) * v_row_b + ch * 16;
            r.v[i] = kv_load16(base + off);
        }
    };

    const int ntiles = (c1 - c0 + kGqaTile - 1) / kGqaTile;
    if (tw < ntiles) {
        if constexpr (!VK) load_v(c0 + tw * kGqaTile, tr);
        load_k(c0 + tw * kGqaTile, tr);
        load_tok(c0 + tw * kGqaTile, tr);
    }

    // (A second register set, refilled two tiles ahead, was measured for the 8-bit and 4-bit formats, whose tiles are
    // half and a quarter of the bytes, and for the 32-heads-per-wave form, whose CUs hold one wave per SIMD: no gain
    // anywhere, a loss on short sequences.  GQA int4 batch 64 x 4096 62.0 us against 59.9, MHA int4 batch 512 x 128
    // 68.5 against 63.2, MQA fp16 batch 32 x 4096 21.6 against 20.8.)
    for (int t = tw; t < ntiles; t += NW) {
        const int tok0 = c0 + t * kGqaTile;
        const bool more = t + NW < ntiles;
        const int tok_next = tok0 + NW * kGqaTile;

        // park V in LDS (row-major, padded pitch), then refill the V registers
        if constexpr (!VK) {
#pragma unroll
        for (int i = 0; i < NVR; ++i) {
            const int slot = i * 64 + lane;
            const int row = slot / CPRL, ch = slot % CPRL;
            if constexpr (KV8) {  // sixteen 8-bit elements become 32 bytes of the 16-bit tile
                *reinterpret_cast<uint4*>(vt + row * VP + ch * 32) =
                    convert8(make_uint2(tr.v[i].x, tr.v[i].y));
                *reinterpret_cast<uint4*>(vt + row * VP + ch * 32 + 16) =
                    convert8(make_uint2(tr.v[i].z, tr.v[i].w));
            } else {
                *reinterpret_cast<uint4*>(vt + row * VP + ch * 16) = tr.v[i];
            }
        }
        // The K registers of this tile, the only loads still in flight, are needed right after: wait for them here,
        // before the V loads of the next tile are issued (on both sides of the branch: the compiler's bookkeeping
        // joins them).  Left to itself the compiler puts a wait for everything behind those V loads, which holds
        // the wave for a whole memory latency every tile.
        if constexpr (PREFETCH) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), the other counters untouched
        if (PREFETCH && more) load_v(tok_next, tr);
        }

        // S^T = K . Q^T for the two 16-token tiles, then refill the K registers
        f32x4 s[2][NT];
        f32x4 sq[2][NT][NG];  // (NG > 1) the sums of the row's runs, apart
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                f32x4 c = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    if constexpr (NG > 1) {
                        if (ks % (KS / NG) == 0 && ks != 0) {
                            sq[mt][nt][ks / (KS / NG) - 1] = c;
                            c = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                        }
                    }
                    uint4 kfrag;
                    if constexpr (KV8) {
                        const uint4 w = tr.k[mt][ks >> 1];
                        kfrag = convert8((ks & 1) ? make_uint2(w.z, w.w) : make_uint2(w.x, w.y));
                    } else {
                        kfrag = tr.k[mt][ks];
                    }
                    if constexpr (VK) {  // (Q in accumulation registers: the ordinary ones hold the K tile)
                        if (ks == 0)
                            MM::mma_bacc0(__builtin_bit_cast(vec8, kfrag), qf[nt][ks], c);
                        else
                            MM::mma_bacc(__builtin_bit_cast(vec8, kfrag), qf[nt][ks], c);
                    } else
                        c = MM::mma(__builtin_bit_cast(vec8, kfrag), qf[nt][ks], c);
                }
                if constexpr (VK) settle(c);
                s[mt][nt] = c;
                sq[mt][nt][NG - 1] = c;
            }
        if constexpr (VK) {
            // the value columns of the tile, from the K registers: lane (n, g) holds 16-byte chunk ks * 4 + g of row
            // mt * 16 + n (8-bit: elements [64 j + 16 g, +16) of it in register j)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
                uint8_t* const row = vt + (mt * 16 + n) * VP;
                if constexpr (KV8) {
#pragma unroll
                    for (int j = 0; j < DV / 64; ++j) {
                        const uint4 w = tr.k[mt][j];
                        *reinterpret_cast<uint4*>(row + j * 128 + g * 32) = convert8(make_uint2(w.x, w.y));
                        *reinterpret_cast<uint4*>(row + j * 128 + g * 32 + 16) =
                            convert8(make_uint2(w.z, w.w));
                    }
                } else {
#pragma unroll
                    for (int ks = 0; ks < DV / 32; ++ks)
                        *reinterpret_cast<uint4*>(row + (ks * 4 + g) * 16) = tr.k[mt][ks];
                }
            }
        }
        if (PREFETCH && more) load_k(tok_next, tr);

        // online softmax; token of s[mt][nt][r]: tok0 + mt*16 + g*4 + r, head nt*16 + n
        vec8 pf[NT];
        vec8 pfg[NT][NG];  // (NG > 1) the probabilities under the V scales of the row's runs
        const bool tail = tok0 + kGqaTile > c1;
        float x[NT][8], mx[NT];
        // (TOK) per token (and run): A = score scale x a_k, Z = z_k plus the conversion's bias; x = sum A (s - Z qsum)
        float tokA[NG][TOK ? 8 : 1], tokZ[NG][TOK ? 8 : 1], tokV[NG][TOK ? 8 : 1], tokW[NG][TOK ? 8 : 1], tokVinv[NG][TOK ? 8 : 1];
        if constexpr (TOK) {
            // tokbuf[((kind * NG + run) * 32 + token]: kind 0 K scale, 1 K zero, 2 V scale, 3 V zero
            float* const mine = tokbuf + (lane >> 5) * (2 * NG * 32) + (lane & 31);
#pragma unroll
            for (int qg = 0; qg < NG; ++qg) {
                mine[qg * 32] = tr.tokp[qg].x;
                mine[(NG + qg) * 32] = tr.tokp[qg].y;
            }
            if (PREFETCH && more) load_tok(tok_next, tr);
#pragma unroll
            for (int qg = 0; qg < NG; ++qg)
#pragma unroll
                for (int mt = 0; mt < 2; ++mt) {
                    const f32x4 ak = *reinterpret_cast<const f32x4*>(tokbuf + (0 * NG + qg) * 32 + mt * 16 + g * 4);
                    const f32x4 zk = *reinterpret_cast<const f32x4*>(tokbuf + (1 * NG + qg) * 32 + mt * 16 + g * 4);
                    const f32x4 av = *reinterpret_cast<const f32x4*>(tokbuf + (2 * NG + qg) * 32 + mt * 16 + g * 4);
                    const f32x4 zv = *reinterpret_cast<const f32x4*>(tokbuf + (3 * NG + qg) * 32 + mt * 16 + g * 4);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        tokA[qg][mt * 4 + r] = sl * ak[r];
                        tokZ[qg][mt * 4 + r] = zk[r] + (B4 ? kInt4Bias : 0.0f);
                        tokV[qg][mt * 4 + r] = av[r];
                        tokW[qg][mt * 4 + r] = zv[r] + (B4 ? kInt4Bias : 0.0f);
                        if constexpr (std::is_same<Tag, bf16_tag>::value)
                            tokVinv[qg][mt * 4 + r] = __builtin_amdgcn_rcpf(av[r]);
                    }
                }
        }
        // the score of token j = mt * 4 + r under the pairs: sum over the row's runs
        auto tok_score = [&](int mt, int nt, int r) __attribute__((always_inline)) {
            float v = (sq[mt][nt][0][r] - tokZ[0][mt * 4 + r] * qsum[nt][0]) * tokA[0][mt * 4 + r];
#pragma unroll
            for (int qg = 1; qg < NG; ++qg)
                v = __builtin_fmaf(sq[mt][nt][qg][r] - tokZ[qg][mt * 4 + r] * qsum[nt][qg], tokA[qg][mt * 4 + r], v);
            return v;
        };
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            mx[nt] = -INFINITY;
            if constexpr (TOK) {
                if (p.is_alibi || tail) {
#pragma unroll
                    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int tok = tok0 + mt * 16 + g * 4 + r;
                            float v = tok_score(mt, nt, r) + slope[nt] * (float)(tok - (len - 1));
                            if (tok >= c1) v = -INFINITY;
                            x[nt][mt * 4 + r] = v;
                            mx[nt] = fmaxf(mx[nt], v);
                        }
                } else {
#pragma unroll
                    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            x[nt][mt * 4 + r] = tok_score(mt, nt, r);
                            mx[nt] = fmaxf(mx[nt], x[nt][mt * 4 + r]);
                        }
                }
            } else if (p.is_alibi || tail) {
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int tok = tok0 + mt * 16 + g * 4 + r;
                        float v = s[mt][nt][r] * sl + slope[nt] * (float)(tok - (len - 1)) - bias_q[nt];
                        if (tok >= c1) v = -INFINITY;
                        x[nt][mt * 4 + r] = v;
                        mx[nt] = fmaxf(mx[nt], v);
                    }
            } else {
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        x[nt][mt * 4 + r] = B4 ? __builtin_fmaf(s[mt][nt][r], sl, -bias_q[nt]) : s[mt][nt][r] * sl;
                        mx[nt] = fmaxf(mx[nt], x[nt][mt * 4 + r]);
                    }
            }
        }
        // the four 16-lane groups hold different tokens of the same heads
        bool up[NT], any_up = false;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            mx[nt] = max_xor32(max_xor16(mx[nt]));
            up[nt] = mx[nt] > m[nt] + kLazy;
            any_up |= up[nt];
        }
        if (__any(any_up)) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const float mn = up[nt] ? mx[nt] : m[nt];
                const float alpha = fast_exp2(m[nt] - mn);
                m[nt] = mn;
                l[nt] *= alpha;
                if constexpr (TOK) {
#pragma unroll
                    for (int qg = 0; qg < NG; ++qg) {
                        corr[nt][qg] *= alpha;
                        if constexpr (LQ) lq[nt][qg] *= alpha;
                    }
                }
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) acc[nt][ct] *= alpha;
            }
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            float xg[NG][8];  // (NG > 1) probabilities under the other runs' V scales
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if constexpr (TOK) {
                    // the second product's operand is p a_v[t], rounded to 16 bits; the zero-point sum uses the
                    // rounded value, and so does the denominator where the rounding is coarse (bf16)
                    const float pe = fast_exp2(x[nt][j] - m[nt]);
                    const float pv = round16<Tag>(pe * tokV[0][j]);
                    // (a scale of zero: the row adds nothing to the columns and its whole probability to the sum)
                    if constexpr (std::is_same<Tag, bf16_tag>::value)
                        l[nt] += tokV[0][j] != 0.0f ? pv * tokVinv[0][j] : pe;
                    else
                        l[nt] += pe;
                    corr[nt][0] = __builtin_fmaf(pv, tokW[0][j], corr[nt][0]);
                    x[nt][j] = pv;
#pragma unroll
                    for (int qg = 1; qg < NG; ++qg) {
                        const float pq = round16<Tag>(pe * tokV[qg][j]);
                        corr[nt][qg] = __builtin_fmaf(pq, tokW[qg][j], corr[nt][qg]);
                        if constexpr (LQ) lq[nt][qg] += tokV[qg][j] != 0.0f ? pq * tokVinv[qg][j] : pe;
                        xg[qg][j] = pq;
                    }
                } else if constexpr (B4) {
                    x[nt][j] = fast_exp2(x[nt][j] - m[nt]);  // (rounded by pack8; the denominator follows below)
                } else {
                    x[nt][j] = as_second_operand<Tag>(fast_exp2(x[nt][j] - m[nt]));
                    l[nt] += x[nt][j];
                }
            }
            pf[nt] = MM::pack8(x[nt]);  // k index j <-> token g*4+j (j<4), 16+g*4+(j-4) (j>=4)
            pfg[nt][0] = pf[nt];
#pragma unroll
            for (int qg = 1; qg < NG; ++qg) pfg[nt][qg] = MM::pack8(xg[qg]);
            if constexpr (B4 && !TOK) {
                // the denominator sums the probabilities as rounded for the matrix instruction (it is also what the
                // bias is taken out with): a dot product of the packed pairs with ones
                constexpr uint32_t kOnes = std::is_same<Tag, f16_tag>::value ? 0x3C003C00u : 0x3F803F80u;
                const uint4 pw = __builtin_bit_cast(uint4, pf[nt]);
                l[nt] = EL::dot2(pw.x, kOnes, l[nt]);
                l[nt] = EL::dot2(pw.y, kOnes, l[nt]);
                l[nt] = EL::dot2(pw.z, kOnes, l[nt]);
                l[nt] = EL::dot2(pw.w, kOnes, l[nt]);
            }
        }

        // O^T += V^T . P^T
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(v_rd + ct * 32));
            const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(v_rd + ct * 32 + 16 * VP));
            const s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            const vec8 a = __builtin_bit_cast(vec8, both);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[nt][ct] = MM::mma(a, pfg[nt][NG > 1 ? ct / (CT / NG) : 0], acc[nt][ct]);
        }

        if (!PREFETCH && more) {
            if constexpr (!VK) load_v(tok_next, tr);
            load_k(tok_next, tr);
            load_tok(tok_next, tr);
        }
    }

    // denominators: each 16-lane group summed its own tokens
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        l[nt] += __shfl_xor(l[nt], 16);
        l[nt] += __shfl_xor(l[nt], 32);
        if constexpr (TOK) {  // the zero points' share (and the bias') comes off every column of the head
#pragma unroll
            for (int qg = 0; qg < NG; ++qg) {
                corr[nt][qg] += __shfl_xor(corr[nt][qg], 16);
                corr[nt][qg] += __shfl_xor(corr[nt][qg], 32);
            }
            float to_l[NG];  // (LQ) run's denominator -> l
            to_l[0] = 1.0f;
            if constexpr (LQ) {
#pragma unroll
                for (int qg = 1; qg < NG; ++qg) {
                    float d = lq[nt][qg];
                    d += __shfl_xor(d, 16);
                    d += __shfl_xor(d, 32);
                    to_l[qg] = d > 0.0f ? l[nt] * __builtin_amdgcn_rcpf(d) : 1.0f;
                }
            }
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const int qg = NG > 1 ? ct / (CT / NG) : 0;
                acc[nt][ct] -= corr[nt][qg];
                if constexpr (LQ)
                    if (qg > 0) acc[nt][ct] *= to_l[qg];
            }
        } else if constexpr (B4) {  // sum_t p (bias + n) = sum_t p n + bias l
            const float off = kInt4Bias * l[nt];
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) acc[nt][ct] -= off;
        }
        if constexpr (B4) {
            // Columns: a run of eight lies in the conversion's order 0, 4, 1, 5 (this lane, 16-lane group g even) and
            // 2, 6, 3, 7 (lane + 16, g odd).  The even group keeps columns 0 and 1 and takes 2 and 3 from its
            // neighbour, the odd one keeps 6 and 7 and takes 4 and 5.
            // v_permlane16_swap(x, y) hands the odd groups' x the even groups' y (of lane - 16) and the even groups' y
            // the odd groups' x (of lane + 16): two of them per tile of sixteen columns.
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                // (elements are copied to scalars first: a bit cast applied to a vector element reads element 0)
                const float a0 = acc[nt][ct][0], a1 = acc[nt][ct][1], a2 = acc[nt][ct][2], a3 = acc[nt][ct][3];
                const auto s01 = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned, a0),
                                                                  __builtin_bit_cast(unsigned, a1), false, false);
                const unsigned c04 = s01[0], c26 = s01[1];
                const auto s23 = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned, a2),
                                                                  __builtin_bit_cast(unsigned, a3), false, false);
                const unsigned c15 = s23[0], c37 = s23[1];
                acc[nt][ct] = f32x4{__builtin_bit_cast(float, c04), __builtin_bit_cast(float, c15),
                                    __builtin_bit_cast(float, c26), __builtin_bit_cast(float, c37)};
            }
        }
    }

    if constexpr (WH) {
        // every wave owns its heads outright: finish from registers.  acc[nt][ct][r] is head nt*16+n,
        // column ct*16 + g*4 + r.
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int hh = nt * 16 + n;
            if (hh < nh) {
                const int h = h_base + hh;
                if (direct) {
                    const float inv = vs / l[nt];
                    uint16_t* orow = o16 + ((size_t)b * p.head_q + h) * DV + g * 4;
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        ushort4 w;
                        w.x = EL::from_f32(acc[nt][ct][0] * inv);
                        w.y = EL::from_f32(acc[nt][ct][1] * inv);
                        w.z = EL::from_f32(acc[nt][ct][2] * inv);
                        w.w = EL::from_f32(acc[nt][ct][3] * inv);
                        *reinterpret_cast<ushort4*>(orow + ct * 16) = w;
                    }
                } else {
                    const size_t part = part0 + (size_t)h * part_stride;
                    float* wrow = p.ws_o + part * DV + g * 4;
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) *reinterpret_cast<f32x4*>(wrow + ct * 16) = acc[nt][ct] * vs;
                    if (g == 0) {
                        p.ws_ml[part * 2 + 0] = m[nt];
                        p.ws_ml[part * 2 + 1] = l[nt];
                    }
                }
            }
        }
        return;
    }

    // merge the four waves through LDS (the V tiles are dead by now).  Rows are padded by four floats so that the
    // sixteen heads a 16-lane group writes (one row each, same columns) fall into different banks.
    constexpr int MW = 4;
    constexpr int AP = gqa_merge_pitch<DV>();
    __syncthreads();
    float* const lds_acc = reinterpret_cast<float*>(smem);                 // [MW][HG][AP]
    float* const lds_ml = lds_acc + MW * HG * AP;                          // [MW][HG][2]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int hh = nt * 16 + n;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
            *reinterpret_cast<f32x4*>(lds_acc + (wave * HG + hh) * AP + ct * 16 + g * 4) = acc[nt][ct];
        if (g == 0) *reinterpret_cast<float2*>(lds_ml + (wave * HG + hh) * 2) = make_float2(m[nt], l[nt]);
    }
    __syncthreads();

    // one thread per (head, four columns): the weights of a head are computed once per thread, and a wave's
    // lanes cover two whole rows, so the weight reads are broadcasts and the rows are read 16 bytes per lane
    constexpr int C4 = DV / 4;
    for (int idx = threadIdx.x; idx < nh * C4; idx += blockDim.x) {
        const int r = idx / C4, col = (idx % C4) * 4;
        float2 ml[MW];
#pragma unroll
        for (int w = 0; w < MW; ++w) ml[w] = *reinterpret_cast<const float2*>(lds_ml + (w * HG + r) * 2);
        float mm = ml[0].x;
#pragma unroll
        for (int w = 1; w < MW; ++w) mm = fmaxf(mm, ml[w].x);
        f32x4 num = {0.0f, 0.0f, 0.0f, 0.0f};
        float den = 0.0f;
#pragma unroll
        for (int w = 0; w < MW; ++w) {
            const float wt = fast_exp2(ml[w].x - mm);
            num += *reinterpret_cast<const f32x4*>(lds_acc + (w * HG + r) * AP + col) * wt;
            den += wt * ml[w].y;
        }
        const int h = h_base + r;
        if (direct) {
            const float inv = vs / den;
            ushort4 w16;
            w16.x = EL::from_f32(num[0] * inv);
            w16.y = EL::from_f32(num[1] * inv);
            w16.z = EL::from_f32(num[2] * inv);
            w16.w = EL::from_f32(num[3] * inv);
            *reinterpret_cast<ushort4*>(o16 + ((size_t)b * p.head_q + h) * DV + col) = w16;
        } else {
            const size_t part = part0 + (size_t)h * part_stride;
            *reinterpret_cast<f32x4*>(p.ws_o + part * DV + col) = num * vs;
            if (col == 0) {
                p.ws_ml[part * 2 + 0] = mm;
                p.ws_ml[part * 2 + 1] = den;
            }
        }
    }
}

// Grid, packed or paged K/V with a fixed split length: (split, KV heads x head groups, sequence).
// Grid, balanced form (p.flat_wgs > 0): (work-group i of W, KV heads x head groups, 1).  The tokens of all
// sequences form one line (positions p.flat_cu, in units of p.flat_unit tokens) whose length the kernel reads from
// p.flat_cu[batch]; work-group i takes positions [i T, (i+1) T) of it, T = flat_share() (the last one to the end),
// whatever sequences they belong to, one segment per sequence it touches.  Every work-group then streams the same number of bytes, which a ragged batch cut into fixed splits
// does not give.  Sequence b spans work-groups first(b) = cu[b] / T ... last(b) = (cu[b+1] - 1) / T (both capped
// at W - 1); its segment in work-group i is the partial in slot i + b (flat_slots), and goes straight to o when
// first(b) == last(b).
template <typename Tag, int D, int DV, int NT, bool PREFETCH, bool WH, int MINW, int KV8 = 0, int PGM = 0>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(MINW))) void gqa_mfma_kernel(const SweepParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    if (p.flat_wgs == 0) {
        int split = blockIdx.x, by = blockIdx.y, b = blockIdx.z;
        // Several head groups per KV head read the same K/V rows.  Work-groups go to the eight XCDs round-robin by
        // linear id, and each XCD has its own L2: renumber so that the groups of one (sequence, KV heads, split) are
        // neighbours on one XCD, and the rows leave HBM once for all of them.
        const int total = (int)(gridDim.x * gridDim.y * gridDim.z);
        if (p.groups > 1 && total % (8 * p.groups) == 0) {
            const int lin = (int)(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z));
            const int slot = lin >> 3;
            const int grp = slot % p.groups;
            int rest = (slot / p.groups) * 8 + (lin & 7);  // index over (split, KV heads, sequence)
            const int nky = (int)gridDim.y / p.groups;
            split = rest % (int)gridDim.x;
            rest /= (int)gridDim.x;
            by = (rest % nky) * p.groups + grp;
            b = rest / nky;
        }
        int start, len;
        seq_range(p, b, start, len);
        const int c0 = split * p.chunk;
        const int c1 = (split == p.nsplit - 1) ? len : min(len, c0 + p.chunk);
        gqa_segment<Tag, D, DV, NT, PREFETCH, WH, KV8, PGM>(p, smem, by, b, start, len, c0, c1,
                                                            (size_t)b * p.head_q * p.nsplit + split, p.nsplit, p.nsplit == 1);
        return;
    }
    const int W = (int)gridDim.x, i = (int)blockIdx.x, fby = (int)blockIdx.y, unit = p.flat_unit;
    const int32_t* const cu = p.flat_cu;
    const int total = cu[p.batch];
    const int T = flat_share(total, W, p.flat_step, p.flat_min);
    const int r0 = (int)min((long long)i * T, (long long)total);
    const int r1 = (i == W - 1) ? total : (int)min((long long)r0 + T, (long long)total);
    if (r0 >= r1) return;
    // the sequence that holds position r0: the last b with cu[b] <= r0 (empty sequences share their position with
    // the next one and are passed over).  A 64-way search: the wave's lanes probe 64 evenly spaced entries at once,
    // so 64 sequences take one round of loads where a binary search takes six dependent ones.
    int lo = 0;
    for (int n = p.batch; n > 1;) {  // invariant: cu[lo] <= r0, and the answer lies in [lo, lo + n)
        const int stride = (n + 63) >> 6;
        const int idx = lo + (int)(threadIdx.x & 63) * stride;
        const bool below = idx < lo + n && cu[idx] <= r0;
        // probes are sorted: the lanes that hold are a prefix, lane 0 among them
        const int k = __popcll(__ballot(below)) - 1;
        lo += k * stride;
        n = min(stride, n - k * stride);
    }
    for (int b = lo; b < p.batch; ++b) {
        const int s = cu[b], e = cu[b + 1];
        if (s >= r1) break;
        if (e <= s) continue;
        int start, len;
        seq_range(p, b, start, len);
        const int first = min(s / T, W - 1), last = min((e - 1) / T, W - 1);
        const int c0 = (max(r0, s) - s) * unit, c1 = min((min(r1, e) - s) * unit, len);
        gqa_segment<Tag, D, DV, NT, PREFETCH, WH, KV8, PGM>(p, smem, fby, b, start, len, c0, c1,
                                                            (size_t)(i + b) * p.head_q, 1, first == last);
        if (!WH) __syncthreads();  // the merge area of this segment is the V tile area of the next
    }
}

// wave_per_head selects the WH form; the grid's y extent must then count groups of four KV heads.
hipError_t launch_gqa_mfma(const SweepParams& p, bool is_bf16, int dim, int heads_per_group, bool wave_per_head,
                           dim3 grid, hipStream_t stream);
// the same with FP8 (e4m3) K and V; dim must be a multiple of 64
hipError_t launch_gqa_mfma_kv8(const SweepParams& p, bool is_bf16, int dim, int heads_per_group, bool wave_per_head,
                               dim3 grid, hipStream_t stream);
// the same with int8 K and V; dim must be a multiple of 64
hipError_t launch_gqa_mfma_i8(const SweepParams& p, bool is_bf16, int dim, int heads_per_group, bool wave_per_head,
                              dim3 grid, hipStream_t stream);
// ... and over an int4 one (two elements to a byte, see kKvInt4 in da_common.h)
hipError_t launch_gqa_mfma_i4(const SweepParams& p, bool is_bf16, int dim, int heads_per_group, bool wave_per_head,
                              dim3 grid, hipStream_t stream);
// ... and over an int4 one whose rows carry their own (scale, zero) pairs (SweepParams::k_tok, v_tok); dim 64, 128, 256
hipError_t launch_gqa_mfma_i4t(const SweepParams& p, bool is_bf16, int dim, int heads_per_group, bool wave_per_head,
                               dim3 grid, hipStream_t stream);
// ... and over an int4 one with a pair per run of 64 elements of each row ([rows, head_k, dim / 64, 2]); dim 128, 256
hipError_t launch_gqa_mfma_i4g(const SweepParams& p, bool is_bf16, int dim, int heads_per_group, bool wave_per_head,
                               dim3 grid, hipStream_t stream);
// ... and over an int8 one with a pair per run of 64 elements
hipError_t launch_gqa_mfma_i8g(const SweepParams& p, bool is_bf16, int dim, int heads_per_group, bool wave_per_head,
                               dim3 grid, hipStream_t stream);
// ... and over an int8 one with such pairs
hipError_t launch_gqa_mfma_i8t(const SweepParams& p, bool is_bf16, int dim, int heads_per_group, bool wave_per_head,
                               dim3 grid, hipStream_t stream);

}  // namespace da
