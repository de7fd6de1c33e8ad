// Software-pipelined MFMA sweep for 65..128 query heads over one latent KV head (key width 576, values = the
// first 512 key columns), 16-bit K.
//
// One work-group of four wavefronts serves one (sequence, 128 heads, sequence split); each wavefront owns 32
// heads: Q as MFMA B-operands in 144 registers, the un-normalised output O^T[512 x 32] in all 256 accumulation
// registers -- one wavefront per SIMD.  K tiles of 32 tokens stream HBM -> LDS with direct-to-LDS loads into four
// buffers (the tile layout of da_mla_dev.h); every tile is read from LDS twice, as K rows for
// S^T = K . Q^T and transposed for O^T += V^T . P^T.
//
// The matrix pipe is the resource to keep busy (2 x 68 matrix instructions of 32 clocks per tile and wavefront), and
// a wavefront's vector-ALU, LDS and load instructions issue beside its own matrix instructions when they do not
// depend on them.  So the tile loop is software-pipelined by one tile and written as one fixed instruction sequence:
//
//   trip t:   phase A   S(t+1) = K(t+1) . Q^T   36 matrix steps, between them the online softmax of S(t)
//                                               (subtract, exp2, sum, pack: two instructions per step) and the
//                                               nine direct-to-LDS loads of tile t+3
//             phase B   O += V(t)^T . P(t)^T    32 matrix steps
//
// Registers.  Q (v112 .. v255), the output tiles (a0 .. a255), the ring of LDS fragments (v80 .. v111) and the
// probability tile (v64 .. v79) are named
// in the instruction text and never seen by the compiler, whose own allocation is confined to v0 .. v63 (kernel
// attribute amdgpu_num_vgpr; the translation unit is built with VGPR-to-AGPR spilling switched off): with 400 of
// the 512 registers pinned down for the whole loop, a register allocator that may move them is the one thing the loop
// cannot afford.  What the compiler allocates: the score tile being accumulated, addresses and scalars.
//
// LDS fragments for the matrix steps run through a ring of eight register sets, requested eight steps ahead of
// their use across the A -> B boundary and, in the steady-state loop, across the trip boundary as well: the barrier
// that makes tile t+2 visible to every wave sits eight matrix steps before the end of trip t's phase B (each wave
// first waits for its own loads of that tile), and the last eight steps request the first K fragments of tile t+2,
// so the matrix pipe finds its operands waiting when trip t+1 starts.  A second, plain barrier at the top of a trip
// keeps the loads of tile t+3 behind every wave's last read of tile t-1, whose buffer they fill.  (A trip has 68
// steps, four more than a multiple of eight, so steady-state trips come in pairs with the ring slots offset by
// four in the second.)  The other trips (the first, the last ones of a split, ALiBi, paged rows) start with an empty
// ring behind one barrier, and the scaling and maximum of S(t+1) are computed while it refills.
//
// Mathematics as in the reference kernel (csrc/kernel/decoding_attn/decoding_fwd_kernel.h:50-235 with the latent
// aliasing of csrc/ops/decoding_attn.cpp:30-37); the structure is unrelated.
#include "da_mla.h"
#include "da_mla_dev.h"

#include <cstdlib>

namespace da {

namespace {

using namespace mla;

constexpr int kPipeBufs = 4;  // LDS tile buffers
constexpr int kRing = 8;      // LDS fragments requested ahead of the matrix step that uses them
constexpr int kDmaRaw = 200;  // phase A's DMA argument: the loads of a raw (8-bit) tile, one every eight steps
// byte offsets of a thread's conversion slot c: of the source in the stage (rows of 576 bytes), of the destination in
// its region (value rows of 1024 bytes, 16-byte columns 16 apart; key-tail rows of 128 bytes)
constexpr int conv_src_off(int c) { return (c / 5) * 16 * 576 + (c % 5) * 128; }
constexpr int conv_dst_off(int c) { return c % 5 < 4 ? (c / 5) * 16 * 1024 + (c % 5) * 256 : (c / 5) * 16 * 128; }
constexpr int kConvSlots = 10;  // 8-byte chunks of a raw tile per thread: two rows x (4 value chunks + the tail chunk)
// LDS operations of the 8-bit form's conversion issued in steps lo .. hi of phase A: a read behind steps 0, 3, ..., 27
// and `wr` writes behind steps 2, 5, ..., 29
constexpr int conv_ops_between(int lo, int hi, int wr) {
    int n = 0;
    for (int s = lo < 0 ? 0 : lo; s <= hi; ++s) {
        if (s % 3 == 0 && s / 3 < kConvSlots) ++n;
        if (s % 3 == 2 && s / 3 < kConvSlots) n += wr;
    }
    return n;
}

typedef short s16x8 __attribute__((__vector_size__(8 * sizeof(short))));

// Registers named in the instruction text (see the header comment).
constexpr int kScV = 64;    // the probability tile: v[64 .. 79]
constexpr int kRingV = 80;  // ring slot s: v[80 + 4 s .. 83 + 4 s]
constexpr int kQV = 112;    // Q fragment of k-step ks: v[112 + 4 ks .. 115 + 4 ks]

// ds_read_b128 into v[R .. R+3] from (base ^ X) + OFF; the XOR goes through `tmp`
template <int R, int X, int OFF>
__device__ __forceinline__ void ring_read_b128(uint32_t base, uint32_t& tmp) {
    if constexpr (X == 0) {
        asm volatile("ds_read_b128 v[%1:%2], %0 offset:%3" ::"v"(base), "n"(R), "n"(R + 3), "n"(OFF));
    } else {
        asm volatile("v_xor_b32 %0, %2, %1\n\tds_read_b128 v[%3:%4], %0 offset:%5"
                     : "=&v"(tmp)
                     : "v"(base), "n"(X), "n"(R), "n"(R + 3), "n"(OFF));
    }
}
// ds_read_b64_tr_b16 into v[R .. R+1]
template <int R, int OFF>
__device__ __forceinline__ void ring_read_tr16(uint32_t addr) {
    asm volatile("ds_read_b64_tr_b16 v[%1:%2], %0 offset:%3" ::"v"(addr), "n"(R), "n"(R + 1), "n"(OFF));
}
template <int N>
__device__ __forceinline__ void wait_lgkm_n() {
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N));
}
template <int X>
__device__ __forceinline__ void xor_const(uint32_t& dst, uint32_t base) {
    asm volatile("v_xor_b32 %0, %2, %1" : "=v"(dst) : "v"(base), "n"(X));
}
// Matrix instructions on the named registers.  S: acc (the compiler's) (+)= v[A..] . v[B..]; O: a[C..] += v[A..] . b
template <typename Tag, int A, int B, bool FIRST>
__device__ __forceinline__ void mma_s(f32x16& acc) {
    if constexpr (std::is_same<Tag, bf16_tag>::value) {
        if constexpr (FIRST)
            asm volatile("v_mfma_f32_32x32x16_bf16 %0, v[%1:%2], v[%3:%4], 0" : "=v"(acc) : "n"(A), "n"(A + 3), "n"(B), "n"(B + 3));
        else
            asm volatile("v_mfma_f32_32x32x16_bf16 %0, v[%1:%2], v[%3:%4], %0" : "+v"(acc) : "n"(A), "n"(A + 3), "n"(B), "n"(B + 3));
    } else {
        if constexpr (FIRST)
            asm volatile("v_mfma_f32_32x32x16_f16 %0, v[%1:%2], v[%3:%4], 0" : "=v"(acc) : "n"(A), "n"(A + 3), "n"(B), "n"(B + 3));
        else
            asm volatile("v_mfma_f32_32x32x16_f16 %0, v[%1:%2], v[%3:%4], %0" : "+v"(acc) : "n"(A), "n"(A + 3), "n"(B), "n"(B + 3));
    }
}
// a[N] *= alpha
template <int N>
__device__ __forceinline__ void scale_acc_n(float alpha) {
    float tmp;
    asm volatile("v_accvgpr_read_b32 %0, a[%2]\n\tv_mul_f32 %0, %0, %1\n\ts_nop 0\n\tv_accvgpr_write_b32 a[%2], %0"
                 : "=&v"(tmp)
                 : "v"(alpha), "n"(N));
}
template <int N>
__device__ __forceinline__ float read_acc_n() {
    float x;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(N));
    return x;
}
template <typename Tag, int A, int B, int C>
__device__ __forceinline__ void mma_o() {
    if constexpr (std::is_same<Tag, bf16_tag>::value)
        asm volatile("v_mfma_f32_32x32x16_bf16 a[%0:%1], v[%2:%3], v[%4:%5], a[%0:%1]" ::"n"(C), "n"(C + 15), "n"(A), "n"(A + 3), "n"(B), "n"(B + 3));
    else
        asm volatile("v_mfma_f32_32x32x16_f16 a[%0:%1], v[%2:%3], v[%4:%5], a[%0:%1]" ::"n"(C), "n"(C + 15), "n"(A), "n"(A + 3), "n"(B), "n"(B + 3));
}
// The probability tile: v[kScV + r], r = 0 .. 15, holds score r of the tile minus the running maximum, then the
// probability, then (r < 8) the probabilities of the pair (2 r, 2 r + 1) packed as one register of two B-operands.
// Single vector-ALU instructions on it, each with a fixed place in the instruction sequence:
template <int I>
__device__ __forceinline__ void sc_set(float x) { asm volatile("v_mov_b32 v[%1], %0" ::"v"(x), "n"(kScV + I)); }
// v[I] = s * scale + negm
template <int I>
__device__ __forceinline__ void sc_fma(float s, float scale, float negm) {
    asm volatile("v_fma_f32 v[%3], %0, %1, %2" ::"v"(s), "v"(scale), "v"(negm), "n"(kScV + I));
}
template <int I>
__device__ __forceinline__ void sc_exp2() { asm volatile("v_exp_f32 v[%0], v[%0]" ::"n"(kScV + I)); }
template <int I>
__device__ __forceinline__ void sc_acc(float& l) { asm volatile("v_add_f32 %0, %0, v[%1]" : "+v"(l) : "n"(kScV + I)); }
__device__ __forceinline__ void v_add(float& x, float y) { asm volatile("v_add_f32 %0, %0, %1" : "+v"(x) : "v"(y)); }
// x += s, s wave-uniform
__device__ __forceinline__ void v_add_s(uint32_t& x, uint32_t s) { asm volatile("v_add_u32 %0, %1, %0" : "+v"(x) : "s"(s)); }
// v[K] = the pair (v[2K], v[2K+1]) rounded to two 16-bit values (round to nearest even).  In place: register K held
// element K, which pair K/2 <= K has consumed by now.  (bf16, s_nop: a result of the transcendental unit needs one
// wait state before an ordinary vector instruction reads it, and there this directly follows the exp2 of v[2K+1].)
template <typename Tag, int K>
__device__ __forceinline__ void sc_pack() {
    if constexpr (std::is_same<Tag, bf16_tag>::value)
        asm volatile("s_nop 0\n\tv_cvt_pk_bf16_f32 v[%0], v[%1], v[%2]" ::"n"(kScV + K), "n"(kScV + 2 * K), "n"(kScV + 2 * K + 1));
    else
        asm volatile("v_cvt_pk_f16_f32 v[%0], v[%1], v[%2]" ::"n"(kScV + K), "n"(kScV + 2 * K), "n"(kScV + 2 * K + 1));
}
// the two 16-bit halves of register K as fp32 values (bf16: the value itself)
template <int K>
__device__ __forceinline__ void sc_bf16_lo(float& dst) { asm volatile("v_lshlrev_b32 %0, 16, v[%1]" : "=v"(dst) : "n"(kScV + K)); }
template <int K>
__device__ __forceinline__ void sc_bf16_hi(float& dst) { asm volatile("v_and_b32 %0, 0xffff0000, v[%1]" : "=v"(dst) : "n"(kScV + K)); }

// PG: paged K/V with pages of fewer than 16 tokens (down to 1): every row of a tile has its own page lookup.
// KV8: K holds 8-bit elements (kKvFp8 or kKvInt8) in rows of 576 bytes (one KV head).  A tile's bytes then stream into
// one of three raw stages (18 KiB, row after row), and the work-group converts a staged tile into the 16-bit tile
// layout two tiles ahead of its use: in the steady-state loop between the matrix steps of phase A (thread (row, j)
// reads the row's 8-byte chunks j, j + 8, ..., converts each to eight 16-bit values -- exactly -- and writes them to
// their swizzled place), in the other trips in one go behind the trip's barrier.  Everything downstream of the 16-bit
// tile is the same instruction sequence, so with unit scales the output equals the 16-bit call's on the widened
// values bit for bit.  LDS: three value regions (the 512 value columns of a tile: one being written, one read as K,
// one read as V), two regions for the remaining 64 key columns (needed only while a tile is written or read as K)
// and the three stages, 158 KiB.
template <typename Tag, bool PG, int KV8 = 0>
__global__ __launch_bounds__(256) __attribute__((amdgpu_num_vgpr(kScV))) void latent_pipe_kernel(const SweepParams p) {
    // the register file as this kernel uses it: v0 .. v255 and a0 .. a255 (the compiler itself stays below v64)
    asm volatile("" ::: "v255", "a255");
    using EL = Elem<Tag>;
    constexpr bool kBf16 = std::is_same<Tag, bf16_tag>::value;
    constexpr int D = 576, DV = 512, NWV = 4;
    constexpr int ROW_A = DV * 2;           // bytes per row, region A (value columns)
    constexpr int ROW_B = (D - DV) * 2;     // bytes per row, region B (remaining key columns)
    constexpr int OFF_B = kTile * ROW_A;    // region B starts here
    constexpr int BUF = kTile * D * 2;      // bytes per tile buffer
    constexpr int NLA = kTile / NWV;        // region-A load instructions per tile per wave (one row each)
    constexpr int NLB = (kTile / 8) / NWV;  // region-B load instructions per tile per wave (eight rows each)
    constexpr int NLW = NLA + NLB;          // load instructions per tile per wave
    constexpr int KS = D / 16;              // k-steps of Q K^T
    constexpr int CT = DV / 32;             // 32-column tiles of the output
    constexpr int NV = CT * 2;              // matrix steps of O += V^T P^T
    constexpr int NB = kPipeBufs;
    static_assert(NLB == 1 && KS == 36 && NV == 32, "schedule below is written for (576, 512), four waves");
    static_assert(!(KV8 && PG), "the 8-bit form takes whole runs of 16 tokens");
    // 8-bit K: region A (value columns) of tile i lives at (i % 3) * ABUF, its region B at OFF_BB + (i % 2) * BBUF,
    // its raw bytes in stage i % 3
    constexpr int KB = KV8 ? 1 : 2;           // bytes per K element in memory
    constexpr int ABUF = kTile * ROW_A;       // 32 KiB
    constexpr int BBUF = kTile * ROW_B;       // 4 KiB
    constexpr int OFF_BB = 3 * ABUF;
    constexpr int OFF_STG = OFF_BB + 2 * BBUF;
    constexpr int STG = kTile * D;            // bytes of a raw tile
    constexpr int NLW8 = 5;                   // load instructions per raw tile per wave: four of 1 KiB, one of 512 bytes
    static_assert(STG == 16 * 1024 + 4 * 512 && (16 * D) % 1024 == 0, "raw tile: 16 whole loads + four half loads; a run of 16 rows ends on a load boundary");

#ifdef DA_PIPE_PROBE
    const long long pr_wk = wall_clock64();
#endif
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];  // NB * BUF bytes
    const uint32_t smem_off = (uint32_t)(uintptr_t)smem;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int half = lane >> 5;
    const int n = lane & 31;

    // Work-groups are handed to the eight XCDs round-robin by linear id, and each XCD has its own L2.  Renumber
    // so that the sequence splits of one (sequence, head group) run on one XCD: they read the same Q block, which
    // then leaves HBM once instead of once per split.
    int split = blockIdx.x, by = blockIdx.y, b = blockIdx.z;
    {
        const int outer_n = gridDim.y * gridDim.z;
        if (gridDim.x > 1 && outer_n % 8 == 0) {
            const int lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
            const int slot = lin >> 3;
            split = slot % (int)gridDim.x;
            const int outer = (slot / (int)gridDim.x) * 8 + (lin & 7);
            by = outer % (int)gridDim.y;
            b = outer / (int)gridDim.y;
        }
    }
    const int hk = by / p.groups;
    const int grp = by % p.groups;

    int start, len;
    seq_range(p, b, start, len);
    const int c0 = split * p.chunk;
    const int c1 = (split == p.nsplit - 1) ? len : min(len, c0 + p.chunk);

    const int wg_heads = min(32 * NWV, p.ratio - grp * 32 * NWV);  // live heads of this work-group
    const int nh = max(0, min(32, wg_heads - wave * 32));          // live heads of this wave
    const int h_base = hk * p.ratio + grp * 32 * NWV + wave * 32;
    uint16_t* const o16 = reinterpret_cast<uint16_t*>(p.o);

    if (c0 >= c1) {
        if (p.nsplit == 1) zero_rows<DV>(p, b, hk * p.ratio + grp * 32 * NWV, wg_heads, 1, 0);
        return;
    }

    const int q_last = max(nh, 1) - 1;
    const uint32_t lane16 = lane * 16;
    const int rb = lane >> 3;  // region B: row within the group of eight, chunk lane & 7
    const int hq = min(h_base + min(n, q_last), p.head_q - 1);
    const float slope = p.is_alibi ? alibi_slope_log2(p.slopes, hq, p.head_q) : 0.0f;

    float m = kNegBig, l = 0.0f;

    const uint8_t* const kbytes = reinterpret_cast<const uint8_t*>(p.k) + (size_t)hk * D * KB;
    const size_t k_row_bytes = (size_t)p.k_row * KB;
    // score scale, log2 units (8-bit K: times the KV head's de-quantisation factor)
    const float sl = KV8 ? p.scale_log2 * head_scale(p.k_scale, hk) : p.scale_log2;

    // One direct-to-LDS load of a tile: region-A row wave + 4 q for q < NLA, then the wave's eight region-B rows.
    // `base` / `base1`: addresses of the rows of the tile's tokens 0 and 16 (a tile is fetched as two runs of 16
    // tokens, each inside one page; for the packed layout and larger pages the second run follows the first); `last`:
    // last valid token of the tile, rows past it re-read that row (they are masked later).
    auto issue_load = [&](auto qc, const uint8_t* base, const uint8_t* base1, int last, int buf) {
        constexpr int q = decltype(qc)::value;
        if constexpr (q < NLA) {
            const int row = wave + NWV * q;  // wave-uniform
            const int rc = min(row, last), run = rc >> 4;
            // lane offset (row part in a scalar register) computed at the load, not kept in a register per q
            uint32_t off;
            asm volatile("v_xor_b32 %0, %1, %2\n\tv_add_u32 %0, %3, %0"
                         : "=&v"(off)
                         : "s"((uint32_t)(swz_a(row) * 16)), "v"(lane16), "s"((uint32_t)(rc - run * 16) * (uint32_t)k_row_bytes));
            lds_dma16<true>(run ? base1 : base, off, smem_off + (uint32_t)(buf * BUF + row * ROW_A));
        } else {
            const int j = wave;
            const int row = j * 8 + rb;
            const int run = min(j >> 1, last >> 4);  // the eight rows of a load lie in one run, clamped or not
            lds_dma16<true>(run ? base1 : base, (uint32_t)(min(row, last) - run * 16) * (uint32_t)k_row_bytes +
                                              (uint32_t)(DV * 2 + (((lane & 7) ^ swz_b(row)) * 16)),
                      smem_off + (uint32_t)(buf * BUF + OFF_B + j * 1024));
        }
    };
    // rows of tokens tok and tok + 16 of the sequence (the second only looked up when the tile has it: the block
    // table ends with the sequence's last page)
    struct TileRows {
        const uint8_t* base;
        const uint8_t* base1;
        int last;
    };
    auto tile_rows = [&](int tok0) {
        const int64_t r0 = row_ref(p, b, start, tok0).k;
        const int64_t r1 = tok0 + 16 < c1 ? row_ref(p, b, start, tok0 + 16).k : r0;
        return TileRows{kbytes + r0 * KB, kbytes + r1 * KB, c1 - 1 - tok0};
    };
    // ---- 8-bit K: raw tiles and their conversion --------------------------------------------------------------------
    // A raw tile is the tile's 32 x 576 bytes row after row (rows are 576 bytes apart in memory, so a run of 16 tokens
    // is 9 KiB of contiguous memory).  Every wave issues five loads per tile: 1 KiB pieces wave, wave + 4, wave + 8,
    // wave + 12 and the 512-byte piece 16 KiB + 512 wave (lanes 0 .. 31).  base / base1: rows of tokens 0 and 16.
    auto issue_raw_whole = [&](const uint8_t* base, const uint8_t* base1, uint32_t lds0) __attribute__((always_inline)) {
        static_for<0, 4>([&](auto qc) {
            const int j = wave + 4 * decltype(qc)::value;  // wave-uniform
            const uint8_t* const src = (j >= 9 ? base1 - 9 * 1024 : base) + j * 1024;
            lds_dma16<true>(src, lane16, lds0 + (uint32_t)(j * 1024));
        });
        if (lane < 32) lds_dma16<true>(base1 + (7 * 1024 + 512 * wave), lane16, lds0 + (uint32_t)(16 * 1024 + 512 * wave));
    };
    // piece q = 0 .. 4 of a whole raw tile (as issue_raw_whole), one at a time between matrix steps
    auto issue_raw_piece = [&](auto qc, const uint8_t* base, const uint8_t* base1, uint32_t lds0) __attribute__((always_inline)) {
        constexpr int q = decltype(qc)::value;
        if constexpr (q < 4) {
            const int j = wave + 4 * q;  // wave-uniform
            lds_dma16<true>((j >= 9 ? base1 - 9 * 1024 : base) + j * 1024, lane16, lds0 + (uint32_t)(j * 1024));
        } else {
            if (lane < 32) lds_dma16<true>(base1 + (7 * 1024 + 512 * wave), lane16, lds0 + (uint32_t)(16 * 1024 + 512 * wave));
        }
    };
    auto issue_raw = [&](int tok0, int stg) {
        const TileRows tr = tile_rows(tok0);
        const uint32_t lds0 = smem_off + (uint32_t)(OFF_STG + stg * STG);
        if (tr.last >= kTile - 1) {
            issue_raw_whole(tr.base, tr.base1, lds0);
            return;
        }
        // the split's last tile: rows past the end re-read the last row (they are masked later), per-lane addresses
        // (the lane's offset passes through an opaque statement: the row arithmetic is then worked out at each call
        // instead of once in the prologue and kept in registers across the loop)
        uint32_t l16 = lane16;
        asm volatile("" : "+v"(l16));
        auto piece = [&](uint32_t at) {
            const uint32_t sb = at + l16, row = sb / (uint32_t)D, within = sb - row * (uint32_t)D;
            const int rc = min((int)row, tr.last), run = rc >> 4;
            lds_dma16_v<true>((run ? tr.base1 : tr.base) + (size_t)(rc - 16 * run) * k_row_bytes + within, lds0 + at);
        };
        static_for<0, 4>([&](auto qc) { piece((uint32_t)((wave + 4 * decltype(qc)::value) * 1024)); });
        if (lane < 32) piece((uint32_t)(16 * 1024 + 512 * wave));
    };
    // Conversion of a staged tile into value region a_off and key-tail region b_off (byte offsets in LDS).  Thread
    // (row r = tid / 16, j = tid % 16) converts, for the rows r and r + 16, the 8-element chunks j, j + 16, j + 32, j + 48
    // of the value columns and, for j < 8, chunk 64 + j (the remaining key columns): ten slots, the last of each row with
    // half the lanes.  Sixteen lanes of a row write sixteen different 16-byte columns (the swizzle permutes them among
    // themselves), so the writes are free of bank conflicts, and since the swizzles of rows r and r + 16 are equal every
    // slot is a constant offset from one source and two destination addresses.
    // (the thread's three addresses are worked out from its index where they are needed, a dozen instructions, rather
    // than kept in registers across the loop: the compiler's 64 registers do not have the room)
    struct ConvAddr {
        uint32_t src, dst_a, dst_b;
    };
    auto conv_addr = [&](uint32_t stg_off, uint32_t a_off, uint32_t b_off) __attribute__((always_inline)) {
        uint32_t tid = threadIdx.x;
        asm volatile("" : "+v"(tid));  // (not to be hoisted out of the loop)
        const int cv_j = (int)tid & 15, cv_r = (int)tid >> 4;
        ConvAddr ca;
        ca.src = smem_off + (uint32_t)(OFF_STG + cv_r * D + cv_j * 8) + stg_off;
        ca.dst_a = smem_off + (uint32_t)(cv_r * ROW_A + ((cv_j ^ swz_a(cv_r)) * 16)) + a_off;
        ca.dst_b = smem_off + (uint32_t)(OFF_BB + cv_r * ROW_B + (((cv_j & 7) ^ swz_b(cv_r)) * 16)) + b_off;
        return ca;
    };
    // slot c = 0 .. 9 of a thread: rows r + 16 (c / 5); c % 5 < 4: value chunk j + 16 (c % 5), else the tail chunk
    // (byte offsets of the source in the stage, of the destination in its region)
    static_assert(D == 576 && ROW_A == 1024 && ROW_B == 128, "conv_src_off / conv_dst_off");
    auto convert_burst = [&](int stg, uint32_t a_off, uint32_t b_off) {
        typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        typedef const __attribute__((address_space(3))) u32x2* lds_src;
        typedef __attribute__((address_space(3))) u32x4* lds_dst;
        const ConvAddr ca = conv_addr((uint32_t)(stg * STG), a_off, b_off);
        const bool tail_lane = (threadIdx.x & 15) < 8;
#pragma unroll
        for (int c = 0; c < kConvSlots; ++c) {
            if (c % 5 == 4 && !tail_lane) continue;
            const u32x2 rv = *reinterpret_cast<lds_src>((uintptr_t)(ca.src + conv_src_off(c)));
            // (this lambda is compiled, and never called, for 16-bit K as well)
            const uint4 cv = kv8x8_to_16<Tag, KV8 ? KV8 : kKvFp8>(make_uint2(rv.x, rv.y));
            const uint32_t dst = (c % 5 < 4 ? ca.dst_a : ca.dst_b) + conv_dst_off(c);
            *reinterpret_cast<lds_dst>((uintptr_t)dst) = u32x4{cv.x, cv.y, cv.z, cv.w};
        }
    };
    auto issue_tile = [&](int tok0, int buf) {
        const TileRows tr = tile_rows(tok0);
        static_for<0, NLW>([&](auto qc) { issue_load(qc, tr.base, tr.base1, tr.last, buf); });
    };

    // PG: the wave's kTile / NWV rows are consecutive here (rows wave * NLA + q), the same rows for both regions, so
    // one set of page lookups (scalar loads) serves both; the second region's load covers eight rows, so its lanes
    // pick their row's address out of the set.
    auto issue_tile_pg = [&](int tok0, int buf) {
        const int last = c1 - 1 - tok0;
        const int mask = (1 << p.page_shift) - 1;
        int64_t rowoff[NLA];  // byte offsets of the wave's rows
#pragma unroll
        for (int q = 0; q < NLA; ++q) {
            const int tok = tok0 + min(wave * NLA + q, last);
            rowoff[q] = ((int64_t)page_of(p, b, tok) * p.k_page + (int64_t)(tok & mask) * p.k_row) * 2;
        }
#pragma unroll
        for (int q = 0; q < NLA; ++q) {
            const int row = wave * NLA + q;
            lds_dma16<true>(kbytes + rowoff[q], lane16 ^ (uint32_t)(swz_a(row) * 16),
                      smem_off + (uint32_t)(buf * BUF + row * ROW_A));
        }
        {
            const int j = wave;
            const int row = j * 8 + rb;
            int64_t mine = rowoff[0];
#pragma unroll
            for (int i = 1; i < 8; ++i) mine = rb == i ? rowoff[i] : mine;
            lds_dma16_v<true>(kbytes + mine + (DV * 2 + (((lane & 7) ^ swz_b(row)) * 16)),
                        smem_off + (uint32_t)(buf * BUF + OFF_B + j * 1024));
        }
    };

    const int ntiles = (c1 - c0 + kTile - 1) / kTile;
    auto issue_any = [&](int i) {
        if constexpr (PG)
            issue_tile_pg(c0 + i * kTile, i);
        else
            issue_tile(c0 + i * kTile, i);
    };
    // Tile 0 goes out behind the first round of Q (buffer 0), tile 1 behind the second, tile 2 when Q is through, tile
    // t + 3 in trip t: the first trip needs Q and tile 0 only, and every work-group of the grid asks for them at the
    // same moment, so nothing else competes with them.  Loads complete in order, so a round's wait leaves the tile
    // issued behind its Q blocks outstanding: the tile arrives while the blocks are read into registers.

    // Q rows of this wave's heads as B-operands: lane (n, half) holds Q[head n][ks*16 + half*8 .. +8).  The wave's
    // 32 x 576 block of Q is staged like a K tile (whole-row direct-to-LDS loads, same swizzle) and read back with
    // the K-row read pattern, which is the same operand layout.  Q passes through buffers 2 and 3, two blocks at a
    // time, so that the first K tiles can be on their way meanwhile (all four blocks at once would need the whole
    // LDS).
    // this wave's share (region-A rows wave + 4 q, region-B rows 8 wave .. 8 wave + 7) of the Q block of wave `blk`
    // (its 32 heads), into tile buffer 2 + blk % 2: the four waves fetch a block together, as they fetch a K tile,
    // because a direct-to-LDS load holds its wave for ~100 clocks (36 of them in a row would be the prologue's longest
    // stretch)
    auto issue_q_share = [&](int blk) {
        const uint8_t* const qb = reinterpret_cast<const uint8_t*>(p.q) + (size_t)b * p.head_q * (D * 2);
        const int first = hk * p.ratio + grp * 32 * NWV + blk * 32;  // first head of the block
        const int last_row = max(min(32, wg_heads - blk * 32), 1) - 1;  // rows past the block's live heads repeat one
        // (8-bit K: through value regions 0 and 1 and the two key-tail regions, while the first raw tiles land in
        // the stages)
        const uint32_t qbuf_a = smem_off + (uint32_t)(KV8 ? (blk & 1) * ABUF : (2 + (blk & 1)) * BUF);
        const uint32_t qbuf_b = smem_off + (uint32_t)(KV8 ? OFF_BB + (blk & 1) * BBUF : (2 + (blk & 1)) * BUF + OFF_B);
#pragma unroll
        for (int q = 0; q < NLA; ++q) {
            const int row = wave + NWV * q;  // wave-uniform
            const int head = min(first + min(row, last_row), p.head_q - 1);
            lds_dma16(qb, (uint32_t)head * (uint32_t)(D * 2) + (lane16 ^ (uint32_t)(swz_a(row) * 16)),
                      qbuf_a + (uint32_t)(row * ROW_A));
        }
        {
            const int row = wave * 8 + rb;
            const int head = min(first + min(row, last_row), p.head_q - 1);
            lds_dma16(qb, (uint32_t)head * (uint32_t)(D * 2) + (uint32_t)(DV * 2 + (((lane & 7) ^ swz_b(row)) * 16)),
                      qbuf_b + (uint32_t)(wave * 1024));
        }
    };
    auto read_q = [&]() {
        const uint32_t qbuf_a = smem_off + (uint32_t)(KV8 ? (wave & 1) * ABUF : (2 + (wave & 1)) * BUF);
        const uint32_t qbuf_b = smem_off + (uint32_t)(KV8 ? OFF_BB + (wave & 1) * BBUF : (2 + (wave & 1)) * BUF + OFF_B);
        const uint32_t qa = qbuf_a + n * ROW_A + ((swz_a(n) ^ half) * 16);
        const uint32_t qbb = qbuf_b + n * ROW_B + ((swz_b(n) ^ half) * 16);
        static_for<0, KS>([&](auto ic) {
            constexpr int ks = decltype(ic)::value;
            uint32_t tmp;
            if constexpr (ks < 32)
                ring_read_b128<kQV + 4 * ks, 32 * (ks & 7), (ks >> 3) * 256>(qa, tmp);
            else
                ring_read_b128<kQV + 4 * ks, 32 * (ks - 32), 0>(qbb, tmp);
            if constexpr (ks % 12 == 11) wait_lgkm_n<0>();  // the counter of outstanding reads is 4 bits wide
        });
    };
    issue_q_share(0);
    issue_q_share(1);
    if constexpr (KV8) {
        // the first three raw tiles go out behind the first round of Q (the stages are free from the start)
        issue_raw(c0, 0);
        if (1 < ntiles) issue_raw(c0 + kTile, 1);
        if (2 < ntiles) issue_raw(c0 + 2 * kTile, 2);
    } else {
        issue_any(0);  // (c0 < c1: there is a tile 0)
    }
    // The output tiles start at zero: 512 register writes, 2048 clocks of a wave alone on its SIMD.  Half of them while
    // the first loads are on their way (all of them would outlast the loads), the other half while the other pair of
    // waves reads its Q blocks.
    auto zero_acc = [&](auto from_c, auto to_c) __attribute__((always_inline)) {
        static_for<decltype(from_c)::value, decltype(to_c)::value>(
            [&](auto ic) { asm volatile("v_accvgpr_write_b32 a[%0], 0" ::"n"(decltype(ic)::value)); });
    };
    constexpr std::integral_constant<int, 0> acc_lo{};
    constexpr std::integral_constant<int, CT * 8> acc_mid{};
    constexpr std::integral_constant<int, CT * 16> acc_hi{};
    zero_acc(acc_lo, acc_mid);
    if constexpr (KV8) {
        // (all but the raw tiles')
        if (2 < ntiles)
            wait_vmcnt<3 * NLW8>();
        else if (1 < ntiles)
            wait_vmcnt<2 * NLW8>();
        else
            wait_vmcnt<NLW8>();
    } else {
        wait_vmcnt<NLW>();  // (all but tile 0's)
    }
    __syncthreads();    // the Q blocks of waves 0 and 1 are in LDS
    if ((wave >> 1) == 0)
        read_q();
    else
        zero_acc(acc_mid, acc_hi);
    __syncthreads();  // ... and in registers: their buffers take the blocks of waves 2 and 3
    issue_q_share(2);
    issue_q_share(3);
    if constexpr (KV8) {
        wait_vmcnt<0>();  // (the raw tiles, issued before, have landed too)
    } else if (1 < ntiles) {
        issue_any(1);
        wait_vmcnt<NLW>();  // (loads complete in order: tile 1's may stay outstanding)
    } else {
        wait_vmcnt<0>();
    }
    __syncthreads();
    if ((wave >> 1) == 1)
        read_q();
    else
        zero_acc(acc_mid, acc_hi);
    __syncthreads();  // the Q buffers are free for K
    if constexpr (KV8) {
        // tile 0 into its 16-bit form (tile 1 follows between the matrix steps of S(0) below); then its stage takes raw
        // tile 3
        convert_burst(0, 0, 0);
        __syncthreads();
        if (3 < ntiles) issue_raw(c0 + 3 * kTile, 0);
    } else {
        if (2 < ntiles) issue_any(2);
    }

    // The fast form of a tile's loads, for whole tiles (no row past the end) between the matrix steps of phase A: the
    // row part of the address is added to the tile's base in scalar registers, the lane part is one XOR.
    // rowoff[j] = (wave + 4 j) * pitch, j < 4: region-A rows of the first run; those of the second run (q >= 4) lie
    // the same distances behind the second run's base.
    uint32_t rowoff[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) rowoff[j] = (uint32_t)(wave + NWV * j) * (uint32_t)k_row_bytes;
    // region B: the wave's eight rows 8 wave .. 8 wave + 7 lie in run wave / 2; lane part (row within the eight,
    // swizzled chunk) kept in a register
    const uint32_t voff_b = (uint32_t)(((wave & 1) * 8 + rb) * (int)k_row_bytes) +
                            (uint32_t)(DV * 2 + (((lane & 7) ^ swz_b(wave * 8 + rb)) * 16));
    const uint32_t lane16w = lane16 ^ (uint32_t)(wave << 6);  // lane16 ^ 16 * (swizzle bits from row & 3 = wave)
    auto issue_load_fast = [&](auto qc, const uint8_t* base, const uint8_t* base1, uint32_t lds_buf) __attribute__((always_inline)) {
        constexpr int q = decltype(qc)::value;
        if constexpr (q < NLA) {
            // row = wave + 4 q: swizzle = wave << 2 | (q & 3)
            uint32_t off;
            if constexpr ((q & 3) == 0)
                off = lane16w;
            else
                asm volatile("v_xor_b32 %0, %1, %2" : "=v"(off) : "n"((q & 3) * 16), "v"(lane16w));
            lds_dma16<true>((q < 4 ? base : base1) + rowoff[q & 3], off,
                      lds_buf + (uint32_t)(q * NWV * ROW_A) + (uint32_t)(wave * ROW_A));
        } else {
            lds_dma16<true>((wave >> 1) ? base1 : base, voff_b, lds_buf + (uint32_t)OFF_B + (uint32_t)(wave * 1024));
        }
    };

    // Per-lane LDS read bases (buffer 0); per-step chunk offsets are XORed in, the rest is instruction offset.
    // K rows: lane (n, half) reads chunk 2 ks + half of row n.
    //   ks < 32: (base_a ^ 32 (ks & 7)) + 256 (ks >> 3)        ks >= 32: base_b ^ 32 (ks - 32)
    const uint32_t base_a = smem_off + n * ROW_A + ((swz_a(n) ^ half) * 16);
    const uint32_t base_b = smem_off + (KV8 ? OFF_BB : OFF_B) + n * ROW_B + ((swz_b(n) ^ half) * 16);
    // LDS offsets of tile i's value region (added to base_a / base_v) and of its key-tail region (added to base_b)
    auto a_of = [](int i) { return KV8 ? (uint32_t)((i % 3) * ABUF) : (uint32_t)((i & (NB - 1)) * BUF); };
    auto b_of = [](int i) { return KV8 ? (uint32_t)((i & 1) * BBUF) : (uint32_t)((i & (NB - 1)) * BUF); };
    // V^T: as a source lane of the transpose read this lane addresses row half*4 + q (+16 s2, +8 for the second
    // read), 8 bytes at chunk 4 c + 2 b1 + b0 of it, q = (lane & 15) >> 2, b1 = lane bit 4, b0 = lane bit 1:
    //   (base_v ^ (64 c | 32 hi)) + 16 KiB s2 + 8 KiB hi
    const uint32_t base_v = smem_off + (half * 4 + ((lane & 15) >> 2)) * ROW_A + 64 * ((lane & 15) >> 2) +
                            16 * ((2 * ((lane >> 4) & 1) + ((lane >> 1) & 1)) ^ half) + 8 * (lane & 1);


    const float bias0 = slope * (float)(half * 4 - (len - 1));  // ALiBi: slope * (token - (len - 1)), split in lane and tile parts

    // ---- the fragment ring -------------------------------------------------------------------------------------
    // Matrix steps of a trip in order: g = 0 .. 35 the k-steps of S = K Q^T (one ds_read_b128 each), g = 36 .. 67 the
    // steps of O += V^T P^T (two transpose reads each).  The reads of step g + kRing are issued behind the matrix
    // instruction of step g; ring slot g % kRing.
    // Addresses of the K reads of the tile being multiplied (region A: one register per k-step % 8, moved from buffer
    // to buffer once a trip; region B: XOR in front of the read)
    constexpr int NKA = (PG || KV8) ? 1 : 8;  // (the 8-bit form needs the registers for its conversion)
    uint32_t ka[NKA];
    uint32_t xa = 0, xb = 0;  // V^T read addresses of the current column tile
    uint32_t xt = 0;          // scratch for K read addresses
    f32x16 sacc;              // S(t+1), being accumulated
    float mxr = 0.0f;         // maximum of the raw scores of the tile in sacc (over the tile's tokens, this lane's head)

    // read for k-step ks of the K tile whose region-B base is tb (region A: ka[]; the PG form, short of registers for
    // its row addresses, keeps one base, ka[0], and XORs in front of every read)
    // RO: where the trip's first step sits in the ring.  A trip has 68 steps, four more than a multiple of the ring's
    // eight slots, so when the ring runs on from one trip into the next (steady-state loop) trips alternate between
    // RO = 0 and RO = 4; a trip that starts with an empty ring starts at 0.
    auto read_k = [&](auto ksc, uint32_t tb, auto ro_c) __attribute__((always_inline)) {
        constexpr int ks = decltype(ksc)::value;
        constexpr int slot = (ks + decltype(ro_c)::value) % kRing;
        if constexpr (ks < 32 && NKA == 1)
            ring_read_b128<kRingV + 4 * slot, 32 * (ks & 7), (ks >> 3) * 256>(ka[0], xt);
        else if constexpr (ks < 32)
            ring_read_b128<kRingV + 4 * slot, 0, (ks >> 3) * 256>(ka[ks & 7], xt);
        else
            ring_read_b128<kRingV + 4 * slot, 32 * (ks - 32), 0>(tb, xt);
    };
    // reads for step i of O += V^T P^T (column tile i / 2, token half i % 2) of the tile at tv; ring slot (KS + i) % kRing
    auto read_v = [&](auto ic, uint32_t tv, auto ro_c) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        constexpr int c = i >> 1, s2 = i & 1, slot = (KS + i + decltype(ro_c)::value) % kRing;
        if constexpr (s2 == 0) {
            if constexpr (c == 0)
                asm volatile("v_mov_b32 %0, %1" : "=v"(xa) : "v"(tv));
            else
                xor_const<64 * c>(xa, tv);
            xor_const<64 * c + 32>(xb, tv);
        }
        ring_read_tr16<kRingV + 4 * slot, s2 * 16 * ROW_A>(xa);
        ring_read_tr16<kRingV + 4 * slot + 2, s2 * 16 * ROW_A + 8 * ROW_A>(xb);
    };

    // softmax of S(t), the part that runs between matrix steps.  sc holds the scores minus the running maximum; for
    // each register pair (2 k, 2 k + 1): exponentiate, add to the denominator, pack.  fp16: 5 instructions a pair,
    // bf16: 7 (the denominator is summed from the rounded values, see as_second_operand in da_common.h).
    constexpr int SMP = kBf16 ? 7 : 5;  // instructions per pair
    constexpr int SMN = 8 * SMP;        // in all
    float tlo, thi;
    auto sm_op = [&](auto jc) __attribute__((always_inline)) {
        constexpr int j = decltype(jc)::value;
        constexpr int k = j / SMP, o = j % SMP;
        if constexpr (o == 0) sc_exp2<2 * k>();
        if constexpr (o == 1) sc_exp2<2 * k + 1>();
        if constexpr (!kBf16) {
            if constexpr (o == 2) sc_acc<2 * k>(l);
            if constexpr (o == 3) sc_acc<2 * k + 1>(l);
            if constexpr (o == 4) sc_pack<Tag, k>();
        } else {
            if constexpr (o == 2) sc_pack<Tag, k>();
            if constexpr (o == 3) sc_bf16_lo<k>(tlo);
            if constexpr (o == 4) sc_bf16_hi<k>(thi);
            if constexpr (o == 5) v_add(l, tlo);
            if constexpr (o == 6) v_add(l, thi);
        }
    };
    // maximum of the raw scores in sacc, between the matrix steps of phase B (its first instruction well behind the
    // last matrix instruction that wrote sacc): eleven instructions
    auto mx_op = [&](auto jc) __attribute__((always_inline)) {
        constexpr int j = decltype(jc)::value;
        if constexpr (j == 0) asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(mxr) : "v"(sacc[0]), "v"(sacc[1]), "v"(sacc[2]));
        if constexpr (j >= 1 && j <= 6)
            asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(mxr) : "v"(sacc[2 * j + 1]), "v"(sacc[2 * j + 2]));
        if constexpr (j == 7) asm volatile("v_max_f32 %0, %0, %1" : "+v"(mxr) : "v"(sacc[15]));
        if constexpr (j == 8) asm volatile("v_mov_b32 %0, %1" : "=v"(tlo) : "v"(mxr));
        // (lanes 32 .. 63 of tlo <-> lanes 0 .. 31 of mxr: tlo = the lower half's maximum everywhere, mxr the upper's)
        if constexpr (j == 9) asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(tlo), "+v"(mxr));
        if constexpr (j == 10) asm volatile("v_max_f32 %0, %0, %1" : "+v"(mxr) : "v"(tlo));
    };

    // ---- 8-bit K: the conversion of tile t+2 between the matrix steps of phase A ---------------------------------------
    // Slot c = 0 .. 9 of this thread (see conv_addr) is read from the stage behind step 3 c's ring read and written,
    // converted, behind step 3 c + 2's; both are LDS operations and count in the waits of the ring (conv_ops_between).
    typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
    typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
    constexpr int kConvWrites = KV8 == kKvInt8 ? 2 : 1;  // LDS writes per converted chunk
    uint32_t csrc = 0, cdst_a = 0, cdst_b = 0;  // this trip's source and destinations (thread's row and chunk)
    u32x2_t craw = {0u, 0u};
    auto conv_read = [&](auto cc) __attribute__((always_inline)) {
        constexpr int c = decltype(cc)::value;
        u32x2_t& raw = craw;  // (named outside the dependent statement, so that the lambda captures them)
        const uint32_t src = csrc;
        if constexpr (c % 5 == 4) {
            if ((threadIdx.x & 15) < 8) asm volatile("ds_read_b64 %0, %1 offset:%2" : "+v"(raw) : "v"(src), "n"(conv_src_off(c)));
        } else {
            asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(raw) : "v"(src), "n"(conv_src_off(c)));
        }
    };
    // VN: the phase goes on into phase B (the ring reads behind steps 28 and up are then two transpose reads each)
    auto conv_write = [&](auto cc, auto vn_c) __attribute__((always_inline)) {
        constexpr int c = decltype(cc)::value;
        constexpr int g = 3 * c + 2;  // the step this runs behind
        // the chunk's read has landed: behind it went the ring reads of this step and the one before
        constexpr int r1 = g - 1 + kRing < KS ? 1 : (decltype(vn_c)::value ? 2 : 0);
        constexpr int r0 = g + kRing < KS ? 1 : (decltype(vn_c)::value ? 2 : 0);
        asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(craw) : "n"(r0 + r1));
        constexpr bool kTail = c % 5 == 4;  // the row's last chunk: key columns 512 .. 575, lanes j < 8
        const uint32_t dbase = kTail ? cdst_b : cdst_a;
        constexpr int OFF = conv_dst_off(c);
        auto write = [&]() __attribute__((always_inline)) {
            if constexpr (kConvWrites == 2) {
                // (int8: four elements at a time, so that two registers of results are live instead of four)
                const uint2 lo = int8x4_to_16<Tag>(craw.x);
                const u32x2_t vlo = {lo.x, lo.y};
                asm volatile("ds_write_b64 %0, %1 offset:%2" ::"v"(dbase), "v"(vlo), "n"(OFF) : "memory");
                const uint2 hi = int8x4_to_16<Tag>(craw.y);
                const u32x2_t vhi = {hi.x, hi.y};
                asm volatile("ds_write_b64 %0, %1 offset:%2" ::"v"(dbase), "v"(vhi), "n"(OFF + 8) : "memory");
            } else {
                const uint4 cv = kv8x8_to_16<Tag, KV8 ? KV8 : kKvFp8>(make_uint2(craw.x, craw.y));
                const u32x4_t v = {cv.x, cv.y, cv.z, cv.w};
                asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(dbase), "v"(v), "n"(OFF) : "memory");
            }
        };
        if constexpr (kTail) {
            if ((threadIdx.x & 15) < 8) write();
        } else {
            write();
        }
    };

    // ---- phase A: S(t+1) = K(t+1) Q^T beside the softmax of S(t) and the loads of tile t+3 ------------------------
    // QK: the matrix steps (else only the softmax runs: last trip); SM: the softmax (else only the matrix steps:
    // prologue); DMA >= 0: the nine loads of a whole tile go out behind steps DMA, DMA + 4, ..., DMA + 32.  (A
    // direct-to-LDS load blocks its wave until the memory path accepts it, ~100 clocks at this kernel's 4 TB/s; giving
    // each of the four waves another DMA, so that their loads do not come together, measured slower, 2970 against
    // 2800 clocks per tile.)
    // CONV (8-bit K, steady-state trips): the conversion of tile t+2 and the five loads of raw tile t+4 (DMA == kDmaRaw,
    // behind steps 1, 9, ..., 33) ride along.
    auto phase_a = [&](auto qk_c, auto sm_c, auto dma_c, uint32_t tb, uint32_t tv, const uint8_t* base,
                       const uint8_t* base1, uint32_t dma_lds, auto ro_c, auto conv_c) __attribute__((always_inline)) {
        constexpr bool QK = decltype(qk_c)::value, SM = decltype(sm_c)::value;
        constexpr bool CONV = decltype(conv_c)::value;
        constexpr int DMA = decltype(dma_c)::value;
        constexpr int RO = decltype(ro_c)::value;
        constexpr bool VNEXT = SM;  // a trip with a softmax continues with phase B
        if constexpr (QK) {
            // the ring was primed by the caller with steps 0 .. kRing-1
            static_for<0, KS>([&](auto gc) {
                constexpr int g = decltype(gc)::value;
                // reads outstanding behind step g's: steps g+1 .. g+kRing-1
                constexpr int last_issued = VNEXT ? g + kRing - 1 : (g + kRing - 1 < KS ? g + kRing - 1 : KS - 1);
                constexpr int nk = (last_issued < KS ? last_issued : KS - 1) - g;           // K reads among them
                constexpr int nv = last_issued >= KS ? last_issued - KS + 1 : 0;            // V steps among them
                // (the counter of outstanding operations has four bits: waiting for fewer than are behind is safe)
                constexpr int behind = nk + 2 * nv + (CONV ? conv_ops_between(g - kRing, g - 1, kConvWrites) : 0);
                wait_lgkm_n<(behind < 15 ? behind : 15)>();
                mma_s<Tag, kRingV + 4 * ((g + RO) % kRing), kQV + 4 * g, g == 0>(sacc);
                if constexpr (g + kRing < KS)
                    read_k(std::integral_constant<int, g + kRing>{}, tb, ro_c);
                else if constexpr (VNEXT)
                    read_v(std::integral_constant<int, g + kRing - KS>{}, tv, ro_c);
                if constexpr (CONV) {
                    if constexpr (g % 3 == 0 && g / 3 < kConvSlots) conv_read(std::integral_constant<int, g / 3>{});
                    if constexpr (g % 3 == 2 && g / 3 < kConvSlots)
                        conv_write(std::integral_constant<int, g / 3>{}, std::integral_constant<bool, VNEXT>{});
                }
                if constexpr (SM) {
                    constexpr int per = (SMN + 27) / 28;  // spread over the first 28 steps (the last 8 carry two reads)
                    static_for<(g * per < SMN ? g * per : SMN), ((g + 1) * per < SMN ? (g + 1) * per : SMN)>(sm_op);
                }
                if constexpr (DMA == kDmaRaw) {
                    if constexpr (g % 8 == 1) issue_raw_piece(std::integral_constant<int, g / 8>{}, base, base1, dma_lds);
                } else if constexpr (DMA >= 0 && g % 4 == (DMA >= 0 ? DMA : 0)) {
                    issue_load_fast(std::integral_constant<int, g / 4>{}, base, base1, dma_lds);
                }
            });
        } else {
            static_for<0, SMN>(sm_op);
            // prime the ring with V steps 0 .. kRing-2 (two reads each; the counter of outstanding reads is 4 bits)
            static_for<0, kRing - 1>([&](auto ic) { read_v(ic, tv, ro_c); });
        }
    };

    // ---- phase B: O += V(t)^T P(t)^T --------------------------------------------------------------------------------
    // AHEAD: V steps requested ahead (kRing behind a phase A with matrix steps, kRing - 1 otherwise); MX: the maximum
    // of the scores in sacc is taken on the way (steps 4 .. 14)
    // NEXTK (steady-state loop; AHEAD = kRing): the ring runs on into the next trip.  Behind step NV - kRing's matrix
    // instruction the wave waits for its own loads of tile t+2 and meets the other waves at a barrier, after which that
    // tile is in LDS for everyone; the last kRing steps then request the first kRing K fragments of tile t+2 (region-B
    // base tb_next; ka[] has moved there by then), which the next trip's phase A finds on their way.
    auto phase_b = [&](auto ahead_c, auto mx_c, uint32_t tv, uint32_t ka_delta, auto ro_c, auto nextk_c, uint32_t tb_next) __attribute__((always_inline)) {
        constexpr int AHEAD = decltype(ahead_c)::value;
        constexpr bool MX = decltype(mx_c)::value;
        constexpr int RO = decltype(ro_c)::value;
        constexpr bool NEXTK = decltype(nextk_c)::value;
        static_assert(!NEXTK || (AHEAD == kRing && MX && 16 + NKA <= NV - kRing), "the K addresses move before they are used");
        static_for<0, NV>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            constexpr int slot = (KS + i + RO) % kRing;
            constexpr int left = NV - 1 - i;
            // reads outstanding behind step i's: V steps (two reads each), then, NEXTK, K steps of the next tile (one each)
            constexpr int nv = left < AHEAD - 1 ? left : AHEAD - 1;
            constexpr int nk = NEXTK ? AHEAD - 1 - nv : 0;
            wait_lgkm_n<2 * nv + nk>();
            mma_o<Tag, kRingV + 4 * slot, kScV + 4 * (i & 1), 16 * (i >> 1)>();
            if constexpr (NEXTK && i == NV - AHEAD) {
                // this wave's share of tile t+2 has landed (tile t+3's loads may be outstanding); 8-bit K: every wave
                // has converted its share of tile t+2 (its writes lie behind the ring reads waited for since)
                if constexpr (!KV8) wait_vmcnt<NLW>();
                asm volatile("s_barrier" ::: "memory");
            }
            if constexpr (i + AHEAD < NV)
                read_v(std::integral_constant<int, i + AHEAD>{}, tv, ro_c);
            else if constexpr (NEXTK)
                read_k(std::integral_constant<int, i + AHEAD - NV>{}, tb_next, std::integral_constant<int, (KS + NV + RO) % kRing>{});
            if constexpr (MX && i >= 4 && i < 15) mx_op(std::integral_constant<int, i - 4>{});
            // the K read addresses move on to the buffer of the tile after next
            if constexpr (MX && i >= 16 && i < 16 + NKA)
                v_add_s(ka[i - 16], ka_delta);
        });
    };

    // the first kRing reads of a K tile (its region-A addresses were moved to it in the preceding phase B)
#pragma unroll
    for (int j = 0; j < NKA; ++j) ka[j] = base_a ^ (uint32_t)(32 * j);
    constexpr std::integral_constant<int, 0> ro0{};
    constexpr std::integral_constant<int, (KS + NV) % kRing> ro1{};  // the trip behind one that started at 0
    static_assert((2 * (KS + NV)) % kRing == 0, "two trips are a whole number of turns of the ring");
    auto prime_k = [&](uint32_t tb) __attribute__((always_inline)) { static_for<0, kRing>([&](auto gc) { read_k(gc, tb, ro0); }); };

    // The part of the softmax of tile t that precedes phase A: running maximum (moved only when exceeded by kLazy;
    // then the denominator and the output tiles are rescaled) and sc = scores - maximum in log2 units.  Whole tiles
    // without ALiBi under a non-negative scale take the maximum of the raw scores from phase B.
    // token of register r: tok0 + (r/4)*8 + half*4 + r%4
    const bool gen_all = p.is_alibi || !(sl >= 0.0f);
    // PLAIN (compile-time): the caller knows that this is a whole tile of a launch without ALiBi and with a
    // non-negative scale
    auto softmax_head = [&](int t, auto plain_c) __attribute__((always_inline)) {
        constexpr bool PLAIN = decltype(plain_c)::value;
        const int tok0 = c0 + t * kTile;
        const bool gen = !PLAIN && (gen_all || tok0 + kTile > c1);
        float mx;
        float xs[16];  // (general form only)
        if (gen) {
            mx = -INFINITY;
            const float b0 = bias0 + slope * (float)tok0;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int off = (r >> 2) * 8 + (r & 3);
                // (fused so that no slope * off products are kept in registers across the loop)
                const float x = __builtin_fmaf(sacc[r], sl, __builtin_fmaf(slope, (float)off, b0));
                xs[r] = (tok0 + half * 4 + off) < c1 ? x : -INFINITY;
                mx = fmaxf(mx, xs[r]);
            }
            mx = max_xor32(mx);
        } else {
            mx = mxr * sl;
        }
        const bool up = mx > m + kLazy;
        if (__any(up)) {
            const float mn = up ? mx : m;
            const float alpha = fast_exp2(m - mn);
            m = mn;
            l *= alpha;
            if (t > 0) {  // (the accumulators are still zero in the first trip)
                static_for<0, CT * 16>([&](auto ic) { scale_acc_n<decltype(ic)::value>(alpha); });
            }
        }
        if (gen) {
            static_for<0, 16>([&](auto rc) { sc_set<decltype(rc)::value>(xs[decltype(rc)::value] - m); });
        } else {
            const float negm = -m;
            static_for<0, 16>([&](auto rc) { sc_fma<decltype(rc)::value>(sacc[decltype(rc)::value], sl, negm); });
        }
    };

    // ---- prologue: S(0) ---------------------------------------------------------------------------------------------
    if constexpr (!KV8) {  // (8-bit K: tile 0 was converted behind the barrier above)
        if (ntiles > 2)
            wait_vmcnt<2 * NLW>();
        else if (ntiles > 1)
            wait_vmcnt<NLW>();
        else
            wait_vmcnt<0>();
        __syncthreads();
    }
#ifdef DA_PIPE_PROBE
    const long long pr_wq = wall_clock64();
#endif
    {
        prime_k(base_b);
        if (KV8 != 0 && 1 < ntiles) {
            const ConvAddr ca = conv_addr((uint32_t)STG, a_of(1), b_of(1));
            csrc = ca.src;
            cdst_a = ca.dst_a;
            cdst_b = ca.dst_b;
            phase_a(std::true_type{}, std::false_type{}, std::integral_constant<int, -1>{}, base_b, base_v, nullptr, nullptr, 0,
                    ro0, std::integral_constant<bool, KV8 != 0>{});
        } else {
            phase_a(std::true_type{}, std::false_type{}, std::integral_constant<int, -1>{}, base_b, base_v, nullptr, nullptr, 0,
                    ro0, std::false_type{});
        }
#pragma unroll
        for (int j = 0; j < NKA; ++j) ka[j] += a_of(1);  // on to tile 1
        // the compiler does not see the matrix instructions inside the assembly: cover the result latency of the
        // last one before anything reads the scores
        asm volatile("s_nop 15\n\ts_nop 7" : "+v"(sacc));
        float mx0 = sacc[0];
#pragma unroll
        for (int r = 1; r < 16; ++r) mx0 = fmaxf(mx0, sacc[r]);
        mxr = max_xor32(mx0);
    }

#ifdef DA_PIPE_PROBE
    const long long pr_t0 = clock64();
    const long long pr_w0 = wall_clock64();
#endif
    // ---- all trips but the last ------------------------------------------------------------------------------------
    // Tile t+3 goes out in trip t: a whole tile between the matrix steps of phase A (fast form), a partial tile (the
    // split's last) or rows looked up one by one (PG) in one go behind the barrier.
    const int nfull = (c1 - c0) / kTile;  // whole tiles
    const bool packed = p.block_table == nullptr;
    const uint8_t* kt3 = kbytes + (size_t)(start + c0 + (NB - 1) * kTile) * k_row_bytes;  // packed: first row of tile t+3
    int t = 0;
#ifdef DA_PIPE_PROBE
    long long pr_top = 0, pr_a = 0, pr_b = 0, pr_x0 = 0, pr_x1 = 0, pr_x2 = 0;
#endif
    // The common case on its own, with nothing left to decide per trip: packed rows, no ALiBi, a whole tile t+3.  Here
    // the fragment ring never drains: the barrier that makes tile t+2 visible sits eight matrix steps before the end
    // of trip t's phase B, whose last steps already request the first K fragments of tile t+2 (phase_b, NEXTK).  A
    // second, plain barrier at the top of a trip keeps the loads of tile t+3 behind every wave's last read of tile
    // t-1, whose buffer they fill.  Trips come in pairs (see RO at read_k).
    bool primed = false;  // the ring holds the first K fragments of tile t+1, which is in LDS for every wave
    if constexpr (KV8 != 0) {
        // ---- 8-bit K.  Entering trip t, tiles t and t+1 are in LDS in 16-bit form, raw tiles t+2 and t+3 are on their
        // way or there.  The trip converts tile t+2 and requests raw tile t+4 into the stage tile t+1 came from.
        if (packed && !gen_all && t + 5 < nfull) {
            // steady state: conversion and loads between the matrix steps, the ring runs on from trip to trip
            uint32_t cur_a = a_of(0), nxt_a = a_of(1), nx2_a = a_of(2), nxt_b = b_of(1), nx2_b = b_of(2);
            uint32_t stg_conv = (uint32_t)(2 * STG), stg_load = (uint32_t)(1 * STG);  // stages of raw tiles t+2, t+4
            const uint8_t* kt4 = kbytes + (size_t)(start + c0 + 4 * kTile) * k_row_bytes;  // first row of tile t+4
            __syncthreads();  // (tile 1 was converted on the way through S(0): now it is there for every wave)
            prime_k(base_b + nxt_b);
            auto steady_trip = [&](auto ro_c) __attribute__((always_inline)) {
                softmax_head(t, std::true_type{});
                wait_vmcnt<NLW8>();  // raw tile t+2 has landed (raw tile t+3's loads may be outstanding)
                // every wave is done with tile t-1, whose value region tile t+2 is converted into (and with the stage
                // of tile t+1, which raw tile t+4 is loaded into)
                asm volatile("s_barrier" ::: "memory");
                {
                    const ConvAddr ca = conv_addr(stg_conv, nx2_a, nx2_b);
                    csrc = ca.src;
                    cdst_a = ca.dst_a;
                    cdst_b = ca.dst_b;
                }
                phase_a(std::true_type{}, std::true_type{}, std::integral_constant<int, kDmaRaw>{}, base_b + nxt_b,
                        base_v + cur_a, kt4, kt4 + 16 * k_row_bytes, smem_off + (uint32_t)OFF_STG + stg_load, ro_c,
                        std::true_type{});
                kt4 += kTile * k_row_bytes;
                phase_b(std::integral_constant<int, kRing>{}, std::true_type{}, base_v + cur_a, nx2_a - nxt_a, ro_c,
                        std::true_type{}, base_b + nx2_b);
                const uint32_t nx3_a = nx2_a == (uint32_t)(2 * ABUF) ? 0u : nx2_a + (uint32_t)ABUF;
                cur_a = nxt_a;
                nxt_a = nx2_a;
                nx2_a = nx3_a;
                const uint32_t b_tmp = nxt_b;
                nxt_b = nx2_b;
                nx2_b = b_tmp;
                stg_conv = stg_conv == (uint32_t)(2 * STG) ? 0u : stg_conv + (uint32_t)STG;
                stg_load = stg_load == (uint32_t)(2 * STG) ? 0u : stg_load + (uint32_t)STG;
                ++t;
            };
            // (both trips of a pair load a whole raw tile: t + 4 and t + 5 lie below nfull)
            for (; t + 5 < nfull;) {
                steady_trip(ro0);
                steady_trip(ro1);
            }
            primed = true;
        }
        for (; t + 1 < ntiles; ++t) {
            const uint32_t cur_a = a_of(t), nxt_a = a_of(t + 1), nxt_b = b_of(t + 1);
            // raw tile t+2 has landed (raw tile t+3's loads may be outstanding); behind the barrier every wave is done
            // with tile t-1 and has converted its share of tile t+1
            if (t + 3 < ntiles)
                wait_vmcnt<NLW8>();
            else
                wait_vmcnt<0>();
            __syncthreads();
            // raw tile t+4: a whole one goes out between the matrix steps below, the split's last one here
            const bool whole4 = t + 4 < nfull;
            if (!whole4 && t + 4 < ntiles) issue_raw(c0 + (t + 4) * kTile, (t + 4) % 3);
            if (primed)
                primed = false;  // (the first K fragments of tile t+1 are on their way already)
            else
                prime_k(base_b + nxt_b);
            softmax_head(t, std::false_type{});
            if (t + 2 < ntiles) {
                // tile t+2 is converted between the matrix steps, as in the steady-state trips
                const ConvAddr ca = conv_addr((uint32_t)(((t + 2) % 3) * STG), a_of(t + 2), b_of(t + 2));
                csrc = ca.src;
                cdst_a = ca.dst_a;
                cdst_b = ca.dst_b;
                if (whole4) {
                    const TileRows tr = tile_rows(c0 + (t + 4) * kTile);
                    phase_a(std::true_type{}, std::true_type{}, std::integral_constant<int, kDmaRaw>{}, base_b + nxt_b,
                            base_v + cur_a, tr.base, tr.base1, smem_off + (uint32_t)(OFF_STG + ((t + 4) % 3) * STG), ro0,
                            std::true_type{});
                } else {
                    phase_a(std::true_type{}, std::true_type{}, std::integral_constant<int, -1>{}, base_b + nxt_b,
                            base_v + cur_a, nullptr, nullptr, 0, ro0, std::true_type{});
                }
            } else {
                phase_a(std::true_type{}, std::true_type{}, std::integral_constant<int, -1>{}, base_b + nxt_b,
                        base_v + cur_a, nullptr, nullptr, 0, ro0, std::false_type{});
            }
            phase_b(std::integral_constant<int, kRing>{}, std::true_type{}, base_v + cur_a, a_of(t + 2) - nxt_a, ro0,
                    std::false_type{}, 0);
        }
    } else {
        if (!PG && packed && !gen_all && t + NB < nfull) {
            uint32_t cur = 0, nxt = (uint32_t)BUF, dst = (uint32_t)((NB - 1) * BUF);  // buffers of tiles t, t+1, t+3
            wait_vmcnt<NLW>();  // tile 1 landed; tile 2 may still be in flight
            __syncthreads();
            prime_k(base_b + nxt);
            auto steady_trip = [&](auto ro_c) __attribute__((always_inline)) {
    #if DA_PIPE_PROBE > 1
                const long long pr_s0 = clock64();
    #endif
                softmax_head(t, std::true_type{});
    #if DA_PIPE_PROBE > 1
                const long long pr_s0b = clock64();
    #endif
                asm volatile("s_barrier" ::: "memory");  // every wave is done with tile t-1
    #if DA_PIPE_PROBE > 1
                const long long pr_s1 = clock64();
                pr_x2 += pr_s1 - pr_s0b;
                pr_top += pr_s1 - pr_s0;
    #endif
                phase_a(std::true_type{}, std::true_type{}, std::integral_constant<int, 1>{}, base_b + nxt, base_v + cur, kt3,
                        kt3 + 16 * k_row_bytes, smem_off + dst, ro_c, std::false_type{});
    #if DA_PIPE_PROBE > 1
                const long long pr_s2 = clock64();
                pr_a += pr_s2 - pr_s1;
    #endif
                kt3 += kTile * k_row_bytes;
                const uint32_t nn = dst == (uint32_t)((NB - 1) * BUF) ? 0u : dst + (uint32_t)BUF;  // buffer after dst = that of tile t+4
                // (tile t+2 lies in the buffer behind nxt)
                const uint32_t nx2 = nxt == (uint32_t)((NB - 1) * BUF) ? 0u : nxt + (uint32_t)BUF;
                phase_b(std::integral_constant<int, kRing>{}, std::true_type{}, base_v + cur, nx2 - nxt, ro_c, std::true_type{},
                        base_b + nx2);
    #if DA_PIPE_PROBE > 1
                pr_b += clock64() - pr_s2;
    #endif
                cur = nxt;
                nxt = nx2;
                dst = nn;
                ++t;
            };
            // (both trips of a pair load a whole tile: t + 3 and t + 4 lie below nfull)
            for (; t + NB < nfull;) {
                steady_trip(ro0);
                steady_trip(ro1);
            }
            primed = true;
        }
        for (; t + 1 < ntiles; ++t) {
    #if DA_PIPE_PROBE > 1
            const long long pr_s0 = clock64();
    #endif
            const uint32_t cur = (uint32_t)((t & (NB - 1)) * BUF), nxt = (uint32_t)(((t + 1) & (NB - 1)) * BUF);
            const bool fast = !PG && t + NB - 1 < nfull;
            TileRows tr{nullptr, nullptr, 0};
            if (fast) {
                if (packed) {  // rows follow each other at the pitch
                    tr.base = kt3;
                    tr.base1 = kt3 + 16 * k_row_bytes;
                    kt3 += kTile * k_row_bytes;
                } else {
                    tr = tile_rows(c0 + (t + NB - 1) * kTile);
                }
            }
    #if DA_PIPE_PROBE > 1
            const long long pr_s0a = clock64();
    #endif
            if (primed) {
                // behind the steady-state loop: tile t+1 is in LDS for every wave and its first K fragments are on their
                // way; what is left to wait for is every wave's last read of tile t-1
                __syncthreads();
                primed = false;
            } else {
                if (t + 2 < ntiles)
                    wait_vmcnt<NLW>();  // tile t+1 landed; tile t+2 may still be in flight
                else
                    wait_vmcnt<0>();
                __syncthreads();  // every wave's share of tile t+1 is in LDS, and every wave is done with tile t-1
                prime_k(base_b + nxt);
            }
            if (!fast && t + NB - 1 < ntiles) {
                if constexpr (PG)
                    issue_tile_pg(c0 + (t + NB - 1) * kTile, (t + NB - 1) & (NB - 1));
                else
                    issue_tile(c0 + (t + NB - 1) * kTile, (t + NB - 1) & (NB - 1));
            }
            softmax_head(t, std::false_type{});
    #if DA_PIPE_PROBE > 1
            const long long pr_s1 = clock64();
            pr_top += pr_s1 - pr_s0;
    #endif
            if (fast)
                phase_a(std::true_type{}, std::true_type{}, std::integral_constant<int, 1>{}, base_b + nxt, base_v + cur, tr.base,
                        tr.base1, smem_off + (uint32_t)(((t + NB - 1) & (NB - 1)) * BUF), ro0, std::false_type{});
            else
                phase_a(std::true_type{}, std::true_type{}, std::integral_constant<int, -1>{}, base_b + nxt, base_v + cur, nullptr,
                        nullptr, 0, ro0, std::false_type{});
    #if DA_PIPE_PROBE > 1
            const long long pr_s2 = clock64();
            pr_a += pr_s2 - pr_s1;
    #endif
            // (tile t+2 lies in buffer (t+2) % NB)
            phase_b(std::integral_constant<int, kRing>{}, std::true_type{}, base_v + cur,
                    (uint32_t)(((t + 2) & (NB - 1)) * BUF) - nxt, ro0, std::false_type{}, 0);
    #if DA_PIPE_PROBE > 1
            pr_b += clock64() - pr_s2;
    #endif
        }
    }
    // ---- the last trip: softmax and O += V^T P^T of the last tile -------------------------------------------------------
    {
        const uint32_t cur = a_of(t);
        softmax_head(t, std::false_type{});
        phase_a(std::false_type{}, std::true_type{}, std::integral_constant<int, -1>{}, 0, base_v + cur, nullptr, nullptr, 0, ro0,
                std::false_type{});
        phase_b(std::integral_constant<int, kRing - 1>{}, std::false_type{}, base_v + cur, 0, ro0, std::false_type{}, 0);
    }

#ifdef DA_PIPE_PROBE
    const long long pr_t1 = clock64();
    const long long pr_w1 = wall_clock64();
#endif
    // finish: the two half-waves hold partial denominators over disjoint tokens
    const float l_tot = l + __shfl_xor(l, 32);
    // (the last matrix instructions' results must have landed before the accumulation registers are read)
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    auto acc_at = [&](auto ic) { return read_acc_n<decltype(ic)::value>(); };
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    // Normalised by the denominator, as 16-bit values: the final output, or (sequence split) the split's partial
    // (ReduceParams::half_partials) beside the running maximum and the denominator as fp32.
    if (p.nsplit > 1) {
        // A split's partial leaves as it lies in the registers (nat_piece in da_common.h): lane (n, half) holds four
        // columns of head n per 32 x 32 tile quarter, the wave stores 1 KiB (two quarters, 16 bytes a lane) per
        // instruction, and the merge kernel reads in that order.  No trip through LDS and no barrier in the tail every work-group of a
        // one-round grid runs at the same moment.
        const float inv = (KV8 ? head_scale(p.v_scale, hk) : 1.0f) / l_tot;  // (8-bit K: times the V factor)
        const int blk = (hk * p.groups + grp) * NWV + wave;
        uint8_t* const rec = reinterpret_cast<uint8_t*>(p.ws_o) +
                             nat_block((size_t)b, p.nsplit, split, nat_blocks(p.head_k, p.groups, NWV), blk) * 8;
        uint8_t* const dst = rec + lane * 16;
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        // (a whole 32 x 32 tile's sixteen values are read before any is converted: the reads are independent, and a
        // lone wave per SIMD has nothing else to cover the wait between a read and its use)
        static_for<0, CT>([&](auto cc) {
            constexpr int c = decltype(cc)::value;
            float a[16];
            static_for<0, 16>([&](auto ic) { a[decltype(ic)::value] = acc_at(std::integral_constant<int, c * 16 + decltype(ic)::value>{}); });
#pragma unroll
            for (int rp = 0; rp < 2; ++rp) {
                u32x4 w;
                w.x = EL::pack2_scaled(a[rp * 8 + 0], a[rp * 8 + 1], inv);
                w.y = EL::pack2_scaled(a[rp * 8 + 2], a[rp * 8 + 3], inv);
                w.z = EL::pack2_scaled(a[rp * 8 + 4], a[rp * 8 + 5], inv);
                w.w = EL::pack2_scaled(a[rp * 8 + 6], a[rp * 8 + 7], inv);
                *reinterpret_cast<u32x4*>(dst + (c * 2 + rp) * 1024) = w;
            }
        });
        if (n < nh && half == 0) reinterpret_cast<float2*>(rec)[nat_ml(n)] = make_float2(m, l_tot);
    } else {
        // The wave's 32 output rows (its heads) leave through LDS: a lane holds groups of four columns of its head's
        // row, so storing from registers would scatter 8-byte pieces over 32 rows per instruction; instead the rows
        // are written to the wave's own tile buffer (pitch 1040 bytes: lanes of one write fall on different banks)
        // and read back a whole row (1 KiB, 16 bytes a lane) per instruction.
        __syncthreads();  // every wave is done with the tile buffers
        constexpr int PITCH = DV * 2 + 16;  // (a multiple of 16: the rows are read back 16 bytes a lane)
        static_assert(32 * PITCH <= BUF, "a wave's rows fit its tile buffer");
        typedef __attribute__((address_space(3))) uint8_t* lds_ptr;
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        const lds_ptr wbuf = (lds_ptr)(uintptr_t)(smem_off + (uint32_t)(wave * BUF));
        const float inv = (KV8 ? head_scale(p.v_scale, hk) : 1.0f) / l_tot;  // (8-bit K: times the V factor)
        static_for<0, CT * 4>([&](auto ic) {
            constexpr int c = decltype(ic)::value / 4, r4 = decltype(ic)::value % 4;
            const int col = c * 32 + r4 * 8 + half * 4;
            u32x2 w;
            w.x = EL::pack2_scaled(acc_at(std::integral_constant<int, c * 16 + r4 * 4 + 0>{}),
                                   acc_at(std::integral_constant<int, c * 16 + r4 * 4 + 1>{}), inv);
            w.y = EL::pack2_scaled(acc_at(std::integral_constant<int, c * 16 + r4 * 4 + 2>{}),
                                   acc_at(std::integral_constant<int, c * 16 + r4 * 4 + 3>{}), inv);
            *reinterpret_cast<__attribute__((address_space(3))) u32x2*>(wbuf + n * PITCH + col * 2) = w;
        });
        // (LDS operations of one wave complete in order: the wave reads its own rows back)
        uint16_t* const dst = o16 + ((size_t)b * p.head_q + h_base) * DV;
        constexpr size_t row_elems = DV;  // elements between consecutive heads' rows
        typedef const __attribute__((address_space(3))) u32x4* lds_row;
        if (nh == 32) {
            // eight rows read, then eight rows stored
#pragma unroll
            for (int r0 = 0; r0 < 32; r0 += 8) {
                u32x4 v[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = *reinterpret_cast<lds_row>(wbuf + (r0 + i) * PITCH + lane * 16);
#pragma unroll
                for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4*>(dst + (size_t)(r0 + i) * row_elems + lane * 8) = v[i];
            }
        } else {
            for (int r = 0; r < nh; ++r) {
                const u32x4 v = *reinterpret_cast<lds_row>(wbuf + r * PITCH + lane * 16);
                *reinterpret_cast<u32x4*>(dst + (size_t)r * row_elems + lane * 8) = v;
            }
        }
    }
#ifdef DA_PIPE_PROBE
    if (p.nsplit > 1) {
        // stamps into the unused last quarter of the fp32-sized partial area, 16 floats per work-group
        const long long pr_w3 = wall_clock64();  // stores issued
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const long long pr_w2 = wall_clock64();
        if (threadIdx.x == 0) {
            float* pa = p.ws_o + (size_t)p.batch * p.head_q * p.nsplit * (DV / 4 * 3) + ((size_t)b * p.nsplit + split) * 16;
            pa[0] = (float)(pr_t1 - pr_t0);
            pa[1] = (float)(pr_w1 - pr_w0);
            pa[2] = (float)pr_top;
            pa[3] = (float)pr_a;
            pa[4] = (float)pr_b;
            pa[5] = (float)ntiles;
            pa[6] = (float)(pr_wk & 0xffffff);
            pa[7] = (float)(pr_w0 & 0xffffff);
            pa[8] = (float)(pr_w1 & 0xffffff);
            pa[9] = (float)(pr_w2 & 0xffffff);
            pa[10] = (float)(pr_wq & 0xffffff);
            pa[11] = (float)pr_x1;
            pa[12] = (float)pr_x2;
            pa[13] = (float)(pr_w3 & 0xffffff);
        }
    }
#endif
}

template <typename Tag, bool PG, int KV8 = 0>
hipError_t launch_form(const SweepParams& p, dim3 grid, hipStream_t stream) {
    auto kern = latent_pipe_kernel<Tag, PG, KV8>;
    // four 16-bit tile buffers; 8-bit K: three value regions, two key-tail regions, three raw stages
    constexpr size_t lds = KV8 ? (size_t)3 * kTile * 512 * 2 + (size_t)2 * kTile * 64 * 2 + (size_t)3 * kTile * 576
                               : (size_t)kPipeBufs * kTile * 576 * 2;
    static_assert(lds <= 160 * 1024, "LDS of one CU");
    static std::atomic<uint64_t> devices_done{0};
    const hipError_t attr_err = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds, devices_done);
    if (attr_err != hipSuccess) return attr_err;
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, p);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_mla_pipe(const SweepParams& p_in, bool is_bf16, dim3 grid, hipStream_t stream) {
    SweepParams p = p_in;
#ifdef DA_PIPE_PROBE
    {
        const char* s = getenv("DA_PIPE_FLAGS");
        p.flat_min = s ? atoi(s) : 0;
    }
#endif
    const bool pg = p.block_table != nullptr && p.page_shift < 4;
    if (is_bf16) return pg ? launch_form<bf16_tag, true>(p, grid, stream) : launch_form<bf16_tag, false>(p, grid, stream);
    return pg ? launch_form<f16_tag, true>(p, grid, stream) : launch_form<f16_tag, false>(p, grid, stream);
}

bool mla_pipe_kv8_supported(const SweepParams& p) {
    // rows of 576 bytes (one KV head), fetched in runs of 16 tokens: the packed layout, or pages of 16 tokens and more
    return p.k_row == 576 && (p.block_table == nullptr || p.page_shift >= 4);
}

hipError_t launch_mla_pipe_kv8(const SweepParams& p, int fmt, bool is_bf16, dim3 grid, hipStream_t stream) {
    if (!mla_pipe_kv8_supported(p)) return hipErrorInvalidValue;
    if (fmt == kKvInt8)
        return is_bf16 ? launch_form<bf16_tag, false, kKvInt8>(p, grid, stream) : launch_form<f16_tag, false, kKvInt8>(p, grid, stream);
    return is_bf16 ? launch_form<bf16_tag, false, kKvFp8>(p, grid, stream) : launch_form<f16_tag, false, kKvFp8>(p, grid, stream);
}

}  // namespace da
