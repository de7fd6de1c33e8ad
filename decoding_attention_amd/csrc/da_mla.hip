// MFMA sweep for many query heads over one KV head whose values are the leading columns of
// the keys (the latent MLA form: 128 heads, key width 576, value width 512).
//
// One work-group serves one (sequence, head group of up to 128 heads, sequence split).  Each of
// its wavefronts owns 32 query heads: their Q rows stay in registers as MFMA B-operands
// (36 k-steps x 4 VGPRs), their un-normalised output O^T[512 x 32] stays in 16 accumulator
// tiles (256 registers), so one wavefront per SIMD uses the whole 512-register budget.
//
// K tiles of 32 tokens stream HBM -> LDS with direct-to-LDS loads (no register staging),
// three buffers deep.  A tile is read from LDS twice and from HBM once:
//   S^T[32 tok x 32 heads] = K_tile . Q^T      K rows as A-operands, ds_read_b128
//   O^T[512 x 32 heads]   += V_tile^T . P^T    V = K[:, :512]; the A-operand needs 8 tokens of
//                                              one column per lane, delivered by the LDS
//                                              transpose read ds_read_b64_tr_b16
// The score tile leaves the MFMA with one head per lane (column n = lane % 32) and 16 tokens
// per lane, so the online softmax is lane-local but for one exchange between the two
// half-waves, and the probabilities feed the second MFMA as its B-operand without any lane
// movement (the token <-> k-index permutation is applied to V's rows instead).
//
// LDS tile layout.  A tile buffer has two regions: the 512 value columns of the 32 rows (1 KiB per row) and
// the remaining 64 key columns (128 B per row).  One direct-to-LDS load instruction fills exactly one row of
// the first region (or eight rows of the second), so its source is a wave-uniform row address plus a per-lane
// chunk offset.  Inside a row the 16-byte chunks are XOR-swizzled with the row index --
//   first region:  chunk c of row r at c ^ ((r & 3) << 2 | (r >> 2) & 3)
//   second region: chunk c of row r at c ^ ((r >> 1) & 7)
// -- which makes both read patterns (16 rows x one chunk for K, 4 rows x 64 bytes for V^T) conflict-free, and
// because XOR commutes with the per-step chunk offsets every read address is one per-lane base XOR a constant.
//
// 8-bit K cache (KV8: FP8 e4m3 or int8): the tile's bytes (32 rows x 576 elements, 18 KiB) are staged in LDS by the
// same direct-to-LDS loads, three stages deep, and the work-group converts each staged tile into the 16-bit tile
// layout above (exact: e4m3 or int8 -> fp16/bf16) one tile ahead of its use, two 16-bit buffers deep; everything downstream of the
// tile is the 16-bit kernel.  The per-head scales fold into the softmax scale and the final normalisation.
//
// Mathematics as in the reference kernel (csrc/kernel/decoding_attn/decoding_fwd_kernel.h:50-235
// with the latent aliasing of csrc/ops/decoding_attn.cpp:30-37); the structure is unrelated.
#include "da_mla.h"
#include "da_mla_dev.h"

#include <cstdlib>

namespace da {

namespace {

using namespace mla;


// PG: paged K/V with pages of fewer than 16 tokens (down to 1): every row of a tile has its own page lookup.
// NB: tile buffers of the 16-bit form.  Three keep two tiles in flight behind the one being read; two (one in
// flight) halve the LDS footprint, so that two work-groups of one or two waves share a CU.
// VD: V is a buffer of its own ([tokens, head_k, 512], not the leading columns of K).  A tile buffer then starts with
// the tile's 32 V rows (the layout of the first K region, read by the same transpose reads) followed by the K tile;
// at 68 KiB a buffer, two of them fit.
template <typename Tag, int D, int DV, int NWV, int KV8, bool PG = false, int NB = kNBuf, bool VD = false>
__global__ __launch_bounds__(64 * NWV) void mfma_latent_kernel(const SweepParams p) {
    // (FP8 with PG: the stage is filled a row per load, 36 of the 64 lanes active, instead of 1 KiB per load)
    using MM = Mma<Tag>;
    using vec8 = typename MM::vec8;
    using EL = Elem<Tag>;
    static_assert(D == 576 && DV == 512 && (NWV == 1 || NWV == 2 || NWV == 4), "tile layout is specific to (576, 512)");
    constexpr int ROW_A = DV * 2;                        // bytes per row, region A (value columns)
    constexpr int ROW_B = (D - DV) * 2;                  // bytes per row, region B (remaining key columns)
    constexpr int OFF_KA = VD ? kTile * ROW_A : 0;       // K's region A starts here (VD: behind the V rows)
    constexpr int OFF_B = OFF_KA + kTile * ROW_A;        // region B starts here
    constexpr int BUF = OFF_B + kTile * ROW_B;           // bytes per tile buffer
    constexpr int QBUF = kTile * D * 2;                  // bytes of a wave's staged Q block (a K tile without V rows)
    constexpr int QOFF_B = kTile * ROW_A;
    constexpr int NLA = kTile / NWV;                     // region-A load instructions per tile per wave (one row each)
    constexpr int NLB = (kTile / 8) / NWV;               // region-B load instructions per tile per wave (eight rows each)
    constexpr int NLW = (VD ? 2 : 1) * NLA + NLB;        // load instructions per tile per wave
    static_assert(!VD || (KV8 == 0 && !PG && NB == 2), "the distinct-V form: 16-bit K/V, runs of 16 tokens, two buffers");
    constexpr int KS = D / 16;                           // k-steps of Q K^T
    constexpr int CT = DV / 32;                          // 32-column tiles of the output
    // FP8 K cache: stages of the tile's raw bytes, filled 1 KiB per load instruction
    static_assert(NB == kNBuf || (NB == 2 && !KV8), "buffer count");
    constexpr int NTB = KV8 ? 2 : NB;                    // 16-bit tile buffers
    constexpr int STG_REAL = kTile * D / 1024;           // load instructions that cover a staged tile (18)
    constexpr int NLW8 = PG ? kTile / NWV : (STG_REAL + NWV - 1) / NWV;  // per wave (the surplus ones repeat the last
                                                                         // KiB); PG: a row per load
    constexpr int STG = ((STG_REAL + NWV - 1) / NWV) * NWV * 1024;  // bytes per stage
    constexpr int STG0 = NTB * BUF;                      // stages start behind the 16-bit buffers
    static_assert((kTile * D) % 1024 == 0, "staged tile");
    static_assert(D % 16 == 0 && DV % 32 == 0 && DV <= D, "shape");

    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];  // lds_bytes<D, NWV, KV8, NB>()
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

    // Q rows of this wave's heads as B-operands: lane (n, half) holds Q[head n][ks*16 + half*8 .. +8).  Loading
    // that layout straight from global memory costs 36 instructions of 32-byte pieces per wave; instead the
    // wave's 32 x 576 block of Q is staged like a K tile (whole-row direct-to-LDS loads, same swizzle, into the
    // wave's own buffer) and read back with the K-row read pattern, which is the same operand layout.
    const int q_last = max(nh, 1) - 1;
    const int hq = min(h_base + min(n, q_last), p.head_q - 1);
    const uint32_t lane16 = lane * 16;
    const int rb = lane >> 3;  // region B: row within the group of eight, chunk lane & 7
    vec8 qf[KS];
    {
        const uint8_t* const qb = reinterpret_cast<const uint8_t*>(p.q) + (size_t)b * p.head_q * (D * 2);
        const uint32_t qbuf = smem_off + wave * QBUF;
        static_for<0, kTile>([&](auto rc) {
            constexpr int row = decltype(rc)::value;
            const int head = min(h_base + min(row, q_last), p.head_q - 1);  // wave-uniform
            lds_dma16(qb, (uint32_t)head * (uint32_t)(D * 2) + (lane16 ^ (uint32_t)(swz_a(row) * 16)),
                      qbuf + (uint32_t)(row * ROW_A));
        });
        static_for<0, kTile / 8>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int row = j * 8 + rb;
            const int head = min(h_base + min(row, q_last), p.head_q - 1);
            lds_dma16(qb, (uint32_t)head * (uint32_t)(D * 2) + (uint32_t)(DV * 2 + (((lane & 7) ^ swz_b(row)) * 16)),
                      qbuf + (uint32_t)(QOFF_B + j * 1024));
        });
        wait_vmcnt<0>();
        const uint32_t qa = qbuf + n * ROW_A + ((swz_a(n) ^ half) * 16);
        const uint32_t qbb = qbuf + QOFF_B + n * ROW_B + ((swz_b(n) ^ half) * 16);
        static_for<0, KS>([&](auto ic) {
            constexpr int ks = decltype(ic)::value;
            if constexpr (ks < 32)
                lds_read_b128<(ks >> 3) * 256>(qf[ks], qa ^ (uint32_t)(32 * (ks & 7)));
            else
                lds_read_b128<0>(qf[ks], qbb ^ (uint32_t)(32 * (ks - 32)));
            if constexpr (ks % 12 == 11) wait_lgkm<0>(qf[ks]);  // the counter of outstanding reads is 4 bits wide
        });
    }
    __syncthreads();  // the tile buffers are free for K once every wave has its Q in registers
    const float slope = p.is_alibi ? alibi_slope_log2(p.slopes, hq, p.head_q) : 0.0f;

    f32x16 acc[CT];
#pragma unroll
    for (int c = 0; c < CT; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[c][r] = 0.0f;
    float m = kNegBig, l = 0.0f;

    constexpr int KB = KV8 ? 1 : 2;  // bytes per K element in memory
    const uint8_t* const kbytes = reinterpret_cast<const uint8_t*>(p.k) + (size_t)hk * D * KB;
    const size_t k_row_bytes = (size_t)p.k_row * KB;
    const uint8_t* const vbytes = reinterpret_cast<const uint8_t*>(p.v) + (size_t)hk * p.v_head * 2;  // (VD)
    const size_t v_row_bytes = (size_t)p.v_row * 2;
    const float sl = p.scale_log2 * head_scale(p.k_scale, hk);  // score scale, log2 units
    const float vs = head_scale(p.v_scale, hk);

    // Stage the tile that starts at token tok0 into buffer `buf`.  Rows past the end of the split re-read the
    // last valid row (they are masked later).  Every wave always issues exactly NLW loads, so the hand-placed
    // vmcnt waits count the same on every wave.
    // `row0` and `row1` are the rows of the tile's tokens 0 and 16 as row_ref() gives them: a tile is fetched as two
    // runs of 16 tokens, each inside one page (pages of paged K/V hold a multiple of 16 tokens and tiles start at
    // multiples of kTile; for the packed layout and larger pages the second run follows the first).  A row past the
    // end re-reads the last valid row, in whichever run that is.
    auto issue_tile = [&](int tok0, RowRef ref0, RowRef ref1, int buf) {
        const uint8_t* const base = kbytes + ref0.k * KB;
        const uint8_t* const base1 = kbytes + ref1.k * KB;
        const int last = c1 - 1 - tok0;
        if constexpr (KV8) {
            // stage `buf`: the tile's bytes in row order, lane l of load j bringing bytes [1024 j + 16 l, +16)
            static_assert(16 * D % 1024 == 0, "the two runs of a staged tile meet on a load boundary");
#pragma unroll
            for (int q = 0; q < NLW8; ++q) {
                const int j = min(wave + NWV * q, STG_REAL - 1);  // wave-uniform; surplus loads repeat the last KiB
                const uint32_t off = (uint32_t)j * 1024u + lane16;
                const uint32_t row = off / (uint32_t)D, within = off - row * (uint32_t)D;
                // rows 0..15 fill loads 0..8 exactly, rows 16..31 loads 9..17: the run is wave-uniform
                const int run = min(j >= 16 * D / 1024 ? 1 : 0, last >> 4);
                lds_dma16<true>(run ? base1 : base,
                          (uint32_t)(min((int)row, last) - run * 16) * (uint32_t)k_row_bytes + within,
                          smem_off + (uint32_t)(STG0 + buf * STG + (wave + NWV * q) * 1024));
            }
            return;
        }
#pragma unroll
        for (int q = 0; q < NLA; ++q) {
            const int row = wave + NWV * q;  // wave-uniform
            const int rc = min(row, last), run = rc >> 4;
            lds_dma16<true>(run ? base1 : base,
                      (uint32_t)(rc - run * 16) * (uint32_t)k_row_bytes + (lane16 ^ (uint32_t)(swz_a(row) * 16)),
                      smem_off + (uint32_t)(buf * BUF + OFF_KA + row * ROW_A));
        }
        if constexpr (VD) {
            const uint8_t* const vbase = vbytes + ref0.v * 2;
            const uint8_t* const vbase1 = vbytes + ref1.v * 2;
#pragma unroll
            for (int q = 0; q < NLA; ++q) {
                const int row = wave + NWV * q;
                const int rc = min(row, last), run = rc >> 4;
                lds_dma16<true>(run ? vbase1 : vbase,
                          (uint32_t)(rc - run * 16) * (uint32_t)v_row_bytes + (lane16 ^ (uint32_t)(swz_a(row) * 16)),
                          smem_off + (uint32_t)(buf * BUF + row * ROW_A));
            }
        }
#pragma unroll
        for (int q = 0; q < NLB; ++q) {
            const int j = wave + NWV * q;
            const int row = j * 8 + rb;
            const int run = min(j >> 1, last >> 4);  // the eight rows of a load lie in one run, clamped or not
            lds_dma16<true>(run ? base1 : base, (uint32_t)(min(row, last) - run * 16) * (uint32_t)k_row_bytes +
                                              (uint32_t)(DV * 2 + (((lane & 7) ^ swz_b(row)) * 16)),
                      smem_off + (uint32_t)(buf * BUF + OFF_B + j * 1024));
        }
    };

    // PG: the wave's kTile / NWV rows are consecutive here (rows wave * NLA + q), the same rows for both regions, so
    // one set of page lookups (scalar loads, fetched a trip ahead like the page of a whole tile otherwise) serves
    // both; the second region's load covers eight rows, so its lanes pick their row's address out of the set.
    struct RowPages {
        int pg[NLA];
    };
    auto lookup_rows = [&](int tok0) {
        RowPages r;
        const int last = c1 - 1 - tok0;
#pragma unroll
        for (int q = 0; q < NLA; ++q) r.pg[q] = page_of(p, b, tok0 + min(wave * NLA + q, last));
        return r;
    };
    auto issue_tile_pg = [&](int tok0, const RowPages& rp, int buf) {
        const int last = c1 - 1 - tok0;
        const int mask = (1 << p.page_shift) - 1;
        int64_t rowoff[NLA];  // byte offsets of the wave's rows
#pragma unroll
        for (int q = 0; q < NLA; ++q) {
            const int tok = tok0 + min(wave * NLA + q, last);
            rowoff[q] = ((int64_t)rp.pg[q] * p.k_page + (int64_t)(tok & mask) * p.k_row) * KB;
        }
        if constexpr (KV8) {
            // stage `buf`: row r of the tile at r * D bytes; one row (D bytes, D / 16 lanes) per load
#pragma unroll
            for (int q = 0; q < NLA; ++q) {
                const int row = wave * NLA + q;
                if (lane < D / 16) lds_dma16<true>(kbytes + rowoff[q], lane16, smem_off + (uint32_t)(STG0 + buf * STG + row * D));
            }
            return;
        }
#pragma unroll
        for (int q = 0; q < NLA; ++q) {
            const int row = wave * NLA + q;
            lds_dma16<true>(kbytes + rowoff[q], lane16 ^ (uint32_t)(swz_a(row) * 16),
                      smem_off + (uint32_t)(buf * BUF + row * ROW_A));
        }
#pragma unroll
        for (int q = 0; q < NLB; ++q) {
            const int j = wave * NLB + q;
            const int row = j * 8 + rb;
            int64_t mine = rowoff[8 * q];
#pragma unroll
            for (int i = 1; i < 8; ++i) mine = rb == i ? rowoff[8 * q + i] : mine;
            lds_dma16_v<true>(kbytes + mine + (DV * 2 + (((lane & 7) ^ swz_b(row)) * 16)),
                        smem_off + (uint32_t)(buf * BUF + OFF_B + j * 1024));
        }
    };

    // FP8: convert stage `stg` into 16-bit tile buffer `tb` (swizzled layout).  Eight threads share a row: thread
    // (row, j) converts the row's 8-element chunks j, j + 8, ..., j + 64, so its swizzles are constants and each
    // chunk costs one address XOR.
    constexpr int RPP = 8 * NWV;  // rows per pass
    const int cv_j = (int)threadIdx.x & 7, cv_r = (int)threadIdx.x >> 3;
    auto convert_stage = [&](int stg, int tb) {
        typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        typedef const __attribute__((address_space(3))) u32x2* lds_src;
        typedef __attribute__((address_space(3))) u32x4* lds_dst;
#pragma unroll
        for (int ps = 0; ps < kTile / RPP; ++ps) {
            const int r = cv_r + ps * RPP;
            const uint32_t src = smem_off + (uint32_t)(STG0 + stg * STG + r * D + cv_j * 8);
            const uint32_t dst_a = smem_off + (uint32_t)(tb * BUF + r * ROW_A + ((cv_j ^ swz_a(r)) * 16));
            const uint32_t dst_b = smem_off + (uint32_t)(tb * BUF + OFF_B + r * ROW_B + ((cv_j ^ swz_b(r)) * 16));
#pragma unroll
            for (int i = 0; i < D / 64; ++i) {
                const u32x2 rv = *reinterpret_cast<lds_src>((uintptr_t)(src + i * 64));
                // (this lambda is compiled, and never called, for 16-bit K as well)
                const uint4 cv = kv8x8_to_16<Tag, KV8 ? KV8 : kKvFp8>(make_uint2(rv.x, rv.y));
                // chunk j + 8 i of the value columns sits at (j + 8 i) ^ swizzle = (j ^ swizzle) ^ 8 i
                const uint32_t dst = i < DV / 64 ? (dst_a ^ (uint32_t)(i * 128)) : dst_b;
                *reinterpret_cast<lds_dst>((uintptr_t)dst) = u32x4{cv.x, cv.y, cv.z, cv.w};
            }
        }
    };

    const int ntiles = (c1 - c0 + kTile - 1) / kTile;
    // rows of tokens tok and tok + 16 (the second only looked up when the tile has it: the block table ends with
    // the sequence's last page)
    auto second_run = [&](int tok, RowRef first) { return tok + 16 < c1 ? row_ref(p, b, start, tok + 16) : first; };
    constexpr int AHEAD = KV8 ? 3 : NB - 1;  // tiles in flight behind the one being read
    RowPages rows_ahead{};
    if constexpr (PG) {
        issue_tile_pg(c0, lookup_rows(c0), 0);
        if (NB > 2 && ntiles > 1) issue_tile_pg(c0 + kTile, lookup_rows(c0 + kTile), 1);
        if (ntiles > NB - 1) rows_ahead = lookup_rows(c0 + (NB - 1) * kTile);
    } else {
        const RowRef r0 = row_ref(p, b, start, c0);
        issue_tile(c0, r0, second_run(c0, r0), 0);
        if (NB > 2 && ntiles > 1) {
            const RowRef r1 = row_ref(p, b, start, c0 + kTile);
            issue_tile(c0 + kTile, r1, second_run(c0 + kTile, r1), 1);
        }
    }
    if constexpr (KV8) {
        // three stages in flight; the first tile is converted here, tile t + 1 at the top of trip t
        if (ntiles > 2) {
            if constexpr (PG) {
                issue_tile_pg(c0 + 2 * kTile, rows_ahead, 2);
                if (ntiles > 3) rows_ahead = lookup_rows(c0 + 3 * kTile);
            } else {
                const RowRef r0 = row_ref(p, b, start, c0 + 2 * kTile);
                issue_tile(c0 + 2 * kTile, r0, second_run(c0 + 2 * kTile, r0), 2);
            }
        }
        if (ntiles > 2)
            wait_vmcnt<(2 * NLW8 < 63 ? 2 * NLW8 : 63)>();  // (the counter has six bits; waiting for fewer is safe)
        else if (ntiles > 1)
            wait_vmcnt<NLW8>();
        else
            wait_vmcnt<0>();
        __syncthreads();
        convert_stage(0, 0);
    }
    // page of the tile after those, fetched one trip ahead of its use (a scalar load for paged K/V)
    int page_ahead = !PG && ntiles > AHEAD ? page_of(p, b, c0 + AHEAD * kTile) : 0;
    int page_ahead1 = !PG && ntiles > AHEAD && c0 + AHEAD * kTile + 16 < c1 ? page_of(p, b, c0 + AHEAD * kTile + 16) : 0;
    // Make the compiler settle its own wait for the Q loads here, before the loop.  It cannot see the
    // direct-to-LDS loads, so a wait for Q placed inside the loop would count down to vmcnt(0) on every trip
    // and drain the tiles in flight.
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[ks]));

    // Per-lane LDS read bases (buffer 0); per-step chunk offsets are XORed in, the rest is instruction offset.
    // K rows: lane (n, half) reads chunk 2 ks + half of row n.
    //   ks < 32: (base_a ^ 32 (ks & 7)) + 256 (ks >> 3)        ks >= 32: base_b ^ 32 (ks - 32)
    const uint32_t base_a = smem_off + OFF_KA + n * ROW_A + ((swz_a(n) ^ half) * 16);
    const uint32_t base_b = smem_off + OFF_B + n * ROW_B + ((swz_b(n) ^ half) * 16);
    // V^T: as a source lane of the transpose read this lane addresses row half*4 + q (+16 s2, +8 for the second
    // read), 8 bytes at chunk 4 c + 2 b1 + b0 of it, q = (lane & 15) >> 2, b1 = lane bit 4, b0 = lane bit 1:
    //   (base_v ^ (64 c | 32 hi)) + 16 KiB s2 + 8 KiB hi
    const uint32_t base_v = smem_off + (half * 4 + ((lane & 15) >> 2)) * ROW_A + 64 * ((lane & 15) >> 2) +
                            16 * ((2 * ((lane >> 4) & 1) + ((lane >> 1) & 1)) ^ half) + 8 * (lane & 1);
    typedef short s16x8 __attribute__((__vector_size__(8 * sizeof(short))));

    const float bias0 = slope * (float)(half * 4 - (len - 1));  // ALiBi: slope * (token - (len - 1)), split in lane and tile parts
    int buf = 0;       // 16-bit buffer that holds tile t
    int buf_next = KV8 ? 0 : NB - 1;  // buffer (FP8: stage) that receives tile t + AHEAD
    int stg_conv = 1;  // FP8: stage that holds tile t + 1
    if constexpr (KV8 != 0) {
        // 8-bit K with fewer than 32 NWV heads: the work-group keeps all its waves for the loads and the conversion;
        // a wave without heads of its own runs only that part of every trip (the same loads, conversions and
        // barriers as in the loop below) and is done.
        if (nh == 0) {
            for (int t = 0; t < ntiles; ++t) {
            // stage of tile t+1 landed (tile t+2 may still be in flight); after the barrier every wave's share of it
            // is in LDS, every wave has converted its share of tile t, and every wave is done with tile t-1
            if (t + 2 < ntiles)
                wait_vmcnt<NLW8>();
            else
                wait_vmcnt<0>();
            __syncthreads();
            if (t + 1 < ntiles) convert_stage(stg_conv, buf ^ 1);
            stg_conv = (stg_conv == 2) ? 0 : stg_conv + 1;
            // (the stage that held tile t was converted before the barrier: free for tile t+3)
            if constexpr (PG) {
                if (t + 3 < ntiles) issue_tile_pg(c0 + (t + 3) * kTile, rows_ahead, buf_next);
                if (t + 4 < ntiles) rows_ahead = lookup_rows(c0 + (t + 4) * kTile);
            } else {
            if (t + 3 < ntiles) {
                const int tk = c0 + (t + 3) * kTile;
                const RowRef r0 = row_in_page(p, start, tk, page_ahead);
                issue_tile(tk, r0, tk + 16 < c1 ? row_in_page(p, start, tk + 16, page_ahead1) : r0, buf_next);
            }
            if (t + 4 < ntiles) {
                const int tk = c0 + (t + 4) * kTile;
                page_ahead = page_of(p, b, tk);
                if (tk + 16 < c1) page_ahead1 = page_of(p, b, tk + 16);
            }
            }
                buf = (buf == NTB - 1) ? 0 : buf + 1;
                buf_next = (buf_next == kNBuf - 1) ? 0 : buf_next + 1;
            }
            return;
        }
    }
    for (int t = 0; t < ntiles; ++t) {
        if constexpr (KV8) {
            // stage of tile t+1 landed (tile t+2 may still be in flight); after the barrier every wave's share of it
            // is in LDS, every wave has converted its share of tile t, and every wave is done with tile t-1
            if (t + 2 < ntiles)
                wait_vmcnt<NLW8>();
            else
                wait_vmcnt<0>();
            __syncthreads();
            if (t + 1 < ntiles) convert_stage(stg_conv, buf ^ 1);
            stg_conv = (stg_conv == 2) ? 0 : stg_conv + 1;
            // (the stage that held tile t was converted before the barrier: free for tile t+3)
            if constexpr (PG) {
                if (t + 3 < ntiles) issue_tile_pg(c0 + (t + 3) * kTile, rows_ahead, buf_next);
                if (t + 4 < ntiles) rows_ahead = lookup_rows(c0 + (t + 4) * kTile);
            } else {
            if (t + 3 < ntiles) {
                const int tk = c0 + (t + 3) * kTile;
                const RowRef r0 = row_in_page(p, start, tk, page_ahead);
                issue_tile(tk, r0, tk + 16 < c1 ? row_in_page(p, start, tk + 16, page_ahead1) : r0, buf_next);
            }
            if (t + 4 < ntiles) {
                const int tk = c0 + (t + 4) * kTile;
                page_ahead = page_of(p, b, tk);
                if (tk + 16 < c1) page_ahead1 = page_of(p, b, tk + 16);
            }
            }
        } else {
        if (AHEAD > 1 && t + 1 < ntiles)
            wait_vmcnt<NLW>();  // tile t landed; tile t+1 may still be in flight
        else
            wait_vmcnt<0>();
        __syncthreads();  // every wave's share of tile t is in LDS, and every wave is done with tile t-1
        if constexpr (PG) {
            if (t + AHEAD < ntiles) issue_tile_pg(c0 + (t + AHEAD) * kTile, rows_ahead, buf_next);
            if (t + AHEAD + 1 < ntiles) rows_ahead = lookup_rows(c0 + (t + AHEAD + 1) * kTile);
        } else {
        if (t + AHEAD < ntiles) {
            const int tk = c0 + (t + AHEAD) * kTile;
            const RowRef r0 = row_in_page(p, start, tk, page_ahead);
            issue_tile(tk, r0, tk + 16 < c1 ? row_in_page(p, start, tk + 16, page_ahead1) : r0, buf_next);
        }
        if (t + AHEAD + 1 < ntiles) {
            const int tk = c0 + (t + AHEAD + 1) * kTile;
            page_ahead = page_of(p, b, tk);
            if (tk + 16 < c1) page_ahead1 = page_of(p, b, tk + 16);
        }
        }
        }

        const int tok0 = c0 + t * kTile;
        // tile base addresses, made opaque so that the constant offsets below stay in the instructions'
        // offset fields instead of being folded into per-read address arithmetic
        const uint32_t ta = base_a + buf * BUF, tb = base_b + buf * BUF, tv = base_v + buf * BUF;
        uint32_t kaddr[8], kaddr_b[4];
#pragma unroll
        for (int j = 0; j < 8; ++j) kaddr[j] = ta ^ (32 * j);
#pragma unroll
        for (int j = 0; j < 4; ++j) kaddr_b[j] = tb ^ (32 * j);
        buf = (buf == NTB - 1) ? 0 : buf + 1;
        buf_next = (buf_next == (KV8 ? kNBuf : NB) - 1) ? 0 : buf_next + 1;  // (NB 16-bit buffers, or three FP8 stages)

        // S^T = K_tile . Q^T : rows = tokens, columns = heads.  K fragments are read kKPD steps ahead.
        f32x16 s;
        {
            constexpr int KPD = kKPD;
            vec8 kf[KPD];
            static_for<0, KPD>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                lds_read_b128<(i >> 3) * 256>(kf[i], kaddr[i & 7]);
            });
            static_for<0, KS>([&](auto ic) {
                constexpr int ks = decltype(ic)::value;
                constexpr int left = KS - 1 - ks;  // reads issued after the one this step consumes
                wait_lgkm<(left < KPD - 1 ? left : KPD - 1)>(kf[ks % KPD]);
                if constexpr (ks == 0)
                    MM::mma_v0(kf[ks % KPD], qf[ks], s);
                else
                    MM::mma_v(kf[ks % KPD], qf[ks], s);
                if constexpr (ks + KPD < 32)
                    lds_read_b128<((ks + KPD) >> 3) * 256>(kf[ks % KPD], kaddr[(ks + KPD) & 7]);
                else if constexpr (ks + KPD < KS)
                    lds_read_b128<0>(kf[ks % KPD], kaddr_b[ks + KPD - 32]);
            });
            // the compiler does not see the matrix instructions inside the assembly: cover the
            // result latency of the last one before anything reads the scores (the scores pass
            // through this statement, so no reader can be scheduled ahead of it)
            asm volatile("s_nop 15\n\ts_nop 7" : "+v"(s));
        }

        // online softmax for head n over this lane's 16 tokens; token of register r: tok0 + (r/4)*8 + half*4 + r%4
        float pv[16];
        float mx = -INFINITY;
        const bool tail = tok0 + kTile > c1;
        if (p.is_alibi || tail) {
            const float b0 = bias0 + slope * (float)tok0;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int off = (r >> 2) * 8 + (r & 3);
                const float x = s[r] * sl + (b0 + slope * (float)off);
                pv[r] = (tok0 + half * 4 + off) < c1 ? x : -INFINITY;
                mx = fmaxf(mx, pv[r]);
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                pv[r] = s[r] * sl;
                mx = fmaxf(mx, pv[r]);
            }
        }
        mx = max_xor32(mx);
        const bool up = mx > m + kLazy;
        if (__any(up)) {
            const float mn = up ? mx : m;
            const float alpha = fast_exp2(m - mn);
            m = mn;
            l *= alpha;
#pragma unroll
            for (int c = 0; c < CT; ++c)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float x = acc[c][r];
                    scale_acc(x, alpha);
                    acc[c][r] = x;
                }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            pv[r] = as_second_operand<Tag>(fast_exp2(pv[r] - m));
            l += pv[r];
        }
        vec8 pf[2];
        pf[0] = MM::pack8(pv);
        pf[1] = MM::pack8(pv + 8);

        // O^T += V_tile^T . P^T : rows = value columns, columns = heads.  V fragment pairs are read kVPD steps ahead.
        {
            constexpr int VPD = kVPD;
            constexpr int NV = CT * 2;  // (column tile, k-step) pairs, column tile major
            static_assert(2 * (VPD - 1) <= 15, "lgkmcnt is a 4-bit counter");
            s16x4 vlo[VPD], vhi[VPD];
            static_for<0, VPD>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                constexpr int c = i >> 1, s2 = i & 1;
                lds_read_tr16_b64<s2 * 16 * ROW_A>(vlo[i], tv ^ (64 * c));
                lds_read_tr16_b64<s2 * 16 * ROW_A + 8 * ROW_A>(vhi[i], tv ^ (64 * c + 32));
            });
            static_for<0, NV>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                constexpr int left = NV - 1 - i;
                wait_lgkm<2 * (left < VPD - 1 ? left : VPD - 1)>(vlo[i % VPD], vhi[i % VPD]);
                const s16x8 both = __builtin_shufflevector(vlo[i % VPD], vhi[i % VPD], 0, 1, 2, 3, 4, 5, 6, 7);
                acc[i >> 1] = MM::mma(__builtin_bit_cast(vec8, both), pf[i & 1], acc[i >> 1]);
                if constexpr (i + VPD < NV) {
                    constexpr int c = (i + VPD) >> 1, s2 = (i + VPD) & 1;
                    lds_read_tr16_b64<s2 * 16 * ROW_A>(vlo[i % VPD], tv ^ (64 * c));
                    lds_read_tr16_b64<s2 * 16 * ROW_A + 8 * ROW_A>(vhi[i % VPD], tv ^ (64 * c + 32));
                }
            });
        }
    }

    // finish: the two half-waves hold partial denominators over disjoint tokens
    const float l_tot = l + __shfl_xor(l, 32);
    if (n < nh) {
        const int h = h_base + n;
        if (p.nsplit == 1) {
            const float inv = vs / l_tot;
            uint16_t* orow = o16 + ((size_t)b * p.head_q + h) * DV;
#pragma unroll
            for (int c = 0; c < CT; ++c)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int col = c * 32 + r4 * 8 + half * 4;
                    ushort4 w;
                    w.x = EL::from_f32(acc[c][r4 * 4 + 0] * inv);
                    w.y = EL::from_f32(acc[c][r4 * 4 + 1] * inv);
                    w.z = EL::from_f32(acc[c][r4 * 4 + 2] * inv);
                    w.w = EL::from_f32(acc[c][r4 * 4 + 3] * inv);
                    *reinterpret_cast<ushort4*>(orow + col) = w;
                }
        } else if (p.nat_partials) {
            // normalised 16-bit values in the order the lanes hold them, the row's (m, l) behind them (nat_block)
            const float inv = vs / l_tot;
            uint8_t* const rec = reinterpret_cast<uint8_t*>(p.ws_o) +
                                 nat_block((size_t)b, p.nsplit, split, nat_blocks(p.head_k, p.groups, NWV),
                                           (hk * p.groups + grp) * NWV + wave) * 8;
            typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
            for (int c = 0; c < CT; ++c)
#pragma unroll
                for (int rp = 0; rp < 2; ++rp) {
                    u32x4 w;
                    w.x = EL::pack2(acc[c][rp * 8 + 0] * inv, acc[c][rp * 8 + 1] * inv);
                    w.y = EL::pack2(acc[c][rp * 8 + 2] * inv, acc[c][rp * 8 + 3] * inv);
                    w.z = EL::pack2(acc[c][rp * 8 + 4] * inv, acc[c][rp * 8 + 5] * inv);
                    w.w = EL::pack2(acc[c][rp * 8 + 6] * inv, acc[c][rp * 8 + 7] * inv);
                    *reinterpret_cast<u32x4*>(rec + (c * 2 + rp) * 1024 + lane * 16) = w;
                }
            if (half == 0) reinterpret_cast<float2*>(rec)[nat_ml(n)] = make_float2(m, l_tot);
        } else {
            const size_t part = ((size_t)b * p.head_q + h) * p.nsplit + split;
            float* wrow = p.ws_o + part * DV;
#pragma unroll
            for (int c = 0; c < CT; ++c)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int col = c * 32 + r4 * 8 + half * 4;
                    float4 w = make_float4(acc[c][r4 * 4 + 0] * vs, acc[c][r4 * 4 + 1] * vs, acc[c][r4 * 4 + 2] * vs,
                                           acc[c][r4 * 4 + 3] * vs);
                    *reinterpret_cast<float4*>(wrow + col) = w;
                }
            if (half == 0) {
                p.ws_ml[part * 2 + 0] = m;
                p.ws_ml[part * 2 + 1] = l_tot;
            }
        }
    }
}

// kNBuf tile buffers (FP8: two of them and three stages of raw bytes); the prologue stages each wave's Q block in a
// buffer of its own.
template <int D, int DV, int NWV, int KV8, int NB, bool VD>
constexpr size_t lds_bytes() {
    constexpr size_t buf = (size_t)kTile * D * 2;
    constexpr size_t stg = (size_t)((kTile * D / 1024 + NWV - 1) / NWV) * NWV * 1024;
    constexpr size_t tiles = KV8 ? 2 * buf + 3 * stg : (size_t)NB * (buf + (VD ? (size_t)kTile * DV * 2 : 0));
    constexpr size_t qstage = (size_t)NWV * buf;
    return tiles > qstage ? tiles : qstage;
}

template <typename Tag, int D, int DV, int NWV, int KV8, bool PG, int NB, bool VD = false>
hipError_t launch_form(const SweepParams& p, dim3 grid, hipStream_t stream) {
    auto kern = mfma_latent_kernel<Tag, D, DV, NWV, KV8, PG, NB, VD>;
    static std::atomic<uint64_t> devices_done{0};
    constexpr size_t lds = lds_bytes<D, DV, NWV, KV8, NB, VD>();
    static_assert(lds <= 160 * 1024, "LDS of one CU");
    const hipError_t attr_err = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds, devices_done);
    if (attr_err != hipSuccess) return attr_err;
    hipLaunchKernelGGL(kern, grid, dim3(64 * NWV), lds, stream, p);
    return hipGetLastError();
}

template <typename Tag, int D, int DV, int NWV, int KV8>
hipError_t launch_one(const SweepParams& p, dim3 grid, hipStream_t stream) {
    const bool pg = p.block_table != nullptr && p.page_shift < 4;
    if constexpr (NWV <= 2 && KV8 == 0) {
        // more work-groups than CUs: the two-buffer form, two work-groups to a CU
        if ((long long)grid.x * grid.y * grid.z > mla_two_per_cu_from()) {
            if (pg) return launch_form<Tag, D, DV, NWV, KV8, true, 2>(p, grid, stream);
            return launch_form<Tag, D, DV, NWV, KV8, false, 2>(p, grid, stream);
        }
    }
    if (pg) return launch_form<Tag, D, DV, NWV, KV8, true, kNBuf>(p, grid, stream);
    return launch_form<Tag, D, DV, NWV, KV8, false, kNBuf>(p, grid, stream);
}

template <typename Tag, int KV8>
hipError_t launch_tag(const SweepParams& p, int rt, dim3 grid, hipStream_t stream) {
    switch (rt) {
        case 32: return launch_one<Tag, 576, 512, 1, KV8>(p, grid, stream);
        case 64: return launch_one<Tag, 576, 512, 2, KV8>(p, grid, stream);
        case 128:
            // 16-bit K: the software-pipelined kernel (da_mla_pipe.hip); this kernel's four-wave form serves 8-bit K
            if constexpr (KV8 == 0) {
                return launch_mla_pipe(p, std::is_same<Tag, bf16_tag>::value, grid, stream);
            } else {
                // (the pipelined kernel's 8-bit form where the live heads fill a work-group's second pair of waves and
                // the layout suits it; this kernel's four-wave form otherwise)
                if (p.ratio > 64 && mla_pipe_kv8_supported(p) && !mla_pipe_kv8_off())
                    return launch_mla_pipe_kv8(p, KV8, std::is_same<Tag, bf16_tag>::value, grid, stream);
                return launch_one<Tag, 576, 512, 4, KV8>(p, grid, stream);
            }
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

bool mla_pipe_kv8_off() {
    static const bool v = [] {
        const char* s = getenv("DA_MLA_PIPE_KV8");
        return s && *s && atoi(s) == 0;
    }();
    return v;
}

int mla_two_per_cu_from() {
    static const int v = [] {
        const char* s = getenv("DA_MLA_TWO_PER_CU_FROM");
        return s && *s ? atoi(s) : 256;
    }();
    return v;
}

bool mla_supported(size_t dim, size_t dim_v, int ratio) { return dim == 576 && dim_v == 512 && ratio >= 1; }

int mla_heads_per_group(int ratio) { return ratio <= 32 ? 32 : (ratio <= 64 ? 64 : 128); }

int mla_rows_per_trip() { return kTile; }

hipError_t launch_mla(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream) {
    return is_bf16 ? launch_tag<bf16_tag, 0>(p, rt, grid, stream) : launch_tag<f16_tag, 0>(p, rt, grid, stream);
}

hipError_t launch_mla_vd(const SweepParams& p, bool is_bf16, int rt, dim3 grid, hipStream_t stream) {
    if (p.block_table != nullptr && p.page_shift < 4) return hipErrorInvalidValue;  // (tiles come as runs of 16 tokens)
    switch (rt) {
        case 32:
            return is_bf16 ? launch_form<bf16_tag, 576, 512, 1, 0, false, 2, true>(p, grid, stream)
                           : launch_form<f16_tag, 576, 512, 1, 0, false, 2, true>(p, grid, stream);
        case 64:
            return is_bf16 ? launch_form<bf16_tag, 576, 512, 2, 0, false, 2, true>(p, grid, stream)
                           : launch_form<f16_tag, 576, 512, 2, 0, false, 2, true>(p, grid, stream);
        case 128:
            return is_bf16 ? launch_form<bf16_tag, 576, 512, 4, 0, false, 2, true>(p, grid, stream)
                           : launch_form<f16_tag, 576, 512, 4, 0, false, 2, true>(p, grid, stream);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_mla_kv8(const SweepParams& p, int fmt, bool is_bf16, int rt, dim3 grid, hipStream_t stream) {
    if (fmt == kKvInt8)
        return is_bf16 ? launch_tag<bf16_tag, kKvInt8>(p, rt, grid, stream)
                       : launch_tag<f16_tag, kKvInt8>(p, rt, grid, stream);
    return is_bf16 ? launch_tag<bf16_tag, kKvFp8>(p, rt, grid, stream) : launch_tag<f16_tag, kKvFp8>(p, rt, grid, stream);
}

}  // namespace da
