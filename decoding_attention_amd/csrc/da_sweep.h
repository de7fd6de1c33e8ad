// Single-query attention as a bandwidth-bound sweep over K and V (wave64, gfx950).
//
// One work-group of four wavefronts serves one (sequence, KV head, query-head group, sequence
// split).  The RT query heads of the group sit in registers as packed 16-bit pairs and are
// shared by every K row that is streamed, so a GQA/MQA group reads its K/V once.
//
// Lane layout: G adjacent lanes cooperate on one K (or V) row, each lane owning the 16-byte
// chunks  g, g+G, g+2G, ...  of the row, so one load instruction covers 64/G rows with
// G*16 contiguous bytes per row.  Each row slot (lane / G) keeps its own online-softmax
// state (running maximum, denominator, un-normalised output) for the rows it has seen; the
// states are merged once at the end (lane shuffles inside a wave, LDS across the four waves),
// which keeps the streaming loop free of cross-lane traffic apart from the G-lane dot-product
// butterfly.
//
// The work-group either finishes the row (nsplit == 1: divide, round to nearest even, store)
// or writes an fp32 partial (un-normalised output, maximum, denominator) for the merge kernel.
//
// Follows the mathematics of the reference kernel (csrc/kernel/decoding_attn/
// decoding_fwd_kernel.h:50-235) and its index rules (block_info.h:14-30), not its structure:
// the reference keeps the whole score row in shared memory and streams K and V once per query
// head.
#pragma once
#include "da_common.h"

namespace da {

// KV8: K and V hold 8-bit elements (1 = FP8 e4m3, 2 = int8), converted exactly to the compute type as they are
// loaded; 0 = 16-bit K/V.
template <typename Tag, int D, int DV, int G, int RT, int U, int KV8 = 0>
__global__ __launch_bounds__(256) void sweep_kernel(const SweepParams p) {
    static_assert(D % (8 * G) == 0 && DV % (8 * G) == 0, "row must split into 16-byte chunks over G lanes");
    constexpr int CPL = D / 8 / G;    // K chunks per lane
    constexpr int CPLV = DV / 8 / G;  // V chunks per lane
    constexpr int E = CPLV * 8;       // output columns per lane
    constexpr int RPI = kWave / G;    // rows per load instruction
    constexpr int NW = 4;             // waves per work-group
    constexpr int TILE = RPI * U;     // rows per wave iteration
    constexpr int KB = KV8 ? 1 : 2;   // bytes per K/V element
    using EL = Elem<Tag>;

    __shared__ float lds_acc[NW][RT][DV];
    __shared__ float lds_ml[NW][RT][2];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int g = lane % G;
    const int slot = lane / G;

    const int split = blockIdx.x;
    const int hk = blockIdx.y / p.groups;
    const int grp = blockIdx.y % p.groups;
    const int b = blockIdx.z;

    int start, len;
    seq_range(p, b, start, len);
    const int c0 = split * p.chunk;
    const int c1 = (split == p.nsplit - 1) ? len : min(len, c0 + p.chunk);

    const int h_base = hk * p.ratio + grp * RT;
    const int nh = min(RT, p.ratio - grp * RT);  // live heads of this group

    if (c0 >= c1) {
        // Nothing to read.  An empty sequence still owns output rows (the merge kernel writes them
        // when the sequence is split).
        if (p.nsplit == 1) zero_rows<DV>(p, b, h_base, nh, 1, 0);
        return;
    }

    // Query heads of the group, as packed pairs, at this lane's chunk positions.
    uint4 qreg[RT][CPL];
    float slope[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        const int h = h_base + min(r, nh - 1);
        const uint16_t* qrow = reinterpret_cast<const uint16_t*>(p.q) + ((size_t)b * p.head_q + h) * D;
#pragma unroll
        for (int c = 0; c < CPL; ++c) qreg[r][c] = *reinterpret_cast<const uint4*>(qrow + (c * G + g) * 8);
        slope[r] = p.is_alibi ? alibi_slope_log2(p.slopes, h, p.head_q) : 0.0f;
    }

    float m[RT], l[RT], acc[RT][E];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        m[r] = kNegBig;
        l[r] = 0.0f;
#pragma unroll
        for (int e = 0; e < E; ++e) acc[r][e] = 0.0f;
    }

    // rows are addressed one by one (row_ref), so paged K/V of any page size costs one table lookup per row
    const uint8_t* kbase = reinterpret_cast<const uint8_t*>(p.k) + ((size_t)hk * D + g * 8) * KB;
    const uint8_t* vbase = reinterpret_cast<const uint8_t*>(p.v) + ((size_t)hk * p.v_head + g * 8) * KB;
    // (an int4 cache's elements come out of the conversion times a power of two, divided out here)
    const float sl = p.scale_log2 * head_scale(p.k_scale, hk) * kv_widening_inverse<KV8>();  // score scale, log2 units
    const float vs = head_scale(p.v_scale, hk) * kv_widening_inverse<KV8>();
    auto load8 = [](const uint8_t* ptr) __attribute__((always_inline)) {  // eight elements as 16-bit pairs
        if constexpr (KV8 == kKvInt4)
            return kv8x8_to_16<Tag, KV8>(kv4_load8(ptr));  // (four bytes from half the address)
        else if constexpr (KV8)
            return kv8x8_to_16<Tag, KV8>(*reinterpret_cast<const uint2*>(ptr));  // (8-byte loads run slower with the non-temporal hint: MHA batch 512 x 128 tokens, FP8, 105 -> 131 us)
        else if constexpr ((D * 2) % 128 != 0)  // (d = 96: neighbouring heads' rows share a 128-byte line, which the
            return *reinterpret_cast<const uint4*>(ptr);  // hint would drop between their reads: MHA batch 8 x 4096
        else                                             // tokens 113.0 us with it, 93.9 without)
            return stream_load16(ptr);
    };

    const int ntiles = (c1 - c0 + TILE - 1) / TILE;
    for (int t = wave; t < ntiles; t += NW) {
        const int base = c0 + t * TILE + slot;
        uint4 kreg[U][CPL];
        uint4 vreg[U][CPLV];
        RowRef rr[U];
#pragma unroll
        for (int u = 0; u < U; ++u)  // rows past the end re-read the last row and are masked
            rr[u] = row_ref(p, b, start, min(base + u * RPI, c1 - 1));
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint8_t* kr = kbase + rr[u].k * KB;
#pragma unroll
            for (int c = 0; c < CPL; ++c) kreg[u][c] = load8(kr + c * G * 8 * KB);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint8_t* vr = vbase + rr[u].v * KB;
#pragma unroll
            for (int c = 0; c < CPLV; ++c) vreg[u][c] = load8(vr + c * G * 8 * KB);
        }

        // scores in log2 units
        float s[U][RT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = base + u * RPI;
#pragma unroll
            for (int r = 0; r < RT; ++r) {
                float d = 0.0f;
#pragma unroll
                for (int c = 0; c < CPL; ++c) {
                    d = EL::dot2(qreg[r][c].x, kreg[u][c].x, d);
                    d = EL::dot2(qreg[r][c].y, kreg[u][c].y, d);
                    d = EL::dot2(qreg[r][c].z, kreg[u][c].z, d);
                    d = EL::dot2(qreg[r][c].w, kreg[u][c].w, d);
                }
                d = group_sum<G>(d);
                d = d * sl + slope[r] * (float)(j - (len - 1));
                s[u][r] = (j < c1) ? d : -INFINITY;
            }
        }

        // online softmax, one rescale per tile
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            float mn = m[r];
#pragma unroll
            for (int u = 0; u < U; ++u) mn = fmaxf(mn, s[u][r]);
            const float alpha = fast_exp2(m[r] - mn);
            m[r] = mn;
            l[r] *= alpha;
#pragma unroll
            for (int e = 0; e < E; ++e) acc[r][e] *= alpha;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                s[u][r] = fast_exp2(s[u][r] - mn);
                l[r] += s[u][r];
            }
        }

        // O += P V
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int c = 0; c < CPLV; ++c) {
                float vf[8];
                vf[0] = EL::lo(vreg[u][c].x);
                vf[1] = EL::hi(vreg[u][c].x);
                vf[2] = EL::lo(vreg[u][c].y);
                vf[3] = EL::hi(vreg[u][c].y);
                vf[4] = EL::lo(vreg[u][c].z);
                vf[5] = EL::hi(vreg[u][c].z);
                vf[6] = EL::lo(vreg[u][c].w);
                vf[7] = EL::hi(vreg[u][c].w);
#pragma unroll
                for (int r = 0; r < RT; ++r) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[r][c * 8 + e] += s[u][r] * vf[e];
                }
            }
        }
    }

    // Merge the row slots of this wave (lanes that own the same columns).
#pragma unroll
    for (int off = G; off < kWave; off <<= 1) {
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const float mo = __shfl_xor(m[r], off);
            const float lo = __shfl_xor(l[r], off);
            const float mn = fmaxf(m[r], mo);
            const float wa = fast_exp2(m[r] - mn);
            const float wb = fast_exp2(mo - mn);
            m[r] = mn;
            l[r] = l[r] * wa + lo * wb;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                const float ao = __shfl_xor(acc[r][e], off);
                acc[r][e] = acc[r][e] * wa + ao * wb;
            }
        }
    }

    if (slot == 0) {
#pragma unroll
        for (int r = 0; r < RT; ++r) {
#pragma unroll
            for (int c = 0; c < CPLV; ++c) {
#pragma unroll
                for (int e = 0; e < 8; ++e) lds_acc[wave][r][(c * G + g) * 8 + e] = acc[r][c * 8 + e];
            }
            if (g == 0) {
                lds_ml[wave][r][0] = m[r];
                lds_ml[wave][r][1] = l[r];
            }
        }
    }
    __syncthreads();

    // Merge the four waves in a fixed order and finish.
    for (int idx = threadIdx.x; idx < nh * DV; idx += blockDim.x) {
        const int r = idx / DV, col = idx % DV;
        float mm = lds_ml[0][r][0];
#pragma unroll
        for (int w = 1; w < NW; ++w) mm = fmaxf(mm, lds_ml[w][r][0]);
        float num = 0.0f, den = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float wt = fast_exp2(lds_ml[w][r][0] - mm);
            num += wt * lds_acc[w][r][col];
            den += wt * lds_ml[w][r][1];
        }
        const int h = h_base + r;
        if (p.nsplit == 1) {
            reinterpret_cast<uint16_t*>(p.o)[((size_t)b * p.head_q + h) * DV + col] = EL::from_f32(num * vs / den);
        } else {
            const size_t part = ((size_t)b * p.head_q + h) * p.nsplit + split;
            p.ws_o[part * DV + col] = num * vs;
            if (col == 0) {
                p.ws_ml[part * 2 + 0] = mm;
                p.ws_ml[part * 2 + 1] = den;
            }
        }
    }
}

// Second pass: merge the per-split partials in split order.  One thread per (sequence, query head, group of four
// output columns); the partials of four splits are fetched together so that their latencies overlap, and the maxima
// are folded in on the way (running maximum, as in the sweeps), so there is no pass over them in front.
// SG > 1 (many splits of few rows: one long sequence): SG lanes share one (row, four columns), lane j of them
// taking splits j, j + SG, ...; a wave covers 64 / SG column groups of one row, and the SG partial sums meet through
// lane exchanges.  The order of summation then differs from SG = 1, not the result's accuracy.
// H16: the partial outputs are normalised 16-bit values (ReduceParams::half_partials); a partial's weight then
// carries its denominator.
template <typename Tag, int SG, bool H16 = false>
__global__ __launch_bounds__(256) void reduce_kernel(const ReduceParams p, int rows) {
    using EL = Elem<Tag>;
    const int nc4 = p.dim_v >> 2;
    int row, c4, sgi = 0;
    size_t nat_b = 0;     // (H16) sequence,
    int nat_blk = 0, nat_n = 0;  // block and row within it
    if constexpr (H16) {
        // (SG > 1 only) the CW = 64 / SG elements of a wave are CW consecutive rows of one block at one column group:
        // consecutive 8-byte pieces of the partials
        static_assert(SG > 1 && 32 % (64 / SG) == 0, "the one-lane-per-element form is reduce16_kernel");
        constexpr int CW = 64 / SG;
        const int wave_id = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
        const long long id = (long long)wave_id * CW + (lane % CW);
        sgi = lane / CW;
        nat_n = (int)(id & 31);
        const long long rest = id >> 5;
        c4 = (int)(rest % nc4);
        const long long bg = rest / nc4;  // sequence * blocks + block
        if (bg >= (long long)(rows / p.head_q) * p.nat_blocks) return;  // (a whole wave: its elements share bg)
        nat_b = (size_t)(bg / p.nat_blocks);
        nat_blk = (int)(bg % p.nat_blocks);
        const int per_kv = p.groups * p.nat_waves;
        const int r = (nat_blk % per_kv) * 32 + nat_n;  // head within its KV head's group of `ratio`
        if (r >= p.ratio) return;                       // (the SG lanes of an element leave together)
        row = (int)nat_b * p.head_q + (nat_blk / per_kv) * p.ratio + r;
    } else if constexpr (SG == 1) {
        const int gid = blockIdx.x * 256 + threadIdx.x;
        row = gid / nc4;  // (sequence, head) index
        c4 = gid - row * nc4;
    } else {
        constexpr int CW = 64 / SG;  // column groups per wave
        const int wave_id = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
        const int waves_per_row = nc4 / CW;
        row = wave_id / waves_per_row;
        c4 = (wave_id - row * waves_per_row) * CW + (lane % CW);
        sgi = lane / CW;
    }
    if (row >= rows) return;  // (whole waves leave together when SG > 1)
    // partial s of this row sits in workspace row part0 + s * pstride (fixed splits: the row's own nsplit slots;
    // balanced grid: slot first share + sequence + s of the batch, see flat_slots, known once the positions are read)
    size_t part0 = (size_t)row * p.nsplit;
    size_t pstride = 1;
    const float2* ml = reinterpret_cast<const float2*>(p.ws_ml) + part0;
    const float4* src = reinterpret_cast<const float4*>(p.ws_o + part0 * p.dim_v) + c4;
    const uint2* const src16 = reinterpret_cast<const uint2*>(p.ws_o);  // (H16) the block records
    // This lane's next four partials: slots s0, s0 + SG, ... (clamped to `last`; the caller masks the rest).
    float2 e[4];
    float4 x[4];
    auto fetch = [&](int s0, int last) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int s = min(s0 + u * SG, last);
            if constexpr (H16) {
                const uint2* const rec = src16 + nat_block(nat_b, p.nsplit, s, p.nat_blocks, nat_blk);
                e[u] = reinterpret_cast<const float2*>(rec)[nat_ml(nat_n)];
                const uint2 h = rec[nat_piece(c4, nat_n)];
                x[u] = make_float4(EL::lo(h.x), EL::hi(h.x), EL::lo(h.y), EL::hi(h.y));
            } else {
                e[u] = ml[(size_t)s * pstride];
                x[u] = src[(size_t)s * pstride * nc4];
            }
        }
    };
    // A small workspace (p.early): the first four are requested before the sequence's length is known, so that
    // their trip to memory overlaps the one for the length; slots past the sequence's last split hold stale data
    // and are masked below.
    if (p.early) fetch(sgi, p.nsplit - 1);
    const int b = row / p.head_q;
    const int len = p.cu_seq_k ? p.cu_seq_k[b + 1] - p.cu_seq_k[b] : p.seq_lens[b];
    int ns = 0;
    if (p.flat_wgs > 0) {
        // balanced sweep grid: the sequence's partials come from the work-groups its tokens fall into; a sequence
        // inside one work-group was written to o by the sweep itself
        if (len > 0) {
            const int lo = p.flat_cu[b], hi = p.flat_cu[b + 1];
            const int T = flat_share(p.flat_cu[p.batch], p.flat_wgs, p.flat_step, p.flat_min);
            const int first = min(lo / T, p.flat_wgs - 1);
            ns = min((hi - 1) / T, p.flat_wgs - 1) - first + 1;
            if (ns == 1) return;
            part0 = (size_t)(first + b) * p.head_q + (size_t)(row - b * p.head_q);
            pstride = (size_t)p.head_q;
            ml = reinterpret_cast<const float2*>(p.ws_ml) + part0;
            src = reinterpret_cast<const float4*>(p.ws_o + part0 * p.dim_v) + c4;
        }
    } else if (len > 0) {
        ns = min(p.nsplit, (len + p.chunk - 1) / p.chunk);
    }
    // One pass with a running maximum (the sum is rescaled when a later partial raises it).
    float mm = kNegBig;
    float4 num = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    float den = 0.0f;
    for (int s0 = sgi; s0 < ns; s0 += 4 * SG) {
        if (!p.early || s0 != sgi) fetch(s0, ns - 1);
        float m_new = mm;
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (s0 + u * SG < ns) m_new = fmaxf(m_new, e[u].x);
        const float keep = fast_exp2(mm - m_new);  // 0 on the first round
        mm = m_new;
        den *= keep;
        num.x *= keep;
        num.y *= keep;
        num.z *= keep;
        num.w *= keep;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const bool valid = s0 + u * SG < ns;
            float w = valid ? fast_exp2(e[u].x - mm) : 0.0f;
            if constexpr (H16) w = valid ? w * e[u].y : 0.0f;  // normalised partial: weight x denominator
            den += valid ? (H16 ? w : w * e[u].y) : 0.0f;
            num.x += valid ? w * x[u].x : 0.0f;
            num.y += valid ? w * x[u].y : 0.0f;
            num.z += valid ? w * x[u].z : 0.0f;
            num.w += valid ? w * x[u].w : 0.0f;
        }
    }
    if constexpr (SG > 1) {
        // the SG lanes of an element bring their sums to a common maximum first
        float m_all = mm;
#pragma unroll
        for (int d = 64 / SG; d < 64; d <<= 1) m_all = fmaxf(m_all, __shfl_xor(m_all, d));
        const float keep = fast_exp2(mm - m_all);
        den *= keep;
        num.x *= keep;
        num.y *= keep;
        num.z *= keep;
        num.w *= keep;
    }
    if constexpr (SG > 1) {
#pragma unroll
        for (int d = 64 / SG; d < 64; d <<= 1) {
            den += __shfl_xor(den, d);
            num.x += __shfl_xor(num.x, d);
            num.y += __shfl_xor(num.y, d);
            num.z += __shfl_xor(num.z, d);
            num.w += __shfl_xor(num.w, d);
        }
        if (sgi != 0) return;
    }
    const float inv = ns > 0 ? 1.0f / den : 0.0f;  // an empty sequence yields a zero row
    ushort4 r;
    r.x = EL::from_f32(num.x * inv);
    r.y = EL::from_f32(num.y * inv);
    r.z = EL::from_f32(num.z * inv);
    r.w = EL::from_f32(num.w * inv);
    *reinterpret_cast<ushort4*>(reinterpret_cast<uint16_t*>(p.o) + (size_t)row * p.dim_v + c4 * 4) = r;
}

// The merge for normalised 16-bit partials (ReduceParams::half_partials, laid out as nat_piece says) in its
// one-lane-per-element form.  Grid: x = sequence, y = 8 * (block of 32 heads within its KV head) + group of four runs,
// z = KV head; thread (run, lane) takes the 16 bytes that lane of the sweep stored in that run of the block's record --
// two groups of four columns of one head -- so a wave's loads are the run's contiguous KiB, one load per split.  With
// eight waves to a SIMD at the benchmark's latent shape the kernel's time is its vector-instruction count (the first
// version, with 600 of them, mostly index arithmetic, took 11 us for 44 MB): everything the work-group shares (record
// addresses, the sequence's length, which splits exist) is scalar, and a value costs one mixed-precision multiply-add.
// The first four splits are requested before the sequence's length is known (slots past the last split hold stale
// data and are skipped).  A partial's weight is 2^(m_i - m) times its denominator l_i.  A work-group covers four runs,
// i.e. 64 columns of the block's 32 rows: its results change hands through LDS so that each row's 128 bytes leave as
// one run.
constexpr int kReduce16Runs = 1;  // runs of a block record per thread (two: no faster, measured)
template <typename Tag>
__global__ __launch_bounds__(256) void reduce16_kernel(const ReduceParams p) {
    using EL = Elem<Tag>;
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    constexpr int NR = kReduce16Runs, NG = 8 / NR;  // NG: groups of four runs along grid y
    __shared__ uint2 out_tile[NR][32][18];  // (a pitch of nine 16-byte units: the rows' writes spread over the banks)
    const int b = (int)blockIdx.x, bpk = (int)blockIdx.y / NG, rg = (int)blockIdx.y % NG, hk = (int)blockIdx.z;
    const int per_kv = p.groups * p.nat_waves;
    const int hr0 = bpk * 32;                   // first head of the block within its KV head's group of `ratio`
    const int live = min(32, p.ratio - hr0);    // live rows of the block
    const size_t row0 = (size_t)b * p.head_q + (size_t)hk * p.ratio + hr0;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int n = lane & 31, half = lane >> 5;  // row of the block, half-wave of the storing lane
    constexpr size_t kRec = (size_t)kNatBlockUnits * 8;
    const uint8_t* const rec0 =
        reinterpret_cast<const uint8_t*>(p.ws_o) + ((size_t)b * p.nsplit * p.nat_blocks + (size_t)(hk * per_kv + bpk)) * kRec;
    const size_t sstride = (size_t)p.nat_blocks * kRec;  // from one split's record to the next
    // this thread's runs: 4 (rg + NG i) + wv, i < NR (the work-group's i-th four runs: columns 64 (rg + NG i) .. + 63)
    const uint32_t xoff = (uint32_t)rg * 4096u + threadIdx.x * 16u;
    const uint32_t eoff = (uint32_t)(64 * 64 * 8) + (uint32_t)n * 8u;
    uint2 r[NR][2];
#pragma unroll
    for (int i = 0; i < NR; ++i) r[i][0] = r[i][1] = make_uint2(0u, 0u);
    if (n < live) {  // (else a dead row of the group's last block)
        float2 e[4];
        u32x4 x[NR][4];
        auto fetch = [&](int s0) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint8_t* const rec = rec0 + (size_t)min(s0 + u, p.nsplit - 1) * sstride;
                e[u] = *reinterpret_cast<const float2*>(rec + eoff);
                // (read once: non-temporal, like the K/V streams)
#pragma unroll
                for (int i = 0; i < NR; ++i)
                    x[i][u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(rec + xoff + i * NG * 4096));
            }
        };
        fetch(0);
        const int len = p.cu_seq_k ? p.cu_seq_k[b + 1] - p.cu_seq_k[b] : p.seq_lens[b];
        float mm = kNegBig, den = 0.0f;
        float num[NR][8];
#pragma unroll
        for (int i = 0; i < NR; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) num[i][j] = 0.0f;
        // split s exists when s < nsplit and s * chunk < len (all scalar)
        for (int s0 = 0; s0 < p.nsplit && (long long)s0 * p.chunk < len; s0 += 4) {
            if (s0 != 0) fetch(s0);
            bool valid[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) valid[u] = s0 + u < p.nsplit && (long long)(s0 + u) * p.chunk < len;
            float m_new = mm;
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (valid[u]) m_new = fmaxf(m_new, e[u].x);
            if (s0 != 0) {
                const float keep = fast_exp2(mm - m_new);
                den *= keep;
#pragma unroll
                for (int i = 0; i < NR; ++i)
#pragma unroll
                    for (int j = 0; j < 8; ++j) num[i][j] *= keep;
            }
            mm = m_new;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (!valid[u]) continue;  // (a slot past the sequence's last split holds stale data, possibly NaN)
                const float w = fast_exp2(e[u].x - mm) * e[u].y;
                den += w;
#pragma unroll
                for (int i = 0; i < NR; ++i) {
                    const uint32_t h[4] = {x[i][u].x, x[i][u].y, x[i][u].z, x[i][u].w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        num[i][2 * j] = __builtin_fmaf(w, EL::lo(h[j]), num[i][2 * j]);
                        num[i][2 * j + 1] = __builtin_fmaf(w, EL::hi(h[j]), num[i][2 * j + 1]);
                    }
                }
            }
        }
        // (the hardware reciprocal, 1 ulp: far below the 16-bit rounding that follows)
        const float inv = len > 0 ? __builtin_amdgcn_rcpf(den) : 0.0f;  // an empty sequence yields a zero row
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            r[i][0] = make_uint2(EL::pack2(num[i][0] * inv, num[i][1] * inv), EL::pack2(num[i][2] * inv, num[i][3] * inv));
            r[i][1] = make_uint2(EL::pack2(num[i][4] * inv, num[i][5] * inv), EL::pack2(num[i][6] * inv, num[i][7] * inv));
        }
    }
    // thread (wave wv, lane (n, half)) holds columns 32 (wv / 2) + 16 (wv % 2) + 4 half .. + 3 and the same + 8 of row n,
    // relative to the first column of its four runs; thread t sends off 16-byte piece t % 8 of row t / 8
    const int u0 = (wv >> 1) * 4 + (wv & 1) * 2;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        out_tile[i][n][u0 * 2 + half] = r[i][0];
        out_tile[i][n][u0 * 2 + 2 + half] = r[i][1];
    }
    __syncthreads();
    const int n2 = threadIdx.x >> 3, seg = threadIdx.x & 7;
    if (n2 < live) {
        uint16_t* const orow = reinterpret_cast<uint16_t*>(p.o) + (row0 + n2) * p.dim_v + rg * 64 + seg * 8;
#pragma unroll
        for (int i = 0; i < NR; ++i)
            *reinterpret_cast<uint4*>(orow + i * NG * 64) = *reinterpret_cast<const uint4*>(&out_tile[i][n2][seg * 2]);
    }
}

}  // namespace da
