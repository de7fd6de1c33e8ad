// C-ABI of libdecoding_attn_hip.so: argument checks, launch planning, workspace, dispatch.
//
// Stands where the reference's csrc/ops/decoding_attn.cpp does (set_dmha_fwd_params :13-62,
// run_dmha_fwd :64-68, decoding_attn :70-76): derive strides from head counts, alias V onto K
// when v is null, choose the kernel for (dtype, dim, dim_v), enqueue on the caller's stream.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <string>
#include <utility>

#include "../../include/decoding_attn_hip.h"
#ifdef DA_BUILD_PROBES
#include "decoding_attn_probe.h"
#endif
#include "da_gqa_mfma.h"
#include "da_mla.h"
#include "da_sweep_launch.h"

namespace {

thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

int env_int(const char* name, int dflt) {
    const char* s = getenv(name);
    if (!s || !*s) return dflt;
    return atoi(s);
}

// Tunables, read once.  DA_TARGET_WGS: work-groups a launch should reach before the sequence
// stops being split further; DA_MAX_CHUNK / DA_MIN_CHUNK: bounds on tokens per split.
struct Tunables {
    int target_wgs, mfma_target_wgs, max_chunk, min_chunk, ragged_chunk, force_kind, group_min_ratio, wave_per_head,
        mla_heads, gqa_heads, flat_wgs, flat_min_tokens, flat_uncounted, flat_uncounted_min, flat_paged_min_mb, nsplit, mfma_small_wgs, group_small_wgs,
        group_small_chunk, mla_group_heads, mla_group_small, fill_rounds, group_target_wgs_d128, mla_distinct_v;
    Tunables() {
        target_wgs = env_int("DA_TARGET_WGS", 512);
        mfma_target_wgs = env_int("DA_MFMA_TARGET_WGS", 256);
        max_chunk = env_int("DA_MAX_CHUNK", 1024);
        min_chunk = env_int("DA_MIN_CHUNK", 512);
        gqa_heads = env_int("DA_GQA_HEADS", 0);  // query heads per work-group and KV head of the grouped kernel (16/32), 0 = by shape
        mla_heads = env_int("DA_MLA_HEADS", 0);  // query heads per work-group of the latent kernel (32/64/128), 0 = by shape
        ragged_chunk = env_int("DA_RAGGED_CHUNK", 256);  // tokens per split when the lengths are known to be ragged
        // balanced grid of the grouped kernel for ragged batches: work-groups in all (0 = off), fewest tokens each
        flat_wgs = env_int("DA_FLAT_WGS", 512);
        flat_min_tokens = env_int("DA_FLAT_MIN_TOKENS", 256);
        // ... also for a batch whose token count the caller did not give (0 = fixed splits then), from this many
        // tokens per share at full length
        flat_uncounted = env_int("DA_FLAT_UNCOUNTED", 1);
        flat_uncounted_min = env_int("DA_FLAT_UNCOUNTED_MIN", 512);
        flat_paged_min_mb = env_int("DA_FLAT_PAGED_MIN_MB", 512);  // paged K/V takes the balanced grid from this many MB of K/V
        mfma_small_wgs = env_int("DA_MFMA_SMALL_WGS", 256);  // latent kernel: below this many 256-token splits, split finer
        // latent form: up to this many query heads take the grouped kernel (0 = never)
        mla_group_heads = env_int("DA_MLA_GROUP_HEADS", 16);
        mla_distinct_v = env_int("DA_MLA_DISTINCT_V", 1);  // (576, 512) with V in its own buffer on the latent kernel (0 = VALU sweep)
        // ... and any head count while groups x batch x max_seq_k stays within this (twice this for two groups)
        mla_group_small = env_int("DA_MLA_GROUP_SMALL", 65536);
        group_target_wgs_d128 = env_int("DA_GROUP_TARGET_WGS_D128", 256);
        fill_rounds = env_int("DA_FILL_ROUNDS", 1);  // grouped kernel: re-plan grids that fill their last round of CUs poorly
        group_small_wgs = env_int("DA_GROUP_SMALL_WGS", 256);  // grouped kernel: likewise
        group_small_chunk = env_int("DA_GROUP_SMALL_CHUNK", 64);
        nsplit = env_int("DA_NSPLIT", 0);  // sequence splits, 0 = by shape (experiments)
        force_kind = env_int("DA_FORCE_KIND", 0);
        wave_per_head = env_int("DA_WAVE_PER_HEAD", 1);
        group_min_ratio = env_int("DA_GROUP_MIN_RATIO", 2);  // smallest head group that takes the grouped MFMA sweep
    }
};
Tunables& tun_storage() {
    static Tunables t;
    return t;
}
const Tunables& tun() { return tun_storage(); }

constexpr int kKindSweep = 1;
constexpr int kKindMfma = 2;
constexpr int kKindGroup = 3;
constexpr int kMaxSplits = 256;
// most sequences of one launch (a grid axis ends at 65535; a multiple of eight, so that the kernels' renumbering of
// work-groups over the eight XCDs stays on); larger batches run as several launches
constexpr size_t kMaxGridBatch = 65528;

struct Plan {
    int kind = 0;
    int rt = 1;      // query heads per work-group
    int groups = 1;  // work-groups per KV head
    int nsplit = 1;
    int chunk = 0;
    size_t ws_bytes = 0;
    bool wave_per_head = false;  // grouped kernel: the four waves of a work-group take four KV heads
    bool v_distinct = false;     // latent kernel: the form that fetches V from a buffer of its own
    // Balanced grid (grouped kernel; a batch known to be ragged, or one whose token count the caller did not give):
    // flat_wgs work-groups per (KV heads, head group), each over an equal share of the concatenated sequences, which
    // the kernels derive from the line's length on the device (da::flat_share; a multiple of flat_step units, at
    // least flat_min).  nsplit then reports the shares along the line and chunk the share in tokens (0 when the
    // host does not know it).
    int flat_wgs = 0, flat_step = 1, flat_min = 1;
    int flat_partials = 0;  // most partials the planner expects one sequence to have
    // paged K/V: the line is measured in units of flat_unit = 32 tokens, every sequence rounded up to whole units
    // (shares then start on tile boundaries), and its positions are computed on the device by a small kernel in
    // front of the sweep, into flat_cu_bytes at the end of the workspace
    int flat_unit = 1;
    size_t flat_cu_bytes = 0;
};

bool supported_dims(size_t dim, size_t dim_v) {
    return (dim == 64 && dim_v == 64) || (dim == 96 && dim_v == 96) || (dim == 128 && dim_v == 128) ||
           (dim == 256 && dim_v == 256) || (dim == 576 && dim_v == 512);
}

int rows_per_trip(size_t dim) {
    switch (dim) {
        case 64: return da::sweep_rows_per_trip<64>();
        case 96: return da::sweep_rows_per_trip<96>();
        case 128: return da::sweep_rows_per_trip<128>();
        case 256: return da::sweep_rows_per_trip<256>();
        default: return da::sweep_rows_per_trip<576>();
    }
}

// v_distinct: V is its own buffer.  At (576, 512) the latent kernels read V out of the K tile; a distinct V takes the
// latent kernel's two-buffer form that stages the V rows beside the K tile (16-bit K/V, packed or in pages of 16 tokens
// and more; otherwise the VALU sweep).
// total_k: sum of the key lengths if the caller knows it (0 = unknown).  The planner never reads cu_seq_k (that
// would need a device synchronisation); when total_k shows that the batch is ragged it cuts the sequences into
// shorter splits so that the work-groups, whose number is sized for max_seq_k, balance.
// page_size: 0 for the packed layout, else tokens per page of paged K/V (any power of two: the MFMA kernels fetch a
// tile whole from pages of 32 tokens and more, as two runs from 16-token pages, row by row below that).
// kv_8bit: K/V are FP8, int8 or int4; the grouped kernel then needs dim % 64 == 0.
// no_latent_kernel: the cache format has no form of the latent kernel (int4): the latent form then runs on the grouped
// kernel whatever its size, as ceil(heads / 16) groups per sequence that read the same rows.
// group_only: the call has a form on the grouped kernel only (per-token quantisation factors): every shape takes it.
// 2 = a pair per 64 elements of a row: at d = 256 its 32-head form would not fit the registers, 16 heads per group.
Plan make_plan(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
               bool v_distinct, size_t total_k, size_t page_size = 0, bool kv_8bit = false,
               bool no_latent_kernel = false, int group_only = 0) {
    const bool packed = page_size == 0;
    Plan pl;
    const int ratio = (int)(head_q / head_k);
    int trip;
    int target_wgs = tun().target_wgs;
    int max_chunk_scale = 1;
    const bool force_sweep = tun().force_kind == kKindSweep;
    const bool latent_vd = v_distinct && da::mla_supported(dim, dim_v, ratio) && !kv_8bit && !force_sweep &&
                           (packed || page_size >= 16) && tun().mla_distinct_v;
    const bool latent = !v_distinct && da::mla_supported(dim, dim_v, ratio);
    // the latent form with up to 16 query heads (a tensor-parallel shard) runs on the grouped kernel, which keeps more
    // bytes in flight per CU than the latent kernel's one-wave form can (its tiles need LDS landing space)
    // (an 8-bit cache: up to twice as many, as two groups that read the same rows; the latent kernel's single
    // computing wave is the slower there: FP8, 32 heads, batch 64 x 4096 tokens 96 -> 60 us)
    // Small problems of any head count go there as well, as ceil(heads / 16) groups per sequence that read the same
    // rows: the latent kernel's work-groups pay ~6 us to stage Q before their first tile, which a few tiles do not
    // win back (measured, 128 heads: batch 1 x 8192 tokens 34.4 -> 24.8 us, batch 16 x 512 29.8 -> 23.4; 32 heads:
    // batch 1 x 16384 33.4 -> 23.0; past the bound below the re-read rows cost more than the staging).
    // (65 heads and more run on the software-pipelined latent kernel, which wins wherever the sequences are split:
    // 128 heads, batch 1 x 4096 tokens 21.4 -> 19.3 us, batch 1 x 512 16.2 -> 15.2, batch 2 x 1024 18.5 -> 16.6, batch
    // 4 x 512 18.4 -> 15.8, batch 4 x 256 17.1 -> 15.2; a single unsplit launch stays, batch 1 x 128 12.9 against 13.8)
    // (its 8-bit form serves rows of one KV head in runs of 16 tokens: the packed layout and pages of 16 tokens and more)
    const bool pipe_kernel = latent && ratio > 64 &&
                             (!kv_8bit || (head_k == 1 && (packed || page_size >= 16) && !no_latent_kernel && !da::mla_pipe_kv8_off()));
    const long long groups16 = (ratio + 15) / 16;
    const long long group_rows = groups16 * (long long)batch * (long long)max_seq_k;
    const long long small_bound =
        pipe_kernel ? (long long)tun().mla_group_small / 4 : (groups16 <= 2 ? 2 : 1) * (long long)tun().mla_group_small;
    const bool latent_small = tun().mla_group_heads > 0 && group_rows <= small_bound && (!pipe_kernel || max_seq_k < 256);
    const bool latent_group = latent && !force_sweep &&
                              (ratio <= (kv_8bit ? 2 * tun().mla_group_heads : tun().mla_group_heads) || latent_small ||
                               no_latent_kernel);
    const bool mfma = (latent && !force_sweep && !latent_group) || latent_vd;
    if (latent_group) {
        pl.kind = kKindGroup;
        pl.rt = 16;
        pl.wave_per_head = false;
        trip = 4 * da::kGqaTile;
        // one work-group (its four V tiles take 132 KB of LDS) per CU, and splits up to twice the usual length
        // (measured, 16 heads: batch 64 x 4096 tokens 73 -> 64 us with 256 work-groups instead of 512; batch 128
        // 126 -> 118 us with 2048-token splits)
        target_wgs = tun().mfma_target_wgs;
        max_chunk_scale = 2;
    } else if (mfma) {
        pl.kind = kKindMfma;
        pl.rt = da::mla_heads_per_group(ratio);
        // few sequences and short ones cannot fill the chip even at the finest split: then two work-groups of 64
        // heads per (sequence, split) beat one of 128 (measured: batch 1, seq 4096: 35 -> 31 us).  The same holds for
        // up to four long sequences (batch 1 x 65536 tokens 64.2 -> 55.7 us, batch 2 x 32768 63.7 -> 56.3, batch 4 x
        // 16384 63.5 -> 56.8; batch 8 x 8192 and larger batches lose, 53.2 -> 57.6).
        // (the compiler-scheduled four-wave form, i.e. an 8-bit cache or a distinct V: the pipelined kernel is faster
        // with 128 heads at every size; batch 8 x 4096 tokens 38.7 -> 30.0 us, batch 16 x 2048 38.9 -> 29.8, batch 4 x
        // 16384 54.4 -> 41.1, batch 32 x 1024 39.2 -> 30.3)
        const long long tiles256 = (long long)batch * (long long)(max_seq_k / 256);
        if (pl.rt == 128 && !pipe_kernel && (tiles256 <= 128 || (batch <= 4 && tiles256 <= 512))) pl.rt = 64;
        if ((tun().mla_heads == 32 || tun().mla_heads == 64 || tun().mla_heads == 128) && tun().mla_heads <= 128 &&
            tun().mla_heads >= 32)
            pl.rt = std::min(tun().mla_heads, da::mla_heads_per_group(ratio));
        // an 8-bit K cache is converted by the whole work-group: always four waves, those without heads of their
        // own only load and convert (measured, FP8, 32 heads, batch 64 x 4096 tokens: 206 us with one wave)
        if (kv_8bit) pl.rt = 128;
        pl.v_distinct = latent_vd;
        trip = da::mla_rows_per_trip();
        target_wgs = tun().mfma_target_wgs;  // one 4-wave work-group fills a CU
        // work-groups of one or two waves over 16-bit K take two tile buffers instead of three when there are more
        // of them than CUs, and then run two to a CU (not with a distinct V, whose two buffers fill the LDS)
        if (pl.rt <= 64 && !kv_8bit && !latent_vd) target_wgs *= 2;
    } else if (dim <= 256 && !force_sweep && (!kv_8bit || dim % 64 == 0) &&
               (ratio >= tun().group_min_ratio || group_only ||
                (tun().group_min_ratio > 1 && (max_seq_k >= 1024 || dim <= 96) &&
                 (long long)batch * (long long)head_k * (long long)max_seq_k >= (1ll << 21)) ||
                // ... and over long sequences of a small batch (measured, 32 heads, 16-bit / FP8: batch 1 x 8192 tokens
                // 26.3 -> 23.9 / 17.8 -> 14.9 us, 1 x 16384 47.9 -> 42.7 / 27.6 -> 24.8, 2 x 4096 25.0 -> 23.7 /
                // 17.7 -> 15.3, 4 x 8192 89.8 -> 82.1 / 46.4 -> 44.6, d 64 1 x 16384 27.7 -> 24.6 / 18.8 -> 15.7; a
                // tie at 1 x 4096 and 1 x 6144; d 256 stays: 1 x 8192 24.9 against 35.2)
                (tun().group_min_ratio > 1 && dim <= 128 && max_seq_k >= 4096 &&
                 (long long)batch * (long long)head_k * (long long)max_seq_k >= (3ll << 16)) ||
                // an int4 cache (the format without a latent kernel): the VALU sweep pays more per nibble than the
                // matrix kernel's word-wise conversion does (measured, MHA 32 heads d 128: batch 512 x 128 tokens 92.0
                // -> 54.8 us, batch 2048 x 128 397 -> 254, batch 32 x 1024 50.5 -> 30.8, batch 32 x 128 8.7 -> 6.8,
                // batch 1 x 4096 16.0 -> 10.2; d 64, batch 16 x 512 14.4 -> 11.0; below 2^17 rows of tokens the sweep's
                // single small launch wins, batch 16 x 128 5.9 against 7.5, and at d 256 it ties or wins)
                (tun().group_min_ratio > 1 && no_latent_kernel && dim <= 128 &&
                 (long long)batch * (long long)head_k * (long long)max_seq_k >= (1ll << 17)))) {
        // Two or more query heads per KV head, or a single one over long sequences of a large batch: the MFMA sweep streams K/V
        // a few percent faster than the VALU sweep even though most of its matrix columns are idle (measured:
        // ratio 2, 2048 tokens: 201 -> 185 us; ratio 1, batch 64 x 2048 tokens: 375 -> 364 us; at batch 1 the VALU sweep wins, and
        // for short sequences it is the steadier one at d = 128 and 256 but the slower one at d = 64 and 96:
        // d 96, 256 x 512 tokens: 366 -> 275 us).
        pl.kind = kKindGroup;
        pl.rt = ratio > 16 ? 32 : 16;
        if (tun().gqa_heads == 16 || tun().gqa_heads == 32) pl.rt = tun().gqa_heads;
        if (group_only == 2 && dim == 256) pl.rt = 16;
        pl.wave_per_head = head_k % 4 == 0 && tun().wave_per_head;
        trip = pl.wave_per_head ? da::kGqaTile : 4 * da::kGqaTile;
        // 16-bit K/V in whole tiles or 16-token runs, rows of 192 bytes and more (d = 96, 128, 256): one work-group per
        // CU saturates what the kernel can pull, and half as many splits halve the partials and the merge.  Measured,
        // 256 against 512 work-groups, bf16: 32/8 heads d 128, batch 64 x 4096 tokens 165.4 -> 159.4 us, batch 128 x 2048
        // 164.4 -> 156.2, batch 32 x 4096 84.5 -> 80.7; 64/8 heads 169.0 -> 160.8; 32/4 heads 88.0 -> 82.9; over 16-token
        // pages 169.9 -> 164.1; MQA 32/1, batch 64 x 4096 35.7 -> 29.6; d 256, 32/8 heads, batch 64 x 4096 317.7 -> 309.0,
        // batch 128 x 2048 320.7 -> 305.7, 16/1 heads, batch 64 x 4096 53.8 -> 46.2, 64/1 heads 93.5 -> 77.9, 32/2 heads
        // 95.7 -> 87.3; d 96, 32/8 heads, batch 64 x 4096 144.1 -> 142.0, batch 128 x 2048 142.5 ->
        // 138.1.  (Before the kernel waited for a tile's K registers ahead of issuing the next tile's V loads, the
        // form with one wave per KV head needed the second work-group per CU to hide that wait: 170.4 against 166.1.)
        // Not at d = 64, whose work-groups stream too few bytes for one per CU (batch 32 x 4096: 47.0 -> 52.2 us), and
        // not over 8-bit K/V or per-row page lookups, which keep fewer bytes in flight per work-group (FP8, 32/8 heads,
        // batch 32 x 4096 tokens 47.8 -> 53.1 us, batch 48 69.3 -> 80.2; int4 30.4 -> 34.3 and 43.8 -> 49.4).
        if (dim >= 96 && !kv_8bit && (packed || page_size >= 16)) target_wgs = tun().group_target_wgs_d128;
    } else {
        pl.kind = kKindSweep;
        const int max_rt = dim > 256 ? 2 : 4;
        pl.rt = ratio >= 3 ? 4 : ratio;  // 1, 2 or 4 (a group of 3 runs as 4 with one idle head)
        if (pl.rt > max_rt) pl.rt = max_rt;
        trip = rows_per_trip(dim);
    }
    pl.groups = (ratio + pl.rt - 1) / pl.rt;
    const long long base = (long long)batch * (long long)(pl.wave_per_head ? head_k / 4 : head_k) * pl.groups;
    const bool ragged = total_k > 0 && (long long)total_k * 10 < (long long)batch * (long long)max_seq_k * 9;
    // The grouped kernel's balanced grid: equal shares of the concatenated tokens instead of fixed splits of every
    // sequence.  Taken for a batch whose token count shows it to be ragged, and for a packed batch whose count the
    // caller did not give (the reference's signature carries none, csrc/ops/decoding_attn.h:29-30) when it is large
    // enough for whole shares: a uniform batch is then cut exactly as fixed splits cut it (batch 64 x 4096 tokens:
    // 256 shares of 1024), and a ragged one is balanced.  The kernels read the line's length from cu_seq_k[batch]
    // themselves.  Paged K/V pays one more (tiny) kernel for the sequences' positions, so it takes this form only
    // when the count is given and the sweep is long enough to win that back.
    const double kv_bytes = (double)total_k * (double)head_k * (double)(dim + dim_v) * (kv_8bit ? 1.0 : 2.0);
    if (pl.kind == kKindGroup && tun().flat_wgs > 0 && batch >= 2) {
        const long long ygrid = base / (long long)batch;
        // (the work-groups the fixed-split plan of this shape aims at, so that a uniform batch without a count is cut
        // the same way -- MQA at d = 128, 256 instead of 512: batch 64 x 4096 tokens 42.1 -> 29.5 us -- and a ragged one
        // gains what the uniform one gains: 32/8 heads d 128 bf16, batch 64 x 1..8192 tokens 209.3 -> 202.0 us, batch
        // 128 x 1..4096 170.6 -> 166.7, 64/8 heads, batch 32 x 1..16384 182.5 -> 175.5; over 16-token pages 197.6 ->
        // 194.8, 177.7 -> 172.0, 185.1 -> 177.6)
        long long w = std::max<long long>(1, std::min(target_wgs, tun().flat_wgs) / ygrid);
        const long long unit = packed ? 1 : da::kGqaTile;
        const long long step = std::max<long long>(1, trip / unit);  // a work-group's waves advance `trip` tokens together
        const long long mn = std::max<long long>(tun().flat_min_tokens / unit, step);
        const bool counted = ragged && total_k < ((size_t)1 << 30) && total_k >= 64 * batch &&
                             (packed || kv_bytes >= (double)tun().flat_paged_min_mb * 1e6);
        const bool uncounted = total_k == 0 && packed && !latent_group && tun().flat_uncounted &&
                               (long long)batch * (long long)max_seq_k >=
                                   std::max<long long>(1, tun().flat_wgs / ygrid) * (long long)tun().flat_uncounted_min &&
                               (long long)batch * (long long)max_seq_k < (1ll << 30);
        if (counted || uncounted) {
            pl.flat_step = (int)step;
            pl.flat_min = (int)mn;
            pl.flat_unit = (int)unit;
            if (counted) {
                const long long line = packed ? (long long)total_k : (long long)total_k / unit + (long long)batch;
                const long long t = da::flat_share(line, (int)w, (int)step, (int)mn);
                w = std::min<long long>(w, (line + t - 1) / t);  // (shares past the line's end would only exit)
                pl.chunk = (int)(da::flat_share(line, (int)w, (int)step, (int)mn) * unit);
            } else {
                pl.chunk = 0;
            }
            pl.flat_wgs = (int)w;
            pl.nsplit = (int)w;
            // partials a sequence of max_seq_k tokens has when the batch is as long as the host knows it can be (the
            // merge picks its form by it; a batch that turns out shorter has more, and is merged correctly all the same)
            const long long line_max = counted ? (packed ? (long long)total_k : (long long)total_k / unit + (long long)batch)
                                               : (long long)batch * (((long long)max_seq_k + unit - 1) / unit);
            const long long t_est = da::flat_share(line_max, (int)w, (int)step, (int)mn);
            pl.flat_partials = (int)std::min<long long>(w, (((long long)max_seq_k + unit - 1) / unit + t_est - 1) / t_est + 1);
            pl.ws_bytes = da::flat_slots((int)w, batch) * head_q * (dim_v + 2) * sizeof(float);
            if (!packed) {
                pl.flat_cu_bytes = ((batch + 1) * sizeof(int32_t) + 15) & ~(size_t)15;
                pl.ws_bytes += pl.flat_cu_bytes;
            }
            return pl;
        }
    }
    int min_chunk = std::max(mfma ? 256 : tun().min_chunk, trip);
    const long long wgs_at_min = base * std::max<long long>(1, (long long)max_seq_k / min_chunk);
    if (mfma) {
        // too few work-groups for the chip even so: 128-token splits, as long as that keeps the merge at 32
        // partials or fewer (measured: batch 1 x 512 tokens 26.8 -> 20.5 us, batch 16 x 512 33.1 -> 29.4 us,
        // batch 4 x 2048 32.9 -> 28.3 us; batch 1 x 8192 with 64 partials loses, 36.0 -> 38.5 us)
        if (wgs_at_min < tun().mfma_small_wgs && max_seq_k <= 32 * 128) min_chunk = std::max(std::min(min_chunk, 128), trip);
        // (the pipelined kernel takes 128-token splits whenever its work-group count, chosen below, asks for them)
        if (pipe_kernel && pl.rt == 128 && max_seq_k <= 32 * 128) min_chunk = std::max(std::min(min_chunk, 128), trip);
    } else {
        // 512-token splits run best; go down to 256 only when that is needed to give every CU a work-group (the
        // VALU sweep: two, measured batch 4 x 1024 tokens 21.4 -> 18.6 us; the grouped kernel loses there)
        const long long fill = pl.kind == kKindSweep ? 2 * 256 : 256;
        if (wgs_at_min < fill) min_chunk = std::max(std::min(min_chunk, 256), trip);
        // the VALU sweep at d = 256 (long rows, long tiles): 128-token splits while the chip is not full
        // (measured, MHA batch 1 x 512 tokens 17.2 -> 13.2 us, batch 2 x 1024 19.7 -> 18.0; no gain at d <= 128)
        if (pl.kind == kKindSweep && dim >= 256 && max_seq_k >= 512 &&
            base * std::max<long long>(1, (long long)max_seq_k / 256) < fill)
            min_chunk = std::max(std::min(min_chunk, 128), trip);
        // One wave per KV head on a chip that even 256-token splits leave half empty: a work-group's time is then
        // mostly the latency of its few serial tiles, so split down to 64 tokens, just far enough to give every CU
        // a work-group and with at most 32 partials to merge (measured, 32/8 heads d 128: batch 1 x 4096 tokens
        // 20.1 -> 15.7 us, batch 4 x 1024 18.9 -> 13.4, batch 16 x 1024 21.1 -> 18.2; 16/8 heads d 256: batch 1 x
        // 2048 29.1 -> 15.5).  Below 512 tokens at d < 128 the second launch costs more than the split saves, and
        // where four waves share one KV head's tokens the finer split changes nothing, except in the latent form
        // (long rows: 16 heads, batch 1 x 4096 tokens 20.0 -> 17.0 us with 128-token splits, one tile per wave).
        if (pl.kind == kKindGroup && (pl.wave_per_head || latent_group) && (max_seq_k >= 512 || dim >= 128) &&
            base * std::max<long long>(1, (long long)max_seq_k / 256) < tun().group_small_wgs) {
            const int by_partials = (int)(((long long)max_seq_k + 31) / 32 + trip - 1) / trip * trip;
            min_chunk = std::max(std::min(min_chunk, std::max(tun().group_small_chunk, by_partials)), trip);
            target_wgs = tun().group_small_wgs;
        }
        if (ragged) min_chunk = std::max(std::min(min_chunk, tun().ragged_chunk), trip);
    }
    long long want = base > 0 ? (target_wgs + base - 1) / base : 1;
    // The latent forms hold one work-group per CU (two for the latent kernel's one- and two-wave forms over 16-bit
    // K, for which the target is doubled): a grid a little over that capacity would run as two rounds, the second
    // nearly empty, so round down there (measured: 48 heads, batch 64 x 256 tokens, 384 work-groups 33.6 us, 192
    // work-groups 19.1 us; 128 heads, batch 100 x 4096 tokens, 300 work-groups 247 us, 200 work-groups 198 us; batch
    // 40 x 8192, 280 work-groups 209 us, 240 work-groups 146 us; 16 heads, batch 150 x 4096, 300 work-groups 183 us,
    // 150 work-groups 153 us).
    if ((latent_group || mfma) && base > 0) want = std::max<long long>(1, target_wgs / base);
    // The pipelined latent kernel: every work-group pays a fixed cost (147 KB of Q in, 131 KB of partials out), and the
    // chip, power-limited under this kernel, runs few active CUs at a higher clock, so the best grid grows with the
    // work: 128 work-groups up to 64 Ki tokens of (sequence, KV head) rows, one more per Ki tokens from there, all
    // 256 CUs from 192 Ki.  Split counts are rounded to the nearest (a half down) and kept to one round of the CUs.
    // Measured, 128 heads, us a call by work-groups: batch 16 x 4096 tokens 128: 33.7, 192: 33.1, 256: 41.8; batch 8 x
    // 8192 128: 34.3, 192: 37.5, 256: 42.2; batch 16 x 1024 64: 21.3, 128: 18.4; batch 8 x 2048 64: 21.6, 128: 19.2;
    // batch 40 x 2048 120: 41.9, 160: 39.0, 200: 40.9; batch 32 x 4096 128: 55.9, 192: 52.7, 256: 56.6; batch 64 x 2048
    // 128: 59.5, 192: 54.5, 256: 59.1; batch 48 x 4096 144: 82.3, 192: 72.7, 240: 71.8; batch 64 x 4096 192: 92.3, 256:
    // 86.6; batch 96 x 1024 96: 52.7, 192: 48.2; batch 128 x 1024 128: 56.1, 256: 59.9.
    // Over an 8-bit cache a tile takes longer (the conversion) and the chip is less power-bound: 192 work-groups up
    // to 64 Ki rows, all CUs from 128 Ki (FP8: batch 16 x 4096 128: 41.0, 192: 35.6, 256: 37.0; batch 24 x 2048 120:
    // 36.9, 192: 30.6; batch 64 x 1024 128: 44.2, 192: 38.2; batch 32 x 4096 192: 54.8, 256: 52.9; batch 128 x 512 128:
    // 38.4, 256: 42.0).
    if (mfma && pipe_kernel && pl.rt == 128 && base > 0) {
        const long long rows = base * (long long)max_seq_k, least = kv_8bit ? 192 : 128;
        const long long w = std::min<long long>(std::max<long long>(least - 64 + rows / 1024, least), target_wgs);
        want = std::max<long long>(1, (2 * w + base - 1) / (2 * base));
        while (want > 1 && base * want > target_wgs) --want;
    }
    const long long by_len = std::max<long long>(1, (long long)max_seq_k / min_chunk);
    // sweep work-groups are also kept short (shorter still for a ragged batch); the latent MFMA kernel's partials
    // are too large (heads x dim_v floats per split) to split more than occupancy asks for
    const int max_chunk = std::max(1, ragged ? tun().ragged_chunk : tun().max_chunk * max_chunk_scale);
    long long by_cap = mfma ? 1 : ((long long)max_seq_k + max_chunk - 1) / max_chunk;
    // the grouped kernel on a batch known to be uniform (token count given, not ragged) needs no cap: fewer, longer
    // splits mean a smaller merge (measured, 32/8 heads d 128: batch 256 x 4096 tokens 726 -> 703 us, batch 128 x
    // 4096 366 -> 360, batch 64 x 16384 727 -> 713); without the count the cap keeps a ragged batch balanced
    // (up to 2048 tokens while the grid is one work-group per CU: with nothing to balance the CUs against each other a
    // longer split loses again, batch 32 x 16384 tokens 360 -> 377 us with 4096-token splits)
    if (pl.kind == kKindGroup && !latent_group && total_k > 0 && !ragged && !kv_8bit && (packed || page_size >= 16))
        by_cap = base >= 512 ? 1 : ((long long)max_seq_k + 2047) / 2048;
    // ... and without a token count (the reference-signature entry point) the same kernel caps at 2048 tokens: as
    // good as the counted plan on a uniform batch and better than the 1024 cap on a ragged one (measured, 32/8 heads,
    // batch 64, d 128: 4096 tokens each 184.6 -> 181.6 us, 181.4 with the count; 1..8192 tokens 264.7 -> 246.1 us; d 96:
    // 152.0 -> 147.0 and 255.8 -> 242.8; d 256: a tie and 540.2 -> 519.9; d 64: a tie and 151.2 -> 146.8)
    if (pl.kind == kKindGroup && !latent_group && total_k == 0 && !kv_8bit && (packed || page_size >= 16))
        by_cap = ((long long)max_seq_k + 2047) / 2048;
    // (one round of long splits beats two rounds with the second nearly empty)
    if (latent_group && base <= target_wgs && base * by_cap > target_wgs) by_cap = 1;
    long long ns = std::max(std::min(want, by_len), std::min(by_cap, by_len));
    ns = std::max<long long>(1, std::min<long long>(ns, kMaxSplits));
    // The grouped kernel's grids and the 256 CUs: work-groups are handed out as CUs free up, so a grid that is not
    // close to a multiple of the CU count ends with most of the chip idle while a few CUs finish (and up to 256
    // work-groups run one per CU, which saturates HBM from about 200).  When the plan above fills its last round of
    // 256 poorly, take the split count that fills it best instead (fewer splits on a tie).  Measured, 32/8 heads d
    // 128, 4096 tokens: batch 40, 7 splits (560 work-groups) 138.6 us, 3 splits (240) 117.9; batch 48, 6 splits (576)
    // 158.8, 5 splits (480) 142.4; batch 100, 4 splits (800) 320.5, 1 split (200) 284.8.
    // (d = 96 counts as long rows, 256 work-groups a round, like its target above: 32/8 heads, 4096 tokens, batch 40
    // 118.0 -> 92.2 us, batch 48 148.3 -> 113.1, batch 72 225.6 -> 166.0, batch 100 243.8 -> 223.1; batch 24 x 8192
    // 151.1 -> 109.4; 32/4 heads, batch 80 x 4096 117.4 -> 90.2)
    // (measured on 16-bit K/V in whole tiles or 16-token runs, and applied there only)
    // (... and on 8-bit K/V at d = 128, whose rows are as short as 16-bit rows at d = 64: FP8, 32/8 heads, batch 100
    // x 4096 tokens 184 -> 154 us, batch 72 131 -> 116, batch 40 74 -> 66)
    const bool whole_tiles = packed || page_size >= 16;
    const bool plain16 = !kv_8bit && whole_tiles;
    const bool short_rows = dim < 96 || kv_8bit;
    if (pl.kind == kKindGroup && (plain16 || (kv_8bit && dim == 128 && whole_tiles)) && dim <= 256 &&
        tun().fill_rounds) {
        // (at d = 64 a work-group streams too few bytes for one per CU to saturate HBM: rounds of two per CU there;
        // 32/8 heads, batch 56 x 4096 tokens 100.1 -> 84.9 us, 32/4 heads, batch 150 x 4096 127.2 -> 112.3)
        const double gran = short_rows ? 512.0 : 256.0, sat = short_rows ? 400.0 : 200.0;
        auto fill = [&](long long c) {
            const double w = (double)(base * c);
            if (w <= gran) return std::min(1.0, w / sat);
            return w / (std::ceil(w / gran) * gran);
        };
        if (fill(ns) < 0.85) {
            long long best_ns = ns;
            double best = fill(ns) - 0.004 * (double)ns;
            for (long long c = 1; c <= std::min<long long>(by_len, 64); ++c) {
                const double score = fill(c) - 0.004 * (double)c;
                if (score > best + 1e-9) {
                    best = score;
                    best_ns = c;
                }
            }
            ns = best_ns;
        }
    }
    if (tun().nsplit > 0) ns = std::min<long long>(tun().nsplit, kMaxSplits);
    long long chunk = ((long long)max_seq_k + ns - 1) / ns;
    chunk = (chunk + trip - 1) / trip * trip;
    if (chunk <= 0) chunk = trip;
    ns = std::max<long long>(1, ((long long)max_seq_k + chunk - 1) / chunk);
    pl.nsplit = (int)ns;
    pl.chunk = (int)chunk;
    pl.ws_bytes = pl.nsplit > 1 ? (size_t)batch * head_q * pl.nsplit * (dim_v + 2) * sizeof(float) : 0;
    return pl;
}

// Workspace bytes of a call: the plan's, or, for a batch beyond one launch (kMaxGridBatch), the largest of its runs'.
size_t plan_ws_bytes(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                     bool v_distinct, size_t total_k, size_t page_size = 0, bool kv_8bit = false,
                     bool no_latent_kernel = false, int group_only = 0) {
    if (batch <= kMaxGridBatch)
        return make_plan(max_seq_k, batch, head_q, head_k, dim, dim_v, v_distinct, total_k, page_size, kv_8bit,
                         no_latent_kernel, group_only).ws_bytes;
    size_t need = make_plan(max_seq_k, kMaxGridBatch, head_q, head_k, dim, dim_v, v_distinct, 0, page_size, kv_8bit,
                            no_latent_kernel, group_only).ws_bytes;
    if (batch % kMaxGridBatch != 0)
        need = std::max(need, make_plan(max_seq_k, batch % kMaxGridBatch, head_q, head_k, dim, dim_v, v_distinct, 0,
                                        page_size, kv_8bit, no_latent_kernel, group_only).ws_bytes);
    return need;
}

struct CachedWs {
    void* ptr = nullptr;
    size_t bytes = 0;
};
std::mutex g_ws_mutex;
std::map<std::pair<int, void*>, CachedWs> g_ws;
bool g_ws_exit_hook = false;
int release_cached_workspaces(bool report);
// Registered when the first workspace is allocated, so after the HIP runtime set itself up: exit handlers run in
// reverse order of registration, which hands the workspaces back while the runtime is still there (at process exit,
// and when the library is unloaded, where the handlers of a shared object run too).
void release_at_exit() { (void)release_cached_workspaces(false); }

// Workspace of the reference-signature entry point: one buffer per (device, stream), grown on demand.
int cached_workspace(size_t bytes, hipStream_t stream, void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(DA_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    CachedWs& w = g_ws[std::make_pair(dev, (void*)stream)];
    if (w.bytes < bytes) {
        if (w.ptr) {
            e = hipFree(w.ptr);  // waits for work that may still read it
            w.ptr = nullptr;
            w.bytes = 0;
            if (e != hipSuccess) return fail(DA_ERR_HIP, "hipFree(workspace): %s", hipGetErrorString(e));
        }
        const size_t want = (bytes + (1u << 20) - 1) & ~((size_t)(1u << 20) - 1);
        e = hipMalloc(&w.ptr, want);
        if (e != hipSuccess) {
            w.ptr = nullptr;
            return fail(DA_ERR_HIP, "hipMalloc(workspace, %zu): %s", want, hipGetErrorString(e));
        }
        w.bytes = want;
        if (!g_ws_exit_hook) {
            g_ws_exit_hook = true;
            (void)std::atexit(release_at_exit);
        }
    }
    *out = w.ptr;
    return DA_OK;
}

// Free every cached workspace (the caller vouches that no enqueued call still uses one).  Errors are reported for an
// explicit release and ignored at exit or unload.
int release_cached_workspaces(bool report) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    int rc = DA_OK;
    if (g_ws.empty()) return rc;  // (and no call into the HIP runtime: it may be gone already)
    int prev = 0;
    const bool have_prev = hipGetDevice(&prev) == hipSuccess;
    for (auto& kv : g_ws) {
        if (!kv.second.ptr) continue;
        hipError_t e = hipSetDevice(kv.first.first);
        if (e == hipSuccess) e = hipFree(kv.second.ptr);
        if (e != hipSuccess && report) rc = fail(DA_ERR_HIP, "hipFree(workspace): %s", hipGetErrorString(e));
        kv.second.ptr = nullptr;
        kv.second.bytes = 0;
    }
    g_ws.clear();
    if (have_prev) (void)hipSetDevice(prev);
    return rc;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

// Workspace of da_decoding_attn_noalloc: a device array that exists on every GPU the library is loaded on, from
// load to process end.  The largest workspace any plan asks for is 256 work-groups x 128 heads x 514 floats =
// 67.4 MB (the latent kernel's split partials), except for the balanced grid on pathologically ragged batches.
#ifdef DA_BUILD_PROBES
// (the measurement build, which only the benchmark loads, holds no such array: its no-alloc entry point serves the
// plans that need no workspace and refuses the rest)
constexpr size_t kScratchBytes = 256;
#else
constexpr size_t kScratchBytes = (size_t)80 << 20;
#endif
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {

// Device address of `scratch` on the current device (each GPU holds its own copy at its own address), looked up on
// the first call per device.  The array's name itself is only a host-side handle.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

int scratch_on_current_device(void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(DA_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(DA_ERR_HIP, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            return fail(DA_ERR_HIP, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return DA_OK;
}

}  // namespace

extern "C" {

const char* da_last_error(void) { return g_last_error.c_str(); }

int da_version(void) { return 100; }

int da_supported_head_dims(size_t dim, size_t dim_v) { return supported_dims(dim, dim_v) ? 1 : 0; }

int da_plan(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v, int is_bf16,
            size_t total_k, int* kernel_kind, int* nsplit, int* chunk, int* heads_per_group) {
    (void)is_bf16;
    if (head_k == 0 || head_q % head_k != 0)
        return fail(DA_ERR_INVALID_ARGUMENT, "head_q (%zu) must be a multiple of head_k (%zu)", head_q, head_k);
    if (!supported_dims(dim, dim_v))
        return fail(DA_ERR_UNSUPPORTED, "unsupported head dims (dim %zu, dim_v %zu)", dim, dim_v);
    const Plan pl = make_plan(max_seq_k, batch, head_q, head_k, dim, dim_v, false, total_k);
    if (kernel_kind) *kernel_kind = pl.kind;
    if (nsplit) *nsplit = pl.nsplit;
    if (chunk) *chunk = pl.chunk;
    if (heads_per_group) *heads_per_group = pl.rt;
    return DA_OK;
}

int da_plan_distinct_v(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                       size_t total_k, size_t page_size, int* kernel_kind, int* nsplit, int* chunk,
                       int* heads_per_group) {
    if (head_k == 0 || head_q % head_k != 0)
        return fail(DA_ERR_INVALID_ARGUMENT, "head_q (%zu) must be a multiple of head_k (%zu)", head_q, head_k);
    if (!supported_dims(dim, dim_v))
        return fail(DA_ERR_UNSUPPORTED, "unsupported head dims (dim %zu, dim_v %zu)", dim, dim_v);
    const Plan pl = make_plan(max_seq_k, batch, head_q, head_k, dim, dim_v, true, total_k, page_size, false);
    if (kernel_kind) *kernel_kind = pl.kind;
    if (nsplit) *nsplit = pl.nsplit;
    if (chunk) *chunk = pl.chunk;
    if (heads_per_group) *heads_per_group = pl.rt;
    return DA_OK;
}

int da_plan_is_balanced(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                        size_t total_k, size_t page_size) {
    if (head_k == 0 || head_q % head_k != 0 || !supported_dims(dim, dim_v)) return -1;
    return make_plan(max_seq_k, batch, head_q, head_k, dim, dim_v, false, total_k, page_size).flat_wgs > 0 ? 1 : 0;
}

int da_plan_call(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v, size_t total_k,
                 size_t page_size, int distinct_v, int kv_bits, int* kernel_kind, int* nsplit, int* chunk,
                 int* heads_per_group, int* balanced) {
    if (head_k == 0 || head_q % head_k != 0)
        return fail(DA_ERR_INVALID_ARGUMENT, "head_q (%zu) must be a multiple of head_k (%zu)", head_q, head_k);
    if (!supported_dims(dim, dim_v))
        return fail(DA_ERR_UNSUPPORTED, "unsupported head dims (dim %zu, dim_v %zu)", dim, dim_v);
    const bool per64 = kv_bits == DA_KV_BITS_INT4_GROUP64 || kv_bits == DA_KV_BITS_INT8_GROUP64;
    const bool per_token = kv_bits == DA_KV_BITS_INT4_PER_TOKEN || kv_bits == DA_KV_BITS_INT8_PER_TOKEN || per64;
    if (kv_bits != 16 && kv_bits != 8 && kv_bits != 4 && !per_token)
        return fail(DA_ERR_INVALID_ARGUMENT,
                    "kv_bits (%d) must be 16, 8, 4 or one of DA_KV_BITS_INT*_PER_TOKEN and DA_KV_BITS_INT*_GROUP64", kv_bits);
    if (per_token && (dim != dim_v || (dim != 64 && dim != 128 && dim != 256) || !distinct_v))
        return fail(DA_ERR_UNSUPPORTED, "per-token factors: head dims (64,64), (128,128) and (256,256), V of its own");
    if (page_size != 0 && (page_size & (page_size - 1)) != 0)
        return fail(DA_ERR_INVALID_ARGUMENT, "page_size (%zu) must be a power of two", page_size);
    // (as run_attention plans one launch; a batch beyond one grid axis is planned run by run, without the count)
    const bool folded = batch > kMaxGridBatch;
    const Plan pl = make_plan(max_seq_k, folded ? kMaxGridBatch : batch, head_q, head_k, dim, dim_v, distinct_v != 0,
                              folded ? 0 : total_k, page_size, kv_bits != 16,
                              kv_bits == 4 || kv_bits == DA_KV_BITS_INT4_PER_TOKEN || kv_bits == DA_KV_BITS_INT4_GROUP64,
                              per64 ? 2 : (per_token ? 1 : 0));
    if (kernel_kind) *kernel_kind = pl.kind;
    if (nsplit) *nsplit = pl.nsplit;
    if (chunk) *chunk = pl.chunk;
    if (heads_per_group) *heads_per_group = pl.rt;
    if (balanced) *balanced = pl.flat_wgs > 0 ? 1 : 0;
    return DA_OK;
}

size_t da_workspace_bytes(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                          size_t total_k) {
    if (head_k == 0 || head_q % head_k != 0 || !supported_dims(dim, dim_v)) return 0;
    const size_t a = plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, false, total_k);
    const size_t b = plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, true, total_k);
    return a > b ? a : b;
}

size_t da_workspace_bytes_paged(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                size_t total_k, size_t page_size) {
    if (head_k == 0 || head_q % head_k != 0 || !supported_dims(dim, dim_v)) return 0;
    const size_t a = plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, false, total_k, page_size, false);
    const size_t b = plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, true, total_k, page_size, false);
    return a > b ? a : b;
}

size_t da_workspace_bytes_fp8kv(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                size_t dim_v, size_t total_k, size_t page_size) {
    if (head_k == 0 || head_q % head_k != 0 || !supported_dims(dim, dim_v)) return 0;
    const size_t a = plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, false, total_k, page_size, true);
    const size_t b = plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, true, total_k, page_size, true);
    return a > b ? a : b;
}

size_t da_workspace_bytes_int8kv(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                 size_t dim_v, size_t total_k, size_t page_size) {
    return da_workspace_bytes_fp8kv(max_seq_k, batch, head_q, head_k, dim, dim_v, total_k, page_size);  // same plans
}

}  // extern "C"

namespace {

// Page-pool description of paged K/V; table == nullptr means the packed layout.
struct Paging {
    const int32_t* table = nullptr;
    const int32_t* seq_lens = nullptr;
    size_t page_size = 0, max_blocks = 0, k_page = 0, v_page = 0;
};

// Element format of K/V: 16-bit like Q (fmt 0), or 8-bit (da::kKvFp8, da::kKvInt8) or 4-bit (da::kKvInt4) with
// per-KV-head de-quantisation factors (null = 1).
struct KvFormat {
    bool sweep_only = false;  // measurement: leave the split partials in the workspace, do not merge them
    int fmt = 0;
    const float* k_scale = nullptr;
    const float* v_scale = nullptr;
    // (int4) a (scale, zero) pair per (token, KV head) instead of the per-head factors
    const float* k_tok = nullptr;
    const float* v_tok = nullptr;
    bool tok_per64 = false;  // ... a pair per run of 64 elements of the row instead: [rows, head_k, dim / 64, 2]
};

KvFormat per_token_format(int fmt, const float* k_params, const float* v_params, bool per64 = false) {
    KvFormat kf;
    kf.fmt = fmt;
    kf.k_tok = k_params;
    kf.v_tok = v_params;
    kf.tok_per64 = per64;
    return kf;
}

KvFormat kv8_format(int fmt, const float* k_scale, const float* v_scale) {
    KvFormat kf;
    kf.fmt = fmt;
    kf.k_scale = k_scale;
    kf.v_scale = v_scale;
    return kf;
}

int run_attention(const void* q, const void* k, const void* v, void* o, const int32_t* cu_seq_k, const Paging& pg,
                  const KvFormat& kf, size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                  int is_alibi, int is_bf16, float softmax_scale, const float* alibi_slopes, size_t total_k,
                  void* workspace, size_t workspace_bytes, void* hip_stream) {
    // the reference's checks (csrc/ops/decoding_attn.cpp:16-22) ...
    if (!q) return fail(DA_ERR_INVALID_ARGUMENT, "q is null");
    if (!k) return fail(DA_ERR_INVALID_ARGUMENT, "k is null");
    if (!o) return fail(DA_ERR_INVALID_ARGUMENT, "o is null");
    if (!pg.table && !cu_seq_k) return fail(DA_ERR_INVALID_ARGUMENT, "cu_seq_k is null");
    if (head_k == 0 || head_q % head_k != 0)
        return fail(DA_ERR_INVALID_ARGUMENT, "head_q (%zu) must be a multiple of head_k (%zu)", head_q, head_k);
    if (dim > 576) return fail(DA_ERR_INVALID_ARGUMENT, "dim (%zu) must be <= 576", dim);
    if (dim_v > 512) return fail(DA_ERR_INVALID_ARGUMENT, "dim_v (%zu) must be <= 512", dim_v);
    // ... and the ones it leaves out
    if (!supported_dims(dim, dim_v))
        return fail(DA_ERR_UNSUPPORTED,
                    "unsupported head dims (dim %zu, dim_v %zu): supported are (64,64) (96,96) (128,128) (256,256) "
                    "(576,512)",
                    dim, dim_v);
    if (!aligned16(q) || !aligned16(k) || (v && !aligned16(v)))
        return fail(DA_ERR_INVALID_ARGUMENT, "q, k and v must be 16-byte aligned");
    // (every finishing path stores 8 or 16 bytes of a row at a time; rows are multiples of 128 bytes)
    if (!aligned16(o)) return fail(DA_ERR_INVALID_ARGUMENT, "o must be 16-byte aligned");
    if (max_seq_k > (size_t)INT32_MAX || batch > (size_t)INT32_MAX || head_q > 65535)
        return fail(DA_ERR_INVALID_ARGUMENT, "shape out of range (max_seq_k %zu, batch %zu, head_q %zu)", max_seq_k, batch,
                    head_q);
    if (batch == 0) return DA_OK;
    if (batch > kMaxGridBatch) {
        // The kernels number the sequences along a grid axis that ends at 65535 (the reference numbers them along
        // grid.x, csrc/kernel/decoding_attn/decoding_fwd_launch_template.h:18, and has no such limit): a larger batch
        // runs as consecutive launches over runs of sequences.  q, o, cu_seq_k and the block table move on with the
        // run; packed K/V stay, cu_seq_k holds absolute rows.  The runs share the workspace: they follow each other
        // on the stream.  (total_k is the whole batch's: the runs are planned without it.)
        for (size_t b0 = 0; b0 < batch; b0 += kMaxGridBatch) {
            const size_t nb = std::min(kMaxGridBatch, batch - b0);
            Paging pgr = pg;
            if (pg.table) {
                pgr.table = pg.table + b0 * pg.max_blocks;
                pgr.seq_lens = pg.seq_lens + b0;
            }
            const int rc = run_attention(static_cast<const uint8_t*>(q) + b0 * head_q * dim * 2, k, v,
                                         static_cast<uint8_t*>(o) + b0 * head_q * dim_v * 2,
                                         cu_seq_k ? cu_seq_k + b0 : nullptr, pgr, kf, max_seq_k, nb, head_q, head_k, dim,
                                         dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes, 0, workspace,
                                         workspace_bytes, hip_stream);
            if (rc != DA_OK) return rc;
        }
        return DA_OK;
    }

    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    const bool per_token = kf.k_tok != nullptr || kf.v_tok != nullptr;
    if (per_token) {
        if ((kf.fmt != da::kKvInt4 && kf.fmt != da::kKvInt8) || !kf.k_tok || !kf.v_tok || !v)
            return fail(DA_ERR_INVALID_ARGUMENT,
                        "per-token factors need an int4 or int8 cache, both k_params and v_params, and v");
        if (dim != dim_v || (dim != 64 && dim != 128 && dim != 256))
            return fail(DA_ERR_UNSUPPORTED, "per-token factors: head dims (64,64), (128,128) and (256,256) only");
        if ((reinterpret_cast<uintptr_t>(kf.k_tok) | reinterpret_cast<uintptr_t>(kf.v_tok)) & 7u)
            return fail(DA_ERR_INVALID_ARGUMENT, "k_params and v_params must be 8-byte aligned");
    }
    const Plan pl = make_plan(max_seq_k, batch, head_q, head_k, dim, dim_v, v != nullptr, total_k,
                              pg.table ? pg.page_size : 0, kf.fmt != 0, kf.fmt == da::kKvInt4,
                              per_token ? (kf.tok_per64 ? 2 : 1) : 0);
    if (per_token && pl.kind != kKindGroup)  // (DA_FORCE_KIND=1 takes the grouped kernel away)
        return fail(DA_ERR_UNSUPPORTED, "per-token factors need the grouped kernel");
    if ((size_t)head_k * pl.groups > 65535)
        return fail(DA_ERR_INVALID_ARGUMENT, "head_k * groups exceeds the grid limit 65535");
    if (kf.fmt == da::kKvInt4 && pl.kind == kKindMfma)  // (DA_MLA_GROUP_HEADS=0 takes the grouped kernel away)
        return fail(DA_ERR_UNSUPPORTED, "an int4 K/V cache at (576, 512) needs the grouped kernel's latent form");

    void* ws = nullptr;
    if (pl.ws_bytes > 0) {
        if (workspace) {
            if (workspace_bytes < pl.ws_bytes)
                return fail(DA_ERR_WORKSPACE, "workspace has %zu bytes, %zu needed", workspace_bytes, pl.ws_bytes);
            if (!aligned16(workspace)) return fail(DA_ERR_INVALID_ARGUMENT, "workspace must be 16-byte aligned");
            ws = workspace;
        } else {
            const int rc = cached_workspace(pl.ws_bytes, stream, &ws);
            if (rc != DA_OK) return rc;
        }
    }

    da::SweepParams sp;
    sp.q = q;
    sp.k = k;
    // V absent: the values are the leading dim_v columns of each K row, read with K's pitch
    // (reference csrc/ops/decoding_attn.cpp:30-37).
    sp.v = v ? v : k;
    if (kf.fmt == da::kKvInt4) {
        // two elements to a byte: the kernels do the int8 cache's address arithmetic on twice the address and halve
        // it at the load (da::kKvInt4 in da_common.h)
        sp.k = reinterpret_cast<const void*>(reinterpret_cast<uintptr_t>(sp.k) * 2);
        sp.v = reinterpret_cast<const void*>(reinterpret_cast<uintptr_t>(sp.v) * 2);
    }
    sp.o = o;
    sp.cu_seq_k = cu_seq_k;
    sp.ws_o = reinterpret_cast<float*>(ws);
    // rows of partials: a slot per (sequence, share) on the balanced grid, nsplit per sequence otherwise
    const size_t partial_rows =
        (pl.flat_wgs ? da::flat_slots(pl.flat_wgs, batch) : (size_t)batch * pl.nsplit) * head_q;
    sp.ws_ml = ws ? reinterpret_cast<float*>(ws) + partial_rows * dim_v : nullptr;
    sp.slopes = is_alibi ? alibi_slopes : nullptr;
    sp.k_row = (int64_t)(head_k * dim);
    sp.v_row = v ? (int64_t)(head_k * dim_v) : (int64_t)(head_k * dim);
    sp.v_head = v ? (int)dim_v : (int)dim;
    sp.head_q = (int)head_q;
    sp.head_k = (int)head_k;
    sp.ratio = (int)(head_q / head_k);
    sp.groups = pl.groups;
    sp.nsplit = pl.nsplit;
    sp.chunk = pl.chunk;
    const float scale = softmax_scale > 0.0f ? softmax_scale : (float)(1.0 / std::sqrt((double)dim));
    sp.scale_log2 = scale * da::kLog2e;
    sp.is_alibi = is_alibi ? 1 : 0;
    sp.k_scale = kf.k_scale;
    sp.v_scale = kf.v_scale;
    sp.k_tok = kf.k_tok;
    sp.v_tok = kf.v_tok;
    sp.block_table = pg.table;
    sp.seq_lens = pg.seq_lens;
    sp.page_shift = 0;
    while (pg.table && ((size_t)1 << sp.page_shift) < pg.page_size) ++sp.page_shift;
    sp.max_blocks = (int)pg.max_blocks;
    sp.k_page = (int64_t)pg.k_page;
    sp.v_page = v ? (int64_t)pg.v_page : (int64_t)pg.k_page;
    sp.flat_wgs = pl.flat_wgs;
    sp.flat_step = pl.flat_step;
    sp.flat_min = pl.flat_min;
    sp.flat_unit = pl.flat_unit;
    sp.flat_cu = cu_seq_k;
    sp.batch = (int)batch;
    if (pl.flat_cu_bytes > 0) {
        // paged: positions of the sequences on the balanced grid's line, computed in front of the sweep
        int32_t* const flat_cu = reinterpret_cast<int32_t*>(static_cast<uint8_t*>(ws) + (pl.ws_bytes - pl.flat_cu_bytes));
        const hipError_t pe = da::launch_flat_prefix(pg.seq_lens, (int)batch, 5, flat_cu, stream);
        if (pe != hipSuccess) return fail(DA_ERR_HIP, "prefix kernel launch: %s", hipGetErrorString(pe));
        sp.flat_cu = flat_cu;
    }

    // the latent kernels' split partials: 16-bit block records where whole blocks of 32 heads fit the area sized for
    // fp32 partials of head_q rows (mla_half_partials), un-normalised fp32 rows otherwise
    const bool half_partials = pl.nsplit > 1 && da::mla_half_partials(pl.kind == kKindMfma, pl.rt, head_q, head_k, pl.groups);
    sp.nat_partials = half_partials ? 1 : 0;
    if (pl.kind == kKindMfma && pl.rt == 128 && kf.fmt == 0 && !pl.v_distinct && pl.nsplit > 1 && !half_partials)
        return fail(DA_ERR_WORKSPACE, "the pipelined kernel's 16-bit partials do not fit the workspace's partial area");
    const dim3 grid((unsigned)(pl.flat_wgs ? pl.flat_wgs : pl.nsplit),
                    (unsigned)((pl.wave_per_head ? head_k / 4 : head_k) * pl.groups),
                    (unsigned)(pl.flat_wgs ? 1 : batch));
    hipError_t e;
    if (kf.fmt != 0) {
        if (pl.kind == kKindMfma)
            e = da::launch_mla_kv8(sp, kf.fmt, is_bf16 != 0, pl.rt, grid, stream);
        else if (pl.kind == kKindGroup && per_token && kf.fmt == da::kKvInt8 && !(kf.tok_per64 && dim > 64))
            e = da::launch_gqa_mfma_i8t(sp, is_bf16 != 0, (int)dim, pl.rt, pl.wave_per_head, grid, stream);
        else if (pl.kind == kKindGroup && per_token && kf.tok_per64 && dim > 64)  // (64: one run is the row)
            e = kf.fmt == da::kKvInt8
                    ? da::launch_gqa_mfma_i8g(sp, is_bf16 != 0, (int)dim, pl.rt, pl.wave_per_head, grid, stream)
                    : da::launch_gqa_mfma_i4g(sp, is_bf16 != 0, (int)dim, pl.rt, pl.wave_per_head, grid, stream);
        else if (pl.kind == kKindGroup && per_token)
            e = da::launch_gqa_mfma_i4t(sp, is_bf16 != 0, (int)dim, pl.rt, pl.wave_per_head, grid, stream);
        else if (pl.kind == kKindGroup && kf.fmt == da::kKvInt8)
            e = da::launch_gqa_mfma_i8(sp, is_bf16 != 0, (int)dim, pl.rt, pl.wave_per_head, grid, stream);
        else if (pl.kind == kKindGroup && kf.fmt == da::kKvInt4)
            e = da::launch_gqa_mfma_i4(sp, is_bf16 != 0, (int)dim, pl.rt, pl.wave_per_head, grid, stream);
        else if (pl.kind == kKindGroup)
            e = da::launch_gqa_mfma_kv8(sp, is_bf16 != 0, (int)dim, pl.rt, pl.wave_per_head, grid, stream);
        else
            e = da::launch_sweep_kv8(sp, kf.fmt, is_bf16 != 0, (int)dim, pl.rt, grid, stream);
    } else if (pl.kind == kKindMfma && pl.v_distinct) {
        e = da::launch_mla_vd(sp, is_bf16 != 0, pl.rt, grid, stream);
    } else if (pl.kind == kKindMfma) {
        e = da::launch_mla(sp, is_bf16 != 0, pl.rt, grid, stream);
    } else if (pl.kind == kKindGroup) {
        e = da::launch_gqa_mfma(sp, is_bf16 != 0, (int)dim, pl.rt, pl.wave_per_head, grid, stream);
    } else {
        switch (dim) {
            case 64: e = da::launch_sweep_d64(sp, is_bf16 != 0, pl.rt, grid, stream); break;
            case 96: e = da::launch_sweep_d96(sp, is_bf16 != 0, pl.rt, grid, stream); break;
            case 128: e = da::launch_sweep_d128(sp, is_bf16 != 0, pl.rt, grid, stream); break;
            case 256: e = da::launch_sweep_d256(sp, is_bf16 != 0, pl.rt, grid, stream); break;
            default: e = da::launch_sweep_d576(sp, is_bf16 != 0, pl.rt, grid, stream); break;
        }
    }
    if (e != hipSuccess) return fail(DA_ERR_HIP, "sweep kernel launch: %s", hipGetErrorString(e));

    if ((pl.nsplit > 1 || pl.flat_wgs) && !kf.sweep_only) {
        da::ReduceParams rp;
        rp.o = o;
        rp.cu_seq_k = cu_seq_k;
        rp.seq_lens = pg.seq_lens;
        rp.ws_o = sp.ws_o;
        rp.ws_ml = sp.ws_ml;
        rp.head_q = (int)head_q;
        rp.dim_v = (int)dim_v;
        rp.nsplit = pl.flat_wgs ? pl.flat_partials : pl.nsplit;
        rp.chunk = pl.chunk;
        rp.flat_wgs = pl.flat_wgs;
        rp.flat_step = pl.flat_step;
        rp.flat_min = pl.flat_min;
        rp.flat_cu = sp.flat_cu;
        rp.batch = (int)batch;
        // (the balanced grid's partial slots are known only once the sequences' positions have been read)
        rp.early = pl.ws_bytes <= ((size_t)8 << 20) && !pl.flat_wgs ? 1 : 0;
        rp.half_partials = half_partials ? 1 : 0;
        rp.ratio = sp.ratio;
        rp.groups = pl.groups;
        rp.nat_waves = half_partials ? pl.rt / 32 : 0;
        rp.nat_blocks = half_partials ? da::nat_blocks((int)head_k, pl.groups, pl.rt / 32) : 0;
        e = da::launch_reduce(rp, is_bf16 != 0, (int)(batch * head_q), stream);
        if (e != hipSuccess) return fail(DA_ERR_HIP, "merge kernel launch: %s", hipGetErrorString(e));
    }
    return DA_OK;
}

int check_paging(const int32_t* block_table, const int32_t* seq_lens, size_t max_seq_k, size_t head_k, size_t dim,
                 size_t dim_v, size_t page_size, size_t max_blocks_per_seq, size_t k_page_stride, size_t v_page_stride,
                 bool has_v, Paging* pg) {
    if (!block_table) return fail(DA_ERR_INVALID_ARGUMENT, "block_table is null");
    if (!seq_lens) return fail(DA_ERR_INVALID_ARGUMENT, "seq_lens is null");
    if (page_size == 0 || (page_size & (page_size - 1)) != 0 || page_size > ((size_t)1 << 20))
        return fail(DA_ERR_INVALID_ARGUMENT, "page_size (%zu) must be a power of two", page_size);
    if (max_blocks_per_seq * page_size < max_seq_k)
        return fail(DA_ERR_INVALID_ARGUMENT, "block table rows (%zu pages of %zu tokens) cannot hold max_seq_k %zu",
                    max_blocks_per_seq, page_size, max_seq_k);
    if (max_blocks_per_seq > (size_t)INT32_MAX)
        return fail(DA_ERR_INVALID_ARGUMENT, "max_blocks_per_seq (%zu) out of range", max_blocks_per_seq);
    // a multiple of 16 elements keeps every row 16-byte aligned for 16-bit and for FP8 elements alike
    if (k_page_stride < page_size * head_k * dim || k_page_stride % 16 != 0)
        return fail(DA_ERR_INVALID_ARGUMENT,
                    "k_page_stride (%zu elements) must be a multiple of 16 and at least page_size * head_k * dim",
                    k_page_stride);
    if (has_v && (v_page_stride < page_size * head_k * dim_v || v_page_stride % 16 != 0))
        return fail(DA_ERR_INVALID_ARGUMENT,
                    "v_page_stride (%zu elements) must be a multiple of 16 and at least page_size * head_k * dim_v",
                    v_page_stride);
    pg->table = block_table;
    pg->seq_lens = seq_lens;
    pg->page_size = page_size;
    pg->max_blocks = max_blocks_per_seq;
    pg->k_page = k_page_stride;
    pg->v_page = v_page_stride;
    return DA_OK;
}

}  // namespace

extern "C" {

int da_decoding_attn_ex(const void* q, const void* k, const void* v, void* o, const int32_t* cu_seq_k,
                        size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                        int is_alibi, int is_bf16, float softmax_scale, const float* alibi_slopes, size_t total_k,
                        void* workspace, size_t workspace_bytes, void* hip_stream) {
    return run_attention(q, k, v, o, cu_seq_k, Paging{}, KvFormat{}, max_seq_k, batch, head_q, head_k, dim, dim_v, is_alibi,
                         is_bf16, softmax_scale, alibi_slopes, total_k, workspace, workspace_bytes, hip_stream);
}

#ifdef DA_BUILD_PROBES
// (libdecoding_attn_probe.so only, declared in decoding_attn_probe.h)
int da_probe_sweep_only(const void* q, const void* k, const void* v, void* o, const int32_t* cu_seq_k, size_t max_seq_k,
                        size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v, int is_alibi, int is_bf16,
                        size_t total_k, void* workspace, size_t workspace_bytes, void* hip_stream) {
    KvFormat kf;
    kf.sweep_only = true;
    return run_attention(q, k, v, o, cu_seq_k, Paging{}, kf, max_seq_k, batch, head_q, head_k, dim, dim_v, is_alibi,
                         is_bf16, 0.0f, nullptr, total_k, workspace, workspace_bytes, hip_stream);
}

// Overrides one planner tunable of this (probe) library in the running process, for sweeps over plans; not
// thread-safe against concurrent calls.
int da_probe_set_tunable(const char* name, int value) {
    if (!name) return DA_ERR_INVALID_ARGUMENT;
    Tunables& t = tun_storage();
    const std::string n(name);
    if (n == "DA_NSPLIT") t.nsplit = value;
    else if (n == "DA_MLA_HEADS") t.mla_heads = value;
    else if (n == "DA_MLA_GROUP_SMALL") t.mla_group_small = value;
    else if (n == "DA_MLA_GROUP_HEADS") t.mla_group_heads = value;
    else if (n == "DA_MFMA_TARGET_WGS") t.mfma_target_wgs = value;
    else if (n == "DA_MFMA_SMALL_WGS") t.mfma_small_wgs = value;
    else if (n == "DA_GROUP_MIN_RATIO") t.group_min_ratio = value;
    else if (n == "DA_FORCE_KIND") t.force_kind = value;
    else return fail(DA_ERR_INVALID_ARGUMENT, "unknown tunable %s", name);
    return DA_OK;
}
#endif

int da_decoding_attn_paged(const void* q, const void* k_pages, const void* v_pages, void* o,
                           const int32_t* block_table, const int32_t* seq_lens, size_t max_seq_k, size_t batch,
                           size_t head_q, size_t head_k, size_t dim, size_t dim_v, size_t page_size,
                           size_t max_blocks_per_seq, size_t k_page_stride, size_t v_page_stride, int is_alibi,
                           int is_bf16, float softmax_scale, const float* alibi_slopes, size_t total_k,
                           void* workspace, size_t workspace_bytes, void* hip_stream) {
    Paging pg;
    const int rc = check_paging(block_table, seq_lens, max_seq_k, head_k, dim, dim_v, page_size, max_blocks_per_seq,
                                k_page_stride, v_page_stride, v_pages != nullptr, &pg);
    if (rc != DA_OK) return rc;
    return run_attention(q, k_pages, v_pages, o, nullptr, pg, KvFormat{}, max_seq_k, batch, head_q, head_k, dim, dim_v,
                         is_alibi, is_bf16, softmax_scale, alibi_slopes, total_k, workspace, workspace_bytes,
                         hip_stream);
}

int da_decoding_attn_fp8kv(const void* q, const void* k8, const void* v8, void* o, const int32_t* cu_seq_k,
                           size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                           int is_alibi, int is_bf16, float softmax_scale, const float* alibi_slopes,
                           const float* k_scale, const float* v_scale, size_t total_k, void* workspace,
                           size_t workspace_bytes, void* hip_stream) {
    return run_attention(q, k8, v8, o, cu_seq_k, Paging{}, kv8_format(da::kKvFp8, k_scale, v_scale), max_seq_k, batch,
                         head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes, total_k,
                         workspace, workspace_bytes, hip_stream);
}

int da_decoding_attn_int8kv(const void* q, const void* k8, const void* v8, void* o, const int32_t* cu_seq_k,
                            size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                            int is_alibi, int is_bf16, float softmax_scale, const float* alibi_slopes,
                            const float* k_scale, const float* v_scale, size_t total_k, void* workspace,
                            size_t workspace_bytes, void* hip_stream) {
    return run_attention(q, k8, v8, o, cu_seq_k, Paging{}, kv8_format(da::kKvInt8, k_scale, v_scale), max_seq_k, batch,
                         head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes, total_k,
                         workspace, workspace_bytes, hip_stream);
}

int da_decoding_attn_paged_fp8kv(const void* q, const void* k_pages, const void* v_pages, void* o,
                                 const int32_t* block_table, const int32_t* seq_lens, size_t max_seq_k, size_t batch,
                                 size_t head_q, size_t head_k, size_t dim, size_t dim_v, size_t page_size,
                                 size_t max_blocks_per_seq, size_t k_page_stride, size_t v_page_stride, int is_alibi,
                                 int is_bf16, float softmax_scale, const float* alibi_slopes, const float* k_scale,
                                 const float* v_scale, size_t total_k, void* workspace, size_t workspace_bytes,
                                 void* hip_stream) {
    Paging pg;
    const int rc = check_paging(block_table, seq_lens, max_seq_k, head_k, dim, dim_v, page_size, max_blocks_per_seq,
                                k_page_stride, v_page_stride, v_pages != nullptr, &pg);
    if (rc != DA_OK) return rc;
    return run_attention(q, k_pages, v_pages, o, nullptr, pg, kv8_format(da::kKvFp8, k_scale, v_scale), max_seq_k,
                         batch, head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes, total_k,
                         workspace, workspace_bytes, hip_stream);
}

int da_decoding_attn_paged_int8kv(const void* q, const void* k_pages, const void* v_pages, void* o,
                                  const int32_t* block_table, const int32_t* seq_lens, size_t max_seq_k, size_t batch,
                                  size_t head_q, size_t head_k, size_t dim, size_t dim_v, size_t page_size,
                                  size_t max_blocks_per_seq, size_t k_page_stride, size_t v_page_stride, int is_alibi,
                                  int is_bf16, float softmax_scale, const float* alibi_slopes, const float* k_scale,
                                  const float* v_scale, size_t total_k, void* workspace, size_t workspace_bytes,
                                  void* hip_stream) {
    Paging pg;
    const int rc = check_paging(block_table, seq_lens, max_seq_k, head_k, dim, dim_v, page_size, max_blocks_per_seq,
                                k_page_stride, v_page_stride, v_pages != nullptr, &pg);
    if (rc != DA_OK) return rc;
    return run_attention(q, k_pages, v_pages, o, nullptr, pg, kv8_format(da::kKvInt8, k_scale, v_scale), max_seq_k,
                         batch, head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes, total_k,
                         workspace, workspace_bytes, hip_stream);
}

int da_decoding_attn_int4kv(const void* q, const void* k4, const void* v4, void* o, const int32_t* cu_seq_k,
                            size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                            int is_alibi, int is_bf16, float softmax_scale, const float* alibi_slopes,
                            const float* k_scale, const float* v_scale, size_t total_k, void* workspace,
                            size_t workspace_bytes, void* hip_stream) {
    return run_attention(q, k4, v4, o, cu_seq_k, Paging{}, kv8_format(da::kKvInt4, k_scale, v_scale), max_seq_k, batch,
                         head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes, total_k,
                         workspace, workspace_bytes, hip_stream);
}

int da_decoding_attn_paged_int4kv(const void* q, const void* k_pages, const void* v_pages, void* o,
                                  const int32_t* block_table, const int32_t* seq_lens, size_t max_seq_k, size_t batch,
                                  size_t head_q, size_t head_k, size_t dim, size_t dim_v, size_t page_size,
                                  size_t max_blocks_per_seq, size_t k_page_stride, size_t v_page_stride, int is_alibi,
                                  int is_bf16, float softmax_scale, const float* alibi_slopes, const float* k_scale,
                                  const float* v_scale, size_t total_k, void* workspace, size_t workspace_bytes,
                                  void* hip_stream) {
    Paging pg;
    const int rc = check_paging(block_table, seq_lens, max_seq_k, head_k, dim, dim_v, page_size, max_blocks_per_seq,
                                k_page_stride, v_page_stride, v_pages != nullptr, &pg);
    if (rc != DA_OK) return rc;
    return run_attention(q, k_pages, v_pages, o, nullptr, pg, kv8_format(da::kKvInt4, k_scale, v_scale), max_seq_k,
                         batch, head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes, total_k,
                         workspace, workspace_bytes, hip_stream);
}

size_t da_workspace_bytes_int4kv(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                 size_t dim_v, size_t total_k, size_t page_size) {
    if (head_k == 0 || head_q % head_k != 0 || !supported_dims(dim, dim_v)) return 0;
    // (as the FP8 cache's plans, but the latent form always on the grouped kernel)
    const size_t a = plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, false, total_k, page_size, true, true);
    const size_t b = plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, true, total_k, page_size, true, true);
    return a > b ? a : b;
}

int da_decoding_attn_int4kv_tok(const void* q, const void* k4, const void* v4, void* o, const int32_t* cu_seq_k,
                                size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                int is_alibi, int is_bf16, float softmax_scale, const float* alibi_slopes,
                                const float* k_params, const float* v_params, size_t total_k, void* workspace,
                                size_t workspace_bytes, void* hip_stream) {
    if (!k_params || !v_params) return fail(DA_ERR_INVALID_ARGUMENT, "k_params or v_params is null");
    return run_attention(q, k4, v4, o, cu_seq_k, Paging{}, per_token_format(da::kKvInt4, k_params, v_params), max_seq_k,
                         batch, head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes, total_k,
                         workspace, workspace_bytes, hip_stream);
}

int da_decoding_attn_paged_int4kv_tok(const void* q, const void* k_pages, const void* v_pages, void* o,
                                      const int32_t* block_table, const int32_t* seq_lens, size_t max_seq_k,
                                      size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                      size_t page_size, size_t max_blocks_per_seq, size_t k_page_stride,
                                      size_t v_page_stride, int is_alibi, int is_bf16, float softmax_scale,
                                      const float* alibi_slopes, const float* k_params, const float* v_params,
                                      size_t total_k, void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (!k_params || !v_params) return fail(DA_ERR_INVALID_ARGUMENT, "k_params or v_params is null");
    Paging pg;
    const int rc = check_paging(block_table, seq_lens, max_seq_k, head_k, dim, dim_v, page_size, max_blocks_per_seq,
                                k_page_stride, v_page_stride, v_pages != nullptr, &pg);
    if (rc != DA_OK) return rc;
    return run_attention(q, k_pages, v_pages, o, nullptr, pg, per_token_format(da::kKvInt4, k_params, v_params),
                         max_seq_k, batch, head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes,
                         total_k, workspace, workspace_bytes, hip_stream);
}

size_t da_workspace_bytes_int4kv_tok(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                     size_t dim_v, size_t total_k, size_t page_size) {
    if (head_k == 0 || head_q % head_k != 0 || dim != dim_v || (dim != 64 && dim != 128 && dim != 256)) return 0;
    return plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, true, total_k, page_size, true, true, true);
}

int da_decoding_attn_int4kv_grp64(const void* q, const void* k4, const void* v4, void* o, const int32_t* cu_seq_k,
                                  size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                  size_t dim_v, int is_alibi, int is_bf16, float softmax_scale,
                                  const float* alibi_slopes, const float* k_params, const float* v_params,
                                  size_t total_k, void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (!k_params || !v_params) return fail(DA_ERR_INVALID_ARGUMENT, "k_params or v_params is null");
    return run_attention(q, k4, v4, o, cu_seq_k, Paging{}, per_token_format(da::kKvInt4, k_params, v_params, true),
                         max_seq_k, batch, head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes,
                         total_k, workspace, workspace_bytes, hip_stream);
}

int da_decoding_attn_paged_int4kv_grp64(const void* q, const void* k_pages, const void* v_pages, void* o,
                                        const int32_t* block_table, const int32_t* seq_lens, size_t max_seq_k,
                                        size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                        size_t page_size, size_t max_blocks_per_seq, size_t k_page_stride,
                                        size_t v_page_stride, int is_alibi, int is_bf16, float softmax_scale,
                                        const float* alibi_slopes, const float* k_params, const float* v_params,
                                        size_t total_k, void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (!k_params || !v_params) return fail(DA_ERR_INVALID_ARGUMENT, "k_params or v_params is null");
    Paging pg;
    const int rc = check_paging(block_table, seq_lens, max_seq_k, head_k, dim, dim_v, page_size, max_blocks_per_seq,
                                k_page_stride, v_page_stride, v_pages != nullptr, &pg);
    if (rc != DA_OK) return rc;
    return run_attention(q, k_pages, v_pages, o, nullptr, pg, per_token_format(da::kKvInt4, k_params, v_params, true),
                         max_seq_k, batch, head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes,
                         total_k, workspace, workspace_bytes, hip_stream);
}

size_t da_workspace_bytes_int4kv_grp64(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                       size_t dim_v, size_t total_k, size_t page_size) {
    if (head_k == 0 || head_q % head_k != 0 || dim != dim_v || (dim != 64 && dim != 128 && dim != 256)) return 0;
    return plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, true, total_k, page_size, true, true, 2);
}

int da_decoding_attn_int8kv_grp64(const void* q, const void* k8, const void* v8, void* o, const int32_t* cu_seq_k,
                                  size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                  size_t dim_v, int is_alibi, int is_bf16, float softmax_scale,
                                  const float* alibi_slopes, const float* k_params, const float* v_params,
                                  size_t total_k, void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (!k_params || !v_params) return fail(DA_ERR_INVALID_ARGUMENT, "k_params or v_params is null");
    return run_attention(q, k8, v8, o, cu_seq_k, Paging{}, per_token_format(da::kKvInt8, k_params, v_params, true),
                         max_seq_k, batch, head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes,
                         total_k, workspace, workspace_bytes, hip_stream);
}

int da_decoding_attn_paged_int8kv_grp64(const void* q, const void* k_pages, const void* v_pages, void* o,
                                        const int32_t* block_table, const int32_t* seq_lens, size_t max_seq_k,
                                        size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                        size_t page_size, size_t max_blocks_per_seq, size_t k_page_stride,
                                        size_t v_page_stride, int is_alibi, int is_bf16, float softmax_scale,
                                        const float* alibi_slopes, const float* k_params, const float* v_params,
                                        size_t total_k, void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (!k_params || !v_params) return fail(DA_ERR_INVALID_ARGUMENT, "k_params or v_params is null");
    Paging pg;
    const int rc = check_paging(block_table, seq_lens, max_seq_k, head_k, dim, dim_v, page_size, max_blocks_per_seq,
                                k_page_stride, v_page_stride, v_pages != nullptr, &pg);
    if (rc != DA_OK) return rc;
    return run_attention(q, k_pages, v_pages, o, nullptr, pg, per_token_format(da::kKvInt8, k_params, v_params, true),
                         max_seq_k, batch, head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes,
                         total_k, workspace, workspace_bytes, hip_stream);
}

size_t da_workspace_bytes_int8kv_grp64(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                       size_t dim_v, size_t total_k, size_t page_size) {
    if (head_k == 0 || head_q % head_k != 0 || dim != dim_v || (dim != 64 && dim != 128 && dim != 256)) return 0;
    return plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, true, total_k, page_size, true, false, 2);
}

int da_decoding_attn_int8kv_tok(const void* q, const void* k8, const void* v8, void* o, const int32_t* cu_seq_k,
                                size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                int is_alibi, int is_bf16, float softmax_scale, const float* alibi_slopes,
                                const float* k_params, const float* v_params, size_t total_k, void* workspace,
                                size_t workspace_bytes, void* hip_stream) {
    if (!k_params || !v_params) return fail(DA_ERR_INVALID_ARGUMENT, "k_params or v_params is null");
    return run_attention(q, k8, v8, o, cu_seq_k, Paging{}, per_token_format(da::kKvInt8, k_params, v_params), max_seq_k,
                         batch, head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes, total_k,
                         workspace, workspace_bytes, hip_stream);
}

int da_decoding_attn_paged_int8kv_tok(const void* q, const void* k_pages, const void* v_pages, void* o,
                                      const int32_t* block_table, const int32_t* seq_lens, size_t max_seq_k,
                                      size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                      size_t page_size, size_t max_blocks_per_seq, size_t k_page_stride,
                                      size_t v_page_stride, int is_alibi, int is_bf16, float softmax_scale,
                                      const float* alibi_slopes, const float* k_params, const float* v_params,
                                      size_t total_k, void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (!k_params || !v_params) return fail(DA_ERR_INVALID_ARGUMENT, "k_params or v_params is null");
    Paging pg;
    const int rc = check_paging(block_table, seq_lens, max_seq_k, head_k, dim, dim_v, page_size, max_blocks_per_seq,
                                k_page_stride, v_page_stride, v_pages != nullptr, &pg);
    if (rc != DA_OK) return rc;
    return run_attention(q, k_pages, v_pages, o, nullptr, pg, per_token_format(da::kKvInt8, k_params, v_params),
                         max_seq_k, batch, head_q, head_k, dim, dim_v, is_alibi, is_bf16, softmax_scale, alibi_slopes,
                         total_k, workspace, workspace_bytes, hip_stream);
}

size_t da_workspace_bytes_int8kv_tok(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                     size_t dim_v, size_t total_k, size_t page_size) {
    if (head_k == 0 || head_q % head_k != 0 || dim != dim_v || (dim != 64 && dim != 128 && dim != 256)) return 0;
    return plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, true, total_k, page_size, true, false, true);
}

int da_release_workspaces(void) { return release_cached_workspaces(true); }

size_t da_noalloc_workspace_limit(void) { return kScratchBytes; }

int da_decoding_attn_noalloc(const void* q, const void* k, const void* v, void* o, const int32_t* cu_seq_k,
                             size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                             int is_alibi, int is_bf16, float softmax_scale, const float* alibi_slopes, size_t total_k,
                             void* hip_stream) {
    // the split partials go to the static device array; a plan that needs more than it holds is refused here, with
    // the numbers, before anything is enqueued (the remaining argument checks are run_attention's)
    if (head_k != 0 && head_q % head_k == 0 && supported_dims(dim, dim_v) && batch > 0) {
        const size_t need = plan_ws_bytes(max_seq_k, batch, head_q, head_k, dim, dim_v, v != nullptr, total_k);
        if (need > kScratchBytes)
            return fail(DA_ERR_WORKSPACE,
                        "this shape needs %zu bytes of split workspace, more than the %zu bytes of the static array "
                        "da_decoding_attn_noalloc works in; use da_decoding_attn_ex with a workspace of your own",
                        need, kScratchBytes);
    }
    void* ws = nullptr;
    const int rc = scratch_on_current_device(&ws);
    if (rc != DA_OK) return rc;
    return run_attention(q, k, v, o, cu_seq_k, Paging{}, KvFormat{}, max_seq_k, batch, head_q, head_k, dim, dim_v, is_alibi,
                         is_bf16, softmax_scale, alibi_slopes, total_k, ws, kScratchBytes, hip_stream);
}

int da_decoding_attn(const void* q, const void* k, const void* v, void* o, const int32_t* cu_seq_k, size_t max_seq_k,
                     size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v, int is_alibi, int is_bf16,
                     void* hip_stream) {
    return da_decoding_attn_ex(q, k, v, o, cu_seq_k, max_seq_k, batch, head_q, head_k, dim, dim_v, is_alibi, is_bf16,
                               0.0f, nullptr, 0, nullptr, 0, hip_stream);
}

}  // extern "C"
