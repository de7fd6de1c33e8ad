/*
 * C-ABI of libdecoding_attn_hip.so — single-query ("decoding") attention for MI355X (gfx950).
 *
 *   O[b,h,:] = softmax_j( scale * <Q[b,h,:], K[cu[b]+j, h/ratio, :]> + slope_h * (j - (len_b - 1)) ) . V[cu[b]+j, h/ratio, :]
 *
 * for MHA / GQA / MQA (dim == dim_v in {64, 96, 128, 256}) and the latent MLA form
 * (dim 576, dim_v 512, v == NULL: V is the first 512 columns of every K row).
 *
 * All pointers are device pointers unless said otherwise; every call only enqueues work on
 * `hip_stream` (a hipStream_t passed as void*, NULL = the default stream) and returns without
 * synchronising.  Functions return 0 on success and a DA_ERR_* code otherwise; the message is
 * available from da_last_error() on the calling thread.  Nothing here calls exit().
 */
#ifndef DECODING_ATTN_HIP_H_
#define DECODING_ATTN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DA_OK 0
#define DA_ERR_INVALID_ARGUMENT 1 /* null pointer, misaligned pointer, head_q % head_k != 0, dim > 576, dim_v > 512 */
#define DA_ERR_UNSUPPORTED 2      /* (dim, dim_v) pair outside the supported set */
#define DA_ERR_WORKSPACE 3        /* caller workspace smaller than da_workspace_bytes() */
#define DA_ERR_HIP 4              /* a HIP runtime call failed */

/*
 * Replaces the reference's
 *   void decoding_attn(void *q, void *k, void *v, void *o, int *cu_seq_k, size_t max_seq_k, size_t batch,
 *                      size_t head_q, size_t head_k, size_t dim, size_t dim_v, bool is_alibi, bool is_bf16,
 *                      cudaStream_t stream)                         (reference csrc/ops/decoding_attn.h:29-30,
 *                                                                    csrc/ops/decoding_attn.cpp:70-76)
 * Same argument order and meaning; softmax scale is 1/sqrt(dim) (decoding_attn.cpp:54) and the ALiBi slope of
 * head h is 2^(-8(h+1)/head_q) (csrc/kernel/decoding_attn/block_info.h:21).
 *   q [batch, head_q, dim]; k [total_k, head_k, dim]; v [total_k, head_k, dim_v] or NULL (MLA);
 *   o [batch, head_q, dim_v]; cu_seq_k [batch + 1] int32 prefix offsets; q/k/v/o 16-byte aligned.
 * Split-sequence partials live in a workspace the library keeps per (device, stream) and grows on demand
 * (growth calls hipMalloc; steady-state calls allocate nothing); da_release_workspaces() frees them, and they are
 * freed at process exit or when the library is unloaded.  Use da_decoding_attn_ex to bring your own.
 */
int da_decoding_attn(const void *q, const void *k, const void *v, void *o, const int32_t *cu_seq_k, size_t max_seq_k,
                     size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v, int is_alibi, int is_bf16,
                     void *hip_stream);

/*
 * Same operation with the two constants of the reference exposed as arguments and a caller-owned workspace.
 * Extends reference csrc/ops/decoding_attn.cpp:13-62 (set_dmha_fwd_params), which hard-codes both.
 *   softmax_scale  <= 0 selects 1/sqrt(dim)
 *   alibi_slopes   device float[head_q] or NULL for the closed form; read only when is_alibi != 0
 *   total_k        number of key tokens (cu_seq_k[batch]) if the caller knows it on the host, else 0.  Only a
 *                  hint: a batch that is much shorter than batch * max_seq_k is cut so that it balances (shorter
 *                  sequence splits, or equal shares of the concatenated tokens across sequence boundaries);
 *                  results are correct for any value, also one that is not the true count.  Pass the same value
 *                  to da_workspace_bytes.
 *   workspace      device buffer of at least da_workspace_bytes(...) bytes, 16-byte aligned, or NULL to use the
 *                  library's cached one
 */
int da_decoding_attn_ex(const void *q, const void *k, const void *v, void *o, const int32_t *cu_seq_k,
                        size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                        int is_alibi, int is_bf16, float softmax_scale, const float *alibi_slopes, size_t total_k,
                        void *workspace, size_t workspace_bytes, void *hip_stream);

/*
 * Frees the workspaces da_decoding_attn (and da_decoding_attn_ex with workspace == NULL) keeps per (device, stream),
 * for long-lived processes that cycle through streams.  The caller must have synchronised every stream whose calls
 * may still use one.  No counterpart in the reference (its kernel needs no workspace).
 */
int da_release_workspaces(void);

/*
 * da_decoding_attn_ex for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  No counterpart in the reference.  The split partials go to a static device array of
 * da_noalloc_workspace_limit() bytes (80 MiB) that every GPU the library is loaded on holds until the process ends;
 * the call allocates nothing, on the device or through any library, and returns DA_ERR_WORKSPACE (nothing enqueued)
 * for a shape whose plan needs more.  All calls on one GPU share that array: calls that overlap on one GPU (two
 * streams, two threads) race on it; calls on one stream do not.  The first call for a shape on a device looks up the
 * array's address there and raises the chosen kernel's LDS limit: make one warm-up call per shape and device outside
 * any graph capture; every later call only enqueues kernels.
 */
int da_decoding_attn_noalloc(const void *q, const void *k, const void *v, void *o, const int32_t *cu_seq_k,
                             size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                             int is_alibi, int is_bf16, float softmax_scale, const float *alibi_slopes, size_t total_k,
                             void *hip_stream);
size_t da_noalloc_workspace_limit(void);

/*
 * Bytes of workspace da_decoding_attn_ex needs for this shape (0 when the sequence is not split).
 * No counterpart in the reference, whose kernel never splits a sequence
 * (csrc/kernel/decoding_attn/decoding_fwd_launch_template.h:12-31).
 */
size_t da_workspace_bytes(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                          size_t total_k);

/*
 * The same attention over a paged K/V cache: K and V live in page pools and each sequence lists its pages.
 * The reference has no paged path of its own; these are the layouts of the libraries it is benchmarked against
 * (benchmarks/python/benchmark_decoding_attn.py:129-151: a [pages, 2, page_size, head_k, dim] pool with one index
 * array per batch; :182-187: a [blocks, 64, 1, 576] latent pool with a [batch, max_blocks] block table).
 *
 *   k_pages        [num_pages, page_size, head_k, dim], consecutive pages k_page_stride elements apart
 *   v_pages        [num_pages, page_size, head_k, dim_v], pages v_page_stride elements apart, or NULL when V is the
 *                  first dim_v columns of each K row (MLA).  A combined [pages, 2, page_size, head_k, dim] pool is
 *                  k_pages = pool, v_pages = pool + page_size * head_k * dim, both strides 2 * page_size * head_k * dim.
 *   block_table    device, int32 [batch, max_blocks_per_seq]: page ids of each sequence in token order; entries
 *                  past ceil(seq_lens[b] / page_size) are not read
 *   seq_lens       device, int32 [batch]: key tokens of each sequence (0 gives zero output rows)
 *   page_size      tokens per page, a power of two (1 included).  All sizes run on the same kernels as the packed
 *                  layout: whole tiles from pages of 32 tokens and more, two runs per tile from 16-token pages,
 *                  a table lookup per row below that.
 * The remaining arguments are those of da_decoding_attn_ex; workspace size from da_workspace_bytes_paged.
 */
int da_decoding_attn_paged(const void *q, const void *k_pages, const void *v_pages, void *o,
                           const int32_t *block_table, const int32_t *seq_lens, size_t max_seq_k, size_t batch,
                           size_t head_q, size_t head_k, size_t dim, size_t dim_v, size_t page_size,
                           size_t max_blocks_per_seq, size_t k_page_stride, size_t v_page_stride, int is_alibi,
                           int is_bf16, float softmax_scale, const float *alibi_slopes, size_t total_k,
                           void *workspace, size_t workspace_bytes, void *hip_stream);

size_t da_workspace_bytes_paged(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                size_t dim_v, size_t total_k, size_t page_size);

/*
 * The same attention over an FP8 K/V cache (the reference lists K/V quantisation as future work, README.md:154-156;
 * it has no such path).  q and o stay fp16 / bf16 (is_bf16); k8 and v8 hold OCP FP8 e4m3 values, one byte per
 * element, in the layouts of the 16-bit entry points (packed [total_k, head_k, dim] with cu_seq_k, or page pools
 * with a block table; strides are in elements).
 *
 *   k_scale, v_scale   device, float [head_k], or NULL for 1: K = k_scale[hk] * fp8 value, V likewise.  FP8
 *                      values convert exactly to fp16 and bf16, so the matrix arithmetic is that of the 16-bit
 *                      path; k_scale is folded into the softmax scale and v_scale into the final normalisation,
 *                      both in fp32.
 * v8 == NULL means V is the first dim_v columns of each K row.  Head dims (64,64), (128,128), (256,256) run on
 * the grouped MFMA kernel and (576,512) with v8 == NULL on the latent MFMA kernel (up to 16 query heads: on the
 * grouped kernel), as the 16-bit forms do; (96,96) runs on the VALU sweep.  Workspace size from da_workspace_bytes_fp8kv (page_size 0 = packed layout).
 */
int da_decoding_attn_fp8kv(const void *q, const void *k8, const void *v8, void *o, const int32_t *cu_seq_k,
                           size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                           int is_alibi, int is_bf16, float softmax_scale, const float *alibi_slopes,
                           const float *k_scale, const float *v_scale, size_t total_k, void *workspace,
                           size_t workspace_bytes, void *hip_stream);

int da_decoding_attn_paged_fp8kv(const void *q, const void *k_pages, const void *v_pages, void *o,
                                 const int32_t *block_table, const int32_t *seq_lens, size_t max_seq_k, size_t batch,
                                 size_t head_q, size_t head_k, size_t dim, size_t dim_v, size_t page_size,
                                 size_t max_blocks_per_seq, size_t k_page_stride, size_t v_page_stride, int is_alibi,
                                 int is_bf16, float softmax_scale, const float *alibi_slopes, const float *k_scale,
                                 const float *v_scale, size_t total_k, void *workspace, size_t workspace_bytes,
                                 void *hip_stream);

size_t da_workspace_bytes_fp8kv(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                size_t dim_v, size_t total_k, size_t page_size);

/*
 * The same attention over an int8 K/V cache (the second format of the reference's quantisation to-do,
 * README.md:154-156; it has no such path).  k8 and v8 hold two's-complement int8 values, symmetric quantisation
 * with one factor per KV head: K = k_scale[hk] * int8 value, V likewise (NULL for 1).  Layouts, arguments and
 * kernels are those of the FP8 entry points above; int8 values convert exactly to fp16 and bf16 too, so with unit
 * scales the result equals the 16-bit call's on the widened values bit for bit.
 */
int da_decoding_attn_int8kv(const void *q, const void *k8, const void *v8, void *o, const int32_t *cu_seq_k,
                            size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                            int is_alibi, int is_bf16, float softmax_scale, const float *alibi_slopes,
                            const float *k_scale, const float *v_scale, size_t total_k, void *workspace,
                            size_t workspace_bytes, void *hip_stream);

int da_decoding_attn_paged_int8kv(const void *q, const void *k_pages, const void *v_pages, void *o,
                                  const int32_t *block_table, const int32_t *seq_lens, size_t max_seq_k,
                                  size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                  size_t page_size, size_t max_blocks_per_seq, size_t k_page_stride,
                                  size_t v_page_stride, int is_alibi, int is_bf16, float softmax_scale,
                                  const float *alibi_slopes, const float *k_scale, const float *v_scale,
                                  size_t total_k, void *workspace, size_t workspace_bytes, void *hip_stream);

size_t da_workspace_bytes_int8kv(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                 size_t dim_v, size_t total_k, size_t page_size);

/*
 * The same attention over an int4 K/V cache (the third format of the reference's quantisation to-do,
 * README.md:154-156; it has no such path).  k4 and v4 hold two's-complement four-bit integers (-8 .. 7), two to a
 * byte, element 2 i of a row in the low half of byte i: k4 [total_k, head_k, dim / 2] bytes, v4 [total_k, head_k,
 * dim_v / 2] bytes or NULL at (576, 512) (V = the leading 512 elements of each K row), 16-byte aligned; page pools
 * likewise, with page strides counted in ELEMENTS as for the other formats.  Symmetric quantisation with one factor
 * per KV head: K = k_scale[hk] * int4 value, V likewise (NULL for 1).  Other arguments as for the FP8 entry points.
 * The values convert exactly to fp16 and bf16, so the only error added is the cache's own quantisation.
 * (576, 512) always runs on the grouped-head kernel, as ceil(heads / 16) groups per sequence that read the same rows
 * (the latent kernel has no int4 form): correct at any head count, but slower than the 8-bit formats from 64 heads up.
 */
int da_decoding_attn_int4kv(const void *q, const void *k4, const void *v4, void *o, const int32_t *cu_seq_k,
                            size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                            int is_alibi, int is_bf16, float softmax_scale, const float *alibi_slopes,
                            const float *k_scale, const float *v_scale, size_t total_k, void *workspace,
                            size_t workspace_bytes, void *hip_stream);

int da_decoding_attn_paged_int4kv(const void *q, const void *k_pages, const void *v_pages, void *o,
                                  const int32_t *block_table, const int32_t *seq_lens, size_t max_seq_k,
                                  size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                  size_t page_size, size_t max_blocks_per_seq, size_t k_page_stride,
                                  size_t v_page_stride, int is_alibi, int is_bf16, float softmax_scale,
                                  const float *alibi_slopes, const float *k_scale, const float *v_scale,
                                  size_t total_k, void *workspace, size_t workspace_bytes, void *hip_stream);

size_t da_workspace_bytes_int4kv(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                 size_t dim_v, size_t total_k, size_t page_size);

/*
 * int4 K/V with a (scale, zero) pair per (token, KV head) -- asymmetric per-token quantisation, the group-wise scheme
 * with the head dimension as the group (the reference's quantisation to-do, README.md:154-156, names no scheme; it
 * has no such path).  k4 and v4 as for da_decoding_attn_int4kv, both required; k_params and v_params hold float pairs
 * laid out like the rows they belong to: [total_k, head_k, 2] for the packed layout, [pages, page_size, head_k, 2]
 * (dense, indexed through the same block table) for page pools, 8-byte aligned:
 *   K[t, hk, c] = k_params[t, hk, 0] * (int4 value - k_params[t, hk, 1]),   V likewise with v_params.
 * Head dims (64,64), (128,128) and (256,256), any head grouping, every page size, ALiBi; all shapes run on the
 * grouped-head kernel, whose matrix instructions work on the integers: the score tile takes one multiply-add per
 * element with the sum of the head's q row (q . K[t] = scale (q . n[t] - zero sum(q))), the probabilities are
 * multiplied by the V scale of their token on the way into the second product, and the zero points' share, one number
 * per head, comes off every output column at the end.  V scales must keep p * scale inside the compute type's range
 * (fp16: below 2^7 is always safe).  Returns DA_ERR_UNSUPPORTED for other head dims.
 */
int da_decoding_attn_int4kv_tok(const void *q, const void *k4, const void *v4, void *o, const int32_t *cu_seq_k,
                                size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                int is_alibi, int is_bf16, float softmax_scale, const float *alibi_slopes,
                                const float *k_params, const float *v_params, size_t total_k, void *workspace,
                                size_t workspace_bytes, void *hip_stream);

int da_decoding_attn_paged_int4kv_tok(const void *q, const void *k_pages, const void *v_pages, void *o,
                                      const int32_t *block_table, const int32_t *seq_lens, size_t max_seq_k,
                                      size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                      size_t page_size, size_t max_blocks_per_seq, size_t k_page_stride,
                                      size_t v_page_stride, int is_alibi, int is_bf16, float softmax_scale,
                                      const float *alibi_slopes, const float *k_params, const float *v_params,
                                      size_t total_k, void *workspace, size_t workspace_bytes, void *hip_stream);

size_t da_workspace_bytes_int4kv_tok(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                     size_t dim_v, size_t total_k, size_t page_size);

/*
 * int4 K/V with a (scale, zero) pair per run of 64 elements of every (token, KV head) row -- group-wise quantisation
 * with groups of 64 (no counterpart in the reference, as above).  k_params and v_params: [total_k, head_k, dim / 64, 2]
 * for the packed layout, [pages, page_size, head_k, dim / 64, 2] for page pools, 8-byte aligned:
 *   K[t, hk, c] = k_params[t, hk, c / 64, 0] * (int4 value - k_params[t, hk, c / 64, 1]),   V likewise.
 * Head dims (64,64) (the per-token scheme itself), (128,128) and (256,256).  The score tile is summed per run before
 * the factors go on; the second product takes one probability operand per run, each multiplied by that run's V
 * scale.  Everything else as for da_decoding_attn_int4kv_tok (at (256,256) a work-group takes 16 query heads, not 32:
 * four sets of factors for 32 heads do not fit the registers).
 */
int da_decoding_attn_int4kv_grp64(const void *q, const void *k4, const void *v4, void *o, const int32_t *cu_seq_k,
                                  size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                  size_t dim_v, int is_alibi, int is_bf16, float softmax_scale,
                                  const float *alibi_slopes, const float *k_params, const float *v_params,
                                  size_t total_k, void *workspace, size_t workspace_bytes, void *hip_stream);

int da_decoding_attn_paged_int4kv_grp64(const void *q, const void *k_pages, const void *v_pages, void *o,
                                        const int32_t *block_table, const int32_t *seq_lens, size_t max_seq_k,
                                        size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                        size_t page_size, size_t max_blocks_per_seq, size_t k_page_stride,
                                        size_t v_page_stride, int is_alibi, int is_bf16, float softmax_scale,
                                        const float *alibi_slopes, const float *k_params, const float *v_params,
                                        size_t total_k, void *workspace, size_t workspace_bytes, void *hip_stream);

size_t da_workspace_bytes_int4kv_grp64(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                       size_t dim_v, size_t total_k, size_t page_size);

/* The same with an int8 cache (k8 and v8 as for da_decoding_attn_int8kv). */
int da_decoding_attn_int8kv_grp64(const void *q, const void *k8, const void *v8, void *o, const int32_t *cu_seq_k,
                                  size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                  size_t dim_v, int is_alibi, int is_bf16, float softmax_scale,
                                  const float *alibi_slopes, const float *k_params, const float *v_params,
                                  size_t total_k, void *workspace, size_t workspace_bytes, void *hip_stream);

int da_decoding_attn_paged_int8kv_grp64(const void *q, const void *k_pages, const void *v_pages, void *o,
                                        const int32_t *block_table, const int32_t *seq_lens, size_t max_seq_k,
                                        size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                        size_t page_size, size_t max_blocks_per_seq, size_t k_page_stride,
                                        size_t v_page_stride, int is_alibi, int is_bf16, float softmax_scale,
                                        const float *alibi_slopes, const float *k_params, const float *v_params,
                                        size_t total_k, void *workspace, size_t workspace_bytes, void *hip_stream);

size_t da_workspace_bytes_int8kv_grp64(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                       size_t dim_v, size_t total_k, size_t page_size);

/*
 * The same per-token scheme over an int8 cache: k8 and v8 as for da_decoding_attn_int8kv (both required),
 * K[t, hk, c] = k_params[t, hk, 0] * (int8 value - k_params[t, hk, 1]), V likewise.  Arguments, layouts, head dims and
 * kernel as for the int4 entry points above.
 */
int da_decoding_attn_int8kv_tok(const void *q, const void *k8, const void *v8, void *o, const int32_t *cu_seq_k,
                                size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                int is_alibi, int is_bf16, float softmax_scale, const float *alibi_slopes,
                                const float *k_params, const float *v_params, size_t total_k, void *workspace,
                                size_t workspace_bytes, void *hip_stream);

int da_decoding_attn_paged_int8kv_tok(const void *q, const void *k_pages, const void *v_pages, void *o,
                                      const int32_t *block_table, const int32_t *seq_lens, size_t max_seq_k,
                                      size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                                      size_t page_size, size_t max_blocks_per_seq, size_t k_page_stride,
                                      size_t v_page_stride, int is_alibi, int is_bf16, float softmax_scale,
                                      const float *alibi_slopes, const float *k_params, const float *v_params,
                                      size_t total_k, void *workspace, size_t workspace_bytes, void *hip_stream);

size_t da_workspace_bytes_int8kv_tok(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim,
                                     size_t dim_v, size_t total_k, size_t page_size);

/*
 * Launch plan the library would use for this shape, for tests and benchmarks:
 *   kernel_kind 1 = VALU sweep, 2 = latent (MLA) MFMA sweep, 3 = grouped-head MFMA sweep (also the latent form with
 *   16 query heads or fewer); nsplit = sequence splits;
 *   chunk = tokens per split; heads_per_group = query heads one work-group serves; total_k as for
 *   da_decoding_attn_ex (0 = unknown).
 * The plan is that of the 16-bit packed call (V inside K for (576, 512)); paged and 8-bit calls may be planned
 * differently.
 * Any output pointer may be NULL.  Returns DA_ERR_UNSUPPORTED for an unsupported (dim, dim_v).
 * Mirrors the role of the reference's per-head-dim tile choice (csrc/kernel/decoding_attn/decoding_fwd_hd*.cu).
 */
int da_plan(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v, int is_bf16,
            size_t total_k, int *kernel_kind, int *nsplit, int *chunk, int *heads_per_group);

/*
 * The same for a call that passes V as a buffer of its own (v != NULL), over the packed layout (page_size 0) or
 * pages of page_size tokens.  It differs from da_plan at (576, 512) only: V outside K takes the latent MFMA kernel's
 * form that stages the V rows beside each K tile (kind 2; it moves both buffers, 1.9x the bytes of the aliased
 * call), except over pages of fewer than 16 tokens, which take the VALU sweep (kind 1, several times slower).
 */
int da_plan_distinct_v(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                       size_t total_k, size_t page_size, int *kernel_kind, int *nsplit, int *chunk,
                       int *heads_per_group);

/*
 * 1 when the 16-bit call (packed: page_size 0; else pages of page_size tokens) takes the grouped kernel's balanced
 * grid -- equal shares of the concatenated sequences per work-group instead of fixed splits of every sequence, the
 * share derived on the device from cu_seq_k[batch] -- 0 when not, negative on an error.  da_plan then reports the
 * shares along the line as nsplit and the share as chunk (0 when no token count was given).  No counterpart in the
 * reference, whose kernel never splits a sequence.
 */
int da_plan_is_balanced(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                        size_t total_k, size_t page_size);

/*
 * The plan of any call of this library, for benchmarks that report it beside a measurement: page_size 0 = packed
 * layout, else pages of page_size tokens; distinct_v != 0 = V passed as a buffer of its own; kv_bits 16 = fp16/bf16
 * K/V, 8 = the FP8 and int8 caches, 4 = the int4 cache, DA_KV_BITS_INT4_PER_TOKEN / DA_KV_BITS_INT8_PER_TOKEN = the
 * int4 / int8 cache with per-token (scale, zero) pairs, DA_KV_BITS_INT4_GROUP64 / DA_KV_BITS_INT8_GROUP64 = the int4 /
 * int8 cache with a pair per 64 elements (distinct_v must be set for the four).  Outputs as da_plan's, balanced as da_plan_is_balanced's result;
 * any output pointer may be NULL.  No counterpart in the reference (one tile shape per head dim,
 * csrc/kernel/decoding_attn/decoding_fwd_hd*.cu).
 */
#define DA_KV_BITS_INT4_PER_TOKEN 5
#define DA_KV_BITS_INT8_PER_TOKEN 9
#define DA_KV_BITS_INT4_GROUP64 6
#define DA_KV_BITS_INT8_GROUP64 10
int da_plan_call(size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v, size_t total_k,
                 size_t page_size, int distinct_v, int kv_bits, int *kernel_kind, int *nsplit, int *chunk,
                 int *heads_per_group, int *balanced);

/* 1 when (dim, dim_v) is a supported pair: the reference's DA_HEADDIM_SWITCH set (csrc/common/common.h:73-96). */
int da_supported_head_dims(size_t dim, size_t dim_v);

/* Message of the last failing call on this thread (never NULL).  Replaces the reference's log-and-exit
 * DA_CHECK / DA_CHECK_CUDART_ERROR macros (csrc/common/common.h:17-49). */
const char *da_last_error(void);

/* Library version, major * 10000 + minor * 100 + patch (reference decoding_attn/__init__.py:15 holds "0.1.0"). */
int da_version(void);

#ifdef __cplusplus
} /* extern "C" */

/*
 * C++ convenience overload with the reference's exact name and parameter list (reference
 * csrc/ops/decoding_attn.h:29-30), the stream being a HIP stream.  Defined inline so that the shared
 * library itself exports C symbols only.  Throws nothing; on failure it prints da_last_error() to stderr
 * and returns (the reference would exit the process).
 */
#include <stdio.h>
struct ihipStream_t;
inline void decoding_attn(void *q, void *k, void *v, void *o, int *cu_seq_k, size_t max_seq_k, size_t batch,
                          size_t head_q, size_t head_k, size_t dim, size_t dim_v, bool is_alibi, bool is_bf16,
                          ihipStream_t *stream) {
    if (da_decoding_attn(q, k, v, o, cu_seq_k, max_seq_k, batch, head_q, head_k, dim, dim_v, is_alibi ? 1 : 0,
                         is_bf16 ? 1 : 0, (void *)stream) != DA_OK) {
        fprintf(stderr, "decoding_attn: %s\n", da_last_error());
    }
}
#endif

#endif /* DECODING_ATTN_HIP_H_ */
