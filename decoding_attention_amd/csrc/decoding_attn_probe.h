/*
 * Measurement aids of the benchmark (bench.py), exported by libdecoding_attn_probe.so only: a second build of the
 * library's sources with these entry points added (and without the static device array of
 * da_decoding_attn_noalloc, which this build answers only for plans that need no workspace).  None of this is part of
 * the drop-in ABI (decoding_attn_hip.h) and nothing here has a counterpart in the reference.
 */
#ifndef DECODING_ATTN_PROBE_H_
#define DECODING_ATTN_PROBE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Enqueue a plain streaming read of `bytes` bytes at `buf` (device memory, 16-byte aligned, at least 128 MiB).  It
 * reads da_probe_stream_read_bytes(bytes) of them, in contiguous slabs with 16-byte loads.  Timing it gives the
 * bandwidth HBM delivers to a kernel that only reads, the practical ceiling for the bandwidth-bound attention
 * kernels.  `sink` may be NULL.
 */
int da_probe_stream_read(const void *buf, size_t bytes, void *sink, void *hip_stream);
size_t da_probe_stream_read_bytes(size_t bytes);

/*
 * Enqueue a kernel that does nothing but matrix instructions: one wave per SIMD on each of 256 work-groups issues
 * `iters` x 32 v_mfma_f32_32x32x16_f16 back to back, each fed by a 16-byte LDS read of the caller's operand values.
 *   operands  32 KiB of fp16 values in device memory, 16-byte aligned (the values matter: a matrix instruction's power
 *             depends on its operands)
 *   sink      256 KiB of device memory the kernel writes its checksums to
 * Timing it gives the matrix rate the chip sustains under its power limit; da_probe_mfma_rate_flops(iters) is the
 * number of floating-point operations of one launch.
 */
int da_probe_mfma_rate(const void *operands, int iters, void *sink, void *hip_stream);
double da_probe_mfma_rate_flops(int iters);

/*
 * da_decoding_attn_ex without its merge kernel, so that the sweep kernel of a call can be timed on its own with
 * events.  When the plan splits the sequences the output rows are NOT written (the partials stay in the
 * workspace): never use it for results.
 */
int da_probe_sweep_only(const void *q, const void *k, const void *v, void *o, const int32_t *cu_seq_k,
                        size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                        int is_alibi, int is_bf16, size_t total_k, void *workspace, size_t workspace_bytes,
                        void *hip_stream);

/*
 * Overrides one planner tunable (by the name of its environment variable: DA_NSPLIT, DA_MLA_HEADS,
 * DA_MLA_GROUP_SMALL, DA_MLA_GROUP_HEADS, DA_MFMA_TARGET_WGS, DA_MFMA_SMALL_WGS, DA_GROUP_MIN_RATIO, DA_FORCE_KIND) for later calls into this library in
 * this process, so that one process can time a shape under several launch plans (bench.py --sweep latent-plan).
 */
int da_probe_set_tunable(const char *name, int value);

#ifdef __cplusplus
}
#endif
#endif /* DECODING_ATTN_PROBE_H_ */
