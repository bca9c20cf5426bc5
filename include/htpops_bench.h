/*
 * htpops_bench.h -- timers and calibration kernels of the bench harness.
 *
 * Exported by the same shared library as include/htpops.h but not part of the op backend's interface: nothing here
 * replaces a reference interface, and no op depends on it. bench.py uses these to time the stream the ops are
 * launched on and to measure the device's own ceilings beside them.
 */
#ifndef HTPOPS_BENCH_H
#define HTPOPS_BENCH_H

#include "htpops.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Records an event on the context's stream / returns elapsed milliseconds between the two most
 * recent start and stop marks after waiting for the stop mark. */
int htpops_timer_start(htpops_context *ctx);
int htpops_timer_stop(htpops_context *ctx);
int htpops_timer_elapsed_ms(htpops_context *ctx, float *ms);

/* Runs `iters` back-to-back v_mfma_i32_32x32x32_i8 (kind 0), v_mfma_i32_16x16x64_i8 (kind 1) or
 * v_mfma_f32_32x32x16_f16 (kind 2) loops on every CU and reports the achieved op rate in Tera-ops/s. */
int htpops_measure_mfma_peak(htpops_context *ctx, int kind, int iters, double *tera_ops);

/* Plain device-to-device copy kernel (16 B per lane, grid-stride) used to calibrate HBM counters and to
 * measure the attainable copy bandwidth; reports bytes read + written per second in GB/s. */
int htpops_measure_copy_bandwidth(htpops_context *ctx, size_t bytes, int iters, double *gbps);

/* Time of one launch that reads `bytes` once and keeps nothing (every wave 4 KiB, 16 bytes per lane and load), averaged
 * over `iters` rounds over `buffers` distinct buffers of that size read in turn (buffers x bytes beyond the 256 MB
 * memory-side cache = every launch reads HBM). The floor under any one-launch weight stream of that size. */
int htpops_measure_read_us(htpops_context *ctx, size_t bytes, int buffers, int iters, double *us_per_launch);

/* Kernel instance and launch geometry of the calling thread's most recent launch of the one-row matmul kernel, as text
 * ("gemv_members_kernel<2,1,512> grid=2400 block=512 lds=..."): the harness checks that the launch it times is the
 * launch its hardware-counter figures were profiled on. */
int htpops_last_gemv_launch(htpops_context *ctx, char *text, size_t cap);

/* Host time of walking a message: `iters` calls of htpops_enqueue_message timed on the host clock while the stream has
 * a backlog (so that no call waits for the GPU); includes the HIP launch calls, nothing of the kernels' run time.
 * Waits for the stream before returning. */
int htpops_measure_host_walk_us(htpops_context *ctx, struct MessageHeader *msg, size_t msg_bytes, int iters,
                                double *us_per_message);

/* The two launches of one-token attention (head_dim 64 or 128, no mask) timed by themselves: `iters` launches of the
 * split-KV kernel in a row, then `iters` of the merge kernel, each between two events on the context's stream, in
 * microseconds per launch. o, q and the `sets` K/V pairs (ks[i], vs[i], read in turn) are device pointers laid out as
 * for htpops_flash_attn_ptr; the partial records go to the context's workspace. */
int htpops_measure_decode_attention_parts(htpops_context *ctx, void *o, const void *q, const void *const *ks,
                                          const void *const *vs, int sets, int kv_len, int n_heads, int n_kv_heads,
                                          int head_dim, int qo_is_f32, int iters, double *split_us, double *merge_us);

#ifdef __cplusplus
}
#endif

#endif /* HTPOPS_BENCH_H */
