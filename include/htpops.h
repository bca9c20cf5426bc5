/*
 * htpops.h -- C ABI of the MI355X (gfx950) op backend.
 *
 * One context owns one HIP stream; ops are enqueued in order on that stream
 * (the reference executes requests strictly in order on one poller thread,
 * src/dsp/commu.c:43, :91-114). Buffer calls and op/message calls on one
 * context may come from different threads (the channel's consumer thread
 * runs messages while the host thread allocates, writes and releases
 * buffers): they are serialised by a lock inside the context. Ordering of
 * the work itself is the caller's: ops run in the order they are enqueued.
 * Every entry point takes that lock, htpops_last_error included (it returns a copy that belongs to the calling
 * thread and stays valid until that thread's next call of it). Several contexts may coexist.
 *
 * Return codes: 0 success, -1 rejected request (same meaning as the
 * reference's ops: bad sizes, null/unknown buffers, misalignment), other
 * negative values below.
 */
#ifndef HTPOPS_H
#define HTPOPS_H

#include "htpops_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

#define HTPOPS_OK            0
#define HTPOPS_ERR_REJECTED  (-1) /* the reference's "return -1" */
#define HTPOPS_ERR_NO_DEVICE (-2) /* compute requested from a context created without a GPU */
#define HTPOPS_ERR_HIP       (-3) /* a HIP runtime call failed; see htpops_last_error() */
#define HTPOPS_ERR_NOMEM     (-4)
#define HTPOPS_ERR_BUSY      (-5) /* channel already active (AEE_EALREADY in the reference) */

#define HTPOPS_DEVICE_NONE (-1)

typedef struct htpops_context htpops_context;

/* ---- session ----------------------------------------------------------- */

/* Replaces open_dsp_session + htp_ops_init_backend (reference: src/host/session.c:14-96,
 * src/dsp/commu.c:239-249). device >= 0 selects a GPU and creates the context's stream.
 * device == HTPOPS_DEVICE_NONE creates a context that can register buffers and validate /
 * frame requests but refuses every compute op with HTPOPS_ERR_NO_DEVICE. */
int htpops_init_backend(htpops_context **out_ctx, int device);

/* Replaces htp_ops_close (reference: src/dsp/commu.c:226-235): stops the channel, releases
 * every buffer the context allocated, destroys the stream. */
int htpops_close(htpops_context *ctx);

/* Text of the most recent failure on this context (never NULL). */
const char *htpops_last_error(const htpops_context *ctx);

/* Switches of a context (no counterpart in the reference): kernel choices that tests and A/B measurements override,
 * and two behaviours a host may want. Each starts from the environment variable HTPOPS_<NAME> (upper case) read when
 * the context is created; nothing on the op path reads the environment afterwards. Unknown names return -1.
 *   "attn_mask_threshold"  0 (default): the attention mask is ADDED to the scaled scores, the convention of the
 *                          reference's scalar routine (src/dsp/ops/flash_attn.c:1505-1512). 1: the mask SELECTS keys,
 *                          keep iff mask > -16 (compared in fp16), every other key is dropped, the convention of the
 *                          kernel the reference dispatches for op 5 (src/dsp/ops/flash_attn.c:448-460). The two agree
 *                          for masks of 0 and -inf only.
 *   "converted_cap_mib"    0 (default): no limit. > 0: converted weight copies beyond this many MiB are evicted, least
 *                          recently used first (copies used by the message being walked stay).
 *   "lane_order", "gemm_fp6", "gemv_rows_kernel", "gemm_tile_units", "attn_key_groups"   force or forbid a kernel
 *                          family / tile shape (for tests; results stay within every op's tolerance).
 *   "log"                  1: failures are also printed to stderr. */
int htpops_set_option(htpops_context *ctx, const char *name, int value);
int htpops_get_option(htpops_context *ctx, const char *name, int *value);

/* Blocks until everything enqueued on the context's stream has finished. */
int htpops_synchronize(htpops_context *ctx);

/* The context's hipStream_t, for callers that order their own HIP work against it. */
void *htpops_get_stream(htpops_context *ctx);

/* ---- buffer registry ---------------------------------------------------
 * Replaces rpcmem_alloc + fastrpc_mmap on the host (reference: src/host/test.c:30-58) and the
 * fd -> address table on the device (reference: src/dsp/mmap_mgr.cc:15-43). Handles are small
 * positive integers that go into RpcmemBufAddr.fd. */

/* Allocates `bytes` of device memory (256-byte aligned); returns a handle > 0 or a negative error. */
int htpops_buffer_alloc(htpops_context *ctx, size_t bytes);

/* Registers caller-owned device memory (e.g. a framework tensor); not freed on release. */
int htpops_buffer_register(htpops_context *ctx, void *device_ptr, size_t bytes);

/* mmap_manager_put_map: forgets the handle, frees the memory if the context allocated it.
 * Unknown handles are ignored and return 0, as in the reference (mmap_mgr.cc:29-37). */
int htpops_buffer_release(htpops_context *ctx, int handle);

/* Device address and size of a handle (NULL / 0 if unknown). The address is for the caller's own kernels and copies.
 * The context keeps converted copies of WEIGHTS that live in buffers it allocated (made on first use by a matmul,
 * dropped by htpops_buffer_write and by ops that write into the buffer): a caller that rewrites such a buffer through
 * this address must say so with htpops_buffer_invalidate before the next op reads it. Activations, KV rows and
 * outputs need nothing. Weights in caller-registered memory get no converted copy (they are converted per call or
 * take the kernels that read them as they are) until the caller asks for one with htpops_buffer_prepare_weights. */
void  *htpops_buffer_device_ptr(htpops_context *ctx, int handle);
size_t htpops_buffer_size(htpops_context *ctx, int handle);

/* Declares the contents of a buffer changed behind the context's back (no counterpart in the reference, whose weights
 * are immutable once mapped, src/dsp/op_executor.cc:130): converted weight copies made from it are dropped and
 * recorded messages that use them refuse to launch. Unknown handles return -1. */
int htpops_buffer_invalidate(htpops_context *ctx, int handle);

/* Makes, now, the converted copy of the weight matrix [n][k/32] (weight_type GGML_TYPE_Q4_0 or GGML_TYPE_Q8_0) at
 * `offset` of the buffer that matmuls over `m_hint` activation rows will use (none at m_hint = 1; operand-order nibbles
 * for 2..16 rows; FP6 tiles or int8 fragments from 33 rows), so that the first matmul does not pay for the conversion
 * and its hipMalloc. The reference maps weights once and treats them as immutable (src/dsp/op_executor.cc:124-130);
 * this call states the same for the buffer: it is the opt-in that puts CALLER-REGISTERED memory under the contract of
 * the context's own buffers -- converted copies of its weights are kept from now on (also those that later matmuls at
 * other row counts make on first use), and the caller says htpops_buffer_invalidate after rewriting it.
 * *converted_bytes (may be NULL) receives the bytes this call added. */
int htpops_buffer_prepare_weights(htpops_context *ctx, int handle, size_t offset, int weight_type, int n, int k,
                                  int m_hint, size_t *converted_bytes);

/* Bytes of converted weight copies the context holds right now / size of its grown-on-demand workspace. */
size_t htpops_converted_bytes(htpops_context *ctx);
size_t htpops_workspace_bytes(htpops_context *ctx);

/* Host <-> device copies ordered on the context's stream; both return after the copy is done. */
int htpops_buffer_write(htpops_context *ctx, int handle, size_t offset, const void *src, size_t bytes);
int htpops_buffer_read(htpops_context *ctx, int handle, size_t offset, void *dst, size_t bytes);

/* ---- op execution ------------------------------------------------------ */

/* Replaces execute_op_simple (reference: include/dsp/op_executor.h:9, src/dsp/op_executor.cc:52-204).
 * Validates the request, resolves handles, enqueues the kernels on the context's stream and returns
 * without waiting. Unknown op ids return -1 (the reference silently returns 0 there). */
int htpops_execute_op(htpops_context *ctx, const struct OpComputeRequest *req);

/* One pass of the reference's consumer loop over a message (src/dsp/commu.c:91-126): runs every
 * request in order, stores each op's return code in RequestHeader.state, honours
 * RPCMEM_MAP.n_puts as handle releases, waits for the stream, then publishes completion by
 * storing state.d = v[0] | (1 << 8). Returns 0, or a negative error if the message is malformed
 * (offsets outside `msg_bytes`; pass 0 to skip the bound check). A compute request that ends before
 * the parameter struct of its op does gets HTPOPS_ERR_REJECTED as its state and is not run (the
 * reference casts without looking at the request's size). The go byte v[0] is not required to be set. */
int htpops_process_message(htpops_context *ctx, struct MessageHeader *msg, size_t msg_bytes);

/* The two halves of htpops_process_message, for producers that keep several messages in flight:
 * htpops_enqueue_message walks the message and enqueues its requests (per-request codes are stored at once; the
 * done byte is not touched); htpops_finish_message waits for the stream and publishes completion. Messages
 * enqueued on one context run in enqueue order (the reference's single consumer thread, src/dsp/commu.c:43). */
int htpops_enqueue_message(htpops_context *ctx, struct MessageHeader *msg, size_t msg_bytes);
int htpops_finish_message(htpops_context *ctx, struct MessageHeader *msg);

/* How many separately submitted units the most recent walk of a message on this context issued: compute requests that
 * were grouped count once (diagnostic; the reference runs one op per request, src/dsp/commu.c:91-100). A group is one
 * kernel launch where all its members take the same kernel (the projections of a decoder layer do); a group of
 * many-row matmuls adds one launch that converts the activations, and a few-row group whose members take different
 * kernels (by shape and weight type) issues one launch per kernel. Grouping never changes a result: a request joins a group only if it neither reads nor
 * overwrites what an earlier member writes and writes nothing an earlier member reads. */
int htpops_last_message_submissions(htpops_context *ctx);

/* A message recorded once and replayed many times: the kernel launches of a whole message (a decoder block that is
 * submitted again for every token, reference: src/dsp/commu.c:91-114 walks it anew each time) are captured into one
 * HIP graph and re-enqueued on the context's stream with a single call.
 * htpops_record_message runs the message once (request states are stored as usual, converted weight copies are made,
 * the workspace is sized), then records a second walk without running it. It rejects messages with an RPCMEM_MAP
 * request or a failing op, and contexts whose channel thread is active. A recording holds device addresses: it refuses
 * to launch (HTPOPS_ERR_REJECTED, record again) once a buffer that its requests name has been released, weights it
 * uses have been rewritten through htpops_buffer_write (their converted copies are dropped), or a later op has needed
 * a larger workspace than the context had. Activations, KV rows and other buffer CONTENTS may change between launches
 * (written by ops, by htpops_buffer_write or by the caller's own kernels); sizes, handles and offsets are those of
 * the recorded message.
 * Request states and the done byte are not touched by a launch; order against other work is stream order.
 * htpops_close releases the recordings that are still alive; their pointers must not be used afterwards. */
typedef struct htpops_recorded_message htpops_recorded_message;
int htpops_record_message(htpops_context *ctx, struct MessageHeader *msg, size_t msg_bytes,
                          htpops_recorded_message **out);
int htpops_launch_recorded_message(htpops_context *ctx, htpops_recorded_message *rec);
int htpops_release_recorded_message(htpops_context *ctx, htpops_recorded_message *rec);

/* Replaces htp_ops_create_channel / htp_ops_destroy_channel (reference: include/htp_ops.idl:11-12,
 * src/dsp/commu.c:151-212): starts a consumer thread that polls msg->state exactly as
 * msg_receiver_loop does (run when v[0] != 0 && v[1] == 0) and calls htpops_process_message.
 * `msg` is ordinary host memory of `max_msg_size` bytes owned by the caller; it is zeroed here. */
int htpops_create_channel(htpops_context *ctx, void *msg, size_t max_msg_size);
int htpops_destroy_channel(htpops_context *ctx);

/* Direct entries with the argument order of the FastRPC interface (reference: include/htp_ops.idl:15-17,
 * include/host/op_export.h:3-5). Both enqueue and then wait, like an RPC. */
int htpops_rms_norm_f32(htpops_context *ctx, int dst_fd, int dst_offset, int src_fd, int src_offset, int ne0,
                        int ne1);
int htpops_mat_mul_permuted_w16a32(htpops_context *ctx, int output_fd, int output_offset, int activation_fd,
                                   int activation_offset, int weight_fd, int weight_offset, int m, int k, int n);

/* ---- raw-pointer op entries ---------------------------------------------
 * Same kernels as htpops_execute_op, for callers that hold device pointers. All pointers are
 * device addresses; all calls enqueue on the context's stream and return without waiting.
 * Each replaces the L1 function named beside it (reference: include/dsp/ops.h:15-26). */

/* hvx_rms_norm_f32 (src/dsp/ops/rms_norm.c:68-84): weight may be NULL (all ones). The reference op
 * is eps = 1e-5f, weight = NULL. Pointers must be 16-byte aligned. */
int htpops_rms_norm_f32_ex_ptr(htpops_context *ctx, float *dst, const float *src, const float *weight, float eps,
                               int ne0, int ne1);

/* Activation quantizer (replaces transfer_activation_chunk_fp32_to_fp16, src/dsp/ops/mat_mul.c:89-128,
 * with ggml's Q8_0 arithmetic): src fp32 [m][k] -> dst block_q8_0 [m][k/32]. k % 32 == 0. */
int htpops_quantize_q8_0_ptr(htpops_context *ctx, void *dst, const float *src, int k, int m);

/* RMSNorm fused with the quantizer: dst block_q8_0 [ne1][ne0/32]. Same result as the two ops in a row. */
int htpops_rms_norm_quantize_q8_0_ptr(htpops_context *ctx, void *dst, const float *src, const float *weight,
                                      float eps, int ne0, int ne1);

/* hmx_mat_mul_permuted_qk_0_d16a32 (src/dsp/ops/mat_mul.c:875-1153) with integer block dots:
 * dst fp32 [m][n]; act block_q8_0 [m][k/32]; weight block_q4_0 or block_q8_0 [n][k/32].
 * weight_type is GGML_TYPE_Q4_0 (2) or GGML_TYPE_Q8_0 (8). k % 32 == 0. */
int htpops_mat_mul_q8_0_act_ptr(htpops_context *ctx, float *dst, const void *act_q8_0, const void *weight, int m,
                                int k, int n, int weight_type);

/* Same with fp32 activations [m][k]; they are quantized into a workspace owned by the context. */
int htpops_mat_mul_f32_act_ptr(htpops_context *ctx, float *dst, const float *act, const void *weight, int m, int k,
                               int n, int weight_type);

/* simple_flash_attn (src/dsp/ops/flash_attn.c:1368-1420). Q/O [qo_len][n_heads][head_dim] as fp32
 * (qo_is_f32 = 1, the reference op) or fp16; K/V fp16 [kv_len][n_kv_heads][head_dim]; mask fp16
 * [qo_len][align_up(kv_len, 64)] added to the scaled scores (or selecting keys, option "attn_mask_threshold"), or
 * NULL; causal as in FlashAttnExParams.
 * head_dim: any even value up to 256 (the reference sends head_dim % 64 != 0 to simple_flash_attn_sp_hdim,
 * src/dsp/ops/flash_attn_sp_hdim.c:782-832, and refuses odd values, :785). */
int htpops_flash_attn_ptr(htpops_context *ctx, void *o, const void *q, const void *k, const void *v,
                          const void *mask, int qo_len, int kv_len, int n_heads, int n_kv_heads, int head_dim,
                          int qo_is_f32, int causal);

/* htpops_flash_attn_ptr for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. Same arguments, same kernels, same
 * results bit for bit; the split-KV partials of decode attention (qo_len == 1) go to a static 8 MiB device array
 * inside the library instead of the context's grown-on-demand workspace, and the call performs no hipMalloc / hipFree
 * of any kind. Limit: n_heads * ceil(kv_len / 64) * (head_dim + 2) * 4 bytes <= 8 MiB (e.g. 32 heads of 128 up to
 * kv_len 32256); larger requests, and outputs that overlap weights the context holds a converted copy of, return -1
 * with a message. All contexts on one GPU share the array, and it keeps the last call's contents: calls on one
 * context are ordered by its stream; a context that calls this while ANOTHER context's calls may still be running
 * (that context has not been through htpops_synchronize, htpops_finish_message or htpops_close since its last such
 * call) gets HTPOPS_ERR_BUSY instead of a race. */
int htpops_flash_attn_noalloc_ptr(htpops_context *ctx, void *o, const void *q, const void *k, const void *v,
                                  const void *mask, int qo_len, int kv_len, int n_heads, int n_kv_heads, int head_dim,
                                  int qo_is_f32, int causal);

#ifdef __cplusplus
}
#endif

#endif /* HTPOPS_H */
