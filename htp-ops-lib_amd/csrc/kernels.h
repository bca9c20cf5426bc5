// Host-callable launchers of the gfx950 kernels. Every launcher validates nothing (the C-ABI layer does),
// enqueues on `stream`, and returns the status of the launch.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace htpops {

enum WeightType { kQ4_0 = 2, kQ8_0 = 8 };  // enum ggml_type values (reference: include/dsp/quants.h:33-74)

// fp32 [m][k] -> block_q8_0 [m][k/32]
hipError_t launch_quantize_q8_0(hipStream_t stream, void *dst, const float *src, int k, int m);

// y = x * rsqrt(mean(x^2) + eps) * w; w may be null
hipError_t launch_rms_norm_f32(hipStream_t stream, float *dst, const float *src, const float *weight, float eps,
                               int ne0, int ne1);
// same, result quantized to block_q8_0 [ne1][ne0/32]; ne0 % 32 == 0
hipError_t launch_rms_norm_quantize_q8_0(hipStream_t stream, void *dst, const float *src, const float *weight,
                                         float eps, int ne0, int ne1);

// out fp32 [m][n] = act block_q8_0 [m][k/32] x weight [n][k/32]
// decode path: one pass over the weight bytes per activation row
hipError_t launch_gemv_q8_0_act(hipStream_t stream, float *out, const void *act, const void *weight, int m, int k,
                                int n, WeightType wt);
// several matrix-vector products (m = 1) in a single launch, each with its own weight matrix, activation row, row
// length k and output; the caller guarantees that no member reads what another writes. hipErrorNotSupported when a
// member does not fit the fast kernel (k % 64, k <= 12288, 4-byte aligned buffers): the caller then launches them one
// by one.
constexpr int kGemvGroupMax = 8;
hipError_t launch_gemv_group_q8_0_act(hipStream_t stream, int count, float *const *outs, const void *const *acts,
                                      const void *const *weights, const int *ns, const int *ks, WeightType wt);
// The same launch with the activation row made inside it: RMSNorm(src [* norm_weight], eps) quantized to Q8_0 is what
// every member multiplies by (all of one k), and it is also written to `q_out`, bit for bit what
// launch_rms_norm_quantize_q8_0 writes (`normalize` false: src quantized as it is, the bytes of launch_quantize_q8_0). hipErrorNotSupported (nothing launched; the caller runs the two steps) unless
// k % 64 == 0, k <= 4096, src / norm_weight are 16-byte aligned and the rows are few enough for this to pay: every
// workgroup makes the row for itself, which beats a launch of its own up to about a thousand workgroups of 16 rows.
hipError_t launch_gemv_group_rms_norm_q8_0_act(hipStream_t stream, int count, float *const *outs, const void *const *weights,
                                               const int *ns, int k, WeightType wt, const float *src,
                                               const float *norm_weight, float eps, void *q_out, bool normalize);
// 2 <= m <= 4 activation rows against several weight matrices in one launch: the decode kernel's stream over the
// weights with the rows held in registers; member i reads the rows acts[i] of length ks[i] (k % 64 == 0, k <= 12288,
// 4-byte aligned buffers; else hipErrorNotSupported)
bool       gemv_rows_fits(int m, int k, WeightType wt);  // whether the launch below is the kernel of choice
hipError_t launch_gemv_rows_group_q8_0_act(hipStream_t stream, int count, float *const *outs, const void *const *acts,
                                           const void *const *weights, const int *ns, int m, const int *ks,
                                           WeightType wt);
// small-batch path (m <= 32, k % 64 == 0, else hipErrorNotSupported): one pass over the weight bytes for all rows,
// block dots on v_mfma_i32_32x32x32_i8
// `workspace` (matmul_skinny_workspace_bytes) holds per-slice partial tiles, `tickets` is an array of
// `ticket_slots` zeroed counters that the kernel leaves zeroed; without them K is not sliced (slower).
size_t     matmul_skinny_workspace_bytes(int m, int k, int n);
hipError_t launch_matmul_skinny(hipStream_t stream, float *out, const void *act, const void *weight, int m, int k,
                                int n, WeightType wt, void *workspace, unsigned *tickets, int ticket_slots);
// several weight matrices against the same 2 <= m <= 8 activation rows in one launch; hipErrorNotSupported when the
// shapes do not fit the K-sliced kernel (the caller then launches them one by one)
size_t     matmul_skinny_group_workspace_bytes(int count, const int *ns, int m, int k);
hipError_t launch_matmul_skinny_group(hipStream_t stream, int count, float *const *outs, const void *act,
                                      const void *const *weights, const int *ns, int m, int k, WeightType wt,
                                      void *workspace, unsigned *tickets, int ticket_slots);
// 2 <= m <= 16 rows against Q4_0 or Q8_0 weights repacked once (launch_weights_to_lane_order into
// matmul_lane_order_weight_bytes, same size as the weights; the caller can cache the copy) into matrix-core operand
// order: every workgroup streams a tile of 16 rows over the whole of K, nothing is exchanged between workgroups.
// Fits when n % 16 == 0 and k % 256 == 0 and the 8 (m <= 8) or 16 activation rows of length k fit LDS; `act` must be
// 16-byte aligned.
bool       matmul_lane_order_fits(int n, int m, int k, WeightType wt);
size_t     matmul_lane_order_weight_bytes(int k, int n, WeightType wt);
hipError_t launch_weights_to_lane_order(hipStream_t stream, void *dst, const void *weight, int k, int n, WeightType wt);
// (one launch for `count` matmuls of the same m, k and weight type; member i reads the activation rows acts[i])
hipError_t launch_matmul_lane_order_group(hipStream_t stream, int count, float *const *outs, const void *const *acts,
                                          const void *const *lane_order_weights, const int *ns, int m, int k,
                                          WeightType wt, int forced_tiles);  // forced_tiles 2 / 3: one / two tiles per workgroup
// 2 <= m <= 8 rows against Q4_0 weights repacked once into another operand order (launch_weights_to_block_pairs, the
// same size again): two blocks per matrix instruction, the second one in the result rows that 8 activation rows leave
// unused. A workgroup keeps its member's activation rows in LDS and streams tiles of 16 weight rows over the whole of
// K; members may differ in k. Conditions: k % 256 == 0, n % 16 == 0, `act` and the repacked weights 16-byte aligned.
bool       matmul_block_pairs_fits(int n, int m, int k, WeightType wt);
hipError_t launch_weights_to_block_pairs(hipStream_t stream, void *dst, const void *weight, int k, int n);
hipError_t launch_matmul_block_pairs_group(hipStream_t stream, int count, float *const *outs, const void *const *acts,
                                           const void *const *pair_order_weights, const int *ns, int m, const int *ks);
// many-row path for Q4_0 weights, k % 64 == 0: FP6 scaled MFMA (exact: int8 = 16 hi + lo, all parts |t| <= 15) over operand
// tiles staged in LDS by DMA. The weight tiles (gemm_fp6_lds_weight_tile_bytes, 1 byte per weight) are converted once
// (launch_q4_0_to_fp6_tiles) and can be cached by the caller; the activation tiles (gemm_fp6_lds_act_tile_bytes) are
// written per call unless `act_tiles_ready`. Buffers 4-byte aligned, else hipErrorNotSupported.
bool       gemm_fp6_lds_fits(int m, int k, int n);
bool       gemm_fp6_lds_fills_device(int m, int n);  // enough 128 x 64 output tiles to keep every compute unit busy
size_t     gemm_fp6_lds_weight_tile_bytes(int k, int n);
size_t     gemm_fp6_lds_act_tile_bytes(int m, int k);
hipError_t launch_q4_0_to_fp6_tiles(hipStream_t stream, void *dst, const void *weight, int k, int n);
hipError_t launch_gemm_fp6_lds(hipStream_t stream, float *out, const void *act_q8_0, const void *weight_tiles, int m, int k,
                               int n, void *act_tiles, bool act_tiles_ready);
// many-row path: int8 MFMA over operands in fragment order. The weights are converted once
// (launch_weights_to_i8_fragments into gemm_i8_weight_fragment_bytes) and can be cached by the caller; the
// activations are converted per call into `act_fragments` (gemm_i8_act_fragment_bytes), unless the caller says that
// buffer already holds the conversion of the same activations (`act_fragments_ready`).
size_t     gemm_i8_weight_fragment_bytes(int k, int n);
size_t     gemm_i8_act_fragment_bytes(int m, int k);
hipError_t launch_weights_to_i8_fragments(hipStream_t stream, void *dst, const void *weight, int k, int n,
                                          WeightType wt);
// `exchange` (gemm_i8_fragments_exchange_bytes; may be 0) and `tickets` (zeroed counters, left zeroed): scratch for shapes
// whose K is split over workgroups. Without them those shapes run unsplit: correct, slower, and rounded differently.
// (`forced_unit` 1 / 2 forces the tile size that the shape would otherwise choose; 0: the kernel's own choice)
size_t     gemm_i8_fragments_exchange_bytes(int m, int n, int k, int forced_unit);
hipError_t launch_gemm_i8_fragments(hipStream_t stream, float *out, const void *act_q8_0, const void *weight_fragments,
                                    int m, int k, int n, void *act_fragments, bool act_fragments_ready, void *exchange,
                                    size_t exchange_bytes, unsigned *tickets, int ticket_slots, int forced_unit);
// The same for up to kGemmGroupMax matmuls of one row count m in one launch each for the conversions and the products:
// member i multiplies the converted activations act_fragments[i] (gemm_i8_act_fragment_bytes(m, ks[i]) each; members
// that read the same rows may share one) by weight_fragments[i]. Every member must be `groupable` (the tile
// configuration it gets depends on (m, n) alone, and a launch has one), else hipErrorNotSupported; a member's result
// is bit for bit what its own launch gives, provided `exchange` holds the sum of the members' exchange bytes.
constexpr int kGemmGroupMax = 8;
bool       gemm_i8_fragments_groupable(int m, int n, int forced_unit);
// launch_gemm_fp6_lds for up to kGemmGroupMax matmuls over the SAME activation rows (one conversion, act_tiles): the
// members that take the same kernel share one launch, whose grid keeps the compute units fed to the end (measured at
// 512 x 11008 x 4096: 65 us alone, 60 / 52 / 50 us per matmul with 2 / 4 / 8 in a launch). A member's result is bit
// for bit what its own launch gives.
hipError_t launch_gemm_fp6_lds_group(hipStream_t stream, int count, float *const *outs, const void *act_q8_0,
                                     const void *const *weight_tiles, int m, int k, const int *ns, void *act_tiles,
                                     bool act_tiles_ready);
hipError_t launch_act_to_i8_fragments_group(hipStream_t stream, int count, void *const *act_fragments,
                                            const void *const *acts_q8_0, const int *ks, int m);
hipError_t launch_gemm_i8_fragments_group(hipStream_t stream, int count, float *const *outs,
                                          const void *const *act_fragments, const void *const *weight_fragments,
                                          const int *ns, const int *ks, int m, void *exchange, size_t exchange_bytes,
                                          unsigned *tickets, int ticket_slots, int forced_unit);
// picks between the one-row and the small-batch kernel by m (any m; many rows are better served by the fragment path)
size_t     mat_mul_workspace_bytes(int m, int k, int n);
hipError_t launch_mat_mul_q8_0_act(hipStream_t stream, float *out, const void *act, const void *weight, int m, int k,
                                   int n, WeightType wt, void *workspace, unsigned *tickets, int ticket_slots);

// The reference's native weight formats (ops 1-4): a weight buffer (weight_kind 1 fp16 tiles, 2 Q4_0, 3 Q8_0,
// 4 IQ4_NL super-blocks) is converted once into MFMA fragment order (permuted_weight_fragment_bytes), then
// out fp32 [m][n] = fp16(act fp16 x W fp16); `act_fragments` is scratch of permuted_act_fragment_bytes.
size_t     permuted_weight_fragment_bytes(int k, int n);
size_t     permuted_act_fragment_bytes(int m, int k);
hipError_t launch_permuted_weight_to_fragments(hipStream_t stream, void *dst, const void *src, int k, int n,
                                               int weight_kind);
hipError_t launch_mat_mul_fragments(hipStream_t stream, float *out, const float *act, const void *weight_fragments,
                                    int m, int k, int n, void *act_fragments);

// attention; see htpops_flash_attn_ptr. `workspace` holds split-KV partials (decode), size from
// flash_attn_workspace_bytes. `q8_out` (or nullptr; used only where flash_attn_writes_q8_0 says so: decode with
// head_dim 64 / 128 and fp32 output): the output row is also written there as Q8_0 blocks, bit for bit what
// launch_quantize_q8_0 makes of it. `forced_key_groups` 1 / 2 forces how many key groups a prefill workgroup holds
// (0: by grid size). `mask_threshold`: the mask selects keys (keep iff mask > -16, reference:
// src/dsp/ops/flash_attn.c:448-460) instead of being added to the scores (:1505-1512).
size_t     flash_attn_workspace_bytes(int qo_len, int kv_len, int n_heads, int head_dim);
hipError_t launch_flash_attn(hipStream_t stream, void *o, const void *q, const void *k, const void *v,
                             const void *mask, int qo_len, int kv_len, int n_heads, int n_kv_heads, int head_dim,
                             bool qo_is_f32, bool causal, void *workspace, void *q8_out, int forced_key_groups,
                             bool mask_threshold);
// One of the two launches of one-token attention by itself, for timing: part 1 = the split-KV launch (writes the
// partial records into `workspace`), part 2 = the merge launch (reads them). Same arguments as above otherwise.
hipError_t launch_flash_attn_decode_part(hipStream_t stream, int part, void *o, const void *q, const void *k,
                                         const void *v, int kv_len, int n_heads, int n_kv_heads, int head_dim,
                                         bool qo_is_f32, void *workspace);
bool       flash_attn_writes_q8_0(int qo_len, int head_dim, bool qo_is_f32);

// What the calling thread's most recent launch of the one-row matmul kernel was: kernel instance and geometry. The bench
// harness compares it with the launch its hardware-counter figures were taken from.
struct LaunchRecord {
  const char *kernel = "";  // kernel family
  int         t0 = 0, t1 = 0, t2 = 0;  // template arguments of the instance
  unsigned    grid = 0, block = 0;
  unsigned    lds = 0;
};
LaunchRecord &last_gemv_launch();

// measurement helpers
hipError_t launch_copy(hipStream_t stream, void *dst, const void *src, size_t bytes);
// one pass over `bytes` (16-byte multiples) that keeps nothing; `sink` is one device word the kernel never writes in practice
hipError_t launch_read(hipStream_t stream, const void *src, size_t bytes, unsigned *sink);
hipError_t launch_mfma_loop(hipStream_t stream, int kind, int iters, int *sink, int n_blocks);

}  // namespace htpops
