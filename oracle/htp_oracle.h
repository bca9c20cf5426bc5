/*
 * htp_oracle.h -- scalar CPU restatement of the op backend's arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing in the shipped library links, loads or calls this code;
 * it exists so that tests, the smoke check and the benchmark's CPU-baseline leg can compare the
 * HIP kernels against an independent, readable definition of every result.
 *
 * Where each function comes from (paths are relative to the reference checkout):
 *   oracle_rms_norm_f32          src/host/test.c:60-80 (rms_norm_f32_ref), src/dsp/ops/rms_norm.c:8-84
 *   oracle_dequantize_*          include/dsp/quants.h:11-31, src/dsp/ops/mat_mul.c:25-32, :260-306
 *   oracle_flash_attn            src/dsp/ops/flash_attn.c:1426-1579 (naive_flash_attn)
 *   oracle_mat_mul_w16a32        src/host/test.c:307-327 (tile layout and fp32 triple loop)
 *   oracle_dequantize_permuted_*,
 *   oracle_mat_mul_permuted      src/dsp/ops/mat_mul.c:308-508 (super-block dequantizers), :758-855, :875-1153.
 *                                The even/odd byte order of the Q4_0 super-block is PARITY UNPINNED (no test
 *                                or fixture in the reference covers it); the rest is pinned by the tile layout.
 *   oracle_quantize_row_q8_0,
 *   oracle_vec_dot_*,
 *   oracle_mat_mul_q*            ggml's Q8_0 quantizer and q4_0 x q8_0 / q8_0 x q8_0 dot product. The reference
 *                                vendors no ggml source and pins no version; these follow the closed forms
 *                                  d = amax/127, id = d ? 1/d : 0, q = roundf(x*id), scale = fp16(d)
 *                                  sumi = sum (w_j) * a_j  (exact int32);  acc += ((float)sumi * d_w) * d_a
 *                                and are pinned by known-answer vectors, an independent numpy restatement and
 *                                exact-integer special cases in tests/ (parity against ggml itself: unpinned).
 *
 * All fp16 values are passed as uint16_t bit patterns; conversions are done in software so the
 * file builds with any C99 compiler. Compile with -ffp-contract=off: the accumulation order and
 * rounding of every fp32 operation is part of the definition.
 */
#ifndef HTP_ORACLE_H
#define HTP_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* IEEE binary16 <-> binary32, round-to-nearest-even, subnormals kept, NaN kept quiet. */
float    oracle_fp16_to_fp32(uint16_t h);
uint16_t oracle_fp32_to_fp16(float f);

/* n_blocks standard blocks -> 32 * n_blocks floats in K order. */
void oracle_dequantize_q4_0(const void *blocks, int n_blocks, float *out);
void oracle_dequantize_q8_0(const void *blocks, int n_blocks, float *out);
void oracle_dequantize_iq4_nl(const void *blocks, int n_blocks, float *out);

/* x fp32 [k] -> block_q8_0 [k/32]. */
void oracle_quantize_row_q8_0(const float *x, void *y, int k);
/* rows: x fp32 [m][k] -> block_q8_0 [m][k/32]. */
void oracle_quantize_q8_0(const float *x, void *y, int k, int m);

/* Exact int32 dot of one weight block with one activation block. */
int32_t oracle_block_dot_q4_0_q8_0(const void *w_block, const void *a_block);
int32_t oracle_block_dot_q8_0_q8_0(const void *w_block, const void *a_block);

/* fp32 dot of a weight row with an activation row, k values, blocks accumulated left to right. */
float oracle_vec_dot_q4_0_q8_0(int k, const void *w_row, const void *a_row);
float oracle_vec_dot_q8_0_q8_0(int k, const void *w_row, const void *a_row);
/* Same terms accumulated in double: the value both the fp32 oracle and a kernel must approach.
 * If abs_sum is not NULL it receives sum |term| (the scale of the 1e-5 tolerance). */
double oracle_vec_dot_q4_0_q8_0_f64(int k, const void *w_row, const void *a_row, double *abs_sum);
double oracle_vec_dot_q8_0_q8_0_f64(int k, const void *w_row, const void *a_row, double *abs_sum);

/* out fp32 [m][n]; act block_q8_0 [m][k/32]; w block_q4_0 / block_q8_0 [n][k/32].
 * weight_type: 2 = Q4_0, 8 = Q8_0 (enum ggml_type, include/dsp/quants.h:33-74).
 * n_threads > 1 splits the n range statically over pthreads. Returns 0 or -1 on bad arguments. */
int oracle_mat_mul_q8_0_act(float *out, const void *act, const void *w, int m, int k, int n, int weight_type,
                            int n_threads);
/* Same from fp32 activations (quantized with oracle_quantize_q8_0 first). */
int oracle_mat_mul_f32_act(float *out, const float *act, const void *w, int m, int k, int n, int weight_type,
                           int n_threads);
/* sum |term| per output, for tolerances: out_abs [m][n]. */
int oracle_mat_mul_q8_0_act_abs(double *out_f64, double *out_abs, const void *act, const void *w, int m, int k,
                                int n, int weight_type);

/* y = x * (1/sqrtf(mean(x^2) + eps)) [* w]; w may be NULL. fp32 left-to-right sum of squares. */
int oracle_rms_norm_f32_ex(float *dst, const float *src, const float *w, float eps, int ne0, int ne1);
/* The reference op: eps = 1e-5f, no weight. */
int oracle_rms_norm_f32(float *dst, const float *src, int ne0, int ne1);

/* Blockwise online-softmax attention, Br = 32 query rows, Bc = 256 keys per block, exp2f with
 * scale = 1/sqrtf(head_dim) * 1.44269504f. Q/O fp32 [qo_len][n_heads][head_dim]; K/V fp16 bit patterns
 * [kv_len][n_kv_heads][head_dim]; mask fp16 bit patterns [qo_len][align_up(kv_len,64)], added to the scaled
 * score, or NULL. causal != 0 additionally hides key j from query i when j > i + kv_len - qo_len.
 * Returns -1 if n_heads % n_kv_heads != 0 or head_dim > 256. */
int oracle_flash_attn(float *O, const float *Q, const uint16_t *K, const uint16_t *V, const uint16_t *mask,
                      int qo_len, int kv_len, int n_heads, int n_kv_heads, int head_dim, int causal);
/* Same with fp16 Q and O (Q widened to fp32 on load, O rounded to fp16 on store). */
int oracle_flash_attn_f16(uint16_t *O, const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                          const uint16_t *mask, int qo_len, int kv_len, int n_heads, int n_kv_heads, int head_dim,
                          int causal);

/* fp16 weights in the 32x32 tile order of the reference (tile = (n/32)*(k/32) + kk/32, element
 * (kk%32 & ~1)*32 + (n%32)*2 + (kk&1)); out[m][n] = sum_k act[m][k] * (float) w[k][n], fp32, k ascending. */
int oracle_mat_mul_w16a32(float *out, const float *act, const uint16_t *w_tiles, int m, int k, int n);

/* Index of weight element (kk, nn) inside the fp16 tile layout above. */
size_t oracle_w16_tile_index(int kk, int nn, int k);

/* Tile-permuted super-blocks of the reference's ops 2-4 (include/dsp/quants.h:16-31): n_super_blocks x 144 B
 * (Q4_0, IQ4_NL) or 272 B (Q8_0) -> 256 fp16 bit patterns each, in fp16 tile order (four super-blocks = one
 * 32x32 tile). Follows src/dsp/ops/mat_mul.c:308-508; see the .c file for what is pinned and what is not. */
void oracle_dequantize_permuted_q4_0(const void *super_blocks, int n_super_blocks, int iq4_nl, uint16_t *out);
void oracle_dequantize_permuted_q8_0(const void *super_blocks, int n_super_blocks, uint16_t *out);

/* Ops 1-4 with the reference's operand precisions: fp16 activations x fp16 (dequantized) weights, result rounded
 * to fp16 and widened. weight_kind = op id (1 fp16 tiles, 2 Q4_0, 3 Q8_0, 4 IQ4_NL). out_f64 may be NULL. */
int oracle_mat_mul_permuted(float *out, double *out_f64, const float *act, const void *weight, int m, int k, int n,
                            int weight_kind);

#ifdef __cplusplus
}
#endif

#endif /* HTP_ORACLE_H */
