// The ops of the MI355X backend: request validation, kernel selection, launches.
//
// This is the replacement for execute_op_simple (reference: src/dsp/op_executor.cc:52-204): a request is validated on
// the host exactly where the reference rejects it (mat_mul.c:878-892, rms_norm.c:69-74, flash_attn.c:1373-1376) plus
// range checks the reference lacks, then its kernels are enqueued on the context's stream.
#include "context.h"

namespace htpops {
namespace host {

// ---- op bodies on raw device pointers (validation that both the handle and the pointer entries share) ----

int op_rms_norm(htpops_context *ctx, float *dst, const float *src, const float *weight, float eps, int ne0, int ne1) {
  // reference: rms_norm.c:69-74 rejects null pointers, zero sizes and misaligned rows
  if (!dst || !src || ne0 <= 0 || ne1 <= 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "rms_norm: null buffer or non-positive size (ne0=%d ne1=%d)", ne0, ne1);
  }
  if (!aligned(dst, 4) || !aligned(src, 4) || (weight && !aligned(weight, 4))) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "rms_norm: buffers must be 4-byte aligned");
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  note_device_write(ctx, dst, (size_t) ne0 * ne1 * 4);
  HTPOPS_HIP(ctx, launch_rms_norm_f32(ctx->stream, dst, src, weight, eps, ne0, ne1));
  return HTPOPS_OK;
}

int op_quantize(htpops_context *ctx, void *dst, const float *src, int k, int m) {
  if (!dst || !src || k <= 0 || m <= 0 || k % 32 != 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "quantize_q8_0: null buffer or bad size (k=%d m=%d, k %% 32 must be 0)", k, m);
  }
  if (!aligned(dst, 4) || !aligned(src, 16)) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "quantize_q8_0: src must be 16-byte and dst 4-byte aligned");
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  note_device_write(ctx, dst, q8_0_bytes((size_t) m, (size_t) k));
  HTPOPS_HIP(ctx, launch_quantize_q8_0(ctx->stream, dst, src, k, m));
  return HTPOPS_OK;
}

int op_rms_norm_quantize(htpops_context *ctx, void *dst, const float *src, const float *weight, float eps, int ne0,
                         int ne1) {
  if (!dst || !src || ne0 <= 0 || ne1 <= 0 || ne0 % 32 != 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "rms_norm_quantize: null buffer or bad size (ne0=%d ne1=%d)", ne0, ne1);
  }
  if (!aligned(dst, 4) || !aligned(src, 16) || (weight && !aligned(weight, 16))) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "rms_norm_quantize: src/weight must be 16-byte and dst 4-byte aligned");
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  if (ne0 <= 16384) {
    note_device_write(ctx, dst, q8_0_bytes((size_t) ne1, (size_t) ne0));
    HTPOPS_HIP(ctx, launch_rms_norm_quantize_q8_0(ctx->stream, dst, src, weight, eps, ne0, ne1));
    return HTPOPS_OK;
  }
  // very long rows: normalize into the workspace, then quantize
  size_t bytes;
  if (!mul3((size_t) ne0, (size_t) ne1, 4, &bytes)) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "rms_norm_quantize: size overflow");
  }
  if (int r = ensure_workspace(ctx, bytes)) {
    return r;
  }
  note_device_write(ctx, dst, q8_0_bytes((size_t) ne1, (size_t) ne0));
  HTPOPS_HIP(ctx, launch_rms_norm_f32(ctx->stream, (float *) ctx->workspace, src, weight, eps, ne0, ne1));
  HTPOPS_HIP(ctx, launch_quantize_q8_0(ctx->stream, dst, (const float *) ctx->workspace, ne0, ne1));
  return HTPOPS_OK;
}

namespace {

int check_mat_mul(htpops_context *ctx, const void *dst, const void *act, const void *weight, int m, int k, int n,
                  int weight_type) {
  // reference: mat_mul.c:878-892
  if (!dst || !act || !weight || m <= 0 || k <= 0 || n <= 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul: null buffer or non-positive size (m=%d k=%d n=%d)", m, k, n);
  }
  if (k % 32 != 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul: k=%d is not a multiple of 32", k);
  }
  if (weight_type != kQ4_0 && weight_type != kQ8_0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul: unsupported weight type %d", weight_type);
  }
  if (!aligned(dst, 4) || !aligned(act, 2) || !aligned(weight, 2)) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul: misaligned buffer");
  }
  return HTPOPS_OK;
}

}  // namespace

// (*out stays nullptr when this matmul does not take the repacked-weight kernel: shape, weight type, activations not
// 16-byte aligned for the DMA into LDS, weights in memory whose copies may not be kept; the caller then uses the
// kernels that read the weights as they are. A failed allocation or conversion launch is an error, not a reason to
// switch kernels.)
bool prefers_block_pairs(const htpops_context *ctx, int m, int k, int n, int wt) {
  return (m == 2 || m == 3) && wt == kQ4_0 && ctx->opt.lane_order == 1 && matmul_block_pairs_fits(n, m, k, (WeightType) wt);
}

int lane_order_weights(htpops_context *ctx, const void *weight, const void *act, int m, int k, int n, int wt,
                       const void **out, bool *block_pairs) {
  *out         = nullptr;
  *block_pairs = ctx->opt.lane_order == 1 && matmul_block_pairs_fits(n, m, k, (WeightType) wt);
  if (ctx->opt.lane_order == 0 || !aligned(act, 16) ||
      !(*block_pairs || matmul_lane_order_fits(n, m, k, (WeightType) wt))) {
    return HTPOPS_OK;
  }
  const int kind = (*block_pairs ? kFragKindBlockPairs : kFragKindLaneOrder) + wt;
  if ((*out = find_copy(ctx, weight, kind, k, n)) != nullptr) {
    return HTPOPS_OK;
  }
  const size_t w_bytes = weight_bytes((size_t) n, (size_t) k, wt);
  if (!may_keep_copies(ctx, weight, w_bytes)) {
    return HTPOPS_OK;
  }
  void *fresh = nullptr;
  if (int r = new_copy(ctx, weight, w_bytes, kind, k, n, matmul_lane_order_weight_bytes(k, n, (WeightType) wt), &fresh)) {
    return r;
  }
  const hipError_t e = *block_pairs ? launch_weights_to_block_pairs(ctx->stream, fresh, weight, k, n) :
                                      launch_weights_to_lane_order(ctx->stream, fresh, weight, k, n, (WeightType) wt);
  if (e != hipSuccess) {
    forget_copy(ctx, fresh);
    return hip_fail(ctx, e, "weight repack launch");
  }
  *out = fresh;
  return HTPOPS_OK;
}

// `act_aligned`: the Q8_0 activations start on a 4-byte boundary (the re-tiling pass of the FP6 kernel reads dwords)
MatMulPlan plan_mat_mul(htpops_context *ctx, const void *weight, bool act_aligned, int m, int k, int n, int wt) {
  MatMulPlan p;
  if (m < kManyRowsMinM || k % 32 != 0) {
    p.ws_bytes = mat_mul_workspace_bytes(m, k, n);
    return p;
  }
  auto lookup_copy = [&](int frag_kind) {
    p.frag_kind = frag_kind;
    p.cached    = find_copy(ctx, weight, frag_kind, k, n);
    p.cacheable = !p.cached && may_keep_copies(ctx, weight, weight_bytes((size_t) n, (size_t) k, wt));
  };
  // Q4_0 weights whose converted copy may be kept, on a shape whose output tiles fill the device: the FP6 kernel over
  // that copy (half the vector-ALU work per block sum of the int8 path). Registered memory that was never prepared
  // (htpops_buffer_prepare_weights) may change behind the context's back, so nothing converted from it is kept, and
  // the FP6 conversion is too slow to redo per call.
  const int use_fp6 = ctx->opt.gemm_fp6;
  if (wt == kQ4_0 && use_fp6 != 0 && gemm_fp6_lds_fits(m, k, n) && aligned(weight, 4) && act_aligned &&
      (use_fp6 > 0 || gemm_fp6_lds_fills_device(m, n))) {
    lookup_copy(kFragKindFp6Tiles + wt);
    if (p.cached || p.cacheable) {
      p.kind         = kPlanLdsFp6;
      p.act_bytes    = (gemm_fp6_lds_act_tile_bytes(m, k) + 255) & ~(size_t) 255;
      p.weight_bytes = gemm_fp6_lds_weight_tile_bytes(k, n);
      p.ws_bytes     = p.act_bytes;
      return p;
    }
  }
  p.kind         = kPlanFragments;
  p.act_bytes    = (gemm_i8_act_fragment_bytes(m, k) + 255) & ~(size_t) 255;
  p.weight_bytes = (gemm_i8_weight_fragment_bytes(k, n) + 255) & ~(size_t) 255;
  lookup_copy(kFragKindRowLayout + wt);
  p.ws_bytes = p.act_bytes + ((p.cached || p.cacheable) ? 0 : p.weight_bytes) +
               ((gemm_i8_fragments_exchange_bytes(m, n, k, ctx->opt.gemm_tile_units) + 255) & ~(size_t) 255);
  return p;
}

int plan_weight_copy(htpops_context *ctx, MatMulPlan &plan, const void *weight, int k, int n, int wt, const void **out) {
  *out = plan.cached;
  if (plan.cached || !plan.cacheable || plan.kind == kPlanFewRows) {
    return HTPOPS_OK;
  }
  void *fresh = nullptr;
  if (int r = new_copy(ctx, weight, weight_bytes((size_t) n, (size_t) k, wt), plan.frag_kind, k, n, plan.weight_bytes, &fresh)) {
    return r;
  }
  const hipError_t e = plan.kind == kPlanLdsFp6 ? launch_q4_0_to_fp6_tiles(ctx->stream, fresh, weight, k, n) :
                                                  launch_weights_to_i8_fragments(ctx->stream, fresh, weight, k, n, (WeightType) wt);
  if (e != hipSuccess) {
    forget_copy(ctx, fresh);
    return fail(ctx, HTPOPS_ERR_HIP, "weight conversion: %s", hipGetErrorString(e));
  }
  plan.cached = fresh, plan.cacheable = false;
  *out = fresh;
  return HTPOPS_OK;
}

namespace {

int run_few_rows(htpops_context *ctx, float *dst, const void *act, const void *weight, int m, int k, int n, int wt,
                 uint8_t *ws) {
  // hipErrorNotSupported from a launcher means "this kernel does not take the shape": try the next one. Any other
  // failure is reported.
  const void *lw    = nullptr;
  bool        pairs = false;
  if (prefers_block_pairs(ctx, m, k, n, wt)) {
    if (int r = lane_order_weights(ctx, weight, act, m, k, n, wt, &lw, &pairs)) {
      return r;
    }
  }
  if (!lw && ctx->opt.gemv_rows_kernel != 0 && gemv_rows_fits(m, k, (WeightType) wt) && aligned(act, 4) && aligned(weight, 4)) {
    const hipError_t e = launch_gemv_rows_group_q8_0_act(ctx->stream, 1, &dst, &act, &weight, &n, m, &k,
                                                                 (WeightType) wt);
    if (e == hipSuccess) {
      return HTPOPS_OK;
    }
    if (e != hipErrorNotSupported) {
      return hip_fail(ctx, e, "few-row mat_mul launch");
    }
    (void) hipGetLastError();
  }
  if (!lw) {
    if (int r = lane_order_weights(ctx, weight, act, m, k, n, wt, &lw, &pairs)) {
      return r;
    }
  }
  if (lw) {
    const hipError_t e = pairs ? launch_matmul_block_pairs_group(ctx->stream, 1, &dst, &act, &lw, &n, m, &k) :
                                 launch_matmul_lane_order_group(ctx->stream, 1, &dst, &act, &lw, &n, m, k, (WeightType) wt,
                                                                ctx->opt.lane_order);
    if (e == hipSuccess) {
      return HTPOPS_OK;
    }
    if (e != hipErrorNotSupported) {
      return hip_fail(ctx, e, "repacked-weight mat_mul launch");
    }
    (void) hipGetLastError();
  }
  HTPOPS_HIP(ctx, launch_mat_mul_q8_0_act(ctx->stream, dst, act, weight, m, k, n, (WeightType) wt, ws,
                                                  ctx->tickets, kTicketSlots));
  return HTPOPS_OK;
}

// `ws` is this matmul's share of the workspace (plan.ws_bytes, already ensured by the caller)
int run_mat_mul(htpops_context *ctx, MatMulPlan &plan, float *dst, const void *act, const void *weight, int m, int k,
                int n, int wt, uint8_t *ws) {
  note_device_write(ctx, dst, (size_t) m * n * 4);
  if (plan.kind == kPlanFewRows) {
    ctx->act_fragments.src = nullptr;  // these kernels put something else at the start of the workspace
    return run_few_rows(ctx, dst, act, weight, m, k, n, wt, ws);
  }
  // the converted copy of the weights, for the kernels that want one: kept with the buffer, or (weights whose copies
  // may not be kept; int8 fragments only) made in the workspace for this call
  const void *frags = nullptr;
  if (int r = plan_weight_copy(ctx, plan, weight, k, n, wt, &frags)) {
    return r;
  }
  if (!frags) {
    void            *fresh = ws + plan.act_bytes;
    const hipError_t e     = launch_weights_to_i8_fragments(ctx->stream, fresh, weight, k, n, (WeightType) wt);
    if (e != hipSuccess) {
      return fail(ctx, HTPOPS_ERR_HIP, "weight conversion: %s", hipGetErrorString(e));
    }
    frags = fresh;
  }
  // The converted activations at the start of the workspace are shared by the requests of a message that read the same
  // rows with the same kernel family (note_device_write above has already cleared the record if this matmul writes
  // into its own activations).
  auto      &af    = ctx->act_fragments;
  const bool ready = af.src == act && af.m == m && af.k == k && af.kind == (int) plan.kind && ws == ctx->workspace;
  const bool keep  = ready || (ctx->in_message && ws == ctx->workspace &&
                               !ranges_overlap(dst, (size_t) m * n * 4, act, q8_0_bytes((size_t) m, (size_t) k)));
  af.src = nullptr;
  if (plan.kind == kPlanLdsFp6) {
    HTPOPS_HIP(ctx, launch_gemm_fp6_lds(ctx->stream, dst, act, frags, m, k, n, ws, ready));
  } else {
    // (scratch for partial tiles at the end of this matmul's share of the workspace)
    const size_t xbytes = gemm_i8_fragments_exchange_bytes(m, n, k, ctx->opt.gemm_tile_units);
    HTPOPS_HIP(ctx, launch_gemm_i8_fragments(ctx->stream, dst, act, frags, m, k, n, ws, ready,
                                             ws + plan.ws_bytes - ((xbytes + 255) & ~(size_t) 255), xbytes, ctx->tickets,
                                             kTicketSlots, ctx->opt.gemm_tile_units));
  }
  if (keep) {
    af.src = act, af.src_bytes = q8_0_bytes((size_t) m, (size_t) k), af.m = m, af.k = k, af.kind = (int) plan.kind;
  }
  return HTPOPS_OK;
}

}  // namespace

int op_mat_mul_q8(htpops_context *ctx, float *dst, const void *act, const void *weight, int m, int k, int n,
                  int weight_type) {
  if (int r = check_mat_mul(ctx, dst, act, weight, m, k, n, weight_type)) {
    return r;
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  MatMulPlan plan = plan_mat_mul(ctx, weight, aligned(act, 4), m, k, n, weight_type);
  if (int r = ensure_workspace(ctx, plan.ws_bytes, /*keep_act_fragments=*/true)) {
    return r;
  }
  return run_mat_mul(ctx, plan, dst, act, weight, m, k, n, weight_type, static_cast<uint8_t *>(ctx->workspace));
}

int op_mat_mul_f32(htpops_context *ctx, float *dst, const float *act, const void *weight, int m, int k, int n,
                   int weight_type) {
  if (int r = check_mat_mul(ctx, dst, act, weight, m, k, n, weight_type)) {
    return r;
  }
  if (!aligned(act, 16)) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul: fp32 activations must be 16-byte aligned");
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  // workspace: [quantized activations][what the matmul itself needs]
  const size_t q_bytes = (q8_0_bytes((size_t) m, (size_t) k) + 255) & ~(size_t) 255;
  MatMulPlan   plan    = plan_mat_mul(ctx, weight, true, m, k, n, weight_type);
  if (int r = ensure_workspace(ctx, q_bytes + plan.ws_bytes)) {
    return r;
  }
  uint8_t *ws = static_cast<uint8_t *>(ctx->workspace);
  HTPOPS_HIP(ctx, launch_quantize_q8_0(ctx->stream, ws, act, k, m));
  return run_mat_mul(ctx, plan, dst, ws, weight, m, k, n, weight_type, ws + q_bytes);
}

// hmx_mat_mul_permuted_w16a32 / hmx_mat_mul_permuted_qk_0_d16a32 (reference: src/dsp/ops/mat_mul.c:758-855, :875-1153)
int op_mat_mul_permuted(htpops_context *ctx, float *dst, const float *act, const void *weight, int m, int k, int n,
                        int kind) {
  // reference: mat_mul.c:760-769, :878-892
  if (!dst || !act || !weight || m <= 0 || k <= 0 || n <= 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul_permuted: null buffer or non-positive size (m=%d k=%d n=%d)", m, k, n);
  }
  if (k % 32 != 0 || n % 32 != 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul_permuted: k=%d and n=%d must be multiples of 32", k, n);
  }
  if (!aligned(dst, 128) || !aligned(act, 128) || !aligned(weight, 128)) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul_permuted: buffers must be 128-byte aligned");
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  note_device_write(ctx, dst, (size_t) m * n * 4);
  const void *frag = find_copy(ctx, weight, kind, k, n);
  // Converted copies are kept only for weights in buffers the context allocated (their contents change only through
  // htpops_buffer_write or as an op's output, both of which drop the copy). Caller-registered memory may be rewritten
  // behind the context's back: it is converted into the workspace on every call.
  const size_t act_bytes  = (permuted_act_fragment_bytes(m, k) + 255) & ~(size_t) 255;
  const size_t frag_bytes = permuted_weight_fragment_bytes(k, n);
  const bool   cacheable  = !frag && may_keep_copies(ctx, weight, permuted_weight_bytes((size_t) n, (size_t) k, kind));
  if (int r = ensure_workspace(ctx, act_bytes + ((frag || cacheable) ? 0 : frag_bytes))) {
    return r;
  }
  if (!frag) {
    void *fresh = static_cast<uint8_t *>(ctx->workspace) + act_bytes;
    if (cacheable) {
      if (int r = new_copy(ctx, weight, permuted_weight_bytes((size_t) n, (size_t) k, kind), kind, k, n, frag_bytes, &fresh)) {
        return r;
      }
    }
    const hipError_t e = launch_permuted_weight_to_fragments(ctx->stream, fresh, weight, k, n, kind);
    if (e != hipSuccess) {
      if (cacheable) {
        forget_copy(ctx, fresh);
      }
      return fail(ctx, HTPOPS_ERR_HIP, "weight conversion: %s", hipGetErrorString(e));
    }
    frag = fresh;
  }
  HTPOPS_HIP(ctx, launch_mat_mul_fragments(ctx->stream, dst, act, frag, m, k, n, ctx->workspace));
  return HTPOPS_OK;
}

int op_flash_attn(htpops_context *ctx, void *o, const void *q, const void *k, const void *v, const void *mask,
                  int qo_len, int kv_len, int n_heads, int n_kv_heads, int head_dim, int qo_is_f32, int causal,
                  bool no_alloc) {
  if (!o || !q || !k || !v || qo_len <= 0 || kv_len <= 0 || n_heads <= 0 || n_kv_heads <= 0 || head_dim <= 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "flash_attn: null buffer or non-positive size");
  }
  // reference: flash_attn.c:1373-1376
  if (n_heads % n_kv_heads != 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "flash_attn: n_heads=%d is not a multiple of n_kv_heads=%d", n_heads,
                n_kv_heads);
  }
  // reference: flash_attn_sp_hdim.c:785-788 (an odd head_dim is refused); 64 and 128 take the MFMA kernels, every
  // other even head_dim up to 256 the general one
  if (head_dim % 2 != 0 || head_dim > 256) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "flash_attn: head_dim=%d (even values up to 256 are built)", head_dim);
  }
  if (!aligned(o, 16) || !aligned(q, 16) || !aligned(k, 16) || !aligned(v, 16) || (mask && !aligned(mask, 8))) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "flash_attn: q/k/v/o must be 16-byte aligned, the mask 8-byte aligned");
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  const size_t ws_bytes = flash_attn_workspace_bytes(qo_len, kv_len, n_heads, head_dim);
  const size_t o_bytes  = (size_t) qo_len * n_heads * head_dim * (qo_is_f32 ? 4 : 2);
  void        *ws       = nullptr;
  if (no_alloc) {
    // nothing may be allocated or freed here: the partials go to this device's static scratch array, and an output
    // that would overwrite weights with a converted copy (whose release is a hipFree) is refused instead
    if (ws_bytes > kNoAllocScratchBytes) {
      return fail(ctx, HTPOPS_ERR_REJECTED,
                  "flash_attn (no allocation): %zu bytes of split-KV partials exceed the %zu-byte static scratch "
                  "(n_heads * ceil(kv_len / 64) * (head_dim + 2) * 4 must fit)", ws_bytes, kNoAllocScratchBytes);
    }
    for (const auto &e : ctx->frag_cache) {
      if (ranges_overlap(o, o_bytes, e.src, e.src_bytes)) {
        return fail(ctx, HTPOPS_ERR_REJECTED, "flash_attn (no allocation): the output overlaps cached weights");
      }
    }
    if (ctx->act_fragments.src && ranges_overlap(o, o_bytes, ctx->act_fragments.src, ctx->act_fragments.src_bytes)) {
      ctx->act_fragments.src = nullptr;
    }
    if (ws_bytes > 0 && !claim_static_scratch(ctx)) {
      return fail(ctx, HTPOPS_ERR_BUSY,
                  "flash_attn (no allocation): another context on this GPU is using the static scratch and has not "
                  "synchronized since");
    }
    ws = ctx->scratch_ptr;
  } else {
    if (int r = ensure_workspace(ctx, ws_bytes)) {
      return r;
    }
    note_device_write(ctx, o, o_bytes);
    ws = ctx->workspace;
  }
  void *q8_out = nullptr;
  if (ctx->attn_q8_out && flash_attn_writes_q8_0(qo_len, head_dim, qo_is_f32 != 0)) {
    q8_out = ctx->attn_q8_out;
    note_device_write(ctx, q8_out, q8_0_bytes(1, (size_t) n_heads * head_dim));
  }
  HTPOPS_HIP(ctx, launch_flash_attn(ctx->stream, o, q, k, v, mask, qo_len, kv_len, n_heads, n_kv_heads, head_dim,
                                    qo_is_f32 != 0, causal != 0, ws, q8_out, ctx->opt.attn_key_groups,
                                    ctx->opt.attn_mask_threshold != 0));
  ctx->attn_q8_done = q8_out != nullptr;
  return HTPOPS_OK;
}


}  // namespace host
}  // namespace htpops

using namespace htpops;
using namespace htpops::host;

// ------------------------------------------------------------------------------------------------ ops

extern "C" int htpops_execute_op(htpops_context *ctx, const struct OpComputeRequest *req) {
  if (!ctx || !req) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  if (!ctx->in_message) {
    ++ctx->use_serial;
  }
  switch (req->op) {
    case HTP_OPS_RMS_NORM_F32:
      {
        // reference: op_executor.cc:82-94
        const auto *p = reinterpret_cast<const RmsNormF32Params *>(req->payload);
        size_t      bytes;
        if (p->ne0 <= 0 || p->ne1 <= 0 || !mul3((size_t) p->ne0, (size_t) p->ne1, 4, &bytes)) {
          return fail(ctx, HTPOPS_ERR_REJECTED, "rms_norm: bad size (ne0=%d ne1=%d)", p->ne0, p->ne1);
        }
        return op_rms_norm(ctx, (float *) resolve(ctx, p->dst, bytes), (const float *) resolve(ctx, p->src, bytes),
                           nullptr, 1e-5f, p->ne0, p->ne1);
      }
    case HTP_OPS_RMS_NORM_F32_EX:
    case HTP_OPS_RMS_NORM_QUANTIZE_Q8_0:
      {
        const auto *p = reinterpret_cast<const RmsNormExParams *>(req->payload);
        size_t      bytes;
        if (p->ne0 <= 0 || p->ne1 <= 0 || !mul3((size_t) p->ne0, (size_t) p->ne1, 4, &bytes)) {
          return fail(ctx, HTPOPS_ERR_REJECTED, "rms_norm: bad size (ne0=%d ne1=%d)", p->ne0, p->ne1);
        }
        const float *w = nullptr;
        if (p->weight.fd >= 0) {
          w = (const float *) resolve(ctx, p->weight, (size_t) p->ne0 * 4);
          if (!w) {
            return fail(ctx, HTPOPS_ERR_REJECTED, "rms_norm: unknown weight buffer");
          }
        }
        const float *src = (const float *) resolve(ctx, p->src, bytes);
        if (req->op == HTP_OPS_RMS_NORM_F32_EX) {
          return op_rms_norm(ctx, (float *) resolve(ctx, p->dst, bytes), src, w, p->eps, p->ne0, p->ne1);
        }
        if (p->ne0 % 32 != 0) {
          return fail(ctx, HTPOPS_ERR_REJECTED, "rms_norm_quantize: ne0=%d is not a multiple of 32", p->ne0);
        }
        return op_rms_norm_quantize(ctx, resolve(ctx, p->dst, q8_0_bytes((size_t) p->ne1, (size_t) p->ne0)), src, w,
                                    p->eps, p->ne0, p->ne1);
      }
    case HTP_OPS_QUANTIZE_Q8_0:
      {
        const auto *p = reinterpret_cast<const RmsNormF32Params *>(req->payload);
        size_t      bytes;
        if (p->ne0 <= 0 || p->ne1 <= 0 || p->ne0 % 32 != 0 || !mul3((size_t) p->ne0, (size_t) p->ne1, 4, &bytes)) {
          return fail(ctx, HTPOPS_ERR_REJECTED, "quantize_q8_0: bad size (ne0=%d ne1=%d)", p->ne0, p->ne1);
        }
        return op_quantize(ctx, resolve(ctx, p->dst, q8_0_bytes((size_t) p->ne1, (size_t) p->ne0)),
                           (const float *) resolve(ctx, p->src, bytes), p->ne0, p->ne1);
      }
    case HTP_OPS_MAT_MUL_Q4_0_Q8_0:
    case HTP_OPS_MAT_MUL_Q8_0_Q8_0:
    case HTP_OPS_MAT_MUL_Q4_0_A32:
    case HTP_OPS_MAT_MUL_Q8_0_A32:
      {
        // reference: op_executor.cc:114-149 (sizes), with ggml row-layout weights
        const auto *p  = reinterpret_cast<const MatMulParams *>(req->payload);
        const int   wt = (req->op == HTP_OPS_MAT_MUL_Q4_0_Q8_0 || req->op == HTP_OPS_MAT_MUL_Q4_0_A32) ? kQ4_0 :
                                                                                                         kQ8_0;
        const bool  f32_act = req->op == HTP_OPS_MAT_MUL_Q4_0_A32 || req->op == HTP_OPS_MAT_MUL_Q8_0_A32;
        size_t      out_bytes, act_bytes;
        if (p->m <= 0 || p->k <= 0 || p->n <= 0 || p->k % 32 != 0 ||
            !mul3((size_t) p->m, (size_t) p->n, 4, &out_bytes) || !mul3((size_t) p->m, (size_t) p->k, 4, &act_bytes)) {
          return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul: bad size (m=%d k=%d n=%d)", p->m, p->k, p->n);
        }
        float      *out = (float *) resolve(ctx, p->output, out_bytes);
        const void *w   = resolve(ctx, p->weight, weight_bytes((size_t) p->n, (size_t) p->k, wt));
        if (f32_act) {
          return op_mat_mul_f32(ctx, out, (const float *) resolve(ctx, p->activation, act_bytes), w, p->m, p->k, p->n,
                                wt);
        }
        return op_mat_mul_q8(ctx, out, resolve(ctx, p->activation, q8_0_bytes((size_t) p->m, (size_t) p->k)), w, p->m,
                             p->k, p->n, wt);
      }
    case HTP_OPS_FLASH_ATTN_QO_F32_KV_F16:
    case HTP_OPS_FLASH_ATTN_F16:
      {
        // reference: op_executor.cc:151-196
        const bool  ext    = req->op == HTP_OPS_FLASH_ATTN_F16;
        const auto *p      = reinterpret_cast<const FlashAttnParams *>(req->payload);
        const int   causal = ext ? reinterpret_cast<const FlashAttnExParams *>(req->payload)->causal : 0;
        if (p->qo_len <= 0 || p->kv_len <= 0 || p->n_heads <= 0 || p->n_kv_heads <= 0 || p->head_dim <= 0) {
          return fail(ctx, HTPOPS_ERR_REJECTED, "flash_attn: non-positive size");
        }
        size_t qo_elems, kv_elems, qo_bytes, kv_bytes, mask_bytes;
        if (!mul3((size_t) p->qo_len, (size_t) p->n_heads, (size_t) p->head_dim, &qo_elems) ||
            !mul3((size_t) p->kv_len, (size_t) p->n_kv_heads, (size_t) p->head_dim, &kv_elems) ||
            !mul3(qo_elems, ext ? 2 : 4, 1, &qo_bytes) || !mul3(kv_elems, 2, 1, &kv_bytes) ||
            !mul3((size_t) p->qo_len, ((size_t) p->kv_len + 63) / 64 * 64, 2, &mask_bytes)) {
          return fail(ctx, HTPOPS_ERR_REJECTED, "flash_attn: size overflow");
        }
        const void *mask = nullptr;
        if (p->mask.fd >= 0 && lookup(ctx, p->mask.fd)) {
          // the kernel strides the mask by align_up(kv_len, 64) (reference: flash_attn.c:152)
          mask = resolve(ctx, p->mask, mask_bytes);
          if (!mask) {
            return fail(ctx, HTPOPS_ERR_REJECTED, "flash_attn: mask buffer smaller than qo_len * align_up(kv_len, 64) * 2");
          }
        }
        return op_flash_attn(ctx, resolve(ctx, p->o, qo_bytes), resolve(ctx, p->q, qo_bytes),
                             resolve(ctx, p->k, kv_bytes), resolve(ctx, p->v, kv_bytes), mask, p->qo_len, p->kv_len,
                             p->n_heads, p->n_kv_heads, p->head_dim, ext ? 0 : 1, causal);
      }
    case HTP_OPS_MAT_MUL_PERMUTED_W16A32:
    case HTP_OPS_MAT_MUL_PERMUTED_W4D16A32:
    case HTP_OPS_MAT_MUL_PERMUTED_W8D16A32:
    case HTP_OPS_MAT_MUL_PERMUTED_W4D16A32_IQ4_NL:
      {
        // reference: op_executor.cc:96-149; the op id doubles as the weight kind
        const auto *p    = reinterpret_cast<const MatMulParams *>(req->payload);
        const int   kind = (int) req->op;
        size_t      out_bytes, act_bytes;
        if (p->m <= 0 || p->k <= 0 || p->n <= 0 || p->k % 32 != 0 || p->n % 32 != 0 ||
            !mul3((size_t) p->m, (size_t) p->n, 4, &out_bytes) || !mul3((size_t) p->m, (size_t) p->k, 4, &act_bytes)) {
          return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul_permuted: bad size (m=%d k=%d n=%d)", p->m, p->k, p->n);
        }
        return op_mat_mul_permuted(ctx, (float *) resolve(ctx, p->output, out_bytes),
                                   (const float *) resolve(ctx, p->activation, act_bytes),
                                   resolve(ctx, p->weight, permuted_weight_bytes((size_t) p->n, (size_t) p->k, kind)),
                                   p->m, p->k, p->n, kind);
      }
    default:
      // the reference returns 0 without touching anything (op_executor.cc:200-203); a silent success on an
      // unknown op hides host bugs, so this backend reports it
      return fail(ctx, HTPOPS_ERR_REJECTED, "unknown op %u", req->op);
  }
}

// ------------------------------------------------------------------------------------------------ direct entries

extern "C" int htpops_rms_norm_f32(htpops_context *ctx, int dst_fd, int dst_offset, int src_fd, int src_offset,
                                   int ne0, int ne1) {
  struct {
    struct OpComputeRequest req;
    struct RmsNormF32Params params;
  } HTPOPS_PACKED r;
  r.req.op     = HTP_OPS_RMS_NORM_F32;
  r.params.dst = { dst_fd, dst_offset };
  r.params.src = { src_fd, src_offset };
  r.params.ne0 = ne0;
  r.params.ne1 = ne1;
  int ret      = htpops_execute_op(ctx, &r.req);
  if (ret != HTPOPS_OK) {
    return ret;
  }
  return htpops_synchronize(ctx);
}

extern "C" int htpops_mat_mul_permuted_w16a32(htpops_context *ctx, int output_fd, int output_offset,
                                              int activation_fd, int activation_offset, int weight_fd,
                                              int weight_offset, int m, int k, int n) {
  struct {
    struct OpComputeRequest req;
    struct MatMulParams     params;
  } HTPOPS_PACKED r;
  r.req.op            = HTP_OPS_MAT_MUL_PERMUTED_W16A32;
  r.params.output     = { output_fd, output_offset };
  r.params.activation = { activation_fd, activation_offset };
  r.params.weight     = { weight_fd, weight_offset };
  r.params.m          = m;
  r.params.k          = k;
  r.params.n          = n;
  int ret             = htpops_execute_op(ctx, &r.req);
  if (ret != HTPOPS_OK) {
    return ret;
  }
  return htpops_synchronize(ctx);
}

// ------------------------------------------------------------------------------------------------ pointer entries

extern "C" int htpops_rms_norm_f32_ex_ptr(htpops_context *ctx, float *dst, const float *src, const float *weight,
                                          float eps, int ne0, int ne1) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  return op_rms_norm(ctx, dst, src, weight, eps, ne0, ne1);
}

extern "C" int htpops_quantize_q8_0_ptr(htpops_context *ctx, void *dst, const float *src, int k, int m) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  return op_quantize(ctx, dst, src, k, m);
}

extern "C" int htpops_rms_norm_quantize_q8_0_ptr(htpops_context *ctx, void *dst, const float *src,
                                                 const float *weight, float eps, int ne0, int ne1) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  return op_rms_norm_quantize(ctx, dst, src, weight, eps, ne0, ne1);
}

extern "C" int htpops_mat_mul_q8_0_act_ptr(htpops_context *ctx, float *dst, const void *act_q8_0, const void *weight,
                                           int m, int k, int n, int weight_type) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  return op_mat_mul_q8(ctx, dst, act_q8_0, weight, m, k, n, weight_type);
}

extern "C" int htpops_mat_mul_f32_act_ptr(htpops_context *ctx, float *dst, const float *act, const void *weight, int m,
                                          int k, int n, int weight_type) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  return op_mat_mul_f32(ctx, dst, act, weight, m, k, n, weight_type);
}

extern "C" int htpops_flash_attn_ptr(htpops_context *ctx, void *o, const void *q, const void *k, const void *v,
                                     const void *mask, int qo_len, int kv_len, int n_heads, int n_kv_heads,
                                     int head_dim, int qo_is_f32, int causal) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  return op_flash_attn(ctx, o, q, k, v, mask, qo_len, kv_len, n_heads, n_kv_heads, head_dim, qo_is_f32, causal);
}

extern "C" int htpops_flash_attn_noalloc_ptr(htpops_context *ctx, void *o, const void *q, const void *k, const void *v,
                                             const void *mask, int qo_len, int kv_len, int n_heads, int n_kv_heads,
                                             int head_dim, int qo_is_f32, int causal) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  return op_flash_attn(ctx, o, q, k, v, mask, qo_len, kv_len, n_heads, n_kv_heads, head_dim, qo_is_f32, causal,
                       /*no_alloc=*/true);
}
