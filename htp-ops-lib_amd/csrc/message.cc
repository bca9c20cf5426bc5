// The consumer's walk over a message (reference: src/dsp/commu.c:91-126): every request in order, each op's return code
// into RequestHeader.state, RPCMEM_MAP puts as handle releases, completion published through the state bytes. On top
// of the reference's one-op-per-request loop, consecutive matmul requests that nothing orders share a kernel launch.
#include "context.h"

#include <cstring>

namespace htpops {
namespace host {

uint64_t load_state(struct MessageHeader *msg) {
  void *p = static_cast<void *>(msg);
  if (aligned(p, 8)) {
    return __atomic_load_n(static_cast<uint64_t *>(__builtin_assume_aligned(p, 8)), __ATOMIC_ACQUIRE);
  }
  uint64_t d;
  memcpy(&d, p, 8);
  __atomic_thread_fence(__ATOMIC_ACQUIRE);
  return d;
}

void store_state(struct MessageHeader *msg, uint64_t d) {
  void *p = static_cast<void *>(msg);
  if (aligned(p, 8)) {
    __atomic_store_n(static_cast<uint64_t *>(__builtin_assume_aligned(p, 8)), d, __ATOMIC_RELEASE);
    return;
  }
  __atomic_thread_fence(__ATOMIC_RELEASE);
  memcpy(p, &d, 8);
}

namespace {


// Consecutive matmul requests of a message are collected and run as one kernel launch when that cannot change any
// result: the result of every request is what its own launch would have produced (same kernel, same arithmetic), the
// requests just stop paying a launch and a ramp-up each. The reference runs requests strictly in order
// (src/dsp/commu.c:91-114); a request therefore joins the open batch only if it neither reads (activations, weights)
// nor overwrites anything an earlier member of the batch writes, and writes nothing an earlier member reads.
//  * one activation row (decode): members may read different activation buffers and have different k -- a whole
//    hazard-free run of matrix-vector products (the seven projections of a layer whose inputs are all ready) is one
//    launch; where a real data dependency exists (o after attention after q/k/v) the run is split there;
//  * 2..16 rows: members of the same k; those that take the repacked-weight kernel share its launch whatever rows
//    they read, the others only with members that read the same rows (q/k/v or gate/up);
//  * many rows on small output tiles: one launch for the products, one for the activation conversions.
struct GemvBatch {
  int                   wt = 0, m = 0, count = 0;
  struct RequestHeader *hdr[kGemvGroupMax];
  float                *out[kGemvGroupMax];
  const void           *w[kGemvGroupMax];
  const void           *act[kGemvGroupMax];
  int                   n[kGemvGroupMax];
  int                   k[kGemvGroupMax];
  // A one-row RMSNorm + Q8_0 (or plain Q8_0 quantization) request that waits for the matmuls that read its row (the
  // decode chain): when only such matmuls follow, one launch makes the row and multiplies by it; anything else runs
  // the request first, as it came.
  struct {
    bool                  waiting = false;
    bool                  normalize = true;  // false: the request is a plain quantization
    struct RequestHeader *hdr     = nullptr;
    void                 *dst     = nullptr;
    const float          *src = nullptr, *weight = nullptr;
    float                 eps = 0.0f;
    int                   ne0 = 0;
  } norm;
  bool fused = false;  // the members read norm.dst and run in the launch that makes it
  bool fp6   = false;  // many-row members of the FP6-tile kernel (all over the same activation rows and k)
  bool pairs_fit = false;  // every member fits the two-blocks-per-instruction kernel (such members may differ in k)
};

// The many-row members of a batch: converted weights from the cache (made now where missing), the distinct activation
// matrices converted side by side in the workspace by one launch, then one launch for all the products. Returns a
// status, or 1 when the members have to be run one by one after all.
static_assert(kGemmGroupMax == kGemvGroupMax, "one batch structure serves both");
int run_fragment_group(htpops_context *ctx, GemvBatch &b) {
  const void *wf[kGemmGroupMax];
  for (int i = 0; i < b.count; ++i) {
    MatMulPlan plan = plan_mat_mul(ctx, b.w[i], true, b.m, b.k[i], b.n[i], b.wt);
    if (plan.kind != kPlanFragments || !(plan.cached || plan.cacheable)) {
      return 1;  // (a converted copy went away since the member joined: the caller runs the members one by one)
    }
    if (int r = plan_weight_copy(ctx, plan, b.w[i], b.k[i], b.n[i], b.wt, &wf[i])) {
      return r;
    }
  }
  // distinct (activation, k) pairs and where their conversions go
  const void *acts[kGemmGroupMax];
  int         act_k[kGemmGroupMax], act_of[kGemmGroupMax], n_acts = 0;
  size_t      offset[kGemmGroupMax], total = 0;
  for (int i = 0; i < b.count; ++i) {
    int j = 0;
    while (j < n_acts && !(acts[j] == b.act[i] && act_k[j] == b.k[i])) {
      ++j;
    }
    if (j == n_acts) {
      acts[j] = b.act[i], act_k[j] = b.k[i], offset[j] = total;
      total += (gemm_i8_act_fragment_bytes(b.m, b.k[i]) + 255) & ~(size_t) 255;
      ++n_acts;
    }
    act_of[i] = j;
  }
  size_t xbytes = 0;  // scratch for the partial tiles of members whose K is split over workgroups, behind the activations
  for (int i = 0; i < b.count; ++i) {
    xbytes += gemm_i8_fragments_exchange_bytes(b.m, b.n[i], b.k[i], ctx->opt.gemm_tile_units);
  }
  if (int r = ensure_workspace(ctx, total + xbytes)) {
    return r;
  }
  ctx->act_fragments.src = nullptr;
  uint8_t    *ws = static_cast<uint8_t *>(ctx->workspace);
  void       *act_dst[kGemmGroupMax];
  const void *af[kGemmGroupMax];
  for (int j = 0; j < n_acts; ++j) {
    act_dst[j] = ws + offset[j];
  }
  for (int i = 0; i < b.count; ++i) {
    af[i] = act_dst[act_of[i]];
  }
  HTPOPS_HIP(ctx, launch_act_to_i8_fragments_group(ctx->stream, n_acts, act_dst, acts, act_k, b.m));
  HTPOPS_HIP(ctx, launch_gemm_i8_fragments_group(ctx->stream, b.count, b.out, af, wf, b.n, b.k, b.m, ws + total, xbytes,
                                                 ctx->tickets, kTicketSlots, ctx->opt.gemm_tile_units));
  return HTPOPS_OK;
}

// The many-row members of a batch that take the FP6-tile kernel over one set of activation rows: converted weights from
// the cache (made now where missing), the activations converted once (or found converted at the start of the
// workspace), one launch per kernel variant for the products. Returns a status, or 1 when the members have to be run
// one by one after all.
int run_fp6_group(htpops_context *ctx, GemvBatch &b) {
  const void *wf[kGemmGroupMax];
  size_t      act_bytes = 0;
  for (int i = 0; i < b.count; ++i) {
    MatMulPlan plan = plan_mat_mul(ctx, b.w[i], true, b.m, b.k[i], b.n[i], b.wt);
    if (plan.kind != kPlanLdsFp6 || !(plan.cached || plan.cacheable)) {
      return 1;  // (a converted copy went away since the member joined: the caller runs the members one by one)
    }
    if (int r = plan_weight_copy(ctx, plan, b.w[i], b.k[i], b.n[i], b.wt, &wf[i])) {
      return r;
    }
    act_bytes = plan.act_bytes;
  }
  if (int r = ensure_workspace(ctx, act_bytes, true)) {  // (tiles already there for these rows stay)
    return r;
  }
  // (note_device_write for the outputs, done by the caller, has already dropped the record if a member writes into
  // the activations)
  const int    m = b.m, k = b.k[0];
  const size_t a_bytes = q8_0_bytes((size_t) m, (size_t) k);
  auto        &af      = ctx->act_fragments;
  const bool   ready   = af.src == b.act[0] && af.m == m && af.k == k && af.kind == (int) kPlanLdsFp6;
  bool         keep    = ready || ctx->in_message;
  for (int i = 0; i < b.count; ++i) {
    keep = keep && !ranges_overlap(b.out[i], (size_t) m * b.n[i] * 4, b.act[0], a_bytes);
  }
  af.src = nullptr;
  HTPOPS_HIP(ctx, launch_gemm_fp6_lds_group(ctx->stream, b.count, b.out, b.act[0], wf, m, k, b.n, ctx->workspace, ready));
  if (keep) {
    af.src = b.act[0], af.src_bytes = a_bytes, af.m = m, af.k = k, af.kind = (int) kPlanLdsFp6;
  }
  return HTPOPS_OK;
}

void flush_batch(htpops_context *ctx, GemvBatch &b) {
  if (b.norm.waiting) {
    b.norm.waiting = false;
    const size_t q_bytes = q8_0_bytes(1, (size_t) b.norm.ne0);
    if (b.fused && b.count > 0) {
      b.fused = false;
      note_device_write(ctx, b.norm.dst, q_bytes);
      for (int i = 0; i < b.count; ++i) {
        note_device_write(ctx, b.out[i], (size_t) b.n[i] * 4);
      }
      const hipError_t e = launch_gemv_group_rms_norm_q8_0_act(ctx->stream, b.count, b.out, b.w, b.n, b.norm.ne0,
                                                                       (WeightType) b.wt, b.norm.src,
                                                                       b.norm.weight, b.norm.eps, b.norm.dst,
                                                                       b.norm.normalize);
      if (e != hipErrorNotSupported) {
        ++ctx->message_submissions;
        if (e != hipSuccess) {
          const int ret = fail(ctx, HTPOPS_ERR_HIP, "rms_norm + mat_mul launch: %s", hipGetErrorString(e));
          b.norm.hdr->state = ret;
          for (int i = 0; i < b.count; ++i) {
            b.hdr[i]->state = ret;
          }
        }
        b.count = 0;
        return;
      }
      (void) hipGetLastError();
    }
    b.fused = false;
    ++ctx->message_submissions;
    b.norm.hdr->state = b.norm.normalize ?
                          op_rms_norm_quantize(ctx, b.norm.dst, b.norm.src, b.norm.weight, b.norm.eps, b.norm.ne0, 1) :
                          op_quantize(ctx, b.norm.dst, b.norm.src, b.norm.ne0, 1);
  }
  if (b.count == 0) {
    return;
  }
  ++ctx->message_submissions;
  int ret = HTPOPS_OK;
  if (b.count > 1) {
    for (int i = 0; i < b.count; ++i) {
      note_device_write(ctx, b.out[i], (size_t) b.m * b.n[i] * 4);
    }
    const int        k0 = b.k[0];
    hipError_t e;
    if (b.m > kBatchMaxM) {
      ret = b.fp6 ? run_fp6_group(ctx, b) : run_fragment_group(ctx, b);
      e   = ret == 1 ? hipErrorNotSupported : hipSuccess;
      ret = ret == 1 ? HTPOPS_OK : ret;
    } else if (b.m == 1) {
      e = launch_gemv_group_q8_0_act(ctx->stream, b.count, b.out, b.act, b.w, b.n, b.k, (WeightType) b.wt);
    } else {
      // 2..16 rows. Which kernel a matrix gets depends on that matrix alone, in the order of the single request
      // (run_few_rows): two and three rows of Q4_0 that fit the two-blocks-per-instruction kernel and have, or get, their
      // repacked copy go there; other two- and three-row members to the weight stream that keeps the rows in
      // registers; the others to the kernel that streams their repacked copy (lane order), and what has no copy to
      // the K-sliced kernel. Every kind is one launch for all its members, each with its own activation rows (and
      // its own k, except in the lane-order kernel: a batch holds members of different k only where each of them fits
      // the two- and three-row kernel or the two-blocks-per-instruction kernel); the K-sliced kernel stages one set
      // of rows per launch.
      struct Group {
        float      *out[kGemvGroupMax];
        const void *w[kGemvGroupMax], *act[kGemvGroupMax];
        int         n[kGemvGroupMax], k[kGemvGroupMax], count = 0;
        void add(float *o, const void *ww, const void *a, int nn, int kk) {
          out[count] = o, w[count] = ww, act[count] = a, n[count] = nn, k[count++] = kk;
        }
      } pairs_g, lane_g, rows_g;
      bool sliced[kGemvGroupMax] = {};
      for (int i = 0; i < b.count; ++i) {
        const void *lw = nullptr;
        bool        member_pairs = false;
        int         r = HTPOPS_OK;
        if (prefers_block_pairs(ctx, b.m, b.k[i], b.n[i], b.wt)) {
          r = lane_order_weights(ctx, b.w[i], b.act[i], b.m, b.k[i], b.n[i], b.wt, &lw, &member_pairs);
        }
        const bool rows = !lw && ctx->opt.gemv_rows_kernel != 0 && gemv_rows_fits(b.m, b.k[i], (WeightType) b.wt);
        if (r == HTPOPS_OK && !lw && !rows) {
          r = lane_order_weights(ctx, b.w[i], b.act[i], b.m, b.k[i], b.n[i], b.wt, &lw, &member_pairs);
        }
        if (r != HTPOPS_OK) {
          b.hdr[i]->state = r;
        } else if (lw) {
          (member_pairs ? pairs_g : lane_g).add(b.out[i], lw, b.act[i], b.n[i], b.k[i]);
        } else if (rows) {
          rows_g.add(b.out[i], b.w[i], b.act[i], b.n[i], b.k[i]);
        } else if (b.m <= kSkinnyGroupMaxM) {
          sliced[i] = true;
        } else {
          // more rows than the K-sliced group launch takes: on its own
          b.hdr[i]->state = op_mat_mul_q8(ctx, b.out[i], b.act[i], b.w[i], b.m, b.k[i], b.n[i], b.wt);
        }
      }
      e = hipSuccess;
      if (pairs_g.count > 0) {
        e = launch_matmul_block_pairs_group(ctx->stream, pairs_g.count, pairs_g.out, pairs_g.act, pairs_g.w, pairs_g.n, b.m,
                                            pairs_g.k);
      }
      if (e == hipSuccess && lane_g.count > 0) {
        e = launch_matmul_lane_order_group(ctx->stream, lane_g.count, lane_g.out, lane_g.act, lane_g.w, lane_g.n, b.m, k0,
                                           (WeightType) b.wt, ctx->opt.lane_order);
      }
      if (e == hipSuccess && rows_g.count > 0) {
        e = launch_gemv_rows_group_q8_0_act(ctx->stream, rows_g.count, rows_g.out, rows_g.act, rows_g.w, rows_g.n, b.m,
                                            rows_g.k, (WeightType) b.wt);
      }
      for (int first = 0; first < b.count && e == hipSuccess && ret == HTPOPS_OK; ++first) {
        if (!sliced[first]) {
          continue;
        }
        float      *out_b[kGemvGroupMax];
        const void *w_b[kGemvGroupMax];
        int         n_b[kGemvGroupMax], count_b = 0;
        for (int i = first; i < b.count; ++i) {  // everybody left that reads the rows of `first`
          if (sliced[i] && b.act[i] == b.act[first] && b.k[i] == b.k[first]) {
            out_b[count_b] = b.out[i], w_b[count_b] = b.w[i], n_b[count_b++] = b.n[i];
            sliced[i] = false;
          }
        }
        const size_t ws = matmul_skinny_group_workspace_bytes(count_b, n_b, b.m, b.k[first]);
        if (int r = ensure_workspace(ctx, ws)) {
          ret = r;
        } else {
          e = launch_matmul_skinny_group(ctx->stream, count_b, out_b, b.act[first], w_b, n_b, b.m, b.k[first],
                                                 (WeightType) b.wt, ctx->workspace, ctx->tickets, kTicketSlots);
        }
      }
    }
    if (e == hipErrorNotSupported) {
      (void) hipGetLastError();
      for (int i = 0; i < b.count; ++i) {
        b.hdr[i]->state = op_mat_mul_q8(ctx, b.out[i], b.act[i], b.w[i], b.m, b.k[i], b.n[i], b.wt);
      }
    } else if (e != hipSuccess) {
      ret = fail(ctx, HTPOPS_ERR_HIP, "grouped mat_mul launch: %s", hipGetErrorString(e));
    }
  } else {
    ret = op_mat_mul_q8(ctx, b.out[0], b.act[0], b.w[0], b.m, b.k[0], b.n[0], b.wt);
  }
  if (ret != HTPOPS_OK) {
    for (int i = 0; i < b.count; ++i) {
      b.hdr[i]->state = ret;
    }
  }
  b.count = 0;
}

// true: the one-row RMSNorm + Q8_0 (op 13) or Q8_0 quantization (op 14) request now waits in the (empty) batch for the
// matmuls behind it; false: run it now
bool try_defer_norm(htpops_context *ctx, const struct OpComputeRequest *req, struct RequestHeader *hdr, GemvBatch &b) {
  const bool   normalize = req->op == HTP_OPS_RMS_NORM_QUANTIZE_Q8_0;
  const auto  *p  = reinterpret_cast<const RmsNormExParams *>(req->payload);
  const auto  *pq = reinterpret_cast<const RmsNormF32Params *>(req->payload);  // (dst, src, ne0, ne1: the same head)
  const int    ne0 = normalize ? p->ne0 : pq->ne0, ne1 = normalize ? p->ne1 : pq->ne1;
  if (!ctx->has_device || ne1 != 1 || ne0 <= 0 || ne0 % 64 != 0 || ne0 > 4096) {
    return false;
  }
  const size_t src_bytes = (size_t) ne0 * 4, q_bytes = q8_0_bytes(1, (size_t) ne0);
  const float *w = nullptr;
  if (normalize && p->weight.fd >= 0 && !(w = (const float *) resolve(ctx, p->weight, src_bytes))) {
    return false;
  }
  const float *src = (const float *) resolve(ctx, normalize ? p->src : pq->src, src_bytes);
  void        *dst = resolve(ctx, normalize ? p->dst : pq->dst, q_bytes);
  if (!src || !dst || !aligned(dst, 4) || !aligned(src, 16) || (w && !aligned(w, 16)) ||
      ranges_overlap(dst, q_bytes, src, src_bytes) || (w && ranges_overlap(dst, q_bytes, w, src_bytes))) {
    return false;  // the ordinary path reports what is wrong; a row quantized in place keeps its own launch
  }
  b.norm.waiting = true, b.norm.hdr = hdr, b.norm.dst = dst, b.norm.src = src, b.norm.weight = w;
  b.norm.eps = normalize ? p->eps : 0.0f, b.norm.ne0 = ne0, b.norm.normalize = normalize;
  hdr->state = HTPOPS_OK;
  return true;
}

// true: the request is now part of the batch and its state is set; false: run it the ordinary way (after a flush)
bool try_batch(htpops_context *ctx, const struct OpComputeRequest *req, struct RequestHeader *hdr, GemvBatch &b) {
  if (!ctx->has_device ||
      (req->op != HTP_OPS_MAT_MUL_Q4_0_Q8_0 && req->op != HTP_OPS_MAT_MUL_Q8_0_Q8_0)) {
    return false;
  }
  const auto *p = reinterpret_cast<const MatMulParams *>(req->payload);
  if (p->m < 1 || p->k <= 0 || p->n <= 0 || p->k % 64 != 0) {
    return false;
  }
  // one activation row, the few rows of the weight-streaming small-batch kernels, or many rows on small tiles
  const int    wt        = req->op == HTP_OPS_MAT_MUL_Q4_0_Q8_0 ? kQ4_0 : kQ8_0;
  const size_t out_bytes = (size_t) p->m * p->n * 4, act_bytes = q8_0_bytes((size_t) p->m, (size_t) p->k);
  const size_t w_bytes   = weight_bytes((size_t) p->n, (size_t) p->k, wt);
  float       *out       = (float *) resolve(ctx, p->output, out_bytes);
  const void  *w         = resolve(ctx, p->weight, w_bytes);
  const void  *act       = resolve(ctx, p->activation, act_bytes);
  if (!out || !w || !act || !aligned(out, 4) || !aligned(w, 4) || !aligned(act, 4) ||
      ranges_overlap(out, out_bytes, act, act_bytes) || ranges_overlap(out, out_bytes, w, w_bytes)) {
    return false;  // the ordinary path reports what is wrong, or handles the aliasing in order
  }
  const bool many_rows = p->m > kBatchMaxM;
  bool       fp6       = false;
  if (many_rows) {
    // only matmuls over a converted copy kept with the weight buffer that take the FP6-tile kernel (members of a launch
    // read the same activation rows) or the fragment kernel in its small-tile configuration; everything else runs on
    // its own
    const MatMulPlan plan = plan_mat_mul(ctx, w, aligned(act, 4), p->m, p->k, p->n, wt);
    if (!(plan.cached || plan.cacheable)) {
      return false;
    }
    fp6 = plan.kind == kPlanLdsFp6;
    if (!fp6 && !(plan.kind == kPlanFragments && gemm_i8_fragments_groupable(p->m, p->n, ctx->opt.gemm_tile_units))) {
      return false;
    }
  }
  // behind a waiting RMSNorm + Q8_0 request: only one-row matmuls over the row it makes, whose outputs leave its
  // operands alone, can run in its launch
  const bool reads_norm = b.norm.waiting && p->m == 1 && act == b.norm.dst && p->k == b.norm.ne0 &&
                          !ranges_overlap(out, out_bytes, b.norm.src, (size_t) p->k * 4) &&
                          !(b.norm.weight && ranges_overlap(out, out_bytes, b.norm.weight, (size_t) p->k * 4)) &&
                          !ranges_overlap(w, w_bytes, b.norm.dst, act_bytes);
  if (b.norm.waiting && b.count == 0) {
    if (reads_norm) {
      b.fused = true;
    } else {
      flush_batch(ctx, b);  // runs the waiting request by itself
    }
  }
  bool join = b.count > 0 && b.count < kGemvGroupMax && b.wt == wt && b.m == p->m && (!b.fused || reads_norm) &&
              b.fp6 == fp6 && (!fp6 || (b.act[0] == act && b.k[0] == p->k)) &&
              (p->m == 1 || many_rows || b.k[0] == p->k ||
               (ctx->opt.gemv_rows_kernel != 0 && gemv_rows_fits(p->m, p->k, (WeightType) wt) &&
                gemv_rows_fits(b.m, b.k[0], (WeightType) wt)) ||
               (ctx->opt.lane_order == 1 && b.pairs_fit && matmul_block_pairs_fits(p->n, p->m, p->k, (WeightType) wt)));
  for (int i = 0; join && i < b.count; ++i) {
    const size_t wi = weight_bytes((size_t) b.n[i], (size_t) b.k[i], b.wt), oi = (size_t) b.m * b.n[i] * 4;
    const size_t ai = q8_0_bytes((size_t) b.m, (size_t) b.k[i]);
    join = !ranges_overlap(out, out_bytes, b.out[i], oi) &&   // two writers of the same bytes must stay ordered
           !ranges_overlap(out, out_bytes, b.w[i], wi) &&     // must not clobber what a member still reads
           !ranges_overlap(out, out_bytes, b.act[i], ai) &&
           !ranges_overlap(b.out[i], oi, w, w_bytes) &&       // must not read what a member is about to write
           !ranges_overlap(b.out[i], oi, act, act_bytes);
  }
  if (!join) {
    if (b.count > 0) {
      flush_batch(ctx, b);
    }
    b.wt = wt, b.m = p->m, b.fp6 = fp6, b.pairs_fit = true;
  }
  b.pairs_fit = b.pairs_fit && matmul_block_pairs_fits(p->n, p->m, p->k, (WeightType) wt);
  b.hdr[b.count] = hdr, b.out[b.count] = out, b.w[b.count] = w, b.act[b.count] = act, b.n[b.count] = p->n, b.k[b.count] = p->k;
  ++b.count;
  hdr->state = HTPOPS_OK;
  return true;
}

// `next` behind a one-token fp32 attention request `req`: if it is the Q8_0 quantization of exactly that attention's
// output row into a buffer that overlaps none of the attention's operands, notes where it wants the row
// (ctx->attn_q8_out) and returns it; nullptr otherwise.
struct RequestHeader *attention_output_quantizer(htpops_context *ctx, const struct OpComputeRequest *req,
                                                 struct RequestHeader *next, size_t next_size) {
  const auto *p = reinterpret_cast<const FlashAttnParams *>(req->payload);
  if (!ctx->has_device || next->type != REQUEST_TYPE_OP_COMPUTE ||
      next_size < sizeof(struct RequestHeader) + sizeof(struct OpComputeRequest) + sizeof(RmsNormF32Params)) {
    return nullptr;
  }
  const auto *nreq = reinterpret_cast<const struct OpComputeRequest *>(next->data);
  const auto *pq   = reinterpret_cast<const RmsNormF32Params *>(nreq->payload);
  if (nreq->op != HTP_OPS_QUANTIZE_Q8_0 || p->qo_len != 1 || p->kv_len <= 0 || p->n_heads <= 0 || p->n_kv_heads <= 0 ||
      p->head_dim <= 0 || p->n_heads > (1 << 20) || p->head_dim > 256 || pq->ne1 != 1 ||
      pq->ne0 != p->n_heads * p->head_dim || !flash_attn_writes_q8_0(1, p->head_dim, true)) {
    return nullptr;
  }
  const size_t row = (size_t) pq->ne0 * 4, q_bytes = q8_0_bytes(1, (size_t) pq->ne0);
  const size_t kv  = (size_t) p->kv_len * p->n_kv_heads * p->head_dim * 2;
  const void  *o = resolve(ctx, p->o, row), *src = resolve(ctx, pq->src, row);
  void        *dst = resolve(ctx, pq->dst, q_bytes);
  const void  *q = resolve(ctx, p->q, row), *k = resolve(ctx, p->k, kv), *v = resolve(ctx, p->v, kv);
  if (!o || o != src || !dst || !q || !k || !v || !aligned(dst, 4) || ranges_overlap(dst, q_bytes, o, row) ||
      ranges_overlap(dst, q_bytes, q, row) || ranges_overlap(dst, q_bytes, k, kv) || ranges_overlap(dst, q_bytes, v, kv)) {
    return nullptr;
  }
  if (p->mask.fd >= 0 && lookup(ctx, p->mask.fd)) {
    const size_t mask_bytes = ((size_t) p->kv_len + 63) / 64 * 64 * 2;
    const void  *mask       = resolve(ctx, p->mask, mask_bytes);
    if (mask && ranges_overlap(dst, q_bytes, mask, mask_bytes)) {
      return nullptr;
    }
  }
  ctx->attn_q8_out = dst;
  return next;
}

}  // namespace

// How many bytes of parameters the op of a compute request reads behind its OpComputeRequest; 0 for an op the
// dispatcher does not know (it reports that itself). The reference casts without looking (op_executor.cc:52-204): a
// request shorter than its op's parameters would make the dispatcher read past it, past the end of the message for
// the last one.
static size_t op_payload_bytes(uint32_t op) {
  switch (op) {
    case HTP_OPS_RMS_NORM_F32:
    case HTP_OPS_QUANTIZE_Q8_0:
      return sizeof(RmsNormF32Params);
    case HTP_OPS_RMS_NORM_F32_EX:
    case HTP_OPS_RMS_NORM_QUANTIZE_Q8_0:
      return sizeof(RmsNormExParams);
    case HTP_OPS_MAT_MUL_PERMUTED_W16A32:
    case HTP_OPS_MAT_MUL_PERMUTED_W4D16A32:
    case HTP_OPS_MAT_MUL_PERMUTED_W8D16A32:
    case HTP_OPS_MAT_MUL_PERMUTED_W4D16A32_IQ4_NL:
    case HTP_OPS_MAT_MUL_Q4_0_Q8_0:
    case HTP_OPS_MAT_MUL_Q8_0_Q8_0:
    case HTP_OPS_MAT_MUL_Q4_0_A32:
    case HTP_OPS_MAT_MUL_Q8_0_A32:
      return sizeof(MatMulParams);
    case HTP_OPS_FLASH_ATTN_QO_F32_KV_F16:
      return sizeof(FlashAttnParams);
    case HTP_OPS_FLASH_ATTN_F16:
      return sizeof(FlashAttnExParams);
    default:
      return 0;
  }
}

int check_message_framing(htpops_context *ctx, const struct MessageHeader *msg, size_t msg_bytes) {
  if (msg_bytes && msg_bytes < sizeof(struct MessageHeader)) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "message: %zu bytes do not hold a header", msg_bytes);
  }
  const int n_reqs = msg->n_reqs;
  if (n_reqs < 0 || n_reqs > (1 << 20)) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "message: n_reqs=%d", n_reqs);
  }
  if (msg_bytes) {
    const size_t hdr = sizeof(struct MessageHeader) + ((size_t) n_reqs + 1) * sizeof(int32_t);
    if (hdr > msg_bytes) {
      return fail(ctx, HTPOPS_ERR_REJECTED, "message: header of %zu bytes does not fit %zu", hdr, msg_bytes);
    }
    int32_t prev = (int32_t) hdr;
    for (int i = 0; i <= n_reqs; ++i) {
      const int32_t off = msg->req_offsets[i];
      if (off < prev || (size_t) off > msg_bytes || (i < n_reqs && (size_t) off + sizeof(struct RequestHeader) > msg_bytes)) {
        return fail(ctx, HTPOPS_ERR_REJECTED, "message: request offset %d (entry %d) outside the message", off, i);
      }
      prev = off;
    }
  }
  return HTPOPS_OK;
}

int enqueue_message(htpops_context *ctx, struct MessageHeader *msg, size_t msg_bytes) {
  if (int r = check_message_framing(ctx, msg, msg_bytes)) {
    return r;
  }
  const int n_reqs = msg->n_reqs;
  GemvBatch batch;
  ctx->act_fragments.src   = nullptr;
  ctx->in_message          = true;
  ctx->message_submissions = 0;
  ++ctx->use_serial;
  for (int i = 0; i < n_reqs; ++i) {
    struct RequestHeader *hdr  = message_header_get_request_ptr(msg, i);
    const size_t          size = message_header_get_request_size(msg, i);
    switch (hdr->type) {
      case REQUEST_TYPE_OP_COMPUTE:
        if (size < sizeof(struct RequestHeader) + sizeof(struct OpComputeRequest)) {
          flush_batch(ctx, batch);
          hdr->state = HTPOPS_ERR_REJECTED;
        } else {
          const auto *req = reinterpret_cast<const struct OpComputeRequest *>(hdr->data);
          if (size < sizeof(struct RequestHeader) + sizeof(struct OpComputeRequest) + op_payload_bytes(req->op)) {
            flush_batch(ctx, batch);
            hdr->state = fail(ctx, HTPOPS_ERR_REJECTED, "message: request %d is shorter than the parameters of op %u", i,
                              req->op);
            break;
          }
          const bool  matmul_payload =
            size >= sizeof(struct RequestHeader) + sizeof(struct OpComputeRequest) + sizeof(MatMulParams);
          const bool  norm_payload =
            (req->op == HTP_OPS_RMS_NORM_QUANTIZE_Q8_0 &&
             size >= sizeof(struct RequestHeader) + sizeof(struct OpComputeRequest) + sizeof(RmsNormExParams)) ||
            (req->op == HTP_OPS_QUANTIZE_Q8_0 &&
             size >= sizeof(struct RequestHeader) + sizeof(struct OpComputeRequest) + sizeof(RmsNormF32Params));
          if (norm_payload) {
            flush_batch(ctx, batch);
          }
          if (!(norm_payload && try_defer_norm(ctx, req, hdr, batch)) &&
              !(matmul_payload && try_batch(ctx, req, hdr, batch))) {
            flush_batch(ctx, batch);
            ++ctx->message_submissions;
            // one-token attention whose fp32 output the NEXT request quantizes to Q8_0 (on its way to the o projection):
            // the launch that finishes the attention writes that row too, and the next request is done with it
            struct RequestHeader *next = nullptr;
            if (req->op == HTP_OPS_FLASH_ATTN_QO_F32_KV_F16 && i + 1 < n_reqs &&
                size >= sizeof(struct RequestHeader) + sizeof(struct OpComputeRequest) + sizeof(FlashAttnParams)) {
              next = attention_output_quantizer(ctx, req, message_header_get_request_ptr(msg, i + 1),
                                                message_header_get_request_size(msg, i + 1));
            }
            ctx->attn_q8_done = false;
            hdr->state        = htpops_execute_op(ctx, req);
            ctx->attn_q8_out  = nullptr;
            if (next && ctx->attn_q8_done && hdr->state == HTPOPS_OK) {
              next->state = HTPOPS_OK;
              ++i;  // (the row is written: that request needs no launch)
            }
          }
        }
        break;
      case REQUEST_TYPE_RPCMEM_MAP:
        {
          flush_batch(ctx, batch);
          // reference: commu.c:102-110 -- only the puts are acted on
          const auto *map = reinterpret_cast<const struct RpcmemMapRequest *>(hdr->data);
          int         ret = 0;
          if (size < sizeof(struct RequestHeader) + sizeof(struct RpcmemMapRequest) || map->n_puts < 0 ||
              size < sizeof(struct RequestHeader) + sizeof(struct RpcmemMapRequest) + (size_t) map->n_puts * 4) {
            ret = HTPOPS_ERR_REJECTED;
          } else {
            for (int j = 0; j < map->n_puts; ++j) {
              htpops_buffer_release(ctx, map->fds[j]);
            }
          }
          hdr->state = ret;
        }
        break;
      default:
        break;  // NO_OP and unknown types are skipped, state untouched (commu.c:111-113)
    }
  }
  flush_batch(ctx, batch);
  ctx->in_message        = false;
  ctx->act_fragments.src = nullptr;
  return HTPOPS_OK;
}


}  // namespace host
}  // namespace htpops

using namespace htpops;
using namespace htpops::host;

extern "C" int htpops_enqueue_message(htpops_context *ctx, struct MessageHeader *msg, size_t msg_bytes) {
  if (!ctx || !msg) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  return enqueue_message(ctx, msg, msg_bytes);
}

extern "C" int htpops_finish_message(htpops_context *ctx, struct MessageHeader *msg) {
  if (!ctx || !msg) {
    return HTPOPS_ERR_REJECTED;
  }
  const uint8_t v0  = msg->state.v[0];
  int           ret = htpops_synchronize(ctx);
  if (ret != HTPOPS_OK) {
    for (int i = 0; i < msg->n_reqs; ++i) {
      struct RequestHeader *hdr = message_header_get_request_ptr(msg, i);
      if (hdr->type == REQUEST_TYPE_OP_COMPUTE && hdr->state == 0) {
        hdr->state = ret;
      }
    }
  }
  // publish completion: state.d = v0 | 1 << 8 with release ordering (reference: commu.c:125-126)
  store_state(msg, (uint64_t) v0 | ((uint64_t) 1 << 8));
  return HTPOPS_OK;
}

extern "C" int htpops_process_message(htpops_context *ctx, struct MessageHeader *msg, size_t msg_bytes) {
  if (!ctx || !msg) {
    return HTPOPS_ERR_REJECTED;
  }
  int ret = htpops_enqueue_message(ctx, msg, msg_bytes);
  if (ret != HTPOPS_OK) {
    return ret;
  }
  return htpops_finish_message(ctx, msg);
}

extern "C" int htpops_last_message_submissions(htpops_context *ctx) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  return ctx->message_submissions;
}
