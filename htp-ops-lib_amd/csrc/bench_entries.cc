// Timers and calibration kernels for the bench harness (include/htpops_bench.h); nothing here is on an op's path and
// nothing has a counterpart in the reference.
#include "context.h"
#include "htpops_bench.h"

#include <chrono>
#include <cstdio>

using namespace htpops;
using namespace htpops::host;

// ------------------------------------------------------------------------------------------------ measurement

extern "C" int htpops_timer_start(htpops_context *ctx) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  HTPOPS_HIP(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
  return HTPOPS_OK;
}

extern "C" int htpops_timer_stop(htpops_context *ctx) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  HTPOPS_HIP(ctx, hipEventRecord(ctx->ev_stop, ctx->stream));
  return HTPOPS_OK;
}

extern "C" int htpops_timer_elapsed_ms(htpops_context *ctx, float *ms) {
  if (!ctx || !ms) {
    return HTPOPS_ERR_REJECTED;
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  HTPOPS_HIP(ctx, hipEventSynchronize(ctx->ev_stop));
  HTPOPS_HIP(ctx, hipEventElapsedTime(ms, ctx->ev_start, ctx->ev_stop));
  return HTPOPS_OK;
}

extern "C" int htpops_measure_mfma_peak(htpops_context *ctx, int kind, int iters, double *tera_ops) {
  if (!ctx || !tera_ops || iters <= 0 || kind < 0 || kind > 2) {
    return HTPOPS_ERR_REJECTED;
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  hipDeviceProp_t prop;
  HTPOPS_HIP(ctx, hipGetDeviceProperties(&prop, ctx->device));
  const int n_blocks = prop.multiProcessorCount * 2;  // 4 waves per block -> 2 waves per SIMD
  int      *sink     = nullptr;
  HTPOPS_HIP(ctx, hipMalloc((void **) &sink, sizeof(int)));
  hipError_t e = launch_mfma_loop(ctx->stream, kind, 16, sink, n_blocks);  // warm-up
  float      ms = 0.f;
  if (e == hipSuccess) e = hipEventRecord(ctx->ev_start, ctx->stream);
  if (e == hipSuccess) e = launch_mfma_loop(ctx->stream, kind, iters, sink, n_blocks);
  if (e == hipSuccess) e = hipEventRecord(ctx->ev_stop, ctx->stream);
  if (e == hipSuccess) e = hipEventSynchronize(ctx->ev_stop);
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, ctx->ev_start, ctx->ev_stop);
  (void) hipFree(sink);
  if (e != hipSuccess) {
    return hip_fail(ctx, e, "mfma loop");
  }
  const double ops_per_mfma = kind == 0 ? 2.0 * 32 * 32 * 32 : (kind == 1 ? 2.0 * 16 * 16 * 64 : 2.0 * 32 * 32 * 16);
  const double total        = (double) n_blocks * 4 /*waves*/ * (double) iters * 4 /*chains*/ * ops_per_mfma;
  *tera_ops                 = total / ((double) ms * 1e-3) / 1e12;
  return HTPOPS_OK;
}

extern "C" int htpops_measure_read_us(htpops_context *ctx, size_t bytes, int buffers, int iters, double *us_per_launch) {
  if (!ctx || !us_per_launch || iters <= 0 || buffers <= 0 || buffers > 64 || bytes < 16) {
    return HTPOPS_ERR_REJECTED;
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  std::vector<void *> bufs;
  unsigned           *sink = nullptr;
  hipError_t          e    = hipMalloc(reinterpret_cast<void **>(&sink), 256);
  for (int b = 0; b < buffers && e == hipSuccess; ++b) {
    void *p = nullptr;
    e       = hipMalloc(&p, bytes);
    if (e == hipSuccess) {
      bufs.push_back(p);
      e = hipMemsetAsync(p, 1, bytes, ctx->stream);
    }
  }
  float ms = 0.f;
  for (size_t b = 0; b < bufs.size() && e == hipSuccess; ++b) {
    e = launch_read(ctx->stream, bufs[b], bytes, sink);
  }
  if (e == hipSuccess) e = hipEventRecord(ctx->ev_start, ctx->stream);
  for (int i = 0; i < iters && e == hipSuccess; ++i) {
    for (size_t b = 0; b < bufs.size() && e == hipSuccess; ++b) {
      e = launch_read(ctx->stream, bufs[b], bytes, sink);
    }
  }
  if (e == hipSuccess) e = hipEventRecord(ctx->ev_stop, ctx->stream);
  if (e == hipSuccess) e = hipEventSynchronize(ctx->ev_stop);
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, ctx->ev_start, ctx->ev_stop);
  (void) hipStreamSynchronize(ctx->stream);
  for (void *p : bufs) {
    (void) hipFree(p);
  }
  (void) hipFree(sink);
  if (e != hipSuccess) {
    return hip_fail(ctx, e, "read loop");
  }
  *us_per_launch = (double) ms * 1e3 / ((double) iters * buffers);
  return HTPOPS_OK;
}

extern "C" int htpops_measure_copy_bandwidth(htpops_context *ctx, size_t bytes, int iters, double *gbps) {
  if (!ctx || !gbps || iters <= 0 || bytes < 16) {
    return HTPOPS_ERR_REJECTED;
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  void *a = nullptr, *b = nullptr;
  HTPOPS_HIP(ctx, hipMalloc(&a, bytes));
  hipError_t e = hipMalloc(&b, bytes);
  if (e != hipSuccess) {
    (void) hipFree(a);
    return hip_fail(ctx, e, "hipMalloc");
  }
  float ms = 0.f;
  e        = hipMemsetAsync(a, 1, bytes, ctx->stream);
  if (e == hipSuccess) e = launch_copy(ctx->stream, b, a, bytes);
  if (e == hipSuccess) e = hipEventRecord(ctx->ev_start, ctx->stream);
  for (int i = 0; i < iters && e == hipSuccess; ++i) {
    e = launch_copy(ctx->stream, b, a, bytes);
  }
  if (e == hipSuccess) e = hipEventRecord(ctx->ev_stop, ctx->stream);
  if (e == hipSuccess) e = hipEventSynchronize(ctx->ev_stop);
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, ctx->ev_start, ctx->ev_stop);
  (void) hipFree(a);
  (void) hipFree(b);
  if (e != hipSuccess) {
    return hip_fail(ctx, e, "copy loop");
  }
  *gbps = 2.0 * (double) (bytes / 16 * 16) * iters / ((double) ms * 1e-3) / 1e9;
  return HTPOPS_OK;
}

extern "C" int htpops_last_gemv_launch(htpops_context *ctx, char *text, size_t cap) {
  if (!ctx || !text || cap == 0) {
    return HTPOPS_ERR_REJECTED;
  }
  const LaunchRecord &r = last_gemv_launch();
  snprintf(text, cap, "%s<%d,%d,%d> grid=%u block=%u lds=%u", r.kernel, r.t0, r.t1, r.t2, r.grid, r.block, r.lds);
  return HTPOPS_OK;
}

extern "C" int htpops_measure_host_walk_us(htpops_context *ctx, struct MessageHeader *msg, size_t msg_bytes, int iters,
                                           double *us_per_message) {
  if (!ctx || !msg || !us_per_message || iters <= 0) {
    return HTPOPS_ERR_REJECTED;
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  // keep the stream busy first: with a backlog in the queue, an enqueue returns as soon as the host side of it is done
  for (int i = 0; i < 64; ++i) {
    if (int r = htpops_enqueue_message(ctx, msg, msg_bytes)) {
      return r;
    }
  }
  const auto t0 = std::chrono::steady_clock::now();
  for (int i = 0; i < iters; ++i) {
    if (int r = htpops_enqueue_message(ctx, msg, msg_bytes)) {
      return r;
    }
  }
  const auto t1 = std::chrono::steady_clock::now();
  *us_per_message = std::chrono::duration<double, std::micro>(t1 - t0).count() / iters;
  return htpops_synchronize(ctx);
}

extern "C" int htpops_measure_decode_attention_parts(htpops_context *ctx, void *o, const void *q, const void *const *ks,
                                                     const void *const *vs, int sets, int kv_len, int n_heads,
                                                     int n_kv_heads, int head_dim, int qo_is_f32, int iters,
                                                     double *split_us, double *merge_us) {
  if (!ctx || !o || !q || !ks || !vs || sets <= 0 || iters <= 0 || !split_us || !merge_us || n_kv_heads <= 0 ||
      n_heads % n_kv_heads != 0 || kv_len <= 0) {
    return HTPOPS_ERR_REJECTED;
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  Lock lock(ctx->mu);
  if (int r = ensure_workspace(ctx, flash_attn_workspace_bytes(1, kv_len, n_heads, head_dim))) {
    return r;
  }
  double *out[2] = { split_us, merge_us };
  for (int part = 1; part <= 2; ++part) {
    for (int i = -8; i < iters; ++i) {  // (eight launches to warm up; the K/V sets take turns so that reads come from HBM)
      if (i == 0) {
        HTPOPS_HIP(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
      }
      const int        s = ((i % sets) + sets) % sets;
      const hipError_t e = launch_flash_attn_decode_part(ctx->stream, part, o, q, ks[s], vs[s], kv_len, n_heads, n_kv_heads,
                                                         head_dim, qo_is_f32 != 0, ctx->workspace);
      if (e != hipSuccess) {
        return hip_fail(ctx, e, "decode attention part");
      }
    }
    HTPOPS_HIP(ctx, hipEventRecord(ctx->ev_stop, ctx->stream));
    HTPOPS_HIP(ctx, hipEventSynchronize(ctx->ev_stop));
    float ms = 0.0f;
    HTPOPS_HIP(ctx, hipEventElapsedTime(&ms, ctx->ev_start, ctx->ev_stop));
    *out[part - 1] = (double) ms * 1e3 / iters;
  }
  return HTPOPS_OK;
}
