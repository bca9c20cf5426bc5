// A message recorded once and replayed many times: the kernel launches of a whole message captured into one HIP graph
// (the reference walks the message anew for every token, src/dsp/commu.c:91-114).
#include "context.h"

using namespace htpops;
using namespace htpops::host;

// ------------------------------------------------------------------------------------------------ recorded messages

extern "C" int htpops_record_message(htpops_context *ctx, struct MessageHeader *msg, size_t msg_bytes,
                                     htpops_recorded_message **out) {
  if (!ctx || !msg || !out) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  *out = nullptr;
  if (int r = need_device(ctx)) {
    return r;
  }
  if (ctx->chan_msg) {
    return fail(ctx, HTPOPS_ERR_BUSY, "record_message: the channel's consumer thread owns the stream");
  }
  if (int r = check_message_framing(ctx, msg, msg_bytes)) {
    return r;
  }
  for (int i = 0; i < msg->n_reqs; ++i) {
    // releasing handles is not something a replay could repeat
    if (message_header_get_request_ptr(msg, i)->type == REQUEST_TYPE_RPCMEM_MAP) {
      return fail(ctx, HTPOPS_ERR_REJECTED, "record_message: request %d releases buffers; only ops can be recorded", i);
    }
  }
  // First walk, executed: sizes the workspace and makes every converted weight copy, so that the recorded walk
  // allocates nothing.
  if (int r = enqueue_message(ctx, msg, msg_bytes)) {
    return r;
  }
  for (int i = 0; i < msg->n_reqs; ++i) {
    const struct RequestHeader *hdr = message_header_get_request_ptr(msg, i);
    if (hdr->type == REQUEST_TYPE_OP_COMPUTE && hdr->state != HTPOPS_OK) {
      return fail(ctx, HTPOPS_ERR_REJECTED, "record_message: request %d failed with %d", i, (int) hdr->state);
    }
  }
  HTPOPS_HIP(ctx, hipStreamSynchronize(ctx->stream));
  const uint64_t generation = ctx->memory_generation;
  std::vector<std::pair<uintptr_t, size_t>> ranges;
  HTPOPS_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
  ctx->collect_ranges = &ranges;
  const int  walked   = enqueue_message(ctx, msg, 0);
  ctx->collect_ranges = nullptr;
  hipGraph_t graph    = nullptr;
  hipError_t e        = hipStreamEndCapture(ctx->stream, &graph);
  bool       all_ok = walked == HTPOPS_OK;
  for (int i = 0; all_ok && i < msg->n_reqs; ++i) {
    const struct RequestHeader *hdr = message_header_get_request_ptr(msg, i);
    all_ok = hdr->type != REQUEST_TYPE_OP_COMPUTE || hdr->state == HTPOPS_OK;
  }
  if (e != hipSuccess || !all_ok || generation != ctx->memory_generation) {
    (void) hipGetLastError();
    if (graph) {
      (void) hipGraphDestroy(graph);
    }
    return fail(ctx, HTPOPS_ERR_HIP, "record_message: the launches could not be captured (%s)",
                e != hipSuccess ? hipGetErrorString(e) : "a request failed or memory moved during the recorded walk");
  }
  hipGraphExec_t exec = nullptr;  // stays null for a message without launches
  size_t         nodes = 0;
  if (graph && (hipGraphGetNodes(graph, nullptr, &nodes) != hipSuccess || nodes == 0)) {
    (void) hipGetLastError();
    (void) hipGraphDestroy(graph);
    graph = nullptr;
  }
  if (graph) {
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
      (void) hipGraphDestroy(graph);
      return hip_fail(ctx, e, "hipGraphInstantiate");
    }
  }
  auto *rec   = new htpops_recorded_message;
  rec->ctx    = ctx;
  rec->graph  = graph;
  rec->exec   = exec;
  rec->ranges = std::move(ranges);
  ctx->recordings.push_back(rec);
  *out = rec;
  return HTPOPS_OK;
}

extern "C" int htpops_launch_recorded_message(htpops_context *ctx, htpops_recorded_message *rec) {
  if (!ctx || !rec || rec->ctx != ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  if (rec->stale) {
    return fail(ctx, HTPOPS_ERR_REJECTED,
                "launch_recorded_message: buffers were released or rewritten since the message was recorded; record it again");
  }
  ctx->act_fragments.src = nullptr;
  if (rec->exec) {
    HTPOPS_HIP(ctx, hipGraphLaunch(rec->exec, ctx->stream));
  }
  return HTPOPS_OK;
}

extern "C" int htpops_release_recorded_message(htpops_context *ctx, htpops_recorded_message *rec) {
  if (!ctx || !rec || rec->ctx != ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  (void) hipStreamSynchronize(ctx->stream);
  if (rec->exec) {
    (void) hipGraphExecDestroy(rec->exec);
    (void) hipGraphDestroy(rec->graph);
  }
  for (size_t i = 0; i < ctx->recordings.size(); ++i) {
    if (ctx->recordings[i] == rec) {
      ctx->recordings[i] = ctx->recordings.back();
      ctx->recordings.pop_back();
      break;
    }
  }
  delete rec;
  return HTPOPS_OK;
}
