// The mailbox channel: a consumer thread that polls the shared message buffer exactly as msg_receiver_loop does
// (reference: src/dsp/commu.c:37-136) and the calls that start and stop it (reference: src/dsp/commu.c:151-212).
#include "context.h"

#include <chrono>
#include <cstring>

using namespace htpops;
using namespace htpops::host;

// ------------------------------------------------------------------------------------------------ channel

namespace {

void poll_loop(htpops_context *ctx) {
  if (ctx->has_device) {
    (void) hipSetDevice(ctx->device);
  }
  while (!ctx->poller_stop.load(std::memory_order_acquire)) {
    const uint64_t d  = load_state(ctx->chan_msg);
    const uint8_t  v0 = d & 0xff, v1 = (d >> 8) & 0xff;
    if (v0 == 0 || v1 != 0) {  // reference: commu.c:70-75
      std::this_thread::sleep_for(std::chrono::microseconds(1));
      continue;
    }
    if (htpops_process_message(ctx, ctx->chan_msg, ctx->chan_bytes) != HTPOPS_OK) {
      // malformed message: still complete the handshake so the producer does not spin forever
      store_state(ctx->chan_msg, (uint64_t) v0 | ((uint64_t) 1 << 8));
    }
  }
}

}  // namespace

extern "C" int htpops_create_channel(htpops_context *ctx, void *msg, size_t max_msg_size) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  if (!msg || max_msg_size < sizeof(struct MessageHeader) + sizeof(int32_t)) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "create_channel: null or too small message buffer");
  }
  if (ctx->chan_msg) {
    return fail(ctx, HTPOPS_ERR_BUSY, "create_channel: a channel is already active");
  }
  memset(msg, 0, max_msg_size);  // reference: commu.c:160-161
  ctx->chan_msg   = static_cast<struct MessageHeader *>(msg);
  ctx->chan_bytes = max_msg_size;
  ctx->poller_stop.store(false);
  ctx->poller = std::thread(poll_loop, ctx);
  return HTPOPS_OK;
}

extern "C" int htpops_destroy_channel(htpops_context *ctx) {
  if (!ctx) {
    return HTPOPS_OK;
  }
  // The thread object is taken out under the lock and joined without it: the consumer thread takes the same lock for
  // every message it walks.
  std::thread poller;
  {
    Lock lock(ctx->mu);
    if (!ctx->chan_msg) {
      return HTPOPS_OK;
    }
    ctx->poller_stop.store(true, std::memory_order_release);
    poller = std::move(ctx->poller);
  }
  if (poller.joinable()) {
    poller.join();
  }
  Lock lock(ctx->mu);
  ctx->chan_msg   = nullptr;
  ctx->chan_bytes = 0;
  return HTPOPS_OK;
}
