// Session of the MI355X op backend: context creation and teardown, its switches, error text, synchronisation.
//
// Replaces open_dsp_session + htp_ops_init_backend / htp_ops_close of the reference (src/host/session.c:14-96,
// src/dsp/commu.c:226-249): there is no FastRPC session, VTCM or HMX to set up, a context is a HIP stream plus the
// tables in context.h.
#include "context.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace {

// Device memory of the entry point that allocates nothing (htpops_flash_attn_noalloc_ptr): the split-KV partials of
// decode attention. Every GPU the library runs on holds its own copy of this array from the moment the code object is
// loaded until the process ends. The name is only a host-side stand-in for the symbol: host code uses the address
// that hipGetSymbolAddress returned for the context's device (htpops_context::scratch_ptr), never the name.
static __device__ __align__(256) unsigned char scratch[htpops::host::kNoAllocScratchBytes];

// Which context's work may be using a device's copy of the array: all contexts on a GPU share it, and two streams
// writing partials into it at once would race. A context claims the array with its first call of the entry point and
// gives it back when it has waited for its stream (htpops_synchronize, htpops_finish_message, htpops_close).
constexpr int kMaxDevices = 64;
std::atomic<htpops_context *> scratch_owner[kMaxDevices];

struct OptionName {
  const char *name;
  int htpops::host::Options::*field;
};
const OptionName kOptions[] = {
  { "lane_order", &htpops::host::Options::lane_order },
  { "gemm_fp6", &htpops::host::Options::gemm_fp6 },
  { "gemv_rows_kernel", &htpops::host::Options::gemv_rows_kernel },
  { "gemm_tile_units", &htpops::host::Options::gemm_tile_units },
  { "attn_key_groups", &htpops::host::Options::attn_key_groups },
  { "attn_mask_threshold", &htpops::host::Options::attn_mask_threshold },
  { "converted_cap_mib", &htpops::host::Options::converted_cap_mib },
  { "log", &htpops::host::Options::log },
};

// HTPOPS_<NAME>: the switch's value when the context is created
void options_from_environment(htpops::host::Options &opt) {
  for (const OptionName &o : kOptions) {
    char env[64] = "HTPOPS_";
    size_t      len = strlen(env);
    for (const char *c = o.name; *c && len + 1 < sizeof(env); ++c) {
      env[len++] = (*c >= 'a' && *c <= 'z') ? (char) (*c - 'a' + 'A') : *c;
    }
    env[len] = 0;
    if (const char *v = getenv(env); v && *v) {
      opt.*(o.field) = atoi(v);
    }
  }
}

}  // namespace

namespace htpops {
namespace host {

int fail(htpops_context *ctx, int code, const char *fmt, ...) {
  char    buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  if (ctx) {
    Lock lock(ctx->mu);  // (recursive: most callers hold it already)
    ctx->last_error = buf;
    if (ctx->opt.log) {
      fprintf(stderr, "[htpops] error %d: %s\n", code, buf);
    }
  }
  return code;
}

int hip_fail(htpops_context *ctx, hipError_t e, const char *what) {
  (void) hipGetLastError();  // the runtime keeps the error for the next caller that asks: it is reported here, once
  return fail(ctx, HTPOPS_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

int need_device(htpops_context *ctx) {
  if (!ctx->has_device) {
    return fail(ctx, HTPOPS_ERR_NO_DEVICE, "context was created without a GPU; compute ops are unavailable");
  }
  return HTPOPS_OK;
}

bool claim_static_scratch(htpops_context *ctx) {
  if (ctx->device < 0 || ctx->device >= kMaxDevices) {
    return false;
  }
  htpops_context *expected = nullptr;
  return scratch_owner[ctx->device].compare_exchange_strong(expected, ctx) || expected == ctx;
}

void release_static_scratch(htpops_context *ctx) {
  if (ctx->device >= 0 && ctx->device < kMaxDevices) {
    htpops_context *expected = ctx;
    scratch_owner[ctx->device].compare_exchange_strong(expected, nullptr);
  }
}

bool mul3(size_t a, size_t b, size_t c, size_t *out) {
  if (a == 0 || b == 0 || c == 0) {
    *out = 0;
    return true;
  }
  if (a > SIZE_MAX / b) {
    return false;
  }
  size_t ab = a * b;
  if (ab > SIZE_MAX / c) {
    return false;
  }
  *out = ab * c;
  return true;
}

}  // namespace host
}  // namespace htpops

using namespace htpops::host;

extern "C" int htpops_init_backend(htpops_context **out_ctx, int device) {
  if (!out_ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  *out_ctx            = nullptr;
  htpops_context *ctx = new (std::nothrow) htpops_context();
  if (!ctx) {
    return HTPOPS_ERR_NOMEM;
  }
  options_from_environment(ctx->opt);
  ctx->buffers.emplace_back();  // handle 0 is never valid
  if (device != HTPOPS_DEVICE_NONE) {
    int        count = 0;
    hipError_t e     = hipGetDeviceCount(&count);
    if (e != hipSuccess || device < 0 || device >= count) {
      if (ctx->opt.log) {
        fprintf(stderr, "[htpops] init_backend: device %d unavailable (%s, %d devices)\n", device,
                hipGetErrorString(e), count);
      }
      delete ctx;
      return HTPOPS_ERR_NO_DEVICE;
    }
    if (hipSetDevice(device) != hipSuccess || hipStreamCreate(&ctx->stream) != hipSuccess ||
        hipEventCreate(&ctx->ev_start) != hipSuccess || hipEventCreate(&ctx->ev_stop) != hipSuccess ||
        hipMalloc(reinterpret_cast<void **>(&ctx->tickets), kTicketSlots * sizeof(unsigned)) != hipSuccess ||
        hipMemset(ctx->tickets, 0, kTicketSlots * sizeof(unsigned)) != hipSuccess) {
      delete ctx;
      return HTPOPS_ERR_HIP;
    }
    // each GPU holds its own copy of the scratch array at its own address: ask for this device's, once, here
    if (hipGetSymbolAddress(&ctx->scratch_ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ctx->scratch_ptr) {
      (void) hipGetLastError();
      (void) hipFree(ctx->tickets);
      (void) hipEventDestroy(ctx->ev_start);
      (void) hipEventDestroy(ctx->ev_stop);
      (void) hipStreamDestroy(ctx->stream);
      delete ctx;
      return HTPOPS_ERR_HIP;
    }
    ctx->device     = device;
    ctx->has_device = true;
  }
  *out_ctx = ctx;
  return HTPOPS_OK;
}

extern "C" int htpops_close(htpops_context *ctx) {
  if (!ctx) {
    return HTPOPS_OK;
  }
  htpops_destroy_channel(ctx);
  if (ctx->has_device) {
    (void) hipSetDevice(ctx->device);
    (void) hipStreamSynchronize(ctx->stream);
    release_static_scratch(ctx);
  }
  for (htpops_recorded_message *rec : ctx->recordings) {  // recordings the caller did not release
    if (rec->exec) {
      (void) hipGraphExecDestroy(rec->exec);
      (void) hipGraphDestroy(rec->graph);
    }
    delete rec;
  }
  ctx->recordings.clear();
  for (size_t h = 1; h < ctx->buffers.size(); ++h) {
    Buffer &b = ctx->buffers[h];
    if (b.live && b.owned) {
      if (ctx->has_device) {
        (void) hipFree(b.ptr);
      } else {
        free(b.ptr);
      }
    }
  }
  if (ctx->has_device) {
    if (ctx->tickets) {
      (void) hipFree(ctx->tickets);
    }
    for (const auto &e : ctx->frag_cache) {
      (void) hipFree(e.frag);
    }
    ctx->frag_cache.clear();
    if (ctx->workspace) {
      (void) hipFree(ctx->workspace);
    }
    (void) hipEventDestroy(ctx->ev_start);
    (void) hipEventDestroy(ctx->ev_stop);
    (void) hipStreamDestroy(ctx->stream);
  }
  delete ctx;
  return HTPOPS_OK;
}

extern "C" const char *htpops_last_error(const htpops_context *ctx) {
  if (!ctx) {
    return "null context";
  }
  // The text is copied under the lock into a buffer of the calling thread, so that a failure recorded by another
  // thread (the channel's consumer) cannot reallocate it under the reader.
  static thread_local std::string copy;
  htpops_context *c = const_cast<htpops_context *>(ctx);
  Lock            lock(c->mu);
  copy = c->last_error;
  return copy.c_str();
}

extern "C" int htpops_set_option(htpops_context *ctx, const char *name, int value) {
  if (!ctx || !name) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  for (const OptionName &o : kOptions) {
    if (strcmp(o.name, name) == 0) {
      ctx->opt.*(o.field) = value;
      return HTPOPS_OK;
    }
  }
  return fail(ctx, HTPOPS_ERR_REJECTED, "set_option: unknown option '%s'", name);
}

extern "C" int htpops_get_option(htpops_context *ctx, const char *name, int *value) {
  if (!ctx || !name || !value) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  for (const OptionName &o : kOptions) {
    if (strcmp(o.name, name) == 0) {
      *value = ctx->opt.*(o.field);
      return HTPOPS_OK;
    }
  }
  return fail(ctx, HTPOPS_ERR_REJECTED, "get_option: unknown option '%s'", name);
}

extern "C" int htpops_synchronize(htpops_context *ctx) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  if (!ctx->has_device) {
    return HTPOPS_OK;
  }
  HTPOPS_HIP(ctx, hipStreamSynchronize(ctx->stream));
  release_static_scratch(ctx);  // (nothing of this context is in flight: another context may take the static scratch)
  return HTPOPS_OK;
}

extern "C" void *htpops_get_stream(htpops_context *ctx) {
  return ctx ? (void *) ctx->stream : nullptr;
}
