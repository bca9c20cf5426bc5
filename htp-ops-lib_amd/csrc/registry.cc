// Buffer registry of the MI355X op backend: handle -> device memory, the context's workspace, and the converted weight
// copies kept with the buffers they were made from.
//
// Replaces rpcmem_alloc + fastrpc_mmap on the host (reference: src/host/test.c:30-58) and the fd -> address table on the
// device (reference: src/dsp/mmap_mgr.cc:15-43). The reference treats mapped weights as immutable
// (src/dsp/op_executor.cc:124-130); the same assumption, made explicit, is what lets converted copies live here.
#include "context.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>

namespace htpops {
namespace host {

Buffer *lookup(htpops_context *ctx, int handle) {
  if (handle <= 0 || (size_t) handle >= ctx->buffers.size() || !ctx->buffers[handle].live) {
    return nullptr;
  }
  return &ctx->buffers[handle];
}

namespace {

int new_handle(htpops_context *ctx, void *ptr, size_t size, bool owned) {
  int h;
  if (!ctx->free_slots.empty()) {
    h = ctx->free_slots.back();
    ctx->free_slots.pop_back();
  } else {
    if (ctx->buffers.size() >= (size_t) kMaxHandles) {
      return fail(ctx, HTPOPS_ERR_NOMEM, "handle table full");
    }
    if (ctx->buffers.empty()) {
      ctx->buffers.emplace_back();  // slot 0: never a valid handle
    }
    h = (int) ctx->buffers.size();
    ctx->buffers.emplace_back();
  }
  Buffer &b      = ctx->buffers[h];
  b.ptr          = ptr;
  b.size         = size;
  b.owned        = owned;
  b.live         = true;
  b.keeps_copies = owned;
  return h;
}

// frees cache entry i (the caller has made sure that no queued kernel still reads it)
void free_entry(htpops_context *ctx, size_t i) {
  const auto &e = ctx->frag_cache[i];
  (void) hipFree(e.frag);
  ctx->converted_bytes -= e.frag_bytes;
  mark_recordings_stale(ctx, e.src, e.src_bytes);
  ctx->frag_cache[i] = ctx->frag_cache.back();
  ctx->frag_cache.pop_back();
}

}  // namespace

void *resolve(htpops_context *ctx, const struct RpcmemBufAddr &addr, size_t need) {
  Buffer *b = lookup(ctx, addr.fd);
  if (!b || addr.offset < 0) {
    return nullptr;
  }
  const size_t off = (size_t) addr.offset;
  if (off > b->size || need > b->size - off) {
    return nullptr;
  }
  if (ctx->collect_ranges) {
    ctx->collect_ranges->emplace_back(reinterpret_cast<uintptr_t>(b->ptr) + off, need);
  }
  return static_cast<uint8_t *>(b->ptr) + off;
}

void mark_recordings_stale(htpops_context *ctx, const void *ptr, size_t bytes) {
  ++ctx->memory_generation;
  const uintptr_t lo = reinterpret_cast<uintptr_t>(ptr);
  for (htpops_recorded_message *rec : ctx->recordings) {
    if (bytes == 0) {
      rec->stale = true;
    }
    for (size_t i = 0; !rec->stale && i < rec->ranges.size(); ++i) {
      rec->stale = rec->ranges[i].first < lo + bytes && lo < rec->ranges[i].first + rec->ranges[i].second;
    }
  }
}

int ensure_workspace(htpops_context *ctx, size_t bytes, bool keep_act_fragments) {
  if (!keep_act_fragments || bytes > ctx->workspace_bytes) {
    ctx->act_fragments.src = nullptr;
  }
  if (bytes <= ctx->workspace_bytes) {
    return HTPOPS_OK;
  }
  mark_recordings_stale(ctx, nullptr, 0);
  if (ctx->workspace) {
    // kernels already enqueued may still use the old block
    HTPOPS_HIP(ctx, hipStreamSynchronize(ctx->stream));
    HTPOPS_HIP(ctx, hipFree(ctx->workspace));
    ctx->workspace       = nullptr;
    ctx->workspace_bytes = 0;
  }
  size_t rounded = (bytes + ((size_t) 1 << 20) - 1) & ~(((size_t) 1 << 20) - 1);
  HTPOPS_HIP(ctx, hipMalloc(&ctx->workspace, rounded));
  ctx->workspace_bytes = rounded;
  return HTPOPS_OK;
}

void drop_fragments(htpops_context *ctx, const void *ptr, size_t bytes) {
  const uintptr_t lo = reinterpret_cast<uintptr_t>(ptr), hi = lo + bytes;
  if (ctx->act_fragments.src) {
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(ctx->act_fragments.src);
    if (a0 < hi && lo < a0 + ctx->act_fragments.src_bytes) {
      ctx->act_fragments.src = nullptr;
    }
  }
  bool synced = false;
  for (size_t i = 0; i < ctx->frag_cache.size();) {
    const auto     &e  = ctx->frag_cache[i];
    const uintptr_t e0 = reinterpret_cast<uintptr_t>(e.src);
    if (e0 < hi && lo < e0 + e.src_bytes) {
      if (!synced && ctx->has_device) {
        (void) hipStreamSynchronize(ctx->stream);  // a queued kernel may still read the fragments
        synced = true;
      }
      free_entry(ctx, i);
    } else {
      ++i;
    }
  }
}

void note_device_write(htpops_context *ctx, const void *ptr, size_t bytes) {
  if ((!ctx->frag_cache.empty() || ctx->act_fragments.src) && ptr) {
    drop_fragments(ctx, ptr, bytes);
  }
}

bool may_keep_copies(htpops_context *ctx, const void *ptr, size_t bytes) {
  const uintptr_t lo = reinterpret_cast<uintptr_t>(ptr);
  for (const Buffer &b : ctx->buffers) {
    const uintptr_t b0 = reinterpret_cast<uintptr_t>(b.ptr);
    if (b.live && b.ptr && b.keeps_copies && lo >= b0 && lo + bytes <= b0 + b.size) {
      return true;
    }
  }
  return false;
}

const void *find_copy(htpops_context *ctx, const void *weight, int kind, int k, int n) {
  for (auto &e : ctx->frag_cache) {
    if (e.src == weight && e.kind == kind && e.k == k && e.n == n) {
      e.last_use = ctx->use_serial;
      return e.frag;
    }
  }
  return nullptr;
}

int new_copy(htpops_context *ctx, const void *weight, size_t src_bytes, int kind, int k, int n, size_t frag_bytes,
             void **out) {
  *out = nullptr;
  // Under a cap, the least recently used copies go first; copies used by the message being walked (or by the op being
  // run) stay, so a message whose own working set exceeds the cap still runs, over it.
  const size_t cap = ctx->opt.converted_cap_mib > 0 ? (size_t) ctx->opt.converted_cap_mib << 20 : 0;
  bool         synced = false;
  while (cap && ctx->converted_bytes + frag_bytes > cap) {
    size_t victim = ctx->frag_cache.size();
    for (size_t i = 0; i < ctx->frag_cache.size(); ++i) {
      const auto &e = ctx->frag_cache[i];
      if (e.last_use < ctx->use_serial && (victim == ctx->frag_cache.size() || e.last_use < ctx->frag_cache[victim].last_use)) {
        victim = i;
      }
    }
    if (victim == ctx->frag_cache.size()) {
      break;
    }
    if (!synced) {
      HTPOPS_HIP(ctx, hipStreamSynchronize(ctx->stream));  // a queued kernel may still read the copy
      synced = true;
    }
    free_entry(ctx, victim);
  }
  void *fresh = nullptr;
  HTPOPS_HIP(ctx, hipMalloc(&fresh, frag_bytes));
  ctx->frag_cache.push_back({ weight, src_bytes, kind, k, n, fresh, frag_bytes, ctx->use_serial });
  ctx->converted_bytes += frag_bytes;
  *out = fresh;
  return HTPOPS_OK;
}

void forget_copy(htpops_context *ctx, void *frag) {
  for (size_t i = 0; i < ctx->frag_cache.size(); ++i) {
    if (ctx->frag_cache[i].frag == frag) {
      (void) hipFree(frag);
      ctx->converted_bytes -= ctx->frag_cache[i].frag_bytes;
      ctx->frag_cache[i] = ctx->frag_cache.back();
      ctx->frag_cache.pop_back();
      return;
    }
  }
}

}  // namespace host
}  // namespace htpops

using namespace htpops;
using namespace htpops::host;

extern "C" int htpops_buffer_alloc(htpops_context *ctx, size_t bytes) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  if (bytes == 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "buffer_alloc: zero size");
  }
  void *p = nullptr;
  if (ctx->has_device) {
    HTPOPS_HIP(ctx, hipMalloc(&p, bytes));
  } else {
    p = aligned_alloc(256, (bytes + 255) & ~(size_t) 255);
    if (!p) {
      return fail(ctx, HTPOPS_ERR_NOMEM, "buffer_alloc: out of host memory");
    }
  }
  int h = new_handle(ctx, p, bytes, true);
  if (h < 0) {
    if (ctx->has_device) {
      (void) hipFree(p);
    } else {
      free(p);
    }
  }
  return h;
}

extern "C" int htpops_buffer_register(htpops_context *ctx, void *device_ptr, size_t bytes) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  if (!device_ptr || bytes == 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "buffer_register: null pointer or zero size");
  }
  return new_handle(ctx, device_ptr, bytes, false);
}

extern "C" int htpops_buffer_release(htpops_context *ctx, int handle) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock    lock(ctx->mu);
  Buffer *b = lookup(ctx, handle);
  if (!b) {
    return HTPOPS_OK;  // unknown handles are ignored (reference: mmap_mgr.cc:29-37)
  }
  int ret = HTPOPS_OK;
  drop_fragments(ctx, b->ptr, b->size);
  mark_recordings_stale(ctx, b->ptr, b->size);
  if (b->owned) {
    if (ctx->has_device) {
      hipError_t e = hipFree(b->ptr);  // waits for work that may still use the block
      if (e != hipSuccess) {
        ret = hip_fail(ctx, e, "hipFree");
      }
    } else {
      free(b->ptr);
    }
  }
  *b = Buffer();
  ctx->free_slots.push_back(handle);
  return ret;
}

extern "C" void *htpops_buffer_device_ptr(htpops_context *ctx, int handle) {
  if (!ctx) {
    return nullptr;
  }
  Lock    lock(ctx->mu);
  Buffer *b = lookup(ctx, handle);
  return b ? b->ptr : nullptr;
}

extern "C" size_t htpops_buffer_size(htpops_context *ctx, int handle) {
  if (!ctx) {
    return 0;
  }
  Lock    lock(ctx->mu);
  Buffer *b = lookup(ctx, handle);
  return b ? b->size : 0;
}

// For weight buffers that the caller's own kernels have rewritten (owned ones through htpops_buffer_device_ptr,
// registered ones at will): drops the converted copies made from the buffer and marks recordings that use it stale.
extern "C" int htpops_buffer_invalidate(htpops_context *ctx, int handle) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock    lock(ctx->mu);
  Buffer *b = lookup(ctx, handle);
  if (!b) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "buffer_invalidate: unknown handle %d", handle);
  }
  drop_fragments(ctx, b->ptr, b->size);
  return HTPOPS_OK;
}

extern "C" int htpops_buffer_prepare_weights(htpops_context *ctx, int handle, size_t offset, int weight_type, int n,
                                             int k, int m_hint, size_t *converted_bytes) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
  if (converted_bytes) {
    *converted_bytes = 0;
  }
  Buffer *b = lookup(ctx, handle);
  if (!b) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "buffer_prepare_weights: unknown handle %d", handle);
  }
  if ((weight_type != kQ4_0 && weight_type != kQ8_0) || n <= 0 || k <= 0 || k % 32 != 0 || m_hint < 1) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "buffer_prepare_weights: bad arguments (type=%d n=%d k=%d m_hint=%d)",
                weight_type, n, k, m_hint);
  }
  const size_t w_bytes = weight_bytes((size_t) n, (size_t) k, weight_type);
  if (offset > b->size || w_bytes > b->size - offset) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "buffer_prepare_weights: %zu bytes at offset %zu do not fit the buffer", w_bytes,
                offset);
  }
  if (int r = need_device(ctx)) {
    return r;
  }
  // From here on the buffer is under the contract of the context's own buffers: its weights are immutable until the
  // caller says otherwise with htpops_buffer_invalidate (or rewrites them through htpops_buffer_write).
  b->keeps_copies    = true;
  const void  *w      = static_cast<const uint8_t *>(b->ptr) + offset;
  const size_t before = ctx->converted_bytes;
  ++ctx->use_serial;
  if (m_hint >= kManyRowsMinM) {
    MatMulPlan  plan = plan_mat_mul(ctx, w, true, m_hint, k, n, weight_type);
    const void *copy = nullptr;
    if (int r = plan_weight_copy(ctx, plan, w, k, n, weight_type, &copy)) {
      return r;
    }
  } else if (m_hint >= 2 && (prefers_block_pairs(ctx, m_hint, k, n, weight_type) ||
                             !(ctx->opt.gemv_rows_kernel != 0 && gemv_rows_fits(m_hint, k, (WeightType) weight_type)))) {
    // (the two- and three-row kernel reads the weights as they are: nothing to make for it)
    const void *copy  = nullptr;
    bool        pairs = false;
    if (int r = lane_order_weights(ctx, w, nullptr, m_hint, k, n, weight_type, &copy, &pairs)) {
      return r;
    }
  }
  if (converted_bytes) {
    *converted_bytes = ctx->converted_bytes - before;
  }
  return HTPOPS_OK;
}

extern "C" size_t htpops_converted_bytes(htpops_context *ctx) {
  if (!ctx) {
    return 0;
  }
  Lock lock(ctx->mu);
  return ctx->converted_bytes;
}

extern "C" size_t htpops_workspace_bytes(htpops_context *ctx) {
  if (!ctx) {
    return 0;
  }
  Lock lock(ctx->mu);
  return ctx->workspace_bytes;
}

extern "C" int htpops_buffer_write(htpops_context *ctx, int handle, size_t offset, const void *src, size_t bytes) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock    lock(ctx->mu);
  Buffer *b = lookup(ctx, handle);
  if (!b || !src || offset > b->size || bytes > b->size - offset) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "buffer_write: unknown handle or range outside the buffer");
  }
  uint8_t *dst = static_cast<uint8_t *>(b->ptr) + offset;
  if (!ctx->has_device) {
    memcpy(dst, src, bytes);
    return HTPOPS_OK;
  }
  drop_fragments(ctx, dst, bytes);  // converted copies of weights that lived here are stale now
  HTPOPS_HIP(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
  HTPOPS_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return HTPOPS_OK;
}

extern "C" int htpops_buffer_read(htpops_context *ctx, int handle, size_t offset, void *dst, size_t bytes) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock    lock(ctx->mu);
  Buffer *b = lookup(ctx, handle);
  if (!b || !dst || offset > b->size || bytes > b->size - offset) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "buffer_read: unknown handle or range outside the buffer");
  }
  const uint8_t *src = static_cast<const uint8_t *>(b->ptr) + offset;
  if (!ctx->has_device) {
    memcpy(dst, src, bytes);
    return HTPOPS_OK;
  }
  HTPOPS_HIP(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
  HTPOPS_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return HTPOPS_OK;
}
