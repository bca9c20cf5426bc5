// C ABI of the MI355X op backend: context, buffer registry, request decoding, mailbox protocol.
//
// This file is the replacement for the reference's dispatch layer: execute_op_simple (src/dsp/op_executor.cc:52-204),
// the fd -> address table (src/dsp/mmap_mgr.cc:15-43) and the consumer side of the shared-memory mailbox
// (src/dsp/commu.c:37-136, :151-212). FastRPC, VTCM/HMX set-up and cache maintenance have no counterpart: a request
// is validated on the host and its kernels are enqueued on the context's HIP stream.
#include "htpops.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <thread>
#include <utility>
#include <vector>

#include "kernels.h"

namespace {

struct Buffer {
  void  *ptr   = nullptr;
  size_t size  = 0;
  bool   owned = false;  // allocated by the context (freed on release)
  bool   live  = false;
};

constexpr int kMaxHandles  = 1 << 20;
constexpr int kTicketSlots = 1 << 16;

// Device memory of the entry point that allocates nothing (htpops_flash_attn_noalloc_ptr): the split-KV partials of
// decode attention. Every GPU the library runs on holds its own copy of this array from the moment the code object is
// loaded until the process ends. The name is only a host-side stand-in for the symbol: host code uses the address
// that hipGetSymbolAddress returned for the context's device (htpops_context::scratch_ptr), never the name.
constexpr size_t kNoAllocScratchBytes = (size_t) 8 << 20;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

}  // namespace

struct htpops_recorded_message {
  htpops_context *ctx   = nullptr;
  hipGraph_t      graph = nullptr;
  hipGraphExec_t  exec  = nullptr;  // null for a message without launches
  bool            stale = false;
  std::vector<std::pair<uintptr_t, size_t>> ranges;
};

struct htpops_context {
  // Guards the buffer registry, the converted-copy caches, the workspace and the recordings: the channel's consumer
  // thread walks messages (resolving handles, making copies) while the host thread may allocate, write or release
  // buffers, as a host of the reference does while its consumer thread runs (reference: src/dsp/mmap_mgr.cc:15-27 maps
  // lazily on that thread). Recursive: a message's RPCMEM_MAP request releases buffers from inside the walk.
  std::recursive_mutex mu;
  // Set by the message walk around an attention request whose output the next request quantizes to Q8_0: where that
  // request wants its row, and whether the attention launch wrote it.
  void               *attn_q8_out  = nullptr;
  bool                attn_q8_done = false;
  int                 device     = HTPOPS_DEVICE_NONE;
  bool                has_device = false;
  hipStream_t         stream     = nullptr;
  std::vector<Buffer> buffers;  // index = handle; slot 0 unused
  std::vector<int>    free_slots;
  std::string         last_error;

  // scratch owned by the context: quantized activations of the fp32-activation matmul, attention partials
  void  *workspace       = nullptr;
  size_t workspace_bytes = 0;
  // zeroed ticket counters of the K-sliced matmul (each launch leaves them zeroed)
  unsigned *tickets = nullptr;

  // weights of ops 1-4 converted to MFMA fragment order, keyed by the source range; dropped when the source
  // buffer is written through the registry or released
  struct FragEntry {
    const void *src;
    size_t      src_bytes;
    int         kind, k, n;
    void       *frag;
  };
  std::vector<FragEntry> frag_cache;

  // Which activations the int8 fragments at the start of `workspace` were made from. Only kept while one message is
  // walked (requests of a message that multiply the same activations share one conversion); any other use of the
  // workspace and any write into the source range clears it.
  struct ActFragments {
    const void *src       = nullptr;
    size_t      src_bytes = 0;
    int         m = 0, k = 0;
    int         kind = 0;  // which kernel family's layout (PlanKind)
  } act_fragments;
  bool in_message = false;
  // how many separately launched units (grouped launches and single ops) the most recent message walk issued
  int  message_submissions = 0;

  // Recorded messages hold device addresses. Each keeps the buffer ranges its requests resolved to (collected through
  // `collect_ranges` while it is recorded) and is marked stale when one of them is released, when a converted copy of
  // weights in one of them is dropped, or when the workspace is replaced. `memory_generation` counts those events, so
  // that a recording can tell whether one happened during its own recorded walk.
  std::vector<htpops_recorded_message *>     recordings;
  std::vector<std::pair<uintptr_t, size_t>> *collect_ranges = nullptr;
  uint64_t                                   memory_generation = 0;

  hipEvent_t ev_start = nullptr, ev_stop = nullptr;

  // this device's copy of the file-scope `scratch` array (hipGetSymbolAddress at init, with the device current)
  void *scratch_ptr = nullptr;

  // mailbox channel
  std::thread           poller;
  std::atomic<bool>     poller_stop{ false };
  struct MessageHeader *chan_msg   = nullptr;
  size_t                chan_bytes = 0;
};

namespace {

using Lock = std::lock_guard<std::recursive_mutex>;

int fail(htpops_context *ctx, int code, const char *fmt, ...) {
  char    buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  if (ctx) {
    ctx->last_error = buf;
  }
  if (getenv("HTPOPS_LOG")) {
    fprintf(stderr, "[htpops] error %d: %s\n", code, buf);
  }
  return code;
}

int hip_fail(htpops_context *ctx, hipError_t e, const char *what) {
  (void) hipGetLastError();  // the runtime keeps the error for the next caller that asks: it is reported here, once
  return fail(ctx, HTPOPS_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define HTPOPS_HIP(ctx, expr)                    \
  do {                                           \
    hipError_t e_ = (expr);                      \
    if (e_ != hipSuccess) {                      \
      return hip_fail((ctx), e_, #expr);         \
    }                                            \
  } while (0)

Buffer *lookup(htpops_context *ctx, int handle) {
  if (handle <= 0 || (size_t) handle >= ctx->buffers.size() || !ctx->buffers[handle].live) {
    return nullptr;
  }
  return &ctx->buffers[handle];
}

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
  Buffer &b = ctx->buffers[h];
  b.ptr     = ptr;
  b.size    = size;
  b.owned   = owned;
  b.live    = true;
  return h;
}

// Resolves (handle, offset) to an address with `need` readable/writable bytes, or null (the reference's
// "mmap_manager_get_map returned NULL" case, op_executor.cc:57-61, extended with range checks).
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

// memory in [ptr, ptr + bytes) is about to go (bytes = 0: the workspace, which every recording may use)
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

bool aligned(const void *p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

// The 8-byte mailbox state is declared packed (alignment 1) but lives at the start of the message buffer, which
// callers allocate at least 8-byte aligned; an unaligned buffer falls back to byte accesses between fences.
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

// size helpers with overflow checks; return false on overflow or non-positive dims
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

int ensure_workspace(htpops_context *ctx, size_t bytes, bool keep_act_fragments = false) {
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
  bool            synced = false;
  for (size_t i = 0; i < ctx->frag_cache.size();) {
    const auto     &e  = ctx->frag_cache[i];
    const uintptr_t e0 = reinterpret_cast<uintptr_t>(e.src);
    if (e0 < hi && lo < e0 + e.src_bytes) {
      if (!synced && ctx->has_device) {
        (void) hipStreamSynchronize(ctx->stream);  // a queued kernel may still read the fragments
        synced = true;
      }
      (void) hipFree(e.frag);
      mark_recordings_stale(ctx, e.src, e.src_bytes);
      ctx->frag_cache[i] = ctx->frag_cache.back();
      ctx->frag_cache.pop_back();
    } else {
      ++i;
    }
  }
}

// an op is about to write [ptr, ptr + bytes): converted weights made from that range are stale
void note_device_write(htpops_context *ctx, const void *ptr, size_t bytes) {
  if ((!ctx->frag_cache.empty() || ctx->act_fragments.src) && ptr) {
    drop_fragments(ctx, ptr, bytes);
  }
}

size_t permuted_weight_bytes(size_t n, size_t k, int kind) {
  // reference: op_executor.cc:100-102, :124-126
  return kind == 1 ? k * n * 2 : k * n / 256 * (kind == 3 ? 272 : 144);
}

size_t q8_0_bytes(size_t rows, size_t k) {
  return rows * (k / 32) * 34;
}

size_t weight_bytes(size_t n, size_t k, int weight_type) {
  return n * (k / 32) * (weight_type == htpops::kQ4_0 ? 18 : 34);
}

int need_device(htpops_context *ctx) {
  if (!ctx->has_device) {
    return fail(ctx, HTPOPS_ERR_NO_DEVICE, "context was created without a GPU; compute ops are unavailable");
  }
  return HTPOPS_OK;
}

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
  HTPOPS_HIP(ctx, htpops::launch_rms_norm_f32(ctx->stream, dst, src, weight, eps, ne0, ne1));
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
  HTPOPS_HIP(ctx, htpops::launch_quantize_q8_0(ctx->stream, dst, src, k, m));
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
    HTPOPS_HIP(ctx, htpops::launch_rms_norm_quantize_q8_0(ctx->stream, dst, src, weight, eps, ne0, ne1));
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
  HTPOPS_HIP(ctx, htpops::launch_rms_norm_f32(ctx->stream, (float *) ctx->workspace, src, weight, eps, ne0, ne1));
  HTPOPS_HIP(ctx, htpops::launch_quantize_q8_0(ctx->stream, dst, (const float *) ctx->workspace, ne0, ne1));
  return HTPOPS_OK;
}

int check_mat_mul(htpops_context *ctx, const void *dst, const void *act, const void *weight, int m, int k, int n,
                  int weight_type) {
  // reference: mat_mul.c:878-892
  if (!dst || !act || !weight || m <= 0 || k <= 0 || n <= 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul: null buffer or non-positive size (m=%d k=%d n=%d)", m, k, n);
  }
  if (k % 32 != 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul: k=%d is not a multiple of 32", k);
  }
  if (weight_type != htpops::kQ4_0 && weight_type != htpops::kQ8_0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul: unsupported weight type %d", weight_type);
  }
  if (!aligned(dst, 4) || !aligned(act, 2) || !aligned(weight, 2)) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "mat_mul: misaligned buffer");
  }
  return HTPOPS_OK;
}

// true when [ptr, ptr + bytes) lies inside a buffer this context allocated: its contents change only through
// htpops_buffer_write or as the output of an op, both of which drop converted copies
bool in_owned_buffer(htpops_context *ctx, const void *ptr, size_t bytes) {
  const uintptr_t lo = reinterpret_cast<uintptr_t>(ptr);
  for (const Buffer &b : ctx->buffers) {
    const uintptr_t b0 = reinterpret_cast<uintptr_t>(b.ptr);
    if (b.ptr && b.owned && lo >= b0 && lo + bytes <= b0 + b.size) {
      return true;
    }
  }
  return false;
}

constexpr int kSkinnyGroupMaxM = 8;   // rows of the K-sliced kernel's grouped launch
constexpr int kBatchMaxM       = 16;  // rows up to which same-activation requests of a message are grouped
constexpr int kManyRowsMinM    = 33;  // rows from which a matmul takes the matrix-core kernels

bool ranges_overlap(const void *a, size_t a_bytes, const void *b, size_t b_bytes) {
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
  return a0 < b0 + b_bytes && b0 < a0 + a_bytes;
}

constexpr int kFragKindRowLayout = 100;  // + ggml type, to keep apart from the tile-permuted kinds 1..4

constexpr int kFragKindLaneOrder = 300;  // + ggml type: Q4_0 weights in matrix-core operand order (2..16 activation rows)

// The repacked copy of `weight` for the few-row kernel: from the cache, or made now and cached. *out stays nullptr when
// this matmul does not take that kernel (shape, weight type, activations not 16-byte aligned for the DMA into LDS,
// weights in memory the context does not own and so cannot watch for writes); the caller then uses the kernels that
// read the weights as they are. A failed allocation or conversion launch is an error, not a reason to switch kernels.
int lane_order_weights(htpops_context *ctx, const void *weight, const void *act, int m, int k, int n, int wt,
                       const void **out) {
  *out = nullptr;
  if (htpops::env_int("HTPOPS_LANE_ORDER", 1) == 0 || !aligned(act, 16) ||
      !htpops::matmul_lane_order_fits(n, m, k, (htpops::WeightType) wt)) {
    return HTPOPS_OK;
  }
  const int kind = kFragKindLaneOrder + wt;
  for (const auto &e : ctx->frag_cache) {
    if (e.src == weight && e.kind == kind && e.k == k && e.n == n) {
      *out = e.frag;
      return HTPOPS_OK;
    }
  }
  if (!in_owned_buffer(ctx, weight, weight_bytes((size_t) n, (size_t) k, wt))) {
    return HTPOPS_OK;
  }
  void *fresh = nullptr;
  HTPOPS_HIP(ctx, hipMalloc(&fresh, htpops::matmul_lane_order_weight_bytes(k, n, (htpops::WeightType) wt)));
  const hipError_t e = htpops::launch_weights_to_lane_order(ctx->stream, fresh, weight, k, n, (htpops::WeightType) wt);
  if (e != hipSuccess) {
    (void) hipFree(fresh);
    return hip_fail(ctx, e, "weight repack launch");
  }
  ctx->frag_cache.push_back({ weight, weight_bytes((size_t) n, (size_t) k, wt), kind, k, n, fresh });
  *out = fresh;
  return HTPOPS_OK;
}

constexpr int kFragKindFp6Tiles = 400;  // + ggml type: FP6 operand tiles of the many-row Q4_0 matmul (LDS kernel)

// Which kernel family a quantized matmul takes and how much of the context's workspace it needs.
enum PlanKind {
  kPlanFewRows,    // m below the many-row threshold: the weight-streaming kernels
  kPlanLdsFp6,     // many rows, Q4_0, k % 64 == 0, enough output tiles, weights the context may keep a converted copy of
  kPlanFragments,  // every other many-row matmul: int8 fragments (converted weights)
};

struct MatMulPlan {
  PlanKind    kind      = kPlanFewRows;
  const void *cached    = nullptr;
  bool        cacheable = false;
  int         frag_kind = 0;
  size_t      act_bytes = 0, weight_bytes = 0;  // converted operand sizes
  size_t      ws_bytes  = 0;
};

// `act_aligned`: the Q8_0 activations start on a 4-byte boundary (the re-tiling pass of the FP6 kernel reads dwords)
MatMulPlan plan_mat_mul(htpops_context *ctx, const void *weight, bool act_aligned, int m, int k, int n, int wt) {
  MatMulPlan p;
  if (m < kManyRowsMinM || k % 32 != 0) {
    p.ws_bytes = htpops::mat_mul_workspace_bytes(m, k, n);
    return p;
  }
  auto lookup_copy = [&](int frag_kind) {
    p.frag_kind = frag_kind;
    p.cached    = nullptr;
    for (const auto &e : ctx->frag_cache) {
      if (e.src == weight && e.kind == frag_kind && e.k == k && e.n == n) {
        p.cached = e.frag;
        return;
      }
    }
    p.cacheable = in_owned_buffer(ctx, weight, weight_bytes((size_t) n, (size_t) k, wt));
  };
  // Q4_0 weights in a buffer of the context's own, on a shape whose output tiles fill the device: the FP6 kernel over
  // a converted copy kept with the buffer (half the vector-ALU work per block sum of the int8 path). Caller-owned
  // memory may change behind the context's back, so nothing converted from it is kept, and the FP6 conversion is too
  // slow to redo per call.
  const int use_fp6 = htpops::env_int("HTPOPS_GEMM_FP6", -1);  // read per call: tests switch kernels
  if (wt == htpops::kQ4_0 && use_fp6 != 0 && htpops::gemm_fp6_lds_fits(m, k, n) && aligned(weight, 4) && act_aligned &&
      (use_fp6 > 0 || htpops::gemm_fp6_lds_fills_device(m, n))) {
    lookup_copy(kFragKindFp6Tiles + wt);
    if (p.cached || p.cacheable) {
      p.kind         = kPlanLdsFp6;
      p.act_bytes    = (htpops::gemm_fp6_lds_act_tile_bytes(m, k) + 255) & ~(size_t) 255;
      p.weight_bytes = htpops::gemm_fp6_lds_weight_tile_bytes(k, n);
      p.ws_bytes     = p.act_bytes;
      return p;
    }
  }
  p.kind         = kPlanFragments;
  p.act_bytes    = (htpops::gemm_i8_act_fragment_bytes(m, k) + 255) & ~(size_t) 255;
  p.weight_bytes = (htpops::gemm_i8_weight_fragment_bytes(k, n) + 255) & ~(size_t) 255;
  lookup_copy(kFragKindRowLayout + wt);
  p.ws_bytes = p.act_bytes + ((p.cached || p.cacheable) ? 0 : p.weight_bytes) +
               ((htpops::gemm_i8_fragments_exchange_bytes(m, n, k) + 255) & ~(size_t) 255);
  return p;
}

int run_few_rows(htpops_context *ctx, float *dst, const void *act, const void *weight, int m, int k, int n, int wt,
                 uint8_t *ws) {
  // hipErrorNotSupported from a launcher means "this kernel does not take the shape": try the next one. Any other
  // failure is reported.
  if (htpops::gemv_rows_fits(m, k, (htpops::WeightType) wt) && aligned(act, 4) && aligned(weight, 4)) {
    const hipError_t e = htpops::launch_gemv_rows_group_q8_0_act(ctx->stream, 1, &dst, &act, &weight, &n, m, &k,
                                                                 (htpops::WeightType) wt);
    if (e == hipSuccess) {
      return HTPOPS_OK;
    }
    if (e != hipErrorNotSupported) {
      return hip_fail(ctx, e, "few-row mat_mul launch");
    }
    (void) hipGetLastError();
  }
  const void *lw = nullptr;
  if (int r = lane_order_weights(ctx, weight, act, m, k, n, wt, &lw)) {
    return r;
  }
  if (lw) {
    const hipError_t e = htpops::launch_matmul_lane_order_group(ctx->stream, 1, &dst, &act, &lw, &n, m, k,
                                                                (htpops::WeightType) wt);
    if (e == hipSuccess) {
      return HTPOPS_OK;
    }
    if (e != hipErrorNotSupported) {
      return hip_fail(ctx, e, "repacked-weight mat_mul launch");
    }
    (void) hipGetLastError();
  }
  HTPOPS_HIP(ctx, htpops::launch_mat_mul_q8_0_act(ctx->stream, dst, act, weight, m, k, n, (htpops::WeightType) wt, ws,
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
  // the converted copy of the weights, for the kernels that want one
  const void *frags = plan.cached;
  if (!frags) {
    void *fresh = ws + plan.act_bytes;
    if (plan.cacheable) {
      HTPOPS_HIP(ctx, hipMalloc(&fresh, plan.weight_bytes));
    }
    const hipError_t e = plan.kind == kPlanLdsFp6 ?
                             htpops::launch_q4_0_to_fp6_tiles(ctx->stream, fresh, weight, k, n) :
                             htpops::launch_weights_to_i8_fragments(ctx->stream, fresh, weight, k, n, (htpops::WeightType) wt);
    if (e != hipSuccess) {
      if (plan.cacheable) {
        (void) hipFree(fresh);
      }
      return fail(ctx, HTPOPS_ERR_HIP, "weight conversion: %s", hipGetErrorString(e));
    }
    if (plan.cacheable) {
      ctx->frag_cache.push_back({ weight, weight_bytes((size_t) n, (size_t) k, wt), plan.frag_kind, k, n, fresh });
    }
    frags = fresh;
  }
  // The converted activations at the start of the workspace are shared by the requests of a message that read the same
  // rows with the same kernel family (note_device_write above has already cleared the record if this matmul writes
  // into its own activations).
  auto      &af    = ctx->act_fragments;
  const bool ready = af.src == act && af.m == m && af.k == k && af.kind == (int) plan.kind && ws == ctx->workspace;
  const bool keep  = ready || (ctx->in_message && ws == ctx->workspace &&
                               in_owned_buffer(ctx, act, q8_0_bytes((size_t) m, (size_t) k)) &&
                               !ranges_overlap(dst, (size_t) m * n * 4, act, q8_0_bytes((size_t) m, (size_t) k)));
  af.src = nullptr;
  if (plan.kind == kPlanLdsFp6) {
    HTPOPS_HIP(ctx, htpops::launch_gemm_fp6_lds(ctx->stream, dst, act, frags, m, k, n, ws, ready));
  } else {
    // (scratch for partial tiles at the end of this matmul's share of the workspace)
    const size_t xbytes = htpops::gemm_i8_fragments_exchange_bytes(m, n, k);
    HTPOPS_HIP(ctx, htpops::launch_gemm_i8_fragments(ctx->stream, dst, act, frags, m, k, n, ws, ready,
                                                     ws + plan.ws_bytes - ((xbytes + 255) & ~(size_t) 255), xbytes,
                                                     ctx->tickets, kTicketSlots));
  }
  if (keep) {
    af.src = act, af.src_bytes = q8_0_bytes((size_t) m, (size_t) k), af.m = m, af.k = k, af.kind = (int) plan.kind;
  }
  return HTPOPS_OK;
}

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
  HTPOPS_HIP(ctx, htpops::launch_quantize_q8_0(ctx->stream, ws, act, k, m));
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
  const void *frag = nullptr;
  for (const auto &e : ctx->frag_cache) {
    if (e.src == weight && e.kind == kind && e.k == k && e.n == n) {
      frag = e.frag;
      break;
    }
  }
  // Converted copies are kept only for weights in buffers the context allocated (their contents change only through
  // htpops_buffer_write or as an op's output, both of which drop the copy). Caller-registered memory may be rewritten
  // behind the context's back: it is converted into the workspace on every call.
  const size_t act_bytes  = (htpops::permuted_act_fragment_bytes(m, k) + 255) & ~(size_t) 255;
  const size_t frag_bytes = htpops::permuted_weight_fragment_bytes(k, n);
  const bool   cacheable  = !frag && in_owned_buffer(ctx, weight, permuted_weight_bytes((size_t) n, (size_t) k, kind));
  if (int r = ensure_workspace(ctx, act_bytes + ((frag || cacheable) ? 0 : frag_bytes))) {
    return r;
  }
  if (!frag) {
    void *fresh = static_cast<uint8_t *>(ctx->workspace) + act_bytes;
    if (cacheable) {
      HTPOPS_HIP(ctx, hipMalloc(&fresh, frag_bytes));
    }
    const hipError_t e = htpops::launch_permuted_weight_to_fragments(ctx->stream, fresh, weight, k, n, kind);
    if (e != hipSuccess) {
      if (cacheable) {
        (void) hipFree(fresh);
      }
      return fail(ctx, HTPOPS_ERR_HIP, "weight conversion: %s", hipGetErrorString(e));
    }
    if (cacheable) {
      ctx->frag_cache.push_back({ weight, permuted_weight_bytes((size_t) n, (size_t) k, kind), kind, k, n, fresh });
    }
    frag = fresh;
  }
  HTPOPS_HIP(ctx, htpops::launch_mat_mul_fragments(ctx->stream, dst, act, frag, m, k, n, ctx->workspace));
  return HTPOPS_OK;
}

int op_flash_attn(htpops_context *ctx, void *o, const void *q, const void *k, const void *v, const void *mask,
                  int qo_len, int kv_len, int n_heads, int n_kv_heads, int head_dim, int qo_is_f32, int causal,
                  bool no_alloc = false) {
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
  const size_t ws_bytes = htpops::flash_attn_workspace_bytes(qo_len, kv_len, n_heads, head_dim);
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
    ws = ctx->scratch_ptr;
  } else {
    if (int r = ensure_workspace(ctx, ws_bytes)) {
      return r;
    }
    note_device_write(ctx, o, o_bytes);
    ws = ctx->workspace;
  }
  void *q8_out = nullptr;
  if (ctx->attn_q8_out && htpops::flash_attn_writes_q8_0(qo_len, head_dim, qo_is_f32 != 0)) {
    q8_out = ctx->attn_q8_out;
    note_device_write(ctx, q8_out, q8_0_bytes(1, (size_t) n_heads * head_dim));
  }
  HTPOPS_HIP(ctx, htpops::launch_flash_attn(ctx->stream, o, q, k, v, mask, qo_len, kv_len, n_heads, n_kv_heads,
                                            head_dim, qo_is_f32 != 0, causal != 0, ws, q8_out));
  ctx->attn_q8_done = q8_out != nullptr;
  return HTPOPS_OK;
}

}  // namespace

// ------------------------------------------------------------------------------------------------ session

extern "C" int htpops_init_backend(htpops_context **out_ctx, int device) {
  if (!out_ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  *out_ctx            = nullptr;
  htpops_context *ctx = new (std::nothrow) htpops_context();
  if (!ctx) {
    return HTPOPS_ERR_NOMEM;
  }
  ctx->buffers.emplace_back();  // handle 0 is never valid
  if (device != HTPOPS_DEVICE_NONE) {
    int        count = 0;
    hipError_t e     = hipGetDeviceCount(&count);
    if (e != hipSuccess || device < 0 || device >= count) {
      if (getenv("HTPOPS_LOG")) {
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
  return ctx ? ctx->last_error.c_str() : "null context";
}

extern "C" int htpops_synchronize(htpops_context *ctx) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  if (!ctx->has_device) {
    return HTPOPS_OK;
  }
  HTPOPS_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return HTPOPS_OK;
}

extern "C" void *htpops_get_stream(htpops_context *ctx) {
  return ctx ? (void *) ctx->stream : nullptr;
}

// ------------------------------------------------------------------------------------------------ buffers

extern "C" int htpops_buffer_alloc(htpops_context *ctx, size_t bytes) {
  if (!ctx || bytes == 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "buffer_alloc: zero size");
  }
  Lock lock(ctx->mu);
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
  if (!ctx || !device_ptr || bytes == 0) {
    return fail(ctx, HTPOPS_ERR_REJECTED, "buffer_register: null pointer or zero size");
  }
  Lock lock(ctx->mu);
  return new_handle(ctx, device_ptr, bytes, false);
}

extern "C" int htpops_buffer_release(htpops_context *ctx, int handle) {
  if (!ctx) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
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

// For owned weight buffers that the caller's own kernels have rewritten through htpops_buffer_device_ptr: drops the
// converted copies made from the buffer and marks recordings that use it stale.
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

// ------------------------------------------------------------------------------------------------ ops

extern "C" int htpops_execute_op(htpops_context *ctx, const struct OpComputeRequest *req) {
  if (!ctx || !req) {
    return HTPOPS_ERR_REJECTED;
  }
  Lock lock(ctx->mu);
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
        const int   wt = (req->op == HTP_OPS_MAT_MUL_Q4_0_Q8_0 || req->op == HTP_OPS_MAT_MUL_Q4_0_A32) ? htpops::kQ4_0 :
                                                                                                         htpops::kQ8_0;
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
  struct RequestHeader *hdr[htpops::kGemvGroupMax];
  float                *out[htpops::kGemvGroupMax];
  const void           *w[htpops::kGemvGroupMax];
  const void           *act[htpops::kGemvGroupMax];
  int                   n[htpops::kGemvGroupMax];
  int                   k[htpops::kGemvGroupMax];
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
};

// The many-row members of a batch: converted weights from the cache (made now where missing), the distinct activation
// matrices converted side by side in the workspace by one launch, then one launch for all the products. Returns a
// status, or 1 when the members have to be run one by one after all.
static_assert(htpops::kGemmGroupMax == htpops::kGemvGroupMax, "one batch structure serves both");
int run_fragment_group(htpops_context *ctx, GemvBatch &b) {
  const void *wf[htpops::kGemmGroupMax];
  for (int i = 0; i < b.count; ++i) {
    MatMulPlan plan = plan_mat_mul(ctx, b.w[i], true, b.m, b.k[i], b.n[i], b.wt);
    if (plan.kind != kPlanFragments || !(plan.cached || plan.cacheable)) {
      return 1;  // (a converted copy went away since the member joined: the caller runs the members one by one)
    }
    if (!plan.cached) {
      void *fresh = nullptr;
      HTPOPS_HIP(ctx, hipMalloc(&fresh, plan.weight_bytes));
      const hipError_t e = htpops::launch_weights_to_i8_fragments(ctx->stream, fresh, b.w[i], b.k[i], b.n[i], (htpops::WeightType) b.wt);
      if (e != hipSuccess) {
        (void) hipFree(fresh);
        return fail(ctx, HTPOPS_ERR_HIP, "weight conversion: %s", hipGetErrorString(e));
      }
      ctx->frag_cache.push_back({ b.w[i], weight_bytes((size_t) b.n[i], (size_t) b.k[i], b.wt), plan.frag_kind, b.k[i], b.n[i], fresh });
      plan.cached = fresh;
    }
    wf[i] = plan.cached;
  }
  // distinct (activation, k) pairs and where their conversions go
  const void *acts[htpops::kGemmGroupMax];
  int         act_k[htpops::kGemmGroupMax], act_of[htpops::kGemmGroupMax], n_acts = 0;
  size_t      offset[htpops::kGemmGroupMax], total = 0;
  for (int i = 0; i < b.count; ++i) {
    int j = 0;
    while (j < n_acts && !(acts[j] == b.act[i] && act_k[j] == b.k[i])) {
      ++j;
    }
    if (j == n_acts) {
      acts[j] = b.act[i], act_k[j] = b.k[i], offset[j] = total;
      total += (htpops::gemm_i8_act_fragment_bytes(b.m, b.k[i]) + 255) & ~(size_t) 255;
      ++n_acts;
    }
    act_of[i] = j;
  }
  size_t xbytes = 0;  // scratch for the partial tiles of members whose K is split over workgroups, behind the activations
  for (int i = 0; i < b.count; ++i) {
    xbytes += htpops::gemm_i8_fragments_exchange_bytes(b.m, b.n[i], b.k[i]);
  }
  if (int r = ensure_workspace(ctx, total + xbytes)) {
    return r;
  }
  ctx->act_fragments.src = nullptr;
  uint8_t    *ws = static_cast<uint8_t *>(ctx->workspace);
  void       *act_dst[htpops::kGemmGroupMax];
  const void *af[htpops::kGemmGroupMax];
  for (int j = 0; j < n_acts; ++j) {
    act_dst[j] = ws + offset[j];
  }
  for (int i = 0; i < b.count; ++i) {
    af[i] = act_dst[act_of[i]];
  }
  HTPOPS_HIP(ctx, htpops::launch_act_to_i8_fragments_group(ctx->stream, n_acts, act_dst, acts, act_k, b.m));
  HTPOPS_HIP(ctx, htpops::launch_gemm_i8_fragments_group(ctx->stream, b.count, b.out, af, wf, b.n, b.k, b.m, ws + total, xbytes,
                                                         ctx->tickets, kTicketSlots));
  return HTPOPS_OK;
}

// The many-row members of a batch that take the FP6-tile kernel over one set of activation rows: converted weights from
// the cache (made now where missing), the activations converted once (or found converted at the start of the
// workspace), one launch per kernel variant for the products. Returns a status, or 1 when the members have to be run
// one by one after all.
int run_fp6_group(htpops_context *ctx, GemvBatch &b) {
  const void *wf[htpops::kGemmGroupMax];
  size_t      act_bytes = 0;
  for (int i = 0; i < b.count; ++i) {
    MatMulPlan plan = plan_mat_mul(ctx, b.w[i], true, b.m, b.k[i], b.n[i], b.wt);
    if (plan.kind != kPlanLdsFp6 || !(plan.cached || plan.cacheable)) {
      return 1;  // (a converted copy went away since the member joined: the caller runs the members one by one)
    }
    if (!plan.cached) {
      void *fresh = nullptr;
      HTPOPS_HIP(ctx, hipMalloc(&fresh, plan.weight_bytes));
      const hipError_t e = htpops::launch_q4_0_to_fp6_tiles(ctx->stream, fresh, b.w[i], b.k[i], b.n[i]);
      if (e != hipSuccess) {
        (void) hipFree(fresh);
        return fail(ctx, HTPOPS_ERR_HIP, "weight conversion: %s", hipGetErrorString(e));
      }
      ctx->frag_cache.push_back({ b.w[i], weight_bytes((size_t) b.n[i], (size_t) b.k[i], b.wt), plan.frag_kind, b.k[i], b.n[i], fresh });
      plan.cached = fresh;
    }
    wf[i]     = plan.cached;
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
  bool         keep    = ready || (ctx->in_message && in_owned_buffer(ctx, b.act[0], a_bytes));
  for (int i = 0; i < b.count; ++i) {
    keep = keep && !ranges_overlap(b.out[i], (size_t) m * b.n[i] * 4, b.act[0], a_bytes);
  }
  af.src = nullptr;
  HTPOPS_HIP(ctx, htpops::launch_gemm_fp6_lds_group(ctx->stream, b.count, b.out, b.act[0], wf, m, k, b.n, ctx->workspace, ready));
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
      const hipError_t e = htpops::launch_gemv_group_rms_norm_q8_0_act(ctx->stream, b.count, b.out, b.w, b.n, b.norm.ne0,
                                                                       (htpops::WeightType) b.wt, b.norm.src,
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
      e = htpops::launch_gemv_group_q8_0_act(ctx->stream, b.count, b.out, b.act, b.w, b.n, b.k, (htpops::WeightType) b.wt);
    } else {
      // 2..16 rows. Two or three rows are one launch of the weight stream that keeps them in registers, each member
      // with its own rows and row length. Otherwise (same k) members whose weights have (or get) a repacked copy go
      // to the kernel that streams it, again each with its own activation rows; the rest go to the K-sliced kernel,
      // one launch per set of rows (it stages one). Which kernel a matrix gets depends on that matrix alone.
      if (htpops::gemv_rows_fits(b.m, k0, (htpops::WeightType) b.wt)) {
        e = htpops::launch_gemv_rows_group_q8_0_act(ctx->stream, b.count, b.out, b.act, b.w, b.n, b.m, b.k,
                                                    (htpops::WeightType) b.wt);
      } else {
        float      *out_a[htpops::kGemvGroupMax];
        const void *w_a[htpops::kGemvGroupMax], *act_a[htpops::kGemvGroupMax];
        int         n_a[htpops::kGemvGroupMax], count_a = 0;
        bool        sliced[htpops::kGemvGroupMax] = {};
        for (int i = 0; i < b.count; ++i) {
          const void *lw = nullptr;
          if (int r = lane_order_weights(ctx, b.w[i], b.act[i], b.m, k0, b.n[i], b.wt, &lw)) {
            b.hdr[i]->state = r;
          } else if (lw) {
            out_a[count_a] = b.out[i], w_a[count_a] = lw, act_a[count_a] = b.act[i], n_a[count_a++] = b.n[i];
          } else if (b.m <= kSkinnyGroupMaxM) {
            sliced[i] = true;
          } else {
            // more rows than the K-sliced group launch takes: on its own
            b.hdr[i]->state = op_mat_mul_q8(ctx, b.out[i], b.act[i], b.w[i], b.m, k0, b.n[i], b.wt);
          }
        }
        e = hipSuccess;
        if (count_a > 0) {
          e = htpops::launch_matmul_lane_order_group(ctx->stream, count_a, out_a, act_a, w_a, n_a, b.m, k0,
                                                     (htpops::WeightType) b.wt);
        }
        for (int first = 0; first < b.count && e == hipSuccess && ret == HTPOPS_OK; ++first) {
          if (!sliced[first]) {
            continue;
          }
          float      *out_b[htpops::kGemvGroupMax];
          const void *w_b[htpops::kGemvGroupMax];
          int         n_b[htpops::kGemvGroupMax], count_b = 0;
          for (int i = first; i < b.count; ++i) {  // everybody left that reads the rows of `first`
            if (sliced[i] && b.act[i] == b.act[first]) {
              out_b[count_b] = b.out[i], w_b[count_b] = b.w[i], n_b[count_b++] = b.n[i];
              sliced[i] = false;
            }
          }
          const size_t ws = htpops::matmul_skinny_group_workspace_bytes(count_b, n_b, b.m, k0);
          if (int r = ensure_workspace(ctx, ws)) {
            ret = r;
          } else {
            e = htpops::launch_matmul_skinny_group(ctx->stream, count_b, out_b, b.act[first], w_b, n_b, b.m, k0,
                                                   (htpops::WeightType) b.wt, ctx->workspace, ctx->tickets, kTicketSlots);
          }
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
  const int    wt        = req->op == HTP_OPS_MAT_MUL_Q4_0_Q8_0 ? htpops::kQ4_0 : htpops::kQ8_0;
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
    if (!fp6 && !(plan.kind == kPlanFragments && htpops::gemm_i8_fragments_groupable(p->m, p->n))) {
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
  bool join = b.count > 0 && b.count < htpops::kGemvGroupMax && b.wt == wt && b.m == p->m && (!b.fused || reads_norm) &&
              b.fp6 == fp6 && (!fp6 || (b.act[0] == act && b.k[0] == p->k)) &&
              (p->m == 1 || many_rows || b.k[0] == p->k ||
               (htpops::gemv_rows_fits(p->m, p->k, (htpops::WeightType) wt) &&
                htpops::gemv_rows_fits(b.m, b.k[0], (htpops::WeightType) wt)));
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
    b.wt = wt, b.m = p->m, b.fp6 = fp6;
  }
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
      pq->ne0 != p->n_heads * p->head_dim || !htpops::flash_attn_writes_q8_0(1, p->head_dim, true)) {
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

// 0, or the error if the request table does not fit `msg_bytes` (0 = unknown size, offsets are trusted)
int check_message_framing(htpops_context *ctx, const struct MessageHeader *msg, size_t msg_bytes) {
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

// Walks a message and enqueues every request in order (reference: src/dsp/commu.c:91-114). Returns 0 or the
// framing error; per-request results go to RequestHeader.state.
int enqueue_message(htpops_context *ctx, struct MessageHeader *msg, size_t msg_bytes) {
  if (int r = check_message_framing(ctx, msg, msg_bytes)) {
    return r;
  }
  const int n_reqs = msg->n_reqs;
  GemvBatch batch;
  ctx->act_fragments.src   = nullptr;
  ctx->in_message          = true;
  ctx->message_submissions = 0;
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

}  // namespace

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
  if (ctx->poller.joinable()) {
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
  if (!ctx || !msg || max_msg_size < sizeof(struct MessageHeader) + sizeof(int32_t)) {
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
  if (!ctx || !ctx->chan_msg) {
    return HTPOPS_OK;
  }
  ctx->poller_stop.store(true, std::memory_order_release);
  if (ctx->poller.joinable()) {
    ctx->poller.join();
  }
  ctx->chan_msg   = nullptr;
  ctx->chan_bytes = 0;
  return HTPOPS_OK;
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
  hipError_t e = htpops::launch_mfma_loop(ctx->stream, kind, 16, sink, n_blocks);  // warm-up
  float      ms = 0.f;
  if (e == hipSuccess) e = hipEventRecord(ctx->ev_start, ctx->stream);
  if (e == hipSuccess) e = htpops::launch_mfma_loop(ctx->stream, kind, iters, sink, n_blocks);
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
    e = htpops::launch_read(ctx->stream, bufs[b], bytes, sink);
  }
  if (e == hipSuccess) e = hipEventRecord(ctx->ev_start, ctx->stream);
  for (int i = 0; i < iters && e == hipSuccess; ++i) {
    for (size_t b = 0; b < bufs.size() && e == hipSuccess; ++b) {
      e = htpops::launch_read(ctx->stream, bufs[b], bytes, sink);
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
  if (e == hipSuccess) e = htpops::launch_copy(ctx->stream, b, a, bytes);
  if (e == hipSuccess) e = hipEventRecord(ctx->ev_start, ctx->stream);
  for (int i = 0; i < iters && e == hipSuccess; ++i) {
    e = htpops::launch_copy(ctx->stream, b, a, bytes);
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
