// What the host-side translation units of the op backend share: the context, its buffer registry and converted-copy
// cache, and the helpers that every entry point uses. The C ABI itself is declared in include/htpops.h; this header is
// internal to the library.
//
//   context.cc   session: init / close / options / synchronize (reference: src/dsp/commu.c:226-249)
//   registry.cc  handle -> device memory table and the converted weight copies kept with it
//                (reference: src/dsp/mmap_mgr.cc:15-43)
//   ops.cc       request validation and kernel selection, one function per op (reference: src/dsp/op_executor.cc:52-204)
//   message.cc   the consumer's walk over a message and the batching of its requests (reference: src/dsp/commu.c:91-126)
//   recorder.cc  a message captured into a HIP graph
//   channel.cc   the polling consumer thread (reference: src/dsp/commu.c:37-136, :151-212)
//   bench_entries.cc  timers and calibration kernels of include/htpops_bench.h
#pragma once

#include "htpops.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <mutex>
#include <string>
#include <thread>
#include <utility>
#include <vector>

#include "kernels.h"

namespace htpops {
namespace host {

struct Buffer {
  void  *ptr   = nullptr;
  size_t size  = 0;
  bool   owned = false;  // allocated by the context (freed on release)
  bool   live  = false;
  // Converted copies of weights in this buffer may be kept: always for owned buffers (their contents change only
  // through htpops_buffer_write or as an op's output, both of which drop the copies); for caller-registered memory
  // once the caller has asked for a copy with htpops_buffer_prepare_weights, which puts the buffer under the same
  // contract (htpops_buffer_invalidate after rewriting it).
  bool   keeps_copies = false;
};

constexpr int kMaxHandles  = 1 << 20;
constexpr int kTicketSlots = 1 << 16;

// size of the static device array behind htpops_flash_attn_noalloc_ptr (context.cc)
constexpr size_t kNoAllocScratchBytes = (size_t) 8 << 20;

// The switches of a context: kernel choices that tests and A/B measurements override. Read once from the environment
// when the context is created (HTPOPS_<NAME> in upper case), changed afterwards only through htpops_set_option; no
// entry point on the op path reads the environment.
struct Options {
  int lane_order          = 1;   // 0: never the repacked-weight kernels; 2 / 3: the one-block kernel with one / two tiles per workgroup
  int gemm_fp6            = -1;  // 0: never the FP6-tile kernel; 1: also on shapes that do not fill the device
  int gemv_rows_kernel    = 1;   // 0: two and three rows take the repacked-weight / K-sliced kernels
  int gemm_tile_units     = 0;   // 1 / 2: force the tile size of the int8 fragment kernel
  int attn_key_groups     = 0;   // 1 / 2: force the number of key groups of the prefill attention kernel
  int attn_mask_threshold = 0;   // 1: the mask selects keys (keep iff mask > -16) instead of being added
  int converted_cap_mib   = 0;   // > 0: converted weight copies are evicted (least recently used first) beyond this
  int log                 = 0;   // errors are also printed to stderr
};

}  // namespace host
}  // namespace htpops

struct htpops_recorded_message {
  htpops_context *ctx   = nullptr;
  hipGraph_t      graph = nullptr;
  hipGraphExec_t  exec  = nullptr;  // null for a message without launches
  bool            stale = false;
  std::vector<std::pair<uintptr_t, size_t>> ranges;
};

struct htpops_context {
  // Guards everything below: the channel's consumer thread walks messages (resolving handles, making copies) while the
  // host thread may allocate, write or release buffers, as a host of the reference does while its consumer thread runs
  // (reference: src/dsp/mmap_mgr.cc:15-27 maps lazily on that thread). Recursive: a message's RPCMEM_MAP request
  // releases buffers from inside the walk.
  std::recursive_mutex mu;
  htpops::host::Options opt;
  // Set by the message walk around an attention request whose output the next request quantizes to Q8_0: where that
  // request wants its row, and whether the attention launch wrote it.
  void               *attn_q8_out  = nullptr;
  bool                attn_q8_done = false;
  int                 device     = HTPOPS_DEVICE_NONE;
  bool                has_device = false;
  hipStream_t         stream     = nullptr;
  std::vector<htpops::host::Buffer> buffers;  // index = handle; slot 0 unused
  std::vector<int>    free_slots;
  std::string         last_error;

  // scratch owned by the context: quantized activations of the fp32-activation matmul, attention partials
  void  *workspace       = nullptr;
  size_t workspace_bytes = 0;
  // zeroed ticket counters of the K-sliced matmul (each launch leaves them zeroed)
  unsigned *tickets = nullptr;

  // Converted copies of weights (MFMA fragment order for ops 1-4, int8 fragments, FP6 tiles, operand-order nibbles),
  // keyed by the source range and the kind; dropped when the source is written through the registry, released or
  // invalidated.
  struct FragEntry {
    const void *src;
    size_t      src_bytes;
    int         kind, k, n;
    void       *frag;
    size_t      frag_bytes;
    uint64_t    last_use;  // message serial of the most recent use (eviction order under Options::converted_cap_mib)
  };
  std::vector<FragEntry> frag_cache;
  size_t                 converted_bytes = 0;  // sum of frag_bytes
  uint64_t               use_serial      = 1;  // advanced per message walk and per single op

  // Which activations the converted operand at the start of `workspace` was made from. Only kept while one message is
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

  // this device's copy of the static scratch array of the entry point that allocates nothing (hipGetSymbolAddress at
  // init, with the device current)
  void *scratch_ptr = nullptr;

  // mailbox channel
  std::thread           poller;
  std::atomic<bool>     poller_stop{ false };
  struct MessageHeader *chan_msg   = nullptr;
  size_t                chan_bytes = 0;
};

namespace htpops {
namespace host {

using Lock = std::lock_guard<std::recursive_mutex>;

// ---- errors ----
int fail(htpops_context *ctx, int code, const char *fmt, ...) __attribute__((format(printf, 3, 4)));
int hip_fail(htpops_context *ctx, hipError_t e, const char *what);

#define HTPOPS_HIP(ctx, expr)                             \
  do {                                                    \
    hipError_t e_ = (expr);                               \
    if (e_ != hipSuccess) {                               \
      return ::htpops::host::hip_fail((ctx), e_, #expr);  \
    }                                                     \
  } while (0)

int need_device(htpops_context *ctx);
// The static device array of the entry point that allocates nothing is shared by the contexts of a GPU: true when
// `ctx` holds it (or has just taken it), false while another context that has not yet waited for its stream does.
bool claim_static_scratch(htpops_context *ctx);
void release_static_scratch(htpops_context *ctx);

// ---- small helpers ----
inline bool aligned(const void *p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}
inline bool ranges_overlap(const void *a, size_t a_bytes, const void *b, size_t b_bytes) {
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
  return a0 < b0 + b_bytes && b0 < a0 + a_bytes;
}
// a * b * c with overflow check; false on overflow
bool mul3(size_t a, size_t b, size_t c, size_t *out);
inline size_t permuted_weight_bytes(size_t n, size_t k, int kind) {
  // reference: op_executor.cc:100-102, :124-126
  return kind == 1 ? k * n * 2 : k * n / 256 * (kind == 3 ? 272 : 144);
}
inline size_t q8_0_bytes(size_t rows, size_t k) {
  return rows * (k / 32) * 34;
}
inline size_t weight_bytes(size_t n, size_t k, int weight_type) {
  return n * (k / 32) * (weight_type == kQ4_0 ? 18 : 34);
}

// ---- registry (registry.cc) ----
Buffer *lookup(htpops_context *ctx, int handle);
// Resolves (handle, offset) to an address with `need` readable/writable bytes, or null (the reference's
// "mmap_manager_get_map returned NULL" case, op_executor.cc:57-61, extended with range checks).
void *resolve(htpops_context *ctx, const struct RpcmemBufAddr &addr, size_t need);
// memory in [ptr, ptr + bytes) is about to go (bytes = 0: the workspace, which every recording may use)
void mark_recordings_stale(htpops_context *ctx, const void *ptr, size_t bytes);
int  ensure_workspace(htpops_context *ctx, size_t bytes, bool keep_act_fragments = false);
// converted copies made from [ptr, ptr + bytes) are stale
void drop_fragments(htpops_context *ctx, const void *ptr, size_t bytes);
// an op is about to write [ptr, ptr + bytes)
void note_device_write(htpops_context *ctx, const void *ptr, size_t bytes);
// true when [ptr, ptr + bytes) lies inside a buffer whose converted copies may be kept (Buffer::keeps_copies)
bool may_keep_copies(htpops_context *ctx, const void *ptr, size_t bytes);
// the cached copy of (weight, kind, k, n) or nullptr; a hit is stamped as used now
const void *find_copy(htpops_context *ctx, const void *weight, int kind, int k, int n);
// Allocates `frag_bytes` for a new converted copy (evicting older ones first when a cap is set) and enters it into
// the cache; the caller fills it with a conversion launch and calls forget_copy if that fails.
int  new_copy(htpops_context *ctx, const void *weight, size_t src_bytes, int kind, int k, int n, size_t frag_bytes,
              void **out);
void forget_copy(htpops_context *ctx, void *frag);

// ---- ops (ops.cc) ----
constexpr int kSkinnyGroupMaxM = 8;   // rows of the K-sliced kernel's grouped launch
constexpr int kBatchMaxM       = 16;  // rows up to which same-activation requests of a message are grouped
constexpr int kManyRowsMinM    = 33;  // rows from which a matmul takes the matrix-core kernels

constexpr int kFragKindRowLayout = 100;  // + ggml type: int8 fragments (kinds 1..4 are the tile-permuted formats of ops 1-4)
constexpr int kFragKindLaneOrder = 300;  // + ggml type: weights in matrix-core operand order (2..16 activation rows)
constexpr int kFragKindBlockPairs = 350; // + ggml type: the same for the two-blocks-per-instruction kernel (2..8 rows)
constexpr int kFragKindFp6Tiles  = 400;  // + ggml type: FP6 operand tiles of the many-row Q4_0 matmul (LDS kernel)

// Which kernel family a quantized matmul takes and how much of the context's workspace it needs.
enum PlanKind {
  kPlanFewRows,    // m below the many-row threshold: the weight-streaming kernels
  kPlanLdsFp6,     // many rows, Q4_0, k % 64 == 0, enough output tiles, weights whose converted copy may be kept
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
MatMulPlan plan_mat_mul(htpops_context *ctx, const void *weight, bool act_aligned, int m, int k, int n, int wt);
// The converted copy a plan wants, from the cache or made now and cached (plan.cacheable); *out stays nullptr for a
// plan whose weights may not be cached (the caller converts into its workspace).
int plan_weight_copy(htpops_context *ctx, MatMulPlan &plan, const void *weight, int k, int n, int wt, const void **out);
// The repacked copy of `weight` for the few-row kernels: from the cache, or made now and cached. *out stays nullptr
// when this matmul takes neither of them. *block_pairs: which of the two operand orders the copy is in (the kernel
// with two blocks per matrix instruction for up to 8 rows of Q4_0, the one-block kernel otherwise); the choice depends
// on (m, k, weight type) and the context's switches only, so the members of a grouped launch agree on it.
// Two and three rows of Q4_0: the two-blocks-per-instruction kernel over a repacked copy where the shape fits it and a
// copy is there or may be kept (a Llama-7B layer: 25 against 28 us at two rows, 25 against 32 us at three); the kernel
// that holds the rows in registers and reads the weights as they are otherwise.
bool prefers_block_pairs(const htpops_context *ctx, int m, int k, int n, int wt);
int lane_order_weights(htpops_context *ctx, const void *weight, const void *act, int m, int k, int n, int wt,
                       const void **out, bool *block_pairs);

int op_rms_norm(htpops_context *ctx, float *dst, const float *src, const float *weight, float eps, int ne0, int ne1);
int op_quantize(htpops_context *ctx, void *dst, const float *src, int k, int m);
int op_rms_norm_quantize(htpops_context *ctx, void *dst, const float *src, const float *weight, float eps, int ne0,
                         int ne1);
int op_mat_mul_q8(htpops_context *ctx, float *dst, const void *act, const void *weight, int m, int k, int n,
                  int weight_type);
int op_mat_mul_f32(htpops_context *ctx, float *dst, const float *act, const void *weight, int m, int k, int n,
                   int weight_type);
int op_mat_mul_permuted(htpops_context *ctx, float *dst, const float *act, const void *weight, int m, int k, int n,
                        int kind);
int op_flash_attn(htpops_context *ctx, void *o, const void *q, const void *k, const void *v, const void *mask,
                  int qo_len, int kv_len, int n_heads, int n_kv_heads, int head_dim, int qo_is_f32, int causal,
                  bool no_alloc = false);

// ---- messages (message.cc) ----
// 0, or the error if the request table does not fit `msg_bytes` (0 = unknown size, offsets are trusted)
int check_message_framing(htpops_context *ctx, const struct MessageHeader *msg, size_t msg_bytes);
// Walks a message and enqueues every request in order (reference: src/dsp/commu.c:91-114). Returns 0 or the
// framing error; per-request results go to RequestHeader.state. The caller holds the context's lock.
int enqueue_message(htpops_context *ctx, struct MessageHeader *msg, size_t msg_bytes);

// The 8-byte mailbox state is declared packed (alignment 1) but lives at the start of the message buffer, which
// callers allocate at least 8-byte aligned; an unaligned buffer falls back to byte accesses between fences.
uint64_t load_state(struct MessageHeader *msg);
void     store_state(struct MessageHeader *msg, uint64_t d);

}  // namespace host
}  // namespace htpops
