// Prefill-sized Q4_0 x Q8_0 matmul on gfx950: out fp32 [m][n] = act block_q8_0 [m][k/32] x W (Q4_0 rows).
//
// Replaces the many-row case of hmx_mat_mul_permuted_qk_0_d16a32 (reference: src/dsp/ops/mat_mul.c:875-1153); the
// arithmetic is ggml's integer block dot: exact block sums, one fp32 product of the two fp16 scales per block.
//
// Per 32 x 32 x 32 block ("unit") the work is
//     S = act_int8 x w_int4     ONE v_mfma_scale_f32_32x32x64_f8f6f4 on FP6 (E2M3) operands, exact:
//                               an int8 activation a = 16 hi + lo with hi in [-8, 7], lo in [0, 15]; hi, lo and the
//                               weight q - 8 in [-8, 7] are all integers of magnitude <= 15, which E2M3 holds exactly
//                               as t / 8 (code = sign bit | magnitude). The instruction's K = 64 is spent as
//                               [hi (32) | lo (32)] against [w (32) | w (32)]; its per-32 block scales (powers of two)
//                               supply the 16 of the hi half and undo the 1/8s. S leaves the matrix core as fp32.
//     C = d_act (x) d_w         one v_mfma_f32_32x32x8_f16 with the two fp16 scales in K slot 0: the exact fp32
//                               product of the scales of every (row, column) pair
//     acc = fma(S, C, acc)      the only vector-ALU work: one fma per block sum
// FP6 runs at twice the int8 rate and S needs no int -> float conversion, so a unit issues 16 vector instructions
// where int8 MFMA + convert + fma issues 32; two waves per SIMD interleave matrix and vector work.
//
// Operands are kept in "panels" whose byte order is the order the matrix core wants, so the inner loop is
// global -> LDS DMA, LDS -> register reads and matrix instructions, with no data shuffling:
//   weights   converted once per weight buffer and cached by the caller (0.875 bytes per weight)
//   act       converted per call from block_q8_0 rows
// A workgroup (8 waves of 64 x 64) owns a 128 x 256 output tile at a time. The (tile, K block) space is cut into
// one equal contiguous range per compute unit, so a tile whose K range is shared by several workgroups is finished
// by whichever of them arrives last, adding the parts in K order (the result does not depend on timing).
#include "device_utils.h"
#include "kernels.h"


namespace htpops {

namespace {

typedef int      v8i __attribute__((ext_vector_type(8)));
typedef int      v2i __attribute__((ext_vector_type(2)));
typedef float    v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ---- panel geometry -----------------------------------------------------------------------------------------------
// A fragment holds, per lane, the 32 FP6 codes of one row (column) of a 32 x 32-element block (24 bytes: element e at
// bits [6 e, 6 e + 6)) and the block's scale as the operand of the scale instruction (8 bytes: fp16 scale, 0, 0, 0),
// as two planes of 16 bytes per lane: plane 0 = code bytes 0..15, plane 1 = code bytes 16..23 + scale.
//   activation fragment: 64 lanes; lane (c, h): row c, h = 0 the hi parts, h = 1 the lo parts; the scale of the
//                        h = 1 lanes is 0 (the scale instruction's K slots 4..7 then add nothing)        2048 bytes
//   weight fragment:     32 lanes; column c (both lane halves read the same 32 bytes)                    1024 bytes
// A block = the fragments of a row group (128 rows) / column group (256 columns) for one K block: 8 KiB each.
constexpr int kTileM = 128, kTileN = 256;
constexpr int kAFrag = 2048, kBFrag = 1024;
constexpr int kABlock = 4 * kAFrag, kBBlock = 8 * kBFrag;  // 8192, 8192

__device__ __forceinline__ uint32_t fp6_code(int t) {  // integer |t| <= 15 as E2M3 value t / 8
  const uint32_t mag = (uint32_t) (t < 0 ? -t : t);
  return (t < 0 ? 32u : 0u) | mag;
}

__device__ __forceinline__ void pack_fp6(uint32_t w[6], const int t[32]) {
#pragma unroll
  for (int i = 0; i < 6; ++i) {
    w[i] = 0;
  }
#pragma unroll
  for (int e = 0; e < 32; ++e) {
    const uint32_t code = fp6_code(t[e]);
    const int      bit  = 6 * e;
    w[bit / 32] |= code << (bit % 32);
    if (bit % 32 > 26) {
      w[bit / 32 + 1] |= code >> (32 - bit % 32);
    }
  }
}

// one thread per (column group, K block, fragment j, column c)
__global__ __launch_bounds__(256) void q4_0_to_fp6_panel_kernel(uint8_t *__restrict__ panel, const uint16_t *__restrict__ w,
                                                                int n, int nblk, size_t total) {
  const size_t t = (size_t) blockIdx.x * 256 + threadIdx.x;
  if (t >= total) {
    return;
  }
  const int    c = (int) (t & 31), j = (int) ((t >> 5) & 7);
  const size_t blk = t >> 8;  // group * nblk + kb
  const int    kb = (int) (blk % (size_t) nblk), group = (int) (blk / (size_t) nblk);
  const int    col = group * kTileN + j * 32 + c;
  uint32_t     o[6] = { 0, 0, 0, 0, 0, 0 };
  uint32_t     sc   = 0;
  if (col < n) {
    const uint16_t *b = w + ((size_t) col * nblk + kb) * 9;  // 18-byte block: fp16 scale, 16 bytes of nibbles
    sc = b[0];
    int v[32];
    // byte i: low nibble = element i, high nibble = element i + 16 (reference: mat_mul.c:266-271)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t q = b[1 + i];
      v[2 * i]          = (int) (q & 15) - 8;
      v[2 * i + 16]     = (int) ((q >> 4) & 15) - 8;
      v[2 * i + 1]      = (int) ((q >> 8) & 15) - 8;
      v[2 * i + 1 + 16] = (int) ((q >> 12) & 15) - 8;
    }
    pack_fp6(o, v);
  }
  uint8_t *frag = panel + blk * kBBlock + j * kBFrag;
  *reinterpret_cast<uint4 *>(frag + c * 16)       = make_uint4(o[0], o[1], o[2], o[3]);
  *reinterpret_cast<uint4 *>(frag + 512 + c * 16) = make_uint4(o[4], o[5], sc, 0);
}

// A workgroup converts 32 rows x 8 K blocks: the raw blocks are read as contiguous runs of halfwords into LDS, then
// thread (K block, row c) builds the hi lane and the lo lane of its row and writes them next to its neighbours'.
__global__ __launch_bounds__(256) void q8_0_to_fp6_panel_kernel(uint8_t *__restrict__ panel, const uint16_t *__restrict__ act,
                                                                int m, int nblk) {
  constexpr int kRowHalfwords = 8 * 17;
  __shared__ uint16_t raw[32 * kRowHalfwords];
  const int tid = threadIdx.x;
  const int group = blockIdx.x >> 2, i = blockIdx.x & 3, kb0 = blockIdx.y * 8;
  const int row0 = group * kTileM + i * 32;
  const int run  = min(8, nblk - kb0) * 17;  // halfwords of a row that exist
#pragma unroll
  for (int j = 0; j < 17; ++j) {
    const int e = tid + 256 * j, r = e / kRowHalfwords, col = e - r * kRowHalfwords;
    raw[e] = (row0 + r < m && col < run) ? act[((size_t) (row0 + r) * nblk + kb0) * 17 + col] : (uint16_t) 0;
  }
  __syncthreads();
  const int kbl = tid >> 5, c = tid & 31;
  if (kb0 + kbl >= nblk) {
    return;
  }
  const uint16_t *b = raw + c * kRowHalfwords + kbl * 17;  // 34-byte block: fp16 scale, 32 int8 (zeros past m)
  int hi[32], lo[32];
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const uint32_t q = b[1 + e];
    const int      a0 = (int) (int8_t) (q & 0xff), a1 = (int) (int8_t) (q >> 8);
    lo[2 * e] = a0 & 15, lo[2 * e + 1] = a1 & 15;  // a = 16 hi + lo, hi = floor(a / 16)
    hi[2 * e] = (a0 - lo[2 * e]) / 16, hi[2 * e + 1] = (a1 - lo[2 * e + 1]) / 16;
  }
  uint32_t oh[6], ol[6];
  pack_fp6(oh, hi);
  pack_fp6(ol, lo);
  uint8_t *frag = panel + ((size_t) group * nblk + kb0 + kbl) * kABlock + i * kAFrag;
  *reinterpret_cast<uint4 *>(frag + c * 16)               = make_uint4(oh[0], oh[1], oh[2], oh[3]);
  *reinterpret_cast<uint4 *>(frag + (32 + c) * 16)        = make_uint4(ol[0], ol[1], ol[2], ol[3]);
  *reinterpret_cast<uint4 *>(frag + 1024 + c * 16)        = make_uint4(oh[4], oh[5], b[0], 0);
  *reinterpret_cast<uint4 *>(frag + 1024 + (32 + c) * 16) = make_uint4(ol[4], ol[5], 0, 0);
}

// ---- the matmul ---------------------------------------------------------------------------------------------------
constexpr int kThreads = 512;
[[maybe_unused]] constexpr int kStages = 8;  // K blocks resident in LDS
// LDS image of one K block: [weight block 8 KiB][activation block 8 KiB]
[[maybe_unused]] constexpr int kImgA = kBBlock;
[[maybe_unused]] constexpr int kImgBytes = kBBlock + kABlock;  // 16384
constexpr int kPartialFloats = kTileM * kTileN;   // one tile of partial sums in the workspace

typedef __attribute__((address_space(1))) const void *gptr_t;
typedef __attribute__((address_space(3))) void       *lptr_t;
typedef int v6i __attribute__((ext_vector_type(6)));
typedef int v4i __attribute__((ext_vector_type(4)));

// ---- who multiplies what ------------------------------------------------------------------------------------------
// G workgroups (one per compute unit) share `tiles` tiles of `nblk` K blocks so that all are busy for the same time
// AND workgroups that run side by side are at the same K block, because then they fetch the same operand blocks at
// the same time and the L2 serves all but the first (tiles of one column group are neighbours in tile order):
//   rounds    tiles 0 .. rounds G - 1 are taken whole, G at a time
//   the rest  the `rest` last tiles are cut at multiples of `len` = ceil(rest nblk / G) K blocks:
//             `full` = nblk / len aligned pieces per tile, one workgroup each (workgroup f rest + t takes piece f
//             of tile t), and a remainder of `rem` = nblk - full len blocks per tile; the remainders, laid end to
//             end, are cut into ranges of `len` blocks for the workgroups that are left.
// A tile that is multiplied in several parts is finished by the workgroup that arrives last.
struct Schedule {
  int tiles, nblk, m_groups, G, rounds, rest, len, full, rem;
};

struct Segment {
  int tile, kb0, kb1;  // K blocks kb0 .. kb1 - 1 of the tile; kb0 < 0: no more segments
};

[[maybe_unused]] __device__ __forceinline__ Segment schedule_segment(const Schedule &sc, int w, int idx) {
  Segment none = { 0, -1, -1 };
  if (idx < sc.rounds) {
    return { idx * sc.G + w, 0, sc.nblk };
  }
  if (sc.rest == 0) {
    return none;
  }
  const int i = idx - sc.rounds, base = sc.rounds * sc.G;
  if (w < sc.rest * sc.full) {
    if (i > 0) {
      return none;
    }
    const int f = w / sc.rest, t = w - f * sc.rest;
    return { base + t, f * sc.len, f * sc.len + sc.len };
  }
  if (sc.rem == 0) {
    return none;
  }
  const int j = w - sc.rest * sc.full;  // range [j len, (j + 1) len) of the remainders laid end to end
  const int x_end = min((j + 1) * sc.len, sc.rest * sc.rem);
  const int t = (j * sc.len) / sc.rem + i;
  const int x0 = max(j * sc.len, t * sc.rem), x1 = min(x_end, (t + 1) * sc.rem);
  if (x0 >= x1) {
    return none;
  }
  return { base + t, sc.full * sc.len + x0 - t * sc.rem, sc.full * sc.len + x1 - t * sc.rem };
}

constexpr int kMaxSegments = 128;  // per workgroup: rounds + the parts of the last, shared round

// ---- the instruction stream of one unit ---------------------------------------------------------------------------
// The vector ALU issue port is what bounds this kernel (one matrix or vector instruction per 4 cycles and SIMD), so
// the order of a unit's instructions is pinned (scheduling barriers): while unit u is accumulated (16 fmas) the two
// matrix instructions of unit u + 1 are issued between the halves, which keeps the matrix pipe (2 x 32 cycles per
// unit) and the port (18 x 4) busy together, and no matrix result is read sooner than 10 instructions after its issue.
#define HTPOPS_FMA8(A, S, C, o)                     \
  _Pragma("unroll") for (int r_ = o; r_ < o + 8; ++r_) { \
    A[r_] = __builtin_fmaf(S[r_], C[r_], A[r_]);    \
  }                                                 \
  __builtin_amdgcn_sched_barrier(0)
#define HTPOPS_MFMA_SUM(S, fa, fb)                                                                              \
  S = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa, fb, zero16, 2, 2, 0, scale_a, 0, scale_b);             \
  __builtin_amdgcn_sched_barrier(0)
#define HTPOPS_MFMA_SCALE(C, fa, fb)                                                                            \
  C = __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(v4h, __builtin_shufflevector(fa, fa, 6, 7)),       \
                                           __builtin_bit_cast(v4h, __builtin_shufflevector(fb, fb, 6, 7)), zero16, 0, 0, 0); \
  __builtin_amdgcn_sched_barrier(0)
// the two matrix instructions of a unit, operands fa (activation fragment) and fb (weight fragment)
#define HTPOPS_UNIT_MATRIX(S, C, fa, fb) \
  HTPOPS_MFMA_SUM(S, fa, fb);            \
  HTPOPS_MFMA_SCALE(C, fa, fb)
// accumulate a unit (from S_cur, C_cur) while issuing the matrix instructions of the next one
#define HTPOPS_UNIT(A, S_cur, C_cur, S_nxt, C_nxt, fa, fb) \
  HTPOPS_MFMA_SUM(S_nxt, fa, fb);                          \
  HTPOPS_FMA8(A, S_cur, C_cur, 0);                         \
  HTPOPS_MFMA_SCALE(C_nxt, fa, fb);                        \
  HTPOPS_FMA8(A, S_cur, C_cur, 8)

__global__ __launch_bounds__(kThreads) void gemm_fp6_panels_kernel(float *__restrict__ out, const uint8_t *__restrict__ a_panel,
                                                                   const uint8_t *__restrict__ b_panel, int m, int n,
                                                                   const Schedule sc, float *__restrict__ partials,
                                                                   unsigned *__restrict__ tickets) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __align__(16) uint8_t lds[kStages * kImgBytes];
  __shared__ int4                  lds_segments[kMaxSegments + 1];  // (tile, kb0, kb1, -): this workgroup's work, in order
  __shared__ unsigned              lds_ticket;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;  // position in the 2 x 4 wave grid
  const int c = lane & 31, h = lane >> 5;
  const int nblk = sc.nblk;
  // Workgroup ids go round-robin over the 8 XCDs (each with its own L2): neighbours in the schedule (tiles of one
  // column group) are given to one XCD.
  const int w = sc.G % 8 == 0 ? (blockIdx.x & 7) * (sc.G / 8) + (blockIdx.x >> 3) : blockIdx.x;

  if (tid <= kMaxSegments) {
    const Segment sg = tid < kMaxSegments ? schedule_segment(sc, w, tid) : Segment{ 0, -1, -1 };
    lds_segments[tid] = make_int4(sg.tile, sg.kb0, sg.kb1, 0);
  }
  __syncthreads();
  // walks the segments K block by K block (scalar registers)
  struct Walker {
    int idx, tile, kb, kb1;
  };
  auto walker_load = [&](Walker &wk, int idx) {
    const int4 e = lds_segments[idx];
    wk.idx = idx, wk.tile = __builtin_amdgcn_readfirstlane(e.x), wk.kb = __builtin_amdgcn_readfirstlane(e.y);
    wk.kb1 = __builtin_amdgcn_readfirstlane(e.z);
  };
  Walker dma, cur;
  walker_load(dma, 0);
  if (dma.kb < 0) {
    return;  // no work (whole workgroup)
  }
  cur = dma;

  // ---- DMA stream: step g goes to stage g % kStages as 16 KiB-sized pieces: wave w moves KiB w of the weight block
  // and KiB w of the activation block ----
  int            dma_g = 0;  // steps issued so far
  const uint8_t *dma_a = nullptr, *dma_b = nullptr;
  auto           dma_seek = [&]() {
    dma_b = b_panel + ((size_t) (dma.tile / sc.m_groups) * nblk + dma.kb) * kBBlock + wave * 1024 + lane * 16;
    dma_a = a_panel + ((size_t) (dma.tile % sc.m_groups) * nblk + dma.kb) * kABlock + wave * 1024 + lane * 16;
  };
  dma_seek();
  // (the DMA instruction is written out: the compiler makes every LDS read that follows a DMA it knows of wait for
  // ALL DMA in flight, which would undo the prefetch distance)
  auto dma_kib = [&](const uint8_t *src, uint32_t dst) {
    asm volatile("s_mov_b32 m0, %1\n s_nop 0\n global_load_lds_dwordx4 %0, off" ::"v"(src), "s"(dst) : "memory");
  };
  const uint32_t lds0 = (uint32_t) (uintptr_t) lds + wave * 1024;
  auto issue = [&](int stage) {
    const uint32_t img = lds0 + stage * kImgBytes;
    dma_kib(dma_b, img);
    dma_kib(dma_a, img + kImgA);
    ++dma_g;
    dma_a += kABlock, dma_b += kBBlock;
    if (++dma.kb == dma.kb1) {
      walker_load(dma, dma.idx + 1);
      if (dma.kb >= 0) {
        dma_seek();
      }
    }
  };
#pragma unroll
  for (int d = 0; d < kStages; ++d) {
    if (dma.kb >= 0) {
      issue(d);
    }
  }
  // Waits until this wave's pieces of step g + 1 have landed (those of later steps may stay in flight), then for
  // everybody's (a bare barrier: __syncthreads would wait for all pieces in flight).
  // s_waitcnt operand: vmcnt in bits 3:0 and 15:14, expcnt (7 = no wait) in 6:4, lgkmcnt in 11:8
  auto wait_next = [&](int g) {
    constexpr int kInFlight = 2 * (kStages - 2);
    if (dma_g - g - 2 >= kStages - 2) {  // steps issued after g + 1
      __builtin_amdgcn_s_waitcnt(0x0070 | (kInFlight & 15) | ((kInFlight >> 4) << 14));  // vmcnt(12) lgkmcnt(0)
    } else {
      __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): the end of the work
    }
    __builtin_amdgcn_s_barrier();
  };

  float acc[4][16];  // unit u = 2 i + j: rows 32 (2 wm + i) .., columns 32 (2 wn + j) ..
  auto  clear_acc = [&]() {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[u][r] = 0.0f;
      }
    }
  };
  clear_acc();
  const v16f zero16 = { 0 };
  // block scales of the FP6 instruction (E8M0 bytes): activations 2^3 (lo half) or 2^7 (hi half: x 16), weights 2^3
  const int scale_a = h ? 127 + 3 : 127 + 7, scale_b = 127 + 3;

  // operands of one K block in registers (codes in elements 0..5, scale operand in 6..7); they are read from LDS one
  // step ahead of their use
  struct Frags {
    v8i a[2], b[2];
  };
  // per-lane LDS offsets of the operands in the stage that is read next; they move on by one image per step
  int  ad_a = kImgA + (2 * wm) * kAFrag + lane * 16, ad_b = (2 * wn) * kBFrag + c * 16;
  int  rd_stage = 0;  // the stage those offsets point at
  auto lds_u4   = [&](int off) { return *reinterpret_cast<const v4i *>(lds + off); };
  auto load_frags = [&](Frags &f) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const v4i a0 = lds_u4(ad_a + i * kAFrag), a1 = lds_u4(ad_a + i * kAFrag + 1024);
      f.a[i] = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
      const v4i b0 = lds_u4(ad_b + i * kBFrag), b1 = lds_u4(ad_b + i * kBFrag + 512);
      f.b[i] = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7);
    }
    const int delta = rd_stage == kStages - 1 ? -(kStages - 1) * kImgBytes : kImgBytes;  // scalar
    rd_stage        = rd_stage == kStages - 1 ? 0 : rd_stage + 1;
    ad_a += delta, ad_b += delta;
  };

  // ---- K blocks kb0 .. kb1 - 1 of `tile` are in the accumulators ----
  // element (u = 2 i + j, r) of this lane: row = 32 (2 wm + i) + 8 (r / 4) + 4 h + r % 4, column = 32 (2 wn + j) + c
  auto finish_segment = [&](int tile, int kb0, int kb1) {
    const int mg = tile % sc.m_groups, ng = tile / sc.m_groups;
    bool      store = kb0 == 0 && kb1 == nblk;
    if (!store) {
      // The tile is one of the `rest` last ones. Its parts, in K order: the aligned pieces 0 .. full - 1, then the
      // ranges of the remainder workgroups that overlap its remainder. Every part leaves its sums in the workspace
      // (slot t (full + 2) + part); the last to arrive adds them in K order. The stores and loads are device-scope
      // atomics (written through to / read from the level all XCDs share) and the ticket is taken only after the
      // stores are acknowledged.
      const int t = tile - sc.rounds * sc.G;
      int       parts = sc.full, part = kb0 / sc.len;
      if (sc.rem > 0) {
        const int j_first = (t * sc.rem) / sc.len, j_last = ((t + 1) * sc.rem - 1) / sc.len;
        parts += j_last - j_first + 1;
        if (kb0 >= sc.full * sc.len) {
          part = sc.full + (w - sc.rest * sc.full) - j_first;
        }
      }
      // a part in the workspace: [wave 8][q 16][lane 64] x 16 bytes, q = 4 u + r / 4
      typedef float v4f __attribute__((ext_vector_type(4)));
      const float *slots = partials + (size_t) t * (sc.full + 2) * kPartialFloats + (size_t) wave * 4096 + lane * 4;
      {
        const float *mine = slots + (size_t) part * kPartialFloats;
#pragma unroll
        for (int q = 0; q < 16; ++q) {
          const v4f v = { acc[q >> 2][4 * (q & 3)], acc[q >> 2][4 * (q & 3) + 1], acc[q >> 2][4 * (q & 3) + 2], acc[q >> 2][4 * (q & 3) + 3] };
          asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(mine + q * 256), "v"(v) : "memory");
        }
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (tid == 0) {
        lds_ticket = __hip_atomic_fetch_add(&tickets[t], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      __syncthreads();
      if (lds_ticket == (unsigned) (parts - 1)) {
        store = true;
        if (tid == 0) {
          __hip_atomic_store(&tickets[t], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // left zeroed for the next launch
        }
        // The parts are added in K order: this workgroup's from its registers, the others read back (8 KiB per wave
        // in flight at once: the parts come from memory, not from this XCD's L2); units 0-1, then units 2-3.
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          float tot[2][16];
          for (int p = 0; p < parts; ++p) {
            if (p == part) {
#pragma unroll
              for (int u = 0; u < 2; ++u) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                  tot[u][r] = p == 0 ? acc[2 * half + u][r] : tot[u][r] + acc[2 * half + u][r];
                }
              }
              continue;
            }
            const float *theirs = slots + (size_t) p * kPartialFloats + half * 2048;
            v4f          v[8];
            asm volatile(
                "global_load_dwordx4 %0, %8, off sc1\n global_load_dwordx4 %1, %8, off offset:1024 sc1\n"
                "global_load_dwordx4 %2, %8, off offset:2048 sc1\n global_load_dwordx4 %3, %8, off offset:3072 sc1\n"
                "global_load_dwordx4 %4, %9, off sc1\n global_load_dwordx4 %5, %9, off offset:1024 sc1\n"
                "global_load_dwordx4 %6, %9, off offset:2048 sc1\n global_load_dwordx4 %7, %9, off offset:3072 sc1\n"
                "s_waitcnt vmcnt(0)"
                : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7])
                : "v"(theirs), "v"(theirs + 1024)
                : "memory");
#pragma unroll
            for (int q = 0; q < 8; ++q) {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                float &a = tot[q >> 2][4 * (q & 3) + e];
                a        = p == 0 ? v[q][e] : a + v[q][e];
              }
            }
          }
#pragma unroll
          for (int u = 0; u < 2; ++u) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              acc[2 * half + u][r] = tot[u][r];
            }
          }
        }
      }
    }
    if (store) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int col = ng * kTileN + (2 * wn + (u & 1)) * 32 + c;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = mg * kTileM + (2 * wm + (u >> 1)) * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
          if (row < m && col < n) {
            out[(size_t) row * n + col] = acc[u][r];
          }
        }
      }
    }
    clear_acc();
  };

  // ---- main loop over the steps of this workgroup ----
  Frags f0, f1;
  v16f  s_a, s_b, c_a, c_b;  // block sums and scale products of the unit being accumulated / the next one
  int   seg_kb0 = cur.kb, g = 0, stage = 0;  // steps done, stage of step g
  __builtin_amdgcn_s_waitcnt(0x0070);
  __builtin_amdgcn_s_barrier();  // (the first steps have landed: all of them, for simplicity)
  load_frags(f0);
  HTPOPS_UNIT_MATRIX(s_a, c_a, f0.a[0], f0.b[0]);
  // One K block: `now` holds step g (and the matrix results of its first unit are under way); step g + 1 is read
  // into `next` while `now` is multiplied. Finishes the segment when the step ends one; false after the last step.
  auto step = [&](Frags &now, Frags &next) {
    if (dma_g > g + 1) {  // there is a step g + 1
      wait_next(g);  // it has landed for everybody, and everybody holds step g in registers ...
      if (dma.kb >= 0) {
        issue(stage);  // ... so its stage can be refilled
      }
    }
    load_frags(next);  // unconditional (after the last step it reads bytes that are never used)
    __builtin_amdgcn_sched_barrier(0);
    HTPOPS_UNIT(acc[0], s_a, c_a, s_b, c_b, now.a[0], now.b[1]);
    HTPOPS_UNIT(acc[1], s_b, c_b, s_a, c_a, now.a[1], now.b[0]);
    HTPOPS_UNIT(acc[2], s_a, c_a, s_b, c_b, now.a[1], now.b[1]);
    HTPOPS_UNIT(acc[3], s_b, c_b, s_a, c_a, next.a[0], next.b[0]);
    stage = stage == kStages - 1 ? 0 : stage + 1;
    ++g;
    if (++cur.kb == cur.kb1) {
      const bool shared = seg_kb0 != 0 || cur.kb1 != nblk;
      finish_segment(cur.tile, seg_kb0, cur.kb1);
      walker_load(cur, cur.idx + 1);
      seg_kb0 = cur.kb;
      if (shared && cur.kb >= 0) {
        // The exchange of a shared tile needs registers: the operands of the next step are read again instead of
        // being kept (their stage has not been refilled yet).
        const int back = rd_stage == 0 ? (kStages - 1) * kImgBytes : -kImgBytes;
        rd_stage       = rd_stage == 0 ? kStages - 1 : rd_stage - 1;
        ad_a += back, ad_b += back;
        load_frags(next);
        HTPOPS_UNIT_MATRIX(s_a, c_a, next.a[0], next.b[0]);
      }
    }
    return cur.kb >= 0;
  };
  while (step(f0, f1) && step(f1, f0)) {
  }
#endif
}

// number of workgroups of the matmul: one per compute unit
int gemm_fp6_workgroups() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
      n = 256;
    }
    return env_int("HTPOPS_GEMM_WORKGROUPS", n);
  }();
  return cus;
}

}  // namespace

size_t gemm_fp6_weight_panel_bytes(int k, int n) {
  return (size_t) ((n + kTileN - 1) / kTileN) * (size_t) (k / 32) * kBBlock;
}

size_t gemm_fp6_act_panel_bytes(int m, int k) {
  return (size_t) ((m + kTileM - 1) / kTileM) * (size_t) (k / 32) * kABlock;
}

size_t gemm_fp6_workspace_bytes() {
  // a tile of the last, shared round has at most full + 2 parts, and rest (full + 2) <= 3 G
  return (size_t) 3 * gemm_fp6_workgroups() * kPartialFloats * sizeof(float);
}

bool gemm_fp6_fills_device(int m, int n) {
  return (size_t) ((m + kTileM - 1) / kTileM) * (size_t) ((n + kTileN - 1) / kTileN) >= (size_t) gemm_fp6_workgroups();
}

hipError_t launch_q4_0_to_fp6_panel(hipStream_t stream, void *dst, const void *weight, int k, int n) {
  if (k % 32 != 0 || n <= 0 || (reinterpret_cast<uintptr_t>(weight) & 1) != 0) {
    return hipErrorInvalidValue;
  }
  const int    nblk  = k / 32;
  const size_t total = (size_t) ((n + kTileN - 1) / kTileN) * nblk * 256;
  hipLaunchKernelGGL(q4_0_to_fp6_panel_kernel, dim3((unsigned) ((total + 255) / 256)), dim3(256), 0, stream,
                     static_cast<uint8_t *>(dst), static_cast<const uint16_t *>(weight), n, nblk, total);
  return hipGetLastError();
}

hipError_t launch_gemm_fp6_panels(hipStream_t stream, float *out, const void *act_q8_0, const void *weight_panel, int m,
                                  int k, int n, void *act_panel, void *workspace, unsigned *tickets, int ticket_slots) {
  const int nblk = k / 32, m_groups = (m + kTileM - 1) / kTileM, n_groups = (n + kTileN - 1) / kTileN;
  if (k % 32 != 0 || m <= 0 || n <= 0 || (size_t) m_groups * n_groups * nblk > (size_t) 1 << 30) {
    return hipErrorInvalidValue;
  }
  hipLaunchKernelGGL(q8_0_to_fp6_panel_kernel, dim3((unsigned) (m_groups * 4), (unsigned) ((nblk + 7) / 8)), dim3(256), 0, stream,
                     static_cast<uint8_t *>(act_panel), static_cast<const uint16_t *>(act_q8_0), m, nblk);
  if (hipError_t e = hipGetLastError(); e != hipSuccess) {
    return e;
  }
  Schedule sc;
  sc.tiles = m_groups * n_groups, sc.nblk = nblk, sc.m_groups = m_groups;
  sc.G      = gemm_fp6_workgroups();
  sc.rounds = sc.tiles / sc.G;
  sc.rest   = sc.tiles - sc.rounds * sc.G;
  sc.len = sc.full = sc.rem = 0;
  if (sc.rest > 0) {
    // no part shorter than 16 K blocks (or the whole K range): a tile of 64 parts would take longer to add up
    // than to multiply
    sc.len  = max((int) (((size_t) sc.rest * nblk + sc.G - 1) / sc.G), min(nblk, 16));
    sc.full = nblk / sc.len;
    sc.rem  = nblk - sc.full * sc.len;
    // no sliver remainders either: a workgroup that collects remainders takes one part from each tile it touches
    while (sc.rem != 0 && sc.rem < max(8, sc.len / 16) && sc.len < nblk) {
      ++sc.len;
      sc.full = nblk / sc.len;
      sc.rem  = nblk - sc.full * sc.len;
    }
  }
  if (sc.G > ticket_slots || sc.rounds + 24 > kMaxSegments) {
    return hipErrorInvalidValue;
  }
  hipLaunchKernelGGL(gemm_fp6_panels_kernel, dim3((unsigned) sc.G), dim3(kThreads), 0, stream, out,
                     static_cast<const uint8_t *>(act_panel), static_cast<const uint8_t *>(weight_panel), m, n, sc,
                     static_cast<float *>(workspace), tickets);
  return hipGetLastError();
}

}  // namespace htpops
