// Q4_0 x Q8_0 matmul for 2..8 activation rows, two blocks per matrix instruction:
// out[m][n] = sum over 32-wide blocks of (int dot of the block) * d_act * d_weight (reference: src/dsp/ops/mat_mul.c:572-640,
// block formats include/dsp/quants.h:8-14, ggml block_q4_0 / block_q8_0).
//
// With at most 8 activation rows, half of a 16 x 16 matrix-instruction result would be rows that do not exist. Here
// those rows carry the NEXT block instead: one v_mfma_i32_16x16x64_i8 multiplies
//     A (16 x 64):  rows 0..7  = the 8 activation rows' block b0 in k slots 0..31, zeros in 32..63
//                   rows 8..15 = zeros in 0..31, the same rows' block b1 in k slots 32..63
//     B (64 x 16):  column n   = weight row n's block b0 in k slots 0..31, its block b1 in 32..63
// so result rows 0..7 are the exact block sums of b0 and rows 8..15 those of b1: every lane of the result is used, and
// a pair of blocks costs one integer product, one scale product and four multiply-adds per lane. The nibbles go in
// unsigned (0..15); the "- 8" of Q4_0 is the instruction's C operand, -8 x (sum of the activation block), from a table
// made once per workgroup. The scale products d_act x d_weight of the same 16 x 16 positions come from one
// v_mfma_f32_16x16x16_f16 with the fp16 scales in k slots 0 (b0) and 1 (b1): exact in fp32.
//
// Weights are repacked once per weight buffer (same size, cached by the caller) so that a lane's operand bytes are one
// 16-byte load per quad of blocks: for a tile of 16 rows and blocks 4 q .. 4 q + 3,
//   1024 B: lane (n, g)'s 16 bytes = nibble bytes 8 (g & 1) .. + 7 of block 4 q + (g >> 1), then of block 4 q + 2 + (g >> 1)
//    128 B: row n's 4 fp16 scales of those blocks
// A workgroup works on one tile at a time over the whole of K (its 8 waves take every eighth quad and add up through
// LDS): nothing is exchanged between workgroups. The activation rows come as they are (block_q8_0 rows) by
// global_load_lds DMA, one row per wave, into a row-major LDS image (row starts 16 bytes past a multiple of 128 apart:
// the 8 rows a wave reads at one offset lie in different banks); lanes whose k slots are zeros read a zeroed corner of
// LDS instead, so no operand needs a select. Bringing the rows in and making the tables is as much work as a tile
// itself, so a launch has only as many workgroups as the device holds at once, each of which keeps its image and walks
// several tiles of its member (tiles wg, wg + stride, ...), with the weights of the steps ahead (also the next tile's)
// always in flight. Members of a launch may differ in k (all seven matrices of a decoder layer in one launch); the
// longest rows decide the LDS size of all workgroups.
#include "device_utils.h"
#include "kernels.h"

#include <stdint.h>

#include <algorithm>

namespace htpops {

namespace {

typedef int      v4i __attribute__((ext_vector_type(4)));
typedef float    v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

constexpr int kBpWaves     = 8;                      // waves of a workgroup
constexpr int kBpThreads   = kBpWaves * kWave;
constexpr int kBpRows      = 16;                     // weight rows per tile
constexpr int kBpActRows   = 8;                      // activation rows of the image
constexpr int kBpQuadBytes = 64 * 16 + kBpRows * 8;  // 1152 = 16 rows x 4 blocks x 18 B
constexpr int kBpZeroBytes = 64;                     // the zeroed corner (a lane reads up to 28 bytes of it)
constexpr size_t kBpLdsLimit = 160 * 1024;

// ---- repack: one thread per (tile, quad, lane) writes its 16 nibble bytes; lanes 0..15 also write the scales ----
__global__ __launch_bounds__(256) void q4_0_to_block_pairs_kernel(uint8_t *__restrict__ dst, const uint8_t *__restrict__ src,
                                                                 int nblk, int n) {
  const int    nquads = nblk / 4;
  const size_t item   = (size_t) blockIdx.x * 256 + threadIdx.x;  // (tile * nquads + quad) * 64 + lane
  const size_t total  = (size_t) (n / kBpRows) * nquads * 64;
  if (item >= total) {
    return;
  }
  const int    lane = (int) (item & 63), nl = lane & 15, g = lane >> 4;
  const size_t tq   = item >> 6;
  const int    quad = (int) (tq % nquads);
  const size_t tile = tq / nquads;
  const uint8_t *row = src + ((size_t) (tile * kBpRows + nl) * nblk + 4 * (size_t) quad) * 18;
  uint8_t       *out = dst + tq * kBpQuadBytes;
  uint32_t       w[4];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const uint8_t *q = row + (2 * p + (g >> 1)) * 18 + 2 + 8 * (g & 1);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      w[2 * p + h] = (uint32_t) q[4 * h] | ((uint32_t) q[4 * h + 1] << 8) | ((uint32_t) q[4 * h + 2] << 16) |
                     ((uint32_t) q[4 * h + 3] << 24);
    }
  }
  *reinterpret_cast<uint4 *>(out + lane * 16) = make_uint4(w[0], w[1], w[2], w[3]);
  if (g == 0) {
    uint16_t s[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      s[j] = (uint16_t) (row[j * 18] | (row[j * 18 + 1] << 8));
    }
    *reinterpret_cast<uint2 *>(out + 1024 + nl * 8) =
      make_uint2((uint32_t) s[0] | ((uint32_t) s[1] << 16), (uint32_t) s[2] | ((uint32_t) s[3] << 16));
  }
}

struct BlockPairsGroupArgs {
  const uint8_t *w[kGemvGroupMax];    // repacked weights
  const uint8_t *act[kGemvGroupMax];  // Q8_0 activation rows of each member (members may share them)
  float         *out[kGemvGroupMax];
  int            n[kGemvGroupMax];
  int            k[kGemvGroupMax];
  int            wg_begin[kGemvGroupMax + 1];  // member i owns workgroups wg_begin[i] .. wg_begin[i + 1] - 1
  int            count;
};

// LDS of a workgroup, in bytes from its start: the zeroed corner, the row image, the table of -8 x (block sums) as the
// integer instruction's C operand ([block][8 rows] int32) and the table of scale operands ([pair of blocks][8 rows]
// dwords: the even block's fp16 scale in the low half-word, the odd block's in the high one; result rows 0..7 keep the
// low half, rows 8..15 the high half).
struct BpLayout {
  int row_stride, image, sums, scales, red, total;
};
__host__ __device__ inline BpLayout bp_layout(int nblk) {
  BpLayout l;
  // rows 16 bytes (4 banks) past a multiple of 128 bytes apart: the 8 rows a wave reads at one offset fall into
  // different banks (a row itself is a multiple of 16 bytes long)
  l.row_stride = (nblk * 34 + 127 - 16) / 128 * 128 + 16;
  l.image      = kBpZeroBytes;
  l.sums       = l.image + kBpActRows * l.row_stride;
  l.scales     = l.sums + nblk * kBpActRows * 4;
  l.red        = l.scales + (nblk / 2) * kBpActRows * 4;   // the waves' sums of a tile, two buffers
  l.total      = l.red + 2 * kBpWaves * 4 * 32 * 4;
  return l;
}

template <int DEPTH>  // steps whose weights are requested ahead
__global__ __launch_bounds__(kBpThreads) void matmul_block_pairs_kernel(BlockPairsGroupArgs grp, int m) {
  extern __shared__ __align__(16) uint8_t bp_lds[];
  int member = 0;
  while (member + 1 < grp.count && (int) blockIdx.x >= grp.wg_begin[member + 1]) {
    ++member;
  }
  const int n = grp.n[member], n_tiles = n / kBpRows;
  const int first_tile = (int) blockIdx.x - grp.wg_begin[member], tile_stride = grp.wg_begin[member + 1] - grp.wg_begin[member];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int nblk = grp.k[member] / 32, nquads = nblk / 4;
  const BpLayout L = bp_layout(nblk);
  const uint8_t *__restrict__ act = grp.act[member];
  float *__restrict__         out = grp.out[member];

  // ---- the activation rows, as they are, by DMA: wave w brings row w in pieces of 1 KiB, the last one shorter (rows
  // past m repeat row m - 1; their results are never stored). The instruction is written out so that the compiler
  // does not make every later LDS read wait for all loads in flight. ----
  const int      a_row = nblk * 34;  // bytes of an activation row, a multiple of 16
  const uint32_t lds0  = (uint32_t) (uintptr_t) bp_lds;
  {
    static_assert(kBpWaves == kBpActRows, "one row per wave");
    const int      row = wave;
    const uint8_t *src = act + (size_t) min(row, m - 1) * a_row;
    const uint32_t to  = lds0 + (uint32_t) (L.image + row * L.row_stride);
    for (int o = 0; o < a_row; o += 1024) {
      if (o + lane * 16 < a_row) {
        const uint8_t *p = src + o + lane * 16;
        asm volatile("s_mov_b32 m0, %1\n s_nop 0\n global_load_lds_dwordx4 %0, off" ::"v"(p), "s"(to + (uint32_t) o) : "memory");
      }
    }
  }
  if (tid < kBpZeroBytes / 4) {
    reinterpret_cast<uint32_t *>(bp_lds)[tid] = 0u;
  }
  // this wave's quads wave, wave + 8, ...: two at a time, the next two in flight behind them
  struct Quad {
    uint4 q;  // this lane's nibble bytes of the quad's two block pairs
    uint2 d;  // the 4 fp16 scales of this lane's weight row
  };
  // A wave's work is a sequence of steps: (tile, h) = its quads wave + 16 h and wave + 16 h + 8 of that tile, tile after
  // tile. The weights of a step are requested two steps ahead, across tile boundaries, so that the stream from memory
  // does not stop while a tile is computed or its sums are added up.
  const int steps = (nquads + 2 * kBpWaves - 1) / (2 * kBpWaves);  // per tile
  auto fetch = [&](Quad (&r)[2], int tile, int h) {
    // (a step past the workgroup's last tile re-reads its last tile, a quad past the end of K the last quad: never used)
    const uint8_t *tw = grp.w[member] + (size_t) min(tile, n_tiles - 1) * nquads * kBpQuadBytes;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int      q = min(wave + (2 * h + c) * kBpWaves, nquads - 1);
      const uint8_t *p = tw + (size_t) q * kBpQuadBytes;
      r[c].q = *reinterpret_cast<const uint4 *>(p + lane * 16);
      r[c].d = *reinterpret_cast<const uint2 *>(p + 1024 + r16 * 8);
      // keep the loads in program order everywhere: the compiler counts the loads that may still be in flight when a
      // register is used, and takes the worst order over all paths that reach the use
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto next_step = [&](int &tile, int &h) {
    if (++h == steps) {
      h = 0, tile += tile_stride;
    }
  };
  // DEPTH register sets take turns: a set is refilled with the step DEPTH ahead as soon as its step is computed
  Quad sets[DEPTH][2];
  int  tf = first_tile, hf = 0;  // the next step to request
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    fetch(sets[d], tf, hf);
    next_step(tf, hf);
  }
  // the DMA pieces of this wave have landed once only the 4 DEPTH weight loads issued after them are outstanding
  // (s_waitcnt operand: vmcnt in bits 3:0 and 15:14, expcnt (7 = no wait) in 6:4, lgkmcnt in 11:8)
  static_assert(4 * DEPTH < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0070 | ((4 * DEPTH) & 15) | (((4 * DEPTH) >> 4) << 14));
  __builtin_amdgcn_s_barrier();  // (bare barriers: __syncthreads would also wait for the weight loads)

  // ---- tables: -8 x block sum per (block, row) and the scale operand per (pair of blocks, result row) ----
  {
    int *sums = reinterpret_cast<int *>(bp_lds + L.sums);
    for (int i = tid; i < nblk * kBpActRows; i += kBpThreads) {
      const int      blk = i / kBpActRows, row = i % kBpActRows;
      const int      s   = blk * 34 + 2;  // the block's 32 int8 start here: 2 bytes off a dword in even blocks
      const uint8_t *p   = bp_lds + L.image + row * L.row_stride + (s & ~3);
      const bool     off = (s & 3) != 0;
      int            acc = 0;
#pragma unroll
      for (int d = 0; d < 9; ++d) {
        const uint32_t v    = reinterpret_cast<const uint32_t *>(p)[d];
        const uint32_t ones = d == 0 ? (off ? 0x01010000u : 0x01010101u) : d == 8 ? (off ? 0x00000101u : 0u) : 0x01010101u;
        acc                 = dot4_i8(v, ones, acc);
      }
      sums[i] = -8 * acc;
    }
    uint32_t *scl = reinterpret_cast<uint32_t *>(bp_lds + L.scales);
    for (int i = tid; i < (nblk / 2) * kBpActRows; i += kBpThreads) {
      const int      pair = i / kBpActRows, r = i % kBpActRows;
      const uint8_t *p    = bp_lds + L.image + r * L.row_stride + 2 * pair * 34;
      scl[i] = (uint32_t) *reinterpret_cast<const uint16_t *>(p) | ((uint32_t) *reinterpret_cast<const uint16_t *>(p + 34) << 16);
    }
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the tables are written; vmcnt untouched
  __builtin_amdgcn_s_barrier();

  // ---- per lane: where its operands of the wave's first pair of blocks lie, and how far apart successive pairs are ----
  // A operand (activations): lane (result row r16, k group g) holds k slots 16 g .. 16 g + 15. Rows 0..7 have data in
  // groups 0, 1 (block b0: bytes 8 g .. + 7 and 16 + 8 g .. + 7 of the row's block), rows 8..15 in groups 2, 3 (block
  // b1); everything else is zeros, read from the zeroed corner with a stride of 0. Even blocks start 2 bytes off a
  // dword: three dwords and two funnel shifts per 8 bytes, with the shift 0 for the aligned odd blocks.
  const bool upper = r16 >= 8, data = upper ? g >= 2 : g < 2;
  const int  pair0 = 2 * wave;                                  // first pair of blocks of this wave
  uint32_t   a_at   = data ? (uint32_t) (L.image + (r16 & 7) * L.row_stride + (upper ? 36 : 0) + 8 * (g & 1) + 68 * pair0) : 0u;
  const uint32_t a_step = data ? 68u : 0u;                      // bytes from a pair to the next
  const uint32_t shift  = (data && !upper) ? 2u : 0u;
  // C operand: rows 4 g + i of the result = rows 4 (g & 1) + i of block b0 + (g >> 1)
  uint32_t c_at = (uint32_t) (L.sums + ((2 * pair0 + (g >> 1)) * kBpActRows + 4 * (g & 1)) * 4);
  // scale operands: only k group 0 carries scales
  uint32_t       s_at   = g == 0 ? (uint32_t) (L.scales + (pair0 * kBpActRows + (r16 & 7)) * 4) : 0u;
  const uint32_t s_step = g == 0 ? (uint32_t) (kBpActRows * 4) : 0u;
  const uint32_t s_mask = upper ? 0xffff0000u : 0x0000ffffu;
  const uint32_t d_mask = g == 0 ? 0xffffffffu : 0u;
  constexpr uint32_t kPairsPerQuadStride = 2 * kBpWaves;        // pairs between a wave's successive quads, minus the two it did

  const uint32_t a_at0 = a_at, c_at0 = c_at, s_at0 = s_at;
  v4f acc;
  auto pair = [&](uint32_t w0, uint32_t w1, uint32_t dw) {
    // activations: bytes [x, x + 8) and [x + 16, x + 24) of the row, x = a_at + shift
    const uint32_t *ap = reinterpret_cast<const uint32_t *>(bp_lds + a_at);
    const uint32_t  t0 = ap[0], t1 = ap[1], t2 = ap[2], t4 = ap[4], t5 = ap[5], t6 = ap[6];
    v4i a;
    a[0] = (int) __builtin_amdgcn_alignbyte(t1, t0, shift);
    a[1] = (int) __builtin_amdgcn_alignbyte(t2, t1, shift);
    a[2] = (int) __builtin_amdgcn_alignbyte(t5, t4, shift);
    a[3] = (int) __builtin_amdgcn_alignbyte(t6, t5, shift);
    const v4i c = *reinterpret_cast<const v4i *>(bp_lds + c_at);
    const uint32_t sa = *reinterpret_cast<const uint32_t *>(bp_lds + s_at) & s_mask;
    // weights: nibbles as they are (0..15), low nibbles = elements e .. e + 7, high nibbles = elements 16 + e ..
    v4i b;
    b[0] = (int) (w0 & 0x0f0f0f0fu), b[1] = (int) (w1 & 0x0f0f0f0fu);
    b[2] = (int) ((w0 >> 4) & 0x0f0f0f0fu), b[3] = (int) ((w1 >> 4) & 0x0f0f0f0fu);
    const v4i sums = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
    const v4f zero = { 0.0f, 0.0f, 0.0f, 0.0f };
    const v4f prod = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(v4h, make_uint2(sa, 0u)),
                                                           __builtin_bit_cast(v4h, make_uint2(dw & d_mask, 0u)), zero, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc[i] = __builtin_fmaf((float) sums[i], prod[i], acc[i]);
    }
    a_at += a_step, c_at += 2 * kBpActRows * 4, s_at += s_step;
  };
  auto skip_to_next_quad = [&]() {  // from behind a quad's second pair to the first pair of the wave's next quad
    a_at += a_step * (kPairsPerQuadStride - 2), c_at += (kPairsPerQuadStride - 2) * 2 * kBpActRows * 4,
      s_at += s_step * (kPairsPerQuadStride - 2);
  };
  // ---- the tiles of this workgroup; the first two steps' weights are already on their way ----
  int buf = 0, tile = first_tile, h = 0;
  acc = (v4f){ 0.0f, 0.0f, 0.0f, 0.0f };
  auto finish_tile = [&]() {
    // result rows 8..15 (k groups 2, 3) hold the odd blocks' share of the same outputs as rows 0..7 of groups 0, 1
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc[i] += __shfl_xor(acc[i], 32, kWave);
    }
    // add the waves of the tile in wave order. Two buffers take turns: a tile's sums are read behind its barrier, and
    // the buffer is written again two tiles later, behind the barrier of the tile in between.
    float *red = reinterpret_cast<float *>(bp_lds + L.red) + buf * (kBpWaves * 4 * 32);
    if (lane < 32) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        red[(wave * 4 + i) * 32 + lane] = acc[i];
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the sums are written; the weight loads stay in flight
    __builtin_amdgcn_s_barrier();
    if (tid < 4 * 32) {
      const int i = tid >> 5, l = tid & 31, row = 4 * (l >> 4) + i;
      float     v = 0.0f;
#pragma unroll
      for (int w = 0; w < kBpWaves; ++w) {
        v += red[(w * 4 + i) * 32 + l];
      }
      if (row < m) {
        out[(size_t) row * n + (size_t) tile * kBpRows + (l & 15)] = v;
      }
    }
    buf ^= 1;
    acc  = (v4f){ 0.0f, 0.0f, 0.0f, 0.0f };
    a_at = a_at0, c_at = c_at0, s_at = s_at0;
  };
  auto step = [&](Quad (&r)[2]) {
#pragma unroll
    for (int cidx = 0; cidx < 2; ++cidx) {
      if (wave + (2 * h + cidx) * kBpWaves < nquads && tile < n_tiles) {
        pair(r[cidx].q.x, r[cidx].q.y, r[cidx].d.x);
        pair(r[cidx].q.z, r[cidx].q.w, r[cidx].d.y);
        skip_to_next_quad();
      }
    }
    fetch(r, tf, hf);
    next_step(tf, hf);
    if (++h == steps && tile < n_tiles) {
      finish_tile();
      h = 0, tile += tile_stride;
    }
  };
  // Always the loads of all DEPTH steps, with no way out between them: the compiler's count of loads in flight at the
  // top of the loop is the worst over every path it sees, and a path that skips a step's loads would make it wait
  // for loads just issued. When the tiles end before the last step, the steps left compute nothing; their loads
  // (of the last tile again, valid addresses) are never used.
#pragma unroll 1
  while (tile < n_tiles) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      step(sets[d]);
    }
  }
}

// How far ahead the weights are requested: two steps (4.6 KB per wave) where three workgroups share a compute unit;
// three where the rows are so long that only one workgroup fits a unit's LDS (k = 11008: 105 KB). Measured on the
// seven matrices of a Llama-7B layer in one launch (8 rows): depth 2 28.3 us, 3 27.2 us, 5 28.1 us, 6 29.5 us; 16 waves
// per workgroup instead of 8 (each tile split 16 ways) 28.3 us.
constexpr int kBpDepthShared = 2, kBpDepthAlone = 3;
bool bp_alone(int nblk) {
  return (size_t) bp_layout(nblk).total * 2 > kBpLdsLimit;
}

}  // namespace

bool matmul_block_pairs_fits(int n, int m, int k, WeightType wt) {
  // k % 256: activation rows (34 B per 32 elements) are whole 16-byte pieces, weight rows whole quads of blocks
  return wt == kQ4_0 && m >= 2 && m <= kBpActRows && k > 0 && k % 256 == 0 && n > 0 && n % kBpRows == 0 &&
         (size_t) bp_layout(k / 32).total <= kBpLdsLimit;
}

hipError_t launch_weights_to_block_pairs(hipStream_t stream, void *dst, const void *weight, int k, int n) {
  if (k % 128 != 0 || n % kBpRows != 0) {
    return hipErrorNotSupported;
  }
  const size_t items = (size_t) (n / kBpRows) * (size_t) (k / 128) * 64;
  hipLaunchKernelGGL(q4_0_to_block_pairs_kernel, dim3((unsigned) ((items + 255) / 256)), dim3(256), 0, stream,
                     static_cast<uint8_t *>(dst), static_cast<const uint8_t *>(weight), k / 32, n);
  return hipGetLastError();
}

hipError_t launch_matmul_block_pairs_group(hipStream_t stream, int count, float *const *outs, const void *const *acts,
                                           const void *const *pair_order_weights, const int *ns, int m, const int *ks) {
  if (count < 1 || count > kGemvGroupMax) {
    return hipErrorNotSupported;
  }
  BlockPairsGroupArgs grp = {};
  int                 k_max = 0;
  for (int i = 0; i < count; ++i) {
    if (!matmul_block_pairs_fits(ns[i], m, ks[i], kQ4_0) || (reinterpret_cast<uintptr_t>(pair_order_weights[i]) & 15) != 0 ||
        (reinterpret_cast<uintptr_t>(acts[i]) & 15) != 0) {
      return hipErrorNotSupported;
    }
    grp.w[i]   = static_cast<const uint8_t *>(pair_order_weights[i]);
    grp.act[i] = static_cast<const uint8_t *>(acts[i]);
    grp.out[i] = outs[i];
    grp.n[i]   = ns[i];
    grp.k[i]   = ks[i];
    k_max      = std::max(k_max, ks[i]);
  }
  // (the longest rows of the launch decide its LDS size and with it how many workgroups share a compute unit)
  const bool   alone = bp_alone(k_max / 32);
  const size_t lds   = (size_t) bp_layout(k_max / 32).total;
  const void  *fn    = alone ? reinterpret_cast<const void *>(matmul_block_pairs_kernel<kBpDepthAlone>) :
                               reinterpret_cast<const void *>(matmul_block_pairs_kernel<kBpDepthShared>);
  static bool attr_set[2] = {};  // more than the default 64 KiB of dynamic LDS for long rows
  if (!attr_set[alone]) {
    const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int) kBpLdsLimit);
    if (e != hipSuccess) {
      return e;
    }
    attr_set[alone] = true;
  }
  // As many workgroups as the device holds at once (LDS decides: three of 43 KB for k = 4096, one of 113 KB for
  // k = 11008, on each of 256 compute units), shared out among the members by their weight bytes; a member's
  // workgroups take its tiles in turn.
  const int  per_cu   = alone ? 1 : (int) std::min<size_t>(3, kBpLdsLimit / lds);
  const long resident = 256L * per_cu;
  long       tiles    = 0;
  for (int i = 0; i < count; ++i) {
    tiles += ns[i] / kBpRows;
  }
  grp.count = count;
  long wgs[kGemvGroupMax];
  if (tiles <= resident) {
    for (int i = 0; i < count; ++i) {
      wgs[i] = ns[i] / kBpRows;
    }
  } else {
    // The launch ends with its busiest workgroup. A workgroup of member i that walks t tiles carries t k_i (weight
    // bytes, up to a factor): find the smallest such load T for which ceil(tiles_i / floor(T / k_i)) workgroups per
    // member fit the device, trying every load some member can produce (tiles-per-workgroup counts are small).
    auto needed = [&](double T, long *out) {
      long sum = 0;
      for (int i = 0; i < count; ++i) {
        const long per = (long) (T / ks[i]);
        if (per < 1) {
          return -1L;
        }
        const long mine = ns[i] / kBpRows;
        out[i] = (mine + per - 1) / per;
        sum += out[i];
      }
      return sum;
    };
    double best_T = 0.0;
    for (int i = 0; i < count; ++i) {
      const long mine = ns[i] / kBpRows;
      for (long t = 1; t <= mine; ++t) {
        const double T = (double) t * ks[i];
        if (best_T > 0.0 && T >= best_T) {
          break;
        }
        long       tmp[kGemvGroupMax];
        const long sum = needed(T, tmp);
        if (sum > 0 && sum <= resident) {
          best_T = T;
          break;  // (larger t of this member only raise T)
        }
      }
    }
    if (best_T <= 0.0 || needed(best_T, wgs) < 0) {
      return hipErrorNotSupported;  // (more members than workgroups: cannot happen with at most 8 members)
    }
  }
  grp.wg_begin[0] = 0;
  for (int i = 0; i < count; ++i) {
    grp.wg_begin[i + 1] = grp.wg_begin[i] + (int) wgs[i];
  }
  const dim3 grid((unsigned) grp.wg_begin[count]), block(kBpThreads);
  if (alone) {
    hipLaunchKernelGGL((matmul_block_pairs_kernel<kBpDepthAlone>), grid, block, lds, stream, grp, m);
  } else {
    hipLaunchKernelGGL((matmul_block_pairs_kernel<kBpDepthShared>), grid, block, lds, stream, grp, m);
  }
  return hipGetLastError();
}

}  // namespace htpops
