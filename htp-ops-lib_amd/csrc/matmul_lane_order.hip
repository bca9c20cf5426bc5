// Q4_0 x Q8_0 matmul for 2..16 activation rows over weights repacked once into the order the matrix core wants:
// out[m][n] = sum over 32-wide blocks of (int dot of the block) * d_act * d_weight (reference: src/dsp/ops/mat_mul.c:572-640,
// block formats include/dsp/quants.h:8-14, ggml block_q4_0 / block_q8_0).
//
// The decode kernel streams Q4_0 rows as they are because one lane can own a whole block. With several activation
// rows the block dots belong on v_mfma_i32_16x16x32_i8 (activation rows x 16 weight rows x 32 k), whose weight operand
// wants, per lane (row n = lane % 16, group g = lane / 16), the 4 nibble bytes 4 g .. 4 g + 3 of row n's block: 4-byte
// pickings from 16 rows, which no wide load delivers from the row layout. So the weights are repacked once per weight
// buffer (same size, cached by the caller): for a tile of 16 rows and a quad of 4 consecutive blocks,
//   1024 B: lane l's 16 bytes = its 4 nibble bytes of blocks 4 q .. 4 q + 3
//    128 B: row n's 4 fp16 scales of those blocks
// so that a wave fetches a quad with one 16-byte and one 8-byte load per lane, fully coalesced, straight into the
// registers the MFMA reads. A workgroup owns one tile over the whole of K (its 8 waves take every eighth quad and add
// up through LDS), so nothing is exchanged between workgroups and a 4096-row matrix still gives 256 of them.
//
// Every workgroup needs all activation rows, as many bytes as its weights. They come as they are (block_q8_0 rows)
// by global_load_lds DMA in 16-byte pieces - no registers, no vector ALU work, in flight together with the first weight
// loads - into LDS with the 8 (or, for m > 8, 16) rows interleaved piece by piece (the rows a wave reads at one byte
// offset lie in different bank groups); the lanes pick their operand bytes out of that image (a funnel shift where a block starts
// 2 bytes off a dword) and the block scales out of a float table made once after the DMA has landed. Measured: laying
// the rows out in operand order with the vector ALU instead cost as much as streaming the weights.
#include "device_utils.h"
#include "kernels.h"

#include <stdint.h>

namespace htpops {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kLoThreads  = 512;
constexpr int kLoWaves    = kLoThreads / kWave;
constexpr int kLoRows     = 16;                       // weight rows per tile
constexpr int kLoMaxActRows = 16;                     // the matrix instruction's other side: 16 activation rows
constexpr int kLoQuadBytes = 64 * 16 + kLoRows * 8;   // 1152 = 16 rows x 4 blocks x 18 B (Q4_0)
constexpr int kLoQuadBytesQ8 = 64 * 32 + kLoRows * 8; // 2176 = 16 rows x 4 blocks x 34 B (Q8_0)
constexpr int quad_bytes(int wt) { return wt == kQ4_0 ? kLoQuadBytes : kLoQuadBytesQ8; }
constexpr size_t kLoLdsLimit = 160 * 1024;

// ---- repack: one thread per (tile, quad, lane) writes its 16 nibble bytes; lanes 0..15 also write the scales ----
__global__ __launch_bounds__(256) void q4_0_to_lane_order_kernel(uint8_t *__restrict__ dst,
                                                                const uint8_t *__restrict__ src, int nblk, int n) {
  const int    nquads = nblk / 4;
  const size_t item   = (size_t) blockIdx.x * 256 + threadIdx.x;  // (tile * nquads + quad) * 64 + lane
  const size_t total  = (size_t) (n / kLoRows) * nquads * 64;
  if (item >= total) {
    return;
  }
  const int    lane = (int) (item & 63), nl = lane & 15, g = lane >> 4;
  const size_t tq   = item >> 6;
  const int    quad = (int) (tq % nquads);
  const size_t tile = tq / nquads;
  const uint8_t *row = src + ((size_t) (tile * kLoRows + nl) * nblk + 4 * (size_t) quad) * 18;
  uint8_t       *out = dst + tq * kLoQuadBytes;
  uint32_t       w[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint8_t *q = row + j * 18 + 2 + 4 * g;
    w[j] = (uint32_t) q[0] | ((uint32_t) q[1] << 8) | ((uint32_t) q[2] << 16) | ((uint32_t) q[3] << 24);
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

// Q8_0: the same tile and quad, 2048 B: lane l's 32 bytes = for each of the 4 blocks its 8 int8 operand bytes, elements
// {4 g .. 4 g + 3, 16 + 4 g .. 16 + 4 g + 3} -- the element order the Q4_0 nibbles unpack to, so that the activation
// operand is formed the same way for both weight types; then the 128 B of scales.
__global__ __launch_bounds__(256) void q8_0_to_lane_order_kernel(uint8_t *__restrict__ dst,
                                                                const uint8_t *__restrict__ src, int nblk, int n) {
  const int    nquads = nblk / 4;
  const size_t item   = (size_t) blockIdx.x * 256 + threadIdx.x;  // (tile * nquads + quad) * 64 + lane
  const size_t total  = (size_t) (n / kLoRows) * nquads * 64;
  if (item >= total) {
    return;
  }
  const int    lane = (int) (item & 63), nl = lane & 15, g = lane >> 4;
  const size_t tq   = item >> 6;
  const int    quad = (int) (tq % nquads);
  const size_t tile = tq / nquads;
  const uint8_t *row = src + ((size_t) (tile * kLoRows + nl) * nblk + 4 * (size_t) quad) * 34;
  uint8_t       *out = dst + tq * kLoQuadBytesQ8;
  uint32_t       w[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint8_t *q = row + j * 34 + 2;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const uint8_t *e = q + 16 * half + 4 * g;
      w[2 * j + half] = (uint32_t) e[0] | ((uint32_t) e[1] << 8) | ((uint32_t) e[2] << 16) | ((uint32_t) e[3] << 24);
    }
  }
  *reinterpret_cast<uint4 *>(out + lane * 32)      = make_uint4(w[0], w[1], w[2], w[3]);
  *reinterpret_cast<uint4 *>(out + lane * 32 + 16) = make_uint4(w[4], w[5], w[6], w[7]);
  if (g == 0) {
    uint16_t s[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      s[j] = (uint16_t) (row[j * 34] | (row[j * 34 + 1] << 8));
    }
    *reinterpret_cast<uint2 *>(out + 2048 + nl * 8) =
      make_uint2((uint32_t) s[0] | ((uint32_t) s[1] << 16), (uint32_t) s[2] | ((uint32_t) s[3] << 16));
  }
}

struct LaneOrderGroupArgs {
  const uint8_t *w[kGemvGroupMax];    // repacked weights
  const uint8_t *act[kGemvGroupMax];  // Q8_0 activation rows of each member (members may share them)
  float         *out[kGemvGroupMax];
  int            n[kGemvGroupMax];
};

template <int WT>
struct QuadRegs {
  uint4 q[WT == kQ4_0 ? 1 : 2];  // this lane's nibble bytes (Q4_0) or operand bytes (Q8_0) of the 4 blocks
  uint2 d;                       // the 4 fp16 scales of this lane's row
};

// ROWS: activation rows in the LDS panel, 8 (m <= 8: lanes 32..63 repeat rows 0..7 and their results are dropped) or 16
// TPW:  16-row weight tiles per workgroup, 1 (8 waves per tile) or 2 (4 waves per tile). The activation panel is as
//       many bytes as a tile's weights and every workgroup fetches it from L2, so two tiles per workgroup cut the
//       traffic into a CU by a quarter; used when that still leaves enough workgroups.
// WT:   weight type of the repacked copy; Q8_0 quads are twice the bytes, so half as many are fetched at a time
template <int ROWS, int TPW, int WT>
__global__ __launch_bounds__(kLoThreads) void matmul_lane_order_kernel(LaneOrderGroupArgs grp, int m, int k) {
  constexpr int kLoChunk    = WT == kQ4_0 ? 4 : 2;  // quads a wave fetches at a time
  constexpr int kQuadBytes  = quad_bytes(WT);
  constexpr int kLoads      = WT == kQ4_0 ? 2 : 3;  // load instructions per quad
  constexpr int kLoActRows  = ROWS;
  constexpr int kLoScaleBlk = ROWS * 4;  // bytes of the scale table per block (one float per row)
  extern __shared__ __align__(16) uint8_t lo_lds[];  // activation panel, later the waves' sums
  const int n = grp.n[blockIdx.y];
  if ((int) (blockIdx.x * kLoRows * TPW) >= n) {
    return;  // whole workgroup: this member has fewer rows than the widest one
  }
  constexpr int WQ = kLoWaves / TPW;  // waves that share a tile
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wph = wave % WQ, tw = wave / WQ;
  const int nl = lane & 15, g = lane >> 4;
  // a second tile past the end of an odd tile count repeats the last one (never stored)
  const int tile = min((int) blockIdx.x * TPW + tw, n / kLoRows - 1);
  const int nblk = k / 32, nquads = nblk / 4;
  const uint8_t *__restrict__ wt  = grp.w[blockIdx.y] + (size_t) tile * nquads * kQuadBytes;
  const uint8_t *__restrict__ act = grp.act[blockIdx.y];
  float *__restrict__         out = grp.out[blockIdx.y];

  auto fetch = [&](QuadRegs<WT> (&r)[kLoChunk], int q0) {  // quads q0, q0 + WQ, ... of this wave (clamped: extra ones unused)
#pragma unroll
    for (int c = 0; c < kLoChunk; ++c) {
      const int      q = min(q0 + c * WQ, nquads - 1);
      const uint8_t *p = wt + (size_t) q * kQuadBytes;
      if (WT == kQ4_0) {
        r[c].q[0] = *reinterpret_cast<const uint4 *>(p + lane * 16);
      } else {
        r[c].q[0]                = *reinterpret_cast<const uint4 *>(p + lane * 32);
        r[c].q[WT == kQ4_0 ? 0 : 1] = *reinterpret_cast<const uint4 *>(p + lane * 32 + 16);
      }
      r[c].d = *reinterpret_cast<const uint2 *>(p + (kQuadBytes - 128) + nl * 8);
    }
  };
  // ---- the activation rows, as they are, by DMA: piece pc of row r goes to piece slot pc * 8 + r. Rows past m repeat
  // row m - 1 (their results are never stored). The DMA instruction is written out so that the compiler does not make
  // every later LDS read wait for all loads in flight. ----
  const int      a_row    = nblk * 34;                 // bytes of an activation row, a multiple of 16
  const int      a_pieces = kLoActRows * (a_row / 16);
  const int      a_bytes  = (a_pieces * 16 + 1023) & ~1023;  // image size: whole DMA instructions
  const uint32_t lds0     = (uint32_t) (uintptr_t) lo_lds;
  for (int i = wave; i * kWave < a_pieces; i += kLoWaves) {
    const int      s   = min(i * kWave + lane, a_pieces - 1), row = min(s % kLoActRows, m - 1), pc = s / kLoActRows;
    const uint8_t *p   = act + (size_t) row * a_row + (size_t) pc * 16;
    const uint32_t to  = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t) i * kWave * 16);
    asm volatile("s_mov_b32 m0, %1\n s_nop 0\n global_load_lds_dwordx4 %0, off" ::"v"(p), "s"(to) : "memory");
  }
  QuadRegs<WT> cur[kLoChunk], nxt[kLoChunk];
  fetch(cur, wph);  // 2 kLoChunk loads, in flight behind the DMA
  // the DMA pieces of this wave have landed once only the weight loads issued after them are outstanding
  // (s_waitcnt operand: vmcnt in bits 3:0 and 15:14, expcnt (7 = no wait) in 6:4, lgkmcnt in 11:8)
  static_assert(kLoads * kLoChunk <= 15, "the wait below leaves exactly the weight loads in flight");
  __builtin_amdgcn_s_waitcnt(0x0070 | (kLoads * kLoChunk));
  __builtin_amdgcn_s_barrier();  // (bare barriers: __syncthreads would also wait for the weight loads)
  // block scales of all rows as floats: [block][row]
  float *s_tab = reinterpret_cast<float *>(lo_lds + a_bytes);
  for (int i = tid; i < nblk * kLoActRows; i += kLoThreads) {
    const int blk = i / kLoActRows, row = i % kLoActRows, o = blk * 34;
    s_tab[i]      = (float) *reinterpret_cast<const _Float16 *>(lo_lds + ((o >> 4) * kLoActRows + row) * 16 + (o & 15));
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the table is written; vmcnt untouched
  __builtin_amdgcn_s_barrier();

  // ---- this wave's quads, kLoChunk at a time, the next chunk in flight behind the current one ----
  // LDS byte offsets of this lane's operand dwords in its first quad (row nl % 8, elements {4 g .., 16 + 4 g ..} of
  // the quad's 4 blocks); the wave's next quad is 8 quads = 1088 B = 68 pieces of every row further on. Even blocks
  // of a quad start 2 bytes off a dword (34 b + 2 with b even): two dwords and a funnel shift; odd blocks are aligned.
  auto a_addr = [&](int o) { return ((o >> 4) * kLoActRows + (nl & (ROWS - 1))) * 16 + (o & 15); };
  int  a_off[4][4];  // [block of the quad][dword]: even blocks use 4, odd blocks 2
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int o = (4 * wph + j) * 34 + 4 * g;  // byte 4 g of the block's row segment (its scale is bytes 0..1)
    if (j % 2 == 0) {
      a_off[j][0] = a_addr(o), a_off[j][1] = a_addr(o + 4), a_off[j][2] = a_addr(o + 16), a_off[j][3] = a_addr(o + 20);
    } else {
      a_off[j][0] = a_addr(o + 2), a_off[j][1] = a_addr(o + 18), a_off[j][2] = 0, a_off[j][3] = 0;
    }
  }
  constexpr int kQuadStep  = WQ * 4 * 34 / 16 * kLoActRows * 16;  // WQ quads further on in the image
  constexpr int kScaleStep = WQ * 4 * kLoScaleBlk;                // and in the scale table
  static_assert(WQ * 4 * 34 % 16 == 0, "a wave's quads are whole pieces apart");
  const uint8_t *s_lane = lo_lds + a_bytes + 4 * wph * kLoScaleBlk + (g & (ROWS / 4 - 1)) * 16;  // scales of rows 4 g ..
  float          acc[4] = { 0.0f, 0.0f, 0.0f, 0.0f };  // rows 4 g + j, column nl (ROWS = 8, lanes with g >= 2: unused rows)
  // nibble -> int8 minus 8 without carries between bytes: (q + 0x78) ^ 0x80 per byte
  auto lo = [](uint32_t q) { return ((q & 0x0f0f0f0fu) + 0x78787878u) ^ 0x80808080u; };
  auto hi = [](uint32_t q) { return (((q >> 4) & 0x0f0f0f0fu) + 0x78787878u) ^ 0x80808080u; };
  for (int q0 = wph; q0 < nquads; q0 += kLoChunk * WQ) {
    const bool more = q0 + kLoChunk * WQ < nquads;
    if (more) {
      fetch(nxt, q0 + kLoChunk * WQ);
    }
#pragma unroll
    for (int c = 0; c < kLoChunk; ++c) {
      const int quad = q0 + c * WQ;
      if (quad < nquads) {
        // Q4_0: wq[j] = the nibble dword of block j; Q8_0: wq[2 j], wq[2 j + 1] = the operand dwords of block j
        uint32_t wq[8];
        wq[0] = cur[c].q[0].x, wq[1] = cur[c].q[0].y, wq[2] = cur[c].q[0].z, wq[3] = cur[c].q[0].w;
        if (WT != kQ4_0) {
          const uint4 q1 = cur[c].q[WT == kQ4_0 ? 0 : 1];
          wq[4] = q1.x, wq[5] = q1.y, wq[6] = q1.z, wq[7] = q1.w;
        }
        union {
          uint2    u;
          _Float16 h[4];
        } sc;
        sc.u = cur[c].d;
        const int      it  = (quad - wph) / WQ;  // this quad is the wave's it-th
        const uint8_t *img = lo_lds + (size_t) it * kQuadStep;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t e0, e1;  // elements 4 g .. 4 g + 3 and 16 + 4 g .. 16 + 4 g + 3 of this lane's activation row
          if (j % 2 == 0) {
            e0 = __builtin_amdgcn_alignbyte(*reinterpret_cast<const uint32_t *>(img + a_off[j][1]),
                                            *reinterpret_cast<const uint32_t *>(img + a_off[j][0]), 2);
            e1 = __builtin_amdgcn_alignbyte(*reinterpret_cast<const uint32_t *>(img + a_off[j][3]),
                                            *reinterpret_cast<const uint32_t *>(img + a_off[j][2]), 2);
          } else {
            e0 = *reinterpret_cast<const uint32_t *>(img + a_off[j][0]);
            e1 = *reinterpret_cast<const uint32_t *>(img + a_off[j][1]);
          }
          const long   a = (long) (((uint64_t) e1 << 32) | e0);
          const float4 s = *reinterpret_cast<const float4 *>(s_lane + (size_t) it * kScaleStep + j * kLoScaleBlk);
          const long   b = WT == kQ4_0 ? (long) (((uint64_t) hi(wq[j]) << 32) | lo(wq[j])) :
                                         (long) (((uint64_t) wq[2 * j + 1] << 32) | wq[2 * j]);
          const v4i    zero = { 0, 0, 0, 0 };
          const v4i    p    = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b, zero, 0, 0, 0);
          const float  dw   = (float) sc.h[j];
          acc[0] += (float) p[0] * (s.x * dw);
          acc[1] += (float) p[1] * (s.y * dw);
          acc[2] += (float) p[2] * (s.z * dw);
          acc[3] += (float) p[3] * (s.w * dw);
        }
      }
    }
    if (more) {
#pragma unroll
      for (int c = 0; c < kLoChunk; ++c) {
        cur[c] = nxt[c];
      }
    }
  }

  // ---- add the waves of a tile in wave order (the panel is no longer needed) ----
  __syncthreads();
  float *red = reinterpret_cast<float *>(lo_lds);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    red[(wave * 4 + j) * kWave + lane] = acc[j];
  }
  __syncthreads();
  if (tid < 4 * kWave * TPW) {
    const int t = tid / (4 * kWave), j = (tid >> 6) & 3, l = tid & 63, row = 4 * (l >> 4) + j;
    float     v = 0.0f;
#pragma unroll
    for (int w = 0; w < WQ; ++w) {
      v += red[((t * WQ + w) * 4 + j) * kWave + l];
    }
    const int n0 = ((int) blockIdx.x * TPW + t) * kLoRows;
    if ((l >> 4) < ROWS / 4 && row < m && n0 < n) {
      out[(size_t) row * n + n0 + (l & 15)] = v;
    }
  }
}

// LDS of a workgroup: the activation rows in whole DMA instructions, the scale table; later the waves' sums
int panel_rows(int m) {
  return m <= 8 ? 8 : kLoMaxActRows;
}

size_t panel_bytes(int k, int rows) {
  const size_t nblk  = (size_t) k / 32;
  const size_t image = (((size_t) rows * (nblk * 34 / 16) * 16) + 1023) & ~(size_t) 1023;
  const size_t panel = image + nblk * (size_t) rows * 4, red = (size_t) kLoWaves * 4 * kWave * sizeof(float);
  return panel > red ? panel : red;
}

}  // namespace

bool matmul_lane_order_fits(int n, int m, int k, WeightType wt) {
  // k % 256: activation rows (34 B per 32 elements) are whole 16-byte pieces, weight rows whole quads of blocks
  return (wt == kQ4_0 || wt == kQ8_0) && m >= 2 && m <= kLoMaxActRows && k > 0 && k % 256 == 0 && n > 0 && n % kLoRows == 0 &&
         panel_bytes(k, panel_rows(m)) <= kLoLdsLimit && n / kLoRows <= 0x7fffffff;
}

size_t matmul_lane_order_weight_bytes(int k, int n, WeightType wt) {
  return (size_t) (n / kLoRows) * (size_t) (k / 128) * quad_bytes(wt);
}

hipError_t launch_weights_to_lane_order(hipStream_t stream, void *dst, const void *weight, int k, int n, WeightType wt) {
  if (k % 128 != 0 || n % kLoRows != 0 || (wt != kQ4_0 && wt != kQ8_0)) {
    return hipErrorNotSupported;
  }
  const size_t items = (size_t) (n / kLoRows) * (size_t) (k / 128) * 64;
  const dim3   grid((unsigned) ((items + 255) / 256));
  if (wt == kQ4_0) {
    hipLaunchKernelGGL(q4_0_to_lane_order_kernel, grid, dim3(256), 0, stream, static_cast<uint8_t *>(dst),
                       static_cast<const uint8_t *>(weight), k / 32, n);
  } else {
    hipLaunchKernelGGL(q8_0_to_lane_order_kernel, grid, dim3(256), 0, stream, static_cast<uint8_t *>(dst),
                       static_cast<const uint8_t *>(weight), k / 32, n);
  }
  return hipGetLastError();
}

hipError_t launch_matmul_lane_order_group(hipStream_t stream, int count, float *const *outs, const void *const *acts,
                                          const void *const *lane_order_weights, const int *ns, int m, int k,
                                          WeightType wt, int forced_tiles) {
  if (count < 1 || count > kGemvGroupMax) {
    return hipErrorNotSupported;
  }
  LaneOrderGroupArgs grp = {};
  int                n_max = 0;
  for (int i = 0; i < count; ++i) {
    if (!matmul_lane_order_fits(ns[i], m, k, wt) || (reinterpret_cast<uintptr_t>(lane_order_weights[i]) & 15) != 0 ||
        (reinterpret_cast<uintptr_t>(acts[i]) & 15) != 0) {
      return hipErrorNotSupported;
    }
    grp.w[i]   = static_cast<const uint8_t *>(lane_order_weights[i]);
    grp.act[i] = static_cast<const uint8_t *>(acts[i]);
    grp.out[i] = outs[i];
    grp.n[i]   = ns[i];
    n_max      = ns[i] > n_max ? ns[i] : n_max;
  }
  typedef void (*Kernel)(LaneOrderGroupArgs, int, int);
  static const Kernel kernels[2][2][2] = {
    { { matmul_lane_order_kernel<8, 1, kQ4_0>, matmul_lane_order_kernel<8, 2, kQ4_0> },
      { matmul_lane_order_kernel<16, 1, kQ4_0>, matmul_lane_order_kernel<16, 2, kQ4_0> } },
    { { matmul_lane_order_kernel<8, 1, kQ8_0>, matmul_lane_order_kernel<8, 2, kQ8_0> },
      { matmul_lane_order_kernel<16, 1, kQ8_0>, matmul_lane_order_kernel<16, 2, kQ8_0> } } };
  static bool attr_set = false;  // more than the default 64 KiB of dynamic LDS for long rows
  if (!attr_set) {
    for (int i = 0; i < 8; ++i) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernels[i / 4][(i / 2) % 2][i % 2]),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int) kLoLdsLimit);
      if (e != hipSuccess) {
        return e;
      }
    }
    attr_set = true;
  }
  // two tiles per workgroup when that still gives every CU two workgroups (measured at m = 8: gate + up, 688 pairs,
  // 19.6 -> 17.6 us; q + k + v, 384 pairs, no gain; single 4096-row matrices lose)
  long pairs = 0;
  for (int i = 0; i < count; ++i) {
    pairs += (ns[i] / kLoRows + 1) / 2;
  }
  const int    tpw    = forced_tiles == 2 || forced_tiles == 3 ? forced_tiles - 1 : (pairs >= 512 ? 2 : 1);
  const dim3   grid((unsigned) ((n_max / kLoRows + tpw - 1) / tpw), (unsigned) count);
  const int    rows = panel_rows(m);
  const size_t lds  = panel_bytes(k, rows);
  hipLaunchKernelGGL(kernels[wt == kQ8_0][rows == 16][tpw - 1], grid, dim3(kLoThreads), lds, stream, grp, m, k);
  return hipGetLastError();
}

}  // namespace htpops
