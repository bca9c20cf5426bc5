// Prefill-sized Q4_0 x Q8_0 matmul on gfx950: out fp32 [m][n] = act block_q8_0 [m][k/32] x W (Q4_0 rows), exact block
// sums on the FP6 matrix instruction, operands staged in LDS by DMA.
//
// Replaces the many-row case of hmx_mat_mul_permuted_qk_0_d16a32 (reference: src/dsp/ops/mat_mul.c:875-1153), whose
// pipeline stages a weight chunk in on-chip memory, converts it there and feeds the matrix unit while the next chunk is
// on its way (:964-999, :1006-1139), with the activations re-tiled once per call (:89-128).
//
// Arithmetic per 32 x 32 x 32 block ("unit"): ggml's integer block dot, exact.
//     S = act_int8 x (q - 8)    ONE v_mfma_scale_f32_32x32x64_f8f6f4 on FP6 (E2M3) operands: an int8 activation is
//                               a = 16 hi + lo with hi in [-8, 7], lo in [0, 15]; hi, lo and q - 8 are integers of
//                               magnitude <= 15, which E2M3 holds exactly as t / 8 (code = sign bit | magnitude).
//                               The instruction's K = 64 is spent as [hi (32) | lo (32)] against [w (32) | w (32)];
//                               its per-32 power-of-two block scales supply the 16 of the hi half and undo the 1/8s.
//                               S leaves the matrix core as fp32, so no int -> float conversion is needed.
//     C = d_act (x) d_w         one v_mfma_f32_32x32x8_f16 with the fp16 scales in K slots 0 / 1: the exact fp32
//                               product of every (row, column) scale pair
//     acc = fma(S, C, acc)      the only vector-ALU work: one fma per block sum (half of what int8 MFMA + convert +
//                               fma issues, and the vector ALU is what bounds this arithmetic)
// Both operands are kept in the byte order the matrix core wants ("tiles"), so that the kernel's memory side is DMA
// straight into LDS and ds_read into operand registers, with no data shuffling and no vector-ALU work:
//   weights      converted once per weight buffer (1 byte per weight incl. scales) and cached by the caller
//   activations  converted per call from block_q8_0 rows; shared by the matmuls of a message that read the same rows
// A workgroup owns 128 x 64 or 128 x 96 outputs over all of K (no exchange between workgroups; a result depends on the
// shape alone): one wave per 64 x 32 outputs (two accumulator tiles, so that an operand read from LDS serves two matrix
// instructions). K advances in steps of two blocks through a ring of LDS stages filled ahead by DMA: three stages of
// 17 KB and three workgroups per compute unit for 128 x 64, four stages of 19 KB and two workgroups for 128 x 96 (a
// third fewer activation bytes per unit of work, for shapes with enough such tiles). With KS = 2 or 3, further groups
// of waves take the other shares of K (shapes with too few tiles to fill the device) and the partial tiles are added
// through LDS in a fixed order.
#include "device_utils.h"
#include "kernels.h"

#include <algorithm>
#include <type_traits>

namespace htpops {

namespace {

typedef int      v4i __attribute__((ext_vector_type(4)));
typedef int      v2i __attribute__((ext_vector_type(2)));
typedef int      v8i __attribute__((ext_vector_type(8)));
typedef float    v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

constexpr int kBM = 128;        // output rows per workgroup; its columns: 32 NT, NT = 2 or 3
constexpr int kMinTiles = 192;  // 128 x 64 output tiles from which the kernel is used

// ---- tiles ----------------------------------------------------------------------------------------------------------
// The 32 FP6 codes of one row (column) of a block are 24 bytes, element e at bits [6 e, 6 e + 6). A step = a block
// pair; its two code strings travel as three 16-byte pieces per lane ("planes"):
//   plane 0 = [lane][block 0 bytes 0..15], plane 1 = [lane][block 0 bytes 16..23] then [lane][block 1 bytes 16..23],
//   plane 2 = [lane][block 1 bytes 0..15]
// so that each block's operand registers are filled by one 16-byte and one 8-byte LDS read.
//   activation tile (32 rows, step): 3 planes x 64 lanes x 16 bytes; lane (c, h): row c, h = 0 the hi parts, h = 1 the lo
//                                    parts. Row scales apart, per 128 rows and step 1 KiB: row r at dwords 2 r, 2 r + 1
//                                    = (even block | odd block << 16, 0): the operand of the scale product as it is read.
//   weight tile (32 columns, step):  2 KiB: plane 0 (32 x 16 B), plane 1 (32 x 8 B block 0, 32 x 8 B block 1), plane 2,
//                                    then the scales as operand dwords of the scale product: [block][64 lanes], lane
//                                    l < 32: the column's fp16 scale in the half-word of its block (K slot 0 or 1),
//                                    lanes 32..63: 0.
constexpr int kATile  = 3 * 1024;
constexpr int kWTile  = 2 * 1024;
constexpr int kSaTile = 1024;
constexpr int kOffA   = 0;
constexpr int kOffW   = kOffA + (kBM / 32) * kATile;

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

// one thread per (column tile of 32, step, column)
__global__ __launch_bounds__(256) void q4_0_to_fp6_tiles_kernel(uint8_t *__restrict__ tiles, const uint32_t *__restrict__ w,
                                                                int n, int pairs, size_t total) {
  const size_t t = (size_t) blockIdx.x * 256 + threadIdx.x;
  if (t >= total) {
    return;
  }
  const int    c = (int) (t & 31);
  const size_t rec = t >> 5;  // tile * pairs + step
  const int    step = (int) (rec % (size_t) pairs), tile = (int) (rec / (size_t) pairs);
  const int    col = tile * 32 + c;
  uint32_t     o0[6] = { 0, 0, 0, 0, 0, 0 }, o1[6] = { 0, 0, 0, 0, 0, 0 };
  uint32_t     d0 = 0, d1 = 0;
  if (col < n) {
    const uint32_t *src = w + ((size_t) col * pairs + step) * 9;  // [d0:2][16 nibble bytes][d1:2][16 nibble bytes]
    uint32_t        r[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) {
      r[i] = src[i];
    }
    d0 = r[0] & 0xffffu;
    d1 = r[4] & 0xffff0000u;
    uint32_t q0[4], q1[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      q0[i] = __builtin_amdgcn_alignbyte(r[i + 1], r[i], 2);
      q1[i] = r[5 + i];
    }
    int v0[32], v1[32];
    // byte j: low nibble = element j, high nibble = element j + 16 (reference: mat_mul.c:266-271)
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const uint32_t b0 = (q0[j / 4] >> (8 * (j % 4))) & 0xffu, b1 = (q1[j / 4] >> (8 * (j % 4))) & 0xffu;
      v0[j] = (int) (b0 & 15) - 8, v0[j + 16] = (int) (b0 >> 4) - 8;
      v1[j] = (int) (b1 & 15) - 8, v1[j + 16] = (int) (b1 >> 4) - 8;
    }
    pack_fp6(o0, v0);
    pack_fp6(o1, v1);
  }
  uint8_t *tile_base = tiles + rec * kWTile;
  reinterpret_cast<uint4 *>(tile_base)[c]        = make_uint4(o0[0], o0[1], o0[2], o0[3]);
  reinterpret_cast<uint2 *>(tile_base + 512)[c]  = make_uint2(o0[4], o0[5]);
  reinterpret_cast<uint2 *>(tile_base + 768)[c]  = make_uint2(o1[4], o1[5]);
  reinterpret_cast<uint4 *>(tile_base + 1024)[c] = make_uint4(o1[0], o1[1], o1[2], o1[3]);
  uint32_t *sc = reinterpret_cast<uint32_t *>(tile_base + 1536);
  sc[c]      = d0;
  sc[32 + c] = 0u;
  sc[64 + c] = d1;
  sc[96 + c] = 0u;
}

// One thread per (row of the padded row count, block, hi or lo half). A wave is one block of the 32 rows of a row tile,
// lanes 0..31 their hi halves and 32..63 their lo halves: its stores are the 1 KiB and the 512 bytes that this block
// owns in the tile's planes, in lane order. Four int8 of a dword are split at once: lo = a & 15 is its own code;
// hi = a >> 4 (arithmetic) as sign and magnitude. Measured on 512 rows of 4096 / 11008 (kernel trace): 5.8 / 7.1 us,
// of which about 3 us are what the smallest kernel costs there. One thread per row and step, with both blocks and both
// halves in a chain of ~1000 vector instructions and a wave per SIMD at most, took 6.0 / 11.2 us; staging the rows
// through LDS so that every load instruction reads consecutive dwords (a lane per row fetches from 32 cache lines)
// took 7.0 / 8.4 us.
__global__ __launch_bounds__(256) void q8_0_to_fp6_tiles_kernel(uint8_t *__restrict__ tiles, uint32_t *__restrict__ scales,
                                                                const uint32_t *__restrict__ act, int m, int pairs,
                                                                int rows_padded) {
  const unsigned t    = blockIdx.x * 256u + threadIdx.x;
  const int      lane = (int) (t & 63u);
  const unsigned wave = t >> 6;
  const int      b    = (int) (wave & 1u);  // block of the step
  const int      step = (int) ((wave >> 1) % (unsigned) pairs);
  const int      rt   = (int) ((wave >> 1) / (unsigned) pairs);
  const int      r    = rt * 32 + (lane & 31);
  const bool     lo   = lane >= 32;
  if (r >= rows_padded) {
    return;  // (whole waves: rows_padded is a multiple of 32)
  }
  // the block's 34 bytes start on a 4-byte boundary (b = 0) or 2 bytes behind one (b = 1): nine aligned dwords hold it
  uint32_t a[9];
  if (r < m) {
    const uint32_t *src = act + ((size_t) r * pairs + step) * 17 + 8 * b;
#pragma unroll
    for (int i = 0; i < 9; ++i) {
      a[i] = src[i];
    }
  } else {
#pragma unroll
    for (int i = 0; i < 9; ++i) {
      a[i] = 0u;
    }
  }
  const uint32_t d = b == 0 ? (a[0] & 0xffffu) : (a[0] >> 16);
  uint32_t       g[8];  // the codes of four elements each, 24 bits
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t q = b == 0 ? __builtin_amdgcn_alignbyte(a[i + 1], a[i], 2) : a[i + 1];
    uint32_t       code;
    if (lo) {
      code = q & 0x0f0f0f0fu;
    } else {
      const uint32_t h   = (q >> 4) & 0x0f0f0f0fu;         // high nibbles: 4-bit two's complement
      const uint32_t neg = (h >> 3) & 0x01010101u;
      const uint32_t mag = (h ^ (neg * 15u)) + neg;        // |hi| <= 8 per byte, no carry between bytes
      code               = mag | (neg << 5);
    }
    g[i] = (code & 0x3fu) | ((code >> 2) & 0xfc0u) | ((code >> 4) & 0x3f000u) | ((code >> 6) & 0xfc0000u);
  }
  const uint4 head = make_uint4(g[0] | (g[1] << 24), (g[1] >> 8) | (g[2] << 16), (g[2] >> 16) | (g[3] << 8), g[4] | (g[5] << 24));
  const uint2 tail = make_uint2((g[5] >> 8) | (g[6] << 16), (g[6] >> 16) | (g[7] << 8));
  uint8_t    *tile = tiles + ((size_t) rt * pairs + step) * kATile;
  reinterpret_cast<uint4 *>(tile + 2048 * b)[lane]      = head;
  reinterpret_cast<uint2 *>(tile + 1024 + 512 * b)[lane] = tail;
  // the scale image: per row and step (fp16 scale of block 0 | of block 1, 0)
  uint16_t *sc = reinterpret_cast<uint16_t *>(scales + (((size_t) (r / kBM) * pairs + step) * kBM + (r % kBM)) * 2);
  if (!lo) {
    sc[b] = (uint16_t) d;
  } else if (b == 0) {
    reinterpret_cast<uint32_t *>(sc)[1] = 0u;
  }
}

// ---- the matmul -----------------------------------------------------------------------------------------------------
// NT: column tiles of 32 per workgroup (2 or 3; a K group has 2 NT waves), NS: LDS stages, KS: K groups
template <int NT>
struct Shape {
  static constexpr int kWaves    = 2 * NT;                            // per K group: 2 (rows of 64) x NT (columns of 32)
  static constexpr int kOffSa    = kOffW + NT * kWTile;
  static constexpr int kStage    = kOffSa + kSaTile;
  static constexpr int kDma      = (kBM / 32) * 3 + 2 * NT + 1;       // 12 activation planes, 2 NT weight KiB, 1 KiB of scales
  static constexpr int kPerWave  = (kDma + kWaves - 1) / kWaves;      // transfers of the waves that issue the most
};

// The matmuls of one launch: the same activation rows against several weight matrices (q/k/v, gate/up of a prefill
// chunk). blockIdx.y is the member; workgroups past a member's own tiles leave at once. One grid for all of them keeps
// every compute unit fed to the end: a launch of its own ends with compute units idle while the last workgroups finish
// (512 x 11008 x 4096: 65 us alone, 60 / 52 / 50 us per matmul with 2 / 4 / 8 in a launch).
struct Fp6Members {
  float         *out[kGemmGroupMax];
  const uint8_t *w_tiles[kGemmGroupMax];
  int            n[kGemmGroupMax];
  int            tiles_n[kGemmGroupMax];
};

template <int NT, int NS, int KS>
__global__ __launch_bounds__(Shape<NT>::kWaves *kWave *KS) void gemm_fp6_lds_kernel(Fp6Members grp,
                                                                                   const uint8_t *__restrict__ a_tiles,
                                                                                   const uint8_t *__restrict__ a_scales,
                                                                                   int m, int pairs, int tiles_m) {
  float *__restrict__ out           = grp.out[blockIdx.y];
  const uint8_t *__restrict__ w_tiles = grp.w_tiles[blockIdx.y];
  const int n = grp.n[blockIdx.y], tiles_n = grp.tiles_n[blockIdx.y];
  using S = Shape<NT>;
  constexpr int kStage = S::kStage, kRing = NS * S::kStage, kOffSa = S::kOffSa;
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kg = wave / S::kWaves, u = wave % S::kWaves;  // K group, wave of the group
  const int wm = u / NT, nt = u % NT;                     // rows 64 wm .. 64 wm + 63, columns 32 nt .. 32 nt + 31

  // Workgroups are handed to the 8 XCDs round-robin, and each XCD has its own L2: the row blocks of one column tile
  // (which read the same weights) are consecutive workgroups of ONE XCD.
  const int xcd = blockIdx.x % 8, j = blockIdx.x / 8;
  const int tile_n = (j / tiles_m) * 8 + xcd, tile_m = j % tiles_m;
  if (tile_n >= tiles_n) {
    return;  // whole workgroup
  }

  // steps of this K group: [s0, s0 + steps); every group runs `iters` iterations (barriers), some of them empty
  const int iters = (pairs + KS - 1) / KS;
  const int s0    = kg * iters;
  const int steps = min(iters, pairs - s0);
  auto step_of = [&](int x) { return s0 + max(0, min(x, steps - 1)); };  // (DMA for steps past the end re-reads the last one)

  uint8_t       *ring  = lds + kg * kRing;
  const uint32_t ring0 = (uint32_t) (uintptr_t) ring;

  // ---- DMA: everything this kernel reads from memory goes straight into LDS (written out as instructions: the
  // compiler would make every LDS read after a DMA it knows of wait for ALL DMA in flight). The transfers of a step
  // (1 KiB each: 12 activation planes, 2 NT weight KiB, the row scales) are dealt to the waves of a K group round
  // robin: wave u issues transfers u, u + kWaves, ... Addresses are a scalar base (tile and step) plus a per-lane
  // offset that never changes, so a transfer costs no vector ALU work. ----
  auto dma16 = [&](const uint8_t *base, uint32_t lane_off, uint32_t dst) {
    asm volatile("s_mov_b32 m0, %2\n s_nop 0\n global_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(dst) : "memory");
  };
  const int last_mt  = (m + 31) / 32 - 1;
  const int last_ct  = (n + 31) / 32 - 1;  // column tiles past the end re-read the last one (their outputs are not stored)
  const uint8_t *src[S::kPerWave];
  uint32_t       dst[S::kPerWave], stride[S::kPerWave];
#pragma unroll
  for (int i = 0; i < S::kPerWave; ++i) {
    const int p = u + S::kWaves * i;  // (p >= kDma: this wave has one transfer less; the entry is never used)
    if (p < 12) {
      const size_t rt = (size_t) min(tile_m * (kBM / 32) + p / 3, last_mt);
      src[i]    = a_tiles + rt * pairs * kATile + (p % 3) * 1024;
      dst[i]    = ring0 + kOffA + (p / 3) * kATile + (p % 3) * 1024;
      stride[i] = kATile;
    } else if (p < 12 + 2 * NT) {
      const int    q  = p - 12;
      const size_t ct = (size_t) min(tile_n * NT + q / 2, last_ct);
      src[i]    = w_tiles + ct * pairs * kWTile + (q % 2) * 1024;
      dst[i]    = ring0 + kOffW + (q / 2) * kWTile + (q % 2) * 1024;
      stride[i] = kWTile;
    } else {
      src[i]    = a_scales + (size_t) tile_m * pairs * kSaTile;
      dst[i]    = ring0 + kOffSa;
      stride[i] = kSaTile;
    }
  }
  const int      mine   = (S::kDma - u + S::kWaves - 1) / S::kWaves;  // transfers of this wave per step
  const uint32_t lane16 = lane * 16;
  auto issue_group = [&](int x, int stage) {  // the transfers of step x into `stage`
    const size_t   s  = (size_t) step_of(x);
    const uint32_t so = (uint32_t) stage * kStage;
#pragma unroll
    for (int i = 0; i < S::kPerWave; ++i) {
      if (i < S::kPerWave - 1 || mine == S::kPerWave) {
        dma16(src[i] + s * stride[i], lane16, dst[i] + so);
      }
    }
  };
  // this wave's transfers of the oldest step in flight have landed (NS - 2 younger groups may stay in flight; s_waitcnt
  // operand: vmcnt in bits 3:0 and 15:14, expcnt 7 = no wait in 6:4, lgkmcnt(0) in 11:8)
  auto wait_oldest_group = [&]() {
    static_assert((NS - 2) * S::kPerWave < 16, "vmcnt fits the low four bits");
    if (mine == S::kPerWave) {
      __builtin_amdgcn_s_waitcnt(0x0070 | ((NS - 2) * S::kPerWave));
    } else {
      __builtin_amdgcn_s_waitcnt(0x0070 | ((NS - 2) * (S::kPerWave - 1)));
    }
  };

#pragma unroll
  for (int x = 0; x < NS - 1; ++x) {
    issue_group(x, x);
  }

  const v16f zero_f = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
  v16f       acc0 = zero_f, acc1 = zero_f;  // rows 64 wm .. + 31 and 64 wm + 32 .. + 63
  // block scales of the FP6 instruction (E8M0 bytes): activations 2^3 (lo half) or 2^7 (hi half: x 16), weights 2^3
  const int scale_a = (lane >> 5) ? 127 + 3 : 127 + 7, scale_b = 127 + 3;
  const uint32_t a_rd  = ring0 + kOffA + (2 * wm) * kATile + lane * 16;
  const uint32_t a_rd8 = ring0 + kOffA + (2 * wm) * kATile + 1024 + lane * 8;  // plane 1: [block 0 tails: 64 x 8][block 1 tails]
  const uint32_t w_rd  = ring0 + kOffW + nt * kWTile + (lane & 31) * 16;       // plane 0; plane 2 at + 1024
  const uint32_t w_rd8 = ring0 + kOffW + nt * kWTile + 512 + (lane & 31) * 8;  // block 0 tails; block 1 at + 256
  const uint32_t sb_rd = ring0 + kOffW + nt * kWTile + 1536 + lane * 4;        // block 0; block 1 at + 256
  const uint32_t sa_rd = ring0 + kOffSa + (2 * wm) * 256 + (lane & 31) * 8;    // upper row tile; the lower one at + 256

  typedef __attribute__((address_space(3))) const uint8_t *lds_ptr;
  auto lds_v4i = [](uint32_t addr, int off) {
    return *reinterpret_cast<__attribute__((address_space(3))) const v4i *>((lds_ptr) (uintptr_t) addr + off);
  };
  auto lds_v2i = [](uint32_t addr, int off) {
    return *reinterpret_cast<__attribute__((address_space(3))) const v2i *>((lds_ptr) (uintptr_t) addr + off);
  };
  auto lds_u32 = [](uint32_t addr, int off) {
    return *reinterpret_cast<__attribute__((address_space(3))) const uint32_t *>((lds_ptr) (uintptr_t) addr + off);
  };
  auto operand = [](v4i lo, v2i hi) {  // (elements 6 and 7 of an FP6 operand are not read by the instruction)
    v8i f;
    f[0] = lo[0], f[1] = lo[1], f[2] = lo[2], f[3] = lo[3], f[4] = hi[0], f[5] = hi[1];
    return f;
  };
  auto fma_half = [](v16f &acc, const v16f &s, const v16f &c, int half) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      acc[half * 8 + i] = __builtin_fmaf(s[half * 8 + i], c[half * 8 + i], acc[half * 8 + i]);
    }
  };

  // Block sums / scale products in flight: x belongs to the upper row tile (acc0), y to the lower one (acc1).
  v16f sx = zero_f, cx = zero_f, sy = zero_f, cy = zero_f;
  // One step out of stage ST (a compile-time constant: every LDS offset is an immediate). A wave's four units of a
  // step -- (row tile, block) = (0, 0), (1, 0), (0, 1), (1, 1) -- are software-pipelined: behind every matrix instruction
  // come eight fmas of the unit before, so that the matrix core and the vector ALU both stay busy from within one
  // wave. The last unit's fmas are deferred past the next barrier, behind the first matrix instructions of the next
  // step. The 8-byte tails are read with written-out instructions so that each lands in the two registers behind its
  // operand's first four.
  auto step = [&](auto stage_tag, int t) {
    constexpr int ST = decltype(stage_tag)::value;
    constexpr int so = ST * kStage;
    // step t is complete in LDS: this wave's transfers of it have landed, then everybody's
    wait_oldest_group();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    v2i a00hi, a01hi, a10hi, a11hi, b0hi, b1hi;  // a<row tile><block>
    asm volatile(
        "ds_read_b64 %0, %6 offset:%c8\n ds_read_b64 %1, %6 offset:%c9\n ds_read_b64 %2, %6 offset:%c10\n"
        " ds_read_b64 %3, %6 offset:%c11\n ds_read_b64 %4, %7 offset:%c12\n ds_read_b64 %5, %7 offset:%c13"
        : "=&v"(a00hi), "=&v"(a01hi), "=&v"(a10hi), "=&v"(a11hi), "=&v"(b0hi), "=&v"(b1hi)
        : "v"(a_rd8), "v"(w_rd8), "i"(so), "i"(so + 512), "i"(so + kATile), "i"(so + kATile + 512), "i"(so), "i"(so + 256)
        : "memory");
    const v4i      a00lo = lds_v4i(a_rd, so), a01lo = lds_v4i(a_rd, so + 2048);
    const v4i      a10lo = lds_v4i(a_rd, so + kATile), a11lo = lds_v4i(a_rd, so + kATile + 2048);
    const v4i      b0lo = lds_v4i(w_rd, so), b1lo = lds_v4i(w_rd, so + 1024);
    const uint32_t sb0 = lds_u32(sb_rd, so), sb1 = lds_u32(sb_rd, so + 256);
    v2i            sa0 = lds_v2i(sa_rd, so), sa1 = lds_v2i(sa_rd, so + 256);  // (scale pair, 0): operands as they are
    // everybody has left step t - 1: its stage takes step t + NS - 1
    issue_group(t + NS - 1, (ST + NS - 1) % NS);
    if (KS > 1) {
      sa0[0] = t < steps ? sa0[0] : 0;  // an iteration past this K group's last step adds zeros
      sa1[0] = t < steps ? sa1[0] : 0;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a00hi), "+v"(a01hi), "+v"(a10hi), "+v"(a11hi), "+v"(b0hi), "+v"(b1hi)::"memory");
    const v8i fa00 = operand(a00lo, a00hi), fa01 = operand(a01lo, a01hi), fa10 = operand(a10lo, a10hi), fa11 = operand(a11lo, a11hi);
    const v8i fb0 = operand(b0lo, b0hi), fb1 = operand(b1lo, b1hi);
    const v4h sa0_op = __builtin_bit_cast(v4h, sa0), sa1_op = __builtin_bit_cast(v4h, sa1);
    const v4h sb0_op = __builtin_bit_cast(v4h, make_uint2(sb0, 0u)), sb1_op = __builtin_bit_cast(v4h, make_uint2(sb1, 0u));
#define HTPOPS_FP6_SUMS(fa, fb) __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa, fb, zero_f, 2, 2, 0, scale_a, 0, scale_b)
#define HTPOPS_SCALE_PRODUCTS(sa, sb) __builtin_amdgcn_mfma_f32_32x32x8f16(sa, sb, zero_f, 0, 0, 0)
#define HTPOPS_FENCE __builtin_amdgcn_sched_barrier(0)
    HTPOPS_FENCE;
    sx = HTPOPS_FP6_SUMS(fa00, fb0);            HTPOPS_FENCE;
    fma_half(acc1, sy, cy, 0);                  HTPOPS_FENCE;  // unit (1, 1) of the step before (zeros at the start)
    cx = HTPOPS_SCALE_PRODUCTS(sa0_op, sb0_op); HTPOPS_FENCE;
    fma_half(acc1, sy, cy, 1);                  HTPOPS_FENCE;
    sy = HTPOPS_FP6_SUMS(fa10, fb0);            HTPOPS_FENCE;
    fma_half(acc0, sx, cx, 0);                  HTPOPS_FENCE;
    cy = HTPOPS_SCALE_PRODUCTS(sa1_op, sb0_op); HTPOPS_FENCE;
    fma_half(acc0, sx, cx, 1);                  HTPOPS_FENCE;
    sx = HTPOPS_FP6_SUMS(fa01, fb1);            HTPOPS_FENCE;
    fma_half(acc1, sy, cy, 0);                  HTPOPS_FENCE;
    cx = HTPOPS_SCALE_PRODUCTS(sa0_op, sb1_op); HTPOPS_FENCE;
    fma_half(acc1, sy, cy, 1);                  HTPOPS_FENCE;
    sy = HTPOPS_FP6_SUMS(fa11, fb1);            HTPOPS_FENCE;
    fma_half(acc0, sx, cx, 0);                  HTPOPS_FENCE;
    cy = HTPOPS_SCALE_PRODUCTS(sa1_op, sb1_op); HTPOPS_FENCE;
    fma_half(acc0, sx, cx, 1);                  HTPOPS_FENCE;
#undef HTPOPS_FP6_SUMS
#undef HTPOPS_SCALE_PRODUCTS
#undef HTPOPS_FENCE
  };
  static_assert(NS == 3 || NS == 4, "the loop is unrolled over the stages");
  for (int t = 0; t < iters; t += NS) {
    step(std::integral_constant<int, 0>(), t);
    if (t + 1 < iters) {
      step(std::integral_constant<int, 1>(), t + 1);
    }
    if (t + 2 < iters) {
      step(std::integral_constant<int, 2>(), t + 2);
    }
    if (NS == 4 && t + 3 < iters) {
      step(std::integral_constant<int, (NS == 4 ? 3 : 0)>(), t + 3);
    }
  }
  fma_half(acc1, sy, cy, 0);  // the last step's unit (1, 1)
  fma_half(acc1, sy, cy, 1);

  // -- the K groups meet: group g > 0 leaves its tiles in LDS, group 0 adds them in order --
  __builtin_amdgcn_s_waitcnt(0x0070);  // (transfers of steps past the end must have landed before LDS is reused or released)
  if (KS > 1) {
    static_assert((KS - 1) * S::kWaves * 32 * 64 * 4 <= KS * kRing, "the partial tiles fit the rings");
    __builtin_amdgcn_s_barrier();
    float *red = reinterpret_cast<float *>(lds);
    if (kg > 0) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        red[(((kg - 1) * S::kWaves + u) * 32 + i) * 64 + lane]      = acc0[i];
        red[(((kg - 1) * S::kWaves + u) * 32 + 16 + i) * 64 + lane] = acc1[i];
      }
    }
    __syncthreads();
    if (kg > 0) {
      return;
    }
#pragma unroll
    for (int g = 1; g < KS; ++g) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        acc0[i] += red[(((g - 1) * S::kWaves + u) * 32 + i) * 64 + lane];
        acc1[i] += red[(((g - 1) * S::kWaves + u) * 32 + 16 + i) * 64 + lane];
      }
    }
  }

  const int col = (tile_n * NT + nt) * 32 + (lane & 31);
  if (col < n) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = tile_m * kBM + wm * 64 + (i / 4) * 8 + (lane >> 5) * 4 + (i & 3);
      if (row < m) {
        out[(size_t) row * n + col] = acc0[i];
      }
      if (row + 32 < m) {
        out[(size_t) (row + 32) * n + col] = acc1[i];
      }
    }
  }
}

// (count members: outs, w_tiles and ns of the matmuls that take this instance)
template <int NT, int NS, int KS>
hipError_t launch_instance(hipStream_t stream, int count, float *const *outs, const uint8_t *a_tiles, const uint8_t *a_scales,
                           const uint8_t *const *w_tiles, int m, const int *ns, int pairs) {
  using S = Shape<NT>;
  const int    tiles_m = (m + kBM - 1) / kBM;
  const size_t lds     = (size_t) KS * NS * S::kStage;
  static_assert((size_t) KS * NS * S::kStage <= 160 * 1024, "the rings fit LDS");
  Fp6Members grp = {};
  int        widest = 0;
  for (int i = 0; i < count; ++i) {
    grp.out[i] = outs[i], grp.w_tiles[i] = w_tiles[i], grp.n[i] = ns[i];
    grp.tiles_n[i] = (ns[i] + 32 * NT - 1) / (32 * NT);
    widest         = std::max(widest, grp.tiles_n[i]);
  }
  const dim3   grid((unsigned) (((widest + 7) / 8) * 8 * tiles_m), (unsigned) count);
  auto         kernel  = gemm_fp6_lds_kernel<NT, NS, KS>;
  static bool  raised  = false;
  if (!raised) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) {
      return e;
    }
    raised = true;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(S::kWaves * kWave * KS), lds, stream, grp, a_tiles, a_scales, m, pairs, tiles_m);
  return hipGetLastError();
}


// ---- 128 x 128 tiles, eight waves ---------------------------------------------------------------------------------
// For shapes with enough such tiles. A step moves 21 transfers of 1 KiB for 32 units instead of 17 for 16, and the
// kernel is written for four waves per SIMD (two workgroups of eight waves per compute unit, at most 128 registers):
// matrix and vector instructions of ONE wave issue far below the rate a SIMD sustains, so it is the number of
// resident waves that keeps its pipes busy. A wave owns 64 x 32 outputs; per unit it issues the block-sum
// instruction, the scale-product instruction and the sixteen fmas in that order, without the 128 x 64 kernel's
// second set of result registers. (Two workgroups sharing a tile, one per half of K, with the partial tiles exchanged
// through memory, did not pay on shapes with fewer tiles: 71 against 62 us at 512 x 11008 x 4096.)
constexpr int kWdWaves  = 8;
constexpr int kWdOffW   = 4 * kATile;
constexpr int kWdOffSa  = kWdOffW + 4 * kWTile;
constexpr int kWdStage  = kWdOffSa + kSaTile;
constexpr int kWdStages = 3;
constexpr int kWdDma    = 12 + 8 + 1;  // activation planes, weight KiB, row scales
constexpr int kWdPerWave = (kWdDma + kWdWaves - 1) / kWdWaves;
constexpr int kWdMinTiles = 512;  // 128 x 128 output tiles from which this kernel is used

__global__ __launch_bounds__(kWdWaves *kWave, 2) void gemm_fp6_lds_wide_kernel(
    Fp6Members grp, const uint8_t *__restrict__ a_tiles, const uint8_t *__restrict__ a_scales, int m, int pairs,
    int tiles_m) {
  float *__restrict__ out           = grp.out[blockIdx.y];
  const uint8_t *__restrict__ w_tiles = grp.w_tiles[blockIdx.y];
  const int n = grp.n[blockIdx.y], tiles_n = grp.tiles_n[blockIdx.y];
  constexpr int NS = kWdStages, kStage = kWdStage;
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const int lane = threadIdx.x & 63;
  const int u    = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = u >> 2, wn = u & 3;  // rows 64 wm .. + 63, columns 32 wn .. + 31 of the tile

  // Consecutive workgroups of one XCD (each has its own L2): the row blocks of a column tile, which read the same
  // weights.
  const int xcd = blockIdx.x % 8, j = blockIdx.x / 8;
  const int tile_m = j % tiles_m, tile_n = (j / tiles_m) * 8 + xcd;
  if (tile_n >= tiles_n) {
    return;  // whole workgroup
  }
  const int steps = pairs;
  auto step_of = [&](int x) { return min(x, steps - 1); };  // (DMA for steps past the end re-reads the last one)

  const uint32_t ring0 = (uint32_t) (uintptr_t) lds;
  auto dma16 = [&](const uint8_t *base, uint32_t lane_off, uint32_t dst) {
    asm volatile("s_mov_b32 m0, %2\n s_nop 0\n global_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(dst) : "memory");
  };
  const int last_mt = (m + 31) / 32 - 1;
  const int last_ct = (n + 31) / 32 - 1;  // tiles past the end re-read the last one (their outputs are not stored)
  const uint8_t *src[kWdPerWave];
  uint32_t       dst[kWdPerWave], stride[kWdPerWave];
#pragma unroll
  for (int i = 0; i < kWdPerWave; ++i) {
    const int p = u + kWdWaves * i;  // (p >= kWdDma: this wave has one transfer less; the entry is never used)
    if (p < 12) {
      const size_t rt = (size_t) min(tile_m * 4 + p / 3, last_mt);
      src[i]    = a_tiles + rt * pairs * kATile + (p % 3) * 1024;
      dst[i]    = ring0 + (p / 3) * kATile + (p % 3) * 1024;
      stride[i] = kATile;
    } else if (p < 20) {
      const int    q  = p - 12;
      const size_t ct = (size_t) min(tile_n * 4 + q / 2, last_ct);
      src[i]    = w_tiles + ct * pairs * kWTile + (q % 2) * 1024;
      dst[i]    = ring0 + kWdOffW + (q / 2) * kWTile + (q % 2) * 1024;
      stride[i] = kWTile;
    } else {
      src[i]    = a_scales + (size_t) tile_m * pairs * kSaTile;
      dst[i]    = ring0 + kWdOffSa;
      stride[i] = kSaTile;
    }
  }
  const int      mine   = (kWdDma - u + kWdWaves - 1) / kWdWaves;  // transfers of this wave per step: 3 or 2
  const uint32_t lane16 = lane * 16;
  auto issue_group = [&](int x, int stage) {
    const size_t   s  = (size_t) step_of(x);
    const uint32_t so = (uint32_t) stage * kStage;
#pragma unroll
    for (int i = 0; i < kWdPerWave; ++i) {
      if (i < kWdPerWave - 1 || mine == kWdPerWave) {
        dma16(src[i] + s * stride[i], lane16, dst[i] + so);
      }
    }
  };
  auto wait_oldest_group = [&]() {  // (see the 128 x 64 kernel: one younger group may stay in flight)
    static_assert((NS - 2) * kWdPerWave < 16, "vmcnt fits the low four bits");
    if (mine == kWdPerWave) {
      __builtin_amdgcn_s_waitcnt(0x0070 | ((NS - 2) * kWdPerWave));
    } else {
      __builtin_amdgcn_s_waitcnt(0x0070 | ((NS - 2) * (kWdPerWave - 1)));
    }
  };
#pragma unroll
  for (int x = 0; x < NS - 1; ++x) {
    issue_group(x, x);
  }

  const v16f zero_f = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
  v16f       acc0 = zero_f, acc1 = zero_f;  // rows 64 wm .. + 31 and 64 wm + 32 .. + 63
  const int  scale_a = (lane >> 5) ? 127 + 3 : 127 + 7, scale_b = 127 + 3;
  const uint32_t a_rd  = ring0 + (2 * wm) * kATile + lane * 16;                    // lower row tile at + kATile; block 1 at + 2048
  const uint32_t a_rd8 = ring0 + (2 * wm) * kATile + 1024 + lane * 8;              // tails; block 1 at + 512
  const uint32_t w_rd  = ring0 + kWdOffW + wn * kWTile + (lane & 31) * 16;         // block 1 at + 1024
  const uint32_t w_rd8 = ring0 + kWdOffW + wn * kWTile + 512 + (lane & 31) * 8;    // tails; block 1 at + 256
  const uint32_t sb_rd = ring0 + kWdOffW + wn * kWTile + 1536 + lane * 4;          // block 1 at + 256
  const uint32_t sa_rd = ring0 + kWdOffSa + (2 * wm) * 256 + (lane & 31) * 8;      // lower row tile at + 256

  typedef __attribute__((address_space(3))) const uint8_t *lds_ptr;
  auto lds_v4i = [](uint32_t addr, int off) {
    return *reinterpret_cast<__attribute__((address_space(3))) const v4i *>((lds_ptr) (uintptr_t) addr + off);
  };
  auto lds_v2i = [](uint32_t addr, int off) {
    return *reinterpret_cast<__attribute__((address_space(3))) const v2i *>((lds_ptr) (uintptr_t) addr + off);
  };
  auto lds_u32 = [](uint32_t addr, int off) {
    return *reinterpret_cast<__attribute__((address_space(3))) const uint32_t *>((lds_ptr) (uintptr_t) addr + off);
  };
  auto operand = [](v4i lo, v2i hi) {
    v8i f;
    f[0] = lo[0], f[1] = lo[1], f[2] = lo[2], f[3] = lo[3], f[4] = hi[0], f[5] = hi[1];
    return f;
  };
#define HTPOPS_FENCE __builtin_amdgcn_sched_barrier(0)
  auto unit = [&](v16f &acc, const v8i &fa, const v8i &fb, v4h sa, v4h sb) {
    const v16f s = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa, fb, zero_f, 2, 2, 0, scale_a, 0, scale_b);
    const v16f c = __builtin_amdgcn_mfma_f32_32x32x8f16(sa, sb, zero_f, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      acc[i] = __builtin_fmaf(s[i], c[i], acc[i]);
    }
    HTPOPS_FENCE;
  };
  // One step out of stage ST (a compile-time constant: every LDS offset is an immediate). Block 1's operands are read
  // from LDS while block 0 is being computed.
  auto step = [&](auto stage_tag, int t) {
    constexpr int ST = decltype(stage_tag)::value;
    constexpr int so = ST * kStage;
    wait_oldest_group();  // this wave's transfers of step t have landed, then everybody's
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    v2i a0hi, a1hi, b0hi;  // block 0: row tiles 0 / 1, the column tile
    asm volatile("ds_read_b64 %0, %3 offset:%c5\n ds_read_b64 %1, %3 offset:%c6\n ds_read_b64 %2, %4 offset:%c7"
                 : "=&v"(a0hi), "=&v"(a1hi), "=&v"(b0hi)
                 : "v"(a_rd8), "v"(w_rd8), "i"(so), "i"(so + kATile), "i"(so)
                 : "memory");
    const v4i      a0lo = lds_v4i(a_rd, so), a1lo = lds_v4i(a_rd, so + kATile), b0lo = lds_v4i(w_rd, so);
    const v2i      sa0 = lds_v2i(sa_rd, so), sa1 = lds_v2i(sa_rd, so + 256);  // (scale pair, 0): operands as they are
    const uint32_t sb0 = lds_u32(sb_rd, so), sb1 = lds_u32(sb_rd, so + 256);
    // everybody has left step t - 1: its stage takes step t + NS - 1
    issue_group(t + NS - 1, (ST + NS - 1) % NS);
    // (the wait as a builtin, so that the compiler knows these reads have landed; the empty statement ties the
    // registers written by the reads above to it)
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    asm volatile("" : "+v"(a0hi), "+v"(a1hi), "+v"(b0hi)::"memory");
    v2i c0hi, c1hi, d0hi;  // block 1, the same three
    asm volatile("ds_read_b64 %0, %3 offset:%c5\n ds_read_b64 %1, %3 offset:%c6\n ds_read_b64 %2, %4 offset:%c7"
                 : "=&v"(c0hi), "=&v"(c1hi), "=&v"(d0hi)
                 : "v"(a_rd8), "v"(w_rd8), "i"(so + 512), "i"(so + kATile + 512), "i"(so + 256)
                 : "memory");
    const v4i c0lo = lds_v4i(a_rd, so + 2048), c1lo = lds_v4i(a_rd, so + kATile + 2048), d0lo = lds_v4i(w_rd, so + 1024);
    const v4h sa0_op = __builtin_bit_cast(v4h, sa0), sa1_op = __builtin_bit_cast(v4h, sa1);
    const v4h sb0_op = __builtin_bit_cast(v4h, make_uint2(sb0, 0u)), sb1_op = __builtin_bit_cast(v4h, make_uint2(sb1, 0u));
    {
      const v8i fa0 = operand(a0lo, a0hi), fa1 = operand(a1lo, a1hi), fb = operand(b0lo, b0hi);
      HTPOPS_FENCE;
      unit(acc0, fa0, fb, sa0_op, sb0_op);
      unit(acc1, fa1, fb, sa1_op, sb0_op);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
    asm volatile("" : "+v"(c0hi), "+v"(c1hi), "+v"(d0hi)::"memory");
    {
      const v8i fa0 = operand(c0lo, c0hi), fa1 = operand(c1lo, c1hi), fb = operand(d0lo, d0hi);
      HTPOPS_FENCE;
      unit(acc0, fa0, fb, sa0_op, sb1_op);
      unit(acc1, fa1, fb, sa1_op, sb1_op);
    }
  };
  for (int t = 0; t < steps; t += NS) {
    step(std::integral_constant<int, 0>(), t);
    if (t + 1 < steps) {
      step(std::integral_constant<int, 1>(), t + 1);
    }
    if (t + 2 < steps) {
      step(std::integral_constant<int, 2>(), t + 2);
    }
  }
#undef HTPOPS_FENCE
  __builtin_amdgcn_s_waitcnt(0x0070);  // (transfers of steps past the end must have landed before LDS is released)

  const int col = tile_n * 128 + wn * 32 + (lane & 31);
  if (col < n) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = tile_m * 128 + wm * 64 + (i / 4) * 8 + (lane >> 5) * 4 + (i & 3);
      if (row < m) {
        out[(size_t) row * n + col] = acc0[i];
      }
      if (row + 32 < m) {
        out[(size_t) (row + 32) * n + col] = acc1[i];
      }
    }
  }
}

hipError_t launch_wide(hipStream_t stream, int count, float *const *outs, const uint8_t *a_tiles, const uint8_t *a_scales,
                       const uint8_t *const *w_tiles, int m, const int *ns, int pairs) {
  const int    tiles_m = (m + 127) / 128;
  const size_t lds     = (size_t) kWdStages * kWdStage;
  Fp6Members   grp     = {};
  int          widest  = 0;
  for (int i = 0; i < count; ++i) {
    grp.out[i] = outs[i], grp.w_tiles[i] = w_tiles[i], grp.n[i] = ns[i], grp.tiles_n[i] = (ns[i] + 127) / 128;
    widest = std::max(widest, grp.tiles_n[i]);
  }
  const dim3   grid((unsigned) (((widest + 7) / 8) * 8 * tiles_m), (unsigned) count);
  static bool  raised  = false;
  if (!raised) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_fp6_lds_wide_kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) {
      return e;
    }
    raised = true;
  }
  hipLaunchKernelGGL(gemm_fp6_lds_wide_kernel, grid, dim3(kWdWaves * kWave), lds, stream, grp, a_tiles, a_scales, m, pairs,
                     tiles_m);
  return hipGetLastError();
}

}  // namespace

bool gemm_fp6_lds_fits(int m, int k, int n) {
  return m >= 1 && n >= 1 && k >= 64 && k % 64 == 0;
}

bool gemm_fp6_lds_fills_device(int m, int n) {
  // Below this the kernel's workgroups (one per tile, K split over at most three wave groups inside it) leave compute
  // units idle, and the fragment kernel, which splits K over workgroups, is faster.
  return (long) ((m + kBM - 1) / kBM) * ((n + 63) / 64) >= kMinTiles;
}

size_t gemm_fp6_lds_weight_tile_bytes(int k, int n) {
  return (size_t) ((n + 31) / 32) * (size_t) (k / 64) * kWTile;
}

size_t gemm_fp6_lds_act_tile_bytes(int m, int k) {
  const size_t m_tiles = ((size_t) m + 31) / 32, m_blocks = ((size_t) m + kBM - 1) / kBM, pairs = (size_t) k / 64;
  return m_tiles * pairs * kATile + m_blocks * pairs * kSaTile;
}

hipError_t launch_q4_0_to_fp6_tiles(hipStream_t stream, void *dst, const void *weight, int k, int n) {
  if (k % 64 != 0 || n <= 0 || (reinterpret_cast<uintptr_t>(weight) & 3) != 0) {
    return hipErrorNotSupported;
  }
  const int    pairs = k / 64;
  const size_t total = (size_t) ((n + 31) / 32) * pairs * 32;
  hipLaunchKernelGGL(q4_0_to_fp6_tiles_kernel, dim3((unsigned) ((total + 255) / 256)), dim3(256), 0, stream,
                     static_cast<uint8_t *>(dst), static_cast<const uint32_t *>(weight), n, pairs, total);
  return hipGetLastError();
}

hipError_t launch_gemm_fp6_lds_group(hipStream_t stream, int count, float *const *outs, const void *act_q8_0,
                                     const void *const *weight_tiles, int m, int k, const int *ns, void *act_tiles,
                                     bool act_tiles_ready) {
  if (count < 1 || count > kGemmGroupMax || (reinterpret_cast<uintptr_t>(act_q8_0) & 3) != 0) {
    return hipErrorNotSupported;
  }
  for (int i = 0; i < count; ++i) {
    if (!gemm_fp6_lds_fits(m, k, ns[i])) {
      return hipErrorNotSupported;
    }
  }
  const int pairs   = k / 64;
  const int m_tiles = (m + 31) / 32;
  uint8_t  *tiles   = static_cast<uint8_t *>(act_tiles);
  uint8_t  *scales  = tiles + (size_t) m_tiles * pairs * kATile;
  if (!act_tiles_ready) {
    const size_t threads = (size_t) m_tiles * pairs * 2 * 64;  // a wave per (row tile, step, block)
    if (threads > 0xffffffffull) {
      return hipErrorNotSupported;
    }
    hipLaunchKernelGGL(q8_0_to_fp6_tiles_kernel, dim3((unsigned) ((threads + 255) / 256)), dim3(256), 0, stream, tiles,
                       reinterpret_cast<uint32_t *>(scales), static_cast<const uint32_t *>(act_q8_0), m, pairs, m_tiles * 32);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
      return e;
    }
  }
  // Which kernel a member takes depends on its own shape, as if it were launched alone:
  // 128 x 128 tiles from where they fill two workgroups per compute unit (10 % faster there: 84 against 95 us at
  // 512 x 16384 x 4096); else
  // 128 x 64 tiles: a K group is 4 waves (one per SIMD) and one ring of three stages, and a compute unit holds three
  // rings: one group per workgroup when the tiles alone give every compute unit three workgroups, otherwise up to
  // three groups per workgroup, each with its share of K, so that the same tiles put more waves on a compute unit.
  // (128 x 96 tiles -- NT = 3, four stages, two workgroups of 6 waves per compute unit, a third fewer activation bytes
  // per unit of work -- measured slower, 84 against 64 us at 512 x 11008 x 4096: six waves do not spread evenly over
  // four SIMDs.) Members that take the same kernel share its launch.
  int kind[kGemmGroupMax];  // 0: 128 x 128 tiles; 1..3: K groups per workgroup of the 128 x 64 kernel
  for (int i = 0; i < count; ++i) {
    if ((long) ((m + 127) / 128) * ((ns[i] + 127) / 128) >= kWdMinTiles) {
      kind[i] = 0;
    } else {
      const long tiles64 = (long) ((m + kBM - 1) / kBM) * ((ns[i] + 63) / 64);
      const int  ks      = tiles64 >= 640 ? 1 : tiles64 >= 384 ? 2 : 3;
      kind[i]            = std::max(1, std::min(ks, pairs / 4));
    }
  }
  for (int which = 0; which <= 3; ++which) {
    float         *o[kGemmGroupMax];
    const uint8_t *w[kGemmGroupMax];
    int            n[kGemmGroupMax], c = 0;
    for (int i = 0; i < count; ++i) {
      if (kind[i] == which) {
        o[c] = outs[i], w[c] = static_cast<const uint8_t *>(weight_tiles[i]), n[c++] = ns[i];
      }
    }
    if (c == 0) {
      continue;
    }
    const hipError_t e = which == 0 ? launch_wide(stream, c, o, tiles, scales, w, m, n, pairs) :
                         which == 1 ? launch_instance<2, 3, 1>(stream, c, o, tiles, scales, w, m, n, pairs) :
                         which == 2 ? launch_instance<2, 3, 2>(stream, c, o, tiles, scales, w, m, n, pairs) :
                                      launch_instance<2, 3, 3>(stream, c, o, tiles, scales, w, m, n, pairs);
    if (e != hipSuccess) {
      return e;
    }
  }
  return hipSuccess;
}

hipError_t launch_gemm_fp6_lds(hipStream_t stream, float *out, const void *act_q8_0, const void *weight_tiles, int m, int k,
                               int n, void *act_tiles, bool act_tiles_ready) {
  return launch_gemm_fp6_lds_group(stream, 1, &out, act_q8_0, &weight_tiles, m, k, &n, act_tiles, act_tiles_ready);
}

}  // namespace htpops
