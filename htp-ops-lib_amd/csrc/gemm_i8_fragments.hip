// Prefill-sized quantized matmul on gfx950: out fp32 [m][n] = act block_q8_0 [m][k/32] x W (Q4_0 or Q8_0 rows).
//
// Replaces the many-row case of hmx_mat_mul_permuted_qk_0_d16a32 (reference: src/dsp/ops/mat_mul.c:875-1153); the
// arithmetic is ggml's integer block dot (exact int32 block sums, one fp32 scale per block pair of scales).
//
// Per 32 x 32 x 32 block ("unit") the work is
//     S = act_int8 x w_int8          one v_mfma_i32_32x32x32_i8 (exact block sums for 32 rows x 32 columns)
//     C = d_act (x) d_w              one v_mfma_f32_32x32x8f16 with the two fp16 scales in K slot 0: the exact fp32
//                                    product of the scales of every (row, column) pair
//     acc = fma((float) S, C, acc)   the only vector-ALU work: one convert and one fma per block sum
// The vector ALU is the floor of this arithmetic (M N K / 32 converts + fmas); everything else is arranged so that it
// never waits: both operands are kept in "fragment order" -- for every 32-row tile and every block the 64 lanes'
// 16-byte MFMA operands form one contiguous KiB -- so the inner loop is loads straight into MFMA registers, no LDS,
// no barrier, no conversion.
//   weights   converted once per weight buffer (nibbles -> int8 with the "- 8" applied, scales -> one dword per row
//             and block) and cached by the caller; Q4_0 grows from 0.5625 to 1.125 bytes per weight in that cache
//   act       converted per call from block_q8_0 rows (a pure re-ordering)
// A wave owns 64 x 64 outputs (2 x 2 units per block) and a share of K; the KSPLIT waves of one tile are summed
// through LDS in a fixed order. Launches with too few such tiles to fill the chip use 32 x 32 tiles (one unit per
// block) instead: four times the workgroups, each with a quarter of the vector-ALU work.
#include "device_utils.h"
#include "kernels.h"

#include <algorithm>
#include <type_traits>

namespace htpops {

namespace {

typedef int      v4i __attribute__((ext_vector_type(4)));
typedef int      v16i __attribute__((ext_vector_type(16)));
typedef float    v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

// ---- operand conversion -------------------------------------------------------------------------------------------
// fragment (tile, block): lane (c = lane % 32, h = lane / 32) holds elements 16 h .. 16 h + 15 of block `block` of row
// 32 tile + c; the scale array holds one dword (fp16 scale, 0) per row and block: weights [tile][block][32],
// activations [tile][block][64] with zeros in the upper 32 (the operand of the scale product as it is loaded), followed
// by one row of 64 zeros.

template <int WT>
__global__ __launch_bounds__(256) void weights_to_i8_fragments_kernel(uint4 *__restrict__ frag, uint32_t *__restrict__ scales,
                                                                      const uint16_t *__restrict__ w, int n, int nblk,
                                                                      int n_tiles) {
  constexpr int WH = WT == kQ4_0 ? 9 : 17;  // halfwords per block
  const size_t  t  = (size_t) blockIdx.x * 256 + threadIdx.x;
  const int     lane = (int) (t & 63);
  const size_t  f    = t >> 6;
  const int     kb = (int) (f % (size_t) nblk), tile = (int) (f / (size_t) nblk);
  if (tile >= n_tiles) {
    return;
  }
  const int c = lane & 31, h = lane >> 5;
  const int row = tile * 32 + c;
  uint32_t  o[4] = { 0, 0, 0, 0 };
  uint32_t  sc   = 0;
  if (row < n) {
    const uint16_t *blk = w + ((size_t) row * nblk + kb) * WH;
    sc = blk[0];
    if (WT == kQ4_0) {
      // byte j: low nibble = element j, high nibble = element j + 16 (reference: mat_mul.c:266-271)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t q  = (uint32_t) blk[1 + 2 * i] | ((uint32_t) blk[2 + 2 * i] << 16);  // bytes 4i .. 4i + 3
        const uint32_t nb = (q >> (4 * h)) & 0x0F0F0F0Fu;
        // per byte: nibble - 8, as int8 (no borrow between bytes: add 0x80 - 8 then flip the top bit)
        o[i] = (nb + 0x78787878u) ^ 0x80808080u;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        o[i] = (uint32_t) blk[1 + 8 * h + 2 * i] | ((uint32_t) blk[2 + 8 * h + 2 * i] << 16);
      }
    }
  }
  frag[t] = make_uint4(o[0], o[1], o[2], o[3]);
  if (h == 0) {
    scales[((size_t) tile * nblk + kb) * 32 + c] = sc;
  }
}

// up to kGemmGroupMax activation matrices of the same row count in one launch
struct ActMember {
  uint4          *frag;
  uint32_t       *scales;
  const uint16_t *act;
  int             nblk;
  unsigned        piece_begin;  // first thread of this member (a multiple of 64)
};
struct ActMembers {
  ActMember m[kGemmGroupMax];
  int       count;
};

__global__ __launch_bounds__(256) void act_to_i8_fragments_kernel(ActMembers grp, int m, int m_tiles, unsigned pieces) {
  const unsigned g = blockIdx.x * 256 + threadIdx.x;
  if (g >= pieces) {
    return;
  }
  int mi = 0;
  for (int i = 1; i < grp.count; ++i) {
    mi = g >= grp.m[i].piece_begin ? i : mi;
  }
  const ActMember &mem  = grp.m[mi];
  const size_t     t    = g - mem.piece_begin;
  const int        nblk = mem.nblk;
  const int        lane = (int) (t & 63);
  const size_t     f    = t >> 6;
  const int        kb = (int) (f % (size_t) nblk), tile = (int) (f / (size_t) nblk);
  if (tile >= m_tiles) {
    return;
  }
  const int c = lane & 31, h = lane >> 5;
  const int row = tile * 32 + c;
  uint32_t  o[4] = { 0, 0, 0, 0 };
  uint32_t  sc   = 0;
  if (row < m) {
    const uint16_t *blk = mem.act + ((size_t) row * nblk + kb) * 17;
    sc = blk[0];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[i] = (uint32_t) blk[1 + 8 * h + 2 * i] | ((uint32_t) blk[2 + 8 * h + 2 * i] << 16);
    }
  }
  mem.frag[t] = make_uint4(o[0], o[1], o[2], o[3]);
  // scale rows of 64 dwords: lanes 32..63 of the scale-product instruction hold K slots that must contribute nothing
  mem.scales[((size_t) tile * nblk + kb) * 64 + lane] = h == 0 ? sc : 0u;
  if (t < 64) {
    mem.scales[(size_t) m_tiles * nblk * 64 + t] = 0u;  // the row that blocks past the end of K are pointed at
  }
}

// The same for even block counts (k % 64 == 0) and 4-byte aligned rows: one thread per (row, block PAIR) reads its 68
// bytes as dwords (five loads instead of eighteen 2-byte ones) and writes the four 16-byte pieces of the pair.
__global__ __launch_bounds__(256) void act_pairs_to_i8_fragments_kernel(ActMembers grp, int m, int m_tiles, unsigned threads) {
  const unsigned g = blockIdx.x * 256 + threadIdx.x;
  if (g >= threads) {
    return;
  }
  int mi = 0;
  for (int i = 1; i < grp.count; ++i) {
    mi = g >= grp.m[i].piece_begin / 4 ? i : mi;  // (a pair of blocks is four pieces)
  }
  const ActMember &mem   = grp.m[mi];
  const unsigned   t     = g - mem.piece_begin / 4;
  const int        nblk  = mem.nblk, pairs = nblk / 2;
  const int        c     = (int) (t & 31);
  const unsigned   f     = t >> 5;
  const int        pr = (int) (f % (unsigned) pairs), tile = (int) (f / (unsigned) pairs);
  if (tile >= m_tiles) {
    return;
  }
  const int row = tile * 32 + c;
  uint32_t  a[17];
  if (row < m) {
    const uint32_t *src = reinterpret_cast<const uint32_t *>(mem.act) + ((size_t) row * pairs + pr) * 17;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const u32x4_a4 v = *reinterpret_cast<const u32x4_a4 *>(src + 4 * i);
      a[4 * i] = v.x, a[4 * i + 1] = v.y, a[4 * i + 2] = v.z, a[4 * i + 3] = v.w;
    }
    a[16] = src[16];
  } else {
#pragma unroll
    for (int i = 0; i < 17; ++i) {
      a[i] = 0u;
    }
  }
  // block 0: scale in the low half of a[0], quants at bytes 2 .. 33; block 1: scale in the high half of a[8], quants
  // at bytes 36 .. 67 (dwords 9 .. 16)
  uint32_t q0[8], q1[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    q0[i] = __builtin_amdgcn_alignbyte(a[i + 1], a[i], 2);
    q1[i] = a[9 + i];
  }
  const size_t base0 = ((size_t) tile * nblk + 2 * pr) * 64, base1 = base0 + 64;
  mem.frag[base0 + c]      = make_uint4(q0[0], q0[1], q0[2], q0[3]);
  mem.frag[base0 + 32 + c] = make_uint4(q0[4], q0[5], q0[6], q0[7]);
  mem.frag[base1 + c]      = make_uint4(q1[0], q1[1], q1[2], q1[3]);
  mem.frag[base1 + 32 + c] = make_uint4(q1[4], q1[5], q1[6], q1[7]);
  mem.scales[base0 + c]      = a[0] & 0xffffu;
  mem.scales[base0 + 32 + c] = 0u;
  mem.scales[base1 + c]      = a[8] >> 16;
  mem.scales[base1 + 32 + c] = 0u;
  if (t < 64) {
    mem.scales[(size_t) m_tiles * nblk * 64 + t] = 0u;  // the row that blocks past the end of K are pointed at
  }
}

// ---- the matmul ---------------------------------------------------------------------------------------------------

constexpr int kGiThreads = 256;
constexpr int kGiWaves   = 4;
#ifndef GI_DEPTH_U1
#define GI_DEPTH_U1 4
#endif
#ifndef GI_DEPTH_U2
#define GI_DEPTH_U2 2
#endif

template <int UM, int UN>
struct FragSet {
  uint4    a[UM], b[UN];
  uint32_t da[UM], dw[UN];
};

// KSPLIT waves share one tile of UM x UN units (each takes every KSPLIT-th block); a workgroup holds 4 / KSPLIT tiles
// that are neighbours along n (they read the same activation fragments).
// A launch serves up to kGemmGroupMax matmuls of the same row count ("members"): each has its own operands, n and k,
// and a range of workgroups that starts at a multiple of 8 (so that the XCD of a workgroup is the same function of
// its index within the member as in a launch of that member alone).
struct FragMember {
  const uint4    *a_frag;
  const uint32_t *a_scale;
  const uint4    *b_frag;
  const uint32_t *b_scale;
  float          *out;
  int             n, nblk, n_tiles;
  int             ksplit;  // waves that share a tile's K (used by the instantiation that takes it at run time)
  int             share;   // small tiles: which operand the workgroup shares through LDS (kShare*)
  int             kparts;  // kShareWeights: workgroups that share a tile's K (partial tiles meet in `exchange`)
  float          *exchange;
  unsigned       *tickets;  // one zeroed counter per (tile, wave) of this member, left zeroed
  unsigned        wg_begin;
};
struct FragMembers {
  FragMember m[kGemmGroupMax];
  int        count;
};

// KSPLIT_T = 0: the split is the member's own (1, 2 or 4), so that members with short and long K share a launch.
template <int KSPLIT_T, int UM, int UN>
struct RedSlots {
  static constexpr int kValue = KSPLIT_T ? (kGiWaves / KSPLIT_T) * (KSPLIT_T - 1) : kGiWaves - 1;
};

__device__ __forceinline__ const FragMember &member_of_workgroup(const FragMembers &grp) {
  int mi = 0;
  for (int i = 1; i < grp.count; ++i) {
    mi = blockIdx.x >= grp.m[i].wg_begin ? i : mi;
  }
  return grp.m[mi];
}

// one workgroup's share of a member; `red`: RedSlots x (UM UN) x 16 x 64 floats of LDS
template <int KSPLIT_T, int UM, int UN>
__device__ __forceinline__ void fragments_workgroup(const FragMember &mem, int m, int m_tiles, float *red_lds) {
  // fragment sets in flight per wave: small tiles run one wave per SIMD and must cover the memory latency alone
  constexpr int kGiDepth = UM == 1 ? GI_DEPTH_U1 : GI_DEPTH_U2;
  float (*red)[UM * UN][16][64] = reinterpret_cast<float (*)[UM * UN][16][64]>(red_lds);  // partial accumulators of the waves with ks > 0

  // the wave index (and everything derived from it) is made scalar so that fragment addresses are scalar base +
  // per-lane offset and cost no vector instructions in the loop
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 31, h = lane >> 5;
  const int         KSPLIT  = KSPLIT_T ? KSPLIT_T : mem.ksplit;
  const int         TILES   = kGiWaves / KSPLIT;
  const int         ks = wave % KSPLIT, tw = wave / KSPLIT;
  float *__restrict__ out   = mem.out;
  const uint4    *a_frag    = mem.a_frag, *b_frag = mem.b_frag;
  const uint32_t *a_scale   = mem.a_scale, *b_scale = mem.b_scale;
  const int       n = mem.n, nblk = mem.nblk, n_tiles = mem.n_tiles;
  const unsigned  wg = blockIdx.x - mem.wg_begin;
  // tile of this wave, in units of 32: m tiles mt0 .. mt0 + UM - 1; n tiles nt0 .. nt0 + UN - 1
  // Workgroup ids go round-robin over the 8 XCDs (each with its own L2). All row blocks of one column group are
  // given consecutive slots of ONE XCD, so the weight fragments they share are fetched into that L2 once.
  const int gy = (m_tiles + UM - 1) / UM, gx = (n_tiles + UN * TILES - 1) / (UN * TILES);
  const int xcd = wg & 7, slot = wg >> 3;
  const int by = slot % gy, bx = (slot / gy) * 8 + xcd;
  if (bx >= gx) {
    return;  // whole workgroup (the grid is padded to a multiple of 8 column groups)
  }
  const int mt0 = by * UM, nt0 = (bx * TILES + tw) * UN;
  const bool tile_ok = nt0 < n_tiles;  // mt0 < m_tiles by construction

  // Operand streams as buffer resources: a load is then resource (scalar) + per-lane offset (a register that never
  // changes) + scalar offset of the block, and costs no vector-ALU instruction.
  auto resource = [](const void *base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int) 0xffffffffu, 0x00020000);
  };
  __amdgpu_buffer_rsrc_t ra[UM], rb[UN], rsa[UM], rsb[UN];
  int                    zero_row[UM];  // byte offset of the row of zero scales from this tile's scale rows
#pragma unroll
  for (int i = 0; i < UM; ++i) {
    const size_t mt = (size_t) min(mt0 + i, m_tiles - 1);
    ra[i]       = resource(a_frag + mt * nblk * 64);
    rsa[i]      = resource(a_scale + mt * nblk * 64);
    zero_row[i] = (int) (((size_t) m_tiles - mt) * nblk * 256);
  }
#pragma unroll
  for (int j = 0; j < UN; ++j) {
    const size_t nt = (size_t) min(nt0 + j, n_tiles - 1);
    rb[j]  = resource(b_frag + nt * nblk * 64);
    rsb[j] = resource(b_scale + nt * nblk * 32);
  }
  const int lane16 = lane * 16, lane4 = lane * 4, c4 = c * 4;
  auto load = [&](FragSet<UM, UN> &s, int kb_raw) {
    const int  kb   = min(kb_raw, nblk - 1);  // branch-free: blocks past the end repeat the last one ...
    const bool live = kb_raw < nblk;          // ... with activation scales of zero: they add nothing
#pragma unroll
    for (int i = 0; i < UM; ++i) {
      s.a[i]  = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(ra[i], lane16, kb * 1024, 0));
      s.da[i] = __builtin_amdgcn_raw_buffer_load_b32(rsa[i], lane4, live ? kb * 256 : zero_row[i], 0);
    }
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      s.b[j]  = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rb[j], lane16, kb * 1024, 0));
      s.dw[j] = __builtin_amdgcn_raw_buffer_load_b32(rsb[j], c4, kb * 128, 0);
    }
  };

  v16f acc[UM][UN];
#pragma unroll
  for (int i = 0; i < UM; ++i) {
#pragma unroll
    for (int j = 0; j < UN; ++j) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[i][j][r] = 0.0f;
      }
    }
  }

  FragSet<UM, UN> ring[kGiDepth];
#pragma unroll
  for (int d = 0; d < kGiDepth; ++d) {
    load(ring[d], ks + d * KSPLIT);
  }
  const v16f zf = { 0 };
  const v16i zi = { 0 };
  // scale operands of a unit: (scale, 0, 0, 0) in K slot 0; the activation side holds zeros in the lanes of K slots
  // 4..7, so whatever the weight side holds there contributes nothing
  auto scale_operand = [&](uint32_t packed) {
    const uint2 u = make_uint2(packed, 0u);
    return __builtin_bit_cast(v4h, u);
  };
  auto mfma_sum = [&](const FragSet<UM, UN> &s, int i, int j) {
    const v4i af = { (int) s.a[i].x, (int) s.a[i].y, (int) s.a[i].z, (int) s.a[i].w };
    const v4i bf = { (int) s.b[j].x, (int) s.b[j].y, (int) s.b[j].z, (int) s.b[j].w };
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bf, zi, 0, 0, 0);
  };
  auto mfma_scale = [&](const FragSet<UM, UN> &s, int i, int j) {
    return __builtin_amdgcn_mfma_f32_32x32x8f16(scale_operand(s.da[i]), scale_operand(s.dw[j]), zf, 0, 0, 0);
  };

  // Software pipeline over units (block, i, j): the two matrix instructions of the NEXT unit are issued between the
  // 16 converts and the 16 fmas of the CURRENT one, so neither pipe waits for the other.
  v16i sum_next = mfma_sum(ring[0], 0, 0);
  v16f scl_next = mfma_scale(ring[0], 0, 0);
  const int steps = (nblk - ks + KSPLIT - 1) / KSPLIT;  // blocks of this wave
  for (int s0 = 0; s0 < steps; s0 += kGiDepth) {
#pragma unroll
    for (int d = 0; d < kGiDepth; ++d) {
#pragma unroll
      for (int u = 0; u < UM * UN; ++u) {
        constexpr int     LAST = UM * UN - 1;
        const int         i = u / UN, j = u % UN;
        const v16i        sum_cur = sum_next;
        const v16f        scl_cur = scl_next;
        const FragSet<UM, UN> &nx = u < LAST ? ring[d] : ring[(d + 1) % kGiDepth];
        const int              ni = u < LAST ? (u + 1) / UN : 0, nj = u < LAST ? (u + 1) % UN : 0;
        // The empty volatile asm statements keep their program order and each pins the value it names: the next
        // unit's block sums exist (in registers of their own) before this unit's converts and fmas are done.
        sum_next = mfma_sum(nx, ni, nj);
        asm volatile("" : "+v"(sum_next));
        v16f f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          f[r] = (float) sum_cur[r];
        }
        asm volatile("" : "+v"(f));
        scl_next = mfma_scale(nx, ni, nj);
        asm volatile("" : "+v"(scl_next));
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          acc[i][j][r] = __builtin_fmaf(f[r], scl_cur[r], acc[i][j][r]);
        }
        asm volatile("" : "+v"(acc[i][j]));
      }
      // every matrix instruction that reads ring[d] has been issued: fetch the set DEPTH steps ahead
      load(ring[d], ks + (s0 + d + kGiDepth) * KSPLIT);
    }
  }

  // ---- the waves of a tile: ks > 0 park their sums in LDS, ks == 0 adds them in order and stores ----
  if (ks > 0) {
#pragma unroll
    for (int i = 0; i < UM; ++i) {
#pragma unroll
      for (int j = 0; j < UN; ++j) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          red[tw * (KSPLIT - 1) + ks - 1][i * UN + j][r][lane] = acc[i][j][r];
        }
      }
    }
  }
  __syncthreads();
  if (ks == 0 && tile_ok) {
#pragma unroll
    for (int i = 0; i < UM; ++i) {
#pragma unroll
      for (int j = 0; j < UN; ++j) {
        if (mt0 + i < m_tiles && nt0 + j < n_tiles) {
          const int col = (nt0 + j) * 32 + c;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float v = acc[i][j][r];
            for (int s = 0; s < KSPLIT - 1; ++s) {
              v += red[tw * (KSPLIT - 1) + s][i * UN + j][r][lane];
            }
            // D[row][col]: col = lane % 32, row = 8 (r / 4) + 4 (lane / 32) + r % 4
            const int row = (mt0 + i) * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
            if (row < m && col < n) {
              out[(size_t) row * n + col] = v;
            }
          }
        }
      }
    }
  }
}

template <int KSPLIT_T, int UM, int UN>
__global__ __launch_bounds__(kGiThreads) void gemm_i8_fragments_kernel(FragMembers grp, int m, int m_tiles) {
  __shared__ float red[RedSlots<KSPLIT_T, UM, UN>::kValue * UM * UN * 16 * 64];
  fragments_workgroup<KSPLIT_T, UM, UN>(member_of_workgroup(grp), m, m_tiles, red);
}

// ---- 32 x 32 tiles with one operand shared through LDS ------------------------------------------------------------
// With 32 x 32 tiles a wave fetches 2.3 KB of operands per block through the vector-memory path and holds four
// blocks of them in registers: too few bytes in flight to cover the latency (a wave spends ~950 clocks per block on
// the Qwen2 shapes at 128 rows). For members whose K is not split over the waves, the four waves of a workgroup
// therefore share one operand: it arrives once per workgroup, by DMA into a ring of LDS stages of four blocks, and the
// registers it leaves free hold eight blocks of the other operand in flight instead of four.
//   kShareWeights      the waves are the four row tiles of ONE column tile (row counts that are whole groups of four
//                      row tiles, e.g. 128): the weight fragments -- the stream that comes from HBM -- go through LDS,
//                      once per column tile and launch
//   kShareActivations  the waves are four neighbouring column tiles of ONE row tile: the activation fragments go
//                      through LDS
// Long K (which the plain body splits over the four waves of a workgroup) is split over `kparts` WORKGROUPS in the
// kShareWeights arrangement: every wave leaves its partial tile in `exchange` (device-scope stores) and takes a
// ticket; the wave that comes last adds all parts in part order and stores the tile, so the result does not depend
// on who that was and nobody waits for anybody. Other members with split K keep the plain body, in the same launch.
constexpr int kShBlocks = 4;                              // blocks per stage
constexpr int kShStages = 3;
constexpr int kShStage  = kShBlocks * (1024 + 256);       // fragments, then the scale rows (256 or 128 bytes a block)
constexpr int kShLds    = kShStages * kShStage > RedSlots<0, 1, 1>::kValue * 16 * 64 * 4 ?
                              kShStages * kShStage : RedSlots<0, 1, 1>::kValue * 16 * 64 * 4;
enum { kSharePlain = 0, kShareActivations = 1, kShareWeights = 2 };

template <bool SHARE_W>
__device__ __forceinline__ void shared_operand_workgroup(const FragMember &mem, int m, int m_tiles, uint8_t *lds) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 31, h = lane >> 5;
  const int n = mem.n, nblk = mem.nblk, n_tiles = mem.n_tiles;
  const unsigned wg = blockIdx.x - mem.wg_begin;
  // grid of the member: gy groups along m, gx along n (padded to 8 for the XCDs), as member_workgroups lays it out
  const int gy = SHARE_W ? m_tiles / kGiWaves : m_tiles;
  const int gx = SHARE_W ? n_tiles : (n_tiles + kGiWaves - 1) / kGiWaves;
  const int kparts = SHARE_W ? mem.kparts : 1;
  const int xcd = wg & 7, slot = (int) (wg >> 3) / kparts, kpart = (int) (wg >> 3) % kparts;
  const int by = slot % gy, bx = (slot / gy) * 8 + xcd;
  if (bx >= gx) {
    return;  // whole workgroup
  }
  const int  mt = SHARE_W ? by * kGiWaves + wave : by;
  const int  nt = SHARE_W ? bx : bx * kGiWaves + wave;
  const bool tile_ok = nt < n_tiles;  // (mt < m_tiles by construction)
  // stages of this workgroup's part of K: [stage0, stage0 + stages)
  const int  all_stages = nblk / kShBlocks;
  const int  stage0 = (int) ((long) kpart * all_stages / kparts);
  const int  stages = (int) ((long) (kpart + 1) * all_stages / kparts) - stage0;
  const size_t ntc = (size_t) min(nt, n_tiles - 1);

  // -- the shared operand: stage s = blocks 4 s .. 4 s + 3 of its tile, 4 KiB of fragments and the scale rows, both
  // contiguous in memory; wave w moves fragment KiB w, wave 0 the scale rows as well --
  constexpr int  kScaleRow = SHARE_W ? 128 : 256;  // bytes of scales per block
  const uint32_t ring0 = (uint32_t) (uintptr_t) lds;
  const uint8_t *sh_src = SHARE_W ? reinterpret_cast<const uint8_t *>(mem.b_frag) + (ntc * nblk) * 1024 + wave * 1024 :
                                    reinterpret_cast<const uint8_t *>(mem.a_frag) + ((size_t) mt * nblk) * 1024 + wave * 1024;
  const uint8_t *sc_src = SHARE_W ? reinterpret_cast<const uint8_t *>(mem.b_scale) + (ntc * nblk) * 128 :
                                    reinterpret_cast<const uint8_t *>(mem.a_scale) + ((size_t) mt * nblk) * 256;
  const uint32_t lane16 = lane * 16;
  auto dma16 = [&](const uint8_t *base, uint32_t dst) {
    asm volatile("s_mov_b32 m0, %2\n s_nop 0\n global_load_lds_dwordx4 %0, %1" ::"v"(lane16), "s"(base), "s"(dst) : "memory");
  };
  auto issue_stage = [&](int s) {  // (stages past the end re-read the last one; nobody reads them)
    const int      sc = stage0 + min(s, stages - 1);
    const uint32_t so = ring0 + (uint32_t) (s % kShStages) * kShStage;
    dma16(sh_src + (size_t) sc * (kShBlocks * 1024), so + wave * 1024);
    if (wave == 0) {
      if (!SHARE_W || lane < 32) {  // 4 x 128 bytes of weight scales are half a transfer
        dma16(sc_src + (size_t) sc * (kShBlocks * kScaleRow), so + kShBlocks * 1024);
      }
    }
  };
  const int mine = wave == 0 ? 2 : 1;  // transfers of this wave per stage

  // -- the wave's own operand: eight blocks in registers (two stages), block q of stage s in slot (s % 2) * 4 + q --
  auto resource = [](const void *base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int) 0xffffffffu, 0x00020000);
  };
  __amdgpu_buffer_rsrc_t ro  = SHARE_W ? resource(mem.a_frag + (size_t) mt * nblk * 64) : resource(mem.b_frag + ntc * nblk * 64);
  __amdgpu_buffer_rsrc_t rso = SHARE_W ? resource(mem.a_scale + (size_t) mt * nblk * 64) : resource(mem.b_scale + ntc * nblk * 32);
  const int own_scale_off = SHARE_W ? lane * 4 : c * 4;
  uint4     oq[2 * kShBlocks];
  uint32_t  dq[2 * kShBlocks];
  auto load_own = [&](int slot_, int kb_raw) {
    const int kb = min(stage0 * kShBlocks + kb_raw, nblk - 1);  // (blocks past the end repeat the last one; they are never used)
    oq[slot_] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(ro, (int) lane16, kb * 1024, 0));
    dq[slot_] = __builtin_amdgcn_raw_buffer_load_b32(rso, own_scale_off, kb * (SHARE_W ? 256 : 128), 0);
  };

  // prologue: order of vector-memory operations = DMA(0), own(0), DMA(1), own(1); from then on DMA(s + 2) at the start
  // of stage s and own(s + 2) block by block during it
  issue_stage(0);
#pragma unroll
  for (int q = 0; q < kShBlocks; ++q) {
    load_own(q, q);
  }
  issue_stage(1);
#pragma unroll
  for (int q = 0; q < kShBlocks; ++q) {
    load_own(kShBlocks + q, kShBlocks + q);
  }

  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    acc[r] = 0.0f;
  }
  const v16f zf = { 0 };
  const v16i zi = { 0 };
  typedef __attribute__((address_space(3))) const uint8_t *lds_ptr;
  const uint32_t sh_rd = ring0 + lane16, sc_rd = ring0 + kShBlocks * 1024 + (SHARE_W ? c * 4 : lane * 4);

  auto stage = [&](auto parity_tag, int s) {
    constexpr int P = decltype(parity_tag)::value;  // s % 2: which half of the own registers
    // This wave's transfers of stage s have landed; what it issued after them -- own(s) [4 x 2 loads], DMA(s + 1)
    // [mine], own(s + 1) [4 x 2] -- may stay in flight.
    if (mine == 2) {
      __builtin_amdgcn_s_waitcnt(0x0F70 | ((8 + 2 + 8) & 15) | (((8 + 2 + 8) >> 4) << 14));
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70 | ((8 + 1 + 8) & 15) | (((8 + 1 + 8) >> 4) << 14));
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    const uint32_t so = (uint32_t) (s % kShStages) * kShStage;
    v4i      sf[kShBlocks];
    uint32_t sd[kShBlocks];
#pragma unroll
    for (int q = 0; q < kShBlocks; ++q) {
      sf[q] = *reinterpret_cast<__attribute__((address_space(3))) const v4i *>((lds_ptr) (uintptr_t) (sh_rd + so) + q * 1024);
      sd[q] = *reinterpret_cast<__attribute__((address_space(3))) const uint32_t *>((lds_ptr) (uintptr_t) (sc_rd + so) + q * kScaleRow);
    }
    // everybody has left stage s - 1: its LDS stage takes stage s + 2
    issue_stage(s + 2);
    // One unit at a time (the empty asm statements pin that order, so that one unit's results are in registers at a
    // time): with four waves per SIMD it is the other waves that fill the pipes meanwhile.
#pragma unroll
    for (int q = 0; q < kShBlocks; ++q) {
      const v4i o4 = { (int) oq[P * kShBlocks + q].x, (int) oq[P * kShBlocks + q].y, (int) oq[P * kShBlocks + q].z,
                       (int) oq[P * kShBlocks + q].w };
      const uint2 uo = make_uint2(dq[P * kShBlocks + q], 0u), us = make_uint2(sd[q], 0u);
      v16i        sum;
      v16f        scl;
      if (SHARE_W) {  // A operand: activations (own), B operand: weights (shared)
        sum = __builtin_amdgcn_mfma_i32_32x32x32_i8(o4, sf[q], zi, 0, 0, 0);
        scl = __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(v4h, uo), __builtin_bit_cast(v4h, us), zf, 0, 0, 0);
      } else {
        sum = __builtin_amdgcn_mfma_i32_32x32x32_i8(sf[q], o4, zi, 0, 0, 0);
        scl = __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(v4h, us), __builtin_bit_cast(v4h, uo), zf, 0, 0, 0);
      }
      asm volatile("" : "+v"(sum), "+v"(scl));
      // both instructions of block q have read its slot: the slot takes its block of stage s + 2
      load_own(P * kShBlocks + q, (s + 2) * kShBlocks + q);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[r] = __builtin_fmaf((float) sum[r], scl[r], acc[r]);
      }
      asm volatile("" : "+v"(acc));
    }
  };
  for (int s = 0; s < stages; s += 2) {
    stage(std::integral_constant<int, 0>(), s);
    if (s + 1 < stages) {
      stage(std::integral_constant<int, 1>(), s + 1);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // (transfers of stages past the end must have landed before LDS is released)
  if (SHARE_W && kparts > 1) {
    const size_t tile_slot = ((size_t) bx * gy + by) * kGiWaves + wave;  // (column tile, row group, wave)
    float       *parts     = mem.exchange + tile_slot * kparts * 1024;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      __hip_atomic_store(&parts[kpart * 1024 + r * 64 + lane], acc[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // Order between the parts and the ticket. In hardware: every part is a device-scope atomic store (written through
    // to the level all XCDs share), the wait below returns when all of them are acknowledged, and only then is the
    // ticket's read-modify-write issued; the wave that comes last reads the parts with device-scope atomic loads, which
    // do not look into this XCD's L2. At compile time: the wait statement and the fence below are compiler barriers,
    // so neither the stores can sink below the ticket nor the loads rise above it. (A release on the ticket and an
    // acquire fence behind it say the same in the memory model, but at device scope they write back and invalidate
    // the whole L2 per tile: measured 49 against 31 us for the Q8_0 block at 128 rows.)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    unsigned ticket = 0;
    if (lane == 0) {
      ticket = __hip_atomic_fetch_add(&mem.tickets[tile_slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    ticket = __builtin_amdgcn_readfirstlane(ticket);
    if (ticket != (unsigned) (kparts - 1)) {
      return;  // the wave that comes last finishes the tile
    }
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[r] = 0.0f;
    }
    for (int p = 0; p < kparts; ++p) {  // all parts, this wave's own included, in part order
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[r] += __hip_atomic_load(&parts[p * 1024 + r * 64 + lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (lane == 0) {
      __hip_atomic_store(&mem.tickets[tile_slot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
    }
  }
  if (tile_ok) {
    const int col = nt * 32 + c;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = mt * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
      if (row < m && col < n) {
        mem.out[(size_t) row * n + col] = acc[r];
      }
    }
  }
}

__global__ __launch_bounds__(kGiThreads, 4) void gemm_i8_fragments_small_kernel(FragMembers grp, int m, int m_tiles) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kShLds];
  const FragMember &mem = member_of_workgroup(grp);
  if (mem.share == kShareWeights) {
    shared_operand_workgroup<true>(mem, m, m_tiles, lds);
  } else if (mem.share == kShareActivations) {
    shared_operand_workgroup<false>(mem, m, m_tiles, lds);
  } else {
    fragments_workgroup<0, 1, 1>(mem, m, m_tiles, reinterpret_cast<float *>(lds));
  }
}

size_t round256(size_t x) {
  return (x + 255) & ~(size_t) 255;
}

}  // namespace

// layout of a converted weight buffer: [fragments: n_tiles * nblk KiB][scales: n_tiles * nblk * 32 dwords]
size_t gemm_i8_weight_fragment_bytes(int k, int n) {
  const size_t n_tiles = ((size_t) n + 31) / 32, nblk = (size_t) k / 32;
  return round256(n_tiles * nblk * 1024) + n_tiles * nblk * 128;
}

size_t gemm_i8_act_fragment_bytes(int m, int k) {
  const size_t m_tiles = ((size_t) m + 31) / 32, nblk = (size_t) k / 32;
  return round256(m_tiles * nblk * 1024) + m_tiles * nblk * 256 + 256;
}

hipError_t launch_weights_to_i8_fragments(hipStream_t stream, void *dst, const void *weight, int k, int n,
                                          WeightType wt) {
  if (k % 32 != 0 || (reinterpret_cast<uintptr_t>(weight) & 1) != 0) {
    return hipErrorInvalidValue;
  }
  const int    nblk = k / 32, n_tiles = (n + 31) / 32;
  const size_t pieces = (size_t) n_tiles * nblk * 64;
  uint4       *frag   = static_cast<uint4 *>(dst);
  uint32_t    *scales = reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(dst) + round256((size_t) n_tiles * nblk * 1024));
  const dim3   grid((unsigned) ((pieces + 255) / 256));
  if (wt == kQ4_0) {
    hipLaunchKernelGGL(weights_to_i8_fragments_kernel<kQ4_0>, grid, dim3(256), 0, stream, frag, scales,
                       static_cast<const uint16_t *>(weight), n, nblk, n_tiles);
  } else {
    hipLaunchKernelGGL(weights_to_i8_fragments_kernel<kQ8_0>, grid, dim3(256), 0, stream, frag, scales,
                       static_cast<const uint16_t *>(weight), n, nblk, n_tiles);
  }
  return hipGetLastError();
}

namespace {

struct TileConfig {
  int unit, ksplit;
};

// enough waves for two per SIMD: split K four ways when the tile count alone gives fewer than ~1500 waves; when even
// that leaves fewer than two workgroups per CU, 32 x 32 tiles
// With 32 x 32 tiles the split follows K alone: a wave should have some 48 blocks or more to work through (its ring of
// loads and its epilogue are paid once), so short K is not split at all and the four waves of a workgroup take four
// neighbouring column tiles instead.
TileConfig tile_config(int m, int n, int k, int forced_unit) {
  const int m_tiles = (m + 31) / 32, n_tiles = (n + 31) / 32, nblk = k / 32;
  const int wave_tiles  = ((m_tiles + 1) / 2) * ((n_tiles + 1) / 2);
  const int unit        = forced_unit == 1 || forced_unit == 2 ? forced_unit : (wave_tiles < 512 ? 1 : 2);
  if (unit == 1) {
    return { 1, nblk >= 192 ? 4 : nblk >= 96 ? 2 : 1 };
  }
  return { 2, wave_tiles * 2 < 1536 ? 4 : 2 };
}

// Column tiles per wave in the small-tile configuration (32 x 32 kSmallUN outputs). Two (one activation fragment
// serving two products: a quarter less operand traffic, half the waves) measured slower, 57-60 against 47.5 us for
// the Qwen2-like block at m = 128: these launches want waves more than they want bytes saved.
constexpr int kSmallUN = 1;

// small tiles: which operand the four waves of a workgroup share (see shared_operand_workgroup) and, with the weights
// shared, over how many workgroups K is split (`split_k`: the caller has scratch for the partial tiles)
struct SmallTilePlan {
  int share, kparts;
};
SmallTilePlan small_tile_plan(int m_tiles, int nblk, TileConfig cfg, bool split_k) {
  if (cfg.unit != 1 || nblk % kShBlocks != 0 || nblk < 2 * kShBlocks) {
    return { kSharePlain, 1 };
  }
  const bool row_groups = m_tiles % kGiWaves == 0;
  if (cfg.ksplit != 1) {
    // a wave should walk some 48 blocks (as the plain body's split of K aims at)
    // (measured on the Qwen2 block at 128 rows, k = 8960: 24 / 32 / 40 / 48 / 64 blocks per part 38.7 / 38.6 / 35.3 / 35.8 / 37.0 us)
    return row_groups && split_k ? SmallTilePlan{ kShareWeights, std::min(8, nblk / 48) } : SmallTilePlan{ kSharePlain, 1 };
  }
  // (measured on the Qwen2 block at 128 rows: weights shared 39.6 us, activations shared 40.2 us, neither 43.9 us)
  return { row_groups ? kShareWeights : kShareActivations, 1 };
}

unsigned member_workgroups(int m_tiles, int n_tiles, TileConfig cfg, SmallTilePlan plan) {
  if (plan.share == kShareWeights) {
    return (unsigned) ((n_tiles + 7) / 8 * 8 * (m_tiles / kGiWaves) * plan.kparts);
  }
  const unsigned tiles_per_wg = kGiWaves / cfg.ksplit;
  const unsigned un = cfg.unit == 1 ? kSmallUN : cfg.unit;
  const unsigned gy = (unsigned) ((m_tiles + cfg.unit - 1) / cfg.unit);
  const unsigned gx = (unsigned) ((n_tiles + un * tiles_per_wg - 1) / (un * tiles_per_wg));
  return (gx + 7) / 8 * 8 * gy;
}

const uint32_t *scales_of(const void *fragments, size_t tiles, size_t nblk) {
  return reinterpret_cast<const uint32_t *>(static_cast<const uint8_t *>(fragments) + round256(tiles * nblk * 1024));
}

}  // namespace

bool gemm_i8_fragments_groupable(int m, int n, int forced_unit) {
  return tile_config(m, n, 32, forced_unit).unit == 1;
}

hipError_t launch_act_to_i8_fragments_group(hipStream_t stream, int count, void *const *act_fragments,
                                            const void *const *acts_q8_0, const int *ks, int m) {
  if (count < 1 || count > kGemmGroupMax || m <= 0) {
    return hipErrorInvalidValue;
  }
  const int  m_tiles = (m + 31) / 32;
  ActMembers grp;
  size_t     pieces = 0;
  bool       by_pairs = true;
  for (int i = 0; i < count; ++i) {
    if (ks[i] <= 0 || ks[i] % 32 != 0 || (reinterpret_cast<uintptr_t>(acts_q8_0[i]) & 1) != 0) {
      return hipErrorInvalidValue;
    }
    by_pairs = by_pairs && ks[i] % 64 == 0 && (reinterpret_cast<uintptr_t>(acts_q8_0[i]) & 3) == 0;
    const int nblk      = ks[i] / 32;
    grp.m[i].frag        = static_cast<uint4 *>(act_fragments[i]);
    grp.m[i].scales      = const_cast<uint32_t *>(scales_of(act_fragments[i], (size_t) m_tiles, (size_t) nblk));
    grp.m[i].act         = static_cast<const uint16_t *>(acts_q8_0[i]);
    grp.m[i].nblk        = nblk;
    grp.m[i].piece_begin = (unsigned) pieces;
    pieces += (size_t) m_tiles * nblk * 64;
  }
  if (pieces > 0xffffff00u) {
    return hipErrorNotSupported;
  }
  grp.count = count;
  if (by_pairs) {
    const unsigned threads = (unsigned) (pieces / 4);
    hipLaunchKernelGGL(act_pairs_to_i8_fragments_kernel, dim3((threads + 255) / 256), dim3(256), 0, stream, grp, m, m_tiles,
                       threads);
  } else {
    hipLaunchKernelGGL(act_to_i8_fragments_kernel, dim3((unsigned) ((pieces + 255) / 256)), dim3(256), 0, stream, grp, m,
                       m_tiles, (unsigned) pieces);
  }
  return hipGetLastError();
}

size_t gemm_i8_fragments_exchange_bytes(int m, int n, int k, int forced_unit) {
  const int           m_tiles = (m + 31) / 32, n_tiles = (n + 31) / 32, nblk = k / 32;
  const SmallTilePlan plan    = small_tile_plan(m_tiles, nblk, tile_config(m, n, k, forced_unit), true);
  return plan.kparts > 1 ? (size_t) ((n_tiles + 7) / 8 * 8) * m_tiles * plan.kparts * 1024 * sizeof(float) : 0;
}

hipError_t launch_gemm_i8_fragments_group(hipStream_t stream, int count, float *const *outs,
                                          const void *const *act_fragments, const void *const *weight_fragments,
                                          const int *ns, const int *ks, int m, void *exchange, size_t exchange_bytes,
                                          unsigned *tickets, int ticket_slots, int forced_unit) {
  if (count < 1 || count > kGemmGroupMax || m <= 0) {
    return hipErrorInvalidValue;
  }
  size_t exchange_used = 0;
  int    tickets_used  = 0;
  const int   m_tiles = (m + 31) / 32;
  FragMembers grp;
  unsigned    total = 0;
  TileConfig  cfg   = { 0, 0 };
  // Workgroups start in block order: the members whose waves have the most blocks to walk go first, so that the launch
  // ends on short waves (members are independent of each other, their order is free).
  int order[kGemmGroupMax];
  for (int i = 0; i < count; ++i) {
    order[i] = i;
  }
  auto walk = [&](int i) { return ks[i] <= 0 || ns[i] <= 0 ? 0 : ks[i] / 32 / tile_config(m, ns[i], ks[i], forced_unit).ksplit; };
  std::stable_sort(order, order + count, [&](int a, int b) { return walk(a) > walk(b); });
  for (int slot = 0; slot < count; ++slot) {
    const int i = order[slot];
    if (ks[i] <= 0 || ks[i] % 32 != 0 || ns[i] <= 0) {
      return hipErrorInvalidValue;
    }
    const TileConfig c = tile_config(m, ns[i], ks[i], forced_unit);
    if (slot > 0 && (c.unit != cfg.unit || (c.unit != 1 && c.ksplit != cfg.ksplit))) {
      return hipErrorNotSupported;  // every member runs in the configuration it would get alone
    }
    cfg               = c;
    const int nblk = ks[i] / 32, n_tiles = (ns[i] + 31) / 32;
    grp.m[slot].a_frag   = static_cast<const uint4 *>(act_fragments[i]);
    grp.m[slot].a_scale  = scales_of(act_fragments[i], (size_t) m_tiles, (size_t) nblk);
    grp.m[slot].b_frag   = static_cast<const uint4 *>(weight_fragments[i]);
    grp.m[slot].b_scale  = scales_of(weight_fragments[i], (size_t) n_tiles, (size_t) nblk);
    grp.m[slot].out      = outs[i];
    grp.m[slot].n        = ns[i];
    grp.m[slot].nblk     = nblk;
    grp.m[slot].n_tiles  = n_tiles;
    grp.m[slot].ksplit   = c.ksplit;
    grp.m[slot].wg_begin = total;
    // K split over workgroups while the caller's scratch for partial tiles and its ticket counters last
    const size_t  xbytes  = gemm_i8_fragments_exchange_bytes(m, ns[i], ks[i], forced_unit);
    const int     xslots  = (n_tiles + 7) / 8 * 8 * m_tiles;
    const bool    split_k = exchange && tickets && xbytes > 0 && exchange_used + xbytes <= exchange_bytes &&
                         tickets_used + xslots <= ticket_slots;
    SmallTilePlan plan    = small_tile_plan(m_tiles, nblk, c, split_k);
    grp.m[slot].share    = plan.share;
    grp.m[slot].kparts   = plan.kparts;
    grp.m[slot].exchange = nullptr;
    grp.m[slot].tickets  = nullptr;
    if (plan.kparts > 1) {
      grp.m[slot].exchange = reinterpret_cast<float *>(static_cast<uint8_t *>(exchange) + exchange_used);
      grp.m[slot].tickets  = tickets + tickets_used;
      exchange_used += xbytes, tickets_used += xslots;
    }
    total += member_workgroups(m_tiles, n_tiles, cfg, plan);
  }
  grp.count = count;
  if (cfg.unit == 1) {
    hipLaunchKernelGGL(gemm_i8_fragments_small_kernel, dim3(total), dim3(kGiThreads), 0, stream, grp, m, m_tiles);
  } else if (cfg.ksplit == 4) {
    hipLaunchKernelGGL((gemm_i8_fragments_kernel<4, 2, 2>), dim3(total), dim3(kGiThreads), 0, stream, grp, m, m_tiles);
  } else {
    hipLaunchKernelGGL((gemm_i8_fragments_kernel<2, 2, 2>), dim3(total), dim3(kGiThreads), 0, stream, grp, m, m_tiles);
  }
  return hipGetLastError();
}

hipError_t launch_gemm_i8_fragments(hipStream_t stream, float *out, const void *act_q8_0, const void *weight_fragments,
                                    int m, int k, int n, void *act_fragments, bool act_fragments_ready, void *exchange,
                                    size_t exchange_bytes, unsigned *tickets, int ticket_slots, int forced_unit) {
  if (k % 32 != 0 || m <= 0 || n <= 0) {
    return hipErrorInvalidValue;
  }
  if (!act_fragments_ready) {
    if (hipError_t e = launch_act_to_i8_fragments_group(stream, 1, &act_fragments, &act_q8_0, &k, m); e != hipSuccess) {
      return e;
    }
  }
  const void *af = act_fragments;
  return launch_gemm_i8_fragments_group(stream, 1, &out, &af, &weight_fragments, &n, &k, m, exchange, exchange_bytes, tickets,
                                        ticket_slots, forced_unit);
}

}  // namespace htpops
