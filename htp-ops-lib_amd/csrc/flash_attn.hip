// Attention for gfx950: O = softmax(Q K^T / sqrt(D) + mask) V per head, GQA by h_kv = h / (n_heads / n_kv_heads).
//
// Replaces simple_flash_attn (reference: src/dsp/ops/flash_attn.c:1368-1420, core :139-825): the same blockwise
// online-softmax recurrence with exp2 and the scale 1/sqrt(D) * log2(e) (reference :210-215, :1440), laid out for
// 64-wide wavefronts and MFMA instead of HVX/HMX tiles in VTCM. Q/O are fp32 (the reference op) or fp16; K/V fp16
// [kv_len][n_kv_heads][D]; the optional fp16 mask [qo_len][align_up(kv_len, 64)] is ADDED to the scaled scores (the
// scalar routine's convention, reference :1505-1512); `causal` hides key j from query i when j > i + kv_len - qo_len.
//
// Three kernels:
//  * prefill (any qo_len, head_dim 64 or 128): one workgroup = 32 query rows x up to 4 query heads of one KV head (one
//    wave per head, so a K/V tile staged in LDS serves the whole GQA group). Scores are computed transposed,
//    S^T = K Q^T with v_mfma_f32_32x32x16_f16, which puts one query per lane: row max / row sum are register
//    reductions plus one exchange between the two lane halves. K and V blocks come into LDS as they lie in memory, by
//    DMA (global_load_lds) into two buffers that take turns: the next block is on its way while one is used. V^T for
//    O^T += V^T P^T is read out of the row-major tile with the transposing LDS read (ds_read_b64_tr_b16); P goes from
//    the score registers straight into the MFMA B operand. Scores are accumulated on top of minus the running
//    maximum, so most blocks need no rescaling. Under `causal`, KV blocks above the diagonal are skipped and the
//    longest query blocks start first. Timing-only builds on the 256-CU device (2048 x 2048 causal, 32 / 8 heads of
//    128: 59 us) put the kernel without any matrix instruction and without the exponentials at 39 us, without the DMA
//    at 51 us: every wave reads the whole K and V tile out of LDS for its 32 queries (1 KiB per matrix instruction:
//    LDS bandwidth would be exhausted at the matrix cores' full rate), and that traffic, not the arithmetic, sets the
//    pace.
//  * decode (qo_len == 1, head_dim 64 or 128): bandwidth bound. The KV range is split across workgroups (n_kv_heads
//    alone would leave the GPU idle); both products run on the matrix cores with the heads of the GQA group as one
//    operand, and a second tiny kernel merges the per-split (max, sum, O) partials in one trip to memory.
//  * any other even head_dim up to 256 (the reference's flash_attn_sp_hdim.c domain): a plain kernel without MFMA.
#include "device_utils.h"
#include "kernels.h"

#include <algorithm>

namespace htpops {

namespace {

// What a mask value contributes to a score. Added as it is (the reference's scalar routine,
// src/dsp/ops/flash_attn.c:1505-1512), or, with `threshold`, selecting the key: kept (0) iff mask > -16, dropped
// (-inf) otherwise, NaN included (the kernel the reference dispatches, src/dsp/ops/flash_attn.c:448-460).
__device__ __forceinline__ float mask_term(_Float16 mv, bool threshold) {
  const float f = (float) mv;
  return threshold ? (f > -16.0f ? 0.0f : -INFINITY) : f;
}

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float    v16f __attribute__((ext_vector_type(16)));

constexpr float kLog2e = 1.44269504f;

__device__ __forceinline__ float fast_exp2(float x) {
  return __builtin_amdgcn_exp2f(x);  // v_exp_f32; exp2(-inf) = 0
}

// ------------------------------------------------------------------------------------------------ prefill

constexpr int kPfThreads = 256;  // threads of one key group: 4 waves, one per query head
constexpr int kBQ        = 32;  // query rows per wave tile
constexpr int kBK        = 64;  // keys per KV block

template <int D>
struct PrefillSmem {
  // K and V tiles of a block of keys, rows as they lie in memory ([key][D] halfs), two buffers each: the next block
  // arrives by DMA while one is used. The 16-byte pieces of a row are stored exclusive-or'ed with low bits of the row
  // number (the DMA chooses what each lane fetches, not where it lands): K rows with key % 8, so that the 16-byte
  // fragment reads of 8 neighbouring keys fall into different banks; V rows with 2 (key % 4), which keeps 32-byte
  // pieces whole for the transposing reads and puts the four rows of such a read into different banks.
  uint8_t k[2][kBK * D * 2];
  uint8_t v[2][kBK * D * 2];
};

// GROUPS = 1 or 2 key groups per workgroup (4 waves each); with 2 they take alternate KV blocks of the same queries
template <int D, bool QO_F32, int GROUPS>
__global__ __launch_bounds__(kPfThreads *GROUPS, 2) void flash_attn_prefill_kernel(void *__restrict__ o_ptr,
                                                                        const void *__restrict__ q_ptr,
                                                                        const _Float16 *__restrict__ k_ptr,
                                                                        const _Float16 *__restrict__ v_ptr,
                                                                        const _Float16 *__restrict__ mask, int qo_len,
                                                                        int kv_len, int n_heads, int n_kv_heads,
                                                                        int flags) {
  const bool causal = (flags & 1) != 0, mask_threshold = (flags & 2) != 0;
  __shared__ __align__(1024) PrefillSmem<D> sm_all[GROUPS];
  constexpr int KSTEPS = D / 16;  // MFMA k-steps over the head dimension
  constexpr int DT     = D / 32;  // 32-row tiles of O^T
  // With GROUPS = 2, two groups of 4 waves work on the same queries and heads: group g takes KV blocks g, g + 2, ...
  // with its own K/V tiles in LDS and its own running (max, sum, O); the two states are merged through LDS at the
  // end. The longest workgroup then walks half as many iterations, which pays when the grid is too small to keep two
  // independent workgroups on every CU busy to the end (few query blocks, or the uneven lengths under `causal`).
  const int           grp = __builtin_amdgcn_readfirstlane((int) threadIdx.x / kPfThreads);  // (the same for a wave)
  PrefillSmem<D>     &sm  = sm_all[grp];

  const int group = n_heads / n_kv_heads;
  const int gc    = group < 4 ? group : 4;  // heads handled by one workgroup
  const int qsub  = 4 / gc;                 // query sub-blocks per workgroup (waves left over when group < 4)
  const int sub_groups = (group + gc - 1) / gc;

  const int tid  = threadIdx.x % kPfThreads;  // within the key group
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int half = lane >> 5;
  const int col  = lane & 31;

  // grid: x = (KV head, head sub-group), y = query block, LAST query block first. Workgroups are dispatched in
  // linear order with x fastest, so under `causal` the long blocks (most visible keys) start first and the short ones
  // fill the tail; consecutive workgroups, which go to different XCDs, work on different KV heads, so one XCD's L2
  // keeps seeing the same K/V stream.
  const int q_block  = (int) (gridDim.y - 1 - blockIdx.y);
  const int h_kv     = blockIdx.x / sub_groups;
  const int h_in_grp = (blockIdx.x % sub_groups) * gc + wave % gc;
  const bool wave_on = h_in_grp < group && wave / gc < qsub;
  const int  head    = h_kv * group + (h_in_grp < group ? h_in_grp : 0);
  const int  q_base  = (q_block * qsub + (wave / gc < qsub ? wave / gc : 0)) * kBQ;
  const int  q_row   = q_base + col;                  // this lane's query
  const bool q_ok    = wave_on && q_row < qo_len;
  const int  q_clamp = q_row < qo_len ? q_row : qo_len - 1;

  const size_t qo_stride = (size_t) n_heads * D;
  const size_t kv_stride = (size_t) n_kv_heads * D;
  const size_t mask_ld   = ((size_t) kv_len + 63) / 64 * 64;
  const float  scale     = (1.0f / sqrtf((float) D)) * kLog2e;

  // Q fragments (B operand of S^T = K Q^T): lane (query, half) holds d = 16 s + 8 half .. + 7 for every k-step s
  v8h qf[KSTEPS];
  {
    const size_t base = (size_t) q_clamp * qo_stride + (size_t) head * D;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int d0 = 16 * s + 8 * half;
      if (QO_F32) {
        const float4 *p  = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(q_ptr) + base + d0);
        const float4  a  = p[0], b = p[1];
        qf[s][0] = (_Float16) (a.x * scale), qf[s][1] = (_Float16) (a.y * scale);
        qf[s][2] = (_Float16) (a.z * scale), qf[s][3] = (_Float16) (a.w * scale);
        qf[s][4] = (_Float16) (b.x * scale), qf[s][5] = (_Float16) (b.y * scale);
        qf[s][6] = (_Float16) (b.z * scale), qf[s][7] = (_Float16) (b.w * scale);
      } else {
        const v8h raw = *reinterpret_cast<const v8h *>(reinterpret_cast<const _Float16 *>(q_ptr) + base + d0);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          qf[s][e] = (_Float16) ((float) raw[e] * scale);
        }
      }
    }
  }

  v16f  oacc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      oacc[t][r] = 0.0f;
    }
  }
  float m_run = -INFINITY;  // running max of this lane's query (same in both halves)
  float l_run = 0.0f;       // running sum over this half's keys only; halves are added at the end

  // keys visible to the LAST query row of the workgroup bound the KV loop under `causal`
  const int q_hi     = min(qo_len, (q_block + 1) * qsub * kBQ) - 1;
  const int kv_limit = causal ? min(kv_len, q_hi + (kv_len - qo_len) + 1) : kv_len;
  const int q_shift  = kv_len - qo_len;
  // last key this lane's query may see, relative to the first key this lane holds in a block (key0 = 4 * half)
  const int vis_last = (causal ? min(kv_len - 1, q_row + q_shift) : kv_len - 1) - 4 * half;

  // The next K/V block travels global memory -> LDS by DMA (global_load_lds, 1 KiB per instruction: no registers, no
  // stores) while the current one is being used. A tile is TILE_B / 1024 instructions, the four waves take every
  // fourth; lane L of an instruction lands at byte 16 L of its KiB = row L / CHUNKS, piece L % CHUNKS, and fetches the
  // piece that belongs there. Per lane the source offsets inside a block never change (kept in registers); what
  // changes per block is a base address the same for all lanes.
  constexpr int ROWB     = D * 2;          // bytes of a K or V row
  constexpr int CHUNKS   = ROWB / 16;      // 16-byte pieces of a row
  constexpr int DMA_ROWS = 1024 / ROWB;    // rows per DMA instruction
  constexpr int TILE_B   = kBK * ROWB;
  constexpr int NDMA     = TILE_B / 1024 / 4;  // instructions per wave and tile
  const int     wave_u   = __builtin_amdgcn_readfirstlane(wave);
  uint32_t      src_off[2][NDMA];  // [K, V]: byte offset of this lane's piece from the block's first row of this KV head
#pragma unroll
  for (int j = 0; j < NDMA; ++j) {
    const int row = (wave_u + 4 * j) * DMA_ROWS + lane / CHUNKS, piece = lane % CHUNKS;
    src_off[0][j] = (uint32_t) row * (uint32_t) (kv_stride * 2) + 16u * (uint32_t) (piece ^ (row & 7));
    src_off[1][j] = (uint32_t) row * (uint32_t) (kv_stride * 2) + 16u * (uint32_t) (piece ^ (2 * (row & 3)));
  }
  auto fetch = [&](int k0, int buf) {
    const uint32_t to_k = (uint32_t) (uintptr_t) sm.k[buf], to_v = (uint32_t) (uintptr_t) sm.v[buf];
    const uint8_t *kb = reinterpret_cast<const uint8_t *>(k_ptr + (size_t) h_kv * D + (size_t) k0 * kv_stride);
    const uint8_t *vb = reinterpret_cast<const uint8_t *>(v_ptr + (size_t) h_kv * D + (size_t) k0 * kv_stride);
    if (k0 + kBK <= kv_len) {
#pragma unroll
      for (int j = 0; j < NDMA; ++j) {
        asm volatile("s_mov_b32 m0, %2\n s_nop 0\n global_load_lds_dwordx4 %0, %1" ::"v"(src_off[0][j]), "s"(kb),
                     "s"(to_k + (uint32_t) ((wave_u + 4 * j) * 1024))
                     : "memory");
      }
#pragma unroll
      for (int j = 0; j < NDMA; ++j) {
        asm volatile("s_mov_b32 m0, %2\n s_nop 0\n global_load_lds_dwordx4 %0, %1" ::"v"(src_off[1][j]), "s"(vb),
                     "s"(to_v + (uint32_t) ((wave_u + 4 * j) * 1024))
                     : "memory");
      }
      return;
    }
    // last, partial block: rows past the end repeat the last key (their scores are hidden below)
#pragma unroll
    for (int j = 0; j < 2 * NDMA; ++j) {
      const int  jj  = j % NDMA;
      const bool isv = j >= NDMA;
      const int  row = (wave_u + 4 * jj) * DMA_ROWS + lane / CHUNKS, piece = lane % CHUNKS;
      const int  key = min(k0 + row, kv_len - 1);
      const int  log = isv ? piece ^ (2 * (row & 3)) : piece ^ (row & 7);
      const _Float16 *src = (isv ? v_ptr : k_ptr) + (size_t) key * kv_stride + (size_t) h_kv * D + 8 * log;
      asm volatile("s_mov_b32 m0, %1\n s_nop 0\n global_load_lds_dwordx4 %0, off" ::"v"(src),
                   "s"((isv ? to_v : to_k) + (uint32_t) ((wave_u + 4 * jj) * 1024))
                   : "memory");
    }
  };
  // additive mask values of this lane's 2 x 16 keys of a block: requested a block ahead, like the tiles
  auto fetch_mask = [&](v4h (&m)[2][4], int k0) {
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        // four consecutive keys: one 8-byte load (rows are padded to a multiple of 64 keys)
        m[kt][rg] = *reinterpret_cast<const v4h *>(mask + (size_t) q_clamp * mask_ld + k0 + 32 * kt + 8 * rg + 4 * half);
      }
    }
  };
  // where this lane's fragments lie in a tile (bytes): K row `col` (+ 32 per tile), piece 2 s + half; V: the lane
  // (16-lane group g = lane / 16, i = lane % 16 = 4 j + q) points at row 4 half + j (+ 16 u + 8 per read), the 8-byte
  // piece q of columns 32 t + 16 (g & 1) .. + 15, and receives column 32 t + 16 (g & 1) + i of four rows
  uint32_t k_at[KSTEPS], v_at[DT];
  {
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      k_at[s] = (uint32_t) (col * ROWB + 16 * ((2 * s + half) ^ (col & 7)));
    }
    const int g = lane >> 4, j = (lane >> 2) & 3, q = lane & 3;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      v_at[t] = (uint32_t) ((4 * half + j) * ROWB + 16 * ((4 * t + 2 * (g & 1) + (q >> 1)) ^ (2 * j)) + 8 * (q & 1));
    }
  }
  typedef short v4s __attribute__((ext_vector_type(4)));

  v4h mreg[2][4], mnext[2][4];
  if (grp * kBK < kv_limit) {
    fetch(grp * kBK, 0);
    if (mask) {
      fetch_mask(mnext, grp * kBK);
    }
  }

  int it = 0;
  for (int kk = 0; kk < kv_limit; kk += GROUPS * kBK, ++it) {
    const int  k0   = kk + grp * kBK;  // this key group's block of the iteration
    const bool live = k0 < kv_limit;   // (the last iteration may have a block for the first group only)
    const int  buf  = it & 1;
    // this wave's share of the block has landed; behind the barrier everybody's has, and nobody reads the other
    // buffer (the previous block) any more
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (mask) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          mreg[kt][rg] = mnext[kt][rg];
        }
      }
    }
    if (k0 + GROUPS * kBK < kv_limit) {
      fetch(k0 + GROUPS * kBK, buf ^ 1);
      if (mask) {
        fetch_mask(mnext, k0 + GROUPS * kBK);
      }
    }
    if (!live) {
      continue;
    }
    const uint8_t *k_tile = sm.k[buf], *v_tile = sm.v[buf];

    // ---- S^T - m = K Q^T - m: two 32-key tiles, accumulated on top of minus the running maximum ----
    // Scores come out of the MFMA already relative to the maximum seen so far, so a block that brings no new maximum
    // to any query of the wave (the usual case after the first few blocks) needs no subtraction and no rescaling.
    const bool  fresh = m_run == -INFINITY;  // nothing visible yet for this query
    const float m_ref = fresh ? 0.0f : m_run;
    v16f st[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        st[kt][r] = -m_ref;
      }
    }
    // the two key tiles advance side by side (independent accumulators), and the fragments of step s + PF are
    // requested before the products of step s
    {
      constexpr int PF = 3;  // steps ahead (an LDS read takes longer to return than two steps' products to issue)
      v8h kf[PF + 1][2];
#pragma unroll
      for (int s = 0; s < PF && s < KSTEPS; ++s) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
          kf[s][kt] = *reinterpret_cast<const v8h *>(k_tile + k_at[s] + 32 * kt * ROWB);
        }
      }
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        if (s + PF < KSTEPS) {
#pragma unroll
          for (int kt = 0; kt < 2; ++kt) {
            kf[(s + PF) % (PF + 1)][kt] = *reinterpret_cast<const v8h *>(k_tile + k_at[s + PF] + 32 * kt * ROWB);
          }
        }
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
          st[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[s % (PF + 1)][kt], qf[s], st[kt], 0, 0, 0);
        }
      }
    }

    // ---- mask (lane = query; register r of tile kt is key k0 + 32 kt + 8 (r / 4) + 4 half + r % 4) ----
    // Only blocks that a mask, the causal diagonal or the end of the keys touches pay for it (the same for the
    // whole wave).
    if (mask != nullptr || k0 + kBK > kv_len || (causal && k0 + kBK - 1 > q_base + q_shift)) {
      const int last = vis_last - k0;  // registers whose key offset 32 kt + 8 (r / 4) + r % 4 exceeds it are hidden
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          float add[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
          if (mask) {
            const v4h mv = mreg[kt][rg];
            add[0] = mask_term(mv[0], mask_threshold), add[1] = mask_term(mv[1], mask_threshold);
            add[2] = mask_term(mv[2], mask_threshold), add[3] = mask_term(mv[3], mask_threshold);
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int r = 4 * rg + e;
            st[kt][r]   = (32 * kt + 8 * rg + e > last) ? -INFINITY : st[kt][r] + add[e];
          }
        }
      }
    }

    // ---- online softmax on scores relative to m_ref ----
    float mx = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        mx = fmaxf(mx, st[kt][r]);
      }
    }
    {
      // both 32-lane halves of the wave hold the same queries: v_permlane32_swap hands each the other's maximum
      const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
      mx            = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
    }
    // the first visible block of a query sets its maximum (either sign), later blocks only raise it
    const bool move = fresh ? (mx != -INFINITY) : (mx > 0.0f);
    if (__builtin_amdgcn_ballot_w64(move) != 0) {
      // (a statement the compiler cannot run ahead of the test: without it the 97 instructions below are turned into
      // selects and run for every block)
      asm volatile("" ::: "memory");
      const float delta = move ? mx : 0.0f;
      const float alpha = fresh ? 0.0f : fast_exp2(-delta);  // O and l of a fresh query are still zero
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          st[kt][r] -= delta;
        }
      }
#pragma unroll
      for (int t = 0; t < DT; ++t) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          oacc[t][r] *= alpha;
        }
      }
      l_run *= alpha;
      m_run = move ? m_ref + mx : m_run;
    }
    // the probabilities, rounded to fp16 in pairs as the matrix instruction takes them; the row sum adds up the
    // rounded values (v_dot2_f32_f16 with ones: two per instruction, fp32 sums), so O and l see the same numbers
    uint32_t pk[2][8];
    float    psum[4] = { 0.0f, 0.0f, 0.0f, 0.0f };  // (four chains: an addition waits for the one before it in its chain)
    {
      const v2h ones = { (_Float16) 1.0f, (_Float16) 1.0f };
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const v2h p2  = { (_Float16) fast_exp2(st[kt][r]), (_Float16) fast_exp2(st[kt][r + 1]) };
          pk[kt][r / 2] = __builtin_bit_cast(uint32_t, p2);
          psum[(r / 2) & 3] = __builtin_amdgcn_fdot2(p2, ones, psum[(r / 2) & 3], false);
        }
      }
    }
    l_run += (psum[0] + psum[1]) + (psum[2] + psum[3]);

    // ---- O^T += V^T P^T ----
    // MFMA (kt, u) covers keys 32 kt + 16 u + {4 half + 0..3, 8 + 4 half + 0..3}: exactly registers 8 u .. 8 u + 7
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const v8h pf = __builtin_bit_cast(v8h, make_uint4(pk[kt][4 * u], pk[kt][4 * u + 1], pk[kt][4 * u + 2], pk[kt][4 * u + 3]));
#pragma unroll
        for (int t = 0; t < DT; ++t) {
          // (V^T fragment: column 32 t + lane % 32 of keys 32 kt + 16 u + 4 half + 0 .. 3 and + 8 .. 11)
          const uint8_t *at = v_tile + v_at[t] + (32 * kt + 16 * u) * ROWB;
          const v4s a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *) at);
          const v4s a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *) (at + 8 * ROWB));
          const v8h vf = __builtin_bit_cast(v8h, (short __attribute__((ext_vector_type(8)))){ a0[0], a0[1], a0[2], a0[3],
                                                                                             a1[0], a1[1], a1[2], a1[3] });
          oacc[t]      = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf, oacc[t], 0, 0, 0);
        }
      }
    }
  }

  // ---- the second key group hands its state over: m, l and O of the same query, lane for lane ----
  float l_tot = l_run + __shfl_xor(l_run, 32, kWave);
  if constexpr (GROUPS == 2) {
    constexpr int STATE = 16 * DT + 2;  // floats per lane
    static_assert((size_t) (kPfThreads / kWave) * STATE * kWave * sizeof(float) <= sizeof(sm_all),
                  "the handed-over state fits the K/V tiles");
    float *xch = reinterpret_cast<float *>(&sm_all[0]) + (size_t) wave * STATE * kWave + lane;
    __syncthreads();  // everybody is done with the tiles
    if (grp == 1) {
      xch[0] = m_run, xch[kWave] = l_tot;
#pragma unroll
      for (int t = 0; t < DT; ++t) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          xch[(2 + 16 * t + r) * kWave] = oacc[t][r];
        }
      }
    }
    __syncthreads();
    if (grp == 1) {
      return;
    }
    const float m1 = xch[0], l1 = xch[kWave];
    const float m_all  = fmaxf(m_run, m1);
    const float m_safe = (m_all == -INFINITY) ? 0.0f : m_all;  // nothing visible at all: keep the exponents finite
    const float a0 = fast_exp2(m_run - m_safe), a1 = fast_exp2(m1 - m_safe);
    l_tot          = a0 * l_tot + a1 * l1;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        oacc[t][r] = a0 * oacc[t][r] + a1 * xch[(2 + 16 * t + r) * kWave];
      }
    }
  }

  // ---- finish: O = O^T / l, one query per lane; register r of tile t is d = 32 t + 8 (r / 4) + 4 half + r % 4 ----
  const float inv   = 1.0f / l_tot;
  if (q_ok) {
    const size_t base = (size_t) q_row * qo_stride + (size_t) head * D;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const int d0 = 32 * t + 8 * rg + 4 * half;
        float     v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = oacc[t][4 * rg + e] * inv;
        }
        if (QO_F32) {
          *reinterpret_cast<float4 *>(reinterpret_cast<float *>(o_ptr) + base + d0) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
          v4h hv = { (_Float16) v[0], (_Float16) v[1], (_Float16) v[2], (_Float16) v[3] };
          *reinterpret_cast<v4h *>(reinterpret_cast<_Float16 *>(o_ptr) + base + d0) = hv;
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------ decode

constexpr int kDecWaveKeys = 32;  // keys of one wave: two 16-key score tiles = one k step of P V
constexpr int kDecMaxGroup = 8;   // query heads scored per pass against one K/V stream
constexpr int kDecSplit    = 128; // keys per workgroup (four waves) ...
constexpr int kDecSplitShort = 64;  // ... and for short contexts (two waves), where 128 would leave most CUs without a workgroup

// partial record per (head, split): m, l, then D floats of un-normalised O.
// A workgroup owns SPLIT consecutive keys of one KV head; each of its SPLIT / 32 waves owns 32 of them and works
// without the others until the end. Both products run on the matrix cores (v_mfma_f32_16x16x32_f16), with up to 16
// query heads of the GQA group as the 16 rows (columns) of a tile:
//  * scores S = K Q^T: K in the A operand as it lies in memory (a lane loads 16 bytes of a key row per k step, all of
//    a wave's K loads issued before the first use); the queries in the B operand, fp32 queries scaled and split into an
//    fp16 pair (two instructions per k step: the scores are those of the fp32 queries to about 2^-22), fp16 queries as
//    they are with the scale applied to the score. A lane then holds, for one head, the scores of 4 keys per tile.
//  * softmax against the wave's own maximum, in those registers; rounded to fp16 they ARE the A operand of
//  * O = P V: the contraction runs over the wave's 32 keys, key 16 t + 4 g + i (tile t, lane group g, register i)
//    in k slot 8 g + 4 t + i. V is the B operand: a lane needs 8 keys at one column. The V rows come into LDS as they
//    are by DMA (global_load_lds, no registers), and ds_read_b64_tr_b16 hands each lane of a 16-lane group one column
//    of the 4 rows x 16 columns that the group's lanes point at (lanes 4 j .. 4 j + 3 at the four 8-byte pieces of
//    row j). Within a row the 32-byte pieces are stored exclusive-or'ed with the row number's low bits (the DMA
//    chooses what each lane fetches, not where it lands), so the four rows of a read lie in different banks.
// The waves' (max, sum, O) are put together through LDS with the factor exp2(m_wave - m_all) per wave and head.
// Measured on MI355X (32 query / 8 KV heads of 128, cold K/V; the split-KV launch alone, kv_len 4096 / 16384): all on
// the vector ALU (8 multiply-adds, 4 lane exchanges and an exponential per key, head and lane) 7.5 / 17.0 us; scores on
// the matrix cores and P V with v_dot2_f32_f16 6.3 / 15.3 us; this version: see the launcher. A variant in which a
// workgroup walks several chunks of keys with the next chunk on its way, about one workgroup per compute unit, was
// slower (17.0 us at 16384), and so was merging inside this launch behind a ticket per KV head (18-19 us at 4096).
template <int D, int GH, bool QO_F32, int SPLIT>
__global__ __launch_bounds__(SPLIT / kDecWaveKeys * kWave) void flash_attn_decode_kernel(
  float *__restrict__ part, const void *__restrict__ q_ptr, const _Float16 *__restrict__ k_ptr,
  const _Float16 *__restrict__ v_ptr, const _Float16 *__restrict__ mask, int kv_len, int n_heads, int n_kv_heads,
  int head0_in_group, int n_splits, int mask_threshold) {
  constexpr int WAVES   = SPLIT / kDecWaveKeys;
  constexpr int THREADS = WAVES * kWave;
  constexpr int KSTEPS  = D / 32;  // k steps of a score tile
  constexpr int CT      = D / 16;  // 16-column tiles of O
  constexpr int ROWB    = D * 2;   // bytes of a K or V row
  constexpr int CHUNKS  = ROWB / 16;            // 16-byte pieces of a row
  constexpr int DMA_ROWS = 1024 / ROWB;         // rows per DMA instruction (1 KiB)
  constexpr int DMAS    = kDecWaveKeys / DMA_ROWS;
  static_assert(GH <= 16 && (D == 64 || D == 128), "heads are the 16 rows of a tile");
  typedef float v4f __attribute__((ext_vector_type(4)));
  typedef short v4s __attribute__((ext_vector_type(4)));
  // LDS: V rows [SPLIT][D] halfs (wave w: rows 32 w ..), then o_w[WAVES][GH][D], red_l[WAVES][GH], red_m[WAVES][GH]
  extern __shared__ __align__(1024) uint8_t dec_lds[];
  float *o_sh  = reinterpret_cast<float *>(dec_lds + SPLIT * ROWB);
  float *red_l = o_sh + WAVES * GH * D, *red_m = red_l + WAVES * GH;

  const int group = n_heads / n_kv_heads;
  const int h_kv  = blockIdx.y;
  const int split = blockIdx.x;
  const int lane  = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col   = lane & 15;   // head of the pass (scores, P), column of the tile (V, O)
  const int kg    = lane >> 4;   // lane group: which 8 of a k step's 32 slots; rows 4 kg .. 4 kg + 3 of a result
  const float scale = (1.0f / sqrtf((float) D)) * kLog2e;
  const size_t kv_stride = (size_t) n_kv_heads * D;

  const int k_end  = min(kv_len, (split + 1) * SPLIT);
  const int k_wave = split * SPLIT + wave * kDecWaveKeys;  // this wave's keys: k_wave + 0 .. 31; keys from k_end on are
                                                           // read as key k_end - 1 and score -inf

  // V first (loads return in order: the K loads the compiler counts are then the youngest, and its waits for them
  // also cover these). DMA instruction i brings rows DMA_ROWS i .. of the wave's 32; lane L lands at byte 16 L of
  // that KiB = row L / CHUNKS, piece L % CHUNKS, and fetches the piece that belongs there.
  uint8_t *v_wave = dec_lds + wave * kDecWaveKeys * ROWB;
  {
    const uint32_t to = (uint32_t) (uintptr_t) v_wave;
#pragma unroll
    for (int i = 0; i < DMAS; ++i) {
      const int row   = i * DMA_ROWS + lane / CHUNKS;
      const int piece = (lane % CHUNKS) ^ (2 * (row & 3));  // (32-byte pieces exclusive-or'ed with the row's low bits)
      const int key   = min(k_wave + row, k_end - 1);
      const _Float16 *src = v_ptr + (size_t) key * kv_stride + (size_t) h_kv * D + 8 * piece;
      asm volatile("s_mov_b32 m0, %1\n s_nop 0\n global_load_lds_dwordx4 %0, off" ::"v"(src), "s"(to + (uint32_t) (i * 1024)) : "memory");
    }
  }
  // the queries: head `col` of the pass, dims 32 s + 8 kg .. + 7
  v8h qf[KSTEPS], qf_lo[KSTEPS];
  {
    const bool   q_on = col < GH && head0_in_group + col < group;
    const size_t base = (size_t) (h_kv * group + min(head0_in_group + col, group - 1)) * D + 8 * kg;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      if (QO_F32) {
        const float4 *qp = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(q_ptr) + base + 32 * s);
        const float4  q0 = qp[0], q1 = qp[1];
        const float   on   = q_on ? scale : 0.0f;
        const float   x[8] = { q0.x * on, q0.y * on, q0.z * on, q0.w * on, q1.x * on, q1.y * on, q1.z * on, q1.w * on };
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          qf[s][e]    = (_Float16) x[e];
          qf_lo[s][e] = (_Float16) (x[e] - (float) qf[s][e]);
        }
      } else {
        const v8h qv = *reinterpret_cast<const v8h *>(reinterpret_cast<const _Float16 *>(q_ptr) + base + 32 * s);
        qf[s]        = q_on ? qv : (v8h){ 0, 0, 0, 0, 0, 0, 0, 0 };
        qf_lo[s]     = (v8h){ 0, 0, 0, 0, 0, 0, 0, 0 };  // (not used)
      }
    }
  }
  // K: row `col` of tile t is key 16 t + col of the wave
  v8h kf[2][KSTEPS];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int    key = min(k_wave + 16 * t + col, k_end - 1);
    const size_t off = (size_t) key * kv_stride + (size_t) h_kv * D + 8 * kg;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      kf[t][s] = *reinterpret_cast<const v8h *>(k_ptr + off + 32 * s);
    }
  }
  // row 0 of the mask (qo_len == 1) for the 8 keys of this lane, requested with the rest
  float mk[2][4];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = k_wave + 16 * t + 4 * kg + i;
      mk[t][i] = (mask && key < k_end) ? mask_term(mask[key], mask_threshold != 0) : 0.0f;
    }
  }

  // scores of head `col` for keys 16 t + 4 kg + i
  float sc[2][4];
  float m_w = -INFINITY;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    v4f acc = { 0.0f, 0.0f, 0.0f, 0.0f };
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[t][s], qf[s], acc, 0, 0, 0);
      if (QO_F32) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[t][s], qf_lo[s], acc, 0, 0, 0);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool  live = k_wave + 16 * t + 4 * kg + i < k_end;
      const float v    = (QO_F32 ? acc[i] : acc[i] * scale) + mk[t][i];
      sc[t][i]         = live ? v : -INFINITY;
      m_w              = fmaxf(m_w, sc[t][i]);
    }
  }
  // the wave's maximum of head `col`: over the four lane groups
  m_w = fmaxf(m_w, __shfl_xor(m_w, 16, kWave));
  m_w = fmaxf(m_w, __shfl_xor(m_w, 32, kWave));
  const float m_safe = (m_w == -INFINITY) ? 0.0f : m_w;
  float       l_w    = 0.0f;
  v8h         pf;  // A operand of P V: k slot 8 kg + 4 t + i
#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float pr = fast_exp2(sc[t][i] - m_safe);
      l_w += pr;
      pf[4 * t + i] = (_Float16) pr;
    }
  }
  l_w += __shfl_xor(l_w, 16, kWave);
  l_w += __shfl_xor(l_w, 32, kWave);
  if (kg == 0 && col < GH) {
    red_m[wave * GH + col] = m_w;
    red_l[wave * GH + col] = l_w;
  }

  // O = P V. (Every load of this wave has returned by now: the K loads were the youngest. The wait is written out
  // because the compiler knows nothing of the DMA.) Read h of tile c: lane (group kg, col = 4 j + q) points at row
  // 16 h + 4 kg + j, halfs 16 c + 4 q .. + 3, and receives column 16 c + col of rows 16 h + 4 kg + 0 .. 3.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  v4f oacc[CT];
  {
    const int j = col >> 2, q = col & 3;
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      v4s b[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int row   = 16 * h + 4 * kg + j;
        const int piece = (2 * c + (q >> 1)) ^ (2 * (row & 3));
        const uint8_t *at = v_wave + row * ROWB + piece * 16 + 8 * (q & 1);
        b[h] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *) at);
      }
      const v8h bf = __builtin_bit_cast(v8h, (short __attribute__((ext_vector_type(8)))){ b[0][0], b[0][1], b[0][2], b[0][3],
                                                                                           b[1][0], b[1][1], b[1][2], b[1][3] });
      const v4f zero = { 0.0f, 0.0f, 0.0f, 0.0f };
      oacc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pf, bf, zero, 0, 0, 0);
    }
  }
  // rows 4 kg + i of the result are heads: this lane's column 16 c + col of each
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int g = 4 * kg + i;
    if (g < GH) {
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        o_sh[((size_t) wave * GH + g) * D + 16 * c + col] = oacc[c][i];
      }
    }
  }
  __syncthreads();
  // put the waves together, each with its factor: two neighbouring columns per thread
  for (int i = threadIdx.x * 2; i < GH * D; i += THREADS * 2) {
    const int g = i / D, d = i % D;
    if (head0_in_group + g >= group) {
      continue;
    }
    float m_all = red_m[g];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) {
      m_all = fmaxf(m_all, red_m[w * GH + g]);
    }
    const float m_ref = (m_all == -INFINITY) ? 0.0f : m_all;
    float       v0 = 0.0f, v1 = 0.0f, l = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float  f = fast_exp2(red_m[w * GH + g] - m_ref);
      const float2 x = *reinterpret_cast<const float2 *>(o_sh + ((size_t) w * GH + g) * D + d);
      l += red_l[w * GH + g] * f;
      v0 += x.x * f, v1 += x.y * f;
    }
    const int head = h_kv * group + head0_in_group + g;
    float    *rec  = part + ((size_t) head * n_splits + split) * (D + 2);
    *reinterpret_cast<float2 *>(rec + 2 + d) = make_float2(v0, v1);
    if (d == 0) {
      *reinterpret_cast<float2 *>(rec) = make_float2(m_all, l);
    }
  }
}

// One workgroup per head: MG groups of D threads, one thread per output column in each; group j merges the j-th part
// of the splits, then the groups' (max, sum, column) are put together through LDS (MG = 1: nothing to put together;
// measured at 32 heads of 128: 32 splits 3.2 us with one group, 4.2 with four; 128 splits 5.7 and 4.0). A group takes its splits
// 64 at a time with every load of a chunk -- the (max, sum) pair of split `lane` and this thread's column of all 64
// records -- requested before the first use, so a chunk costs one trip to memory (kv_len up to 32768 at 128 keys per
// split: the whole merge is one trip). Each wave works the rescale factors out for itself (lane s holds that of split
// s, read back with v_readlane); chunks are folded into a running (max, sum, column) like KV blocks are.
constexpr int kMergeChunk  = 64;
constexpr int kMergeGroups = 4;  // for more than kMergeChunk splits

template <int D, bool QO_F32, int MG>
__global__ __launch_bounds__(D *MG) void flash_attn_decode_merge_kernel(void *__restrict__ o_ptr,
                                                                        const float *__restrict__ part, int n_splits,
                                                                        uint8_t *__restrict__ q8_out) {
  // (q8_out, fp32 output only: the output row is also written as Q8_0 blocks, the bytes the Q8_0 quantizer makes of
  // it; a block is 32 neighbouring columns, one half of a wave)
  extern __shared__ float merge_lds[];  // MG > 1 only: the groups' columns [MG][D], then their (max, sum) [MG][2]
  static_assert(D % kWave == 0, "a wave lies in one group");
  const int    head = blockIdx.x, d = threadIdx.x % D, lane = threadIdx.x & (kWave - 1);
  // (the same for the whole wave, and known to be: the bounds below then stay in scalar registers and the 64 loads of a
  // chunk are switched by scalar branches instead of one lane mask each)
  const int    grp  = __builtin_amdgcn_readfirstlane((int) threadIdx.x / D);
  const float *rec0 = part + (size_t) head * n_splits * (D + 2);
  const int    per  = (n_splits + MG - 1) / MG;  // splits of a group
  const int    s_begin = grp * per, s_end = min(n_splits, s_begin + per);
  float        m_run = -INFINITY, l_run = 0.0f, v_run = 0.0f;
  for (int s0 = s_begin; s0 < s_end; s0 += kMergeChunk) {
    const int  left = s_end - s0;  // >= 1
    const bool mine = lane < kMergeChunk && lane < left;
    float      m_s = -INFINITY, l_s = 0.0f;
    if (mine) {
      const float2 ml = *reinterpret_cast<const float2 *>(rec0 + (size_t) (s0 + lane) * (D + 2));
      m_s = ml.x, l_s = ml.y;
    }
    float x[kMergeChunk];
#pragma unroll
    for (int u = 0; u < kMergeChunk; ++u) {
      x[u] = u < left ? rec0[(size_t) (s0 + u) * (D + 2) + 2 + d] : 0.0f;
    }
    const float m_new  = fmaxf(m_run, wave_max(m_s));
    const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
    const float keep   = fast_exp2(m_run - m_safe);  // 0 for the first chunk
    const float f      = fast_exp2(m_s - m_safe);    // 0 in lanes without a split
    l_run              = l_run * keep + wave_sum(l_s * f);
    float v            = 0.0f;
#pragma unroll
    for (int u = 0; u < kMergeChunk; ++u) {
      v += x[u] * __int_as_float(__builtin_amdgcn_readlane(__float_as_int(f), u));
    }
    v_run = v_run * keep + v;
    m_run = m_new;
  }
  if (MG > 1) {
    float *grp_v = merge_lds, *grp_ml = merge_lds + MG * D;
    grp_v[grp * D + d] = v_run;
    if (d == 0) {
      grp_ml[2 * grp] = m_run, grp_ml[2 * grp + 1] = l_run;
    }
    __syncthreads();
    if (grp != 0) {
      return;
    }
    float m_all = grp_ml[0];
#pragma unroll
    for (int j = 1; j < MG; ++j) {
      m_all = fmaxf(m_all, grp_ml[2 * j]);
    }
    const float m_safe = (m_all == -INFINITY) ? 0.0f : m_all;
    l_run = 0.0f, v_run = 0.0f;
#pragma unroll
    for (int j = 0; j < MG; ++j) {  // (a group without splits has m = -inf, l = v = 0)
      const float f = fast_exp2(grp_ml[2 * j] - m_safe);
      l_run += grp_ml[2 * j + 1] * f;
      v_run += grp_v[j * D + d] * f;
    }
  }
  const float out = v_run * (1.0f / l_run);
  if (QO_F32) {
    reinterpret_cast<float *>(o_ptr)[(size_t) head * D + d] = out;
    if (q8_out != nullptr) {
      float amax = fabsf(out);
#define HTPOPS_DPP_MAX(ctrl) \
  amax = fmaxf(amax, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(amax), __float_as_int(amax), ctrl, 0xf, 0xf, false)))
      HTPOPS_DPP_MAX(0xB1);   // quad_perm [1,0,3,2]
      HTPOPS_DPP_MAX(0x4E);   // quad_perm [2,3,0,1]
      HTPOPS_DPP_MAX(0x141);  // row_half_mirror
      HTPOPS_DPP_MAX(0x140);  // row_mirror: the 16 lanes of a row
#undef HTPOPS_DPP_MAX
      amax            = fmaxf(amax, __shfl_xor(amax, 16, kWave));  // the two rows of the block
      const float dq  = amax / 127.0f;
      const float id  = (dq != 0.0f) ? 1.0f / dq : 0.0f;
      const int   col = head * D + d;
      uint8_t    *blk = q8_out + (size_t) (col >> 5) * 34;
      blk[2 + (col & 31)] = (uint8_t) (int) roundf(out * id);
      if ((col & 31) == 0) {
        *reinterpret_cast<uint16_t *>(blk) = __half_as_ushort(__float2half_rn(dq));
      }
    }
  } else {
    reinterpret_cast<_Float16 *>(o_ptr)[(size_t) head * D + d] = (_Float16) out;
  }
}

// ------------------------------------------------------------------------------------------------ any even head_dim

// Head dims the MFMA kernels above are not built for (anything but 64 and 128; the reference routes head_dim % 64 != 0
// to its own variant, src/dsp/ops/flash_attn_sp_hdim.c:782-832, which only asks for an even head_dim). One workgroup
// per (query row, head); its four waves take every fourth 64-key block, with one key per lane for the scores (dot
// products of fp16 pairs, v_dot2_f32_f16) and one output column per lane (d = lane + 64 i) for O += p V, then merge their
// (max, sum, O) through LDS. Built for coverage, not speed: K rows are read straight from global memory.
constexpr int kGenThreads = 256;
constexpr int kGenMaxD    = 256;

template <bool QO_F32>
__global__ __launch_bounds__(kGenThreads) void flash_attn_any_dim_kernel(void *__restrict__ o_ptr,
                                                                         const void *__restrict__ q_ptr,
                                                                         const _Float16 *__restrict__ k_ptr,
                                                                         const _Float16 *__restrict__ v_ptr,
                                                                         const _Float16 *__restrict__ mask, int qo_len,
                                                                         int kv_len, int n_heads, int n_kv_heads,
                                                                         int head_dim, int flags) {
  const bool causal = (flags & 1) != 0, mask_threshold = (flags & 2) != 0;
  __shared__ v2h   q_sh[kGenMaxD / 2];
  __shared__ float part_o[4][kGenMaxD];
  __shared__ float part_ml[4][2];

  const int D     = head_dim;
  const int tid   = threadIdx.x;
  const int lane  = tid & 63;
  const int wave  = tid >> 6;
  const int row   = blockIdx.x;
  const int head  = blockIdx.y;
  const int h_kv  = head / (n_heads / n_kv_heads);
  const float scale = (1.0f / sqrtf((float) D)) * kLog2e;
  const size_t qo_base   = ((size_t) row * n_heads + head) * D;
  const size_t kv_stride = (size_t) n_kv_heads * D;
  const size_t mask_ld   = ((size_t) kv_len + 63) / 64 * 64;

  // the scaled query, rounded to fp16 like the MFMA kernels' B operand
  for (int i = tid; i < D / 2; i += kGenThreads) {
    float a, b;
    if (QO_F32) {
      a = reinterpret_cast<const float *>(q_ptr)[qo_base + 2 * i];
      b = reinterpret_cast<const float *>(q_ptr)[qo_base + 2 * i + 1];
    } else {
      a = (float) reinterpret_cast<const _Float16 *>(q_ptr)[qo_base + 2 * i];
      b = (float) reinterpret_cast<const _Float16 *>(q_ptr)[qo_base + 2 * i + 1];
    }
    q_sh[i] = v2h{ (_Float16) (a * scale), (_Float16) (b * scale) };
  }
  __syncthreads();

  const int kv_vis = causal ? min(kv_len, row + (kv_len - qo_len) + 1) : kv_len;  // keys 0 .. kv_vis - 1 are visible
  float m_run = -INFINITY, l_run = 0.0f;
  float acc[kGenMaxD / 64] = { 0.0f, 0.0f, 0.0f, 0.0f };
  for (int k0 = wave * 64; k0 < kv_vis; k0 += 4 * 64) {
    const int  key = k0 + lane;
    const bool on  = key < kv_vis;
    float      s   = -INFINITY;
    if (on) {
      const v2h *kr = reinterpret_cast<const v2h *>(k_ptr + (size_t) key * kv_stride + (size_t) h_kv * D);
      float      d0 = 0.0f, d1 = 0.0f;
      int        i  = 0;
      for (; i + 1 < D / 2; i += 2) {
        d0 = __builtin_amdgcn_fdot2(q_sh[i], kr[i], d0, false);
        d1 = __builtin_amdgcn_fdot2(q_sh[i + 1], kr[i + 1], d1, false);
      }
      if (i < D / 2) {
        d0 = __builtin_amdgcn_fdot2(q_sh[i], kr[i], d0, false);
      }
      s = d0 + d1;
      if (mask) {
        s += mask_term(mask[(size_t) row * mask_ld + key], mask_threshold);
      }
    }
    float mx = s;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
    }
    const float m_new  = fmaxf(m_run, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;  // everything masked so far: keep exp2 arguments finite
    const float alpha  = fast_exp2(m_run - m_safe);
    const float p      = fast_exp2(s - m_safe);  // 0 for hidden keys
    float       psum   = p;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      psum += __shfl_xor(psum, off, kWave);
    }
    l_run = l_run * alpha + psum;
    m_run = m_new;
#pragma unroll
    for (int i = 0; i < kGenMaxD / 64; ++i) {
      acc[i] *= alpha;
    }
    const int n_keys = min(64, kv_vis - k0);
    for (int j = 0; j < n_keys; ++j) {
      const float     pj = __shfl(p, j, kWave);
      const _Float16 *vr = v_ptr + (size_t) (k0 + j) * kv_stride + (size_t) h_kv * D;
#pragma unroll
      for (int i = 0; i < kGenMaxD / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < D) {
          acc[i] += pj * (float) vr[d];
        }
      }
    }
  }

  // merge the four waves
  if (lane == 0) {
    part_ml[wave][0] = m_run;
    part_ml[wave][1] = l_run;
  }
#pragma unroll
  for (int i = 0; i < kGenMaxD / 64; ++i) {
    part_o[wave][lane + 64 * i] = acc[i];
  }
  __syncthreads();
  float m_all = -INFINITY;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    m_all = fmaxf(m_all, part_ml[w][0]);
  }
  const float m_safe = (m_all == -INFINITY) ? 0.0f : m_all;
  float       l_all  = 0.0f;
  float       wgt[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    wgt[w] = fast_exp2(part_ml[w][0] - m_safe);
    l_all += wgt[w] * part_ml[w][1];
  }
  for (int d = tid; d < D; d += kGenThreads) {
    float o = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      o += wgt[w] * part_o[w][d];
    }
    o /= l_all;
    if (QO_F32) {
      reinterpret_cast<float *>(o_ptr)[qo_base + d] = o;
    } else {
      reinterpret_cast<_Float16 *>(o_ptr)[qo_base + d] = (_Float16) o;
    }
  }
}

template <int D, bool QO_F32>
hipError_t launch_prefill(hipStream_t stream, void *o, const void *q, const void *k, const void *v, const void *mask,
                          int qo_len, int kv_len, int n_heads, int n_kv_heads, bool causal, int forced, bool mask_threshold) {
  const int group      = n_heads / n_kv_heads;
  const int gc         = group < 4 ? group : 4;
  const int qsub       = 4 / gc;
  const int sub_groups = (group + gc - 1) / gc;
  const unsigned q_blocks = (unsigned) ((qo_len + qsub * kBQ - 1) / (qsub * kBQ));
  if (q_blocks > 65535u) {
    return hipErrorInvalidValue;
  }
  const dim3 grid((unsigned) (n_kv_heads * sub_groups), q_blocks);
  // Two key groups per workgroup when the grid leaves CUs without a second workgroup, or (causal) when the workgroups
  // all fit at once and their uneven lengths would leave the long ones running alone. Measured on the 256-CU device,
  // 32 query / 8 KV heads of 128: 2048 x 2048 causal 59 us against 65 us, 1024 x 1024 without `causal` 30 against
  // 33 us; but 2048 x 2048 without `causal` 101 against 92 us.
  constexpr unsigned kCus = 256;
  const unsigned     wgs  = grid.x * grid.y;
  const bool         two  = forced ? forced == 2 : (wgs <= kCus || (causal && wgs <= 2 * kCus));
  if (two) {
    hipLaunchKernelGGL((flash_attn_prefill_kernel<D, QO_F32, 2>), grid, dim3(kPfThreads * 2), 0, stream, o, q,
                       (const _Float16 *) k, (const _Float16 *) v, (const _Float16 *) mask, qo_len, kv_len, n_heads,
                       n_kv_heads, (causal ? 1 : 0) | (mask_threshold ? 2 : 0));
  } else {
    hipLaunchKernelGGL((flash_attn_prefill_kernel<D, QO_F32, 1>), grid, dim3(kPfThreads), 0, stream, o, q,
                       (const _Float16 *) k, (const _Float16 *) v, (const _Float16 *) mask, qo_len, kv_len, n_heads,
                       n_kv_heads, (causal ? 1 : 0) | (mask_threshold ? 2 : 0));
  }
  return hipGetLastError();
}

template <int D, int GH, bool QO_F32, int SPLIT>
hipError_t launch_decode_pass(hipStream_t stream, dim3 grid, float *workspace, const void *q, const void *k, const void *v,
                              const void *mask, int kv_len, int n_heads, int n_kv_heads, int h0, int n_splits,
                              bool mask_threshold) {
  constexpr int    kWaves = SPLIT / kDecWaveKeys;
  // (the V rows; the waves' O, their sums and maxima)
  constexpr size_t kLds = (size_t) SPLIT * D * 2 + ((size_t) kWaves * GH * D + 2 * (size_t) kWaves * GH) * sizeof(float);
  static_assert(kLds <= 64 * 1024, "dynamic LDS without raising the limit");
  hipLaunchKernelGGL((flash_attn_decode_kernel<D, GH, QO_F32, SPLIT>), grid, dim3(kWaves * kWave), kLds, stream, workspace,
                     q, (const _Float16 *) k, (const _Float16 *) v, (const _Float16 *) mask, kv_len, n_heads, n_kv_heads,
                     h0, n_splits, mask_threshold ? 1 : 0);
  return hipGetLastError();
}

template <int D, bool QO_F32>
hipError_t launch_decode(hipStream_t stream, void *o, const void *q, const void *k, const void *v, const void *mask,
                         int kv_len, int n_heads, int n_kv_heads, float *workspace, void *q8_out, bool mask_threshold,
                         int parts = 3) {  // (bit 0: the split-KV launch, bit 1: the merge launch)
  const int  group    = n_heads / n_kv_heads;
  // 64-key chunks while 128-key ones would give fewer than 128 workgroups (measured at 8 KV heads: kv = 512 8.8 -> 7.1 us;
  // kv = 4096 and 16384 are 1 and 6 us slower with 64)
  const bool short_kv = (long) ((kv_len + kDecSplit - 1) / kDecSplit) * n_kv_heads < 128;
  const int  split    = short_kv ? kDecSplitShort : kDecSplit;
  const int  n_splits = (kv_len + split - 1) / split;
  const dim3 grid((unsigned) n_splits, (unsigned) n_kv_heads);
  for (int h0 = 0; h0 < group && (parts & 1); h0 += kDecMaxGroup) {
    const int  gh = group - h0;
    hipError_t e;
#define HTPOPS_DECODE(GH)                                                                                           \
  e = short_kv ? launch_decode_pass<D, GH, QO_F32, kDecSplitShort>(stream, grid, workspace, q, k, v, mask, kv_len, n_heads, \
                                                                  n_kv_heads, h0, n_splits, mask_threshold) :      \
                 launch_decode_pass<D, GH, QO_F32, kDecSplit>(stream, grid, workspace, q, k, v, mask, kv_len, n_heads,  \
                                                              n_kv_heads, h0, n_splits, mask_threshold)
    if (gh > 4) {
      HTPOPS_DECODE(8);
    } else if (gh > 2) {
      HTPOPS_DECODE(4);
    } else if (gh == 2) {
      HTPOPS_DECODE(2);
    } else {
      HTPOPS_DECODE(1);
    }
#undef HTPOPS_DECODE
    if (e != hipSuccess) {
      return e;
    }
  }
  if (!(parts & 2)) {
    return hipGetLastError();
  }
  uint8_t *q8 = QO_F32 ? static_cast<uint8_t *>(q8_out) : nullptr;
  if (n_splits > kMergeChunk) {
    hipLaunchKernelGGL((flash_attn_decode_merge_kernel<D, QO_F32, kMergeGroups>), dim3((unsigned) n_heads),
                       dim3(D * kMergeGroups), (size_t) kMergeGroups * (D + 2) * sizeof(float), stream, o, workspace,
                       n_splits, q8);
  } else {
    hipLaunchKernelGGL((flash_attn_decode_merge_kernel<D, QO_F32, 1>), dim3((unsigned) n_heads), dim3(D), 0, stream, o,
                       workspace, n_splits, q8);
  }
  return hipGetLastError();
}

}  // namespace

bool flash_attn_writes_q8_0(int qo_len, int head_dim, bool qo_is_f32) {
  return qo_len == 1 && qo_is_f32 && (head_dim == 64 || head_dim == 128);
}

size_t flash_attn_workspace_bytes(int qo_len, int kv_len, int n_heads, int head_dim) {
  if (qo_len != 1 || (head_dim != 64 && head_dim != 128)) {
    return 0;
  }
  const size_t n_splits = ((size_t) kv_len + kDecSplitShort - 1) / kDecSplitShort;  // the most there can be
  return (size_t) n_heads * n_splits * ((size_t) head_dim + 2) * sizeof(float);
}

hipError_t launch_flash_attn_decode_part(hipStream_t stream, int part, void *o, const void *q, const void *k,
                                         const void *v, int kv_len, int n_heads, int n_kv_heads, int head_dim,
                                         bool qo_is_f32, void *workspace) {
  if ((head_dim != 64 && head_dim != 128) || (part != 1 && part != 2) || !workspace) {
    return hipErrorNotSupported;
  }
  float *ws = static_cast<float *>(workspace);
  if (head_dim == 128) {
    return qo_is_f32 ? launch_decode<128, true>(stream, o, q, k, v, nullptr, kv_len, n_heads, n_kv_heads, ws, nullptr, false, part) :
                       launch_decode<128, false>(stream, o, q, k, v, nullptr, kv_len, n_heads, n_kv_heads, ws, nullptr, false, part);
  }
  return qo_is_f32 ? launch_decode<64, true>(stream, o, q, k, v, nullptr, kv_len, n_heads, n_kv_heads, ws, nullptr, false, part) :
                     launch_decode<64, false>(stream, o, q, k, v, nullptr, kv_len, n_heads, n_kv_heads, ws, nullptr, false, part);
}

hipError_t launch_flash_attn(hipStream_t stream, void *o, const void *q, const void *k, const void *v,
                             const void *mask, int qo_len, int kv_len, int n_heads, int n_kv_heads, int head_dim,
                             bool qo_is_f32, bool causal, void *workspace, void *q8_out, int forced_key_groups,
                             bool mask_threshold) {
  if (head_dim != 64 && head_dim != 128) {
    if (head_dim <= 0 || head_dim % 2 != 0 || head_dim > kGenMaxD || qo_len > 0x7fffffff || n_heads > 65535) {
      return hipErrorNotSupported;
    }
    const dim3 grid((unsigned) qo_len, (unsigned) n_heads);
    if (qo_is_f32) {
      hipLaunchKernelGGL(flash_attn_any_dim_kernel<true>, grid, dim3(kGenThreads), 0, stream, o, q,
                         (const _Float16 *) k, (const _Float16 *) v, (const _Float16 *) mask, qo_len, kv_len, n_heads,
                         n_kv_heads, head_dim, (causal ? 1 : 0) | (mask_threshold ? 2 : 0));
    } else {
      hipLaunchKernelGGL(flash_attn_any_dim_kernel<false>, grid, dim3(kGenThreads), 0, stream, o, q,
                         (const _Float16 *) k, (const _Float16 *) v, (const _Float16 *) mask, qo_len, kv_len, n_heads,
                         n_kv_heads, head_dim, (causal ? 1 : 0) | (mask_threshold ? 2 : 0));
    }
    return hipGetLastError();
  }
  // with a single query row the causal rule (key j visible iff j <= kv_len - 1) hides nothing
  if (qo_len == 1) {
    float *ws = static_cast<float *>(workspace);
    if (head_dim == 128) {
      return qo_is_f32 ? launch_decode<128, true>(stream, o, q, k, v, mask, kv_len, n_heads, n_kv_heads, ws, q8_out, mask_threshold) :
                         launch_decode<128, false>(stream, o, q, k, v, mask, kv_len, n_heads, n_kv_heads, ws, q8_out, mask_threshold);
    }
    return qo_is_f32 ? launch_decode<64, true>(stream, o, q, k, v, mask, kv_len, n_heads, n_kv_heads, ws, q8_out, mask_threshold) :
                       launch_decode<64, false>(stream, o, q, k, v, mask, kv_len, n_heads, n_kv_heads, ws, q8_out, mask_threshold);
  }
  if (head_dim == 128) {
    return qo_is_f32 ?
             launch_prefill<128, true>(stream, o, q, k, v, mask, qo_len, kv_len, n_heads, n_kv_heads, causal,
                                        forced_key_groups, mask_threshold) :
             launch_prefill<128, false>(stream, o, q, k, v, mask, qo_len, kv_len, n_heads, n_kv_heads, causal,
                                        forced_key_groups, mask_threshold);
  }
  return qo_is_f32 ? launch_prefill<64, true>(stream, o, q, k, v, mask, qo_len, kv_len, n_heads, n_kv_heads, causal,
                                        forced_key_groups, mask_threshold) :
                     launch_prefill<64, false>(stream, o, q, k, v, mask, qo_len, kv_len, n_heads, n_kv_heads, causal,
                                        forced_key_groups, mask_threshold);
}

}  // namespace htpops
