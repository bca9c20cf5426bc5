// Decode-path matrix-vector product for gfx950: Q4_0 or Q8_0 weight rows times one Q8_0 activation row.
//
// Replaces hmx_mat_mul_permuted_qk_0_d16a32 at m = 1 (reference: src/dsp/ops/mat_mul.c:875-1153), which dequantizes
// every weight to fp16 in on-chip memory and runs a 32-row matrix tile for one useful row. Here the op is what it
// is on this machine: a stream over the weight bytes (18 or 34 bytes per 32 weights, each read once) with the
// integer block dots done in registers.
//
// Unit of work: a PAIR of blocks (64 weights). A pair is 36 bytes (Q4_0) or 68 bytes (Q8_0), i.e. a whole number
// of dwords, and every row starts on a pair boundary when k % 64 == 0, so lanes load pairs as dwords with no byte
// realignment. Inside a pair the first block's quants sit two bytes off a dword boundary, behind its fp16 scale.
// Instead of shifting weight bytes, the activation pair (which has the same skew in its own wire layout) is masked
// once per wave so that its bytes line up with the weight dwords and carry zeros under the scale bytes; the
// integer dot is order independent, so v_dot4_i32_i8 over the skewed dwords gives the exact block sums.
// Q4_0 nibbles stay unsigned (0..15): sum (q - 8) a = sum q a - 8 sum a, and sum a is per activation block.
//
// Mapping: G lanes (16, 32 or 64) share a row and stride over its pairs; a wave works on 64 / G rows at once and
// R such row sets, with every weight load issued before the first use (the whole matrix is a few tens of KB per
// CU, so the kernel is latency bound and wants all bytes in flight). fp32 partial sums are reduced over the G lanes.
#include "device_utils.h"
#include "kernels.h"

#include <stdlib.h>

#include <algorithm>

namespace htpops {

namespace {

constexpr int kThreads = 256;
constexpr int kWaves   = kThreads / kWave;

template <int WT>
struct Pair;
template <>
struct Pair<kQ4_0> {
  static constexpr int kDwords = 9;
};
template <>
struct Pair<kQ8_0> {
  static constexpr int kDwords = 17;
};
constexpr int kActPairDwords = 17;

// Activation pair prepared for dotting against raw weight dwords.
template <int WT>
struct ActPair;

template <>
struct ActPair<kQ4_0> {
  uint32_t lo[9];  // bytes that meet the low nibbles of weight dword i
  uint32_t hi[9];  // bytes that meet the high nibbles of weight dword i
  float    d0, d1; // activation scales of the two blocks
  int      off0, off1;  // 8 * (sum of the block's activation bytes)
};

template <>
struct ActPair<kQ8_0> {
  uint32_t a[17];
  float    d0, d1;
};

template <int N>
__device__ __forceinline__ void load_dwords(uint32_t (&dst)[N], const uint32_t *__restrict__ p) {
  constexpr int n4 = N / 4;
#pragma unroll
  for (int i = 0; i < n4; ++i) {
    const u32x4_a4 v = *reinterpret_cast<const u32x4_a4 *>(p + 4 * i);
    dst[4 * i + 0]   = v.x;
    dst[4 * i + 1]   = v.y;
    dst[4 * i + 2]   = v.z;
    dst[4 * i + 3]   = v.w;
  }
#pragma unroll
  for (int i = 4 * n4; i < N; ++i) {
    dst[i] = p[i];
  }
}

template <int N>
__device__ __forceinline__ void zero_dwords(uint32_t (&dst)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) {
    dst[i] = 0u;
  }
}

__device__ __forceinline__ void prepare(ActPair<kQ4_0> &ap, const uint32_t (&a)[17]) {
  ap.lo[0] = a[0] & 0xffff0000u;  // elements 0,1 of block 0 (under weight bytes 2,3); scale bytes -> 0
  ap.lo[1] = a[1];
  ap.lo[2] = a[2];
  ap.lo[3] = a[3];
  ap.lo[4] = a[4] & 0x0000ffffu;  // elements 14,15; the next two weight bytes are block 1's scale
  ap.hi[0] = a[4] & 0xffff0000u;  // elements 16,17
  ap.hi[1] = a[5];
  ap.hi[2] = a[6];
  ap.hi[3] = a[7];
  ap.hi[4] = a[8] & 0x0000ffffu;  // elements 30,31
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    ap.lo[5 + i] = a[9 + i];   // block 1, elements 0..15
    ap.hi[5 + i] = a[13 + i];  // block 1, elements 16..31
  }
  ap.d0 = half_bits_to_float(a[0]);
  ap.d1 = half_bits_to_float(a[8] >> 16);
  int s0 = 0, s1 = 0;
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    s0 = dot4_i8(ap.lo[i], 0x01010101u, s0);
    s0 = dot4_i8(ap.hi[i], 0x01010101u, s0);
  }
#pragma unroll
  for (int i = 5; i < 9; ++i) {
    s1 = dot4_i8(ap.lo[i], 0x01010101u, s1);
    s1 = dot4_i8(ap.hi[i], 0x01010101u, s1);
  }
  ap.off0 = 8 * s0;
  ap.off1 = 8 * s1;
}

__device__ __forceinline__ void prepare(ActPair<kQ8_0> &ap, const uint32_t (&a)[17]) {
#pragma unroll
  for (int i = 0; i < 17; ++i) {
    ap.a[i] = a[i];
  }
  ap.d0 = half_bits_to_float(a[0]);
  ap.d1 = half_bits_to_float(a[8] >> 16);
}

// fp32 contribution of one weight pair: ((float) sumi0 * d_w0) * d_a0 + ((float) sumi1 * d_w1) * d_a1
__device__ __forceinline__ float pair_dot(const uint32_t (&w)[9], const ActPair<kQ4_0> &ap) {
  int s0 = -ap.off0, s1 = -ap.off1;
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    s0 = dot4_i8(w[i] & 0x0f0f0f0fu, ap.lo[i], s0);
    s0 = dot4_i8((w[i] >> 4) & 0x0f0f0f0fu, ap.hi[i], s0);
  }
#pragma unroll
  for (int i = 5; i < 9; ++i) {
    s1 = dot4_i8(w[i] & 0x0f0f0f0fu, ap.lo[i], s1);
    s1 = dot4_i8((w[i] >> 4) & 0x0f0f0f0fu, ap.hi[i], s1);
  }
  const float dw0 = half_bits_to_float(w[0]);
  const float dw1 = half_bits_to_float(w[4] >> 16);
  float       t   = ((float) s0 * dw0) * ap.d0;
  t += ((float) s1 * dw1) * ap.d1;
  return t;
}

__device__ __forceinline__ float pair_dot(const uint32_t (&w)[17], const ActPair<kQ8_0> &ap) {
  int s0 = 0, s1 = 0;
  s0 = dot4_i8(w[0], ap.a[0] & 0xffff0000u, s0);
#pragma unroll
  for (int i = 1; i < 8; ++i) {
    s0 = dot4_i8(w[i], ap.a[i], s0);
  }
  s0 = dot4_i8(w[8], ap.a[8] & 0x0000ffffu, s0);
#pragma unroll
  for (int i = 9; i < 17; ++i) {
    s1 = dot4_i8(w[i], ap.a[i], s1);
  }
  const float dw0 = half_bits_to_float(w[0]);
  const float dw1 = half_bits_to_float(w[8] >> 16);
  float       t   = ((float) s0 * dw0) * ap.d0;
  t += ((float) s1 * dw1) * ap.d1;
  return t;
}

// ---- activation pairs prepared once per workgroup ------------------------------------------------------------------
// The decode kernel keeps the PREPARED form of the activation row in LDS as a table of kEntries words per pair, entry e
// of pair p at tab[e * TS + p] (consecutive lanes read consecutive words: no bank conflicts): the masked dwords that
// meet the weight dwords, the two scales as floats and, for Q4_0 weights, 8 x the two block sums. One thread prepares
// one pair; every wave of the workgroup then reads operands from the table right where it uses them, so the sums and
// masks are computed once per workgroup instead of once per wave and no wave holds a prepared pair in registers.
template <int WT>
struct Prepared;
template <>
struct Prepared<kQ4_0> {
  static constexpr int kEntries = 22;  // lo[9], hi[9], d0, d1, off0, off1
};
template <>
struct Prepared<kQ8_0> {
  static constexpr int kEntries = 19;  // a[17] (scale bytes zeroed), d0, d1
};

template <int TS>
__device__ __forceinline__ void store_prepared(uint32_t *tab, int p, const ActPair<kQ4_0> &ap) {
#pragma unroll
  for (int i = 0; i < 9; ++i) {
    tab[i * TS + p]       = ap.lo[i];
    tab[(9 + i) * TS + p] = ap.hi[i];
  }
  tab[18 * TS + p] = __float_as_uint(ap.d0);
  tab[19 * TS + p] = __float_as_uint(ap.d1);
  tab[20 * TS + p] = (uint32_t) ap.off0;
  tab[21 * TS + p] = (uint32_t) ap.off1;
}

template <int TS>
__device__ __forceinline__ void store_prepared(uint32_t *tab, int p, const ActPair<kQ8_0> &ap) {
  tab[p] = ap.a[0] & 0xffff0000u;
#pragma unroll
  for (int i = 1; i < 8; ++i) {
    tab[i * TS + p] = ap.a[i];
  }
  tab[8 * TS + p] = ap.a[8] & 0x0000ffffu;
#pragma unroll
  for (int i = 9; i < 17; ++i) {
    tab[i * TS + p] = ap.a[i];
  }
  tab[17 * TS + p] = __float_as_uint(ap.d0);
  tab[18 * TS + p] = __float_as_uint(ap.d1);
}

// the same arithmetic as pair_dot, operands from the table
template <int TS>
__device__ __forceinline__ float pair_dot_prepared(const uint32_t (&w)[9], const uint32_t *tab, int p, Prepared<kQ4_0>) {
  int s0 = -(int) tab[20 * TS + p], s1 = -(int) tab[21 * TS + p];
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    s0 = dot4_i8(w[i] & 0x0f0f0f0fu, tab[i * TS + p], s0);
    s0 = dot4_i8((w[i] >> 4) & 0x0f0f0f0fu, tab[(9 + i) * TS + p], s0);
  }
#pragma unroll
  for (int i = 5; i < 9; ++i) {
    s1 = dot4_i8(w[i] & 0x0f0f0f0fu, tab[i * TS + p], s1);
    s1 = dot4_i8((w[i] >> 4) & 0x0f0f0f0fu, tab[(9 + i) * TS + p], s1);
  }
  const float dw0 = half_bits_to_float(w[0]);
  const float dw1 = half_bits_to_float(w[4] >> 16);
  float       t   = ((float) s0 * dw0) * __uint_as_float(tab[18 * TS + p]);
  t += ((float) s1 * dw1) * __uint_as_float(tab[19 * TS + p]);
  return t;
}

template <int TS>
__device__ __forceinline__ float pair_dot_prepared(const uint32_t (&w)[17], const uint32_t *tab, int p, Prepared<kQ8_0>) {
  int s0 = 0, s1 = 0;
#pragma unroll
  for (int i = 0; i < 9; ++i) {
    s0 = dot4_i8(w[i], tab[i * TS + p], s0);
  }
#pragma unroll
  for (int i = 9; i < 17; ++i) {
    s1 = dot4_i8(w[i], tab[i * TS + p], s1);
  }
  const float dw0 = half_bits_to_float(w[0]);
  const float dw1 = half_bits_to_float(w[8] >> 16);
  float       t   = ((float) s0 * dw0) * __uint_as_float(tab[17 * TS + p]);
  t += ((float) s1 * dw1) * __uint_as_float(tab[18 * TS + p]);
  return t;
}

// Any number of pairs per row: lanes loop over the row, activations are re-read (L2) for every row set.
template <int WT, int R>
__global__ __launch_bounds__(kThreads) void gemv_pairs_loop_kernel(float *__restrict__ out,
                                                                   const uint32_t *__restrict__ act,
                                                                   const uint32_t *__restrict__ w, int n, int pairs) {
  constexpr int PD   = Pair<WT>::kDwords;
  const int     lane = threadIdx.x & (kWave - 1);
  const int     wave = threadIdx.x / kWave;
  const int     row0 = (blockIdx.x * kWaves + wave) * R;
  if (row0 >= n) {
    return;
  }
  const size_t row_dwords = (size_t) pairs * PD;
  float        acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    acc[r] = 0.0f;
  }
  for (int p = lane; p < pairs; p += kWave) {
    uint32_t wreg[R][PD];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (row0 + r < n) {
        load_dwords<PD>(wreg[r], w + (size_t) (row0 + r) * row_dwords + (size_t) p * PD);
      } else {
        zero_dwords<PD>(wreg[r]);
      }
    }
    uint32_t a[kActPairDwords];
    load_dwords<kActPairDwords>(a, act + (size_t) p * kActPairDwords);
    ActPair<WT> ap;
    prepare(ap, a);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      acc[r] += pair_dot(wreg[r], ap);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const float s = group_sum<kWave>(acc[r]);
    if (lane == 0 && row0 + r < n) {
      out[row0 + r] = s;
    }
  }
}

// sum over the G consecutive lanes of a group; valid in the group's last lane
template <int G>
__device__ __forceinline__ float group_sum_dpp(float v) {
#define HTPOPS_DPP_ADD(ctrl, row_mask) \
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, row_mask, 0xf, false))
  HTPOPS_DPP_ADD(0xB1, 0xf);   // quad_perm [1,0,3,2]
  HTPOPS_DPP_ADD(0x4E, 0xf);   // quad_perm [2,3,0,1]
  HTPOPS_DPP_ADD(0x141, 0xf);  // row_half_mirror
  HTPOPS_DPP_ADD(0x140, 0xf);  // row_mirror: every lane of a 16-lane row holds the row sum
  if (G >= 32) {
    HTPOPS_DPP_ADD(0x142, 0xa);  // row_bcast15 into rows 1 and 3
  }
  if (G >= 64) {
    HTPOPS_DPP_ADD(0x143, 0xc);  // row_bcast31 into rows 2 and 3
  }
#undef HTPOPS_DPP_ADD
  return v;
}

// ---- the decode kernel -------------------------------------------------------------------------------------------
// The activation row is staged in LDS once per workgroup instead of being fetched by every wave: the texture path then
// carries (almost) only weight bytes. Weight loads are issued right behind the activation loads, so the weights are in
// flight while the workgroup synchronises. Partial sums are reduced with DPP row operations instead of LDS permutes.
//
// One launch serves up to kGemvGroupMax matrix-vector products ("members"), each with its own weight matrix, output,
// row count, row length and ACTIVATION ROW: a workgroup finds its member from a table of first-workgroup indices
// (blockIdx.x is one-dimensional over all members) and then runs the row-set body compiled for that member's row
// length. The caller guarantees that no member reads what another member writes; members that share an activation
// row (q/k/v, gate/up of a decoder layer) are simply members with equal `act`.
struct GemvMember {
  const uint32_t *w;
  const uint32_t *act;
  float          *out;
  int             n;       // weight rows
  int             pairs;   // block pairs per row (k / 64)
  int             block0;  // first workgroup of this member
  int             shape;   // kShape* below: lanes per row and pairs per lane
  int             r;       // row sets per wave (1 or 2; 4 only in the launch that makes its activation row)
};

struct GemvMembers {
  GemvMember m[kGemvGroupMax];
  int        count;
};

// The fused form of the launch: the activation row of EVERY member is the RMS-normalized, Q8_0-quantized image of one
// fp32 row (the decode chain norm -> quantize -> projections as one launch). Each workgroup makes that image for itself
// in LDS -- the first 256 threads repeat the fused RMSNorm + Q8_0 kernel's arithmetic thread for thread, so the bytes
// are the ones that kernel writes -- and the first workgroup of the launch also writes it to `q_out`, where the
// message asked for it. Without `normalize` the row is quantized as it is: the bytes of the Q8_0 quantizer (the same
// block arithmetic), for projections behind a plain quantization (attention output -> Q8_0 -> o projection).
struct GemvNorm {
  const float *src;     // fp32 [k]
  const float *weight;  // fp32 [k] or nullptr
  float        eps;
  uint8_t     *q_out;   // block_q8_0 [k / 32]
  int          normalize;
};

// lanes per row x pairs per lane x waves per row
enum { kShapeG16 = 0, kShapeG32 = 1, kShapeG64 = 2, kShapeG64x2 = 3, kShapeG64x2S2 = 4 };

constexpr int kSharedActMaxPairs = 192;  // longest activation row the kernel stages (k = 12288)
constexpr int kFusedNormMaxBlocks = 1024;  // most workgroups for which making the activation row in each of them pays
constexpr int kRedDwords         = 16;   // LDS words in front of the staged row: partial sums of rows split over waves

// One workgroup of WAVES waves. SEG = 1: wave `wave` computes rows row0 .. row0 + SLOTS * R - 1, SLOTS = 64 / G rows at
// a time. SEG = 2 (G = 64, R = 1): a row is split into two halves taken by two neighbouring waves, whose partial sums
// meet in LDS and are added in a fixed order (first half + second half) -- measured on MI355X, a wave that requests
// more than about 4.6 KB of the stream at once (three pairs per lane, the k = 11008 rows on one wave) streams 10-25 %
// slower than two waves with half of it each.
template <int WT, int G, int ITERS, int R, int SEG, int WAVES, bool FUSED>
__device__ __forceinline__ void gemv_row_sets(const GemvMember &mem, int wg, uint32_t *lds, const GemvNorm &norm) {
  static_assert(SEG == 1 || (G == kWave && R == 1 && WAVES % SEG == 0), "split rows: one row per wave pair");
  constexpr int PD      = Pair<WT>::kDwords;
  constexpr int SLOTS   = kWave / G;
  constexpr int THREADS = WAVES * kWave;
  constexpr int TS      = G * ITERS * SEG < kSharedActMaxPairs ? G * ITERS * SEG : kSharedActMaxPairs;  // pairs in the table
  static_assert(TS <= THREADS, "one thread prepares one activation pair");
  uint32_t *tab = lds + kRedDwords;
  const int                    n     = mem.n;
  const int                    pairs = mem.pairs;
  float *__restrict__          out   = mem.out;
  const uint32_t *__restrict__ w     = mem.w;
  const uint32_t *__restrict__ act   = mem.act;
  const int    lane = threadIdx.x & (kWave - 1);
  const int    wave = threadIdx.x / kWave;
  const int    g    = lane % G;
  const int    slot = lane / G;
  const int    seg  = SEG == 1 ? 0 : wave % SEG;
  const int    row0 = SEG == 1 ? (wg * WAVES + wave) * (SLOTS * R) : wg * (WAVES / SEG) + wave / SEG;
  const int    seg_pairs = SEG == 1 ? pairs : (pairs + SEG - 1) / SEG;
  const int    p_begin   = seg * seg_pairs;
  const int    p_end     = min(pairs, p_begin + seg_pairs);  // may be <= p_begin for a very short row: no live pair
  const size_t row_dwords = (size_t) pairs * PD;

  // The activation pair this thread prepares is requested FIRST and the weights right behind it: loads retire in
  // order, so the (L2 resident, quickly served) activations never wait behind the HBM stream, while the weights are
  // already in flight during the workgroup's LDS exchange. Only waves that have a pair to prepare issue these loads
  // (a wave-uniform branch): measured, the address processing of five more load instructions in every wave costs
  // about 4 % of a decoder layer's stream. Threads beyond the row inside such a wave re-read its last pair.
  uint32_t   araw[kActPairDwords];
  const bool stager = wave * kWave < pairs;
  if (!FUSED && stager) {
    const int my_pair = min((int) threadIdx.x, pairs - 1);
    load_dwords<kActPairDwords>(araw, act + (size_t) my_pair * kActPairDwords);
  }
  // fused form: this thread's slices of the fp32 row (8 floats each, slice = thread / 4 + 64 b is a quant block's
  // quarter `thread % 4`), requested before the weights for the same reason
  constexpr int BPT = FUSED ? (2 * TS + 63) / 64 : 1;
  // (the norm weights too, instead of behind the sum of squares)
  static_assert(!FUSED || BPT <= 2, "the fused form is for rows of up to 64 pairs");
  float          xv[BPT][8], gv[BPT][8];
  const int      nb = 2 * pairs, part = threadIdx.x & 3;
  if (FUSED && threadIdx.x < 256) {
#pragma unroll
    for (int b = 0; b < BPT; ++b) {
      const int blk = ((int) threadIdx.x >> 2) + b * 64;
      if (blk < nb) {
        const float4 *xp = reinterpret_cast<const float4 *>(norm.src + blk * kQK + part * 8);
        const float4  a0 = xp[0], a1 = xp[1];
        xv[b][0] = a0.x, xv[b][1] = a0.y, xv[b][2] = a0.z, xv[b][3] = a0.w;
        xv[b][4] = a1.x, xv[b][5] = a1.y, xv[b][6] = a1.z, xv[b][7] = a1.w;
        if (norm.weight) {
          const float4 *wp = reinterpret_cast<const float4 *>(norm.weight + blk * kQK + part * 8);
          const float4  w0 = wp[0], w1 = wp[1];
          gv[b][0] = w0.x, gv[b][1] = w0.y, gv[b][2] = w0.z, gv[b][3] = w0.w;
          gv[b][4] = w1.x, gv[b][5] = w1.y, gv[b][6] = w1.z, gv[b][7] = w1.w;
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          xv[b][i] = 0.0f;
        }
      }
    }
  }

  // Branch-free weight loads (so that the compiler can count them and wait per use): lanes without work read a
  // clamped, valid address and get their two scale fields zeroed afterwards, which makes the pair contribute 0.
  uint32_t wreg[R][ITERS][PD];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int row = min(row0 + r * SLOTS + slot, n - 1);
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int p = min(p_begin + g + i * G, pairs - 1);
      load_dwords<PD>(wreg[r][i], w + (size_t) row * row_dwords + (size_t) p * PD);
    }
  }

  if (FUSED) {
    // RMSNorm + Q8_0 of the row into an LDS image of its block_q8_0 bytes, in the arithmetic and the order of sums of
    // rms_norm_quantize_kernel (256 threads, slices as above; the other waves add zeros)
    float   *red = reinterpret_cast<float *>(lds);
    uint8_t *img = reinterpret_cast<uint8_t *>(tab + TS * Prepared<WT>::kEntries);
    float    ss  = 0.0f;
    if (threadIdx.x < 256) {
#pragma unroll
      for (int b = 0; b < BPT; ++b) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          ss = __fmaf_rn(xv[b][i], xv[b][i], ss);
        }
      }
    }
    ss = wave_sum(ss);
    if (lane == 0 && wave < 4) {
      red[wave] = ss;
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // LDS only: the weight loads stay in flight
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    const float sum   = ((red[0] + red[1]) + red[2]) + red[3];
    const float mean  = sum / (float) (nb * kQK);
    const float scale = norm.normalize ? 1.0f / sqrtf(mean + norm.eps) : 1.0f;  // (x * 1.0f is x)
    if (threadIdx.x < 256) {
#pragma unroll
      for (int b = 0; b < BPT; ++b) {
        const int blk  = ((int) threadIdx.x >> 2) + b * 64;
        float     amax = 0.0f;
        float     y[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          y[i] = xv[b][i] * scale;
        }
        if (norm.weight && blk < nb) {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            y[i] *= gv[b][i];
          }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          amax = fmaxf(amax, fabsf(y[i]));
        }
        amax           = quad_max(amax);
        const float d  = amax / 127.0f;
        const float id = (d != 0.0f) ? 1.0f / d : 0.0f;
        if (blk < nb) {
          uint16_t      *o16 = reinterpret_cast<uint16_t *>(img + (size_t) blk * 34);
          uint16_t      *g16 = reinterpret_cast<uint16_t *>(norm.q_out + (size_t) blk * 34);
          const bool     pub = blockIdx.x == 0;  // the first workgroup of the launch writes the row where it was asked for
          const uint16_t dh  = __half_as_ushort(__float2half_rn(d));
          if (part == 0) {
            o16[0] = dh;
            if (pub) {
              g16[0] = dh;
            }
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int      q0 = (int) roundf(y[2 * i] * id), q1 = (int) roundf(y[2 * i + 1] * id);
            const uint16_t qq = (uint16_t) ((q0 & 0xff) | ((q1 & 0xff) << 8));
            o16[1 + part * 4 + i] = qq;
            if (pub) {
              g16[1 + part * 4 + i] = qq;
            }
          }
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // LDS only: the weight loads stay in flight
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (stager) {
      const int       my_pair = min((int) threadIdx.x, pairs - 1);
      const uint32_t *ip      = reinterpret_cast<const uint32_t *>(img) + (size_t) my_pair * kActPairDwords;
#pragma unroll
      for (int i = 0; i < kActPairDwords; ++i) {
        araw[i] = ip[i];
      }
    }
  }
  if (stager) {
    ActPair<WT> ap;
    prepare(ap, araw);
    if ((int) threadIdx.x < pairs) {
      store_prepared<TS>(tab, (int) threadIdx.x, ap);
    }
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the LDS writes have landed; vmcnt is left alone
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");

#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int row = row0 + r * SLOTS + slot;
    float     acc = 0.0f;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int  p    = p_begin + g + i * G;
      const bool live = row < n && p < p_end;
      constexpr int kScale1 = WT == kQ4_0 ? 4 : 8;  // dword holding the second block's scale (upper half)
      wreg[r][i][0]         = live ? wreg[r][i][0] : 0u;
      wreg[r][i][kScale1]   = live ? wreg[r][i][kScale1] : 0u;
      acc += pair_dot_prepared<TS>(wreg[r][i], tab, min(p, pairs - 1), Prepared<WT>());
    }
    acc = group_sum_dpp<G>(acc);
    if (SEG == 1) {
      if (g == G - 1 && row < n) {
        out[row] = acc;
      }
    } else {
      float *red = reinterpret_cast<float *>(lds);
      if (lane == kWave - 1) {
        red[wave] = acc;
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      if (lane == kWave - 1 && seg == 0 && row < n) {
        float total = acc;
#pragma unroll
        for (int sg = 1; sg < SEG; ++sg) {
          total += red[wave + sg];
        }
        out[row] = total;
      }
    }
  }
}

// LONG = false: every member has at most 64 pairs per row (k <= 4096); the kernel then holds only the one-pair bodies
// and keeps their small register footprint. LONG = true adds the bodies for longer rows.
// The first workgroup of members 1..7 travels as plain leading arguments (INT_MAX for members that do not exist), the
// first words of the argument block: a wave knows its member after one scalar load and fetches that member's record with
// a second one, instead of walking the table in memory.
template <int WT, bool LONG, int THREADS, bool FUSED>
__device__ __forceinline__ void gemv_members_body(int b1, int b2, int b3, int b4, int b5, int b6, int b7,
                                                  const GemvMembers &grp, const GemvNorm &norm) {
  static_assert(kGemvGroupMax == 8, "one leading argument per member after the first");
  extern __shared__ __attribute__((aligned(16))) uint32_t gemv_lds[];
  constexpr int W   = THREADS / kWave;
  const int     bid = (int) blockIdx.x;
  const int     mi  = bid >= b7 ? 7 : bid >= b6 ? 6 : bid >= b5 ? 5 : bid >= b4 ? 4 : bid >= b3 ? 3 : bid >= b2 ? 2 : bid >= b1 ? 1 : 0;
  const GemvMember &mem = grp.m[mi];
  const int         wg  = (int) blockIdx.x - mem.block0;
  if constexpr (FUSED) {
    if (mem.r == 4) {  // (rows of 33..64 pairs only: see the launcher)
      gemv_row_sets<WT, 64, 1, 4, 1, W, FUSED>(mem, wg, gemv_lds, norm);
      return;
    }
  }
  const int         sel = mem.shape * 2 + (mem.r - 1);
  switch (sel) {
    case kShapeG16 * 2 + 0: gemv_row_sets<WT, 16, 1, 1, 1, W, FUSED>(mem, wg, gemv_lds, norm); break;
    case kShapeG16 * 2 + 1: gemv_row_sets<WT, 16, 1, 2, 1, W, FUSED>(mem, wg, gemv_lds, norm); break;
    case kShapeG32 * 2 + 0: gemv_row_sets<WT, 32, 1, 1, 1, W, FUSED>(mem, wg, gemv_lds, norm); break;
    case kShapeG32 * 2 + 1: gemv_row_sets<WT, 32, 1, 2, 1, W, FUSED>(mem, wg, gemv_lds, norm); break;
    case kShapeG64 * 2 + 0: gemv_row_sets<WT, 64, 1, 1, 1, W, FUSED>(mem, wg, gemv_lds, norm); break;
    case kShapeG64 * 2 + 1: gemv_row_sets<WT, 64, 1, 2, 1, W, FUSED>(mem, wg, gemv_lds, norm); break;
    default:
      if constexpr (LONG) {
        switch (sel) {
          case kShapeG64x2 * 2 + 0: gemv_row_sets<WT, 64, 2, 1, 1, W, FUSED>(mem, wg, gemv_lds, norm); break;
          case kShapeG64x2S2 * 2 + 0: gemv_row_sets<WT, 64, 2, 1, 2, W, FUSED>(mem, wg, gemv_lds, norm); break;
          default: break;
        }
      }
      break;
  }
}

template <int WT, bool LONG, int THREADS>
__global__ __launch_bounds__(THREADS) void gemv_members_kernel(int b1, int b2, int b3, int b4, int b5, int b6, int b7,
                                                               GemvMembers grp) {
  gemv_members_body<WT, LONG, THREADS, false>(b1, b2, b3, b4, b5, b6, b7, grp, GemvNorm{});
}

template <int WT, bool LONG, int THREADS>
__global__ __launch_bounds__(THREADS) void gemv_members_norm_kernel(int b1, int b2, int b3, int b4, int b5, int b6, int b7,
                                                                    GemvMembers grp, GemvNorm norm) {
  gemv_members_body<WT, LONG, THREADS, true>(b1, b2, b3, b4, b5, b6, b7, grp, norm);
}

// Fills shape, r and block0 of every member and launches; with `norm`, the fused form (see GemvNorm).
template <int WT>
hipError_t launch_gemv_members(hipStream_t stream, GemvMembers &grp, const GemvNorm *norm = nullptr) {
  // measured on MI355X: short-lived waves (one row set each) stream best; only very wide launches of short rows
  // (gate + up of a 7B layer: 22016 rows of 64 pairs) gain from two rows per lane group
  long total_short_rows = 0;
  for (int i = 0; i < grp.count; ++i) {
    if (grp.m[i].pairs <= 64) {
      total_short_rows += grp.m[i].n;
    }
  }
  // Workgroups of 512 threads stage the activation row half as often per weight byte (measured on a 7B layer's seven
  // projections in one launch: 20.3 us against 20.9 us); launches too small to give every compute unit a few of them
  // keep 256 threads.
  auto place = [&](int threads, bool commit) {
    const int waves  = threads / kWave;
    int       blocks = 0;
    for (int i = 0; i < grp.count; ++i) {
      GemvMember &mem            = grp.m[i];
      const int   lanes_per_row  = mem.shape == kShapeG16 ? 16 : mem.shape == kShapeG32 ? 32 : 64;
      const int   rows_per_group = mem.shape == kShapeG64x2S2 ? waves / 2 : waves * (kWave / lanes_per_row) * mem.r;
      if (commit) {
        mem.block0 = blocks;
      }
      blocks += (mem.n + rows_per_group - 1) / rows_per_group;
    }
    return blocks;
  };
  int  max_pairs = 0;
  bool any_long  = false;
  for (int i = 0; i < grp.count; ++i) {
    GemvMember &mem = grp.m[i];
    const int   p   = mem.pairs;
    if (p < 1 || p > kSharedActMaxPairs || mem.n < 1) {
      return hipErrorNotSupported;
    }
    mem.shape = p <= 16 ? kShapeG16 : p <= 32 ? kShapeG32 : p <= 64 ? kShapeG64 : p <= 128 ? kShapeG64x2 : kShapeG64x2S2;
    mem.r     = (p <= 64 && (total_short_rows >= 16384 || norm)) ? 2 : 1;
    if (norm && p > 32 && p <= 64 && total_short_rows > kFusedNormMaxBlocks * 16) {
      mem.r = 4;  // gate and up of a 7B layer: 32 rows per workgroup halve the number of times the row is made
    }
    max_pairs = p > max_pairs ? p : max_pairs;
    any_long  = any_long || p > 64;
  }
  // (making the activation row is work per workgroup: the fused form takes the fewest, largest workgroups)
  const int threads = (norm || place(512, false) >= 1024) ? 512 : kThreads;
  const int blocks = place(threads, true);
  // Measured on MI355X with Q4_0 weights of k = 4096: making the row costs every workgroup about as much as 8 KB of its
  // weight stream, which beats a launch of its own (3.5-4 us behind another) up to about a thousand workgroups:
  // n = 4096: 5.2 us against 7.0 us, 3 x 4096: 9.0 / 10.4, 2 x 11008: 16.4 / 14.5 with 16 rows per workgroup, 14.2 with
  // 32 (and 16.0 with 64: too few workgroups). Longer rows cost in proportion.
  if (norm && (any_long || blocks > kFusedNormMaxBlocks)) {
    return hipErrorNotSupported;
  }
  // the table stride of the widest body among the members (see TS in gemv_row_sets)
  const int    table_pairs = max_pairs <= 16 ? 16 : max_pairs <= 32 ? 32 : max_pairs <= 64 ? 64 : max_pairs <= 128 ? 128 : kSharedActMaxPairs;
  const size_t lds = (size_t) (kRedDwords + table_pairs * Prepared<WT>::kEntries) * 4 +
                     (norm ? (size_t) max_pairs * 2 * 34 + 4 : 0);  // + the LDS image of the quantized row
  const dim3   grid((unsigned) blocks);
  int b[kGemvGroupMax];
  for (int i = 1; i < kGemvGroupMax; ++i) {
    b[i] = i < grp.count ? grp.m[i].block0 : 0x7fffffff;
  }
#define HTPOPS_GEMV_LAUNCH(LONG, T) \
  hipLaunchKernelGGL((gemv_members_kernel<WT, LONG, T>), grid, dim3(T), lds, stream, b[1], b[2], b[3], b[4], b[5], b[6], b[7], grp)
  last_gemv_launch() = { norm ? "gemv_members_norm_kernel" : "gemv_members_kernel", WT, norm ? 0 : (int) any_long,
                         threads, (unsigned) blocks, (unsigned) threads, (unsigned) lds };
  if (norm) {
    hipLaunchKernelGGL((gemv_members_norm_kernel<WT, false, 512>), grid, dim3(512), lds, stream, b[1], b[2], b[3], b[4],
                       b[5], b[6], b[7], grp, *norm);
  } else if (threads == 512) {
    if (any_long) {
      HTPOPS_GEMV_LAUNCH(true, 512);
    } else {
      HTPOPS_GEMV_LAUNCH(false, 512);
    }
  } else if (any_long) {
    HTPOPS_GEMV_LAUNCH(true, kThreads);
  } else {
    HTPOPS_GEMV_LAUNCH(false, kThreads);
  }
#undef HTPOPS_GEMV_LAUNCH
  return hipGetLastError();
}

// Catch-all (odd block counts, any m): one wave per weight row, 16-bit loads, scalar integer arithmetic.
template <int WT>
__global__ __launch_bounds__(kThreads) void gemv_blocks_generic_kernel(float *__restrict__ out,
                                                                       const uint16_t *__restrict__ act,
                                                                       const uint16_t *__restrict__ w, int m, int n,
                                                                       int nblk) {
  constexpr int WH   = WT == kQ4_0 ? 9 : 17;  // halfwords per weight block
  const int     lane = threadIdx.x & (kWave - 1);
  const int     row  = blockIdx.x * kWaves + threadIdx.x / kWave;
  if (row >= n) {
    return;
  }
  for (int mi = 0; mi < m; ++mi) {
    float acc = 0.0f;
    for (int b = lane; b < nblk; b += kWave) {
      const uint16_t *wb   = w + ((size_t) row * nblk + b) * WH;
      const uint16_t *ab   = act + ((size_t) mi * nblk + b) * 17;
      int             sumi = 0;
      if (WT == kQ4_0) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int wq = wb[1 + j], al = ab[1 + j], ah = ab[9 + j];
          sumi += ((wq & 15) - 8) * (int) (int8_t) (al & 0xff) + (((wq >> 8) & 15) - 8) * (int) (int8_t) (al >> 8);
          sumi += (((wq >> 4) & 15) - 8) * (int) (int8_t) (ah & 0xff) + (((wq >> 12) & 15) - 8) * (int) (int8_t) (ah >> 8);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int wq = wb[1 + j], aq = ab[1 + j];
          sumi += (int) (int8_t) (wq & 0xff) * (int) (int8_t) (aq & 0xff) + (int) (int8_t) (wq >> 8) * (int) (int8_t) (aq >> 8);
        }
      }
      acc += ((float) sumi * half_bits_to_float(wb[0])) * half_bits_to_float(ab[0]);
    }
    acc = group_sum<kWave>(acc);
    if (lane == 0) {
      out[(size_t) mi * n + row] = acc;
    }
  }
}

// ---- two to four activation rows, held in registers ---------------------------------------------------------------
// The stream over the weights again, arranged so that nothing is shared and nothing waits: a wave owns one chunk of 64
// pairs of K (lane = pair), prepares its pairs of all M activation rows ONCE into registers, and then walks a range of
// weight rows -- one pair per lane and row, requested three rows ahead -- dotting each against the M rows (the nibble
// unpacking is shared between them). The C = 1, 2 or 3 waves that cover all of K for the same range of weight rows are
// a team: with C = 1 a wave stores its sums itself, otherwise the chunk sums of a row meet in LDS after the walk and
// are added in chunk order. A workgroup has three waves: three teams of short rows, or one team (and an idle wave
// when C = 2). The extra rows cost vector-ALU work only (about 5 us per row and Llama-7B layer, which is why the
// kernel is used up to three rows); every member of a launch brings its own activation rows and row length.
struct RowsMember {
  const uint32_t *w;
  const uint32_t *act;  // M rows
  float          *out;  // [M][n]
  int             n;
  int             pairs;   // block pairs per row (k / 64)
  int             block0;  // first workgroup of this member
};

struct RowsMembers {
  RowsMember m[kGemvGroupMax];
  int        count;
};

constexpr int kRowsDepth   = 3;   // weight rows in flight per wave
constexpr int kRowsMaxWalk = 64;  // weight rows per team at most (the LDS image of the chunk sums)
constexpr int kRowsWaves   = 3;   // = the most chunks a row has (kSharedActMaxPairs / 64)

template <int WT, int M>
__global__ __launch_bounds__(kRowsWaves *kWave) void gemv_rows_in_registers_kernel(RowsMembers grp, int walk) {
  constexpr int PD = Pair<WT>::kDwords;
  __shared__ float red[kRowsMaxWalk * kRowsWaves * M];
  int mi = 0;
#pragma unroll
  for (int i = 1; i < kGemvGroupMax; ++i) {
    mi = (i < grp.count && (int) blockIdx.x >= grp.m[i].block0) ? i : mi;
  }
  const RowsMember &mem = grp.m[mi];
  const int                    n     = mem.n;
  const int                    pairs = mem.pairs;
  const uint32_t *__restrict__ w     = mem.w;
  float *__restrict__          out   = mem.out;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int C    = (pairs + kWave - 1) / kWave;  // chunks of K = waves of a team
  const int c = wave % C, team = wave / C, teams = kRowsWaves / C;
  // (a wave without a team -- the third one when C = 2 -- and a team past the member's last row walk nothing)
  const int row_begin = team < teams ? min(n, (((int) blockIdx.x - mem.block0) * teams + team) * walk) : n;
  const int row_end   = min(n, row_begin + walk);
  const int  p    = c * kWave + lane;
  const bool live = p < pairs;
  const int  pc   = min(p, pairs - 1);
  const size_t row_dwords = (size_t) pairs * PD;

  // the first weight rows are requested before the activations are prepared
  uint32_t        wreg[kRowsDepth][PD];
  const uint32_t *wp = w + (size_t) pc * PD;
#pragma unroll
  for (int d = 0; d < kRowsDepth; ++d) {
    load_dwords<PD>(wreg[d], wp + (size_t) min(row_begin + d, n - 1) * row_dwords);
  }
  ActPair<WT> ap[M];
#pragma unroll
  for (int mm = 0; mm < M; ++mm) {
    uint32_t a[kActPairDwords];
    load_dwords<kActPairDwords>(a, mem.act + ((size_t) mm * pairs + pc) * kActPairDwords);
    prepare(ap[mm], a);
    if (!live) {
      ap[mm].d0 = 0.0f, ap[mm].d1 = 0.0f;  // a pair past the end of the row adds nothing
    }
  }

  for (int r0 = row_begin; r0 < row_end; r0 += kRowsDepth) {
#pragma unroll
    for (int d = 0; d < kRowsDepth; ++d) {
      const int r = r0 + d;
      if (r < row_end) {  // (uniform)
        float v[M];
#pragma unroll
        for (int mm = 0; mm < M; ++mm) {
          v[mm] = pair_dot(wreg[d], ap[mm]);
        }
        // the slot is free: its next row
        load_dwords<PD>(wreg[d], wp + (size_t) min(r + kRowsDepth, n - 1) * row_dwords);
#pragma unroll
        for (int mm = 0; mm < M; ++mm) {
          v[mm] = group_sum_dpp<kWave>(v[mm]);
        }
        if (lane == kWave - 1) {
#pragma unroll
          for (int mm = 0; mm < M; ++mm) {
            if (C == 1) {
              out[(size_t) mm * n + r] = v[mm];
            } else {
              red[((r - row_begin) * C + c) * M + mm] = v[mm];
            }
          }
        }
      }
    }
  }
  if (C > 1) {  // (the same for the whole workgroup: one team)
    __syncthreads();
    const int rb = min(n, ((int) blockIdx.x - mem.block0) * walk), re = min(n, rb + walk);  // the team's rows
    for (int t = threadIdx.x; t < (re - rb) * M; t += kRowsWaves * kWave) {
      const int r = t / M, mm = t % M;
      float     total = red[(r * C) * M + mm];
      for (int cc = 1; cc < C; ++cc) {
        total += red[(r * C + cc) * M + mm];
      }
      out[(size_t) mm * n + rb + r] = total;
    }
  }
}

template <int WT>
hipError_t launch_rows_in_registers(hipStream_t stream, const RowsMembers &grp, int blocks, int m, int walk) {
  const dim3 grid((unsigned) blocks), block((unsigned) (kRowsWaves * kWave));
  switch (m) {
    case 2: hipLaunchKernelGGL((gemv_rows_in_registers_kernel<WT, 2>), grid, block, 0, stream, grp, walk); break;
    case 3: hipLaunchKernelGGL((gemv_rows_in_registers_kernel<WT, 3>), grid, block, 0, stream, grp, walk); break;
    case 4: hipLaunchKernelGGL((gemv_rows_in_registers_kernel<WT, 4>), grid, block, 0, stream, grp, walk); break;
    default: return hipErrorNotSupported;
  }
  return hipGetLastError();
}

template <int WT>
hipError_t launch_gemv_row(hipStream_t stream, float *out, const uint32_t *act, const uint32_t *w, int n, int pairs) {
  if (pairs <= kSharedActMaxPairs) {
    GemvMembers grp = {};
    grp.count       = 1;
    grp.m[0].w = w, grp.m[0].act = act, grp.m[0].out = out, grp.m[0].n = n, grp.m[0].pairs = pairs;
    return launch_gemv_members<WT>(stream, grp);
  }
  hipLaunchKernelGGL((gemv_pairs_loop_kernel<WT, 2>), dim3((unsigned) ((n + kWaves * 2 - 1) / (kWaves * 2))),
                     dim3(kThreads), 0, stream, out, act, w, n, pairs);
  return hipGetLastError();
}

}  // namespace

LaunchRecord &last_gemv_launch() {
  static thread_local LaunchRecord rec;
  return rec;
}

// m rows of activations, one pass over the weights per activation row. The caller routes larger m to the MFMA path.
hipError_t launch_gemv_q8_0_act(hipStream_t stream, float *out, const void *act, const void *weight, int m, int k,
                                int n, WeightType wt) {
  const int  nblk       = k / kQK;
  const bool pair_path  = (nblk % 2 == 0) && ((reinterpret_cast<uintptr_t>(act) | reinterpret_cast<uintptr_t>(weight)) & 3) == 0;
  if (!pair_path) {
    dim3 grid((unsigned) ((n + kWaves - 1) / kWaves));
    if (wt == kQ4_0) {
      hipLaunchKernelGGL(gemv_blocks_generic_kernel<kQ4_0>, grid, dim3(kThreads), 0, stream, out,
                         (const uint16_t *) act, (const uint16_t *) weight, m, n, nblk);
    } else {
      hipLaunchKernelGGL(gemv_blocks_generic_kernel<kQ8_0>, grid, dim3(kThreads), 0, stream, out,
                         (const uint16_t *) act, (const uint16_t *) weight, m, n, nblk);
    }
    return hipGetLastError();
  }
  const int pairs = nblk / 2;
  for (int mi = 0; mi < m; ++mi) {
    const uint32_t *a = reinterpret_cast<const uint32_t *>(act) + (size_t) mi * pairs * kActPairDwords;
    float          *o = out + (size_t) mi * n;
    hipError_t      e = wt == kQ4_0 ? launch_gemv_row<kQ4_0>(stream, o, a, (const uint32_t *) weight, n, pairs) :
                                      launch_gemv_row<kQ8_0>(stream, o, a, (const uint32_t *) weight, n, pairs);
    if (e != hipSuccess) {
      return e;
    }
  }
  return hipSuccess;
}

hipError_t launch_gemv_group_q8_0_act(hipStream_t stream, int count, float *const *outs, const void *const *acts,
                                      const void *const *weights, const int *ns, const int *ks, WeightType wt) {
  if (count < 1 || count > kGemvGroupMax) {
    return hipErrorNotSupported;
  }
  GemvMembers grp = {};
  grp.count       = count;
  // The members are laid out over the workgroups in order of their size, largest first:
  // workgroups start in index order, and a launch that ends with the workgroups of its small matrices ends sooner
  // than one that ends with those of a large one (a 7B layer's seven projections: 19.9 us as gate, up, down, q, k, v, o
  // against 20.2 us as q, k, v, o, gate, up, down). A member's own workgroups and sums do not depend on its place.
  int order[kGemvGroupMax];
  for (int i = 0; i < count; ++i) {
    order[i] = i;
  }
  std::stable_sort(order, order + count, [&](int a, int b) {
    const long sa = (long) ns[a] * ks[a], sb = (long) ns[b] * ks[b];
    return sa != sb ? sa > sb : ks[a] < ks[b];  // (equal sizes: the shorter rows first -- gate, down, up measured 20.5 us)
  });
  for (int j = 0; j < count; ++j) {
    const int i    = order[j];
    const int nblk = ks[i] / kQK;
    if (ks[i] % (2 * kQK) != 0 || nblk / 2 > kSharedActMaxPairs ||
        ((reinterpret_cast<uintptr_t>(weights[i]) | reinterpret_cast<uintptr_t>(acts[i])) & 3) != 0) {
      return hipErrorNotSupported;
    }
    grp.m[j].w = static_cast<const uint32_t *>(weights[i]), grp.m[j].act = static_cast<const uint32_t *>(acts[i]);
    grp.m[j].out = outs[i], grp.m[j].n = ns[i], grp.m[j].pairs = nblk / 2;
  }
  return wt == kQ4_0 ? launch_gemv_members<kQ4_0>(stream, grp) : launch_gemv_members<kQ8_0>(stream, grp);
}

// The decode chain as one launch: every member's activation row is RMSNorm(src [* norm_weight]) quantized to Q8_0,
// made by each workgroup for itself and also written to `q_out` (k / 32 blocks), bit for bit what
// launch_rms_norm_quantize_q8_0 writes (`normalize` false: src quantized as it is, what launch_quantize_q8_0 writes). k % 64 == 0, k <= 4096, 16-byte aligned src / norm_weight and few enough
// weight rows that it pays (see launch_gemv_members), else hipErrorNotSupported and nothing is launched.
hipError_t launch_gemv_group_rms_norm_q8_0_act(hipStream_t stream, int count, float *const *outs, const void *const *weights,
                                               const int *ns, int k, WeightType wt, const float *src,
                                               const float *norm_weight, float eps, void *q_out, bool normalize) {
  const int nblk = k / kQK;
  if (count < 1 || count > kGemvGroupMax || k % (2 * kQK) != 0 || nblk / 2 > kSharedActMaxPairs ||
      (reinterpret_cast<uintptr_t>(src) & 15) != 0 || (reinterpret_cast<uintptr_t>(norm_weight) & 15) != 0 ||
      (reinterpret_cast<uintptr_t>(q_out) & 3) != 0) {
    return hipErrorNotSupported;
  }
  GemvMembers grp = {};
  grp.count       = count;
  for (int i = 0; i < count; ++i) {
    if ((reinterpret_cast<uintptr_t>(weights[i]) & 3) != 0) {
      return hipErrorNotSupported;
    }
    grp.m[i].w = static_cast<const uint32_t *>(weights[i]), grp.m[i].act = static_cast<const uint32_t *>(q_out);
    grp.m[i].out = outs[i], grp.m[i].n = ns[i], grp.m[i].pairs = nblk / 2;
  }
  const GemvNorm norm = { src, normalize ? norm_weight : nullptr, eps, static_cast<uint8_t *>(q_out), normalize ? 1 : 0 };
  return wt == kQ4_0 ? launch_gemv_members<kQ4_0>(stream, grp, &norm) : launch_gemv_members<kQ8_0>(stream, grp, &norm);
}

bool gemv_rows_fits(int m, int k, WeightType wt) {
  // measured on Llama-7B (Q4_0) and Qwen2-1.5B (Q8_0) layers: up to three rows the kernel beats the repacked-weight and
  // K-sliced kernels (28.2 / 31.8 against 38.9 / 39.3 us and 13.3 / 14.8 against 18.3 / 18.5 us), at four rows they
  // are level (39.0 against 38.2, 18.4 against 18.6 us); every further row costs it as much again while theirs come
  // free up to eight. (Two and three rows of Q4_0 go to the two-blocks-per-instruction kernel instead where a repacked
  // copy of the weights is there or may be kept, 25 against 28 and 32 us; the caller decides that.)
  (void) wt;
  const int nblk = k / kQK;
  return m >= 2 && m <= 3 && k % (2 * kQK) == 0 && nblk / 2 <= kSharedActMaxPairs;
}

hipError_t launch_gemv_rows_group_q8_0_act(hipStream_t stream, int count, float *const *outs, const void *const *acts,
                                           const void *const *weights, const int *ns, int m, const int *ks,
                                           WeightType wt) {
  if (count < 1 || count > kGemvGroupMax || m < 2 || m > 4) {
    return hipErrorNotSupported;
  }
  long waves_per_row = 0;  // summed over all weight rows
  for (int i = 0; i < count; ++i) {
    const int pairs = ks[i] / (2 * kQK);
    if (ns[i] < 1 || ks[i] % (2 * kQK) != 0 || pairs < 1 || pairs > kSharedActMaxPairs ||
        ((reinterpret_cast<uintptr_t>(weights[i]) | reinterpret_cast<uintptr_t>(acts[i])) & 3) != 0) {
      return hipErrorNotSupported;
    }
    waves_per_row += (long) ns[i] * ((pairs + kWave - 1) / kWave);
  }
  // about twelve waves per compute unit, each with at least eight weight rows to set its prepared activations against
  // (measured on the Llama-7B layer at two rows: 4 / 8 / 16 / 32 rows per wave 45.9 / 41.9 / 48.6 / 75.4 us)
  int walk = kRowsMaxWalk;
  while (walk > 8 && waves_per_row / walk < 3072) {
    walk /= 2;
  }
  RowsMembers grp = {};
  grp.count       = count;
  int blocks      = 0;
  for (int i = 0; i < count; ++i) {
    const int pairs = ks[i] / (2 * kQK);
    const int rows_per_block = walk * (kRowsWaves / ((pairs + kWave - 1) / kWave));
    grp.m[i].w = static_cast<const uint32_t *>(weights[i]), grp.m[i].act = static_cast<const uint32_t *>(acts[i]);
    grp.m[i].out = outs[i], grp.m[i].n = ns[i], grp.m[i].pairs = pairs, grp.m[i].block0 = blocks;
    blocks += (ns[i] + rows_per_block - 1) / rows_per_block;
  }
  return wt == kQ4_0 ? launch_rows_in_registers<kQ4_0>(stream, grp, blocks, m, walk) :
                       launch_rows_in_registers<kQ8_0>(stream, grp, blocks, m, walk);
}

}  // namespace htpops
