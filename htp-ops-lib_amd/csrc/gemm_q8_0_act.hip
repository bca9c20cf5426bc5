// Prefill-path quantized matmul for gfx950: out[m][n] = sum over 32-wide K blocks of
//   (float) (int dot of weight block (n, kb) with activation block (m, kb)) * d_w(n, kb) * d_a(m, kb).
//
// Replaces hmx_mat_mul_permuted_qk_0_d16a32 for m > 1 (reference: src/dsp/ops/mat_mul.c:875-1153): there, weights
// are dequantized (scale applied) to fp16 tiles in on-chip memory and multiplied on the fp16 matrix unit. Here the
// scales never touch the operands, so every block sum is the exact integer:
//
// Both operands carry a scale per 32 K-values, so an accumulator may only span one block, and each of the m n k / 32
// block sums must be multiplied by its own scale pair. On this machine that epilogue, not the dot products, is the
// bottleneck: the VALU retires 16 lanes per clock per SIMD while one 32x32x32 matrix instruction produces 1024 block
// sums in 32 clocks. Two kernels:
//
//  * large m (>= 64), `gemm_mfma3_kernel`: everything except one FMA per block sum runs on the matrix cores.
//      S  = act_int x weight_int   two v_mfma_f32_32x32x16_f16 on integer-valued fp16 operands: products and the
//                                  fp32 accumulation of 32 of them are exact (|S| < 2^24), so S is the exact block
//                                  sum, already in floating point (no int -> float conversion);
//      C  = d_a (x) d_w            one v_mfma_f32_32x32x8f16 with the scales in K-slot 0: the exact fp32 product of
//                                  two fp16 scales for all 32 x 32 (m, n) pairs (fp16 subnormals are not flushed);
//      acc = fma(S, C, acc)        the only VALU work per block sum.
//    Activations are converted once per launch by a pre-pass (int8 -> integer-valued fp16, laid out [k / 8][m] in
//    16-byte pieces so that a tile is contiguous) and reach LDS by global_load_lds DMA; Q4_0 / Q8_0 weights are
//    converted on their way into LDS (nibble or byte -> fp16 through v_perm + one packed fp16 add).
//    Tile 128 x 64, K step 64, 256 threads = 2 x 2 waves of 64 x 32, double-buffered LDS.
//  * small m, `gemm_q8_0_act_kernel`: v_mfma_i32_32x32x32_i8 on int8 tiles with the convert-and-scale epilogue on
//    the VALU; tile 32 x 128.
// The MFMA output layout puts n on lanes (lane % 32) and 16 values of m in registers.
#include "device_utils.h"
#include "kernels.h"

namespace htpops {

namespace {

typedef int   v4i __attribute__((ext_vector_type(4)));
typedef int   v16i __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int KB_STEP  = 4;  // quant blocks per K step (two pairs)

// one K block in LDS
template <int BM, int BN>
struct __attribute__((aligned(16))) StageBlock {
  uint4 a[2][BM];  // [half][m row]
  uint4 b[2][BN];  // [half][n row]
  float da[BM];
  float dw[BN];
};
template <int BM, int BN>
struct Stage {
  StageBlock<BM, BN> blk[KB_STEP];
};

template <int WT>
struct WPair;
template <>
struct WPair<kQ4_0> {
  static constexpr int kDwords = 9;
};
template <>
struct WPair<kQ8_0> {
  static constexpr int kDwords = 17;
};

__device__ __forceinline__ uint32_t alignbyte2(uint32_t hi, uint32_t lo) {
  return __builtin_amdgcn_alignbyte(hi, lo, 2);  // bytes 2..5 of the 8-byte value hi:lo
}

// 4 unsigned nibbles (one per byte, 0..15) -> 4 signed bytes (q - 8)
__device__ __forceinline__ uint32_t nibbles_to_s8(uint32_t q) {
  return ((q | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
}

template <int N>
__device__ __forceinline__ void load_pair(uint32_t (&dst)[N], const uint32_t *__restrict__ p) {
  constexpr int n4 = N / 4;
#pragma unroll
  for (int i = 0; i < n4; ++i) {
    const u32x4_a4 v = *reinterpret_cast<const u32x4_a4 *>(p + 4 * i);
    dst[4 * i + 0] = v.x, dst[4 * i + 1] = v.y, dst[4 * i + 2] = v.z, dst[4 * i + 3] = v.w;
  }
#pragma unroll
  for (int i = 4 * n4; i < N; ++i) {
    dst[i] = p[i];
  }
}

// a Q8_0 pair (17 dwords) -> two blocks of 32 int8 as 2 x 2 uint4 (half 0 / half 1) and two scales
__device__ __forceinline__ void split_q8_pair(const uint32_t (&p)[17], uint4 (&h0)[2], uint4 (&h1)[2], float (&d)[2]) {
  uint32_t q[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    q[i] = alignbyte2(p[i + 1], p[i]);  // block 0 quants start at byte 2
  }
  h0[0] = make_uint4(q[0], q[1], q[2], q[3]);
  h1[0] = make_uint4(q[4], q[5], q[6], q[7]);
  h0[1] = make_uint4(p[9], p[10], p[11], p[12]);
  h1[1] = make_uint4(p[13], p[14], p[15], p[16]);
  d[0]  = half_bits_to_float(p[0]);
  d[1]  = half_bits_to_float(p[8] >> 16);
}

// a Q4_0 pair (9 dwords) -> the same, values q - 8
__device__ __forceinline__ void split_q4_pair(const uint32_t (&p)[9], uint4 (&h0)[2], uint4 (&h1)[2], float (&d)[2]) {
  uint32_t q0[4], q1[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    q0[i] = alignbyte2(p[i + 1], p[i]);  // block 0: bytes 2..17
    q1[i] = p[5 + i];                    // block 1: bytes 20..35
  }
  h0[0] = make_uint4(nibbles_to_s8(q0[0] & 0x0f0f0f0fu), nibbles_to_s8(q0[1] & 0x0f0f0f0fu),
                     nibbles_to_s8(q0[2] & 0x0f0f0f0fu), nibbles_to_s8(q0[3] & 0x0f0f0f0fu));
  h1[0] = make_uint4(nibbles_to_s8((q0[0] >> 4) & 0x0f0f0f0fu), nibbles_to_s8((q0[1] >> 4) & 0x0f0f0f0fu),
                     nibbles_to_s8((q0[2] >> 4) & 0x0f0f0f0fu), nibbles_to_s8((q0[3] >> 4) & 0x0f0f0f0fu));
  h0[1] = make_uint4(nibbles_to_s8(q1[0] & 0x0f0f0f0fu), nibbles_to_s8(q1[1] & 0x0f0f0f0fu),
                     nibbles_to_s8(q1[2] & 0x0f0f0f0fu), nibbles_to_s8(q1[3] & 0x0f0f0f0fu));
  h1[1] = make_uint4(nibbles_to_s8((q1[0] >> 4) & 0x0f0f0f0fu), nibbles_to_s8((q1[1] >> 4) & 0x0f0f0f0fu),
                     nibbles_to_s8((q1[2] >> 4) & 0x0f0f0f0fu), nibbles_to_s8((q1[3] >> 4) & 0x0f0f0f0fu));
  d[0]  = half_bits_to_float(p[0]);
  d[1]  = half_bits_to_float(p[4] >> 16);
}

// WM waves along m, TM MFMA tiles per wave along m; the remaining waves lie along n.
template <int WT, int WM, int TM>
__global__ __launch_bounds__(kThreads) void gemm_q8_0_act_kernel(float *__restrict__ out,
                                                                 const uint32_t *__restrict__ act,
                                                                 const uint32_t *__restrict__ w, int m, int n,
                                                                 int pairs) {
  constexpr int WN = 4 / WM;
  constexpr int BM = WM * TM * 32;
  constexpr int BN = WN * 32;
  constexpr int WD = WPair<WT>::kDwords;
  constexpr int AD = 17;
  static_assert(BM * 2 <= kThreads && BN * 2 <= kThreads, "one staging task per thread");
  using StageT = Stage<BM, BN>;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  StageT *stages = reinterpret_cast<StageT *>(smem);

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm   = wave / WN;
  const int wn   = wave % WN;
  const int m0   = blockIdx.y * BM;
  const int n0   = blockIdx.x * BN;

  // staging roles per K step: thread t < 2 BM moves activation pair (row t / 2, pair t % 2); thread t < 2 BN moves
  // weight pair (row t / 2, pair t % 2). Rows past the matrix edge are clamped: their outputs are never stored.
  const int  s_row  = tid >> 1;
  const int  s_pair = tid & 1;
  const bool has_a  = tid < 2 * BM;
  const bool has_w  = tid < 2 * BN;
  const int  a_m    = min(m0 + s_row, m - 1);
  const int  w_n    = min(n0 + s_row, n - 1);

  const uint32_t *a_ptr = act + (size_t) a_m * pairs * AD;
  const uint32_t *w_ptr = w + (size_t) w_n * pairs * WD;

  uint32_t areg[AD], wreg[WD];
  // K steps past the end (odd number of pairs) re-read the last pair; its scales are zeroed at store time
  auto fetch = [&](int step) {
    const int p = min(step * 2 + s_pair, pairs - 1);
    if (has_a) {
      load_pair<AD>(areg, a_ptr + (size_t) p * AD);
    }
    if (has_w) {
      load_pair<WD>(wreg, w_ptr + (size_t) p * WD);
    }
  };
  auto stash = [&](int step, StageT &st) {
    uint4      h0[2], h1[2];
    float      d[2];
    const bool live = step * 2 + s_pair < pairs;
    if (has_a) {
      split_q8_pair(areg, h0, h1, d);
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        auto &sb        = st.blk[s_pair * 2 + b];
        sb.a[0][s_row] = h0[b];
        sb.a[1][s_row] = h1[b];
        sb.da[s_row]   = live ? d[b] : 0.0f;
      }
    }
    if (has_w) {
      if constexpr (WT == kQ4_0) {
        split_q4_pair(wreg, h0, h1, d);
      } else {
        split_q8_pair(wreg, h0, h1, d);
      }
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        auto &sb        = st.blk[s_pair * 2 + b];
        sb.b[0][s_row] = h0[b];
        sb.b[1][s_row] = h1[b];
        sb.dw[s_row]   = live ? d[b] : 0.0f;
      }
    }
  };

  float acc[TM][16];
#pragma unroll
  for (int t = 0; t < TM; ++t) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[t][r] = 0.0f;
    }
  }

  const int n_steps = (pairs + 1) / 2;
  const int half    = lane >> 5;  // which 16 K-values of the block this lane feeds
  const int col     = lane & 31;  // n within the wave tile (B operand row, D column)

  fetch(0);
  stash(0, stages[0]);
  __syncthreads();

  for (int step = 0; step < n_steps; ++step) {
    StageT &cur = stages[step & 1];
    if (step + 1 < n_steps) {
      fetch(step + 1);
    }
#pragma unroll
    for (int kb = 0; kb < KB_STEP; ++kb) {
      const auto &sb = cur.blk[kb];
      const uint4 bq = sb.b[half][wn * 32 + col];
      const float dw = sb.dw[wn * 32 + col];
      const v4i   bf = { (int) bq.x, (int) bq.y, (int) bq.z, (int) bq.w };
#pragma unroll
      for (int t = 0; t < TM; ++t) {
        const int   mrow = (wm * TM + t) * 32;
        const uint4 aq   = sb.a[half][mrow + col];
        const v4i   af   = { (int) aq.x, (int) aq.y, (int) aq.z, (int) aq.w };
        v16i        s    = { 0 };
        s                = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bf, s, 0, 0, 0);
        // D[i][j]: j = lane % 32 (n), i = 8 * (r / 4) + 4 * (lane / 32) + r % 4 (m)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int   i  = 8 * (r >> 2) + 4 * half + (r & 3);
          const float da = sb.da[mrow + i];
          acc[t][r] += ((float) s[r] * dw) * da;
        }
      }
    }
    if (step + 1 < n_steps) {
      stash(step + 1, stages[(step + 1) & 1]);
    }
    __syncthreads();
  }

  // store: out[m][n], n contiguous across lanes
#pragma unroll
  for (int t = 0; t < TM; ++t) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int mi = m0 + (wm * TM + t) * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
      const int ni = n0 + wn * 32 + col;
      if (mi < m && ni < n) {
        out[(size_t) mi * n + ni] = acc[t][r];
      }
    }
  }
}

template <int WT, int WM, int TM>
hipError_t launch_gemm_instance(hipStream_t stream, float *out, const uint32_t *act, const uint32_t *w, int m, int n,
                                int pairs) {
  constexpr int BM = WM * TM * 32, BN = (4 / WM) * 32;
  const dim3    grid((unsigned) ((n + BN - 1) / BN), (unsigned) ((m + BM - 1) / BM));
  hipLaunchKernelGGL((gemm_q8_0_act_kernel<WT, WM, TM>), grid, dim3(kThreads), 2 * sizeof(Stage<BM, BN>), stream, out,
                     act, w, m, n, pairs);
  return hipGetLastError();
}

// ================================================================================================ large m

typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float    v16f __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(1))) const void *gptr_t;
typedef __attribute__((address_space(3))) void       *lptr_t;

constexpr int G3_BM = 128, G3_BN = 64, G3_KB = 2;  // tile and quant blocks per K step
constexpr int G3_SLICES = G3_KB * 4;               // 16-byte (8 x fp16) K slices per row per step

// 4 bytes (each 0..255 after the caller's bias) -> 4 integer-valued halfs minus `bias`, as two packed registers
__device__ __forceinline__ void bytes_to_halfs(uint32_t u, float bias, uint32_t &lo, uint32_t &hi) {
  const uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);  // 0x6400 | byte0, 0x6400 | byte1
  const uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);  // 1024 + byte as fp16
  const v2h      b  = { (_Float16) bias, (_Float16) bias };
  const v2h      r0 = __builtin_bit_cast(v2h, p0) - b;
  const v2h      r1 = __builtin_bit_cast(v2h, p1) - b;
  lo                = __builtin_bit_cast(uint32_t, r0);
  hi                = __builtin_bit_cast(uint32_t, r1);
}

// Pre-pass: block_q8_0 [m][pairs * 2] -> aq [pairs * 8][mp] 16-byte pieces (8 integer-valued halfs), da [pairs * 2][mp]
// fp16 scales. Rows m .. mp - 1 are zero filled. One thread per (row, pair).
__global__ __launch_bounds__(256) void gemm_prepare_act_kernel(uint4 *__restrict__ aq, uint16_t *__restrict__ da,
                                                               const uint32_t *__restrict__ act, int m, int mp,
                                                               int pairs) {
  const int row  = blockIdx.x * 64 + (threadIdx.x & 63);
  const int pair = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (row >= mp || pair >= pairs) {
    return;
  }
  uint32_t q[16];
  uint16_t d0 = 0, d1 = 0;
  if (row < m) {
    uint32_t p[17];
    load_pair<17>(p, act + ((size_t) row * pairs + pair) * 17);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      q[i]     = alignbyte2(p[i + 1], p[i]);
      q[8 + i] = p[9 + i];
    }
    d0 = (uint16_t) (p[0] & 0xffffu);
    d1 = (uint16_t) (p[8] >> 16);
#pragma unroll
    for (int s = 0; s < 8; ++s) {  // slice s = bytes 8 s .. 8 s + 7 of the pair's 64 values
      uint4 o;
      bytes_to_halfs(q[2 * s] ^ 0x80808080u, 1152.0f, o.x, o.y);
      bytes_to_halfs(q[2 * s + 1] ^ 0x80808080u, 1152.0f, o.z, o.w);
      aq[((size_t) pair * 8 + s) * mp + row] = o;
    }
  } else {
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      aq[((size_t) pair * 8 + s) * mp + row] = make_uint4(0, 0, 0, 0);
    }
  }
  da[((size_t) pair * 2 + 0) * mp + row] = d0;
  da[((size_t) pair * 2 + 1) * mp + row] = d1;
}

template <int WT>
struct G3Raw {
  static constexpr int kDwords = WPair<WT>::kDwords;              // per row per K step
  static constexpr int kInstrs = (16 * kDwords + kWave - 1) / kWave;  // DMA dword instructions per wave per step
};

// ring slot filled by DMA two K steps ahead: activation tile, activation scales, raw weight pairs
template <int WT>
struct __attribute__((aligned(16))) G3Slot {
  uint4    a[G3_SLICES][G3_BM];  // [kb * 4 + kstep * 2 + half][m row]: 8 halfs each
  uint16_t da[kWave * 8];        // 1 KiB DMA target: [kb][m row] in the first G3_KB * G3_BM entries
  uint32_t raw[4][G3Raw<WT>::kInstrs * kWave];  // per wave: 16 rows x kDwords, row-major
};
// converted weights of one K step
struct __attribute__((aligned(16))) G3B {
  uint4    b[G3_SLICES][G3_BN + 1];  // one piece of padding per slice: the four converting lanes of a row hit four banks
  uint16_t dw[G3_KB][G3_BN];
};

template <int N>
__device__ __forceinline__ void g3_wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// LDS traffic of this wave has landed, then a workgroup barrier without the global-memory fence of __syncthreads()
// (that fence would wait for the DMA that is meant to stay in flight)
__device__ __forceinline__ void g3_block_sync() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <int WT>
__global__ __launch_bounds__(256) void gemm_mfma3_kernel(float *__restrict__ out, const uint4 *__restrict__ aq,
                                                         const uint16_t *__restrict__ da_g,
                                                         const uint32_t *__restrict__ w, int m, int mp, int n,
                                                         int pairs) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  using Slot            = G3Slot<WT>;
  Slot         *slots   = reinterpret_cast<Slot *>(smem);
  G3B          *bbuf    = reinterpret_cast<G3B *>(smem + 3 * sizeof(Slot));
  constexpr int WD      = G3Raw<WT>::kDwords;
  constexpr int RAW_INS = G3Raw<WT>::kInstrs;
  constexpr int PER_STEP = 4 + RAW_INS;  // DMA instructions per wave per K step (wave 0 issues one more)

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm   = wave >> 1, wn = wave & 1;
  const int half = lane >> 5, col = lane & 31;
  // Tile mapping: workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2. When the number of
  // m-tiles divides 8, every XCD is given one m-tile only, so the activation tile (re-read by every n-tile) stays
  // in that XCD's L2 instead of streaming from memory for each of the n / 64 workgroups.
  const int m_tiles = mp / G3_BM, n_tiles = (n + G3_BN - 1) / G3_BN;
  int       mt, nt;
  if (m_tiles <= 8 && 8 % m_tiles == 0) {
    const int per = 8 / m_tiles, xcd = blockIdx.x & 7;
    mt            = xcd % m_tiles;
    nt            = (blockIdx.x >> 3) * per + xcd / m_tiles;
  } else {
    mt = blockIdx.x % m_tiles;
    nt = blockIdx.x / m_tiles;
  }
  if (nt >= n_tiles) {
    return;  // whole workgroup, before any barrier
  }
  const int m0 = mt * G3_BM;
  const int n0 = nt * G3_BN;

  // conversion task of this lane: (row of the wave's 16, block of the pair, 8-byte half (Q4_0) / 16-byte k-step (Q8_0))
  const int t_row = lane >> 2, t_blk = (lane >> 1) & 1, t_sub = lane & 1;

  // Everything the K loop needs arrives by global_load_lds DMA, so the only vmcnt traffic is counted by hand:
  // 4 x 1 KiB of the activation tile, RAW_INS dword-wide instructions for the wave's own 16 weight rows (lane e of
  // instruction j fetches dword (j * 64 + e) of the 16 x WD block, i.e. each row's pair is read contiguously), and on
  // wave 0 the 512 bytes of activation scales. Steps past the end repeat the last one (keeps the counts fixed).
  // per-lane source pointers of step 0; every K step advances them by a fixed stride
  const uint4 *a_src[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int inst = wave * 4 + j;  // 0..15: slice = inst / 2, rows (inst % 2) * 64 ..
    a_src[j]       = aq + (size_t) (inst >> 1) * mp + m0 + (inst & 1) * 64 + lane;
  }
  const uint32_t *raw_src[RAW_INS];
#pragma unroll
  for (int j = 0; j < RAW_INS; ++j) {
    const int e   = min(j * kWave + lane, 16 * WD - 1);
    const int row = e / WD, d = e % WD;
    raw_src[j]    = w + (size_t) min(n0 + wave * 16 + row, n - 1) * pairs * WD + d;
  }
  const uint16_t *da_src    = da_g + (size_t) ((lane >> 4) & 1) * mp + m0 + (lane & 15) * 8;
  const size_t    a_stride  = (size_t) G3_SLICES * mp;  // uint4 units per step
  const size_t    da_stride = (size_t) G3_KB * mp;
  auto            dma       = [&](int step_raw, Slot &sl) {
    const size_t step = (size_t) min(step_raw, pairs - 1);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int inst = wave * 4 + j;
      __builtin_amdgcn_global_load_lds((gptr_t) (a_src[j] + step * a_stride), (lptr_t) &sl.a[inst >> 1][(inst & 1) * 64], 16,
                                       0, 0);
    }
#pragma unroll
    for (int j = 0; j < RAW_INS; ++j) {
      __builtin_amdgcn_global_load_lds((gptr_t) (raw_src[j] + step * WD), (lptr_t) &sl.raw[wave][j * kWave], 4, 0, 0);
    }
    if (wave == 0) {
      // lanes 0..15: block 0, 16..31: block 1 (256 bytes = 128 rows each); the upper lanes repeat into the padding
      __builtin_amdgcn_global_load_lds((gptr_t) (da_src + step * da_stride), (lptr_t) &sl.da[0], 16, 0, 0);
    }
  };
  // the wave's own raw rows -> integer-valued fp16 slices + scales
  auto convert = [&](const Slot &sl, G3B &bb) {
    const uint32_t *p    = &sl.raw[wave][t_row * WD];
    const int       brow = wave * 16 + t_row;
    if (WT == kQ4_0) {
      // block b's quants start at byte 18 b + 2 of the pair; this task takes bytes 8 sub .. 8 sub + 7 of them
      const int off = t_blk ? 5 + 2 * t_sub : 2 * t_sub;
      uint32_t  x0 = p[off], x1 = p[off + 1];
      if (!t_blk) {
        const uint32_t x2 = p[off + 2];  // block 0 is skewed by two bytes
        x0 = alignbyte2(x1, x0);
        x1 = alignbyte2(x2, x1);
      }
      uint4 lo, hi;
      bytes_to_halfs(x0 & 0x0f0f0f0fu, 1032.0f, lo.x, lo.y);
      bytes_to_halfs(x1 & 0x0f0f0f0fu, 1032.0f, lo.z, lo.w);
      bytes_to_halfs((x0 >> 4) & 0x0f0f0f0fu, 1032.0f, hi.x, hi.y);
      bytes_to_halfs((x1 >> 4) & 0x0f0f0f0fu, 1032.0f, hi.z, hi.w);
      // low nibbles = elements 8 sub .. 8 sub + 7: k-step 0, half = sub; high nibbles: k-step 1
      bb.b[t_blk * 4 + 0 + t_sub][brow] = lo;
      bb.b[t_blk * 4 + 2 + t_sub][brow] = hi;
      if (t_sub == 0) {
        bb.dw[t_blk][brow] = (uint16_t) (t_blk ? p[4] >> 16 : p[0] & 0xffffu);
      }
    } else {
      // block b's quants start at byte 34 b + 2; this task takes bytes 16 sub .. 16 sub + 15
      const int off = t_blk ? 9 + 4 * t_sub : 4 * t_sub;
      uint32_t  x[4] = { p[off], p[off + 1], p[off + 2], p[off + 3] };
      if (!t_blk) {
        const uint32_t x4 = p[off + 4];
        x[0] = alignbyte2(x[1], x[0]);
        x[1] = alignbyte2(x[2], x[1]);
        x[2] = alignbyte2(x[3], x[2]);
        x[3] = alignbyte2(x4, x[3]);
      }
      uint4 s0, s1;  // k-step = sub, halves 0 and 1
      bytes_to_halfs(x[0] ^ 0x80808080u, 1152.0f, s0.x, s0.y);
      bytes_to_halfs(x[1] ^ 0x80808080u, 1152.0f, s0.z, s0.w);
      bytes_to_halfs(x[2] ^ 0x80808080u, 1152.0f, s1.x, s1.y);
      bytes_to_halfs(x[3] ^ 0x80808080u, 1152.0f, s1.z, s1.w);
      bb.b[t_blk * 4 + t_sub * 2 + 0][brow] = s0;
      bb.b[t_blk * 4 + t_sub * 2 + 1][brow] = s1;
      if (t_sub == 0) {
        bb.dw[t_blk][brow] = (uint16_t) (t_blk ? p[8] >> 16 : p[0] & 0xffffu);
      }
    }
  };
  auto wait_older = [&]() {  // everything except the newest step's DMA has landed
    if (wave == 0) {
      g3_wait_vmcnt<PER_STEP + 1>();
    } else {
      g3_wait_vmcnt<PER_STEP>();
    }
  };

  v16f acc[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[t][r] = 0.0f;
    }
  }

  dma(0, slots[0]);
  dma(1, slots[1]);
  wait_older();
  convert(slots[0], bbuf[0]);
  g3_block_sync();

  // Per K step: the DMA for step + 1 was requested a full step ago and is awaited first; the request for
  // step + 2 goes out next; then the MFMA work of this step and the conversion of the next step's weights sit in
  // one basic block with nothing between them, so the conversion runs in the shadow of the matrix instructions.
  for (int step = 0; step < pairs; ++step) {
    const Slot &cur = slots[step % 3];
    const G3B  &cb  = bbuf[step & 1];
    g3_wait_vmcnt<0>();
    dma(step + 2, slots[(step + 2) % 3]);
    // four (kb, m-tile) units per step; the FMAs of a unit are issued behind the MFMAs of the next one so that the
    // vector ALU works in the shadow of the matrix pipe
    v16f c_prev, s_prev;
    int  t_prev = 0;
#pragma unroll
    for (int u = 0; u < 2 * G3_KB; ++u) {
      const int      kb   = u >> 1, t = u & 1;
      const uint16_t dwb  = cb.dw[kb][wn * 32 + col];
      const v4h      dwf  = { half == 0 ? __builtin_bit_cast(_Float16, dwb) : (_Float16) 0, 0, 0, 0 };
      const int      mrow = wm * 64 + t * 32;
      const uint16_t dab  = cur.da[kb * G3_BM + mrow + col];
      const v4h      daf  = { half == 0 ? __builtin_bit_cast(_Float16, dab) : (_Float16) 0, 0, 0, 0 };
      v16f           c    = { 0 };
      c                   = __builtin_amdgcn_mfma_f32_32x32x8f16(daf, dwf, c, 0, 0, 0);
      v16f sum            = { 0 };
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const v8h af = __builtin_bit_cast(v8h, cur.a[kb * 4 + s2 * 2 + half][mrow + col]);
        const v8h bf = __builtin_bit_cast(v8h, cb.b[kb * 4 + s2 * 2 + half][wn * 32 + col]);
        sum          = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, sum, 0, 0, 0);
      }
      if (u > 0) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          acc[t_prev][r] = __builtin_fmaf(s_prev[r], c_prev[r], acc[t_prev][r]);
        }
      }
      c_prev = c, s_prev = sum, t_prev = t;
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[t_prev][r] = __builtin_fmaf(s_prev[r], c_prev[r], acc[t_prev][r]);
    }
    if (step + 1 < pairs) {
      convert(slots[(step + 1) % 3], bbuf[(step + 1) & 1]);
    }
    g3_block_sync();
  }
  g3_wait_vmcnt<0>();  // nothing may still be writing into this workgroup's LDS when it exits

#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int mi = m0 + wm * 64 + t * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
      const int ni = n0 + wn * 32 + col;
      if (mi < m && ni < n) {
        out[(size_t) mi * n + ni] = acc[t][r];
      }
    }
  }
}

template <int WT>
size_t g3_lds_bytes() {
  return 3 * sizeof(G3Slot<WT>) + 2 * sizeof(G3B);
}

}  // namespace

size_t gemm_workspace_bytes(int m, int k) {
  if (m < 64 || (k / kQK) % 2 != 0) {
    return 0;
  }
  const size_t mp = ((size_t) m + G3_BM - 1) / G3_BM * G3_BM;
  return mp * (size_t) k * 2 + mp * (size_t) (k / kQK) * 2 + 256;
}

hipError_t launch_gemm_q8_0_act(hipStream_t stream, float *out, const void *act, const void *weight, int m, int k,
                                int n, WeightType wt, void *workspace) {
  static const int use_mfma3 = env_int("HTPOPS_GEMM_MFMA3", 1);
  const int nblk = k / kQK;
  if (nblk % 2 != 0 || ((reinterpret_cast<uintptr_t>(act) | reinterpret_cast<uintptr_t>(weight)) & 3) != 0) {
    return hipErrorNotSupported;  // odd block counts / unaligned rows go to the generic kernel
  }
  const int       pairs = nblk / 2;
  const uint32_t *a     = (const uint32_t *) act;
  const uint32_t *w     = (const uint32_t *) weight;
  if (m >= 64 && workspace && use_mfma3) {
    const int mp  = (m + G3_BM - 1) / G3_BM * G3_BM;
    uint4    *aq  = static_cast<uint4 *>(workspace);
    uint16_t *da  = reinterpret_cast<uint16_t *>(static_cast<uint8_t *>(workspace) + (size_t) mp * k * 2);
    hipLaunchKernelGGL(gemm_prepare_act_kernel, dim3((unsigned) (mp / 64), (unsigned) ((pairs + 3) / 4)), dim3(256), 0,
                       stream, aq, da, a, m, mp, pairs);
    const int m_tiles = mp / G3_BM, n_tiles = (n + G3_BN - 1) / G3_BN;
    unsigned  n_groups;
    if (m_tiles <= 8 && 8 % m_tiles == 0) {
      const int per = 8 / m_tiles;
      n_groups      = 8u * (unsigned) ((n_tiles + per - 1) / per);
    } else {
      n_groups = (unsigned) m_tiles * (unsigned) n_tiles;
    }
    const dim3 grid(n_groups);
    static bool raised = false;
    if (!raised) {
      hipError_t e1 = hipFuncSetAttribute((const void *) gemm_mfma3_kernel<kQ4_0>,
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int) g3_lds_bytes<kQ4_0>());
      hipError_t e2 = hipFuncSetAttribute((const void *) gemm_mfma3_kernel<kQ8_0>,
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int) g3_lds_bytes<kQ8_0>());
      if (e1 != hipSuccess || e2 != hipSuccess) {
        return e1 != hipSuccess ? e1 : e2;
      }
      raised = true;
    }
    if (wt == kQ4_0) {
      hipLaunchKernelGGL(gemm_mfma3_kernel<kQ4_0>, grid, dim3(256), g3_lds_bytes<kQ4_0>(), stream, out, aq, da, w, m,
                         mp, n, pairs);
    } else {
      hipLaunchKernelGGL(gemm_mfma3_kernel<kQ8_0>, grid, dim3(256), g3_lds_bytes<kQ8_0>(), stream, out, aq, da, w, m,
                         mp, n, pairs);
    }
    return hipGetLastError();
  }
  if (m <= 32) {
    return wt == kQ4_0 ? launch_gemm_instance<kQ4_0, 1, 1>(stream, out, a, w, m, n, pairs) :
                         launch_gemm_instance<kQ8_0, 1, 1>(stream, out, a, w, m, n, pairs);
  }
  return wt == kQ4_0 ? launch_gemm_instance<kQ4_0, 2, 2>(stream, out, a, w, m, n, pairs) :
                       launch_gemm_instance<kQ8_0, 2, 2>(stream, out, a, w, m, n, pairs);
}

}  // namespace htpops
