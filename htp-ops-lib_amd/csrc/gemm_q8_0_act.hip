// Prefill-path quantized matmul for gfx950: out[m][n] = sum over 32-wide K blocks of
//   (float) (int dot of weight block (n, kb) with activation block (m, kb)) * d_w(n, kb) * d_a(m, kb)
// with the integer dots on the matrix cores (v_mfma_i32_32x32x32_i8: one instruction = 32 x 32 outputs x one quant
// block of K) and the per-block scales applied in fp32 on the vector ALU.
//
// Replaces hmx_mat_mul_permuted_qk_0_d16a32 for m > 1 (reference: src/dsp/ops/mat_mul.c:875-1153): there, weights
// are dequantized to fp16 tiles in on-chip memory and multiplied on the fp16 matrix unit; here they are unpacked to
// int8 tiles in LDS (Q4_0 nibbles - 8, Q8_0 bytes as they are), activations stay int8, and only the block sums are
// converted to floating point.
//
// Workgroup = 256 threads = 4 waves, K step = 128 (four quant blocks). Two tile shapes:
//   prefill: BM x BN = 128 x 64, waves in a 2 x 2 grid, each 64 (m) x 32 (n) = two MFMA tiles sharing the weight
//            fragment;
//   small m: BM x BN = 32 x 128, the four waves side by side along n, one MFMA tile each.
//   LDS, per K block: A[h][row] and B[h][row], 16 bytes each: the 16 K-values of half h (0: elements 0..15,
//   1: elements 16..31 -- for Q4_0 that is low nibbles / high nibbles of the same 16 bytes), so a fragment read is
//   one conflict-free ds_read_b128 per lane. Scales sit beside them as fp32.
//   Global -> LDS goes through registers one K step ahead of the MFMA loop (double-buffered LDS); the unit of
//   transfer is a pair of blocks (68 / 36 bytes: dword aligned when k % 64 == 0).
// The MFMA output layout puts n on lanes (lane % 32) and 16 values of m in registers, so the weight scale is one
// value per lane and the activation scales are LDS broadcasts.
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

}  // namespace

hipError_t launch_gemm_q8_0_act(hipStream_t stream, float *out, const void *act, const void *weight, int m, int k,
                                int n, WeightType wt) {
  const int nblk = k / kQK;
  if (nblk % 2 != 0 || ((reinterpret_cast<uintptr_t>(act) | reinterpret_cast<uintptr_t>(weight)) & 3) != 0) {
    return hipErrorNotSupported;  // odd block counts / unaligned rows go to the generic kernel
  }
  const int       pairs = nblk / 2;
  const uint32_t *a     = (const uint32_t *) act;
  const uint32_t *w     = (const uint32_t *) weight;
  if (m <= 32) {
    return wt == kQ4_0 ? launch_gemm_instance<kQ4_0, 1, 1>(stream, out, a, w, m, n, pairs) :
                         launch_gemm_instance<kQ8_0, 1, 1>(stream, out, a, w, m, n, pairs);
  }
  return wt == kQ4_0 ? launch_gemm_instance<kQ4_0, 2, 2>(stream, out, a, w, m, n, pairs) :
                       launch_gemm_instance<kQ8_0, 2, 2>(stream, out, a, w, m, n, pairs);
}

}  // namespace htpops
