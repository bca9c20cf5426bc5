// The reference's native weight formats (its ops 1-4) on gfx950.
//
// The Hexagon backend keeps weights in the order its matrix unit consumes: fp16 in 32x32 tiles
// (hmx_mat_mul_permuted_w16a32, reference: src/dsp/ops/mat_mul.c:758-855, layout src/host/test.c:300-312) or
// quantized "super-blocks" of 8 K rows x 32 N columns with one fp16 scale per 2 x 16 patch
// (hmx_mat_mul_permuted_qk_0_d16a32, mat_mul.c:875-1153; dequantizers :308-508). Both paths multiply fp16
// activations by fp16 weights and round the result to fp16.
//
// Here a weight buffer is converted ONCE (weights are immutable for the reference too, op_executor.cc:130) into the
// order the gfx950 matrix core consumes, and cached by the caller: for every 32-column tile and every 16-wide K step
// the 64 lanes' 16-byte B operands of v_mfma_f32_32x32x16_f16 lie in one contiguous KiB ("fragment order"), so the
// matmul kernel needs neither LDS nor any shuffling: both operands are loaded straight into MFMA registers.
//   lane (c = lane % 32, h = lane / 32) of fragment (tile, step) holds W[16 step + 8 h .. + 7][32 tile + c].
// Activations are converted per call (fp32 -> fp16, round to nearest even) into the same order with rows on lanes.
#include "device_utils.h"
#include "kernels.h"

namespace htpops {

namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float    v16f __attribute__((ext_vector_type(16)));

// IQ4_NL code book (reference: src/dsp/ops/mat_mul.c:29-32)
__constant__ int8_t kIq4nlDev[16] = { -127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113 };

// one thread = one 16-byte fragment piece: 8 consecutive K of one column
struct PieceCoord {
  int  tile_n, step, c, h;  // fragment coordinates
  int  k_tile, kb;          // 32x32 source tile along K, first K row inside it (0, 8, 16, 24)
  bool ok;
};

__device__ __forceinline__ PieceCoord piece_coord(size_t t, int k_steps, int n_tiles) {
  PieceCoord p;
  const int lane = (int) (t & 63);
  const size_t f = t >> 6;
  p.step   = (int) (f % (size_t) k_steps);
  p.tile_n = (int) (f / (size_t) k_steps);
  p.c = lane & 31, p.h = lane >> 5;
  const int k0 = 16 * p.step + 8 * p.h;
  p.k_tile = k0 >> 5, p.kb = k0 & 31;
  p.ok = p.tile_n < n_tiles;
  return p;
}

// fp16 tiles: element (k1, n1) of a tile sits at (k1 & ~1) * 32 + n1 * 2 + (k1 & 1)
__global__ __launch_bounds__(256) void repack_w16_tiles_kernel(uint4 *__restrict__ dst, const uint32_t *__restrict__ src,
                                                               int k_steps, int n_tiles) {
  const size_t     t = (size_t) blockIdx.x * 256 + threadIdx.x;
  const PieceCoord p = piece_coord(t, k_steps, n_tiles);
  if (!p.ok) {
    return;
  }
  const size_t tile = (size_t) p.tile_n * (k_steps / 2) + p.k_tile;
  const uint32_t *s = src + tile * 512 + (size_t) (p.kb * 32 + p.c * 2) / 2;  // dword = one K pair of column c
  dst[t] = make_uint4(s[0], s[32], s[64], s[96]);                             // row pairs are 64 halfs apart
}

__device__ __forceinline__ uint32_t pack_halfs(float a, float b) {
  // fp16(q) * fp16(scale) is exact in fp32 (|q| <= 127, 11-bit significand); one rounding to fp16
  const _Float16 x = (_Float16) a, y = (_Float16) b;
  return (uint32_t) __builtin_bit_cast(uint16_t, x) | ((uint32_t) __builtin_bit_cast(uint16_t, y) << 16);
}

// Q4_0 / IQ4_NL super-blocks (144 B: 8 scales, 128 quant bytes). The 8 K rows of a piece are the four vectors of
// ONE super-block at elements 2c and 2c + 1: vector v takes the low (v < 2) or high nibble of bytes 4c + (v & 1)
// and 4c + 2 + (v & 1), scale 2v + c / 16 (reference: mat_mul.c:319-325, :383-405).
template <bool IQ4_NL>
__global__ __launch_bounds__(256) void dequant_permuted_q4_kernel(uint4 *__restrict__ dst, const uint8_t *__restrict__ src,
                                                                  int k_steps, int n_tiles) {
  const size_t     t = (size_t) blockIdx.x * 256 + threadIdx.x;
  const PieceCoord p = piece_coord(t, k_steps, n_tiles);
  if (!p.ok) {
    return;
  }
  const size_t    tile = (size_t) p.tile_n * (k_steps / 2) + p.k_tile;
  const uint8_t  *sb   = src + (tile * 4 + (size_t) (p.kb >> 3)) * 144;
  const uint16_t *sc   = reinterpret_cast<const uint16_t *>(sb);
  const uint8_t  *qs   = sb + 16 + 4 * p.c;
  uint32_t        out[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const float d  = half_bits_to_float(sc[2 * v + (p.c >> 4)]);
    const int   b0 = qs[v & 1], b1 = qs[2 + (v & 1)];
    const int   n0 = (v & 2) ? (b0 >> 4) : (b0 & 15), n1 = (v & 2) ? (b1 >> 4) : (b1 & 15);
    const int   q0 = IQ4_NL ? (int) kIq4nlDev[n0] : n0 - 8, q1 = IQ4_NL ? (int) kIq4nlDev[n1] : n1 - 8;
    out[v]         = pack_halfs((float) q0 * d, (float) q1 * d);
  }
  dst[t] = make_uint4(out[0], out[1], out[2], out[3]);
}

// Q8_0 super-blocks (272 B: 8 scales, 256 int8): vector v = quants[64 v .. 64 v + 63] (mat_mul.c:483-505)
__global__ __launch_bounds__(256) void dequant_permuted_q8_kernel(uint4 *__restrict__ dst, const uint8_t *__restrict__ src,
                                                                  int k_steps, int n_tiles) {
  const size_t     t = (size_t) blockIdx.x * 256 + threadIdx.x;
  const PieceCoord p = piece_coord(t, k_steps, n_tiles);
  if (!p.ok) {
    return;
  }
  const size_t    tile = (size_t) p.tile_n * (k_steps / 2) + p.k_tile;
  const uint8_t  *sb   = src + (tile * 4 + (size_t) (p.kb >> 3)) * 272;
  const uint16_t *sc   = reinterpret_cast<const uint16_t *>(sb);
  const int8_t   *qs   = reinterpret_cast<const int8_t *>(sb + 16) + 2 * p.c;
  uint32_t        out[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const float d = half_bits_to_float(sc[2 * v + (p.c >> 4)]);
    out[v]        = pack_halfs((float) qs[64 * v] * d, (float) qs[64 * v + 1] * d);
  }
  dst[t] = make_uint4(out[0], out[1], out[2], out[3]);
}

// activations fp32 [m][k] -> fragment order with rows on lanes; rows >= m are zero
__global__ __launch_bounds__(256) void act_to_fragments_kernel(uint4 *__restrict__ dst, const float *__restrict__ act,
                                                               int m, int k, int m_tiles) {
  const size_t t = (size_t) blockIdx.x * 256 + threadIdx.x;
  const int    k_steps = k / 16;
  const int    lane = (int) (t & 63);
  const size_t f    = t >> 6;
  const int    step = (int) (f % (size_t) k_steps), tile = (int) (f / (size_t) k_steps);
  if (tile >= m_tiles) {
    return;
  }
  const int row = tile * 32 + (lane & 31);
  uint4     o   = make_uint4(0, 0, 0, 0);
  if (row < m) {
    const float4 *s = reinterpret_cast<const float4 *>(act + (size_t) row * k + 16 * step + 8 * (lane >> 5));
    const float4  a = s[0], b = s[1];
    o = make_uint4(pack_halfs(a.x, a.y), pack_halfs(a.z, a.w), pack_halfs(b.x, b.y), pack_halfs(b.z, b.w));
  }
  dst[t] = o;
}

// out[m][n] = fp16(sum_k A[m][k] * W[k][n]) widened to fp32; both operands in fragment order.
// A workgroup is WM x WN waves, a wave owns MT x NT tiles of 32 x 32 and walks K with DEPTH fragment sets in flight.
template <int MT, int NT, int WM, int WN>
__global__ __launch_bounds__(WM *WN * 64) void gemm_f16_fragments_kernel(float *__restrict__ out,
                                                                         const uint4 *__restrict__ a_frag,
                                                                         const uint4 *__restrict__ b_frag, int m, int n,
                                                                         int k_steps, int m_tiles, int n_tiles) {
  constexpr int DEPTH = 4;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int mt0 = (blockIdx.y * WM + wm) * MT, nt0 = (blockIdx.x * WN + wn) * NT;
  if (mt0 >= m_tiles || nt0 >= n_tiles) {
    return;  // no barriers in this kernel
  }
  const uint4 *ap[MT], *bp[NT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    ap[i] = a_frag + (size_t) min(mt0 + i, m_tiles - 1) * k_steps * 64 + lane;
  }
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    bp[j] = b_frag + (size_t) min(nt0 + j, n_tiles - 1) * k_steps * 64 + lane;
  }
  v16f acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[i][j][r] = 0.0f;
      }
    }
  }
  uint4 ar[DEPTH][MT], br[DEPTH][NT];
  auto  load = [&](int d, int step) {
    const size_t off = (size_t) min(step, k_steps - 1) * 64;  // branch-free: steps past the end repeat the last one
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      ar[d][i] = ap[i][off];
    }
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      br[d][j] = bp[j][off];
    }
  };
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    load(d, d);
  }
  for (int s0 = 0; s0 < k_steps; s0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (s0 + d < k_steps) {
#pragma unroll
        for (int i = 0; i < MT; ++i) {
#pragma unroll
          for (int j = 0; j < NT; ++j) {
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, ar[d][i]),
                                                               __builtin_bit_cast(v8h, br[d][j]), acc[i][j], 0, 0, 0);
          }
        }
      }
      load(d, s0 + d + DEPTH);
    }
  }
  // D[i][j]: j = lane % 32 (column), i = 8 (r / 4) + 4 (lane / 32) + r % 4 (row)
#pragma unroll
  for (int i = 0; i < MT; ++i) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      if (mt0 + i < m_tiles && nt0 + j < n_tiles) {
        const int col = (nt0 + j) * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = (mt0 + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          if (row < m) {
            out[(size_t) row * n + col] = (float) (_Float16) acc[i][j][r];  // the reference stores fp16 results
          }
        }
      }
    }
  }
}

}  // namespace

size_t permuted_weight_fragment_bytes(int k, int n) {
  return (size_t) k * (size_t) n * 2;
}

size_t permuted_act_fragment_bytes(int m, int k) {
  return (size_t) ((m + 31) / 32) * 32 * (size_t) k * 2;
}

hipError_t launch_permuted_weight_to_fragments(hipStream_t stream, void *dst, const void *src, int k, int n,
                                               int weight_kind) {
  if (k % 32 != 0 || n % 32 != 0 || weight_kind < 1 || weight_kind > 4) {
    return hipErrorInvalidValue;
  }
  const int    k_steps = k / 16, n_tiles = n / 32;
  const size_t pieces  = (size_t) k_steps * n_tiles * 64;
  const dim3   grid((unsigned) ((pieces + 255) / 256));
  uint4       *d = static_cast<uint4 *>(dst);
  switch (weight_kind) {
    case 1:
      hipLaunchKernelGGL(repack_w16_tiles_kernel, grid, dim3(256), 0, stream, d, static_cast<const uint32_t *>(src),
                         k_steps, n_tiles);
      break;
    case 2:
      hipLaunchKernelGGL(dequant_permuted_q4_kernel<false>, grid, dim3(256), 0, stream, d,
                         static_cast<const uint8_t *>(src), k_steps, n_tiles);
      break;
    case 3:
      hipLaunchKernelGGL(dequant_permuted_q8_kernel, grid, dim3(256), 0, stream, d, static_cast<const uint8_t *>(src),
                         k_steps, n_tiles);
      break;
    default:
      hipLaunchKernelGGL(dequant_permuted_q4_kernel<true>, grid, dim3(256), 0, stream, d,
                         static_cast<const uint8_t *>(src), k_steps, n_tiles);
      break;
  }
  return hipGetLastError();
}

hipError_t launch_mat_mul_fragments(hipStream_t stream, float *out, const float *act, const void *weight_fragments,
                                    int m, int k, int n, void *act_fragments) {
  if (k % 32 != 0 || n % 32 != 0 || m <= 0) {
    return hipErrorInvalidValue;
  }
  const int    k_steps = k / 16, n_tiles = n / 32, m_tiles = (m + 31) / 32;
  const size_t a_pieces = (size_t) m_tiles * k_steps * 64;
  hipLaunchKernelGGL(act_to_fragments_kernel, dim3((unsigned) ((a_pieces + 255) / 256)), dim3(256), 0, stream,
                     static_cast<uint4 *>(act_fragments), act, m, k, m_tiles);
  if (hipError_t e = hipGetLastError(); e != hipSuccess) {
    return e;
  }
  const uint4 *a = static_cast<const uint4 *>(act_fragments), *b = static_cast<const uint4 *>(weight_fragments);
  if (m_tiles == 1) {
    // weight streaming: one 32-column tile per wave, as many workgroups as possible
    hipLaunchKernelGGL((gemm_f16_fragments_kernel<1, 1, 1, 2>), dim3((unsigned) ((n_tiles + 1) / 2), 1), dim3(128), 0,
                       stream, out, a, b, m, n, k_steps, m_tiles, n_tiles);
  } else if (m_tiles <= 4) {
    hipLaunchKernelGGL((gemm_f16_fragments_kernel<1, 2, 2, 2>), dim3((unsigned) ((n_tiles + 3) / 4),
                                                                      (unsigned) ((m_tiles + 1) / 2)),
                       dim3(256), 0, stream, out, a, b, m, n, k_steps, m_tiles, n_tiles);
  } else {
    hipLaunchKernelGGL((gemm_f16_fragments_kernel<2, 2, 2, 2>), dim3((unsigned) ((n_tiles + 3) / 4),
                                                                      (unsigned) ((m_tiles + 3) / 4)),
                       dim3(256), 0, stream, out, a, b, m, n, k_steps, m_tiles, n_tiles);
  }
  return hipGetLastError();
}

}  // namespace htpops
