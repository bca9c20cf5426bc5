// RMSNorm for gfx950: y = x * (1 / sqrtf(mean(x^2) + eps)) [* w].
//
// Replaces hvx_rms_norm_f32 (reference: src/dsp/ops/rms_norm.c:8-84), which makes two passes per row and handles
// rows one after another. Here one workgroup owns a row, keeps it in registers (rows up to 16384 floats), reduces
// the sum of squares with wave shuffles plus one LDS exchange, and writes the scaled row: 4 bytes read and
// 4 bytes written per element. Longer rows take a second read that hits L2.
// The fused variant quantizes the normalized row to Q8_0 without writing the fp32 intermediate.
#include "device_utils.h"
#include "kernels.h"

namespace htpops {

namespace {

constexpr int kThreads = 256;
constexpr int kWaves   = kThreads / kWave;

__device__ __forceinline__ float block_sum(float v, float *lds) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) {
    lds[wave] = v;
  }
  __syncthreads();
  float total = 0.0f;
#pragma unroll
  for (int i = 0; i < kWaves; ++i) {
    total += lds[i];
  }
  return total;
}

// Each thread keeps PAIRS slices of 8 consecutive floats in registers (slice index = thread + i * kThreads), which
// covers rows up to kThreads * 8 * PAIRS floats. The slice mapping and the order of the partial sums are the same
// as in the fused quantizing kernel below, so both compute bit-identical row scales. Needs ne0 % 8 == 0 and
// 16-byte aligned rows (the launcher falls back otherwise).
template <int PAIRS>
__global__ __launch_bounds__(kThreads) void rms_norm_reg_kernel(float *__restrict__ dst, const float *__restrict__ src,
                                                                const float *__restrict__ weight, float eps, int ne0) {
  __shared__ float lds[kWaves];
  const size_t row = blockIdx.x;
  const float *x   = src + row * ne0;
  float       *y   = dst + row * ne0;
  const int    n8  = ne0 / 8;

  // (short rows fetch their norm weights together with the row instead of behind the sum of squares: one trip to
  // memory less in a kernel that is a chain of such trips; longer rows would pay for that with registers)
  constexpr bool kEarly = PAIRS <= 2;
  float v[PAIRS][8], gw[kEarly ? PAIRS : 1][8];
  float ss = 0.0f;
#pragma unroll
  for (int b = 0; b < PAIRS; ++b) {
    const int idx = threadIdx.x + b * kThreads;
    if (idx < n8) {
      const float4 *p  = reinterpret_cast<const float4 *>(x + idx * 8);
      const float4  a0 = p[0], a1 = p[1];
      v[b][0] = a0.x, v[b][1] = a0.y, v[b][2] = a0.z, v[b][3] = a0.w;
      v[b][4] = a1.x, v[b][5] = a1.y, v[b][6] = a1.z, v[b][7] = a1.w;
      if (kEarly && weight) {
        const float4 *wp = reinterpret_cast<const float4 *>(weight + idx * 8);
        const float4  w0 = wp[0], w1 = wp[1];
        float        *g  = gw[kEarly ? b : 0];
        g[0] = w0.x, g[1] = w0.y, g[2] = w0.z, g[3] = w0.w, g[4] = w1.x, g[5] = w1.y, g[6] = w1.z, g[7] = w1.w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        v[b][i] = 0.0f;
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      ss = __fmaf_rn(v[b][i], v[b][i], ss);
    }
  }
  const float sum   = block_sum(ss, lds);
  const float mean  = sum / (float) ne0;
  const float scale = 1.0f / sqrtf(mean + eps);
#pragma unroll
  for (int b = 0; b < PAIRS; ++b) {
    const int idx = threadIdx.x + b * kThreads;
    if (idx < n8) {
      float o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        o[i] = v[b][i] * scale;
      }
      if (weight && kEarly) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          o[i] *= gw[kEarly ? b : 0][i];
        }
      } else if (weight) {
        const float4 *wp = reinterpret_cast<const float4 *>(weight + idx * 8);
        const float4  w0 = wp[0], w1 = wp[1];
        o[0] *= w0.x, o[1] *= w0.y, o[2] *= w0.z, o[3] *= w0.w;
        o[4] *= w1.x, o[5] *= w1.y, o[6] *= w1.z, o[7] *= w1.w;
      }
      float4 *q = reinterpret_cast<float4 *>(y + idx * 8);
      q[0]      = make_float4(o[0], o[1], o[2], o[3]);
      q[1]      = make_float4(o[4], o[5], o[6], o[7]);
    }
  }
}

// Any ne0 / alignment: scalar loads, two reads of the row.
__global__ __launch_bounds__(kThreads) void rms_norm_generic_kernel(float *__restrict__ dst,
                                                                    const float *__restrict__ src,
                                                                    const float *__restrict__ weight, float eps,
                                                                    int ne0) {
  __shared__ float lds[kWaves];
  const size_t row = blockIdx.x;
  const float *x   = src + row * ne0;
  float       *y   = dst + row * ne0;
  float        ss  = 0.0f;
  for (int i = threadIdx.x; i < ne0; i += kThreads) {
    ss += x[i] * x[i];
  }
  const float sum   = block_sum(ss, lds);
  const float mean  = sum / (float) ne0;
  const float scale = 1.0f / sqrtf(mean + eps);
  for (int i = threadIdx.x; i < ne0; i += kThreads) {
    float o = x[i] * scale;
    if (weight) {
      o *= weight[i];
    }
    y[i] = o;
  }
}

// Fused RMSNorm -> Q8_0. Four neighbouring lanes hold one quant block (8 floats each) and exchange amax inside the
// quad; BPT slices per thread in registers (rows up to kThreads * 8 * BPT floats). Needs ne0 % 32 == 0.
template <int BPT>
__global__ __launch_bounds__(kThreads) void rms_norm_quantize_kernel(uint8_t *__restrict__ dst,
                                                                     const float *__restrict__ src,
                                                                     const float *__restrict__ weight, float eps,
                                                                     int ne0) {
  __shared__ float lds[kWaves];
  const size_t row = blockIdx.x;
  const int    nb  = ne0 / kQK;
  const float *x   = src + row * ne0;
  uint8_t     *out = dst + row * (size_t) nb * 34;

  // slice s = thread + b * kThreads holds floats 8 s .. 8 s + 7: a quad of lanes covers one quant block
  const int      part   = threadIdx.x & 3;
  constexpr bool kEarly = BPT <= 2;  // (norm weights of short rows together with the row, see rms_norm_reg_kernel)
  float          v[BPT][8], gw[kEarly ? BPT : 1][8];
  float          ss = 0.0f;
#pragma unroll
  for (int b = 0; b < BPT; ++b) {
    const int blk = (threadIdx.x >> 2) + b * (kThreads / 4);
    if (blk < nb) {
      const float4 *p  = reinterpret_cast<const float4 *>(x + blk * kQK + part * 8);
      const float4  a0 = p[0], a1 = p[1];
      v[b][0] = a0.x, v[b][1] = a0.y, v[b][2] = a0.z, v[b][3] = a0.w;
      v[b][4] = a1.x, v[b][5] = a1.y, v[b][6] = a1.z, v[b][7] = a1.w;
      if (kEarly && weight) {
        const float4 *wp = reinterpret_cast<const float4 *>(weight + blk * kQK + part * 8);
        const float4  w0 = wp[0], w1 = wp[1];
        float        *g  = gw[kEarly ? b : 0];
        g[0] = w0.x, g[1] = w0.y, g[2] = w0.z, g[3] = w0.w, g[4] = w1.x, g[5] = w1.y, g[6] = w1.z, g[7] = w1.w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        v[b][i] = 0.0f;
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      ss = __fmaf_rn(v[b][i], v[b][i], ss);
    }
  }
  const float sum   = block_sum(ss, lds);
  const float mean  = sum / (float) ne0;
  const float scale = 1.0f / sqrtf(mean + eps);

#pragma unroll
  for (int b = 0; b < BPT; ++b) {
    const int blk = (threadIdx.x >> 2) + b * (kThreads / 4);
    float     amax = 0.0f;
    float     y[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      y[i] = v[b][i] * scale;
    }
    if (weight && blk < nb && kEarly) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        y[i] *= gw[kEarly ? b : 0][i];
      }
    } else if (weight && blk < nb) {
      const float4 *wp = reinterpret_cast<const float4 *>(weight + blk * kQK + part * 8);
      const float4  w0 = wp[0], w1 = wp[1];
      y[0] *= w0.x, y[1] *= w0.y, y[2] *= w0.z, y[3] *= w0.w;
      y[4] *= w1.x, y[5] *= w1.y, y[6] *= w1.z, y[7] *= w1.w;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      amax = fmaxf(amax, fabsf(y[i]));
    }
    amax           = quad_max(amax);
    const float d  = amax / 127.0f;
    const float id = (d != 0.0f) ? 1.0f / d : 0.0f;
    if (blk < nb) {
      uint16_t *o16 = reinterpret_cast<uint16_t *>(out + (size_t) blk * 34);
      if (part == 0) {
        o16[0] = __half_as_ushort(__float2half_rn(d));
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int q0 = (int) roundf(y[2 * i] * id), q1 = (int) roundf(y[2 * i + 1] * id);
        o16[1 + part * 4 + i] = (uint16_t) ((q0 & 0xff) | ((q1 & 0xff) << 8));
      }
    }
  }
}

bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

}  // namespace

hipError_t launch_rms_norm_f32(hipStream_t stream, float *dst, const float *src, const float *weight, float eps,
                               int ne0, int ne1) {
  const bool vec_ok = (ne0 % 8 == 0) && aligned16(dst) && aligned16(src) && (!weight || aligned16(weight));
  const int  n8     = ne0 / 8;
  dim3       grid((unsigned) ne1), block(kThreads);
  if (vec_ok && n8 <= kThreads * 1) {
    hipLaunchKernelGGL(rms_norm_reg_kernel<1>, grid, block, 0, stream, dst, src, weight, eps, ne0);
  } else if (vec_ok && n8 <= kThreads * 2) {
    hipLaunchKernelGGL(rms_norm_reg_kernel<2>, grid, block, 0, stream, dst, src, weight, eps, ne0);
  } else if (vec_ok && n8 <= kThreads * 4) {
    hipLaunchKernelGGL(rms_norm_reg_kernel<4>, grid, block, 0, stream, dst, src, weight, eps, ne0);
  } else if (vec_ok && n8 <= kThreads * 8) {
    hipLaunchKernelGGL(rms_norm_reg_kernel<8>, grid, block, 0, stream, dst, src, weight, eps, ne0);
  } else {
    hipLaunchKernelGGL(rms_norm_generic_kernel, grid, block, 0, stream, dst, src, weight, eps, ne0);
  }
  return hipGetLastError();
}

hipError_t launch_rms_norm_quantize_q8_0(hipStream_t stream, void *dst, const float *src, const float *weight,
                                         float eps, int ne0, int ne1) {
  const int nb = ne0 / kQK;
  dim3      grid((unsigned) ne1), block(kThreads);
  uint8_t  *out = (uint8_t *) dst;
  if (nb <= (kThreads / 4) * 1) {
    hipLaunchKernelGGL(rms_norm_quantize_kernel<1>, grid, block, 0, stream, out, src, weight, eps, ne0);
  } else if (nb <= (kThreads / 4) * 2) {
    hipLaunchKernelGGL(rms_norm_quantize_kernel<2>, grid, block, 0, stream, out, src, weight, eps, ne0);
  } else if (nb <= (kThreads / 4) * 4) {
    hipLaunchKernelGGL(rms_norm_quantize_kernel<4>, grid, block, 0, stream, out, src, weight, eps, ne0);
  } else if (nb <= (kThreads / 4) * 8) {
    hipLaunchKernelGGL(rms_norm_quantize_kernel<8>, grid, block, 0, stream, out, src, weight, eps, ne0);
  } else {
    return hipErrorInvalidValue;  // rows longer than 16384: the C-ABI layer runs the two ops separately
  }
  return hipGetLastError();
}

}  // namespace htpops
