// Device-side helpers shared by the gfx950 kernels: bit casts, fp16 scale decoding, wave64 reductions.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace htpops {

constexpr int kWave = 64;
constexpr int kQK   = 32;  // values per quant block (reference: include/dsp/quants.h:7)

// 4-byte aligned 16-byte vector: quant rows are only dword aligned (18- and 34-byte blocks).
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));

__device__ __forceinline__ float half_bits_to_float(uint32_t bits16) {
  return __half2float(__ushort_as_half((unsigned short) (bits16 & 0xffffu)));
}

__device__ __forceinline__ int dot4_i8(uint32_t a, uint32_t b, int acc) {
  return __builtin_amdgcn_sdot4((int) a, (int) b, acc, false);
}

// Sum over the `width` (power of two, <= 64) consecutive lanes that share lane / width.
template <int width>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int off = width / 2; off > 0; off >>= 1) {
    v += __shfl_xor(v, off, kWave);
  }
  return v;
}

template <int width>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int off = width / 2; off > 0; off >>= 1) {
    v = fmaxf(v, __shfl_xor(v, off, kWave));
  }
  return v;
}

}  // namespace htpops
