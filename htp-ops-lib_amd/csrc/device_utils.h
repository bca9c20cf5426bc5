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

// The same over the 64 lanes of a wave and over quads with DPP row operations: no trip through the LDS crossbar, which
// is what a kernel that is one chain of dependent latencies wants. Every lane gets the result. (The additions of
// wave_sum come in another order than group_sum's; kernels that must agree bit for bit use the same one.)
#define HTPOPS_DPP_STEP(op, ctrl, rows) \
  v = op(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(ident), __float_as_int(v), ctrl, rows, 0xf, false)))
__device__ __forceinline__ float dpp_add(float a, float b) {
  return a + b;
}
__device__ __forceinline__ float wave_max(float v) {
  const float ident = -INFINITY;
  HTPOPS_DPP_STEP(fmaxf, 0xB1, 0xf);   // quad_perm [1,0,3,2]
  HTPOPS_DPP_STEP(fmaxf, 0x4E, 0xf);   // quad_perm [2,3,0,1]
  HTPOPS_DPP_STEP(fmaxf, 0x141, 0xf);  // row_half_mirror
  HTPOPS_DPP_STEP(fmaxf, 0x140, 0xf);  // row_mirror: every lane of a 16-lane row holds the row's
  HTPOPS_DPP_STEP(fmaxf, 0x142, 0xa);  // row_bcast15 into rows 1 and 3
  HTPOPS_DPP_STEP(fmaxf, 0x143, 0xc);  // row_bcast31 into rows 2 and 3: lane 63 holds the wave's
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
__device__ __forceinline__ float wave_sum(float v) {
  const float ident = 0.0f;
  HTPOPS_DPP_STEP(dpp_add, 0xB1, 0xf);
  HTPOPS_DPP_STEP(dpp_add, 0x4E, 0xf);
  HTPOPS_DPP_STEP(dpp_add, 0x141, 0xf);
  HTPOPS_DPP_STEP(dpp_add, 0x140, 0xf);
  HTPOPS_DPP_STEP(dpp_add, 0x142, 0xa);
  HTPOPS_DPP_STEP(dpp_add, 0x143, 0xc);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
// maximum over the four lanes of a quad (the same pairs in the same order as group_max<4>)
__device__ __forceinline__ float quad_max(float v) {
  const float ident = -INFINITY;
  HTPOPS_DPP_STEP(fmaxf, 0x4E, 0xf);  // quad_perm [2,3,0,1]
  HTPOPS_DPP_STEP(fmaxf, 0xB1, 0xf);  // quad_perm [1,0,3,2]
  return v;
}
#undef HTPOPS_DPP_STEP

}  // namespace htpops
