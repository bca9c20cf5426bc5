// Q8_0 activation quantizer for gfx950.
//
// Replaces the fp32 -> fp16 activation staging of the reference (src/dsp/ops/mat_mul.c:89-128) with ggml's
// Q8_0 arithmetic: per 32-value block d = amax / 127, id = d ? 1/d : 0, q = roundf(x * id), scale = fp16(d).
// Bandwidth bound: 128 B read and 34 B written per block.
//
// Mapping: four lanes share a block (8 floats = two 16-byte loads each). amax is exchanged inside the quad,
// each lane rounds its eight values, and a wave's sixteen blocks (544 contiguous bytes) are assembled in LDS so
// that the 34-byte blocks leave as aligned dword stores.
#include "device_utils.h"
#include "kernels.h"

namespace htpops {

namespace {

constexpr int kThreads        = 256;
constexpr int kBlocksPerWave  = 16;                        // 64 lanes / 4 lanes per block
constexpr int kBlocksPerGroup = kBlocksPerWave * (kThreads / kWave);
constexpr int kWaveOutBytes   = kBlocksPerWave * 34;       // 544
constexpr int kWaveOutDwords  = kWaveOutBytes / 4;         // 136

// total_blocks = m * k / 32; blocks are contiguous in both src (128 B each) and dst (34 B each).
__global__ __launch_bounds__(kThreads) void quantize_q8_0_kernel(uint8_t *__restrict__ dst,
                                                                  const float *__restrict__ src,
                                                                  long long total_blocks) {
  __shared__ __attribute__((aligned(16))) uint16_t stage[kThreads / kWave][kWaveOutBytes / 2];

  const int       lane       = threadIdx.x & (kWave - 1);
  const int       wave       = threadIdx.x / kWave;
  const long long wave_block = ((long long) blockIdx.x * (kThreads / kWave) + wave) * kBlocksPerWave;
  if (wave_block >= total_blocks) {
    return;
  }
  const long long block = wave_block + (lane >> 2);
  const int       part  = lane & 3;  // which 8 of the block's 32 values
  const bool      live  = block < total_blocks;

  float x[8];
  if (live) {
    const float4 *p  = reinterpret_cast<const float4 *>(src + block * kQK + part * 8);
    const float4  v0 = p[0];
    const float4  v1 = p[1];
    x[0] = v0.x, x[1] = v0.y, x[2] = v0.z, x[3] = v0.w;
    x[4] = v1.x, x[5] = v1.y, x[6] = v1.z, x[7] = v1.w;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      x[i] = 0.0f;
    }
  }

  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    amax = fmaxf(amax, fabsf(x[i]));
  }
  amax = quad_max(amax);

  const float d  = amax / 127.0f;
  const float id = (d != 0.0f) ? 1.0f / d : 0.0f;

  int q[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    q[i] = (int) roundf(x[i] * id);
  }

  // LDS image of this wave's 16 blocks: block b at byte 34 b; its quants start at 34 b + 2 + 8 part.
  uint16_t *img  = stage[wave];
  const int base = ((lane >> 2) * 34 + 2 + part * 8) / 2;  // in uint16 units
  img[base + 0]  = (uint16_t) ((q[0] & 0xff) | ((q[1] & 0xff) << 8));
  img[base + 1]  = (uint16_t) ((q[2] & 0xff) | ((q[3] & 0xff) << 8));
  img[base + 2]  = (uint16_t) ((q[4] & 0xff) | ((q[5] & 0xff) << 8));
  img[base + 3]  = (uint16_t) ((q[6] & 0xff) | ((q[7] & 0xff) << 8));
  if (part == 0) {
    img[(lane >> 2) * 17] = __half_as_ushort(__float2half_rn(d));
  }
  // the image is private to this wave: a wavefront-scope release/acquire pair orders the LDS traffic
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  // 16 blocks start at a multiple of 16 blocks = 544 bytes, so the image is dword aligned in dst.
  long long remaining = total_blocks - wave_block;
  const int n_dwords  = remaining >= kBlocksPerWave ? kWaveOutDwords : (int) (remaining * 34 / 4);
  const int n_bytes   = remaining >= kBlocksPerWave ? kWaveOutBytes : (int) (remaining * 34);
  uint32_t       *out32 = reinterpret_cast<uint32_t *>(dst + wave_block * 34);
  const uint32_t *img32 = reinterpret_cast<const uint32_t *>(img);
  for (int i = lane; i < n_dwords; i += kWave) {
    out32[i] = img32[i];
  }
  // an odd number of trailing blocks leaves two bytes
  if (lane == 0 && (n_bytes & 3)) {
    reinterpret_cast<uint16_t *>(dst + wave_block * 34)[n_bytes / 2 - 1] = img[n_bytes / 2 - 1];
  }
}

}  // namespace

hipError_t launch_quantize_q8_0(hipStream_t stream, void *dst, const float *src, int k, int m) {
  const long long total_blocks = (long long) m * (k / kQK);
  const long long groups       = (total_blocks + kBlocksPerGroup - 1) / kBlocksPerGroup;
  hipLaunchKernelGGL(quantize_q8_0_kernel, dim3((unsigned) groups), dim3(kThreads), 0, stream, (uint8_t *) dst, src,
                     total_blocks);
  return hipGetLastError();
}

}  // namespace htpops
