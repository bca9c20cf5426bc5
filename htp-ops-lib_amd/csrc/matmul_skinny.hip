// Quantized matmul for a handful of activation rows (2 <= m <= 32) on gfx950: out[m][n] = act_q8_0[m][k] x W[n][k].
//
// Replaces the small-batch case of hmx_mat_mul_permuted_qk_0_d16a32 (reference: src/dsp/ops/mat_mul.c:875-1153;
// the per-block arithmetic is ggml's integer block dot, restated by the CPU oracle). Like the one-row kernel the
// job is to stream the weight bytes exactly once; unlike it, every weight block meets all m activation rows, and
// that product runs on the matrix core:
//
//   v_mfma_i32_32x32x32_i8 with A = activations (one row per lane, garbage rows beyond m are never read back) and
//   B = 32 weight rows (one per lane). One instruction is one 32-element block: lane half 0 supplies elements
//   0..15 (the low nibbles of a Q4_0 block), half 1 elements 16..31 (the high nibbles), so a lane unpacks with one
//   shift and one mask per dword. The "- 8" of Q4_0 never touches the weights: the accumulator input of the MFMA
//   is preloaded with -8 * sum(act block), computed once per workgroup while the activations are staged.
//   The output holds n on lanes and m in registers: m <= 8 needs 4 of the 16 registers, so the scale epilogue is
//   4 x (convert, multiply, fma) per block instead of 16.
//
// Work is cut into (32 weight rows) x (K slice of 1024 elements) workgroups; inside one, the waves take weight
// pairs (two blocks = 36 or 68 bytes, the smallest dword-aligned unit) round-robin and are reduced through LDS.
// Activations are staged in LDS in MFMA operand order. A second kernel without K slicing (rows gathered straight
// from global memory) covers row sizes that are not multiples of 16 bytes.
#include "device_utils.h"
#include "kernels.h"

namespace htpops {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kSkThreads = 512;
constexpr int kSkWaves   = kSkThreads / kWave;
constexpr int kSkRows    = 32;  // weight rows per workgroup
constexpr int kSkPrefetch  = 2;   // weight pairs in flight per wave (gather kernel)

__device__ __forceinline__ uint32_t shift_in_2(uint32_t hi, uint32_t lo) {
  return __builtin_amdgcn_alignbyte(hi, lo, 2);  // bytes 2..5 of the 8-byte value hi:lo
}

// Weight pair -> two B operands and two scales. Q4_0: the 9 dwords of the pair; Q8_0: this half's 16 bytes of each
// block plus the two scale dwords.
template <WeightType WT>
struct PairRegs;

template <>
struct PairRegs<kQ4_0> {
  uint32_t w[9];

  __device__ __forceinline__ void load(const uint8_t *row, int pair, int) {
    const uint32_t *p = reinterpret_cast<const uint32_t *>(row + (size_t) pair * 36);
    const uint4     a = *reinterpret_cast<const uint4 *>(p);
    const uint4     b = *reinterpret_cast<const uint4 *>(p + 4);
    w[0] = a.x, w[1] = a.y, w[2] = a.z, w[3] = a.w;
    w[4] = b.x, w[5] = b.y, w[6] = b.z, w[7] = b.w;
    w[8] = p[8];
  }

  // same pair from an LDS image of the row (4-byte aligned)
  __device__ __forceinline__ void load_lds(const uint32_t *p, int) {
#pragma unroll
    for (int i = 0; i < 9; ++i) {
      w[i] = p[i];
    }
  }

  __device__ __forceinline__ void unpack(int half, v4i &b0, v4i &b1, float &d0, float &d1) const {
    const int sh = 4 * half;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      b0[i] = (int) ((shift_in_2(w[i + 1], w[i]) >> sh) & 0x0F0F0F0Fu);
      b1[i] = (int) ((w[5 + i] >> sh) & 0x0F0F0F0Fu);
    }
    d0 = half_bits_to_float((uint16_t) (w[0] & 0xffffu));
    d1 = half_bits_to_float((uint16_t) (w[4] >> 16));
  }
};

template <>
struct PairRegs<kQ8_0> {
  uint32_t u[5], v[4], s0, s1;

  __device__ __forceinline__ void load(const uint8_t *row, int pair, int half) {
    const uint32_t *p = reinterpret_cast<const uint32_t *>(row + (size_t) pair * 68);
    const uint4     a = *reinterpret_cast<const uint4 *>(p + 4 * half);
    const uint4     b = *reinterpret_cast<const uint4 *>(p + 9 + 4 * half);
    u[0] = a.x, u[1] = a.y, u[2] = a.z, u[3] = a.w;
    u[4] = p[4 * half + 4];
    v[0] = b.x, v[1] = b.y, v[2] = b.z, v[3] = b.w;
    s0 = p[0], s1 = p[8];
  }

  __device__ __forceinline__ void load_lds(const uint32_t *p, int half) {
#pragma unroll
    for (int i = 0; i < 5; ++i) {
      u[i] = p[4 * half + i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = p[9 + 4 * half + i];
    }
    s0 = p[0], s1 = p[8];
  }

  __device__ __forceinline__ void unpack(int, v4i &b0, v4i &b1, float &d0, float &d1) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      b0[i] = (int) shift_in_2(u[i + 1], u[i]);
      b1[i] = (int) v[i];
    }
    d0 = half_bits_to_float((uint16_t) (s0 & 0xffffu));
    d1 = half_bits_to_float((uint16_t) (s1 >> 16));
  }
};

// MR = registers of the MFMA result that carry real rows: rows 8 (r / 4) + 4 half + r % 4 for r < MR, i.e.
// MR = 4 / 8 / 16 covers m <= 8 / 16 / 32. MPAD = 2 MR activation-row slots are staged per block.
//
// LDS image of an activation chunk of kc blocks: a[kc][2][MPAD] 16-byte operand pieces, da[kc][2][MR] floats,
// off[kc][2][MR] ints (-8 * block sum for Q4_0 weights, 0 for Q8_0).
template <int MR>
struct ActChunk {
  static constexpr int MPAD   = 2 * MR;
  static constexpr int PER_KB = 32 * MPAD + 16 * MR;  // bytes per block
  uint4 *a;
  float *da;
  int   *off;

  __device__ __forceinline__ ActChunk(uint8_t *base, int kc) {
    a   = reinterpret_cast<uint4 *>(base);
    da  = reinterpret_cast<float *>(base + (size_t) kc * 2 * MPAD * 16);
    off = reinterpret_cast<int *>(base + (size_t) kc * 2 * MPAD * 16 + (size_t) kc * 2 * MR * 4);
  }

  // One task = (activation row, pair) -> four operand pieces, two scales, two offsets. Tasks are taken
  // kStageUnroll per thread at a time with all their loads issued before the first use.
  template <WeightType WT, int THREADS, int kStageUnroll>
  __device__ __forceinline__ void stage(const uint8_t *__restrict__ act, int m, int nblk, int pair0, int cpairs,
                                        int tid) const {
    const int n_tasks = cpairs * MPAD;
    for (int t0 = tid; t0 < n_tasks; t0 += kStageUnroll * THREADS) {
      uint32_t w[kStageUnroll][17];
#pragma unroll
      for (int u = 0; u < kStageUnroll; ++u) {
        const int t    = min(t0 + u * THREADS, n_tasks - 1);
        const int mrow = min(t % MPAD, m - 1), pl = t / MPAD;
        const uint32_t *src =
          reinterpret_cast<const uint32_t *>(act + ((size_t) mrow * nblk + 2 * (size_t) (pair0 + pl)) * 34);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint4 x = *reinterpret_cast<const uint4 *>(src + 4 * i);
          w[u][4 * i] = x.x, w[u][4 * i + 1] = x.y, w[u][4 * i + 2] = x.z, w[u][4 * i + 3] = x.w;
        }
        w[u][16] = src[16];
      }
#pragma unroll
      for (int u = 0; u < kStageUnroll; ++u) {
        const int t    = t0 + u * THREADS;
        const int mrow = t % MPAD, pl = t / MPAD;
        if (t >= n_tasks || mrow >= m) {
          continue;
        }
        uint32_t e0[8], e1[8];
        int      s0 = 0, s1 = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          e0[i] = shift_in_2(w[u][i + 1], w[u][i]);
          e1[i] = w[u][9 + i];
          s0    = __builtin_amdgcn_sdot4((int) e0[i], 0x01010101, s0, false);
          s1    = __builtin_amdgcn_sdot4((int) e1[i], 0x01010101, s1, false);
        }
        const int kl = 2 * pl;
        a[((kl + 0) * 2 + 0) * MPAD + mrow] = make_uint4(e0[0], e0[1], e0[2], e0[3]);
        a[((kl + 0) * 2 + 1) * MPAD + mrow] = make_uint4(e0[4], e0[5], e0[6], e0[7]);
        a[((kl + 1) * 2 + 0) * MPAD + mrow] = make_uint4(e1[0], e1[1], e1[2], e1[3]);
        a[((kl + 1) * 2 + 1) * MPAD + mrow] = make_uint4(e1[4], e1[5], e1[6], e1[7]);
        // result row mrow lives in lane half (mrow / 4) % 2, register 4 (mrow / 8) + mrow % 4
        const int hs = (mrow >> 2) & 1, r = 4 * (mrow >> 3) + (mrow & 3);
        da[((kl + 0) * 2 + hs) * MR + r]  = half_bits_to_float((uint16_t) (w[u][0] & 0xffffu));
        da[((kl + 1) * 2 + hs) * MR + r]  = half_bits_to_float((uint16_t) (w[u][8] >> 16));
        off[((kl + 0) * 2 + hs) * MR + r] = WT == kQ4_0 ? -8 * s0 : 0;
        off[((kl + 1) * 2 + hs) * MR + r] = WT == kQ4_0 ? -8 * s1 : 0;
      }
    }
  }

  // acc += scales * (act block kl x the 32 weight rows in bq)
  __device__ __forceinline__ void block_mac(float (&acc)[MR], int kl, int half, int a_slot, v4i bq, float dw) const {
    const uint4 aq = a[(kl * 2 + half) * MPAD + a_slot];
    const v4i   af = { (int) aq.x, (int) aq.y, (int) aq.z, (int) aq.w };
    v16i        c  = { 0 };
    float       dav[MR];
#pragma unroll
    for (int r4 = 0; r4 < MR / 4; ++r4) {
      const int4   o = *reinterpret_cast<const int4 *>(&off[(kl * 2 + half) * MR + 4 * r4]);
      const float4 d = *reinterpret_cast<const float4 *>(&da[(kl * 2 + half) * MR + 4 * r4]);
      c[4 * r4] = o.x, c[4 * r4 + 1] = o.y, c[4 * r4 + 2] = o.z, c[4 * r4 + 3] = o.w;
      dav[4 * r4] = d.x, dav[4 * r4 + 1] = d.y, dav[4 * r4 + 2] = d.z, dav[4 * r4 + 3] = d.w;
    }
    const v16i s = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bq, c, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      acc[r] = __builtin_fmaf((float) s[r], dw * dav[r], acc[r]);
    }
  }
};

// sum of the waves' accumulators through LDS (all waves must be done with the LDS they overwrite), then store
template <int MR>
__device__ __forceinline__ void reduce_and_store(float *__restrict__ out, float *red, const float (&acc)[MR], int m,
                                                 int n, int n0, int tid) {
  const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    red[(wave * MR + r) * 64 + lane] = acc[r];
  }
  __syncthreads();
  for (int i = tid; i < MR * 64; i += kSkThreads) {
    const int r = i >> 6, l = i & 63;
    float     v = 0.0f;
#pragma unroll
    for (int w = 0; w < kSkWaves; ++w) {
      v += red[(w * MR + r) * 64 + l];
    }
    const int mrow = 8 * (r >> 2) + 4 * (l >> 5) + (r & 3);
    const int col  = n0 + (l & 31);
    if (mrow < m && col < n) {
      out[(size_t) mrow * n + col] = v;
    }
  }
}

// Fallback for rows that are not 16-byte multiples: every lane gathers its own row's pairs from global memory.
template <WeightType WT, int MR, int PF>
__global__ __launch_bounds__(kSkThreads) void matmul_skinny_kernel(float *__restrict__ out,
                                                                  const uint8_t *__restrict__ act,
                                                                  const uint8_t *__restrict__ weight, int m, int k,
                                                                  int n, int kc) {
  constexpr int MPAD     = 2 * MR;
  constexpr int WROW_BLK = WT == kQ4_0 ? 18 : 34;
  extern __shared__ __align__(16) uint8_t sk_lds[];
  const ActChunk<MR> chunk(sk_lds, kc);

  const int tid  = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int nl = lane & 31, half = lane >> 5;
  const int nblk  = k / 32;
  const int n0    = blockIdx.x * kSkRows;
  const int row   = min(n0 + nl, n - 1);
  const uint8_t *wrow = weight + (size_t) row * nblk * WROW_BLK;
  const int a_slot = min(nl, MPAD - 1);

  float acc[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    acc[r] = 0.0f;
  }

  const int total_pairs = nblk / 2;
  for (int kb0 = 0; kb0 < nblk; kb0 += kc) {
    const int cblk   = min(kc, nblk - kb0);
    const int cpairs = cblk / 2;
    const int pair0  = kb0 / 2;

    // the first PF weight pairs of this wave are in flight while the activations are staged
    PairRegs<WT> ring[PF];
#pragma unroll
    for (int j = 0; j < PF; ++j) {
      ring[j].load(wrow, min(pair0 + wave + j * kSkWaves, total_pairs - 1), half);
    }
    if (kb0 > 0) {
      __syncthreads();  // every wave is done with the previous chunk
    }
    chunk.template stage<WT, kSkThreads, 3>(act, m, nblk, pair0, cpairs, tid);
    __syncthreads();

    // stream this wave's weight pairs: PF pairs in flight, reloaded branch-free with a clamped index
    for (int pl0 = wave; pl0 < cpairs; pl0 += PF * kSkWaves) {
#pragma unroll
      for (int j = 0; j < PF; ++j) {
        const int pl = pl0 + j * kSkWaves;
        if (pl < cpairs) {
          v4i   bq[2];
          float dw[2];
          ring[j].unpack(half, bq[0], bq[1], dw[0], dw[1]);
          chunk.block_mac(acc, 2 * pl, half, a_slot, bq[0], dw[0]);
          chunk.block_mac(acc, 2 * pl + 1, half, a_slot, bq[1], dw[1]);
        }
        ring[j].load(wrow, min(pair0 + pl + PF * kSkWaves, total_pairs - 1), half);
      }
    }
  }
  __syncthreads();
  reduce_and_store<MR>(out, reinterpret_cast<float *>(sk_lds), acc, m, n, n0, tid);
}

// ---------------------------------------------------------------------------------------------------------------
// Main kernel: one workgroup = 32 weight rows x one K slice of 16 pairs (1024 elements), so the grid has enough
// small workgroups to keep every CU streaming. The slice of the 32 rows reaches LDS by global_load_lds DMA in
// 16-byte pieces (contiguous 576- or 1088-byte runs of HBM), all requested before anything else happens; lanes then
// pick their row's pairs out of LDS. The K slices of a row tile are summed in a fixed order by whichever workgroup
// of the tile finishes last (a ticket counter per tile), so the result does not depend on scheduling.
// Needs row byte counts that are multiples of 16.
constexpr int kSlThreads = 256;
constexpr int kSlWaves   = kSlThreads / kWave;
constexpr int kSlPairs   = 16;  // pairs per K slice

template <WeightType WT>
struct SliceGeom {
  static constexpr int PAIRB  = WT == kQ4_0 ? 36 : 68;
  static constexpr int SEG    = kSlPairs * PAIRB;      // bytes of one row in a slice: 576 / 1088
  static constexpr int PPR    = SEG / 16 + 1;          // 16-byte pieces per LDS row, odd: 37 / 69 (one spare piece)
  static constexpr int PIECES = kSkRows * PPR;
  static constexpr int INSTRS = (PIECES + kWave - 1) / kWave;  // DMA instructions per slice: 19 / 35
  static constexpr int BYTES  = INSTRS * kWave * 16;
};

typedef __attribute__((address_space(1))) const void *sk_gptr_t;
typedef __attribute__((address_space(3))) void       *sk_lptr_t;

// Several weight matrices that meet the same activation rows (the q/k/v or gate/up projections of a decoder layer)
// share one launch: blockIdx.z picks the member, whose weight pointer, output pointer, row count and first tile
// (for its partial tiles and ticket counters) come from the argument table.
struct SkinnyGroupArgs {
  const uint8_t *w[kGemvGroupMax];
  float         *out[kGemvGroupMax];
  int            n[kGemvGroupMax];
  int            tile0[kGemvGroupMax];
};

template <WeightType WT, int MR>
__global__ __launch_bounds__(kSlThreads) void matmul_skinny_slice_kernel(SkinnyGroupArgs grp,
                                                                        const uint8_t *__restrict__ act, int m,
                                                                        int k, float *__restrict__ partials,
                                                                        unsigned *__restrict__ tickets) {
  typedef SliceGeom<WT> G;
  const int                     n      = grp.n[blockIdx.z];
  float *__restrict__           out    = grp.out[blockIdx.z];
  const uint8_t *__restrict__   weight = grp.w[blockIdx.z];
  if ((int) (blockIdx.x * kSkRows) >= n) {
    return;  // whole workgroup: this member has fewer rows than the widest one
  }
  constexpr int MPAD     = 2 * MR;
  constexpr int WROW_BLK = WT == kQ4_0 ? 18 : 34;
  constexpr int ACT_BYTES = 2 * kSlPairs * ActChunk<MR>::PER_KB;
  constexpr int RED_BYTES = kSlWaves * MR * 64 * 4;
  __shared__ __align__(16) uint8_t lds_w[G::BYTES];
  __shared__ __align__(16) uint8_t lds_act[ACT_BYTES > RED_BYTES ? ACT_BYTES : RED_BYTES];
  __shared__ unsigned              lds_ticket;
  const ActChunk<MR> chunk(lds_act, 2 * kSlPairs);

  const int tid  = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int nl = lane & 31, half = lane >> 5;
  const int nblk    = k / 32;
  const int tile    = blockIdx.x, slice = blockIdx.y, nslices = gridDim.y;
  const int gtile   = grp.tile0[blockIdx.z] + tile;  // among all members: partial tiles and tickets
  const int n0      = tile * kSkRows;
  const int a_slot  = min(nl, MPAD - 1);
  const int pair0   = slice * kSlPairs;
  const int cpairs  = min(kSlPairs, nblk / 2 - pair0);
  const size_t row_bytes  = (size_t) nblk * WROW_BLK;
  const size_t last_piece = (size_t) n * row_bytes - 16;  // clamp for reads past the end of the matrix

  // ---- all weight bytes of the slice: instruction i moves pieces 64 i .. 64 i + 63 of the [32][PPR] image ----
#pragma unroll
  for (int j = 0; j < (G::INSTRS + kSlWaves - 1) / kSlWaves; ++j) {
    const int i = j * kSlWaves + wave;
    if (i < G::INSTRS) {
      const int    q   = i * kWave + lane;
      const int    row = min(q / G::PPR, kSkRows - 1), pc = q % G::PPR;
      const size_t off = (size_t) min(n0 + row, n - 1) * row_bytes + (size_t) pair0 * G::PAIRB + (size_t) pc * 16;
      __builtin_amdgcn_global_load_lds((sk_gptr_t) (weight + min(off, last_piece)),
                                       (sk_lptr_t) (lds_w + (size_t) i * kWave * 16), 16, 0, 0);
    }
  }
  // ---- activations of the slice in MFMA operand order ----
  chunk.template stage<WT, kSlThreads, (kSlPairs * MPAD + kSlThreads - 1) / kSlThreads>(act, m, nblk, pair0, cpairs, tid);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  float acc[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    acc[r] = 0.0f;
  }
  const uint8_t *img = lds_w + (size_t) nl * G::PPR * 16;
#pragma unroll
  for (int j = 0; j < kSlPairs / kSlWaves; ++j) {
    const int pl = j * kSlWaves + wave;
    if (pl < cpairs) {
      PairRegs<WT> pr;
      pr.load_lds(reinterpret_cast<const uint32_t *>(img + (size_t) pl * G::PAIRB), half);
      v4i   bq[2];
      float dw[2];
      pr.unpack(half, bq[0], bq[1], dw[0], dw[1]);
      chunk.block_mac(acc, 2 * pl, half, a_slot, bq[0], dw[0]);
      chunk.block_mac(acc, 2 * pl + 1, half, a_slot, bq[1], dw[1]);
    }
  }

  // ---- sum the waves; thread t owns result elements e = t, t + 256, ... of the [MR][64] tile ----
  __syncthreads();
  float *red = reinterpret_cast<float *>(lds_act);
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    red[(wave * MR + r) * 64 + lane] = acc[r];
  }
  __syncthreads();
  constexpr int EPT = MR * 64 / kSlThreads;  // 1, 2 or 4
  float v[EPT];
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int i = e * kSlThreads + tid;
    v[e]        = 0.0f;
#pragma unroll
    for (int w = 0; w < kSlWaves; ++w) {
      v[e] += red[w * MR * 64 + i];
    }
  }
  if (nslices > 1) {
    // Publish this slice's partial tile, take a ticket; the last workgroup of the tile adds all slices in order.
    // The partials travel as device-scope atomic stores and loads (written through to / read from the level all
    // XCDs share) and the ticket is taken only after the stores are acknowledged; a device-scope fence would do the
    // same job by writing back the whole L2, which costs tens of microseconds per workgroup.
    float *mine = partials + ((size_t) gtile * nslices + slice) * (MR * 64);
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      __hip_atomic_store(&mine[e * kSlThreads + tid], v[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
      lds_ticket = __hip_atomic_fetch_add(&tickets[gtile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (lds_ticket != (unsigned) (nslices - 1)) {
      return;
    }
    __atomic_signal_fence(__ATOMIC_SEQ_CST);  // (compile time: the loads below stay behind the ticket; the barrier above orders them in hardware)
    const float *all = partials + (size_t) gtile * nslices * (MR * 64);
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      v[e] = 0.0f;
    }
    // eight slices are requested together (each load travels to the level all XCDs share and back), then added in
    // slice order
    for (int sl0 = 0; sl0 < nslices; sl0 += 8) {
      float x[8][EPT];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int sl = min(sl0 + u, nslices - 1);
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
          x[u][e] = __hip_atomic_load(&all[(size_t) sl * (MR * 64) + e * kSlThreads + tid], __ATOMIC_RELAXED,
                                      __HIP_MEMORY_SCOPE_AGENT);
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (sl0 + u < nslices) {
#pragma unroll
          for (int e = 0; e < EPT; ++e) {
            v[e] += x[u][e];
          }
        }
      }
    }
    if (tid == 0) {
      __hip_atomic_store(&tickets[gtile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
    }
  }
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int i = e * kSlThreads + tid;
    const int r = i >> 6, l = i & 63;
    const int mrow = 8 * (r >> 2) + 4 * (l >> 5) + (r & 3);
    const int col  = n0 + (l & 31);
    if (mrow < m && col < n) {
      out[(size_t) mrow * n + col] = v[e];
    }
  }
}

constexpr size_t kSkLdsLimit = 160 * 1024;

template <typename K>
hipError_t allow_big_lds(K kernel) {
  return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                             (int) kSkLdsLimit);
}

template <int MR>
size_t slice_partial_bytes(int k, int n) {
  const size_t tiles = ((size_t) n + kSkRows - 1) / kSkRows, nslices = ((size_t) k / 64 + kSlPairs - 1) / kSlPairs;
  return nslices > 1 ? tiles * nslices * MR * 64 * sizeof(float) : 0;
}

template <WeightType WT, int MR>
hipError_t launch_skinny_slices(hipStream_t stream, const SkinnyGroupArgs &grp, int count, const void *act, int m, int k,
                                void *workspace, unsigned *tickets) {
  int n_max = 0;
  for (int i = 0; i < count; ++i) {
    n_max = grp.n[i] > n_max ? grp.n[i] : n_max;
  }
  const unsigned tiles = (unsigned) ((n_max + kSkRows - 1) / kSkRows), nslices = (unsigned) ((k / 64 + kSlPairs - 1) / kSlPairs);
  hipLaunchKernelGGL((matmul_skinny_slice_kernel<WT, MR>), dim3(tiles, nslices, (unsigned) count), dim3(kSlThreads), 0, stream,
                     grp, static_cast<const uint8_t *>(act), m, k, static_cast<float *>(workspace), tickets);
  return hipGetLastError();
}

// true when the K-sliced kernel can take these matrices in one launch
template <WeightType WT>
bool slices_fit(const SkinnyGroupArgs &grp, int count, int k, const void *workspace, const unsigned *tickets, int ticket_slots) {
  const size_t row_bytes = (size_t) (k / 32) * (WT == kQ4_0 ? 18 : 34);
  const bool   split     = k / 64 > kSlPairs;
  int          tiles     = 0;
  for (int i = 0; i < count; ++i) {
    if (reinterpret_cast<uintptr_t>(grp.w[i]) % 16 != 0 || (grp.n[i] + kSkRows - 1) / kSkRows > 65535) {
      return false;
    }
    tiles += (grp.n[i] + kSkRows - 1) / kSkRows;
  }
  return row_bytes % 16 == 0 && (!split || (workspace && tickets && tiles <= ticket_slots));
}

template <WeightType WT, int MR>
hipError_t launch_skinny(hipStream_t stream, float *out, const void *act, const void *weight, int m, int k, int n,
                         void *workspace, unsigned *tickets, int ticket_slots) {
  const int nblk = k / 32;
  SkinnyGroupArgs  one = {};
  one.w[0] = static_cast<const uint8_t *>(weight), one.out[0] = out, one.n[0] = n, one.tile0[0] = 0;
  if (slices_fit<WT>(one, 1, k, workspace, tickets, ticket_slots)) {
    return launch_skinny_slices<WT, MR>(stream, one, 1, act, m, k, workspace, tickets);
  }
  constexpr int per_kb = ActChunk<MR>::PER_KB;
  const size_t  budget = 96 * 1024;
  const int nchunks = (int) (((size_t) nblk * per_kb + budget - 1) / budget);
  int       kc      = (nblk + nchunks - 1) / nchunks;
  kc                = (kc + 1) & ~1;
  size_t lds        = (size_t) kc * per_kb;
  const size_t red  = (size_t) kSkWaves * MR * 64 * sizeof(float);
  lds               = lds > red ? lds : red;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipError_t e = allow_big_lds(&matmul_skinny_kernel<WT, MR, kSkPrefetch>); e != hipSuccess) {
      return e;
    }
    attr_set = true;
  }
  const unsigned grid = (unsigned) ((n + kSkRows - 1) / kSkRows);
  hipLaunchKernelGGL((matmul_skinny_kernel<WT, MR, kSkPrefetch>), dim3(grid), dim3(kSkThreads), lds, stream, out,
                     static_cast<const uint8_t *>(act), static_cast<const uint8_t *>(weight), m, k, n, kc);
  return hipGetLastError();
}

template <WeightType WT>
hipError_t launch_skinny_m(hipStream_t stream, float *out, const void *act, const void *weight, int m, int k, int n,
                           void *workspace, unsigned *tickets, int ticket_slots) {
  if (m <= 8) {
    return launch_skinny<WT, 4>(stream, out, act, weight, m, k, n, workspace, tickets, ticket_slots);
  }
  if (m <= 16) {
    return launch_skinny<WT, 8>(stream, out, act, weight, m, k, n, workspace, tickets, ticket_slots);
  }
  return launch_skinny<WT, 16>(stream, out, act, weight, m, k, n, workspace, tickets, ticket_slots);
}

}  // namespace

size_t matmul_skinny_workspace_bytes(int m, int k, int n) {
  if (m < 1 || k % 64 != 0) {
    return 0;
  }
  const int rows = m < 32 ? m : 32;
  return rows <= 8 ? slice_partial_bytes<4>(k, n) : rows <= 16 ? slice_partial_bytes<8>(k, n) : slice_partial_bytes<16>(k, n);
}

size_t matmul_skinny_group_workspace_bytes(int count, const int *ns, int m, int k) {
  size_t total = 0;
  for (int i = 0; i < count; ++i) {
    total += matmul_skinny_workspace_bytes(m, k, ns[i]);
  }
  return total;
}

hipError_t launch_matmul_skinny_group(hipStream_t stream, int count, float *const *outs, const void *act,
                                      const void *const *weights, const int *ns, int m, int k, WeightType wt,
                                      void *workspace, unsigned *tickets, int ticket_slots) {
  if (count < 1 || count > kGemvGroupMax || k % 64 != 0 || m < 2 || m > 8) {
    return hipErrorNotSupported;
  }
  SkinnyGroupArgs grp = {};
  int             tile0 = 0;
  for (int i = 0; i < count; ++i) {
    grp.w[i] = static_cast<const uint8_t *>(weights[i]), grp.out[i] = outs[i], grp.n[i] = ns[i], grp.tile0[i] = tile0;
    tile0 += (ns[i] + kSkRows - 1) / kSkRows;
  }
  if (wt == kQ4_0) {
    return slices_fit<kQ4_0>(grp, count, k, workspace, tickets, ticket_slots) ?
             launch_skinny_slices<kQ4_0, 4>(stream, grp, count, act, m, k, workspace, tickets) : hipErrorNotSupported;
  }
  return slices_fit<kQ8_0>(grp, count, k, workspace, tickets, ticket_slots) ?
           launch_skinny_slices<kQ8_0, 4>(stream, grp, count, act, m, k, workspace, tickets) : hipErrorNotSupported;
}

hipError_t launch_matmul_skinny(hipStream_t stream, float *out, const void *act, const void *weight, int m, int k,
                                int n, WeightType wt, void *workspace, unsigned *tickets, int ticket_slots) {
  if (k % 64 != 0 || m < 1 || m > 32) {
    return hipErrorNotSupported;
  }
  return wt == kQ4_0 ? launch_skinny_m<kQ4_0>(stream, out, act, weight, m, k, n, workspace, tickets, ticket_slots) :
                       launch_skinny_m<kQ8_0>(stream, out, act, weight, m, k, n, workspace, tickets, ticket_slots);
}

}  // namespace htpops
