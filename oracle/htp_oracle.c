/*
 * htp_oracle.c -- scalar CPU restatement of the op backend's arithmetic.
 * TEST INFRASTRUCTURE ONLY; see htp_oracle.h for what each function restates and how it is pinned.
 * Build: gcc -O3 -ffp-contract=off -fPIC -shared -pthread (see Makefile).
 */
#include "htp_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define QK 32

/* packed block layouts, include/dsp/quants.h:11-14 and :23-26 */
typedef struct {
  uint16_t d;
  uint8_t  qs[QK / 2];
} __attribute__((packed)) blk_q4_0;

typedef struct {
  uint16_t d;
  int8_t   qs[QK];
} __attribute__((packed)) blk_q8_0;

/* src/dsp/ops/mat_mul.c:29-32 */
static const int8_t kIq4nl[16] = { -127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113 };

/* ------------------------------------------------------------------ fp16 */

float oracle_fp16_to_fp32(uint16_t h) {
  uint32_t sign = (uint32_t) (h & 0x8000u) << 16;
  uint32_t exp  = (h >> 10) & 0x1fu;
  uint32_t man  = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      /* subnormal: value = man * 2^-24, exactly representable in fp32 */
      float    v = (float) man * 5.9604644775390625e-8f;
      uint32_t vb;
      memcpy(&vb, &v, 4);
      bits = sign | vb;
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

uint16_t oracle_fp32_to_fp16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint16_t sign = (uint16_t) ((x >> 16) & 0x8000u);
  uint32_t ax   = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    return (uint16_t) (sign | 0x7c00u | ((ax > 0x7f800000u) ? (0x200u | ((ax >> 13) & 0x3ffu)) : 0u));
  }
  if (ax >= 0x477ff000u) { /* >= 65520 rounds to inf */
    return (uint16_t) (sign | 0x7c00u);
  }
  if (ax < 0x33000001u) { /* <= 2^-25 rounds to zero (ties-to-even at exactly 2^-25) */
    return sign;
  }
  int32_t  e   = (int32_t) (ax >> 23) - 127;
  uint32_t man = (ax & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  uint32_t shift;
  uint32_t half_exp;
  if (e < -14) { /* subnormal result: unit is 2^-24 */
    shift    = (uint32_t) (13 + (-14 - e));
    half_exp = 0;
  } else {
    shift    = 13;
    half_exp = (uint32_t) (e + 15);
  }
  uint32_t q    = man >> shift;
  uint32_t rem  = man & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) {
    q += 1;
  }
  uint32_t out;
  if (half_exp == 0) {
    out = q; /* may carry into the smallest normal, which is the right encoding */
  } else {
    out = ((half_exp - 1) << 10) + q; /* q holds the implicit bit; a carry bumps the exponent */
  }
  return (uint16_t) (sign | out);
}

/* ------------------------------------------------------------ dequantize */

void oracle_dequantize_q4_0(const void *blocks, int n_blocks, float *out) {
  const blk_q4_0 *b = (const blk_q4_0 *) blocks;
  for (int i = 0; i < n_blocks; ++i) {
    float d = oracle_fp16_to_fp32(b[i].d);
    for (int j = 0; j < QK / 2; ++j) {
      out[i * QK + j]          = (float) ((int) (b[i].qs[j] & 0x0f) - 8) * d;
      out[i * QK + j + QK / 2] = (float) ((int) (b[i].qs[j] >> 4) - 8) * d;
    }
  }
}

void oracle_dequantize_iq4_nl(const void *blocks, int n_blocks, float *out) {
  const blk_q4_0 *b = (const blk_q4_0 *) blocks;
  for (int i = 0; i < n_blocks; ++i) {
    float d = oracle_fp16_to_fp32(b[i].d);
    for (int j = 0; j < QK / 2; ++j) {
      out[i * QK + j]          = (float) kIq4nl[b[i].qs[j] & 0x0f] * d;
      out[i * QK + j + QK / 2] = (float) kIq4nl[b[i].qs[j] >> 4] * d;
    }
  }
}

void oracle_dequantize_q8_0(const void *blocks, int n_blocks, float *out) {
  const blk_q8_0 *b = (const blk_q8_0 *) blocks;
  for (int i = 0; i < n_blocks; ++i) {
    float d = oracle_fp16_to_fp32(b[i].d);
    for (int j = 0; j < QK; ++j) {
      out[i * QK + j] = (float) b[i].qs[j] * d;
    }
  }
}

/* -------------------------------------------------------------- quantize */

void oracle_quantize_row_q8_0(const float *x, void *y, int k) {
  blk_q8_0 *b  = (blk_q8_0 *) y;
  const int nb = k / QK;
  for (int i = 0; i < nb; ++i) {
    float amax = 0.0f;
    for (int j = 0; j < QK; ++j) {
      float v = fabsf(x[i * QK + j]);
      if (v > amax) {
        amax = v;
      }
    }
    const float d  = amax / 127.0f;
    const float id = d ? 1.0f / d : 0.0f;
    b[i].d         = oracle_fp32_to_fp16(d);
    for (int j = 0; j < QK; ++j) {
      b[i].qs[j] = (int8_t) roundf(x[i * QK + j] * id);
    }
  }
}

void oracle_quantize_q8_0(const float *x, void *y, int k, int m) {
  for (int r = 0; r < m; ++r) {
    oracle_quantize_row_q8_0(x + (size_t) r * k, (uint8_t *) y + (size_t) r * (k / QK) * sizeof(blk_q8_0), k);
  }
}

/* ------------------------------------------------------------------ dots */

int32_t oracle_block_dot_q4_0_q8_0(const void *w_block, const void *a_block) {
  const blk_q4_0 *w    = (const blk_q4_0 *) w_block;
  const blk_q8_0 *a    = (const blk_q8_0 *) a_block;
  int32_t         sumi = 0;
  for (int j = 0; j < QK / 2; ++j) {
    const int v0 = (w->qs[j] & 0x0f) - 8;
    const int v1 = (w->qs[j] >> 4) - 8;
    sumi += v0 * a->qs[j] + v1 * a->qs[j + QK / 2];
  }
  return sumi;
}

int32_t oracle_block_dot_q8_0_q8_0(const void *w_block, const void *a_block) {
  const blk_q8_0 *w    = (const blk_q8_0 *) w_block;
  const blk_q8_0 *a    = (const blk_q8_0 *) a_block;
  int32_t         sumi = 0;
  for (int j = 0; j < QK; ++j) {
    sumi += (int) w->qs[j] * (int) a->qs[j];
  }
  return sumi;
}

float oracle_vec_dot_q4_0_q8_0(int k, const void *w_row, const void *a_row) {
  const blk_q4_0 *w   = (const blk_q4_0 *) w_row;
  const blk_q8_0 *a   = (const blk_q8_0 *) a_row;
  float           acc = 0.0f;
  for (int i = 0; i < k / QK; ++i) {
    const int32_t sumi = oracle_block_dot_q4_0_q8_0(&w[i], &a[i]);
    acc += ((float) sumi * oracle_fp16_to_fp32(w[i].d)) * oracle_fp16_to_fp32(a[i].d);
  }
  return acc;
}

float oracle_vec_dot_q8_0_q8_0(int k, const void *w_row, const void *a_row) {
  const blk_q8_0 *w   = (const blk_q8_0 *) w_row;
  const blk_q8_0 *a   = (const blk_q8_0 *) a_row;
  float           acc = 0.0f;
  for (int i = 0; i < k / QK; ++i) {
    const int32_t sumi = oracle_block_dot_q8_0_q8_0(&w[i], &a[i]);
    acc += ((float) sumi * oracle_fp16_to_fp32(w[i].d)) * oracle_fp16_to_fp32(a[i].d);
  }
  return acc;
}

double oracle_vec_dot_q4_0_q8_0_f64(int k, const void *w_row, const void *a_row, double *abs_sum) {
  const blk_q4_0 *w = (const blk_q4_0 *) w_row;
  const blk_q8_0 *a = (const blk_q8_0 *) a_row;
  double          acc = 0.0, mag = 0.0;
  for (int i = 0; i < k / QK; ++i) {
    const double t = (double) oracle_block_dot_q4_0_q8_0(&w[i], &a[i]) * (double) oracle_fp16_to_fp32(w[i].d) *
                     (double) oracle_fp16_to_fp32(a[i].d);
    acc += t;
    mag += fabs(t);
  }
  if (abs_sum) {
    *abs_sum = mag;
  }
  return acc;
}

double oracle_vec_dot_q8_0_q8_0_f64(int k, const void *w_row, const void *a_row, double *abs_sum) {
  const blk_q8_0 *w = (const blk_q8_0 *) w_row;
  const blk_q8_0 *a = (const blk_q8_0 *) a_row;
  double          acc = 0.0, mag = 0.0;
  for (int i = 0; i < k / QK; ++i) {
    const double t = (double) oracle_block_dot_q8_0_q8_0(&w[i], &a[i]) * (double) oracle_fp16_to_fp32(w[i].d) *
                     (double) oracle_fp16_to_fp32(a[i].d);
    acc += t;
    mag += fabs(t);
  }
  if (abs_sum) {
    *abs_sum = mag;
  }
  return acc;
}

/* ---------------------------------------------------------------- matmul */

typedef struct {
  float       *out;
  const void  *act;
  const void  *w;
  int          m, k, n, weight_type;
  int          n_begin, n_end;
} mm_job;

static void mm_range(const mm_job *j) {
  const size_t a_row_bytes = (size_t) (j->k / QK) * sizeof(blk_q8_0);
  const size_t w_row_bytes = (size_t) (j->k / QK) * (j->weight_type == 2 ? sizeof(blk_q4_0) : sizeof(blk_q8_0));
  for (int r = 0; r < j->m; ++r) {
    const uint8_t *a_row = (const uint8_t *) j->act + (size_t) r * a_row_bytes;
    for (int c = j->n_begin; c < j->n_end; ++c) {
      const uint8_t *w_row = (const uint8_t *) j->w + (size_t) c * w_row_bytes;
      j->out[(size_t) r * j->n + c] = j->weight_type == 2 ? oracle_vec_dot_q4_0_q8_0(j->k, w_row, a_row) :
                                                            oracle_vec_dot_q8_0_q8_0(j->k, w_row, a_row);
    }
  }
}

static void *mm_thread(void *p) {
  mm_range((const mm_job *) p);
  return NULL;
}

int oracle_mat_mul_q8_0_act(float *out, const void *act, const void *w, int m, int k, int n, int weight_type,
                            int n_threads) {
  if (!out || !act || !w || m <= 0 || k <= 0 || n <= 0 || k % QK != 0) {
    return -1;
  }
  if (weight_type != 2 && weight_type != 8) {
    return -1;
  }
  if (n_threads < 1) {
    n_threads = 1;
  }
  if (n_threads > 256) {
    n_threads = 256;
  }
  if (n_threads > n) {
    n_threads = n;
  }
  mm_job    jobs[256];
  pthread_t tids[256];
  for (int t = 0; t < n_threads; ++t) {
    jobs[t].out         = out;
    jobs[t].act         = act;
    jobs[t].w           = w;
    jobs[t].m           = m;
    jobs[t].k           = k;
    jobs[t].n           = n;
    jobs[t].weight_type = weight_type;
    jobs[t].n_begin     = (int) ((long long) n * t / n_threads);
    jobs[t].n_end       = (int) ((long long) n * (t + 1) / n_threads);
  }
  if (n_threads == 1) {
    mm_range(&jobs[0]);
    return 0;
  }
  for (int t = 0; t < n_threads; ++t) {
    if (pthread_create(&tids[t], NULL, mm_thread, &jobs[t]) != 0) {
      /* run what could not be spawned inline */
      mm_range(&jobs[t]);
      tids[t] = 0;
    }
  }
  for (int t = 0; t < n_threads; ++t) {
    if (tids[t]) {
      pthread_join(tids[t], NULL);
    }
  }
  return 0;
}

int oracle_mat_mul_f32_act(float *out, const float *act, const void *w, int m, int k, int n, int weight_type,
                           int n_threads) {
  if (!act || m <= 0 || k <= 0 || k % QK != 0) {
    return -1;
  }
  void *q = malloc((size_t) m * (k / QK) * sizeof(blk_q8_0));
  if (!q) {
    return -1;
  }
  oracle_quantize_q8_0(act, q, k, m);
  int ret = oracle_mat_mul_q8_0_act(out, q, w, m, k, n, weight_type, n_threads);
  free(q);
  return ret;
}

int oracle_mat_mul_q8_0_act_abs(double *out_f64, double *out_abs, const void *act, const void *w, int m, int k,
                                int n, int weight_type) {
  if (!act || !w || m <= 0 || k <= 0 || n <= 0 || k % QK != 0 || (weight_type != 2 && weight_type != 8)) {
    return -1;
  }
  const size_t a_row_bytes = (size_t) (k / QK) * sizeof(blk_q8_0);
  const size_t w_row_bytes = (size_t) (k / QK) * (weight_type == 2 ? sizeof(blk_q4_0) : sizeof(blk_q8_0));
  for (int r = 0; r < m; ++r) {
    const uint8_t *a_row = (const uint8_t *) act + (size_t) r * a_row_bytes;
    for (int c = 0; c < n; ++c) {
      const uint8_t *w_row = (const uint8_t *) w + (size_t) c * w_row_bytes;
      double         mag   = 0.0;
      double         v     = weight_type == 2 ? oracle_vec_dot_q4_0_q8_0_f64(k, w_row, a_row, &mag) :
                                                oracle_vec_dot_q8_0_q8_0_f64(k, w_row, a_row, &mag);
      if (out_f64) {
        out_f64[(size_t) r * n + c] = v;
      }
      if (out_abs) {
        out_abs[(size_t) r * n + c] = mag;
      }
    }
  }
  return 0;
}

/* --------------------------------------------------------------- rmsnorm */

int oracle_rms_norm_f32_ex(float *dst, const float *src, const float *w, float eps, int ne0, int ne1) {
  if (!dst || !src || ne0 <= 0 || ne1 <= 0) {
    return -1;
  }
  for (int j = 0; j < ne1; ++j) {
    const float *x   = src + (size_t) j * ne0;
    float       *y   = dst + (size_t) j * ne0;
    float        sum = 0.0f;
    for (int i = 0; i < ne0; ++i) {
      sum += x[i] * x[i];
    }
    const float mean  = sum / ne0;
    const float scale = 1.0f / sqrtf(mean + eps);
    if (w) {
      for (int i = 0; i < ne0; ++i) {
        y[i] = (x[i] * scale) * w[i];
      }
    } else {
      for (int i = 0; i < ne0; ++i) {
        y[i] = x[i] * scale;
      }
    }
  }
  return 0;
}

int oracle_rms_norm_f32(float *dst, const float *src, int ne0, int ne1) {
  return oracle_rms_norm_f32_ex(dst, src, NULL, 1e-5f, ne0, ne1);
}

/* ------------------------------------------------------------- attention */

#define FA_BR 32
#define FA_BC 256

static int flash_attn_impl(float *O32, uint16_t *O16, const float *Q32, const uint16_t *Q16, const uint16_t *K,
                           const uint16_t *V, const uint16_t *mask, int qo_len, int kv_len, int n_heads,
                           int n_kv_heads, int head_dim, int causal) {
  if (n_kv_heads <= 0 || n_heads % n_kv_heads != 0 || head_dim <= 0 || head_dim > 256) {
    return -1;
  }
  const int    group     = n_heads / n_kv_heads;
  const size_t mask_ld   = ((size_t) kv_len + 63) / 64 * 64;
  const size_t qo_stride = (size_t) n_heads * head_dim;
  const size_t kv_stride = (size_t) n_kv_heads * head_dim;
  const float  qk_scale  = 1.0f / sqrtf((float) head_dim) * 1.44269504f;
  const int    D         = head_dim;

  float *Qi = (float *) malloc(sizeof(float) * FA_BR * D);
  float *Oi = (float *) malloc(sizeof(float) * FA_BR * D);
  float *Kj = (float *) malloc(sizeof(float) * FA_BC * D);
  float *Vj = (float *) malloc(sizeof(float) * FA_BC * D);
  float *S  = (float *) malloc(sizeof(float) * FA_BR * FA_BC);
  float *P  = (float *) malloc(sizeof(float) * FA_BC);
  if (!Qi || !Oi || !Kj || !Vj || !S || !P) {
    free(Qi), free(Oi), free(Kj), free(Vj), free(S), free(P);
    return -1;
  }
  float m_run[FA_BR], l_run[FA_BR];

  for (int h = 0; h < n_heads; ++h) {
    const int h_kv = h / group;
    for (int q0 = 0; q0 < qo_len; q0 += FA_BR) {
      const int br = (q0 + FA_BR < qo_len) ? FA_BR : qo_len - q0;
      for (int r = 0; r < br; ++r) {
        const size_t base = (size_t) (q0 + r) * qo_stride + (size_t) h * D;
        for (int d = 0; d < D; ++d) {
          Qi[r * D + d] = Q32 ? Q32[base + d] : oracle_fp16_to_fp32(Q16[base + d]);
          Oi[r * D + d] = 0.0f;
        }
        m_run[r] = -INFINITY;
        l_run[r] = 0.0f;
      }
      for (int k0 = 0; k0 < kv_len; k0 += FA_BC) {
        const int bc = (k0 + FA_BC < kv_len) ? FA_BC : kv_len - k0;
        for (int c = 0; c < bc; ++c) {
          const size_t base = (size_t) (k0 + c) * kv_stride + (size_t) h_kv * D;
          for (int d = 0; d < D; ++d) {
            Kj[c * D + d] = oracle_fp16_to_fp32(K[base + d]);
            Vj[c * D + d] = oracle_fp16_to_fp32(V[base + d]);
          }
        }
        for (int r = 0; r < br; ++r) {
          for (int c = 0; c < bc; ++c) {
            float sum = 0.0f;
            for (int d = 0; d < D; ++d) {
              sum += Qi[r * D + d] * Kj[c * D + d];
            }
            float s = sum * qk_scale;
            if (mask) {
              s += oracle_fp16_to_fp32(mask[(size_t) (q0 + r) * mask_ld + (size_t) (k0 + c)]);
            }
            if (causal && (k0 + c) > (q0 + r) + (kv_len - qo_len)) {
              s = -INFINITY;
            }
            S[r * FA_BC + c] = s;
          }
        }
        for (int r = 0; r < br; ++r) {
          float m_blk = -INFINITY;
          for (int c = 0; c < bc; ++c) {
            if (S[r * FA_BC + c] > m_blk) {
              m_blk = S[r * FA_BC + c];
            }
          }
          const float m_new = fmaxf(m_run[r], m_blk);
          float       p_sum = 0.0f;
          for (int c = 0; c < bc; ++c) {
            P[c] = exp2f(S[r * FA_BC + c] - m_new);
            p_sum += P[c];
          }
          const float f     = exp2f(m_run[r] - m_new);
          const float l_new = l_run[r] * f + p_sum;
          for (int d = 0; d < D; ++d) {
            Oi[r * D + d] *= f;
            float acc = 0.0f;
            for (int c = 0; c < bc; ++c) {
              acc += P[c] * Vj[c * D + d];
            }
            Oi[r * D + d] += acc;
          }
          m_run[r] = m_new;
          l_run[r] = l_new;
        }
      }
      for (int r = 0; r < br; ++r) {
        const float  inv  = 1.0f / l_run[r];
        const size_t base = (size_t) (q0 + r) * qo_stride + (size_t) h * D;
        for (int d = 0; d < D; ++d) {
          const float o = Oi[r * D + d] * inv;
          if (O32) {
            O32[base + d] = o;
          } else {
            O16[base + d] = oracle_fp32_to_fp16(o);
          }
        }
      }
    }
  }
  free(Qi), free(Oi), free(Kj), free(Vj), free(S), free(P);
  return 0;
}

int oracle_flash_attn(float *O, const float *Q, const uint16_t *K, const uint16_t *V, const uint16_t *mask,
                      int qo_len, int kv_len, int n_heads, int n_kv_heads, int head_dim, int causal) {
  if (!O || !Q || !K || !V) {
    return -1;
  }
  return flash_attn_impl(O, NULL, Q, NULL, K, V, mask, qo_len, kv_len, n_heads, n_kv_heads, head_dim, causal);
}

int oracle_flash_attn_f16(uint16_t *O, const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                          const uint16_t *mask, int qo_len, int kv_len, int n_heads, int n_kv_heads, int head_dim,
                          int causal) {
  if (!O || !Q || !K || !V) {
    return -1;
  }
  return flash_attn_impl(NULL, O, NULL, Q, K, V, mask, qo_len, kv_len, n_heads, n_kv_heads, head_dim, causal);
}

/* -------------------------------------------------------- fp16 tile matmul */

size_t oracle_w16_tile_index(int kk, int nn, int k) {
  const int k0 = kk / 32, k1 = kk % 32;
  const int n0 = nn / 32, n1 = nn % 32;
  const size_t tile = (size_t) n0 * (size_t) (k / 32) + (size_t) k0;
  return tile * 1024 + (size_t) ((k1 & ~1) * 32 + n1 * 2 + (k1 & 1));
}

int oracle_mat_mul_w16a32(float *out, const float *act, const uint16_t *w_tiles, int m, int k, int n) {
  if (!out || !act || !w_tiles || m <= 0 || k <= 0 || n <= 0 || k % 32 != 0 || n % 32 != 0) {
    return -1;
  }
  for (int i = 0; i < m; ++i) {
    for (int j = 0; j < n; ++j) {
      float acc = 0.0f;
      for (int l = 0; l < k; ++l) {
        acc += act[(size_t) i * k + l] * oracle_fp16_to_fp32(w_tiles[oracle_w16_tile_index(l, j, k)]);
      }
      out[(size_t) i * n + j] = acc;
    }
  }
  return 0;
}

/* ----------------------------------------------- tile-permuted super-blocks
 * my_block_q4_0 (144 B = 8 fp16 scales + 128 quant bytes) and my_block_q8_0 (272 B = 8 scales + 256 int8)
 * hold 256 weights of one 32x32 HMX tile: 8 K rows x 32 N columns. The dequantizer writes four 64-element
 * vectors per super-block (reference: src/dsp/ops/mat_mul.c:383-405 and :483-505); vector v is tile row pair
 * 4 * (super-block % 4) + v, element e of a vector is column e / 2, K parity e % 2 (the fp16 tile order of
 * src/host/test.c:307-312), and elements 0..31 / 32..63 of vector v use scales 2v / 2v + 1 (the scale index
 * table at :319-325: a scale covers 2 K rows x 16 columns).
 *   Q4_0 / IQ4_NL: vectors 0, 1 come from the low nibbles of the even / odd quant bytes, vectors 2, 3 from
 *   the high nibbles of the even / odd bytes (vlut16 sends even bytes to the low and odd bytes to the high
 *   vector of its result pair, :383-384 with :402-405) -- this even/odd assignment is read off the HVX
 *   instruction's documented behaviour and has no test in the reference: PARITY UNPINNED for it.
 *   Q8_0: vunpack keeps byte order, vector v = quants[64 v .. 64 v + 63] (:483-489).
 * Every value is fp16(q) * fp16(scale), rounded once to fp16 (qf16 multiply then convert, :402-405). */

static uint16_t dequant_fp16_product(int q, uint16_t scale_bits) {
  /* |q| <= 127 times an 11-bit significand is exact in fp32; one rounding to fp16 */
  return oracle_fp32_to_fp16((float) q * oracle_fp16_to_fp32(scale_bits));
}

void oracle_dequantize_permuted_q4_0(const void *super_blocks, int n_super_blocks, int iq4_nl, uint16_t *out) {
  const uint8_t *src = (const uint8_t *) super_blocks;
  for (int i = 0; i < n_super_blocks; ++i, src += 144, out += 256) {
    uint16_t scales[8];
    memcpy(scales, src, 16);
    const uint8_t *qs = src + 16;
    for (int v = 0; v < 4; ++v) {
      for (int e = 0; e < 64; ++e) {
        const uint8_t byte = qs[2 * e + (v & 1)];
        const int     nib  = (v & 2) ? (byte >> 4) : (byte & 0x0f);
        const int     q    = iq4_nl ? kIq4nl[nib] : nib - 8;
        out[v * 64 + e]    = dequant_fp16_product(q, scales[2 * v + (e >> 5)]);
      }
    }
  }
}

void oracle_dequantize_permuted_q8_0(const void *super_blocks, int n_super_blocks, uint16_t *out) {
  const uint8_t *src = (const uint8_t *) super_blocks;
  for (int i = 0; i < n_super_blocks; ++i, src += 272, out += 256) {
    uint16_t scales[8];
    memcpy(scales, src, 16);
    const int8_t *qs = (const int8_t *) (src + 16);
    for (int v = 0; v < 4; ++v) {
      for (int e = 0; e < 64; ++e) {
        out[v * 64 + e] = dequant_fp16_product(qs[v * 64 + e], scales[2 * v + (e >> 5)]);
      }
    }
  }
}

/* The reference's matmul ops 1-4 (src/dsp/ops/mat_mul.c:758-855, :875-1153): activations fp32 -> fp16, weights
 * fp16 tiles (op 1) or tiles dequantized as above (ops 2-4), products accumulated by the matrix unit, result
 * rounded to fp16 and widened to fp32 (:909, hmx_consume_accumulator_fp16). The accumulation precision of the
 * HMX is not documented; here products of the fp16 operands are summed in double (exact to well below one
 * fp16 ulp) and rounded once. weight_kind: 1 fp16 tiles, 2 Q4_0, 3 Q8_0, 4 IQ4_NL super-blocks (the op ids).
 * out_f64, if not NULL, receives the unrounded sums. */
int oracle_mat_mul_permuted(float *out, double *out_f64, const float *act, const void *weight, int m, int k, int n,
                            int weight_kind) {
  if (!out || !act || !weight || m <= 0 || k <= 0 || n <= 0 || k % 32 != 0 || n % 32 != 0 || weight_kind < 1 ||
      weight_kind > 4) {
    return -1;
  }
  const size_t    n_tiles = (size_t) (k / 32) * (size_t) (n / 32);
  uint16_t       *tiles   = NULL;
  const uint16_t *w16     = (const uint16_t *) weight;
  if (weight_kind != 1) {
    tiles = (uint16_t *) malloc(n_tiles * 1024 * sizeof(uint16_t));
    if (!tiles) {
      return -1;
    }
    if (weight_kind == 3) {
      oracle_dequantize_permuted_q8_0(weight, (int) (n_tiles * 4), tiles);
    } else {
      oracle_dequantize_permuted_q4_0(weight, (int) (n_tiles * 4), weight_kind == 4, tiles);
    }
    w16 = tiles;
  }
  float *a16 = (float *) malloc((size_t) k * sizeof(float));
  float *col = (float *) malloc((size_t) k * sizeof(float));
  if (!a16 || !col) {
    free(tiles), free(a16), free(col);
    return -1;
  }
  for (int j = 0; j < n; ++j) {
    for (int l = 0; l < k; ++l) {
      col[l] = oracle_fp16_to_fp32(w16[oracle_w16_tile_index(l, j, k)]);
    }
    for (int i = 0; i < m; ++i) {
      double acc = 0.0;
      for (int l = 0; l < k; ++l) {
        const float a = oracle_fp16_to_fp32(oracle_fp32_to_fp16(act[(size_t) i * k + l]));
        acc += (double) a * (double) col[l];
      }
      if (out_f64) {
        out_f64[(size_t) i * n + j] = acc;
      }
      out[(size_t) i * n + j] = oracle_fp16_to_fp32(oracle_fp32_to_fp16((float) acc));
    }
  }
  free(tiles), free(a16), free(col);
  return 0;
}
