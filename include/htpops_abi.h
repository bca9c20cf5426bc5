/*
 * htpops_abi.h -- wire formats shared by callers and the MI355X op backend.
 *
 * Everything in this header is a byte-for-byte layout contract:
 *   - op ids and packed parameter structs   (reference: include/op_reg.h:5-47)
 *   - mailbox message / request framing      (reference: include/message.h:6-58)
 *   - quantized weight / activation blocks   (reference: include/dsp/quants.h:5-31)
 *
 * A host that already includes the reference's own op_reg.h / message.h can
 * define HTPOPS_USE_REFERENCE_HEADERS before including this file; the structs
 * are then taken from those headers and only checked here.
 *
 * Ops 0..5 keep the reference numbering. Ops >= HTP_OPS_EXT_BASE are additions
 * of this backend (ggml-style Q8_0 activation arithmetic, fp16 attention with
 * a causal flag, RMSNorm with weight and eps); they are appended, never
 * renumbered, so a reference host never emits them by accident.
 */
#ifndef HTPOPS_ABI_H
#define HTPOPS_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
#  define HTPOPS_STATIC_ASSERT(c, m) static_assert(c, m)
#else
#  define HTPOPS_STATIC_ASSERT(c, m) _Static_assert(c, m)
#endif

#define HTPOPS_PACKED __attribute__((packed))

#ifdef HTPOPS_USE_REFERENCE_HEADERS
#  include "message.h"
#  include "op_reg.h"
#else

/* ---- op ids (reference: include/op_reg.h:5-13) ------------------------- */
enum HtpOpsIndex {
  HTP_OPS_RMS_NORM_F32                     = 0, /* fp32 rows, eps 1e-5, no weight              */
  HTP_OPS_MAT_MUL_PERMUTED_W16A32          = 1, /* fp16 weights in 32x32 tile order            */
  HTP_OPS_MAT_MUL_PERMUTED_W4D16A32        = 2, /* Q4_0 super-blocks (144 B / 256 weights)     */
  HTP_OPS_MAT_MUL_PERMUTED_W8D16A32        = 3, /* Q8_0 super-blocks (272 B / 256 weights)     */
  HTP_OPS_MAT_MUL_PERMUTED_W4D16A32_IQ4_NL = 4, /* IQ4_NL code book, same super-block          */
  HTP_OPS_FLASH_ATTN_QO_F32_KV_F16         = 5, /* fp32 Q/O, fp16 K/V, optional additive mask  */
  HTP_OPS_COUNT                            = 6,
};

/* A buffer is named by (handle, byte offset). The reference passes an rpcmem
 * file descriptor in `fd`; this backend passes a handle issued by
 * htpops_buffer_alloc / htpops_buffer_register (reference: op_reg.h:15-18). */
struct RpcmemBufAddr {
  int32_t fd;
  int32_t offset;
} HTPOPS_PACKED;

/* reference: op_reg.h:20-25 */
struct RmsNormF32Params {
  struct RpcmemBufAddr dst;
  struct RpcmemBufAddr src;
  int32_t              ne0; /* row length   */
  int32_t              ne1; /* number of rows */
} HTPOPS_PACKED;

/* reference: op_reg.h:27-34 */
struct MatMulParams {
  struct RpcmemBufAddr output;     /* fp32 [m][n]          */
  struct RpcmemBufAddr activation; /* [m][k]               */
  struct RpcmemBufAddr weight;     /* [n][k] in some format */
  int32_t              m;
  int32_t              k;
  int32_t              n;
} HTPOPS_PACKED;

/* reference: op_reg.h:36-47 */
struct FlashAttnParams {
  struct RpcmemBufAddr o;
  struct RpcmemBufAddr q;
  struct RpcmemBufAddr k;
  struct RpcmemBufAddr v;
  struct RpcmemBufAddr mask; /* fd < 0 means "no mask" */
  int32_t              qo_len;
  int32_t              kv_len;
  int32_t              n_heads;
  int32_t              n_kv_heads;
  int32_t              head_dim;
} HTPOPS_PACKED;

/* ---- mailbox framing (reference: include/message.h:6-42) --------------- */
struct MessageState {
  union {
    volatile uint8_t  v[8]; /* v[0]: producer "go", v[1]: consumer "done" */
    volatile uint64_t d;
  };
} HTPOPS_PACKED;

struct MessageHeader {
  struct MessageState state;
  uint32_t            checksum;
  int32_t             n_reqs;
  int32_t             req_offsets[0]; /* n_reqs + 1 byte offsets from the header start */
} HTPOPS_PACKED;

struct RequestHeader {
  int32_t state; /* written by the consumer: the op's return code */
  int32_t type;  /* enum RequestType */
  uint8_t data[0];
} HTPOPS_PACKED;

enum RequestType {
  REQUEST_TYPE_NO_OP      = 0,
  REQUEST_TYPE_RPCMEM_MAP = 1,
  REQUEST_TYPE_OP_COMPUTE = 2,
  REQUEST_TYPE_COUNT      = 3,
};

struct RpcmemMapRequest {
  int32_t n_puts; /* handles to release */
  int32_t n_gets; /* ignored, as in the reference */
  int32_t fds[0];
} HTPOPS_PACKED;

struct OpComputeRequest {
  uint32_t op; /* enum HtpOpsIndex or enum HtpOpsExtIndex */
  uint8_t  payload[0];
} HTPOPS_PACKED;

/* accessors with the reference's names (message.h:44-58) */
static inline size_t message_header_size(const struct MessageHeader *h) {
  return sizeof(struct MessageHeader) + ((size_t) h->n_reqs + 1) * sizeof(int32_t);
}
static inline size_t message_total_size(const struct MessageHeader *h) {
  return (size_t) h->req_offsets[h->n_reqs];
}
static inline size_t message_header_get_request_size(const struct MessageHeader *h, int i) {
  return (size_t) (h->req_offsets[i + 1] - h->req_offsets[i]);
}
static inline struct RequestHeader *message_header_get_request_ptr(struct MessageHeader *h, int i) {
  return (struct RequestHeader *) ((uintptr_t) h + (uintptr_t) h->req_offsets[i]);
}

#endif /* HTPOPS_USE_REFERENCE_HEADERS */

HTPOPS_STATIC_ASSERT(sizeof(struct RpcmemBufAddr) == 8, "RpcmemBufAddr is 8 bytes");
HTPOPS_STATIC_ASSERT(sizeof(struct RmsNormF32Params) == 24, "RmsNormF32Params is 24 bytes");
HTPOPS_STATIC_ASSERT(sizeof(struct MatMulParams) == 36, "MatMulParams is 36 bytes");
HTPOPS_STATIC_ASSERT(sizeof(struct FlashAttnParams) == 60, "FlashAttnParams is 60 bytes");
HTPOPS_STATIC_ASSERT(sizeof(struct MessageState) == 8, "MessageState is 8 bytes");
HTPOPS_STATIC_ASSERT(sizeof(struct MessageHeader) == 16, "MessageHeader is 16 bytes before req_offsets");
HTPOPS_STATIC_ASSERT(sizeof(struct RequestHeader) == 8, "RequestHeader is 8 bytes");
HTPOPS_STATIC_ASSERT(sizeof(struct RpcmemMapRequest) == 8, "RpcmemMapRequest is 8 bytes before fds");
HTPOPS_STATIC_ASSERT(sizeof(struct OpComputeRequest) == 4, "OpComputeRequest is 4 bytes before payload");

/* ---- ops added by this backend ----------------------------------------- */
#define HTP_OPS_EXT_BASE 6

enum HtpOpsExtIndex {
  /* fp32 [ne1][ne0] -> block_q8_0 [ne1][ne0/32]; params: RmsNormF32Params */
  HTP_OPS_QUANTIZE_Q8_0 = HTP_OPS_EXT_BASE + 0,
  /* weights block_q4_0 [n][k/32] (ggml row layout), activations block_q8_0 [m][k/32],
   * output fp32 [m][n]; params: MatMulParams */
  HTP_OPS_MAT_MUL_Q4_0_Q8_0 = HTP_OPS_EXT_BASE + 1,
  /* same with block_q8_0 weights */
  HTP_OPS_MAT_MUL_Q8_0_Q8_0 = HTP_OPS_EXT_BASE + 2,
  /* fp32 activations [m][k]; quantized to Q8_0 inside the op, then as above */
  HTP_OPS_MAT_MUL_Q4_0_A32 = HTP_OPS_EXT_BASE + 3,
  HTP_OPS_MAT_MUL_Q8_0_A32 = HTP_OPS_EXT_BASE + 4,
  /* y = x * rsqrt(mean(x^2) + eps) * w ; params: RmsNormExParams */
  HTP_OPS_RMS_NORM_F32_EX = HTP_OPS_EXT_BASE + 5,
  /* fp16 Q/O/K/V, optional fp16 additive mask, optional causal flag; params: FlashAttnExParams */
  HTP_OPS_FLASH_ATTN_F16 = HTP_OPS_EXT_BASE + 6,
  /* RMSNorm (weight, eps) fused with Q8_0 quantization of the result; params: RmsNormExParams,
   * dst receives block_q8_0 [ne1][ne0/32] */
  HTP_OPS_RMS_NORM_QUANTIZE_Q8_0 = HTP_OPS_EXT_BASE + 7,
  HTP_OPS_EXT_END
};

struct RmsNormExParams {
  struct RpcmemBufAddr dst;
  struct RpcmemBufAddr src;
  struct RpcmemBufAddr weight; /* fp32 [ne0]; fd < 0 means all ones */
  int32_t              ne0;
  int32_t              ne1;
  float                eps;
} HTPOPS_PACKED;
HTPOPS_STATIC_ASSERT(sizeof(struct RmsNormExParams) == 36, "RmsNormExParams is 36 bytes");

struct FlashAttnExParams {
  struct FlashAttnParams base; /* o and q are fp16 here */
  int32_t                causal; /* 1: key j visible to query i iff j <= i + kv_len - qo_len */
} HTPOPS_PACKED;
HTPOPS_STATIC_ASSERT(sizeof(struct FlashAttnExParams) == 64, "FlashAttnExParams is 64 bytes");

/* ---- quantized blocks (reference: include/dsp/quants.h:5-31) ----------- */
#define HTPOPS_QK 32        /* values per block, QK4_0 == QK8_0 == QK_0 */
#define HTPOPS_QK_SUPER 256 /* values per permuted super-block, QK_K     */

typedef uint16_t htpops_fp16_t; /* IEEE binary16 bit pattern */

/* 32 weights: value j (j<16) = (quants[j] & 15) - 8, value j+16 = (quants[j] >> 4) - 8, times scale */
typedef struct {
  htpops_fp16_t scale;
  uint8_t       quants[HTPOPS_QK / 2];
} HTPOPS_PACKED htpops_block_q4_0;

/* 32 values: (int8) quants[j] times scale */
typedef struct {
  htpops_fp16_t scale;
  int8_t        quants[HTPOPS_QK];
} HTPOPS_PACKED htpops_block_q8_0;

/* permuted super-blocks: 8 scales, then the quants of 8 groups */
typedef struct {
  htpops_fp16_t scales[8];
  uint8_t       quants[8 * HTPOPS_QK / 2];
} HTPOPS_PACKED htpops_super_block_q4_0;

typedef struct {
  htpops_fp16_t scales[8];
  int8_t        quants[8 * HTPOPS_QK];
} HTPOPS_PACKED htpops_super_block_q8_0;

HTPOPS_STATIC_ASSERT(sizeof(htpops_block_q4_0) == 18, "block_q4_0 is 18 bytes");
HTPOPS_STATIC_ASSERT(sizeof(htpops_block_q8_0) == 34, "block_q8_0 is 34 bytes");
HTPOPS_STATIC_ASSERT(sizeof(htpops_super_block_q4_0) == 144, "my_block_q4_0 is 144 bytes");
HTPOPS_STATIC_ASSERT(sizeof(htpops_super_block_q8_0) == 272, "my_block_q8_0 is 272 bytes");

/* IQ4_NL code book (reference: src/dsp/ops/mat_mul.c:29-32) */
#define HTPOPS_IQ4_NL_VALUES \
  { -127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113 }

#endif /* HTPOPS_ABI_H */
