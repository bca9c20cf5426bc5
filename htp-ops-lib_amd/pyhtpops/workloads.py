"""Seeded synthetic inputs for the benchmark configurations and the parity tests.

Every generator takes a numpy Generator (PCG64) so that host oracle and GPU see identical bytes.
Quantized tensors are returned as uint8 arrays in the wire layout (block_q4_0 = 18 B, block_q8_0 = 34 B,
reference: include/dsp/quants.h:11-26).
"""
import numpy as np

QK = 32
Q4_0_BLOCK_BYTES = 18
Q8_0_BLOCK_BYTES = 34
GGML_TYPE_Q4_0 = 2
GGML_TYPE_Q8_0 = 8


def rng_for(config, case=0):
    """Generator for benchmark config `config`, case `case`: seed = 1000 * config + case."""
    return np.random.Generator(np.random.PCG64(1000 * int(config) + int(case)))


def block_bytes(weight_type):
    return Q4_0_BLOCK_BYTES if weight_type == GGML_TYPE_Q4_0 else Q8_0_BLOCK_BYTES


def row_bytes(k, weight_type):
    return k // QK * block_bytes(weight_type)


def make_q4_0_weights(rng, n, k, scale_mul=0.02):
    """[n][k/32] block_q4_0: scale = fp16(|N(0,1)| * scale_mul), 16 bytes of two uniform 0..15 nibbles."""
    nb = n * (k // QK)
    out = np.empty((nb, Q4_0_BLOCK_BYTES), dtype=np.uint8)
    d = (np.abs(rng.standard_normal(nb, dtype=np.float32)) * np.float32(scale_mul)).astype(np.float16)
    out[:, 0:2] = d.view(np.uint8).reshape(nb, 2)
    out[:, 2:] = rng.integers(0, 256, size=(nb, QK // 2), dtype=np.uint8)
    return out.reshape(n, -1)


def make_q8_0_weights(rng, n, k, scale_mul=0.01):
    """[n][k/32] block_q8_0: scale = fp16(|N(0,1)| * scale_mul), int8 uniform in [-127, 127]."""
    nb = n * (k // QK)
    out = np.empty((nb, Q8_0_BLOCK_BYTES), dtype=np.uint8)
    d = (np.abs(rng.standard_normal(nb, dtype=np.float32)) * np.float32(scale_mul)).astype(np.float16)
    out[:, 0:2] = d.view(np.uint8).reshape(nb, 2)
    q = rng.integers(-127, 128, size=(nb, QK), dtype=np.int8)
    out[:, 2:] = q.view(np.uint8)
    return out.reshape(n, -1)


def make_weights(rng, n, k, weight_type):
    if weight_type == GGML_TYPE_Q4_0:
        return make_q4_0_weights(rng, n, k)
    if weight_type == GGML_TYPE_Q8_0:
        return make_q8_0_weights(rng, n, k)
    raise ValueError("unsupported weight type %r" % (weight_type,))


def make_activations(rng, m, k):
    """fp32 [m][k] drawn from N(0, 1)."""
    return rng.standard_normal((m, k), dtype=np.float32)


def make_attention_inputs(rng, qo_len, kv_len, n_heads, n_kv_heads, head_dim):
    """Q [qo_len, n_heads, D], K and V [kv_len, n_kv_heads, D], all N(0,1) rounded to fp16."""
    q = rng.standard_normal((qo_len, n_heads, head_dim), dtype=np.float32).astype(np.float16)
    k = rng.standard_normal((kv_len, n_kv_heads, head_dim), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((kv_len, n_kv_heads, head_dim), dtype=np.float32).astype(np.float16)
    return q, k, v


def make_causal_mask(qo_len, kv_len):
    """fp16 [qo_len][align_up(kv_len, 64)] additive mask: 0 where key j <= i + kv_len - qo_len, -inf elsewhere
    (padding columns are -inf). Layout of the reference op (src/dsp/ops/flash_attn.c:152, :1508)."""
    ld = (kv_len + 63) // 64 * 64
    i = np.arange(qo_len)[:, None]
    j = np.arange(ld)[None, :]
    visible = (j <= i + (kv_len - qo_len)) & (j < kv_len)
    return np.where(visible, np.float16(0), np.float16(-np.inf)).astype(np.float16)


# ---- numpy views of the block formats (host-side helpers, no arithmetic of the ops themselves) ----

def q8_0_split(blocks, k):
    """uint8 [m][k/32*34] -> (fp16 scales [m][k/32], int8 quants [m][k])."""
    m = blocks.shape[0]
    b = blocks.reshape(m, k // QK, Q8_0_BLOCK_BYTES)
    d = np.ascontiguousarray(b[:, :, 0:2]).view(np.float16).reshape(m, k // QK)
    q = np.ascontiguousarray(b[:, :, 2:]).view(np.int8).reshape(m, k)
    return d, q


def q4_0_split(blocks, k):
    """uint8 [n][k/32*18] -> (fp16 scales [n][k/32], int8 values (q - 8) [n][k] in K order)."""
    n = blocks.shape[0]
    b = blocks.reshape(n, k // QK, Q4_0_BLOCK_BYTES)
    d = np.ascontiguousarray(b[:, :, 0:2]).view(np.float16).reshape(n, k // QK)
    qs = b[:, :, 2:]
    lo = (qs & 0x0F).astype(np.int8) - 8
    hi = (qs >> 4).astype(np.int8) - 8
    q = np.concatenate([lo, hi], axis=2).reshape(n, k)
    return d, q


# ---- benchmark shapes -----------------------------------------------------------------------------

# (name, n, k) of the seven matmuls of one Llama-7B decoder layer (config 1)
LLAMA7B_LAYER = [
    ("q", 4096, 4096), ("k", 4096, 4096), ("v", 4096, 4096), ("o", 4096, 4096),
    ("gate", 11008, 4096), ("up", 11008, 4096), ("down", 4096, 11008),
]

# Qwen2-1.5B-like block (config 4), Q8_0 weights
QWEN2_1P5B_LAYER = [
    ("q", 1536, 1536), ("k", 256, 1536), ("v", 256, 1536), ("o", 1536, 1536),
    ("gate", 8960, 1536), ("up", 8960, 1536), ("down", 1536, 8960),
]


def matmul_algorithmic_bytes(m, k, n, weight_type):
    """Compulsory traffic: every weight byte once, Q8_0 activations once, fp32 outputs once."""
    return n * row_bytes(k, weight_type) + m * row_bytes(k, GGML_TYPE_Q8_0) + m * n * 4


# ---------------------------------------------------------------------------- the reference's native weight formats
IQ4_NL_VALUES = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.int32)


def w16_tile_layout(w_kn):
    """fp16 weights W[k][n] -> the 32x32 tile order of the reference's fp16 matmul (reference: src/host/test.c:300-312):
    tile (n/32)*(K/32) + k/32, element (k%32 & ~1)*32 + (n%32)*2 + (k&1)."""
    k, n = w_kn.shape
    kk, nn = np.meshgrid(np.arange(k), np.arange(n), indexing="ij")
    idx = ((nn // 32) * (k // 32) + kk // 32) * 1024 + ((kk % 32) & ~1) * 32 + (nn % 32) * 2 + (kk & 1)
    out = np.empty(k * n, np.float16)
    out[idx.reshape(-1)] = w_kn.astype(np.float16).reshape(-1)
    return out


def make_permuted_weights(rng, n, k, kind):
    """Random weights in the super-block formats of ops 2-4 (kind = op id: 2 Q4_0, 3 Q8_0, 4 IQ4_NL): per 32x32 tile
    four super-blocks of 8 fp16 scales + 128 nibble bytes (144 B) or 256 int8 (272 B). Returns the raw bytes."""
    n_sb = (n // 32) * (k // 32) * 4
    scale = 0.01 if kind == 3 else 0.02
    d = (np.abs(rng.standard_normal((n_sb, 8))) * scale).astype(np.float16)
    if kind == 3:
        q = rng.integers(-127, 128, (n_sb, 256), dtype=np.int8).view(np.uint8)
    else:
        q = rng.integers(0, 256, (n_sb, 128), dtype=np.uint8)
    return np.concatenate([d.view(np.uint8).reshape(n_sb, 16), q], axis=1).reshape(-1)


def permuted_to_kn(raw, n, k, kind):
    """Independent numpy reading of the super-block formats: raw bytes -> float32 W[k][n] with values
    fp16(q * scale). Built from the tile geometry alone (a scale covers 2 K rows x 16 columns; a 64-element vector
    is one row pair, columns interleaved with K parity), used to cross-check the C oracle."""
    size = 272 if kind == 3 else 144
    sb = np.asarray(raw, np.uint8).reshape(-1, size)
    n_sb = sb.shape[0]
    scales = sb[:, :16].copy().view(np.float16).astype(np.float32)           # [n_sb][8]
    if kind == 3:
        q = sb[:, 16:].copy().view(np.int8).astype(np.int32).reshape(n_sb, 4, 64)   # vector v = bytes 64v..64v+63
    else:
        b = sb[:, 16:].astype(np.int32).reshape(n_sb, 64, 2)                 # [e][byte parity]
        lo, hi = b & 15, b >> 4
        nib = np.stack([lo[:, :, 0], lo[:, :, 1], hi[:, :, 0], hi[:, :, 1]], axis=1)  # vectors 0..3
        q = IQ4_NL_VALUES[nib] if kind == 4 else nib - 8
    sc = np.repeat(scales.reshape(n_sb, 4, 2), 32, axis=2)                   # [n_sb][v][64]
    vals = (q.astype(np.float32) * sc).astype(np.float16).astype(np.float32)  # one rounding to fp16
    # super-block s of tile t holds row pairs 4s..4s+3; element e = column e//2, K parity e%2
    tiles = vals.reshape(n // 32, k // 32, 4, 4, 32, 2)                       # [n0][k0][s][v][col][par]
    w = tiles.transpose(1, 2, 3, 5, 0, 4).reshape(k, n)                       # k = k0*32 + (4s+v)*2 + par
    return w
