"""ctypes binding of the CPU oracle (test infrastructure only).

Imported by tests/, by __graft_entry__.smoke() and by the CPU-baseline leg of bench.py; the shipped
library and its Python harness never import this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_NAME = "libhtp_oracle.so"

GGML_TYPE_Q4_0 = 2
GGML_TYPE_Q8_0 = 8

_c_void_p = ctypes.c_void_p
_c_int = ctypes.c_int


def build(native=False):
    """Compiles the oracle with make (gcc). Returns the path of the shared object."""
    target = "native" if native else "libhtp_oracle.so"
    subprocess.run(["make", "-C", _HERE, target], check=True, capture_output=True)
    return os.path.join(_HERE, "libhtp_oracle_native.so" if native else _LIB_NAME)


def _ptr(a):
    return a.ctypes.data_as(_c_void_p) if a is not None else None


class Oracle:
    """Thin numpy-facing wrapper. Quantized data travels as uint8 arrays, fp16 as uint16 bit patterns."""

    def __init__(self, path=None):
        if path is None:
            path = os.path.join(_HERE, _LIB_NAME)
            if not os.path.exists(path):
                build()
        lib = ctypes.CDLL(path)
        self.lib = lib
        lib.oracle_fp16_to_fp32.restype = ctypes.c_float
        lib.oracle_fp16_to_fp32.argtypes = [ctypes.c_uint16]
        lib.oracle_fp32_to_fp16.restype = ctypes.c_uint16
        lib.oracle_fp32_to_fp16.argtypes = [ctypes.c_float]
        for name in ("oracle_dequantize_q4_0", "oracle_dequantize_q8_0", "oracle_dequantize_iq4_nl"):
            getattr(lib, name).restype = None
            getattr(lib, name).argtypes = [_c_void_p, _c_int, _c_void_p]
        lib.oracle_quantize_q8_0.restype = None
        lib.oracle_quantize_q8_0.argtypes = [_c_void_p, _c_void_p, _c_int, _c_int]
        for name in ("oracle_block_dot_q4_0_q8_0", "oracle_block_dot_q8_0_q8_0"):
            getattr(lib, name).restype = ctypes.c_int32
            getattr(lib, name).argtypes = [_c_void_p, _c_void_p]
        for name in ("oracle_vec_dot_q4_0_q8_0", "oracle_vec_dot_q8_0_q8_0"):
            getattr(lib, name).restype = ctypes.c_float
            getattr(lib, name).argtypes = [_c_int, _c_void_p, _c_void_p]
        lib.oracle_mat_mul_q8_0_act.restype = _c_int
        lib.oracle_mat_mul_q8_0_act.argtypes = [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int]
        lib.oracle_mat_mul_f32_act.restype = _c_int
        lib.oracle_mat_mul_f32_act.argtypes = [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int]
        lib.oracle_mat_mul_q8_0_act_abs.restype = _c_int
        lib.oracle_mat_mul_q8_0_act_abs.argtypes = [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int]
        lib.oracle_rms_norm_f32_ex.restype = _c_int
        lib.oracle_rms_norm_f32_ex.argtypes = [_c_void_p, _c_void_p, _c_void_p, ctypes.c_float, _c_int, _c_int]
        lib.oracle_rms_norm_f32.restype = _c_int
        lib.oracle_rms_norm_f32.argtypes = [_c_void_p, _c_void_p, _c_int, _c_int]
        for name in ("oracle_flash_attn", "oracle_flash_attn_f16"):
            getattr(lib, name).restype = _c_int
            getattr(lib, name).argtypes = [_c_void_p] * 5 + [_c_int] * 6
        lib.oracle_mat_mul_w16a32.restype = _c_int
        lib.oracle_mat_mul_w16a32.argtypes = [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int]
        lib.oracle_dequantize_permuted_q4_0.restype = None
        lib.oracle_dequantize_permuted_q4_0.argtypes = [_c_void_p, _c_int, _c_int, _c_void_p]
        lib.oracle_dequantize_permuted_q8_0.restype = None
        lib.oracle_dequantize_permuted_q8_0.argtypes = [_c_void_p, _c_int, _c_void_p]
        lib.oracle_mat_mul_permuted.restype = _c_int
        lib.oracle_mat_mul_permuted.argtypes = [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int]
        lib.oracle_w16_tile_index.restype = ctypes.c_size_t
        lib.oracle_w16_tile_index.argtypes = [_c_int, _c_int, _c_int]

    # -- scalars ---------------------------------------------------------
    def fp16_to_fp32(self, h):
        return float(self.lib.oracle_fp16_to_fp32(int(h)))

    def fp32_to_fp16(self, f):
        return int(self.lib.oracle_fp32_to_fp16(float(f)))

    # -- formats ---------------------------------------------------------
    def dequantize(self, blocks, kind):
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        bsz = {"q4_0": 18, "iq4_nl": 18, "q8_0": 34}[kind]
        nb = blocks.size // bsz
        out = np.empty(nb * 32, dtype=np.float32)
        getattr(self.lib, "oracle_dequantize_" + kind)(_ptr(blocks), nb, _ptr(out))
        return out

    def quantize_q8_0(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        m, k = x.shape
        assert k % 32 == 0
        out = np.empty((m, k // 32 * 34), dtype=np.uint8)
        self.lib.oracle_quantize_q8_0(_ptr(x), _ptr(out), k, m)
        return out

    def block_dot(self, w_block, a_block, weight_type):
        w_block = np.ascontiguousarray(w_block, dtype=np.uint8)
        a_block = np.ascontiguousarray(a_block, dtype=np.uint8)
        fn = self.lib.oracle_block_dot_q4_0_q8_0 if weight_type == GGML_TYPE_Q4_0 else self.lib.oracle_block_dot_q8_0_q8_0
        return int(fn(_ptr(w_block), _ptr(a_block)))

    def vec_dot(self, k, w_row, a_row, weight_type):
        w_row = np.ascontiguousarray(w_row, dtype=np.uint8)
        a_row = np.ascontiguousarray(a_row, dtype=np.uint8)
        fn = self.lib.oracle_vec_dot_q4_0_q8_0 if weight_type == GGML_TYPE_Q4_0 else self.lib.oracle_vec_dot_q8_0_q8_0
        return float(fn(k, _ptr(w_row), _ptr(a_row)))

    # -- matmul ----------------------------------------------------------
    def mat_mul_q8_0_act(self, act_q8, w, m, k, n, weight_type, n_threads=1):
        act_q8 = np.ascontiguousarray(act_q8, dtype=np.uint8)
        w = np.ascontiguousarray(w, dtype=np.uint8)
        out = np.empty((m, n), dtype=np.float32)
        ret = self.lib.oracle_mat_mul_q8_0_act(_ptr(out), _ptr(act_q8), _ptr(w), m, k, n, weight_type, n_threads)
        if ret != 0:
            raise ValueError("oracle_mat_mul_q8_0_act rejected its arguments")
        return out

    def mat_mul_f32_act(self, act, w, m, k, n, weight_type, n_threads=1):
        act = np.ascontiguousarray(act, dtype=np.float32)
        w = np.ascontiguousarray(w, dtype=np.uint8)
        out = np.empty((m, n), dtype=np.float32)
        ret = self.lib.oracle_mat_mul_f32_act(_ptr(out), _ptr(act), _ptr(w), m, k, n, weight_type, n_threads)
        if ret != 0:
            raise ValueError("oracle_mat_mul_f32_act rejected its arguments")
        return out

    def mat_mul_q8_0_act_f64(self, act_q8, w, m, k, n, weight_type):
        """Returns (value accumulated in double, sum of |terms|) per output."""
        act_q8 = np.ascontiguousarray(act_q8, dtype=np.uint8)
        w = np.ascontiguousarray(w, dtype=np.uint8)
        out = np.empty((m, n), dtype=np.float64)
        mag = np.empty((m, n), dtype=np.float64)
        ret = self.lib.oracle_mat_mul_q8_0_act_abs(_ptr(out), _ptr(mag), _ptr(act_q8), _ptr(w), m, k, n, weight_type)
        if ret != 0:
            raise ValueError("oracle_mat_mul_q8_0_act_abs rejected its arguments")
        return out, mag

    # -- rmsnorm ---------------------------------------------------------
    def rms_norm(self, x, w=None, eps=1e-5):
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        ne1, ne0 = x.shape
        out = np.empty_like(x)
        if w is not None:
            w = np.ascontiguousarray(w, dtype=np.float32)
        ret = self.lib.oracle_rms_norm_f32_ex(_ptr(out), _ptr(x), _ptr(w), eps, ne0, ne1)
        if ret != 0:
            raise ValueError("oracle_rms_norm_f32_ex rejected its arguments")
        return out

    # -- attention -------------------------------------------------------
    def flash_attn(self, q, k, v, mask, n_heads, n_kv_heads, head_dim, causal=False):
        """q fp32 or fp16 [qo_len, n_heads, head_dim]; k, v fp16 [kv_len, n_kv_heads, head_dim];
        mask fp16 [qo_len, align_up(kv_len, 64)] or None. Output has q's dtype."""
        k = np.ascontiguousarray(k, dtype=np.float16)
        v = np.ascontiguousarray(v, dtype=np.float16)
        qo_len, kv_len = q.shape[0], k.shape[0]
        if mask is not None:
            mask = np.ascontiguousarray(mask, dtype=np.float16)
            assert mask.shape[1] == (kv_len + 63) // 64 * 64 and mask.shape[0] >= qo_len
        if q.dtype == np.float16:
            q = np.ascontiguousarray(q)
            out = np.empty_like(q)
            fn = self.lib.oracle_flash_attn_f16
        else:
            q = np.ascontiguousarray(q, dtype=np.float32)
            out = np.empty_like(q)
            fn = self.lib.oracle_flash_attn
        ret = fn(_ptr(out), _ptr(q), _ptr(k), _ptr(v), _ptr(mask), qo_len, kv_len, n_heads, n_kv_heads, head_dim,
                 1 if causal else 0)
        if ret != 0:
            raise ValueError("oracle_flash_attn rejected its arguments")
        return out

    @staticmethod
    def threshold_mask(mask):
        """The additive mask that selects the same keys as the kernel the reference dispatches for op 5: that kernel
        keeps a key iff its fp16 mask value is > -16 and sets the score of every other key to -inf
        (src/dsp/ops/flash_attn.c:448-460: Q6_Q_vcmp_gt_VhfVhf against 0xcc00, then a mux with -inf); a NaN compares
        false and is dropped. flash_attn(..., threshold_mask(mask)) is therefore that kernel's rule on top of the
        scalar routine's arithmetic."""
        m = np.asarray(mask, dtype=np.float16)
        with np.errstate(invalid="ignore"):
            keep = m > np.float16(-16.0)
        return np.where(keep, np.float16(0.0), np.float16(-np.inf)).astype(np.float16)

    # -- fp16 tiles --------------------------------------------------------
    def mat_mul_w16a32(self, act, w_tiles, m, k, n):
        act = np.ascontiguousarray(act, dtype=np.float32)
        w_tiles = np.ascontiguousarray(w_tiles, dtype=np.float16)
        out = np.empty((m, n), dtype=np.float32)
        ret = self.lib.oracle_mat_mul_w16a32(_ptr(out), _ptr(act), _ptr(w_tiles), m, k, n)
        if ret != 0:
            raise ValueError("oracle_mat_mul_w16a32 rejected its arguments")
        return out

    def dequantize_permuted(self, super_blocks, kind):
        """kind: 2 Q4_0, 3 Q8_0, 4 IQ4_NL (the op ids) -> fp16 [n_super_blocks][256] in tile order."""
        sb = np.ascontiguousarray(super_blocks, dtype=np.uint8).reshape(-1)
        size = 272 if kind == 3 else 144
        n = sb.size // size
        out = np.empty((n, 256), dtype=np.float16)
        if kind == 3:
            self.lib.oracle_dequantize_permuted_q8_0(_ptr(sb), n, _ptr(out))
        else:
            self.lib.oracle_dequantize_permuted_q4_0(_ptr(sb), n, 1 if kind == 4 else 0, _ptr(out))
        return out

    def mat_mul_permuted(self, act, weight, m, k, n, kind, want_f64=False):
        """Ops 1-4: returns fp32 [m][n] (fp16-rounded values), optionally also the unrounded double sums."""
        act = np.ascontiguousarray(act, dtype=np.float32)
        weight = np.ascontiguousarray(weight)
        out = np.empty((m, n), dtype=np.float32)
        f64 = np.empty((m, n), dtype=np.float64)
        ret = self.lib.oracle_mat_mul_permuted(_ptr(out), _ptr(f64), _ptr(act), _ptr(weight), m, k, n, kind)
        if ret != 0:
            raise ValueError("oracle_mat_mul_permuted rejected its arguments")
        return (out, f64) if want_f64 else out

    def w16_tile_index(self, kk, nn, k):
        return int(self.lib.oracle_w16_tile_index(kk, nn, k))


class RefNaiveFlashAttn:
    """The reference's own scalar attention routine, when oracle/_ref has been built (see Makefile)."""

    def __init__(self):
        path = os.path.join(_HERE, "_ref", "libref_naive_flash_attn.so")
        if not os.path.exists(path):
            raise FileNotFoundError(path)
        self.lib = ctypes.CDLL(path)
        self.lib.naive_flash_attn.restype = _c_int
        self.lib.naive_flash_attn.argtypes = [_c_void_p] * 5 + [_c_int] * 5

    def __call__(self, q, k, v, mask, n_heads, n_kv_heads, head_dim):
        q = np.ascontiguousarray(q, dtype=np.float32)
        k = np.ascontiguousarray(k, dtype=np.float16)
        v = np.ascontiguousarray(v, dtype=np.float16)
        if mask is not None:
            mask = np.ascontiguousarray(mask, dtype=np.float16)
        out = np.empty_like(q)
        ret = self.lib.naive_flash_attn(_ptr(out), _ptr(q), _ptr(k), _ptr(v), _ptr(mask), q.shape[0], k.shape[0],
                                        n_heads, n_kv_heads, head_dim)
        if ret != 0:
            raise ValueError("naive_flash_attn returned %d" % ret)
        return out
