"""ctypes binding of libhtpops_mi355x.so plus builders for the wire structs.

This is harness code for tests and benchmarks: it mirrors the reference's host-side usage (allocate shared
buffers, fill a request, run it; reference: src/host/test.c:30-58, :166-200) on top of the C ABI declared in
include/htpops.h. It contains no arithmetic of the ops and no fallback: if the shared library or a GPU is
missing, calls fail.
"""
import ctypes
import os
import struct
import subprocess

import numpy as np

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG_DIR, "libhtpops_mi355x.so")

# op ids (include/htpops_abi.h)
HTP_OPS_RMS_NORM_F32 = 0
HTP_OPS_MAT_MUL_PERMUTED_W16A32 = 1
HTP_OPS_MAT_MUL_PERMUTED_W4D16A32 = 2
HTP_OPS_MAT_MUL_PERMUTED_W8D16A32 = 3
HTP_OPS_MAT_MUL_PERMUTED_W4D16A32_IQ4_NL = 4
HTP_OPS_FLASH_ATTN_QO_F32_KV_F16 = 5
HTP_OPS_QUANTIZE_Q8_0 = 6
HTP_OPS_MAT_MUL_Q4_0_Q8_0 = 7
HTP_OPS_MAT_MUL_Q8_0_Q8_0 = 8
HTP_OPS_MAT_MUL_Q4_0_A32 = 9
HTP_OPS_MAT_MUL_Q8_0_A32 = 10
HTP_OPS_RMS_NORM_F32_EX = 11
HTP_OPS_FLASH_ATTN_F16 = 12
HTP_OPS_RMS_NORM_QUANTIZE_Q8_0 = 13

REQUEST_TYPE_NO_OP = 0
REQUEST_TYPE_RPCMEM_MAP = 1
REQUEST_TYPE_OP_COMPUTE = 2

HTPOPS_OK = 0
HTPOPS_ERR_REJECTED = -1
HTPOPS_ERR_NO_DEVICE = -2
HTPOPS_ERR_HIP = -3
HTPOPS_ERR_NOMEM = -4
HTPOPS_ERR_BUSY = -5
HTPOPS_DEVICE_NONE = -1

GGML_TYPE_Q4_0 = 2
GGML_TYPE_Q8_0 = 8

EXPORTED_SYMBOLS = [
    "htpops_init_backend", "htpops_close", "htpops_last_error", "htpops_set_option", "htpops_get_option",
    "htpops_synchronize", "htpops_get_stream", "htpops_buffer_prepare_weights", "htpops_converted_bytes",
    "htpops_workspace_bytes",
    "htpops_buffer_alloc", "htpops_buffer_register", "htpops_buffer_release", "htpops_buffer_device_ptr",
    "htpops_buffer_size", "htpops_buffer_invalidate", "htpops_buffer_write", "htpops_buffer_read", "htpops_execute_op",
    "htpops_process_message", "htpops_enqueue_message", "htpops_finish_message", "htpops_last_message_submissions",
    "htpops_record_message", "htpops_launch_recorded_message", "htpops_release_recorded_message", "htpops_create_channel", "htpops_destroy_channel", "htpops_rms_norm_f32",
    "htpops_mat_mul_permuted_w16a32", "htpops_rms_norm_f32_ex_ptr", "htpops_quantize_q8_0_ptr",
    "htpops_rms_norm_quantize_q8_0_ptr", "htpops_mat_mul_q8_0_act_ptr", "htpops_mat_mul_f32_act_ptr",
    "htpops_flash_attn_ptr", "htpops_flash_attn_noalloc_ptr", "htpops_timer_start", "htpops_timer_stop", "htpops_timer_elapsed_ms",
    "htpops_measure_mfma_peak", "htpops_measure_copy_bandwidth", "htpops_measure_read_us", "htpops_last_gemv_launch",
    "htpops_measure_host_walk_us",
    "htpops_measure_decode_attention_parts",
]


# the switches of a context (htpops_set_option) and the values they start from
DEFAULT_OPTIONS = {"lane_order": 1, "gemm_fp6": -1, "gemv_rows_kernel": 1, "gemm_tile_units": 0, "attn_key_groups": 0,
                   "attn_mask_threshold": 0, "converted_cap_mib": 0, "log": 0}


def build_library():
    """Compiles the shared library with make + hipcc (gfx950). Raises on failure."""
    subprocess.run(["make", "-C", _PKG_DIR, "-j8"], check=True, capture_output=True)
    return LIB_PATH


def load_library(path=None):
    path = path or LIB_PATH
    if not os.path.exists(path):
        raise FileNotFoundError(
            "%s is missing: build it with `make -C %s` (hipcc, gfx950) before running" % (path, _PKG_DIR))
    lib = ctypes.CDLL(path)
    vp, ci, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    sig = {
        "htpops_init_backend": (ci, [ctypes.POINTER(vp), ci]),
        "htpops_close": (ci, [vp]),
        "htpops_last_error": (ctypes.c_char_p, [vp]),
        "htpops_set_option": (ci, [vp, ctypes.c_char_p, ci]),
        "htpops_get_option": (ci, [vp, ctypes.c_char_p, ctypes.POINTER(ci)]),
        "htpops_buffer_prepare_weights": (ci, [vp, ci, sz, ci, ci, ci, ci, ctypes.POINTER(sz)]),
        "htpops_converted_bytes": (sz, [vp]),
        "htpops_workspace_bytes": (sz, [vp]),
        "htpops_synchronize": (ci, [vp]),
        "htpops_get_stream": (vp, [vp]),
        "htpops_buffer_alloc": (ci, [vp, sz]),
        "htpops_buffer_register": (ci, [vp, vp, sz]),
        "htpops_buffer_release": (ci, [vp, ci]),
        "htpops_buffer_device_ptr": (vp, [vp, ci]),
        "htpops_buffer_size": (sz, [vp, ci]),
        "htpops_buffer_invalidate": (ci, [vp, ci]),
        "htpops_buffer_write": (ci, [vp, ci, sz, vp, sz]),
        "htpops_buffer_read": (ci, [vp, ci, sz, vp, sz]),
        "htpops_execute_op": (ci, [vp, vp]),
        "htpops_process_message": (ci, [vp, vp, sz]),
        "htpops_enqueue_message": (ci, [vp, vp, sz]),
        "htpops_finish_message": (ci, [vp, vp]),
        "htpops_last_message_submissions": (ci, [vp]),
        "htpops_record_message": (ci, [vp, vp, sz, ctypes.POINTER(vp)]),
        "htpops_launch_recorded_message": (ci, [vp, vp]),
        "htpops_release_recorded_message": (ci, [vp, vp]),
        "htpops_create_channel": (ci, [vp, vp, sz]),
        "htpops_destroy_channel": (ci, [vp]),
        "htpops_rms_norm_f32": (ci, [vp, ci, ci, ci, ci, ci, ci]),
        "htpops_mat_mul_permuted_w16a32": (ci, [vp] + [ci] * 9),
        "htpops_rms_norm_f32_ex_ptr": (ci, [vp, vp, vp, vp, ctypes.c_float, ci, ci]),
        "htpops_quantize_q8_0_ptr": (ci, [vp, vp, vp, ci, ci]),
        "htpops_rms_norm_quantize_q8_0_ptr": (ci, [vp, vp, vp, vp, ctypes.c_float, ci, ci]),
        "htpops_mat_mul_q8_0_act_ptr": (ci, [vp, vp, vp, vp, ci, ci, ci, ci]),
        "htpops_mat_mul_f32_act_ptr": (ci, [vp, vp, vp, vp, ci, ci, ci, ci]),
        "htpops_flash_attn_ptr": (ci, [vp] * 6 + [ci] * 7),
        "htpops_flash_attn_noalloc_ptr": (ci, [vp] * 6 + [ci] * 7),
        "htpops_timer_start": (ci, [vp]),
        "htpops_timer_stop": (ci, [vp]),
        "htpops_timer_elapsed_ms": (ci, [vp, ctypes.POINTER(ctypes.c_float)]),
        "htpops_measure_mfma_peak": (ci, [vp, ci, ci, ctypes.POINTER(ctypes.c_double)]),
        "htpops_measure_copy_bandwidth": (ci, [vp, sz, ci, ctypes.POINTER(ctypes.c_double)]),
        "htpops_measure_read_us": (ci, [vp, sz, ci, ci, ctypes.POINTER(ctypes.c_double)]),
        "htpops_last_gemv_launch": (ci, [vp, ctypes.c_char_p, sz]),
        "htpops_measure_host_walk_us": (ci, [vp, vp, sz, ci, ctypes.POINTER(ctypes.c_double)]),
        "htpops_measure_decode_attention_parts": (ci, [vp, vp, vp, ctypes.POINTER(vp), ctypes.POINTER(vp), ci, ci, ci, ci, ci,
                                                       ci, ci, ctypes.POINTER(ctypes.c_double),
                                                       ctypes.POINTER(ctypes.c_double)]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


# ---- wire structs (little endian, packed; include/htpops_abi.h) --------------------------------------

def buf_addr(fd, offset=0):
    return struct.pack("<ii", fd, offset)


def rms_norm_params(dst, src, ne0, ne1):
    return buf_addr(*dst) + buf_addr(*src) + struct.pack("<ii", ne0, ne1)


def rms_norm_ex_params(dst, src, weight, ne0, ne1, eps):
    return buf_addr(*dst) + buf_addr(*src) + buf_addr(*weight) + struct.pack("<iif", ne0, ne1, eps)


def mat_mul_params(output, activation, weight, m, k, n):
    return buf_addr(*output) + buf_addr(*activation) + buf_addr(*weight) + struct.pack("<iii", m, k, n)


def flash_attn_params(o, q, k, v, mask, qo_len, kv_len, n_heads, n_kv_heads, head_dim, causal=None):
    body = (buf_addr(*o) + buf_addr(*q) + buf_addr(*k) + buf_addr(*v) + buf_addr(*mask) +
            struct.pack("<iiiii", qo_len, kv_len, n_heads, n_kv_heads, head_dim))
    if causal is not None:
        body += struct.pack("<i", int(causal))
    return body


def op_compute_request(op, payload):
    return struct.pack("<I", op) + payload


def build_message(requests):
    """requests: list of (request_type, body_bytes). Returns a bytearray laid out like the reference's host code
    does (src/host/test.c:166-194): MessageHeader, n + 1 offsets, then RequestHeader + body per request."""
    n = len(requests)
    header_size = 16 + 4 * (n + 1)
    offsets = [header_size]
    for _, body in requests:
        offsets.append(offsets[-1] + 8 + len(body))
    msg = bytearray(offsets[-1])
    struct.pack_into("<QIi", msg, 0, 0, 0, n)
    struct.pack_into("<%di" % (n + 1), msg, 16, *offsets)
    for i, (rtype, body) in enumerate(requests):
        struct.pack_into("<ii", msg, offsets[i], 0, rtype)
        msg[offsets[i] + 8:offsets[i] + 8 + len(body)] = body
    return msg


def message_request_states(msg):
    n = struct.unpack_from("<i", msg, 12)[0]
    offsets = struct.unpack_from("<%di" % (n + 1), msg, 16)
    return [struct.unpack_from("<i", msg, offsets[i])[0] for i in range(n)]


class HtpOpsError(RuntimeError):
    def __init__(self, code, text):
        RuntimeError.__init__(self, "htpops error %d: %s" % (code, text))
        self.code = code


class Context:
    """One backend context (one HIP stream). device=None creates a validation-only context."""

    def __init__(self, device=0, lib=None):
        self.lib = lib or load_library()
        self._ctx = ctypes.c_void_p()
        dev = HTPOPS_DEVICE_NONE if device is None else int(device)
        ret = self.lib.htpops_init_backend(ctypes.byref(self._ctx), dev)
        if ret != HTPOPS_OK:
            raise HtpOpsError(ret, "htpops_init_backend(device=%r) failed" % (device,))
        self.has_device = device is not None

    # -- lifetime --
    def close(self):
        if self._ctx:
            self.lib.htpops_close(self._ctx)
            self._ctx = ctypes.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def last_error(self):
        return self.lib.htpops_last_error(self._ctx).decode()

    def _check(self, ret):
        if ret < 0:
            raise HtpOpsError(ret, self.last_error())
        return ret

    def synchronize(self):
        self._check(self.lib.htpops_synchronize(self._ctx))

    # -- switches --
    def set_option(self, name, value):
        self._check(self.lib.htpops_set_option(self._ctx, name.encode(), int(value)))

    def get_option(self, name):
        v = ctypes.c_int()
        self._check(self.lib.htpops_get_option(self._ctx, name.encode(), ctypes.byref(v)))
        return int(v.value)

    def option(self, name, value):
        """Context manager: the switch `name` holds `value` inside the with block and its old value afterwards."""
        ctx = self

        class _Scoped:
            def __enter__(self_inner):
                self_inner.old = ctx.get_option(name)
                ctx.set_option(name, value)
                return ctx

            def __exit__(self_inner, *exc):
                ctx.set_option(name, self_inner.old)

        return _Scoped()

    # -- buffers --
    def alloc(self, nbytes):
        return self._check(self.lib.htpops_buffer_alloc(self._ctx, int(nbytes)))

    def register(self, device_ptr, nbytes):
        """Registers caller-owned device memory (not freed on release); returns a handle."""
        return self._check(self.lib.htpops_buffer_register(self._ctx, ctypes.c_void_p(device_ptr), int(nbytes)))

    def release(self, handle):
        return self.lib.htpops_buffer_release(self._ctx, int(handle))

    def size(self, handle):
        return int(self.lib.htpops_buffer_size(self._ctx, int(handle)))

    def device_ptr(self, handle):
        return self.lib.htpops_buffer_device_ptr(self._ctx, int(handle))

    def invalidate(self, handle):
        return self.lib.htpops_buffer_invalidate(self._ctx, int(handle))

    def prepare_weights(self, handle, weight_type, n, k, m_hint, offset=0):
        """htpops_buffer_prepare_weights; returns the bytes of converted copies the call added."""
        added = ctypes.c_size_t()
        self._check(self.lib.htpops_buffer_prepare_weights(self._ctx, int(handle), int(offset), int(weight_type), int(n),
                                                           int(k), int(m_hint), ctypes.byref(added)))
        return int(added.value)

    def converted_bytes(self):
        return int(self.lib.htpops_converted_bytes(self._ctx))

    def workspace_bytes(self):
        return int(self.lib.htpops_workspace_bytes(self._ctx))

    def write(self, handle, array, offset=0):
        a = np.ascontiguousarray(array)
        self._check(self.lib.htpops_buffer_write(self._ctx, handle, offset, a.ctypes.data_as(ctypes.c_void_p), a.nbytes))

    def read(self, handle, dtype, count, offset=0):
        out = np.empty(count, dtype=dtype)
        self._check(self.lib.htpops_buffer_read(self._ctx, handle, offset, out.ctypes.data_as(ctypes.c_void_p), out.nbytes))
        return out

    def upload(self, array):
        """Allocates a buffer of the array's size and copies it in; returns the handle."""
        a = np.ascontiguousarray(array)
        h = self.alloc(max(a.nbytes, 1))
        if a.nbytes:
            self.write(h, a)
        return h

    # -- ops --
    def execute(self, op, payload):
        """htpops_execute_op; returns the raw return code (0 / negative)."""
        req = op_compute_request(op, payload)
        buf = (ctypes.c_char * len(req)).from_buffer_copy(req)
        return self.lib.htpops_execute_op(self._ctx, ctypes.cast(buf, ctypes.c_void_p))

    def process_message(self, msg, bound=True):
        """Runs a message built by build_message in place; returns htpops_process_message's code."""
        buf = (ctypes.c_char * len(msg)).from_buffer(msg)
        return self.lib.htpops_process_message(self._ctx, ctypes.cast(buf, ctypes.c_void_p), len(msg) if bound else 0)

    def enqueue_message(self, msg):
        """htpops_enqueue_message: enqueue only. `msg` must stay alive until finish_message."""
        buf = (ctypes.c_char * len(msg)).from_buffer(msg)
        return self.lib.htpops_enqueue_message(self._ctx, ctypes.cast(buf, ctypes.c_void_p), len(msg))

    def message_handle(self, msg):
        """(address, length) of a message buffer for enqueue_message_handle: a driver loop that submits the same
        messages again and again pays the buffer lookup once. `msg` must stay alive as long as the handle is used."""
        buf = (ctypes.c_char * len(msg)).from_buffer(msg)
        return ctypes.cast(buf, ctypes.c_void_p), len(msg)

    def enqueue_message_handle(self, handle):
        return self.lib.htpops_enqueue_message(self._ctx, handle[0], handle[1])

    def finish_message(self, msg):
        buf = (ctypes.c_char * len(msg)).from_buffer(msg)
        return self.lib.htpops_finish_message(self._ctx, ctypes.cast(buf, ctypes.c_void_p))

    def last_message_submissions(self):
        return self.lib.htpops_last_message_submissions(self._ctx)

    def record_message(self, msg):
        """htpops_record_message: runs `msg` once and returns (code, recording); the recording is None on failure."""
        buf = (ctypes.c_char * len(msg)).from_buffer(msg)
        rec = ctypes.c_void_p()
        ret = self.lib.htpops_record_message(self._ctx, ctypes.cast(buf, ctypes.c_void_p), len(msg), ctypes.byref(rec))
        return ret, (rec if ret == 0 else None)

    def launch_recorded_message(self, rec):
        return self.lib.htpops_launch_recorded_message(self._ctx, rec)

    def release_recorded_message(self, rec):
        return self.lib.htpops_release_recorded_message(self._ctx, rec)

    # -- timing --
    def timer_start(self):
        self._check(self.lib.htpops_timer_start(self._ctx))

    def timer_stop_ms(self):
        self._check(self.lib.htpops_timer_stop(self._ctx))
        ms = ctypes.c_float()
        self._check(self.lib.htpops_timer_elapsed_ms(self._ctx, ctypes.byref(ms)))
        return float(ms.value)

    def measure_mfma_peak(self, kind, iters=20000):
        v = ctypes.c_double()
        self._check(self.lib.htpops_measure_mfma_peak(self._ctx, kind, iters, ctypes.byref(v)))
        return float(v.value)

    def measure_read_us(self, nbytes, buffers, iters=10):
        v = ctypes.c_double()
        self._check(self.lib.htpops_measure_read_us(self._ctx, int(nbytes), buffers, iters, ctypes.byref(v)))
        return v.value

    def last_gemv_launch(self):
        buf = ctypes.create_string_buffer(256)
        self._check(self.lib.htpops_last_gemv_launch(self._ctx, buf, len(buf)))
        return buf.value.decode()

    def measure_host_walk_us(self, msg, iters=2000):
        """Host microseconds per htpops_enqueue_message of `msg` with the stream kept busy (no kernel time)."""
        buf = (ctypes.c_char * len(msg)).from_buffer(msg)
        v = ctypes.c_double()
        self._check(self.lib.htpops_measure_host_walk_us(self._ctx, ctypes.cast(buf, ctypes.c_void_p), len(msg), iters,
                                                         ctypes.byref(v)))
        return float(v.value)

    def measure_decode_attention_parts(self, o, q, ks, vs, kv_len, n_heads, n_kv_heads, head_dim, qo_is_f32, iters=100):
        """(split-KV launch, merge launch) of one-token attention in microseconds per launch; o, q, ks[i], vs[i] are
        buffer handles."""
        n = len(ks)
        kp = (ctypes.c_void_p * n)(*[self.device_ptr(h) for h in ks])
        vpp = (ctypes.c_void_p * n)(*[self.device_ptr(h) for h in vs])
        a, b = ctypes.c_double(), ctypes.c_double()
        self._check(self.lib.htpops_measure_decode_attention_parts(
            self._ctx, ctypes.c_void_p(self.device_ptr(o)), ctypes.c_void_p(self.device_ptr(q)), kp, vpp, n, kv_len,
            n_heads, n_kv_heads, head_dim, int(qo_is_f32), iters, ctypes.byref(a), ctypes.byref(b)))
        return float(a.value), float(b.value)

    def measure_copy_bandwidth(self, nbytes, iters=20):
        v = ctypes.c_double()
        self._check(self.lib.htpops_measure_copy_bandwidth(self._ctx, int(nbytes), iters, ctypes.byref(v)))
        return float(v.value)

    # -- convenience wrappers used by tests and the benchmark: upload, run through the op ABI, download --
    def run_quantize_q8_0(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        m, k = x.shape
        hx, hy = self.upload(x), self.alloc(m * (k // 32) * 34)
        try:
            self._check(self.execute(HTP_OPS_QUANTIZE_Q8_0, rms_norm_params((hy, 0), (hx, 0), k, m)))
            self.synchronize()
            return self.read(hy, np.uint8, m * (k // 32) * 34).reshape(m, -1)
        finally:
            self.release(hx), self.release(hy)

    def run_rms_norm(self, x, weight=None, eps=None, quantize=False):
        x = np.ascontiguousarray(x, dtype=np.float32)
        ne1, ne0 = x.shape
        out_bytes = ne1 * (ne0 // 32) * 34 if quantize else x.nbytes
        hx, hy = self.upload(x), self.alloc(out_bytes)
        hw = self.upload(np.ascontiguousarray(weight, dtype=np.float32)) if weight is not None else -1
        try:
            if eps is None and weight is None and not quantize:
                ret = self.execute(HTP_OPS_RMS_NORM_F32, rms_norm_params((hy, 0), (hx, 0), ne0, ne1))
            else:
                op = HTP_OPS_RMS_NORM_QUANTIZE_Q8_0 if quantize else HTP_OPS_RMS_NORM_F32_EX
                ret = self.execute(op, rms_norm_ex_params((hy, 0), (hx, 0), (hw, 0), ne0, ne1,
                                                          1e-5 if eps is None else eps))
            self._check(ret)
            self.synchronize()
            if quantize:
                return self.read(hy, np.uint8, out_bytes).reshape(ne1, -1)
            return self.read(hy, np.float32, ne0 * ne1).reshape(ne1, ne0)
        finally:
            self.release(hx), self.release(hy)
            if hw > 0:
                self.release(hw)

    def run_mat_mul(self, act, weight, m, k, n, weight_type, act_is_f32=False):
        if act_is_f32:
            op = HTP_OPS_MAT_MUL_Q4_0_A32 if weight_type == GGML_TYPE_Q4_0 else HTP_OPS_MAT_MUL_Q8_0_A32
            act = np.ascontiguousarray(act, dtype=np.float32)
        else:
            op = HTP_OPS_MAT_MUL_Q4_0_Q8_0 if weight_type == GGML_TYPE_Q4_0 else HTP_OPS_MAT_MUL_Q8_0_Q8_0
            act = np.ascontiguousarray(act, dtype=np.uint8)
        ha, hw, ho = self.upload(act), self.upload(np.ascontiguousarray(weight, dtype=np.uint8)), self.alloc(m * n * 4)
        try:
            self._check(self.execute(op, mat_mul_params((ho, 0), (ha, 0), (hw, 0), m, k, n)))
            self.synchronize()
            return self.read(ho, np.float32, m * n).reshape(m, n)
        finally:
            self.release(ha), self.release(hw), self.release(ho)

    def run_mat_mul_permuted(self, act, weight_raw, m, k, n, op, repeats=1):
        """The reference's ops 1-4: fp32 activations, weights in the reference's tile order (raw bytes)."""
        act = np.ascontiguousarray(act, dtype=np.float32)
        ha, hw, ho = self.upload(act), self.upload(np.ascontiguousarray(weight_raw).view(np.uint8)), self.alloc(m * n * 4)
        try:
            for _ in range(repeats):
                self._check(self.execute(op, mat_mul_params((ho, 0), (ha, 0), (hw, 0), m, k, n)))
            self.synchronize()
            return self.read(ho, np.float32, m * n).reshape(m, n)
        finally:
            self.release(ha), self.release(hw), self.release(ho)

    def run_flash_attn(self, q, k, v, mask, n_heads, n_kv_heads, head_dim, causal=False):
        """q fp32 -> the reference op (id 5); q fp16 -> the extended op with the causal flag."""
        qo_len, kv_len = q.shape[0], k.shape[0]
        f16 = q.dtype == np.float16
        q = np.ascontiguousarray(q)
        hq, hk, hv = self.upload(q), self.upload(np.ascontiguousarray(k, np.float16)), self.upload(np.ascontiguousarray(v, np.float16))
        ho = self.alloc(q.nbytes)
        hm = self.upload(np.ascontiguousarray(mask, np.float16)) if mask is not None else -1
        try:
            if f16:
                payload = flash_attn_params((ho, 0), (hq, 0), (hk, 0), (hv, 0), (hm, 0), qo_len, kv_len, n_heads,
                                            n_kv_heads, head_dim, causal=causal)
                ret = self.execute(HTP_OPS_FLASH_ATTN_F16, payload)
            else:
                assert not causal, "the reference op has no causal flag; pass a mask"
                payload = flash_attn_params((ho, 0), (hq, 0), (hk, 0), (hv, 0), (hm, 0), qo_len, kv_len, n_heads,
                                            n_kv_heads, head_dim)
                ret = self.execute(HTP_OPS_FLASH_ATTN_QO_F32_KV_F16, payload)
            self._check(ret)
            self.synchronize()
            return self.read(ho, q.dtype, q.size).reshape(q.shape)
        finally:
            for h in (hq, hk, hv, ho):
                self.release(h)
            if hm > 0:
                self.release(hm)
