"""CPU-only checks of the boundary: struct layouts, exported symbols, buffer registry, request validation,
message framing and the mailbox handshake. No kernel runs here (contexts are created without a device)."""
import ctypes
import os
import re
import struct
import subprocess
import threading
import time

import numpy as np
import pytest

from pyhtpops import api

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(api.LIB_PATH):
        api.build_library()
    return api.load_library()


@pytest.fixture()
def ctx(lib):
    c = api.Context(device=None, lib=lib)
    yield c
    c.close()


def test_abi_header_compiles_as_c_and_cxx_with_the_reference_sizes(tmp_path):
    src = tmp_path / "probe.c"
    src.write_text('#include "htpops.h"\n#include "htpops_bench.h"\nint main(void){return 0;}\n')
    inc = os.path.join(ROOT, "include")
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-I", inc, "-c", str(src), "-o", str(tmp_path / "c.o")], check=True)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-I", inc, "-x", "c++", "-c", str(src), "-o", str(tmp_path / "cc.o")], check=True)


def test_library_exports_every_symbol_the_header_declares(lib):
    header = "".join(open(os.path.join(ROOT, "include", h)).read() for h in ("htpops.h", "htpops_bench.h"))
    declared = sorted(set(re.findall(r"\b(htpops_[a-z0-9_]+)\s*\(", header)))
    assert declared == sorted(api.EXPORTED_SYMBOLS)
    for name in declared:
        assert hasattr(lib, name), name


def test_python_wire_builders_match_the_packed_struct_sizes():
    assert len(api.rms_norm_params((1, 0), (2, 0), 3, 4)) == 24
    assert len(api.mat_mul_params((1, 0), (2, 0), (3, 0), 1, 2, 3)) == 36
    assert len(api.flash_attn_params((1, 0), (2, 0), (3, 0), (4, 0), (5, 0), 1, 2, 3, 4, 5)) == 60
    assert len(api.flash_attn_params((1, 0), (2, 0), (3, 0), (4, 0), (5, 0), 1, 2, 3, 4, 5, causal=1)) == 64
    assert len(api.rms_norm_ex_params((1, 0), (2, 0), (3, 0), 1, 2, 1e-6)) == 36
    # a one-request RMSNorm message is 16 + 2*4 + 8 + 4 + 24 = 60 bytes (reference: src/host/test.c:166-194)
    msg = api.build_message([(api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(0, api.rms_norm_params((7, 0), (9, 0), 60000, 1)))])
    assert len(msg) == 60
    assert struct.unpack_from("<QIi2i", msg, 0) == (0, 0, 1, 24, 60)
    assert struct.unpack_from("<iiI", msg, 24) == (0, api.REQUEST_TYPE_OP_COMPUTE, api.HTP_OPS_RMS_NORM_F32)
    assert struct.unpack_from("<iiiiii", msg, 36) == (7, 0, 9, 0, 60000, 1)


def test_buffer_registry(ctx):
    h1, h2 = ctx.alloc(1000), ctx.alloc(64)
    assert h1 > 0 and h2 > 0 and h1 != h2
    assert ctx.size(h1) == 1000 and ctx.device_ptr(h1)
    data = np.arange(250, dtype=np.int32)
    ctx.write(h1, data)
    assert np.array_equal(ctx.read(h1, np.int32, 250), data)
    assert np.array_equal(ctx.read(h1, np.int32, 10, offset=40), data[10:20])
    with pytest.raises(api.HtpOpsError):
        ctx.write(h2, data)  # does not fit
    with pytest.raises(api.HtpOpsError):
        ctx.read(h1, np.int32, 2, offset=996)
    assert ctx.release(h1) == 0 and ctx.size(h1) == 0 and not ctx.device_ptr(h1)
    assert ctx.release(h1) == 0 and ctx.release(12345) == 0  # unknown handles are ignored, as in the reference
    h3 = ctx.alloc(8)
    assert h3 == h1  # slots are reused
    with pytest.raises(api.HtpOpsError):
        ctx.alloc(0)


def test_requests_are_rejected_like_the_reference_rejects_them(ctx):
    src, dst = ctx.alloc(4096 * 4), ctx.alloc(4096 * 4)
    R = api.HTPOPS_ERR_REJECTED
    # zero sizes (rms_norm.c:69-71), unknown handle -> null pointer (op_executor.cc:58-60), range overflow
    assert ctx.execute(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((dst, 0), (src, 0), 0, 1)) == R
    assert ctx.execute(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((dst, 0), (src, 0), 4096, 0)) == R
    assert ctx.execute(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((999, 0), (src, 0), 4096, 1)) == R
    assert ctx.execute(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((dst, 0), (src, 0), 4097, 1)) == R
    assert ctx.execute(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((dst, 16), (src, 0), 4096, 1)) == R
    assert ctx.execute(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((dst, -4), (src, 0), 16, 1)) == R
    # a well-formed request reaches the device check
    assert ctx.execute(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((dst, 0), (src, 0), 4096, 1)) == api.HTPOPS_ERR_NO_DEVICE
    assert "GPU" in ctx.last_error()
    # matmul preconditions (mat_mul.c:878-887): k % 32, non-zero dims
    w, a, o = ctx.alloc(64 * 2 * 18), ctx.alloc(2 * 34), ctx.alloc(64 * 4)
    assert ctx.execute(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0, api.mat_mul_params((o, 0), (a, 0), (w, 0), 1, 48, 64)) == R
    assert ctx.execute(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0, api.mat_mul_params((o, 0), (a, 0), (w, 0), 0, 64, 64)) == R
    assert ctx.execute(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0, api.mat_mul_params((o, 0), (a, 0), (w, 0), 1, 64, 65)) == R  # weight too small
    assert ctx.execute(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0, api.mat_mul_params((o, 0), (a, 0), (w, 0), 1, 64, 64)) == api.HTPOPS_ERR_NO_DEVICE
    # attention: n_heads % n_kv_heads (flash_attn.c:1373-1376)
    q, k = ctx.alloc(8 * 128 * 4), ctx.alloc(64 * 3 * 128 * 2)
    p = api.flash_attn_params((q, 0), (q, 0), (k, 0), (k, 0), (-1, 0), 1, 64, 8, 3, 128)
    assert ctx.execute(api.HTP_OPS_FLASH_ATTN_QO_F32_KV_F16, p) == R
    # unknown op: reported (the reference returns 0 silently, op_executor.cc:200-203)
    assert ctx.execute(77, b"\0" * 64) == R


def test_process_message_walks_requests_and_completes_the_handshake(ctx):
    src, dst = ctx.alloc(256), ctx.alloc(256)
    spare = ctx.alloc(16)
    good = api.op_compute_request(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((dst, 0), (src, 0), 64, 1))
    bad = api.op_compute_request(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((dst, 0), (src, 0), 0, 1))
    unmap = struct.pack("<ii2i", 2, 0, spare, 4242)
    msg = api.build_message([(api.REQUEST_TYPE_OP_COMPUTE, good), (api.REQUEST_TYPE_OP_COMPUTE, bad),
                             (api.REQUEST_TYPE_RPCMEM_MAP, unmap), (api.REQUEST_TYPE_NO_OP, b"")])
    msg[0] = 1  # producer's go byte
    for i, off in enumerate(struct.unpack_from("<4i", msg, 16)):
        struct.pack_into("<i", msg, off, 1000 + i)  # poison the per-request states
    assert ctx.process_message(msg) == 0
    assert api.message_request_states(msg) == [api.HTPOPS_ERR_NO_DEVICE, api.HTPOPS_ERR_REJECTED, 0, 1003]
    assert msg[0] == 1 and msg[1] == 1 and bytes(msg[2:8]) == b"\0" * 6  # state.d = v0 | 1 << 8 (commu.c:125)
    assert ctx.size(spare) == 0  # n_puts released the handle (commu.c:104-108)


def test_process_message_rejects_malformed_framing(ctx):
    body = api.op_compute_request(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((1, 0), (2, 0), 64, 1))
    msg = api.build_message([(api.REQUEST_TYPE_OP_COMPUTE, body)])
    broken = bytearray(msg)
    struct.pack_into("<i", broken, 12, 5)  # claims more requests than the buffer holds
    assert ctx.process_message(broken) == api.HTPOPS_ERR_REJECTED
    broken = bytearray(msg)
    struct.pack_into("<i", broken, 16, 4000)  # offset outside the message
    assert ctx.process_message(broken) == api.HTPOPS_ERR_REJECTED
    broken = bytearray(msg)
    struct.pack_into("<i", broken, 12, -1)
    assert ctx.process_message(broken) == api.HTPOPS_ERR_REJECTED
    assert ctx.process_message(bytearray(msg[:12])) == api.HTPOPS_ERR_REJECTED  # not even a header


def test_process_message_rejects_requests_shorter_than_their_parameters(ctx):
    # The reference casts a request's bytes to its op's parameter struct without looking at the request's size
    # (op_executor.cc:52-204); here a compute request that ends before its op's parameters do is refused with its own
    # state, the requests around it run, and nothing behind the request is read (for the last request that would be
    # memory behind the message).
    src, dst = ctx.alloc(256), ctx.alloc(256)
    good = api.op_compute_request(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((dst, 0), (src, 0), 64, 1))
    bodies = {
        api.HTP_OPS_RMS_NORM_F32: good,
        api.HTP_OPS_MAT_MUL_Q4_0_Q8_0: api.op_compute_request(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0, api.mat_mul_params((dst, 0), (src, 0), (src, 0), 1, 32, 1)),
        api.HTP_OPS_MAT_MUL_PERMUTED_W16A32: api.op_compute_request(api.HTP_OPS_MAT_MUL_PERMUTED_W16A32, api.mat_mul_params((dst, 0), (src, 0), (src, 0), 1, 32, 32)),
        api.HTP_OPS_FLASH_ATTN_QO_F32_KV_F16: api.op_compute_request(api.HTP_OPS_FLASH_ATTN_QO_F32_KV_F16, b"\0" * 60),
        api.HTP_OPS_FLASH_ATTN_F16: api.op_compute_request(api.HTP_OPS_FLASH_ATTN_F16, b"\0" * 64),
        api.HTP_OPS_RMS_NORM_QUANTIZE_Q8_0: api.op_compute_request(api.HTP_OPS_RMS_NORM_QUANTIZE_Q8_0, b"\0" * 36),
    }
    for op, body in bodies.items():
        for cut in (1, 4, len(body) - 4):  # one byte short, one field short, the op word alone
            msg = api.build_message([(api.REQUEST_TYPE_OP_COMPUTE, good), (api.REQUEST_TYPE_OP_COMPUTE, body[:len(body) - cut])])
            assert ctx.process_message(msg) == 0
            states = api.message_request_states(msg)
            assert states == [api.HTPOPS_ERR_NO_DEVICE, api.HTPOPS_ERR_REJECTED], (op, cut, states)
            assert "shorter than the parameters" in ctx.last_error()
        whole = api.build_message([(api.REQUEST_TYPE_OP_COMPUTE, body)])
        assert ctx.process_message(whole) == 0
        assert "shorter than the parameters" not in ctx.last_error()


def test_channel_poller_follows_the_state_byte_protocol(ctx, lib):
    size = 4096
    raw = ctypes.create_string_buffer(size + 64)
    base = (ctypes.addressof(raw) + 63) & ~63
    assert lib.htpops_create_channel(ctx._ctx, base, size) == 0
    assert lib.htpops_create_channel(ctx._ctx, base, size) == api.HTPOPS_ERR_BUSY
    view = (ctypes.c_ubyte * size).from_address(base)
    try:
        for round_ in range(3):
            body = api.op_compute_request(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((999, 0), (998, 0), 64, 1))
            msg = api.build_message([(api.REQUEST_TYPE_OP_COMPUTE, body)])
            # as the reference host does: state.d = 0, fill the requests, then set the go byte last
            for i in range(8):
                view[i] = 0
            ctypes.memmove(base + 8, bytes(msg[8:]), len(msg) - 8)
            time.sleep(0.01)
            assert view[1] == 0  # nothing happens until v[0] is set
            view[0] = 1
            deadline = time.time() + 5
            while view[1] != 1 and time.time() < deadline:
                time.sleep(0.0005)
            assert view[1] == 1
            state = struct.unpack_from("<i", bytes(view[:len(msg)]), 24)[0]
            assert state == api.HTPOPS_ERR_REJECTED  # unknown handles -> -1
    finally:
        assert lib.htpops_destroy_channel(ctx._ctx) == 0
    assert lib.htpops_destroy_channel(ctx._ctx) == 0


def test_device_context_fails_loudly_without_a_gpu(lib):
    # on a machine without a GPU the backend must refuse to initialise instead of falling back
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(api.HtpOpsError) as e:
        api.Context(device=0, lib=lib)
    assert e.value.code == api.HTPOPS_ERR_NO_DEVICE
