"""GPU: the entry point that allocates nothing (htpops_flash_attn_noalloc_ptr, partials in a static device array)
against the ordinary entry point (htpops_flash_attn_ptr, partials in the context's workspace), through the C ABI on raw
device pointers: bit-identical outputs, on two calls in a row with the second one smaller (the array keeps the first
call's contents), then each against the oracle; sizes beyond the static array are refused; the context's workspace and
converted-copy accounting do not move across a call (nothing was allocated or freed through the context); two contexts
cannot use the shared array at the same time."""
import ctypes

import numpy as np
import pytest

from pyhtpops import api
from pyhtpops import workloads as wl

pytestmark = pytest.mark.gpu

ATTN_ATOL = 2e-3


def vp(x):
    return ctypes.c_void_p(x)


def run_both(ctx, oracle, rng, qo, kv, nh, nkv, hd, qo_f32, with_mask):
    q, k, v = wl.make_attention_inputs(rng, qo, kv, nh, nkv, hd)
    if qo_f32:
        q = q.astype(np.float32)
    mask = None
    if with_mask:
        ld = (kv + 63) // 64 * 64
        mask = np.where(rng.random((qo, ld)) < 0.2, -np.inf, 0.0).astype(np.float16)
        mask[:, 0] = 0
    hq, hk, hv = ctx.upload(q), ctx.upload(k), ctx.upload(v)
    hm = ctx.upload(mask) if mask is not None else None
    outs = []
    handles = [hq, hk, hv] + ([hm] if hm else [])
    try:
        for fn in (ctx.lib.htpops_flash_attn_ptr, ctx.lib.htpops_flash_attn_noalloc_ptr):
            ho = ctx.alloc(q.nbytes)
            handles.append(ho)
            ctx.write(ho, np.full(q.nbytes, 0xA5, np.uint8))
            print("attention %s qo=%d kv=%d heads=%d/%d D=%d f32=%d mask=%d" % (
                "noalloc" if fn is ctx.lib.htpops_flash_attn_noalloc_ptr else "ordinary", qo, kv, nh, nkv, hd, qo_f32, with_mask), flush=True)
            ret = fn(ctx._ctx, vp(ctx.device_ptr(ho)), vp(ctx.device_ptr(hq)), vp(ctx.device_ptr(hk)), vp(ctx.device_ptr(hv)),
                     vp(ctx.device_ptr(hm)) if hm else None, qo, kv, nh, nkv, hd, int(qo_f32), 0 if with_mask else 1)
            assert ret == 0, ctx.last_error()
            ctx.synchronize()
            outs.append(ctx.read(ho, q.dtype, q.size).reshape(q.shape))
    finally:
        for h in handles:
            ctx.release(h)
    assert np.array_equal(outs[0].view(np.uint8), outs[1].view(np.uint8)), "the two entry points differ"
    ref = oracle.flash_attn(q, k, v, mask, nh, nkv, hd, not with_mask)
    assert np.abs(outs[1].astype(np.float32) - ref.astype(np.float32)).max() <= ATTN_ATOL


def test_no_alloc_attention_equals_the_ordinary_entry_point(oracle):
    rng = wl.rng_for(90, 0)
    with api.Context(device=0) as ctx:
        # decode (the path that uses the scratch): a long context first, then a shorter one, then other shapes
        run_both(ctx, oracle, rng, 1, 4096, 32, 8, 128, False, False)
        run_both(ctx, oracle, rng, 1, 300, 32, 8, 128, False, False)
        run_both(ctx, oracle, rng, 1, 1000, 8, 2, 64, True, True)
        run_both(ctx, oracle, rng, 1, 70, 4, 4, 128, True, False)
        # prefill and odd head dims take no scratch but go through the same entry
        run_both(ctx, oracle, rng, 48, 200, 8, 2, 128, False, False)
        run_both(ctx, oracle, rng, 3, 133, 4, 2, 80, True, True)


def test_no_alloc_attention_refuses_what_does_not_fit(oracle):
    with api.Context(device=0) as ctx:
        h = ctx.alloc(1 << 16)
        p = vp(ctx.device_ptr(h))
        # 32 heads x ceil(40000 / 64) splits x 130 floats = 10.4 MB > 8 MiB: refused before anything is launched
        ret = ctx.lib.htpops_flash_attn_noalloc_ptr(ctx._ctx, p, p, p, p, None, 1, 40000, 32, 8, 128, 0, 1)
        assert ret == api.HTPOPS_ERR_REJECTED and "static scratch" in ctx.last_error()
        # the same rejections as the ordinary entry
        assert ctx.lib.htpops_flash_attn_noalloc_ptr(ctx._ctx, p, p, p, p, None, 1, 64, 6, 4, 128, 0, 1) == api.HTPOPS_ERR_REJECTED
        assert ctx.lib.htpops_flash_attn_noalloc_ptr(ctx._ctx, None, p, p, p, None, 1, 64, 8, 4, 128, 0, 1) == api.HTPOPS_ERR_REJECTED
        ctx.release(h)
    with api.Context(device=None) as host_only:
        x = np.zeros(16, np.uint8)
        h = host_only.alloc(4096)
        p = vp(host_only.device_ptr(h))
        assert host_only.lib.htpops_flash_attn_noalloc_ptr(host_only._ctx, p, p, p, p, None, 1, 16, 1, 1, 128, 0, 1) == api.HTPOPS_ERR_NO_DEVICE


def test_no_alloc_attention_leaves_the_contexts_memory_alone(oracle):
    # The property the entry point exists for. The context's own allocations are its workspace (grown on demand by
    # the ordinary entry) and its converted weight copies: neither may move across a no-alloc call, not even for a
    # context length far beyond anything the ordinary entry has sized the workspace for.
    rng = wl.rng_for(91, 0)
    nh, nkv, hd = 32, 8, 128
    with api.Context(device=0) as ctx:
        # grow the workspace with an ordinary decode call, and hold a converted weight copy (m = 8 repacks Q4_0 weights)
        q, k, v = wl.make_attention_inputs(rng, 1, 512, nh, nkv, hd)
        ctx.run_flash_attn(q, k, v, None, nh, nkv, hd, causal=True)
        w = wl.make_q4_0_weights(rng, 64, 512)
        a = oracle.quantize_q8_0(wl.make_activations(rng, 8, 512))
        hw, ha, hout = ctx.upload(w), ctx.upload(a), ctx.alloc(8 * 64 * 4)
        assert ctx.execute(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0, api.mat_mul_params((hout, 0), (ha, 0), (hw, 0), 8, 512, 64)) == 0
        ctx.synchronize()
        ws_before, conv_before = ctx.workspace_bytes(), ctx.converted_bytes()
        assert ws_before > 0 and conv_before > 0
        kv = 16384  # partials: 32 heads x 256 splits x 130 floats = 4.3 MB, four times the workspace so far
        assert nh * ((kv + 63) // 64) * (hd + 2) * 4 > ws_before
        q, k, v = wl.make_attention_inputs(rng, 1, kv, nh, nkv, hd)
        hq, hk, hv, ho = ctx.upload(q), ctx.upload(k), ctx.upload(v), ctx.alloc(q.nbytes)
        try:
            print("no-alloc decode kv=%d on a context with %d bytes of workspace" % (kv, ws_before), flush=True)
            ret = ctx.lib.htpops_flash_attn_noalloc_ptr(ctx._ctx, vp(ctx.device_ptr(ho)), vp(ctx.device_ptr(hq)),
                                                        vp(ctx.device_ptr(hk)), vp(ctx.device_ptr(hv)), None, 1, kv, nh, nkv,
                                                        hd, 0, 1)
            assert ret == 0, ctx.last_error()
            assert ctx.workspace_bytes() == ws_before and ctx.converted_bytes() == conv_before
            ctx.synchronize()
            got = ctx.read(ho, np.float16, q.size).reshape(q.shape)
            ref = oracle.flash_attn(q, k, v, None, nh, nkv, hd, True)
            assert np.abs(got.astype(np.float32) - ref.astype(np.float32)).max() <= ATTN_ATOL
            # an output over cached weights would force the copy's release (a hipFree): refused, copy kept
            ret = ctx.lib.htpops_flash_attn_noalloc_ptr(ctx._ctx, vp(ctx.device_ptr(hw)), vp(ctx.device_ptr(hq)),
                                                        vp(ctx.device_ptr(hk)), vp(ctx.device_ptr(hv)), None, 1, 64, 2, 1,
                                                        128, 0, 1)
            assert ret == api.HTPOPS_ERR_REJECTED and ctx.converted_bytes() == conv_before
        finally:
            for h in (hq, hk, hv, ho, hw, ha, hout):
                ctx.release(h)


def test_no_alloc_attention_is_one_context_at_a_time_per_gpu(oracle):
    # All contexts of a GPU share the static array. A second context that asks for it while the first one's call may
    # still be running is told so (HTPOPS_ERR_BUSY) instead of racing; once the first has waited for its stream the
    # second goes ahead, and gets the right answer.
    rng = wl.rng_for(92, 0)
    nh, nkv, hd, kv = 8, 2, 128, 2000
    q, k, v = wl.make_attention_inputs(rng, 1, kv, nh, nkv, hd)
    ref = oracle.flash_attn(q, k, v, None, nh, nkv, hd, True)
    with api.Context(device=0) as first, api.Context(device=0) as second:
        def call(ctx):
            hs = [ctx.upload(q), ctx.upload(k), ctx.upload(v), ctx.alloc(q.nbytes)]
            ret = ctx.lib.htpops_flash_attn_noalloc_ptr(ctx._ctx, vp(ctx.device_ptr(hs[3])), vp(ctx.device_ptr(hs[0])),
                                                        vp(ctx.device_ptr(hs[1])), vp(ctx.device_ptr(hs[2])), None, 1, kv, nh,
                                                        nkv, hd, 0, 1)
            return ret, hs
        ret1, h1 = call(first)
        assert ret1 == 0, first.last_error()
        ret2, h2 = call(second)
        assert ret2 == api.HTPOPS_ERR_BUSY and "another context" in second.last_error()
        first.synchronize()
        ret2 = second.lib.htpops_flash_attn_noalloc_ptr(second._ctx, vp(second.device_ptr(h2[3])), vp(second.device_ptr(h2[0])),
                                                        vp(second.device_ptr(h2[1])), vp(second.device_ptr(h2[2])), None, 1, kv,
                                                        nh, nkv, hd, 0, 1)
        assert ret2 == 0, second.last_error()
        second.synchronize()
        for ctx, hs in ((first, h1), (second, h2)):
            got = ctx.read(hs[3], np.float16, q.size).reshape(q.shape)
            assert np.abs(got.astype(np.float32) - ref.astype(np.float32)).max() <= ATTN_ATOL
            for h in hs:
                ctx.release(h)
