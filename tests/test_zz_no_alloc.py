"""GPU: the entry point that allocates nothing (htpops_flash_attn_noalloc_ptr, partials in a static device array)
against the ordinary entry point (htpops_flash_attn_ptr, partials in the context's workspace), through the C ABI on raw
device pointers: bit-identical outputs, on two calls in a row with the second one smaller (the array keeps the first
call's contents), then each against the oracle; sizes beyond the static array are refused."""
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
