"""GPU parity of the reference's own matmul ops (ids 1-4: fp16 tiles and tile-permuted Q4_0 / Q8_0 / IQ4_NL
super-blocks) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from pyhtpops import api
from pyhtpops import workloads as wl

pytestmark = pytest.mark.gpu

@pytest.fixture(scope="module")
def ctx():
    c = api.Context(device=0)
    yield c
    c.close()


OPS = {1: api.HTP_OPS_MAT_MUL_PERMUTED_W16A32, 2: api.HTP_OPS_MAT_MUL_PERMUTED_W4D16A32,
       3: api.HTP_OPS_MAT_MUL_PERMUTED_W8D16A32, 4: api.HTP_OPS_MAT_MUL_PERMUTED_W4D16A32_IQ4_NL}


def make_weights(rng, n, k, kind):
    """raw bytes in the reference's layout and the same weights as float32 W[k][n]"""
    if kind == 1:
        w = (rng.standard_normal((k, n)) * 0.05).astype(np.float16)
        return wl.w16_tile_layout(w), w.astype(np.float32)
    raw = wl.make_permuted_weights(rng, n, k, kind)
    return raw, wl.permuted_to_kn(raw, n, k, kind)


def check(ctx, oracle, kind, m, k, n, seed):
    rng = wl.rng_for(80 + kind, seed)
    x = wl.make_activations(rng, m, k)
    raw, w = make_weights(rng, n, k, kind)
    print("permuted matmul kind=%d m=%d k=%d n=%d" % (kind, m, k, n), flush=True)
    got = ctx.run_mat_mul_permuted(x, raw, m, k, n, OPS[kind])
    want, f64 = oracle.mat_mul_permuted(x, raw, m, k, n, kind, want_f64=True)
    # Both sides round a sum of exact fp16 x fp16 products to fp16; the GPU accumulates in fp32 (matrix core), the
    # oracle in double. Tolerance: the fp32 accumulation error, 1e-6 of sum |terms|, plus one fp16 spacing for sums
    # that land on different sides of a rounding boundary.
    mag = np.abs(x.astype(np.float16).astype(np.float64)) @ np.abs(w.astype(np.float64))
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0 ** -14))) - 10)   # spacing of fp16 at |want|
    assert np.all(np.abs(got - f64) <= 1e-6 * mag + ulp), float((np.abs(got - f64) / (1e-6 * mag + ulp)).max())
    assert np.all(np.abs(got - want) <= 1e-6 * mag + ulp)
    assert np.mean(got == want) > 0.9
    # every output is a value fp16 can hold (the reference stores fp16 results)
    assert np.array_equal(got, got.astype(np.float16).astype(np.float32))


@pytest.mark.parametrize("kind", [1, 2, 3, 4])
@pytest.mark.parametrize("m,k,n", [(1, 4096, 512), (5, 96, 64), (32, 1024, 256), (33, 256, 96), (100, 512, 160),
                                   (300, 2048, 320), (8, 32, 32)])
def test_permuted_matmul(ctx, oracle, kind, m, k, n):
    check(ctx, oracle, kind, m, k, n, m + k + n)


def test_fp16_tile_layout_is_the_reference_tests_layout(ctx):
    # the reference's own host test (src/host/test.c:300-327) fills tiles with this index formula and compares with
    # a plain triple loop: one weight set to 1 selects one activation column
    m, k, n = 2, 64, 64
    x = np.arange(m * k, dtype=np.float32).reshape(m, k) / 64.0
    for kk, nn in [(0, 0), (1, 0), (0, 1), (33, 2), (63, 63), (31, 32)]:
        tiles = np.zeros(k * n, np.float16)
        k0, k1, n0, n1 = kk // 32, kk % 32, nn // 32, nn % 32
        tiles[(n0 * (k // 32) + k0) * 1024 + (k1 & ~1) * 32 + n1 * 2 + (k1 & 1)] = 1.0
        got = ctx.run_mat_mul_permuted(x, tiles, m, k, n, OPS[1])
        want = np.zeros((m, n), np.float32)
        want[:, nn] = x[:, kk].astype(np.float16).astype(np.float32)
        assert np.array_equal(got, want), (kk, nn)


def test_converted_weights_are_cached_and_dropped_on_write(ctx, oracle):
    rng = wl.rng_for(85, 0)
    m, k, n = 4, 128, 64
    x = wl.make_activations(rng, m, k)
    raw_a, raw_b = wl.make_permuted_weights(rng, n, k, 2), wl.make_permuted_weights(rng, n, k, 2)
    ha, hw, ho = ctx.upload(x), ctx.upload(raw_a), ctx.alloc(m * n * 4)
    try:
        payload = api.mat_mul_params((ho, 0), (ha, 0), (hw, 0), m, k, n)
        for raw in (raw_a, raw_a, raw_b, raw_a):
            ctx.write(hw, raw)
            for _ in range(2):  # second call reuses the converted weights
                assert ctx.execute(OPS[2], payload) == 0
            ctx.synchronize()
            got = ctx.read(ho, np.float32, m * n).reshape(m, n)
            want = oracle.mat_mul_permuted(x, raw, m, k, n, 2)
            assert np.mean(got == want) > 0.98 and np.allclose(got, want, rtol=2e-3, atol=1e-4)
    finally:
        ctx.release(ha), ctx.release(hw), ctx.release(ho)


@pytest.mark.parametrize("bad", ["k", "n", "null"])
def test_permuted_matmul_rejects_what_the_reference_rejects(ctx, bad):
    # reference: src/dsp/ops/mat_mul.c:760-769, :878-892 (k % 32, n % 32, null buffers -> -1)
    m, k, n = 1, 64, 64
    if bad == "k":
        k = 48
    if bad == "n":
        n = 40
    ha, hw, ho = ctx.alloc(m * 64 * 4), ctx.alloc(64 * 64 * 2), ctx.alloc(m * 64 * 4)
    try:
        w = (hw, 0) if bad != "null" else (12345, 0)
        assert ctx.execute(OPS[1], api.mat_mul_params((ho, 0), (ha, 0), w, m, k, n)) == -1
    finally:
        ctx.release(ha), ctx.release(hw), ctx.release(ho)


def test_weights_in_caller_owned_memory_are_converted_on_every_call(oracle):
    # Memory the context did not allocate can change without the context seeing it: a second context owns the buffer
    # here and rewrites it, the first one only has it registered. No converted copy may survive between calls.
    rng = wl.rng_for(86, 0)
    m, k, n = 4, 128, 64
    x = wl.make_activations(rng, m, k)
    raws = [wl.make_permuted_weights(rng, n, k, 2) for _ in range(3)]
    with api.Context(device=0) as owner, api.Context(device=0) as user:
        hw_owner = owner.upload(raws[0])
        hw = user.register(owner.device_ptr(hw_owner), raws[0].nbytes)
        ha, ho = user.upload(x), user.alloc(m * n * 4)
        payload = api.mat_mul_params((ho, 0), (ha, 0), (hw, 0), m, k, n)
        for raw in (raws[0], raws[1], raws[2], raws[0]):
            owner.write(hw_owner, raw)
            for _ in range(2):
                assert user.execute(OPS[2], payload) == 0
                user.synchronize()
                got = user.read(ho, np.float32, m * n).reshape(m, n)
                want = oracle.mat_mul_permuted(x, raw, m, k, n, 2)
                assert np.mean(got == want) > 0.98 and np.allclose(got, want, rtol=2e-3, atol=1e-4)
