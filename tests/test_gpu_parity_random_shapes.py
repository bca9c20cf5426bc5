"""Seeded random shapes through the C ABI against the oracle: the parametrized parity tests sit on the shapes of the
benchmark's configurations and on both sides of every kernel switch that was known when they were written; these draw
row counts, row lengths, output widths, head counts and key counts at random so that a switch nobody listed is hit too.
Same bars as there: 1e-5 of the sum of |block terms| for the matmuls (fp32 summation order differs from the oracle's),
2e-3 absolute for attention; a repeat of a matmul must be bit-identical."""
import numpy as np
import pytest

from pyhtpops import api
from pyhtpops import workloads as wl

pytestmark = pytest.mark.gpu

MATMUL_RTOL = 1e-5
ATTN_ATOL = 2e-3


@pytest.fixture(scope="module")
def ctx():
    c = api.Context(device=0)
    yield c
    c.close()


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_random_matmul_shapes(ctx, oracle, seed):
    rng = np.random.default_rng(9000 + seed)
    for _ in range(40):
        wt = int(rng.choice([wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0]))
        m = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 17, 24, 32, 33, 48, 64, 100, 128, 200, 257, 512]))
        k = [32 * int(rng.integers(1, 40)), 256 * int(rng.integers(1, 48)), 64 * int(rng.integers(1, 192)),
             int(rng.choice([4096, 11008, 1536, 8960, 2048, 8192, 12288, 4096 + 32]))][int(rng.integers(0, 4))]
        n = [int(rng.integers(1, 70)), 16 * int(rng.integers(1, 300)), int(rng.integers(1, 5000)),
             64 * int(rng.integers(1, 180))][int(rng.integers(0, 4))]
        while m * k * n > 2e8:
            n = max(1, n // 2)
        w = wl.make_weights(rng, n, k, wt)
        a = oracle.quantize_q8_0(wl.make_activations(rng, m, k))
        print("mat_mul case m=%d k=%d n=%d wt=%d" % (m, k, n, wt), flush=True)
        got = ctx.run_mat_mul(a, w, m, k, n, wt)
        want, mag = oracle.mat_mul_q8_0_act_f64(a, w, m, k, n, wt)
        assert np.all(np.abs(got - want) <= MATMUL_RTOL * mag), (m, k, n, wt, float((np.abs(got - want) / mag).max()))
        assert np.array_equal(ctx.run_mat_mul(a, w, m, k, n, wt), got), (m, k, n, wt)


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_random_attention_shapes(ctx, oracle, seed):
    rng = np.random.default_rng(9100 + seed)
    for _ in range(30):
        d = int(rng.choice([64, 128, 128, 64, 80, 96, 32, 256, 2, 112]))
        nkv = int(rng.choice([1, 2, 3, 4, 8]))
        nh = nkv * int(rng.choice([1, 2, 3, 4, 6, 8]))
        if rng.integers(0, 2) == 0:  # one token against a cache
            qo = 1
            kv = int(rng.choice([1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 500, 1000, 2047, 2048, 2049, 4096, 5000, 8191]))
            if rng.integers(0, 2):
                kv = int(rng.integers(1, 6000))
        else:
            qo = int(rng.integers(1, 200))
            kv = qo + int(rng.integers(0, 400)) if rng.integers(0, 2) else int(rng.integers(1, 600))
        while qo * kv * nh * d > 2e8:
            kv = max(1, kv // 2)
        q, k, v = wl.make_attention_inputs(rng, qo, kv, nh, nkv, d)
        f32 = rng.integers(0, 2) == 0
        mode = int(rng.integers(0, 3))  # no mask | additive causal mask | the causal flag of the fp16 op
        if (f32 and mode == 2) or (mode != 0 and kv < qo):
            mode = 0 if kv < qo else 1
        mask = wl.make_causal_mask(qo, kv) if mode == 1 else None
        print("attention case qo=%d kv=%d heads=%d/%d d=%d f32=%d mode=%d" % (qo, kv, nh, nkv, d, f32, mode), flush=True)
        if f32:
            q32 = q.astype(np.float32)
            got = ctx.run_flash_attn(q32, k, v, mask, nh, nkv, d)
            want = oracle.flash_attn(q32, k, v, mask, nh, nkv, d)
        else:
            got = ctx.run_flash_attn(q, k, v, mask, nh, nkv, d, causal=(mode == 2))
            want = oracle.flash_attn(q, k, v, mask, nh, nkv, d, mode == 2)
        err = float(np.abs(got.astype(np.float32) - want.astype(np.float32)).max())
        assert err <= ATTN_ATOL, (qo, kv, nh, nkv, d, f32, mode, err)
