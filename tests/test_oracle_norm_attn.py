"""Pins the oracle's RMSNorm, attention and fp16-tile matmul against closed forms, float64 numpy,
the fixtures written from the reference's own scalar attention routine, and (when built) that routine itself."""
import glob
import os

import numpy as np
import pytest

from pyhtpops import workloads as wl


# ---------------------------------------------------------------------------------------- rmsnorm

def test_rms_norm_closed_forms(oracle):
    for c in (3.0, -0.25, 100.0):
        x = np.full(4096, c, np.float32)
        y = oracle.rms_norm(x, eps=1e-6)[0]
        assert np.allclose(y, c / np.sqrt(c * c + 1e-6), rtol=1e-6)
    x = np.zeros(64, np.float32)
    x[5] = 8.0  # one-hot: mean = 1, y = 8 / sqrt(1 + eps)
    y = oracle.rms_norm(x, eps=1e-5)[0]
    assert y[5] == np.float32(8.0) * (np.float32(1.0) / np.sqrt(np.float32(1.0) + np.float32(1e-5))) and not y[:5].any()
    assert not oracle.rms_norm(np.zeros(32, np.float32))[0].any()


def test_rms_norm_matches_float64_with_weight_and_eps(oracle):
    rng = wl.rng_for(95, 1)
    for ne0, ne1 in ((4096, 1), (1536, 128), (60000, 1), (33, 3)):
        x = (rng.uniform(-20, 20, (ne1, ne0))).astype(np.float32)
        w = (1 + 0.1 * rng.standard_normal(ne0)).astype(np.float32)
        for eps, ww in ((1e-5, None), (1e-6, w)):
            y = oracle.rms_norm(x, ww, eps)
            x64 = x.astype(np.float64)
            want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + eps) * (1 if ww is None else ww)
            assert np.abs(y - want).max() <= 1e-5  # the reference's own tolerance (src/host/test.c:116-118)


def test_rms_norm_is_scale_invariant_for_large_inputs(oracle):
    rng = wl.rng_for(95, 2)
    x = wl.make_activations(rng, 2, 2048)
    assert np.allclose(oracle.rms_norm(x * 64.0, eps=1e-6), oracle.rms_norm(x, eps=1e-6), rtol=0, atol=2e-6)


# -------------------------------------------------------------------------------------- attention

def numpy_attention(q, k, v, mask, causal):
    """softmax(Q K^T / sqrt(D) + mask) V in float64, GQA by integer division of the head index."""
    qo, nh, d = q.shape
    kv, nkv, _ = k.shape
    g = nh // nkv
    out = np.zeros((qo, nh, d))
    q64, k64, v64 = q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)
    for h in range(nh):
        s = q64[:, h, :] @ k64[:, h // g, :].T / np.sqrt(d)
        if mask is not None:
            s = s + mask[:qo, :kv].astype(np.float64)
        if causal:
            i, j = np.arange(qo)[:, None], np.arange(kv)[None, :]
            s = np.where(j <= i + (kv - qo), s, -np.inf)
        s = s - s.max(axis=1, keepdims=True)
        p = np.exp(s)
        out[:, h, :] = (p / p.sum(axis=1, keepdims=True)) @ v64[:, h // g, :]
    return out


@pytest.mark.parametrize("qo,kv,nh,nkv,d", [(5, 70, 4, 2, 64), (1, 300, 8, 2, 128), (33, 517, 4, 4, 128),
                                             (64, 64, 2, 1, 64)])
def test_attention_matches_float64_softmax(oracle, qo, kv, nh, nkv, d):
    rng = wl.rng_for(94, qo)
    q, k, v = wl.make_attention_inputs(rng, qo, kv, nh, nkv, d)
    mask = wl.make_causal_mask(qo, kv)
    for m, causal in ((None, False), (mask, False), (None, True)):
        got = oracle.flash_attn(q.astype(np.float32), k, v, m, nh, nkv, d, causal)
        want = numpy_attention(q, k, v, m, causal)
        assert np.abs(got - want).max() < 2e-6
    # causal flag == causal mask, bit for bit
    assert np.array_equal(oracle.flash_attn(q.astype(np.float32), k, v, mask, nh, nkv, d, False),
                          oracle.flash_attn(q.astype(np.float32), k, v, None, nh, nkv, d, True))
    # fp16 Q/O variant is the fp32 one rounded once
    got16 = oracle.flash_attn(q, k, v, None, nh, nkv, d, True)
    assert got16.dtype == np.float16
    assert np.array_equal(got16, oracle.flash_attn(q.astype(np.float32), k, v, None, nh, nkv, d, True).astype(np.float16))


def test_attention_invariants(oracle):
    rng = wl.rng_for(94, 100)
    qo, kv, nh, nkv, d = 7, 200, 8, 2, 128
    q, k, v = wl.make_attention_inputs(rng, qo, kv, nh, nkv, d)
    q32 = q.astype(np.float32)
    # rows of softmax sum to one
    ones = np.ones_like(v)
    assert np.allclose(oracle.flash_attn(q32, k, ones, None, nh, nkv, d), 1.0, atol=1e-6)
    # a single key returns its value
    out = oracle.flash_attn(q32, k[:1], v[:1], None, nh, nkv, d)
    assert np.allclose(out, np.repeat(v[:1].astype(np.float32), nh // nkv, axis=1), atol=1e-7)
    # decode equals the last row of causal prefill
    qq, kk, vv = wl.make_attention_inputs(rng, 40, 40, 4, 2, 64)
    full = oracle.flash_attn(qq.astype(np.float32), kk, vv, None, 4, 2, 64, True)
    last = oracle.flash_attn(qq[-1:].astype(np.float32), kk, vv, None, 4, 2, 64, True)
    assert np.allclose(full[-1], last[0], atol=1e-6)
    # masked-out keys do not matter
    mask = wl.make_causal_mask(qo, kv)
    k2, v2 = k.copy(), v.copy()
    k2[kv - 3:], v2[kv - 3:] = k[kv - 3:][::-1], v[kv - 3:][::-1]
    a = oracle.flash_attn(q32[:1], k, v, mask[:1], nh, nkv, d)
    b = oracle.flash_attn(q32[:1], k2, v2, mask[:1], nh, nkv, d)
    assert np.array_equal(a, b)  # query 0 sees keys 0..kv-qo only
    # query heads of one group share K/V: swapping two query heads of a group swaps their outputs
    qs = q32.copy()
    qs[:, [0, 1]] = q32[:, [1, 0]]
    o1 = oracle.flash_attn(q32, k, v, None, nh, nkv, d)
    o2 = oracle.flash_attn(qs, k, v, None, nh, nkv, d)
    assert np.array_equal(o1[:, 0], o2[:, 1]) and np.array_equal(o1[:, 1], o2[:, 0])
    # rejects what the reference rejects (flash_attn.c:1373-1376)
    with pytest.raises(ValueError):
        oracle.flash_attn(q32, k, v, None, 8, 3, d)


def _load_goldens(golden_dir):
    files = sorted(glob.glob(os.path.join(golden_dir, "naive_flash_attn_*.npz")))
    assert len(files) >= 3
    for f in files:
        z = np.load(f)
        qo, kv, nh, nkv, d, masked = [int(t) for t in z["dims"]]
        yield os.path.basename(f), z["q"], z["k"], z["v"], (z["mask"] if masked else None), nh, nkv, d, z["out"]


def test_attention_reproduces_reference_routine_fixtures(oracle, golden_dir):
    for name, q, k, v, mask, nh, nkv, d, want in _load_goldens(golden_dir):
        got = oracle.flash_attn(q, k, v, mask, nh, nkv, d)
        # same block sizes, same operation order: agreement is at rounding level of exp2f/sqrtf only
        assert np.abs(got - want).max() <= 1e-6, name


def test_attention_against_reference_routine_when_built(oracle):
    import oracle_py
    try:
        ref = oracle_py.RefNaiveFlashAttn()
    except FileNotFoundError:
        pytest.skip("oracle/_ref not built (no reference checkout on this machine)")
    rng = wl.rng_for(94, 200)
    for qo, kv, nh, nkv, d in ((3, 64, 2, 2, 64), (37, 300, 4, 2, 128), (1, 1000, 8, 8, 128), (65, 257, 2, 1, 96)):
        q, k, v = wl.make_attention_inputs(rng, qo, kv, nh, nkv, d)
        q32 = q.astype(np.float32)
        for mask in (None, wl.make_causal_mask(qo, kv)):
            want = ref(q32, k, v, mask, nh, nkv, d)
            got = oracle.flash_attn(q32, k, v, mask, nh, nkv, d)
            assert np.abs(got - want).max() <= 1e-6


# ------------------------------------------------------------------------------ fp16 tile matmul

def test_w16_tile_layout_and_matmul(oracle):
    # reference: src/host/test.c:307-312
    k, n, m = 64, 96, 3
    for kk, nn in ((0, 0), (1, 0), (2, 0), (0, 1), (31, 31), (32, 0), (0, 32), (63, 95), (33, 40)):
        tile = (nn // 32) * (k // 32) + kk // 32
        want = tile * 1024 + ((kk % 32) & ~1) * 32 + (nn % 32) * 2 + (kk & 1)
        assert oracle.w16_tile_index(kk, nn, k) == want
    idx = np.array([[oracle.w16_tile_index(kk, nn, k) for nn in range(n)] for kk in range(k)])
    assert sorted(idx.ravel().tolist()) == list(range(k * n))  # a permutation
    rng = wl.rng_for(93, 1)
    w = rng.uniform(0, 1, (k, n)).astype(np.float16)
    tiles = np.empty(k * n, np.float16)
    tiles[idx.ravel()] = w.ravel()
    act = rng.uniform(0, 1, (m, k)).astype(np.float32)
    got = oracle.mat_mul_w16a32(act, tiles, m, k, n)
    want = act.astype(np.float64) @ w.astype(np.float64)
    assert np.abs(got - want).max() < 1e-4


def test_threshold_mask_follows_the_dispatched_kernels_rule(oracle):
    # src/dsp/ops/flash_attn.c:452-455: keep iff mask > -16.0 in fp16 (0xcc00); equality, anything below, and NaN
    # (an ordered compare is false) are dropped; 0, positive biases, +inf and -15.99 (rounds to an fp16 above -16) stay
    vals = np.array([0.0, -15.99, -16.0, -16.02, -1e4, -np.inf, 3.0, np.inf, np.nan, -0.0], np.float16)
    got = oracle.threshold_mask(vals)
    want = np.array([0, 0, -np.inf, -np.inf, -np.inf, -np.inf, 0, 0, -np.inf, 0], np.float16)
    assert np.array_equal(got, want)
    assert vals[1] > np.float16(-16) and vals[3] < np.float16(-16)
    # on a 0 / -inf mask the two conventions are the same function
    rng = np.random.default_rng(5)
    q = rng.standard_normal((3, 2, 64)).astype(np.float32)
    k = rng.standard_normal((70, 1, 64)).astype(np.float16)
    v = rng.standard_normal((70, 1, 64)).astype(np.float16)
    mask = np.where(rng.random((3, 128)) < 0.3, -np.inf, 0.0).astype(np.float16)
    mask[:, 0] = 0
    a = oracle.flash_attn(q, k, v, mask, 2, 1, 64)
    b = oracle.flash_attn(q, k, v, oracle.threshold_mask(mask), 2, 1, 64)
    assert np.array_equal(a, b)
    # with finite biases they differ: a bias of -3 lowers a key's weight when added and leaves it alone when it selects
    biased = np.zeros((3, 128), np.float16)
    biased[:, 5] = -3.0
    assert np.abs(oracle.flash_attn(q, k, v, biased, 2, 1, 64) - oracle.flash_attn(q, k, v, oracle.threshold_mask(biased), 2, 1, 64)).max() > 1e-3
    assert np.array_equal(oracle.flash_attn(q, k, v, oracle.threshold_mask(biased), 2, 1, 64), oracle.flash_attn(q, k, v, None, 2, 1, 64))
