"""GPU parity of the attention op against the oracle (2e-3 absolute, the bar for fp16 attention), the fixtures
written from the reference's scalar routine, and size-independent invariants at the benchmark's full sizes."""
import glob
import os

import numpy as np
import pytest

from pyhtpops import api
from pyhtpops import workloads as wl

pytestmark = pytest.mark.gpu

ATOL = 2e-3


@pytest.fixture(scope="module")
def ctx():
    c = api.Context(device=0)
    yield c
    c.close()


@pytest.fixture(autouse=True)
def default_switches(ctx):
    """Tests that force a kernel or the mask convention do it through htpops_set_option; every test starts from the
    defaults again."""
    yield
    for name, value in api.DEFAULT_OPTIONS.items():
        ctx.set_option(name, value)


CASES = [
    # qo, kv, heads, kv heads, D
    (1, 300, 8, 2, 128), (1, 4096, 32, 8, 128), (1, 70, 4, 4, 64), (1, 129, 16, 1, 128), (1, 1, 4, 2, 64),
    (5, 70, 4, 2, 64), (40, 300, 4, 1, 128), (33, 517, 4, 4, 128), (64, 64, 2, 1, 64), (128, 128, 8, 2, 128),
    (100, 260, 6, 2, 128), (31, 95, 3, 1, 64), (2, 2, 2, 2, 64), (96, 200, 8, 1, 128),
    # decode on both sides of the switch between 64- and 128-key chunks (128 workgroups of 128 keys)
    (1, 64, 8, 8, 128), (1, 65, 8, 2, 64), (1, 2048, 32, 8, 128), (1, 1920, 32, 8, 128), (1, 1900, 16, 4, 64),
    (1, 2100, 16, 16, 64),
    # decode long enough for a workgroup to walk several chunks of keys (about one workgroup per compute unit): ragged
    # last workgroup, odd and even chunk counts, every group width, both head dims
    (1, 4100, 32, 32, 128), (1, 9000, 16, 8, 64), (1, 6000, 12, 12, 128), (1, 20000, 12, 4, 128), (1, 9000, 48, 8, 64),
    (1, 12500, 32, 8, 128),
    # head dims other than 64 and 128 (the reference's flash_attn_sp_hdim.c domain: any even head_dim)
    (1, 300, 8, 2, 80), (7, 133, 4, 2, 96), (33, 70, 6, 3, 40), (1, 1, 2, 1, 2), (20, 517, 4, 1, 256), (3, 64, 2, 2, 112),
    (1, 1000, 4, 4, 192), (65, 65, 2, 1, 30),
]


@pytest.mark.parametrize("qo,kv,nh,nkv,d", CASES)
def test_reference_op_fp32_qo_with_and_without_mask(ctx, oracle, qo, kv, nh, nkv, d):
    rng = wl.rng_for(61, qo * 1000 + kv + nh)
    q, k, v = wl.make_attention_inputs(rng, qo, kv, nh, nkv, d)
    q32 = q.astype(np.float32)
    print("attention case", qo, kv, nh, nkv, d, flush=True)
    for mask in (None, wl.make_causal_mask(qo, kv)):
        got = ctx.run_flash_attn(q32, k, v, mask, nh, nkv, d)
        want = oracle.flash_attn(q32, k, v, mask, nh, nkv, d)
        assert got.dtype == np.float32 and np.abs(got - want).max() <= ATOL


@pytest.mark.parametrize("qo,kv,nh,nkv,d", CASES)
def test_fp16_op_with_causal_flag(ctx, oracle, qo, kv, nh, nkv, d):
    rng = wl.rng_for(62, qo * 1000 + kv + nh)
    q, k, v = wl.make_attention_inputs(rng, qo, kv, nh, nkv, d)
    got = ctx.run_flash_attn(q, k, v, None, nh, nkv, d, causal=True)
    want = oracle.flash_attn(q, k, v, None, nh, nkv, d, True)
    assert got.dtype == np.float16
    assert np.abs(got.astype(np.float32) - want.astype(np.float32)).max() <= ATOL
    # the causal flag and the equivalent additive mask agree
    masked = ctx.run_flash_attn(q, k, v, wl.make_causal_mask(qo, kv), nh, nkv, d, causal=False)
    assert np.abs(got.astype(np.float32) - masked.astype(np.float32)).max() <= 1e-3


@pytest.mark.parametrize("groups", ["1", "2"])
@pytest.mark.parametrize("qo,kv,nh,nkv,d", [(40, 300, 4, 1, 128), (33, 517, 4, 4, 128), (64, 96, 2, 1, 64), (70, 200, 8, 2, 128),
                                            (128, 129, 8, 2, 128)])
def test_prefill_with_one_and_two_key_groups(ctx, oracle, groups, qo, kv, nh, nkv, d):
    # the prefill kernel runs its KV blocks in one or two key groups per workgroup depending on the grid; both must
    # meet the oracle on every shape (odd block counts leave the second group idle in the last iteration)
    ctx.set_option("attn_key_groups", int(groups))
    rng = wl.rng_for(63, qo * 1000 + kv + nh)
    q, k, v = wl.make_attention_inputs(rng, qo, kv, nh, nkv, d)
    for causal, mask in ((True, None), (False, wl.make_causal_mask(qo, kv)), (False, None)):
        got = ctx.run_flash_attn(q, k, v, mask, nh, nkv, d, causal=causal)
        want = oracle.flash_attn(q, k, v, mask, nh, nkv, d, causal)
        assert np.abs(got.astype(np.float32) - want.astype(np.float32)).max() <= ATOL


@pytest.mark.parametrize("kv,nh,nkv,d", [(300, 8, 2, 128), (4096, 32, 8, 128), (70, 4, 4, 64), (1, 4, 2, 64), (9000, 16, 2, 128)])
def test_message_attention_then_quantization_of_its_output(ctx, oracle, kv, nh, nkv, d):
    # One-token attention followed by the Q8_0 quantization of its output row (on its way to the o projection): the
    # launch that finishes the attention writes the Q8_0 row too. The fp32 output is the attention's own, and the row
    # is bit for bit the quantizer's (the oracle's) of that output. A quantization of other rows, a two-token
    # attention and a head dim of the plain kernel keep their own launches.
    rng = wl.rng_for(62, kv * 100 + nh)
    q, k, v = wl.make_attention_inputs(rng, 1, kv, nh, nkv, d)
    q32 = q.astype(np.float32)
    ne0 = nh * d
    hq, hk, hv = ctx.upload(q32), ctx.upload(k), ctx.upload(v)
    ho, hq8 = ctx.alloc(ne0 * 4), ctx.alloc(ne0 // 32 * 34)
    hother = ctx.upload(wl.make_activations(rng, 1, ne0))
    try:
        def op(o, payload):
            return (api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(o, payload))

        attn = op(api.HTP_OPS_FLASH_ATTN_QO_F32_KV_F16,
                  api.flash_attn_params((ho, 0), (hq, 0), (hk, 0), (hv, 0), (-1, 0), 1, kv, nh, nkv, d))
        want_o = ctx.run_flash_attn(q32, k, v, None, nh, nkv, d)
        for src, launches in ((ho, 1), (hother, 2)):
            ctx.write(hq8, np.full(ne0 // 32 * 34, 0xA5, np.uint8))
            ctx.write(ho, np.full(ne0, np.nan, np.float32))
            msg = api.build_message([attn, op(api.HTP_OPS_QUANTIZE_Q8_0, api.rms_norm_params((hq8, 0), (src, 0), ne0, 1))])
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0, 0], ctx.last_error()
            assert ctx.last_message_submissions() == launches
            got_o = ctx.read(ho, np.float32, ne0).reshape(1, nh, d)
            assert np.array_equal(got_o, want_o)
            row = got_o.reshape(1, ne0) if src == ho else ctx.read(hother, np.float32, ne0).reshape(1, ne0)
            assert np.array_equal(ctx.read(hq8, np.uint8, ne0 // 32 * 34), oracle.quantize_q8_0(row)[0])
    finally:
        for h in (hq, hk, hv, ho, hq8, hother):
            ctx.release(h)


def test_fixtures_from_the_reference_routine(ctx, golden_dir):
    files = sorted(glob.glob(os.path.join(golden_dir, "naive_flash_attn_*.npz")))
    assert len(files) >= 3
    for f in files:
        z = np.load(f)
        qo, kv, nh, nkv, d, masked = [int(t) for t in z["dims"]]
        got = ctx.run_flash_attn(z["q"], z["k"], z["v"], z["mask"] if masked else None, nh, nkv, d)
        assert np.abs(got - z["out"]).max() <= ATOL, os.path.basename(f)


def test_additive_mask_with_finite_biases(ctx, oracle):
    # the op follows the scalar routine's additive convention (reference flash_attn.c:1505-1512)
    rng = wl.rng_for(63, 0)
    qo, kv, nh, nkv, d = 37, 130, 4, 2, 128
    q, k, v = wl.make_attention_inputs(rng, qo, kv, nh, nkv, d)
    mask = np.full((qo, 192), -np.inf, np.float16)
    mask[:, :kv] = (rng.standard_normal((qo, kv)) * 2).astype(np.float16)
    q32 = q.astype(np.float32)
    got = ctx.run_flash_attn(q32, k, v, mask, nh, nkv, d)
    assert np.abs(got - oracle.flash_attn(q32, k, v, mask, nh, nkv, d)).max() <= ATOL


def test_full_size_invariants(ctx):
    # benchmark shapes: 32 query heads, 8 KV heads, D = 128; decode kv = 4096, prefill q = kv = 2048 (causal)
    rng = wl.rng_for(3, 0)
    nh, nkv, d = 32, 8, 128
    q, k, v = wl.make_attention_inputs(rng, 2048, 2048, nh, nkv, d)
    print("full-size prefill", flush=True)
    out = ctx.run_flash_attn(q, k, v, None, nh, nkv, d, causal=True).astype(np.float32)
    # (a) rows of softmax sum to one: V = ones gives O = ones
    ones = ctx.run_flash_attn(q, k, np.ones_like(v), None, nh, nkv, d, causal=True).astype(np.float32)
    assert np.abs(ones - 1.0).max() <= 2e-3
    # (b) query 0 sees key 0 only
    assert np.abs(out[0] - np.repeat(v[0].astype(np.float32), nh // nkv, axis=0)).max() <= 2e-3
    # (c) decode over the same keys equals the last row of the causal prefill
    print("full-size decode", flush=True)
    last = ctx.run_flash_attn(q[-1:], k, v, None, nh, nkv, d, causal=True).astype(np.float32)
    assert np.abs(last[0] - out[-1]).max() <= 2e-3
    # (d) decode at kv = 4096: convex combination of values stays inside their range, permuting keys changes nothing
    q1, k4, v4 = wl.make_attention_inputs(rng, 1, 4096, nh, nkv, d)
    o1 = ctx.run_flash_attn(q1, k4, v4, None, nh, nkv, d, causal=True).astype(np.float32)
    perm = rng.permutation(4096)
    o2 = ctx.run_flash_attn(q1, k4[perm], v4[perm], None, nh, nkv, d, causal=True).astype(np.float32)
    assert np.abs(o1 - o2).max() <= 2e-3
    vmax = np.repeat(np.abs(v4.astype(np.float32)).max(axis=0), nh // nkv, axis=0)
    assert np.all(np.abs(o1[0]) <= vmax + 1e-3)


def test_rejections(ctx):
    q, k = ctx.alloc(8 * 128 * 4), ctx.alloc(64 * 3 * 128 * 2)
    R = api.HTPOPS_ERR_REJECTED
    p = api.flash_attn_params((q, 0), (q, 0), (k, 0), (k, 0), (-1, 0), 1, 64, 8, 3, 128)
    assert ctx.execute(api.HTP_OPS_FLASH_ATTN_QO_F32_KV_F16, p) == R     # n_heads % n_kv_heads
    p = api.flash_attn_params((q, 0), (q, 0), (k, 0), (k, 0), (-1, 0), 1, 64, 4, 2, 95)
    assert ctx.execute(api.HTP_OPS_FLASH_ATTN_QO_F32_KV_F16, p) == R     # odd head_dim (flash_attn_sp_hdim.c:785)
    p = api.flash_attn_params((q, 0), (q, 0), (k, 0), (k, 0), (-1, 0), 1, 2, 2, 2, 258)
    assert ctx.execute(api.HTP_OPS_FLASH_ATTN_QO_F32_KV_F16, p) == R     # head_dim above what is built
    p = api.flash_attn_params((q, 0), (q, 0), (k, 0), (k, 0), (-1, 0), 1, 4096, 8, 2, 128)
    assert ctx.execute(api.HTP_OPS_FLASH_ATTN_QO_F32_KV_F16, p) == R     # K/V buffer too small
    ctx.release(q), ctx.release(k)


@pytest.mark.parametrize("qo,kv,nh,nkv,d", [(1, 300, 8, 2, 128), (1, 4096, 32, 8, 128), (40, 300, 4, 1, 128), (5, 70, 4, 2, 64),
                                            (3, 130, 2, 1, 80), (70, 200, 8, 2, 128)])
def test_mask_selects_keys_when_the_threshold_option_is_set(ctx, oracle, qo, kv, nh, nkv, d):
    # The kernel the reference dispatches for op 5 keeps a key iff mask > -16 (src/dsp/ops/flash_attn.c:448-460); its
    # scalar routine adds the mask (:1505-1512). The default here is the additive convention; with the option
    # "attn_mask_threshold" the same op selects keys. A mask with finite biases on both sides of -16, exact -16, -inf and
    # NaN tells the two apart; each mode is checked against the oracle under its own convention.
    rng = wl.rng_for(64, qo * 1000 + kv + nh)
    q, k, v = wl.make_attention_inputs(rng, qo, kv, nh, nkv, d)
    q = q.astype(np.float32)  # the reference op (id 5): fp32 Q / O
    ld = (kv + 63) // 64 * 64
    values = np.array([0.0, 0.0, 0.0, -3.0, -15.5, -16.0, -17.0, -40.0, -np.inf, 2.0], np.float16)
    mask = values[rng.integers(0, len(values), size=(qo, ld))]
    mask[:, 0] = 0
    additive = ctx.run_flash_attn(q, k, v, mask, nh, nkv, d)
    assert np.abs(additive - oracle.flash_attn(q, k, v, mask, nh, nkv, d)).max() <= ATOL
    with_nan = mask.copy()
    with_nan[:, 1] = np.nan  # dropped by the selecting convention (an ordered compare), poison for the additive one
    ctx.set_option("attn_mask_threshold", 1)
    selecting = ctx.run_flash_attn(q, k, v, with_nan, nh, nkv, d)
    want = oracle.flash_attn(q, k, v, oracle.threshold_mask(with_nan), nh, nkv, d)
    assert np.all(np.isfinite(selecting))
    assert np.abs(selecting - want).max() <= ATOL
    assert np.abs(selecting - additive).max() > 10 * ATOL  # (the two conventions really differ on this mask)
    # 0 / -inf masks: the same answer either way
    plain = np.where(mask > np.float16(-16), np.float16(0), np.float16(-np.inf)).astype(np.float16)
    a = ctx.run_flash_attn(q, k, v, plain, nh, nkv, d)
    ctx.set_option("attn_mask_threshold", 0)
    assert np.array_equal(a, ctx.run_flash_attn(q, k, v, plain, nh, nkv, d))
