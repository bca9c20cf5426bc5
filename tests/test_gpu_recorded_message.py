"""GPU: a message recorded into a HIP graph must give, on every replay, exactly what the same message gives when it is
walked and launched the ordinary way on the same buffer contents -- with other work and synchronizations in between,
and it must refuse to launch once memory it holds addresses of has gone."""
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


def op(op_id, payload):
    return (api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(op_id, payload))


class Block:
    """One decoder-block-like message over `m` rows: fused RMSNorm -> Q8_0, three Q4_0 matmuls on it (one launch when
    m <= 8), fp16 attention over a KV cache, Q8_0 quantization and a Q8_0 matmul of the result."""

    def __init__(self, ctx, rng, m, k=1024, n_heads=8, n_kv_heads=2, head_dim=128, kv_len=320):
        self.ctx, self.m, self.k = ctx, m, k
        self.ns = [n_heads * head_dim, 256, 272]
        self.n_out = 512
        self.w = [wl.make_q4_0_weights(rng, n, k) for n in self.ns]
        self.w_out = wl.make_q8_0_weights(rng, self.n_out, n_heads * head_dim)
        self.norm_w = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
        self.kcache = (0.5 * rng.standard_normal((kv_len, n_kv_heads, head_dim))).astype(np.float16)
        self.vcache = (0.5 * rng.standard_normal((kv_len, n_kv_heads, head_dim))).astype(np.float16)
        c = ctx
        self.hx = c.alloc(m * k * 4)
        self.hq = c.alloc(m * (k // 32) * 34)
        self.hnw = c.upload(self.norm_w)
        self.hw = [c.upload(w) for w in self.w]
        self.hmm = [c.alloc(m * n * 4) for n in self.ns]
        self.hk, self.hv = c.upload(self.kcache), c.upload(self.vcache)
        self.hattn = c.alloc(m * n_heads * head_dim * 4)
        self.hattn_q = c.alloc(m * (n_heads * head_dim // 32) * 34)
        self.hw_out = c.upload(self.w_out)
        self.hout = c.alloc(m * self.n_out * 4)
        self.handles = [self.hx, self.hq, self.hnw, self.hk, self.hv, self.hattn, self.hattn_q, self.hw_out, self.hout] + \
            self.hw + self.hmm
        reqs = [op(api.HTP_OPS_RMS_NORM_QUANTIZE_Q8_0, api.rms_norm_ex_params((self.hq, 0), (self.hx, 0), (self.hnw, 0), k, m, 1e-6))]
        reqs += [op(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0, api.mat_mul_params((ho, 0), (self.hq, 0), (hw, 0), m, k, n))
                 for ho, hw, n in zip(self.hmm, self.hw, self.ns)]
        # the first matmul's fp32 output [m][n_heads * head_dim] is the query of the reference attention op (no mask)
        reqs += [op(api.HTP_OPS_FLASH_ATTN_QO_F32_KV_F16,
                    api.flash_attn_params((self.hattn, 0), (self.hmm[0], 0), (self.hk, 0), (self.hv, 0), (-1, 0), m, kv_len,
                                          n_heads, n_kv_heads, head_dim))]
        reqs += [op(api.HTP_OPS_QUANTIZE_Q8_0, api.rms_norm_params((self.hattn_q, 0), (self.hattn, 0), n_heads * head_dim, m))]
        reqs += [op(api.HTP_OPS_MAT_MUL_Q8_0_Q8_0, api.mat_mul_params((self.hout, 0), (self.hattn_q, 0), (self.hw_out, 0), m,
                                                                     n_heads * head_dim, self.n_out))]
        self.msg = api.build_message(reqs)

    def outputs(self):
        c = self.ctx
        return [c.read(h, np.uint8, c.size(h)) for h in self.hmm + [self.hq, self.hattn, self.hattn_q, self.hout]]

    def scrub(self):
        for h in self.hmm + [self.hq, self.hattn, self.hattn_q, self.hout]:
            self.ctx.write(h, np.full(self.ctx.size(h), 0xA5, np.uint8))

    def release(self):
        for h in self.handles:
            self.ctx.release(h)


@pytest.mark.parametrize("m", [1, 8, 96])
def test_replays_equal_the_ordinary_walk(ctx, m):
    rng = wl.rng_for(70, m)
    blk = Block(ctx, rng, m)
    other_w = wl.make_q4_0_weights(rng, 640, 1024)
    rec = None
    try:
        ctx.write(blk.hx, wl.make_activations(rng, m, blk.k))
        # the unrelated work of the loop below, once beforehand: if it had to enlarge the shared workspace after the
        # recording, the recording would (rightly) refuse to launch
        ctx.run_mat_mul(ctx.run_quantize_q8_0(wl.make_activations(rng, 40, 1024)), other_w, 40, 1024, 640, wl.GGML_TYPE_Q4_0)
        ret, rec = ctx.record_message(blk.msg)
        assert ret == 0, ctx.last_error()
        assert all(s == 0 for s in api.message_request_states(blk.msg))
        for replay in range(4):
            x = wl.make_activations(rng, m, blk.k)
            ctx.write(blk.hx, x)
            ctx.write(blk.hk, np.roll(blk.kcache, replay + 1, axis=0))  # new contents, same addresses
            assert ctx.process_message(blk.msg) == 0
            want = blk.outputs()
            blk.scrub()
            # unrelated work on the same context between the walk and the replay (it uses the shared workspace)
            a = ctx.run_quantize_q8_0(wl.make_activations(rng, 40, 1024))
            ctx.run_mat_mul(a, other_w, 40, 1024, 640, wl.GGML_TYPE_Q4_0)
            assert ctx.launch_recorded_message(rec) == 0, ctx.last_error()
            if replay % 2:
                assert ctx.launch_recorded_message(rec) == 0  # twice in a row: same inputs, same result
            ctx.synchronize()
            got = blk.outputs()
            for g, w in zip(got, want):
                assert np.array_equal(g, w), "replay %d differs from the ordinary walk" % replay
    finally:
        if rec is not None:
            assert ctx.release_recorded_message(rec) == 0
        blk.release()


def test_recording_refuses_to_launch_after_its_memory_has_gone(ctx):
    rng = wl.rng_for(71, 0)
    blk = Block(ctx, rng, 8)
    rec = None
    try:
        ctx.write(blk.hx, wl.make_activations(rng, 8, blk.k))
        ret, rec = ctx.record_message(blk.msg)
        assert ret == 0, ctx.last_error()
        assert ctx.launch_recorded_message(rec) == 0
        # rewriting weights drops their converted copies, which the recording points at
        ctx.write(blk.hw[0], blk.w[0])
        assert ctx.launch_recorded_message(rec) == -1
        assert "record it again" in ctx.last_error()
        assert ctx.release_recorded_message(rec) == 0
        ret, rec = ctx.record_message(blk.msg)
        assert ret == 0, ctx.last_error()
        assert ctx.launch_recorded_message(rec) == 0
        # releasing a buffer the message does not name changes nothing ...
        spare = ctx.alloc(1024)
        ctx.release(spare)
        assert ctx.launch_recorded_message(rec) == 0
        ctx.synchronize()
        # ... releasing one that it names does
        ctx.release(blk.hmm[1])
        assert ctx.launch_recorded_message(rec) == -1
    finally:
        if rec is not None:
            assert ctx.release_recorded_message(rec) == 0
        blk.release()


def test_messages_that_cannot_be_recorded(ctx):
    rng = wl.rng_for(72, 0)
    spare = ctx.alloc(4096)
    hx = ctx.upload(wl.make_activations(rng, 1, 1024))
    hy = ctx.alloc(1024 * 4)
    try:
        # a handle release inside the message: rejected before anything runs (the handle stays valid)
        import struct
        map_req = (api.REQUEST_TYPE_RPCMEM_MAP, struct.pack("<iii", 1, 0, spare))
        norm = op(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((hy, 0), (hx, 0), 1024, 1))
        ret, rec = ctx.record_message(api.build_message([norm, map_req]))
        assert ret == -1 and rec is None
        assert ctx.size(spare) == 4096
        # a failing op
        bad = op(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((hy, 0), (hx, 0), 0, 1))
        ret, rec = ctx.record_message(api.build_message([norm, bad]))
        assert ret == -1 and rec is None
        # an empty message records and replays as nothing
        ret, rec = ctx.record_message(api.build_message([]))
        assert ret == 0
        assert ctx.launch_recorded_message(rec) == 0
        assert ctx.release_recorded_message(rec) == 0
        # the context still works
        assert ctx.process_message(api.build_message([norm])) == 0
    finally:
        for h in (spare, hx, hy):
            ctx.release(h)


def test_close_releases_recordings_left_alive():
    c = api.Context(device=0)
    rng = wl.rng_for(73, 0)
    hx = c.upload(wl.make_activations(rng, 4, 1024))
    hy = c.alloc(4 * 1024 * 4)
    msg = api.build_message([op(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((hy, 0), (hx, 0), 1024, 4))])
    ret, rec = c.record_message(msg)
    assert ret == 0 and rec is not None
    assert c.launch_recorded_message(rec) == 0
    c.close()  # neither the recording nor the buffers were released by hand
