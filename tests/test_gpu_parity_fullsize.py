"""GPU parity at the benchmark's full sizes, with the benchmark's launch geometry: the requests travel as mailbox
messages built like the reference's host code does (src/host/test.c:166-204: message written, run, per-request state
read back), so grouped launches (q+k+v, gate+up) and the kernels picked for the full row counts are what is checked.
The scalar oracle is too slow for whole outputs at these sizes: every output matrix is compared on a sample of weight
rows (columns of the output) for every activation row, against the float64 accumulation of the oracle's exact
integer block terms (|gpu - f64| <= 1e-5 * sum |terms|)."""
import numpy as np
import pytest

from pyhtpops import api
from pyhtpops import workloads as wl

pytestmark = pytest.mark.gpu

MATMUL_RTOL = 1e-5
Q4, Q8 = wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0
# which activation buffer a projection reads (the data flow of a decoder layer; the backend groups requests by it)
ACT_OF = {"q": 0, "k": 0, "v": 0, "o": 1, "gate": 2, "up": 2, "down": 3}


@pytest.fixture(scope="module")
def ctx():
    c = api.Context(device=0)
    yield c
    c.close()


def sampled_rows(n, count=96):
    return np.unique(np.concatenate([np.linspace(0, n - 1, count).astype(int), [0, 1, n - 2, n - 1]]))


def run_layer_message(ctx, oracle, shapes, weights, acts, m, wt, act_rows=None, launches=None):
    """One message with one matmul request per entry of `shapes`; returns nothing, asserts parity of every output
    (and, with `launches`, how many submissions the message became)."""
    op = api.HTP_OPS_MAT_MUL_Q4_0_Q8_0 if wt == Q4 else api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    h_act = {g: ctx.upload(a) for g, a in acts.items()}
    h_w = [ctx.upload(weights[(n, k)]) for _, n, k in shapes]
    h_out = [ctx.alloc(m * n * 4) for _, n, _ in shapes]
    try:
        for h, (_, n, _) in zip(h_out, shapes):
            ctx.write(h, np.full(m * n, np.nan, np.float32))
        reqs = [(api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(
            op, api.mat_mul_params((h_out[i], 0), (h_act[ACT_OF[name]], 0), (h_w[i], 0), m, k, n)))
            for i, (name, n, k) in enumerate(shapes)]
        msg = api.build_message(reqs)
        msg[0] = 1
        for rep in range(2):  # a second pass runs on the converted weight copies the first one cached
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0] * len(shapes), ctx.last_error()
            assert msg[1] == 1
            if launches is not None:
                assert ctx.last_message_submissions() == launches
            for i, (name, n, k) in enumerate(shapes):
                print("full-size message m=%d %s n=%d k=%d pass %d" % (m, name, n, k, rep), flush=True)
                got = ctx.read(h_out[i], np.float32, m * n).reshape(m, n)
                assert np.all(np.isfinite(got)), "%s: output not fully written" % name
                cols = sampled_rows(n)
                rows = np.arange(m) if act_rows is None else act_rows
                a = acts[ACT_OF[name]][rows]
                want, mag = oracle.mat_mul_q8_0_act_f64(a, weights[(n, k)][cols], len(rows), k, len(cols), wt)
                err = np.abs(got[np.ix_(rows, cols)] - want) / mag
                assert np.all(err <= MATMUL_RTOL), "%s m=%d: %g" % (name, m, err.max())
    finally:
        for h in list(h_act.values()) + h_w + h_out:
            ctx.release(h)


@pytest.fixture(scope="module")
def llama_weights():
    rng = wl.rng_for(1, 0)
    return {(n, k): wl.make_q4_0_weights(rng, n, k) for n, k in {(n, k) for _, n, k in wl.LLAMA7B_LAYER}}


@pytest.mark.parametrize("m", [1, 2, 3, 8])
def test_llama7b_layer_message_at_full_size(ctx, oracle, llama_weights, m):
    # config 1: q/k/v/o 4096x4096, gate/up 11008x4096, down 4096x11008, seven requests in one message
    rng = wl.rng_for(1, 100 + m)
    acts = {g: oracle.quantize_q8_0(wl.make_activations(rng, m, k)) for g, k in {0: 4096, 1: 4096, 2: 4096, 3: 11008}.items()}
    # the seven requests are one launch: two rows in the kernel that keeps the rows in registers, three and eight rows
    # in the two-blocks-per-instruction kernel, whose members may differ in k
    run_layer_message(ctx, oracle, wl.LLAMA7B_LAYER, llama_weights, acts, m, Q4, launches=1)


@pytest.mark.parametrize("n,k", [(11008, 4096), (4096, 11008)])
def test_prefill_gemm_m512_at_full_size(ctx, oracle, llama_weights, n, k):
    # config 2, both shapes; the activations are quantized on the GPU (bit-exact against the oracle's quantizer)
    rng = wl.rng_for(2, n)
    m = 512
    x = wl.make_activations(rng, m, k)
    a = ctx.run_quantize_q8_0(x)
    assert np.array_equal(a, oracle.quantize_q8_0(x))
    w = llama_weights[(n, k)]
    print("full-size prefill m=%d n=%d k=%d" % (m, n, k), flush=True)
    got = ctx.run_mat_mul(a, w, m, k, n, Q4)
    rows = np.array([0, 1, 31, 32, 63, 64, 255, 256, 300, 510, 511])
    cols = sampled_rows(n, 64)
    want, mag = oracle.mat_mul_q8_0_act_f64(a[rows], w[cols], len(rows), k, len(cols), Q4)
    assert np.all(np.abs(got[np.ix_(rows, cols)] - want) <= MATMUL_RTOL * mag)
    # every row against the one-row kernel of the same row (independent kernel, same arithmetic)
    for r in (5, 130, 257, 500):
        gemv = ctx.run_mat_mul(a[r:r + 1], w, 1, k, n, Q4)
        assert np.abs(gemv[0] - got[r]).max() <= 2e-5 * np.abs(gemv).max()
    # the fp32-activation op (quantize + matmul) gives the same bits
    assert np.array_equal(ctx.run_mat_mul(x, w, m, k, n, Q4, act_is_f32=True), got)


@pytest.mark.parametrize("m", [1, 2, 128])
def test_qwen2_q8_0_block_message_at_full_size(ctx, oracle, m):
    # config 4: RMSNorm (1536, eps 1e-6, weight N(1, 0.1)) -> Q8_0 -> Q8_0-weight matmuls 1536x1536 (q, o), 256x1536
    # (k, v), 8960x1536 (gate, up), 1536x8960 (down)
    rng = wl.rng_for(4, 100 + m)
    weights = {(n, k): wl.make_q8_0_weights(rng, n, k) for n, k in {(n, k) for _, n, k in wl.QWEN2_1P5B_LAYER}}
    x = wl.make_activations(rng, m, 1536)
    g = (1 + 0.1 * rng.standard_normal(1536)).astype(np.float32)
    normed = ctx.run_rms_norm(x, g, 1e-6)
    assert np.abs(normed - oracle.rms_norm(x, g, 1e-6)).max() <= 2e-3
    fused = ctx.run_rms_norm(x, g, 1e-6, quantize=True)
    assert np.array_equal(fused, oracle.quantize_q8_0(normed))  # the chain on the GPU's own normalized rows: bit-exact
    acts = {0: fused, 1: oracle.quantize_q8_0(wl.make_activations(rng, m, 1536)),
            2: oracle.quantize_q8_0(wl.make_activations(rng, m, 1536)), 3: oracle.quantize_q8_0(wl.make_activations(rng, m, 8960))}
    act_rows = None if m <= 8 else np.array([0, 1, 31, 32, 63, 64, 100, 126, 127])
    run_layer_message(ctx, oracle, wl.QWEN2_1P5B_LAYER, weights, acts, m, Q8, act_rows, launches=1)


ATTN_ATOL = 2e-3


@pytest.mark.parametrize("qo,kv", [(2048, 2048), (1, 4096), (1, 16384)])
def test_attention_at_full_size_against_the_oracle_on_sampled_rows(ctx, oracle, qo, kv):
    # config 3 (32 query / 8 KV heads of 128, fp16, causal): the kernel the benchmark times, against the oracle's scalar
    # attention for sampled query rows -- both ends, both sides of a 32-row tile edge, the middle, and the whole last
    # tile -- every head. The oracle gets the sampled rows with their rows of the causal mask written out (0 on and
    # below the diagonal, -inf above: the convention both reference variants agree on, flash_attn.c:452-455 / :1505-1512).
    nh, nkv, hd = 32, 8, 128
    rng = wl.rng_for(3, qo * 7 + kv)
    q, k, v = wl.make_attention_inputs(rng, qo, kv, nh, nkv, hd)
    print("full-size attention qo=%d kv=%d" % (qo, kv), flush=True)
    got = ctx.run_flash_attn(q, k, v, None, nh, nkv, hd, causal=True)
    rows = np.array(sorted({0, 31, 32, qo // 2 - 1, qo // 2} | set(range(max(0, qo - 32), qo)))) if qo > 1 else np.array([0])
    rows = rows[rows >= 0]
    ld = (kv + 63) // 64 * 64
    mask = np.full((len(rows), ld), -np.inf, np.float16)
    for i, r in enumerate(rows):
        mask[i, :r + (kv - qo) + 1] = 0
    want = oracle.flash_attn(np.ascontiguousarray(q[rows]), k, v, mask, nh, nkv, hd, False)
    err = np.abs(got[rows].astype(np.float32) - want.astype(np.float32)).max()
    assert err <= ATTN_ATOL, err
    # the reference op (id 5: fp32 Q / O, the mask as a buffer) on the same rows gives the same values
    got32 = ctx.run_flash_attn(np.ascontiguousarray(q[rows]).astype(np.float32), k, v, mask, nh, nkv, hd)
    assert np.abs(got32 - want.astype(np.float32)).max() <= ATTN_ATOL


def test_decoder_layer_for_one_token_as_one_message(ctx, oracle, llama_weights):
    # The twelve requests of a Llama-7B-like layer for one token, as ONE message: RMSNorm+Q8_0 -> q, k, v -> attention
    # over 4096 cached keys -> Q8_0 -> o -> RMSNorm+Q8_0 -> gate, up -> Q8_0 -> down. The walk fuses and groups them
    # into 6 submissions; every buffer the message writes must hold, byte for byte, what the same requests give when
    # each is sent as a message of its own (12 submissions: the reference's one-op-per-request order,
    # src/dsp/commu.c:91-114), and every stage must meet the oracle applied to the stage's own input.
    nh, nkv, hd, kv = 32, 8, 128, 4096
    rng = wl.rng_for(6, 1)
    shapes = {name: (n, k) for name, n, k in wl.LLAMA7B_LAYER}
    _, kk, vv = wl.make_attention_inputs(rng, 1, kv, nh, nkv, hd)
    x = wl.make_activations(rng, 1, 4096)
    g = (1 + 0.1 * rng.standard_normal(4096)).astype(np.float32)
    hidden = wl.make_activations(rng, 1, 11008)
    h_w = {name: ctx.upload(llama_weights[shapes[name]]) for name in shapes}
    hx, hg, hh, hk, hv = ctx.upload(x), ctx.upload(g), ctx.upload(hidden), ctx.upload(kk), ctx.upload(vv)
    sizes = {"qa": 4096 // 32 * 34, "qo": 4096 // 32 * 34, "qb": 4096 // 32 * 34, "qd": 11008 // 32 * 34, "attn": 4096 * 4}
    sizes.update({name: shapes[name][0] * 4 for name in shapes})

    def build(bufs):
        def op(code, payload):
            return (api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(code, payload))

        def mm(name, act):
            n, k = shapes[name]
            return op(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0, api.mat_mul_params((bufs[name], 0), (bufs[act], 0), (h_w[name], 0), 1, k, n))
        return [
            op(api.HTP_OPS_RMS_NORM_QUANTIZE_Q8_0, api.rms_norm_ex_params((bufs["qa"], 0), (hx, 0), (hg, 0), 4096, 1, 1e-6)),
            mm("q", "qa"), mm("k", "qa"), mm("v", "qa"),
            op(api.HTP_OPS_FLASH_ATTN_QO_F32_KV_F16,
               api.flash_attn_params((bufs["attn"], 0), (bufs["q"], 0), (hk, 0), (hv, 0), (-1, 0), 1, kv, nh, nkv, hd)),
            op(api.HTP_OPS_QUANTIZE_Q8_0, api.rms_norm_params((bufs["qo"], 0), (bufs["attn"], 0), 4096, 1)),
            mm("o", "qo"),
            op(api.HTP_OPS_RMS_NORM_QUANTIZE_Q8_0, api.rms_norm_ex_params((bufs["qb"], 0), (bufs["o"], 0), (hg, 0), 4096, 1, 1e-6)),
            mm("gate", "qb"), mm("up", "qb"),
            op(api.HTP_OPS_QUANTIZE_Q8_0, api.rms_norm_params((bufs["qd"], 0), (hh, 0), 11008, 1)),
            mm("down", "qd")]

    sets = [{name: ctx.alloc(nbytes) for name, nbytes in sizes.items()} for _ in range(2)]
    try:
        for bufs in sets:
            for name, nbytes in sizes.items():
                ctx.write(bufs[name], np.full(nbytes, 0xA5, np.uint8))
        print("decoder layer: twelve requests in one message", flush=True)
        msg = api.build_message(build(sets[0]))
        assert ctx.process_message(msg) == 0 and api.message_request_states(msg) == [0] * 12, ctx.last_error()
        assert ctx.last_message_submissions() == 6
        print("decoder layer: one message per request", flush=True)
        for req in build(sets[1]):
            one = api.build_message([req])
            assert ctx.process_message(one) == 0 and api.message_request_states(one) == [0], ctx.last_error()
        out = [{name: ctx.read(bufs[name], np.uint8, nbytes) for name, nbytes in sizes.items()} for bufs in sets]
        for name in sizes:
            assert np.array_equal(out[0][name], out[1][name]), "%s differs between the one message and the twelve" % name
        o = out[0]
        f32 = {name: o[name].view(np.float32) for name in list(shapes) + ["attn"]}

        def check_matmul(name, act):
            n, k = shapes[name]
            want, mag = oracle.mat_mul_q8_0_act_f64(o[act].reshape(1, -1), llama_weights[(n, k)], 1, k, n, Q4)
            assert np.all(np.abs(f32[name] - want[0]) <= MATMUL_RTOL * mag[0]), name

        def check_norm_row(name, src_row):
            # RMSNorm is held to 2e-3, so its Q8_0 row is: the oracle's quantizer applied to some row within 2e-3 of
            # the oracle's normalized row -- every dequantized value within half a quantization step plus 2e-3 of it
            normed = oracle.rms_norm(src_row.reshape(1, -1), g, 1e-6)[0]
            blocks = o[name].reshape(-1, 34)
            d = blocks[:, :2].copy().view(np.float16).astype(np.float32)
            deq = (blocks[:, 2:].view(np.int8).astype(np.float32) * d).reshape(-1)
            step = np.repeat(d[:, 0], 32)
            assert np.all(np.abs(deq - normed) <= 0.5 * step * 1.002 + 2e-3), name

        check_norm_row("qa", x[0])
        for name in ("q", "k", "v"):
            check_matmul(name, "qa")
        want_attn = oracle.flash_attn(f32["q"].reshape(1, nh, hd), kk, vv, None, nh, nkv, hd)
        assert np.abs(f32["attn"] - want_attn.reshape(-1)).max() <= ATTN_ATOL
        assert np.array_equal(o["qo"], oracle.quantize_q8_0(f32["attn"].reshape(1, -1)).reshape(-1))
        check_matmul("o", "qo")
        check_norm_row("qb", f32["o"])
        check_matmul("gate", "qb")
        check_matmul("up", "qb")
        assert np.array_equal(o["qd"], oracle.quantize_q8_0(hidden).reshape(-1))
        check_matmul("down", "qd")
    finally:
        for bufs in sets:
            for h in bufs.values():
                ctx.release(h)
        for h in list(h_w.values()) + [hx, hg, hh, hk, hv]:
            ctx.release(h)
