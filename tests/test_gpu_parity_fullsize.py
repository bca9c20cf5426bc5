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
    # up to three rows the seven requests are one launch; eight rows: the six k = 4096 projections share one, down is
    # alone
    run_layer_message(ctx, oracle, wl.LLAMA7B_LAYER, llama_weights, acts, m, Q4, launches=1 if m <= 3 else 2)


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
