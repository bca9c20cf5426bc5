"""GPU parity: Q8_0 quantizer (bit-exact), RMSNorm (2e-3 absolute; in practice ~1e-6), quantized matmul
(|gpu - f64| <= 1e-5 * sum|terms|, and the same against the fp32 oracle), all through the op ABI."""
import os

import numpy as np
import pytest

from pyhtpops import api
from pyhtpops import workloads as wl

pytestmark = pytest.mark.gpu

MATMUL_RTOL = 1e-5      # relative to sum |block terms| (fp32 accumulation order differs from the oracle's)
NORM_ATOL = 2e-3


@pytest.fixture(scope="module")
def ctx():
    c = api.Context(device=0)
    yield c
    c.close()


@pytest.fixture(autouse=True)
def default_switches(ctx):
    """Tests that force a kernel do it through htpops_set_option; every test starts from the defaults again."""
    yield
    for name, value in api.DEFAULT_OPTIONS.items():
        ctx.set_option(name, value)


# ---------------------------------------------------------------------------------------- quantizer

@pytest.mark.parametrize("m,k", [(1, 4096), (8, 4096), (1, 11008), (3, 32), (5, 96), (128, 1536), (512, 4096), (7, 8960)])
def test_quantize_q8_0_bit_exact(ctx, oracle, m, k):
    rng = wl.rng_for(51, m * 100000 + k)
    x = wl.make_activations(rng, m, k)
    if m >= 3:
        x[1] *= 1e-5          # tiny scales (fp16 subnormal d)
        x[2] *= 2e3
        x[0, :32] = 0         # an all-zero block
    print("quantize case m=%d k=%d" % (m, k), flush=True)
    got = ctx.run_quantize_q8_0(x)
    want = oracle.quantize_q8_0(x)
    assert np.array_equal(got, want)


def test_quantize_q8_0_ties_and_extremes_bit_exact(ctx, oracle):
    x = np.zeros((2, 64), np.float32)
    x[0, 0] = 127.0
    x[0, 1:9] = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5]
    x[0, 32:64] = np.arange(32) - 16
    x[1, :32] = np.linspace(-3e-6 * 127, 3e-6 * 127, 32)
    x[1, 32:] = np.linspace(-6e4, 6e4, 32)
    assert np.array_equal(ctx.run_quantize_q8_0(x), oracle.quantize_q8_0(x))


# ------------------------------------------------------------------------------------------ rmsnorm

@pytest.mark.parametrize("ne0,ne1", [(4096, 1), (1536, 1), (1536, 128), (4096, 512), (60000, 1), (33, 3), (8192, 4), (16384, 2), (24576, 2)])
def test_rms_norm_reference_op(ctx, oracle, ne0, ne1):
    rng = wl.rng_for(52, ne0 + ne1)
    x = rng.uniform(-20, 20, (ne1, ne0)).astype(np.float32)   # the reference test's input range (test.c:99-102)
    print("rms_norm case ne0=%d ne1=%d" % (ne0, ne1), flush=True)
    got = ctx.run_rms_norm(x)
    want = oracle.rms_norm(x, None, 1e-5)
    assert np.abs(got - want).max() <= 1e-5   # the reference's own tolerance (test.c:116-118)


@pytest.mark.parametrize("ne0,ne1", [(4096, 1), (1536, 128), (1536, 1), (96, 5)])
def test_rms_norm_with_weight_and_eps(ctx, oracle, ne0, ne1):
    rng = wl.rng_for(52, 1000 + ne0 + ne1)
    x = wl.make_activations(rng, ne1, ne0)
    w = (1 + 0.1 * rng.standard_normal(ne0)).astype(np.float32)
    got = ctx.run_rms_norm(x, w, 1e-6)
    want = oracle.rms_norm(x, w, 1e-6)
    assert np.abs(got - want).max() <= NORM_ATOL
    # tighter: the reference's own 1e-5 (the oracle's sequential fp32 row sum is the noisier side)
    assert np.abs(got - want).max() <= 1e-5
    x64 = x.astype(np.float64)
    exact = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-6) * w
    assert np.abs(got - exact).max() <= 1e-6
    got1 = ctx.run_rms_norm(x, None, 1e-6)
    assert np.abs(got1 - oracle.rms_norm(x, None, 1e-6)).max() <= 1e-5


@pytest.mark.parametrize("ne0,ne1", [(4096, 1), (1536, 128), (4096, 8), (16384, 2)])
def test_fused_rms_norm_quantize_equals_the_two_ops_in_a_row(ctx, oracle, ne0, ne1):
    rng = wl.rng_for(52, 2000 + ne0 + ne1)
    x = wl.make_activations(rng, ne1, ne0)
    w = (1 + 0.1 * rng.standard_normal(ne0)).astype(np.float32)
    fused = ctx.run_rms_norm(x, w, 1e-6, quantize=True)
    two_step = ctx.run_quantize_q8_0(ctx.run_rms_norm(x, w, 1e-6))
    assert np.array_equal(fused, two_step)
    # and against the oracle chain: quants within one step, scales within one fp16 ulp (the row sums differ in order)
    want = oracle.quantize_q8_0(oracle.rms_norm(x, w, 1e-6))
    dg, qg = wl.q8_0_split(fused, ne0)
    dw, qw = wl.q8_0_split(want, ne0)
    assert np.abs(qg.astype(np.int32) - qw.astype(np.int32)).max() <= 1
    assert np.abs(dg.view(np.int16).astype(np.int32) - dw.view(np.int16).astype(np.int32)).max() <= 1


# ------------------------------------------------------------------------------------------- matmul

def check_mat_mul(ctx, oracle, rng, m, k, n, wt):
    w = wl.make_weights(rng, n, k, wt)
    x = wl.make_activations(rng, m, k)
    a = oracle.quantize_q8_0(x)
    print("mat_mul case m=%d k=%d n=%d wt=%d" % (m, k, n, wt), flush=True)
    got = ctx.run_mat_mul(a, w, m, k, n, wt)
    want32 = oracle.mat_mul_q8_0_act(a, w, m, k, n, wt, n_threads=8)
    want64, mag = oracle.mat_mul_q8_0_act_f64(a, w, m, k, n, wt)
    assert np.all(np.abs(got - want64) <= MATMUL_RTOL * mag), float((np.abs(got - want64) / mag).max())
    assert np.all(np.abs(got - want32) <= MATMUL_RTOL * mag)
    return got, x, w


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
@pytest.mark.parametrize("k,n", [(4096, 4096), (4096, 1024), (11008, 512), (1536, 1536), (1536, 256), (8960, 384),
                                 (64, 32), (128, 7), (2048, 100), (1024, 33), (12288 + 64, 40), (96, 64), (32, 5), (4128, 16)])
def test_gemv_m1(ctx, oracle, wt, k, n):
    check_mat_mul(ctx, oracle, wl.rng_for(53, k * 7 + n + wt), 1, k, n, wt)


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
@pytest.mark.parametrize("m,k,n", [(8, 4096, 512), (2, 11008, 96), (3, 1536, 256), (8, 96, 40), (5, 64, 32), (16, 1024, 128),
                                   (8, 11008, 1024), (8, 4096, 100), (13, 2048, 70), (32, 4096, 64), (31, 11008, 40),
                                   (40, 1024, 96), (63, 640, 33), (9, 64, 32), (4, 8960, 1536)])
def test_small_batch(ctx, oracle, wt, m, k, n):
    got, x, w = check_mat_mul(ctx, oracle, wl.rng_for(54, m * 31 + k + n + wt), m, k, n, wt)
    # the fp32-activation op quantizes on the device and must give the same bits
    assert np.array_equal(ctx.run_mat_mul(x, w, m, k, n, wt, act_is_f32=True), got)


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
def test_mat_mul_integer_exact_special_case(ctx, wt):
    # scales 1.0 and small integers: every partial sum is an exactly representable integer
    rng = wl.rng_for(55, wt)
    m, k, n = 2, 256, 96
    w = wl.make_weights(rng, n, k, wt).reshape(n, k // 32, -1)
    w[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    w = w.reshape(n, -1)
    a = np.empty((m, k // 32, 34), np.uint8)
    a[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    a[:, :, 2:] = rng.integers(-20, 21, (m, k // 32, 32), dtype=np.int8).view(np.uint8)
    a = a.reshape(m, -1)
    got = ctx.run_mat_mul(a, w, m, k, n, wt)
    _, qa = wl.q8_0_split(a, k)
    _, qw = (wl.q4_0_split if wt == wl.GGML_TYPE_Q4_0 else wl.q8_0_split)(w, k)
    assert np.array_equal(got, (qa.astype(np.int64) @ qw.astype(np.int64).T).astype(np.float32))


def test_block_dot_extremes_are_exact(ctx):
    # all weights -8 and all activations -127: 32512 per block, times scales 1 -> exact
    k, n = 128, 32
    w = np.zeros((n, k // 32, 18), np.uint8)
    w[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    a = np.empty((1, k // 32, 34), np.uint8)
    a[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    a[:, :, 2:] = np.int8(-127).view(np.uint8)
    got = ctx.run_mat_mul(a.reshape(1, -1), w.reshape(n, -1), 1, k, n, wl.GGML_TYPE_Q4_0)
    assert np.all(got == 4 * 32512.0)
    w[:] = 0xFF
    w[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    got = ctx.run_mat_mul(a.reshape(1, -1), w.reshape(n, -1), 1, k, n, wl.GGML_TYPE_Q4_0)
    assert np.all(got == 4 * (-7 * 127 * 32.0))


def test_message_with_a_decode_chain_runs_in_order(ctx, oracle):
    # RMSNorm -> quantize -> GEMV submitted as one mailbox message (config 0 of the benchmark, small n)
    rng = wl.rng_for(0, 0)
    k, n = 4096, 256
    w = wl.make_q4_0_weights(rng, n, k)
    x = wl.make_activations(rng, 1, k)
    hx, hn, hq, hw, ho = ctx.upload(x), ctx.alloc(k * 4), ctx.alloc(k // 32 * 34), ctx.upload(w), ctx.alloc(n * 4)
    ones = ctx.upload(np.ones(k, np.float32))
    reqs = [
        (api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(api.HTP_OPS_RMS_NORM_F32_EX, api.rms_norm_ex_params((hn, 0), (hx, 0), (ones, 0), k, 1, 1e-6))),
        (api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(api.HTP_OPS_QUANTIZE_Q8_0, api.rms_norm_params((hq, 0), (hn, 0), k, 1))),
        (api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0, api.mat_mul_params((ho, 0), (hq, 0), (hw, 0), 1, k, n))),
        (api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(api.HTP_OPS_RMS_NORM_F32, api.rms_norm_params((hn, 0), (hx, 0), 0, 1))),
    ]
    msg = api.build_message(reqs)
    msg[0] = 1
    assert ctx.process_message(msg) == 0
    assert api.message_request_states(msg) == [0, 0, 0, -1] and msg[1] == 1
    got = ctx.read(ho, np.float32, n)
    normed = oracle.rms_norm(x, np.ones(k, np.float32), 1e-6)
    gpu_normed = ctx.read(hn, np.float32, k)
    assert np.abs(gpu_normed - normed[0]).max() <= 1e-5
    # quantization of the GPU's own normalized row is bit-exact, and the GEMV on it matches the oracle
    a = oracle.quantize_q8_0(gpu_normed[None, :])
    assert np.array_equal(ctx.read(hq, np.uint8, k // 32 * 34), a[0])
    want64, mag = oracle.mat_mul_q8_0_act_f64(a, w, 1, k, n, wl.GGML_TYPE_Q4_0)
    assert np.all(np.abs(got - want64[0]) <= MATMUL_RTOL * mag[0])
    for h in (hx, hn, hq, hw, ho, ones):
        ctx.release(h)


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
@pytest.mark.parametrize("m", [2, 8, 12, 27])
def test_small_batch_integer_exact(ctx, wt, m):
    # scales 1.0, full-range int8 activations: the output is the exact integer matrix product
    rng = wl.rng_for(58, wt + m)
    k, n = 640, 77
    w = wl.make_weights(rng, n, k, wt).reshape(n, k // 32, -1)
    w[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    w = w.reshape(n, -1)
    a = np.empty((m, k // 32, 34), np.uint8)
    a[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    a[:, :, 2:] = rng.integers(-127, 128, (m, k // 32, 32), dtype=np.int8).view(np.uint8)
    a = a.reshape(m, -1)
    got = ctx.run_mat_mul(a, w, m, k, n, wt)
    _, qa = wl.q8_0_split(a, k)
    _, qw = (wl.q4_0_split if wt == wl.GGML_TYPE_Q4_0 else wl.q8_0_split)(w, k)
    assert np.array_equal(got, (qa.astype(np.int64) @ qw.astype(np.int64).T).astype(np.float32))


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
def test_message_batches_same_activation_gemvs(ctx, oracle, wt):
    # One message: ten one-row matmuls on activation A with different n (they run as grouped launches of up to
    # eight), one on activation B, then one more on A whose output buffer is B's output (must stay ordered).
    rng = wl.rng_for(60, wt)
    k = 1536
    op = api.HTP_OPS_MAT_MUL_Q4_0_Q8_0 if wt == wl.GGML_TYPE_Q4_0 else api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    ns = [256, 1536, 33, 1, 640, 64, 100, 8, 2048, 17]
    ws = [wl.make_weights(rng, n, k, wt) for n in ns]
    a = oracle.quantize_q8_0(wl.make_activations(rng, 1, k))
    b = oracle.quantize_q8_0(wl.make_activations(rng, 1, k))
    ha, hb = ctx.upload(a), ctx.upload(b)
    hws = [ctx.upload(w) for w in ws]
    houts = [ctx.alloc(n * 4) for n in ns]
    handles = [ha, hb] + hws + houts
    try:
        reqs = [(api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(op, api.mat_mul_params((ho, 0), (ha, 0), (hw, 0), 1, k, n)))
                for ho, hw, n in zip(houts, hws, ns)]
        # activation B into output 0, then activation A into output 0 again: the last writer must win
        reqs.append((api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(op, api.mat_mul_params((houts[0], 0), (hb, 0), (hws[0], 0), 1, k, ns[0]))))
        reqs.append((api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(op, api.mat_mul_params((houts[1], 0), (ha, 0), (hws[1], 0), 1, k, ns[1]))))
        msg = api.build_message(reqs)
        assert ctx.process_message(msg) == 0
        assert all(s == 0 for s in api.message_request_states(msg))
        got = [ctx.read(ho, np.float32, n) for ho, n in zip(houts, ns)]
        for i, (w, n) in enumerate(zip(ws, ns)):
            act = b if i == 0 else a
            single = ctx.run_mat_mul(act, w, 1, k, n, wt)[0]
            assert np.array_equal(got[i], single), "request %d differs from its own launch" % i
            want64, mag = oracle.mat_mul_q8_0_act_f64(act, w, 1, k, n, wt)
            assert np.all(np.abs(got[i] - want64[0]) <= MATMUL_RTOL * mag[0])
    finally:
        for h in handles:
            ctx.release(h)


@pytest.mark.parametrize("wt,m,k", [(wl.GGML_TYPE_Q4_0, 8, 4096), (wl.GGML_TYPE_Q8_0, 3, 1536), (wl.GGML_TYPE_Q4_0, 2, 2048 + 64),
                                    (wl.GGML_TYPE_Q4_0, 12, 4096), (wl.GGML_TYPE_Q8_0, 10, 1536), (wl.GGML_TYPE_Q4_0, 16, 2048 + 64)])
def test_message_batches_same_activation_small_batches(ctx, oracle, wt, m, k):
    # The same grouping for 2..16 activation rows: matrices of different n on activation A, then the same weights on
    # activation B. Members that take the repacked-weight kernel share launches across A and B (each member reads its
    # own rows), those of the K-sliced kernel (each with its own partial tiles and ticket counters) only within A or B.
    # Every request must equal its own launch bit for bit, twice in a row (the counters come back to zero).
    rng = wl.rng_for(65, wt * 100 + m)
    op = api.HTP_OPS_MAT_MUL_Q4_0_Q8_0 if wt == wl.GGML_TYPE_Q4_0 else api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    ns = [256, 1536, 33, 640, 100]
    ws = [wl.make_weights(rng, n, k, wt) for n in ns]
    a = oracle.quantize_q8_0(wl.make_activations(rng, m, k))
    b = oracle.quantize_q8_0(wl.make_activations(rng, m, k))
    ha, hb = ctx.upload(a), ctx.upload(b)
    hws = [ctx.upload(w) for w in ws]
    houts_a = [ctx.alloc(m * n * 4) for n in ns]
    houts_b = [ctx.alloc(m * n * 4) for n in ns]
    handles = [ha, hb] + hws + houts_a + houts_b
    try:
        reqs = [(api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(op, api.mat_mul_params((ho, 0), (ha, 0), (hw, 0), m, k, n)))
                for ho, hw, n in zip(houts_a, hws, ns)]
        reqs += [(api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(op, api.mat_mul_params((ho, 0), (hb, 0), (hw, 0), m, k, n)))
                 for ho, hw, n in zip(houts_b, hws, ns)]
        msg = api.build_message(reqs)
        for _ in range(2):
            assert ctx.process_message(msg) == 0
            assert all(s == 0 for s in api.message_request_states(msg))
            for act, houts in ((a, houts_a), (b, houts_b)):
                for ho, w, n in zip(houts, ws, ns):
                    got = ctx.read(ho, np.float32, m * n).reshape(m, n)
                    assert np.array_equal(got, ctx.run_mat_mul(act, w, m, k, n, wt)), "a request differs from its own launch"
                    want64, mag = oracle.mat_mul_q8_0_act_f64(act, w, m, k, n, wt)
                    assert np.all(np.abs(got - want64) <= MATMUL_RTOL * mag)
    finally:
        for h in handles:
            ctx.release(h)


def test_small_batch_repeated_launches_are_bit_identical(ctx):
    # K is cut into slices that are summed in a fixed order by the last workgroup of a row tile: the result must not
    # depend on which workgroup that is, and the ticket counters must come back to zero after every launch
    rng = wl.rng_for(59, 0)
    m, k, n = 8, 11008, 2048
    w = wl.make_q4_0_weights(rng, n, k)
    a = wl.quantize_q8_0_numpy(wl.make_activations(rng, m, k)) if hasattr(wl, "quantize_q8_0_numpy") else \
        ctx.run_quantize_q8_0(wl.make_activations(rng, m, k))
    first = ctx.run_mat_mul(a, w, m, k, n, wl.GGML_TYPE_Q4_0)
    for _ in range(5):
        assert np.array_equal(ctx.run_mat_mul(a, w, m, k, n, wl.GGML_TYPE_Q4_0), first)
    # every row agrees with the one-row kernel
    for r in (0, 3, 7):
        one = ctx.run_mat_mul(a[r:r + 1], w, 1, k, n, wl.GGML_TYPE_Q4_0)
        assert np.abs(one[0] - first[r]).max() <= 2e-5 * np.abs(one).max()


@pytest.mark.parametrize("wt,m", [(wl.GGML_TYPE_Q4_0, 2), (wl.GGML_TYPE_Q4_0, 3), (wl.GGML_TYPE_Q8_0, 2), (wl.GGML_TYPE_Q8_0, 3)])
@pytest.mark.parametrize("k,n", [(64, 1), (128, 33), (1024, 100), (4096, 4096), (4096 + 64, 70), (8192, 9), (11008, 272),
                                 (12288, 64), (2048 + 64, 1000)])
def test_two_and_three_rows_on_the_decode_kernels_weight_stream(ctx, oracle, wt, m, k, n):
    # 2 and 3 rows run the decode kernel's stream over the weights with the rows held in registers: one, two or three
    # waves per weight row (k <= 4096, <= 8192, <= 12288), rows past the last whole walk of a workgroup, one lane of a
    # chunk only (k = 4096 + 64). HTPOPS_LANE_ORDER=0 pins that kernel (by default Q4_0 with n % 16 == 0 and
    # k % 256 == 0 goes to the kernel over repacked weights instead). Against the oracle, bit for bit on a repeat,
    # every row against the one-row kernel (same block sums and lane mapping; the compiler is free to fuse the scale
    # multiplications differently in the two kernels, so to rounding), and against what the default switches and
    # HTPOPS_GEMV_ROWS_KERNEL=0 choose for the same matmul.
    rng = wl.rng_for(69, wt * 1000 + m * 100 + k + n)
    ctx.set_option("lane_order", 0)
    got, x, w = check_mat_mul(ctx, oracle, rng, m, k, n, wt)
    a = oracle.quantize_q8_0(x)
    assert np.array_equal(ctx.run_mat_mul(a, w, m, k, n, wt), got)
    _, mag = oracle.mat_mul_q8_0_act_f64(a, w, m, k, n, wt)
    for r in range(m):
        one = ctx.run_mat_mul(a[r:r + 1], w, 1, k, n, wt)[0]
        assert np.all(np.abs(one - got[r]) <= 1e-6 * mag[r]), "row %d differs from the one-row kernel" % r
    ctx.set_option("lane_order", 1)
    default = ctx.run_mat_mul(a, w, m, k, n, wt)
    assert np.all(np.abs(default - got) <= 2 * MATMUL_RTOL * mag)
    ctx.set_option("gemv_rows_kernel", 0)
    other = ctx.run_mat_mul(a, w, m, k, n, wt)
    assert np.all(np.abs(other - got) <= 2 * MATMUL_RTOL * mag)


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
def test_mat_mul_on_both_sides_of_every_kernel_switch(ctx, oracle, wt):
    # which kernel a matmul takes depends on m (1 | 2..8 | 9..16 | 17..32 | 33..), on k (multiples of 32, 64, 256; the
    # LDS panel of the few-row kernel) and on n (multiples of 16, tile counts): seeded random shapes around each switch,
    # every one against the oracle
    rng = wl.rng_for(68, wt)
    ms = [1, 2, 7, 8, 9, 15, 16, 17, 31, 32, 33, 34, 63, 64, 65, 127, 128, 129, 200]
    for m in ms:
        for _ in range(2):
            k = int(rng.choice([32, 64, 96, 256, 288, 512, 1024 + 64, 2048, 4096 + 256, 8192, 8960]))
            n = int(rng.choice([1, 15, 16, 17, 48, 100, 256, 272, 1000, 1536]))
            if m * k * n > 200e6:
                n = 48
            check_mat_mul(ctx, oracle, rng, m, k, n, wt)


# --------------------------------------------------------------------------------- prefill (MFMA) path

@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
@pytest.mark.parametrize("m,k,n", [(128, 1536, 256), (512, 4096, 128), (100, 11008, 96), (33, 2048, 70),
                                   (64, 192, 64), (129, 320, 65), (32, 4096, 512), (17, 1536, 130), (512, 128, 64)])
def test_gemm_mfma(ctx, oracle, wt, m, k, n):
    check_mat_mul(ctx, oracle, wl.rng_for(56, m * 131 + k + n + wt), m, k, n, wt)


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
def test_gemm_mfma_integer_exact(ctx, wt):
    # scales 1.0 and small integers: the block sums come straight out of the matrix cores
    rng = wl.rng_for(57, wt)
    m, k, n = 96, 512, 160
    w = wl.make_weights(rng, n, k, wt).reshape(n, k // 32, -1)
    w[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    w = w.reshape(n, -1)
    a = np.empty((m, k // 32, 34), np.uint8)
    a[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    a[:, :, 2:] = rng.integers(-127, 128, (m, k // 32, 32), dtype=np.int8).view(np.uint8)
    a = a.reshape(m, -1)
    got = ctx.run_mat_mul(a, w, m, k, n, wt)
    _, qa = wl.q8_0_split(a, k)
    _, qw = (wl.q4_0_split if wt == wl.GGML_TYPE_Q4_0 else wl.q8_0_split)(w, k)
    assert np.array_equal(got, (qa.astype(np.int64) @ qw.astype(np.int64).T).astype(np.float32))


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
@pytest.mark.parametrize("m,k,n", [(128, 1536, 256), (129, 320, 65), (100, 11008, 96), (33, 2048, 70), (256, 4096, 512)])
def test_gemm_mfma_with_small_and_large_tiles(ctx, oracle, wt, m, k, n):
    # launches with few output tiles run 32 x 32 tiles per workgroup, the others 64 x 64 (HTPOPS_GEMM_TILE_UNITS forces
    # one or the other): both must meet the oracle on the same inputs
    ctx.set_option("gemm_fp6", 0)
    got = {}
    for units in ("1", "2"):
        ctx.set_option("gemm_tile_units", int(units))
        got[units], _, _ = check_mat_mul(ctx, oracle, wl.rng_for(58, m * 131 + k + n + wt), m, k, n, wt)
    scale = np.abs(got["1"]).max()
    assert np.abs(got["1"] - got["2"]).max() <= 2e-5 * scale


def test_message_shares_one_activation_conversion_between_many_row_matmuls(ctx, oracle):
    # Many-row matmuls of one message that multiply the same activations reuse the converted copy of those
    # activations. The copy must be dropped when a request of the message rewrites the activations, when another
    # activation (or another kernel) takes the workspace, and at the end of the message. Every request must equal its
    # own launch bit for bit.
    rng = wl.rng_for(66, 0)
    m, k = 96, 1536
    wt = wl.GGML_TYPE_Q8_0
    op = api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    ns = [256, 1536, 320]
    ws = [wl.make_weights(rng, n, k, wt) for n in ns]
    x1, x2, xb = (wl.make_activations(rng, m, k) for _ in range(3))
    a1, a2, b = (oracle.quantize_q8_0(x) for x in (x1, x2, xb))
    hx2 = ctx.upload(x2)
    ha, hb = ctx.upload(a1), ctx.upload(b)
    hws = [ctx.upload(w) for w in ws]
    w1row = wl.make_weights(rng, 64, k, wt)  # a one-row matmul in between uses the workspace for something else
    hw1 = ctx.upload(w1row)
    ho1 = ctx.alloc(64 * 4)
    # outputs: 0..2 = A (first contents) x W0..W2, 3..5 = A (second contents) x W0..W2, 6 = B x W0, 7 = A x W1, 8 = A x W2
    out_ns = ns + ns + [ns[0], ns[1], ns[2]]
    houts = [ctx.alloc(m * n * 4) for n in out_ns]
    handles = [hx2, ha, hb, hw1, ho1] + hws + houts
    mm = lambda ho, hact, hw, n: (api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(op, api.mat_mul_params((ho, 0), (hact, 0), (hw, 0), m, k, n)))
    try:
        reqs = [mm(houts[i], ha, hws[i], ns[i]) for i in range(3)]
        reqs += [(api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(api.HTP_OPS_QUANTIZE_Q8_0, api.rms_norm_params((ha, 0), (hx2, 0), k, m)))]
        reqs += [mm(houts[3 + i], ha, hws[i], ns[i]) for i in range(3)]
        reqs += [mm(houts[6], hb, hws[0], ns[0]), mm(houts[7], ha, hws[1], ns[1])]
        reqs += [(api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(op, api.mat_mul_params((ho1, 0), (ha, 0), (hw1, 0), 1, k, 64)))]
        reqs += [mm(houts[8], ha, hws[2], ns[2])]
        msg = api.build_message(reqs)
        for _ in range(2):
            ctx.write(ha, a1)
            assert ctx.process_message(msg) == 0
            assert all(s == 0 for s in api.message_request_states(msg))
            acts = [a1] * 3 + [a2] * 3 + [b, a2, a2]
            wsel = [0, 1, 2, 0, 1, 2, 0, 1, 2]
            for ho, act, wi, n in zip(houts, acts, wsel, out_ns):
                got = ctx.read(ho, np.float32, m * n).reshape(m, n)
                assert np.array_equal(got, ctx.run_mat_mul(act, ws[wi], m, k, n, wt)), "a request differs from its own launch"
            assert np.array_equal(ctx.read(ha, np.uint8, a2.size).reshape(a2.shape), a2)
            assert np.array_equal(ctx.read(ho1, np.float32, 64), ctx.run_mat_mul(a2[:1], w1row, 1, k, 64, wt)[0])
        want64, mag = oracle.mat_mul_q8_0_act_f64(a2, ws[1], m, k, ns[1], wt)
        got = ctx.read(houts[7], np.float32, m * ns[1]).reshape(m, ns[1])
        assert np.all(np.abs(got - want64) <= MATMUL_RTOL * mag)
    finally:
        for h in handles:
            ctx.release(h)


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
@pytest.mark.parametrize("m,k,n", [(2, 256, 16), (8, 256, 48), (3, 512, 4096), (8, 4096, 4096), (5, 11008, 272), (8, 2048 + 256, 1024),
                                   (7, 8960, 1536), (9, 256, 32), (16, 4096, 4096), (12, 2048 + 256, 1040), (13, 8192, 48),
                                   (16, 8960, 64), (11, 11008, 64)])
def test_few_rows_over_repacked_weights(ctx, oracle, wt, m, k, n):
    # 2..16 rows against Q4_0 or Q8_0 weights with n % 16 == 0, k % 256 == 0 run on a copy of the weights repacked into
    # matrix-core operand order (9..16 rows only while 16 activation rows fit the LDS panel: k = 8960 does not,
    # nor 11008; they take the K-sliced kernel). It must meet the oracle, agree with the kernels that read the weights as they are
    # (switch HTPOPS_LANE_ORDER=0) to summation order, and repeat bit for bit.
    rng = wl.rng_for(66, m * 17 + k + n + wt)
    got, x, w = check_mat_mul(ctx, oracle, rng, m, k, n, wt)
    a = oracle.quantize_q8_0(x)
    assert np.array_equal(ctx.run_mat_mul(a, w, m, k, n, wt), got)
    _, mag = oracle.mat_mul_q8_0_act_f64(a, w, m, k, n, wt)
    # one and two weight tiles per workgroup (the launcher picks by the number of tiles; HTPOPS_LANE_ORDER=2 / 3 force
    # one / two) sum the same blocks in different wave order
    for tiles in ("2", "3"):
        ctx.set_option("lane_order", int(tiles))
        forced = ctx.run_mat_mul(a, w, m, k, n, wt)
        assert np.all(np.abs(forced - got) <= 2 * MATMUL_RTOL * mag)
        assert np.array_equal(forced, ctx.run_mat_mul(a, w, m, k, n, wt))
    ctx.set_option("lane_order", 0)
    plain = ctx.run_mat_mul(a, w, m, k, n, wt)
    assert np.all(np.abs(plain - got) <= 2 * MATMUL_RTOL * mag)


def test_few_rows_repacked_weights_extremes_and_cache(ctx, oracle):
    # every weight -8 against every activation -127 with unit scales: 32512 per block, exact in fp32 for k = 512;
    # then the cached repacked copy must follow a rewrite of the weight buffer, and caller-owned memory (nothing
    # cached, the weights are read as they are) must give the same values
    m, k, n = 8, 512, 64
    one = np.array([1.0], np.float16).view(np.uint8)
    w = np.zeros((n, k // 32, 18), np.uint8)
    w[:, :, 0:2] = one
    a = np.empty((m, k // 32, 34), np.uint8)
    a[:, :, 0:2] = one
    a[:, :, 2:] = np.int8(-127).view(np.uint8)
    w, a = w.reshape(n, -1), a.reshape(m, -1)
    ha, hw, ho = ctx.upload(a), ctx.upload(w), ctx.alloc(m * n * 4)
    alias = ctx.register(ctx.device_ptr(hw), w.nbytes)
    try:
        def run(h):
            assert ctx.execute(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0, api.mat_mul_params((ho, 0), (ha, 0), (h, 0), m, k, n)) == 0
            ctx.synchronize()
            return ctx.read(ho, np.float32, m * n).reshape(m, n)
        assert np.array_equal(run(hw), np.full((m, n), 32512.0 * (k // 32), np.float32))
        rng = wl.rng_for(67, 0)
        w2 = wl.make_q4_0_weights(rng, n, k)
        a2 = oracle.quantize_q8_0(wl.make_activations(rng, m, k))
        ctx.write(hw, w2), ctx.write(ha, a2)
        want, mag = oracle.mat_mul_q8_0_act_f64(a2, w2, m, k, n, wl.GGML_TYPE_Q4_0)
        assert np.all(np.abs(run(hw) - want) <= MATMUL_RTOL * mag)
        assert np.all(np.abs(run(alias) - want) <= MATMUL_RTOL * mag)
    finally:
        for h in (alias, ha, hw, ho):
            ctx.release(h)


@pytest.fixture
def fp6_kernel(ctx):
    """Forces the FP6 many-row kernel (by default it only takes shapes that fill the device with whole tiles)."""
    ctx.set_option("gemm_fp6", 1)


# ragged rows / columns / odd K-block counts; one tile shared by many workgroups (k = 4128, 11008); several tiles per
# workgroup is covered by test_gemm_fp6_whole_tiles_on_every_workgroup
@pytest.mark.parametrize("m,k,n", [(64, 64, 128), (128, 128, 128), (100, 96, 200), (33, 4096, 4000), (512, 32, 1024),
                                   (300, 4128, 1000), (129, 320, 257), (512, 4096, 128), (100, 11008, 96)])
def test_gemm_fp6(ctx, oracle, fp6_kernel, m, k, n):
    check_mat_mul(ctx, oracle, wl.rng_for(62, m * 131 + k + n), m, k, n, wl.GGML_TYPE_Q4_0)


def test_gemm_fp6_integer_exact_and_repeatable(ctx, fp6_kernel):
    # scales 1.0: the block sums come straight out of the FP6 matrix instruction (int8 = 16 hi + lo, every part
    # exact), including the extremes -127 x -8; tiles shared between workgroups are added in a fixed order, so
    # repeated launches are bit-identical and the ticket counters come back to zero
    rng = wl.rng_for(63, 0)
    m, k, n = 160, 2048, 300
    w = wl.make_weights(rng, n, k, wl.GGML_TYPE_Q4_0).reshape(n, k // 32, -1)
    w[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    w[0, :, 2:] = 0x00  # all weights -8
    w = w.reshape(n, -1)
    a = np.empty((m, k // 32, 34), np.uint8)
    a[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    a[:, :, 2:] = rng.integers(-127, 128, (m, k // 32, 32), dtype=np.int8).view(np.uint8)
    a[0, :, 2:] = np.int8(-127).view(np.uint8)
    a = a.reshape(m, -1)
    got = ctx.run_mat_mul(a, w, m, k, n, wl.GGML_TYPE_Q4_0)
    _, qa = wl.q8_0_split(a, k)
    _, qw = wl.q4_0_split(w, k)
    assert np.array_equal(got, (qa.astype(np.int64) @ qw.astype(np.int64).T).astype(np.float32))
    assert got[0, 0] == 32512.0 * (k // 32)
    for _ in range(3):
        assert np.array_equal(ctx.run_mat_mul(a, w, m, k, n, wl.GGML_TYPE_Q4_0), got)


def test_gemm_fp6_whole_tiles_on_every_workgroup(ctx, oracle):
    # 2048 x 4096 outputs = 256 tiles of 128 x 256: the shape class the FP6 kernel takes by default; rows are checked
    # against the oracle and against the one-row kernel
    rng = wl.rng_for(64, 0)
    m, k, n = 2048, 1024, 4096 + 256
    w = wl.make_q4_0_weights(rng, n, k)
    a = ctx.run_quantize_q8_0(wl.make_activations(rng, m, k))
    got = ctx.run_mat_mul(a, w, m, k, n, wl.GGML_TYPE_Q4_0)
    rows = [0, 127, 128, 1000, 2047]
    want64, mag = oracle.mat_mul_q8_0_act_f64(a[rows], w, len(rows), k, n, wl.GGML_TYPE_Q4_0)
    assert np.all(np.abs(got[rows] - want64) <= MATMUL_RTOL * mag)
    for r in (5, 1300):
        gemv = ctx.run_mat_mul(a[r:r + 1], w, 1, k, n, wl.GGML_TYPE_Q4_0)
        assert np.abs(gemv[0] - got[r]).max() <= 2e-5 * np.abs(gemv).max()


def test_gemm_fp6_128x128_tiles_ragged_and_exact(ctx, oracle):
    # 1000 x 8200 outputs = 8 x 65 tiles of 128 x 128 (the last ones ragged both ways), from where the FP6 path uses
    # its 128 x 128 kernel; k = 192 is three steps, one pass of its ring. Unit scales first (block sums exact, the
    # extremes -127 x -8 included), then random scales against the oracle on sampled rows and against the one-row
    # kernel.
    rng = wl.rng_for(68, 0)
    m, k, n = 1000, 192, 8200
    w = wl.make_q4_0_weights(rng, n, k).reshape(n, k // 32, -1)
    a = ctx.run_quantize_q8_0(wl.make_activations(rng, m, k)).reshape(m, k // 32, -1)
    w1, a1 = w.copy(), a.copy()
    w1[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    a1[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    w1[n - 1, :, 2:] = 0x00  # all weights -8
    a1[m - 1, :, 2:] = np.int8(-127).view(np.uint8)
    w1, a1, w, a = w1.reshape(n, -1), a1.reshape(m, -1), w.reshape(n, -1), a.reshape(m, -1)
    got = ctx.run_mat_mul(a1, w1, m, k, n, wl.GGML_TYPE_Q4_0)
    _, qa = wl.q8_0_split(a1, k)
    _, qw = wl.q4_0_split(w1, k)
    assert np.array_equal(got, (qa.astype(np.int64) @ qw.astype(np.int64).T).astype(np.float32))
    assert got[m - 1, n - 1] == 32512.0 * (k // 32)
    got = ctx.run_mat_mul(a, w, m, k, n, wl.GGML_TYPE_Q4_0)
    assert np.array_equal(ctx.run_mat_mul(a, w, m, k, n, wl.GGML_TYPE_Q4_0), got)
    rows = [0, 31, 64, 127, 128, 500, 895, 896, 999]
    want64, mag = oracle.mat_mul_q8_0_act_f64(a[rows], w, len(rows), k, n, wl.GGML_TYPE_Q4_0)
    assert np.all(np.abs(got[rows] - want64) <= MATMUL_RTOL * mag)
    for r in (77, 999):
        gemv = ctx.run_mat_mul(a[r:r + 1], w, 1, k, n, wl.GGML_TYPE_Q4_0)
        assert np.abs(gemv[0] - got[r]).max() <= 2e-5 * np.abs(gemv).max()


def test_gemm_weight_conversion_cache_follows_the_weights(ctx, oracle):
    # Many-row matmuls run on weights converted to MFMA operand order. For buffers the context allocated the converted
    # copy is cached and must be dropped when the buffer is rewritten; for caller-owned (registered) memory nothing is
    # cached, so the caller may change it freely between calls.
    rng = wl.rng_for(61, 0)
    m, k, n = 96, 512, 160
    a = oracle.quantize_q8_0(wl.make_activations(rng, m, k))
    w1, w2 = wl.make_q4_0_weights(rng, n, k), wl.make_q4_0_weights(rng, n, k)
    ha, hw, ho = ctx.upload(a), ctx.upload(w1), ctx.alloc(m * n * 4)
    alias = ctx.register(ctx.device_ptr(hw), w1.nbytes)  # the same memory seen as caller-owned
    try:
        def run(h):
            assert ctx.execute(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0, api.mat_mul_params((ho, 0), (ha, 0), (h, 0), m, k, n)) == 0
            ctx.synchronize()
            return ctx.read(ho, np.float32, m * n).reshape(m, n)
        want1, mag1 = oracle.mat_mul_q8_0_act_f64(a, w1, m, k, n, wl.GGML_TYPE_Q4_0)
        want2, mag2 = oracle.mat_mul_q8_0_act_f64(a, w2, m, k, n, wl.GGML_TYPE_Q4_0)
        for _ in range(2):
            assert np.all(np.abs(run(hw) - want1) <= MATMUL_RTOL * mag1)
        ctx.write(hw, w2)
        assert np.all(np.abs(run(hw) - want2) <= MATMUL_RTOL * mag2)
        assert np.all(np.abs(run(alias) - want2) <= MATMUL_RTOL * mag2)
    finally:
        for h in (alias, ha, hw, ho):
            ctx.release(h)


def test_gemm_full_prefill_shape_rows_match_the_decode_kernel(ctx, oracle):
    # M = 512, K = 4096, N = 11008 is too large for the scalar oracle in a test: check (a) a sample of rows against
    # the oracle and (b) every row against the GEMV kernel of the same row (independent kernel, same arithmetic)
    rng = wl.rng_for(2, 0)
    m, k, n = 512, 4096, 11008
    w = wl.make_q4_0_weights(rng, n, k)
    x = wl.make_activations(rng, m, k)
    a = oracle.quantize_q8_0(x)
    print("full prefill shape", flush=True)
    got = ctx.run_mat_mul(a, w, m, k, n, wl.GGML_TYPE_Q4_0)
    rows = [0, 1, 31, 32, 255, 256, 511]
    want64, mag = oracle.mat_mul_q8_0_act_f64(a[rows], w, len(rows), k, n, wl.GGML_TYPE_Q4_0)
    assert np.all(np.abs(got[rows] - want64) <= MATMUL_RTOL * mag)
    for r in (5, 130, 300, 500):
        gemv = ctx.run_mat_mul(a[r:r + 1], w, 1, k, n, wl.GGML_TYPE_Q4_0)
        scale = np.abs(gemv).max()
        assert np.abs(gemv[0] - got[r]).max() <= 2e-5 * scale


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
@pytest.mark.parametrize("m", [1, 2, 8, 16, 40])
def test_mat_mul_with_activations_at_a_4_byte_aligned_offset(ctx, oracle, wt, m):
    # the request only promises 2-byte aligned activations; kernels that want 16-byte alignment (the DMA of the
    # repacked-weight kernel) must not be picked, alone or inside a message's grouped launch
    rng = wl.rng_for(71, wt * 100 + m)
    k, n = 1024, 256
    op = api.HTP_OPS_MAT_MUL_Q4_0_Q8_0 if wt == wl.GGML_TYPE_Q4_0 else api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    w = wl.make_weights(rng, n, k, wt)
    a = oracle.quantize_q8_0(wl.make_activations(rng, m, k))
    want, mag = oracle.mat_mul_q8_0_act_f64(a, w, m, k, n, wt)
    hw, ho, ho2 = ctx.upload(w), ctx.alloc(m * n * 4), ctx.alloc(m * n * 4)
    ha = ctx.alloc(a.nbytes + 64)
    try:
        for off in (4, 8, 2):
            ctx.write(ha, a, offset=off)
            print("offset activations m=%d wt=%d off=%d" % (m, wt, off), flush=True)
            assert ctx.execute(op, api.mat_mul_params((ho, 0), (ha, off), (hw, 0), m, k, n)) == 0, ctx.last_error()
            ctx.synchronize()
            got = ctx.read(ho, np.float32, m * n).reshape(m, n)
            assert np.all(np.abs(got - want) <= MATMUL_RTOL * mag)
            msg = api.build_message([(api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(op, api.mat_mul_params((h, 0), (ha, off), (hw, 0), m, k, n)))
                                     for h in (ho, ho2)])
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0, 0], ctx.last_error()
            for h in (ho, ho2):
                got = ctx.read(h, np.float32, m * n).reshape(m, n)
                assert np.all(np.abs(got - want) <= MATMUL_RTOL * mag)
    finally:
        for h in (hw, ho, ho2, ha):
            ctx.release(h)


def test_buffer_invalidate_drops_converted_weight_copies(ctx, oracle):
    # an owned weight buffer rewritten through its device address (here by a second context that has the address
    # registered) keeps its converted copy until the caller says so
    rng = wl.rng_for(72, 0)
    m, k, n = 8, 512, 64
    w1, w2 = wl.make_q4_0_weights(rng, n, k), wl.make_q4_0_weights(rng, n, k)
    a = oracle.quantize_q8_0(wl.make_activations(rng, m, k))
    ha, hw, ho = ctx.upload(a), ctx.upload(w1), ctx.alloc(m * n * 4)
    try:
        def run():
            assert ctx.execute(api.HTP_OPS_MAT_MUL_Q4_0_Q8_0, api.mat_mul_params((ho, 0), (ha, 0), (hw, 0), m, k, n)) == 0
            ctx.synchronize()
            return ctx.read(ho, np.float32, m * n).reshape(m, n)
        first = run()
        want2, mag2 = oracle.mat_mul_q8_0_act_f64(a, w2, m, k, n, wl.GGML_TYPE_Q4_0)
        with api.Context(device=0) as other:
            alias = other.register(ctx.device_ptr(hw), w2.nbytes)
            other.write(alias, w2)
        assert np.array_equal(run(), first)          # the repacked copy of the old weights is still in use
        assert ctx.invalidate(hw) == 0
        assert np.all(np.abs(run() - want2) <= MATMUL_RTOL * mag2)
        assert ctx.invalidate(987654) == -1
    finally:
        for h in (ha, hw, ho):
            ctx.release(h)


def _mm(op, ho, ha, hw, m, k, n, out_off=0, act_off=0):
    return (api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(op, api.mat_mul_params((ho, out_off), (ha, act_off), (hw, 0), m, k, n)))


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
def test_message_groups_independent_gemvs_of_different_activations(ctx, oracle, wt):
    # one-row matmuls whose inputs and outputs are all independent run as ONE launch even when they read different
    # activation buffers and have different k (the reference runs them one after the other, commu.c:91-114; with no
    # data dependency between them the order cannot be observed). Every request must equal its own launch bit for bit.
    rng = wl.rng_for(73, wt)
    op = api.HTP_OPS_MAT_MUL_Q4_0_Q8_0 if wt == wl.GGML_TYPE_Q4_0 else api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    shapes = [(256, 1536), (272, 1536), (100, 4096), (1536, 8960), (33, 64), (640, 11008), (7, 2048)]   # (n, k)
    ws = [wl.make_weights(rng, n, k, wt) for n, k in shapes]
    acts = [oracle.quantize_q8_0(wl.make_activations(rng, 1, k)) for _, k in shapes]
    acts[1] = acts[0]  # two members share an activation row
    has = [ctx.upload(a) for a in acts]
    ctx.release(has[1])
    has[1] = has[0]
    hws = [ctx.upload(w) for w in ws]
    hos = [ctx.alloc(n * 4) for n, _ in shapes]
    try:
        msg = api.build_message([_mm(op, ho, ha, hw, 1, k, n) for ho, ha, hw, (n, k) in zip(hos, has, hws, shapes)])
        for _ in range(2):
            for ho, (n, _) in zip(hos, shapes):
                ctx.write(ho, np.full(n, np.nan, np.float32))
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0] * len(shapes), ctx.last_error()
            assert ctx.last_message_submissions() == 1
            for ho, a, w, (n, k) in zip(hos, acts, ws, shapes):
                got = ctx.read(ho, np.float32, n)
                assert np.array_equal(got, ctx.run_mat_mul(a, w, 1, k, n, wt)[0]), "a request differs from its own launch"
                want, mag = oracle.mat_mul_q8_0_act_f64(a, w, 1, k, n, wt)
                assert np.all(np.abs(got - want[0]) <= MATMUL_RTOL * mag[0])
    finally:
        for h in set(has) | set(hws) | set(hos):
            ctx.release(h)


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
def test_message_groups_independent_many_row_matmuls(ctx, oracle, wt):
    # Many-row matmuls on small output tiles (the projections of a small model at a prefill chunk of 128 rows) share
    # one launch for the products and one for the activation conversions when nothing orders them; members read
    # different activation matrices with different k. Every request must equal its own launch bit for bit. A request
    # that writes what an earlier one reads ends the group.
    rng = wl.rng_for(75, wt)
    op = api.HTP_OPS_MAT_MUL_Q4_0_Q8_0 if wt == wl.GGML_TYPE_Q4_0 else api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    m = 100
    shapes = [(192, 1536), (64, 1536), (40, 1536), (192, 1536), (1120, 1536), (1120, 1536), (192, 8960)]   # (n, k)
    act_of = [0, 0, 0, 1, 2, 2, 3]
    act_k = [1536, 1536, 1536, 8960]
    ws = [wl.make_weights(rng, n, k, wt) for n, k in shapes]
    acts = [oracle.quantize_q8_0(wl.make_activations(rng, m, k)) for k in act_k]
    has = [ctx.upload(a) for a in acts]
    hws = [ctx.upload(w) for w in ws]
    hos = [ctx.alloc(m * n * 4) for n, _ in shapes]
    try:
        reqs = [_mm(op, ho, has[g], hw, m, k, n) for ho, g, hw, (n, k) in zip(hos, act_of, hws, shapes)]
        msg = api.build_message(reqs)
        for _ in range(2):
            for ho, (n, _) in zip(hos, shapes):
                ctx.write(ho, np.full(m * n, np.nan, np.float32))
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0] * len(shapes), ctx.last_error()
            assert ctx.last_message_submissions() == 1
            for ho, g, w, (n, k) in zip(hos, act_of, ws, shapes):
                got = ctx.read(ho, np.float32, m * n).reshape(m, n)
                assert np.array_equal(got, ctx.run_mat_mul(acts[g], w, m, k, n, wt)), "a request differs from its own launch"
                want, mag = oracle.mat_mul_q8_0_act_f64(acts[g], w, m, k, n, wt)
                assert np.all(np.abs(got - want) <= MATMUL_RTOL * mag)
        # the same output twice: two launches, the later request wins
        msg2 = api.build_message([_mm(op, hos[0], has[0], hws[0], m, 1536, 192), _mm(op, hos[0], has[1], hws[3], m, 1536, 192)])
        assert ctx.process_message(msg2) == 0
        assert ctx.last_message_submissions() == 2
        assert np.array_equal(ctx.read(hos[0], np.float32, m * 192).reshape(m, 192),
                              ctx.run_mat_mul(acts[1], ws[3], m, 1536, 192, wt))
    finally:
        for h in has + hws + hos:
            ctx.release(h)


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
@pytest.mark.parametrize("m", [2, 3, 8])
def test_message_groups_independent_few_row_matmuls(ctx, oracle, wt, m):
    # Few-row matmuls of the same k that nothing orders share a launch although they read different activation rows
    # (2, 3 rows: the weight stream with the rows in registers, or for Q4_0 members that fit it the kernel over
    # repacked weights, one launch of each kind; 8: the kernel over repacked weights for Q4_0, one launch per set of
    # rows otherwise). Every request must equal its own launch bit for bit.
    # With two and three rows the members may also differ in k (one, two and three waves per weight row here).
    rng = wl.rng_for(76, wt * 10 + m)
    op = api.HTP_OPS_MAT_MUL_Q4_0_Q8_0 if wt == wl.GGML_TYPE_Q4_0 else api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    ns = [256, 64, 48, 256, 1000, 130]
    act_of = [0, 0, 0, 1, 2, 3]
    ks = [1024] * 4 + ([1024, 1024] if m == 8 else [8192, 11008])
    act_k = [1024, 1024, ks[4], ks[5]]
    ws = [wl.make_weights(rng, n, k, wt) for n, k in zip(ns, ks)]
    acts = [oracle.quantize_q8_0(wl.make_activations(rng, m, k)) for k in act_k]
    has = [ctx.upload(a) for a in acts]
    hws = [ctx.upload(w) for w in ws]
    hos = [ctx.alloc(m * n * 4) for n in ns]
    try:
        msg = api.build_message([_mm(op, ho, has[g], hw, m, k, n) for ho, g, hw, n, k in zip(hos, act_of, hws, ns, ks)])
        for _ in range(2):
            for ho, n in zip(hos, ns):
                ctx.write(ho, np.full(m * n, np.nan, np.float32))
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0] * len(ns), ctx.last_error()
            assert ctx.last_message_submissions() == 1
            for ho, g, w, n, k in zip(hos, act_of, ws, ns, ks):
                got = ctx.read(ho, np.float32, m * n).reshape(m, n)
                assert np.array_equal(got, ctx.run_mat_mul(acts[g], w, m, k, n, wt)), "a request differs from its own launch"
                want, mag = oracle.mat_mul_q8_0_act_f64(acts[g], w, m, k, n, wt)
                assert np.all(np.abs(got - want) <= MATMUL_RTOL * mag)
    finally:
        for h in has + hws + hos:
            ctx.release(h)


@pytest.mark.parametrize("m", [2, 5, 8])
def test_message_groups_few_row_q4_0_matmuls_of_different_k(ctx, oracle, m):
    # 2..8 rows against Q4_0 weights with n % 16 == 0, k % 256 == 0 take the two-blocks-per-instruction kernel, whose
    # members bring their own k: matmuls over rows of different length share a launch (the longest rows size its LDS;
    # k = 11008 leaves one workgroup per compute unit, which also changes how far ahead the weights are requested). A
    # member of the first one's k that does not fit that kernel (n = 40) still joins the batch, and runs on the kernel
    # that reads the weights as they are. Every request must equal its own launch bit for bit and meet the oracle.
    ctx.set_option("gemv_rows_kernel", 0)  # (two and three rows would otherwise stay on the decode kernel's stream)
    rng = wl.rng_for(77, m)
    wt, op = wl.GGML_TYPE_Q4_0, api.HTP_OPS_MAT_MUL_Q4_0_Q8_0
    ks = [512, 2048, 11008, 256, 2048, 512]
    ns = [64, 48, 32, 16, 1008, 40]
    ws = [wl.make_weights(rng, n, k, wt) for n, k in zip(ns, ks)]
    acts = [oracle.quantize_q8_0(wl.make_activations(rng, m, k)) for k in ks]
    has = [ctx.upload(a) for a in acts]
    hws = [ctx.upload(w) for w in ws]
    hos = [ctx.alloc(m * n * 4) for n in ns]
    try:
        msg = api.build_message([_mm(op, ho, ha, hw, m, k, n) for ho, ha, hw, n, k in zip(hos, has, hws, ns, ks)])
        for _ in range(2):
            for ho, n in zip(hos, ns):
                ctx.write(ho, np.full(m * n, np.nan, np.float32))
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0] * len(ns), ctx.last_error()
            assert ctx.last_message_submissions() == 1
            for ho, a, w, n, k in zip(hos, acts, ws, ns, ks):
                got = ctx.read(ho, np.float32, m * n).reshape(m, n)
                assert np.array_equal(got, ctx.run_mat_mul(a, w, m, k, n, wt)), "a request differs from its own launch"
                want, mag = oracle.mat_mul_q8_0_act_f64(a, w, m, k, n, wt)
                assert np.all(np.abs(got - want) <= MATMUL_RTOL * mag)
    finally:
        for h in has + hws + hos:
            ctx.release(h)


def test_message_groups_many_row_matmuls_over_the_same_rows(ctx, oracle):
    # Independent many-row Q4_0 matmuls over the SAME activation rows (q/k/v or gate/up of a prefill chunk) whose
    # weights live in buffers of the context share the launch of the FP6-tile kernel (one grid keeps the compute units
    # fed to the end). Every request must equal its own launch bit for bit; one that reads other rows starts a new launch.
    wt, op = wl.GGML_TYPE_Q4_0, api.HTP_OPS_MAT_MUL_Q4_0_Q8_0
    fp6 = ctx.get_option("gemm_fp6") != 0   # (switched off, every request is a launch of the int8 kernel)
    rng = wl.rng_for(81, 0)
    m, k = 512, 1024
    ns = [4096, 3072, 6144, 3072]
    act_of = [0, 0, 0, 1]
    ws = [wl.make_weights(rng, n, k, wt) for n in ns]
    acts = [oracle.quantize_q8_0(wl.make_activations(rng, m, k)) for _ in range(2)]
    has, hws = [ctx.upload(a) for a in acts], [ctx.upload(w) for w in ws]
    hos = [ctx.alloc(m * n * 4) for n in ns]
    try:
        msg = api.build_message([_mm(op, ho, has[g], hw, m, k, n) for ho, g, hw, n in zip(hos, act_of, hws, ns)])
        for _ in range(2):
            for ho, n in zip(hos, ns):
                ctx.write(ho, np.full(m * n, np.nan, np.float32))
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0] * len(ns), ctx.last_error()
            assert ctx.last_message_submissions() == (2 if fp6 else 4)
            for ho, g, w, n in zip(hos, act_of, ws, ns):
                got = ctx.read(ho, np.float32, m * n).reshape(m, n)
                assert np.array_equal(got, ctx.run_mat_mul(acts[g], w, m, k, n, wt)), "a request differs from its own launch"
                rows = [0, 31, 32, 300, m - 1]
                cols = np.unique(np.linspace(0, n - 1, 40).astype(int))
                want, mag = oracle.mat_mul_q8_0_act_f64(acts[g][rows], w[cols], len(rows), k, len(cols), wt)
                assert np.all(np.abs(got[np.ix_(rows, cols)] - want) <= MATMUL_RTOL * mag)
        # ten requests over the same rows: a launch takes eight, the ninth starts another that finds the rows converted
        more = [ctx.alloc(m * ns[1] * 4) for _ in range(10)]
        try:
            msg = api.build_message([_mm(op, ho, has[0], hws[1], m, k, ns[1]) for ho in more])
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0] * 10, ctx.last_error()
            assert ctx.last_message_submissions() == (2 if fp6 else 10)
            want = ctx.run_mat_mul(acts[0], ws[1], m, k, ns[1], wt)
            for ho in more:
                assert np.array_equal(ctx.read(ho, np.float32, m * ns[1]).reshape(m, ns[1]), want)
        finally:
            for h in more:
                ctx.release(h)
    finally:
        for h in has + hws + hos:
            ctx.release(h)


def _norm_q(hq, hx, hg, k, rows, eps):
    return (api.REQUEST_TYPE_OP_COMPUTE,
            api.op_compute_request(api.HTP_OPS_RMS_NORM_QUANTIZE_Q8_0, api.rms_norm_ex_params((hq, 0), (hx, 0), (hg, 0), k, rows, eps)))


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
@pytest.mark.parametrize("k,wide", [(64, 0), (1024, 0), (1536, 0), (4096, 0), (4096, 2), (4096, 4), (8192, 0), (11008, 0)])
@pytest.mark.parametrize("with_weight", [True, False])
def test_message_decode_chain_in_one_launch(ctx, oracle, wt, k, wide, with_weight):
    # RMSNorm -> Q8_0 of one row followed by the one-row matmuls that read it (q/k/v or gate/up of a decoder layer) is one
    # launch: every workgroup makes the row for itself. The Q8_0 row written must be the bytes of the op run alone, and
    # every product the bits of its own launch over that row (`wide` = 2: gate and up of a 7B layer, 32 weight rows per
    # workgroup instead of 16). Rows longer than 4096 and launches that would still need more than about a thousand
    # workgroups (`wide` = 4 matrices of 11008 rows) keep the two launches, where that is faster.
    rng = wl.rng_for(77, wt * 100000 + k * 8 + int(with_weight) * 4 + wide // 2)
    op = api.HTP_OPS_MAT_MUL_Q4_0_Q8_0 if wt == wl.GGML_TYPE_Q4_0 else api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    ns = [11008] * wide if wide else [256, 1000, 48]
    launches = 1 if k <= 4096 and wide < 4 else 2
    x = wl.make_activations(rng, 1, k)
    g = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32) if with_weight else None
    ws = [wl.make_weights(rng, n, k, wt) for n in ns]
    hx, hq = ctx.upload(x), ctx.alloc(k // 32 * 34)
    hg = ctx.upload(g) if with_weight else -1
    hws, hos = [ctx.upload(w) for w in ws], [ctx.alloc(n * 4) for n in ns]
    try:
        q_alone = ctx.run_rms_norm(x, g, 1e-6, quantize=True)
        want_q = oracle.quantize_q8_0(oracle.rms_norm(x, g if with_weight else np.ones(k, np.float32), 1e-6))
        assert np.count_nonzero(q_alone != want_q) <= q_alone.size // 100   # (last-bit differences before rounding only)
        msg = api.build_message([_norm_q(hq, hx, hg, k, 1, 1e-6)] + [_mm(op, ho, hq, hw, 1, k, n) for ho, hw, n in zip(hos, hws, ns)])
        for _ in range(2):
            ctx.write(hq, np.full(k // 32 * 34, 0xA5, np.uint8))
            for ho, n in zip(hos, ns):
                ctx.write(ho, np.full(n, np.nan, np.float32))
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0] * (1 + len(ns)), ctx.last_error()
            assert ctx.last_message_submissions() == launches
            assert np.array_equal(ctx.read(hq, np.uint8, k // 32 * 34), q_alone[0]), "the row differs from the op run alone"
            for ho, w, n in zip(hos, ws, ns):
                got = ctx.read(ho, np.float32, n)
                assert np.array_equal(got, ctx.run_mat_mul(q_alone, w, 1, k, n, wt)[0]), "a request differs from its own launch"
                want, mag = oracle.mat_mul_q8_0_act_f64(q_alone, w, 1, k, n, wt)
                assert np.all(np.abs(got - want[0]) <= MATMUL_RTOL * mag[0])
    finally:
        for h in [hx, hq] + hws + hos + ([hg] if with_weight else []):
            ctx.release(h)


@pytest.mark.parametrize("wt", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
@pytest.mark.parametrize("k", [128, 1536, 4096, 8192])
def test_message_quantize_then_projections_in_one_launch(ctx, oracle, wt, k):
    # A one-row Q8_0 quantization (op 14: the attention output on its way to the o projection) followed by one-row
    # matmuls over the row it writes runs inside their launch like the RMSNorm + Q8_0 request does: the row written is the
    # quantizer's, bit for bit (which is the oracle's), and so are the products. Rows longer than 4096 keep two launches.
    rng = wl.rng_for(80, wt * 100000 + k)
    op = api.HTP_OPS_MAT_MUL_Q4_0_Q8_0 if wt == wl.GGML_TYPE_Q4_0 else api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    ns = [4096, 48]
    x = wl.make_activations(rng, 1, k)
    ws = [wl.make_weights(rng, n, k, wt) for n in ns]
    hx, hq = ctx.upload(x), ctx.alloc(k // 32 * 34)
    hws, hos = [ctx.upload(w) for w in ws], [ctx.alloc(n * 4) for n in ns]
    try:
        want_q = oracle.quantize_q8_0(x)
        quant = (api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(api.HTP_OPS_QUANTIZE_Q8_0, api.rms_norm_params((hq, 0), (hx, 0), k, 1)))
        msg = api.build_message([quant] + [_mm(op, ho, hq, hw, 1, k, n) for ho, hw, n in zip(hos, hws, ns)])
        for _ in range(2):
            ctx.write(hq, np.full(k // 32 * 34, 0xA5, np.uint8))
            for ho, n in zip(hos, ns):
                ctx.write(ho, np.full(n, np.nan, np.float32))
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0] * (1 + len(ns)), ctx.last_error()
            assert ctx.last_message_submissions() == (1 if k <= 4096 else 2)
            assert np.array_equal(ctx.read(hq, np.uint8, k // 32 * 34), want_q[0]), "the row differs from the quantizer's"
            for ho, w, n in zip(hos, ws, ns):
                got = ctx.read(ho, np.float32, n)
                assert np.array_equal(got, ctx.run_mat_mul(want_q, w, 1, k, n, wt)[0]), "a request differs from its own launch"
    finally:
        for h in [hx, hq] + hws + hos:
            ctx.release(h)


def test_message_decode_chain_keeps_its_own_launch_when_it_must(ctx, oracle):
    # The RMSNorm -> Q8_0 request runs by itself, in order, when what follows cannot share its launch: a matmul over another
    # row, a matmul whose output lands on the request's input, several rows, the end of the message; and matmuls that
    # read the new row after a request that could not join still see it.
    wt, op = wl.GGML_TYPE_Q8_0, api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    rng = wl.rng_for(78, 0)
    k, n = 1024, 256
    x = wl.make_activations(rng, 2, k)
    g = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    w, w2 = wl.make_weights(rng, n, k, wt), wl.make_weights(rng, n, k, wt)
    other = oracle.quantize_q8_0(wl.make_activations(rng, 1, k))
    hx, hg, hw, hw2, hother = ctx.upload(x), ctx.upload(g), ctx.upload(w), ctx.upload(w2), ctx.upload(other)
    hq, ho, ho2 = ctx.alloc(2 * (k // 32) * 34), ctx.alloc(2 * n * 4), ctx.alloc(n * 4)
    hxo = ctx.alloc(k * 4)                                     # a row that a matmul overwrites (n = 256 of its floats)
    try:
        q1 = ctx.run_rms_norm(x[:1], g, 1e-6, quantize=True)
        q2 = ctx.run_rms_norm(x, g, 1e-6, quantize=True)

        def run(reqs, submissions):
            ctx.write(hq, np.full(2 * (k // 32) * 34, 0xA5, np.uint8))
            ctx.write(hxo, x[0])
            msg = api.build_message(reqs)
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0] * len(reqs), ctx.last_error()
            assert ctx.last_message_submissions() == submissions

        # another row first, then the new one: the norm by itself, then the two matmuls together
        run([_norm_q(hq, hx, hg, k, 1, 1e-6), _mm(op, ho2, hother, hw2, 1, k, n), _mm(op, ho, hq, hw, 1, k, n)], 2)
        assert np.array_equal(ctx.read(hq, np.uint8, k // 32 * 34), q1[0])
        assert np.array_equal(ctx.read(ho, np.float32, n), ctx.run_mat_mul(q1, w, 1, k, n, wt)[0])
        assert np.array_equal(ctx.read(ho2, np.float32, n), ctx.run_mat_mul(other, w2, 1, k, n, wt)[0])
        # the new row, then a request over another row: the first two share a launch, the third has its own
        run([_norm_q(hq, hx, hg, k, 1, 1e-6), _mm(op, ho, hq, hw, 1, k, n), _mm(op, ho2, hother, hw2, 1, k, n)], 2)
        assert np.array_equal(ctx.read(ho, np.float32, n), ctx.run_mat_mul(q1, w, 1, k, n, wt)[0])
        assert np.array_equal(ctx.read(ho2, np.float32, n), ctx.run_mat_mul(other, w2, 1, k, n, wt)[0])
        # the matmul writes over the row that the norm reads: norm first, then the matmul
        run([_norm_q(hq, hxo, hg, k, 1, 1e-6), _mm(op, hxo, hq, hw, 1, k, n)], 2)
        assert np.array_equal(ctx.read(hq, np.uint8, k // 32 * 34), q1[0])
        assert np.array_equal(ctx.read(hxo, np.float32, n), ctx.run_mat_mul(q1, w, 1, k, n, wt)[0])
        # two rows: the ordinary two launches
        run([_norm_q(hq, hx, hg, k, 2, 1e-6), _mm(op, ho, hq, hw, 2, k, n)], 2)
        assert np.array_equal(ctx.read(hq, np.uint8, 2 * (k // 32) * 34), q2.reshape(-1))
        assert np.array_equal(ctx.read(ho, np.float32, 2 * n).reshape(2, n), ctx.run_mat_mul(q2, w, 2, k, n, wt))
        # nothing behind it
        run([_norm_q(hq, hx, hg, k, 1, 1e-6)], 1)
        assert np.array_equal(ctx.read(hq, np.uint8, k // 32 * 34), q1[0])
        # two chains in one message: each is one launch
        run([_norm_q(hq, hx, hg, k, 1, 1e-6), _mm(op, ho, hq, hw, 1, k, n),
             _norm_q(hq, hx, hg, k, 1, 1e-6), _mm(op, ho2, hq, hw2, 1, k, n)], 2)
        assert np.array_equal(ctx.read(ho, np.float32, n), ctx.run_mat_mul(q1, w, 1, k, n, wt)[0])
        assert np.array_equal(ctx.read(ho2, np.float32, n), ctx.run_mat_mul(q1, w2, 1, k, n, wt)[0])
    finally:
        for h in (hx, hg, hw, hw2, hother, hq, ho, ho2, hxo):
            ctx.release(h)


@pytest.mark.parametrize("seed", range(60))
def test_message_batching_equals_one_request_at_a_time(ctx, seed):
    # Random programs over a small pool of buffers, so that requests read what earlier ones wrote, overwrite what earlier
    # ones read, and write the same bytes twice: RMSNorm -> Q8_0 (op 13), Q8_0 quantization (op 14) and matmuls of 1, 2,
    # 3, 5, 8 and 64 rows whose outputs feed later norms -- or land on Q8_0 rows that later matmuls read as they are (whatever
    # those bytes mean as blocks: both walks must agree on every byte, NaNs included). The walk of ONE message (which
    # shares launches where it may) must leave every buffer exactly as one message per request does, where nothing can
    # share.
    rng = wl.rng_for(79, seed)
    k = n = (256, 512, 1024)[seed % 3]        # outputs are as long as inputs, so that they can be normalized again
    rows = 72
    wt = wl.GGML_TYPE_Q4_0 if seed % 2 == 0 else wl.GGML_TYPE_Q8_0
    op_mm = api.HTP_OPS_MAT_MUL_Q4_0_Q8_0 if wt == wl.GGML_TYPE_Q4_0 else api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    q_row = k // 32 * 34
    f_init = [wl.make_activations(rng, rows, k) for _ in range(4)]
    q_init = [np.zeros(rows * q_row, np.uint8) for _ in range(2)]   # (zero scales and values: finite whatever reads them)
    ws = [wl.make_weights(rng, n, k, wt) for _ in range(4)]
    g = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    hf, hq = [ctx.upload(x) for x in f_init], [ctx.upload(x) for x in q_init]
    hw, hg = [ctx.upload(w) for w in ws], ctx.upload(g)
    try:
        reqs = []
        for _ in range(16):
            kind = rng.integers(0, 10)
            m = int(rng.choice([1, 1, 1, 1, 2, 3, 5, 8, 64]))
            row = int(rng.integers(0, rows - m + 1))          # requests work on rows row .. row + m - 1 of their buffers
            f, q = int(rng.integers(0, len(hf))), int(rng.integers(0, len(hq)))
            if kind < 3:
                weight = (hg, 0) if rng.integers(0, 2) else (-1, 0)
                reqs.append((api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(
                    api.HTP_OPS_RMS_NORM_QUANTIZE_Q8_0,
                    api.rms_norm_ex_params((hq[q], row * q_row), (hf[f], row * k * 4), weight, k, m, 1e-6))))
            elif kind < 4:
                reqs.append((api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(
                    api.HTP_OPS_QUANTIZE_Q8_0, api.rms_norm_params((hq[q], row * q_row), (hf[f], row * k * 4), k, m))))
            else:
                # the output rows start wherever they fit: m x n floats somewhere in the fp32 buffer
                out_row = int(rng.integers(0, rows - m + 1))
                ho, out_off = hf[f], out_row * n * 4
                if m <= 2 and rng.integers(0, 5) < 2:    # m x n floats over the Q8_0 rows of another (or the same) buffer
                    qo, off = int(rng.integers(0, len(hq))), 4 * int(rng.integers(0, (rows * q_row - m * n * 4) // 4 + 1))
                    # (not over the rows this very request reads: a request that overwrites its own input while its
                    # workgroups still read it has no defined result)
                    if qo != q or off + m * n * 4 <= row * q_row or off >= (row + m) * q_row:
                        ho, out_off = hq[qo], off
                reqs.append(_mm(op_mm, ho, hq[q], hw[int(rng.integers(0, len(hw)))], m, k, n,
                                out_off=out_off, act_off=row * q_row))

        def run(messages):
            for h, x in zip(hf + hq, f_init + q_init):
                ctx.write(h, x)
            for msg in messages:
                assert ctx.process_message(msg) == 0
                assert all(st == 0 for st in api.message_request_states(msg)), ctx.last_error()
            return [ctx.read(h, np.uint8, ctx.size(h)) for h in hf + hq]

        one_by_one = run([api.build_message([r]) for r in reqs])
        together = run([api.build_message(reqs)])
        assert ctx.last_message_submissions() <= len(reqs)
        for i, (a, b) in enumerate(zip(one_by_one, together)):
            assert np.array_equal(a, b), "buffer %d differs between the two walks" % i
    finally:
        for h in hf + hq + hw + [hg]:
            ctx.release(h)


def test_message_keeps_dependent_gemvs_in_order(ctx, oracle):
    # Requests with a data dependency must not share a launch. (1) read-after-write: request 1's fp32 output bytes are
    # request 2's Q8_0 activation row (unit scales and small integers make those bytes finite Q8_0 blocks);
    # (2) write-after-read: request 3 reads activation A, request 4 writes its output over A;
    # (3) write-after-write: requests 5 and 6 write the same output, the later one wins.
    wt, op = wl.GGML_TYPE_Q8_0, api.HTP_OPS_MAT_MUL_Q8_0_Q8_0
    rng = wl.rng_for(74, 0)
    one = np.array([1.0], np.float16).view(np.uint8)
    k1, n1 = 256, 272                      # 272 floats = 1088 bytes = 32 Q8_0 blocks -> k2 = 1024
    k2, n2 = 1024, 96
    w1 = wl.make_q8_0_weights(rng, n1, k1).reshape(n1, k1 // 32, 34)
    w1[:, :, 0:2] = one
    w1[:, :, 2:] = rng.integers(-3, 4, (n1, k1 // 32, 32), dtype=np.int8).view(np.uint8)
    w1 = w1.reshape(n1, -1)
    a1 = np.empty((1, k1 // 32, 34), np.uint8)
    a1[:, :, 0:2] = one
    a1[:, :, 2:] = rng.integers(-3, 4, (1, k1 // 32, 32), dtype=np.int8).view(np.uint8)
    a1 = a1.reshape(1, -1)
    w2 = wl.make_q8_0_weights(rng, n2, k2)
    stale = oracle.quantize_q8_0(wl.make_activations(rng, 1, k2))       # what the buffer holds before request 1 runs
    a3 = oracle.quantize_q8_0(wl.make_activations(rng, 1, k2))
    w4 = wl.make_q8_0_weights(rng, 272, k1)                              # 272 floats overwrite the 1088 bytes of a3
    h = {name: ctx.upload(x) for name, x in dict(w1=w1, a1=a1, w2=w2, mid=stale, a3=a3, w4=w4).items()}
    h.update(o2=ctx.alloc(n2 * 4), o3=ctx.alloc(n2 * 4), o5=ctx.alloc(n2 * 4))
    try:
        msg = api.build_message([
            _mm(op, h["mid"], h["a1"], h["w1"], 1, k1, n1),       # 1
            _mm(op, h["o2"], h["mid"], h["w2"], 1, k2, n2),       # 2 reads what 1 writes
            _mm(op, h["o3"], h["a3"], h["w2"], 1, k2, n2),        # 3
            _mm(op, h["a3"], h["a1"], h["w4"], 1, k1, 272),       # 4 overwrites what 3 reads
            _mm(op, h["o5"], h["a3"], h["w2"], 1, k2, n2),        # 5 reads what 4 wrote
            _mm(op, h["o5"], h["a1"], h["w1"], 1, k1, n2),        # 6 overwrites 5's output
        ])
        for _ in range(3):
            ctx.write(h["mid"], stale), ctx.write(h["a3"], a3)
            assert ctx.process_message(msg) == 0
            assert api.message_request_states(msg) == [0] * 6, ctx.last_error()
            assert ctx.last_message_submissions() >= 4
            out1 = ctx.read(h["mid"], np.float32, n1)
            _, q1 = wl.q8_0_split(a1, k1)
            _, qw1 = wl.q8_0_split(w1, k1)
            assert np.array_equal(out1, (q1.astype(np.int64) @ qw1.astype(np.int64).T)[0].astype(np.float32))
            act2 = out1.view(np.uint8).reshape(1, -1)
            assert np.array_equal(ctx.read(h["o2"], np.float32, n2), ctx.run_mat_mul(act2, w2, 1, k2, n2, wt)[0])
            want2, mag2 = oracle.mat_mul_q8_0_act_f64(act2, w2, 1, k2, n2, wt)
            assert np.all(np.isfinite(want2)) and np.all(np.abs(ctx.read(h["o2"], np.float32, n2) - want2[0]) <= MATMUL_RTOL * mag2[0])
            assert np.array_equal(ctx.read(h["o3"], np.float32, n2), ctx.run_mat_mul(a3, w2, 1, k2, n2, wt)[0])
            out4 = ctx.read(h["a3"], np.float32, 272)
            assert np.array_equal(out4, ctx.run_mat_mul(a1, w4, 1, k1, 272, wt)[0])
            assert np.array_equal(ctx.read(h["o5"], np.float32, n2), out1[:n2])
    finally:
        for v in h.values():
            ctx.release(v)


def test_a_failed_device_allocation_is_reported_and_the_context_stays_usable(ctx, oracle):
    # Split-KV partials of a decode attention over 2^31 - 64 keys and 4096 heads would need some 70 TB of workspace:
    # the allocation fails before anything is launched, the call returns HTPOPS_ERR_HIP with the runtime's message,
    # and the error is not left behind for the next op to trip over.
    h = ctx.alloc(4096)
    try:
        p = ctx.device_ptr(h)
        ret = ctx.lib.htpops_flash_attn_ptr(ctx._ctx, p, p, p, p, None, 1, 2**31 - 64, 4096, 4096, 128, 0, 1)
        assert ret == api.HTPOPS_ERR_HIP, ret
        assert "hipMalloc" in ctx.last_error(), ctx.last_error()
        x = wl.make_activations(wl.rng_for(76, 0), 3, 256)
        assert np.array_equal(ctx.run_quantize_q8_0(x), oracle.quantize_q8_0(x))
        w = wl.make_q4_0_weights(wl.rng_for(76, 1), 48, 256)
        a = oracle.quantize_q8_0(x)
        got = ctx.run_mat_mul(a, w, 3, 256, 48, wl.GGML_TYPE_Q4_0)
        want, mag = oracle.mat_mul_q8_0_act_f64(a, w, 3, 256, 48, wl.GGML_TYPE_Q4_0)
        assert np.all(np.abs(got - want) <= MATMUL_RTOL * mag)
    finally:
        ctx.release(h)


def test_registered_weights_take_the_fast_kernels_once_prepared(ctx, oracle):
    # Weights in memory the context does not own (a framework's tensor, here a buffer of a second context registered by
    # address) get no converted copy on their own: nothing tells the context when they change. htpops_buffer_prepare_weights
    # is the opt-in (the reference maps weights once and treats them as immutable, src/dsp/op_executor.cc:124-130): it
    # makes the copy now, and from then on the buffer is treated like one of the context's own, htpops_buffer_invalidate
    # included. Same kernel = same bits as the owned-buffer run (the kernels that read the weights as they are sum in
    # another order).
    wt, op = wl.GGML_TYPE_Q4_0, api.HTP_OPS_MAT_MUL_Q4_0_Q8_0
    rng = wl.rng_for(95, 0)
    k, n = 1024, 3072
    w = wl.make_q4_0_weights(rng, n, k)
    acts = {m: oracle.quantize_q8_0(wl.make_activations(rng, m, k)) for m in (8, 512)}
    with api.Context(device=0) as owner:
        theirs = owner.upload(w)
        ours = ctx.upload(w)
        alias = ctx.register(owner.device_ptr(theirs), w.nbytes)
        h_act = {m: ctx.upload(a) for m, a in acts.items()}
        h_out = {m: ctx.alloc(m * n * 4) for m in acts}

        def run(hw, m):
            msg = api.build_message([(api.REQUEST_TYPE_OP_COMPUTE, api.op_compute_request(
                op, api.mat_mul_params((h_out[m], 0), (h_act[m], 0), (hw, 0), m, k, n)))])
            assert ctx.process_message(msg) == 0 and api.message_request_states(msg) == [0], ctx.last_error()
            assert ctx.last_message_submissions() == 1
            return ctx.read(h_out[m], np.float32, m * n).reshape(m, n)

        def check(got, m, weights):
            cols = np.unique(np.linspace(0, n - 1, 40).astype(int))
            rows = np.arange(m) if m <= 8 else np.array([0, 1, 31, 32, 127, 128, 300, 511])
            want, mag = oracle.mat_mul_q8_0_act_f64(acts[m][rows], weights[cols], len(rows), k, len(cols), wt)
            assert np.all(np.abs(got[np.ix_(rows, cols)] - want) <= MATMUL_RTOL * mag)

        try:
            base = ctx.converted_bytes()
            owned = {m: run(ours, m) for m in (8, 512)}   # repacked-weight kernel / FP6-tile kernel over cached copies
            owned_bytes = ctx.converted_bytes() - base
            assert owned_bytes >= 2 * w.nbytes             # operand-order nibbles (1 x) + FP6 tiles (1.78 x)
            for m in (8, 512):
                check(owned[m], m, w)
            # before the opt-in: right answers, nothing kept
            before = ctx.converted_bytes()
            for m in (8, 512):
                check(run(alias, m), m, w)
            assert ctx.converted_bytes() == before
            # the opt-in, one row count at a time
            added8 = ctx.prepare_weights(alias, wt, n, k, 8)
            assert added8 == w.nbytes and ctx.converted_bytes() == before + added8
            assert ctx.prepare_weights(alias, wt, n, k, 8) == 0          # already there
            assert np.array_equal(run(alias, 8), owned[8])
            added512 = ctx.prepare_weights(alias, wt, n, k, 512)
            assert added8 + added512 == owned_bytes
            assert np.array_equal(run(alias, 512), owned[512])
            assert ctx.converted_bytes() == before + owned_bytes          # the matmuls made nothing more
            # the owner rewrites its memory and says so: the copies go, the next matmuls see the new weights and, the
            # buffer staying under the contract, keep new copies
            w2 = wl.make_q4_0_weights(rng, n, k)
            owner.write(theirs, w2)
            assert ctx.invalidate(alias) == 0
            assert ctx.converted_bytes() == before
            for m in (8, 512):
                check(run(alias, m), m, w2)
            assert ctx.converted_bytes() == before + owned_bytes
            # bad arguments
            assert ctx.lib.htpops_buffer_prepare_weights(ctx._ctx, alias, 0, wt, n, k + 32, 8, None) == api.HTPOPS_ERR_REJECTED
            assert ctx.lib.htpops_buffer_prepare_weights(ctx._ctx, 12345, 0, wt, n, k, 8, None) == api.HTPOPS_ERR_REJECTED
            assert ctx.lib.htpops_buffer_prepare_weights(ctx._ctx, alias, 0, 3, n, k, 8, None) == api.HTPOPS_ERR_REJECTED
        finally:
            for h in [alias, ours] + list(h_act.values()) + list(h_out.values()):
                ctx.release(h)
            owner.release(theirs)


def test_converted_copies_stay_under_the_cap(ctx, oracle):
    # With "converted_cap_mib" set, the least recently used converted copies are evicted when a new one would pass the
    # cap; results do not change, and a copy that went is simply made again.
    wt, op = wl.GGML_TYPE_Q4_0, api.HTP_OPS_MAT_MUL_Q4_0_Q8_0
    rng = wl.rng_for(96, 0)
    m, k, n = 8, 2048, 4096                       # 4.5 MiB of weights each, the same again as a repacked copy
    ws = [wl.make_q4_0_weights(rng, n, k) for _ in range(3)]
    a = oracle.quantize_q8_0(wl.make_activations(rng, m, k))
    hws, ha, ho = [ctx.upload(w) for w in ws], ctx.upload(a), ctx.alloc(m * n * 4)
    try:
        base = ctx.converted_bytes()
        ctx.set_option("converted_cap_mib", (base >> 20) + 10)   # room for two copies, not three

        def run(i):
            assert ctx.execute(op, api.mat_mul_params((ho, 0), (ha, 0), (hws[i], 0), m, k, n)) == 0
            ctx.synchronize()
            return ctx.read(ho, np.float32, m * n).reshape(m, n)
        first = [run(i) for i in range(3)]
        assert ctx.converted_bytes() - base == 2 * ws[0].nbytes   # the copy of weights 0 went when weights 2 came
        for i in (0, 1, 2, 0):
            assert np.array_equal(run(i), first[i])
            assert ctx.converted_bytes() - base <= 2 * ws[0].nbytes
        cols = np.unique(np.linspace(0, n - 1, 32).astype(int))
        want, mag = oracle.mat_mul_q8_0_act_f64(a, ws[2][cols], m, k, len(cols), wt)
        assert np.all(np.abs(first[2][:, cols] - want) <= MATMUL_RTOL * mag)
    finally:
        for h in hws + [ha, ho]:
            ctx.release(h)
