"""Pins the oracle's fp16 conversion, block decoders, Q8_0 quantizer and integer block dots.

The quantizer and the integer dots are ggml arithmetic that the reference neither vendors nor tests
(parity with ggml itself: unpinned); they are pinned here by hand-computed answers, by an independent
numpy restatement, and by exact-integer special cases.
"""
import numpy as np
import pytest

from pyhtpops import workloads as wl

IQ4_NL = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.float32)


def q4_block(scale, qs):
    b = np.empty(18, dtype=np.uint8)
    b[0:2] = np.array([scale], dtype=np.float16).view(np.uint8)
    b[2:] = np.asarray(qs, dtype=np.uint8)
    return b


def q8_block(scale, qs):
    b = np.empty(34, dtype=np.uint8)
    b[0:2] = np.array([scale], dtype=np.float16).view(np.uint8)
    b[2:] = np.asarray(qs, dtype=np.int8).view(np.uint8)
    return b


# ------------------------------------------------------------------------------------------- fp16

def test_fp16_to_fp32_matches_numpy_for_every_bit_pattern(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.fp16_to_fp32(int(b)) for b in bits], dtype=np.float32)
    finite = np.isfinite(want)
    assert np.array_equal(got[finite].view(np.uint32), want[finite].view(np.uint32))
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(np.isinf(got), np.isinf(want))


def test_fp32_to_fp16_round_to_nearest_even_matches_numpy(oracle):
    rng = np.random.Generator(np.random.PCG64(11))
    xs = [0.0, -0.0, 1.0, 65504.0, 65519.9, 65520.0, 1e9, 5.9604645e-8, 2.9802322e-8, 2.9802326e-8, 6.1035156e-5,
          6.0975552e-5, 0.1, 1.0 / 3.0, 2049.0, 2051.0, 1.00048828125, 1.0014648, float("inf"), -float("inf")]
    xs += list(rng.standard_normal(4000).astype(np.float32) * np.float32(0.02))
    xs += list(np.exp(rng.uniform(-20, 12, 4000)).astype(np.float32) * rng.choice([-1, 1], 4000))
    # exact midpoints between neighbouring halves must go to the even one
    h = rng.integers(1, 0x7BFF, 2000).astype(np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    xs += list(((lo + hi) / 2).astype(np.float32))
    xs = np.array(xs, dtype=np.float32)
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([oracle.fp32_to_fp16(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert oracle.fp32_to_fp16(float("nan")) & 0x7C00 == 0x7C00 and oracle.fp32_to_fp16(float("nan")) & 0x3FF != 0


# ---------------------------------------------------------------------------------------- decoders

def test_q4_0_decode_every_nibble_times_scale(oracle):
    for scale in (1.0, 0.5, 0.0131, 6.1e-5, 3.0e-7):
        s16 = np.float32(np.float16(scale))
        for q in range(16):
            blk = q4_block(scale, [q | ((15 - q) << 4)] * 16)
            out = oracle.dequantize(blk, "q4_0")
            assert np.all(out[:16] == np.float32(q - 8) * s16)
            assert np.all(out[16:] == np.float32(15 - q - 8) * s16)


def test_q4_0_decode_element_order_hand_computed(oracle):
    # byte j = j | (15 - j) << 4: element j is j - 8, element j + 16 is 7 - j (low nibbles first, then high)
    blk = q4_block(2.0, [j | ((15 - j) << 4) for j in range(16)])
    out = oracle.dequantize(blk, "q4_0")
    want = np.array([2.0 * (j - 8) for j in range(16)] + [2.0 * (7 - j) for j in range(16)], dtype=np.float32)
    assert np.array_equal(out, want)


def test_iq4_nl_decode_uses_the_code_book(oracle):
    blk = q4_block(0.25, [j | ((15 - j) << 4) for j in range(16)])
    out = oracle.dequantize(blk, "iq4_nl")
    want = np.concatenate([IQ4_NL, IQ4_NL[::-1]]) * np.float32(0.25)
    assert np.array_equal(out, want)


def test_q8_0_decode_is_signed(oracle):
    qs = np.arange(-16, 16)
    qs[0] = -128
    qs[31] = 127
    out = oracle.dequantize(q8_block(0.5, qs), "q8_0")
    assert np.array_equal(out, qs.astype(np.float32) * np.float32(0.5))


def test_split_helpers_agree_with_the_decoders(oracle):
    rng = wl.rng_for(99, 1)
    w4 = wl.make_q4_0_weights(rng, 3, 128)
    d, q = wl.q4_0_split(w4, 128)
    deq = oracle.dequantize(w4, "q4_0").reshape(3, 128)
    assert np.array_equal(deq, q.astype(np.float32) * np.repeat(d.astype(np.float32), 32, axis=1))
    w8 = wl.make_q8_0_weights(rng, 3, 128)
    d, q = wl.q8_0_split(w8, 128)
    deq = oracle.dequantize(w8, "q8_0").reshape(3, 128)
    assert np.array_equal(deq, q.astype(np.float32) * np.repeat(d.astype(np.float32), 32, axis=1))


# --------------------------------------------------------------------------------------- quantizer

def numpy_quantize_q8_0(x):
    """Independent restatement with numpy float32 operations."""
    x = np.asarray(x, dtype=np.float32).reshape(-1, 32)
    amax = np.max(np.abs(x), axis=1).astype(np.float32)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    y = (x * inv[:, None]).astype(np.float32)
    q = (np.sign(y) * np.floor(np.abs(y) + np.float32(0.5))).astype(np.int8)  # half away from zero
    return d.astype(np.float16), q


def test_quantize_q8_0_known_answers(oracle):
    # all zeros -> scale 0, quants 0
    d, q = wl.q8_0_split(oracle.quantize_q8_0(np.zeros(32, np.float32)), 32)
    assert d[0, 0] == 0 and not q.any()
    # x_j = j - 16: amax 16, d = 16/127, q_j = round((j - 16) * 127 / 16)
    x = np.arange(32, dtype=np.float32) - 16
    d, q = wl.q8_0_split(oracle.quantize_q8_0(x), 32)
    assert d[0, 0] == np.float16(np.float32(16.0) / np.float32(127.0))
    inv = np.float32(1.0) / (np.float32(16.0) / np.float32(127.0))
    want = [int(np.sign(v) * np.floor(abs(np.float32(v) * inv) + 0.5)) for v in x]
    assert q[0].tolist() == want
    assert q[0, 0] == -127 and q[0, 16] == 0 and q[0, 17] == 8  # 7.9375 -> 8
    # +-127 c -> +-127
    for c in (1.0, 0.37, 123.0, 1e-6):
        x = np.full(32, 0.5 * c, np.float32)
        x[3], x[7] = 127 * c, -127 * c
        d, q = wl.q8_0_split(oracle.quantize_q8_0(x), 32)
        assert q[0, 3] == 127 and q[0, 7] == -127


def test_quantize_q8_0_ties_round_away_from_zero(oracle):
    # amax = 127 -> d = 1, id = 1 exactly, so x + 0.5 ties are exact
    x = np.zeros(32, np.float32)
    x[0] = 127.0
    x[1:9] = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5]
    d, q = wl.q8_0_split(oracle.quantize_q8_0(x), 32)
    assert d[0, 0] == np.float16(1.0)
    assert q[0, :9].tolist() == [127, 1, -1, 2, -2, 3, -3, 127, -127]


def test_quantize_q8_0_scale_is_fp16_of_unrounded_d_and_subnormal_scales_survive(oracle):
    x = np.zeros(32, np.float32)
    x[5] = 127 * 3.0e-6  # d = 3e-6 is an fp16 subnormal
    x[6] = 3.0e-6
    d, q = wl.q8_0_split(oracle.quantize_q8_0(x), 32)
    assert d[0, 0] == np.float16(np.float32(x[5]) / np.float32(127.0)) and d[0, 0] != 0
    assert q[0, 5] == 127 and q[0, 6] == 1


def test_quantize_q8_0_matches_numpy_restatement(oracle):
    rng = wl.rng_for(98, 2)
    x = wl.make_activations(rng, 7, 4096)
    x[2] *= 1e-4
    x[3] *= 3e3
    x[4, 64:96] = 0
    got_d, got_q = wl.q8_0_split(oracle.quantize_q8_0(x), 4096)
    want_d, want_q = numpy_quantize_q8_0(x)
    assert np.array_equal(got_d.view(np.uint16).ravel(), want_d.view(np.uint16).ravel())
    assert np.array_equal(got_q.ravel(), want_q.ravel())


def test_quantize_q8_0_is_stable_under_requantization(oracle):
    rng = wl.rng_for(98, 3)
    x = wl.make_activations(rng, 2, 512)
    b1 = oracle.quantize_q8_0(x)
    deq = oracle.dequantize(b1, "q8_0").reshape(2, 512)
    d1, q1 = wl.q8_0_split(b1, 512)
    d2, q2 = wl.q8_0_split(oracle.quantize_q8_0(deq), 512)
    # the extreme element stays at +-127 and the scale moves by at most one fp16 rounding
    assert np.array_equal(np.abs(q2).max(axis=1), np.abs(q1).max(axis=1))
    assert np.allclose(d2.astype(np.float32), d1.astype(np.float32), rtol=2 ** -10)


# ------------------------------------------------------------------------------------ integer dots

def test_block_dots_match_numpy_integer_arithmetic(oracle):
    rng = wl.rng_for(97, 1)
    k = 32 * 64
    w4 = wl.make_q4_0_weights(rng, 1, k)
    w8 = wl.make_q8_0_weights(rng, 1, k)
    a = oracle.quantize_q8_0(wl.make_activations(rng, 1, k))
    _, q4 = wl.q4_0_split(w4, k)
    _, q8 = wl.q8_0_split(w8, k)
    _, qa = wl.q8_0_split(a, k)
    for b in range(k // 32):
        sl = slice(32 * b, 32 * b + 32)
        assert oracle.block_dot(w4[0, 18 * b:18 * b + 18], a[0, 34 * b:34 * b + 34], wl.GGML_TYPE_Q4_0) == int(
            np.dot(q4[0, sl].astype(np.int32), qa[0, sl].astype(np.int32)))
        assert oracle.block_dot(w8[0, 34 * b:34 * b + 34], a[0, 34 * b:34 * b + 34], wl.GGML_TYPE_Q8_0) == int(
            np.dot(q8[0, sl].astype(np.int32), qa[0, sl].astype(np.int32)))


def test_block_dot_extremes_and_low_high_nibble_pairing(oracle):
    # all weights -8, all activations -127 -> 32 * 8 * 127
    assert oracle.block_dot(q4_block(1, [0x00] * 16), q8_block(1, [-127] * 32), wl.GGML_TYPE_Q4_0) == 32512
    assert oracle.block_dot(q4_block(1, [0xFF] * 16), q8_block(1, [-127] * 32), wl.GGML_TYPE_Q4_0) == -7 * 127 * 32
    assert oracle.block_dot(q8_block(1, [-128] * 32), q8_block(1, [-128] * 32), wl.GGML_TYPE_Q8_0) == 32 * 16384
    # low nibbles pair with activations 0..15, high nibbles with 16..31: a transposed pairing fails this
    a = np.zeros(32, np.int8)
    a[3] = 5
    a[19] = 11
    w = [0x88] * 16
    w[3] = (0xC << 4) | 0x9  # low nibble 9 -> +1, high nibble 12 -> +4
    assert oracle.block_dot(q4_block(1, w), q8_block(1, a), wl.GGML_TYPE_Q4_0) == 1 * 5 + 4 * 11


def test_vec_dot_applies_both_scales_per_block_in_order(oracle):
    # two blocks with different scales; values chosen so that fp32 arithmetic is exact
    w = np.concatenate([q4_block(0.5, [0x99] * 16), q4_block(2.0, [0xAA] * 16)])  # +1 ... , +2 ...
    a = np.concatenate([q8_block(0.25, [3] * 32), q8_block(4.0, [-1] * 32)])
    got = oracle.vec_dot(64, w, a, wl.GGML_TYPE_Q4_0)
    assert got == (32 * 1 * 3) * 0.5 * 0.25 + (32 * 2 * -1) * 2.0 * 4.0
    w8 = np.concatenate([q8_block(0.5, [7] * 32), q8_block(2.0, [-3] * 32)])
    got = oracle.vec_dot(64, w8, a, wl.GGML_TYPE_Q8_0)
    assert got == (32 * 7 * 3) * 0.5 * 0.25 + (32 * -3 * -1) * 2.0 * 4.0


@pytest.mark.parametrize("weight_type", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
def test_mat_mul_integer_exact_when_scales_are_one(oracle, weight_type):
    rng = wl.rng_for(96, weight_type)
    m, k, n = 2, 64, 64
    w = wl.make_weights(rng, n, k, weight_type).reshape(n, k // 32, -1)
    w[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    w = w.reshape(n, -1)
    a = np.empty((m, k // 32, 34), np.uint8)
    a[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    a[:, :, 2:] = rng.integers(-20, 21, (m, k // 32, 32), dtype=np.int8).view(np.uint8)
    a = a.reshape(m, -1)
    out = oracle.mat_mul_q8_0_act(a, w, m, k, n, weight_type)
    _, qa = wl.q8_0_split(a, k)
    _, qw = (wl.q4_0_split if weight_type == wl.GGML_TYPE_Q4_0 else wl.q8_0_split)(w, k)
    want = qa.astype(np.int64) @ qw.astype(np.int64).T
    assert np.array_equal(out.astype(np.int64), want) and np.array_equal(out, want.astype(np.float32))


@pytest.mark.parametrize("weight_type", [wl.GGML_TYPE_Q4_0, wl.GGML_TYPE_Q8_0])
def test_mat_mul_against_float64_and_row_independence(oracle, weight_type):
    rng = wl.rng_for(96, 10 + weight_type)
    m, k, n = 8, 1536, 96
    w = wl.make_weights(rng, n, k, weight_type)
    x = wl.make_activations(rng, m, k)
    a = oracle.quantize_q8_0(x)
    out = oracle.mat_mul_q8_0_act(a, w, m, k, n, weight_type)
    # independent float64 evaluation from the split views
    da, qa = wl.q8_0_split(a, k)
    dw, qw = (wl.q4_0_split if weight_type == wl.GGML_TYPE_Q4_0 else wl.q8_0_split)(w, k)
    sumi = np.einsum("mbj,nbj->mnb", qa.reshape(m, -1, 32).astype(np.int64), qw.reshape(n, -1, 32).astype(np.int64))
    terms = sumi * da.astype(np.float64)[:, None, :] * dw.astype(np.float64)[None, :, :]
    want, mag = terms.sum(axis=2), np.abs(terms).sum(axis=2)
    assert np.all(np.abs(out - want) <= 1e-6 * mag)
    f64, mag2 = oracle.mat_mul_q8_0_act_f64(a, w, m, k, n, weight_type)
    assert np.allclose(f64, want, rtol=0, atol=1e-12 * mag.max()) and np.allclose(mag2, mag, rtol=1e-12)
    # one row alone gives bit-identical results to the same row inside the batch; threads do not change bits
    assert np.array_equal(oracle.mat_mul_q8_0_act(a[3:4], w, 1, k, n, weight_type)[0], out[3])
    assert np.array_equal(oracle.mat_mul_q8_0_act(a, w, m, k, n, weight_type, n_threads=4), out)
    assert np.array_equal(oracle.mat_mul_f32_act(x, w, m, k, n, weight_type), out)


# --------------------------------------------------------------------------- reference-native formats (ops 1-4)

def test_permuted_q4_0_known_answers(oracle):
    # hand-computed from the dequantizer's vector order (reference: src/dsp/ops/mat_mul.c:383-405): quant bytes
    # 0..127, scales 1..8
    sb = np.zeros(144, np.uint8)
    sb[:16] = np.arange(1, 9, dtype=np.float16).view(np.uint8)
    sb[16:] = np.arange(128, dtype=np.uint8)
    d = oracle.dequantize_permuted(sb, 2)[0].astype(np.float32)
    assert d[0] == (0 - 8) * 1          # vector 0, e 0: low nibble of byte 0, scale 0
    assert d[1] == (2 - 8) * 1          # e 1: low nibble of byte 2
    assert d[32] == ((64 & 15) - 8) * 2  # e 32: byte 64, scale 1
    assert d[64] == (1 - 8) * 3         # vector 1: low nibble of byte 1, scale 2
    assert d[128] == (0 - 8) * 5        # vector 2: high nibble of byte 0, scale 4
    assert d[192 + 33] == ((67 >> 4) - 8) * 8  # vector 3, e 33: high nibble of byte 67, scale 7
    nl = oracle.dequantize_permuted(sb, 4)[0].astype(np.float32)
    assert nl[0] == -127 * 1 and nl[1] == -83 * 1 and nl[128] == -127 * 5


def test_permuted_q8_0_known_answers(oracle):
    sb = np.zeros(272, np.uint8)
    sb[:16] = np.array([1, 2, 3, 4, 5, 6, 7, 8], np.float16).view(np.uint8) 
    sb[16:] = (np.arange(256) - 128).astype(np.int8).view(np.uint8)
    d = oracle.dequantize_permuted(sb, 3)[0].astype(np.float32)
    assert d[0] == -128 * 1 and d[31] == -97 * 1 and d[32] == -96 * 2 and d[64] == -64 * 3 and d[255] == 127 * 8


@pytest.mark.parametrize("kind", [2, 3, 4])
def test_permuted_dequantizer_matches_numpy_reading(oracle, kind):
    rng = wl.rng_for(70, kind)
    n, k = 64, 96
    raw = wl.make_permuted_weights(rng, n, k, kind)
    tiles = oracle.dequantize_permuted(raw, kind).reshape(-1)       # fp16 tile order
    w = wl.permuted_to_kn(raw, n, k, kind)                          # [k][n] from the tile geometry
    for kk, nn in [(0, 0), (1, 0), (0, 1), (31, 31), (33, 2), (95, 63), (64, 40), (7, 17), (8, 16)]:
        assert tiles[oracle.w16_tile_index(kk, nn, k)] == np.float16(w[kk, nn])
    assert np.array_equal(wl.w16_tile_layout(w).view(np.uint16), tiles.view(np.uint16))


@pytest.mark.parametrize("kind", [1, 2, 3, 4])
def test_mat_mul_permuted_against_numpy(oracle, kind):
    rng = wl.rng_for(71, kind)
    m, k, n = 3, 96, 64
    x = wl.make_activations(rng, m, k)
    if kind == 1:
        w = (rng.standard_normal((k, n)) * 0.05).astype(np.float16).astype(np.float32)
        raw = wl.w16_tile_layout(w)
    else:
        raw = wl.make_permuted_weights(rng, n, k, kind)
        w = wl.permuted_to_kn(raw, n, k, kind)
    got, f64 = oracle.mat_mul_permuted(x, raw, m, k, n, kind, want_f64=True)
    want = x.astype(np.float16).astype(np.float64) @ w.astype(np.float64)
    assert np.allclose(f64, want, rtol=1e-12, atol=1e-12)
    assert np.array_equal(got, want.astype(np.float32).astype(np.float16).astype(np.float32))
    # the fp32 triple loop of the reference's own test differs only by the fp16 rounding of activations and result
    if kind == 1:
        loose = oracle.mat_mul_w16a32(x, raw, m, k, n)
        assert np.allclose(got, loose, rtol=4e-3, atol=4e-3)
