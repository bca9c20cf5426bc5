"""CPU: which of a super-block's 8 scales multiplies which of its 256 outputs (ops 2-4).

The oracle's restatement of the reference's fast dequantization path (src/dsp/ops/mat_mul.c:383-405, :483-505) says:
output vector v (64 elements) uses scale 2 v for elements 0..31 and scale 2 v + 1 for elements 32..63. The reference
holds two more statements of the same map that can be read without running it, and this test checks the oracle
against all three, each derived here from the reference's description of the data movement and not from the oracle:
  * the scale index table of the fast path (:319-326) looked up by vlut16, which sends the even bytes of its index
    vector to the low and the odd bytes to the high vector of the result pair;
  * the scalar expansion macro (:236-257): vs{v}_c = valign(splat(s[2v+1]), splat(s[2v]), 64 bytes);
  * the `no_group_coalesce` path (:347-370): output vector v = group 2v (32 halfwords) followed by group 2v + 1, each
    group multiplied by its own scale.
The map is probed through the oracle with constant quants and eight distinct scales, so it does not depend on the
order of the nibbles inside a vector (which stays unpinned: no test or fixture of the reference fixes it).
"""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "oracle"))
import oracle_py  # noqa: E402


@pytest.fixture(scope="module")
def oracle():
    return oracle_py.Oracle()


def scale_map_from_index_table():
    # index bytes of the two lookups: 0, 2 alternating over the first 64 bytes, 1, 3 over the last 64; the second table
    # adds 4 (mat_mul.c:319-326). The lookup returns a pair: halfword j of the low vector comes from index byte 2 j,
    # halfword j of the high vector from index byte 2 j + 1; vectors 0, 1 are the low / high result of the first
    # lookup, vectors 2, 3 of the second (:397-400).
    idx0 = np.array([(b % 2) * 2 + b // 64 for b in range(128)])
    out = np.empty((4, 64), int)
    for t, idx in enumerate((idx0, idx0 + 4)):
        out[2 * t] = idx[0::2]
        out[2 * t + 1] = idx[1::2]
    return out


def scale_map_from_scalar_macro():
    # vs{v}_c = valign(splat(s[2 v + 1]), splat(s[2 v]), 64): bytes 64..127 of the second operand followed by bytes
    # 0..63 of the first; both are splats, so the first 32 halfwords carry s[2 v] and the last 32 carry s[2 v + 1]
    return np.array([[2 * v + e // 32 for e in range(64)] for v in range(4)])


def scale_map_from_no_group_coalesce():
    # eight groups of 32 dequantized halfwords, each multiplied by its own scale g; output vector v is group 2 v
    # rotated to the low half joined with group 2 v + 1 in the high half
    groups = [np.full(32, g) for g in range(8)]
    return np.array([np.concatenate([groups[2 * v], groups[2 * v + 1]]) for v in range(4)])


def probe_oracle(oracle, kind):
    # every quant decodes to +1, scales are 1..8: the output IS the scale index + 1
    scales = np.arange(1, 9, dtype=np.float16).view(np.uint8)
    if kind == 3:
        quants = np.full(256, 1, np.int8).view(np.uint8)
    else:
        nib = 9 if kind == 2 else 8  # Q4_0: 9 - 8 = 1; IQ4_NL: table entry 8 is +1
        quants = np.full(128, nib | (nib << 4), np.uint8)
    sb = np.concatenate([scales, quants])
    out = oracle.dequantize_permuted(np.tile(sb, 3), kind).astype(np.float64)  # three super-blocks: the map repeats
    assert out.shape == (3, 256)
    assert np.array_equal(out[0], out[1]) and np.array_equal(out[0], out[2])
    return (out[0] - 1).astype(int).reshape(4, 64)


@pytest.mark.parametrize("kind", [2, 3, 4])
def test_scale_to_element_map_matches_every_statement_of_it_in_the_reference(oracle, kind):
    want = scale_map_from_index_table()
    assert np.array_equal(want, scale_map_from_scalar_macro())
    assert np.array_equal(want, scale_map_from_no_group_coalesce())
    assert np.array_equal(probe_oracle(oracle, kind), want)
