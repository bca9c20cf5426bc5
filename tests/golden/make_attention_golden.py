"""Writes tests/golden/naive_flash_attn_*.npz from the reference's own scalar attention routine.

Run in the development container only (it needs oracle/_ref, which is built from the reference checkout by
`make -C oracle ref`). The fixtures hold inputs and the routine's outputs; no reference source is stored.

    python tests/golden/make_attention_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
sys.path.insert(0, os.path.join(ROOT, "htp-ops-lib_amd"))

import oracle_py  # noqa: E402
from pyhtpops import workloads  # noqa: E402

CASES = [
    # name, qo_len, kv_len, n_heads, n_kv_heads, head_dim, masked, seed
    ("q5_kv70_h4x2_d64_causal", 5, 70, 4, 2, 64, True, 9001),
    ("q1_kv300_h8x2_d128_nomask", 1, 300, 8, 2, 128, False, 9002),
    ("q40_kv300_h4x1_d128_causal", 40, 300, 4, 1, 128, True, 9003),
]


def main():
    ref = oracle_py.RefNaiveFlashAttn()
    for name, qo, kv, nh, nkv, d, masked, seed in CASES:
        rng = np.random.Generator(np.random.PCG64(seed))
        q16, k16, v16 = workloads.make_attention_inputs(rng, qo, kv, nh, nkv, d)
        q32 = q16.astype(np.float32)
        mask = workloads.make_causal_mask(qo, kv) if masked else None
        out = ref(q32, k16, v16, mask, nh, nkv, d)
        path = os.path.join(HERE, "naive_flash_attn_%s.npz" % name)
        np.savez_compressed(path, q=q32, k=k16, v=v16, mask=(mask if mask is not None else np.zeros((0, 0), np.float16)),
                            out=out, dims=np.array([qo, kv, nh, nkv, d, int(masked)], dtype=np.int32))
        print("wrote", path, out.shape, float(np.abs(out).max()))


if __name__ == "__main__":
    main()
