#!/usr/bin/env python3
"""Writes tests/golden/colsum_golden.npz: small inputs and their expected column means.

The expected values come from a pure-Python float64 brute force (math.exp, explicit
loops, explicit visibility rule) that shares no code with the oracle, the package or
torch's softmax/matmul.  The reference ships no golden vectors for this path; these pin
the oracle and the HIP kernels to an independent evaluation of the definition
(reference semantics: flash_colsum/baselines.py:35-78).

Inputs are drawn in float32 and rounded to fp16-representable values so the kernels (fp16
inputs) and the oracle (fp32 inputs) see exactly the same numbers.
Run from the repo root:  python tests/golden/make_golden.py
"""
import math
import os

import numpy as np

CASES = [
    # name, B, H, Sq, Sk, D, causal, cls_len, scale
    ("nc_small", 2, 2, 5, 5, 64, False, None, None),
    ("nc_ragged", 1, 3, 37, 37, 64, False, None, 0.2),
    ("nc_cls3", 2, 2, 37, 37, 64, False, 3, None),
    ("nc_cls_gt_s", 1, 2, 9, 9, 64, False, 50, None),
    ("nc_d128", 1, 2, 33, 33, 128, False, None, None),
    ("nc_negscale", 1, 2, 20, 20, 64, False, None, -0.25),
    ("c_long", 1, 2, 7, 70, 64, True, None, None),
    ("c_square", 1, 2, 40, 40, 64, True, None, None),
    ("c_kshort", 1, 2, 40, 11, 64, True, None, None),
    ("c_q1", 1, 3, 1, 45, 128, True, None, None),
    ("c_d128", 1, 2, 35, 99, 128, True, None, 0.05),
]


def brute(q, k, causal, cls_len, scale):
    b_n, h_n, s_q, d = q.shape
    s_k = k.shape[2]
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    rows = s_q if (causal or cls_len is None) else min(cls_len, s_q)
    k_past = max(0, s_k - s_q)
    out = [[0.0] * s_k for _ in range(b_n)]
    for b in range(b_n):
        for h in range(h_n):
            for i in range(rows):
                seen = [j for j in range(s_k) if (not causal) or j <= k_past + i]
                sc = {j: scale * sum(float(q[b, h, i, t]) * float(k[b, h, j, t]) for t in range(d)) for j in seen}
                top = max(sc.values())
                den = sum(math.exp(v - top) for v in sc.values())
                for j in seen:
                    out[b][j] += math.exp(sc[j] - top) / den
    return np.array(out, dtype=np.float64) / (h_n * rows)


def main():
    rng = np.random.default_rng(20240607)
    blob = {}
    for name, b, h, sq, sk, d, causal, cls_len, scale in CASES:
        q = rng.standard_normal((b, h, sq, d)).astype(np.float16).astype(np.float32)
        k = rng.standard_normal((b, h, sk, d)).astype(np.float16).astype(np.float32)
        blob[name + "/q"] = q.astype(np.float16)
        blob[name + "/k"] = k.astype(np.float16)
        blob[name + "/out"] = brute(q, k, causal, cls_len, scale)
        blob[name + "/meta"] = np.array([int(causal), -1 if cls_len is None else cls_len], dtype=np.int64)
        blob[name + "/scale"] = np.array([np.nan if scale is None else scale], dtype=np.float64)
        print(name, blob[name + "/out"].sum(axis=-1))
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "colsum_golden.npz"), **blob)


if __name__ == "__main__":
    main()
