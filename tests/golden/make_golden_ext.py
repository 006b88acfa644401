#!/usr/bin/env python3
"""Writes tests/golden/colsum_ext_golden.npz: small inputs and expected column means for the
shapes beyond the reference operator's domain (grouped key heads, batched causal calls, causal
calls restricted to their first rows, explicit k_past, non-causal S_q != S_k).

Definition evaluated here, by a pure-Python float64 brute force that shares no code with the
oracle, the package or torch:
    key head of query head h   = h // (H_q // H_k)
    key j visible to query i   <=>  not causal, or j <= k_past + i   (k_past defaults to max(0, S_k - S_q))
    rows averaged              = first min(cls_len, S_q) query rows (all when cls_len is None)
    out[b][j] = 1 / (H_q * rows) * sum_h sum_{i < rows} softmax_j(scale * <q[b,h,i], k[b,h // g,j]>)
With H_q == H_k this is the reference's definition (flash_colsum/baselines.py:35-78).
Run from the repo root:  python tests/golden/make_golden_ext.py
"""
import math
import os

import numpy as np

CASES = [
    # name, B, Hq, Hk, Sq, Sk, D, causal, cls_len, k_past, scale
    ("gqa_nc", 2, 4, 2, 19, 19, 64, False, None, None, None),
    ("mqa_nc_cls", 1, 6, 1, 33, 33, 64, False, 2, None, 0.2),
    ("gqa_causal_b3", 3, 4, 2, 7, 41, 64, True, None, None, None),
    ("causal_b2", 2, 2, 2, 35, 35, 128, True, None, None, 0.05),
    ("causal_cls", 1, 3, 3, 20, 50, 64, True, 6, None, None),
    ("causal_kpast", 2, 2, 1, 9, 30, 64, True, None, 4, None),
    ("cross_nc", 2, 2, 2, 11, 37, 64, False, None, None, None),
    ("gqa_cross_cls", 1, 8, 2, 40, 13, 128, False, 5, None, -0.1),
]


def brute(q, k, causal, cls_len, k_past, scale):
    b_n, hq, s_q, d = q.shape
    hk, s_k = k.shape[1], k.shape[2]
    grp = hq // hk
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    rows = s_q if cls_len is None else min(cls_len, s_q)
    if k_past is None:
        k_past = max(0, s_k - s_q)
    out = [[0.0] * s_k for _ in range(b_n)]
    for b in range(b_n):
        for h in range(hq):
            kh = h // grp
            for i in range(rows):
                seen = [j for j in range(s_k) if (not causal) or j <= k_past + i]
                sc = {j: scale * sum(float(q[b, h, i, t]) * float(k[b, kh, j, t]) for t in range(d)) for j in seen}
                top = max(sc.values())
                den = sum(math.exp(v - top) for v in sc.values())
                for j, v in sc.items():
                    out[b][j] += math.exp(v - top) / den
    return np.array(out, dtype=np.float64) / (hq * rows)


def main():
    rng = np.random.default_rng(20250309)
    blob = {}
    for name, b, hq, hk, sq, sk, d, causal, cls_len, k_past, scale in CASES:
        q = rng.standard_normal((b, hq, sq, d)).astype(np.float16).astype(np.float32)
        k = rng.standard_normal((b, hk, sk, d)).astype(np.float16).astype(np.float32)
        blob[name + "/q"] = q.astype(np.float16)
        blob[name + "/k"] = k.astype(np.float16)
        blob[name + "/out"] = brute(q, k, causal, cls_len, k_past, scale)
        blob[name + "/meta"] = np.array([int(causal), -1 if cls_len is None else cls_len, -1 if k_past is None else k_past],
                                        dtype=np.int64)
        blob[name + "/scale"] = np.array([np.nan if scale is None else scale], dtype=np.float64)
        print(name, blob[name + "/out"].sum(axis=-1))
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "colsum_ext_golden.npz"), **blob)


if __name__ == "__main__":
    main()
