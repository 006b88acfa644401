#!/usr/bin/env python3
"""Latency / peak-memory sweeps of `flash_colsum` on one MI355X, as CSV.

Counterpart of the reference's three sweeps (reference: benchmarks/benchmark_colsum.py:289-424):

  noncausal_batched   S = 1024, H = 16, D = 64, B in {1, 2, ..., 1024}
  noncausal           B = 1, H = 16, D = 64, S in {2048, ..., 262144}
  causal              B = 1, H = 32, Q_len = 128, D = 128, K_len in {16384, ..., 262144}

plus one of this repository's own: `vit`, non-causal token counts of common vision encoders
(197, 257, 577, 729, 1025, 1370), none of them a multiple of the kernels' 32-key tile.

Timing follows the reference's `measure_latency` (benchmark_colsum.py:42-56): warm-up calls,
then `iters` x (call + device synchronize) under one wall clock, so launch and host overhead
are included.  Peak memory is `torch.cuda.max_memory_allocated` around one call
(benchmark_colsum.py:59-71); the kernels' workspace is allocated once per stream by the host
layer and reported in its own column.  The eager baseline that materialises the attention matrix runs
on the GPU too.  Where its score tensors would not fit it runs in chunks (`eager_kind` says how), each
chunk the same eager code on a slice: over the batch for the batched sweep, over query rows elsewhere
(a row's softmax needs all keys, so rows are what can be cut).  The reference's benchmark has the same
fallback (benchmarks/benchmark_colsum.py:74-196, 234-274; it estimates the batched case from the largest
batch that fitted, here it is run).

    python bench_sweep.py --sweep all --out sweep.csv
"""
import argparse
import csv
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "flash-colsum_amd"))

SWEEPS = {
    "noncausal_batched": [dict(B=b, H=16, Sq=1024, Sk=1024, D=64, causal=False) for b in (1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024)],
    "noncausal": [dict(B=1, H=16, Sq=s, Sk=s, D=64, causal=False) for s in (2048, 4096, 8192, 16384, 32768, 65536, 131072, 262144)],
    "causal": [dict(B=1, H=32, Sq=128, Sk=k, D=128, causal=True) for k in (16384, 32768, 65536, 131072, 262144)],
    # not in the reference: token counts of common vision encoders (n*n patches + 1 class token)
    "vit": [dict(B=b, H=h, Sq=s, Sk=s, D=64, causal=False) for (b, h, s) in
            ((64, 12, 197), (32, 16, 257), (32, 16, 577), (16, 16, 729), (16, 16, 1025), (8, 16, 1370))],
}
EAGER_MAX_BYTES = 40 << 30  # logits + fp32 softmax + cast of the eager baseline must fit well inside HBM


def measure_latency(fn, warmup, iters):
    import torch

    with torch.no_grad():
        for _ in range(warmup):
            fn()
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
            torch.cuda.synchronize()
        return (time.perf_counter() - t0) / iters


def peak_memory(fn):
    import torch

    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    with torch.no_grad():
        fn()
    torch.cuda.synchronize()
    return torch.cuda.max_memory_allocated() - base


def chunked_eager(naive_colsum, q, k, scale, causal, budget_bytes):
    """The eager baseline on slices that fit `budget_bytes` of score tensors; returns (fn, kind, chunk).

    Batch > 1: slices of the batch (results concatenated).  Batch 1: slices of query rows; a slice's means
    are weighted by its rows and added (causal: rows [r0, r1) see the keys below k_past + r1 and are aligned
    to the end of that prefix, which is the alignment the eager code infers from the shapes)."""
    import torch

    b, h, sq, _ = q.shape
    sk = k.shape[2]
    per_score = 2 + 4 + 2 + 2  # logits, fp32 softmax, its cast, one temporary
    if b > 1:
        chunk = max(1, min(b, budget_bytes // (h * sq * sk * per_score)))

        def fn():
            return torch.cat([naive_colsum(q[i:i + chunk], k[i:i + chunk], scale=scale, is_causal=causal)
                              for i in range(0, b, chunk)], dim=0)
        return fn, "chunked_batch", chunk
    chunk = max(1, min(sq, budget_bytes // (h * sk * per_score)))
    k_past = max(0, sk - sq) if causal else 0

    def fn():
        out = torch.zeros((1, sk), dtype=torch.float32, device=q.device)
        for r0 in range(0, sq, chunk):
            r1 = min(sq, r0 + chunk)
            if causal:
                part = naive_colsum(q[:, :, r0:r1], k[:, :, :k_past + r1], scale=scale, is_causal=True)
                out[:, :k_past + r1] += part.float() * (r1 - r0)
            else:
                out += naive_colsum(q[:, :, r0:r1], k, scale=scale).float() * (r1 - r0)
        return out / sq
    return fn, "chunked_rows", chunk


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--sweep", default="all", choices=sorted(SWEEPS) + ["all"])
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--out", default="-", help="CSV file, or - for stdout")
    ap.add_argument("--no-eager", action="store_true", help="skip the eager baseline")
    ap.add_argument("--max-points", type=int, default=0, help="only the first N points of each sweep (0 = all)")
    args = ap.parse_args()

    import torch
    from flash_colsum import _hip, flash_colsum, naive_colsum

    if not torch.cuda.is_available():
        sys.exit("bench_sweep.py needs a GPU")
    names = sorted(SWEEPS) if args.sweep == "all" else [args.sweep]
    fields = ["sweep", "B", "H", "Sq", "Sk", "D", "causal", "flash_ms", "flash_peak_mib", "workspace_mib", "flash_tflops",
              "eager_ms", "eager_peak_mib", "speedup", "max_abs_diff_vs_eager", "eager_kind", "eager_chunk"]
    out = sys.stdout if args.out == "-" else open(args.out, "w", newline="")
    wr = csv.DictWriter(out, fieldnames=fields)
    wr.writeheader()
    for name in names:
        points = SWEEPS[name][: args.max_points] if args.max_points else SWEEPS[name]
        for pt in points:
            g = torch.Generator(device="cuda").manual_seed(0)
            q = torch.randn((pt["B"], pt["H"], pt["Sq"], pt["D"]), generator=g, device="cuda", dtype=torch.float16)
            k = torch.randn((pt["B"], pt["H"], pt["Sk"], pt["D"]), generator=g, device="cuda", dtype=torch.float16)
            scale = pt["D"] ** -0.5
            run = lambda: flash_colsum(q, k, scale=scale, is_causal=pt["causal"])
            # long points: fewer iterations, at least 3
            t_probe = measure_latency(run, 1, 1)
            iters = max(3, min(args.iters, int(2.0 / max(t_probe, 1e-6))))
            t_fast = measure_latency(run, min(args.warmup, iters), iters)
            m_fast = peak_memory(run)
            row = dict(sweep=name, causal=int(pt["causal"]), flash_ms=round(t_fast * 1e3, 4),
                       flash_peak_mib=round(m_fast / 2**20, 2),
                       # kept by the host layer between calls, so not part of the per-call peak
                       workspace_mib=round(_hip.workspace_bytes(pt["causal"], pt["B"], pt["H"], pt["Sq"], pt["Sk"], pt["D"]) / 2**20, 2),
                       flash_tflops=round(4.0 * pt["B"] * pt["H"] * pt["Sq"] * pt["Sk"] * pt["D"] / t_fast / 1e12, 1),
                       **{f: pt[f] for f in ("B", "H", "Sq", "Sk", "D")})
            scores = pt["B"] * pt["H"] * pt["Sq"] * pt["Sk"]
            if not args.no_eager:
                if scores * (2 + 4 + 2 + 2) <= EAGER_MAX_BYTES:
                    ref, kind, chunk = (lambda: naive_colsum(q, k, scale=scale, is_causal=pt["causal"])), "full", ""
                else:
                    ref, kind, chunk = chunked_eager(naive_colsum, q, k, scale, pt["causal"], EAGER_MAX_BYTES // 2)
                row.update(eager_kind=kind, eager_chunk=chunk)
                try:
                    t_probe_ref = measure_latency(ref, 0, 1)  # long points: one warm-up is the probe itself
                    n_ref = max(1, min(iters, int(2.0 / max(t_probe_ref, 1e-6))))
                    t_ref = t_probe_ref if n_ref == 1 and t_probe_ref > 2.0 else measure_latency(ref, 0, max(n_ref, 2))
                    m_ref = peak_memory(ref)
                    diff = (run().float() - ref().float()).abs().max().item()
                    row.update(eager_ms=round(t_ref * 1e3, 4), eager_peak_mib=round(m_ref / 2**20, 2),
                               speedup=round(t_ref / t_fast, 2), max_abs_diff_vs_eager=f"{diff:.3e}")
                except torch.OutOfMemoryError:
                    torch.cuda.empty_cache()
            wr.writerow(row)
            out.flush()
            print(f"[sweep] {name} {pt}: {row['flash_ms']} ms, eager {row.get('eager_ms')}", file=sys.stderr, flush=True)
            del q, k
            torch.cuda.empty_cache()
    if out is not sys.stdout:
        out.close()


if __name__ == "__main__":
    main()
