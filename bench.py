#!/usr/bin/env python3
"""Benchmark of the attention column-mean hot path on one MI355X.

A step is one call of `flash_colsum(Q, K, ...)` on synthetic inputs that are already
resident in HBM.  The default workload is the batched non-causal self-attention shape
B=8, H=16, S=2048, D=64 with K = Q.clone().  Prints ONE JSON line on stdout; everything
else goes to stderr.

  value          effective TFLOP/s of the whole call (wall clock, launch + epilogue
                 included), counting two QK^T passes: 4*B*H*Sq*Sk*D / t
  ms_per_step    wall-clock milliseconds per call, calls issued back to back
  ms_per_call_synced / value_synced
                 the same with a device synchronize after every call, the reference benchmark's
                 own clock (reference: benchmarks/benchmark_colsum.py:42-56)
  roofline       kernels-only time of one call (HIP events on the launch stream around the
                 C-ABI call with output and workspace preallocated) against the dense
                 fp16 MFMA peak
  cpu_baseline   the eager materialising baseline (oracle/naive_colsum.py, a port of the
                 reference's naive path) on this host's cores, same workload
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "flash-colsum_amd"))
sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2516.6  # MI355X dense fp16 MFMA: 256 CU x 2.4 GHz x 4096 FLOP/clk/CU
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # name: (q shape, k shape, kwargs, K = Q.clone())
    "noncausal_b2_h4_s512_d64": ((2, 4, 512, 64), (2, 4, 512, 64), dict(scale=0.125), False),
    "noncausal_b8_h16_s2048_d64": ((8, 16, 2048, 64), (8, 16, 2048, 64), dict(), True),
    "cls1_b32_h16_s577_d64": ((32, 16, 577, 64), (32, 16, 577, 64), dict(cls_len=1), False),
    # a point of the reference's own batched sweep (benchmarks/benchmark_colsum.py:289-330), not a headline config
    "noncausal_b256_h16_s1024_d64": ((256, 16, 1024, 64), (256, 16, 1024, 64), dict(), False),
    # not in the reference's benchmarks: a vision encoder's token count (short-sequence kernel) and 128-wide heads
    "noncausal_b64_h12_s197_d64": ((64, 12, 197, 64), (64, 12, 197, 64), dict(), False),
    "noncausal_b8_h16_s1024_d128": ((8, 16, 1024, 128), (8, 16, 1024, 128), dict(), False),
    # further variants of the single-pass kernels, for their profiles: nine-tile short sequences, two key groups,
    # ragged key tiles (no multiple of 32), a head dim between 64 and 128
    "noncausal_b32_h16_s257_d64": ((32, 16, 257, 64), (32, 16, 257, 64), dict(), False),
    "noncausal_b128_h16_s512_d64": ((128, 16, 512, 64), (128, 16, 512, 64), dict(), False),
    "noncausal_b32_h16_s577_d64": ((32, 16, 577, 64), (32, 16, 577, 64), dict(), False),
    "noncausal_b8_h16_s1024_d96": ((8, 16, 1024, 96), (8, 16, 1024, 96), dict(), False),
    "causal_h32_q128_k4096_d128": ((1, 32, 128, 128), (1, 32, 4096, 128), dict(is_causal=True), False),
    "causal_h32_q128_k16384_d128": ((1, 32, 128, 128), (1, 32, 16384, 128), dict(is_causal=True), False),
    "causal_h32_q512_k65536_d128_peaky": ((1, 32, 512, 128), (1, 32, 65536, 128), dict(is_causal=True), False),
}
DEFAULT = "noncausal_b8_h16_s2048_d64"
SETTLE_CALLS = 150  # untimed calls before the --warmup steps (the GPU's clocks settle under load); reported in the record


def make_inputs(name):
    """fp32 CPU tensors from a CPU generator (seed 0, Q drawn first), identical on every host."""
    import torch

    qs, ks, kwargs, same = WORKLOADS[name]
    g = torch.Generator().manual_seed(0)
    q = torch.randn(qs, generator=g, dtype=torch.float32)
    if same:
        k = q.clone()
    else:
        k = torch.randn(ks, generator=g, dtype=torch.float32)
    if name.endswith("peaky"):
        # four head-dim channels scaled x8; first 64 keys pushed +3 sigma along Q's mean direction
        k[..., [7, 31, 64, 101]] *= 8.0
        u = q[0].mean(dim=1)
        u = u / u.norm(dim=-1, keepdim=True)
        k[0, :, :64, :] += 3.0 * u[:, None, :]
    return q, k, kwargs


def flops(name):
    """Nominal work of one call: two QK^T passes over all Sq rows, 4*B*H*Sq*Sk*D."""
    qs, ks, _, _ = WORKLOADS[name]
    b, h, sq, d = qs
    return 4.0 * b * h * sq * ks[2] * d


def needed_rows(name):
    qs, _, kwargs, _ = WORKLOADS[name]
    return min(kwargs.get("cls_len") or qs[2], qs[2])


def algorithmic_bytes(name):
    """Bytes one call must move: the Q rows it averages, K, and the fp32 output."""
    qs, ks, _, _ = WORKLOADS[name]
    b, h, _, d = qs
    return b * h * needed_rows(name) * d * 2 + ks[0] * ks[1] * ks[2] * d * 2 + ks[0] * ks[2] * 4


def hbm_bound(name):
    """With cls_len only a few query rows are needed: the call is a batch of GEMVs over K."""
    return needed_rows(name) * 16 <= WORKLOADS[name][0][2] and needed_rows(name) <= 16


def kernel_source_sha16():
    """First 16 hex digits of the SHA-256 over the library's kernel sources, in name order."""
    import hashlib

    h = hashlib.sha256()
    src = os.path.join(ROOT, "flash-colsum_amd", "csrc")
    for fn in sorted(os.listdir(src)):
        with open(os.path.join(src, fn), "rb") as f:
            h.update(fn.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--workload", default=DEFAULT, choices=sorted(WORKLOADS))
    ap.add_argument("--dtype", default="fp16", choices=["fp16", "bf16"], help="operand type (the headline is fp16)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--sweep", action="store_true",
                    help="instead of the benchmark line: run the reference's three sweeps (bench_sweep.py) and write "
                         "their summary as CSV to --sweep-out")
    ap.add_argument("--sweep-out", default=os.path.join(ROOT, "gpurun_out", "sweeps_mi355x.csv"))
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy five times, so that a rocprofv3 --pmc run over this "
                         "command sees a kernel of known HBM traffic next to the workload's kernels")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one MI355X: this path has no multi-GPU part, run with --gpus 1")

    import torch
    from flash_colsum import flash_colsum, _hip

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    if args.sweep:
        import bench_sweep

        os.makedirs(os.path.dirname(args.sweep_out), exist_ok=True)
        sys.argv = ["bench_sweep.py", "--sweep", "all", "--out", args.sweep_out, "--iters", str(max(3, min(args.steps, 50))),
                    "--warmup", str(max(1, min(args.warmup, 10)))]
        bench_sweep.main()
        print(json.dumps({"sweep_csv": args.sweep_out}), flush=True)
        return
    name = args.workload
    q32, k32, kwargs = make_inputs(name)
    op_dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float16
    q = q32.to(op_dtype).cuda()
    k = k32.to(op_dtype).cuda()
    torch.cuda.synchronize()

    # ---- whole-call wall clock (the headline): K calls back to back between two syncs.
    # The GPU's clocks take a few tens of milliseconds of load to settle; untimed calls first.
    for _ in range(SETTLE_CALLS):
        flash_colsum(q, k, **kwargs)
    for _ in range(args.warmup):
        flash_colsum(q, k, **kwargs)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        flash_colsum(q, k, **kwargs)
    torch.cuda.synchronize()
    ms_call = (time.perf_counter() - t0) * 1e3 / args.steps
    fl = flops(name)
    tflops = fl / (ms_call * 1e-3) / 1e12
    # the reference's own clock (benchmarks/benchmark_colsum.py:42-56): call + synchronize per iteration
    t0 = time.perf_counter()
    for _ in range(args.steps):
        flash_colsum(q, k, **kwargs)
        torch.cuda.synchronize()
    ms_call_synced = (time.perf_counter() - t0) * 1e3 / args.steps

    # ---- kernels only: HIP events on the launch stream around the C-ABI call
    b, h, sq, d = q.shape
    sk = k.shape[2]
    causal = bool(kwargs.get("is_causal", False))
    cls_n = int(kwargs.get("cls_len") or -1)
    scale = float(kwargs.get("scale") or d ** -0.5)
    lib = _hip.lib()
    stream = torch.cuda.current_stream().cuda_stream
    # the call as the host layer issues it: fcs_colsum_call
    call, call_ref, n_ws = _hip._prepared_call(causal, q, k, scale, cls_n, max(0, sk - sq) if causal else 0)
    ws = torch.empty(max(n_ws, 1), dtype=torch.uint8, device="cuda")
    out = torch.empty((b, sk), dtype=torch.float32, device="cuda")
    call.q, call.k, call.out, call.out_f16 = q.data_ptr(), k.data_ptr(), out.data_ptr(), None
    call.ws, call.ws_bytes, call.hip_stream = ws.data_ptr(), n_ws, stream
    plan_text = _hip.plan_description(q.shape, k.shape, causal=causal, cls_n=cls_n, scale=scale, bf16=args.dtype == "bf16")

    def launch():
        rc = lib.fcs_colsum_call(call_ref)
        if rc != 0:
            raise RuntimeError(_hip.strerror(rc))

    for _ in range(args.warmup):
        launch()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        launch()
    torch.cuda.synchronize()
    raw_ms = (time.perf_counter() - t0) * 1e3 / args.steps  # C-ABI calls back to back, no Python layer
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for e0, e1 in evs:
        e0.record()
        launch()
        e1.record()
    torch.cuda.synchronize()
    ker_ms = statistics.mean(e0.elapsed_time(e1) for e0, e1 in evs)
    ker_tflops = fl / (ker_ms * 1e-3) / 1e12
    by = algorithmic_bytes(name)
    ker_gbs = by / (ker_ms * 1e-3) / 1e9
    roofline = {
        "bound": "mfma",
        "kernel": plan_text + " (all kernels of one call)",
        "achieved": round(ker_tflops, 2),
        "peak": PEAK_FP16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(ker_tflops / PEAK_FP16_TFLOPS, 4),
        "kernel_ms": round(ker_ms, 5),
        "c_abi_back_to_back_ms": round(raw_ms, 5),
        "algorithmic_flops": fl,
        "algorithmic_bytes": by,
        "hbm_frac": round(ker_gbs / PEAK_HBM_GBS, 4),
        "traffic": None,
    }
    if hbm_bound(name):
        # only `cls_len` rows are needed, so the nominal FLOP count is not the work: price against HBM
        roofline.update({"bound": "hbm", "achieved": round(ker_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(ker_gbs / PEAK_HBM_GBS, 4),
                         "needed_tflops": round(fl * needed_rows(name) / q.shape[2] / (ker_ms * 1e-3) / 1e12, 3)})
    print(f"[bench] {name}: {ms_call:.4f} ms/call wall ({ms_call_synced:.4f} with a synchronize per call), "
          f"{raw_ms:.4f} ms C-ABI back-to-back, {ker_ms:.4f} ms kernels, "
          f"{tflops:.1f} / {ker_tflops:.1f} TFLOP/s", file=sys.stderr)

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()

    # measured offline with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (see profiles/), bytes per call; only
    # valid for the kernels it was measured with: the file names the hash of the kernel sources
    traffic_file = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(traffic_file):
        with open(traffic_file) as f:
            measured = json.load(f)
        if measured.get("kernel_source_sha16") == kernel_source_sha16():
            roofline["traffic"] = measured.get(name if args.dtype == "fp16" else name + "_" + args.dtype)
        else:
            roofline["traffic_note"] = "profiles/hbm_traffic.json was measured with other kernel sources: ignored"

    # ---- CPU baseline: eager materialising path on the host cores, same workload
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import naive_colsum

        qc, kc = q32.to(op_dtype).float(), k32.to(op_dtype).float()
        naive_colsum(qc, kc, **kwargs)
        ts = []
        for _ in range(3):
            t0 = time.perf_counter()
            naive_colsum(qc, kc, **kwargs)
            ts.append(time.perf_counter() - t0)
        t_cpu = statistics.median(ts)
        cpu = {
            "value": round(fl / t_cpu / 1e12, 5),
            "unit": "TFLOP/s",
            "ms_per_call": round(t_cpu * 1e3, 2),
            "cores": torch.get_num_threads(),
            "host_cpus": os.cpu_count(),
            "kind": "port",
            "sample": f"full workload {name}, fp32 torch eager on CPU, 1 warm-up + median of 3 calls",
        }
        print(f"[bench] cpu baseline: {t_cpu * 1e3:.1f} ms/call on {torch.get_num_threads()} threads", file=sys.stderr)

    rec = {
        "metric": "ms/call + effective TFLOP/s (% fp16 MFMA peak), B8 H16 S2048 D64 non-causal"
        if name == DEFAULT else f"ms/call + effective TFLOP/s (% fp16 MFMA peak), {name}",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_calls": SETTLE_CALLS,
        "ms_per_step": round(ms_call, 5),
        "ms_per_call_synced": round(ms_call_synced, 5),
        "value_synced": round(fl / (ms_call_synced * 1e-3) / 1e12, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "dtype_note": f"{args.dtype} MFMA operands, fp32 accumulation, fp32 softmax and column sums",
        "data": f"synthetic: N(0,1) from torch.Generator(seed 0) on CPU, rounded to {args.dtype}",
        "config": {"workload": name, "q_shape": list(q.shape), "k_shape": list(k.shape), **{k_: v for k_, v in kwargs.items()}},
        "frac_of_fp16_mfma_peak": round(tflops / PEAK_FP16_TFLOPS, 4),
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    print(json.dumps(rec), flush=True)


if __name__ == "__main__":
    main()
