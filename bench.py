"""Benchmark of the fused attention forward on one MI355X.

One step = one forward pass (softmax(Q K^T / sqrt(H)) V for every batch and head) over one
synthetic batch resident in HBM.  Prints one JSON line: whole-job TFLOP/s with
flop = 4*B*R*L^2*H, the MFMA roofline of the kernel (average launch duration from HIP events
recorded on the launch stream inside the kernel library) and, beside it, the naive float32 CPU
evaluation of the same workload timed on the host cores over a bounded sample of (batch, head)
pairs.  Counterpart of the reference's benchmark (reference tests/benchmark_fused_attn.py:8-45),
which prints wall-clock milliseconds of 128 naive and 128 fused launches.

usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1|c2|c3|c4|c5a|c5b|readme] [--causal]
"""
import argparse
import json
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

PEAK_TFLOPS_FP16 = 2500.0   # MI355X dense fp16 MFMA, published

# HBM bytes per launch of the forward kernel, measured with rocprofv3 (FETCH_SIZE and WRITE_SIZE
# in separate --pmc runs of this script, each scaled by what the same counter reads for the 1 GiB
# calibration copy below: 2.000 for fetch, 1.000 for write).  Summaries:
# profiles/fwd_kernel_pingpong_c3.md and profiles/fwd_kernel_pingpong_c4.md.
MEASURED_TRAFFIC_BYTES = {"c3": 134.4e6, "c4": 808.2e6}


def cpu_baseline(w, q, k, v, gpu_out, budget_s):
    """Naive float32 attention on the host cores for a bounded sample of (batch, head) pairs.

    The checker (oracle/) is used here as the timed CPU baseline and to report the error of the
    GPU result on the sampled pairs; it never produces anything the benchmark's `value` uses.
    """
    import torch

    from oracle import attention_per_head

    cores = torch.get_num_threads()
    pairs_all = [(b, h) for b in range(w.B) for h in range(w.R)]
    t0 = time.perf_counter()
    attention_per_head(q, k, v, w.H, heads=pairs_all[:1])         # warm-up, also sizes the sample
    per_pair = time.perf_counter() - t0
    n = max(1, min(len(pairs_all), int(budget_s / max(per_pair, 1e-6))))
    stride = max(1, len(pairs_all) // n)
    pairs = pairs_all[::stride][:n]
    t0 = time.perf_counter()
    ref = attention_per_head(q, k, v, w.H, heads=pairs)
    dt = time.perf_counter() - t0
    flop = 4.0 * len(pairs) * w.L * w.L * w.H
    sel = ~torch.isnan(ref)
    err = (gpu_out.float().cpu()[sel] - ref[sel]).abs().max().item()
    return {
        "value": flop / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": "%d of %d (batch, head) pairs of %s, torch float32 per-head loop, %.2f s"
                  % (len(pairs), len(pairs_all), w.name, dt),
        "ms_per_step_extrapolated": dt / len(pairs) * len(pairs_all) * 1e3,
        "gpu_max_abs_err_on_sample": err,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default="c3")
    ap.add_argument("--causal", action="store_true",
                    help="the causal extension of the C ABI instead of the reference's non-causal forward: "
                         "counts the flops of the keys at or below the diagonal, no CPU baseline")
    ap.add_argument("--calibration-copy-mib", type=int, default=1024,
                    help="size of the plain copy run before the timed region (0 disables it)")
    ap.add_argument("--cpu-budget-s", type=float, default=15.0,
                    help="seconds of host time for the CPU baseline sample (0 disables it)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the forward has no multi-GPU path "
                 "(every (batch, head) pair is independent); run with --gpus 1")

    import torch

    import fused_attn
    from fused_attention_amd import capi, workloads

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    capi.load_library()     # fail loudly if the kernel library is not built
    w = workloads.WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    q, k, v = workloads.make_inputs(w)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    chunk = min(128, w.H * 2)

    # A plain device-to-device copy of known size, outside the timed region: the reference point
    # against which the HBM counters (FETCH_SIZE / WRITE_SIZE) of a profiler run are scaled.
    if args.calibration_copy_mib > 0:
        src = torch.arange(args.calibration_copy_mib * (1 << 18), dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.causal:
        out = torch.empty_like(qd)

        def step():
            return capi.forward(qd, kd, vd, w.H, out=out, causal=True)
    else:
        def step():
            return fused_attn.attention_forward(w.H, chunk, qd, kd, vd)

    for _ in range(args.warmup):
        out = step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3

    # Kernel duration: HIP events on the launch stream around back-to-back launches.
    if args.causal:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            step()
        e1.record()
        torch.cuda.synchronize()
        kernel_ms = e0.elapsed_time(e1) / args.steps
    else:
        kernel_ms = capi.forward_timed(qd, kd, vd, w.H, out, iters=args.steps)

    # causal: query i attends to i + 1 keys
    flop = 2.0 * w.B * w.R * w.L * (w.L + 1) * w.H if args.causal else workloads.flops(w)
    value = flop / (ms_per_step * 1e-3) / 1e12
    achieved = flop / (kernel_ms * 1e-3) / 1e12
    line = {
        "metric": "fused attn fwd causal TFLOP/s (2*B*R*L*(L+1)*H)" if args.causal else "fused attn fwd TFLOP/s (4*B*R*L^2*H)",
        "value": value,
        "unit": "TFLOP/s",
        "pct_of_fp16_mfma_peak": 100.0 * value / PEAK_TFLOPS_FP16,
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "%s: B=%d R=%d L=%d H=%d %s, fp16 N(0,%g) seeded on the host, "
                        "fed as [B, L, R*H]" % (w.name, w.B, w.R, w.L, w.H, "causal" if args.causal else "non-causal",
                                                w.q_std),
            "flop_per_step": flop,
            "bytes_per_step": workloads.io_bytes(w),
        },
        "roofline": {
            "bound": "mfma",
            "achieved": achieved,
            "peak": PEAK_TFLOPS_FP16,
            "unit": "TFLOP/s",
            "frac": achieved / PEAK_TFLOPS_FP16,
            "traffic": None if args.causal else MEASURED_TRAFFIC_BYTES.get(w.name),
            "kernel_ms": kernel_ms,
        },
    }
    if args.cpu_budget_s > 0 and not args.causal:
        line["cpu_baseline"] = cpu_baseline(w, q, k, v, out, args.cpu_budget_s)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
