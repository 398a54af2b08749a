"""Benchmark of the fused attention forward on one MI355X.

One step = one forward pass (softmax(Q K^T / sqrt(H)) V for every batch and head) over one
synthetic batch resident in HBM.  Prints one JSON line: whole-job TFLOP/s with
flop = 4*B*R*L^2*H, the MFMA roofline of the kernel (average launch duration from HIP events
recorded on the launch stream inside the kernel library) and, beside it, the naive float32 CPU
evaluation of the same workload timed on the host cores over a bounded sample of (batch, head)
pairs.  Counterpart of the reference's benchmark (reference tests/benchmark_fused_attn.py:8-45),
which prints wall-clock milliseconds of 128 naive and 128 fused launches.

Before the counted warm-up the step is launched for half a second, so that the chip's clock has
settled ("settle_launches"); "value_cold" is the same measurement taken before that loop, after
the --warmup launches only.  With the default workload the line also carries "workloads": kernel
time, TFLOP/s, roofline fraction and error on a bounded sample for the other configurations and for
the QKV projection front end.

usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1|c2|c3|c4|c5a|c5b|readme] [--causal]
                       [--mask causal|zero] [--projection plain|rotary] [--others auto|on|off]
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

# HBM bytes per launch of the forward kernel.  They are not measured by this script: they were read
# with rocprofv3 (FETCH_SIZE and WRITE_SIZE in separate --pmc runs of this script, each scaled by
# what the same counter reads for the 1 GiB calibration copy below: 2.000 for fetch, 1.000 for
# write) and are quoted here with the file that holds the counter summary.  Workloads without a
# counter run report null.  The counter runs were made at the commit that last touched each file's
# counters (c3, c4 and readme at the commit that gave the 16 x 16 kernel its conflict-free K chunk order; c3_mask c1f4501; the projection at the commit that rewrote it on 16 x 16 x 32 instructions); the kernel
# each of these workloads runs has not changed since.
MEASURED_TRAFFIC = {
    "c3": (134.4e6, "profiles/fwd_kernel_pp16_c3.md"),
    "c3_mask": (470.0e6, "profiles/fwd_kernel_pingpong_mask.md"),
    "c4": (805.5e6, "profiles/fwd_kernel_pp16_c4.md"),
    "readme": (335.7e6, "profiles/fwd_kernel_pp16_readme.md"),
    "qkv_proj_c3": (268.6e6, "profiles/qkv_proj_kernel_c3.md"),
    "qkv_proj_readme": (2181.2e6, "profiles/qkv_proj_kernel_readme.md"),
}

# Launches made before the counted warm-up until this much time has passed: the chip needs a few
# hundred milliseconds of work before its clock settles (a 25-launch run reads about 10 % low).
SETTLE_SECONDS = 0.5

# The other benchmark configurations, measured after the headline line's timed region: seconds of
# event-timed launches per workload, and host seconds for the error check of each.
OTHER_WORKLOADS = ("c1", "c2", "c4", "c5a", "c5b", "readme")


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


def settle(step, seconds):
    """Launches `step` until `seconds` have passed; returns the number of launches."""
    import torch

    n = 0
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            step()
        torch.cuda.synchronize()
        n += 8
    return n


def side_workload(name, dev, check_budget_s):
    """Kernel time, TFLOP/s and error on a bounded sample of (batch, head) pairs for one of the
    configurations that are not the headline: HIP events around back-to-back launches inside the
    kernel library, after a settle loop of its own."""
    import torch

    import fused_attn
    from fused_attention_amd import capi, workloads
    from oracle import attention_per_head

    w = workloads.WORKLOADS[name]
    q, k, v = workloads.make_inputs(w)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    out = fused_attn.attention_forward(w.H, min(128, 2 * w.H), qd, kd, vd)
    torch.cuda.synchronize()
    one = max(capi.forward_timed(qd, kd, vd, w.H, out, iters=3), 1e-3)
    settle_iters = max(8, int(0.3e3 / one))
    capi.forward_timed(qd, kd, vd, w.H, out, iters=settle_iters)
    iters = max(50, min(5000, int(0.3e3 / one)))
    kernel_ms = capi.forward_timed(qd, kd, vd, w.H, out, iters=iters)
    flop = workloads.flops(w)
    tflops = flop / (kernel_ms * 1e-3) / 1e12
    entry = {
        "shape": "B=%d R=%d L=%d H=%d" % (w.B, w.R, w.L, w.H),
        "kernel_ms": kernel_ms,
        "launches_timed": iters,
        "tflops": tflops,
        "frac": tflops / PEAK_TFLOPS_FP16,
    }
    if check_budget_s > 0:
        pairs_all = [(b, h) for b in range(w.B) for h in range(w.R)]
        t0 = time.perf_counter()
        ref = attention_per_head(q, k, v, w.H, heads=pairs_all[:1])
        per_pair = time.perf_counter() - t0
        n = max(1, min(len(pairs_all), int(check_budget_s / max(per_pair, 1e-6))))
        # spread over batches and heads; the first pair has been computed already
        extra = pairs_all[1::max(1, len(pairs_all) // n)][:n - 1]
        if extra:
            more = attention_per_head(q, k, v, w.H, heads=extra)
            ref = torch.where(torch.isnan(ref), more, ref)
        got = out.float().cpu()
        sel = ~torch.isnan(ref)
        entry["max_abs_err"] = (got[sel] - ref[sel]).abs().max().item()
        entry["finite"] = bool(torch.isfinite(got).all())
        entry["pairs_checked"] = 1 + len(extra)
    return entry


def variant_workload(name, dev, variant):
    """The extensions of the C ABI on a benchmark configuration: 'bf16' (bfloat16 tensors), 'causal',
    'mask' (an additive fp16 [B, L, L] mask of zeros below and -inf above the diagonal, which gives
    the causal result).  Kernel time from HIP events around back-to-back launches inside the kernel
    library (fa_fwd_timed_ex), after a settle loop; flop counts every (query, key) pair the variant
    attends to; error against the float32 oracle on four (batch, head) pairs."""
    import torch

    from fused_attention_amd import capi, workloads
    from oracle import attention, causal_mask

    w = workloads.WORKLOADS[name]
    q, k, v = workloads.make_inputs(w)
    dt = torch.bfloat16 if variant == "bf16" else torch.float16
    q, k, v = q.to(dt), k.to(dt), v.to(dt)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    causal = variant == "causal"
    mask = None
    if variant == "mask":
        mask = torch.full((w.L, w.L), float("-inf")).triu(1).to(torch.float16).expand(w.B, w.L, w.L).contiguous().to(dev)
    out = torch.empty_like(qd)

    capi.forward(qd, kd, vd, w.H, out=out, causal=causal, mask=mask)
    torch.cuda.synchronize()
    flop = workloads.flops(w) if variant == "bf16" else 2.0 * w.B * w.R * w.L * (w.L + 1) * w.H

    def timed(iters):
        return capi.forward_timed(qd, kd, vd, w.H, out, iters=iters, causal=causal, mask=mask)

    one = max(timed(3), 1e-3)
    timed(max(8, int(0.3e3 / one)))                 # settle
    iters = max(50, min(5000, int(0.3e3 / one)))
    kernel_ms = timed(iters)
    # four (batch, head) pairs spread over batches and heads, each as a one-head problem of its own
    pairs = sorted({(b, h) for b, h in ((0, 0), (w.B - 1, w.R - 1), (w.B // 2, w.R // 3), (w.B // 3, (2 * w.R) // 3))})
    err = 0.0
    for b, h in pairs:
        cols = slice(h * w.H, (h + 1) * w.H)
        q1, k1, v1 = (t[b:b + 1, :, cols].float() for t in (q, k, v))
        ref = attention(q1, k1, v1, w.H, mask=None if variant == "bf16" else causal_mask(1, w.L))
        err = max(err, (out[b:b + 1, :, cols].float().cpu() - ref).abs().max().item())
    tflops = flop / (kernel_ms * 1e-3) / 1e12
    return {
        "shape": "B=%d R=%d L=%d H=%d %s" % (w.B, w.R, w.L, w.H, variant),
        "kernel_ms": kernel_ms,
        "launches_timed": iters,
        "flop_counted": "4*B*R*L^2*H" if variant == "bf16" else "2*B*R*L*(L+1)*H (pairs at or below the diagonal)",
        "tflops": tflops,
        "frac": tflops / PEAK_TFLOPS_FP16,
        "max_abs_err": err,
        "finite": bool(torch.isfinite(out.float()).all()),
        "pairs_checked": len(pairs),
        "traffic": MEASURED_TRAFFIC.get(name + "_" + variant, (None, None))[0],
        "traffic_source": MEASURED_TRAFFIC.get(name + "_" + variant, (None, None))[1],
    }


def projection_workload(name, dev, rope, iters=None):
    """The fused QKV projection front end (fa_qkv_proj) at the feature sizes of a benchmark
    configuration: hidden [B, L, R*H] times weight [R*H, 3*R*H] into the packed qkv tensor the
    attention kernel reads.  Kernel time from events on the launch stream (torch's current stream);
    flop = 2 * B*L * R*H * 3*R*H; error against the float32 oracle on a sample of rows."""
    import math

    import torch

    from fused_attention_amd import capi, workloads
    from oracle import qkv_projection, rope_tables

    w = workloads.WORKLOADS[name]
    F = w.R * w.H
    gen = torch.Generator().manual_seed(w.seed * 1000 + 7)
    x = torch.randn(w.B, w.L, F, generator=gen).to(torch.float16)
    wt = (torch.randn(F, 3 * F, generator=gen) / math.sqrt(F)).to(torch.float16)
    tables = rope_tables(w.L, w.H) if rope else None
    xd, wd = x.to(dev), wt.to(dev)
    td = tuple(t.to(dev) for t in tables) if rope else None
    out = torch.empty(w.B, w.L, 3, F, dtype=torch.float16, device=dev)

    def step():
        return capi.qkv_project(xd, wd, w.R, w.H, rope=td, out=out)

    flop = 2.0 * w.B * w.L * F * 3 * F
    step()
    torch.cuda.synchronize()
    profiled_iters = iters
    if iters is None:
        iters = max(20, min(2000, int(0.3 / (flop / 0.9e15))))
    for _ in range(iters):
        step()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        step()
    e1.record()
    torch.cuda.synchronize()
    kernel_ms = e0.elapsed_time(e1) / iters
    # for scale, the vendor library's plain GEMM on the same operands (no bias, no rotation, an
    # [M, 3F] result), timed the same way; left out of profiled runs (iters given)
    vendor = None
    if profiled_iters is None and not rope:
        x2, o2 = xd.view(w.B * w.L, F), torch.empty(w.B * w.L, 3 * F, dtype=torch.float16, device=dev)
        for _ in range(iters):
            torch.matmul(x2, wd, out=o2)
        e0.record()
        for _ in range(iters):
            torch.matmul(x2, wd, out=o2)
        e1.record()
        torch.cuda.synchronize()
        vendor_ms = e0.elapsed_time(e1) / iters
        vendor = {"what": "torch.matmul (hipBLASLt) on the same x and w", "kernel_ms": vendor_ms,
                  "tflops": flop / (vendor_ms * 1e-3) / 1e12}
    rows = torch.arange(0, w.L, max(1, w.L // 64))
    want = qkv_projection(x[:1, rows], wt, None, w.R, w.H, *((tables[0][rows], tables[1][rows]) if rope else (None, None)))
    got = out[:1, rows.to(dev)].float().cpu()
    tflops = flop / (kernel_ms * 1e-3) / 1e12
    return {
        "shape": "B=%d L=%d F_in=%d R=%d H=%d%s" % (w.B, w.L, F, w.R, w.H, " rotary" if rope else ""),
        "kernel_ms": kernel_ms,
        "launches_timed": iters,
        "tflops": tflops,
        "frac": tflops / PEAK_TFLOPS_FP16,
        "max_abs_err": (got - want).abs().max().item(),
        "finite": bool(torch.isfinite(out.float()).all()),
        "rows_checked": int(rows.numel()),
        "bytes_algorithmic": (w.B * w.L * F + F * 3 * F + w.B * w.L * 3 * F) * 2,
        "traffic": None if rope else MEASURED_TRAFFIC.get("qkv_proj_" + name, (None, None))[0],
        "traffic_source": None if rope else MEASURED_TRAFFIC.get("qkv_proj_" + name, (None, None))[1],
        "vendor_gemm": vendor,
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
    ap.add_argument("--mask", choices=["causal", "zero"], default=None,
                    help="the additive-mask path instead of the plain forward: an fp16 [B, L, L] mask of zeros below "
                         "and -inf above the diagonal (the causal result; counts the flops of the pairs at or below "
                         "the diagonal), or a mask of zeros (the plain result, all flops); no CPU baseline")
    ap.add_argument("--calibration-copy-mib", type=int, default=1024,
                    help="size of the plain copy run before the timed region (0 disables it)")
    ap.add_argument("--cpu-budget-s", type=float, default=15.0,
                    help="seconds of host time for the CPU baseline sample (0 disables it)")
    ap.add_argument("--projection", choices=["plain", "rotary"], default=None,
                    help="measure the fused QKV projection front end at the workload's feature sizes "
                         "instead of the attention forward (one JSON line, flop = 2*B*L*F*3F)")
    ap.add_argument("--others", choices=["auto", "on", "off"], default="auto",
                    help="also measure the other benchmark configurations into \"workloads\" "
                         "(auto: with the default headline workload, non-causal)")
    ap.add_argument("--check-budget-s", type=float, default=4.0,
                    help="host seconds per workload for the error check of the other configurations")
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
    # A plain device-to-device copy of known size, outside the timed region: the reference point
    # against which the HBM counters (FETCH_SIZE / WRITE_SIZE) of a profiler run are scaled.
    if args.calibration_copy_mib > 0:
        src = torch.arange(args.calibration_copy_mib * (1 << 18), dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.projection:
        entry = projection_workload(args.workload, dev, rope=args.projection == "rotary", iters=args.steps)
        print(json.dumps({
            "metric": "fused qkv projection TFLOP/s (2*B*L*F*3F)", "value": entry["tflops"], "unit": "TFLOP/s",
            "n_gpus": 1, "steps": entry["launches_timed"], "warmup": entry["launches_timed"],
            "ms_per_step": entry["kernel_ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "f16", "data": "synthetic", "config": {"workload": "qkv projection, " + entry["shape"]},
            "roofline": {"bound": "mfma", "achieved": entry["tflops"], "peak": PEAK_TFLOPS_FP16, "unit": "TFLOP/s",
                         "frac": entry["frac"], "traffic": None, "kernel_ms": entry["kernel_ms"]},
            "max_abs_err": entry["max_abs_err"]}))
        return
    q, k, v = workloads.make_inputs(w)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    chunk = min(128, w.H * 2)

    if args.causal and args.mask:
        sys.exit("--causal and --mask are two ways to the same result: pick one")
    mask = None
    if args.mask == "causal":
        mask = torch.full((w.L, w.L), float("-inf")).triu(1).to(torch.float16).expand(w.B, w.L, w.L).contiguous().to(dev)
    elif args.mask == "zero":
        mask = torch.zeros(w.B, w.L, w.L, dtype=torch.float16, device=dev)
    if args.causal or mask is not None:
        out = torch.empty_like(qd)

        def step():
            return capi.forward(qd, kd, vd, w.H, out=out, causal=args.causal, mask=mask)
    else:
        def step():
            return fused_attn.attention_forward(w.H, chunk, qd, kd, vd)

    def timed_steps():
        for _ in range(args.warmup):
            o = step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            o = step()
        torch.cuda.synchronize()
        return o, (time.perf_counter() - t0) / args.steps * 1e3

    # First without the settle loop ("value_cold": what --warmup and --steps alone read, the
    # figure earlier versions of this script reported as `value`), then after it.
    out, ms_per_step_cold = timed_steps()
    settle_launches = settle(step, SETTLE_SECONDS)
    out, ms_per_step = timed_steps()

    # Kernel duration: HIP events on the launch stream around back-to-back launches, inside the library.
    kernel_ms = capi.forward_timed(qd, kd, vd, w.H, out, iters=args.steps, causal=args.causal, mask=mask)

    # causal (flag or mask pattern): query i attends to i + 1 keys
    half = args.causal or args.mask == "causal"
    variant = "causal" if args.causal else ("additive mask (%s pattern)" % args.mask if args.mask else "non-causal")
    flop = 2.0 * w.B * w.R * w.L * (w.L + 1) * w.H if half else workloads.flops(w)
    value = flop / (ms_per_step * 1e-3) / 1e12
    achieved = flop / (kernel_ms * 1e-3) / 1e12
    traffic_key = w.name + ("_causal" if args.causal else "_mask" if args.mask == "causal" else "_mask_zero" if args.mask else "")
    line = {
        "metric": "fused attn fwd causal TFLOP/s (2*B*R*L*(L+1)*H)" if half else "fused attn fwd TFLOP/s (4*B*R*L^2*H)",
        "value": value,
        "unit": "TFLOP/s",
        "pct_of_fp16_mfma_peak": 100.0 * value / PEAK_TFLOPS_FP16,
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_launches": settle_launches,
        "ms_per_step": ms_per_step,
        "value_cold": flop / (ms_per_step_cold * 1e-3) / 1e12,
        "ms_per_step_cold": ms_per_step_cold,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "%s: B=%d R=%d L=%d H=%d %s, fp16 N(0,%g) seeded on the host, "
                        "fed as [B, L, R*H]" % (w.name, w.B, w.R, w.L, w.H, variant, w.q_std),
            "flop_per_step": flop,
            "bytes_per_step": workloads.io_bytes(w),
        },
        "roofline": {
            "bound": "mfma",
            "achieved": achieved,
            "peak": PEAK_TFLOPS_FP16,
            "unit": "TFLOP/s",
            "frac": achieved / PEAK_TFLOPS_FP16,
            "traffic": MEASURED_TRAFFIC.get(traffic_key, (None, None))[0],
            "traffic_source": MEASURED_TRAFFIC.get(traffic_key, (None, None))[1],
            "kernel_ms": kernel_ms,
        },
    }
    if args.cpu_budget_s > 0 and not args.causal and mask is None:
        line["cpu_baseline"] = cpu_baseline(w, q, k, v, out, args.cpu_budget_s)
    others = args.others == "on" or (args.others == "auto" and args.workload == "c3" and not args.causal and mask is None)
    if others:
        del qd, kd, vd, out
        torch.cuda.empty_cache()
        line["workloads"] = {name: side_workload(name, dev, args.check_budget_s)
                             for name in OTHER_WORKLOADS if name != args.workload}
        # the extensions of the C ABI on the headline configuration
        for variant in ("bf16", "causal", "mask"):
            line["workloads"]["c3_" + variant] = variant_workload("c3", dev, variant)
        # the projection front end at the headline's and the reference benchmark's feature sizes
        line["workloads"]["qkv_proj_c3"] = projection_workload("c3", dev, rope=False)
        line["workloads"]["qkv_proj_c3_rotary"] = projection_workload("c3", dev, rope=True)
        line["workloads"]["qkv_proj_readme"] = projection_workload("readme", dev, rope=False)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
