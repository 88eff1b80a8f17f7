#!/usr/bin/env python3
"""Benchmark of the fused-bias attention forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one launch of the dense fused-bias forward at the op-level T5-base shape
(batch 16, 12 heads, head_dim 64, Lq = Lk = 1024, bf16, bidirectional buckets, no
1/sqrt(d) scaling), inputs resident in HBM.  Prints ONE JSON line: the TFLOP/s of that
workload (4*B*H*L*L*D algorithmic FLOPs per launch), the MFMA roofline fraction of the
kernel measured with device events, a sweep over longer sequences, and the CPU 'basic'
baseline timed on the host cores for a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published
B, H, L, D = 16, 12, 1024, 64


def make_inputs(torch, dev, b, h, l, d, seed=0):
    g = torch.Generator().manual_seed(seed)
    q, k, v = ((0.5 * torch.randn(b, h, l, d, generator=g)).to(torch.bfloat16).to(dev) for _ in range(3))
    table = torch.randn(32, h, generator=g).to(dev)
    return q, k, v, table


def time_kernel(torch, fn, steps, warmup):
    """(wall ms per step with host syncs on both sides, device-event ms per launch)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for s, e in ev:
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    dev_ms = sum(s.elapsed_time(e) for s, e in ev) / steps
    return wall, dev_ms


def cpu_baseline(torch, seconds_budget=20.0):
    """The oracle's 'basic' path (materialised bias, einsum, fp32 softmax, einsum) on the host cores,
    on whole batch elements of the bench workload until ~the budget is used."""
    from oracle import t5_basic as O
    threads = torch.get_num_threads()
    g = torch.Generator().manual_seed(0)
    q, k, v = (0.5 * torch.randn(1, H, L, D, generator=g) for _ in range(3))
    table = torch.randn(32, H, generator=g)
    O.dense_attention(q, k, v, table, False, 1.0)          # warm-up
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < seconds_budget and len(times) < 16):
        t0 = time.perf_counter()
        O.dense_attention(q, k, v, table, False, 1.0)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    flops = 4.0 * H * L * L * D
    return {"value": flops / med / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"{len(times)} runs of 1 of the {B} batch elements (H{H} L{L} D{D}, fp32 'basic' with "
                      f"materialised bias), median {med * 1e3:.1f} ms"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sweep", action="store_true", help="skip the longer-sequence sweep")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    from turbot5_amd.ops import flash_attention_with_fusing_bias
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    props = torch.cuda.get_device_properties(dev)

    q, k, v, table = make_inputs(torch, dev, B, H, L, D)
    fn = lambda: flash_attention_with_fusing_bias(q, k, v, table, causal=False, sm_scale=1.0)  # noqa: E731
    wall_ms, dev_ms = time_kernel(torch, fn, args.steps, args.warmup)
    flops = 4.0 * B * H * L * L * D
    value = flops / (wall_ms * 1e-3) / 1e12
    achieved = flops / (dev_ms * 1e-3) / 1e12

    sweep = {}
    if not args.no_sweep:
        for l in (2048, 4096, 8192, 16384):
            b = max(1, 16384 // l)
            qs, ks, vs, ts = make_inputs(torch, dev, b, H, l, D, seed=l)
            f = lambda: flash_attention_with_fusing_bias(qs, ks, vs, ts, causal=False, sm_scale=1.0)  # noqa: E731
            _, ms = time_kernel(torch, f, max(5, args.steps // 5), 3)
            tf = 4.0 * b * H * l * l * D / (ms * 1e-3) / 1e12
            sweep[f"B{b}_L{l}"] = {"ms": round(ms, 4), "tflops": round(tf, 1), "frac_mfma_peak": round(tf / PEAK_BF16_TFLOPS, 4)}
            del qs, ks, vs, ts

    line = {
        "metric": "fused-bias attn fwd TFLOP/s + % MFMA peak; T5-base encoder tokens/s @8k",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"dense bidirectional fused-bias attention forward, B{B} H{H} Lq=Lk={L} D{D} bf16, "
                               "32 buckets max_distance 128, sm_scale 1.0 (BASELINE config 2)",
                   "device": props.name, "compute_units": props.multi_processor_count},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": None,
                     "kernel": "t5a::fwd_kernel<bf16,64,dense,false>", "kernel_ms": round(dev_ms, 5),
                     "algorithmic_flops_per_launch": flops},
        "tokens_per_s": round(B * L / (wall_ms * 1e-3), 1),
        "sweep": sweep,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(torch)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
