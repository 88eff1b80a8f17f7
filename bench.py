#!/usr/bin/env python3
"""Benchmark of the fused-bias attention forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--full] [--no-cpu] [--no-extra] [--shape BxL[c]]

A step is one launch of the dense fused-bias forward at the op-level T5-base shape (batch 16,
12 heads, head_dim 64, Lq = Lk = 1024, bf16, bidirectional buckets, no 1/sqrt(d) scaling) with
inputs resident in HBM.  Prints ONE JSON line:

  value / ms_per_step   TFLOP/s of that workload (4*B*H*L*L*D algorithmic FLOPs per launch), wall
                        clock around K launches with a device synchronise on both sides
  roofline              the same kernel timed with device events on the launch stream, against the
                        published dense bf16 MFMA peak
  sweep                 longer sequences at constant B*L = 16384 (the "seq >= 4096" target)
  extra                 the other workloads of the baseline: packed variable-length batch (bidirectional
                        and causal), the three sparse patterns at L = 16384, T5-base encoder tokens/s at
                        8k tokens; with --full also the 100k-token encoder pass and batch-64 greedy
                        decoding over an 8192-token memory (split-K cross-attention)
  cpu_baseline          the CPU 'basic' path (materialised bias, einsum, fp32 softmax, einsum) timed on
                        the host cores on a bounded sample of the same workload
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
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, published
# HBM bytes per launch of the headline kernel: rocprofv3 FETCH_SIZE and WRITE_SIZE, each scaled by what the
# same counter reads for a 256 MiB device copy (profiles/fwd_kernel_bf16_d64_dense_B16_L1024.hbm_traffic.txt)
MEASURED_TRAFFIC_BYTES = 1.0212e8
B, H, L, D = 16, 12, 1024, 64


def make_inputs(torch, dev, b, h, l, d, seed=0):
    g = torch.Generator().manual_seed(seed)
    q, k, v = ((0.5 * torch.randn(b, h, l, d, generator=g)).to(torch.bfloat16).to(dev) for _ in range(3))
    table = torch.randn(32, h, generator=g).to(dev)
    return q, k, v, table


def time_kernel(torch, fn, steps, warmup, ramp_ms=120.0):
    """(wall ms per step with host syncs on both sides, device ms per launch).

    After an idle period the device needs some tens of milliseconds of uninterrupted work before its clocks
    settle (the same launch runs 20-40 % slower during that ramp), so the workload first runs untimed for
    about ``ramp_ms``; then the W warm-up steps, then exactly K timed steps.  The device figure comes from
    one pair of events recorded on the launch stream (torch's current stream, the one the library is
    handed) around the K back-to-back launches; events between the launches would put marker packets into
    the queue and stretch the region they measure."""
    t_ramp = time.perf_counter()
    while (time.perf_counter() - t_ramp) * 1e3 < ramp_ms:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return wall, start.elapsed_time(stop) / steps


def c3_lengths(torch):
    return torch.randint(128, 4097, (32,), generator=torch.Generator().manual_seed(1)).tolist()


def extra_workloads(torch, dev, steps, full):
    from turbot5_amd import ops
    out = {}
    reps, warm = max(10, steps // 2), 5

    # ---- packed variable-length batch: 32 sequences, lengths U[128, 4096] (seed 1)
    lens = c3_lengths(torch)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=dev)
    tot = sum(lens)
    g = torch.Generator().manual_seed(3)
    q, k, v = ((0.5 * torch.randn(tot, H, D, generator=g)).to(torch.bfloat16).to(dev) for _ in range(3))
    table = torch.randn(32, H, generator=g).to(dev)
    for causal in (False, True):
        f = lambda: ops.flash_attention_with_fusing_bias_varlen(q, k, v, table, cu, cu, max(lens), max(lens),  # noqa: E731
                                                                causal=causal, sm_scale=1.0)
        _, ms = time_kernel(torch, f, reps, warm)
        pairs = sum(n * (n + 1) // 2 for n in lens) if causal else sum(n * n for n in lens)
        tf = 4.0 * H * D * pairs / (ms * 1e-3) / 1e12
        out["varlen_causal" if causal else "varlen_bidirectional"] = {
            "total_tokens": tot, "ms": round(ms, 4), "tflops": round(tf, 1), "frac_mfma_peak": round(tf / PEAK_BF16_TFLOPS, 4)}
    del q, k, v

    # ---- causal dense (decoder self-attention over a prompt): FLOPs of the visible pairs only
    for bsz, ln in ((16, 1024), (4, 4096)):
        q, k, v, table = make_inputs(torch, dev, bsz, H, ln, D, seed=7)
        f = lambda: ops.flash_attention_with_fusing_bias(q, k, v, table, causal=True, sm_scale=1.0)  # noqa: E731
        _, ms = time_kernel(torch, f, reps, warm)
        tf = 4.0 * bsz * H * D * (ln * (ln + 1) // 2) / (ms * 1e-3) / 1e12
        out[f"dense_causal_B{bsz}_H{H}_L{ln}"] = {"ms": round(ms, 4), "tflops": round(tf, 1),
                                                 "frac_mfma_peak": round(tf / PEAK_BF16_TFLOPS, 4)}
        del q, k, v

    # ---- head_dim 128 (the T5-3B / 11B head shape): B4 H6 L4096, same FLOPs as the B4 H12 D64 sweep point
    g = torch.Generator().manual_seed(6)
    q, k, v = ((0.5 * torch.randn(4, 6, 4096, 128, generator=g)).to(torch.bfloat16).to(dev) for _ in range(3))
    table = torch.randn(32, 6, generator=g).to(dev)
    f = lambda: ops.flash_attention_with_fusing_bias(q, k, v, table, causal=False, sm_scale=1.0)  # noqa: E731
    _, ms = time_kernel(torch, f, reps, warm)
    tf = 4.0 * 4 * 6 * 4096 * 4096 * 128 / (ms * 1e-3) / 1e12
    out["dense_head_dim_128_B4_H6_L4096"] = {"ms": round(ms, 4), "tflops": round(tf, 1), "frac_mfma_peak": round(tf / PEAK_BF16_TFLOPS, 4)}
    del q, k, v

    # ---- sparse patterns, B1 H12 L16384 D64
    Ls = 16384
    q, k, v, table = make_inputs(torch, dev, 1, H, Ls, D, seed=4)
    bytes_min = 4 * H * Ls * D * 2
    f = lambda: ops.local_attention_with_fusing_bias(q, k, v, table, 128)  # noqa: E731
    _, ms = time_kernel(torch, f, reps, warm)
    pairs = Ls * 255 - 127 * 128
    out["local_r127"] = {"ms": round(ms, 4), "tflops_live_pairs": round(4.0 * H * D * pairs / ms / 1e9, 1),
                         "gbs_min_bytes": round(bytes_min / ms / 1e6, 1)}
    f = lambda: ops.block_attention_with_fusing_bias(q, k, v, table, 128, 64)  # noqa: E731
    _, ms = time_kernel(torch, f, reps, warm)
    pairs = 64 * Ls + (Ls - 64) * 192 - 64 * 64
    out["block_128_g64"] = {"ms": round(ms, 4), "tflops_live_pairs": round(4.0 * H * D * pairs / ms / 1e9, 1),
                            "gbs_min_bytes": round(bytes_min / ms / 1e6, 1)}
    g = torch.Generator().manual_seed(5)
    sk, sv = ((0.5 * torch.randn(1, H, Ls // 16, D, generator=g)).to(torch.bfloat16).to(dev) for _ in range(2))
    f = lambda: ops.transient_global_attention_with_fusing_bias(q, k, v, sk, sv, table, 128, 16)  # noqa: E731
    _, ms = time_kernel(torch, f, reps, warm)
    pairs = Ls * 255 - 127 * 128 + Ls * (Ls // 16)
    out["tglobal_r127_g16"] = {"ms": round(ms, 4), "tflops_live_pairs": round(4.0 * H * D * pairs / ms / 1e9, 1)}
    del q, k, v, sk, sv

    # ---- T5-base encoder, tokens/s at 8k tokens
    from turbot5_amd import T5Config, T5EncoderModel, T5Model
    base = dict(vocab_size=32128, d_model=768, d_kv=64, d_ff=3072, num_layers=12, num_heads=12, dropout_rate=0.0,
                attention_type="flash")
    torch.manual_seed(0)
    enc = T5EncoderModel(T5Config(attention_dtype=torch.bfloat16, **base)).eval().to(dev)
    ids_g = torch.Generator().manual_seed(0)
    with torch.no_grad():
        for bsz in (2, 1):
            ids = torch.randint(0, 32128, (bsz, 8192), generator=ids_g).to(dev)
            f = lambda: enc(ids)  # noqa: E731
            _, ms = time_kernel(torch, f, 5, 2)
            out[f"t5_base_encoder_8k_B{bsz}_fp32_act_bf16_attn"] = {
                "ms": round(ms, 2), "tokens_per_s": round(bsz * 8192 / (ms * 1e-3), 1)}
        enc16 = enc.to(torch.bfloat16)
        enc16.config.attention_dtype = None
        for blk in enc16.encoder.block:
            blk.layer[0].SelfAttention.config.attention_dtype = None
        ids = torch.randint(0, 32128, (2, 8192), generator=ids_g).to(dev)
        f = lambda: enc16(ids)  # noqa: E731
        _, ms = time_kernel(torch, f, 5, 2)
        out["t5_base_encoder_8k_B2_bf16"] = {"ms": round(ms, 2), "tokens_per_s": round(2 * 8192 / (ms * 1e-3), 1)}
        # a padded batch: 16 rows of 4096 positions, 128..4096 valid tokens each (right padding); the stack packs
        # the valid tokens once and runs all 12 layers on them, with one launch plan shared by the layers
        plens = torch.randint(128, 4097, (16,), generator=torch.Generator().manual_seed(2))
        pmask = (torch.arange(4096)[None, :] < plens[:, None]).to(torch.float32).to(dev)
        ids = torch.randint(0, 32128, (16, 4096), generator=ids_g).to(dev)
        f = lambda: enc16(ids, pmask)  # noqa: E731
        _, ms = time_kernel(torch, f, 5, 2)
        out["t5_base_encoder_padded_B16_L4096_bf16"] = {
            "ms": round(ms, 2), "valid_tokens": int(plens.sum()), "valid_tokens_per_s": round(int(plens.sum()) / (ms * 1e-3), 1)}
        if full:
            ids = torch.randint(0, 32128, (1, 100000), generator=ids_g).to(dev)
            f = lambda: enc16(ids)  # noqa: E731
            _, ms = time_kernel(torch, f, 2, 1, ramp_ms=0.0)
            attn_flops = 12 * 4.0 * 12 * 64 * 1e5 * 1e5
            out["t5_base_encoder_100k_B1_bf16"] = {"ms": round(ms, 1), "tokens_per_s": round(1e5 / (ms * 1e-3), 1),
                                                   "attention_tflops_lower_bound": round(attn_flops / ms / 1e9, 1)}
    del enc
    if full:
        # ---- the baseline's small configuration (T5-small, 4 x 512 ids): a pass is a hundred short launches, bound by
        # the host; the same pass as one HIP graph
        from turbot5_amd import GraphedForward
        small = dict(vocab_size=32128, d_model=512, d_kv=64, d_ff=2048, num_layers=6, num_heads=8, dropout_rate=0.0,
                     attention_type="flash")
        torch.manual_seed(0)
        for dt, tag in ((torch.float32, "fp32"), (torch.bfloat16, "bf16")):
            sm = T5EncoderModel(T5Config(**small)).eval().to(dev).to(dt)
            ids = torch.randint(0, 32128, (4, 512), generator=torch.Generator().manual_seed(0)).to(dev)
            graphed = GraphedForward(sm, ids)
            with torch.no_grad():
                _, ms_e = time_kernel(torch, lambda: sm(ids), 50, 10)
            _, ms_g = time_kernel(torch, lambda: graphed(ids), 50, 10)
            out[f"t5_small_encoder_B4_L512_{tag}"] = {"eager_ms": round(ms_e, 3), "graphed_ms": round(ms_g, 3),
                                                      "graphed_tokens_per_s": round(2048 / (ms_g * 1e-3), 1)}
            del sm, graphed
        # ---- greedy decoding, batch 64 over an 8192-token encoder memory, 64 steps
        torch.manual_seed(0)
        model = T5Model(T5Config(attention_dtype=torch.bfloat16, **base)).eval().to(dev)
        mem = torch.randn(64, 8192, 768, generator=torch.Generator().manual_seed(6)).to(dev)
        steps_dec = 64
        with torch.no_grad():
            # the baseline's end-to-end case: 100k-token encoder input, 128-token decoder, fp32 activations, bf16 attention
            ids = torch.randint(0, 32128, (1, 100000), generator=torch.Generator().manual_seed(8)).to(dev)
            dec_ids = torch.randint(0, 32128, (1, 128), generator=torch.Generator().manual_seed(9)).to(dev)
            f = lambda: model(ids, dec_ids)  # noqa: E731
            _, ms = time_kernel(torch, f, 2, 1, ramp_ms=0.0)
            out["t5_base_encdec_100k_enc_128_dec_fp32_act_bf16_attn"] = {
                "ms": round(ms, 1), "encoder_tokens_per_s": round(1e5 / (ms * 1e-3), 1)}
            del ids, dec_ids
            model.greedy_decode(encoder_outputs=mem, max_new_tokens=4)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            model.greedy_decode(encoder_outputs=mem, max_new_tokens=steps_dec)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
        out["greedy_decode_B64_mem8192"] = {"steps": steps_dec, "ms_per_step": round(dt / steps_dec * 1e3, 3),
                                            "tokens_per_s": round(64 * steps_dec / dt, 1)}
        # small batches are bound by host launches: the same loop against one HIP graph per step
        # (whole calls timed: cross-attention K/V projection of the memory + 64 steps)
        with torch.no_grad():
            for bsz in (8, 1):
                memb = mem[:bsz].contiguous()
                res = {}
                for name, fn in (("eager", lambda: model.greedy_decode(encoder_outputs=memb, max_new_tokens=steps_dec)),
                                 ("graphed", lambda: model.greedy_decode_graphed(memb, steps_dec))):
                    fn()
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    fn()
                    torch.cuda.synchronize()
                    res[name] = time.perf_counter() - t0
                out[f"greedy_decode_B{bsz}_mem8192"] = {
                    "steps": steps_dec, "eager_ms_per_step": round(res["eager"] / steps_dec * 1e3, 3),
                    "graphed_ms_per_step": round(res["graphed"] / steps_dec * 1e3, 3),
                    "graphed_tokens_per_s": round(bsz * steps_dec / res["graphed"], 1)}
        # the split-K cross-attention alone: one layer-step reads K and V of the whole memory once
        g = torch.Generator().manual_seed(7)
        kc = (0.5 * torch.randn(64, 8192, 12, 64, generator=g)).to(torch.bfloat16).to(dev).transpose(1, 2)
        vc = (0.5 * torch.randn(64, 8192, 12, 64, generator=g)).to(torch.bfloat16).to(dev).transpose(1, 2)
        qd = (0.5 * torch.randn(64, 12, 1, 64, generator=g)).to(torch.bfloat16).to(dev)
        f = lambda: ops.flash_decoding_attention(qd, kc, vc, None, 1.0)  # noqa: E731
        _, ms = time_kernel(torch, f, 20, 5)
        nbytes = 2 * 64 * 8192 * 768 * 2
        out["splitk_cross_attention_layer_step"] = {"ms": round(ms, 4), "gbs": round(nbytes / ms / 1e6, 1),
                                                    "frac_hbm_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
    return out


def cpu_baseline(torch, seconds_budget=20.0):
    """The oracle's 'basic' path (materialised bias, einsum, fp32 softmax, einsum) on the host cores,
    on whole batch elements of the bench workload until about the budget is used."""
    from oracle import t5_basic as O
    threads = torch.get_num_threads()
    g = torch.Generator().manual_seed(0)
    q, k, v = (0.5 * torch.randn(1, H, L, D, generator=g) for _ in range(3))
    table = torch.randn(32, H, generator=g)
    O.dense_attention(q, k, v, table, False, 1.0)          # warm-up
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < seconds_budget and len(times) < 64):
        t0 = time.perf_counter()
        O.dense_attention(q, k, v, table, False, 1.0)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    flops = 4.0 * H * L * L * D
    return {"value": round(flops / med / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"{len(times)} runs of 1 of the {B} batch elements (H{H} L{L} D{D}, fp32 'basic' with "
                      f"materialised bias), median {med * 1e3:.1f} ms"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--full", action="store_true", help="also run the 100k-token encoder pass and the decode loop")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="only the headline workload (no sweep, no extra legs)")
    ap.add_argument("--shape", default=None, metavar="BxL[c]",
                    help="only time the dense forward at batch B, length L (suffix c: causal); for profiling runs")
    ap.add_argument("--copy-probe", action="store_true",
                    help="only run five plain 256 MiB device copies (calibrates the HBM traffic counters)")
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
    if args.copy_probe:
        x = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev)
        y = torch.empty_like(x)
        for _ in range(5):
            y.copy_(x)
        torch.cuda.synchronize()
        print(json.dumps({"copy_probe_bytes_per_copy": x.numel()}))
        return

    if args.shape:
        causal = args.shape.endswith("c")
        b, l = (int(x) for x in args.shape.rstrip("c").split("x"))
        q, k, v, table = make_inputs(torch, dev, b, H, l, D, seed=l)
        f = lambda: flash_attention_with_fusing_bias(q, k, v, table, causal=causal, sm_scale=1.0)  # noqa: E731
        _, ms = time_kernel(torch, f, args.steps, args.warmup)
        fl = 4.0 * b * H * D * (l * (l + 1) // 2 if causal else l * l)
        print(json.dumps({"shape": args.shape, "kernel_ms": round(ms, 5), "tflops": round(fl / ms / 1e9, 1),
                          "frac_mfma_peak": round(fl / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}))
        return

    q, k, v, table = make_inputs(torch, dev, B, H, L, D)
    fn = lambda: flash_attention_with_fusing_bias(q, k, v, table, causal=False, sm_scale=1.0)  # noqa: E731
    wall_ms, dev_ms = time_kernel(torch, fn, args.steps, args.warmup)
    flops = 4.0 * B * H * L * L * D
    value = flops / (wall_ms * 1e-3) / 1e12
    achieved = flops / (dev_ms * 1e-3) / 1e12

    sweep, extra = {}, {}
    if not args.no_extra:
        for l in (2048, 4096, 8192, 16384):
            b = max(1, 16384 // l)
            qs, ks, vs, ts = make_inputs(torch, dev, b, H, l, D, seed=l)
            f = lambda: flash_attention_with_fusing_bias(qs, ks, vs, ts, causal=False, sm_scale=1.0)  # noqa: E731
            _, ms = time_kernel(torch, f, args.steps, args.warmup)
            tf = 4.0 * b * H * l * l * D / (ms * 1e-3) / 1e12
            sweep[f"B{b}_L{l}"] = {"ms": round(ms, 4), "tflops": round(tf, 1), "frac_mfma_peak": round(tf / PEAK_BF16_TFLOPS, 4)}
            del qs, ks, vs, ts
        extra = extra_workloads(torch, dev, args.steps, args.full)

    line = {
        "metric": "fused-bias attn fwd TFLOP/s + % MFMA peak; T5-base encoder tokens/s @8k",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"dense bidirectional fused-bias attention forward, B{B} H{H} Lq=Lk={L} D{D} bf16, "
                               "32 buckets max_distance 128, sm_scale 1.0 (baseline configuration 2)",
                   "device": props.name, "compute_units": props.multi_processor_count},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": MEASURED_TRAFFIC_BYTES,
                     "kernel": "t5a::fwd_kernel<bf16, 64, dense, non-causal>", "kernel_ms": round(dev_ms, 5),
                     "algorithmic_flops_per_launch": flops},
        "tokens_per_s": round(B * L / (wall_ms * 1e-3), 1),
        "sweep": sweep,
        "extra": extra,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(torch)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
