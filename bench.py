#!/usr/bin/env python3
"""Benchmark of the fused-bias attention forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick] [--no-cpu] [--leg NAME]

A step is one launch of the dense fused-bias forward at the op-level T5-base shape (batch 16,
12 heads, head_dim 64, Lq = Lk = 1024, bf16, bidirectional buckets, no 1/sqrt(d) scaling) with
inputs resident in HBM.  Prints ONE JSON line:

  value / ms_per_step   TFLOP/s of that workload (4*B*H*L*L*D algorithmic FLOPs per launch), wall
                        clock around K launches with a device synchronise on both sides
  roofline              the same kernel timed with device events on the launch stream, against the
                        published dense bf16 MFMA peak; `traffic` is the HBM bytes per launch that the
                        committed counter summary under profiles/ reports (null when that file is absent)
  sweep                 longer sequences at constant B*L = 16384 (the "seq >= 4096" target)
  extra                 the other workloads of the baseline: packed variable-length batch (bidirectional
                        and causal), the three sparse patterns at L = 16384, split-K cross-attention at batch
                        64 over an 8192-token memory (HBM-bound: its own roofline entry), T5-base encoder
                        tokens/s at 8k tokens with the share of the attention kernel, the 100k-token encoder +
                        128-token decoder pass, greedy decoding at batch 64 (skipped with --quick)
  cpu_baseline          the CPU 'basic' path (materialised bias, einsum, fp32 softmax, einsum) timed on
                        the host cores on bounded samples of the same workloads, and `checks`: the max-abs
                        difference between what the timed launches wrote and that CPU path on row subsets

--leg NAME runs one kernel K times and nothing else, for profiling:
    dense:BxL[c][:exact|:prescaled]  bwd:BxL[c][:fp32|:d128]  dense_f32_c1  local  block  tglobal  splitk  varlen  varlen_causal  copy
--leg NAME --timeline does the same with the measurement build of the library (`python -m turbot5_amd.build --trace`)
and prints where the work items of the last launch spent their shader-clock cycles.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published
PEAK_F32_TFLOPS = 157.3     # MI355X dense fp32 MFMA, published
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, published
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "fwd_kernel_bf16_d64_dense_B16_L1024.hbm_traffic.txt")
B, H, L, D = 16, 12, 1024, 64
SPARSE_L = 16384


def measured_traffic_bytes():
    """HBM bytes per launch of the headline kernel as the committed rocprofv3 counter summary states them
    (FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for a plain device copy)."""
    try:
        with open(TRAFFIC_PROFILE) as f:
            m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", f.read(), re.M)
        return float(m.group(1)) if m else None
    except OSError:
        return None


def device_max_clock_ghz():
    """Maximum shader clock of the first GPU agent that rocminfo lists (GHz), or None."""
    import subprocess
    try:
        txt = subprocess.run(["rocminfo"], capture_output=True, text=True, timeout=20).stdout
    except (OSError, subprocess.SubprocessError):
        return None
    gpu = False
    for line in txt.splitlines():
        if "Device Type:" in line:
            gpu = "GPU" in line
        m = re.search(r"Max Clock Freq\. \(MHz\):\s*(\d+)", line)
        if m and gpu:
            return int(m.group(1)) / 1000.0
    # the clock line comes before the device type line of an agent: second pass keyed on the agent's name
    blocks = txt.split("*******")
    for blk in blocks:
        if "Device Type:             GPU" in blk or re.search(r"Device Type:\s+GPU", blk):
            m = re.search(r"Max Clock Freq\. \(MHz\):\s*(\d+)", blk)
            if m:
                return int(m.group(1)) / 1000.0
    return None


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


def c3_lengths():
    with open(os.path.join(ROOT, "tests", "golden", "c3_lengths.json")) as f:
        return json.load(f)["lengths"]


def pick_rows(torch, n_rows, count, seed, extra=()):
    r = torch.randperm(n_rows, generator=torch.Generator().manual_seed(seed))[:count]
    return torch.cat([r, torch.tensor([e for e in extra if 0 <= e < n_rows], dtype=torch.long)]).unique()


# ---------------------------------------------------------------------------------------------------------------
# Samples: small host copies of what a timed launch read and wrote, kept for the CPU leg's checks.
# kind, rows, q rows, keys, values, table column(s), output rows, parameters
# ---------------------------------------------------------------------------------------------------------------
class Sample:
    def __init__(self, name, kind, **kw):
        self.name, self.kind, self.kw = name, kind, kw


def dense_sample(torch, name, q, k, v, table, out, causal, b=0, h=0, seed=0):
    rows = pick_rows(torch, q.shape[2], 24, seed, extra=(0, 1, 127, 128, q.shape[2] - 1))
    return Sample(name, "dense", rows=rows, q=q[b, h, rows.to(q.device)].float().cpu(), k=k[b, h].float().cpu(),
                  v=v[b, h].float().cpu(), t=table[:, h].float().cpu(), o=out[b, h, rows.to(q.device)].float().cpu(),
                  causal=causal, offset=k.shape[2] - q.shape[2])


# ---------------------------------------------------------------------------------------------------------------
# GPU legs
# ---------------------------------------------------------------------------------------------------------------
def sparse_inputs(torch, dev):
    q, k, v, table = make_inputs(torch, dev, 1, H, SPARSE_L, D, seed=4)
    g = torch.Generator().manual_seed(5)
    sk, sv = ((0.5 * torch.randn(1, H, SPARSE_L // 16, D, generator=g)).to(torch.bfloat16).to(dev) for _ in range(2))
    return q, k, v, table, sk, sv


def splitk_inputs(torch, dev):
    g = torch.Generator().manual_seed(7)
    kc = (0.5 * torch.randn(64, 8192, 12, 64, generator=g)).to(torch.bfloat16).to(dev).transpose(1, 2)
    vc = (0.5 * torch.randn(64, 8192, 12, 64, generator=g)).to(torch.bfloat16).to(dev).transpose(1, 2)
    qd = (0.5 * torch.randn(64, 12, 1, 64, generator=g)).to(torch.bfloat16).to(dev)
    return qd, kc, vc


def varlen_inputs(torch, dev):
    lens = c3_lengths()
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32, device=dev)
    g = torch.Generator().manual_seed(3)
    q, k, v = ((0.5 * torch.randn(sum(lens), H, D, generator=g)).to(torch.bfloat16).to(dev) for _ in range(3))
    table = torch.randn(32, H, generator=g).to(dev)
    return lens, cu, q, k, v, table


def extra_workloads(torch, dev, steps, samples):
    from turbot5_amd import ops
    out = {}
    reps, warm = max(10, steps // 2), 5

    # ---- packed variable-length batch: 32 sequences, lengths U[128, 4096] (seed 1, tests/golden/c3_lengths.json)
    lens, cu, q, k, v, table = varlen_inputs(torch, dev)
    tot = sum(lens)
    for causal in (False, True):
        f = lambda: ops.flash_attention_with_fusing_bias_varlen(q, k, v, table, cu, cu, max(lens), max(lens),  # noqa: E731
                                                                causal=causal, sm_scale=1.0)
        _, ms = time_kernel(torch, f, reps, warm)
        pairs = sum(n * (n + 1) // 2 for n in lens) if causal else sum(n * n for n in lens)
        tf = 4.0 * H * D * pairs / (ms * 1e-3) / 1e12
        name = "varlen_causal" if causal else "varlen_bidirectional"
        out[name] = {"total_tokens": tot, "ms": round(ms, 4), "tflops": round(tf, 1),
                     "frac_mfma_peak": round(tf / PEAK_BF16_TFLOPS, 4)}
        o = f()
        b = lens.index(max(lens))            # the longest sequence, one head
        s, e = int(cu[b]), int(cu[b + 1])
        samples.append(dense_sample(torch, name, q[s:e].transpose(0, 1)[None], k[s:e].transpose(0, 1)[None],
                                    v[s:e].transpose(0, 1)[None], table, o[s:e].transpose(0, 1)[None], causal, 0, 7, 31))
    del q, k, v

    # ---- causal dense (decoder self-attention over a prompt): FLOPs of the visible pairs only
    for bsz, ln in ((16, 1024), (4, 4096)):
        q, k, v, table = make_inputs(torch, dev, bsz, H, ln, D, seed=7)
        f = lambda: ops.flash_attention_with_fusing_bias(q, k, v, table, causal=True, sm_scale=1.0)  # noqa: E731
        _, ms = time_kernel(torch, f, reps, warm)
        tf = 4.0 * bsz * H * D * (ln * (ln + 1) // 2) / (ms * 1e-3) / 1e12
        out[f"dense_causal_B{bsz}_H{H}_L{ln}"] = {"ms": round(ms, 4), "tflops": round(tf, 1),
                                                 "frac_mfma_peak": round(tf / PEAK_BF16_TFLOPS, 4)}
        samples.append(dense_sample(torch, f"dense_causal_B{bsz}_L{ln}", q, k, v, table, f(), True, bsz - 1, 3, 32))
        del q, k, v

    # ---- score precision modes at the headline shape and at L = 16384: the default (Q * log2 e rounded to bf16 in
    # the kernel), exact (the factor applied to the fp32 product) and prescaled (what the attention modules do: the
    # factor folded into the query projection, nothing applied in the kernel)
    modes = {}
    for bsz, ln in ((B, L), (1, 16384)):
        q, k, v, table = make_inputs(torch, dev, bsz, H, ln, D, seed=ln if ln != L else 0)
        qs = (q.float() * ops.LOG2E).to(q.dtype)
        for mode, qq, arg in (("default", q, None), ("exact", q, True), ("prescaled", qs, "prescaled")):
            f = lambda: ops.flash_attention_with_fusing_bias(qq, k, v, table, causal=False, sm_scale=1.0, exact_scores=arg)  # noqa: E731
            _, ms = time_kernel(torch, f, reps, warm)
            tf = 4.0 * bsz * H * D * ln * ln / (ms * 1e-3) / 1e12
            modes[f"B{bsz}_L{ln}_{mode}"] = {"ms": round(ms, 4), "tflops": round(tf, 1), "frac_mfma_peak": round(tf / PEAK_BF16_TFLOPS, 4)}
            if mode != "default":
                # (prescaled: the oracle gets the rows the kernel was given, divided by log2 e again)
                qref = qq if mode == "exact" else (qq.float() / ops.LOG2E)
                samples.append(dense_sample(torch, f"dense_B{bsz}_L{ln}_{mode}", qref, k, v, table, f(), False, bsz - 1, 2, 34))
        del q, k, v, qs
    out["score_modes"] = modes

    # ---- backward of the dense forward (dq, dk, dv, table gradient): the headline shape and one sweep point on the
    # 16-bit matrix cores, the headline shape on the fp32 ones as well (fp32_math), with the largest difference
    # between the two paths' gradients relative to the gradient's scale
    bw = {}
    for bsz, ln in ((B, L), (4, 4096)):
        q, k, v, table = make_inputs(torch, dev, bsz, H, ln, D, seed=ln if (bsz, ln) != (B, L) else 0)
        o, lse = ops.flash_attention_with_fusing_bias(q, k, v, table, causal=False, sm_scale=1.0, return_lse=True)
        gout = torch.randn_like(o)
        f = lambda: ops._dense_backward(q, k, v, table, o, lse, gout, False, 1.0, 32, 128, None)  # noqa: E731
        _, ms = time_kernel(torch, f, reps, warm)
        grads = f()
        tf = 10.0 * bsz * H * D * ln * ln / (ms * 1e-3) / 1e12
        bw[f"B{bsz}_L{ln}"] = {"ms": round(ms, 4), "tflops": round(tf, 1), "frac_mfma_peak": round(tf / PEAK_BF16_TFLOPS, 4)}
        if (bsz, ln) == (B, L):
            ops.BACKWARD_FP32_MATH = True
            try:
                _, ms32 = time_kernel(torch, f, max(reps // 4, 3), 2, ramp_ms=30.0)
                ref = f()
            finally:
                ops.BACKWARD_FP32_MATH = False
            tf32 = 10.0 * bsz * H * D * ln * ln / (ms32 * 1e-3) / 1e12
            bw[f"B{bsz}_L{ln}_fp32_math"] = {"ms": round(ms32, 4), "tflops": round(tf32, 1), "frac_fp32_mfma_peak": round(tf32 / PEAK_F32_TFLOPS, 4)}
            diff = 0.0
            for got, want in zip(grads, ref):
                if got is not None:
                    diff = max(diff, ((got.float() - want.float()).abs().max() / want.float().abs().max().clamp_min(1e-6)).item())
            bw["max_rel_diff_16bit_vs_fp32_math"] = round(diff, 5)
        del q, k, v, o, gout, grads
    bw["note"] = "three kernels (row statistics, dq pass, dk / dv pass); 2.5 x the forward's FLOPs"
    out["backward"] = bw
    q = k = v = o = gout = None
    del q, k, v, o, gout

    # ---- head_dim 128 (the T5-3B / 11B head shape): B4 H6 L4096, same FLOPs as the B4 H12 D64 sweep point
    g = torch.Generator().manual_seed(6)
    q, k, v = ((0.5 * torch.randn(4, 6, 4096, 128, generator=g)).to(torch.bfloat16).to(dev) for _ in range(3))
    table = torch.randn(32, 6, generator=g).to(dev)
    f = lambda: ops.flash_attention_with_fusing_bias(q, k, v, table, causal=False, sm_scale=1.0)  # noqa: E731
    _, ms = time_kernel(torch, f, reps, warm)
    tf = 4.0 * 4 * 6 * 4096 * 4096 * 128 / (ms * 1e-3) / 1e12
    out["dense_head_dim_128_B4_H6_L4096"] = {"ms": round(ms, 4), "tflops": round(tf, 1), "frac_mfma_peak": round(tf / PEAK_BF16_TFLOPS, 4)}
    samples.append(dense_sample(torch, "dense_head_dim_128", q, k, v, table, f(), False, 2, 5, 33))
    del q, k, v

    # ---- sparse patterns, B1 H12 L16384 D64 (algorithmic bytes: q, k, v read once, o written once)
    Ls = SPARSE_L
    q, k, v, table, sk, sv = sparse_inputs(torch, dev)
    bytes_min = 4 * H * Ls * D * 2
    hs = 9      # head sampled for the checks
    f = lambda: ops.local_attention_with_fusing_bias(q, k, v, table, 128)  # noqa: E731
    _, ms = time_kernel(torch, f, reps, warm)
    pairs = Ls * 255 - 127 * 128
    out["local_r127"] = {"ms": round(ms, 4), "tflops_live_pairs": round(4.0 * H * D * pairs / ms / 1e9, 1),
                         "gbs_min_bytes": round(bytes_min / ms / 1e6, 1),
                         "frac_mfma_peak": round(4.0 * H * D * pairs / ms / 1e9 / PEAK_BF16_TFLOPS, 4),
                         "frac_hbm_peak": round(bytes_min / ms / 1e6 / PEAK_HBM_GBS, 4)}
    rows = pick_rows(torch, Ls, 32, 41, extra=(0, 1, 127, 128, Ls - 128, Ls - 1))
    host = dict(k=k[0, hs].float().cpu(), v=v[0, hs].float().cpu(), t=table[:, hs].float().cpu())
    samples.append(Sample("local_r127", "local", rows=rows, q=q[0, hs, rows.to(dev)].float().cpu(),
                          o=f()[0, hs, rows.to(dev)].float().cpu(), block_len=128, **host))
    f = lambda: ops.block_attention_with_fusing_bias(q, k, v, table, 128, 64)  # noqa: E731
    _, ms = time_kernel(torch, f, reps, warm)
    pairs = 64 * Ls + (Ls - 64) * 192 - 64 * 64
    out["block_128_g64"] = {"ms": round(ms, 4), "tflops_live_pairs": round(4.0 * H * D * pairs / ms / 1e9, 1),
                            "gbs_min_bytes": round(bytes_min / ms / 1e6, 1),
                            "frac_mfma_peak": round(4.0 * H * D * pairs / ms / 1e9 / PEAK_BF16_TFLOPS, 4),
                            "frac_hbm_peak": round(bytes_min / ms / 1e6 / PEAK_HBM_GBS, 4)}
    rows = pick_rows(torch, Ls, 32, 42, extra=(0, 63, 64, 65, 127, 128, Ls - 1))
    samples.append(Sample("block_128_g64", "block", rows=rows, q=q[0, hs, rows.to(dev)].float().cpu(),
                          o=f()[0, hs, rows.to(dev)].float().cpu(), block_len=128, n_global=64, **host))
    f = lambda: ops.transient_global_attention_with_fusing_bias(q, k, v, sk, sv, table, 128, 16)  # noqa: E731
    _, ms = time_kernel(torch, f, reps, warm)
    pairs = Ls * 255 - 127 * 128 + Ls * (Ls // 16)
    out["tglobal_r127_g16"] = {"ms": round(ms, 4), "tflops_live_pairs": round(4.0 * H * D * pairs / ms / 1e9, 1),
                               "frac_mfma_peak": round(4.0 * H * D * pairs / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}
    rows = pick_rows(torch, Ls, 24, 43, extra=(0, 15, 16, Ls - 1))
    samples.append(Sample("tglobal_r127_g16", "tglobal", rows=rows, q=q[0, hs, rows.to(dev)].float().cpu(),
                          o=f()[0, hs, rows.to(dev)].float().cpu(), block_len=128, gbs=16,
                          sk=sk[0, hs].float().cpu(), sv=sv[0, hs].float().cpu(), **host))
    del q, k, v, sk, sv

    # ---- split-K cross-attention of one decoder layer-step: reads K and V of the whole memory once (HBM-bound)
    qd, kc, vc = splitk_inputs(torch, dev)
    f = lambda: ops.flash_decoding_attention(qd, kc, vc, None, 1.0)  # noqa: E731
    _, ms = time_kernel(torch, f, 20, 5)
    nbytes = 2 * 64 * 8192 * 768 * 2
    out["splitk_cross_attention_layer_step"] = {
        "ms": round(ms, 4),
        "roofline": {"bound": "hbm", "achieved": round(nbytes / ms / 1e6, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4), "traffic": None,
                     "kernel": "t5a::splitk_partial_kernel<bf16, 64, 1> + splitk_merge_kernel",
                     "algorithmic_bytes_per_launch": nbytes}}
    o = f()
    samples.append(Sample("splitk_cross_attention", "dense", rows=torch.tensor([0]), q=qd[37, 5].float().cpu(),
                          k=kc[37, 5].float().cpu(), v=vc[37, 5].float().cpu(), t=None, o=o[37, 5].float().cpu(),
                          causal=False, offset=0))
    del qd, kc, vc
    return out


def model_workloads(torch, dev, steps):
    """T5-base (random init) legs: encoder tokens/s at 8k tokens, the 100k + 128 pass, greedy decoding."""
    from turbot5_amd import T5Config, T5EncoderModel, T5Model, ops
    out = {}
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
            # the attention kernel alone at this shape, times the 12 layers: its share of the pass
            q, k, v, table = make_inputs(torch, dev, bsz, 12, 8192, 64, seed=8)
            fa = lambda: ops.flash_attention_with_fusing_bias(q, k, v, table, causal=False, sm_scale=1.0)  # noqa: E731
            _, ms_a = time_kernel(torch, fa, 10, 3)
            out[f"t5_base_encoder_8k_B{bsz}_fp32_act_bf16_attn"] = {
                "ms": round(ms, 2), "tokens_per_s": round(bsz * 8192 / (ms * 1e-3), 1),
                "attention_kernel_ms_12_layers": round(12 * ms_a, 2), "attention_share": round(12 * ms_a / ms, 3),
                "note": "the rest is fp32 GEMMs (projections, feed-forward) through torch / hipBLASLt and RMS norms"}
            del q, k, v
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
        ids = torch.randint(0, 32128, (1, 100000), generator=ids_g).to(dev)
        f = lambda: enc16(ids)  # noqa: E731
        _, ms = time_kernel(torch, f, 2, 1, ramp_ms=0.0)
        attn_flops = 12 * 4.0 * 12 * 64 * 1e5 * 1e5
        out["t5_base_encoder_100k_B1_bf16"] = {"ms": round(ms, 1), "tokens_per_s": round(1e5 / (ms * 1e-3), 1),
                                               "attention_tflops_lower_bound": round(attn_flops / ms / 1e9, 1)}
    del enc, enc16
    # ---- the baseline's end-to-end case and greedy decoding, fp32 activations with bf16 attention
    torch.manual_seed(0)
    model = T5Model(T5Config(attention_dtype=torch.bfloat16, **base)).eval().to(dev)
    mem = torch.randn(64, 8192, 768, generator=torch.Generator().manual_seed(6)).to(dev)
    steps_dec = 32
    with torch.no_grad():
        ids = torch.randint(0, 32128, (1, 100000), generator=torch.Generator().manual_seed(8)).to(dev)
        dec_ids = torch.randint(0, 32128, (1, 128), generator=torch.Generator().manual_seed(9)).to(dev)
        f = lambda: model(ids, dec_ids)  # noqa: E731
        _, ms = time_kernel(torch, f, 2, 1, ramp_ms=0.0)
        logits = f()[0]
        out["t5_base_encdec_100k_enc_128_dec_fp32_act_bf16_attn"] = {
            "ms": round(ms, 1), "encoder_tokens_per_s": round(1e5 / (ms * 1e-3), 1),
            "logits_finite": bool(torch.isfinite(logits).all())}
        del ids, dec_ids, logits
        model.greedy_decode(encoder_outputs=mem, max_new_tokens=4)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        toks = model.greedy_decode(encoder_outputs=mem, max_new_tokens=steps_dec)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        out["greedy_decode_B64_mem8192"] = {"steps": steps_dec, "ms_per_step": round(dt / steps_dec * 1e3, 3),
                                            "tokens_per_s": round(64 * steps_dec / dt, 1)}
        model.greedy_decode_graphed(mem, steps_dec)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        toks_g = model.greedy_decode_graphed(mem, steps_dec)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        out["greedy_decode_B64_mem8192_graphed"] = {
            "steps": steps_dec, "ms_per_step": round(dt / steps_dec * 1e3, 3), "tokens_per_s": round(64 * steps_dec / dt, 1),
            "tokens_equal_to_eager_loop": round(float((toks == toks_g).float().mean()), 4),
            "note": "whole call: cross-attention K/V projection of the memory + the steps"}
    return out


# ---------------------------------------------------------------------------------------------------------------
# CPU leg: the oracle timed on the host, and the timed launches checked against it
# ---------------------------------------------------------------------------------------------------------------
def check_sample(torch, O, s):
    """max-abs difference between the rows a timed launch wrote and the 'basic' math on the same inputs."""
    kw = s.kw
    rows, q, k, v, t = kw["rows"], kw["q"], kw["k"], kw["v"], kw["t"]
    n = k.shape[0]
    j = torch.arange(n)[None, :]
    i = rows[:, None]

    def bias_of(rel, bidirectional=True):
        return t[O.relative_position_bucket(rel, bidirectional, 32, 128)] if t is not None else torch.zeros(rel.shape)

    if s.kind == "dense":
        i = i + kw["offset"]
        sc = q @ k.T + bias_of(j - i, not kw["causal"])
        if kw["causal"]:
            sc = sc.masked_fill(j > i, float("-inf"))
        want = torch.softmax(sc, -1) @ v
    elif s.kind in ("local", "tglobal"):
        sc = q @ k.T + bias_of(j - i)
        sc = sc.masked_fill((j - i).abs() >= kw["block_len"], float("-inf"))
        vv = v
        if s.kind == "tglobal":
            g = torch.arange(kw["sk"].shape[0])[None, :]
            side = q @ kw["sk"].T + bias_of(g - torch.clamp(i // kw["gbs"], max=kw["sk"].shape[0] - 1))
            sc, vv = torch.cat([sc, side], 1), torch.cat([v, kw["sv"]], 0)
        want = torch.softmax(sc, -1) @ vv
    else:   # block pattern, the reference's key list: [G global tokens | own block], rel = column - (G + row in block)
        Bl, G = kw["block_len"], kw["n_global"]
        want = torch.empty_like(kw["o"])
        for x, r in enumerate(rows.tolist()):
            if r < G:
                sc = q[x] @ k.T + bias_of(j[0] - r)
                want[x] = torch.softmax(sc, -1) @ v
                continue
            blk, rr = r // Bl, r % Bl
            c = torch.arange(G + Bl)
            ids = torch.where(c < G, c, blk * Bl + c - G)
            inside = (ids < n)[:, None]                      # keys of a ragged last block past the end count as zeros
            kk = torch.where(inside, k[ids.clamp(max=n - 1)], torch.zeros(()))
            vv = torch.where(inside, v[ids.clamp(max=n - 1)], torch.zeros(()))
            sc = kk @ q[x] + bias_of(c - (G + rr))
            if blk == 0:
                sc[Bl:] = float("-inf")                      # block 0 loses its last G list columns
            want[x] = torch.softmax(sc, -1) @ vv
    return float((kw["o"] - want).abs().max())


def cpu_baseline(torch, samples, seconds_budget=24.0):
    """The oracle's 'basic' path (materialised bias, einsum, fp32 softmax, einsum) on the host cores: bounded
    samples of the headline workload (C2), of the packed batch (C3), the T5-small encoder (C1), the sparse patterns
    at L = 16384 (C4, one head) and the decode shape (C5, 8 of 64 batch elements); and the checks of the timed GPU
    launches.  This function is the only place where bench.py uses the oracle."""
    from oracle import t5_basic as O
    from oracle import t5_model as OM
    torch.set_num_threads(os.cpu_count() or 1)
    threads = torch.get_num_threads()
    g = torch.Generator().manual_seed(0)
    q, k, v = (0.5 * torch.randn(1, H, L, D, generator=g) for _ in range(3))
    table = torch.randn(32, H, generator=g)
    O.dense_attention(q, k, v, table, False, 1.0)          # warm-up
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < seconds_budget / 2 and len(times) < 64):
        t0 = time.perf_counter()
        O.dense_attention(q, k, v, table, False, 1.0)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    flops = 4.0 * H * L * L * D
    res = {"value": round(flops / med / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
           "host_logical_cpus": os.cpu_count(), "torch_threads": threads,
           "sample": f"{len(times)} runs of 1 of the {B} batch elements (H{H} L{L} D{D}, fp32 'basic' with "
                     f"materialised bias), median {med * 1e3:.1f} ms"}
    other = {}
    # C3: one sequence of the packed batch (the median length), bidirectional, all 12 heads
    lens = sorted(c3_lengths())
    n = lens[len(lens) // 2]
    qs, ks, vs = (0.5 * torch.randn(1, H, n, D, generator=g) for _ in range(3))
    t0 = time.perf_counter()
    O.dense_attention(qs, ks, vs, table, False, 1.0)
    dt = time.perf_counter() - t0
    other["packed_batch_one_sequence"] = {"length": n, "ms": round(dt * 1e3, 1),
                                          "tflops": round(4.0 * H * n * n * D / dt / 1e12, 4)}
    # C1: T5-small encoder, 4 x 512 ids, fp32, through the oracle's layer stack
    from turbot5_amd import T5Config, T5EncoderModel
    torch.manual_seed(0)
    cfg = T5Config(vocab_size=32128, d_model=512, d_kv=64, d_ff=2048, num_layers=6, num_heads=8, dropout_rate=0.0)
    sd = {kk: vv.detach() for kk, vv in T5EncoderModel(cfg).state_dict().items()}
    ids = torch.randint(0, 32128, (4, 512), generator=torch.Generator().manual_seed(0))
    OM.encoder_forward(sd, cfg, ids[:1])
    t0 = time.perf_counter()
    OM.encoder_forward(sd, cfg, ids)
    dt = time.perf_counter() - t0
    other["t5_small_encoder_B4_L512_fp32"] = {"ms": round(dt * 1e3, 1), "tokens_per_s": round(2048 / dt, 1)}
    # C4: the three sparse patterns at the full L = 16384, one head each (the oracle's blocked evaluation
    # materialises the bias and mask per block, as the reference's modules do)
    Ls = SPARSE_L
    qs, ks, vs = (0.5 * torch.randn(1, 1, Ls, D, generator=g) for _ in range(3))
    t1 = table[:, :1]
    sk, sv = (0.5 * torch.randn(1, 1, Ls // 16, D, generator=g) for _ in range(2))
    for name, fn, pairs in (
            ("local_r127", lambda: O.local_attention_blocked(qs, ks, vs, t1, 128), Ls * 255 - 127 * 128),
            ("block_128_g64", lambda: O.block_attention_blocked(qs, ks, vs, t1, 128, 64), 64 * Ls + (Ls - 64) * 192 - 64 * 64),
            ("tglobal_r127_g16", lambda: O.tglobal_attention_blocked(qs, ks, vs, sk, sv, t1, 128, 16),
             Ls * 255 - 127 * 128 + Ls * (Ls // 16))):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        other[f"sparse_{name}_one_head_L{Ls}"] = {"ms": round(dt * 1e3, 1), "heads_timed": 1, "of_heads": H,
                                                 "tflops_live_pairs": round(4.0 * D * pairs / dt / 1e12, 4)}
    # C5 decode: one query row over an 8192-token memory, 8 of the 64 batch elements, 12 heads, no bias
    qd = 0.5 * torch.randn(8, H, 1, D, generator=g)
    kd, vd = (0.5 * torch.randn(8, H, 8192, D, generator=g) for _ in range(2))
    O.basic_attention(qd, kd, vd, None)
    t0 = time.perf_counter()
    O.basic_attention(qd, kd, vd, None)
    dt = time.perf_counter() - t0
    other["cross_attention_layer_step_B8_of_64_N8192"] = {
        "ms": round(dt * 1e3, 2), "gbytes_per_s_bf16_equivalent": round(2 * 8 * 8192 * 768 * 2 / dt / 1e9, 2),
        "note": "fp32 'basic' on the host; bytes counted as the bf16 cache the GPU kernel reads"}
    res["other_workloads"] = other
    res["checks"] = {s.name: round(check_sample(torch, O, s), 5) for s in samples}
    res["checks_note"] = ("max-abs of (what the timed launch wrote) - ('basic' math in fp32 on the same bf16 inputs) over "
                          "a subset of rows of one (batch, head); bar 2e-2")
    return res


# ---------------------------------------------------------------------------------------------------------------
def run_leg(torch, dev, name, steps, warmup, timeline=False):
    """One kernel, K launches, for profiling runs."""
    from turbot5_amd import ops
    if name == "copy":
        x = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev)
        y = torch.empty_like(x)
        for _ in range(5):
            y.copy_(x)
        torch.cuda.synchronize()
        return {"leg": "copy", "bytes_per_copy": x.numel()}
    peak = PEAK_BF16_TFLOPS
    if name.startswith("dense:"):
        parts = name.split(":")
        shape, mode = parts[1], (parts[2] if len(parts) > 2 else None)
        causal = shape.endswith("c")
        b, l = (int(x) for x in shape.rstrip("c").split("x"))
        q, k, v, table = make_inputs(torch, dev, b, H, l, D, seed=l if (b, l) != (B, L) else 0)
        exact = {None: None, "exact": True, "prescaled": "prescaled"}[mode]
        f = lambda: ops.flash_attention_with_fusing_bias(q, k, v, table, causal=causal, sm_scale=1.0, exact_scores=exact)  # noqa: E731
        fl = 4.0 * b * H * D * (l * (l + 1) // 2 if causal else l * l)
    elif name.startswith("bwd:"):
        # the backward kernels alone (dq pass, dk / dv pass, row statistics) on saved forward results: 2.5 x the
        # forward's FLOPs (five products instead of two); bwd:BxL[c]:fp32 runs them on the fp32 matrix cores
        # (bwd:BxL[c]:d128 is the T5-3B / 11B head shape: 6 heads of 128, the same FLOPs)
        fp32_math = name.endswith(":fp32")
        ops.BACKWARD_FP32_MATH = fp32_math
        hb, db = (H // 2, 2 * D) if name.endswith(":d128") else (H, D)
        shape = name.split(":")[1]
        causal = shape.endswith("c")
        b, l = (int(x) for x in shape.rstrip("c").split("x"))
        q, k, v, table = make_inputs(torch, dev, b, hb, l, db, seed=l if (b, l) != (B, L) else 0)
        o, lse = ops.flash_attention_with_fusing_bias(q, k, v, table, causal=causal, sm_scale=1.0, return_lse=True)
        g = torch.randn_like(o)
        f = lambda: ops._dense_backward(q, k, v, table, o, lse, g, causal, 1.0, 32, 128, None)  # noqa: E731
        fl = 10.0 * b * hb * db * (l * (l + 1) // 2 if causal else l * l)
        peak = PEAK_F32_TFLOPS if fp32_math else PEAK_BF16_TFLOPS
    elif name == "dense_f32_c1":
        # the attention of baseline configuration 1 (T5-small encoder): B4 H8 L512 D64 in fp32, on the fp32 matrix cores
        g = torch.Generator().manual_seed(3)
        q, k, v = ((0.5 * torch.randn(4, 8, 512, 64, generator=g)).to(dev) for _ in range(3))
        table = torch.randn(32, 8, generator=g).to(dev)
        f = lambda: ops.flash_attention_with_fusing_bias(q, k, v, table, causal=False, sm_scale=1.0)  # noqa: E731
        fl = 4.0 * 4 * 8 * 512 * 512 * 64
        peak = PEAK_F32_TFLOPS
    elif name in ("local", "block", "tglobal"):
        q, k, v, table, sk, sv = sparse_inputs(torch, dev)
        if name == "local":
            f = lambda: ops.local_attention_with_fusing_bias(q, k, v, table, 128)  # noqa: E731
            fl = 4.0 * H * D * (SPARSE_L * 255 - 127 * 128)
        elif name == "block":
            f = lambda: ops.block_attention_with_fusing_bias(q, k, v, table, 128, 64)  # noqa: E731
            fl = 4.0 * H * D * (64 * SPARSE_L + (SPARSE_L - 64) * 192 - 64 * 64)
        else:
            f = lambda: ops.transient_global_attention_with_fusing_bias(q, k, v, sk, sv, table, 128, 16)  # noqa: E731
            fl = 4.0 * H * D * (SPARSE_L * 255 - 127 * 128 + SPARSE_L * (SPARSE_L // 16))
    elif name == "splitk":
        qd, kc, vc = splitk_inputs(torch, dev)
        f = lambda: ops.flash_decoding_attention(qd, kc, vc, None, 1.0)  # noqa: E731
        fl = None      # HBM-bound: the K and V rows are read once (2 tensors x 64 x 12 x 8192 x 64 bf16)
        nbytes = 2.0 * 64 * 12 * 8192 * 64 * 2
    elif name in ("varlen", "varlen_causal"):
        lens, cu, q, k, v, table = varlen_inputs(torch, dev)
        causal = name.endswith("causal")
        f = lambda: ops.flash_attention_with_fusing_bias_varlen(q, k, v, table, cu, cu, max(lens), max(lens),  # noqa: E731
                                                                causal=causal, sm_scale=1.0)
        fl = 4.0 * H * D * (sum(n * (n + 1) // 2 for n in lens) if causal else sum(n * n for n in lens))
    else:
        raise SystemExit(f"unknown leg {name!r}")
    _, ms = time_kernel(torch, f, steps, warmup)
    if fl is None:
        out = {"leg": name, "kernel_ms": round(ms, 5), "gbytes_per_s": round(nbytes / ms / 1e6, 1),
               "frac_hbm_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
    else:
        out = {"leg": name, "kernel_ms": round(ms, 5), "tflops": round(fl / ms / 1e9, 1),
               "frac_mfma_peak": round(fl / ms / 1e9 / peak, 4), "mfma_peak_tflops": peak}
    if timeline:
        out["timeline"] = read_timeline(torch, f)
    return out


def read_timeline(torch, fn):
    """Cycle stamps of the work items of ONE launch from the measurement build (see T5A_STAMP in attn_fwd.hip)."""
    import ctypes as C
    import numpy as np
    from turbot5_amd import _lib
    lib = _lib.load()
    items, slots = 4096, 16
    buf = np.zeros(items * slots, dtype=np.uint64)
    torch.cuda.synchronize()
    lib.t5a_trace_read(buf.ctypes.data_as(C.c_void_p), 1)       # clear what earlier launches left
    fn()
    torch.cuda.synchronize()
    rc = lib.t5a_trace_read(buf.ctypes.data_as(C.c_void_p), 0)
    t = buf.reshape(items, slots).astype(np.int64)
    t = t[t[:, 0] != 0]
    if rc != 0 or len(t) == 0:
        return {"error": f"no stamps (rc {rc})"}
    names = ["entry -> first requests issued", "-> LUT barrier passed", "-> first score product (tile loop starts)"]
    res = {"workgroups_stamped": int(len(t)), "unit": "shader-clock cycles, median over workgroups", "phases": []}
    prev = t[:, 0]
    for i in range(1, 12):
        ok = t[:, i] != 0
        if not ok.any():
            break
        label = names[i - 1] if i <= 3 else ("-> end of a q tile's tile loop" if i % 2 == 0 else "-> next q tile of the run set up")
        res["phases"].append({"stamp": i, "what": label, "cycles": int(np.median((t[:, i] - prev)[ok])), "workgroups": int(ok.sum())})
        prev = np.where(ok, t[:, i], prev)
    fast = t[:, 14] > 0
    if fast.any():      # wavefront 0's fast steps, split at the step's barrier
        n = t[fast, 14].astype(float)
        res["fast_steps"] = {"per_work_item": float(np.median(n)),
                             "cycles_own_work_per_step": round(float(np.median(t[fast, 12] / n)), 1),
                             "cycles_waiting_at_the_barrier_per_step": round(float(np.median(t[fast, 13] / n)), 1)}
    total = t[:, :12].max(axis=1) - t[:, 0]
    res["work_item_total"] = {"median": int(np.median(total)), "min": int(total.min()), "max": int(total.max())}
    # the counters of different XCDs are not synchronised: only differences inside one workgroup mean anything
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--quick", "--no-extra", dest="quick", action="store_true",
                    help="only the headline workload (no sweep, no extra legs)")
    ap.add_argument("--no-models", action="store_true", help="skip the T5-base model legs (encoder, 100k pass, decoding)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg and its checks")
    ap.add_argument("--leg", default=None, metavar="NAME",
                    help="run only one kernel: dense:BxL[c][:exact|:prescaled], bwd:BxL[c][:fp32|:d128], dense_f32_c1, local, block, tglobal, splitk, varlen, varlen_causal, copy")
    ap.add_argument("--timeline", action="store_true",
                    help="with --leg: use the measurement build (libt5attn_trace.so) and print the work items' cycle stamps")
    ap.add_argument("--full", action="store_true", help="accepted for compatibility: the default run is the full one")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    if args.timeline:
        from turbot5_amd import _lib, build as t5a_build
        if not args.leg or not os.path.exists(t5a_build.TRACE_LIB):
            print("--timeline needs --leg and the measurement build: python -m turbot5_amd.build --trace", file=sys.stderr)
            sys.exit(2)
        _lib.LIB_PATH = t5a_build.TRACE_LIB
    from turbot5_amd.ops import flash_attention_with_fusing_bias
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    props = torch.cuda.get_device_properties(dev)
    if args.leg:
        print(json.dumps(run_leg(torch, dev, args.leg, args.steps, args.warmup, args.timeline)))
        return

    samples = []
    q, k, v, table = make_inputs(torch, dev, B, H, L, D)
    fn = lambda: flash_attention_with_fusing_bias(q, k, v, table, causal=False, sm_scale=1.0)  # noqa: E731
    wall_ms, dev_ms = time_kernel(torch, fn, args.steps, args.warmup)
    flops = 4.0 * B * H * L * L * D
    value = flops / (wall_ms * 1e-3) / 1e12
    achieved = flops / (dev_ms * 1e-3) / 1e12
    samples.append(dense_sample(torch, f"dense_B{B}_L{L}", q, k, v, table, fn(), False, 11, 4, 30))
    del q, k, v

    sweep, extra = {}, {}
    if not args.quick:
        for l in (2048, 4096, 8192, 16384):
            b = max(1, 16384 // l)
            qs, ks, vs, ts = make_inputs(torch, dev, b, H, l, D, seed=l)
            f = lambda: flash_attention_with_fusing_bias(qs, ks, vs, ts, causal=False, sm_scale=1.0)  # noqa: E731
            _, ms = time_kernel(torch, f, args.steps, args.warmup)
            tf = 4.0 * b * H * l * l * D / (ms * 1e-3) / 1e12
            sweep[f"B{b}_L{l}"] = {"ms": round(ms, 4), "tflops": round(tf, 1), "frac_mfma_peak": round(tf / PEAK_BF16_TFLOPS, 4)}
            samples.append(dense_sample(torch, f"dense_B{b}_L{l}", qs, ks, vs, ts, f(), False, b - 1, 6, l))
            del qs, ks, vs, ts
        extra = extra_workloads(torch, dev, args.steps, samples)
        if not args.no_models:
            extra.update(model_workloads(torch, dev, args.steps))

    # the peak the device itself implies: compute units x 4096 dense bf16 FLOP per clock x its maximum clock
    clock_ghz = props.clock_rate / 1e6 if getattr(props, "clock_rate", 0) else device_max_clock_ghz()
    device_peak = round(props.multi_processor_count * 4096 * clock_ghz / 1e3, 1) if clock_ghz else None
    line = {
        "metric": "fused-bias attn fwd TFLOP/s + % MFMA peak; T5-base encoder tokens/s @8k",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"dense bidirectional fused-bias attention forward, B{B} H{H} Lq=Lk={L} D{D} bf16, "
                               "32 buckets max_distance 128, sm_scale 1.0 (baseline configuration 2)",
                   "device": props.name, "compute_units": props.multi_processor_count,
                   "max_clock_ghz": clock_ghz, "bf16_peak_from_cus_and_clock_tflops": device_peak},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": measured_traffic_bytes(),
                     "traffic_source": os.path.relpath(TRAFFIC_PROFILE, ROOT),
                     "kernel": "t5a::fwd_kernel<bf16, 64, dense, non-causal>", "kernel_ms": round(dev_ms, 5),
                     "algorithmic_flops_per_launch": flops},
        "tokens_per_s": round(B * L / (wall_ms * 1e-3), 1),
        "sweep": sweep,
        "extra": extra,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(torch, samples)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
