"""The baseline's configurations at their exact sizes, each against the oracle:

  configuration 1   T5-small encoder, 4 x 512 ids, fp32: every attention op inside the model held to 1e-4
  configuration 3   packed batch of 32 sequences with lengths U[128, 4096] (seed 1, tests/golden/c3_lengths.json),
                    12 heads, head_dim 64, bf16, bidirectional and causal
  configuration 5   T5-base: 100k-token encoder + 128-token decoder forward (fp32 activations, bf16 attention),
                    split-K cross-attention at batch 64 over an 8192-token memory, greedy decoding at batch 64

(configuration 2 is in test_gpu_dense.py, configuration 4 in test_gpu_full_size.py.)"""
import json
import os

import pytest
import torch

from oracle import t5_basic as O
from oracle import t5_model as OM

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
T5_BASE = dict(vocab_size=32128, d_model=768, d_kv=64, d_ff=3072, num_layers=12, num_heads=12, dropout_rate=0.0,
               attention_type="flash")


def rnd(*shape, seed, scale=0.5, dtype=torch.bfloat16):
    return (scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed))).to(dtype)


# ------------------------------------------------------------------------------------------------ configuration 3
@pytest.mark.parametrize("causal", [False, True])
def test_config3_packed_batch(gpu_device, causal):
    from turbot5_amd.ops import flash_attention_with_fusing_bias_varlen
    with open(os.path.join(HERE, "golden", "c3_lengths.json")) as f:
        lens = json.load(f)["lengths"]
    assert len(lens) == 32 and min(lens) >= 128 and max(lens) <= 4096
    H, D = 12, 64
    total = sum(lens)
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    q, k, v = (rnd(total, H, D, seed=200 + i) for i in range(3))
    table = rnd(32, H, seed=203, scale=1.0, dtype=torch.float32)
    out, lse = flash_attention_with_fusing_bias_varlen(
        q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), table.to(gpu_device), cu.to(gpu_device),
        cu.to(gpu_device), max(lens), max(lens), causal=causal, sm_scale=1.0, return_lse=True)
    out, lse = out.float().cpu(), lse.cpu()
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    # whole sequences against the oracle: the shortest, the longest, the first and the last
    picks = sorted({lens.index(min(lens)), lens.index(max(lens)), 0, 31})
    assert len(picks) >= 3
    for b in picks:
        s, e = int(cu[b]), int(cu[b + 1])
        want = O.dense_attention(q[s:e].transpose(0, 1)[None], k[s:e].transpose(0, 1)[None],
                                 v[s:e].transpose(0, 1)[None], table, causal, 1.0)[0].transpose(0, 1)
        err = (out[s:e] - want).abs().max().item()
        assert err <= 2e-2, f"sequence {b} (length {e - s}): max-abs {err}"
        want_lse = O.dense_lse(q[s:e].transpose(0, 1)[None], k[s:e].transpose(0, 1)[None], table, causal, 1.0)[0]
        assert (lse[s:e] - want_lse.transpose(0, 1)).abs().max().item() <= 2e-2
    # every other sequence: random rows against the oracle's row formula
    g = torch.Generator().manual_seed(7)
    for b in range(32):
        if b in picks:
            continue
        s, n = int(cu[b]), lens[b]
        rows = torch.randint(0, n, (8,), generator=g)
        j = torch.arange(n)[None, :]
        i = rows[:, None]
        for h in (0, 5, 11):
            sc = q[s + rows, h].float() @ k[s:s + n, h].float().T + \
                table[O.relative_position_bucket(j - i, not causal, 32, 128), h]
            if causal:
                sc = sc.masked_fill(j > i, float("-inf"))
            want = torch.softmax(sc, -1) @ v[s:s + n, h].float()
            assert (out[s + rows, h] - want).abs().max().item() <= 2e-2, (b, h)


# ------------------------------------------------------------------------------------------------ configuration 5
def test_config5_splitk_cross_attention_batch64(gpu_device):
    """B64 H12 over an 8192-token memory in the decoder's cache layout (B, N, H, D): merged output of every
    batch element against the oracle on four of them, and against the dense kernel on all."""
    from turbot5_amd.ops import flash_attention_with_fusing_bias, flash_decoding_attention
    B, H, N, D = 64, 12, 8192, 64
    g = torch.Generator().manual_seed(300)
    kc = (0.5 * torch.randn(B, N, H, D, generator=g)).to(torch.bfloat16)
    vc = (0.5 * torch.randn(B, N, H, D, generator=g)).to(torch.bfloat16)
    q = (0.5 * torch.randn(B, H, 1, D, generator=g)).to(torch.bfloat16)
    dk, dv, dq = kc.to(gpu_device).transpose(1, 2), vc.to(gpu_device).transpose(1, 2), q.to(gpu_device)
    out = flash_decoding_attention(dq, dk, dv, None, 1.0)
    dense = flash_attention_with_fusing_bias(dq, dk, dv, None, causal=False, sm_scale=1.0)
    assert (out.float() - dense.float()).abs().max().item() <= 1e-2
    out = out.float().cpu()
    for b in (0, 17, 40, 63):
        want = O.dense_attention(q[b:b + 1], kc[b:b + 1].transpose(1, 2), vc[b:b + 1].transpose(1, 2), None, False, 1.0)
        assert (out[b:b + 1] - want).abs().max().item() <= 1e-2, b


@pytest.fixture(scope="module")
def t5_base(gpu_device):
    from turbot5_amd import T5Config, T5Model
    torch.manual_seed(0)
    cfg = T5Config(attention_dtype=torch.bfloat16, **T5_BASE)
    m = T5Model(cfg).eval()
    with torch.no_grad():
        for name, p in m.named_parameters():
            if "relative_attention_bias" in name:
                p.copy_(torch.randn_like(p))
    sd = {k: v.detach().clone() for k, v in m.state_dict().items()}
    return cfg, m.to(gpu_device), sd


def test_config5_t5_base_100k_encoder_128_decoder(gpu_device, t5_base):
    """One forward pass of the whole model at the baseline's size.  Checked: everything finite; the first
    encoder layer's attention (100k x 100k scores per head, bf16 kernel inside fp32 activations) on a random
    subset of rows against the oracle's row formula, from the very tensors the layer saw."""
    cfg, m, sd = t5_base
    L, Ld = 100000, 128
    ids = torch.randint(0, 32128, (1, L), generator=torch.Generator().manual_seed(8))
    dec = torch.randint(0, 32128, (1, Ld), generator=torch.Generator().manual_seed(9))
    attn0 = m.encoder.block[0].layer[0].SelfAttention
    seen = {}
    h1 = attn0.register_forward_pre_hook(lambda mod, args: seen.__setitem__("x", args[0].detach().float().cpu()))
    h2 = attn0.o.register_forward_pre_hook(lambda mod, args: seen.__setitem__("attn", args[0].detach().float().cpu()))
    try:
        with torch.no_grad():
            logits, enc, _ = m(ids.to(gpu_device), dec.to(gpu_device))
    finally:
        h1.remove()
        h2.remove()
    assert logits.shape == (1, Ld, 32128) and enc.shape == (1, L, 768)
    assert torch.isfinite(logits).all() and torch.isfinite(enc).all()
    x, attn = seen["x"][0], seen["attn"][0]                     # (L, 768) normed input, (L, 768) merged heads
    H, D = 12, 64
    p = "encoder.block.0.layer.0.SelfAttention."
    kk = (x @ sd[p + "k.weight"].T).to(torch.bfloat16).float().view(L, H, D)
    vv = (x @ sd[p + "v.weight"].T).to(torch.bfloat16).float().view(L, H, D)
    rows = torch.cat([torch.randperm(L, generator=torch.Generator().manual_seed(10))[:20],
                      torch.tensor([0, 1, 127, 128, L - 1])])
    qq = (x[rows] @ sd[p + "q.weight"].T).to(torch.bfloat16).float().view(-1, H, D)
    table = sd[p + "relative_attention_bias.weight"]
    j = torch.arange(L)[None, :]
    bucket = O.relative_position_bucket(j - rows[:, None], True, 32, 128)
    for h in range(H):
        s = qq[:, h] @ kk[:, h].T + table[bucket, h]
        want = torch.softmax(s, -1) @ vv[:, h]
        got = attn[rows].view(-1, H, D)[:, h]
        assert (got - want).abs().max().item() <= 2e-2, h


def test_config5_greedy_decode_batch64(gpu_device, t5_base):
    """Four greedy steps at batch 64 over an 8192-token memory (KV cache + split-K cross-attention), eager
    loop and graphed loop; logits of three batch elements against the oracle's full decoder pass fed with the
    tokens the device chose."""
    cfg, m, sd = t5_base
    B, N, steps = 64, 8192, 4
    mem = torch.randn(B, N, 768, generator=torch.Generator().manual_seed(6))
    dmem = mem.to(gpu_device)
    with torch.no_grad():
        toks = m.greedy_decode(encoder_outputs=dmem, max_new_tokens=steps)
        toks_g, logits_g = m.greedy_decode_graphed(dmem, steps, return_logits=True)
    assert toks.shape == (B, steps)
    toks, toks_g, logits_g = toks.cpu(), toks_g.cpu(), logits_g.cpu()
    start = torch.full((B, 1), cfg.decoder_start_token_id, dtype=torch.long)
    for b in (0, 31, 63):
        dec_in = torch.cat([start[b:b + 1], toks_g[b:b + 1, :-1]], dim=1)
        want = OM.lm_logits(sd, cfg, OM.decoder_forward(sd, cfg, dec_in, mem[b:b + 1]))[0]     # (steps, vocab)
        err = (logits_g[b] - want).abs().max().item()
        assert err <= 5e-2, f"batch element {b}: logits max-abs {err}"
        # the tokens are the argmax wherever the oracle's decision is not within the tolerance of a tie
        top2 = want.topk(2, dim=-1).values
        clear = (top2[:, 0] - top2[:, 1]) > 1e-1
        assert torch.equal(toks_g[b][clear], want.argmax(-1)[clear])
        assert torch.equal(toks[b][clear], want.argmax(-1)[clear])


# ------------------------------------------------------------------------------------------------ configuration 1
def test_config1_every_attention_op_within_1e4(gpu_device):
    """T5-small encoder (seed 0), 4 x 512 ids, all-ones mask, fp32: each of the six attention ops is compared
    with the oracle on the tensors that op saw inside the model (its own q, k, v), to the per-op fp32 bar."""
    from turbot5_amd import T5Config, T5EncoderModel
    torch.manual_seed(0)
    cfg = T5Config(vocab_size=32128, d_model=512, d_kv=64, d_ff=2048, num_layers=6, num_heads=8, dropout_rate=0.0,
                   attention_type="flash")
    m = T5EncoderModel(cfg).eval()
    with torch.no_grad():
        for name, p in m.named_parameters():
            if "relative_attention_bias" in name:
                p.copy_(torch.randn_like(p))
    sd = {k: v.detach().clone() for k, v in m.state_dict().items()}
    ids = torch.randint(0, 32128, (4, 512), generator=torch.Generator().manual_seed(0))
    seen = []
    hooks = []
    for i, blk in enumerate(m.encoder.block):
        att = blk.layer[0].SelfAttention
        rec = {}
        seen.append(rec)
        hooks.append(att.register_forward_pre_hook(lambda mod, args, rec=rec: rec.__setitem__("x", args[0].detach().cpu())))
        hooks.append(att.o.register_forward_pre_hook(lambda mod, args, rec=rec: rec.__setitem__("attn", args[0].detach().cpu())))
    m = m.to(gpu_device)
    with torch.no_grad():
        got = m(ids.to(gpu_device), torch.ones(4, 512, device=gpu_device)).cpu()
    for h in hooks:
        h.remove()
    table = sd["encoder.block.0.layer.0.SelfAttention.relative_attention_bias.weight"]
    B, L, H, D = 4, 512, 8, 64
    worst = 0.0
    for i, rec in enumerate(seen):
        p = f"encoder.block.{i}.layer.0.SelfAttention."
        q, k, v = ((rec["x"] @ sd[p + n + ".weight"].T).view(B, L, H, D).transpose(1, 2) for n in ("q", "k", "v"))
        want = O.dense_attention(q, k, v, table, False, 1.0).transpose(1, 2).reshape(B, L, H * D)
        err = (rec["attn"] - want).abs().max().item()
        worst = max(worst, err)
        assert err <= 1e-4, f"layer {i}: attention op max-abs {err}"
    want = OM.encoder_forward(sd, cfg, ids)
    assert (got - want).abs().max().item() <= 2e-3     # six layers end to end (GEMM rounding on both sides)
