"""Size-independent checks at the full sizes of the baseline configurations: 100k tokens dense
(bidirectional and causal), the three sparse patterns at L = 16384 with 12 heads (baseline configuration 4).  The oracle is applied to a random
subset of query rows (every key of those rows), which it finishes in seconds."""
import pytest
import torch

from oracle import t5_basic as O

pytestmark = pytest.mark.gpu


def rnd(*shape, seed, scale=0.5, dtype=torch.bfloat16):
    return (scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed))).to(dtype)


def rows_oracle(q, k, v, table, rows, h, key_ids, rel, live):
    """softmax(q.k + T[bucket(rel)]) v for the given rows of head h.  key_ids (R,K) indexes k/v (−1: zero
    vector), rel (R,K) relative positions, live (R,K) bool."""
    qh = q[0, h, rows].float()
    kk = torch.where(key_ids[..., None] >= 0, k[0, h].float()[key_ids.clamp(min=0)], torch.zeros(()))
    vv = torch.where(key_ids[..., None] >= 0, v[0, h].float()[key_ids.clamp(min=0)], torch.zeros(()))
    s = torch.einsum("rd,rkd->rk", qh, kk) + table[O.relative_position_bucket(rel, True, 32, 128), h]
    s = s.masked_fill(~live, float("-inf"))
    return torch.einsum("rk,rkd->rd", torch.softmax(s, -1), vv)


def pick(L, n, seed, extra=()):
    r = torch.randperm(L, generator=torch.Generator().manual_seed(seed))[:n]
    return torch.cat([r, torch.tensor(list(extra), dtype=torch.long)]).unique()


@pytest.mark.parametrize("causal", [False, True])
def test_dense_100k_tokens(gpu_device, causal):
    from turbot5_amd.ops import flash_attention_with_fusing_bias
    L, H, D = 100000, 2, 64
    q, k, v = (rnd(1, H, L, D, seed=70 + i) for i in range(3))
    table = rnd(32, H, seed=73, scale=1.0, dtype=torch.float32)
    dev = [t.to(gpu_device) for t in (q, k, v, table)]
    out = flash_attention_with_fusing_bias(*dev, causal=causal, sm_scale=1.0).cpu()
    ones = flash_attention_with_fusing_bias(dev[0], dev[1], torch.ones_like(dev[2]), dev[3], causal=causal, sm_scale=1.0)
    assert (ones.float() - 1.0).abs().max().item() <= 1e-2                    # weights sum to one in every row
    if causal:
        assert torch.equal(out[0, :, 0], v[0, :, 0])                          # the first row sees only itself
    rows = pick(L, 40, 74, extra=(0, 1, 127, 128, L - 1))
    j = torch.arange(L)[None, :]
    i = rows[:, None]
    for h in range(H):
        qh = q[0, h, rows].float()
        s = qh @ k[0, h].float().T + table[O.relative_position_bucket(j - i, not causal, 32, 128), h]
        if causal:
            s = s.masked_fill(j > i, float("-inf"))
        want = torch.softmax(s, -1) @ v[0, h].float()
        assert (out[0, h, rows].float() - want).abs().max().item() <= 2e-2


def test_local_16k(gpu_device):
    from turbot5_amd.ops import local_attention_with_fusing_bias
    L, H, D, Bl = 16384, 12, 64, 128
    q, k, v = (rnd(1, H, L, D, seed=80 + i) for i in range(3))
    table = rnd(32, H, seed=83, scale=1.0, dtype=torch.float32)
    out = local_attention_with_fusing_bias(*(t.to(gpu_device) for t in (q, k, v, table)), Bl).cpu()
    rows = pick(L, 64, 84, extra=(0, 1, Bl - 1, Bl, L - Bl, L - 1))
    key_ids = rows[:, None] + torch.arange(-Bl + 1, Bl)[None, :]
    live = (key_ids >= 0) & (key_ids < L)
    rel = key_ids - rows[:, None]
    for h in range(H):
        want = rows_oracle(q, k, v, table, rows, h, torch.where(live, key_ids, -1), rel, live)
        assert (out[0, h, rows].float() - want).abs().max().item() <= 2e-2


def test_block_16k(gpu_device):
    """[G global tokens | own block] with rel = c - (G + r) over the list column c; block 0 loses its last
    G columns; the first G rows see every key (reference layout, attentions.py:685-691, :722-732, :788-814)."""
    from turbot5_amd.ops import block_attention_with_fusing_bias
    L, H, D, Bl, G = 16384, 12, 64, 128, 64
    q, k, v = (rnd(1, H, L, D, seed=90 + i) for i in range(3))
    table = rnd(32, H, seed=93, scale=1.0, dtype=torch.float32)
    out = block_attention_with_fusing_bias(*(t.to(gpu_device) for t in (q, k, v, table)), Bl, G).cpu()
    # global rows: dense
    rows = torch.tensor([0, 1, G - 1])
    j = torch.arange(L)[None, :]
    for h in range(H):
        s = q[0, h, rows].float() @ k[0, h].float().T + table[O.relative_position_bucket(j - rows[:, None], True, 32, 128), h]
        want = torch.softmax(s, -1) @ v[0, h].float()
        assert (out[0, h, rows].float() - want).abs().max().item() <= 2e-2
    # other rows: the list
    rows = pick(L - G, 64, 94, extra=(0, Bl - G - 1, Bl - G, L - G - 1)) + G
    blk, r = rows // Bl, rows % Bl
    c = torch.arange(G + Bl)[None, :]
    key_ids = torch.where(c < G, c, blk[:, None] * Bl + (c - G))
    live = ~((blk[:, None] == 0) & (c >= Bl))
    rel = c - (G + r[:, None])
    for h in range(H):
        want = rows_oracle(q, k, v, table, rows, h, key_ids, rel, live)
        assert (out[0, h, rows].float() - want).abs().max().item() <= 2e-2


def test_tglobal_16k(gpu_device):
    from turbot5_amd.ops import transient_global_attention_with_fusing_bias
    L, H, D, Bl, gbs = 16384, 12, 64, 128, 16
    Gn = L // gbs
    q, k, v = (rnd(1, H, L, D, seed=100 + i) for i in range(3))
    sk, sv = (rnd(1, H, Gn, D, seed=103 + i) for i in range(2))
    table = rnd(32, H, seed=105, scale=1.0, dtype=torch.float32)
    out = transient_global_attention_with_fusing_bias(*(t.to(gpu_device) for t in (q, k, v, sk, sv, table)), Bl, gbs).cpu()
    rows = pick(L, 48, 106, extra=(0, gbs - 1, gbs, L - 1))
    loc = rows[:, None] + torch.arange(-Bl + 1, Bl)[None, :]
    live_loc = (loc >= 0) & (loc < L)
    g = torch.arange(Gn)[None, :].expand(len(rows), Gn)
    kcat = torch.cat([k, sk], 2)
    vcat = torch.cat([v, sv], 2)
    key_ids = torch.cat([torch.where(live_loc, loc, -1), L + g], 1)
    rel = torch.cat([loc - rows[:, None], g - (rows // gbs)[:, None]], 1)
    live = torch.cat([live_loc, torch.ones_like(g, dtype=torch.bool)], 1)
    for h in range(H):
        want = rows_oracle(q, kcat, vcat, table, rows, h, key_ids, rel, live)
        assert (out[0, h, rows].float() - want).abs().max().item() <= 2e-2


def test_padded_sequences_equal_the_sequences_alone_16k(gpu_device):
    """Size-independent property of the per-sequence lengths at L = 16384: a right-padded sequence of n
    tokens gives, on its n rows, what the n tokens give as a batch of their own (local and transient-global
    patterns; n a multiple of the side block so that both runs build the same side tokens)."""
    from turbot5_amd.ops import local_attention_with_fusing_bias, transient_global_attention_with_fusing_bias
    H, L, D, Bl, gbs = 12, 16384, 64, 128, 16
    lens = [16384, 9600, 4112]
    B = len(lens)
    q, k, v = (rnd(B, H, L, D, seed=120 + i).to(gpu_device) for i in range(3))
    sk, sv = (rnd(B, H, L // gbs, D, seed=123 + i).to(gpu_device) for i in range(2))
    table = rnd(32, H, seed=125, scale=1.0, dtype=torch.float32).to(gpu_device)
    tl = torch.tensor(lens, dtype=torch.int32, device=gpu_device)
    loc = local_attention_with_fusing_bias(q, k, v, table, Bl, seq_lens=tl)
    tg = transient_global_attention_with_fusing_bias(q, k, v, sk, sv, table, Bl, gbs, seq_lens=tl)
    assert torch.isfinite(loc).all() and torch.isfinite(tg).all()
    for b, n in enumerate(lens):
        qa, ka, va = (t[b:b + 1, :, :n].contiguous() for t in (q, k, v))
        alone = local_attention_with_fusing_bias(qa, ka, va, table, Bl)
        assert (loc[b, :, :n].float() - alone[0].float()).abs().max().item() <= 2e-2, ("local", b)
        ska, sva = (t[b:b + 1, :, :n // gbs].contiguous() for t in (sk, sv))
        alone = transient_global_attention_with_fusing_bias(qa, ka, va, ska, sva, table, Bl, gbs)
        assert (tg[b, :, :n].float() - alone[0].float()).abs().max().item() <= 2e-2, ("tglobal", b)
