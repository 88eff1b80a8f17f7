"""Pins the sparse-pattern parts of the oracle (reference att.py:523-1065, utils.py:84-258).

* blocking helpers and the local / transient-global ops: HuggingFace LongT5
  (third-party library with the same lineage) and brute-force closed forms;
* block attention: brute-force closed form only (no third-party counterpart).
"""
import numpy as np
import pytest
import torch

from oracle import t5_basic as O
from tests import closed_forms as CF


def rnd(*shape, seed=0, scale=0.5):
    g = torch.Generator().manual_seed(seed)
    return scale * torch.randn(*shape, generator=g)


@pytest.fixture(scope="module")
def hf():
    from transformers.models.longt5 import modeling_longt5 as L
    return L


# ---------------------------------------------------------------- helpers vs HF
def test_helpers_against_huggingface(hf):
    x = rnd(2, 50, 3, 4, seed=1)                      # HF layout (B,L,H,D): blocks at dim 1, no swap
    for bl in (8, 10, 64):
        a = O.split_into_blocks(x, bl, 1, swap12=False)
        if 50 // bl >= 1:
            assert torch.equal(a, hf._split_into_blocks(x, bl, 1))
            assert torch.equal(O.concatenate_3_blocks(a, 1, 2), hf._concatenate_3_blocks(a, 1, 2))
    mask = torch.ones(2, 48)
    mask[1, 37:] = 0
    for bl in (8, 16):
        want = hf._get_local_attention_mask(mask, bl, torch.device("cpu"))   # (B,1,nb,Bl,3Bl)
        got = O.local_attention_mask(mask, bl)                               # (B,nb,1,Bl,3Bl)
        assert torch.equal(got, want.transpose(1, 2))
    for gbs in (4, 8, 16):
        ids, seg = O.make_global_fixed_block_ids(mask, gbs)
        ids2, seg2 = hf._make_global_fixed_block_ids(mask, gbs)
        assert torch.equal(ids, ids2) and torch.equal(seg, seg2)
        h = rnd(2, 48, 6, seed=2)
        assert torch.allclose(O.create_global_aggregates(h, ids, seg.shape[-1]),
                              hf._create_global_aggregates(h, ids2, seg2.shape[-1]))


def test_data_split_swaps_blocks_before_heads():
    x = rnd(2, 3, 32, 4, seed=3)                      # reference layout (B,H,L,D), dim=2, then transpose(1,2)
    y = O.split_into_blocks(x, 8, 2)
    assert y.shape == (2, 4, 3, 8, 4)
    assert torch.equal(y[1, 2, 0], x[1, 0, 16:24])
    short = O.split_into_blocks(x[:, :, :5], 8, 2)    # shorter than one block: one block of the whole length
    assert short.shape == (2, 1, 3, 5, 4)


# ---------------------------------------------------------------- local
def _hf_cfg(hf, H, D, Bl, gbs=None):
    from transformers import LongT5Config
    return LongT5Config(d_model=H * D, d_kv=D, num_heads=H, local_radius=Bl - 1, global_block_size=gbs or 16,
                        relative_attention_num_buckets=32, relative_attention_max_distance=128, dropout_rate=0.0,
                        is_decoder=False)


@pytest.mark.parametrize("L,Bl", [(64, 16), (96, 32), (16, 16)])
def test_local_against_huggingface(hf, L, Bl):
    B, H, D = 2, 3, 8
    mod = hf.LongT5LocalAttention(_hf_cfg(hf, H, D, Bl), has_relative_attention_bias=True).eval()
    table = rnd(32, H, seed=4, scale=1.0)
    with torch.no_grad():
        mod.relative_attention_bias.weight.copy_(table)
        mod.o.weight.copy_(torch.eye(H * D))
        x = rnd(B, L, H * D, seed=5, scale=1.0)
        am = torch.ones(B, L)
        want = mod(x, mask=hf._get_local_attention_mask(am, Bl, x.device))[0]        # (B,L,H*D)
        q = mod.q(x).view(B, L, H, D).transpose(1, 2)
        k = mod.k(x).view(B, L, H, D).transpose(1, 2)
        v = mod.v(x).view(B, L, H, D).transpose(1, 2)
    got = O.local_attention_blocked(q, k, v, table, Bl).transpose(1, 2).reshape(B, L, H * D)
    assert torch.allclose(got, want, atol=2e-5)


@pytest.mark.parametrize("L,Bl", [(64, 16), (96, 32)])
def test_local_with_padding_against_huggingface(hf, L, Bl):
    """Right-padded batch: the oracle's mask path against LongT5LocalAttention with the same mask,
    compared on the valid query rows (padded rows attend a uniformly masked window in both)."""
    B, H, D = 3, 2, 8
    mod = hf.LongT5LocalAttention(_hf_cfg(hf, H, D, Bl), has_relative_attention_bias=True).eval()
    table = rnd(32, H, seed=24, scale=1.0)
    am = torch.ones(B, L)
    am[0, L - 5:] = 0
    am[1, Bl + 3:] = 0
    with torch.no_grad():
        mod.relative_attention_bias.weight.copy_(table)
        mod.o.weight.copy_(torch.eye(H * D))
        x = rnd(B, L, H * D, seed=25, scale=1.0)
        want = mod(x, mask=hf._get_local_attention_mask(am, Bl, x.device))[0]
        q = mod.q(x).view(B, L, H, D).transpose(1, 2)
        k = mod.k(x).view(B, L, H, D).transpose(1, 2)
        v = mod.v(x).view(B, L, H, D).transpose(1, 2)
    got = O.local_attention_blocked(q, k, v, table, Bl, am).transpose(1, 2).reshape(B, L, H * D)
    valid = am.bool()
    assert torch.allclose(got[valid], want[valid], atol=2e-5)


def test_local_with_padding_against_brute_force():
    """Valid rows of a right-padded batch equal plain attention over the valid keys inside the window."""
    B, H, L, D, Bl = 2, 2, 48, 4, 16
    q, k, v = (rnd(B, H, L, D, seed=26 + i) for i in range(3))
    table = rnd(32, H, seed=29, scale=1.0)
    lens = [37, 9]
    am = (torch.arange(L)[None, :] < torch.tensor(lens)[:, None]).float()
    got = O.local_attention_blocked(q, k, v, table, Bl, am)
    i = torch.arange(L)[:, None]
    j = torch.arange(L)[None, :]
    bias = table[O.relative_position_bucket(j - i, True, 32, 128)].permute(2, 0, 1).unsqueeze(0)
    for b, n in enumerate(lens):
        keep = ((j - i).abs() < Bl) & (j < n)
        want = O.basic_attention(q[b:b + 1], k[b:b + 1], v[b:b + 1], bias.masked_fill(~keep, float("-inf")))
        assert (got[b, :, :n] - want[0, :, :n]).abs().max().item() < 2e-6


@pytest.mark.parametrize("L,Bl", [(40, 8), (48, 16), (8, 8), (5, 8)])
def test_local_against_closed_form(L, Bl):
    H, D = 2, 4
    q, k, v = rnd(1, H, L, D, seed=6), rnd(1, H, L, D, seed=7), rnd(1, H, L, D, seed=8)
    table = rnd(32, H, seed=9, scale=1.0)
    got = O.local_attention_blocked(q, k, v, table, Bl)[0].numpy()
    want = CF.local(q[0].numpy(), k[0].numpy(), v[0].numpy(), table.numpy(), min(Bl, L))
    assert np.abs(got - want).max() < 2e-6


def test_local_long_distance_saturation():
    """block_len above the saturation distance exercises the far buckets."""
    H, D, L, Bl = 1, 4, 300, 150
    q, k, v = rnd(1, H, L, D, seed=10), rnd(1, H, L, D, seed=11), rnd(1, H, L, D, seed=12)
    table = rnd(32, H, seed=13, scale=1.0)
    got = O.local_attention_blocked(q, k, v, table, Bl)[0].numpy()
    want = CF.local(q[0].numpy(), k[0].numpy(), v[0].numpy(), table.numpy(), Bl)
    assert np.abs(got - want).max() < 2e-6


# ---------------------------------------------------------------- transient-global
@pytest.mark.parametrize("L,Bl,gbs", [(64, 16, 4), (96, 32, 8)])
def test_tglobal_against_huggingface(hf, L, Bl, gbs):
    B, H, D = 2, 3, 8
    mod = hf.LongT5TransientGlobalAttention(_hf_cfg(hf, H, D, Bl, gbs), has_relative_attention_bias=True).eval()
    table = rnd(32, H, seed=14, scale=1.0)
    with torch.no_grad():
        mod.relative_attention_bias.weight.copy_(table)
        mod.global_relative_attention_bias.weight.copy_(table)   # the reference reads the local table (att.py:918-919)
        mod.global_input_layer_norm.weight.copy_(1.0 + rnd(H * D, seed=15, scale=0.1))
        mod.o.weight.copy_(torch.eye(H * D))
        x = rnd(B, L, H * D, seed=16, scale=1.0)
        am = torch.ones(B, L)
        want = mod(x, mask=am)[0]
        q = mod.q(x).view(B, L, H, D).transpose(1, 2)
        k = mod.k(x).view(B, L, H, D).transpose(1, 2)
        v = mod.v(x).view(B, L, H, D).transpose(1, 2)
        side = O.tglobal_side_inputs(x, am, gbs, mod.global_input_layer_norm.weight, 1e-6)
        sk = mod.k(side).view(B, -1, H, D).transpose(1, 2)
        sv = mod.v(side).view(B, -1, H, D).transpose(1, 2)
    got = O.tglobal_attention_blocked(q, k, v, sk, sv, table, Bl, gbs).transpose(1, 2).reshape(B, L, H * D)
    assert torch.allclose(got, want, atol=3e-5)


@pytest.mark.parametrize("L,Bl,gbs", [(64, 16, 4), (96, 32, 8)])
def test_tglobal_with_padding_against_huggingface(hf, L, Bl, gbs):
    """Right-padded batch: the oracle's mask path (block ids, side-token validity, orphan tokens) against
    LongT5TransientGlobalAttention with the same mask, on the valid query rows."""
    B, H, D = 3, 2, 8
    mod = hf.LongT5TransientGlobalAttention(_hf_cfg(hf, H, D, Bl, gbs), has_relative_attention_bias=True).eval()
    table = rnd(32, H, seed=34, scale=1.0)
    am = torch.ones(B, L)
    am[0, L - gbs - 3:] = 0          # orphan tokens after the last full block
    am[1, Bl + 1:] = 0
    with torch.no_grad():
        mod.relative_attention_bias.weight.copy_(table)
        mod.global_relative_attention_bias.weight.copy_(table)
        mod.global_input_layer_norm.weight.copy_(1.0 + rnd(H * D, seed=35, scale=0.1))
        mod.o.weight.copy_(torch.eye(H * D))
        x = rnd(B, L, H * D, seed=36, scale=1.0)
        want = mod(x, mask=am)[0]
        q = mod.q(x).view(B, L, H, D).transpose(1, 2)
        k = mod.k(x).view(B, L, H, D).transpose(1, 2)
        v = mod.v(x).view(B, L, H, D).transpose(1, 2)
        side = O.tglobal_side_inputs(x, am, gbs, mod.global_input_layer_norm.weight, 1e-6)
        sk = mod.k(side).view(B, -1, H, D).transpose(1, 2)
        sv = mod.v(side).view(B, -1, H, D).transpose(1, 2)
    got = O.tglobal_attention_blocked(q, k, v, sk, sv, table, Bl, gbs, am).transpose(1, 2).reshape(B, L, H * D)
    valid = am.bool()
    assert torch.allclose(got[valid], want[valid], atol=3e-5)


def test_tglobal_with_padding_equals_the_sequence_alone():
    """A right-padded sequence of n valid tokens (n a multiple of the block length) gives, on its valid rows,
    what the same n tokens give as an unpadded batch: side tokens n // gbs, keys up to n."""
    H, D, L, Bl, gbs, n = 2, 4, 64, 16, 4, 32
    q, k, v = (rnd(1, H, L, D, seed=37 + i) for i in range(3))
    hidden = rnd(1, L, 6, seed=40, scale=1.0)
    w = 1.0 + rnd(6, seed=41, scale=0.1)
    proj = rnd(6, H * D, seed=42)
    table = rnd(32, H, seed=43, scale=1.0)
    am = (torch.arange(L)[None, :] < n).float()
    def side(h, m):
        s_ = O.tglobal_side_inputs(h, m, gbs, w) @ proj
        return s_.view(1, -1, H, D).transpose(1, 2)
    got = O.tglobal_attention_blocked(q, k, v, side(hidden, am), side(hidden, am), table, Bl, gbs, am)
    want = O.tglobal_attention_blocked(q[:, :, :n], k[:, :, :n], v[:, :, :n], side(hidden[:, :n], None),
                                       side(hidden[:, :n], None), table, Bl, gbs)
    assert (got[:, :, :n] - want).abs().max().item() < 2e-6


@pytest.mark.parametrize("L,Bl,gbs", [(48, 16, 4), (64, 8, 16), (256, 32, 1)])
def test_tglobal_against_closed_form(L, Bl, gbs):
    H, D = 2, 4
    q, k, v = rnd(1, H, L, D, seed=17), rnd(1, H, L, D, seed=18), rnd(1, H, L, D, seed=19)
    sk, sv = rnd(1, H, L // gbs, D, seed=20), rnd(1, H, L // gbs, D, seed=21)
    table = rnd(32, H, seed=22, scale=1.0)
    got = O.tglobal_attention_blocked(q, k, v, sk, sv, table, Bl, gbs)[0].numpy()
    want = CF.tglobal(q[0].numpy(), k[0].numpy(), v[0].numpy(), sk[0].numpy(), sv[0].numpy(), table.numpy(), Bl, gbs)
    assert np.abs(got - want).max() < 2e-6


def test_tglobal_side_inputs_are_normalised_block_sums():
    x = rnd(1, 32, 6, seed=23, scale=1.0)
    w = 1.0 + rnd(6, seed=24, scale=0.1)
    got = O.tglobal_side_inputs(x, None, 8, w)
    sums = x.view(1, 4, 8, 6).sum(2)
    want = w * sums / torch.sqrt(sums.pow(2).mean(-1, keepdim=True) + 1e-6)
    assert torch.allclose(got, want, atol=1e-6)


# ---------------------------------------------------------------- block + global tokens
@pytest.mark.parametrize("L,Bl,G", [(64, 16, 4), (48, 16, 16), (40, 16, 8), (10, 16, 4), (160, 32, 8)])
def test_block_against_closed_form(L, Bl, G):
    H, D = 2, 4
    q, k, v = rnd(1, H, L, D, seed=25), rnd(1, H, L, D, seed=26), rnd(1, H, L, D, seed=27)
    table = rnd(32, H, seed=28, scale=1.0)
    got = O.block_attention_blocked(q, k, v, table, Bl, G)[0].numpy()
    want = CF.block(q[0].numpy(), k[0].numpy(), v[0].numpy(), table.numpy(), Bl, G)
    assert np.abs(got - want).max() < 2e-6


def test_block_zero_quirk_is_visible():
    """In block 0 the rows past the global tokens never see tokens [Bl-G, Bl): changing them changes nothing."""
    H, D, L, Bl, G = 1, 4, 32, 16, 4
    q, k, v = rnd(1, H, L, D, seed=29), rnd(1, H, L, D, seed=30), rnd(1, H, L, D, seed=31)
    table = rnd(32, H, seed=32, scale=1.0)
    a = O.block_attention_blocked(q, k, v, table, Bl, G)
    k2, v2 = k.clone(), v.clone()
    k2[:, :, Bl - G:Bl] += 1.0
    v2[:, :, Bl - G:Bl] -= 2.0
    b = O.block_attention_blocked(q, k2, v2, table, Bl, G)
    assert torch.allclose(a[:, :, G:Bl], b[:, :, G:Bl], atol=1e-6)
    assert not torch.allclose(a[:, :, :G], b[:, :, :G], atol=1e-3)     # the global queries do see them
