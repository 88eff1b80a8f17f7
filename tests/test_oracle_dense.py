"""Pins the dense / varlen / split-K parts of the oracle (reference naive.py:4-23,
att.py:126-141, :229-236, decoding.py:47-55) against library routines, invariants
and a brute-force closed form."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import t5_basic as O
from tests import closed_forms as CF


def rnd(*shape, seed=0, scale=0.5):
    g = torch.Generator().manual_seed(seed)
    return scale * torch.randn(*shape, generator=g)


def test_basic_equals_sdpa_fp64():
    q, k, v = rnd(2, 3, 17, 8, seed=1), rnd(2, 3, 23, 8, seed=2), rnd(2, 3, 23, 8, seed=3)
    bias = rnd(1, 3, 17, 23, seed=4, scale=1.0)
    got = O.basic_attention(q, k, v, bias)
    want = F.scaled_dot_product_attention(q.double(), k.double(), v.double(), attn_mask=bias.double(), scale=1.0)
    assert torch.allclose(got.double(), want, atol=2e-6)


def test_zero_table_is_plain_unscaled_sdpa():
    q, k, v = rnd(1, 2, 9, 16, seed=5), rnd(1, 2, 9, 16, seed=6), rnd(1, 2, 9, 16, seed=7)
    got = O.dense_attention(q, k, v, torch.zeros(32, 2), sm_scale=1.0)
    want = F.scaled_dot_product_attention(q, k, v, scale=1.0)
    assert torch.allclose(got, want, atol=1e-6)
    got2 = O.dense_attention(q, k, v, None)           # default scale 1/sqrt(D)
    assert torch.allclose(got2, F.scaled_dot_product_attention(q, k, v), atol=1e-6)


def test_invariants():
    q, k = rnd(1, 2, 12, 8, seed=8), rnd(1, 2, 20, 8, seed=9)
    table = rnd(32, 2, seed=10, scale=1.0)
    ones = torch.ones(1, 2, 20, 8)
    assert torch.allclose(O.dense_attention(q, k, ones, table, sm_scale=1.0), torch.ones(1, 2, 12, 8), atol=1e-6)
    v = rnd(1, 2, 20, 8, seed=11)
    a = O.dense_attention(q, k, v, table, sm_scale=1.0)
    b = O.dense_attention(q, k, v, table + 3.25, sm_scale=1.0)      # uniform table shift is softmax-invariant
    assert torch.allclose(a, b, atol=1e-5)
    # causal, M == N: row 0 sees only key 0
    c = O.dense_attention(q, k[:, :, :12], v[:, :, :12], table, causal=True, sm_scale=1.0)
    assert torch.allclose(c[:, :, 0], v[:, :, 0], atol=1e-6)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("M,N", [(9, 9), (5, 150), (1, 40), (140, 140)])
def test_dense_against_closed_form(causal, M, N):
    H, D = 2, 4
    q, k, v = rnd(1, H, M, D, seed=12), rnd(1, H, N, D, seed=13), rnd(1, H, N, D, seed=14)
    table = rnd(32, H, seed=15, scale=1.0)
    got = O.dense_attention(q, k, v, table, causal=causal, sm_scale=0.7)
    want = CF.dense(q[0].numpy(), k[0].numpy(), v[0].numpy(), table.numpy(), causal, 0.7)
    assert np.abs(got[0].numpy() - want).max() < 2e-6


def test_dense_bias_matches_basic_cache_alignment():
    """rel = j - (i + N - M): the last M rows of the N x N bias (att.py:229-234)."""
    table = rnd(32, 3, seed=16, scale=1.0)
    full = O.compute_bias(table, 50, 50, True)
    assert torch.equal(O.dense_bias(table, 7, 50, False), full[:, :, -7:, :])
    uni = O.compute_bias(table, 50, 50, False)
    cb = O.dense_bias(table, 1, 50, True)
    assert torch.equal(cb, uni[:, :, -1:, :])             # last row: nothing is masked


def test_m_greater_than_n_causal_rows_are_zero():
    q, k, v = rnd(1, 1, 6, 4, seed=17), rnd(1, 1, 3, 4, seed=18), rnd(1, 1, 3, 4, seed=19)
    out = O.dense_attention(q, k, v, None, causal=True, sm_scale=1.0)
    assert torch.equal(out[0, 0, :3], torch.zeros(3, 4))  # rows with i + N - M < 0 see no key
    assert torch.allclose(out[0, 0, 3], v[0, 0, 0])


def test_row_chunking_changes_nothing():
    q, k, v = rnd(1, 2, 70, 8, seed=20), rnd(1, 2, 70, 8, seed=21), rnd(1, 2, 70, 8, seed=22)
    table = rnd(32, 2, seed=23, scale=1.0)
    a = O.dense_attention(q, k, v, table, sm_scale=1.0, row_chunk=1024)
    b = O.dense_attention(q, k, v, table, sm_scale=1.0, row_chunk=13)
    assert torch.allclose(a, b, atol=1e-6)


def test_lse():
    q, k = rnd(1, 2, 5, 8, seed=24), rnd(1, 2, 9, 8, seed=25)
    table = rnd(32, 2, seed=26, scale=1.0)
    lse = O.dense_lse(q, k, table, sm_scale=1.0)
    s = torch.einsum("bhqd,bhkd->bhqk", q, k) + O.compute_bias(table, 9, 9, True)[:, :, -5:]
    assert torch.allclose(lse, torch.log(torch.exp(s.double()).sum(-1)).float(), atol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
def test_varlen_equals_per_sequence_dense(causal):
    H, D = 2, 8
    lens = [5, 1, 33, 0, 12]
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    tot = int(cu[-1])
    q, k, v = rnd(tot, H, D, seed=27), rnd(tot, H, D, seed=28), rnd(tot, H, D, seed=29)
    table = rnd(32, H, seed=30, scale=1.0)
    out = O.varlen_attention(q, k, v, table, cu, cu, causal=causal, sm_scale=1.0)
    for b, n in enumerate(lens):
        if n == 0:
            continue
        s = int(cu[b])
        want = CF.dense(q[s:s + n].transpose(0, 1).numpy(), k[s:s + n].transpose(0, 1).numpy(),
                        v[s:s + n].transpose(0, 1).numpy(), table.numpy(), causal, 1.0)
        assert np.abs(out[s:s + n].transpose(0, 1).numpy() - want).max() < 2e-6


def test_unpad_data():
    mask = torch.tensor([[1, 1, 1, 0], [1, 0, 0, 0], [1, 1, 1, 1]])
    idx, cu, mx = O.unpad_data(mask)
    assert idx.tolist() == [0, 1, 2, 4, 8, 9, 10, 11]
    assert cu.tolist() == [0, 3, 4, 8] and cu.dtype == torch.int32 and mx == 4


@pytest.mark.parametrize("S", [1, 2, 3, 8])
def test_splitk_merge_is_dense(S):
    q, k, v = rnd(2, 3, 1, 16, seed=31), rnd(2, 3, 41, 16, seed=32), rnd(2, 3, 41, 16, seed=33)
    so, l, ml = O.splitk_partials(q, k, v, S, 1.0)
    got = O.splitk_merge(so, l, ml)
    want = F.scaled_dot_product_attention(q, k, v, scale=1.0)
    assert torch.allclose(got, want, atol=1e-5)
