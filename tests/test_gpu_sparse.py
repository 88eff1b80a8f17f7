"""GPU parity of the local / block / transient-global forwards and the split-K decode kernel."""
import pytest
import torch

from oracle import t5_basic as O

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-2, torch.float16: 2e-2, torch.float32: 1e-4}


def rnd(*shape, seed=0, scale=0.5, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("L,Bl", [(512, 128), (256, 16), (384, 64), (1024, 512), (100, 128), (640, 128)])
def test_local(gpu_device, dtype, L, Bl):
    from turbot5_amd.ops import local_attention_with_fusing_bias
    B, H, D = 2, 3, 64
    q, k, v = (rnd(B, H, L, D, seed=40 + i, dtype=dtype) for i in range(3))
    table = rnd(32, H, seed=43, scale=1.0)
    out = local_attention_with_fusing_bias(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device),
                                           table.to(gpu_device), Bl)
    want = O.local_attention_blocked(q, k, v, table, Bl)
    assert (out.float().cpu() - want).abs().max().item() <= TOL[dtype]


def test_local_ragged_length_matches_closed_form(gpu_device):
    """L not a multiple of block_len: the reference's blocked code cannot run; the window definition can."""
    from turbot5_amd.ops import local_attention_with_fusing_bias
    B, H, L, D, Bl = 1, 2, 333, 64, 100
    q, k, v = (rnd(B, H, L, D, seed=50 + i) for i in range(3))
    table = rnd(32, H, seed=53, scale=1.0)
    out = local_attention_with_fusing_bias(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device),
                                           table.to(gpu_device), Bl)
    i = torch.arange(L)[:, None]
    j = torch.arange(L)[None, :]
    bias = table[O.relative_position_bucket(j - i, True, 32, 128)].permute(2, 0, 1).unsqueeze(0)
    bias = bias.masked_fill((j - i).abs() >= Bl, float("-inf"))
    want = O.basic_attention(q, k, v, bias)
    assert (out.cpu() - want).abs().max().item() <= 1e-4


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("L,Bl,G", [(512, 128, 64), (256, 32, 8), (384, 128, 128), (300, 128, 64), (100, 128, 64),
                                    (1024, 512, 32), (256, 64, 0)])
def test_block(gpu_device, dtype, L, Bl, G):
    from turbot5_amd.ops import block_attention_with_fusing_bias
    B, H, D = 2, 3, 64
    q, k, v = (rnd(B, H, L, D, seed=60 + i, dtype=dtype) for i in range(3))
    table = rnd(32, H, seed=63, scale=1.0)
    out = block_attention_with_fusing_bias(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device),
                                           table.to(gpu_device), Bl, G)
    want = O.block_attention_blocked(q, k, v, table, Bl, G)
    assert (out.float().cpu() - want).abs().max().item() <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("L,Bl,G,D", [(2048, 128, 64, 64), (1900, 128, 33, 64), (4096, 256, 128, 32), (1536, 64, 16, 128)])
def test_block_global_rows_as_key_splits(gpu_device, dtype, L, Bl, G, D):
    """Long sequences: the G global rows are computed as key splits and merged (workspace given) or by one
    workgroup per (batch, head) (no workspace); both against the oracle."""
    from turbot5_amd.ops import block_attention_with_fusing_bias
    from turbot5_amd import _lib
    B, H = 2, 3
    assert _lib.load().t5a_sparse_workspace_bytes(_lib.PATTERN_BLOCK, B, H, L, D, Bl, G) > 0
    q, k, v = (rnd(B, H, L, D, seed=160 + i, dtype=dtype) for i in range(3))
    table = rnd(32, H, seed=163, scale=1.0)
    dev = [t.to(gpu_device) for t in (q, k, v, table)]
    split = block_attention_with_fusing_bias(*dev, Bl, G)
    single = block_attention_with_fusing_bias(*dev, Bl, G, key_splits=False)
    if L % Bl == 0:
        want = O.block_attention_blocked(q, k, v, table, Bl, G)
        assert (split.float().cpu() - want).abs().max().item() <= TOL[dtype]
        assert (single.float().cpu() - want).abs().max().item() <= TOL[dtype]
    # the two ways differ only in the rounding of the merge, and only in the global rows
    assert (split[:, :, :G].float() - single[:, :, :G].float()).abs().max().item() <= TOL[dtype]
    assert torch.equal(split[:, :, G:], single[:, :, G:])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("L,Bl,gbs", [(512, 128, 16), (256, 32, 8), (2048, 128, 16), (384, 64, 1)])
def test_tglobal(gpu_device, dtype, L, Bl, gbs):
    from turbot5_amd.ops import transient_global_attention_with_fusing_bias
    B, H, D = 2, 3, 64
    q, k, v = (rnd(B, H, L, D, seed=70 + i, dtype=dtype) for i in range(3))
    sk, sv = (rnd(B, H, L // gbs, D, seed=73 + i, dtype=dtype) for i in range(2))
    table = rnd(32, H, seed=75, scale=1.0)
    out = transient_global_attention_with_fusing_bias(*(t.to(gpu_device) for t in (q, k, v, sk, sv)),
                                                      table.to(gpu_device), Bl, gbs)
    want = O.tglobal_attention_blocked(q, k, v, sk, sv, table, Bl, gbs)
    assert (out.float().cpu() - want).abs().max().item() <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,N,S", [(1, 1000, 4), (1, 8192, 8), (3, 500, 7), (8, 257, 2), (1, 5, 8), (1, 300, None)])
def test_splitk(gpu_device, dtype, M, N, S):
    from turbot5_amd.ops import flash_attn_v2_fwd, flash_decoding_attention
    B, H, D = 3, 4, 64
    # (B,H,N,D) views of a (B,N,H,D) cache, as the decoder keeps it
    q = rnd(B, H, M, D, seed=80, dtype=dtype)
    k = rnd(B, N, H, D, seed=81, dtype=dtype).transpose(1, 2)
    v = rnd(B, N, H, D, seed=82, dtype=dtype).transpose(1, 2)
    res, Lsum, ml = flash_attn_v2_fwd(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), None, False, 1.0, S)
    want = O.dense_attention(q, k, v, None, False, 1.0)
    assert res.dtype == torch.float32
    assert (res.cpu() - want).abs().max().item() <= TOL[dtype]
    if S is not None:
        so, l, m = O.splitk_partials(q, k, v, S, 1.0)
        l_, m_ = (l.squeeze(-1), m.squeeze(-1)) if M == 1 else (l, m)
        live = l_ > 0
        assert (ml.cpu()[live] - m_[live]).abs().max().item() <= 2e-2
        assert ((Lsum.cpu()[live] - l_[live]).abs() / l_[live]).max().item() <= 2e-2
    out = flash_decoding_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), None, 1.0, S)
    assert out.dtype == dtype and (out.float().cpu() - want).abs().max().item() <= TOL[dtype]


def test_splitk_with_bias_and_head_dims(gpu_device):
    from turbot5_amd.ops import flash_attn_v2_fwd
    for D in (16, 32, 128):
        B, H, M, N = 2, 2, 2, 333
        q, k, v = rnd(B, H, M, D, seed=90), rnd(B, H, N, D, seed=91), rnd(B, H, N, D, seed=92)
        bias = rnd(1, H, M, N, seed=93, scale=1.0)
        res, _, _ = flash_attn_v2_fwd(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), bias.to(gpu_device),
                                      False, 0.8, 3)
        s = torch.einsum("bhqd,bhkd->bhqk", q * 0.8, k) + bias
        want = torch.softmax(s, -1) @ v
        assert (res.cpu() - want).abs().max().item() <= 1e-4


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("L,Bl,lens", [(512, 128, [512, 300, 1, 129]), (384, 64, [100, 0, 384, 63]),
                                       (256, 16, [255, 17, 16, 200]), (1024, 512, [700, 1024, 511, 5])])
def test_local_with_sequence_lengths(gpu_device, dtype, L, Bl, lens):
    """Right-padded batch through the local pattern: valid rows equal the oracle's mask path
    (key valid and query valid and inside the window, utils.py:174-188)."""
    from turbot5_amd.ops import local_attention_with_fusing_bias
    B, H, D = len(lens), 3, 64
    q, k, v = (rnd(B, H, L, D, seed=60 + i, dtype=dtype) for i in range(3))
    table = rnd(32, H, seed=63, scale=1.0)
    mask = (torch.arange(L)[None, :] < torch.tensor(lens)[:, None]).float()
    out = local_attention_with_fusing_bias(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), table.to(gpu_device), Bl,
                                           seq_lens=torch.tensor(lens, dtype=torch.int32, device=gpu_device))
    want = O.local_attention_blocked(q, k, v, table, Bl, mask)
    assert torch.isfinite(out).all()
    for b, n in enumerate(lens):
        if n:
            assert (out.float().cpu()[b, :, :n] - want[b, :, :n]).abs().max().item() <= TOL[dtype], (b, n)
    # full lengths: the same numbers as the call without lengths
    full = torch.full((B,), L, dtype=torch.int32, device=gpu_device)
    a = local_attention_with_fusing_bias(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), table.to(gpu_device), Bl, seq_lens=full)
    b_ = local_attention_with_fusing_bias(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), table.to(gpu_device), Bl)
    assert torch.equal(a, b_)


def test_sequence_length_arguments_are_checked(gpu_device):
    from turbot5_amd import ops
    q = torch.zeros(1, 1, 128, 64, device=gpu_device, dtype=torch.bfloat16)
    lens = torch.tensor([100], dtype=torch.int32, device=gpu_device)
    with pytest.raises(ValueError):          # first rows are for the windowed patterns
        ops._sparse(ops.L.PATTERN_BLOCK, q, q, q, None, 64, 16, seq_lens=lens, seq_starts=lens)
    with pytest.raises(ValueError):          # ... and need lengths
        ops.local_attention_with_fusing_bias(q, q, q, None, 64, seq_starts=lens)
    with pytest.raises(ValueError):
        ops.local_attention_with_fusing_bias(q, q, q, None, 64, seq_lens=lens.long())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("L,Bl,gbs,lens", [(512, 128, 16, [512, 300, 17, 129]), (256, 32, 8, [255, 7, 0, 64]),
                                           (1024, 128, 16, [1000, 1024, 130, 15])])
def test_tglobal_with_sequence_lengths(gpu_device, dtype, L, Bl, gbs, lens):
    """Right-padded batch through the transient-global pattern: valid rows equal the oracle's mask path
    (local mask, block ids with orphan tokens, side-token validity; utils.py:174-237)."""
    from turbot5_amd.ops import transient_global_attention_with_fusing_bias
    B, H, D = len(lens), 3, 64
    q, k, v = (rnd(B, H, L, D, seed=80 + i, dtype=dtype) for i in range(3))
    sk, sv = (rnd(B, H, L // gbs, D, seed=83 + i, dtype=dtype) for i in range(2))
    table = rnd(32, H, seed=85, scale=1.0)
    mask = (torch.arange(L)[None, :] < torch.tensor(lens)[:, None]).float()
    out = transient_global_attention_with_fusing_bias(*(t.to(gpu_device) for t in (q, k, v, sk, sv)),
                                                      table.to(gpu_device), Bl, gbs,
                                                      seq_lens=torch.tensor(lens, dtype=torch.int32, device=gpu_device))
    want = O.tglobal_attention_blocked(q, k, v, sk, sv, table, Bl, gbs, mask)
    assert torch.isfinite(out).all()
    for b, n in enumerate(lens):
        if n:
            assert (out.float().cpu()[b, :, :n] - want[b, :, :n]).abs().max().item() <= TOL[dtype], (b, n)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,N,S", [(1, 1000, 4), (1, 8192, None), (3, 500, 7)])
def test_splitk_over_padded_memories(gpu_device, dtype, M, N, S):
    """Each batch element only has the keys [start, start + len) of its N rows: equal to dense attention over
    exactly those keys; an element without keys comes out zero; splits that hold no valid key drop out."""
    from turbot5_amd.ops import flash_decoding_attention
    B, H, D = 5, 3, 64
    q = rnd(B, H, M, D, seed=90, dtype=dtype)
    k, v = (rnd(B, H, N, D, seed=91 + i, dtype=dtype) for i in range(2))
    lens = [N, N // 3, 1, 0, N - 7]
    starts = [0, 5, N - 1, 0, 7]
    dq, dk, dv = (t.to(gpu_device) for t in (q, k, v))
    tl = torch.tensor(lens, dtype=torch.int32, device=gpu_device)
    ts = torch.tensor(starts, dtype=torch.int32, device=gpu_device)
    out = flash_decoding_attention(dq, dk, dv, None, 1.0, num_splits=S, key_lens=tl, key_starts=ts).float().cpu()
    for b in range(B):
        if lens[b] == 0:
            assert (out[b] == 0).all()
            continue
        sl = slice(starts[b], starts[b] + lens[b])
        want = O.basic_attention(q[b:b + 1].float(), k[b:b + 1, :, sl].float(), v[b:b + 1, :, sl].float(), None)
        assert (out[b] - want[0]).abs().max().item() <= TOL[dtype], b
    # right padding only: starts may be left out
    right = flash_decoding_attention(dq, dk, dv, None, 1.0, num_splits=S, key_lens=tl).float().cpu()
    want = O.basic_attention(q[1:2].float(), k[1:2, :, :lens[1]].float(), v[1:2, :, :lens[1]].float(), None)
    assert (right[1] - want[0]).abs().max().item() <= TOL[dtype]
    with pytest.raises(ValueError):
        flash_decoding_attention(dq, dk, dv, None, 1.0, key_starts=ts)


@pytest.mark.parametrize("run_len", [1, 2, 3, 5, 16])
@pytest.mark.parametrize("L,Bl", [(640, 128), (333, 100), (1000, 16), (896, 256), (700, 300)])
def test_local_with_runs_of_q_tiles(gpu_device, monkeypatch, run_len, L, Bl):
    """The local pattern's work items are runs of consecutive q tiles (one stream of key tiles through the LDS
    rings, the distance LUT built once per run); a run may end inside a (batch, head) or cross into the next
    one.  Every run length must give what the window definition gives, for sequence lengths that are no
    multiple of anything, with per-sequence lengths, and for windows too wide for the LUT (masked path)."""
    from turbot5_amd import ops
    from turbot5_amd.ops import local_attention_with_fusing_bias
    monkeypatch.setattr(ops, "RUN_LEN", run_len)
    B, H, D = 2, 3, 64
    q, k, v = (rnd(B, H, L, D, seed=300 + i, dtype=torch.bfloat16) for i in range(3))
    table = rnd(32, H, seed=303, scale=1.0)
    lens = torch.tensor([L, max(1, L - 217)], dtype=torch.int32)
    dev = [t.to(gpu_device) for t in (q, k, v, table)]
    out = local_attention_with_fusing_bias(*dev, Bl).float().cpu()
    out_l = local_attention_with_fusing_bias(*dev, Bl, seq_lens=lens.to(gpu_device)).float().cpu()
    i = torch.arange(L)[:, None]
    j = torch.arange(L)[None, :]
    bias = table[O.relative_position_bucket(j - i, True, 32, 128)].permute(2, 0, 1).unsqueeze(0)
    bias = bias.masked_fill((j - i).abs() >= Bl, float("-inf"))
    want = O.basic_attention(q.float(), k.float(), v.float(), bias)
    assert (out - want).abs().max().item() <= 2e-2
    for b in range(B):
        n = int(lens[b])
        wb = O.basic_attention(q[b:b + 1, :, :n].float(), k[b:b + 1, :, :n].float(), v[b:b + 1, :, :n].float(),
                               bias[:, :, :n, :n])
        assert (out_l[b:b + 1, :, :n] - wb).abs().max().item() <= 2e-2, b


@pytest.mark.parametrize("run_len", [1, 2, 3, 7, 16])
@pytest.mark.parametrize("L,Bl,G", [(1024, 128, 64), (900, 100, 20), (768, 256, 32), (640, 64, 64)])
def test_block_with_runs_of_q_tiles(gpu_device, monkeypatch, run_len, L, Bl, G):
    """The block pattern's work items are runs of consecutive q tiles as well, with the global rows' key splits
    behind them in the same launch (or a pass of their own without a workspace).  Every run length gives the
    oracle's result, with guard rows behind the output untouched."""
    from turbot5_amd import ops
    monkeypatch.setattr(ops, "RUN_LEN", run_len)
    B, H, D = 2, 3, 64
    q, k, v = (rnd(B, H, L, D, seed=310 + i, dtype=torch.bfloat16) for i in range(3))
    table = rnd(32, H, seed=313, scale=1.0)
    want = O.block_attention_blocked(q.float(), k.float(), v.float(), table, Bl, G)
    for key_splits in (True, False):
        out = ops.block_attention_with_fusing_bias(*(t.to(gpu_device) for t in (q, k, v, table)), Bl, G,
                                                   key_splits=key_splits).float().cpu()
        assert torch.isfinite(out).all()
        assert (out - want).abs().max().item() <= 2e-2, key_splits


@pytest.mark.parametrize("B,H,L,Bl,G", [(8, 12, 1024, 128, 64), (16, 12, 1024, 128, 64), (4, 16, 2048, 64, 32)])
def test_block_with_many_batch_heads(gpu_device, B, H, L, Bl, G):
    """Shapes with so many (batch, head) pairs that the launch plan leaves the global rows ONE key split per pair
    (t5a_sparse_launch_plan says so): the single split is still an item of its own behind the runs.  Output
    written into a larger buffer whose guard rows must stay as they were."""
    import ctypes as C
    from turbot5_amd import _lib, ops
    plan = (C.c_int32 * 6)()
    _lib.check(_lib.load().t5a_sparse_launch_plan(_lib.PATTERN_BLOCK, _lib.T5A_BF16, B, H, L, 64, Bl, G, 1, 0, 0, plan))
    run_len, items, block_items, nsplit, split_rows, tps = list(plan)
    assert block_items > 0 and items == block_items + nsplit * B * H
    D = 64
    q, k, v = (rnd(B, H, L, D, seed=320 + i, dtype=torch.bfloat16) for i in range(3))
    table = rnd(32, H, seed=323, scale=1.0)
    out = ops.block_attention_with_fusing_bias(*(t.to(gpu_device) for t in (q, k, v, table)), Bl, G).float().cpu()
    assert torch.isfinite(out).all()
    # the oracle on a few (batch, head) pairs: first, last and one in the middle
    for b, h in ((0, 0), (B - 1, H - 1), (B // 2, H // 2)):
        want = O.block_attention_blocked(q[b:b + 1, h:h + 1].float(), k[b:b + 1, h:h + 1].float(),
                                         v[b:b + 1, h:h + 1].float(), table[:, h:h + 1], Bl, G)
        assert (out[b:b + 1, h:h + 1] - want).abs().max().item() <= 2e-2, (b, h)
    # size-independent property on everything: V = 1 gives 1
    ones = torch.ones_like(v).to(gpu_device)
    out1 = ops.block_attention_with_fusing_bias(q.to(gpu_device), k.to(gpu_device), ones, table.to(gpu_device), Bl, G)
    assert (out1.float() - 1.0).abs().max().item() <= 1e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("L,Bl,G", [(1024, 128, 64), (512, 64, 64), (768, 256, 32), (640, 128, 0)])
def test_block_with_right_padded_sequences(gpu_device, dtype, L, Bl, G):
    """Per-sequence lengths in the block pattern against the oracle's mask path (pinned by vectors from the
    reference module): lengths inside block 0, inside a later block on either side of its first G columns, at a
    block boundary, and a full sequence; with and without key splits for the global rows."""
    from turbot5_amd.ops import block_attention_with_fusing_bias
    H, D = 3, 64
    lens = [L, Bl // 2, Bl + G // 2 + 1, 2 * Bl + G + 5, 3 * Bl, L - 1]
    B = len(lens)
    q, k, v = (rnd(B, H, L, D, seed=400 + i, dtype=dtype) for i in range(3))
    table = rnd(32, H, seed=403, scale=1.0)
    mask = (torch.arange(L)[None, :] < torch.tensor(lens)[:, None]).float()
    want = O.block_attention_blocked(q, k, v, table, Bl, G, mask)
    tl = torch.tensor(lens, dtype=torch.int32, device=gpu_device)
    dev = [t.to(gpu_device) for t in (q, k, v, table)]
    for splits in (True, False):
        out = block_attention_with_fusing_bias(*dev, Bl, G, seq_lens=tl, key_splits=splits).float().cpu()
        for b, n in enumerate(lens):
            err = (out[b, :, :n] - want[b, :, :n]).abs().max().item()
            assert err <= TOL[dtype], (b, n, splits, err)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("L,Bl", [(1024, 128), (512, 64), (1536, 512)])
def test_local_with_padding_on_either_side(gpu_device, dtype, L, Bl):
    from turbot5_amd.ops import local_attention_with_fusing_bias
    H, D = 3, 64
    spans = [(0, L), (37, L - 37), (Bl + 3, 2 * Bl), (L - 70, 70), (5, 1), (0, 0)]
    B = len(spans)
    q, k, v = (rnd(B, H, L, D, seed=410 + i, dtype=dtype) for i in range(3))
    table = rnd(32, H, seed=413, scale=1.0)
    pos = torch.arange(L)[None, :]
    st, ln = torch.tensor([s for s, _ in spans])[:, None], torch.tensor([n for _, n in spans])[:, None]
    mask = ((pos >= st) & (pos < st + ln)).float()
    want = O.local_attention_blocked(q, k, v, table, Bl, mask)
    out = local_attention_with_fusing_bias(
        *(t.to(gpu_device) for t in (q, k, v, table)), Bl,
        seq_lens=ln[:, 0].to(torch.int32).to(gpu_device), seq_starts=st[:, 0].to(torch.int32).to(gpu_device)).float().cpu()
    valid = mask.bool()
    assert torch.isfinite(out[valid[:, None, :].expand(B, H, L)]).all()
    err = (out - want).abs()[valid[:, None, :, None].expand(B, H, L, D)].max().item()
    assert err <= TOL[dtype], err


@pytest.mark.parametrize("L,Bl", [(1024, 128), (700, 64), (512, 32)])
def test_local_windowed_lut_buffer_gives_identical_results(gpu_device, L, Bl):
    """The local pattern's LUT images (sliding window folded in), built once into a buffer and fetched by later
    launches, are the images its work items otherwise fill for themselves: outputs are bit-identical without the
    buffer, on the launch that builds it and on those that find it ready; buffers for different windows and the plain
    one of the same table are separate entries."""
    from turbot5_amd import ops
    B, H, D = 2, 3, 64
    q, k, v = (rnd(B, H, L, D, seed=140 + i, dtype=torch.bfloat16).to(gpu_device) for i in range(3))
    table = rnd(32, H, seed=143, scale=1.0).to(gpu_device)
    run = lambda bl=Bl: ops.local_attention_with_fusing_bias(q, k, v, table, bl).cpu()  # noqa: E731
    ops.clear_bias_luts()
    ops.BIAS_LUT_CACHE = False
    try:
        plain = run()
        other_plain = run(2 * Bl)
        dense_plain = ops.flash_attention_with_fusing_bias(q, k, v, table, causal=False, sm_scale=1.0).cpu()
    finally:
        ops.BIAS_LUT_CACHE = True
    assert len(ops._BIAS_LUTS) == 0
    first, second = run(), run()
    assert len(ops._BIAS_LUTS) == 1
    assert torch.equal(plain.view(torch.int16), first.view(torch.int16))
    assert torch.equal(plain.view(torch.int16), second.view(torch.int16))
    other = run(2 * Bl)                # another window: its own images
    dense = ops.flash_attention_with_fusing_bias(q, k, v, table, causal=False, sm_scale=1.0).cpu()   # the plain ones
    from turbot5_amd import _lib
    has_other = _lib.load().t5a_bias_lut_bytes_windowed(H, 32, 128, 2 * Bl) > 0   # (a window of 256 is too long to fetch)
    assert len(ops._BIAS_LUTS) == (3 if has_other else 2)
    assert torch.equal(other_plain.view(torch.int16), other.view(torch.int16))
    assert torch.equal(dense_plain.view(torch.int16), dense.view(torch.int16))
    assert torch.equal(plain.view(torch.int16), run().view(torch.int16))
    want = O.local_attention_blocked(q.cpu(), k.cpu(), v.cpu(), table.cpu(), Bl) if L % Bl == 0 else None
    if want is not None:
        assert (first.float() - want).abs().max().item() <= 2e-2
    ops.clear_bias_luts()


def test_windowed_lut_buffer_is_only_for_its_window(gpu_device):
    """A buffer of windowed images is refused by every call that would read it as something else; a plain buffer
    handed to the local pattern is ignored."""
    import ctypes as C
    from turbot5_amd import _lib as lib_mod, ops
    lib = lib_mod.load()
    B, H, L, D, Bl = 1, 2, 256, 64, 64
    q, k, v = (rnd(B, H, L, D, seed=150 + i, dtype=torch.bfloat16).to(gpu_device) for i in range(3))
    table = rnd(32, H, seed=153, scale=1.0).to(gpu_device)
    o = torch.empty_like(q)
    nbytes = lib.t5a_bias_lut_bytes_windowed(H, 32, 128, Bl)
    assert nbytes > 0
    lut = torch.zeros(nbytes, dtype=torch.uint8, device=gpu_device)

    def sparse_args(block_len, window):
        a = lib_mod.T5ASparseArgs()
        a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
        for name, t in (("q_strides", q), ("k_strides", k), ("v_strides", v), ("o_strides", o)):
            setattr(a, name, (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2)))
        a.dtype, a.B, a.H, a.L, a.D = lib_mod.T5A_BF16, B, H, L, D
        a.pattern, a.block_len, a.aux, a.sm_scale = lib_mod.PATTERN_LOCAL, block_len, 0, 1.0
        a.bias.table, a.bias.table_dtype = table.data_ptr(), lib_mod.T5A_F32
        a.bias.num_buckets, a.bias.max_distance = 32, 128
        a.bias.stride_bucket, a.bias.stride_head = table.stride(0), table.stride(1)
        a.bias.lut, a.bias.lut_bytes, a.bias.lut_window, a.bias.lut_ready = lut.data_ptr(), nbytes, window, 0
        return a

    stream = ops._stream(q)
    with torch.cuda.device(gpu_device):
        assert lib.t5a_fwd_sparse(C.byref(sparse_args(Bl, Bl)), stream) == 0           # builds and uses it
        built = o.clone()
        assert lib.t5a_fwd_sparse(C.byref(sparse_args(2 * Bl, Bl)), stream) != 0       # another window: refused
        assert b"window" in lib.t5a_last_error()
        a = sparse_args(Bl, 0)                                                         # declared plain: ignored
        a.bias.lut_ready = 1
        o.zero_()
        assert lib.t5a_fwd_sparse(C.byref(a), stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(o.view(torch.int16), built.view(torch.int16))
        a = sparse_args(Bl, -3)
        assert lib.t5a_fwd_sparse(C.byref(a), stream) != 0


def _random_masks(B, L, seed):
    """rows: holes everywhere, left padding, padding on both sides, a long run of zeros inside, all ones"""
    g = torch.Generator().manual_seed(seed)
    m = torch.ones(B, L)
    m[0] = (torch.rand(L, generator=g) > 0.3).float()
    if B > 1:
        m[1, : L // 3] = 0
    if B > 2:
        m[2, : L // 5] = 0
        m[2, -(L // 4):] = 0
    if B > 3:
        m[3, L // 3: L // 3 + min(L // 2, 300)] = 0
    m[:, L // 2] = 1   # no empty row
    return m


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("L,Bl", [(512, 128), (384, 64), (640, 32), (1024, 256), (768, 384)])
def test_local_with_masks_of_any_shape(gpu_device, dtype, L, Bl):
    """key_bits: the key half of the reference's local mask for masks with holes and padding on either side;
    rows of valid tokens against the oracle's mask path"""
    from turbot5_amd import ops
    B, H, D = 5, 2, 64
    q, k, v = (rnd(B, H, L, D, seed=160 + i, dtype=dtype) for i in range(3))
    table = rnd(32, H, seed=163, scale=1.0)
    mask = _random_masks(B, L, 164)
    bits = ops.pack_key_bits(mask.to(gpu_device), Bl)
    out = ops.local_attention_with_fusing_bias(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device),
                                               table.to(gpu_device), Bl, key_bits=bits).float().cpu()
    want = O.local_attention_blocked(q, k, v, table, Bl, attention_mask=mask)
    rows = mask.bool()[:, None, :, None].expand_as(out)
    assert torch.isfinite(out[rows]).all()
    assert (out - want)[rows].abs().max().item() <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("L,Bl,G", [(512, 128, 64), (384, 64, 16), (1024, 256, 32), (640, 128, 128), (500, 100, 20)])
def test_block_with_masks_of_any_shape(gpu_device, dtype, L, Bl, G):
    """key_bits: the reference's additive mask over its key list, [own block | global tokens] laid over
    [global tokens | own block], for masks of any shape; rows of valid tokens against the oracle"""
    from turbot5_amd import ops
    B, H, D = 5, 2, 64
    q, k, v = (rnd(B, H, L, D, seed=170 + i, dtype=dtype) for i in range(3))
    table = rnd(32, H, seed=173, scale=1.0)
    mask = _random_masks(B, L, 174)
    bits = ops.pack_key_bits(mask.to(gpu_device), Bl, G)
    out = ops.block_attention_with_fusing_bias(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device),
                                               table.to(gpu_device), Bl, G, key_bits=bits).float().cpu()
    want = O.block_attention_blocked(q, k, v, table, Bl, G, attention_mask=mask)
    # Every row of a valid token keeps a visible column: the first G rows see every key; a row of block b >= 1 always
    # sees the last G list columns; a row of block 0 sees list column c iff token c is valid, and it is such a token
    # itself.  So the set of compared rows comes from the mask alone, and the kernel must be finite on all of them.
    rows = mask.bool()[:, None, :, None].expand_as(out)
    assert rows.float().mean().item() > 0.5
    assert torch.isfinite(out[rows]).all()
    assert (out - want)[rows].abs().max().item() <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("L,Bl,gbs", [(512, 128, 16), (384, 64, 8), (640, 32, 16), (1000, 127, 16), (300, 64, 32)])
def test_tglobal_with_masks_of_any_shape(gpu_device, dtype, L, Bl, gbs):
    """key_bits and side_counts: window keys by their validity, side tokens counted by the valid block ENDs, a
    token's side token min(row // gbs, count - 1) (utils.py:191-237); rows of valid tokens against the oracle"""
    from turbot5_amd import ops
    B, H, D = 5, 2, 64
    q, k, v = (rnd(B, H, L, D, seed=180 + i, dtype=dtype) for i in range(3))
    sk, sv = (rnd(B, H, L // gbs, D, seed=183 + i, dtype=dtype) for i in range(2))
    table = rnd(32, H, seed=185, scale=1.0)
    mask = _random_masks(B, L, 186)
    dmask = mask.to(gpu_device)
    bits = ops.pack_key_bits(dmask, Bl, gbs)
    counts = ops.side_token_counts(dmask, gbs)
    assert counts.tolist() == [int(mask[b, gbs - 1::gbs].sum()) for b in range(B)]
    out = ops.transient_global_attention_with_fusing_bias(
        *(t.to(gpu_device) for t in (q, k, v, sk, sv)), table.to(gpu_device), Bl, gbs, key_bits=bits,
        side_counts=counts).float().cpu()
    want = O.tglobal_attention_blocked(q, k, v, sk, sv, table, Bl, gbs, mask)
    rows = mask.bool()[:, None, :, None].expand_as(out)
    assert torch.isfinite(out[rows]).all()
    assert (out - want)[rows].abs().max().item() <= TOL[dtype]
    with pytest.raises(ValueError):   # the counts are not optional
        ops.transient_global_attention_with_fusing_bias(
            *(t.to(gpu_device) for t in (q, k, v, sk, sv)), table.to(gpu_device), Bl, gbs, key_bits=bits)
