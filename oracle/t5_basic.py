"""CPU restatement of the reference's 'basic' T5 attention math (pure torch).

TEST INFRASTRUCTURE ONLY -- see ``oracle/__init__.py``.  Every function cites
the reference lines (relative to the reference checkout) it restates.

Pinning status (what checks each function besides this file itself):

* ``relative_position_bucket``  -- known-answer table, the installed HuggingFace
  ``transformers`` T5 implementation (third-party), brute-force integer closed
  form.  tests/test_oracle_bucket.py
* ``compute_bias`` / ``basic_attention`` / ``dense_attention`` -- torch SDPA in
  fp64, invariants (V=1, constant table shift, causal row 0).
  tests/test_oracle_dense.py
* ``local_attention_blocked`` and the blocking helpers -- HuggingFace LongT5
  helpers / ``LongT5LocalAttention`` (third-party) and a brute-force dense-mask
  closed form.  tests/test_oracle_sparse.py
* ``tglobal_attention_blocked`` -- HuggingFace ``LongT5TransientGlobalAttention``
  (with its side table set equal to the local table) and the closed form.
* ``block_attention_blocked`` -- vectors written from the reference's own
  ``T5BlockAttention`` (all-ones, right-padded, left-padded and holed masks,
  ragged last block, sequences shorter than a block; tests/golden/
  sparse_modules.npz, made by tests/golden/make_sparse_fixtures.py in the build
  container) and a brute-force closed form.  tests/test_oracle_fixtures.py
* the local and transient-global functions with left padding and holes in the
  mask -- the same fixture file (``T5LocalAttention``,
  ``T5TransientGlobalAttention`` end to end).
* ``splitk_merge`` -- identity with un-split dense attention.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

NEG_MASK = -1e10  # the additive "masked" value the sparse modules use (att.py:602, :697)


# --------------------------------------------------------------------------
# a1  bucket function                                           att.py:78-124
# --------------------------------------------------------------------------
def relative_position_bucket(relative_position: torch.Tensor, bidirectional: bool = True,
                             num_buckets: int = 32, max_distance: int = 128) -> torch.Tensor:
    """int64 tensor of (memory_pos - query_pos) -> int64 bucket ids (att.py:78-124).

    The fp32 ``log`` and the truncating cast are kept exactly as the reference
    has them; that is what fixes the bucket boundaries.
    """
    rp = relative_position.to(torch.long)
    out = torch.zeros_like(rp)
    nb = num_buckets
    if bidirectional:
        nb //= 2
        out = out + (rp > 0).to(torch.long) * nb            # att.py:99
        rp = rp.abs()                                       # att.py:100
    else:
        rp = -torch.minimum(rp, torch.zeros_like(rp))       # att.py:102
    max_exact = nb // 2                                     # att.py:106
    small = rp < max_exact
    big = max_exact + (
        torch.log(rp.float() / max_exact) / math.log(max_distance / max_exact) * (nb - max_exact)
    ).to(torch.long)                                        # att.py:110-114
    big = torch.minimum(big, torch.full_like(big, nb - 1))  # att.py:115-117
    return out + torch.where(small, rp, big)


# --------------------------------------------------------------------------
# a2  materialised bias                                        att.py:126-141
# --------------------------------------------------------------------------
def compute_bias(table: torch.Tensor, query_length: int, key_length: int, bidirectional: bool,
                 num_buckets: int = 32, max_distance: int = 128) -> torch.Tensor:
    """(num_buckets, H) table -> (1, H, query_length, key_length) bias (att.py:126-141)."""
    ctx = torch.arange(query_length, dtype=torch.long)[:, None]
    mem = torch.arange(key_length, dtype=torch.long)[None, :]
    buckets = relative_position_bucket(mem - ctx, bidirectional, num_buckets, max_distance)
    return table[buckets].permute(2, 0, 1).unsqueeze(0)


# --------------------------------------------------------------------------
# a3  'basic' attention                                         naive.py:4-23
# --------------------------------------------------------------------------
def basic_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                    position_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """softmax(q k^T + bias) v with NO 1/sqrt(d), softmax in fp32 (naive.py:4-23, eval mode)."""
    scores = torch.einsum("...qd,...kd->...qk", q, k)
    if position_bias is not None:
        scores = scores + position_bias.to(scores.dtype)
    weights = F.softmax(scores.float(), dim=-1).type_as(scores)
    return torch.einsum("...hqk,...hkd->...hqd", weights, v)


def dense_bias(table: Optional[torch.Tensor], M: int, N: int, causal: bool,
               num_buckets: int = 32, max_distance: int = 128, H: int = 1,
               dtype=torch.float32) -> torch.Tensor:
    """Bias + causal mask of one dense call, (1,H,M,N).

    Queries are aligned to the END of the keys as 'basic' does with a KV cache:
    bias is computed for N x N and the last M query rows are kept
    (att.py:229-234).  Bucket mode is unidirectional iff causal, because
    T5FlashAttention ties both to ``is_decoder`` (att.py:390, :135).  The causal
    mask is the decoder's extended mask: key j visible iff j <= i + (N - M).
    """
    if table is not None and M <= N:
        bias = compute_bias(table.to(dtype), N, N, not causal, num_buckets, max_distance)[:, :, N - M:, :]
        if causal:
            i = torch.arange(M)[:, None] + (N - M)
            bias = bias.masked_fill(torch.arange(N)[None, :] > i, float("-inf"))
        return bias
    # no table (zeros, att.py:222-227) or M > N (never happens in 'basic'): same closed form
    return _dense_bias_rows(table, 0, M, M, N, causal, num_buckets, max_distance, H, dtype)


def dense_attention(q, k, v, table=None, causal=False, sm_scale=None, num_buckets=32, max_distance=128,
                    compute_dtype=torch.float32, row_chunk: int = 1024) -> torch.Tensor:
    """Oracle for one ``flash_attention_with_fusing_bias`` call (fused.py:876-890).

    q (B,H,M,D); k,v (B,H,N,D).  ``sm_scale=None`` means 1/sqrt(D) (fused.py:833-834).
    Inputs are first converted to ``compute_dtype`` (fp32 by default: "fp32 math
    on the rounded inputs"); pass the input dtype for the literal low-precision
    'basic'.  Rows are processed in chunks so long sequences fit in host RAM;
    chunking changes nothing numerically (rows are independent).  Fully masked
    rows (causal with M > N) give zeros, as fused.py:352-355 does.
    """
    B, H, M, D = q.shape
    N = k.shape[2]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    qf, kf, vf = (t.to(compute_dtype) for t in (q, k, v))
    out = torch.empty(B, H, M, D, dtype=compute_dtype)
    for r0 in range(0, M, row_chunk):
        r1 = min(M, r0 + row_chunk)
        bias = _dense_bias_rows(table, r0, r1, M, N, causal, num_buckets, max_distance, H, compute_dtype)
        qs = qf[:, :, r0:r1] * sm_scale if sm_scale != 1.0 else qf[:, :, r0:r1]
        o = basic_attention(qs, kf, vf, bias)
        out[:, :, r0:r1] = torch.nan_to_num(o, nan=0.0)
    return out


def _dense_bias_rows(table, r0, r1, M, N, causal, nb, md, H, dtype):
    i = torch.arange(r0, r1, dtype=torch.long)[:, None] + (N - M)
    j = torch.arange(N, dtype=torch.long)[None, :]
    if table is not None:
        bias = table.to(dtype)[relative_position_bucket(j - i, not causal, nb, md)].permute(2, 0, 1).unsqueeze(0)
    else:
        bias = torch.zeros(1, H, r1 - r0, N, dtype=dtype)
    if causal:
        bias = bias.masked_fill(j > i, float("-inf"))
    return bias


def dense_lse(q, k, table=None, causal=False, sm_scale=None, num_buckets=32, max_distance=128) -> torch.Tensor:
    """Natural-log normaliser per query row, (B,H,M) fp32 (fused.py:358)."""
    B, H, M, D = q.shape
    N = k.shape[2]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    s = torch.einsum("bhqd,bhkd->bhqk", q.float() * sm_scale, k.float())
    s = s + dense_bias(table, M, N, causal, num_buckets, max_distance, H)
    return torch.logsumexp(s, dim=-1)


# --------------------------------------------------------------------------
# a7  varlen = per-sequence dense                            varlen.py:870-889
# --------------------------------------------------------------------------
def varlen_attention(q, k, v, table, cu_seqlens_q, cu_seqlens_k, causal=False, sm_scale=None,
                     num_buckets=32, max_distance=128, compute_dtype=torch.float32) -> torch.Tensor:
    """q (total_q,H,D), k/v (total_k,H,D) packed; positions are in-sequence (varlen.py:254, :303)."""
    out = torch.zeros(q.shape, dtype=compute_dtype)
    cq = [int(x) for x in cu_seqlens_q]
    ck = [int(x) for x in cu_seqlens_k]
    for b in range(len(cq) - 1):
        qs, qe, ks, ke = cq[b], cq[b + 1], ck[b], ck[b + 1]
        if qe == qs:
            continue
        if ke == ks:
            continue  # no keys: rows stay zero
        o = dense_attention(q[qs:qe].transpose(0, 1)[None], k[ks:ke].transpose(0, 1)[None],
                            v[ks:ke].transpose(0, 1)[None], table, causal, sm_scale,
                            num_buckets, max_distance, compute_dtype)
        out[qs:qe] = o[0].transpose(0, 1)
    return out


# --------------------------------------------------------------------------
# a8  unpad / pad                                             padding.py:79-150
# --------------------------------------------------------------------------
def unpad_data(attention_mask: torch.Tensor):
    """(B,L) 0/1 mask -> (indices of valid tokens in the flattened batch, cu_seqlens int32, max len)
    (padding.py:79-88)."""
    seqlens = attention_mask.sum(dim=-1, dtype=torch.int32)
    indices = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
    cu = F.pad(torch.cumsum(seqlens, dim=0, dtype=torch.int32), (1, 0))
    return indices, cu, int(seqlens.max())


# --------------------------------------------------------------------------
# a7-helpers  LongT5-style blocking                              utils.py:84-188
# --------------------------------------------------------------------------
def pad_to_multiple(x: torch.Tensor, block_len: int, dim: int, pad_value=0) -> torch.Tensor:
    """utils.py:84-97."""
    dim = dim % x.ndim
    pad_len = -x.shape[dim] % block_len
    if not all(x.shape):
        shape = list(x.shape)
        shape[dim] += pad_len
        return torch.zeros(shape, dtype=x.dtype)
    widths = [0, 0] * x.ndim
    widths[2 * (x.ndim - 1 - dim) + 1] = pad_len
    return F.pad(x, widths, mode="constant", value=pad_value)


def split_into_blocks(x: torch.Tensor, block_len: int, dim: int, swap12: bool = True) -> torch.Tensor:
    """utils.py:99-113 (``swap12``) and :139-154 (no swap: the mask variant).

    Pads to a multiple of block_len when at least one full block exists, else
    uses the whole length as the single block; inserts (num_blocks, block_len)
    at ``dim``; the data variant then swaps dims 1 and 2 (blocks before heads).
    """
    dim = dim % x.ndim
    n = x.shape[dim]
    if n % block_len != 0 and n // block_len >= 1:
        x = pad_to_multiple(x, block_len, dim, 0)
    elif n // block_len < 1:
        block_len = n
    nb = x.shape[dim] // block_len
    shape = x.shape[:dim] + (nb, block_len) + x.shape[dim + 1:]
    y = x.reshape(shape)
    return y.transpose(1, 2) if swap12 else y


def concatenate_3_blocks(x: torch.Tensor, block_dim: int, sequence_dim: int, pad_value=0) -> torch.Tensor:
    """[prev | own | next] block along ``sequence_dim``, zero blocks at both ends (utils.py:115-137)."""
    nb = x.shape[block_dim]
    widths = [0, 0] * x.ndim
    widths[2 * (x.ndim - 1 - block_dim)] = 1
    widths[2 * (x.ndim - 1 - block_dim) + 1] = 1
    xp = F.pad(x, widths, mode="constant", value=pad_value)
    parts = [xp.narrow(block_dim, s, nb) for s in range(3)]
    return torch.cat(parts, dim=sequence_dim)


def local_attention_mask(attention_mask: torch.Tensor, block_len: int) -> torch.Tensor:
    """(B,L) 0/1 -> (B,nb,1,Bl,3Bl) bool: query valid & key valid & |rel| < Bl (utils.py:174-188, :156-172)."""
    blocked = split_into_blocks(attention_mask, block_len, 1, swap12=False)       # (B,nb,Bl)
    three = concatenate_3_blocks(blocked, block_dim=1, sequence_dim=2)           # (B,nb,3Bl)
    m = torch.logical_and(blocked.unsqueeze(-1), three.unsqueeze(-2))            # (B,nb,Bl,3Bl)
    bl = m.shape[2]
    pos = torch.arange(3 * bl, dtype=torch.int32)
    rel = pos[None, :] - pos[bl:2 * bl][:, None]
    m = torch.logical_and(m, (rel.abs() < bl)[None, None])
    return m.unsqueeze(2)


def local_block_bias(table: torch.Tensor, block_len: int, bidirectional: bool, nb: int, md: int) -> torch.Tensor:
    """(1,1,H,Bl,3Bl): rel = j3 - (Bl + r) (att.py:529-551)."""
    mem = torch.arange(3 * block_len, dtype=torch.long)
    ctx = mem[block_len:-block_len]
    b = relative_position_bucket(mem[None, :] - ctx[:, None], bidirectional, nb, md)
    return table[b].permute(2, 0, 1)[None, None]


def _flatten_blocks(x):          # "shape_blocks" att.py:575-576 (reshape: tolerant of the non-viewable case)
    return x.reshape(-1, x.size(2), x.size(3), x.size(4))


def _unblock(o, B, L):           # (B*nb,H,Bl,D) -> (B,H,L,D)   (unshape att.py:578-580 without the head merge)
    nbk, H, Bl, D = o.shape
    return o.reshape(B, nbk // B, H, Bl, D).permute(0, 2, 1, 3, 4).reshape(B, H, -1, D)[:, :, :L]


def local_attention_blocked(q, k, v, table, block_len: int, attention_mask: Optional[torch.Tensor] = None,
                            num_buckets=32, max_distance=128, compute_dtype=torch.float32) -> torch.Tensor:
    """Literal blocked evaluation of T5LocalAttention's op (att.py:583-638), in-model mask path.

    q,k,v (B,H,L,D); ``attention_mask`` (B,L) 0/1 (None = all ones, what T5Stack
    supplies: modeling.py:479-480, :488-489).  Returns (B,H,L,D).
    """
    B, H, L, D = q.shape
    q, k, v = (t.to(compute_dtype) for t in (q, k, v))
    if attention_mask is None:
        attention_mask = torch.ones(B, L)
    qb = _flatten_blocks(split_into_blocks(q, block_len, 2))
    kb = _flatten_blocks(concatenate_3_blocks(split_into_blocks(k, block_len, 2), 1, 3))
    vb = _flatten_blocks(concatenate_3_blocks(split_into_blocks(v, block_len, 2), 1, 3))
    m = local_attention_mask(attention_mask, block_len)
    m = torch.where(m > 0, 0.0, NEG_MASK).to(compute_dtype)                       # att.py:600-602
    m = _flatten_blocks(m)
    bl = qb.shape[2]
    if table is not None:
        bias = _flatten_blocks(local_block_bias(table.to(compute_dtype), bl, True, num_buckets, max_distance))
    else:
        bias = torch.zeros(1, H, bl, 3 * bl, dtype=compute_dtype)
    bias = bias + m                                                               # att.py:619-621
    return _unblock(basic_attention(qb, kb, vb, bias), B, L)


# --------------------------------------------------------------------------
# a10  block attention with global tokens                        att.py:652-862
# --------------------------------------------------------------------------
def block_attention_blocked(q, k, v, table, block_len: int, n_global: int,
                            attention_mask: Optional[torch.Tensor] = None,
                            num_buckets=32, max_distance=128, compute_dtype=torch.float32) -> torch.Tensor:
    """Literal blocked evaluation of T5BlockAttention's op (att.py:734-862), mask path.

    Keeps the reference's layout quirk: the additive mask is laid out
    [local Bl | side G] (att.py:722-732) while the keys are [side G | local Bl]
    (att.py:807-814), so in block 0 the last G key columns are disabled.
    """
    B, H, L, D = q.shape
    q, k, v = (t.to(compute_dtype) for t in (q, k, v))
    G, Bl = n_global, block_len
    if attention_mask is None:
        attention_mask = torch.ones(B, L)
    full_blocks = L // Bl >= 1                                                    # att.py:752
    ext = (1.0 - attention_mask.to(compute_dtype)[:, None, None, :]) * NEG_MASK   # att.py:694-707
    key_target = L + (-L % Bl) + G                                                # att.py:780
    bias_rows = Bl + G if full_blocks else L                                      # att.py:782
    if table is not None:
        pos_bias = _block_compute_bias(table.to(compute_dtype), bias_rows, key_target, num_buckets, max_distance)
    else:
        pos_bias = torch.zeros(1, H, bias_rows, key_target, dtype=compute_dtype)
    side_out = None
    if full_blocks:
        side_bias = pos_bias[:, :, :G, :L]                                        # att.py:680-683
        side_out = basic_attention(q[:, :, :G], k, v, side_bias)                  # att.py:795-800 (no mask)
    kb = split_into_blocks(k, Bl, 2)
    qb = split_into_blocks(q, Bl, 2)
    vb = split_into_blocks(v, Bl, 2)
    if full_blocks:
        nblk = kb.shape[1]
        sk = k[:, :, :G][:, None].expand(B, nblk, H, G, D)
        sv = v[:, :, :G][:, None].expand(B, nblk, H, G, D)
        kb = torch.cat([sk, kb], dim=3)                                           # att.py:813
        vb = torch.cat([sv, vb], dim=3)
        side_length = G
        block_bias = pos_bias[:, :, G:, :Bl + G]                                  # att.py:688-689
    else:
        side_length = 0
        block_bias = pos_bias[:, :, :L, :L]                                       # att.py:691
    qb, kb, vb = _flatten_blocks(qb), _flatten_blocks(kb), _flatten_blocks(vb)
    # prepare_side_attention, att.py:722-732
    lm = split_into_blocks(ext, Bl, 3)                                            # (B,1,1,nb,Bl')
    if L // Bl >= 1:
        sm = torch.zeros(B, 1, 1, lm.shape[3], G, dtype=compute_dtype)
        sm[:, :, :, 0, :] = NEG_MASK
        lm = torch.cat([lm, sm], dim=-1)
    lm = lm.squeeze(1).squeeze(1)[:, :, None, None, :]                            # (B,nb,1,1,Bl+G)
    bias = _flatten_blocks(lm + block_bias)                                       # att.py:830, :839
    o = basic_attention(qb, kb, vb, bias)
    out = _unblock(o, B, L).clone()
    if full_blocks:
        out[:, :, :G] = side_out                                                  # att.py:852-853
    return out


def _block_compute_bias(table, query_length, key_length, nb, md, side_length=0):
    """att.py:659-678 with its default side_length=0 (the only way forward() calls it, att.py:791)."""
    side = torch.arange(side_length, dtype=torch.long)
    ctx = torch.arange(side_length, query_length + side_length, dtype=torch.long)[:, None]
    mem = torch.cat([torch.arange(side_length, key_length, dtype=torch.long), side])[None, :]
    b = relative_position_bucket(mem - ctx, True, nb, md)
    return table[b].permute(2, 0, 1).unsqueeze(0)


# --------------------------------------------------------------------------
# a11  transient-global                               att.py:865-1065, utils.py:191-258
# --------------------------------------------------------------------------
def make_global_fixed_block_ids(attention_mask: torch.Tensor, gbs: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """(B,L) 0/1 float mask -> (block id per token, -1 for padding; 0/1 validity per side token)
    (utils.py:191-237)."""
    B, L = attention_mask.shape[:2]
    am = attention_mask.to(torch.float32)
    frac = torch.ones_like(am) / gbs
    frac = torch.cumsum(frac, dim=1) - frac
    keep = torch.where(am != 0.0, 1.0, -1000.0)
    ids = torch.floor(keep + frac - 1.0)
    ids = torch.where(ids > -1.0, ids, torch.tensor(-1.0))
    ids = ids * am + (am - 1)
    # orphan tokens join the last full block (utils.py:206-212)
    ends = (torch.arange(L) % gbs) == gbs - 1
    full = torch.logical_and(ends, ids >= 0).sum(-1).unsqueeze(-1).to(ids.dtype) - 1
    ids = torch.where(ids < full, ids, full)
    ng = L // gbs
    if ng > 0:
        idmax = ids.max(dim=-1).values[:, None].expand(B, ng)
    else:
        idmax = torch.zeros(B, 0, dtype=ids.dtype)
    seg = torch.cumsum(torch.ones(B, ng), dim=-1) - 1
    seg = torch.where(seg <= idmax, 1, 0)
    return ids.to(torch.int), seg.to(torch.int)


def create_global_aggregates(hidden: torch.Tensor, block_ids: torch.Tensor, ng: int) -> torch.Tensor:
    """Per-block sums of hidden states, (B,ng,d) (utils.py:249-258)."""
    ids = torch.where(block_ids >= 0, block_ids, torch.tensor(ng, dtype=block_ids.dtype))
    one_hot = F.one_hot(ids.to(torch.int64), ng + 1)[:, :, :-1]
    return torch.einsum("...nd,...ng->...gd", hidden, one_hot.to(hidden.dtype))


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """T5LayerNorm, no mean subtraction, no bias (modules.py:52-60)."""
    var = x.to(torch.float32).pow(2).mean(-1, keepdim=True)
    y = x * torch.rsqrt(var + eps)
    if weight.dtype in (torch.float16, torch.bfloat16):
        y = y.to(weight.dtype)
    return weight * y


def tglobal_side_bias(table, attention_mask, seg_ids, block_ids, bidirectional, nb, md):
    """(B,H,L,Gn): bucket(g - block_id(i)) through the LOCAL table + 0/-1e10 where
    mask[i] != segment_id[g] (att.py:905-925; the local table at :918-919)."""
    eq = torch.eq(attention_mask[..., None], seg_ids[:, None, :])[:, None]
    add = torch.where(eq > 0, 0.0, NEG_MASK)
    gpos = torch.arange(seg_ids.shape[-1])
    rel = (gpos - block_ids[..., None]).to(torch.int64)                           # utils.py:240-247
    b = relative_position_bucket(rel, bidirectional, nb, md)
    return add + table[b].permute(0, 3, 1, 2)


def tglobal_attention_blocked(q, k, v, side_k, side_v, table, block_len: int, gbs: int,
                              attention_mask: Optional[torch.Tensor] = None,
                              num_buckets=32, max_distance=128, compute_dtype=torch.float32) -> torch.Tensor:
    """Literal blocked evaluation of T5TransientGlobalAttention's op (att.py:977-1052), mask path.

    q,k,v (B,H,L,D); side_k, side_v (B,H,Gn,D) with Gn = L // gbs, already
    projected from the normalised block sums (att.py:959-974).  Returns the
    head-correct (B,H,L,D) output (the module's missing head transpose,
    att.py:951-953, sits outside the op).
    """
    B, H, L, D = q.shape
    q, k, v, side_k, side_v = (t.to(compute_dtype) for t in (q, k, v, side_k, side_v))
    if attention_mask is None:
        attention_mask = torch.ones(B, L)
    block_ids, seg_ids = make_global_fixed_block_ids(attention_mask, gbs)
    qb = split_into_blocks(q, block_len, 2)
    kb = concatenate_3_blocks(split_into_blocks(k, block_len, 2), 1, 3)
    vb = concatenate_3_blocks(split_into_blocks(v, block_len, 2), 1, 3)
    nblk = kb.shape[1]
    Gn = side_k.shape[2]
    kb = torch.cat([kb, side_k[:, None].expand(B, nblk, H, Gn, D)], dim=3)         # att.py:989-995
    vb = torch.cat([vb, side_v[:, None].expand(B, nblk, H, Gn, D)], dim=3)
    qb, kb, vb = _flatten_blocks(qb), _flatten_blocks(kb), _flatten_blocks(vb)
    bl = qb.shape[2]
    lm = torch.where(local_attention_mask(attention_mask, block_len) > 0, 0.0, NEG_MASK).to(compute_dtype)
    if table is not None:
        tb = table.to(compute_dtype)
        bias = local_block_bias(tb, bl, True, num_buckets, max_distance) + lm     # (B,nb,H,Bl,3Bl)
        side = tglobal_side_bias(tb, attention_mask, seg_ids, block_ids, True, num_buckets, max_distance)
    else:
        bias = torch.zeros(1, 1, H, bl, 3 * bl, dtype=compute_dtype) + lm
        side = tglobal_side_bias(torch.zeros(num_buckets, H, dtype=compute_dtype), attention_mask, seg_ids,
                                 block_ids, True, num_buckets, max_distance)
    side = split_into_blocks(side.to(compute_dtype), bl, -2)                       # (B,nb,H,Bl,Gn)
    bias = _flatten_blocks(torch.cat([bias.expand(B, nblk, H, bl, 3 * bl), side], dim=-1))
    return _unblock(basic_attention(qb, kb, vb, bias), B, L)


def tglobal_side_inputs(hidden: torch.Tensor, attention_mask: Optional[torch.Tensor], gbs: int,
                        norm_weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """RMSNorm(block sums of hidden) -> (B, L//gbs, d_model) (att.py:959-966)."""
    B, L = hidden.shape[:2]
    if attention_mask is None:
        attention_mask = torch.ones(B, L)
    block_ids, seg_ids = make_global_fixed_block_ids(attention_mask, gbs)
    agg = create_global_aggregates(hidden, block_ids, seg_ids.shape[-1])
    return rms_norm(agg, norm_weight, eps)


# --------------------------------------------------------------------------
# a13  split-K merge                                          decoding.py:47-55
# --------------------------------------------------------------------------
def splitk_merge(so: torch.Tensor, l: torch.Tensor, ml: torch.Tensor) -> torch.Tensor:
    """so (B,H,S,M,D) per-split normalised outputs, l (B,H,S,M) per-split sum of exp,
    ml (B,H,S,M) per-split max -> (B,H,M,D) (decoding.py:47-55, kept for any M)."""
    a_max = ml.max(dim=2, keepdim=True).values
    alpha = torch.exp(ml - a_max)
    w = torch.softmax(torch.log(alpha * l), dim=2)
    return (w.unsqueeze(-1) * so).sum(dim=2)


def splitk_partials(q, k, v, num_splits: int, sm_scale: float = 1.0, bias: Optional[torch.Tensor] = None):
    """What the split kernel writes (decoding.py:78-80, :172-178): split s covers keys
    [s*(N//S), (s+1)*(N//S)), the last split takes the remainder."""
    B, H, M, D = q.shape
    N = k.shape[2]
    per = N // num_splits
    so = torch.zeros(B, H, num_splits, M, D)
    l = torch.zeros(B, H, num_splits, M)
    ml = torch.full((B, H, num_splits, M), float("-inf"))
    for s in range(num_splits):
        lo = s * per
        hi = N if s == num_splits - 1 else lo + per
        if hi <= lo:
            continue
        sc = torch.einsum("bhqd,bhkd->bhqk", q.float() * sm_scale, k[:, :, lo:hi].float())
        if bias is not None:
            sc = sc + bias[..., lo:hi].float()
        mx = sc.max(dim=-1).values
        p = torch.exp(sc - mx[..., None])
        l[:, :, s] = p.sum(-1)
        ml[:, :, s] = mx
        so[:, :, s] = torch.einsum("bhqk,bhkd->bhqd", p, v[:, :, lo:hi].float()) / l[:, :, s][..., None]
    return so, l, ml
