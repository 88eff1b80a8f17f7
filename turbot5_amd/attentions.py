"""Attention modules of the T5 encoder/decoder, drop-in for the reference's plugin classes.

``T5ATTENTION_TYPES[config.attention_type](config, has_relative_attention_bias=...)`` builds the
self-attention of an encoder layer exactly as the reference does
(src/turbot5/model/modeling.py:54-61, :137).  Constructor and ``forward`` signatures, the
returned tuple ``(attn_output, present_key_value, position_bias[, attn_weights])`` and the
parameter names (``q k v o relative_attention_bias``, plus ``global_relative_attention_bias``
and ``global_input_layer_norm`` for transient-global) are the reference's
(src/turbot5/model/attentions.py:387-521, :523-649, :652-862, :865-1065), so HuggingFace T5 /
LongT5 state dicts load unchanged.  The attention itself always runs in the HIP kernels of
libt5attn.so; there is no torch fallback in this package.

Differences from the reference, all on purpose:
* every module hands the (num_buckets, H) TABLE on as ``position_bias`` (the reference does so
  for 'flash' only; the sparse modules materialise a bias tensor), and never builds an L x L bias;
* the sparse modules take attention masks whose rows are one run of valid tokens (all ones, right padding,
  and for local / transient-global also left padding); masks with holes raise ``NotImplementedError``;
* transient-global returns the head-correct layout (the reference's ``unshape`` omits the
  head transpose, attentions.py:951-953);
* ``layer_head_mask`` is not available on fused paths; ``output_attentions=True`` adds a fourth element None to the
  returned tuple, as the reference's fused modules do (attentions.py:483, :519-520, :647, :860, :1063).
"""
from __future__ import annotations

import warnings
import weakref
from collections import OrderedDict
from typing import Optional

import torch
from torch import nn

from . import ops
from .config import T5Config
from .padding import _get_unpad_data, _upad_input, index_first_axis, pad_input


class T5LayerNorm(nn.Module):
    """RMS norm without mean subtraction or bias (reference src/turbot5/model/modules.py:24-67)."""

    def __init__(self, dim: int, eps: float = 1e-6, use_triton: bool = False):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor, group: int = 1, seq_lens: Optional[torch.Tensor] = None,
                seq_starts: Optional[torch.Tensor] = None, key_bits: Optional[torch.Tensor] = None,
                group_counts: Optional[torch.Tensor] = None) -> torch.Tensor:
        """On a ROCm device: the fused HIP kernel (the reference switches to its Triton kernel there,
        modules.py:61-66).  Host tensors take the reference's eager formula (modules.py:51-59).
        ``group`` > 1 norms the sums of ``group`` consecutive rows of each sequence (side tokens)."""
        # (the kernel has no backward: a module in training mode that is being differentiated takes the eager formula)
        differentiated = self.training and torch.is_grad_enabled() and (x.requires_grad or self.weight.requires_grad)
        if x.is_cuda and not (differentiated and seq_lens is None and key_bits is None):
            from .ops import rms_norm
            return rms_norm(x, self.weight, self.eps, group, seq_lens=seq_lens, seq_starts=seq_starts,
                            key_bits=key_bits, group_counts=group_counts)
        if group > 1:
            B, L, d = x.shape
            n = L // group
            agg = x[:, :n * group].reshape(B, n, group, d).sum(dim=2)
            if L > n * group and n > 0:
                agg = torch.cat([agg[:, :-1], agg[:, -1:] + x[:, n * group:].sum(dim=1, keepdim=True)], dim=1)
            x = agg
        variance = x.to(torch.float32).pow(2).mean(-1, keepdim=True)
        x = x * torch.rsqrt(variance + self.eps)
        if self.weight.dtype in (torch.float16, torch.bfloat16):
            x = x.to(self.weight.dtype)
        return self.weight * x

    def add_norm(self, x: torch.Tensor, residual: Optional[torch.Tensor]):
        """``(x + residual, norm(x + residual))``: the residual add that closes one sub-layer and the norm
        that opens the next (reference src/turbot5/model/modeling.py:159-161, :113-114), one kernel on a
        ROCm device.  ``residual`` None: ``(x, norm(x))``."""
        if residual is None:
            return x, self.forward(x)
        differentiated = torch.is_grad_enabled() and (x.requires_grad or residual.requires_grad or
                                                      (self.training and self.weight.requires_grad))
        if x.is_cuda and residual.dtype == x.dtype and not differentiated:
            from .ops import rms_norm
            return rms_norm(x, self.weight, self.eps, 1, residual)
        total = x + residual
        return total, self.forward(total)


# ---------------------------------------------------------------------------------------------
# One host synchronisation per distinct mask tensor (not per layer): is it all ones, and if not,
# where are the valid tokens.  The reference asks the same question in every layer
# (attentions.py:410-418) and again inside the unpad helper (padding.py:82).
_MASK_INFO: "OrderedDict[tuple, tuple]" = OrderedDict()


def _mask_info(mask: torch.Tensor):
    # The entry remembers WHICH tensor it describes (weakly): a later mask that happens to get the freed
    # tensor's address, shape and version must not inherit its lengths.
    key = (mask.data_ptr(), mask._version, tuple(mask.shape), str(mask.device), mask.dtype)
    hit = _MASK_INFO.get(key)
    if hit is not None and hit[0]() is mask:
        return hit[1], hit[2]
    if mask.dim() != 2:
        raise ValueError(f"attention mask must be (batch, key_length) of 0/1, got shape {tuple(mask.shape)}")
    valid = mask != 0
    lens = valid.sum(-1, dtype=torch.int32)
    steps = torch.arange(mask.shape[1], device=mask.device)
    first = valid.to(torch.int8).argmax(-1)   # first valid token of a row (0 for an empty row)
    # one transfer for both questions: all ones?  every row ONE run of ones (padding left, right or both)?
    all_ones, one_run, from_zero = (bool(x) for x in torch.stack(
        [valid.all(), (valid == ((steps[None, :] >= first[:, None]) &
                                 (steps[None, :] < (first + lens)[:, None]))).all(),
         (first == 0).all()]).tolist())
    unpad = None
    if not all_ones:
        # batches whose rows are one run of valid tokens run in place, with a start row and a length per
        # sequence; anything else (holes) is packed first.  The last element collects the launch plans of
        # this batch, one per kind of attention call, so that the layers of a stack build each only once.
        if one_run:
            B, L = mask.shape
            cu = torch.arange(0, (B + 1) * L, L, dtype=torch.int32, device=mask.device)
            cu[:B] += first.to(torch.int32)
            unpad = ("lens", (lens, cu), {"right_padded": from_zero})
        else:
            unpad = ("packed", _get_unpad_data(valid.to(torch.int32)), {})
    _MASK_INFO[key] = (weakref.ref(mask), all_ones, unpad)
    _MASK_INFO.move_to_end(key)
    while len(_MASK_INFO) > 16:
        _MASK_INFO.popitem(last=False)
    return all_ones, unpad


class PackedBatch:
    """The valid tokens of a padded (B, L) batch laid back to back: what a whole layer stack needs to run
    on ``total`` rows instead of ``B * L`` (the reference packs and pads around every attention call,
    attentions.py:492-511, and runs everything else on the padded rows)."""
    __slots__ = ("indices", "cu_seqlens", "max_len", "batch", "length", "plans")

    def __init__(self, indices, cu_seqlens, max_len, batch, length, plans):
        self.indices, self.cu_seqlens, self.max_len = indices, cu_seqlens, max_len
        self.batch, self.length, self.plans = batch, length, plans


def packed_batch(mask: torch.Tensor) -> Optional[PackedBatch]:
    """None for an all-ones mask; otherwise the packed layout of its valid tokens, remembered with the
    mask (one more host synchronisation per distinct mask tensor: the number of valid tokens)."""
    all_ones, unpad = _mask_info(mask)
    if all_ones:
        return None
    kind, data, plans = unpad
    hit = plans.get("packed_batch")
    if hit is None:
        indices, cu, max_len = data if kind == "packed" else _get_unpad_data((mask != 0).to(torch.int32))
        hit = plans["packed_batch"] = PackedBatch(indices, cu, max_len, mask.shape[0], mask.shape[1], {})
    return hit


class _T5AttentionBase(nn.Module):
    """Parameters and shape helpers shared by the attention modules (attentions.py:36-66)."""

    def __init__(self, config: T5Config, has_relative_attention_bias: bool = False):
        super().__init__()
        self.config = config
        self.is_decoder = config.is_decoder
        self.has_relative_attention_bias = has_relative_attention_bias
        self.relative_attention_num_buckets = config.relative_attention_num_buckets
        self.relative_attention_max_distance = config.relative_attention_max_distance
        self.d_model = config.d_model
        self.key_value_proj_dim = config.d_kv
        self.n_heads = config.num_heads
        self.dropout = config.dropout_rate
        self.inner_dim = self.n_heads * self.key_value_proj_dim
        self.q = nn.Linear(self.d_model, self.inner_dim, bias=False)
        self.k = nn.Linear(self.d_model, self.inner_dim, bias=False)
        self.v = nn.Linear(self.d_model, self.inner_dim, bias=False)
        self.o = nn.Linear(self.inner_dim, self.d_model, bias=False)
        if self.has_relative_attention_bias:
            self.relative_attention_bias = nn.Embedding(self.relative_attention_num_buckets, self.n_heads)
        self.pruned_heads = set()
        self.gradient_checkpointing = False

    # (B, L, H*D) -> strided (B, H, L, D) view; the kernels take the strides as they are
    def _shape(self, states: torch.Tensor, batch_size: int) -> torch.Tensor:
        return states.view(batch_size, -1, self.n_heads, self.key_value_proj_dim).transpose(1, 2)

    def _unshape(self, states: torch.Tensor, batch_size: int) -> torch.Tensor:
        return states.transpose(1, 2).contiguous().view(batch_size, -1, self.inner_dim)

    def _attn_dtype(self, x: torch.Tensor) -> torch.dtype:
        return self.config.attention_dtype or x.dtype

    def _query(self, hidden_states: torch.Tensor, adt: torch.dtype):
        """-> (query rows (..., H*D) in the attention dtype, the ``exact_scores`` argument that goes with them).

        16-bit attention, ``config.attention_exact_scores`` None: log2(e) is folded into the projection
        (``ops.prescaled_query``), so the rows are rounded to the attention dtype once and the kernel applies no
        factor to them -- the reference applies its factor to the fp32 product (fused_bias_attention.py:323-337);
        this gives the same accuracy without the multiply per score.  True / False: plain projection, the
        kernel scales the fp32 product / multiplies and re-rounds the rows."""
        choice = getattr(self.config, "attention_exact_scores", None)
        if choice is None and adt in (torch.bfloat16, torch.float16) and hidden_states.is_cuda:
            return ops.prescaled_query(hidden_states, self.q.weight, adt, 1.0), "prescaled"
        return self.q(hidden_states).to(adt), choice

    def _table(self, position_bias):
        if position_bias is None and self.has_relative_attention_bias:
            position_bias = self.relative_attention_bias.weight
        if position_bias is not None and position_bias.dim() != 2:
            raise ValueError("position_bias must be the (num_buckets, n_heads) table handed on by the first "
                             f"layer, got shape {tuple(position_bias.shape)}")
        return position_bias

    @staticmethod
    def _reject(layer_head_mask, output_attentions):
        """``output_attentions=True`` is accepted as in the reference's fused modules, whose fourth tuple element is
        then None (attentions.py:483, :519-520, :647, :860, :1063): the weights are never materialised."""
        if layer_head_mask is not None:
            raise NotImplementedError("layer_head_mask is not supported by the fused attention kernels")

    @staticmethod
    def _outputs(attn_output, present_key_value, table, output_attentions):
        outputs = (attn_output, present_key_value, table)
        return outputs + (None,) if output_attentions else outputs


class T5FlashAttention(_T5AttentionBase):
    """Full attention with the bias fused into the kernel (reference attentions.py:387-521).

    Encoder self-attention (bidirectional buckets), decoder self-attention (``config.is_decoder``:
    causal mask + unidirectional buckets, KV cache through ``past_key_value``) and cross-attention
    (``cross_attention=True``: no causal mask; no bias unless a table is passed).
    """

    def __init__(self, config: T5Config, cross_attention: bool = False, *args, **kwargs) -> None:
        super().__init__(config, *args, **kwargs)
        self.causal = config.is_decoder and not cross_attention

    def forward(self, hidden_states, mask=None, key_value_states=None, position_bias=None, past_key_value=None,
                layer_head_mask=None, query_length=None, use_cache=False, output_attentions=False):
        self._reject(layer_head_mask, output_attentions)
        batch_size, seq_length = hidden_states.shape[:2]
        varlen, unpad = False, None
        if mask is not None:
            all_ones, unpad = _mask_info(mask)
            varlen = not all_ones

        if past_key_value is not None and len(past_key_value) != 2:
            raise ValueError(
                f"past_key_value should have 2 past states: keys and values. Got { len(past_key_value)} past states")
        adt = self._attn_dtype(hidden_states)

        # A padded memory (cross-attention without cached keys): its k and v projections run on the valid rows
        # only and are scattered into zeros; the padding rows are never attended.
        memory_rows, memory_layout = None, None
        if (key_value_states is not None and varlen and key_value_states.is_cuda
                and (past_key_value is None or past_key_value[0].shape[2] != key_value_states.shape[1])):
            layout = packed_batch(mask)
            n_rows = key_value_states.shape[0] * key_value_states.shape[1]
            if layout is not None and 0 < layout.indices.numel() <= 0.85 * n_rows and mask.shape[1] == key_value_states.shape[1]:
                memory_layout = layout
                memory_rows = index_first_axis(key_value_states.reshape(n_rows, -1), layout.indices)

        def project(proj_layer, past):
            """keys or values: (B, H, key_length, D) in the attention dtype (attentions.py:444-469)."""
            if key_value_states is None:
                states = self._shape(proj_layer(hidden_states), batch_size).to(adt)
                if past is not None:
                    states = torch.cat([past, states], dim=2)
                return states
            if past is None or past.shape[2] != key_value_states.shape[1]:
                if memory_rows is not None:
                    padded = pad_input(proj_layer(memory_rows).to(adt), memory_layout.indices,
                                       memory_layout.batch, memory_layout.length)
                    return self._shape(padded, batch_size)
                return self._shape(proj_layer(key_value_states), batch_size).to(adt)
            return past

        query_rows, exact = self._query(hidden_states, adt)
        query_states = self._shape(query_rows, batch_size)
        # (the split-K kernel scales the fp32 product: rows that carry log2(e) already get ln 2 as their scale)
        dec_scale = 1.0 / ops.LOG2E if exact == "prescaled" else 1.0
        key_states = project(self.k, past_key_value[0] if past_key_value is not None else None)
        value_states = project(self.v, past_key_value[1] if past_key_value is not None else None)
        table = self._table(position_bias)
        nb, md = self.relative_attention_num_buckets, self.relative_attention_max_distance
        key_length = key_states.shape[2]

        if not varlen:
            if table is None and not self.causal and seq_length <= 8 and key_length >= 512:
                # few query rows over a long memory (incremental decoding): split-K kernel
                attn_output = ops.flash_decoding_attention(query_states, key_states, value_states, None, dec_scale)
            else:
                attn_output = ops.flash_attention_with_fusing_bias(
                    query_states, key_states, value_states, table, causal=self.causal, sm_scale=1.0, exact_scores=exact,
                    NUM_BUCKETS=nb, MAX_DISTANCE=md)
        else:
            if mask.shape[1] != key_length:
                raise ValueError(f"mask covers {mask.shape[1]} keys but there are {key_length}")
            q_blhd = query_states.transpose(1, 2)
            k_blhd = key_states.transpose(1, 2)
            v_blhd = value_states.transpose(1, 2)
            kind, unpad, plans = unpad
            dev = hidden_states.device
            # self-attention over the batch: cu_seqlens come from the per-mask cache, so the layers can share
            # one plan; other calls make their cu_q on the spot and plan per call
            plan = True
            if key_value_states is None and seq_length == key_length:
                plan = plans.setdefault((self.causal, self.n_heads, self.key_value_proj_dim, adt, seq_length,
                                         ops._stream(hidden_states)), ops.LaunchPlan())   # one per stream
            if kind == "lens" and table is None and not self.causal and seq_length <= 8 and key_length >= 512:
                # few query rows over long padded memories (incremental decoding): the split-K kernel with
                # each memory's first key and key count
                lens_k, cu_k = unpad
                starts = plans.get("key_starts")
                if starts is None:
                    starts = plans["key_starts"] = (cu_k[:batch_size] - torch.arange(
                        batch_size, device=dev, dtype=torch.int32) * key_length).contiguous()
                attn_output = ops.flash_decoding_attention(query_states, key_states, value_states, None, dec_scale,
                                                           key_lens=lens_k, key_starts=starts)
                kind = "done"
            elif kind == "lens":
                # rows padded on either side: the kernel walks the padded (B*L, H, D) layout with a start row
                # and a length per sequence; nothing is gathered or scattered (the reference unpads and pads, attentions.py:492-511)
                def rows(t, n):
                    t = t if t.is_contiguous() else t.contiguous()
                    return t.view(batch_size * n, self.n_heads, -1)
                unpad, cu_k = unpad
                self_attn = key_value_states is None and seq_length == key_length
                cu_q = cu_k if self_attn else torch.arange(0, (batch_size + 1) * seq_length, seq_length,
                                                           dtype=torch.int32, device=dev)
                out_p = ops.flash_attention_with_fusing_bias_varlen(
                    rows(q_blhd, seq_length), rows(k_blhd, key_length), rows(v_blhd, key_length), table, cu_q, cu_k,
                    seq_length, key_length, causal=self.causal, sm_scale=1.0, exact_scores=exact, NUM_BUCKETS=nb, MAX_DISTANCE=md,
                    seq_lens_q=unpad if self_attn else None, seq_lens_k=unpad,
                    launch_plan=plan)
                attn_output = out_p.view(batch_size, seq_length, self.n_heads, -1).transpose(1, 2)
            elif key_value_states is None and seq_length == key_length:
                q_p, k_p, v_p, indices_q, (cu_q, cu_k), (max_q, max_k) = _upad_input(
                    q_blhd, k_blhd, v_blhd, mask, seq_length, self.n_heads, unpad_data=unpad)
            else:
                # queries are all valid; only the keys carry padding (cross-attention, cached decoding)
                indices_k, cu_k, max_k = unpad
                k_p = index_first_axis(k_blhd.reshape(batch_size * key_length, self.n_heads, -1), indices_k)
                v_p = index_first_axis(v_blhd.reshape(batch_size * key_length, self.n_heads, -1), indices_k)
                q_p = q_blhd.reshape(batch_size * seq_length, self.n_heads, -1)
                cu_q = torch.arange(0, (batch_size + 1) * seq_length, seq_length, dtype=torch.int32,
                                    device=hidden_states.device)
                indices_q, max_q = None, seq_length
            if kind not in ("lens", "done"):
                out_p = ops.flash_attention_with_fusing_bias_varlen(
                    q_p, k_p, v_p, table, cu_q, cu_k, max_q, max_k, causal=self.causal, sm_scale=1.0, exact_scores=exact,
                    NUM_BUCKETS=nb, MAX_DISTANCE=md, launch_plan=plan)
                if indices_q is not None:
                    attn_output = pad_input(out_p, indices_q, batch_size, seq_length).transpose(1, 2)
                else:
                    attn_output = out_p.view(batch_size, seq_length, self.n_heads, -1).transpose(1, 2)

        attn_output = self.o(self._unshape(attn_output, batch_size).to(hidden_states.dtype))
        present_key_value_state = (key_states, value_states) if (self.is_decoder and use_cache) else None
        return self._outputs(attn_output, present_key_value_state, table, output_attentions)

    def forward_packed(self, hidden_states, packed: PackedBatch, position_bias=None):
        """Self-attention over hidden states that are already packed: (total, d_model), sequences back to
        back as ``packed.cu_seqlens`` says.  No gather, no scatter; positions count the tokens of a
        sequence, as in the reference's packed call (varlen_fused_bias_attn.py:254, :303)."""
        total = hidden_states.shape[0]
        adt = self._attn_dtype(hidden_states)
        q, exact = self._query(hidden_states, adt)
        q = q.view(total, self.n_heads, self.key_value_proj_dim)
        k, v = (p(hidden_states).view(total, self.n_heads, self.key_value_proj_dim).to(adt) for p in (self.k, self.v))
        table = self._table(position_bias)
        plan = packed.plans.setdefault((self.causal, self.n_heads, self.key_value_proj_dim, adt,
                                        ops._stream(hidden_states)), ops.LaunchPlan())
        out = ops.flash_attention_with_fusing_bias_varlen(
            q, k, v, table, packed.cu_seqlens, packed.cu_seqlens, packed.max_len, packed.max_len,
            causal=self.causal, sm_scale=1.0, exact_scores=exact, NUM_BUCKETS=self.relative_attention_num_buckets,
            MAX_DISTANCE=self.relative_attention_max_distance, launch_plan=plan)
        return (self.o(out.reshape(total, self.inner_dim).to(hidden_states.dtype)), None, table)


class _SparseBase(_T5AttentionBase):
    def _key_bits(self, mask, block_len, aux=0):
        """Validity bit sets of a mask of any shape (ops.pack_key_bits), kept with the mask's other derived data."""
        _, unpad = _mask_info(mask)
        plans = unpad[2]
        key = ("key_bits", int(block_len), int(aux))
        bits = plans.get(key)
        if bits is None:
            bits = plans[key] = ops.pack_key_bits(mask, block_len, aux)
        return bits

    def _check_call(self, mask, layer_head_mask, past_key_value, use_cache, output_attentions, left_padding_ok=True):
        """-> (lengths, first rows): (B,) int32 device tensors for a batch whose rows are each ONE run of valid
        tokens (padding on the right, and on the left where the pattern takes it); (None, None) for all ones.
        First rows are None for right padding.  Any other mask gives ("bits", None): the caller passes validity
        bit sets instead."""
        if past_key_value is not None:
            warnings.warn('Currently, passing past key value states is not supported.')
        if use_cache is not None:
            warnings.warn('Currently, using cache is not supported for chosen attention type.')
        self._reject(layer_head_mask, output_attentions)
        if mask is not None:
            all_ones, unpad = _mask_info(mask)
            if not all_ones:
                if unpad[0] == "lens":
                    plans = unpad[2]
                    if plans.get("right_padded"):
                        return unpad[1][0], None
                    if left_padding_ok:
                        starts = plans.get("starts")
                        if starts is None:   # first row of each sequence, from the start rows of the flat (B*L) layout
                            B, L = mask.shape
                            starts = plans["starts"] = (unpad[1][1][:B] - torch.arange(
                                B, device=mask.device, dtype=torch.int32) * L).contiguous()
                        return unpad[1][0], starts
                return "bits", None
        return None, None

    def _qkv(self, hidden_states):
        """-> q, k, v as (B, H, L, D) views in the attention dtype and the ``exact_scores`` argument for q"""
        batch_size = hidden_states.shape[0]
        adt = self._attn_dtype(hidden_states)
        q, exact = self._query(hidden_states, adt)
        k, v = (self._shape(p(hidden_states), batch_size).to(adt) for p in (self.k, self.v))
        return self._shape(q, batch_size), k, v, exact

    def _finish(self, attn_output, hidden_states, table, output_attentions=False):
        batch_size = hidden_states.shape[0]
        out = self.o(self._unshape(attn_output, batch_size).to(hidden_states.dtype))
        return self._outputs(out, None, table, output_attentions)


class T5LocalAttention(_SparseBase):
    """Sliding-window attention, |j - i| < sliding_window (reference attentions.py:523-649)."""

    def __init__(self, config: T5Config, *args, **kwargs) -> None:
        super().__init__(config, *args, **kwargs)
        self.block_len = config.sliding_window

    def forward(self, hidden_states, mask=None, position_bias=None, layer_head_mask=None, past_key_value=None,
                use_cache=None, output_attentions=False):
        # right-padded batches: the keys of a sequence end at its length (the key half of the reference's
        # local mask, utils.py:174-188); outputs at padded positions mean nothing, as in the reference
        seq_lens, seq_starts = self._check_call(mask, layer_head_mask, past_key_value, use_cache, output_attentions)
        q, k, v, exact = self._qkv(hidden_states)
        table = self._table(position_bias)
        # a sequence shorter than one block is a single block of its own length (utils.py:107-108)
        block_len = min(self.block_len, hidden_states.shape[1])
        key_bits = None
        if isinstance(seq_lens, str):   # a mask with holes: the keys' validity as bit sets
            seq_lens, key_bits = None, self._key_bits(mask, block_len)
        out = ops.local_attention_with_fusing_bias(
            q, k, v, table, block_len, 1.0, self.relative_attention_num_buckets,
            self.relative_attention_max_distance, seq_lens=seq_lens, seq_starts=seq_starts,
            exact_scores=exact, key_bits=key_bits)
        return self._finish(out, hidden_states, table, output_attentions)


class T5BlockAttention(_SparseBase):
    """Own block plus ``global_block_size`` leading global tokens (reference attentions.py:652-862)."""

    def __init__(self, config: T5Config, *args, **kwargs) -> None:
        super().__init__(config, *args, **kwargs)
        self.block_len = config.sliding_window
        self.n_global_tokens = config.global_block_size

    def forward(self, hidden_states, mask=None, position_bias=None, layer_head_mask=None, past_key_value=None,
                use_cache=None, output_attentions=False):
        # right-padded batches: the reference's additive mask over its key list (attentions.py:722-732)
        # (left padding and holes: validity bit sets, looked up per tile)
        seq_lens, _ = self._check_call(mask, layer_head_mask, past_key_value, use_cache, output_attentions,
                                       left_padding_ok=False)
        q, k, v, exact = self._qkv(hidden_states)
        table = self._table(position_bias)
        key_bits = None
        seq_length = hidden_states.shape[1]
        if seq_lens is not None and seq_length < self.block_len:
            # A padded batch shorter than one block: the reference's single block of seq_length keys under the
            # additive key mask, bias of the row distance (attentions.py:752, :691, :722-732) -- full attention
            # over the valid keys with positions = row indices, which is the windowed kernel with a window that
            # spans the sequence.
            if isinstance(seq_lens, str):
                seq_lens, key_bits = None, self._key_bits(mask, seq_length)
            out = ops.local_attention_with_fusing_bias(
                q, k, v, table, seq_length, 1.0, self.relative_attention_num_buckets,
                self.relative_attention_max_distance, seq_lens=seq_lens, exact_scores=exact, key_bits=key_bits)
            return self._finish(out, hidden_states, table, output_attentions)
        if isinstance(seq_lens, str):
            seq_lens, key_bits = None, self._key_bits(mask, self.block_len, self.n_global_tokens)
        out = ops.block_attention_with_fusing_bias(
            q, k, v, table, self.block_len, self.n_global_tokens, 1.0, self.relative_attention_num_buckets,
            self.relative_attention_max_distance, exact_scores=exact, seq_lens=seq_lens, key_bits=key_bits)
        return self._finish(out, hidden_states, table, output_attentions)


class T5TransientGlobalAttention(_SparseBase):
    """Sliding window plus one side token per ``global_block_size`` tokens (reference attentions.py:865-1065)."""

    def __init__(self, config: T5Config, *args, **kwargs) -> None:
        super().__init__(config, *args, **kwargs)
        self.block_len = config.sliding_window
        self.global_block_size = config.global_block_size
        if self.has_relative_attention_bias:
            # kept for checkpoint compatibility; the reference reads the local table for the side
            # bias as well (attentions.py:918-919)
            self.global_relative_attention_bias = nn.Embedding(self.relative_attention_num_buckets, self.n_heads)
        self.global_input_layer_norm = T5LayerNorm(config.d_model, eps=config.layer_norm_epsilon)

    def side_inputs(self, hidden_states: torch.Tensor, seq_lens: Optional[torch.Tensor] = None,
                    seq_starts: Optional[torch.Tensor] = None, key_bits: Optional[torch.Tensor] = None,
                    side_counts: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Normalised block sums, (B, L // global_block_size, d_model); trailing tokens that do not fill
        a block join the last one (utils.py:206-212, :249-258; attentions.py:959-966).  With ``seq_lens``
        (or ``key_bits`` and ``side_counts``, for masks of any shape) each sequence counts its valid tokens only."""
        B, L, d = hidden_states.shape
        gbs = self.global_block_size
        n_side = L // gbs
        if n_side == 0:
            return hidden_states.new_zeros(B, 0, d)
        # block sums and norm in one kernel
        return self.global_input_layer_norm(hidden_states, group=gbs, seq_lens=seq_lens, seq_starts=seq_starts,
                                            key_bits=key_bits, group_counts=side_counts)

    def forward(self, hidden_states, mask=None, position_bias=None, layer_head_mask=None, past_key_value=None,
                use_cache=None, output_attentions=False):
        # right-padded batches: per-sequence key limit and side-token count in the kernels (utils.py:174-237)
        seq_lens, seq_starts = self._check_call(mask, layer_head_mask, past_key_value, use_cache, output_attentions)
        batch_size = hidden_states.shape[0]
        adt = self._attn_dtype(hidden_states)
        block_len = min(self.block_len, hidden_states.shape[1])
        key_bits = side_counts = None
        if isinstance(seq_lens, str):   # a mask with holes: validity bit sets and the side tokens of each sequence
            seq_lens = None
            key_bits = self._key_bits(mask, block_len, self.global_block_size)
            plans = _mask_info(mask)[1][2]
            side_counts = plans.get(("side_counts", self.global_block_size))
            if side_counts is None:
                side_counts = plans[("side_counts", self.global_block_size)] = ops.side_token_counts(mask, self.global_block_size)
        q, k, v, exact = self._qkv(hidden_states)
        side = self.side_inputs(hidden_states, seq_lens, seq_starts, key_bits, side_counts)
        side_k = self._shape(self.k(side), batch_size).to(adt)
        side_v = self._shape(self.v(side), batch_size).to(adt)
        table = self._table(position_bias)
        out = ops.transient_global_attention_with_fusing_bias(
            q, k, v, side_k, side_v, table, block_len, self.global_block_size, 1.0,
            self.relative_attention_num_buckets, self.relative_attention_max_distance, seq_lens=seq_lens,
            seq_starts=seq_starts, exact_scores=exact, key_bits=key_bits, side_counts=side_counts)
        return self._finish(out, hidden_states, table, output_attentions)


T5ATTENTION_TYPES = {
    # 'basic' is the reference's eager T5Attention (attentions.py:36-257): the same math as 'flash', which is what
    # runs here (no attention weights, head mask or attention dropout; those raise NotImplementedError)
    "basic": T5FlashAttention,
    "flash": T5FlashAttention,
    "triton-basic": T5FlashAttention,   # same math as 'flash'; the materialised-bias kernel is not rebuilt
    "local": T5LocalAttention,
    "block": T5BlockAttention,
    "transient-global": T5TransientGlobalAttention,
}
