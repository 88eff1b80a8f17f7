"""Unpad / pad glue either side of the packed (cu_seqlens) kernel.

Same contract as the reference's src/turbot5/model/padding.py (:79-150, :30-44):
valid tokens of a (B, L) 0/1 mask are gathered into one packed (total, ...)
tensor, the kernel runs on it, and the result is scattered back into zeros.
The only host synchronisation is the size of ``nonzero``; the maximum length
handed to the kernel is the padded length (an upper bound is all it needs),
so there is no ``.item()`` per call.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def _get_unpad_data(attention_mask: torch.Tensor):
    """(B,L) 0/1 mask -> (flat indices of the valid tokens, cu_seqlens int32 (B+1,), upper bound of the
    longest sequence) (padding.py:79-88)."""
    seqlens_in_batch = attention_mask.sum(dim=-1, dtype=torch.int32)
    indices = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
    cu_seqlens = F.pad(torch.cumsum(seqlens_in_batch, dim=0, dtype=torch.int32), (1, 0))
    return indices, cu_seqlens, attention_mask.shape[-1]


def index_first_axis(x: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """Rows ``indices`` of x along dim 0 (padding.py:5-27, forward only)."""
    return x.index_select(0, indices)


def unpad_input(hidden_states: torch.Tensor, attention_mask: torch.Tensor):
    """(B,L,...) -> (total, ...) of the valid tokens plus the unpad metadata (padding.py:90-111)."""
    indices, cu_seqlens, max_len = _get_unpad_data(attention_mask)
    flat = hidden_states.reshape(-1, *hidden_states.shape[2:])
    return index_first_axis(flat, indices), indices, cu_seqlens, max_len


def _upad_input(query_layer, key_layer, value_layer, attention_mask, query_length, NH, unpad_data=None):
    """Packed q, k, v for the varlen kernel (padding.py:113-150).  Inputs are (B,L,H,D)."""
    indices_k, cu_seqlens_k, max_k = unpad_data if unpad_data is not None else _get_unpad_data(attention_mask)
    batch_size, kv_seq_len, num_kv_heads, head_dim = key_layer.shape
    key_layer = index_first_axis(key_layer.reshape(batch_size * kv_seq_len, num_kv_heads, head_dim), indices_k)
    value_layer = index_first_axis(value_layer.reshape(batch_size * kv_seq_len, num_kv_heads, head_dim), indices_k)
    if query_length == kv_seq_len:
        query_layer = index_first_axis(query_layer.reshape(batch_size * kv_seq_len, NH, head_dim), indices_k)
        cu_seqlens_q, max_q, indices_q = cu_seqlens_k, max_k, indices_k
    elif query_length == 1:
        max_q = 1
        cu_seqlens_q = torch.arange(batch_size + 1, dtype=torch.int32, device=query_layer.device)
        indices_q = cu_seqlens_q[:-1]
        query_layer = query_layer.squeeze(1)
    else:
        # the -query_length: slice assumes left padding, as the reference does
        attention_mask = attention_mask[:, -query_length:]
        query_layer, indices_q, cu_seqlens_q, max_q = unpad_input(query_layer, attention_mask)
    return query_layer, key_layer, value_layer, indices_q, (cu_seqlens_q, cu_seqlens_k), (max_q, max_k)


def pad_input(hidden_states: torch.Tensor, indices: torch.Tensor, batch: int, seqlen: int) -> torch.Tensor:
    """(total, ...) -> (B, L, ...) with zeros at the padded positions (padding.py:30-44, :47-76)."""
    out = torch.zeros(batch * seqlen, *hidden_states.shape[1:], device=hidden_states.device,
                      dtype=hidden_states.dtype)
    out.index_copy_(0, indices, hidden_states)
    return out.view(batch, seqlen, *hidden_states.shape[1:])
