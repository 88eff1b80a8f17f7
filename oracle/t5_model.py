"""CPU restatement of the reference's T5 layer stack with 'basic' attention (pure torch).

TEST INFRASTRUCTURE ONLY -- see ``oracle/__init__.py``.  Functional: works on a ``state_dict``
with HuggingFace T5 parameter names, so the same weights drive this oracle and the HIP-backed
stack.  Follows src/turbot5/model/modeling.py (:142-164 self-attention layer, :178-201
cross-attention layer, :104-128 feed-forward layer, :232-342 block, :421-632 stack incl. the
sharing of layer 0's position bias, :589) and src/turbot5/model/attentions.py:144-257
(T5Attention.forward, 'basic').  Masks use the standard T5 semantics (additive, broadcast over
heads and query rows); the reference's encoder hands 'basic' a raw 0/1 mask that only
broadcasts for batch 1 (modeling.py:490-491) -- identical for all-ones masks up to a
softmax-invariant constant.

Pinning: the dense-attention core is pinned in tests/test_oracle_dense.py; the stack is pinned
against the installed HuggingFace ``T5EncoderModel`` / ``T5ForConditionalGeneration``
(third-party) in tests/test_oracle_model.py.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch
import torch.nn.functional as F

from . import t5_basic as O

SD = Dict[str, torch.Tensor]


def _act(name: str):
    return {"relu": F.relu, "gelu": F.gelu, "silu": F.silu,
            "gelu_new": lambda x: F.gelu(x, approximate="tanh")}[name]


def _heads(x: torch.Tensor, H: int, D: int) -> torch.Tensor:
    B, L, _ = x.shape
    return x.view(B, L, H, D).transpose(1, 2)


def _merge(x: torch.Tensor) -> torch.Tensor:
    B, H, L, D = x.shape
    return x.transpose(1, 2).reshape(B, L, H * D)


def basic_self_attention(sd: SD, prefix: str, cfg, hidden: torch.Tensor, table: torch.Tensor,
                         key_mask: Optional[torch.Tensor], causal: bool, attention_type: str = "basic") -> torch.Tensor:
    """T5Attention.forward for self-attention (attentions.py:144-257) or the sparse modules' math."""
    H, D = cfg.num_heads, cfg.d_kv
    q = _heads(hidden @ sd[prefix + "q.weight"].T, H, D)
    k = _heads(hidden @ sd[prefix + "k.weight"].T, H, D)
    v = _heads(hidden @ sd[prefix + "v.weight"].T, H, D)
    nb, md = cfg.relative_attention_num_buckets, cfg.relative_attention_max_distance
    L = hidden.shape[1]
    if attention_type in ("basic", "flash"):
        bias = O.dense_bias(table, L, L, causal, nb, md, H)
        if key_mask is not None:
            bias = bias + torch.where(key_mask[:, None, None, :] > 0, 0.0, float("-inf"))
        out = torch.nan_to_num(O.basic_attention(q, k, v, bias), nan=0.0)
    elif attention_type == "local":
        out = O.local_attention_blocked(q, k, v, table, cfg.sliding_window, key_mask, nb, md)
    elif attention_type == "block":
        out = O.block_attention_blocked(q, k, v, table, cfg.sliding_window, cfg.global_block_size, key_mask, nb, md)
    elif attention_type == "transient-global":
        gbs = cfg.global_block_size
        side = tglobal_side_inputs(hidden, gbs, sd[prefix + "global_input_layer_norm.weight"], cfg.layer_norm_epsilon,
                                   key_mask)
        sk = _heads(side @ sd[prefix + "k.weight"].T, H, D)
        sv = _heads(side @ sd[prefix + "v.weight"].T, H, D)
        out = tglobal_attention(q, k, v, sk, sv, table, cfg.sliding_window, gbs, nb, md, key_mask)
    else:
        raise KeyError(attention_type)
    return _merge(out) @ sd[prefix + "o.weight"].T


def tglobal_side_inputs(hidden, gbs, norm_weight, eps, attention_mask=None):
    """Block sums (trailing tokens join the last full block, utils.py:206-212) -> RMSNorm."""
    B, L, _ = hidden.shape
    block_ids, seg = O.make_global_fixed_block_ids(torch.ones(B, L) if attention_mask is None else attention_mask, gbs)
    agg = O.create_global_aggregates(hidden, block_ids, seg.shape[-1])
    return O.rms_norm(agg, norm_weight, eps)


def tglobal_attention(q, k, v, sk, sv, table, Bl, gbs, nb, md, attention_mask=None):
    """Blocked oracle when the reference's blocking applies, dense closed form otherwise
    (L not a multiple of the block length breaks the reference's reshape, attentions.py:575-576)."""
    B, H, L, D = q.shape
    if L % Bl == 0 or L < Bl:
        return O.tglobal_attention_blocked(q, k, v, sk, sv, table, Bl, gbs, attention_mask, nb, md)
    if attention_mask is not None:
        raise NotImplementedError("padding mask with a length that the reference's blocking cannot take")
    i = torch.arange(L)[:, None]
    j = torch.arange(L)[None, :]
    local = table[O.relative_position_bucket(j - i, True, nb, md)].permute(2, 0, 1).unsqueeze(0)
    local = local.masked_fill((j - i).abs() >= Bl, float("-inf"))
    block_ids, _ = O.make_global_fixed_block_ids(torch.ones(1, L), gbs)
    g = torch.arange(sk.shape[2])[None, :]
    side = table[O.relative_position_bucket(g - block_ids[0][:, None].long(), True, nb, md)].permute(2, 0, 1).unsqueeze(0)
    return O.basic_attention(q, torch.cat([k, sk], 2), torch.cat([v, sv], 2), torch.cat([local, side], -1))


def cross_attention(sd: SD, prefix: str, cfg, hidden, memory, key_mask) -> torch.Tensor:
    """T5Attention.forward with key_value_states: no position bias (attentions.py:222-227)."""
    H, D = cfg.num_heads, cfg.d_kv
    q = _heads(hidden @ sd[prefix + "q.weight"].T, H, D)
    k = _heads(memory @ sd[prefix + "k.weight"].T, H, D)
    v = _heads(memory @ sd[prefix + "v.weight"].T, H, D)
    bias = None
    if key_mask is not None:
        bias = torch.where(key_mask[:, None, None, :] > 0, 0.0, float("-inf"))
    return _merge(O.basic_attention(q, k, v, bias)) @ sd[prefix + "o.weight"].T


def feed_forward(sd: SD, prefix: str, cfg, hidden) -> torch.Tensor:
    x = O.rms_norm(hidden, sd[prefix + "layer_norm.weight"], cfg.layer_norm_epsilon)
    act = _act(cfg.dense_act_fn)
    p = prefix + "DenseReluDense."
    if cfg.is_gated_act:
        y = act(x @ sd[p + "wi_0.weight"].T) * (x @ sd[p + "wi_1.weight"].T)
    else:
        y = act(x @ sd[p + "wi.weight"].T)
    return hidden + y @ sd[p + "wo.weight"].T


def encoder_forward(sd: SD, cfg, input_ids: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                    attention_type: str = "basic", num_layers: Optional[int] = None) -> torch.Tensor:
    hidden = sd["shared.weight"][input_ids]
    table = sd["encoder.block.0.layer.0.SelfAttention.relative_attention_bias.weight"]
    n = cfg.num_layers if num_layers is None else num_layers
    for i in range(n):
        p = f"encoder.block.{i}.layer."
        x = O.rms_norm(hidden, sd[p + "0.layer_norm.weight"], cfg.layer_norm_epsilon)
        hidden = hidden + basic_self_attention(sd, p + "0.SelfAttention.", cfg, x, table, attention_mask, False,
                                               attention_type)
        hidden = feed_forward(sd, p + "1.", cfg, hidden)
    hidden = O.rms_norm(hidden, sd["encoder.final_layer_norm.weight"], cfg.layer_norm_epsilon)
    if attention_mask is not None:
        hidden = hidden * (attention_mask[..., None] > 0)     # padded rows carry no meaning: zero them
    return hidden


def decoder_forward(sd: SD, cfg, decoder_input_ids: torch.Tensor, memory: torch.Tensor,
                    memory_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Full (non-incremental) decoder pass; equals the incremental pass with a KV cache."""
    hidden = sd["shared.weight"][decoder_input_ids]
    table = sd["decoder.block.0.layer.0.SelfAttention.relative_attention_bias.weight"]
    for i in range(cfg.num_decoder_layers):
        p = f"decoder.block.{i}.layer."
        x = O.rms_norm(hidden, sd[p + "0.layer_norm.weight"], cfg.layer_norm_epsilon)
        hidden = hidden + basic_self_attention(sd, p + "0.SelfAttention.", cfg, x, table, None, True)
        x = O.rms_norm(hidden, sd[p + "1.layer_norm.weight"], cfg.layer_norm_epsilon)
        hidden = hidden + cross_attention(sd, p + "1.EncDecAttention.", cfg, x, memory, memory_mask)
        hidden = feed_forward(sd, p + "2.", cfg, hidden)
    return O.rms_norm(hidden, sd["decoder.final_layer_norm.weight"], cfg.layer_norm_epsilon)


def lm_logits(sd: SD, cfg, hidden: torch.Tensor) -> torch.Tensor:
    """Tied embeddings: rescale by d_model**-0.5 before the head; untied: no rescale (modeling.py:704)."""
    if getattr(cfg, "tie_word_embeddings", True):
        hidden = hidden * (cfg.d_model ** -0.5)
    return hidden @ sd["lm_head.weight"].T
