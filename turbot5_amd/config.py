"""Configuration of the T5 modules on the attention hot path.

A plain dataclass with the field names of the reference's ``T5Config``
(src/turbot5/model/config.py:84-154) that the attention modules and the layer
stack read.  ``attention_type`` selects the encoder self-attention class from
``T5ATTENTION_TYPES``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import torch


@dataclass
class T5Config:
    vocab_size: int = 32128
    d_model: int = 512
    d_kv: int = 64
    d_ff: int = 2048
    num_layers: int = 6
    num_decoder_layers: Optional[int] = None
    num_heads: int = 8
    relative_attention_num_buckets: int = 32
    relative_attention_max_distance: int = 128
    dropout_rate: float = 0.1
    layer_norm_epsilon: float = 1e-6
    initializer_factor: float = 1.0
    feed_forward_proj: str = "relu"
    is_encoder_decoder: bool = True
    use_cache: bool = True
    pad_token_id: int = 0
    eos_token_id: int = 1
    decoder_start_token_id: int = 0
    # T5 v1.0 ties the lm head to the input embedding and rescales the decoder output by d_model**-0.5 before
    # it; T5 v1.1 / Flan (gated-gelu) have an untied head and no rescale (reference modeling.py:704)
    tie_word_embeddings: bool = True
    attention_type: str = "flash"        # key of T5ATTENTION_TYPES
    sliding_window: int = 512            # block_len of local / block / transient-global
    global_block_size: int = 32          # block: number of global tokens; transient-global: tokens per side token
    use_triton: bool = True              # accepted for compatibility; the HIP kernels are always used
    is_decoder: bool = False
    # dtype the attention kernels run in; None = the dtype of the activations.  torch.bfloat16 with
    # fp32 activations gives "fp32 activations, bf16 attention".
    attention_dtype: Optional[torch.dtype] = None
    # bf16 / fp16 attention: apply the score scale to the fp32 product instead of to the query rows (closer to
    # fp32 math at large scores, about 11 % slower); None = the default of ``turbot5_amd.ops.EXACT_SCORES``
    attention_exact_scores: Optional[bool] = None
    dense_act_fn: str = field(init=False, default="relu")
    is_gated_act: bool = field(init=False, default=False)

    def __post_init__(self):
        if self.num_decoder_layers is None:
            self.num_decoder_layers = self.num_layers
        act_info = self.feed_forward_proj.split("-")       # config.py:128-141
        self.dense_act_fn = act_info[-1]
        self.is_gated_act = act_info[0] == "gated"
        if len(act_info) > 1 and act_info[0] != "gated" or len(act_info) > 2:
            raise ValueError(f"`feed_forward_proj`: {self.feed_forward_proj} is not a valid activation function "
                             "of the dense layer. Please make sure `feed_forward_proj` is of the format "
                             "`gated-{ACT_FN}` or `{ACT_FN}`, e.g. 'gated-gelu' or 'relu'")
        if self.feed_forward_proj == "gated-gelu":
            self.dense_act_fn = "gelu_new"

    def copy(self, **changes) -> "T5Config":
        kw = {f: getattr(self, f) for f in self.__dataclass_fields__ if self.__dataclass_fields__[f].init}
        kw.update(changes)
        return T5Config(**kw)
