"""Lean T5 layer stack around the attention modules (the caller of the hot path).

Restates the wiring of the reference's src/turbot5/model/modeling.py -- layer wrappers
(:131-201), T5Block (:221-342), T5Stack (:352-632), T5EncoderModel (:834-942), T5Model (:635-831)
-- without the HuggingFace ``PreTrainedModel`` machinery.  Parameter names equal HF T5's, so a
T5 ``state_dict`` loads with ``load_state_dict``.  Differences from the reference:

* every attention in the stack runs in the HIP kernels: the encoder uses
  ``T5ATTENTION_TYPES[config.attention_type]``; the decoder self-attention is ``T5FlashAttention``
  in causal mode with a KV cache, the cross-attention ``T5FlashAttention(cross_attention=True)``,
  which switches to the split-K kernel for single-token steps (the reference keeps both on the
  torch 'basic' path, modeling.py:134-135, :170);
* layers receive the raw (batch, length) 0/1 mask (or None when the caller gives none) and the
  (num_buckets, H) table of layer 0 as ``position_bias`` (modeling.py:589), never an L x L tensor.
"""
from __future__ import annotations

import copy
from typing import List, Optional, Tuple

import torch
from torch import nn

from .attentions import T5ATTENTION_TYPES, T5FlashAttention, T5LayerNorm, packed_batch
from .padding import index_first_axis, pad_input
from .config import T5Config

_ACT = {"relu": nn.functional.relu, "gelu": nn.functional.gelu, "silu": nn.functional.silu,
        "gelu_new": lambda x: nn.functional.gelu(x, approximate="tanh")}


def _epilogue_ok(x, weight, zero_bias) -> bool:
    """Inference on a ROCm device with one floating dtype throughout: the GEMM library can apply the
    activation in the epilogue of the first projection (a private torch entry point, checked for)."""
    return (hasattr(torch, "_addmm_activation") and x.is_cuda
            and x.dtype in (torch.bfloat16, torch.float16, torch.float32)
            and weight.dtype == x.dtype and zero_bias.dtype == x.dtype
            and not (torch.is_grad_enabled() and (x.requires_grad or weight.requires_grad)))


class T5DenseActDense(nn.Module):
    def __init__(self, config: T5Config):
        super().__init__()
        self.wi = nn.Linear(config.d_model, config.d_ff, bias=False)
        self.wo = nn.Linear(config.d_ff, config.d_model, bias=False)
        self.act = _ACT[config.dense_act_fn]
        # a zero bias lets the GEMM library apply ReLU in the epilogue of wi (no separate pass over
        # the (tokens, d_ff) activations); not part of the state_dict
        self._relu = config.dense_act_fn == "relu"
        self.register_buffer("_zero_bias", torch.zeros(config.d_ff), persistent=False)

    def forward(self, hidden_states):
        if self._relu and _epilogue_ok(hidden_states, self.wi.weight, self._zero_bias):
            x = hidden_states.reshape(-1, hidden_states.shape[-1])
            mid = torch._addmm_activation(self._zero_bias, x, self.wi.weight.t(), use_gelu=False)
            return self.wo(mid).view(*hidden_states.shape[:-1], -1)
        return self.wo(self.act(self.wi(hidden_states)))


class T5DenseGatedActDense(nn.Module):
    def __init__(self, config: T5Config):
        super().__init__()
        self.wi_0 = nn.Linear(config.d_model, config.d_ff, bias=False)
        self.wi_1 = nn.Linear(config.d_model, config.d_ff, bias=False)
        self.wo = nn.Linear(config.d_ff, config.d_model, bias=False)
        self.act = _ACT[config.dense_act_fn]
        # tanh-GELU (the 'gated-gelu' of T5 v1.1 / Flan-T5) is the GEMM library's GELU epilogue: it is applied
        # to the fp32 accumulator of wi_0 before the one rounding to the activation type
        self._gelu_tanh = config.dense_act_fn == "gelu_new"
        self.register_buffer("_zero_bias", torch.zeros(config.d_ff), persistent=False)

    def forward(self, hidden_states):
        if self._gelu_tanh and _epilogue_ok(hidden_states, self.wi_0.weight, self._zero_bias):
            x = hidden_states.reshape(-1, hidden_states.shape[-1])
            gate = torch._addmm_activation(self._zero_bias, x, self.wi_0.weight.t(), use_gelu=True)
            return self.wo(gate * self.wi_1(x)).view(*hidden_states.shape[:-1], -1)
        return self.wo(self.act(self.wi_0(hidden_states)) * self.wi_1(hidden_states))


class T5LayerFF(nn.Module):
    def __init__(self, config: T5Config):
        super().__init__()
        self.DenseReluDense = T5DenseGatedActDense(config) if config.is_gated_act else T5DenseActDense(config)
        self.layer_norm = T5LayerNorm(config.d_model, eps=config.layer_norm_epsilon)

    def step(self, hidden_states, pending=None):
        """(residual stream, this sub-layer's update): ``pending`` is the previous sub-layer's update, added
        to the stream by the same kernel that norms it; the caller adds (or passes on) the returned update."""
        hidden_states, normed = self.layer_norm.add_norm(hidden_states, pending)
        return hidden_states, self.DenseReluDense(normed)

    def forward(self, hidden_states):
        hidden_states, update = self.step(hidden_states)
        return hidden_states + update


class T5LayerSelfAttention(nn.Module):
    def __init__(self, config: T5Config, has_relative_attention_bias=False):
        super().__init__()
        if config.is_decoder:
            self.SelfAttention = T5FlashAttention(config, has_relative_attention_bias=has_relative_attention_bias)
        else:
            try:
                cls = T5ATTENTION_TYPES[config.attention_type]
            except KeyError:
                raise KeyError(f"attention_type={config.attention_type!r}; available: {sorted(T5ATTENTION_TYPES)}") from None
            self.SelfAttention = cls(config, has_relative_attention_bias=has_relative_attention_bias)
        self.layer_norm = T5LayerNorm(config.d_model, eps=config.layer_norm_epsilon)

    def step(self, hidden_states, pending=None, attention_mask=None, position_bias=None, layer_head_mask=None,
             past_key_value=None, use_cache=False, output_attentions=False, packed=None):
        """(residual stream, the attention module's tuple); element 0 of the tuple is the update to add.
        ``packed``: the hidden states are the packed valid tokens of a padded batch (flash attention only)."""
        hidden_states, normed = self.layer_norm.add_norm(hidden_states, pending)
        if packed is not None:
            return hidden_states, self.SelfAttention.forward_packed(normed, packed, position_bias)
        kwargs = dict(mask=attention_mask, position_bias=position_bias, layer_head_mask=layer_head_mask,
                      past_key_value=past_key_value, output_attentions=output_attentions)
        if isinstance(self.SelfAttention, T5FlashAttention):
            kwargs["use_cache"] = use_cache
        return hidden_states, self.SelfAttention(normed, **kwargs)

    def forward(self, hidden_states, attention_mask=None, position_bias=None, layer_head_mask=None,
                past_key_value=None, use_cache=False, output_attentions=False):
        hidden_states, out = self.step(hidden_states, None, attention_mask, position_bias, layer_head_mask,
                                       past_key_value, use_cache, output_attentions)
        return (hidden_states + out[0],) + out[1:]


class T5LayerCrossAttention(nn.Module):
    def __init__(self, config: T5Config):
        super().__init__()
        self.EncDecAttention = T5FlashAttention(config, cross_attention=True, has_relative_attention_bias=False)
        self.layer_norm = T5LayerNorm(config.d_model, eps=config.layer_norm_epsilon)

    def step(self, hidden_states, pending, key_value_states, attention_mask=None, position_bias=None,
             past_key_value=None, use_cache=False, query_length=None):
        hidden_states, normed = self.layer_norm.add_norm(hidden_states, pending)
        return hidden_states, self.EncDecAttention(normed, mask=attention_mask, key_value_states=key_value_states,
                                                   position_bias=position_bias, past_key_value=past_key_value,
                                                   use_cache=use_cache, query_length=query_length)

    def forward(self, hidden_states, key_value_states, attention_mask=None, position_bias=None,
                past_key_value=None, use_cache=False, query_length=None):
        hidden_states, out = self.step(hidden_states, None, key_value_states, attention_mask, position_bias,
                                       past_key_value, use_cache, query_length)
        return (hidden_states + out[0],) + out[1:]


class T5Block(nn.Module):
    def __init__(self, config: T5Config, has_relative_attention_bias=False):
        super().__init__()
        self.is_decoder = config.is_decoder
        self.layer = nn.ModuleList([T5LayerSelfAttention(config, has_relative_attention_bias)])
        if self.is_decoder:
            self.layer.append(T5LayerCrossAttention(config))
        self.layer.append(T5LayerFF(config))

    def step(self, hidden_states, pending=None, attention_mask=None, position_bias=None, encoder_hidden_states=None,
             encoder_attention_mask=None, past_key_value=None, use_cache=False, packed=None):
        """The block with its last residual add left to the caller: returns (residual stream, update of the
        feed-forward sub-layer, present, position_bias).  ``pending`` is the previous block's update.  Every
        add between sub-layers happens inside the kernel that norms the sum for the next sub-layer."""
        self_past = past_key_value[:2] if past_key_value is not None else None
        cross_past = past_key_value[2:] if past_key_value is not None and len(past_key_value) == 4 else None
        hidden_states, sa = self.layer[0].step(hidden_states, pending, attention_mask=attention_mask,
                                               position_bias=position_bias, past_key_value=self_past,
                                               use_cache=use_cache, packed=packed)
        pending, present, position_bias = sa[0], sa[1], sa[2]
        if self.is_decoder and encoder_hidden_states is not None:
            hidden_states, ca = self.layer[1].step(hidden_states, pending, key_value_states=encoder_hidden_states,
                                                   attention_mask=encoder_attention_mask, past_key_value=cross_past,
                                                   use_cache=use_cache)
            pending = ca[0]
            if present is not None and ca[1] is not None:
                present = present + ca[1]
        hidden_states, pending = self.layer[-1].step(hidden_states, pending)
        return hidden_states, pending, present, position_bias

    def forward(self, hidden_states, attention_mask=None, position_bias=None, encoder_hidden_states=None,
                encoder_attention_mask=None, past_key_value=None, use_cache=False):
        hidden_states, update, present, position_bias = self.step(
            hidden_states, None, attention_mask, position_bias, encoder_hidden_states, encoder_attention_mask,
            past_key_value, use_cache)
        return hidden_states + update, present, position_bias


class T5Stack(nn.Module):
    def __init__(self, config: T5Config, embed_tokens: Optional[nn.Embedding] = None):
        super().__init__()
        self.config = config
        self.embed_tokens = embed_tokens
        self.is_decoder = config.is_decoder
        n = config.num_decoder_layers if config.is_decoder else config.num_layers
        self.block = nn.ModuleList([T5Block(config, has_relative_attention_bias=bool(i == 0)) for i in range(n)])
        self.final_layer_norm = T5LayerNorm(config.d_model, eps=config.layer_norm_epsilon)
        # An encoder with full ('flash') attention runs a padded batch on its valid tokens only: they are
        # packed once after the embedding, every layer (projections, attention through cu_seqlens, norms,
        # feed-forward) works on (total, d_model), and the result is scattered back into zeros at the end.
        # The reference packs and pads around each attention call only (attentions.py:492-511) and spends
        # the dense layers on the padding too.  Outputs at valid positions are the same; padded positions
        # of the result are zero.  Set to False to keep the padded layout through the stack.
        self.pack_padded_batches = (not config.is_decoder) and all(
            isinstance(b.layer[0].SelfAttention, T5FlashAttention) for b in self.block)

    def forward(self, input_ids=None, attention_mask=None, encoder_hidden_states=None, encoder_attention_mask=None,
                inputs_embeds=None, past_key_values=None, use_cache=False):
        if inputs_embeds is None:
            inputs_embeds = self.embed_tokens(input_ids)
        hidden_states = inputs_embeds
        if past_key_values is None:
            past_key_values = [None] * len(self.block)
        position_bias = None
        presents: List[Optional[Tuple[torch.Tensor, ...]]] = []
        # the decoder's own padding mask has no meaning under causal attention with right padding;
        # only the encoder mask is routed down (as key padding of self- and cross-attention).  Left padding
        # or holes would change the positions the reference computes (it unpads with the mask), so they
        # are refused rather than silently ignored.
        if self.is_decoder and attention_mask is not None and attention_mask.is_cuda:
            from .attentions import _mask_info
            all_ones, unpad = _mask_info(attention_mask)
            if not all_ones and not (unpad[0] == "lens" and unpad[2].get("right_padded")):
                raise NotImplementedError("the decoder takes all-ones or right-padded attention masks only")
        self_mask = None if self.is_decoder else attention_mask
        packed = None
        if self.pack_padded_batches and self_mask is not None and hidden_states.is_cuda:
            packed = packed_batch(self_mask)
            if packed is not None and packed.indices.numel() == 0:
                packed = None       # nothing valid anywhere: the padded route handles empty sequences
            if packed is not None:
                hidden_states = index_first_axis(hidden_states.reshape(-1, hidden_states.shape[-1]), packed.indices)
        pending = None      # the last sub-layer's update, not yet added to the residual stream
        for blk, past in zip(self.block, past_key_values):
            hidden_states, pending, present, position_bias = blk.step(
                hidden_states, pending, attention_mask=self_mask, position_bias=position_bias,
                encoder_hidden_states=encoder_hidden_states, encoder_attention_mask=encoder_attention_mask,
                past_key_value=past, use_cache=use_cache, packed=packed)
            presents.append(present)
        hidden_states = self.final_layer_norm.add_norm(hidden_states, pending)[1]
        if packed is not None:
            hidden_states = pad_input(hidden_states, packed.indices, packed.batch, packed.length)
        return hidden_states, (presents if use_cache else None)


def _init_t5_weights(module: nn.Module, config: T5Config) -> None:
    """HuggingFace T5 initialisation scheme (the reference inherits it, modeling.py:344-350)."""
    f = config.initializer_factor
    d_model, d_kv, n_heads, d_ff = config.d_model, config.d_kv, config.num_heads, config.d_ff
    for m in module.modules():
        if isinstance(m, T5LayerNorm):
            m.weight.data.fill_(f * 1.0)
        elif isinstance(m, T5DenseActDense):
            m.wi.weight.data.normal_(mean=0.0, std=f * (d_model ** -0.5))
            m.wo.weight.data.normal_(mean=0.0, std=f * (d_ff ** -0.5))
        elif isinstance(m, T5DenseGatedActDense):
            m.wi_0.weight.data.normal_(mean=0.0, std=f * (d_model ** -0.5))
            m.wi_1.weight.data.normal_(mean=0.0, std=f * (d_model ** -0.5))
            m.wo.weight.data.normal_(mean=0.0, std=f * (d_ff ** -0.5))
        elif hasattr(m, "q") and hasattr(m, "o") and hasattr(m, "key_value_proj_dim"):
            m.q.weight.data.normal_(mean=0.0, std=f * ((d_model * d_kv) ** -0.5))
            m.k.weight.data.normal_(mean=0.0, std=f * (d_model ** -0.5))
            m.v.weight.data.normal_(mean=0.0, std=f * (d_model ** -0.5))
            m.o.weight.data.normal_(mean=0.0, std=f * ((n_heads * d_kv) ** -0.5))
            if getattr(m, "has_relative_attention_bias", False):
                m.relative_attention_bias.weight.data.normal_(mean=0.0, std=f * (d_model ** -0.5))
                if hasattr(m, "global_relative_attention_bias"):
                    m.global_relative_attention_bias.weight.data.normal_(mean=0.0, std=f * (d_model ** -0.5))
    # writes through .data do not bump the version counter that the distance-LUT cache keys on
    from . import ops
    ops.clear_bias_luts()


class T5EncoderModel(nn.Module):
    def __init__(self, config: T5Config):
        super().__init__()
        self.config = config
        self.shared = nn.Embedding(config.vocab_size, config.d_model)
        enc_cfg = config.copy(is_decoder=False, use_cache=False, is_encoder_decoder=False)
        self.encoder = T5Stack(enc_cfg, self.shared)
        self.shared.weight.data.normal_(mean=0.0, std=config.initializer_factor * 1.0)
        _init_t5_weights(self, config)

    def forward(self, input_ids=None, attention_mask=None, inputs_embeds=None):
        return self.encoder(input_ids=input_ids, attention_mask=attention_mask, inputs_embeds=inputs_embeds)[0]


class T5Model(nn.Module):
    """Encoder-decoder with tied embeddings, an lm head and a greedy decoding loop."""

    def __init__(self, config: T5Config):
        super().__init__()
        self.config = config
        self.shared = nn.Embedding(config.vocab_size, config.d_model)
        enc_cfg = config.copy(is_decoder=False, use_cache=False, is_encoder_decoder=False)
        dec_cfg = config.copy(is_decoder=True, is_encoder_decoder=False)
        self.encoder = T5Stack(enc_cfg, self.shared)
        self.decoder = T5Stack(dec_cfg, self.shared)
        self.lm_head = nn.Linear(config.d_model, config.vocab_size, bias=False)
        self.shared.weight.data.normal_(mean=0.0, std=config.initializer_factor * 1.0)
        self.lm_head.weight.data.normal_(mean=0.0, std=config.initializer_factor * 1.0)
        if config.tie_word_embeddings:
            self.lm_head.weight = self.shared.weight
        # tied embeddings are rescaled before the head, untied ones are not (reference modeling.py:704)
        self.lm_scale = config.d_model ** -0.5 if config.tie_word_embeddings else 1.0
        _init_t5_weights(self, config)

    def forward(self, input_ids, decoder_input_ids, attention_mask=None, encoder_outputs=None,
                past_key_values=None, use_cache=False):
        if encoder_outputs is None:
            encoder_outputs = self.encoder(input_ids=input_ids, attention_mask=attention_mask)[0]
        hidden, presents = self.decoder(input_ids=decoder_input_ids, encoder_hidden_states=encoder_outputs,
                                        encoder_attention_mask=attention_mask, past_key_values=past_key_values,
                                        use_cache=use_cache)
        logits = self.lm_head(hidden * self.lm_scale if self.lm_scale != 1.0 else hidden)
        return logits, encoder_outputs, presents

    @torch.no_grad()
    def greedy_decode(self, input_ids=None, attention_mask=None, max_new_tokens: int = 16, encoder_outputs=None,
                      batch_size: Optional[int] = None):
        """Incremental greedy decoding: one token per step, self-attention over the KV cache through the
        dense kernel, cross-attention over the encoder memory through the split-K kernel."""
        if encoder_outputs is None:
            encoder_outputs = self.encoder(input_ids=input_ids, attention_mask=attention_mask)[0]
        B = encoder_outputs.shape[0] if batch_size is None else batch_size
        dev = encoder_outputs.device
        tokens = torch.full((B, 1), self.config.decoder_start_token_id, dtype=torch.long, device=dev)
        out, past = [], None
        for _ in range(max_new_tokens):
            logits, _, past = self.forward(None, tokens, attention_mask=attention_mask,
                                           encoder_outputs=encoder_outputs, past_key_values=past, use_cache=True)
            tokens = logits[:, -1].argmax(dim=-1, keepdim=True)
            out.append(tokens)
        return torch.cat(out, dim=1)

    @torch.no_grad()
    def greedy_decode_graphed(self, encoder_outputs: torch.Tensor, max_new_tokens: int = 16,
                              return_logits: bool = False, attention_mask: Optional[torch.Tensor] = None):
        """Greedy decoding with one HIP graph per decoding step instead of a few hundred launches.

        The step has fixed shapes: the self-attention keys and values live in preallocated
        (B, max_new_tokens, H, D) caches that the step appends to at a position held in device memory, and
        the packed kernel reads the current key length of every sequence from device memory too
        (``seq_lens_k``); cross-attention keys and values are projected once, outside the graph, and read
        by the split-K kernel.  The graph and its buffers are kept per (batch, memory length, step count)
        and reused by later calls (the two most recent shapes; ``model._decode_graphs.clear()`` frees them).
        Same tokens as ``greedy_decode`` up to rounding in the logits (the
        self-attention runs through the packed instead of the dense entry point).
        ``attention_mask``: the encoder's (B, N) mask.  Memories padded on either side are read by the split-K
        kernel with the first key and the key count of every memory in device buffers of the graph (so later
        calls may bring other lengths); masks with holes are not taken here.
        """
        from .attentions import _mask_info
        mem_rows = None
        if attention_mask is not None:
            all_ones, unpad = _mask_info(attention_mask)
            if not all_ones:
                if unpad[0] != "lens":
                    raise NotImplementedError("greedy_decode_graphed takes encoder masks without holes; use greedy_decode")
                mem_rows = unpad[1]          # (lengths, first rows in the (B*N) layout)
        from . import ops
        dec, cfg = self.decoder, self.config
        B, N, d = encoder_outputs.shape
        dev = encoder_outputs.device
        first = dec.block[0].layer[0].SelfAttention
        H, D = first.n_heads, first.key_value_proj_dim
        adt = first._attn_dtype(encoder_outputs)
        key = (B, N, int(max_new_tokens), str(dev), encoder_outputs.dtype, adt, bool(return_logits), mem_rows is not None)
        # a graph holds the addresses of the weights it was captured with: parameters that moved since
        # (``.to(...)``, a new ``nn.Parameter``) invalidate every captured step; values copied in place do not
        weights = tuple(p.data_ptr() for p in self.decoder.parameters()) + (self.lm_head.weight.data_ptr(),)
        cache = self.__dict__.setdefault("_decode_graphs", {})
        if self.__dict__.get("_decode_graph_weights") != weights:
            cache.clear()
            self.__dict__["_decode_graph_weights"] = weights
        st = cache.get(key)
        if st is None:
            while len(cache) >= 2:      # each entry owns the K/V buffers of its batch: keep the two latest shapes
                cache.pop(next(iter(cache)))
            T = int(max_new_tokens)
            st = cache[key] = dict(
                tok=torch.zeros(B, 1, dtype=torch.long, device=dev), pos=torch.zeros(1, dtype=torch.long, device=dev),
                lens=torch.ones(B, dtype=torch.int32, device=dev), out=torch.zeros(B, T, dtype=torch.long, device=dev),
                # self-attention cache: keys and values of a position side by side, so one copy appends both
                kv=[torch.zeros(B, T, 2, H, D, dtype=adt, device=dev) for _ in dec.block],
                # q, k and v projections of the self-attention as one GEMM: a copy of the three weights
                wqkv=[torch.empty(3 * H * D, cfg.d_model, dtype=first.q.weight.dtype, device=dev) for _ in dec.block],
                ck=[torch.empty(B, N, H, D, dtype=adt, device=dev) for _ in dec.block],
                cv=[torch.empty(B, N, H, D, dtype=adt, device=dev) for _ in dec.block],
                cu_q=torch.arange(B + 1, dtype=torch.int32, device=dev),
                cu_k=torch.arange(B + 1, dtype=torch.int32, device=dev) * T,
                mem_lens=torch.zeros(B, dtype=torch.int32, device=dev),
                mem_starts=torch.zeros(B, dtype=torch.int32, device=dev),
                logits=torch.zeros(B, T, cfg.vocab_size, device=dev) if return_logits else None, graph=None)
        T = st["out"].shape[1]
        table = first.relative_attention_bias.weight
        nb, md = first.relative_attention_num_buckets, first.relative_attention_max_distance
        scale = self.lm_scale

        def step():
            tok, pos, lens = st["tok"], st["pos"], st["lens"]
            hidden, pending = dec.embed_tokens(tok), None
            for l, blk in enumerate(dec.block):
                sa, ca, ff = blk.layer[0], blk.layer[1], blk.layer[2]
                attn, cross = sa.SelfAttention, ca.EncDecAttention
                hidden, normed = sa.layer_norm.add_norm(hidden, pending)
                qkv = nn.functional.linear(normed, st["wqkv"][l]).view(B, 3, H, D).to(adt)
                kv = st["kv"][l]
                kv.index_copy_(1, pos, qkv[:, 1:].unsqueeze(1))
                rows = kv.view(B * T, 2, H, D)
                o = ops.flash_attention_with_fusing_bias_varlen(
                    qkv[:, 0], rows[:, 0], rows[:, 1], table, st["cu_q"], st["cu_k"],
                    1, T, causal=True, sm_scale=1.0, NUM_BUCKETS=nb, MAX_DISTANCE=md, seq_lens_k=lens,
                    launch_plan=False)
                pending = attn.o(o.reshape(B, 1, H * D).to(hidden.dtype))
                hidden, normed = ca.layer_norm.add_norm(hidden, pending)
                q = cross._shape(cross.q(normed), B).to(adt)
                o = ops.flash_decoding_attention(
                    q, st["ck"][l].transpose(1, 2), st["cv"][l].transpose(1, 2), None, 1.0,
                    key_lens=st["mem_lens"] if mem_rows is not None else None,
                    key_starts=st["mem_starts"] if mem_rows is not None else None)
                pending = cross.o(cross._unshape(o, B).to(hidden.dtype))
                hidden, pending = ff.step(hidden, pending)
            hidden = dec.final_layer_norm.add_norm(hidden, pending)[1]
            logits = self.lm_head(hidden * scale)[:, -1]
            if st["logits"] is not None:
                st["logits"].index_copy_(1, pos, logits.float().unsqueeze(1))
            nxt = logits.argmax(dim=-1, keepdim=True)
            st["out"].index_copy_(1, pos, nxt)
            tok.copy_(nxt)
            pos.add_(1)
            lens.add_(1)

        def reset():
            st["tok"].fill_(cfg.decoder_start_token_id)
            st["pos"].zero_()
            st["lens"].fill_(1)

        if mem_rows is not None:
            st["mem_lens"].copy_(mem_rows[0])
            st["mem_starts"].copy_(mem_rows[1][:B] - torch.arange(B, device=dev, dtype=torch.int32) * N)
        # cross-attention keys and values of this memory, once; of padded memories only the valid rows are
        # projected (gathered once for all layers), the other rows of the buffers are never read
        valid_rows = packed_batch(attention_mask) if mem_rows is not None else None
        if valid_rows is not None and not 0 < valid_rows.indices.numel() <= 0.85 * B * N:
            valid_rows = None
        mem_valid = index_first_axis(encoder_outputs.reshape(B * N, d), valid_rows.indices) if valid_rows is not None else None
        for l, blk in enumerate(dec.block):
            attn = blk.layer[0].SelfAttention
            torch.cat([attn.q.weight, attn.k.weight, attn.v.weight], dim=0, out=st["wqkv"][l])   # current values
            cross = blk.layer[1].EncDecAttention
            for proj, buf in ((cross.k, st["ck"][l]), (cross.v, st["cv"][l])):
                if mem_valid is None:
                    buf.copy_(proj(encoder_outputs).view(B, N, H, D))
                else:
                    buf.view(B * N, H, D).index_copy_(0, valid_rows.indices, proj(mem_valid).view(-1, H, D).to(adt))
        if st["graph"] is None:
            reset()
            side = torch.cuda.Stream(device=dev)
            side.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(side):        # warm-up outside the capture: library handles, allocator
                step()
            torch.cuda.current_stream(dev).wait_stream(side)
            reset()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            st["graph"] = graph
        reset()
        for _ in range(T):
            st["graph"].replay()
        return (st["out"].clone(), st["logits"].clone()) if return_logits else st["out"].clone()
