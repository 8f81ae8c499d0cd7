"""Hugging Face DeBERTa-v2/v3 modules with the attention core running on the fused MI355X kernel.

Class names follow TurboDeBERTa's ``model.py`` (``FlashDisentangledSelfAttention``,
``FlashDebertaV2Attention/Layer/Encoder/Model``).  Submodule and parameter names are Hugging Face's,
so a stock DeBERTa-v2/v3 ``state_dict`` loads unchanged; ``patch_model`` switches an already built
(e.g. ``from_pretrained``) model over in place.

What differs from the reference glue (model.py:34-186):
* no ``[B, H, L, 2*span]`` strips: the per-head projections of the relative embeddings go to the
  kernel, which contracts them on the matrix cores (``pos_key_layer`` / ``pos_query_layer``);
* q, k, v are passed as strided ``[B, H, L, D]`` views of the projection outputs -- no
  ``permute().contiguous()`` (model.py:70-78), and the output is written token-major so the final
  ``[B, L, H*D]`` is a view;
* padding is handled by per-sequence lengths inside the fixed-length kernel: no un-pad / re-pad
  gathers (model.py:138-183) and no host synchronisation (model.py:55-63, padding.py:82);
* the position index is Hugging Face's for both terms (modeling_deberta_v2.py:318, :336-343).
"""
from __future__ import annotations

import math
from typing import Optional

import torch
from torch import nn
from transformers.models.deberta_v2.modeling_deberta_v2 import (
    DebertaV2Attention,
    DebertaV2Encoder,
    DebertaV2Layer,
    DebertaV2Model,
    DisentangledSelfAttention,
)

from .ops.flash_attention import flash_attention_with_disentangled
from .padding import key_padding_mask


class FlashDisentangledSelfAttention(DisentangledSelfAttention):
    """``DisentangledSelfAttention`` (modeling_deberta_v2.py:137-345) with the score / softmax / value
    product replaced by one kernel launch.  Same constructor, parameters and ``forward`` signature.

    Masks: sequences must be right-padded (valid tokens first), which is what the DeBERTa tokenizers
    produce; the valid length of each sequence is taken from the mask.  Rows of padded query tokens
    are returned as zeros (the eager module gives them a meaningless uniform average,
    modeling_deberta_v2.py:256-259); downstream layers mask them anyway.
    ``output_attentions=True`` needs the probability matrix, which the fused kernel never forms: that
    call is served by the eager parent class."""

    def forward(self, hidden_states, attention_mask, output_attentions=False, query_states=None,
                relative_pos=None, rel_embeddings=None):
        if output_attentions:
            return super().forward(hidden_states, attention_mask, output_attentions, query_states,
                                   relative_pos, rel_embeddings)
        if query_states is None:
            query_states = hidden_states
        B, L, _ = hidden_states.shape
        H, D = self.num_attention_heads, self.attention_head_size
        if query_states.shape[1] != L:
            raise ValueError("self-attention only: query_states and hidden_states must have one length")

        heads = lambda x: x.view(B, L, H, D).permute(0, 2, 1, 3)          # [B, H, L, D] view, token-major storage
        q = heads(self.query_proj(query_states))
        k = heads(self.key_proj(hidden_states))
        v = heads(self.value_proj(hidden_states))

        scale_factor = 1 + int("c2p" in self.pos_att_type) + int("p2c" in self.pos_att_type)
        pos_key = pos_query = None
        buckets = max_rel = 0
        if self.relative_attention:
            buckets, max_rel = self.position_buckets, self.max_relative_positions
            span = self.pos_ebd_size
            rel = self.pos_dropout(rel_embeddings)[0:2 * span]                                   # HF:295
            table = lambda proj: proj(rel).view(2 * span, H, D).permute(1, 0, 2)                 # [H, 2*span, D] view
            if "c2p" in self.pos_att_type:
                pos_key = table(self.key_proj if self.share_att_key else self.pos_key_proj)      # HF:296-312
            if "p2c" in self.pos_att_type:
                pos_query = table(self.query_proj if self.share_att_key else self.pos_query_proj)
        else:
            scale_factor = 1
        sm_scale = 1.0 / math.sqrt(D * scale_factor)                                             # HF:120-121, :243

        seqlens = None
        if attention_mask is not None:
            seqlens = key_padding_mask(attention_mask).sum(dim=-1, dtype=torch.int32)
        out = flash_attention_with_disentangled(q, k, v, None, None, False, sm_scale, buckets, max_rel,
                                                pos_key_layer=pos_key, pos_query_layer=pos_query,
                                                seqlens_k=seqlens)
        # out has q's strides: [B, H, L, D] view of token-major [B, L, H, D] storage
        return (out.permute(0, 2, 1, 3).reshape(B, L, H * D), None)


class FlashDebertaV2Attention(DebertaV2Attention):
    def __init__(self, config):
        super().__init__(config)
        self.self = FlashDisentangledSelfAttention(config)


class FlashDebertaV2Layer(DebertaV2Layer):
    def __init__(self, config):
        super().__init__(config)
        self.attention = FlashDebertaV2Attention(config)


class FlashDebertaV2Encoder(DebertaV2Encoder):
    def __init__(self, config):
        super().__init__(config)
        self.layer = nn.ModuleList([FlashDebertaV2Layer(config) for _ in range(config.num_hidden_layers)])


class FlashDebertaV2Model(DebertaV2Model):
    def __init__(self, config):
        super().__init__(config)
        self.encoder = FlashDebertaV2Encoder(config)
        self.post_init()


def patch_model(model: nn.Module) -> nn.Module:
    """Switch every ``DisentangledSelfAttention`` inside ``model`` (any DeBERTa-v2/v3 model or task head,
    e.g. one loaded with ``from_pretrained``) to the fused kernel, in place.  Parameters are untouched."""
    for module in model.modules():
        if type(module) is DisentangledSelfAttention:
            module.__class__ = FlashDisentangledSelfAttention
    return model
