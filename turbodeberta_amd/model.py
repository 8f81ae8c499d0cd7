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
* the position index is Hugging Face's for both terms (modeling_deberta_v2.py:318, :336-343);
* in eval mode, work that does not depend on the input is done once instead of once per call: the
  per-head position tables (a function of the layer's weights and the shared relative embeddings
  only; the reference recomputes both strip GEMMs every call, model.py:94-110) and the
  concatenated Q/K/V weight of the single fused projection GEMM; the valid lengths are computed by
  the first layer that sees a mask and reused by the others (the reference recomputes them, with
  a host synchronisation, in every layer: model.py:55-63).
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


def _versions(*tensors):
    """Identity of a set of tensors for cache keys: storage address and in-place modification counter."""
    return tuple((t.data_ptr(), t._version, t.dtype, t.device) if t is not None else None for t in tensors)


def _lengths_of(attention_mask):
    """int32 [B] valid lengths of a right-padded batch.  The result is attached to the mask tensor, so the
    layers of an encoder, which all receive the same mask object (modeling_deberta_v2.py:651-660), compute it
    once per forward."""
    cached = getattr(attention_mask, "_tdb_lengths", None)
    if cached is not None and cached[0] == attention_mask._version:
        return cached[1]
    lengths = key_padding_mask(attention_mask).sum(dim=-1, dtype=torch.int32)
    try:
        attention_mask._tdb_lengths = (attention_mask._version, lengths)
    except AttributeError:      # tensor subclasses without a __dict__
        pass
    return lengths


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

        frozen = not self.training and not torch.is_grad_enabled()       # nothing below can change between calls
        if frozen and query_states is hidden_states:
            # one projection GEMM; q, k, v are views into its [B, L, 3, H, D] output (token stride 3*H*D)
            w, b = self._fused_qkv()
            qkv = nn.functional.linear(hidden_states, w, b).view(B, L, 3, H, D)
            q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        else:
            heads = lambda x: x.view(B, L, H, D).permute(0, 2, 1, 3)      # [B, H, L, D] view, token-major storage
            q = heads(self.query_proj(query_states))
            k = heads(self.key_proj(hidden_states))
            v = heads(self.value_proj(hidden_states))

        scale_factor = 1 + int("c2p" in self.pos_att_type) + int("p2c" in self.pos_att_type)
        pos_key = pos_query = None
        buckets = max_rel = 0
        if self.relative_attention:
            buckets, max_rel = self.position_buckets, self.max_relative_positions
            span = self.pos_ebd_size
            if frozen:
                pos_key, pos_query = self._position_tables(rel_embeddings, hidden_states.dtype)
            else:
                pos_key, pos_query = self._project_tables(self.pos_dropout(rel_embeddings)[0:2 * span])   # HF:295
        else:
            scale_factor = 1
        sm_scale = 1.0 / math.sqrt(D * scale_factor)                                             # HF:120-121, :243

        seqlens = _lengths_of(attention_mask) if attention_mask is not None else None
        out = flash_attention_with_disentangled(q, k, v, None, None, False, sm_scale, buckets, max_rel,
                                                pos_key_layer=pos_key, pos_query_layer=pos_query,
                                                seqlens_k=seqlens)
        # out has q's strides: [B, H, L, D] view of token-major storage
        return (out.permute(0, 2, 1, 3).reshape(B, L, H * D), None)

    def _project_tables(self, rel):
        """Per-head projections of the relative embeddings, ``[H, 2*span, D]`` views (modeling_deberta_v2.py:296-312)."""
        H, D = self.num_attention_heads, self.attention_head_size
        table = lambda proj: proj(rel).view(rel.shape[0], H, D).permute(1, 0, 2)
        pos_key = pos_query = None
        if "c2p" in self.pos_att_type:
            pos_key = table(self.key_proj if self.share_att_key else self.pos_key_proj)
        if "p2c" in self.pos_att_type:
            pos_query = table(self.query_proj if self.share_att_key else self.pos_query_proj)
        return pos_key, pos_query

    def _position_tables(self, rel_embeddings, dtype):
        """Eval-mode cache of ``_project_tables``: recomputed only when the relative embeddings or the
        projection weights have been modified (or moved / cast)."""
        kp = self.key_proj if self.share_att_key else getattr(self, "pos_key_proj", None)
        qp = self.query_proj if self.share_att_key else getattr(self, "pos_query_proj", None)
        key = (_versions(rel_embeddings, *(t for m in (kp, qp) if m is not None for t in (m.weight, m.bias))), dtype)
        cached = self.__dict__.get("_tdb_tables")
        if cached is None or cached[0] != key:
            rel = rel_embeddings[0:2 * self.pos_ebd_size]                # dropout is the identity in eval mode
            cached = (key, self._project_tables(rel))
            self.__dict__["_tdb_tables"] = cached
        return cached[1]

    def _fused_qkv(self):
        """Eval-mode cache of the concatenated ``[3*H*D, hidden]`` projection weight (and bias)."""
        mods = (self.query_proj, self.key_proj, self.value_proj)
        key = _versions(*(t for m in mods for t in (m.weight, m.bias)))
        cached = self.__dict__.get("_tdb_qkv")
        if cached is None or cached[0] != key:
            w = torch.cat([m.weight for m in mods], dim=0)
            b = torch.cat([m.bias for m in mods], dim=0) if all(m.bias is not None for m in mods) else None
            if b is None and any(m.bias is not None for m in mods):
                b = torch.cat([m.bias if m.bias is not None else m.weight.new_zeros(m.weight.shape[0]) for m in mods])
            cached = (key, (w, b))
            self.__dict__["_tdb_qkv"] = cached
        return cached[1]


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
