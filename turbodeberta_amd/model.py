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
  a host synchronisation, in every layer: model.py:55-63);
* in eval mode the encoder keeps a batch with padding packed from the embeddings to the last layer:
  projections, LayerNorms and feed-forward blocks run on ``[valid_tokens, hidden]`` and the packed
  attention kernel is called with views of the projection output, so padded positions cost
  nothing anywhere.  The reference packs and re-pads around the attention call of every layer
  (model.py:138-183); here there is one gather after the embeddings, one scatter at the end and one
  host synchronisation (the number of valid tokens) per forward.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
from torch import nn
from transformers.modeling_outputs import BaseModelOutput
from transformers.models.deberta_v2.modeling_deberta_v2 import (
    DebertaV2Attention,
    DebertaV2Encoder,
    DebertaV2ForMaskedLM,
    DebertaV2ForMultipleChoice,
    DebertaV2ForQuestionAnswering,
    DebertaV2ForSequenceClassification,
    DebertaV2ForTokenClassification,
    DebertaV2Layer,
    DebertaV2Model,
    DisentangledSelfAttention,
)

from .ops.flash_attention import flash_attention_with_disentangled
from .ops.flash_attention_varlen import flash_attention_with_disentangled_varlen
from .padding import index_first_axis, key_padding_mask, pad_input


def _versions(*tensors):
    """Identity of a set of live tensors (parameters) for cache keys: object, storage address and in-place
    modification counter.  Only meaningful for tensors that stay alive between the calls that compare keys."""
    return tuple((id(t), t.data_ptr(), t._version, t.dtype, t.device) if t is not None else None for t in tensors)


def _version_of(t):
    """In-place modification counter of a tensor, or None where there is none to read (inference tensors do not
    track one and raise on access)."""
    try:
        return t._version
    except (RuntimeError, AttributeError):
        return None


class _MaskInfo:
    """What the fused paths need to know about an attention mask: ``lengths`` int32 ``[B]`` on the device and
    ``total``, the number of valid tokens (a host int; ``None`` when the caller declared the lengths without it)."""
    __slots__ = ("lengths", "total")

    def __init__(self, lengths, total):
        self.lengths, self.total = lengths, total


def _mask_info(attention_mask):
    """Valid lengths of a batch whose mask is **right padded** (valid tokens first), verified: the kernels take
    per-sequence lengths, so a mask with holes or left padding cannot be expressed and raises ``ValueError`` instead
    of attending to the wrong tokens.  A 3-D / 4-D mask must be the outer product ``m_i * m_j`` Hugging Face's
    encoder builds (modeling_deberta_v2.py:601-608), or one row ``[.., 1, L]`` that broadcasts over the queries, and the
    same for every head; other shapes raise ``ValueError`` in ``key_padding_mask``.  The check costs one host synchronisation per mask object;
    the result is attached to the tensor, so the layers of an encoder, which all receive the same mask object
    (modeling_deberta_v2.py:651-660), share it.  (A mask without a modification counter -- an inference tensor --
    is trusted not to be modified in place between calls.)"""
    version = _version_of(attention_mask)
    cached = getattr(attention_mask, "_tdb_info", None)
    if cached is not None and cached[0] == version:
        return cached[1]
    valid = key_padding_mask(attention_mask) != 0                               # [B, L]
    L = valid.shape[-1]
    lengths = valid.sum(dim=-1, dtype=torch.int32)
    ok = (valid == (torch.arange(L, device=valid.device)[None, :] < lengths[:, None])).all()
    if attention_mask.dim() == 4 and attention_mask.shape[1] > 1:
        ok = ok & ((attention_mask != 0) == (attention_mask[:, :1] != 0)).all()      # one length per sequence: no per-head masks
    if attention_mask.dim() > 2 and attention_mask.shape[-2] == L and L > 1:
        full = attention_mask if attention_mask.dim() == 3 else attention_mask[:, 0]
        ok = ok & ((full != 0) == (valid[:, :, None] & valid[:, None, :])).all()
    ok_host, total = torch.stack([ok.to(torch.int64), lengths.sum(dtype=torch.int64)]).tolist()   # the one synchronisation
    if not ok_host:
        raise ValueError("attention_mask must be right padded (valid tokens first, no holes) and, if 3-D or 4-D, the "
                         "outer product of a key-padding mask with itself (or one broadcast row of it), equal for all "
                         "heads: the fused attention takes per-sequence lengths.  Use the eager Hugging Face modules for "
                         "other masks.")
    info = _MaskInfo(lengths, int(total))
    try:
        attention_mask._tdb_info = (version, info)
    except AttributeError:      # tensor subclasses without a __dict__
        pass
    return info


def declare_right_padded(attention_mask, lengths, total=None):
    """Opt out of the mask inspection: the caller vouches that ``attention_mask`` is right padded with ``lengths``
    (int32 ``[B]`` on the mask's device) valid tokens per sequence.  The facts are attached to the mask tensor the way
    ``_mask_info`` caches its own findings, so every fused module that receives this mask object uses them and none
    synchronises with the host: a forward on such a mask can be captured into a HIP graph.  ``total`` (a host int, the
    sum of the lengths) additionally lets the encoder pack the batch; without it the encoder keeps the padded layout,
    because the packed token count sizes host-side allocations.  Nothing is verified: wrong lengths give wrong
    attention.  Returns the mask."""
    if lengths.dtype != torch.int32 or lengths.dim() != 1 or lengths.shape[0] != attention_mask.shape[0]:
        raise ValueError("lengths must be an int32 tensor with one entry per sequence of the mask")
    if lengths.device != attention_mask.device:
        raise ValueError("lengths must live on the mask's device")
    attention_mask._tdb_info = (_version_of(attention_mask), _MaskInfo(lengths, None if total is None else int(total)))
    return attention_mask


def _packing_of(info, batch, seqlen, device):
    """``(indices, cu_seqlens)`` of a verified right-padded batch without a further synchronisation: positions of the
    valid tokens in the flattened ``[B*L]`` batch, int32 boundaries with a leading 0."""
    cu = torch.nn.functional.pad(torch.cumsum(info.lengths, dim=0, dtype=torch.int32), (1, 0))
    seq = torch.repeat_interleave(torch.arange(batch, device=device), info.lengths.long(), output_size=info.total)
    indices = torch.arange(info.total, device=device) - cu[:-1].long()[seq] + seq * seqlen
    return indices, cu


class FlashDisentangledSelfAttention(DisentangledSelfAttention):
    """``DisentangledSelfAttention`` (modeling_deberta_v2.py:137-345) with the score / softmax / value
    product replaced by one kernel launch.  Same constructor, parameters and ``forward`` signature.

    Masks: sequences must be right-padded (valid tokens first), which is what the DeBERTa tokenizers
    produce; the valid length of each sequence is taken from the mask, and a mask of any other shape
    (holes, left padding, a 3-D / 4-D mask that is not ``m_i * m_j``) raises ``ValueError`` -- checked
    once per mask object, with one host synchronisation.  Rows of padded query tokens
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

        pos_key, pos_query, sm_scale, buckets, max_rel = self._position_terms(rel_embeddings, hidden_states.dtype,
                                                                              frozen)
        seqlens = _mask_info(attention_mask).lengths if attention_mask is not None else None
        out = flash_attention_with_disentangled(q, k, v, None, None, False, sm_scale, buckets, max_rel,
                                                pos_key_layer=pos_key, pos_query_layer=pos_query,
                                                seqlens_k=seqlens)
        # out has q's strides: [B, H, L, D] view of token-major storage
        return (out.permute(0, 2, 1, 3).reshape(B, L, H * D), None)

    def forward_packed(self, hidden_states, cu_seqlens, max_seqlen, rel_embeddings=None):
        """Eval-mode forward on packed tokens: ``hidden_states [T, hidden]`` holds the valid tokens of all
        sequences back to back, ``cu_seqlens`` int32 ``[B+1]`` their boundaries.  Returns ``[T, H*D]``.
        The counterpart of the reference's packed branch (model.py:138-183) without its per-layer gathers."""
        T = hidden_states.shape[0]
        H, D = self.num_attention_heads, self.attention_head_size
        w, b = self._fused_qkv()
        qkv = nn.functional.linear(hidden_states, w, b).view(T, 3, H, D)
        pos_key, pos_query, sm_scale, buckets, max_rel = self._position_terms(rel_embeddings, hidden_states.dtype, True)
        out = flash_attention_with_disentangled_varlen(qkv[:, 0], qkv[:, 1], qkv[:, 2], None, None, cu_seqlens,
                                                       cu_seqlens, max_seqlen, max_seqlen, False, sm_scale, buckets,
                                                       max_rel, pos_key_layer=pos_key, pos_query_layer=pos_query,
                                                       zero_output=False)      # the packing comes from the verified mask
        return out.reshape(T, H * D)

    def _position_terms(self, rel_embeddings, dtype, frozen):
        """``(pos_key, pos_query, sm_scale, position_buckets, max_relative_positions)`` of one call."""
        scale_factor = 1
        pos_key = pos_query = None
        buckets = max_rel = 0
        if self.relative_attention:
            scale_factor += int("c2p" in self.pos_att_type) + int("p2c" in self.pos_att_type)
            buckets, max_rel = self.position_buckets, self.max_relative_positions
            if frozen:
                pos_key, pos_query = self._position_tables(rel_embeddings, dtype)
            else:
                rel = self.pos_dropout(rel_embeddings)[0:2 * self.pos_ebd_size]                 # HF:295
                pos_key, pos_query = self._project_tables(rel)
        return pos_key, pos_query, 1.0 / math.sqrt(self.attention_head_size * scale_factor), buckets, max_rel   # HF:120-121, :243

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
        # Identity of the relative embeddings: the encoder's layer-normed copy is a temporary, whose address says
        # nothing (it can be reused by a later, different tensor); FlashDebertaV2Encoder tags what it hands out with
        # the identity of its sources.  A parameter speaks for itself.  Anything else is not cached.
        source = getattr(rel_embeddings, "_tdb_source", None)
        if source is None and isinstance(rel_embeddings, nn.Parameter):
            source = _versions(rel_embeddings)
        if source is None:
            return self._project_tables(rel_embeddings[0:2 * self.pos_ebd_size])
        key = (source, _versions(*(t for m in (kp, qp) if m is not None for t in (m.weight, m.bias))), dtype)
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
    """``DebertaV2Encoder`` (modeling_deberta_v2.py:565-686) over ``FlashDebertaV2Layer``.

    In eval mode under ``torch.no_grad()`` a batch that contains padding runs **packed**: the valid tokens
    are gathered once, every layer works on ``[valid_tokens, hidden]`` (``forward_packed`` of the attention
    module, then Hugging Face's own output / feed-forward submodules, which are shape agnostic), and the
    result is scattered back to ``[B, L, hidden]`` with zeros at padded positions.  Verifying the mask and
    counting the valid tokens is the only host synchronisation of the forward.  Everything else -- training,
    gradients, ``output_attentions``, ``query_states``, CPU tensors, batches without padding -- takes the
    parent's loop over the (fused, padded) layers.  Masks must be right padded in either path (see
    ``FlashDisentangledSelfAttention``); others raise ``ValueError``.

    ``pack_sequences = False`` switches the packed path off."""

    pack_sequences = True

    def __init__(self, config):
        super().__init__(config)
        self.layer = nn.ModuleList([FlashDebertaV2Layer(config) for _ in range(config.num_hidden_layers)])

    def get_rel_embedding(self):
        """As the parent (modeling_deberta_v2.py:593-597); in eval mode under ``no_grad`` the (layer-normed) result is
        computed once per state of its sources and tagged with their identity, which the attention modules key
        their position-table caches on."""
        if self.training or torch.is_grad_enabled() or not self.relative_attention:
            return super().get_rel_embedding()
        sources = [self.rel_embeddings.weight]
        if "layer_norm" in self.norm_rel_ebd:
            sources += [self.LayerNorm.weight, self.LayerNorm.bias]
        key = _versions(*sources)
        cached = self.__dict__.get("_tdb_rel")
        if cached is None or cached[0] != key:
            rel = super().get_rel_embedding()
            if rel is self.rel_embeddings.weight:
                rel = rel.detach()           # a tensor of its own to carry the tag (shares the storage)
            rel._tdb_source = key
            cached = (key, rel)
            self.__dict__["_tdb_rel"] = cached
        return cached[1]

    def forward(self, hidden_states, attention_mask, output_hidden_states=True, output_attentions=False,
                query_states=None, relative_pos=None, return_dict=True, intermediate_states=True):
        """As the parent (modeling_deberta_v2.py:634-695).  ``intermediate_states=False`` (an argument of this class
        only) says that of the hidden states the caller reads just the first and the last: the packed path then
        leaves the layers in between out of the returned tuple instead of scattering each back to ``[B, L, hidden]``."""
        fused = (not output_attentions and torch.is_tensor(hidden_states)
                 and all(isinstance(l.attention.self, FlashDisentangledSelfAttention) for l in self.layer))
        packable = (fused and self.pack_sequences and not self.training and not torch.is_grad_enabled()
                    and query_states is None and hidden_states.is_cuda and attention_mask.dim() in (2, 3, 4))
        if packable:
            B, L, _ = hidden_states.shape
            info = _mask_info(attention_mask)                                # the one host synchronisation
            packable = info.total is not None and info.total < B * L      # (no total: declared by the caller)
            if packable:
                indices, cu_seqlens = _packing_of(info, B, L, hidden_states.device)
        if not packable:
            if fused and relative_pos is None and self.relative_attention:
                relative_pos = hidden_states.new_empty(0)    # fused layers never read the [L, L] matrix: do not build it
            return super().forward(hidden_states, attention_mask, output_hidden_states, output_attentions,
                                   query_states, relative_pos, return_dict)

        keep_all = output_hidden_states and intermediate_states
        padded = lambda t: pad_input(t, indices, B, L)
        all_hidden_states = (hidden_states,) if output_hidden_states else None
        rel_embeddings = self.get_rel_embedding()
        x = index_first_axis(hidden_states.reshape(B * L, -1), indices)
        for i, layer in enumerate(self.layer):
            attn = layer.attention
            attended = attn.output(attn.self.forward_packed(x, cu_seqlens, L, rel_embeddings), x)     # HF:368-378
            x = layer.output(layer.intermediate(attended), attended)                                   # HF:431-432
            if i == 0 and self.conv is not None:                                                       # HF:666-667
                x = index_first_axis(self.conv(hidden_states, padded(x), key_padding_mask(attention_mask).long())
                                     .reshape(B * L, -1), indices)
            if keep_all and i + 1 < len(self.layer):
                all_hidden_states = all_hidden_states + (padded(x),)
        output_states = padded(x)
        if output_hidden_states:
            all_hidden_states = all_hidden_states + (output_states,)
        if not return_dict:
            return tuple(v for v in [output_states, all_hidden_states, None] if v is not None)
        return BaseModelOutput(last_hidden_state=output_states, hidden_states=all_hidden_states, attentions=None)


class FlashDebertaV2Model(DebertaV2Model):
    def __init__(self, config):
        super().__init__(config)
        self.encoder = FlashDebertaV2Encoder(config)
        self.post_init()

    def forward(self, input_ids=None, attention_mask=None, token_type_ids=None, position_ids=None,
                inputs_embeds=None, output_attentions=None, output_hidden_states=None, return_dict=None, **kwargs):
        """As the parent (modeling_deberta_v2.py:711-793), which always asks the encoder for every layer's output and
        then uses the last one (modeling_deberta_v2.py:760-768).  When the caller did not ask for the hidden states
        (and no ``z_steps`` pass needs the last but one), the encoder is told so through its ``intermediate_states``
        argument, so that the packed path does not scatter every layer's result back to ``[B, L, hidden]`` for
        nothing.  Nothing is stored on the modules: concurrent calls on one model do not see each other's flags."""
        cfg = self.config
        want_hidden = output_hidden_states if output_hidden_states is not None else cfg.output_hidden_states
        if want_hidden or self.z_steps > 1 or kwargs:
            return super().forward(input_ids=input_ids, attention_mask=attention_mask, token_type_ids=token_type_ids,
                                   position_ids=position_ids, inputs_embeds=inputs_embeds,
                                   output_attentions=output_attentions, output_hidden_states=output_hidden_states,
                                   return_dict=return_dict, **kwargs)
        output_attentions = output_attentions if output_attentions is not None else cfg.output_attentions
        return_dict = return_dict if return_dict is not None else cfg.return_dict
        if (input_ids is None) == (inputs_embeds is None):
            raise ValueError("You have to specify exactly one of input_ids and inputs_embeds")
        given = input_ids if input_ids is not None else inputs_embeds[..., 0]
        if input_ids is not None:
            self.warn_if_padding_and_no_attention_mask(input_ids, attention_mask)
        if attention_mask is None:
            attention_mask = torch.ones(given.shape, device=given.device)
        if token_type_ids is None:
            token_type_ids = torch.zeros(given.shape, dtype=torch.long, device=given.device)
        embedded = self.embeddings(input_ids=input_ids, token_type_ids=token_type_ids, position_ids=position_ids,
                                   mask=attention_mask, inputs_embeds=inputs_embeds)
        encoded = self.encoder(embedded, attention_mask, output_hidden_states=True, output_attentions=output_attentions,
                               return_dict=return_dict, intermediate_states=False)
        sequence_output = encoded[1][-1]
        if not return_dict:
            return (sequence_output,) + tuple(encoded[2:])
        return BaseModelOutput(last_hidden_state=sequence_output, hidden_states=None, attentions=encoded.attentions)


class _FusedHead:
    """Task models with the reference's class names (model.py:244-314).  The Hugging Face parent builds the whole
    model -- so parameter names, weight tying and initialisation are exactly Hugging Face's and stock checkpoints
    load with ``from_pretrained`` -- and the attention / encoder / model classes inside are then switched to the fused
    ones.  (The reference's own constructors call ``DebertaV2PreTrainedModel().__init__(config)`` on a fresh,
    argument-less instance and cannot be instantiated.)"""

    def __init__(self, config):
        super().__init__(config)
        patch_model(self)


class FlashDebertaV2ForMaskedLM(_FusedHead, DebertaV2ForMaskedLM):
    pass


class FlashDebertaV2ForSequenceClassification(_FusedHead, DebertaV2ForSequenceClassification):
    pass


class FlashDebertaV2ForTokenClassification(_FusedHead, DebertaV2ForTokenClassification):
    pass


class FlashDebertaV2ForQuestionAnswering(_FusedHead, DebertaV2ForQuestionAnswering):
    pass


class FlashDebertaV2ForMultipleChoice(_FusedHead, DebertaV2ForMultipleChoice):
    pass


def patch_model(model: nn.Module) -> nn.Module:
    """Switch every ``DisentangledSelfAttention`` inside ``model`` (any DeBERTa-v2/v3 model or task head,
    e.g. one loaded with ``from_pretrained``) to the fused kernel, in place.  Parameters are untouched."""
    swaps = {DisentangledSelfAttention: FlashDisentangledSelfAttention, DebertaV2Encoder: FlashDebertaV2Encoder,
             DebertaV2Model: FlashDebertaV2Model}        # none of them adds parameters or constructor state
    for module in model.modules():
        if type(module) in swaps:
            module.__class__ = swaps[type(module)]
    return model
