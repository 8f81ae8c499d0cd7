"""Packing helpers with the names and return values of TurboDeBERTa's ``padding.py``.

They are kept for callers that hold packed data or want it; the attention glue in ``model.py``
does not need them (the fixed-length kernel takes per-sequence valid lengths and skips padding by
itself, so nothing is gathered or scattered around the attention call)."""
from __future__ import annotations

import torch
import torch.nn.functional as F


def key_padding_mask(attention_mask: torch.Tensor) -> torch.Tensor:
    """``[B, L]`` validity of every token from the masks Hugging Face passes around: a 2-D mask is
    returned as is; the encoder's ``[B, 1, L, L]`` (``m_i * m_j``, modeling_deberta_v2.py:601-608) or a
    ``[B, L, L]`` mask is reduced through its diagonal ``m_i * m_i`` -- a view, no reduction kernel; a
    mask with one query row that broadcasts over the queries (``[B, 1, L]``, ``[B, 1, 1, L]``, the
    "extended" key mask of other Hugging Face models) is that row.  Of a mask with several heads, head 0 is
    taken.  Any other shape raises ``ValueError``: a mask whose last two dimensions differ has no diagonal to
    read the tokens from.  (The reference assumes 2-D, padding.py:79-83, and breaks on the encoder's 4-D mask.)"""
    if attention_mask.dim() == 2:
        return attention_mask
    if attention_mask.dim() == 4:
        attention_mask = attention_mask[:, 0]
    if attention_mask.dim() != 3:
        raise ValueError(f"attention_mask must have 2, 3 or 4 dims, got {attention_mask.dim()}")
    rows, cols = attention_mask.shape[-2:]
    if rows == cols:
        return torch.diagonal(attention_mask, dim1=-2, dim2=-1)
    if rows == 1:
        return attention_mask[:, 0]
    raise ValueError(f"attention_mask of shape {tuple(attention_mask.shape)}: the last two dimensions must be "
                     f"[L, L] or [1, L]")


def sequence_lengths(attention_mask: torch.Tensor) -> torch.Tensor:
    """int32 ``[B]`` number of valid tokens per sequence (device tensor, no host sync)."""
    return key_padding_mask(attention_mask).sum(dim=-1, dtype=torch.int32)


def _get_unpad_data(attention_mask: torch.Tensor):
    """``(indices, cu_seqlens, max_seqlen_in_batch)`` as in the reference (padding.py:79-88):
    ``indices`` int64 positions of valid tokens in the flattened ``[B*L]`` batch, ``cu_seqlens`` int32
    ``[B+1]`` with a leading 0.  ``max_seqlen_in_batch`` is the padded length ``L`` -- an upper bound
    the kernels accept -- instead of the reference's ``.max().item()``, which costs a host sync."""
    mask = key_padding_mask(attention_mask)
    seqlens_in_batch = mask.sum(dim=-1, dtype=torch.int32)
    indices = torch.nonzero(mask.flatten(), as_tuple=False).flatten()
    cu_seqlens = F.pad(torch.cumsum(seqlens_in_batch, dim=0, dtype=torch.int32), (1, 0))
    return indices, cu_seqlens, int(mask.shape[-1])


def index_first_axis(input: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """Rows ``indices`` of ``input`` along dim 0 (padding.py:46-76, forward only)."""
    return input.index_select(0, indices)


def index_put_first_axis(values: torch.Tensor, indices: torch.Tensor, first_axis_dim: int) -> torch.Tensor:
    """Scatter ``values`` to rows ``indices`` of a zero tensor with ``first_axis_dim`` rows
    (padding.py:5-27, forward only)."""
    out = torch.zeros(first_axis_dim, *values.shape[1:], device=values.device, dtype=values.dtype)
    out.index_copy_(0, indices, values)
    return out


def pad_input(hidden_states: torch.Tensor, indices: torch.Tensor, batch: int, seqlen: int) -> torch.Tensor:
    """``[total, ...]`` -> ``[batch, seqlen, ...]`` with zeros at padded positions (padding.py:30-44)."""
    out = index_put_first_axis(hidden_states, indices, batch * seqlen)
    return out.view(batch, seqlen, *hidden_states.shape[1:])


def unpad_input(hidden_states: torch.Tensor, attention_mask: torch.Tensor):
    """``(packed [total, ...], indices, cu_seqlens, max_seqlen)`` (padding.py:90-111)."""
    indices, cu_seqlens, max_len = _get_unpad_data(attention_mask)
    flat = hidden_states.reshape(-1, *hidden_states.shape[2:])
    return index_first_axis(flat, indices), indices, cu_seqlens, max_len


def _upad_input(query_layer, key_layer, value_layer, pos_key, pos_query, attention_mask, query_length, NH):
    """Pack ``[B, L, H, D]`` q/k/v (and optional ``[B, L, H, 2*span]`` strips) by the mask, with the
    reference's return tuple (padding.py:113-166).  Self-attention only: ``query_length`` must equal
    the key length."""
    batch, kv_len, heads, head_dim = key_layer.shape
    if query_length != kv_len:
        raise ValueError("self-attention only: query_length must equal the key length")
    indices, cu_seqlens, max_len = _get_unpad_data(attention_mask)
    take = lambda t: None if t is None else index_first_axis(t.reshape(batch * kv_len, *t.shape[2:]), indices)
    return (take(query_layer), take(key_layer), take(value_layer), take(pos_key), take(pos_query), indices,
            (cu_seqlens, cu_seqlens), (max_len, max_len))
