"""CPU oracle for DeBERTa-v2/v3 disentangled attention.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain torch-CPU / numpy, the eager arithmetic of Hugging Face
``transformers`` (5.15.0) ``models/deberta_v2/modeling_deberta_v2.py`` -- the third-party
routine the reference (TurboDeBERTa) subclasses and is graded against.  Abbreviation used in
citations below:  HF = that file.  Nothing in the shipped package may import this module;
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do,
and only as the checker.

Pin status of each function (what independent evidence fixes it):

* ``log_bucket_position`` / ``relative_position_index`` -- pinned: closed-form zones, spot
  values, antisymmetry/monotonicity, a float64 margin proof, a float64 scalar restatement
  (``bucket_scalar`` below) and golden tables written by HF's own
  ``make_log_bucket_position`` (``tests/golden/hf_bucket_table.npz``).
* ``disentangled_bias`` / ``attention`` -- pinned: brute-force triple loop on tiny shapes,
  Toeplitz invariant, reduction to ``torch.nn.functional.scaled_dot_product_attention`` when
  the position terms vanish, and golden outputs written by HF's
  ``DisentangledSelfAttention.forward`` (``tests/golden/hf_layer_outputs.npz``).
* ``self_attention_layer`` -- pinned by the same HF golden outputs (config-1 layer);
  a two-layer model output is in ``tests/golden/hf_tiny_model.npz``.
* ``encoder_attention_mask`` -- pinned by an HF golden 2x8 toy
  (``tests/golden/hf_mask_toy.npz``).
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import numpy as np
import torch


# ----------------------------------------------------------------------------------------
# relative-position bucketing (integer stage; must be bit exact)
# ----------------------------------------------------------------------------------------

def log_bucket_position(rel: torch.Tensor, bucket_size: int, max_position: int) -> torch.Tensor:
    """Signed log-bucket of an integer relative position.  Follows HF:57-69
    (``make_log_bucket_position``): identity for ``|rel| <= bucket_size//2``, then
    ``ceil(log(|rel|/mid) / log((max_position-1)/mid) * (mid-1)) + mid`` with the sign restored.
    The floating-point part is evaluated the way torch evaluates it for an int64 input:
    the integer division promotes to float32, everything after stays float32.
    Returns a float32 tensor (HF returns the float ``log_pos`` dtype; the caller casts to long).
    """
    mid = bucket_size // 2
    sign = torch.sign(rel)
    inner = (rel < mid) & (rel > -mid)
    abs_pos = torch.where(inner, torch.full_like(rel, mid - 1), rel.abs())
    num = torch.log(abs_pos / mid)                       # int64 / int -> float32
    den = torch.log(torch.tensor((max_position - 1) / mid))   # python float -> float32 scalar
    log_pos = torch.ceil(num / den * (mid - 1)) + mid
    return torch.where(abs_pos <= mid, rel.to(log_pos.dtype), log_pos * sign)


def relative_position(q_len: int, k_len: int, bucket_size: int = -1, max_position: int = -1) -> torch.Tensor:
    """``[q_len, k_len]`` int64 matrix of (bucketed) ``i - j``.  Follows HF:72-101
    (``build_relative_position``): bucketing is applied only when both ``bucket_size`` and
    ``max_position`` are positive (HF:96)."""
    rel = torch.arange(q_len, dtype=torch.long)[:, None] - torch.arange(k_len, dtype=torch.long)[None, :]
    if bucket_size > 0 and max_position > 0:
        rel = log_bucket_position(rel, bucket_size, max_position)
    return rel.to(torch.long)


def att_span(position_buckets: int, max_relative_positions: int) -> int:
    """Half-width of the relative-embedding table.  HF:168-174 (``pos_ebd_size``)."""
    return position_buckets if position_buckets > 0 else max_relative_positions


def relative_position_index(q_len: int, k_len: int, position_buckets: int, max_relative_positions: int) -> torch.Tensor:
    """delta(i, j) = clamp(bucket(i - j) + span, 0, 2*span - 1), int64 ``[q_len, k_len]``.
    This single index serves both terms at score position (i, j):  c2p uses it directly
    (HF:318); p2c gathers row j of ``K.Q_r^T`` at ``clamp(span - bucket(j - i))`` and then
    transposes (HF:336-343), which equals the same delta(i, j) because the bucket is odd."""
    span = att_span(position_buckets, max_relative_positions)
    rel = relative_position(q_len, k_len, position_buckets, max_relative_positions)
    return torch.clamp(rel + span, 0, 2 * span - 1)


def delta_table(max_len: int, position_buckets: int, max_relative_positions: int) -> np.ndarray:
    """delta as a function of r = i - j for r in [-(max_len-1), max_len-1]; int32
    ``[2*max_len - 1]``, entry ``r + max_len - 1``.  Same arithmetic as
    ``relative_position_index`` on a 1-D range (the bucket depends on i - j only)."""
    span = att_span(position_buckets, max_relative_positions)
    rel = torch.arange(-(max_len - 1), max_len, dtype=torch.long)
    if position_buckets > 0 and max_relative_positions > 0:
        rel = log_bucket_position(rel, position_buckets, max_relative_positions).to(torch.long)
    return torch.clamp(rel + span, 0, 2 * span - 1).to(torch.int32).numpy()


# ----------------------------------------------------------------------------------------
# attention on explicit per-head tensors
# ----------------------------------------------------------------------------------------

def scale_factor_of(pos_att_type: Sequence[str]) -> int:
    """1 + [c2p] + [p2c].  HF:237-241."""
    return 1 + int("c2p" in pos_att_type) + int("p2c" in pos_att_type)


def _scale(d: int, scale_factor: int) -> torch.Tensor:
    """sqrt(float(d) * scale_factor) as a float32 tensor.  HF:120-121 (``scaled_size_sqrt``)."""
    return torch.sqrt(torch.tensor(d, dtype=torch.float) * scale_factor)


def disentangled_bias(q: torch.Tensor, k: torch.Tensor, pos_key: Optional[torch.Tensor],
                      pos_query: Optional[torch.Tensor], position_buckets: int,
                      max_relative_positions: int, pos_att_type: Sequence[str]) -> torch.Tensor:
    """c2p + p2c score bias, ``[B, H, Lq, Lk]``, already divided by sqrt(d*scale_factor).
    Follows HF:276-345.  ``q, k``: ``[B, H, L, D]``; ``pos_key, pos_query``: ``[H, 2*span, D]``
    (the per-head projections of ``rel_embeddings[0:2*span]``, HF:295-312).  The gathers and
    the transpose of the p2c term are kept literally as HF writes them."""
    B, H, Lq, D = q.shape
    Lk = k.shape[2]
    span = att_span(position_buckets, max_relative_positions)
    sf = scale_factor_of(pos_att_type)
    rel = relative_position(Lq, Lk, position_buckets, max_relative_positions)       # [Lq, Lk]
    score = torch.zeros(B, H, Lq, Lk, dtype=q.dtype)
    if "c2p" in pos_att_type:
        scale = _scale(pos_key.shape[-1], sf)
        c2p_att = torch.matmul(q, pos_key.transpose(-1, -2)[None])                 # [B,H,Lq,2s]  HF:317
        c2p_pos = torch.clamp(rel + span, 0, 2 * span - 1)                          # HF:318
        c2p_att = torch.gather(c2p_att, -1, c2p_pos[None, None].expand(B, H, Lq, Lk))
        score = score + c2p_att / scale.to(c2p_att.dtype)                           # HF:324
    if "p2c" in pos_att_type:
        scale = _scale(pos_query.shape[-1], sf)
        assert Lq == Lk, "self-attention only (HF:327-334 rebuilds r_pos otherwise)"
        p2c_pos = torch.clamp(-rel + span, 0, 2 * span - 1)                         # HF:336
        p2c_att = torch.matmul(k, pos_query.transpose(-1, -2)[None])               # [B,H,Lk,2s]  HF:337
        p2c_att = torch.gather(p2c_att, -1, p2c_pos[None, None].expand(B, H, Lk, Lk)).transpose(-1, -2)
        score = score + p2c_att / scale.to(p2c_att.dtype)                           # HF:343
    return score


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
              pos_key: Optional[torch.Tensor], pos_query: Optional[torch.Tensor],
              key_mask: Optional[torch.Tensor] = None, *, position_buckets: int = 256,
              max_relative_positions: int = 512, pos_att_type: Sequence[str] = ("c2p", "p2c"),
              return_probs: bool = False):
    """softmax(QK^T/s + c2p/s + p2c/s, masked) V on ``[B, H, L, D]`` tensors, in the dtype of
    ``q`` with HF's operation order (HF:242-264): K is divided by the scale *before* QK^T, each
    term is produced in the working dtype, masked scores become ``finfo.min``.
    ``key_mask``: bool broadcastable to ``[B, 1, Lq, Lk]`` (True = attend) or None.
    Returns ``[B, H, L, D]``."""
    D = q.shape[-1]
    sf = scale_factor_of(pos_att_type)
    scale = _scale(D, sf)
    scores = torch.matmul(q, (k.transpose(-1, -2) / scale.to(q.dtype)))           # HF:243
    if len(pos_att_type):
        scores = scores + disentangled_bias(q, k, pos_key, pos_query, position_buckets,
                                            max_relative_positions, pos_att_type)
    if key_mask is not None:
        scores = scores.masked_fill(~key_mask.bool(), torch.finfo(q.dtype).min)    # HF:256-257
    probs = torch.softmax(scores, dim=-1)                                           # HF:259
    out = torch.matmul(probs, v)                                                    # HF:262-264
    return (out, probs) if return_probs else out


def attention_lengths(q, k, v, pos_key, pos_query, seqlens: Optional[torch.Tensor], **kw) -> torch.Tensor:
    """``attention`` with a right-padding mask built from per-sequence valid lengths the way the
    HF encoder expands a 2-D mask (HF:601-608: ``m_i * m_j``); rows ``i >= len`` are zeroed in
    the result because parity is defined on valid tokens only."""
    B, H, L, D = q.shape
    if seqlens is None:
        return attention(q, k, v, pos_key, pos_query, None, **kw)
    m = (torch.arange(L)[None, :] < seqlens.to(torch.long)[:, None])               # [B, L]
    out = attention(q, k, v, pos_key, pos_query, encoder_attention_mask(m), **kw)
    return out * m[:, None, :, None].to(out.dtype)


def encoder_attention_mask(mask2d: torch.Tensor) -> torch.Tensor:
    """``[B, L]`` -> ``[B, 1, L, L]`` with entry ``m_i * m_j``.  HF:601-608."""
    ext = mask2d.unsqueeze(1).unsqueeze(2)
    return ext * ext.squeeze(-2).unsqueeze(-1)


def attention_varlen(q, k, v, pos_key, pos_query, cu_seqlens, **kw) -> torch.Tensor:
    """Packed ``[T, H, D]`` attention: every sequence ``cu[b]:cu[b+1]`` is attended on its own
    with in-sequence positions, which equals HF on a right-padded batch restricted to valid
    tokens."""
    out = torch.empty_like(q)
    cu = [int(x) for x in cu_seqlens]
    for b in range(len(cu) - 1):
        s, e = cu[b], cu[b + 1]
        if e == s:
            continue
        qb, kb, vb = (t[s:e].transpose(0, 1)[None] for t in (q, k, v))
        out[s:e] = attention(qb, kb, vb, pos_key, pos_query, None, **kw)[0].transpose(0, 1)
    return out


# ----------------------------------------------------------------------------------------
# whole self-attention layer from hidden states (config-1 shape)
# ----------------------------------------------------------------------------------------

def split_heads(x: torch.Tensor, heads: int) -> torch.Tensor:
    """``[B, L, H*D]`` -> ``[B, H, L, D]``.  HF:186-189."""
    B, L, _ = x.shape
    return x.view(B, L, heads, -1).permute(0, 2, 1, 3)


def position_projections(rel_embeddings, span, heads, w_pk, b_pk, w_pq, b_pq):
    """Per-head projections of the first ``2*span`` relative embeddings: ``[H, 2*span, D]`` each.
    HF:295-312; with ``share_att_key`` the caller passes the key/query projection weights."""
    rel = rel_embeddings[0:2 * span]
    pk = torch.nn.functional.linear(rel, w_pk, b_pk).view(2 * span, heads, -1).permute(1, 0, 2)
    pq = torch.nn.functional.linear(rel, w_pq, b_pq).view(2 * span, heads, -1).permute(1, 0, 2)
    return pk, pq


def self_attention_layer(hidden, mask4d, rel_embeddings, wq, bq, wk, bk, wv, bv, heads, *,
                         w_pos_key=None, b_pos_key=None, w_pos_query=None, b_pos_query=None,
                         position_buckets=256, max_relative_positions=512,
                         pos_att_type=("c2p", "p2c")) -> torch.Tensor:
    """``DisentangledSelfAttention.forward`` (HF:191-274) from hidden states: returns the
    context layer ``[B, L, H*D]``.  ``w_pos_* is None`` means ``share_att_key`` (HF:296-302)."""
    lin = torch.nn.functional.linear
    q = split_heads(lin(hidden, wq, bq), heads)
    k = split_heads(lin(hidden, wk, bk), heads)
    v = split_heads(lin(hidden, wv, bv), heads)
    span = att_span(position_buckets, max_relative_positions)
    if w_pos_key is None:
        w_pos_key, b_pos_key = wk, bk
    if w_pos_query is None:
        w_pos_query, b_pos_query = wq, bq
    pk, pq = position_projections(rel_embeddings, span, heads, w_pos_key, b_pos_key, w_pos_query, b_pos_query)
    ctx = attention(q, k, v, pk, pq, mask4d, position_buckets=position_buckets,
                    max_relative_positions=max_relative_positions, pos_att_type=pos_att_type)
    B, H, L, D = ctx.shape
    return ctx.permute(0, 2, 1, 3).reshape(B, L, H * D)


# ----------------------------------------------------------------------------------------
# brute force (pure Python loops; tiny shapes only) -- an independent statement of the maths
# ----------------------------------------------------------------------------------------

def bucket_scalar(r: int, bucket_size: int, max_position: int) -> int:
    """Scalar bucket in float64 ``math`` (independent of torch's float32 kernels)."""
    if bucket_size <= 0 or max_position <= 0:
        return r
    mid = bucket_size // 2
    a = abs(r)
    if a <= mid:
        return r
    val = math.ceil(math.log(a / mid) / math.log((max_position - 1) / mid) * (mid - 1)) + mid
    return val if r > 0 else -val


def attention_bruteforce(q, k, v, pos_key, pos_query, key_len=None, *, position_buckets,
                         max_relative_positions, pos_att_type=("c2p", "p2c")) -> torch.Tensor:
    """Triple loop over (i, j, d) for one ``[L, D]`` head in float64.
    S[i,j] = (Q_i.K_j + Q_i.K_r[delta] + K_j.Q_r[delta]) / sqrt(d*f), keys j >= key_len masked."""
    L, D = q.shape
    span = att_span(position_buckets, max_relative_positions)
    f = scale_factor_of(pos_att_type)
    n_keys = L if key_len is None else int(key_len)
    q, k, v = q.double(), k.double(), v.double()
    pk = pos_key.double() if pos_key is not None else None
    pq = pos_query.double() if pos_query is not None else None
    out = torch.zeros(L, D, dtype=torch.float64)
    for i in range(L):
        s = []
        for j in range(n_keys):
            dl = min(max(bucket_scalar(i - j, position_buckets, max_relative_positions) + span, 0), 2 * span - 1)
            acc = 0.0
            for d in range(D):
                acc += float(q[i, d]) * float(k[j, d])
                if "c2p" in pos_att_type:
                    acc += float(q[i, d]) * float(pk[dl, d])
                if "p2c" in pos_att_type:
                    acc += float(k[j, d]) * float(pq[dl, d])
            s.append(acc / math.sqrt(D * f))
        m = max(s)
        e = [math.exp(x - m) for x in s]
        z = sum(e)
        for j in range(n_keys):
            out[i] += (e[j] / z) * v[j]
    return out
