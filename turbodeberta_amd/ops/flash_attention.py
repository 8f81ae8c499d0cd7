"""Fixed-length fused disentangled attention.

Drop-in for TurboDeBERTa's ``turbodeberta.ops.flash_attention`` (ops/flash_attention.py): same
function name, positional parameters and return value.  The device work is one launch of a
hand-written gfx950 kernel through ``tdb_attn_fwd_fixed`` (include/tdb_attn.h)."""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from .. import _lib
from . import _launch as L


def prepare(q, k, v, q_pos, k_pos, causal=False, sm_scale=None, position_buckets=0, max_relative_distance=0, *,
            pos_key_layer=None, pos_query_layer=None, seqlens_k=None, force_generic=False) -> L.PreparedLaunch:
    """Validate and pack one call of ``flash_attention_with_disentangled`` without launching it."""
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be [B, H, L, D]")
    Dq, Dk, Dv = q.shape[-1], k.shape[-1], v.shape[-1]
    assert Dq == Dk == Dv, "Query, key, and value must have the same head dimension"
    dev = L.require_gpu(q, k, v, q_pos, k_pos, pos_key_layer, pos_query_layer, seqlens_k)
    B, H, M, D = q.shape
    N = k.shape[2]
    if k.shape != (B, H, N, D) or v.shape != (B, H, N, D):
        raise ValueError(f"k/v shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
    if M != N:
        raise ValueError(f"self-attention only: query length {M} != key length {N}")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError("q, k, v must share one dtype")
    if causal:
        raise ValueError("causal=True is not supported (the reference glue never enables it, model.py:116)")
    if (q_pos is not None and pos_key_layer is not None) or (k_pos is not None and pos_query_layer is not None):
        raise ValueError("pass a position term either as a strip (q_pos/k_pos) or as a table (pos_*_layer), not both")

    span = L.att_span(position_buckets, max_relative_distance)
    q, k, v = L.as_rows(q), L.as_rows(k), L.as_rows(v)
    o = torch.empty_like(q)
    if not L.rows_ok(o):
        o = torch.empty(q.shape, dtype=q.dtype, device=dev)
    keep = [q, k, v]

    a = _lib.FixedArgs()
    a.dtype = L.dtype_code(q)
    a.batch, a.heads, a.head_dim, a.seqlen = B, H, D, M
    a.causal = 0
    a.flags = _lib.TDB_FLAG_FORCE_GENERIC if force_generic else 0
    a.sm_scale = L.default_scale(sm_scale, D)
    a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
    for nm, t in (("q", q), ("k", k), ("v", v), ("o", o)):
        setattr(a, nm + "_stride_b", t.stride(0))
        setattr(a, nm + "_stride_h", t.stride(1))
        setattr(a, nm + "_stride_l", t.stride(2))
    if seqlens_k is not None:
        if seqlens_k.shape != (B,):
            raise ValueError(f"seqlens_k must be [B={B}], got {tuple(seqlens_k.shape)}")
        seqlens_k = seqlens_k.to(torch.int32).contiguous()
        keep.append(seqlens_k)
        a.seqlens_k = seqlens_k.data_ptr()

    strips = []
    for name, s in (("q_pos", q_pos), ("k_pos", k_pos)):
        if s is not None:
            if s.dim() != 4 or s.shape[:3] != (B, H, M) or s.dtype != q.dtype:
                raise ValueError(f"{name}: expected a [B, H, L, 2*span] strip of dtype {q.dtype}, got {tuple(s.shape)} {s.dtype}")
            s = s if s.stride(-1) == 1 else s.contiguous()
        strips.append(s)
    pk = L.fused_table(pos_key_layer, H, span, D, "pos_key_layer")
    pq = L.fused_table(pos_query_layer, H, span, D, "pos_query_layer")
    for t in (pk, pq):
        if t is not None and t.dtype != q.dtype:
            raise ValueError("position tables must have the dtype of q")
    L.fill_pos(a.pos, dev=dev, max_len=M, span=span, position_buckets=position_buckets,
               max_relative_distance=max_relative_distance, pos_key=pk, pos_query=pq,
               c2p_strip=strips[0], p2c_strip=strips[1], varlen=False, keep=keep)
    keep += [t for t in (strips[0], strips[1], pk, pq) if t is not None]
    return L.PreparedLaunch(_lib.load().tdb_attn_fwd_fixed, a, o, keep, dev)


class FlashAttentionDisentangled(torch.autograd.Function):
    """Forward-only, like the reference (ops/flash_attention.py:319-343)."""

    @staticmethod
    def forward(ctx, q, k, v, q_pos, k_pos, causal, sm_scale, position_buckets, max_relative_distance,
                pos_key_layer, pos_query_layer, seqlens_k, force_generic):
        return prepare(q, k, v, q_pos, k_pos, causal, sm_scale, position_buckets, max_relative_distance,
                       pos_key_layer=pos_key_layer, pos_query_layer=pos_query_layer, seqlens_k=seqlens_k,
                       force_generic=force_generic).launch()

    @staticmethod
    def backward(ctx, grad_output):
        raise RuntimeError(L.BACKWARD_MESSAGE)


def flash_attention_with_disentangled(q, k, v, q_pos, k_pos, causal=False, sm_scale=None,
                                      position_buckets=0, max_relative_distance=0, *,
                                      pos_key_layer: Optional[torch.Tensor] = None,
                                      pos_query_layer: Optional[torch.Tensor] = None,
                                      seqlens_k: Optional[torch.Tensor] = None,
                                      force_generic: bool = False):
    """softmax(sm_scale * (Q K^T + c2p + p2c)) V with DeBERTa's log-bucketed relative positions.

    Positional parameters are the reference's (ops/flash_attention.py:345-369):

    q, k, v : ``[B, H, L, D]`` (any strides with a contiguous last dim, e.g. a permuted
        ``[B, L, H, D]`` projection output -- no copy is made).
    q_pos : content->position strip ``Q K_r^T``, ``[B, H, L, 2*span]``, or None.  (The reference
        glue passes its ``pos_key`` strip here, model.py:127-137.)
    k_pos : position->content strip ``K Q_r^T``, ``[B, H, L, 2*span]``, or None.
    causal : must be False.
    sm_scale : None means ``1/sqrt(D)``.
    position_buckets, max_relative_distance : bucket configuration; ``span`` is
        ``position_buckets`` if positive, else ``max_relative_distance``.

    Keyword-only extensions (fused mode -- no strips in HBM):

    pos_key_layer, pos_query_layer : ``[H, 2*span, D]`` or ``[1, H, 2*span, D]`` projections of the
        relative embeddings (``K_r``, ``Q_r``); the kernel contracts them on the matrix cores.
    seqlens_k : int32 ``[B]`` valid lengths of right-padded sequences; keys beyond are masked and
        query rows beyond are returned as zeros.
    force_generic : run the vector-ALU kernel even where the matrix-core kernel applies.

    Score position (i, j) reads column ``clamp(bucket(i-j) + span, 0, 2*span-1)`` of BOTH strips,
    which is Hugging Face's eager indexing (modeling_deberta_v2.py:318, :336-343).  The reference's
    Triton kernel mirrors the p2c column (ops/flash_attention.py:127); that deviation from the
    model definition is not reproduced.

    Returns ``o`` with the shape and dtype of ``q``.  Forward only: backward raises RuntimeError.
    """
    return FlashAttentionDisentangled.apply(q, k, v, q_pos, k_pos, causal, sm_scale, position_buckets,
                                            max_relative_distance, pos_key_layer, pos_query_layer,
                                            seqlens_k, force_generic)
