"""Packed variable-length fused disentangled attention.

Drop-in for TurboDeBERTa's ``turbodeberta.ops.flash_attention_varlen``
(ops/flash_attention_varlen.py): same function name, positional parameters and return value.  One
launch through ``tdb_attn_fwd_varlen`` (include/tdb_attn.h); the tile -> sequence work list the
reference builds on the host with one ``.item()`` per sequence (get_mid, :10-22) is resolved on
the device from ``cu_seqlens``."""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from .. import _lib
from . import _launch as L


def prepare(q, k, v, q_pos, k_pos, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal=False, sm_scale=None,
            position_buckets=0, max_relative_distance=0, *, pos_key_layer=None, pos_query_layer=None,
            force_generic=False, check_cu_seqlens=False, zero_output=True) -> L.PreparedLaunch:
    """Validate and pack one call of ``flash_attention_with_disentangled_varlen`` without launching it.

    ``max_seqlen`` must be a true upper bound and ``cu_seqlens[-1]`` must equal the token count: the kernels
    clamp a longer sequence to ``max_seqlen`` and never touch rows past ``cu_seqlens[-1]``.  Neither can be
    seen without reading ``cu_seqlens`` on the host, so the default makes no such read; rows the kernels do
    not cover are zeros (``zero_output``; callers that know their packing is exact, like the packed encoder,
    pass False and save the fill).  ``check_cu_seqlens=True`` copies the offsets to the host (one
    synchronisation) and raises ``ValueError`` on the first inconsistency."""
    if q.dim() != 3 or k.dim() != 3 or v.dim() != 3:
        raise ValueError("q, k, v must be [total_tokens, H, D]")
    Dq, Dk, Dv = q.shape[-1], k.shape[-1], v.shape[-1]
    assert Dq == Dk == Dv
    dev = L.require_gpu(q, k, v, q_pos, k_pos, cu_seqlens_q, cu_seqlens_k, pos_key_layer, pos_query_layer)
    T, H, D = q.shape
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError("self-attention only: q, k, v must have one shape")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError("q, k, v must share one dtype")
    if causal:
        raise ValueError("causal=True is not supported (the reference glue never enables it, model.py:116)")
    if cu_seqlens_k is not cu_seqlens_q and (cu_seqlens_k.shape != cu_seqlens_q.shape):
        raise ValueError("self-attention only: cu_seqlens_q and cu_seqlens_k must describe the same packing")
    if int(max_seqlen_q) != int(max_seqlen_k):
        raise ValueError("self-attention only: max_seqlen_q != max_seqlen_k")
    if cu_seqlens_q.dim() != 1 or cu_seqlens_q.numel() < 1:
        raise ValueError("cu_seqlens must be a 1-D tensor of B+1 offsets")
    if (q_pos is not None and pos_key_layer is not None) or (k_pos is not None and pos_query_layer is not None):
        raise ValueError("pass a position term either as a strip (q_pos/k_pos) or as a table (pos_*_layer), not both")

    B = cu_seqlens_q.numel() - 1
    span = L.att_span(position_buckets, max_relative_distance)
    q, k, v = L.as_rows(q), L.as_rows(k), L.as_rows(v)
    o = torch.empty_like(q)              # q's strides where the kernels can address them, else contiguous
    if not L.rows_ok(o):
        o = torch.empty(q.shape, dtype=q.dtype, device=dev)
    if zero_output:
        o.zero_()
    cu = cu_seqlens_q.to(torch.int32).contiguous()
    if check_cu_seqlens:
        _lib.check_cu_seqlens(cu.cpu().numpy(), T, max(int(max_seqlen_q), 1))
    keep = [cu, q, k, v]

    a = _lib.VarlenArgs()
    a.dtype = L.dtype_code(q)
    a.batch, a.heads, a.head_dim = B, H, D
    a.total_tokens, a.max_seqlen = T, max(int(max_seqlen_q), 1)
    a.causal = 0
    a.flags = _lib.TDB_FLAG_FORCE_GENERIC if force_generic else 0
    a.sm_scale = L.default_scale(sm_scale, D)
    a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
    for nm, t in (("q", q), ("k", k), ("v", v), ("o", o)):
        setattr(a, nm + "_stride_t", t.stride(0))
        setattr(a, nm + "_stride_h", t.stride(1))
    a.cu_seqlens = cu.data_ptr()

    strips = []
    for name, s in (("q_pos", q_pos), ("k_pos", k_pos)):
        if s is not None:
            if s.dim() != 3 or s.shape[:2] != (T, H) or s.dtype != q.dtype:
                raise ValueError(f"{name}: expected a [total, H, 2*span] strip of dtype {q.dtype}, got {tuple(s.shape)} {s.dtype}")
            s = s if s.stride(-1) == 1 else s.contiguous()
        strips.append(s)
    pk = L.fused_table(pos_key_layer, H, span, D, "pos_key_layer")
    pq = L.fused_table(pos_query_layer, H, span, D, "pos_query_layer")
    for t in (pk, pq):
        if t is not None and t.dtype != q.dtype:
            raise ValueError("position tables must have the dtype of q")
    L.fill_pos(a.pos, dev=dev, max_len=a.max_seqlen, span=span, position_buckets=position_buckets,
               max_relative_distance=max_relative_distance, pos_key=pk, pos_query=pq,
               c2p_strip=strips[0], p2c_strip=strips[1], varlen=True, keep=keep)
    keep += [t for t in (strips[0], strips[1], pk, pq) if t is not None]
    return L.PreparedLaunch(_lib.load().tdb_attn_fwd_varlen, a, o, keep, dev)


class FlashAttentionDisentangled(torch.autograd.Function):
    """Forward-only, like the reference (ops/flash_attention_varlen.py:317-346)."""

    @staticmethod
    def forward(ctx, q, k, v, q_pos, k_pos, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal,
                sm_scale, position_buckets, max_relative_distance, pos_key_layer, pos_query_layer, force_generic,
                check_cu_seqlens=False, zero_output=True):
        return prepare(q, k, v, q_pos, k_pos, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal,
                       sm_scale, position_buckets, max_relative_distance, pos_key_layer=pos_key_layer,
                       pos_query_layer=pos_query_layer, force_generic=force_generic,
                       check_cu_seqlens=check_cu_seqlens, zero_output=zero_output).launch()

    @staticmethod
    def backward(ctx, grad_output):
        raise RuntimeError(L.BACKWARD_MESSAGE)


def flash_attention_with_disentangled_varlen(q, k, v, q_pos, k_pos, cu_seqlens_q, cu_seqlens_k,
                                             max_seqlen_q, max_seqlen_k, causal=False, sm_scale=None,
                                             position_buckets=0, max_relative_distance=0, *,
                                             pos_key_layer: Optional[torch.Tensor] = None,
                                             pos_query_layer: Optional[torch.Tensor] = None,
                                             force_generic: bool = False, check_cu_seqlens: bool = False,
                                             zero_output: bool = True):
    """Packed-sequence form of ``flash_attention_with_disentangled``.

    Positional parameters are the reference's (ops/flash_attention_varlen.py:348-374):

    q, k, v : ``[total_tokens, H, D]``, sequences concatenated without padding.
    q_pos, k_pos : c2p / p2c strips ``[total_tokens, H, 2*span]`` or None.
    cu_seqlens_q, cu_seqlens_k : int32 ``[B+1]`` cumulative lengths (leading 0), as produced by
        ``padding._get_unpad_data``; both must describe the same packing.
    max_seqlen_q, max_seqlen_k : longest sequence (an upper bound is fine; a smaller value truncates longer
        sequences, their remaining rows come back as zeros).
    causal, sm_scale, position_buckets, max_relative_distance : as in the fixed-length operator.

    Keyword-only: ``pos_key_layer`` / ``pos_query_layer`` ``[H, 2*span, D]`` fused tables,
    ``force_generic``, ``check_cu_seqlens`` (validate the offsets on the host: one synchronisation,
    ``ValueError`` when they are malformed, exceed ``max_seqlen`` or do not end at the token count) and
    ``zero_output`` (see ``prepare``).  Relative positions are in-sequence offsets
    (ops/flash_attention_varlen.py:70,118); each key is masked by its own sequence's length.
    No host synchronisation is made unless ``check_cu_seqlens`` asks for one.  Returns ``o [total_tokens, H, D]``; forward only."""
    return FlashAttentionDisentangled.apply(q, k, v, q_pos, k_pos, cu_seqlens_q, cu_seqlens_k, max_seqlen_q,
                                            max_seqlen_k, causal, sm_scale, position_buckets,
                                            max_relative_distance, pos_key_layer, pos_query_layer, force_generic,
                                            check_cu_seqlens, zero_output)
