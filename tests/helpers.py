"""Shared builders for the parity tests: seeded inputs, oracle evaluation, comparison rules."""
from __future__ import annotations

import numpy as np
import torch

from oracle import hf_eager as O

# Tolerances of the parity bar: float32 outputs within 1e-4 relative, bfloat16 within 2e-2 max-abs.
FP32_REL = 1e-4
BF16_MAX_ABS = 2e-2


def span_of(buckets, max_rel):
    return buckets if buckets > 0 else max_rel


def make_inputs(seed, B, H, L, D, buckets, max_rel, dtype=torch.float32, scale=1.0, lengths=None):
    """Per-head tensors on the CPU, already rounded to ``dtype``."""
    g = torch.Generator().manual_seed(seed)
    span = span_of(buckets, max_rel)
    mk = lambda *s: (torch.randn(*s, generator=g) * scale).to(dtype)
    d = dict(q=mk(B, H, L, D), k=mk(B, H, L, D), v=mk(B, H, L, D), pk=mk(H, 2 * span, D), pq=mk(H, 2 * span, D))
    if lengths is not None:
        d["lengths"] = torch.as_tensor(lengths, dtype=torch.int32)
    return d


def oracle_fixed(inp, buckets, max_rel, pos_att_type=("c2p", "p2c"), dtype=torch.float32):
    """Oracle on the (already rounded) inputs, evaluated in ``dtype``; zeros on padded rows."""
    c = lambda t: None if t is None else t.to(dtype)
    pk = c(inp["pk"]) if "c2p" in pos_att_type else None
    pq = c(inp["pq"]) if "p2c" in pos_att_type else None
    return O.attention_lengths(c(inp["q"]), c(inp["k"]), c(inp["v"]), pk, pq, inp.get("lengths"),
                               position_buckets=buckets, max_relative_positions=max_rel,
                               pos_att_type=pos_att_type).float()


def assert_close_fp32(got, ref, what=""):
    got, ref = got.float().cpu(), ref.float().cpu()
    denom = ref.abs().max().clamp_min(1e-30)
    rel = ((got - ref).abs().max() / denom).item()
    assert rel <= FP32_REL, f"{what}: max relative error {rel:.3e} > {FP32_REL}"


def assert_close_bf16(got, ref, what="", tol=BF16_MAX_ABS):
    got, ref = got.float().cpu(), ref.float().cpu()
    err = (got - ref).abs().max().item()
    assert err <= tol, f"{what}: max abs error {err:.3e} > {tol}"


def pack(inp, lengths):
    """[B,H,L,D] -> packed [T,H,D] for q, k, v plus int32 cu_seqlens."""
    lengths = [int(x) for x in lengths]
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int32)
    out = {}
    for nm in ("q", "k", "v"):
        out[nm] = torch.cat([inp[nm][b, :, :n].transpose(0, 1) for b, n in enumerate(lengths)], 0).contiguous()
    return out, cu
