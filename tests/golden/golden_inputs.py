"""Seeded inputs for the golden fixtures.  Shared by ``make_golden.py`` (which feeds them to
Hugging Face's eager DeBERTa-v2 code and stores the outputs) and by the tests (which feed the
same arrays to the oracle and to the HIP path).  Everything is drawn from
``numpy.random.RandomState`` so the stream never changes."""
from __future__ import annotations

import numpy as np

# name -> case description.  ``lengths`` None means an all-ones mask.
LAYER_CASES = {
    # BASELINE config 1: B2 x L128 x 768, 12 heads x 64, buckets 256 / max_rel 512, shared keys.
    "cfg1_fp32": dict(B=2, L=128, hidden=768, heads=12, buckets=256, max_rel=512, share=True,
                      pos_att_type=("c2p", "p2c"), dtype="fp32", lengths=None, bias=False, seed=0),
    "cfg1_bf16": dict(B=2, L=128, hidden=768, heads=12, buckets=256, max_rel=512, share=True,
                      pos_att_type=("c2p", "p2c"), dtype="bf16", lengths=None, bias=False, seed=0),
    "d64_fp32_masked": dict(B=2, L=96, hidden=256, heads=4, buckets=256, max_rel=512, share=True,
                            pos_att_type=("c2p", "p2c"), dtype="fp32", lengths=(96, 50), bias=True, seed=1),
    "tiny_fp32_masked": dict(B=2, L=24, hidden=64, heads=2, buckets=8, max_rel=16, share=True,
                             pos_att_type=("c2p", "p2c"), dtype="fp32", lengths=(24, 13), bias=True, seed=2),
    "noshare_fp32": dict(B=2, L=64, hidden=128, heads=2, buckets=16, max_rel=64, share=False,
                         pos_att_type=("c2p", "p2c"), dtype="fp32", lengths=(40, 64), bias=True, seed=3),
    "c2p_only_fp32": dict(B=1, L=48, hidden=128, heads=2, buckets=16, max_rel=64, share=True,
                          pos_att_type=("c2p",), dtype="fp32", lengths=None, bias=True, seed=4),
    "p2c_only_fp32": dict(B=1, L=48, hidden=128, heads=2, buckets=16, max_rel=64, share=True,
                          pos_att_type=("p2c",), dtype="fp32", lengths=None, bias=True, seed=5),
    "nopos_fp32": dict(B=1, L=48, hidden=128, heads=2, buckets=16, max_rel=64, share=True,
                       pos_att_type=(), dtype="fp32", lengths=(37,), bias=True, seed=6),
    "nobucket_fp32": dict(B=1, L=80, hidden=128, heads=2, buckets=-1, max_rel=32, share=True,
                          pos_att_type=("c2p", "p2c"), dtype="fp32", lengths=None, bias=True, seed=7),
    # sequence longer than max_rel: every |i-j| >= 512 saturates to index 0 / 2*span-1
    "far_fp32": dict(B=1, L=640, hidden=64, heads=1, buckets=256, max_rel=512, share=True,
                     pos_att_type=("c2p", "p2c"), dtype="fp32", lengths=None, bias=False, seed=8),
}


def span_of(case) -> int:
    return case["buckets"] if case["buckets"] > 0 else case["max_rel"]


def layer_inputs(case) -> dict:
    """hidden ~ N(0,1), rel_embeddings ~ N(0,1), weights ~ N(0,0.02), biases ~ N(0,0.02) or 0."""
    rs = np.random.RandomState(case["seed"])
    B, L, hid = case["B"], case["L"], case["hidden"]
    f32 = np.float32
    out = {
        "hidden": rs.standard_normal((B, L, hid)).astype(f32),
        "rel_embeddings": rs.standard_normal((2 * span_of(case), hid)).astype(f32),
    }
    for nm in ("q", "k", "v", "pk", "pq"):
        out["w" + nm] = (0.02 * rs.standard_normal((hid, hid))).astype(f32)
        b = (0.02 * rs.standard_normal((hid,))).astype(f32)
        out["b" + nm] = b if case["bias"] else np.zeros_like(b)
    lengths = case["lengths"] if case["lengths"] is not None else (L,) * B
    out["lengths"] = np.asarray(lengths, dtype=np.int32)
    out["mask2d"] = (np.arange(L)[None, :] < out["lengths"][:, None]).astype(np.int64)
    return out


def tiny_model_config() -> dict:
    """Keyword arguments of a 2-layer DeBERTa-v3-style config (rel-embedding LayerNorm on)."""
    return dict(vocab_size=100, hidden_size=128, num_hidden_layers=2, num_attention_heads=2,
                intermediate_size=256, hidden_act="gelu", hidden_dropout_prob=0.0,
                attention_probs_dropout_prob=0.0, max_position_embeddings=64, type_vocab_size=0,
                relative_attention=True, position_buckets=16, max_relative_positions=64,
                share_att_key=True, pos_att_type=["c2p", "p2c"], norm_rel_ebd="layer_norm",
                position_biased_input=False, layer_norm_eps=1e-7, pad_token_id=0)


def tiny_model_inputs():
    rs = np.random.RandomState(11)
    ids = rs.randint(1, 100, size=(3, 40)).astype(np.int64)
    lengths = np.array([40, 23, 1], dtype=np.int64)
    mask = (np.arange(40)[None, :] < lengths[:, None]).astype(np.int64)
    ids = ids * mask
    return ids, mask


def fill_params(model, seed: int = 12) -> None:
    """Overwrite every parameter, in sorted-name order, with seeded values: matrices ~ N(0,0.05),
    vectors ~ 1 + N(0,0.05) when the name says LayerNorm weight, else N(0,0.05)."""
    import torch

    rs = np.random.RandomState(seed)
    with torch.no_grad():
        for name, p in sorted(model.named_parameters(), key=lambda kv: kv[0]):
            val = (0.05 * rs.standard_normal(tuple(p.shape))).astype(np.float32)
            if name.endswith("LayerNorm.weight"):
                val = val + 1.0
            p.copy_(torch.from_numpy(val))
