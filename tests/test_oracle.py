"""Pins the CPU oracle (oracle/hf_eager.py) against evidence that does not come from the oracle:
golden outputs written by Hugging Face's eager code, closed forms, a library routine (torch SDPA),
a float64 brute-force loop and structural invariants."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import hf_eager as O
from golden_inputs import LAYER_CASES, layer_inputs, span_of


# ------------------------------------------------------------------------------ bucket function

def _bucket_1d(lo, hi, buckets, max_pos):
    rel = torch.arange(lo, hi + 1, dtype=torch.long)
    return O.log_bucket_position(rel, buckets, max_pos).to(torch.long).numpy()


def test_bucket_matches_hf_golden_tables(golden_dir):
    g = np.load(os.path.join(golden_dir, "hf_bucket_table.npz"))
    for key in g.files:
        if not key.startswith("b"):
            continue
        buckets, max_pos, max_len = (int(x[1:]) for x in key.split("_"))
        got = _bucket_1d(-(max_len - 1), max_len - 1, buckets, max_pos)
        assert np.array_equal(got, g[key].astype(np.int64)), key
    m = O.relative_position(40, 40, 16, 32).numpy()
    assert np.array_equal(m, g["matrix_b16_p32_l40"].astype(np.int64))
    m = O.relative_position(40, 40, -1, 32).numpy()
    assert np.array_equal(m, g["matrix_nobucket_l40"].astype(np.int64))


def test_bucket_closed_forms_256_512():
    b = _bucket_1d(-4095, 4095, 256, 512)
    at = lambda r: int(b[r + 4095])
    for r in range(-128, 129):                       # identity zone
        assert at(r) == r
    assert [at(r) for r in range(129, 136)] == [129, 130, 131, 131, 132, 133, 133]
    assert [at(r) for r in range(505, 512)] == [254, 255, 255, 255, 255, 255, 255]
    assert at(511) == 255 and at(512) >= 256 and at(4095) == 446
    assert np.array_equal(b, -b[::-1])               # odd function
    assert np.all(np.diff(b) >= 0)                   # monotone
    assert len(np.unique(b[4095:4095 + 512])) == 256  # 256 distinct values on [0, 511]


def test_bucket_float64_margin_and_scalar_agreement():
    # float64 evaluation agrees everywhere, and the ceil argument stays >= 1e-4 from an integer
    # wherever the result is not clamped away, so no float32 log implementation can flip it.
    mid, P = 128, 512
    worst = 1.0
    for n in range(129, 511):
        x = math.log(n / mid) / math.log((P - 1) / mid) * (mid - 1)
        worst = min(worst, abs(x - round(x)))
    assert worst > 1e-3
    b = _bucket_1d(-4095, 4095, 256, 512)
    for r in list(range(-700, 701)) + [-4095, -2650, 1471, 2040, 4095]:
        assert int(b[r + 4095]) == O.bucket_scalar(r, 256, 512), r


def test_delta_table_is_clamped_bucket_plus_span():
    d = O.delta_table(4096, 256, 512)
    assert d.dtype == np.int32 and d.shape == (8191,)
    assert d.min() == 0 and d.max() == 511
    assert d[4095] == 256 and d[4095 + 511] == 511 and d[4095 + 512] == 511 and d[4095 - 512] == 0
    assert d[4095 - 511] == 1
    full = O.relative_position_index(300, 300, 256, 512).numpy()
    i, j = np.meshgrid(np.arange(300), np.arange(300), indexing="ij")
    assert np.array_equal(full, d[i - j + 4095])
    nb = O.delta_table(100, -1, 32)                  # no bucketing: clamp(r + 32, 0, 63)
    assert np.array_equal(nb, np.clip(np.arange(-99, 100) + 32, 0, 63))


# ------------------------------------------------------------------------------ attention maths

def _rand_heads(seed, B, H, L, D, span, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g) * scale
    return mk(B, H, L, D), mk(B, H, L, D), mk(B, H, L, D), mk(H, 2 * span, D), mk(H, 2 * span, D)


@pytest.mark.parametrize("buckets,max_rel,L,klen", [(4, 8, 14, None), (-1, 4, 12, None), (8, 16, 16, 9), (4, 64, 10, 1)])
def test_attention_equals_bruteforce(buckets, max_rel, L, klen):
    span = O.att_span(buckets, max_rel)
    q, k, v, pk, pq = _rand_heads(5, 1, 2, L, 8, span)
    lens = None if klen is None else torch.tensor([klen])
    out = O.attention_lengths(q, k, v, pk, pq, lens, position_buckets=buckets, max_relative_positions=max_rel)
    for h in range(2):
        ref = O.attention_bruteforce(q[0, h], k[0, h], v[0, h], pk[h], pq[h], klen,
                                     position_buckets=buckets, max_relative_positions=max_rel)
        n = L if klen is None else klen
        assert torch.allclose(out[0, h, :n].double(), ref[:n], atol=2e-6, rtol=1e-5)
        assert torch.all(out[0, h, n:] == 0)


@pytest.mark.parametrize("types", [("c2p",), ("p2c",)])
def test_single_term_equals_bruteforce(types):
    q, k, v, pk, pq = _rand_heads(6, 1, 1, 12, 8, 4)
    out = O.attention(q, k, v, pk, pq, None, position_buckets=4, max_relative_positions=8, pos_att_type=types)
    ref = O.attention_bruteforce(q[0, 0], k[0, 0], v[0, 0], pk[0], pq[0], None, position_buckets=4,
                                 max_relative_positions=8, pos_att_type=types)
    assert torch.allclose(out[0, 0].double(), ref, atol=2e-6, rtol=1e-5)


def test_zero_position_tables_reduce_to_sdpa():
    q, k, v, pk, pq = _rand_heads(7, 2, 3, 33, 16, 8)
    out = O.attention(q, k, v, torch.zeros_like(pk), torch.zeros_like(pq), None,
                      position_buckets=8, max_relative_positions=16)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, scale=1.0 / math.sqrt(3 * 16))
    assert torch.allclose(out, ref, atol=1e-6, rtol=1e-5)
    out = O.attention(q, k, v, None, None, None, pos_att_type=())
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v)        # 1/sqrt(d)
    assert torch.allclose(out, ref, atol=1e-6, rtol=1e-5)


def test_key_padding_mask_equals_sdpa_on_valid_rows():
    q, k, v, pk, pq = _rand_heads(8, 2, 2, 20, 16, 8)
    lens = torch.tensor([20, 7])
    out = O.attention_lengths(q, k, v, torch.zeros_like(pk), torch.zeros_like(pq), lens,
                              position_buckets=8, max_relative_positions=16)
    keep = (torch.arange(20)[None] < lens[:, None])[:, None, None, :]
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=keep, scale=1.0 / math.sqrt(48))
    assert torch.allclose(out[1, :, :7], ref[1, :, :7], atol=1e-6, rtol=1e-5)
    assert torch.allclose(out[0], ref[0], atol=1e-6, rtol=1e-5)


def test_toeplitz_invariant_and_probability_rows():
    # all query rows equal and all key rows equal => the score depends on i - j only
    _, _, v, pk, pq = _rand_heads(9, 1, 1, 24, 8, 8)
    q = torch.randn(8).expand(1, 1, 24, 8).contiguous()
    k = torch.randn(8).expand(1, 1, 24, 8).contiguous()
    _, probs = O.attention(q, k, v, pk, pq, None, position_buckets=8, max_relative_positions=16, return_probs=True)
    logit = torch.log(probs[0, 0])
    logit = logit - logit[:, :1] + logit[:1, :1]      # undo the per-row normaliser using column 0 ...
    assert torch.allclose(probs.sum(-1), torch.ones(1, 1, 24), atol=1e-6)
    bias = O.disentangled_bias(q, k, pk, pq, 8, 16, ("c2p", "p2c"))[0, 0]
    for off in range(-5, 6):
        d = torch.diagonal(bias, off)
        assert torch.allclose(d, d[:1].expand_as(d), atol=1e-6)


def test_p2c_index_convention_is_hf_not_mirrored():
    # HF gathers row j of K.Q_r^T at clamp(span - bucket(j - i)); the mirrored convention
    # clamp(span - bucket(i - j)) is a different matrix.  Keeps the index direction pinned.
    L, span = 6, 4
    g = torch.Generator().manual_seed(3)
    strip = torch.randn(L, 2 * span, generator=g)                    # K.Q_r^T for one head
    rel = O.relative_position(L, L, -1, span)
    hf_literal = torch.gather(strip, -1, torch.clamp(-rel + span, 0, 2 * span - 1)).t()
    same_delta = torch.stack([strip[j, torch.clamp(rel[:, j] + span, 0, 2 * span - 1)] for j in range(L)], 1)
    mirrored = torch.stack([strip[j, torch.clamp(-rel[:, j] + span, 0, 2 * span - 1)] for j in range(L)], 1)
    assert torch.equal(hf_literal, same_delta)
    assert not torch.equal(hf_literal, mirrored)


def test_single_key_sequence_returns_value_row():
    q, k, v, pk, pq = _rand_heads(10, 1, 2, 5, 8, 4)
    out = O.attention_lengths(q, k, v, pk, pq, torch.tensor([1]), position_buckets=4, max_relative_positions=8)
    assert torch.allclose(out[0, :, 0], v[0, :, 0], atol=1e-6)


def test_varlen_equals_per_sequence_fixed():
    H, D, span = 2, 8, 4
    lens = [5, 1, 9, 3]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    g = torch.Generator().manual_seed(4)
    q, k, v = (torch.randn(int(cu[-1]), H, D, generator=g) for _ in range(3))
    pk, pq = torch.randn(H, 2 * span, D, generator=g), torch.randn(H, 2 * span, D, generator=g)
    out = O.attention_varlen(q, k, v, pk, pq, cu, position_buckets=4, max_relative_positions=8)
    Lmax = max(lens)
    qp, kp, vp = (torch.zeros(len(lens), H, Lmax, D) for _ in range(3))
    for b, n in enumerate(lens):
        for dst, src in ((qp, q), (kp, k), (vp, v)):
            dst[b, :, :n] = src[cu[b]:cu[b + 1]].transpose(0, 1)
    ref = O.attention_lengths(qp, kp, vp, pk, pq, torch.tensor(lens), position_buckets=4, max_relative_positions=8)
    for b, n in enumerate(lens):
        assert torch.allclose(out[cu[b]:cu[b + 1]], ref[b, :, :n].transpose(0, 1), atol=1e-6)


# ------------------------------------------------------------------------------ HF golden outputs

def _oracle_layer(case, inp, dtype):
    t = lambda a: torch.from_numpy(a).to(dtype)
    mask4 = O.encoder_attention_mask(torch.from_numpy(inp["mask2d"]))
    kw = {}
    if not case["share"]:
        kw = dict(w_pos_key=t(inp["wpk"]), b_pos_key=t(inp["bpk"]), w_pos_query=t(inp["wpq"]), b_pos_query=t(inp["bpq"]))
    return O.self_attention_layer(t(inp["hidden"]), mask4, t(inp["rel_embeddings"]), t(inp["wq"]), t(inp["bq"]),
                                  t(inp["wk"]), t(inp["bk"]), t(inp["wv"]), t(inp["bv"]), case["heads"],
                                  position_buckets=case["buckets"], max_relative_positions=case["max_rel"],
                                  pos_att_type=case["pos_att_type"], **kw)


@pytest.mark.parametrize("name", sorted(LAYER_CASES))
def test_layer_matches_hf_golden(name, golden_dir):
    case = LAYER_CASES[name]
    inp = layer_inputs(case)
    gold = torch.from_numpy(np.load(os.path.join(golden_dir, "hf_layer_outputs.npz"))[name])
    dtype = torch.bfloat16 if case["dtype"] == "bf16" else torch.float32
    out = _oracle_layer(case, inp, dtype).float()
    valid = torch.from_numpy(inp["mask2d"]).bool()
    if case["dtype"] == "fp32":
        assert torch.allclose(out[valid], gold[valid], rtol=1e-5, atol=1e-6), (out - gold)[valid].abs().max()
    else:
        # same op order in the same dtype: only matmul blocking may differ
        assert (out[valid] - gold[valid]).abs().max() <= 2e-3


def test_mask_toy_matches_hf(golden_dir):
    g = np.load(os.path.join(golden_dir, "hf_mask_toy.npz"))
    m = torch.from_numpy(g["mask2d"])
    assert np.array_equal(O.encoder_attention_mask(m).numpy(), g["ext"])
    # padded QUERY rows: every score is finfo.min -> uniform softmax over all 8 keys
    probs = g["probs"]
    assert np.allclose(probs[0, :, 5:, :], 1.0 / 8)
    # valid rows put zero weight on padded keys
    assert np.all(probs[0, :, :5, 5:] == 0)
