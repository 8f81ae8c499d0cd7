"""Bit-exact use of the relative-position index by the matrix-core kernel (bf16 and fp16, head_dim 64).

The kernel turns i - j into a table row through its window / ring addressing; random data at bf16
tolerance would not notice one wrong row among thousands.  Here the tables are indicator functions of
the BITS of the index: head h marks every table row x whose bit h is set (score 0) and suppresses the
others (score -512), Q and K are unit vectors that pick the marked component and make Q.K^T vanish, and
V is +-1.  The output row of query i is then the plain average of V over the keys j whose delta(i - j)
has bit h set -- exact arithmetic up to the final rounding -- so it moves by about 1/count when a single
key is taken with a wrong index, while the rounding of the result is 2^-9 (bf16) of a value of size
1/sqrt(count).  Two different indices differ in some bit, so a wrong row shows in the head of that bit.

Expected values: delta(r) comes from the oracle's table (pinned against Hugging Face's own function in
test_oracle.py); the average itself is evaluated in float64 with torch.  The formula is tied back to the
oracle's full attention on the smallest case.  Reference for the index: modeling_deberta_v2.py:318,
:336-343 (both terms use the same delta)."""
import math

import numpy as np
import pytest
import torch

from oracle import hf_eager as O
from turbodeberta_amd.ops.flash_attention import flash_attention_with_disentangled
from turbodeberta_amd.ops.flash_attention_varlen import flash_attention_with_disentangled_varlen

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = 64
BIG = 512.0


def _tables(span, nbits, dtype):
    """pk[h, x, h] marks bit h of x; pq[h, x, 32 + h] marks bit (h + 3) % nbits of x."""
    x = torch.arange(2 * span)
    pk = torch.zeros(nbits, 2 * span, D)
    pq = torch.zeros(nbits, 2 * span, D)
    for h in range(nbits):
        pk[h, :, h] = torch.where((x >> h) & 1 == 1, 0.0, -BIG)
        pq[h, :, 32 + h] = torch.where((x >> ((h + 3) % nbits)) & 1 == 1, 0.0, -BIG)
    return pk.to(dtype), pq.to(dtype)


def _inputs(lengths, nbits, dtype, seed):
    """Packed q, k, v [T, H, D]: Q = e_h, K = e_{32+h} (so Q.K = 0, Q.pk[x] = pk[h, x, h], K.pq[x] = pq[h, x, 32+h])."""
    T = int(sum(lengths))
    g = torch.Generator().manual_seed(seed)
    q = torch.zeros(T, nbits, D)
    k = torch.zeros(T, nbits, D)
    for h in range(nbits):
        q[:, h, h] = 1.0
        k[:, h, 32 + h] = 1.0
    v = (torch.randint(0, 2, (T, nbits, D), generator=g) * 2 - 1).float()
    return q.to(dtype), k.to(dtype), v.to(dtype)


def _expected(v, lengths, span, nbits, buckets, max_rel, terms, wrong_row=None):
    """float64 [T, H, D]: softmax over the keys of each sequence of scale * (mark_c2p + mark_p2c)(delta(i - j)), times V.
    ``wrong_row = (r, d)``: pretend relative position r is looked up in table row d (to show what the bound notices)."""
    f = 1 + len(terms)
    scale = 1.0 / math.sqrt(D * f)
    out = torch.empty(v.shape, dtype=torch.float64, device=DEV)
    x = torch.arange(2 * span, device=DEV)
    start = 0
    for n in lengths:
        delta = torch.from_numpy(O.delta_table(n, buckets, max_rel).astype(np.int64)).to(DEV)      # entry r + n - 1
        if wrong_row is not None and abs(wrong_row[0]) < n:
            delta[wrong_row[0] + n - 1] = wrong_row[1]
        idx = (torch.arange(n, device=DEV)[:, None] - torch.arange(n, device=DEV)[None, :]) + n - 1
        dmat = delta[idx]                                                                            # [n, n] delta(i - j)
        for h in range(nbits):
            mark = torch.zeros(2 * span, dtype=torch.float64, device=DEV)
            if "c2p" in terms:
                mark += torch.where((x >> h) & 1 == 1, 0.0, -BIG).double()
            if "p2c" in terms:
                mark += torch.where((x >> ((h + 3) % nbits)) & 1 == 1, 0.0, -BIG).double()
            probs = torch.softmax(mark[dmat] * scale, dim=-1)
            out[start:start + n, h] = probs @ v[start:start + n, h].to(DEV).double()
        start += n
    return out


def _check(got, want, dtype, what):
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -10       # twice the rounding of the stored result
    err = (got.double() - want).abs()
    bound = ulp * want.abs() + 2e-6
    worst = (err / bound).max().item()
    assert worst <= 1.0, f"{what}: error / bound = {worst:.2f}"


CASES = [(300, [300, 129, 1, 64]), (640, [640, 300]), (4096, [4096, 700])]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("buckets,max_rel", [(256, 512), (-1, 512)], ids=["bucketed", "unbucketed"])
@pytest.mark.parametrize("L,lengths", CASES, ids=[f"L{c[0]}" for c in CASES])
def test_matrix_core_kernel_uses_exact_indices(dtype, buckets, max_rel, L, lengths):
    span = O.att_span(buckets, max_rel)
    nbits = int(math.log2(2 * span))
    pk, pq = _tables(span, nbits, dtype)
    q, k, v = _inputs(lengths, nbits, dtype, seed=L)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int32)
    g = lambda t: t.to(DEV)
    term_sets = [("c2p",), ("p2c",), ("c2p", "p2c")]       # each term alone shows every bit; together: the shared path
    for terms in term_sets:
        scale = 1.0 / math.sqrt(D * (1 + len(terms)))
        want = _expected(v, lengths, span, nbits, buckets, max_rel, terms)
        kw = dict(pos_key_layer=g(pk) if "c2p" in terms else None, pos_query_layer=g(pq) if "p2c" in terms else None)
        print(f"[case] index exactness packed {dtype} L={L} buckets={buckets} terms={terms}", flush=True)
        out = flash_attention_with_disentangled_varlen(g(q), g(k), g(v), None, None, g(cu), g(cu), L, L, False, scale,
                                                       buckets, max_rel, **kw)
        torch.cuda.synchronize()
        _check(out, want, dtype, f"packed {terms}")
        # the same sequences right-padded to L through the fixed-length operator
        B = len(lengths)
        pad = lambda t: torch.stack([torch.nn.functional.pad(t[int(cu[b]):int(cu[b + 1])], (0, 0, 0, 0, 0, L - lengths[b]))
                                     for b in range(B)]).permute(0, 2, 1, 3)            # [B, H, L, D]
        lens = torch.tensor(lengths, dtype=torch.int32)
        print(f"[case] index exactness fixed {dtype} L={L} buckets={buckets} terms={terms}", flush=True)
        outf = flash_attention_with_disentangled(g(pad(q)), g(pad(k)), g(pad(v)), None, None, False, scale, buckets,
                                                 max_rel, seqlens_k=g(lens), **kw)
        torch.cuda.synchronize()
        for b in range(B):
            s, e = int(cu[b]), int(cu[b + 1])
            _check(outf[b, :, :lengths[b]].permute(1, 0, 2), want[s:e], dtype, f"fixed seq {b} {terms}")


def test_expected_values_are_the_oracle():
    """The closed form used above equals the oracle's full attention on the same inputs (float32, small case)."""
    buckets, max_rel, lengths = 256, 512, [300]
    span, nbits = 256, 9
    pk, pq = _tables(span, nbits, torch.float32)
    q, k, v = _inputs(lengths, nbits, torch.float32, seed=1)
    want = _expected(v, lengths, span, nbits, buckets, max_rel, ("c2p", "p2c")).cpu()
    heads = lambda t: t.permute(1, 0, 2)[None]
    ref = O.attention(heads(q), heads(k), heads(v), pk, pq, None, position_buckets=buckets,
                      max_relative_positions=max_rel)[0].permute(1, 0, 2)
    assert (ref.double() - want).abs().max().item() <= 1e-5


@pytest.mark.parametrize("L,r", [(300, 5), (640, -200), (4096, 1500), (4096, -3)])
def test_bound_notices_one_wrong_row(L, r):
    """What the comparison above is worth: looking one relative position up in another table row moves the
    expected output beyond the bound, at every length tested (bf16 bound, the looser one)."""
    buckets, max_rel, span, nbits = 256, 512, 256, 9
    _, _, v = _inputs([L], nbits, torch.bfloat16, seed=L)
    right = _expected(v, [L], span, nbits, buckets, max_rel, ("c2p",))
    d = int(O.delta_table(L, buckets, max_rel)[r + L - 1])
    for flip in (1, 4, 64):                                       # another row: one bit of the index flipped
        wrong = _expected(v, [L], span, nbits, buckets, max_rel, ("c2p",), wrong_row=(r, d ^ flip))
        with pytest.raises(AssertionError):
            _check(wrong, right, torch.bfloat16, "one wrong row")
