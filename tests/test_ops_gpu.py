"""Parity of the HIP kernels (called through the C ABI by the Python operators) against the CPU
oracle and against golden outputs written by Hugging Face's eager code.

Bar: float32 outputs within 1e-4 relative of the oracle; bfloat16 within 2e-2 max-abs of the
bfloat16 eager oracle (and much closer to the float32 oracle evaluated on the same rounded inputs);
relative-position indices bit exact (host tables are checked in test_capi_cpu.py; here the kernel's
use of them is pinned by one-hot position tables that make the output reveal the index)."""
import math
import os

import numpy as np
import pytest
import torch

from helpers import (assert_close_bf16, assert_close_fp32, make_inputs, oracle_fixed, pack, span_of)
from golden_inputs import LAYER_CASES, layer_inputs
from oracle import hf_eager as O

pytestmark = pytest.mark.gpu

from turbodeberta_amd.ops.flash_attention import flash_attention_with_disentangled
from turbodeberta_amd.ops.flash_attention_varlen import flash_attention_with_disentangled_varlen

DEV = "cuda:0"


def run_fixed(inp, buckets, max_rel, pos_att_type=("c2p", "p2c"), **kw):
    g = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in inp.items()}
    D = inp["q"].shape[-1]
    f = O.scale_factor_of(pos_att_type)
    print(f"[case] fixed q={tuple(inp['q'].shape)} {inp['q'].dtype} buckets={buckets} max_rel={max_rel} "
          f"types={pos_att_type} kw={list(kw)}", flush=True)
    out = flash_attention_with_disentangled(
        g["q"], g["k"], g["v"], None, None, False, 1.0 / math.sqrt(D * f), buckets, max_rel,
        pos_key_layer=g["pk"] if "c2p" in pos_att_type else None,
        pos_query_layer=g["pq"] if "p2c" in pos_att_type else None,
        seqlens_k=g.get("lengths"), **kw)
    torch.cuda.synchronize()
    return out.cpu()


# ------------------------------------------------------------------ float32: 1e-4 relative

@pytest.mark.parametrize("B,H,L,D,buckets,max_rel,lengths", [
    (2, 12, 128, 64, 256, 512, None),            # config-1 head shapes
    (2, 3, 1, 64, 256, 512, None),
    (1, 2, 5, 8, 4, 8, None),
    (2, 2, 17, 32, 8, 16, (17, 9)),
    (3, 2, 63, 64, 16, 64, (63, 1, 40)),
    (1, 2, 65, 128, 16, 64, None),
    (1, 1, 100, 256, -1, 32, (77,)),
    (1, 2, 200, 72, 32, 128, None),
    (1, 1, 640, 64, 256, 512, None),             # beyond max_rel: saturated indices
])
def test_fp32_fixed_vs_oracle(B, H, L, D, buckets, max_rel, lengths):
    inp = make_inputs(1, B, H, L, D, buckets, max_rel, lengths=lengths)
    ref = oracle_fixed(inp, buckets, max_rel)
    assert_close_fp32(run_fixed(inp, buckets, max_rel), ref, "fp32 fixed")


def test_fp32_sharp_softmax():
    # large logits: the softmax is far from uniform, so an index or sign error moves the output a lot
    inp = make_inputs(2, 1, 2, 96, 64, 256, 512, scale=3.0)
    ref = oracle_fixed(inp, 256, 512)
    assert_close_fp32(run_fixed(inp, 256, 512), ref, "fp32 sharp")


@pytest.mark.parametrize("types", [("c2p",), ("p2c",), ()])
def test_fp32_term_subsets(types):
    inp = make_inputs(3, 1, 2, 80, 64, 16, 64)
    ref = oracle_fixed(inp, 16, 64, pos_att_type=types)
    assert_close_fp32(run_fixed(inp, 16, 64, pos_att_type=types), ref, f"fp32 {types}")


def test_index_exactness_via_one_hot_tables():
    # K_r[x] = e_x-like rows make c2p(i,j) = Q_i[delta mod D] * [delta // D == block]: any wrong
    # delta changes which query component is read.  Values are exactly representable, scores small.
    B, H, L, D, buckets, max_rel = 1, 1, 300, 64, 256, 512
    span = 256
    inp = make_inputs(4, B, H, L, D, buckets, max_rel)
    pk = torch.zeros(H, 2 * span, D)
    pq = torch.zeros(H, 2 * span, D)
    for x in range(2 * span):
        pk[0, x, x % D] = 1.0 + (x // D)
        pq[0, x, (7 * x) % D] = 1.0 + (x // D)
    inp["pk"], inp["pq"] = pk, pq
    ref = oracle_fixed(inp, buckets, max_rel)
    assert_close_fp32(run_fixed(inp, buckets, max_rel), ref, "one-hot tables")


def test_fp32_strips_equal_fused():
    B, H, L, D, buckets, max_rel = 2, 2, 70, 64, 16, 64
    inp = make_inputs(5, B, H, L, D, buckets, max_rel, lengths=(70, 33))
    ref = oracle_fixed(inp, buckets, max_rel)
    g = {k: v.to(DEV) for k, v in inp.items()}
    c2p = torch.matmul(g["q"], g["pk"].transpose(-1, -2)[None])       # the strips the reference glue builds
    p2c = torch.matmul(g["k"], g["pq"].transpose(-1, -2)[None])
    print("[case] fixed strips", flush=True)
    out = flash_attention_with_disentangled(g["q"], g["k"], g["v"], c2p, p2c, False, 1 / math.sqrt(3 * D),
                                            buckets, max_rel, seqlens_k=g["lengths"])
    assert_close_fp32(out.cpu(), ref, "strip mode")


def test_fp32_strided_views_no_copy():
    B, H, L, D = 2, 3, 50, 64
    inp = make_inputs(6, B, H, L, D, 16, 64)
    ref = oracle_fixed(inp, 16, 64)
    g = {k: v.to(DEV) for k, v in inp.items()}
    # [B, L, H, D] storage viewed as [B, H, L, D], as a projection output would be
    q, k, v = (g[n].permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3) for n in "qkv")
    assert not q.is_contiguous()
    print("[case] fixed strided", flush=True)
    out = flash_attention_with_disentangled(q, k, v, None, None, False, 1 / math.sqrt(3 * D), 16, 64,
                                            pos_key_layer=g["pk"], pos_query_layer=g["pq"])
    assert out.stride() == q.stride()
    assert_close_fp32(out.cpu(), ref, "strided")


def test_fp32_varlen_vs_oracle():
    H, D, buckets, max_rel = 2, 64, 16, 64
    lengths = [37, 1, 64, 16, 17, 90]
    inp = make_inputs(7, len(lengths), H, max(lengths), D, buckets, max_rel)
    packed, cu = pack(inp, lengths)
    ref = O.attention_varlen(packed["q"], packed["k"], packed["v"], inp["pk"], inp["pq"], cu,
                             position_buckets=buckets, max_relative_positions=max_rel)
    print("[case] varlen fused", flush=True)
    out = flash_attention_with_disentangled_varlen(
        packed["q"].to(DEV), packed["k"].to(DEV), packed["v"].to(DEV), None, None, cu.to(DEV), cu.to(DEV),
        max(lengths), max(lengths), False, 1 / math.sqrt(3 * D), buckets, max_rel,
        pos_key_layer=inp["pk"].to(DEV), pos_query_layer=inp["pq"].to(DEV))
    assert_close_fp32(out.cpu(), ref, "varlen")
    # strips, packed
    c2p = torch.einsum("thd,hmd->thm", packed["q"], inp["pk"]).to(DEV)
    p2c = torch.einsum("thd,hmd->thm", packed["k"], inp["pq"]).to(DEV)
    print("[case] varlen strips", flush=True)
    out2 = flash_attention_with_disentangled_varlen(
        packed["q"].to(DEV), packed["k"].to(DEV), packed["v"].to(DEV), c2p, p2c, cu.to(DEV), cu.to(DEV),
        max(lengths), max(lengths), False, 1 / math.sqrt(3 * D), buckets, max_rel)
    assert_close_fp32(out2.cpu(), ref, "varlen strips")


def test_varlen_with_empty_sequences_and_default_scale():
    H, D = 1, 64
    lengths = [0, 5, 0, 3]
    inp = make_inputs(8, 4, H, 5, D, 4, 8)
    packed, cu = pack(inp, lengths)
    ref = O.attention_varlen(packed["q"], packed["k"], packed["v"], None, None, cu, pos_att_type=())
    print("[case] varlen empty seqs", flush=True)
    out = flash_attention_with_disentangled_varlen(packed["q"].to(DEV), packed["k"].to(DEV), packed["v"].to(DEV),
                                                   None, None, cu.to(DEV), cu.to(DEV), 5, 5)
    assert_close_fp32(out.cpu(), ref, "varlen empty")          # sm_scale=None -> 1/sqrt(D)


# ------------------------------------------------------------------ golden outputs from HF eager

def _run_layer(case, inp, dtype):
    t = lambda a: torch.from_numpy(a).to(DEV, dtype)
    lin = torch.nn.functional.linear
    heads, span = case["heads"], span_of(case["buckets"], case["max_rel"])
    hidden, rel = t(inp["hidden"]), t(inp["rel_embeddings"])[: 2 * span]
    B, L, hid = hidden.shape
    split = lambda x: x.view(B, L, heads, -1).permute(0, 2, 1, 3)          # view, no copy
    q, k, v = split(lin(hidden, t(inp["wq"]), t(inp["bq"]))), split(lin(hidden, t(inp["wk"]), t(inp["bk"]))), \
        split(lin(hidden, t(inp["wv"]), t(inp["bv"])))
    wpk, bpk = (t(inp["wk"]), t(inp["bk"])) if case["share"] else (t(inp["wpk"]), t(inp["bpk"]))
    wpq, bpq = (t(inp["wq"]), t(inp["bq"])) if case["share"] else (t(inp["wpq"]), t(inp["bpq"]))
    types = case["pos_att_type"]
    pk = lin(rel, wpk, bpk).view(2 * span, heads, -1).permute(1, 0, 2).contiguous() if "c2p" in types else None
    pq = lin(rel, wpq, bpq).view(2 * span, heads, -1).permute(1, 0, 2).contiguous() if "p2c" in types else None
    D = q.shape[-1]
    lens = torch.from_numpy(inp["lengths"]).to(DEV)
    print(f"[case] golden layer {case}", flush=True)
    out = flash_attention_with_disentangled(q, k, v, None, None, False, 1 / math.sqrt(D * O.scale_factor_of(types)),
                                            case["buckets"], case["max_rel"], pos_key_layer=pk, pos_query_layer=pq,
                                            seqlens_k=lens)
    return out.permute(0, 2, 1, 3).reshape(B, L, hid).float().cpu()


@pytest.mark.parametrize("name", sorted(LAYER_CASES))
def test_layer_matches_hf_golden(name, golden_dir):
    case = LAYER_CASES[name]
    inp = layer_inputs(case)
    gold = torch.from_numpy(np.load(os.path.join(golden_dir, "hf_layer_outputs.npz"))[name])
    valid = torch.from_numpy(inp["mask2d"]).bool()
    if case["dtype"] == "fp32":
        out = _run_layer(case, inp, torch.float32)
        assert_close_fp32(out[valid], gold[valid], name)
    else:
        out = _run_layer(case, inp, torch.bfloat16)
        assert_close_bf16(out[valid], gold[valid], name)
    assert torch.all(out[~valid] == 0)


# ------------------------------------------------------------------ bfloat16: 2e-2 max-abs

@pytest.mark.parametrize("force_generic", [False, True])
@pytest.mark.parametrize("B,H,L,buckets,max_rel,lengths", [
    (2, 12, 128, 256, 512, None),
    (2, 2, 512, 256, 512, (512, 389)),
    (1, 2, 1, 256, 512, None),
    (3, 1, 129, 256, 512, (129, 64, 3)),
    (1, 2, 300, 32, 128, None),
    (1, 1, 333, -1, 64, (250,)),
    (1, 1, 1100, 256, 512, None),
    (1, 1, 2200, 256, 512, (2111,)),        # long enough for the instance with far key steps
])
def test_bf16_fixed_vs_oracle(B, H, L, buckets, max_rel, lengths, force_generic):
    inp = make_inputs(9, B, H, L, 64, buckets, max_rel, dtype=torch.bfloat16, lengths=lengths)
    out = run_fixed(inp, buckets, max_rel, force_generic=force_generic)
    ref32 = oracle_fixed(inp, buckets, max_rel, dtype=torch.float32)
    assert_close_bf16(out, ref32, "bf16 vs fp32 oracle on rounded inputs", tol=1e-2)
    if L <= 512:
        ref16 = oracle_fixed(inp, buckets, max_rel, dtype=torch.bfloat16)
        assert_close_bf16(out, ref16, "bf16 vs bf16 eager oracle")


@pytest.mark.parametrize("force_generic", [False, True])
def test_bf16_varlen_vs_oracle(force_generic):
    H, D, buckets, max_rel = 4, 64, 256, 512
    rs = np.random.RandomState(0)
    lengths = [int(x) for x in rs.randint(16, 513, size=12)] + [1, 128, 129]
    inp = make_inputs(10, len(lengths), H, max(lengths), D, buckets, max_rel, dtype=torch.bfloat16)
    packed, cu = pack(inp, lengths)
    f = lambda t: t.float()
    ref = O.attention_varlen(f(packed["q"]), f(packed["k"]), f(packed["v"]), f(inp["pk"]), f(inp["pq"]), cu,
                             position_buckets=buckets, max_relative_positions=max_rel)
    print(f"[case] bf16 varlen generic={force_generic} lengths={lengths}", flush=True)
    out = flash_attention_with_disentangled_varlen(
        packed["q"].to(DEV), packed["k"].to(DEV), packed["v"].to(DEV), None, None, cu.to(DEV), cu.to(DEV),
        max(lengths), max(lengths), False, 1 / math.sqrt(3 * D), buckets, max_rel,
        pos_key_layer=inp["pk"].to(DEV), pos_query_layer=inp["pq"].to(DEV), force_generic=force_generic)
    assert_close_bf16(out.cpu(), ref, "bf16 varlen", tol=1e-2)


@pytest.mark.parametrize("force_generic", [False, True])
def test_bf16_varlen_more_than_64_sequences(force_generic):
    """150 short sequences, more than the 64 whose boundaries a wave holds in its lanes: the matrix-core path goes out
    as three launches of 50 (the result must equal, bit for bit, what separate calls on the three parts give), the
    vector-ALU kernel scans the boundaries in chunks of 64."""
    H, D, buckets, max_rel = 2, 64, 256, 512
    rs = np.random.RandomState(4)
    lengths = [int(x) for x in rs.randint(1, 200, size=150)]
    lengths[70], lengths[140] = 0, 130
    inp = make_inputs(11, len(lengths), H, max(lengths), D, buckets, max_rel, dtype=torch.bfloat16)
    packed, cu = pack(inp, lengths)
    f = lambda t: t.float()
    ref = O.attention_varlen(f(packed["q"]), f(packed["k"]), f(packed["v"]), f(inp["pk"]), f(inp["pq"]), cu,
                             position_buckets=buckets, max_relative_positions=max_rel)
    print(f"[case] bf16 varlen 150 sequences generic={force_generic}", flush=True)
    out = flash_attention_with_disentangled_varlen(
        packed["q"].to(DEV), packed["k"].to(DEV), packed["v"].to(DEV), None, None, cu.to(DEV), cu.to(DEV),
        max(lengths), max(lengths), False, 1 / math.sqrt(3 * D), buckets, max_rel,
        pos_key_layer=inp["pk"].to(DEV), pos_query_layer=inp["pq"].to(DEV), force_generic=force_generic)
    assert_close_bf16(out.cpu(), ref, "bf16 varlen, 150 sequences", tol=1e-2)
    if not force_generic:
        for first in (0, 50, 100):
            lo, hi = int(cu[first]), int(cu[first + 50])
            part_cu = (cu[first:first + 51] - cu[first]).to(DEV)
            part = flash_attention_with_disentangled_varlen(
                packed["q"][lo:hi].to(DEV), packed["k"][lo:hi].to(DEV), packed["v"][lo:hi].to(DEV), None, None, part_cu,
                part_cu, max(lengths), max(lengths), False, 1 / math.sqrt(3 * D), buckets, max_rel,
                pos_key_layer=inp["pk"].to(DEV), pos_query_layer=inp["pq"].to(DEV))
            assert torch.equal(part, out[lo:hi]), f"sequences {first}..{first + 49}"


def test_repeated_launches_are_bit_identical():
    """The kernels have no atomics and no order-dependent reduction: the same launch must give the same bits every
    time.  A difference between repetitions would mean a race between the waves of a workgroup (a missing barrier,
    an LDS slot overwritten early) that the parity tolerances could hide.  Fixed layout with ragged lengths, packed
    batch, and a sequence long enough for the instances with far key steps, 100 launches each."""
    H, D, buckets, max_rel = 12, 64, 256, 512
    rs = np.random.RandomState(5)
    lengths = [int(x) for x in rs.randint(16, 513, size=24)]
    inp = make_inputs(31, len(lengths), H, 512, D, buckets, max_rel, dtype=torch.bfloat16, lengths=lengths)
    dev = {k: inp[k].to(DEV) for k in ("q", "k", "v", "pk", "pq")}
    seqlens = torch.tensor(lengths, dtype=torch.int32, device=DEV)
    packed, cu = pack(inp, lengths)
    pdev = {k: packed[k].to(DEV) for k in ("q", "k", "v")}
    cud = cu.to(DEV)
    long_inp = make_inputs(32, 1, 2, 2304, D, buckets, max_rel, dtype=torch.bfloat16)
    ldev = {k: long_inp[k].to(DEV) for k in ("q", "k", "v", "pk", "pq")}
    scale = 1 / math.sqrt(3 * D)
    runs = {
        "fixed": lambda: flash_attention_with_disentangled(dev["q"], dev["k"], dev["v"], None, None, False, scale, buckets, max_rel,
                                                           pos_key_layer=dev["pk"], pos_query_layer=dev["pq"], seqlens_k=seqlens),
        "packed": lambda: flash_attention_with_disentangled_varlen(pdev["q"], pdev["k"], pdev["v"], None, None, cud, cud, 512, 512,
                                                                   False, scale, buckets, max_rel, pos_key_layer=dev["pk"],
                                                                   pos_query_layer=dev["pq"]),
        "long": lambda: flash_attention_with_disentangled(ldev["q"], ldev["k"], ldev["v"], None, None, False, scale, buckets,
                                                          max_rel, pos_key_layer=ldev["pk"], pos_query_layer=ldev["pq"]),
    }
    for name, run in runs.items():
        print(f"[case] repeated launches, {name}", flush=True)
        first = run().clone()
        for rep in range(100):
            assert torch.equal(run(), first), f"{name}: launch {rep + 2} differs from the first"


def test_packed_tile_deal_at_other_grid_sizes():
    """The packed launch deals its tiles to the persistent workgroups inside the kernel.  Grids of 8, 24 and 40
    workgroups and the full device must all produce every tile:
    the output is zero-filled first, so a tile that nobody took would stay zero, and each result must equal the
    full-grid one bit for bit (a tile's arithmetic does not depend on who computes it)."""
    from turbodeberta_amd import _lib
    H, D, buckets, max_rel = 16, 64, 256, 512
    rs = np.random.RandomState(7)
    lengths = [int(x) for x in rs.randint(1, 260, size=64)]
    for i in (0, 5, 31, 63):
        lengths[i] = 0
    lengths[17] = 300
    inp = make_inputs(21, len(lengths), H, max(lengths), D, buckets, max_rel, dtype=torch.bfloat16)
    packed, cu = pack(inp, lengths)
    f = lambda t: t.float()
    ref = O.attention_varlen(f(packed["q"]), f(packed["k"]), f(packed["v"]), f(inp["pk"]), f(inp["pq"]), cu,
                             position_buckets=buckets, max_relative_positions=max_rel)
    dev = {k: packed[k].to(DEV) for k in ("q", "k", "v")}
    run = lambda: flash_attention_with_disentangled_varlen(
        dev["q"], dev["k"], dev["v"], None, None, cu.to(DEV), cu.to(DEV), max(lengths), max(lengths), False,
        1 / math.sqrt(3 * D), buckets, max_rel, pos_key_layer=inp["pk"].to(DEV), pos_query_layer=inp["pq"].to(DEV))
    try:
        print("[case] packed deal, full grid", flush=True)
        assert _lib.set_workgroup_limit(0) == 0
        full = run()
        assert_close_bf16(full.cpu(), ref, "packed deal, full grid")
        for grid in (8, 24, 40, 250):
            print(f"[case] packed deal, at most {grid} workgroups", flush=True)
            assert _lib.set_workgroup_limit(grid) == grid // 8 * 8
            assert torch.equal(run(), full), f"grid {grid}"
    finally:
        _lib.set_workgroup_limit(0)


@pytest.mark.parametrize("force_generic", [False, True])
@pytest.mark.parametrize("B,H,L,buckets,max_rel,lengths", [
    (2, 4, 512, 256, 512, (512, 389)),
    (3, 1, 129, 256, 512, (129, 64, 3)),
    (1, 2, 300, 32, 128, None),
    (1, 1, 1100, 256, 512, None),
    (1, 1, 2200, 256, 512, (2111,)),
])
def test_fp16_fixed_vs_oracle(B, H, L, buckets, max_rel, lengths, force_generic):
    """float16 inputs take the matrix-core kernel too (fp16 MFMA, fp32 accumulation); 11 significant bits give a
    tighter bound than bfloat16."""
    inp = make_inputs(12, B, H, L, 64, buckets, max_rel, dtype=torch.float16, lengths=lengths)
    out = run_fixed(inp, buckets, max_rel, force_generic=force_generic)
    assert out.dtype == torch.float16
    ref32 = oracle_fixed(inp, buckets, max_rel, dtype=torch.float32)
    assert_close_bf16(out, ref32, "fp16 vs fp32 oracle on rounded inputs", tol=2e-3)


def test_fp16_varlen_matrix_core_equals_vector_alu():
    H, D, buckets, max_rel = 4, 64, 256, 512
    rs = np.random.RandomState(2)
    lengths = [int(x) for x in rs.randint(16, 513, size=10)] + [1, 128, 129]
    inp = make_inputs(13, len(lengths), H, max(lengths), D, buckets, max_rel, dtype=torch.float16)
    packed, cu = pack(inp, lengths)
    f = lambda t: t.float()
    ref = O.attention_varlen(f(packed["q"]), f(packed["k"]), f(packed["v"]), f(inp["pk"]), f(inp["pq"]), cu,
                             position_buckets=buckets, max_relative_positions=max_rel)
    outs = []
    for gen in (False, True):
        print(f"[case] fp16 varlen generic={gen}", flush=True)
        outs.append(flash_attention_with_disentangled_varlen(
            packed["q"].to(DEV), packed["k"].to(DEV), packed["v"].to(DEV), None, None, cu.to(DEV), cu.to(DEV),
            max(lengths), max(lengths), False, 1 / math.sqrt(3 * D), buckets, max_rel,
            pos_key_layer=inp["pk"].to(DEV), pos_query_layer=inp["pq"].to(DEV), force_generic=gen).cpu())
        assert_close_bf16(outs[-1], ref, f"fp16 varlen generic={gen}", tol=2e-3)


# ------------------------------------------------------------------ padded batches in the projection layout

def _as_projection_output(t):
    """The same values stored as [B, L, H, D] and viewed as [B, H, L, D]: what a projection followed by a head split
    gives."""
    return t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,L,lengths", [
    (5, 3, 400, (400, 1, 129, 256, 37)),        # whole tiles of padding (zeros from the up-front fill) and partial ones
    (2, 12, 512, (512, 389)),
    (3, 2, 128, (0, 128, 5)),                   # an empty sequence
    (70, 1, 130, None),                         # more than 64 sequences: several launches
    (2, 1, 2200, (2111, 1700)),                 # the instances with far key steps
])
def test_padded_projection_layout_equals_head_major_layout(B, H, L, lengths, dtype):
    """A right-padded batch (a call with lengths: its tiles are dealt like those of packed sequences, its rows addressed
    through the batch strides) gives the same bits whether its tensors are stored [B, L, H, D] or [B, H, L, D], and
    matches the oracle; padded rows are zeros in both, whole tiles of them included."""
    buckets, max_rel = 256, 512
    if lengths is None:
        lengths = tuple(int(x) for x in np.random.RandomState(B).randint(0, L + 1, size=B))
    inp = make_inputs(31, B, H, L, 64, buckets, max_rel, dtype=dtype, lengths=lengths)
    head_major = run_fixed(inp, buckets, max_rel)
    proj = dict(inp)
    for n in "qkv":
        proj[n] = _as_projection_output(inp[n])
        assert proj[n].stride(0) == L * proj[n].stride(2)
    row_major = run_fixed(proj, buckets, max_rel)
    assert torch.equal(row_major, head_major)
    for b, n in enumerate(lengths):
        assert torch.all(row_major[b, :, n:] == 0)
    if L <= 512 and B <= 8:
        ref = oracle_fixed(inp, buckets, max_rel, dtype=torch.float32)
        assert_close_bf16(row_major, ref, "padded projection layout vs fp32 oracle", tol=1e-2 if dtype == torch.bfloat16 else 2e-3)


def test_padded_batch_at_other_grid_sizes():
    """A padded batch with whole tiles of padding at grids of 8, 40 and 248 workgroups: the deal and the up-front fill of
    the padded tiles are both strided over the grid, and every grid must give the full-grid result bit for bit (the
    output is allocated uninitialised, so a tile nobody filled would show)."""
    from turbodeberta_amd import _lib
    B, H, L, buckets, max_rel = 9, 5, 500, 256, 512
    lengths = (500, 0, 3, 128, 129, 257, 384, 40, 499)
    inp = make_inputs(33, B, H, L, 64, buckets, max_rel, dtype=torch.bfloat16, lengths=lengths)
    try:
        assert _lib.set_workgroup_limit(0) == 0
        full = run_fixed(inp, buckets, max_rel)
        assert_close_bf16(full, oracle_fixed(inp, buckets, max_rel, dtype=torch.float32), "padded batch, full grid", tol=1e-2)
        for b, n in enumerate(lengths):
            assert torch.all(full[b, :, n:] == 0)
        for grid in (8, 40, 248):
            assert _lib.set_workgroup_limit(grid) == grid
            garbage = torch.full((64, 1024, 1024), 7.0, device=DEV)          # what the next allocations will reuse
            del garbage
            assert torch.equal(run_fixed(inp, buckets, max_rel), full), f"grid {grid}"
    finally:
        _lib.set_workgroup_limit(0)


def test_padded_projection_layout_with_strips():
    B, H, L, buckets, max_rel = 4, 2, 300, 256, 512
    lengths = (300, 40, 170, 129)
    inp = make_inputs(32, B, H, L, 64, buckets, max_rel, dtype=torch.bfloat16, lengths=lengths)
    c2p, p2c = _strips(inp)
    head_major = _run_strips(inp, c2p, p2c, buckets, max_rel)
    proj = dict(inp)
    for n in "qkv":
        proj[n] = _as_projection_output(inp[n])
    row_major = _run_strips(proj, _as_projection_output(c2p), _as_projection_output(p2c), buckets, max_rel)
    assert torch.equal(row_major, head_major)
    for b, n in enumerate(lengths):
        assert torch.all(row_major[b, :, n:] == 0)


# ------------------------------------------------------------------ 16-bit strips (the reference's own operator signature)

def _strips(inp, types=("c2p", "p2c")):
    """The strips the reference glue hands to its kernel (model.py:122-125, :146-148): Q.K_r^T and K.Q_r^T, computed
    and rounded in the element type."""
    c2p = torch.matmul(inp["q"], inp["pk"].transpose(-1, -2)[None]) if "c2p" in types else None
    p2c = torch.matmul(inp["k"], inp["pq"].transpose(-1, -2)[None]) if "p2c" in types else None
    return c2p, p2c


def _run_strips(inp, c2p, p2c, buckets, max_rel, n_terms=2, **kw):
    dev = lambda t: None if t is None else t.to(DEV)
    D = inp["q"].shape[-1]
    print(f"[case] fixed strips q={tuple(inp['q'].shape)} {inp['q'].dtype} buckets={buckets} max_rel={max_rel} "
          f"c2p={c2p is not None} p2c={p2c is not None} kw={kw}", flush=True)
    out = flash_attention_with_disentangled(dev(inp["q"]), dev(inp["k"]), dev(inp["v"]), dev(c2p), dev(p2c), False,
                                            1.0 / math.sqrt(D * (1 + n_terms)), buckets, max_rel,
                                            seqlens_k=dev(inp.get("lengths")), **kw)
    torch.cuda.synchronize()
    return out.cpu()


@pytest.mark.parametrize("force_generic", [False, True])
@pytest.mark.parametrize("B,H,L,buckets,max_rel,lengths", [
    (2, 12, 128, 256, 512, None),
    (2, 2, 512, 256, 512, (512, 389)),
    (1, 2, 1, 256, 512, None),
    (3, 1, 129, 256, 512, (129, 64, 3)),
    (1, 2, 300, 32, 128, None),
    (1, 1, 333, -1, 64, (250,)),
    (1, 1, 1100, 256, 512, None),
])
def test_bf16_strips_fixed_vs_oracle(B, H, L, buckets, max_rel, lengths, force_generic):
    """Strips in bf16, as Hugging Face's eager code holds them before its gather: the bf16 eager oracle is the same
    computation, the fp32 oracle differs by the rounding of the strips."""
    inp = make_inputs(21, B, H, L, 64, buckets, max_rel, dtype=torch.bfloat16, lengths=lengths)
    c2p, p2c = _strips(inp)
    out = _run_strips(inp, c2p, p2c, buckets, max_rel, force_generic=force_generic)
    ref32 = oracle_fixed(inp, buckets, max_rel, dtype=torch.float32)
    assert_close_bf16(out, ref32, "bf16 strips vs fp32 oracle on rounded inputs", tol=1e-2)
    if L <= 512:
        ref16 = oracle_fixed(inp, buckets, max_rel, dtype=torch.bfloat16)
        assert_close_bf16(out, ref16, "bf16 strips vs bf16 eager oracle")
    if lengths is not None:
        for b, n in enumerate(lengths):
            assert torch.all(out[b, :, n:] == 0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("types", [("c2p", "p2c"), ("c2p",), ("p2c",)])
def test_random_strips_matrix_core_equals_vector_alu(types, dtype):
    """Strips of independent random values (no table behind them): every (row, column) of a strip holds its own
    number, so a wrong row, a wrong column or a value filed under the wrong key moves the output.  The vector-ALU
    kernel, pinned against the oracle in fp32, reads the same strips element by element."""
    B, H, L, buckets, max_rel = 2, 3, 400, 256, 512
    inp = make_inputs(22, B, H, L, 64, buckets, max_rel, dtype=dtype, lengths=(400, 213))
    g = torch.Generator().manual_seed(23)
    c2p = (torch.randn(B, H, L, 2 * buckets, generator=g) * 4).to(dtype) if "c2p" in types else None
    p2c = (torch.randn(B, H, L, 2 * buckets, generator=g) * 4).to(dtype) if "p2c" in types else None
    fast = _run_strips(inp, c2p, p2c, buckets, max_rel, n_terms=len(types))
    slow = _run_strips(inp, c2p, p2c, buckets, max_rel, n_terms=len(types), force_generic=True)
    assert_close_bf16(fast, slow, f"random strips {types} {dtype}", tol=4e-3 if dtype == torch.float16 else 1e-2)
    # and against the definition, on the valid rows of the first sequence
    f = lambda t: t[0].float()
    idx = O.relative_position_index(400, 400, buckets, max_rel)                   # [L, L] columns delta(i - j)
    s = torch.einsum("hid,hjd->hij", f(inp["q"]), f(inp["k"]))
    if c2p is not None:
        s = s + torch.gather(f(c2p), 2, idx[None].expand(H, -1, -1))
    if p2c is not None:
        s = s + torch.gather(f(p2c), 2, idx.t()[None].expand(H, -1, -1)).transpose(1, 2)
    ref = torch.softmax(s / math.sqrt(64 * (1 + len(types))), -1) @ f(inp["v"])
    assert_close_bf16(fast[0], ref, f"random strips {types} {dtype} vs definition", tol=1e-2)


def test_bf16_strips_varlen_vs_oracle():
    H, D, buckets, max_rel = 4, 64, 256, 512
    rs = np.random.RandomState(1)
    lengths = [int(x) for x in rs.randint(16, 513, size=10)] + [1, 128, 129, 0, 64]
    inp = make_inputs(24, len(lengths), H, max(lengths), D, buckets, max_rel, dtype=torch.bfloat16)
    packed, cu = pack(inp, lengths)
    f = lambda t: t.float()
    ref = O.attention_varlen(f(packed["q"]), f(packed["k"]), f(packed["v"]), f(inp["pk"]), f(inp["pq"]), cu,
                             position_buckets=buckets, max_relative_positions=max_rel)
    c2p = torch.einsum("thd,hmd->thm", packed["q"], inp["pk"])
    p2c = torch.einsum("thd,hmd->thm", packed["k"], inp["pq"])
    outs = []
    for force_generic in (False, True):
        print(f"[case] bf16 varlen strips generic={force_generic} lengths={lengths}", flush=True)
        out = flash_attention_with_disentangled_varlen(
            packed["q"].to(DEV), packed["k"].to(DEV), packed["v"].to(DEV), c2p.to(DEV), p2c.to(DEV), cu.to(DEV),
            cu.to(DEV), max(lengths), max(lengths), False, 1 / math.sqrt(3 * D), buckets, max_rel,
            force_generic=force_generic)
        torch.cuda.synchronize()
        assert_close_bf16(out.cpu(), ref, f"bf16 varlen strips generic={force_generic}", tol=1e-2)
        outs.append(out.cpu())
    assert_close_bf16(outs[0], outs[1], "bf16 varlen strips, matrix cores vs vector ALUs", tol=4e-3)


def test_backward_raises_like_the_reference():
    q = torch.randn(1, 1, 8, 64, device=DEV, requires_grad=True)
    out = flash_attention_with_disentangled(q, q, q, None, None)
    with pytest.raises(RuntimeError, match="Backward pass is not implemented"):
        out.sum().backward()
