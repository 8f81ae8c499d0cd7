#!/usr/bin/env python3
"""Benchmark of the fused disentangled-attention forward on one MI355X.

A "step" is one attention forward over one batch of synthetic DeBERTa-v3-base attention inputs
(12 heads x 64, rel-pos buckets 256 / max 512), bf16, inputs resident in HBM:

  fixed   batch 32 x seq 512, right-padded, valid lengths uniform in [384, 512]   (headline `value`)
  varlen  64 sequences with lengths uniform in [16, 512], packed with cu_seqlens  (reported beside it)
  padded  batch 32 x seq 512 as in `fixed`, but with valid lengths uniform in [64, 512]: a padded batch as it reaches
          the operator when nothing packs it   (`fixed_wide`, part of `all`)
  long    batch 4 x seq 4096, full mask, and its packed variant (8 sequences U[1024, 4096])   (`long`, `long_varlen`)
  strips  the reference's own call signature -- c2p / p2c strips [B, H, L, 2*span] computed by the caller -- on the
          matrix-core kernel: batch 8 x seq 256 and batch 32 x seq 512, bf16, priced against HBM (the strips are
          most of the bytes)   (`strips`)
  generic the vector-ALU kernel that serves float32 inputs and what the matrix-core kernel does not take: the
          attention of the config-1 layer (batch 2 x seq 128, float32), and the batch 8 x seq 256 strip call forced
          onto it for comparison   (`generic`)

Prints ONE JSON line.  `value` is algorithmic attention TFLOP/s of the fixed workload over the timed
region; FLOPs per sequence of valid length l and per head:  4*l*l*d (QK^T + PV) + 4*l*W*d (c2p + p2c),
W = min(2*span, 2*l - 1) -- no credit for padding, window recompute or projections.
`roofline` prices the kernel's average launch duration (two HIP events on the launch stream that bracket the timed
region, divided by the number of launches) against the MI355X dense bf16 MFMA peak; `cpu_baseline` times the CPU oracle (eager float32 restatement of
Hugging Face's DisentangledSelfAttention) on a bounded sample of the same workload and on the config-1 layer.

Before the warm-up launches of every workload the GPU is kept busy for `--prewarm-ms` (default 30 ms of launches of
that workload, untimed, reported as `prewarm_ms`): the first milliseconds of load after an idle period run at a lower
clock, and the timed region of a short run (`--steps 20 --warmup 5` is 2.5 ms) would otherwise sit inside that ramp.
`--warmup` and `--steps` keep their meaning.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

H, D, HID = 12, 64, 768
BUCKETS, MAX_REL, SPAN = 256, 512, 256
PEAK_BF16_TFLOPS = 2500.0       # MI355X dense bf16 MFMA, AMD public spec
PEAK_HBM_GBS = 8000.0
METRIC = "attn TFLOP/s + tokens/s, DeBERTa-v3-base b32xL512 bf16, fixed and varlen"
PEAK_FP32_VALU_TFLOPS = 157.3   # MI355X vector fp32, AMD public spec (what the generic kernel is priced against)
# HBM bytes per launch are not measured by this script: they come from `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE`
# runs of it, each counter scaled by what it reads for a plain 512 MiB device copy.  The figures, the commands, the
# commit and a digest of the kernel source they were taken at are recorded in the files named here; `roofline.traffic`
# repeats them with that source, and `roofline.traffic_stale` is true when the kernel source has changed since.
RECORDED_TRAFFIC = {
    "fixed": "profiles/attn_mfma_kernel_fixed_b32xL512.md",
    "varlen": "profiles/attn_mfma_kernel_varlen_64seq.md",
    "long": "profiles/attn_mfma_kernel_long_b4xL4096.md",
    "long_varlen": "profiles/attn_mfma_kernel_long_b4xL4096.md",
    "strips_b32xL512": "profiles/attn_mfma_kernel_strips_b32xL512.md",
    "strips_b8xL256": "profiles/attn_mfma_kernel_strips_b32xL512.md",
}
KERNEL_SOURCES = ("turbodeberta_amd/csrc/attn_mfma.hip", "turbodeberta_amd/csrc/tdb_internal.h")


def kernel_source_digest():
    """First 16 hex digits of the SHA-256 over the matrix-core kernel's source files, in the order of KERNEL_SOURCES:
    what a profile summary records as `kernel_source_sha256:` when its counters are taken."""
    import hashlib
    h = hashlib.sha256()
    try:
        for rel in KERNEL_SOURCES:
            h.update(open(os.path.join(ROOT, rel), "rb").read())
    except OSError:
        return None
    return h.hexdigest()[:16]


def recorded_traffic(name):
    """(bytes, source, stale) from the profile summary of a workload: the line `traffic_bytes_per_launch: <number>`
    (`traffic_bytes_per_launch[<name>]:` when one file covers several workloads), the line `commit: <hash>` and the
    line `kernel_source_sha256: <digest>` of the file.  `stale` says that the kernel source has changed since the
    counters were read (or that the summary does not say what it was read from); (None, None, None) when the file or
    the line is missing."""
    path = RECORDED_TRAFFIC.get(name)
    if path is None:
        return None, None, None
    try:
        text = open(os.path.join(ROOT, path)).read()
    except OSError:
        return None, None, None
    val = commit = digest = None
    for line in text.splitlines():
        for key in ("traffic_bytes_per_launch:", f"traffic_bytes_per_launch[{name}]:"):
            if line.startswith(key):
                val = float(line.split(":", 1)[1])
        if line.startswith("commit:"):
            commit = line.split(":", 1)[1].strip()
        if line.startswith("kernel_source_sha256:"):
            digest = line.split(":", 1)[1].strip()
    if val is None:
        return None, None, None
    source = f"{path} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, calibrated on a 512 MiB copy; commit {commit})"
    return val, source, digest is None or digest != kernel_source_digest()


def flops_of(lengths, heads=H) -> float:
    tot = 0.0
    for l in lengths:
        l = int(l)
        w = min(2 * SPAN, 2 * l - 1)
        tot += 4.0 * l * l * D + 4.0 * l * w * D
    return heads * tot


def algorithmic_bytes(lengths) -> float:
    t = float(sum(int(x) for x in lengths))
    return 2.0 * 4 * t * H * D + 2 * H * 2 * SPAN * D * 2.0


def make_weights(dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    mk = lambda *s, std: (torch.randn(*s, generator=g, device=dev, dtype=torch.float32) * std)
    w = {n: mk(HID, HID, std=0.02).to(torch.bfloat16) for n in ("wq", "wk", "wv")}
    w["rel"] = mk(2 * SPAN, HID, std=1.0).to(torch.bfloat16)
    return w, g


def position_tables(w):
    lin = torch.nn.functional.linear
    pk = lin(w["rel"], w["wk"]).view(2 * SPAN, H, D).permute(1, 0, 2).contiguous()     # K_r [H, 2s, D]
    pq = lin(w["rel"], w["wq"]).view(2 * SPAN, H, D).permute(1, 0, 2).contiguous()     # Q_r
    return pk, pq


def build_fixed(dev, B=32, L=512, shortest=384):
    from turbodeberta_amd.ops import flash_attention as fa
    w, g = make_weights(dev)
    lengths = np.random.RandomState(0).randint(shortest, 513, size=B)
    hidden = torch.randn(B, L, HID, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    lin = torch.nn.functional.linear
    heads = lambda x: x.view(B, L, H, D).permute(0, 2, 1, 3)       # projection-native storage, [B,H,L,D] view
    q, k, v = heads(lin(hidden, w["wq"])), heads(lin(hidden, w["wk"])), heads(lin(hidden, w["wv"]))
    pk, pq = position_tables(w)
    lens = torch.from_numpy(lengths.astype(np.int32)).to(dev)
    plan = fa.prepare(q, k, v, None, None, False, 1.0 / math.sqrt(3 * D), BUCKETS, MAX_REL,
                      pos_key_layer=pk, pos_query_layer=pq, seqlens_k=lens)
    return plan, lengths, dict(q=q, k=k, v=v, pk=pk, pq=pq)


def build_long(dev, B=4, L=4096):
    """Config 5: batch 4 x seq 4096, full mask."""
    from turbodeberta_amd.ops import flash_attention as fa
    w, g = make_weights(dev)
    hidden = torch.randn(B, L, HID, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    lin = torch.nn.functional.linear
    heads = lambda x: x.view(B, L, H, D).permute(0, 2, 1, 3)
    q, k, v = heads(lin(hidden, w["wq"])), heads(lin(hidden, w["wk"])), heads(lin(hidden, w["wv"]))
    pk, pq = position_tables(w)
    plan = fa.prepare(q, k, v, None, None, False, 1.0 / math.sqrt(3 * D), BUCKETS, MAX_REL,
                      pos_key_layer=pk, pos_query_layer=pq)
    return plan, np.full(B, L)


def _strip_call(dev, w, g, B, L, dt, force_generic=False):
    """The reference's literal call shape: c2p / p2c strips [B, H, L, 2*span] computed by the caller (model.py:122-137
    of the reference), full mask."""
    from turbodeberta_amd.ops import flash_attention as fa
    lin = torch.nn.functional.linear
    hidden = torch.randn(B, L, HID, generator=g, device=dev, dtype=torch.float32).to(dt)
    heads = lambda x: x.view(B, L, H, D).permute(0, 2, 1, 3)
    q, k, v = (heads(lin(hidden, w[n].to(dt))) for n in ("wq", "wk", "wv"))
    pk, pq = (t.to(dt) for t in position_tables(w))
    c2p = torch.matmul(q, pk.transpose(-1, -2)[None])
    p2c = torch.matmul(k, pq.transpose(-1, -2)[None])
    return fa.prepare(q, k, v, c2p, p2c, False, 1.0 / math.sqrt(3 * D), BUCKETS, MAX_REL, force_generic=force_generic)


def build_generic(dev):
    """The vector-ALU kernel: (a) the attention of the config-1 layer -- batch 2 x seq 128, 12 heads, float32, full
    mask, the case it exists for; (b) the strip call at batch 8 x seq 256 in bf16 forced onto it (without the flag that
    call runs on the matrix cores: `build_strips`)."""
    from turbodeberta_amd.ops import flash_attention as fa
    w, g = make_weights(dev)
    lin = torch.nn.functional.linear
    B, L, dt = 2, 128, torch.float32
    hidden = torch.randn(B, L, HID, generator=g, device=dev, dtype=torch.float32).to(dt)
    heads = lambda x: x.view(B, L, H, D).permute(0, 2, 1, 3)
    q, k, v = (heads(lin(hidden, w[n].to(dt))) for n in ("wq", "wk", "wv"))
    pk, pq = (t.to(dt) for t in position_tables(w))
    plan = fa.prepare(q, k, v, None, None, False, 1.0 / math.sqrt(3 * D), BUCKETS, MAX_REL,
                      pos_key_layer=pk, pos_query_layer=pq)
    return {"config1_fp32": (plan, np.full(B, L)),
            "strips_bf16_forced": (_strip_call(dev, w, g, 8, 256, torch.bfloat16, force_generic=True), np.full(8, 256))}


def build_strips(dev):
    """The strip call on the matrix-core kernel at batch 8 x seq 256 and at the headline shape, batch 32 x seq 512."""
    w, g = make_weights(dev)
    return {"b8xL256": (_strip_call(dev, w, g, 8, 256, torch.bfloat16), np.full(8, 256)),
            "b32xL512": (_strip_call(dev, w, g, 32, 512, torch.bfloat16), np.full(32, 512))}


def strip_bytes(lengths) -> float:
    """Algorithmic bytes of a strip call: q, k, v read and o written once, plus every strip element that some score
    position addresses -- row i of either strip is read at the columns delta(i - j), j < l, a contiguous range because
    delta is monotone."""
    from turbodeberta_amd import _lib
    tot = 0.0
    for l in lengths:
        l = int(l)
        lut = _lib.delta_table(l, BUCKETS, MAX_REL).astype(np.int64)       # entry r + l - 1
        i = np.arange(l)
        cols = lut[i + l - 1] - lut[i] + 1                                   # delta(i - 0) - delta(i - (l - 1)) + 1
        tot += 2.0 * 4 * l * H * D + 2 * 2.0 * H * float(cols.sum())
    return tot


def build_varlen(dev, n_seq=64, lo=16, hi=512):
    from turbodeberta_amd.ops import flash_attention_varlen as fv
    w, g = make_weights(dev)
    lengths = np.random.RandomState(0).randint(lo, hi + 1, size=n_seq)
    T = int(lengths.sum())
    hidden = torch.randn(T, HID, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    lin = torch.nn.functional.linear
    q, k, v = (lin(hidden, w[n]).view(T, H, D) for n in ("wq", "wk", "wv"))
    pk, pq = position_tables(w)
    cu = torch.from_numpy(np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)).to(dev)
    plan = fv.prepare(q, k, v, None, None, cu, cu, int(lengths.max()), int(lengths.max()), False,
                      1.0 / math.sqrt(3 * D), BUCKETS, MAX_REL, pos_key_layer=pk, pos_query_layer=pq)
    return plan, lengths


def prewarm(plan, budget_ms):
    """Keeps the GPU busy with launches of `plan` until `budget_ms` of wall clock have passed; returns the ms spent."""
    if budget_ms <= 0:
        return 0.0
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while True:
        for _ in range(20):
            plan.launch()
        torch.cuda.synchronize()
        spent = (time.perf_counter() - t0) * 1e3
        if spent >= budget_ms:
            return spent


def time_steps(plan, steps, warmup, prewarm_ms=0.0):
    """Times exactly `steps` back-to-back launches after `warmup` untimed ones (and, before those, `prewarm_ms` of
    untimed launches that bring the clock up).  Returns
    (wall ms per step between two synchronisations, kernel ms = span between two HIP events that bracket the same
    timed region on the launch stream / steps, then median and minimum of per-launch event pairs from a second pass;
    an event pair around a single launch reads about 3 us more than the launch takes in a back-to-back stream;
    ms spent pre-warming)."""
    spent = prewarm(plan, prewarm_ms)
    for _ in range(warmup):
        plan.launch()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        plan.launch()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    span_ms = e0.elapsed_time(e1) / steps
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in ev:
        a.record()
        plan.launch()
        b.record()
    torch.cuda.synchronize()
    durs = sorted(a.elapsed_time(b) for a, b in ev)
    return wall_ms, span_ms, durs[len(durs) // 2], durs[0], spent


def cpu_baseline(tensors, lengths, budget_s=12.0):
    """Oracle (float32 eager restatement of HF) on the first 2 sequences of the fixed workload."""
    from oracle import hf_eager as O
    nb = 2
    f = lambda t: t[:nb].float().cpu().contiguous()
    q, k, v = f(tensors["q"]), f(tensors["k"]), f(tensors["v"])
    pk, pq = tensors["pk"].float().cpu(), tensors["pq"].float().cpu()
    lens = torch.from_numpy(lengths[:nb].astype(np.int32))
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    run = lambda: O.attention_lengths(q, k, v, pk, pq, lens, position_buckets=BUCKETS, max_relative_positions=MAX_REL)
    run()
    times, t_start = [], time.perf_counter()
    while len(times) < 5 or (time.perf_counter() - t_start < budget_s and len(times) < 200):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {"value": round(flops_of(lengths[:nb]) / med / 1e12, 5), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port", "ms_per_sample": round(med * 1e3, 2),
            "sample": f"first {nb} of the 32 sequences of the fixed workload (lengths {lengths[:nb].tolist()}), "
                      f"float32 torch-CPU oracle, median of {len(times)} runs",
            "config1_layer": cpu_config1_layer()}


def cpu_config1_layer(budget_s=6.0):
    """BASELINE config 1 on the host: one DisentangledSelfAttention layer from hidden states (projections, position
    tables, attention), batch 2 x seq 128 x hidden 768, 12 heads, float32, full mask, seed 0 -- the oracle's
    restatement of the eager layer."""
    from oracle import hf_eager as O
    g = torch.Generator().manual_seed(0)
    B, L = 2, 128
    hidden = torch.randn(B, L, HID, generator=g)
    rel = torch.randn(2 * SPAN, HID, generator=g)
    wq, wk, wv = (torch.randn(HID, HID, generator=g) * 0.02 for _ in range(3))
    zero = torch.zeros(HID)
    mask = O.encoder_attention_mask(torch.ones(B, L, dtype=torch.long))
    run = lambda: O.self_attention_layer(hidden, mask, rel, wq, zero, wk, zero, wv, zero, H, position_buckets=BUCKETS,
                                         max_relative_positions=MAX_REL)
    run()
    run()
    times, t_start = [], time.perf_counter()
    while len(times) < 5 or (time.perf_counter() - t_start < budget_s and len(times) < 200):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    attn_flops = flops_of([L] * B)
    proj_flops = 2.0 * HID * HID * (3 * B * L + 2 * 2 * SPAN)
    return {"ms_per_layer": round(med * 1e3, 3), "tokens_per_s": round(B * L / med, 1),
            "attention_gflops": round(attn_flops / med / 1e9, 2), "with_projections_gflops": round((attn_flops + proj_flops) / med / 1e9, 2),
            "cores": torch.get_num_threads(),
            "sample": f"whole layer, batch {B} x seq {L} x hidden {HID}, float32, median of {len(times)} runs"}


def model_benchmark(dev, steps=30, warmup=10):
    """End-to-end forward of a DeBERTa-v3-large-shaped model (24 layers x 1024, 16 heads x 64, FFN 4096, vocabulary
    128100, buckets 256, max_rel 512, shared keys, c2p|p2c, layer-normed relative embeddings; random N(0, 0.02)
    weights, eval mode, bf16) on ids [16, 512] with right-padded lengths U[64, 512]: valid tokens per second with the
    attention core on the fused kernel (encoder packed: the default; and with padded layers), and with Hugging Face's
    eager attention in the same model on the same GPU."""
    from transformers import DebertaV2Config, DebertaV2Model
    from turbodeberta_amd.model import patch_model
    cfg = DebertaV2Config(vocab_size=128100, hidden_size=1024, num_hidden_layers=24, num_attention_heads=16,
                          intermediate_size=4096, hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0,
                          max_position_embeddings=512, type_vocab_size=0, relative_attention=True, position_buckets=256,
                          max_relative_positions=512, share_att_key=True, pos_att_type=["c2p", "p2c"],
                          norm_rel_ebd="layer_norm", position_biased_input=False, layer_norm_eps=1e-7,
                          initializer_range=0.02)
    torch.manual_seed(0)
    with torch.device(dev):
        model = DebertaV2Model(cfg)
    model = model.to(torch.bfloat16).eval()
    rs = np.random.RandomState(0)
    lengths = rs.randint(64, 513, size=16)
    ids = torch.from_numpy(rs.randint(0, 128000, size=(16, 512))).to(dev)
    mask = torch.from_numpy((np.arange(512)[None] < lengths[:, None]).astype(np.int64)).to(dev)

    def run(m):
        with torch.no_grad():
            for _ in range(warmup):
                m(input_ids=ids, attention_mask=mask)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                m(input_ids=ids, attention_mask=mask)
            torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps

    t_eager = run(model)
    patch_model(model)
    model.encoder.pack_sequences = False
    t_padded = run(model)
    model.encoder.pack_sequences = True
    t_fused = run(model)
    tokens = float(lengths.sum())
    return {"workload": "v3-large-shaped model, ids [16, 512], lengths U[64,512] seed 0 (%d valid tokens), bf16" % int(tokens),
            "steps": steps, "warmup": warmup,
            "fused": {"ms_per_forward": round(t_fused * 1e3, 3), "valid_tokens_per_s": round(tokens / t_fused, 1)},
            "fused_padded_layers": {"ms_per_forward": round(t_padded * 1e3, 3),
                                    "valid_tokens_per_s": round(tokens / t_padded, 1)},
            "hf_eager_same_gpu": {"ms_per_forward": round(t_eager * 1e3, 3), "valid_tokens_per_s": round(tokens / t_eager, 1)},
            "speedup": round(t_eager / t_fused, 3)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20, help="untimed launches right before the timed region")
    ap.add_argument("--prewarm-ms", type=float, default=30.0,
                    help="untimed launches of the workload for this many ms before the warm-up, to get past the clock "
                         "ramp that follows an idle period (0 switches it off)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--workload", choices=["all", "both", "fixed", "varlen", "long", "strips", "generic"], default="all",
                    help="all = fixed + varlen + long + long_varlen + strips + generic; both = fixed + varlen")
    ap.add_argument("--with-model", action="store_true",
                    help="add the end-to-end forward of a v3-large-shaped model (fused attention vs Hugging Face eager "
                         "attention on the same GPU) to the JSON line as \"model\"")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain device copy of 512 MiB (read) + 512 MiB (write), the yardstick the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every figure of this path is per GPU (no collectives); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the operators have no CPU implementation", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda", int(os.environ.get("LOCAL_RANK", "0")))
    torch.cuda.set_device(dev)

    if args.calibrate_copy:
        src = torch.zeros(256 * 1024 * 1024, dtype=torch.bfloat16, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    out = {"metric": METRIC, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic"}
    spent_prewarm = []

    def measure(plan, lengths, name, kernel, peak=PEAK_BF16_TFLOPS, bound="mfma", steps=None, nbytes=None):
        steps = steps or args.steps
        wall_ms, mean_ms, med_ms, min_ms, spent = time_steps(plan, steps, args.warmup, args.prewarm_ms)
        spent_prewarm.append(spent)
        fl = flops_of(lengths)
        nbytes = algorithmic_bytes(lengths) if nbytes is None else nbytes
        if bound == "hbm":                                         # priced by bytes: GB/s against the HBM peak
            ach, peak, unit = nbytes / (mean_ms * 1e-3) / 1e9, PEAK_HBM_GBS, "GB/s"
        else:
            ach, unit = fl / (mean_ms * 1e-3) / 1e12, "TFLOP/s"
        traffic, traffic_source, traffic_stale = recorded_traffic(name)
        return {
            "value": round(fl / (wall_ms * 1e-3) / 1e12, 2), "ms_per_step": round(wall_ms, 4), "steps": steps,
            "tokens_per_s": round(float(lengths.sum()) / (wall_ms * 1e-3), 1),
            "core_tflops": round(H * sum(4.0 * int(l) ** 2 * D for l in lengths) / (wall_ms * 1e-3) / 1e12, 2),
            "roofline": {"bound": bound, "achieved": round(ach, 2), "peak": peak, "unit": unit,
                         "frac": round(ach / peak, 4), "traffic": traffic, "traffic_source": traffic_source, "traffic_stale": traffic_stale,
                         "kernel": kernel,
                         "kernel_ms_mean": round(mean_ms, 4), "kernel_ms_pair_median": round(med_ms, 4),
                         "kernel_ms_pair_min": round(min_ms, 4), "algorithmic_gflop": round(fl / 1e9, 3), "algorithmic_bytes": nbytes,
                         "hbm_gbs_algorithmic": round(nbytes / (mean_ms * 1e-3) / 1e9, 1)},
        }

    res_fixed = res_var = None
    tensors = lengths_f = None
    if args.workload in ("all", "both", "fixed"):
        plan, lengths_f, tensors = build_fixed(dev)
        res_fixed = measure(plan, lengths_f, "fixed", "attn_mfma_kernel<c2p,p2c>")
    if args.workload in ("all", "both", "varlen"):
        plan_v, lengths_v = build_varlen(dev)
        res_var = measure(plan_v, lengths_v, "varlen", "attn_mfma_kernel<c2p,p2c>")
    extra = {}
    if args.workload == "all":
        plan_w, lengths_w, _ = build_fixed(dev, shortest=64)
        extra["fixed_wide"] = {"workload": "fixed b32xL512, valid lengths U[64,512] seed 0 (%d valid tokens), 12 heads x 64, c2p|p2c"
                                           % int(lengths_w.sum()),
                               **measure(plan_w, lengths_w, "fixed_wide", "attn_mfma_kernel<c2p,p2c>")}
        del plan_w
    if args.workload in ("all", "long"):
        few = max(5, min(args.steps, 40))                      # a launch takes ~1 ms: fewer steps keep the run short
        plan_l, lengths_l = build_long(dev)
        extra["long"] = {"workload": "fixed b4xL4096, full mask, 12 heads x 64, buckets 256, max_rel 512, c2p|p2c",
                         **measure(plan_l, lengths_l, "long", "attn_mfma_kernel<c2p,p2c>", steps=few)}
        del plan_l
        plan_lv, lengths_lv = build_varlen(dev, n_seq=8, lo=1024, hi=4096)
        extra["long_varlen"] = {"workload": "8 packed sequences, lengths U[1024,4096] seed 0, total tokens %d" % int(lengths_lv.sum()),
                                **measure(plan_lv, lengths_lv, "long_varlen", "attn_mfma_kernel<c2p,p2c>", steps=few)}
        del plan_lv
    if args.workload in ("all", "strips"):
        extra["strips"] = {}
        for name, (pl, ln) in build_strips(dev).items():
            extra["strips"][name] = {"workload": "strip-taking signature (c2p / p2c strips [B,H,L,512] from the caller), "
                                                 "batch %d x seq %d, full mask, bf16" % (len(ln), int(ln[0])),
                                     **measure(pl, ln, "strips_" + name, "attn_mfma_kernel<c2p,p2c,strips>", bound="hbm",
                                               nbytes=strip_bytes(ln))}
            del pl
        torch.cuda.empty_cache()
    if args.workload in ("all", "generic"):
        notes = {"config1_fp32": "attention of the config-1 layer: batch 2 x seq 128, 12 heads x 64, float32, fused tables",
                 "strips_bf16_forced": "strip-taking signature, batch 8 x seq 256, bf16, forced onto the vector-ALU kernel "
                                       "(without the flag it runs on the matrix cores: `strips.b8xL256`)"}
        extra["generic"] = {name: {"workload": notes[name],
                                   **measure(pl, ln, name, "attn_generic_kernel", peak=PEAK_FP32_VALU_TFLOPS, bound="valu")}
                            for name, (pl, ln) in build_generic(dev).items()}
    head = res_fixed or res_var or extra.get("long") or next(iter((extra.get("strips") or extra["generic"]).values()))
    out.update({"value": head["value"], "ms_per_step": head["ms_per_step"], "tokens_per_s": head["tokens_per_s"],
                "core_tflops": head["core_tflops"], "roofline": head["roofline"]})
    out["config"] = {"workload": ("fixed b32xL512, valid lengths U[384,512] seed 0" if res_fixed else
                                  "varlen 64 seqs U[16,512] seed 0") + ", 12 heads x 64, buckets 256, max_rel 512, c2p|p2c",
                     "global_batch": 32 if res_fixed else 64, "seq_len": 512}
    if res_fixed and res_var:
        out["varlen"] = {"workload": "64 packed sequences, lengths U[16,512] seed 0, total tokens %d" % int(lengths_v.sum()),
                         **res_var}
    out.update(extra)
    out["prewarm_ms"] = round(float(np.mean(spent_prewarm)), 2) if spent_prewarm else 0.0
    if not args.no_cpu_baseline and tensors is not None:
        out["cpu_baseline"] = cpu_baseline(tensors, lengths_f)
    if args.with_model:
        del tensors
        torch.cuda.empty_cache()
        out["model"] = model_benchmark(dev)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
