#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

One "step" = one forward (O + log-sum-exp) followed by one tile-recompute backward (dQ, dK, dV), inputs
resident in HBM.  The headline workload is the DiT joint-attention configuration B=1 H=24 S=4608 (512 text
+ 4096 image tokens) D=128 bf16: the line's `value`, `ms_per_step`, `roofline` and `cpu_baseline` are its.
Without `--config` the other four configurations (1 small, 3 ragged cross attention, 4 long causal, 5 the
inference-only int8-QK forward, whose step is quantisation + forward) are then timed the same way at up to
20 steps each and reported as rows of `configs`; `--config 1..5` runs one configuration alone.  Prints ONE JSON line.

Three timed loops after the warm-up, all with the same inputs:
  1. `--steps` steps bracketed by a device synchronisation on both sides, nothing else running on the
     host side: `ms_per_step` and `value` come from this one;
  2. the same steps with a HIP event before the forward, between forward and backward, and after the
     backward (events on the stream the kernels are launched on): medians in `timing`;
  3. at most 50 steps with the library's own event pair around every kernel launch: `kernels_ms`, and from
     them the roofline of the dominant kernel.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA, published
PEAK_INT8_TOPS = 5000.0        # MI355X dense int8 MFMA, published
METRIC = "fwd+bwd attn TFLOP/s & % MFMA peak, S=4608 D=128 bf16; saved-activation bytes"


def profile_path(workload_name: str) -> str:
    return os.path.join(ROOT, "profiles", f"attention_kernels_{workload_name}.md")


def recorded_traffic(workload_name: str, kernel):
    """HBM bytes per launch of `kernel` as recorded in this workload's rocprofv3 summary under profiles/
    (FETCH_SIZE and WRITE_SIZE passes, already scaled by the copy-kernel calibration that the summary
    states next to the commands).  Counters cannot be read from inside this script; None when the
    summary or the row is missing."""
    try:
        text = open(profile_path(workload_name)).read()
    except OSError:
        return None
    sec = text.split("## HBM traffic", 1)
    if len(sec) < 2:
        return None
    total = None
    for name in ([kernel] if isinstance(kernel, str) else kernel):      # several kernels: one entry-point call launches them all
        for line in sec[1].splitlines():
            m = re.match(r"\|\s*`fattn::%s[<`][^|]*\|\s*[\d.]+\s*\|\s*([\d.]+)\s*\|\s*[\d.]+\s*\|\s*([\d.]+)\s*\|" % re.escape(name), line)
            if m:
                total = (total or 0) + int((float(m.group(1)) + float(m.group(2))) * 1e6)
                break
    return total


def cpu_baseline(w):
    """Naive materialised fp32 SDPA forward+backward (the parity checker) timed on the host cores, on a
    bounded sample of the same workload: whole passes while they are short, else one band of query
    rows of every head (a band costs rows x Sk)."""
    from oracle import oracle as O
    O.lib()
    B, H, Sq, Sk, D = w.shape
    cores = O.num_threads()
    heads = B * H
    rows = (0, Sq)
    sample_pairs = w.valid_pairs()
    what = f"all {heads} (batch,head) slices"
    if w.flops() > 4e12:                                     # long causal: the last 1024 query rows of every head
        rows = (Sq - 1024, Sq)
        sample_pairs = heads * sum(min(i + 1, Sk) if w.causal else Sk for i in range(*rows))
        what = f"query rows {rows[0]}..{rows[1]} of all {heads} (batch,head) slices"
    passes, dt = 0, 0.0
    t0 = time.perf_counter()
    while dt < 10.0 and passes < 5000:           # repeated to about 10 s of CPU work
        o, _ = O.sdpa_fwd(w.q, w.k, w.v, w.scale, causal=w.causal, kv_len=w.kv_len, heads=(0, heads), rows=rows)
        O.sdpa_bwd(w.q, w.k, w.v, o, w.do, w.scale, causal=w.causal, kv_len=w.kv_len, heads=(0, heads), rows=rows)
        passes += 1
        dt = time.perf_counter() - t0
    flops = 14.0 * sample_pairs * D * passes
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"{passes} passes over {what} of the same workload, naive fp32 fwd+bwd, {dt:.1f} s wall",
            "seconds": dt}


def cpu_baseline_sage(w):
    """The oracle's quantiser + int8-QK forward, whole passes over the same workload for about 10 s."""
    from oracle import oracle as O
    O.lib()
    B, H, Sq, Sk, D = w.shape
    passes, dt = 0, 0.0
    t0 = time.perf_counter()
    while dt < 10.0 and passes < 5000:
        z = O.sage_quant(w.q, w.k)
        O.sage_fwd(z["qi8"], z["ki8"], z["sq"], z["sk"], w.v, w.scale)
        passes += 1
        dt = time.perf_counter() - t0
    ops = 4.0 * w.valid_pairs() * D * passes
    return {"value": ops / dt / 1e12, "unit": "TOP/s", "cores": O.num_threads(), "kind": "port",
            "sample": f"{passes} passes of quantisation + int8-QK forward over all {B * H} (batch,head) slices of the "
                      f"same workload, {dt:.1f} s wall", "seconds": dt}


def input_prep_rate(capi, W, torch, B, H, N, D, dev, iters=20):
    """Fused RMS-norm + RoPE + layout change of one [B,N,H,D] projection output (the caller of the hot
    path on the input side), outside the timed step: HBM-bound, reported against 8 TB/s."""
    x = torch.randn((B, N, H, D), device=dev, dtype=torch.float32).to(torch.bfloat16)
    wgt = torch.ones((D,), device=dev, dtype=torch.bfloat16)
    side = int(round((N - 512) ** 0.5))
    cos, sin = W.axial_rope_tables(N - side * side, side, side, D)
    cos, sin = torch.from_numpy(cos).to(dev), torch.from_numpy(sin).to(dev)
    y = torch.empty((B, H, N, D), device=dev, dtype=torch.bfloat16)
    for _ in range(3):
        capi.prep_rmsnorm_rope(x, wgt, cos, sin, out=y)
    torch.cuda.synchronize()
    capi.profiling_enable(True)
    for _ in range(iters):
        capi.prep_rmsnorm_rope(x, wgt, cos, sin, out=y)
    torch.cuda.synchronize()
    tot, n = capi.profiling_read()["input_prep"]
    capi.profiling_enable(False)
    ms = tot / max(n, 1)
    nbytes = 2 * x.numel() * 2 + 2 * cos.numel() * 4 + D * 2       # read x, write y, read both tables and the scale
    return {"kernel": "prep_qk_kernel", "ms_per_tensor": ms, "algorithmic_bytes": nbytes,
            "GB_per_s": nbytes / (ms * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 8e12}


def tile_ops_line(args, capi, torch, dev):
    """The element-wise tile primitives on one tile of the headline shape (all 24 heads, 1024 query rows, 4608
    keys): median HIP-event time per call and the algorithmic bytes each moves, against 8 TB/s."""
    BH, q_t, k_t = 24, 1024, 4608
    n = BH * q_t * k_t
    g = torch.Generator(device=dev).manual_seed(7)
    logits = torch.randn((BH, q_t, k_t), device=dev, generator=g)
    scores = logits.view(1, BH, q_t, k_t)
    keep = (torch.rand((1, BH, q_t, k_t), device=dev, generator=g) < 0.9).to(torch.uint8)
    keep_pad = torch.ones((1, BH, q_t, k_t), device=dev, dtype=torch.uint8)
    keep_pad[..., k_t - k_t // 10:] = 0
    add = torch.randn((BH, k_t), device=dev, generator=g)
    lse = torch.logsumexp(logits, -1)
    lse_other = lse.clone()
    probs = torch.rand((BH, q_t, k_t), device=dev, generator=g).to(torch.bfloat16)
    saved = torch.randn((4, 24, 4608, 128), device=dev, generator=g).to(torch.bfloat16)
    saved_fp8 = torch.empty(saved.shape, device=dev, dtype=torch.uint8)
    n_future = int((torch.arange(k_t, device=dev)[None, :] > torch.arange(q_t, device=dev)[:, None]).sum()) * BH
    n_dropped = int((keep == 0).sum())
    cases = [
        ("flame_apply_causal_mask_fp32", lambda: capi.tile_causal_mask(scores), 4 * n_future),
        ("flame_apply_attn_mask_fp32 (last tenth of the keys excluded)", lambda: capi.tile_attn_mask(scores, keep_pad),
         n + 4 * int((keep_pad == 0).sum())),
        ("flame_apply_attn_mask_fp32 (a random tenth excluded: scattered 4-byte stores)", lambda: capi.tile_attn_mask(scores, keep),
         n + 4 * n_dropped),
        ("flame_sdpa_add_mask_tile_fp32", lambda: capi.tile_add_mask(logits, keep.view(BH, q_t, k_t), add, bool_rank=3,
                                                                      add_rank=2, k_total=k_t, causal=True), 9 * n + 4 * BH * k_t),
        ("flame_sdpa_lse_from_logits_tile", lambda: capi.tile_lse_from_logits(logits), 4 * n + 4 * BH * q_t),
        ("flame_sdpa_softmax_from_lse_tile", lambda: capi.tile_softmax_from_lse(logits, lse, out=probs), 6 * n + 4 * BH * q_t),
        ("flame_sdpa_lse_merge_rows", lambda: capi.tile_lse_merge(lse, lse_other), 12 * BH * q_t),
        ("flame_sdpa_dropout_bf16_inplace", lambda: capi.tile_dropout(probs, 0.1, 2024), 4 * n),
        # the saved set of the headline shape on its way to the offload pool: Q, K, V, O = 4 x [1, 24, 4608, 128] bf16
        ("flame_bf16_to_fp8 (saved Q,K,V,O of cfg 2)", lambda: capi.bf16_to_fp8(saved, 56.0, out=saved_fp8), 3 * saved.numel()),
        ("flame_fp8_to_bf16 (saved Q,K,V,O of cfg 2)", lambda: capi.fp8_to_bf16(saved_fp8, 1.0 / 56.0, out=saved), 3 * saved.numel()),
    ]
    out = {}
    for name, fn, nbytes in cases:
        for _ in range(3):
            fn()
        times = []
        for _ in range(20):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            e1.synchronize()
            times.append(e0.elapsed_time(e1))
        ms = sorted(times)[len(times) // 2]
        out[name] = {"ms_median": ms, "algorithmic_bytes": nbytes, "GB_per_s": nbytes / (ms * 1e-3) / 1e9,
                     "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 8e12}
    print(json.dumps({"metric": "element-wise tile primitives, GB/s of algorithmic bytes", "unit": "GB/s", "n_gpus": 1,
                      "dtype": "f32/bf16/u8", "data": "synthetic",
                      "config": {"workload": "score tile [24, 1024, 4608]; FP8 pair on 4 x [1, 24, 4608, 128] bf16"}, "primitives": out}))
    return 0


def big_head_dims_line(args, capi, torch, dev):
    """The forward for head dims above 128 on four shapes (one with a single head of one image, the case of a VAE mid
    block), next to torch's materialised bf16 matmul - fp32 softmax - matmul on the same GPU: median HIP-event
    times, useful TFLOP/s (4 B H S^2 D)."""
    import math
    out = {}
    g = torch.Generator(device=dev).manual_seed(11)
    for (B, H, S, D) in [(16, 1, 4096, 512), (1, 1, 4096, 512), (2, 8, 4096, 384), (2, 8, 4096, 256)]:
        q, k, v = (torch.randn((B, H, S, D), device=dev, generator=g).to(torch.bfloat16) for _ in range(3))
        sc = 1.0 / math.sqrt(D)

        def materialised():
            p = torch.softmax(torch.matmul(q, k.transpose(-1, -2)).float() * sc, -1).to(torch.bfloat16)
            return torch.matmul(p, v)

        res = {}
        for name, fn, iters in (("fused", lambda: capi.attn_fwd(q, k, v, sc), 20), ("materialised_torch", materialised, 8)):
            for _ in range(3):
                fn()
            times = []
            for _ in range(iters):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                fn()
                e1.record()
                e1.synchronize()
                times.append(e0.elapsed_time(e1))
            res[name + "_ms_median"] = sorted(times)[len(times) // 2]
        res["fused_useful_TFLOPs"] = 4.0 * B * H * S * S * D / (res["fused_ms_median"] * 1e-3) / 1e12
        out[f"B={B} H={H} S={S} D={D}"] = res
    print(json.dumps({"metric": "forward for head dims above 128, ms", "unit": "ms", "n_gpus": 1, "dtype": "bf16",
                      "data": "synthetic", "higher_is_better": False,
                      "config": {"workload": "forward only, non-causal, head dims 256 / 384 / 512"}, "shapes": out}))
    return 0


def materialised_path_line(args, capi, torch, dev):
    """The library's own materialised path (flame_attn_fwd_materialised_bf16 / flame_attn_bwd_materialised_bf16: the
    shapes the fused kernels refuse) on three shapes: median HIP-event times of forward and backward with the
    workspace the size query recommends, useful TFLOP/s (4 / 10 B H S^2 D), and the bytes its element-wise passes move
    over the scores (forward 4 + 4 + 4 + 2 + 2 per score element: write logits, two reads for maximum and sum, a read
    and the bf16 P written, read by the P V product; backward 8 more for dP and dS), as a rate."""
    import math
    out = {}
    g = torch.Generator(device=dev).manual_seed(13)
    for (B, H, S, D, masked) in [(1, 8, 2048, 256, True), (2, 4, 4096, 520, False), (1, 24, 2048, 20, False)]:
        q, k, v, do = (torch.randn((B, H, S, D), device=dev, generator=g).to(torch.bfloat16) for _ in range(4))
        mask = torch.ones((1, 1, S, S), dtype=torch.uint8, device=dev) if masked else None
        sc = 1.0 / math.sqrt(D)
        ws_f = torch.empty(capi.materialised_workspace_bytes(B, H, S, S, D, D, False), dtype=torch.uint8, device=dev)
        ws_b = torch.empty(capi.materialised_workspace_bytes(B, H, S, S, D, D, True), dtype=torch.uint8, device=dev)
        o, lse = capi.attn_fwd_materialised(q, k, v, sc, mask=mask, workspace=ws_f)
        grads = tuple(torch.empty_like(q) for _ in range(3))
        res = {"workspace_MiB": {"forward": ws_f.numel() / 2 ** 20, "backward": ws_b.numel() / 2 ** 20}}
        for name, fn in (("forward", lambda: capi.attn_fwd_materialised(q, k, v, sc, mask=mask, out=o, workspace=ws_f)),
                         ("backward", lambda: capi.attn_bwd_materialised(q, k, v, o, do, lse, sc, mask=mask, workspace=ws_b, grads=grads))):
            for _ in range(2):
                fn()
            times = []
            for _ in range(8):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                fn()
                e1.record()
                e1.synchronize()
                times.append(e0.elapsed_time(e1))
            ms = sorted(times)[len(times) // 2]
            flops = (4.0 if name == "forward" else 10.0) * B * H * S * S * D
            score_bytes = (16.0 if name == "forward" else 30.0) * B * H * S * S
            res[name] = {"ms_median": ms, "useful_TFLOPs": flops / (ms * 1e-3) / 1e12, "score_traffic_GB_per_s": score_bytes / (ms * 1e-3) / 1e9}
        out[f"B={B} H={H} S={S} D={D}" + (" keep-mask" if masked else "")] = res
        del q, k, v, do, o, lse, grads, ws_f, ws_b
    print(json.dumps({"metric": "materialised path (shapes the fused kernels refuse), ms", "unit": "ms", "n_gpus": 1, "dtype": "bf16",
                      "data": "synthetic", "higher_is_better": False,
                      "config": {"workload": "forward and backward, head dims 256 with a keep-mask, 520 and 20"}, "shapes": out}))
    return 0


def materialised_comparator(capi, torch, q, k, v, do, scale, o_fused, grads_fused, iters=5):
    """The structure this path replaces, run on the same GPU for comparison: scores = Q K^T as one library GEMM
    per head, softmax through this library's tile primitives, P kept in bf16 for the backward, PV / dV / dP / dQ /
    dK as library GEMMs (the reference's materialised path: src/sdpa.rs:788-961, backward
    src/autograd.rs:3918-3969).  Reports its time, its peak device memory next to the fused path's, and how far its
    results are from the fused kernels'.  Unmasked problems only."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    BH = B * H
    q3, k3, v3, do3 = (t.reshape(BH, -1, D) for t in (q, k, v, do))

    def fwd():
        s = torch.bmm(q3, k3.transpose(1, 2)).float()            # bf16 GEMM, fp32 scores
        s *= scale
        lse = capi.tile_lse_from_logits(s)
        p = capi.tile_softmax_from_lse(s, lse)                    # bf16 [BH, Sq, Sk]: what is saved for the backward
        return p, torch.bmm(p, v3)

    def bwd(p):
        dv = torch.bmm(p.transpose(1, 2), do3)
        dp = torch.bmm(do3, v3.transpose(1, 2)).float()
        pf = p.float()
        ds = (pf * (dp - (dp * pf).sum(-1, keepdim=True)) * scale).to(torch.bfloat16)
        return torch.bmm(ds, k3), torch.bmm(ds.transpose(1, 2), q3), dv

    p, o = fwd()
    dq, dk, dv = bwd(p)
    torch.cuda.synchronize()

    def rel(a, b):
        return float((a.float() - b.reshape(a.shape).float()).norm() / b.float().norm())

    diffs = {"O": rel(o, o_fused), "dQ": rel(dq, grads_fused[0]), "dK": rel(dk, grads_fused[1]), "dV": rel(dv, grads_fused[2])}
    del p, o, dq, dk, dv
    torch.cuda.empty_cache()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    tf, tb = [], []
    for _ in range(iters):
        e = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        e[0].record()
        p, o = fwd()
        e[1].record()
        g = bwd(p)
        e[2].record()
        e[2].synchronize()
        tf.append(e[0].elapsed_time(e[1]))
        tb.append(e[1].elapsed_time(e[2]))
        del p, o, g
    peak = torch.cuda.max_memory_allocated() - base
    return {"what": "QK^T / PV / backward products as library GEMMs, softmax by the tile primitives, bf16 P saved",
            "forward_ms_median": sorted(tf)[len(tf) // 2], "backward_ms_median": sorted(tb)[len(tb) // 2],
            "saved_between_forward_and_backward_bytes": BH * Sq * Sk * 2 + BH * Sq * D * 2,
            "peak_device_MiB_beyond_inputs": peak / 2 ** 20, "rel_l2_vs_fused": diffs}


def timed_loops(torch, capi, first, second, steps, warmup):
    """The three loops of the module docstring.  `first` / `second`: the two halves of a step (forward and
    backward; quantisation and forward).  Returns (wall ms per step, event medians, per-kernel averages)."""
    for _ in range(warmup):
        first()
        second()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        first()
        second()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps

    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    for e in ev:
        e[0].record()
        first()
        e[1].record()
        second()
        e[2].record()
    torch.cuda.synchronize()
    a = [e[0].elapsed_time(e[1]) for e in ev]
    b = [e[1].elapsed_time(e[2]) for e in ev]
    j = [e[0].elapsed_time(e[2]) for e in ev]
    medians = {"first_ms_median": statistics.median(a), "second_ms_median": statistics.median(b),
               "step_ms_median": statistics.median(j), "step_ms_min": min(j), "step_ms_max": max(j), "samples": steps}

    capi.profiling_enable(True)          # an event pair around every kernel, on the launch stream
    for _ in range(min(steps, 50)):
        first()
        second()
    torch.cuda.synchronize()
    times = capi.profiling_read()
    capi.profiling_enable(False)
    per_kernel = {kname: tot / n for kname, (tot, n) in times.items() if n}
    return wall_ms, medians, per_kernel


def sage_line(args, capi, torch, w, dev, steps=None, warmup=None, with_cpu_baseline=True):
    """Inference-only configuration: one step = quantise Q and K to int8 + the int8-QK forward.  Returns the line."""
    import numpy as np
    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    B, H, Sq, Sk, D = w.shape
    q, k, v = (torch.from_numpy(np.ascontiguousarray(t).view(np.int16)).view(torch.bfloat16).to(dev) for t in (w.q, w.k, w.v))
    o = torch.empty_like(q)
    state = {}

    def quant():
        state["qz"] = capi.sage_quant(q, k)

    def fwd():
        capi.sage_fwd(state["qz"], v, w.scale, out=o)

    torch.cuda.reset_peak_memory_stats()
    ms, med, per_kernel = timed_loops(torch, capi, quant, fwd, steps, warmup)
    # the bf16 forward on the same inputs, for the comparison the int8 path has to win
    for _ in range(5):
        capi.attn_fwd(q, k, v, w.scale, want_lse=False, out=o)
    e = [torch.cuda.Event(enable_timing=True) for _ in range(21)]
    for i in range(20):
        e[i].record()
        capi.attn_fwd(q, k, v, w.scale, want_lse=False, out=o)
    e[20].record()
    torch.cuda.synchronize()
    bf16_fwd_ms = statistics.median(e[i].elapsed_time(e[i + 1]) for i in range(20))
    ops = 4.0 * w.valid_pairs() * D            # 2*pairs*D int8 (QK^T) + 2*pairs*D bf16 (PV)
    t_fwd = per_kernel["sage_fwd"] * 1e-3
    # time-weighted blend of the two peaks: the int8 half is priced at 5.0 POP/s, the bf16 half at 2.5 PFLOP/s
    ideal = 0.5 * ops / (PEAK_INT8_TOPS * 1e12) + 0.5 * ops / (PEAK_BF16_TFLOPS * 1e12)
    out = {
        "metric": "int8-QK attention forward incl. quantisation, T(FL)OP/s", "value": ops / (ms * 1e-3) / 1e12,
        "unit": "TOP/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8+bf16", "data": "synthetic",
        "config": {"workload": w.name, "B": B, "H": H, "Sq": Sq, "Sk": Sk, "D": D, "causal": bool(w.causal),
                   "step": "quantise Q,K (per-block int8, mean-smoothed K) + int8-QK forward"},
        "timing": {"quantise_ms_median": med["first_ms_median"], "forward_ms_median": med["second_ms_median"],
                   "step_ms_median": med["step_ms_median"], "samples": med["samples"], "clock": "HIP events on the launch stream",
                   "bf16_forward_same_inputs_ms_median": bf16_fwd_ms},
        "roofline": {"bound": "mfma", "kernel": "sage_fwd_wide_kernel + sage_fwd_kernel (last partial round)", "achieved": ops / t_fwd / 1e12,
                     "peak": ops / ideal / 1e12, "unit": "TOP/s", "frac": ideal / t_fwd,
                     "traffic": recorded_traffic(w.name, ["sage_fwd_wide_kernel", "sage_fwd_kernel"]),
                     "avg_launch_ms": per_kernel["sage_fwd"], "ops_per_launch": ops,
                     "note": "peak = time-weighted blend of 5.0 POP/s int8 and 2.5 PFLOP/s bf16"},
        "kernels_ms": per_kernel,
        "peak_device_MiB": torch.cuda.max_memory_allocated() / 2 ** 20}
    if with_cpu_baseline and not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_sage(w)
    return out


# Instructions other than MFMAs that the kernels compiled for head dim 64 issue per MFMA (vector ALU + LDS, from the
# SQ_INSTS_* counters in profiles/attention_kernels_cfg3_ragged_cross.md): at D = 64 a 64-key tile has half the MFMAs
# of a D = 128 tile for the same softmax / dS arithmetic.
OTHERS_PER_MFMA_D64 = {"fwd": 12.9, "bwd_dq": 9.1, "bwd_dkdv": 7.1}
ISSUE_CYCLES_PER_INSTRUCTION = 5.5     # measured: next to an MFMA stream a SIMD issues one other instruction every 5-6 cycles


def bound_of(w, kname, launch_ms):
    """What bounds kernel `kname` at workload `w`, and the rate that bound allows for its algorithmic flops:
    'launch' when a launch is over before the chip fills (under 20 us), 'valu-issue' at head dim 64, where the
    instructions between two MFMAs take longer to issue than the MFMA (32 cycles) takes to run, else 'mfma'."""
    D = w.shape[4]
    if launch_ms < 0.020:
        return "launch", None, "a launch of a few microseconds: fixed launch and prologue time, not a pipe, sets the rate"
    if D <= 64:
        k = OTHERS_PER_MFMA_D64[kname]
        frac = 32.0 / max(32.0, ISSUE_CYCLES_PER_INSTRUCTION * k)
        return ("valu-issue", PEAK_BF16_TFLOPS * frac,
                f"{k} other instructions per MFMA x {ISSUE_CYCLES_PER_INSTRUCTION} issue cycles against 32 cycles per MFMA: "
                f"{frac:.2f} of the MFMA peak is the most this instruction mix can reach")
    return "mfma", PEAK_BF16_TFLOPS, None


def attention_line(args, capi, torch, W, w, dev, steps, warmup, headline):
    """Forward + backward of one workload: the three timed loops and the line built from them.  `headline`: also
    the input-preparation rate, the materialised comparator and the CPU baseline."""
    B, H, Sq, Sk, D = w.shape

    def dev_t(bits):
        import numpy as np
        return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16).to(dev)

    torch.cuda.reset_peak_memory_stats()
    q, k, v, do = (dev_t(t) for t in (w.q, w.k, w.v, w.do))
    kvl = None if w.kv_len is None else torch.from_numpy(w.kv_len).to(dev)
    o = torch.empty_like(q)
    grads = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))
    ws = torch.empty(capi.bwd_workspace_bytes(B, H, Sq, D), dtype=torch.uint8, device=dev)
    mask = torch.ones(1, 1, Sq, Sk, dtype=torch.uint8, device=dev) if args.keep_mask else None
    state = {}
    drop = args.dropout

    def fwd():
        if drop > 0.0:
            _, state["lse"] = capi.attn_fwd_dropout(q, k, v, w.scale, drop, 2024, causal=w.causal, kv_len=kvl, mask=mask, out=o)
        else:
            _, state["lse"] = capi.attn_fwd(q, k, v, w.scale, causal=w.causal, kv_len=kvl, mask=mask, out=o)

    def bwd():
        if drop > 0.0:
            state["grads"] = capi.attn_bwd_dropout(q, k, v, o, do, state["lse"], w.scale, drop, 2024, causal=w.causal, kv_len=kvl,
                                                   mask=mask, workspace=ws)
        else:
            capi.attn_bwd(q, k, v, o, do, state["lse"], w.scale, causal=w.causal, kv_len=kvl, mask=mask, workspace=ws, grads=grads)

    ms, med, per_kernel = timed_loops(torch, capi, fwd, bwd, steps, warmup)
    peak_mib = torch.cuda.max_memory_allocated() / 2 ** 20

    flops_fwd, flops_bwd = w.flops(True, False), w.flops(False, True)
    tflops = (flops_fwd + flops_bwd) / (ms * 1e-3) / 1e12
    # Dominant kernel: bwd_dkdv_kernel.  Per launch it carries four of the five backward GEMMs over
    # every attended (query, key) pair: S recompute, dP, dV, dK = 8 * pairs * D flops.  The fifth
    # (dQ) runs in bwd_dq_kernel, which recomputes S and dP (6 * pairs * D executed, 2 * pairs * D
    # algorithmic).  The forward kernel carries its two GEMMs (4 * pairs * D).  With the joint schedule one
    # launch (bwd_joint_kernel) carries all five backward GEMMs: 10 * pairs * D algorithmic, 14 executed.
    pairs_d = w.valid_pairs() * D
    kern_flops = {"fwd": (4 * pairs_d, 4 * pairs_d), "bwd_dkdv": (8 * pairs_d, 8 * pairs_d),
                  "bwd_dq": (2 * pairs_d, 6 * pairs_d), "bwd_joint": (10 * pairs_d, 14 * pairs_d)}          # (algorithmic, executed)
    kernels = {}
    for kname, (alg, exe) in kern_flops.items():
        if kname in per_kernel:
            t = per_kernel[kname] * 1e-3
            kernels[kname] = {"avg_launch_ms": per_kernel[kname], "algorithmic_tflops": alg / t / 1e12,
                              "executed_tflops": exe / t / 1e12, "frac_of_peak_executed": exe / t / 1e12 / PEAK_BF16_TFLOPS}
    dom = "bwd_joint" if "bwd_joint" in kernels else "bwd_dkdv"
    achieved = kernels[dom]["algorithmic_tflops"]
    bound, bound_peak, bound_note = bound_of(w, dom, per_kernel[dom]) if dom != "bwd_joint" else ("mfma", PEAK_BF16_TFLOPS, None)
    plain = not args.keep_mask and drop == 0.0 and args.head_dim == 0 and args.bwd_schedule == "default"
    out = {
        "metric": METRIC, "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w.name, "B": B, "H": H, "Sq": Sq, "Sk": Sk, "D": D, "causal": bool(w.causal),
                   "step": "forward (O+LSE) + recompute backward (dQ,dK,dV)", "keep_mask": bool(args.keep_mask),
                   "dropout_p": drop, "bwd_schedule": args.bwd_schedule},
        "frac_of_bf16_mfma_peak": tflops / PEAK_BF16_TFLOPS,
        "timing": {"forward_ms_median": med["first_ms_median"], "backward_ms_median": med["second_ms_median"],
                   "step_ms_median": med["step_ms_median"], "step_ms_min": med["step_ms_min"], "step_ms_max": med["step_ms_max"],
                   "samples": med["samples"], "clock": "HIP events on the launch stream",
                   "forward_tflops": flops_fwd / (med["first_ms_median"] * 1e-3) / 1e12,
                   "backward_tflops": flops_bwd / (med["second_ms_median"] * 1e-3) / 1e12,
                   "step_tflops": (flops_fwd + flops_bwd) / (med["step_ms_median"] * 1e-3) / 1e12},
        # `peak` is always the published MFMA peak and `frac` the fraction of it; where something else bounds the
        # kernel, `bound` names it and `bound_peak` / `frac_of_bound` give the rate that bound allows
        "roofline": {"bound": bound, "kernel": f"{dom}_kernel", "achieved": achieved, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / PEAK_BF16_TFLOPS,
                     "traffic": recorded_traffic(w.name, f"{dom}_kernel") if plain else None,
                     "avg_launch_ms": per_kernel[dom], "flops_per_launch": kern_flops[dom][0]},
        "kernels": kernels,
        "kernels_ms": per_kernel,
        "peak_device_MiB": peak_mib,
        "saved_activations": w.saved_activation_bytes(),
    }
    if bound != "mfma":
        out["roofline"]["bound_note"] = bound_note
        if bound_peak:
            out["roofline"]["bound_peak"] = bound_peak
            out["roofline"]["frac_of_bound"] = achieved / bound_peak
    if headline:
        out["input_prep"] = input_prep_rate(capi, W, torch, B, H, Sq, D, dev)
        if plain:
            del ws
            out["materialised_comparator"] = materialised_comparator(capi, torch, q, k, v, do, w.scale, o, grads)
        if not args.no_cpu_baseline:
            out["cpu_baseline"] = cpu_baseline(w)
    return out


def summary_of(line):
    """The row a configuration contributes to the headline line's `configs`."""
    r = line["roofline"]
    row = {"workload": line["config"]["workload"], "steps": line["steps"], "ms_per_step": line["ms_per_step"],
           "step_ms_median_hip_events": line["timing"]["step_ms_median"],
           "value": line["value"], "unit": line["unit"], "dominant_kernel": r["kernel"], "roofline_bound": r["bound"],
           "roofline_frac": r["frac"], "dominant_kernel_avg_launch_ms": r["avg_launch_ms"], "kernels_ms": line["kernels_ms"]}
    if "frac_of_bf16_mfma_peak" in line:
        row["frac_of_bf16_mfma_peak"] = line["frac_of_bf16_mfma_peak"]
        row["forward_ms"] = line["timing"]["forward_ms_median"]
        row["backward_ms"] = line["timing"]["backward_ms_median"]
    else:
        row["quantise_ms"] = line["timing"]["quantise_ms_median"]
        row["forward_ms"] = line["timing"]["forward_ms_median"]
        row["frac_of_int8_bf16_blend"] = r["frac"]
    for key in ("bound_peak", "frac_of_bound", "bound_note"):
        if key in r:
            row["roofline_" + key] = r[key]
    return row


def mfma_ceiling_line(args, capi, torch, W, dev):
    """What the matrix pipe alone allows: a loop of nothing but bf16 MFMAs on bf16 N(0,1) operands, one wavefront per
    SIMD on every compute unit, with as many MFMAs as each attention kernel of the headline shape executes, next to
    those kernels' own times from the same process.  Under rocprofv3 --pmc GRBM_GUI_ACTIVE the same run gives the
    clock each of them is granted."""
    import ctypes
    from flame_amd import build as fb
    probe = ctypes.CDLL(fb.PROBE_LIB_PATH)
    probe.flame_probe_mfma_data_bytes.restype = ctypes.c_size_t
    nbytes = probe.flame_probe_mfma_data_bytes()
    g = torch.Generator(device=dev).manual_seed(5)
    data = torch.randn(nbytes // 2, device=dev, generator=g).to(torch.bfloat16)
    sink = torch.zeros(16, device=dev)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    w = W.CONFIGS[2]()
    B, H, Sq, Sk, D = w.shape
    line = attention_line(args, capi, torch, W, w, dev, min(args.steps, 50), min(args.warmup, 10), headline=False)
    pairs_d = w.valid_pairs() * D
    executed = {"fwd": 4 * pairs_d, "bwd_dq": 6 * pairs_d, "bwd_dkdv": 8 * pairs_d}
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ones = torch.ones_like(data)           # the same loop on constant operands: far fewer bits toggle per MFMA

    def time_loop(operands, iters, waves=4):
        def run():
            rc = probe.flame_probe_mfma_loop(ctypes.c_void_p(operands.data_ptr()), ctypes.c_void_p(sink.data_ptr()), cus, waves, iters, stream)
            assert rc == 0, rc

        for _ in range(5):
            run()
        times = []
        for _ in range(20):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            run()
            e1.record()
            e1.synchronize()
            times.append(e0.elapsed_time(e1))
        return statistics.median(times)

    rows = {}
    for kname, flops in executed.items():
        per_wave = flops / 32768.0 / (cus * 4)                 # MFMAs (32x32x16: 32768 flops) per wavefront
        iters = max(1, int(round(per_wave / 8)))
        loop_flops = iters * 8 * 32768.0 * cus * 4
        t_loop = time_loop(data, iters)
        t_const = time_loop(ones, iters)
        t_two = time_loop(data, max(1, iters // 2), waves=8)   # two wavefronts per SIMD, half the MFMAs each
        t_kernel = line["kernels_ms"][kname]
        rows[kname] = {"executed_flops": flops, "kernel_ms": t_kernel, "kernel_executed_tflops": flops / (t_kernel * 1e-3) / 1e12,
                       "mfma_only_loop_ms_same_mfma_count": t_loop, "mfma_only_loop_tflops": loop_flops / (t_loop * 1e-3) / 1e12,
                       "mfma_only_loop_two_wavefronts_per_simd_ms": t_two,
                       "mfma_only_loop_constant_operands_ms": t_const,
                       "mfma_only_loop_constant_operands_tflops": loop_flops / (t_const * 1e-3) / 1e12,
                       "kernel_time_over_mfma_only_time": t_kernel / t_loop}
    return {"metric": "attention kernels against an MFMA-only loop of the same MFMA count", "unit": "ms", "n_gpus": 1,
            "dtype": "bf16", "data": "synthetic", "higher_is_better": False,
            "config": {"workload": w.name, "probe": "v_mfma_f32_32x32x16_bf16 only, N(0,1) bf16 operands, 4 wavefronts per compute unit"},
            "kernels": rows, "step_ms": line["ms_per_step"]}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--config", type=int, default=0,
                    help="workload configuration 1..5 alone; default: the headline shape (2) with its extras, then 1, 3, 4, 5 "
                         "at up to 20 steps each, reported under `configs` of the one line")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--keep-mask", action="store_true",
                    help="pass an all-ones [1,1,Sq,Sk] keep-mask, which times the kernels that read an explicit mask "
                         "(same arithmetic and flop count as the unmasked step)")
    ap.add_argument("--dropout", type=float, default=0.0,
                    help="dropout probability of the attention weights: times the DROPOUT builds of the kernels")
    ap.add_argument("--head-dim", type=int, default=0,
                    help="the headline shape with another head dim (e.g. 96, which runs zero-padded on the 128-wide kernels)")
    ap.add_argument("--bwd-schedule", choices=("default", "joint", "rows"), default="default",
                    help="how the backward of the unmasked shapes is launched (FLAME_ATTN_BWD_SCHEDULE): dQ then dK/dV kernel; "
                         "a rows pre-pass and both in one grid; the pre-pass and the two kernels")
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="also run one plain 256 MiB device copy, so that FETCH_SIZE / WRITE_SIZE read under "
                         "rocprofv3 --pmc can be scaled by what the same counters report for a known size")
    ap.add_argument("--big-head-dims", action="store_true",
                    help="time the forward for head dims above 128 next to a materialised comparator (a line of its own)")
    ap.add_argument("--materialised", action="store_true",
                    help="time the materialised path (library GEMMs + element-wise kernels) on shapes the fused kernels refuse "
                         "(a line of its own)")
    ap.add_argument("--tile-ops", action="store_true",
                    help="time the element-wise tile primitives instead of an attention workload (a line of its own)")
    ap.add_argument("--mfma-ceiling", action="store_true",
                    help="time an MFMA-only loop with the MFMA count of each kernel of the headline shape (a line of its own)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (heads shard without communication; "
              "no multi-GPU path exists). Re-run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    from flame_amd import capi, workloads as W
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    capi.lib()      # fails loudly when the HIP library is missing
    if args.bwd_schedule != "default":
        os.environ["FLAME_ATTN_BWD_SCHEDULE"] = args.bwd_schedule

    dev = torch.device("cuda:0")
    if args.traffic_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        torch.empty_like(src).copy_(src)          # one elementwise copy kernel: reads 256 MiB, writes 256 MiB
        del src
    if args.tile_ops:
        return tile_ops_line(args, capi, torch, dev)
    if args.big_head_dims:
        return big_head_dims_line(args, capi, torch, dev)
    if args.materialised:
        return materialised_path_line(args, capi, torch, dev)
    if args.mfma_ceiling:
        print(json.dumps(mfma_ceiling_line(args, capi, torch, W, dev)))
        return 0

    variant = args.keep_mask or args.dropout > 0.0 or args.head_dim != 0 or args.bwd_schedule != "default"
    all_configs = args.config == 0 and not variant
    cfg = args.config or 2
    w = W.config2(D=args.head_dim) if (args.head_dim and cfg == 2) else W.CONFIGS[cfg]()
    if w.do is None:            # inference-only workload (int8-QK forward)
        print(json.dumps(sage_line(args, capi, torch, w, dev)))
        return 0
    line = attention_line(args, capi, torch, W, w, dev, args.steps, args.warmup, headline=(cfg == 2 and not args.head_dim))
    if all_configs:
        # the other four configurations, timed the same way at up to 20 steps each (cfg 4 takes 8 ms per step), one row each
        rows = {"cfg2": summary_of(line)}
        del w
        for other in (1, 3, 4, 5):
            torch.cuda.empty_cache()
            wo = W.CONFIGS[other]()
            n, nw = min(args.steps, 20), min(args.warmup, 5)
            lo = (sage_line(args, capi, torch, wo, dev, n, nw, with_cpu_baseline=False) if wo.do is None
                  else attention_line(args, capi, torch, W, wo, dev, n, nw, headline=False))
            rows[f"cfg{other}"] = summary_of(lo)
            del wo, lo
        line["configs"] = dict(sorted(rows.items()))
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
