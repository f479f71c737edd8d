#!/usr/bin/env python3
"""Benchmark of the ternary linear-layer hot path on one MI355X.

Headline workload (benchmark configuration 3): the LLaMA-3-8B decode projection sweep at batch 1 -
7 ternary GEMVs per layer (q, k, v, o, gate, up, down) x 32 layers, 1.854 GB of packed weights + scales
resident in HBM, issued as ONE launch of the multi-problem plan. A "step" is one sweep. The metric is the
packed weight+scale stream rate in GB/s (algorithmic bytes = 0.265625 * rows * cols per matrix) and its
fraction of the 8 TB/s HBM peak.

The same run measures every other benchmark configuration and reports them in `configs`:
  cfg1  one 2048 x 2048 GEMV (cache-resident, and rotated over > 512 MB of distinct matrices)
  cfg2  the LLaMA-1B layer set x 16 layers as one plan (cache-resident 258 MB, and rotated over 775 MB)
  cfg3  the 8B sweep at batch 1 (the headline), 4 and 16
  cfg4  the prefill GEMM, M in {16, 128, 512, 2048} x {gate/up 14336 x 4096, down 4096 x 14336}
  cfg5  LLaMA-70B, all 80 layers resident (18.2 GB packed), batch 1 and 16, at P(0) = 0.42, 0.2 and 0.7
  lm_head  the ternary output head (128256 x 4096 and 128256 x 8192), one GEMV per call
plus `single_calls` (the reference's own call pattern, one operator call per matrix, replayed from a
captured HIP graph so that no host time is in the figure: fp16 and int8 activations, and the dependent
chain of a decode step), `copy_ceiling` (what this GPU streams with a plain read / copy kernel) and
`cpu_baseline` (the reference's host loop, restated in C, on this machine's cores).

Every time is taken with HIP events on the launch stream around back-to-back launches, after an untimed
settle phase (the GPU idles near 100 MHz and needs tens of milliseconds of load to reach its working
clocks); `mean`, `median` and `min` are per step, the last two over groups of consecutive steps.

Prints one JSON line. `--gpus` above 1 is refused: this build measures one GPU.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0   # MI355X dense FP16 matrix peak
# HBM bytes one launch moves, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by a copy kernel of known size
# (the profile named beside each figure); valid for that workload only, and only for the kernel source it was
# profiled on: `sha256_16` is the first 16 hex digits of the sha256 of that csrc file then. The bench recomputes the
# hash and marks the figure `traffic_stale` when the file has changed since.
TRAFFIC = {
    "headline": {"bytes": 1922930278, "file": "gemv_mfma.hip", "sha256_16": "a91bf3a0bdad1f50",
                 "source": "rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE of this workload (profiles/gemv_mfma_wide__llama8b_sweep_b1.md), not read in this run"},
    4: {"bytes": 2251384729, "file": "gemv_mfma.hip", "sha256_16": "a91bf3a0bdad1f50",
        "source": "rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE of this workload (profiles/gemv_batch__llama8b_sweep_b4_b16.md), not read in this run"},
    16: {"bytes": 2085173453, "file": "gemv_batch.hip", "sha256_16": "8f870ce9ea664d7b",
         "source": "rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE of this workload (profiles/gemv_batch__llama8b_sweep_b4_b16.md), not read in this run"},
}


def traffic_fields(key, algorithmic_bytes):
    """The profiled HBM bytes per launch of a workload, with the check that the kernel source is still the one profiled."""
    import hashlib
    t = TRAFFIC[key]
    path = os.path.join(ROOT, "ternary-llm_amd", "csrc", t["file"])
    with open(path, "rb") as f:
        now = hashlib.sha256(f.read()).hexdigest()[:16]
    return {"traffic": t["bytes"], "traffic_over_algorithmic": round(t["bytes"] / algorithmic_bytes, 3),
            "traffic_source": t["source"], "traffic_profiled_on": f"{t['file']} sha256 {t['sha256_16']}",
            "traffic_stale": now != t["sha256_16"]}


SHAPES = {
    # name: (hidden, q_dim, kv_dim, ffn, layers)
    "llama1b": (2048, 2048, 512, 8192, 16),
    "llama8b": (4096, 4096, 1024, 14336, 32),
    "llama70b": (8192, 8192, 1024, 28672, 80),
}

CUSTOM = []  # filled by --matrices "ROWSxCOLS,..." (replaces the model's per-layer matrix list)


def layer_matrices(model):
    if CUSTOM:
        return [(f"m{i}", r, c) for i, (r, c) in enumerate(CUSTOM)]
    h, q, kv, ffn, _ = SHAPES[model]
    return [("q_proj", q, h), ("k_proj", kv, h), ("v_proj", kv, h), ("o_proj", h, q),
            ("gate_proj", ffn, h), ("up_proj", ffn, h), ("down_proj", h, ffn)]


def packed_bytes(rows, cols, group=128):
    return rows * (cols // 32) * 8 + rows * (cols // group) * 2


def gen_masks(torch, rows, cols, p_zero, gen):
    """i.i.d. ternary weights packed on the device: P(0)=p_zero, P(+1)=P(-1); sign bit 0 under zeros."""
    words = cols // 32
    pw = (torch.ones(32, dtype=torch.int64, device="cuda") << torch.arange(32, device="cuda"))
    nz = torch.empty((rows, words), dtype=torch.int32, device="cuda")
    sg = torch.empty((rows, words), dtype=torch.int32, device="cuda")
    step = max(1, (1 << 25) // cols)
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        u = torch.rand((r1 - r0, words, 32), device="cuda", generator=gen)
        for dst, thr in ((nz, 1.0 - p_zero), (sg, (1.0 - p_zero) / 2)):
            v = ((u < thr).to(torch.int64) * pw).sum(dim=2)
            dst[r0:r1] = torch.where(v >= 2 ** 31, v - 2 ** 32, v).to(torch.int32)
    return nz, sg


def build_sweep(torch, model, layers, batch, p_zero, scale_lo, scale_hi, seed, unit_rms=False):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    problems, meta = [], []
    for layer in range(layers):
        for name, rows, cols in layer_matrices(model):
            nz, sg = gen_masks(torch, rows, cols, p_zero, gen)
            sc = (torch.rand((rows, cols // 128), device="cuda", generator=gen) * (scale_hi - scale_lo)
                  + scale_lo).to(torch.float16)
            x = torch.randn((batch, cols), device="cuda", generator=gen)
            if unit_rms:
                x = x / torch.sqrt(torch.mean(x * x, dim=1, keepdim=True))
            x = x.to(torch.float16)
            y = torch.zeros((batch, rows), dtype=torch.float16, device="cuda")
            problems.append((nz, sg, sc, x, y, rows, cols, batch))
            meta.append((layer, name))
    return problems, meta


def with_batch(torch, problems, batch, seed):
    """The same weights with `batch` activation rows per matrix."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    out = []
    for (nz, sg, sc, _, _, rows, cols, _) in problems:
        x = torch.randn((batch, cols), device="cuda", generator=gen).to(torch.float16)
        y = torch.zeros((batch, rows), dtype=torch.float16, device="cuda")
        out.append((nz, sg, sc, x, y, rows, cols, batch))
    return out


def check_sample(oracle, problems, idxs, rows_per=64, seed=0):
    """Sampled rows of a few problems against the fp64 oracle; returns the worst max_rel."""
    rng = np.random.default_rng(seed)
    worst = 0.0
    for i in idxs:
        nz, sg, sc, x, y, rows, cols, batch = problems[i]
        pick = np.sort(rng.choice(rows, size=min(rows_per, rows), replace=False))
        nzs = nz[pick].cpu().numpy().view(np.uint32)
        sgs = sg[pick].cpu().numpy().view(np.uint32)
        scs = sc[pick].cpu().numpy().view(np.uint16)
        xs = x.cpu().numpy().view(np.uint16)
        got = y[:, pick].cpu().numpy().astype(np.float64)
        ref = oracle.gemm_f64(xs, nzs, sgs, scs)
        # the error floor uses the rms of the whole output vector, not of the sample
        full = y.float()
        tau = float((full * full).mean().sqrt().item()) / 64.0
        rel = np.abs(got - ref) / np.maximum(np.abs(ref), tau)
        worst = max(worst, float(rel.max()))
    return worst


class Timer:
    """HIP-event timing of back-to-back launches on torch's current stream (the stream every launch of
    this file uses). Untimed: launches for `settle_ms`, then `warmup` more. Timed: `steps` launches, with an
    event between groups of consecutive launches so that a median and a minimum exist beside the mean."""

    def __init__(self, torch, settle_ms):
        self.torch = torch
        self.settle_ms = settle_ms

    def run(self, fn, steps, warmup):
        torch = self.torch
        untimed = 0
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < self.settle_ms:
            for _ in range(10):
                fn()
            untimed += 10
            torch.cuda.synchronize()
        for _ in range(warmup):
            fn()
        untimed += warmup
        torch.cuda.synchronize()
        group = max(1, steps // 20)
        n_groups = (steps + group - 1) // group
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(n_groups + 1)]
        done = 0
        ev[0].record()
        for g in range(n_groups):
            n = min(group, steps - done)
            for _ in range(n):
                fn()
            done += n
            ev[g + 1].record()
        torch.cuda.synchronize()
        per = []
        done = 0
        for g in range(n_groups):
            n = min(group, steps - done)
            done += n
            per.append(ev[g].elapsed_time(ev[g + 1]) / n)
        total = ev[0].elapsed_time(ev[n_groups])
        return {"mean_ms": total / steps, "median_ms": float(np.median(per)), "min_ms": float(np.min(per)),
                "steps": steps, "untimed_launches": untimed, "steps_per_timing_group": group}


def stats_us(t):
    return {"us": round(t["mean_ms"] * 1e3, 2), "us_median": round(t["median_ms"] * 1e3, 2),
            "us_min": round(t["min_ms"] * 1e3, 2), "steps": t["steps"], "untimed_launches": t["untimed_launches"]}


def hbm_row(name, t, nbytes, kernel, parity=None, note=None):
    gbps = nbytes / (t["mean_ms"] * 1e-3) / 1e9
    row = {"config": name, **stats_us(t), "packed_bytes": nbytes, "GBps": round(gbps, 1),
           "GBps_best": round(nbytes / (t["min_ms"] * 1e-3) / 1e9, 1), "bound": "hbm",
           "frac_hbm_peak": round(gbps / HBM_PEAK_GBS, 4), "kernel": kernel}
    if parity is not None:
        row["parity_max_rel_sampled"] = parity
    if note:
        row["note"] = note
    return row


def capture(torch, fn):
    """Records fn's launches into a HIP graph on a side stream; returns the graph (replay() = one step)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        fn()                      # warm-up on the capture stream (per-stream state is created here, not under capture)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            fn()
    torch.cuda.synchronize()
    return graph


def cfg1_rows(torch, tl, orc, timer, seed):
    """One 2048 x 2048 GEMV per call (the reference's own test shape, 1.1 MB packed). A call is far below
    the launch floor, so the row is latency, not bandwidth. Calls are replayed from a captured graph (no
    host time): 256 calls on ONE matrix (cache-resident) and 512 calls over 512 distinct matrices
    (582 MB, beyond L2 and the 256 MB Infinity Cache)."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed + 11)
    rows = cols = 2048
    n_distinct = 512
    nz, sg = gen_masks(torch, rows * 8, cols, 0.42, gen)    # 8 matrices of random bits, reused with offsets below
    nz_all = nz.repeat(n_distinct // 8, 1).contiguous()
    sg_all = sg.repeat(n_distinct // 8, 1).contiguous()
    sc_all = (torch.rand((rows * n_distinct, cols // 128), device="cuda", generator=gen) * 0.02 + 0.01).to(torch.float16)
    x = torch.randn((1, cols), device="cuda", generator=gen).to(torch.float16)
    y = torch.zeros((n_distinct, rows), dtype=torch.float16, device="cuda")
    mats = [(nz_all[i * rows:(i + 1) * rows], sg_all[i * rows:(i + 1) * rows], sc_all[i * rows:(i + 1) * rows]) for i in range(n_distinct)]

    def same():
        for _ in range(256):
            tl.ternary_gemv(*mats[0], x, y[0], rows, cols, 128)

    def rotated():
        for i in range(n_distinct):
            tl.ternary_gemv(*mats[i], x, y[i], rows, cols, 128)

    out = []
    nbytes = packed_bytes(rows, cols)
    for name, fn, calls, note in (("cfg1: 2048x2048 GEMV, same matrix (cache-resident)", same, 256,
                                   "1.1 MB of weights stay in L2: latency of one launch, not HBM bandwidth"),
                                  ("cfg1: 2048x2048 GEMV, rotated over 512 distinct matrices (582 MB)", rotated, n_distinct,
                                   "every call reads weights that left the caches")):
        graph = capture(torch, fn)
        t = timer.run(graph.replay, 20, 3)
        per_call = {k: v / calls for k, v in t.items() if k.endswith("_ms")}
        row = hbm_row(name, {**t, **per_call}, nbytes, "tllm::gemv_mfma_kernel<Wide, fine>", note=note)
        row["calls_per_graph_replay"] = calls
        out.append(row)
        del graph
    probs = [(mats[3][0], mats[3][1], mats[3][2], x, y[3:4], rows, cols, 1)]
    out[1]["parity_max_rel_sampled"] = check_sample(orc, probs, [0])
    return out


def plan_rows(torch, tl, orc, timer, label, model, layers, batches, p_zero, lo, hi, seed, steps, warmup, copies=1,
              unit_rms=False, problems=None):
    """A model's projection sweep as one plan launch per step, for each batch size. copies > 1: that many
    distinct weight sets, launched in turn (a step = one set), so that no set is still in a cache when its
    turn comes again."""
    sets = [problems] if problems is not None else []
    while len(sets) < copies:
        sets.append(build_sweep(torch, model, layers, 1, p_zero, lo, hi, seed + 1000 * len(sets), unit_rms)[0])
    nbytes = sum(packed_bytes(p[5], p[6]) for p in sets[0])
    rows = []
    for b in batches:
        psets = [s if b == 1 else with_batch(torch, s, b, seed + 100 + b) for s in sets]
        plans = [tl.LinearPlan(ps) for ps in psets]
        turn = [0]

        def step():
            plans[turn[0] % len(plans)].launch()
            turn[0] += 1

        t = timer.run(step, steps, warmup)
        n = len(psets[0])
        parity = check_sample(orc, psets[-1], sorted(set([0, 1, 4, 6, n - 1, n // 2])))
        note = None
        if copies > 1:
            note = f"rotated over {copies} distinct weight sets ({copies * nbytes} bytes)"
        elif nbytes < 512 * 1024 * 1024:
            note = "cache-resident: the set fits the 256 MB Infinity Cache, so the figure is not an HBM rate"
        rows.append(hbm_row(f"{label}, batch {b}", t, nbytes, plans[0].kernel, parity, note))
        rows[-1]["matrices_per_launch"] = n
        for pl in plans:
            pl.close()
        del psets, plans
    return rows, sets[0]


def int8_sweep_row(torch, tl, orc, timer, label, problems, steps, warmup):
    """The same sweep on INT8 activations (the reference's decode path, ternary_gemv_int8 per linear): every input
    vector quantised once by quantize_absmax_int8 outside the timed region, then one plan launch per step over the
    int8 vectors and their device-resident scales. Sampled rows against the oracle's integer arithmetic."""
    probs, scales = [], []
    for (nz, sg, sc, x, y, rows, cols, _) in problems:
        q = torch.zeros(cols, dtype=torch.int8, device="cuda")
        qs = torch.zeros(1, dtype=torch.float32, device="cuda")
        tl.quantize_absmax_int8(x, q, qs, cols)
        probs.append((nz, sg, sc, q, torch.zeros((1, rows), dtype=torch.float16, device="cuda"), rows, cols, 1))
        scales.append(qs)
    torch.cuda.synchronize()
    plan = tl.LinearPlan(probs, input_scales=scales)
    t = timer.run(plan.launch, steps, warmup)
    nbytes = sum(packed_bytes(p[5], p[6]) for p in probs)
    rng = np.random.default_rng(3)
    worst = 0.0
    n = len(probs)
    for i in sorted(set([0, 1, 4, 6, n - 1, n // 2])):
        nz, sg, sc, q, y, rows, cols, _ = probs[i]
        pick = np.sort(rng.choice(rows, size=min(64, rows), replace=False))
        ref = orc.gemv_i8_f64(nz[pick].cpu().numpy().view(np.uint32), sg[pick].cpu().numpy().view(np.uint32),
                              sc[pick].cpu().numpy().view(np.uint16), q.cpu().numpy(), float(scales[i].item()))
        full = y.float()
        tau = float((full * full).mean().sqrt().item()) / 64.0
        got = y[0, pick].cpu().numpy().astype(np.float64)
        worst = max(worst, float((np.abs(got - ref) / np.maximum(np.abs(ref), tau)).max()))
    row = hbm_row(label, t, nbytes, plan.kernel + " on int8 activations", worst)
    row["matrices_per_launch"] = n
    plan.close()
    return row


def gemm_rows(torch, tl, orc, timer, seed, m_list, p_zero, calls, warm):
    """Prefill GEMM (cfg4): LLaMA-3-8B gate/up 14336x4096 and down 4096x14336, M tokens each; dense-equivalent
    2*M*N*K flops against the FP16 matrix peak (M = 16 is HBM-bound and also gets its weight-stream rate).
    For M > 16 the same shape is also timed as a dense fp16 product of the vendor library (torch.matmul on a
    dense fp16 matrix with the same value distribution: 42 % zeros, +-scale): what the matrix cores of this
    box deliver on these operands when the weights need no decoding (`dense_fp16_us`, `vs_dense_fp16` =
    that time / ours)."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed + 4)
    rows = []
    for (n, k) in ((14336, 4096), (4096, 14336)):
        nz, sg = gen_masks(torch, n, k, p_zero, gen)
        sc = (torch.rand((n, k // 128), device="cuda", generator=gen) * 0.02 + 0.01).to(torch.float16)
        dense = None
        if any(m > 16 for m in m_list):
            dense = torch.empty((n, k), dtype=torch.float16, device="cuda")
            step = max(1, (1 << 24) // k)
            for r0 in range(0, n, step):
                r1 = min(n, r0 + step)
                u = torch.rand((r1 - r0, k), device="cuda", generator=gen)
                w = torch.where(u < p_zero, 0.0, torch.where(u < (1.0 + p_zero) / 2, 1.0, -1.0))
                dense[r0:r1] = (w * sc[r0:r1].float().repeat_interleave(128, dim=1)).to(torch.float16)
                del u, w
        for m in m_list:
            a = torch.randn((m, k), device="cuda", generator=gen).to(torch.float16)
            c = torch.zeros((m, n), dtype=torch.float16, device="cuda")
            t = timer.run(lambda: tl.ternary_gemm(a, nz, sg, sc, c, m, n, k, 128), calls, warm)
            t_dense = None
            if dense is not None and m > 16:
                cd = torch.empty((m, n), dtype=torch.float16, device="cuda")
                t_dense = timer.run(lambda: torch.matmul(a, dense.t(), out=cd), calls, warm)
                del cd
            rng = np.random.default_rng(m + n)
            ms_ = np.unique(rng.integers(0, m, 4))
            ns_ = np.unique(rng.integers(0, n, 96))
            ref = orc.gemm_f64(a[ms_].cpu().numpy().view(np.uint16), nz[ns_].cpu().numpy().view(np.uint32),
                               sg[ns_].cpu().numpy().view(np.uint32), sc[ns_].cpu().numpy().view(np.uint16))
            full = c.float()
            tau = float(torch.sqrt(torch.mean(full * full)).item()) / 64.0
            got = full.cpu().numpy().astype(np.float64)[np.ix_(ms_, ns_)]
            rel = float((np.abs(got - ref) / np.maximum(np.abs(ref), tau)).max())
            tflops = 2.0 * m * n * k / (t["mean_ms"] * 1e-3) / 1e12
            row = {"config": f"cfg4: prefill GEMM M={m}, W {n}x{k}", "M": m, "N": n, "K": k, **stats_us(t),
                   "tflops": round(tflops, 1), "tflops_best": round(2.0 * m * n * k / (t["min_ms"] * 1e-3) / 1e12, 1),
                   "bound": "mfma" if m > 16 else "hbm", "frac_mfma_peak": round(tflops / MFMA_F16_PEAK_TFLOPS, 4),
                   "kernel": tl.gemm_kernel(m, n, k), "max_rel_sampled": rel}
            if t_dense is not None:
                row["dense_fp16_us"] = round(t_dense["mean_ms"] * 1e3, 2)
                row["dense_fp16_tflops"] = round(2.0 * m * n * k / (t_dense["mean_ms"] * 1e-3) / 1e12, 1)
                row["vs_dense_fp16"] = round(t_dense["mean_ms"] / t["mean_ms"], 3)
            if m <= 16:
                gb = packed_bytes(n, k) / (t["mean_ms"] * 1e-3) / 1e9
                row["GBps"] = round(gb, 1)
                row["frac_hbm_peak"] = round(gb / HBM_PEAK_GBS, 4)
            rows.append(row)
            del a, c, full
        del dense
        del nz, sg, sc
    return rows


def ffn_front_rows(torch, tl, timer, seed, m_list, p_zero, calls, warm):
    """The FFN front half of a prefill step on the 8B shapes (reference src/transformer.cpp:264-286 at n_tokens > 1):
    ternary_gemm on gate, ternary_gemm on up and silu_mul as the reference issues them, and as ONE launch
    (tllm_ternary_gemm_swiglu_f16). Flops counted for both products (4*M*N*K); the outputs are compared bit for bit."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed + 44)
    n, k = 14336, 4096
    rows = []
    g_nz, g_sg = gen_masks(torch, n, k, p_zero, gen)
    u_nz, u_sg = gen_masks(torch, n, k, p_zero, gen)
    g_sc = (torch.rand((n, k // 128), device="cuda", generator=gen) * 0.02 + 0.01).to(torch.float16)
    u_sc = (torch.rand((n, k // 128), device="cuda", generator=gen) * 0.02 + 0.01).to(torch.float16)
    for m in m_list:
        if m <= 16:
            continue
        a = torch.randn((m, k), device="cuda", generator=gen).to(torch.float16)
        g, u, one = (torch.zeros((m, n), dtype=torch.float16, device="cuda") for _ in range(3))

        def three():
            tl.ternary_gemm(a, g_nz, g_sg, g_sc, g, m, n, k, 128)
            tl.ternary_gemm(a, u_nz, u_sg, u_sc, u, m, n, k, 128)
            tl.silu_mul(g, u, g, m * n)

        t3 = timer.run(three, calls, warm)
        t1 = timer.run(lambda: tl.ternary_gemm_swiglu(a, g_nz, g_sg, g_sc, u_nz, u_sg, u_sc, one, m, n, k, 128), calls, warm)
        floor = float(torch.sqrt(torch.mean(g.float() ** 2)).item()) / 64.0
        rel = float(((one.float() - g.float()).abs() / torch.clamp(g.float().abs(), min=floor)).max().item())
        flops = 4.0 * m * n * k
        for name, t, kern in (("gate GEMM + up GEMM + SiLU*mul, three launches", t3, tl.gemm_kernel(m, n, k) + " x 2, silu_mul_kernel"),
                              ("gate/up/SiLU*mul in one launch", t1, "tllm::gemm_ns_kernel<4, 2, pair>")):
            tf = flops / (t["mean_ms"] * 1e-3) / 1e12
            rows.append({"config": f"cfg4: prefill FFN front half M={m}, 2 x W {n}x{k}: {name}", "M": m, "N": n, "K": k, **stats_us(t),
                         "tflops": round(tf, 1), "bound": "mfma", "frac_mfma_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                         "kernel": kern, "max_rel_one_launch_vs_three": rel})
        del a, g, u, one
    return rows


def qkv_prefill_rows(torch, tl, timer, seed, m_list, p_zero, calls, warm):
    """The q, k and v projections of a prefill step on the 8B shapes (reference src/transformer.cpp:199-217 at
    n_tokens > 1): three ternary_gemm calls as the reference issues them, and ONE launch whose tiles are dealt to the
    workgroups together (tllm_ternary_gemm_group_f16). Flops of the three products; the outputs of the two ways are
    compared (same arithmetic; where a tile is split along K the order of the fp32 additions may differ)."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed + 45)
    k, ns = 4096, (4096, 1024, 1024)
    ws = []
    for n in ns:
        nz, sg = gen_masks(torch, n, k, p_zero, gen)
        ws.append((nz, sg, (torch.rand((n, k // 128), device="cuda", generator=gen) * 0.02 + 0.01).to(torch.float16)))
    rows = []
    for m in m_list:
        if m <= 16:
            continue
        a = torch.randn((m, k), device="cuda", generator=gen).to(torch.float16)
        sep = [torch.zeros((m, n), dtype=torch.float16, device="cuda") for n in ns]
        grp = [torch.zeros((m, n), dtype=torch.float16, device="cuda") for n in ns]

        def three():
            for n, w, o in zip(ns, ws, sep):
                tl.ternary_gemm(a, *w, o, m, n, k, 128)

        t3 = timer.run(three, calls, warm)
        t1 = timer.run(lambda: tl.ternary_gemm_group(a, ws, grp, m, k), calls, warm)
        rel = 0.0
        for x, y in zip(sep, grp):
            floor = float(torch.sqrt(torch.mean(x.float() ** 2)).item()) / 64.0
            rel = max(rel, float(((y.float() - x.float()).abs() / torch.clamp(x.float().abs(), min=floor)).max().item()))
        flops = 2.0 * m * sum(ns) * k
        for name, t, kern in (("three launches", t3, " + ".join(tl.gemm_kernel(m, n, k) for n in ns)),
                              ("one launch", t1, "tllm::gemm_ns_kernel<4, 1, group>")):
            tf = flops / (t["mean_ms"] * 1e-3) / 1e12
            rows.append({"config": f"cfg4: prefill q/k/v M={m}, W 4096+1024+1024 x {k}: {name}", "M": m, "N": sum(ns), "K": k, **stats_us(t),
                         "tflops": round(tf, 1), "bound": "mfma", "frac_mfma_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                         "kernel": kern, "max_rel_one_launch_vs_three": rel})
        del a, sep, grp
    return rows


def single_call_rows(torch, tl, timer, problems, model, layers):
    """The reference's call pattern on the headline weights: one operator call per matrix
    (src/transformer.cpp:102-118), all calls of a sweep captured once into a HIP graph and replayed, so the
    time holds launch and kernel costs but no host time. fp16 activations (ternary_gemv), int8 activations
    (quantize_absmax_int8 once per layer input + ternary_gemv_int8 with the device-resident scale), and the
    dependent chain of a decode step's linear side in its three forms."""
    n = len(problems)
    nbytes = sum(packed_bytes(p[5], p[6]) for p in problems)
    out = []

    def f16_calls():
        for nz, sg, sc, x, y, rows, cols, _ in problems:
            tl.ternary_gemv(nz, sg, sc, x, y, rows, cols, 128)

    q8 = {c: torch.zeros(c, dtype=torch.int8, device="cuda") for c in {p[6] for p in problems}}
    qs = {c: torch.zeros(1, dtype=torch.float32, device="cuda") for c in q8}

    def i8_calls():   # the reference's ternary_linear_int8 (src/transformer.cpp:132-142), without its device-to-host copy of the scale
        for nz, sg, sc, x, y, rows, cols, _ in problems:
            tl.quantize_absmax_int8(x, q8[cols], qs[cols], cols)
            tl.ternary_gemv_int8(nz, sg, sc, q8[cols], qs[cols], y, rows, cols, 128)

    def i8_fused_calls():   # the same linear as ONE launch: quantised inside the GEMV, bit-identical to the pair
        for nz, sg, sc, x, y, rows, cols, _ in problems:
            tl.ternary_linear_int8(nz, sg, sc, x, y, rows, cols, 128)

    for name, fn, kernel in ((f"single calls, fp16 activations: {n} x ternary_gemv from one graph", f16_calls, "tllm::gemv_mfma_kernel<Wide, fine>"),
                             (f"single calls, int8 linear in one launch: {n} x ternary_linear_int8 (quantised inside the GEMV) from one graph", i8_fused_calls,
                              "tllm::gemv_mfma_kernel<Wide, fine>, input quantised in the staging pass"),
                             (f"single calls, int8 activations: {n} x (quantize_absmax_int8 + ternary_gemv_int8) from one graph", i8_calls,
                              "tllm::gemv_mfma_kernel<Wide, fine> on int8 activations")):
        graph = capture(torch, fn)
        t = timer.run(graph.replay, 30, 5)
        row = hbm_row(name, t, nbytes, kernel)
        row["us_per_call"] = round(t["mean_ms"] * 1e3 / n, 2)
        out.append(row)
        del graph
    chain = decode_chain(torch, tl, problems, model, layers)
    for name, fn, launches in chain["variants"]:
        graph = capture(torch, fn)
        t = timer.run(graph.replay, 30, 5)
        row = hbm_row(f"decode chain ({name}), {layers} layers, dependent order, from one graph", t, nbytes, "several")
        row["launches_per_token"] = launches * layers
        row["us_per_launch"] = round(t["mean_ms"] * 1e3 / (launches * layers), 2)
        out.append(row)
        del graph
    chain["close"]()
    return out


def decode_chain(torch, tl, problems, model, layers):
    """The linear-side launches of a batch-1 decode step over the sweep's own weights, issued in the order a
    transformer needs them (every launch after the one before, as reference src/transformer.cpp:193-296
    does): (a) the reference's ten launches per layer, (b) q/k/v and gate/up as plans, (c) RMSNorm prologue +
    SwiGLU pair: four launches per layer."""
    h, qd, kvd, ffn, _ = SHAPES[model]
    f16 = dict(dtype=torch.float16, device="cuda")
    x = torch.randn((1, h), device="cuda").to(torch.float16)
    xn, att = torch.empty_like(x), torch.randn((1, qd), device="cuda").to(torch.float16)
    q, k, v = torch.zeros((1, qd), **f16), torch.zeros((1, kvd), **f16), torch.zeros((1, kvd), **f16)
    o, g, u, d = torch.zeros((1, h), **f16), torch.zeros((1, ffn), **f16), torch.zeros((1, ffn), **f16), torch.zeros((1, h), **f16)
    eps, L = 1e-5, []
    for l in range(layers):
        w = {name: problems[7 * l + i][:3] for i, name in enumerate(("q", "k", "v", "o", "g", "u", "d"))}
        w["n1"], w["n2"] = torch.ones(h, **f16), torch.ones(h, **f16)
        w["qkv"] = tl.LinearPlan([(*w["q"], xn, q, qd, h, 1), (*w["k"], xn, k, kvd, h, 1), (*w["v"], xn, v, kvd, h, 1)])
        w["gu"] = tl.LinearPlan([(*w["g"], xn, g, ffn, h, 1), (*w["u"], xn, u, ffn, h, 1)])
        w["qkv_n"] = tl.LinearPlan([(*w["q"], x, q, qd, h, 1), (*w["k"], x, k, kvd, h, 1), (*w["v"], x, v, kvd, h, 1)],
                                   norm_weights=[w["n1"]] * 3, eps=eps)
        w["gu_n"] = tl.LinearPlan([(*w["g"], x, g, ffn, h, 1, tl.SWIGLU_GATE), (*w["u"], x, None, ffn, h, 1)],
                                  norm_weights=[w["n2"]] * 2, eps=eps)
        L.append(w)

    def ten():
        for w in L:
            tl.rmsnorm(x, w["n1"], xn, None, None, 1, h, eps)
            tl.ternary_gemv(*w["q"], xn, q, qd, h, 128)
            tl.ternary_gemv(*w["k"], xn, k, kvd, h, 128)
            tl.ternary_gemv(*w["v"], xn, v, kvd, h, 128)
            tl.ternary_gemv(*w["o"], att, o, h, qd, 128)
            tl.rmsnorm(x, w["n2"], xn, None, None, 1, h, eps)
            tl.ternary_gemv(*w["g"], xn, g, ffn, h, 128)
            tl.ternary_gemv(*w["u"], xn, u, ffn, h, 128)
            tl.silu_mul(g, u, g, ffn)
            tl.ternary_gemv(*w["d"], g, d, h, ffn, 128)

    def seven():
        for w in L:
            tl.rmsnorm(x, w["n1"], xn, None, None, 1, h, eps)
            w["qkv"].launch()
            tl.ternary_gemv(*w["o"], att, o, h, qd, 128)
            tl.rmsnorm(x, w["n2"], xn, None, None, 1, h, eps)
            w["gu"].launch()
            tl.silu_mul(g, u, g, ffn)
            tl.ternary_gemv(*w["d"], g, d, h, ffn, 128)

    def four():
        for w in L:
            w["qkv_n"].launch()
            tl.ternary_gemv(*w["o"], att, o, h, qd, 128)
            w["gu_n"].launch()
            tl.ternary_gemv(*w["d"], g, d, h, ffn, 128)

    # Staged plans: the dependent launches of a layer as stages of one launch (waits at device counters between the
    # stages instead of kernel boundaries); the residual adds ride in the epilogues of o_proj and down_proj.
    # (the residual stream goes x -> xs -> x3 and is not fed back from layer to layer here: every layer adds to the
    # same start vector, so that replaying the chain thousands of times does not walk the stream off to infinity)
    xs, x3 = torch.zeros((1, h), **f16), torch.zeros((1, h), **f16)
    for l, w in enumerate(L):
        nxt = L[l + 1] if l + 1 < len(L) else None
        ogd = [(*w["o"], att, xs, h, qd, 1), (*w["g"], xs, g, ffn, h, 1, tl.SWIGLU_GATE), (*w["u"], xs, None, ffn, h, 1),
               (*w["d"], g, x3, h, ffn, 1)]
        norms, res, stages = [None, w["n2"], w["n2"], None], [x, None, None, xs], [0, 1, 1, 2]
        w["ogd"] = tl.LinearPlan(ogd, norm_weights=norms, eps=eps, stages=stages, residuals=res)
        if nxt is not None:
            ogd = ogd + [(*nxt["q"], x3, q, qd, h, 1), (*nxt["k"], x3, k, kvd, h, 1), (*nxt["v"], x3, v, kvd, h, 1)]
            w["ogdq"] = tl.LinearPlan(ogd, norm_weights=norms + [nxt["n1"]] * 3, eps=eps, stages=stages + [3, 3, 3],
                                      residuals=res + [None] * 3)
        else:
            w["ogdq"] = w["ogd"]
        w["qkv_s"] = tl.LinearPlan([(*w["q"], x3, q, qd, h, 1), (*w["k"], x3, k, kvd, h, 1), (*w["v"], x3, v, kvd, h, 1)],
                                   norm_weights=[w["n1"]] * 3, eps=eps)

    # The reference's decode step proper is INT8 (src/transformer.cpp:176: use_int8 = n_tokens == 1): every linear runs
    # on the absmax-quantised input, the int8 vector shared inside a group. Its launches (the four copies of the scale
    # to the host per layer left out: the scale stays on the device here), the same as four launches per layer (norm
    # prologue + quantisation inside the launch + SwiGLU pair), and as one staged launch per layer.
    Q = tl.QUANTIZE_INPUT
    i8, i8s = torch.zeros(max(h, qd, ffn), dtype=torch.int8, device="cuda"), torch.zeros(1, dtype=torch.float32, device="cuda")
    for l, w in enumerate(L):
        nxt = L[l + 1] if l + 1 < len(L) else None
        w["qkv_q"] = tl.LinearPlan([(*w["q"], x, q, qd, h, 1, Q), (*w["k"], x, k, kvd, h, 1, Q), (*w["v"], x, v, kvd, h, 1, Q)],
                                   norm_weights=[w["n1"]] * 3, eps=eps)
        w["gu_q"] = tl.LinearPlan([(*w["g"], x, g, ffn, h, 1, tl.SWIGLU_GATE | Q), (*w["u"], x, None, ffn, h, 1)],
                                  norm_weights=[w["n2"]] * 2, eps=eps)
        ogd = [(*w["o"], att, xs, h, qd, 1, Q), (*w["g"], xs, g, ffn, h, 1, tl.SWIGLU_GATE | Q), (*w["u"], xs, None, ffn, h, 1),
               (*w["d"], g, x3, h, ffn, 1, Q)]
        norms, res, stages = [None, w["n2"], w["n2"], None], [x, None, None, xs], [0, 1, 1, 2]
        if nxt is not None:
            ogd = ogd + [(*nxt["q"], x3, q, qd, h, 1, Q), (*nxt["k"], x3, k, kvd, h, 1, Q), (*nxt["v"], x3, v, kvd, h, 1, Q)]
            norms, res, stages = norms + [nxt["n1"]] * 3, res + [None] * 3, stages + [3, 3, 3]
        w["ogdq_q"] = tl.LinearPlan(ogd, norm_weights=norms, eps=eps, stages=stages, residuals=res)

    def int8_reference():
        for w in L:
            tl.rmsnorm(x, w["n1"], xn, None, None, 1, h, eps)
            tl.quantize_absmax_int8(xn, i8, i8s, h)
            tl.ternary_gemv_int8(*w["q"], i8, i8s, q, qd, h, 128)
            tl.ternary_gemv_int8(*w["k"], i8, i8s, k, kvd, h, 128)
            tl.ternary_gemv_int8(*w["v"], i8, i8s, v, kvd, h, 128)
            tl.quantize_absmax_int8(att, i8, i8s, qd)
            tl.ternary_gemv_int8(*w["o"], i8, i8s, o, h, qd, 128)
            tl.rmsnorm(x, w["n2"], xn, None, None, 1, h, eps)
            tl.quantize_absmax_int8(xn, i8, i8s, h)
            tl.ternary_gemv_int8(*w["g"], i8, i8s, g, ffn, h, 128)
            tl.ternary_gemv_int8(*w["u"], i8, i8s, u, ffn, h, 128)
            tl.silu_mul(g, u, g, ffn)
            tl.quantize_absmax_int8(g, i8, i8s, ffn)
            tl.ternary_gemv_int8(*w["d"], i8, i8s, d, h, ffn, 128)

    def int8_four():
        for w in L:
            w["qkv_q"].launch()
            tl.ternary_linear_int8(*w["o"], att, o, h, qd, 128)
            w["gu_q"].launch()
            tl.ternary_linear_int8(*w["d"], g, d, h, ffn, 128)

    def int8_one():
        L[0]["qkv_q"].launch()
        for w in L:
            w["ogdq_q"].launch()

    def two():
        for w in L:
            w["qkv_s"].launch()
            w["ogd"].launch()

    def one():
        L[0]["qkv_s"].launch()
        for w in L:
            w["ogdq"].launch()

    def close():
        for w in L:
            for key in ("qkv", "gu", "qkv_n", "gu_n", "qkv_s", "ogd", "qkv_q", "gu_q", "ogdq_q"):
                w[key].close()
            if w["ogdq"] is not w["ogd"]:
                w["ogdq"].close()

    return {"variants": (("the reference's 10 launches per layer", ten, 10), ("q/k/v and gate/up as plans: 7 per layer", seven, 7),
                         ("RMSNorm prologue + SwiGLU pair: 4 per layer", four, 4),
                         ("staged plan o_proj -> gate/up -> down_proj with the residual adds, q/k/v apart: 2 launches per layer", two, 2),
                         ("staged plan o_proj -> gate/up -> down_proj -> q/k/v of the next layer: 1 launch per layer", one, 1),
                         ("INT8 decode as the reference issues it: 14 launches per layer, scales kept on the device", int8_reference, 14),
                         ("INT8 decode, RMSNorm prologue + quantisation in the launch + SwiGLU pair: 4 per layer", int8_four, 4),
                         ("INT8 decode as one staged launch per layer", int8_one, 1)),
            "close": close}


def lm_head_rows(torch, tl, orc, timer, seed):
    """The ternary output head of a .tllm model (reference src/transformer.cpp:308-311: ternary_linear on
    vocab x hidden): one batch-1 GEMV per call on 128256 x 4096 (8B) and 128256 x 8192 (70B), back-to-back calls."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed + 77)
    out = []
    for rows, cols in ((128256, 4096), (128256, 8192)):
        nz, sg = gen_masks(torch, rows, cols, 0.42, gen)
        sc = (torch.rand((rows, cols // 128), device="cuda", generator=gen) * 0.02 + 0.01).to(torch.float16)
        x = torch.randn((1, cols), device="cuda", generator=gen).to(torch.float16)
        y = torch.zeros((1, rows), dtype=torch.float16, device="cuda")
        t = timer.run(lambda: tl.ternary_gemv(nz, sg, sc, x, y, rows, cols, 128), 100, 10)
        parity = check_sample(orc, [(nz, sg, sc, x, y, rows, cols, 1)], [0])
        out.append(hbm_row(f"lm_head: {rows}x{cols} GEMV, one call", t, packed_bytes(rows, cols), "tllm::gemv_mfma_kernel<Wide>", parity,
                           "the same matrix every call: " + ("fits" if packed_bytes(rows, cols) < 256 * 2 ** 20 else "exceeds") + " the 256 MB Infinity Cache"))
        del nz, sg, sc
    return out


def copy_ceiling(torch, tl, timer):
    """What this GPU moves with nothing to compute: a read-only pass over 4 GiB (the library's streaming kernel:
    16-byte non-temporal loads; a few launch shapes are tried and the best is kept) and a device-to-device copy of
    2 GiB (bytes read + bytes written)."""
    src = torch.ones(1 << 30, dtype=torch.int32, device="cuda")
    best = None
    for shape in ("3,16", "8,8", "24,4", "32,8"):   # workgroups per CU, loads in flight per thread
        per_cu, flight = (int(v) for v in shape.split(","))
        tl.set_tuning("read_wgs_per_cu", per_cu)
        tl.set_tuning("read_in_flight", flight)
        t = timer.run(lambda: tl.read_stream(src), 20, 3)
        rate = src.numel() * 4 / (t["mean_ms"] * 1e-3) / 1e9
        if best is None or rate > best[0]:
            best = (rate, src.numel() * 4 / (t["min_ms"] * 1e-3) / 1e9, shape)
    tl.set_tuning("read_wgs_per_cu", 8)
    tl.set_tuning("read_in_flight", 8)
    half = src[: 1 << 29]
    dst = torch.empty_like(half)
    t2 = timer.run(lambda: dst.copy_(half), 20, 3)
    copy = 2 * half.numel() * 4 / (t2["mean_ms"] * 1e-3) / 1e9
    del src, dst
    return {"read_only_GBps": round(best[0], 1), "read_only_GBps_best": round(best[1], 1), "read_only_frac_hbm_peak": round(best[0] / HBM_PEAK_GBS, 4),
            "read_only_launch_shape": best[2], "copy_read_plus_write_GBps": round(copy, 1),
            "what": "tllm_read_stream over 4 GiB (best of four launch shapes); torch copy_ of 2 GiB (hipMemcpy device to device)"}


def cpu_baseline(oracle, torch, shape_sets, threads):
    """The reference's fp32 host loop (tests/test_ternary_gemv.cu:40-75, restated in C in oracle/), batch 1,
    on this machine's host cores: every matrix shape of configurations 1-3 and one full 70B layer, single
    threaded (the reference's own form) and split by rows over `threads` threads. A bounded sample: about
    10-20 s of CPU time."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(99)
    rows_out = []
    tot = {"st_bytes": 0, "st_s": 0.0, "mt_bytes": 0, "mt_s": 0.0}
    for label, shapes in shape_sets:
        st_b = st_t = mt_t = 0.0
        for (rows, cols) in shapes:
            nz, sg = gen_masks(torch, rows, cols, 0.42, gen)
            sc = (torch.rand((rows, cols // 128), device="cuda", generator=gen) * 0.02 + 0.01).float()
            x = torch.randn(cols, device="cuda", generator=gen).to(torch.float16).float()
            nzh, sgh = nz.cpu().numpy().view(np.uint32), sg.cpu().numpy().view(np.uint32)
            sch, xh = sc.cpu().numpy(), x.cpu().numpy()
            t0 = time.perf_counter()
            oracle.gemv_hostloop(nzh, sgh, sch, xh, threads=1)
            st_t += time.perf_counter() - t0
            t0 = time.perf_counter()
            oracle.gemv_hostloop(nzh, sgh, sch, xh, threads=threads)
            mt_t += time.perf_counter() - t0
            st_b += packed_bytes(rows, cols)
            del nz, sg, sc, x
        rows_out.append({"shapes": label, "packed_bytes": int(st_b), "single_thread_ms": round(st_t * 1e3, 2),
                         "single_thread_GBps": round(st_b / st_t / 1e9, 4), f"threads_{threads}_ms": round(mt_t * 1e3, 2),
                         f"threads_{threads}_GBps": round(st_b / mt_t / 1e9, 4)})
        tot["st_bytes"] += st_b
        tot["st_s"] += st_t
        tot["mt_bytes"] += st_b
        tot["mt_s"] += mt_t
    return {
        "value": round(tot["mt_bytes"] / tot["mt_s"] / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": f"one GEMV per matrix shape of configurations 1-3 and of one LLaMA-70B layer ({int(tot['st_bytes'])} packed bytes in all), "
                  f"rows split over {threads} threads: {tot['mt_s']:.2f} s; single thread: {tot['st_s']:.2f} s; "
                  "loop = tests/test_ternary_gemv.cu:40-75 restated in C; the 80-layer 70B figure would be 80 x the layer's time",
        "single_thread_GBps": round(tot["st_bytes"] / tot["st_s"] / 1e9, 4),
        "per_shape_set": rows_out,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # A step is 0.33 ms. The GPU idles at ~100 MHz and takes tens of milliseconds of load to settle at its working
    # clocks, so every timed region is preceded by --settle-ms of the same launches, whatever --warmup says.
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--settle-ms", type=float, default=200.0,
                    help="untimed launches for this long before the warm-up launches of every timed region")
    ap.add_argument("--model", default="llama8b", choices=sorted(SHAPES))
    ap.add_argument("--layers", type=int, default=0, help="0 = the model's own layer count")
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--p-zero", type=float, default=0.42)
    ap.add_argument("--mode", default="plan", choices=["plan", "calls"],
                    help="plan: the whole sweep as one launch; calls: one operator call per matrix")
    ap.add_argument("--matrices", default="", help='per-layer matrix list "ROWSxCOLS,..." instead of the model\'s')
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only-headline", action="store_true", help="skip configs, single_calls and copy_ceiling (profiling runs)")
    ap.add_argument("--configs", default="1,2,3,4,5", help="benchmark configurations to add to `configs`")
    ap.add_argument("--also-batch", default="4,16", help="extra activation-row counts of configuration 3")
    ap.add_argument("--gemm-m", default="16,128,512,2048", help="token counts M of configuration 4")
    ap.add_argument("--gemm-calls", type=int, default=200, help="timed launches per GEMM case")
    ap.add_argument("--gemm-warm", type=int, default=20, help="untimed launches before them (after the settle phase)")
    ap.add_argument("--no-sparsity-sweep", action="store_true", help="configuration 5 at P(0) = 0.42 only (default: also 0.2 and 0.7)")
    ap.add_argument("--no-single-calls", action="store_true")
    ap.add_argument("--seed", type=int, default=20240611)
    args = ap.parse_args()
    for item in filter(None, args.matrices.split(",")):
        r, c = item.lower().split("x")
        CUSTOM.append((int(r), int(c)))
    if args.gpus != 1:
        print("bench.py measures ONE GPU: this build has no multi-GPU path (--gpus must be 1).", file=sys.stderr)
        sys.exit(2)

    import torch
    import ternary_llm_amd as tl
    if not torch.cuda.is_available():
        print("bench.py needs the MI355X (no CPU fallback exists).", file=sys.stderr)
        sys.exit(2)
    tl.lib()
    from oracle import oracle as orc
    if not os.path.exists(orc.LIB):
        orc.build()
    orc.load()
    timer = Timer(torch, args.settle_ms)
    layers = args.layers or SHAPES[args.model][4]
    lo, hi = (0.005, 0.02) if args.model == "llama70b" else (0.01, 0.03)
    problems, meta = build_sweep(torch, args.model, layers, args.batch, args.p_zero, lo, hi, args.seed)
    n_mats = len(layer_matrices(args.model))
    sweep_bytes = sum(packed_bytes(r, c) for (_, _, _, _, _, r, c, _) in problems)
    torch.cuda.synchronize()

    if args.mode == "plan":
        plan = tl.LinearPlan(problems)
        assert plan.weight_bytes == sweep_bytes
        step = plan.launch
        launches_per_step = 1
    else:
        def step():
            for nz, sg, sc, x, y, rows, cols, batch in problems:
                if batch == 1:
                    tl.ternary_gemv(nz, sg, sc, x, y, rows, cols, 128)
                else:
                    tl.ternary_gemm(x, nz, sg, sc, y, batch, rows, cols, 128)
        launches_per_step = len(problems)

    headline = (args.model == "llama8b" and not CUSTOM and args.batch == 1 and args.mode == "plan"
                and layers == SHAPES["llama8b"][4] and args.p_zero == 0.42)
    t0 = time.perf_counter()
    t = timer.run(step, args.steps, args.warmup)
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = t["mean_ms"]
    gbps = sweep_bytes / (ms_per_step * 1e-3) / 1e9
    sample_idx = sorted(set([0, 1, 4, 6, len(problems) - 1, len(problems) // 2]))
    parity = check_sample(orc, problems, [i for i in sample_idx if i < len(problems)])

    out = {
        "metric": "ternary GEMV packed-weight GB/s (% HBM peak) at B=1; GEMM TOPS at M=512",
        "value": round(gbps, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "settle_ms": args.settle_ms, "untimed_launches": t["untimed_launches"],
        "ms_per_step": round(ms_per_step, 5), "ms_per_step_median": round(t["median_ms"], 5), "ms_per_step_min": round(t["min_ms"], 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "dtype_detail": "fp16 activations x 2-bit ternary weights (fp16 group scales), fp32 accumulation, fp16 outputs",
        "data": "synthetic (seeded; P(0)=%.2f, fp16 scales U[%.3f,%.3f], x ~ N(0,1))" % (args.p_zero, lo, hi),
        "config": {
            "workload": f"cfg3: {args.model} {layers}-layer decode projection sweep "
                        f"({len(problems)} ternary GEMVs, {sweep_bytes} packed bytes), batch {args.batch}",
            "mode": args.mode, "launches_per_step": launches_per_step, "group_size": 128,
        },
        "pct_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBS, 2),
        "timing": "HIP events on the launch stream around back-to-back launches; mean over all timed steps, median and min over "
                  f"groups of {t['steps_per_timing_group']} consecutive steps; {t['untimed_launches']} untimed launches first "
                  f"({args.settle_ms:.0f} ms settle + {args.warmup} warm-up)",
        "wall_ms_per_step_with_untimed": round(wall_ms / args.steps, 5),
        "parity_max_rel_sampled": parity,
        "roofline": {
            "bound": "hbm", "achieved": round(gbps, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(gbps / HBM_PEAK_GBS, 4),
            "frac_best_group": round(sweep_bytes / (t["min_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            **(traffic_fields("headline", sweep_bytes) if headline else {"traffic": None}),
            "kernel": plan.kernel if args.mode == "plan" else "per-matrix launches",
            "bytes_per_launch": sweep_bytes // launches_per_step,
        },
    }
    if not args.only_headline:
        want = {int(v) for v in args.configs.split(",") if v.strip()}
        cfgs = []
        cfg_steps = max(50, min(args.steps, 400))
        if 1 in want:
            cfgs += cfg1_rows(torch, tl, orc, timer, args.seed)
        if 2 in want:
            r, _ = plan_rows(torch, tl, orc, timer, "cfg2: llama1b 16-layer sweep (unit-RMS activations)", "llama1b", 16, [1], 0.42, 0.01, 0.03,
                             args.seed + 2, cfg_steps, 20, unit_rms=True)
            cfgs += r
            r, _ = plan_rows(torch, tl, orc, timer, "cfg2: llama1b 16-layer sweep, rotated", "llama1b", 16, [1], 0.42, 0.01, 0.03,
                             args.seed + 2, cfg_steps, 20, copies=3, unit_rms=True)
            cfgs += r
        if 3 in want and headline:
            cfgs.append(hbm_row("cfg3: llama8b 32-layer sweep, batch 1 (the headline value)", t, sweep_bytes, plan.kernel, parity))
            extra = [int(v) for v in args.also_batch.split(",") if v.strip()]
            r, _ = plan_rows(torch, tl, orc, timer, "cfg3: llama8b 32-layer sweep", "llama8b", 32, extra, 0.42, 0.01, 0.03,
                             args.seed, cfg_steps, 20, problems=problems)
            for row, b in zip(r, extra):
                if b in TRAFFIC:
                    row.update(traffic_fields(b, sweep_bytes))
            cfgs += r
            cfgs.append(int8_sweep_row(torch, tl, orc, timer, "cfg3: llama8b 32-layer sweep, batch 1, int8 activations (plan of ternary_gemv_int8)",
                                       problems, cfg_steps, 20))
        if 4 in want:
            gemm_m = [int(v) for v in args.gemm_m.split(",") if v.strip()]
            g = gemm_rows(torch, tl, orc, timer, args.seed, gemm_m, 0.42, args.gemm_calls, args.gemm_warm)
            cfgs += g
            cfgs += ffn_front_rows(torch, tl, timer, args.seed, [m for m in gemm_m if m in (512, 2048)], 0.42, args.gemm_calls, args.gemm_warm)
            cfgs += qkv_prefill_rows(torch, tl, timer, args.seed, [m for m in gemm_m if m in (128, 512, 2048)], 0.42, args.gemm_calls, args.gemm_warm)
            m512 = [c for c in g if c["M"] == 512]
            if m512:
                agg = sum(2.0 * c["M"] * c["N"] * c["K"] for c in m512) / sum(c["us"] for c in m512) / 1e6
                out["gemm_m512"] = {"tflops_both_shapes": round(agg, 1), "frac_mfma_peak": round(agg / MFMA_F16_PEAK_TFLOPS, 4),
                                    "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s (2*M*N*K)",
                                    "per_shape": [{k: c[k] for k in ("N", "K", "us", "tflops", "frac_mfma_peak", "kernel", "dense_fp16_us", "vs_dense_fp16")
                                                   if k in c} for c in m512]}
        if not args.no_single_calls and headline:
            out["single_calls"] = single_call_rows(torch, tl, timer, problems, "llama8b", 32)
        if 5 in want:
            zs = [0.42] + ([] if args.no_sparsity_sweep else [0.2, 0.7])
            for pz in zs:
                r, _ = plan_rows(torch, tl, orc, timer, f"cfg5: llama70b 80-layer sweep resident, P(0)={pz}", "llama70b", 80, [1, 16],
                                 pz, 0.005, 0.02, args.seed + 5, 40, 5)
                cfgs += r
        if 3 in want and headline:
            cfgs += lm_head_rows(torch, tl, orc, timer, args.seed)
            # the headline once more from idle clocks: no settle phase, the driver's own warm-up and step counts
            cold = Timer(torch, 0.0).run(step, 20, 5)
            out["cold_start"] = {"ms_per_step": round(cold["mean_ms"], 5), "GBps": round(sweep_bytes / (cold["mean_ms"] * 1e-3) / 1e9, 1),
                                 "frac_hbm_peak": round(sweep_bytes / (cold["mean_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                 "what": "the headline step with settle_ms 0, warmup 5, steps 20, measured right after host-side work (clocks not settled)"}
        out["configs"] = cfgs
        out["copy_ceiling"] = copy_ceiling(torch, tl, timer)
    if not args.no_cpu_baseline:
        threads = min(os.cpu_count() or 1, 16)
        sets = [("cfg1: 2048x2048", [(2048, 2048)]),
                ("cfg2: one llama1b layer", [(r, c) for _, r, c in layer_matrices("llama1b")] if not CUSTOM else [(2048, 2048)]),
                ("cfg3: one llama8b layer", [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096), (4096, 14336)]),
                ("cfg5: one llama70b layer", [(8192, 8192), (1024, 8192), (1024, 8192), (8192, 8192), (28672, 8192), (28672, 8192), (8192, 28672)])]
        if CUSTOM:
            sets = sets[:1]
        out["cpu_baseline"] = cpu_baseline(orc, torch, sets, threads)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
