#!/usr/bin/env python3
"""Benchmark of the fused 3S attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg3_chunglu_233k]
                    [--no-other-configs] [--no-cpu-baseline]

A step is one launch of the fused SDDMM -> softmax -> SpMM kernel (through the C ABI,
f3s_attention_fwd, heavy-first window order) over the whole synthetic graph, with the CSR,
the TC-block structure and Q/K/V already resident in HBM. Preprocessing is timed separately and
reported in the same JSON line, as are compact results of the other benchmark configurations
(`other_configs`) and a sanity check of the timed output. Prints exactly one JSON line on stdout;
progress goes to stderr.

Figures (all exact functions of the generated graph):
  value              effective TFLOP/s  = 4*d*E / t                    (useful flops over edges)
  roofline.achieved  MFMA TFLOP/s       = 1024*d*nTCB / t_kernel       (flops issued to MFMA)
  padded_tflops      reference's figure = 256*(4d+5)*nTCB / t
                     (scripts/baseline_comp/baseline_comp_kernel_only.py:132-146)
  hbm_min_gbps       compulsory bytes   = 3*N*d*2 + 4*N*d + 96*nTCB + 4*(2*nRW+1), over t
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_MFMA_F16_TFLOPS = 2500.0  # MI355X dense fp16/bf16
PEAK_HBM_GBPS = 8000.0
# what the 256 vector L1s can hand to their CUs: 64 bytes per clock each at the 2.4 GHz peak engine
# clock. Every K/V row of every TC block passes through them, so this bounds the gather whatever
# the caches do (an attention call cannot be faster than B_gather over this).
PEAK_L1_GBPS = 256 * 64 * 2.4


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def host_bits(t):
    """fp16 / bf16 device tensor -> numpy array the oracle takes (float16, or uint16 bits)."""
    t = t.contiguous().cpu()
    if t.dtype == torch.float16:
        return t.numpy()
    return t.view(torch.int16).numpy().view(np.uint16)


def cpu_baseline(rowPtr, colIdx, N, Q, K, V, scale, d, budget_s=12.0):
    """Time the CPU oracle (C + OpenMP restatement of textbook SDDMM/softmax/SpMM over CSR) on a
    bounded sample: equally spaced slices of rows, grown until ~budget_s of CPU work is done.
    Q, K, V: [N, d] of one head."""
    import oracle
    oracle.build()
    rp = rowPtr.cpu().numpy()
    ci = colIdx.cpu().numpy()
    dt = 0 if Q.dtype == torch.float16 else 1
    Qh, Kh, Vh = (host_bits(x) for x in (Q, K, V))
    threads = oracle.num_threads()
    # calibrate on ~N/2048 evenly spaced rows, then size the sample for ~budget_s
    step = max(1, N // 512)
    t0 = time.time()
    oracle.attention_textbook(rp, ci, N, Qh, Kh, Vh, scale, dtype=dt, row_step=step)
    t_cal = time.time() - t0
    t0 = time.time()
    oracle.attention_textbook(rp, ci, N, Qh, Kh, Vh, scale, dtype=dt, rows=(0, 1))
    t_fixed = time.time() - t0  # fp16 -> fp32 conversion of Q/K/V, paid by every call
    per_row = max(1e-9, (t_cal - t_fixed) / (N // step + 1))
    rows_target = int(min(N, max(64, budget_s / per_row)))
    step = max(1, N // rows_target)
    sel = np.arange(0, N, step)
    edges = int((rp[sel + 1] - rp[sel]).sum())
    t0 = time.time()
    oracle.attention_textbook(rp, ci, N, Qh, Kh, Vh, scale, dtype=dt, row_step=step)
    spent = time.time() - t0 - t_fixed
    rows_done = len(sel)
    tflops = 4.0 * d * edges / spent / 1e12 if spent > 0 else 0.0
    return {"value": tflops, "unit": "TFLOP/s (effective, 4*d*E/t)", "cores": threads,
            "kind": "port",
            "sample": "oracle textbook attention (C+OpenMP, fp64 accumulate) on every %d-th row "
                      "(%d rows, %d edges), %.1f s wall" % (step, rows_done, edges, spent)}


def cpu_baseline_torch(rowPtr, colIdx, N, Q, K, V, scale, d, max_edges=4_000_000):
    """The reference's own CPU formulation of the computation, edge-wise SDDMM -> segment softmax
    -> SpMM with plain PyTorch ops (scripts/baseline_comp/baseline_comp_kernel_only.py:667-686
    does it with PyG's softmax / scatter; PyG is not installed here, so index_add_ / index_reduce_
    stand in), fp32 on the host cores, on the first rows of the graph up to max_edges edges."""
    rp = rowPtr.cpu().long()
    rows_n = int(torch.searchsorted(rp, torch.tensor(max_edges)).clamp(min=1, max=N))
    e = int(rp[rows_n])
    if e == 0:
        return None
    col = colIdx[:e].cpu().long()
    row = torch.repeat_interleave(torch.arange(rows_n), rp[1:rows_n + 1] - rp[:rows_n])
    Qf, Kf, Vf = (x.float().cpu() for x in (Q, K, V))
    torch.set_num_threads(os.cpu_count() or 1)

    def run():
        s_e = (Qf[row] * Kf[col]).sum(-1) / scale
        mx = torch.full((rows_n,), float("-inf")).index_reduce_(0, row, s_e, "amax")
        p = torch.exp(s_e - mx[row])
        den = torch.zeros(rows_n).index_add_(0, row, p)
        out = torch.zeros((rows_n, d)).index_add_(0, row, (p / den[row]).unsqueeze(1) * Vf[col])
        return out
    run()
    t0 = time.time()
    run()
    dt = time.time() - t0
    return {"value": 4.0 * d * e / dt / 1e12, "unit": "TFLOP/s (effective, 4*d*E/t)",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": "edge-wise PyTorch CPU ops (gather, index_reduce_, index_add_) on the first "
                      "%d rows (%d edges), %.2f s" % (rows_n, e, dt)}


def bucketed_order(pre, N, buckets):
    """An experimental launch order (results do not depend on the order): windows grouped by the
    column range (one of `buckets` equal parts) that most of their TC blocks start in, heavy
    windows first inside a group. For graphs whose K + V exceed the caches, so that windows that
    run together name neighbouring rows."""
    import torch
    rwo = pre["rowWindowOffset"].long()
    nrw = rwo.numel() - 1
    counts = rwo[1:] - rwo[:-1]
    first_col = pre["sparseAToXidx"].view(-1, 16)[:, 0].long()
    win = torch.repeat_interleave(torch.arange(nrw, device=rwo.device), counts)
    part = torch.clamp(first_col * buckets // max(N, 1), max=buckets - 1)
    hist = torch.bincount(win * buckets + part, minlength=nrw * buckets).view(nrw, buckets)
    bucket = hist.argmax(dim=1)
    key = bucket * (int(counts.max()) + 1) + (int(counts.max()) - counts)
    return torch.argsort(key, stable=True).to(torch.int32)


def recorded_traffic(config, schedule, scale, natural_order):
    """HBM-side bytes per attention call as rocprofv3 counted them in an EARLIER run (FETCH_SIZE
    and WRITE_SIZE, scaled by what the same counters read for a plain copy): counters cannot be
    read from inside this process, so the figure is a record, labelled with the profile summary
    it comes from, and is only given for the workload and schedule it was taken on."""
    path = os.path.join(ROOT, "profiles", "traffic_recorded.json")
    if scale != 1.0 or natural_order or not os.path.exists(path):
        return None
    for rec in json.load(open(path)).get("records", []):
        if rec.get("config") == config and rec.get("schedule") == schedule:
            return rec
    return None


def run_config(name, args, dev, headline):
    """Generate one configuration, preprocess it, time the attention call; returns the result
    dict (the full line for the headline configuration, a compact one otherwise)."""
    from fused3s_amd import capi, synth
    cfg = synth.CONFIGS[name]
    d = cfg["d"]
    heads = cfg["heads"]
    tdtype = torch.float16 if cfg["dtype"] == "fp16" else torch.bfloat16
    scale_graph = args.scale if headline else 1.0

    t0 = time.time()
    rowPtr, colIdx = synth.make_graph(name, seed=0, device=dev, scale=scale_graph)
    torch.cuda.synchronize()
    N = rowPtr.numel() - 1
    E = colIdx.numel()
    deg = (rowPtr[1:] - rowPtr[:-1])
    max_degree = int(deg.max())
    log("graph %s: N=%d E=%d max_degree=%d (%.1f s to generate on the GPU)"
        % (name, N, E, max_degree, time.time() - t0))
    # single head: [N, d] ~ N(0, 1); multi-head: [N, heads, d] ~ N(0, 1/d)
    Q, K, V = synth.features(N, heads * d, seed=0, device=dev, dtype=tdtype,
                             std=1.0 if heads == 1 else d ** -0.5)
    if heads > 1:
        Q, K, V = (x.view(N, heads, d) for x in (Q, K, V))
    scale = float(np.sqrt(d))

    # preprocessing (timed on its own; not part of the step)
    two_phase = bool(getattr(args, "two_phase_preprocess", False))
    capi.preprocess(rowPtr, colIdx, N, two_phase=two_phase)  # warm-up (module load, allocator)
    torch.cuda.synchronize()
    pre_ms = []
    for _ in range(7):
        t0 = time.time()
        pre = capi.preprocess(rowPtr, colIdx, N, two_phase=two_phase)
        torch.cuda.synchronize()
        pre_ms.append((time.time() - t0) * 1e3)
    pre_ms = float(np.median(pre_ms))
    nTCB = pre["blockCount"]
    nRW = (N + 15) // 16
    cnt = (pre["rowWindowOffset"][1:] - pre["rowWindowOffset"][:-1])
    # scan bound of the preprocessing: CSR read once, ids + bitmaps written once
    pre_bytes = 4.0 * E + 4.0 * (N + 1) + 96.0 * nTCB
    pre_hbm_frac = pre_bytes / (pre_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS
    log("preprocess: nTCB=%d nRW=%d max TCB/window=%d mean=%.1f  %.2f ms (%.2f G edges/s, %.1f%% "
        "of the HBM scan bound)" % (nTCB, nRW, int(cnt.max()), float(cnt.float().mean()), pre_ms,
                                    E / pre_ms / 1e6, 100 * pre_hbm_frac))

    if headline and args.preprocess_only:
        return {"metric": "preprocess_ms", "value": pre_ms, "unit": "ms", "n_gpus": 1,
                "higher_is_better": False, "data": "synthetic",
                "config": {"workload": "%s: N=%d E=%d, CSR -> TC blocks" % (name, N, E),
                           "nTCB": nTCB, "nRW": nRW},
                "preprocess_gedges_per_s": E / pre_ms / 1e6, "preprocess_hbm_frac": pre_hbm_frac}
    if os.path.basename(capi.LIB_PATH).startswith("libf3s_amd_pre_"):
        raise SystemExit("bench.py: %s is a preprocessing probe whose block arrays are incomplete; "
                         "it may only be timed with --preprocess-only" % capi.LIB_PATH)

    if headline and args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)  # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    natural = headline and args.natural_order
    order = None if natural else pre["sortedRowWindows"]
    if headline and args.column_buckets > 0:
        order = bucketed_order(pre, N, args.column_buckets)
    out = torch.empty((N, heads * d), dtype=torch.float32, device=dev)
    # scratch of the column-sliced schedule, which the library picks for graphs with long windows
    workspace = capi.attention_workspace(N, d, dev, nTCB=nTCB, dtype=tdtype,
                                         heads=0 if heads == 1 else heads)
    if workspace is not None:
        # the schedule's index depends on the structure only: built once, like the structure
        capi.attention_prepare(pre["rowWindowOffset"], pre["sparseAToXidx"], N, d,
                               workspace, heads=0 if heads == 1 else heads)
    schedule = "column-sliced" if workspace is not None else "window"
    log("attention schedule: %s" % ("column-sliced (%.0f MB workspace)" % (workspace.numel() / 1e6)
                                    if workspace is not None else "workgroup per window"))

    layout = getattr(args, "kv_layout", "") if headline else ""
    if heads == 1 and layout:
        # experiment: K and V rows placed differently in memory, through the multi-head entry
        # with one head (which takes any row pitch); the values are the same
        def placed(t, pitch_bytes, offset_bytes=0, store=None):
            pe, oe = pitch_bytes // t.element_size(), offset_bytes // t.element_size()
            if store is None:
                store = torch.zeros((N, pe), dtype=t.dtype, device=dev)
            store[:, oe:oe + d] = t
            return store[:, oe:oe + d].unflatten(1, (1, d)), store
        row = d * Q.element_size()
        if layout == "interleaved":  # one array of 2-row records: K in the first half, V behind it
            pitch = 2 * row
            Kh, kv = placed(K, pitch)
            Vh, _ = placed(V, pitch, row, kv)
        elif layout.startswith("odd"):  # rows at pitch P, each one row beyond the pitch boundary
            pitch = int(layout[3:])
            Kh, _ = placed(K, pitch, row)
            Vh, _ = placed(V, pitch, row)
        else:  # "pitch<bytes>"
            pitch = int(layout[5:])
            Kh, _ = placed(K, pitch)
            Vh, _ = placed(V, pitch)
        Qh, _ = placed(Q, pitch)  # the entry takes one pitch for Q, K and V
        workspace = capi.attention_workspace(N, d, dev, nTCB=nTCB, dtype=tdtype, heads=1)
        if workspace is not None:
            capi.attention_prepare(pre["rowWindowOffset"], pre["sparseAToXidx"], N, d, workspace,
                                   heads=1)
        log("K / V layout: %s (multi-head entry, one head)" % layout)

        def step(v=V, o=out):
            vh = Vh if v is V else placed(v, pitch)[0]
            capi.attention_heads(pre["rowWindowOffset"], order, pre["sparseAToXidx"],
                                 pre["tcbBitMap"], N, Qh, Kh, vh, scale, True, out=o,
                                 workspace=workspace, prepared=workspace is not None)
    elif heads == 1:
        def step(v=V, o=out):
            capi.attention(pre["rowWindowOffset"], order, pre["sparseAToXidx"], pre["tcbBitMap"],
                           N, Q, K, v, scale, True, out=o, workspace=workspace,
                           prepared=workspace is not None)
    else:
        def step(v=V, o=out):
            capi.attention_heads(pre["rowWindowOffset"], order, pre["sparseAToXidx"],
                                 pre["tcbBitMap"], N, Q, K, v, scale, True, out=o,
                                 workspace=workspace, prepared=workspace is not None)

    steps, warmup = (args.steps, args.warmup) if headline else (10, 3)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    events = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    events[0].record()
    for i in range(steps):
        step()
        events[i + 1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kern_ms = np.array([events[i].elapsed_time(events[i + 1]) for i in range(steps)])
    ms_per_step = wall * 1e3 / steps
    t_avg = float(kern_ms.mean()) * 1e-3
    t_med = float(np.median(kern_ms)) * 1e-3

    # sanity of what was timed: finite output, and softmax weights that sum to one (with V = 1
    # every row that has an edge must come out as 1, every other row as 0)
    finite = bool(torch.isfinite(out).all())
    ones = torch.ones_like(V)
    o1 = torch.empty_like(out)
    step(ones, o1)
    torch.cuda.synchronize()
    has = (deg > 0).unsqueeze(1).to(o1.dtype)
    rowsum_err = float((o1 - has).abs().max())
    del ones, o1
    sanity = {"finite": finite, "rowsum_max_err": rowsum_err, "ok": finite and rowsum_err < 2e-3}

    D = heads * d  # all per-node byte and flop counts scale with the concatenated width
    f_eff = 4.0 * D * E
    f_mfma = 1024.0 * D * nTCB
    f_pad = 256.0 * (4 * d + 5) * nTCB * heads
    b_min = 3.0 * N * D * 2 + 4.0 * N * D + 96.0 * nTCB + 4.0 * (2 * nRW + 1)
    b_gather = N * D * 2.0 + nTCB * (2 * 16 * D * 2.0 + 96.0 * heads) + 4.0 * N * D
    achieved = f_mfma / t_avg / 1e12

    # the bound that binds on paper: t_roof = max(F_mfma / P_mfma, B_min / BW_hbm)
    if f_mfma / (PEAK_MFMA_F16_TFLOPS * 1e12) >= b_min / (PEAK_HBM_GBPS * 1e9):
        roofline = {"bound": "mfma", "achieved": achieved, "peak": PEAK_MFMA_F16_TFLOPS,
                    "unit": "TFLOP/s", "frac": achieved / PEAK_MFMA_F16_TFLOPS, "traffic": None}
    else:
        gbps = b_min / t_avg / 1e9
        roofline = {"bound": "hbm", "achieved": gbps, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                    "frac": gbps / PEAK_HBM_GBPS, "traffic": None}
    log("%s kernel: median %.3f ms  mean %.3f ms  effective %.1f TFLOP/s  MFMA %.1f TFLOP/s "
        "(%.1f%%)  gather %.0f GB/s  sanity %s"
        % (name, t_med * 1e3, t_avg * 1e3, f_eff / t_med / 1e12, achieved,
           100 * achieved / PEAK_MFMA_F16_TFLOPS, b_gather / t_med / 1e9, sanity))
    if not headline:
        return {"config": name, "N": N, "E": E, "nTCB": nTCB, "d": d, "heads": heads,
                "dtype": "f16" if cfg["dtype"] == "fp16" else "bf16", "schedule": schedule,
                "kernel_ms_median": t_med * 1e3, "effective_tflops": f_eff / t_med / 1e12,
                "bound": roofline["bound"], "achieved": roofline["achieved"],
                "frac": roofline["frac"], "gather_gbps": b_gather / t_med / 1e9,
                "preprocess_ms": pre_ms, "preprocess_hbm_frac": pre_hbm_frac,
                "sanity_ok": sanity["ok"]}

    result = {
        "metric": "fused_3s_attention_effective_tflops_d%d_%s%s"
                  % (d, cfg["dtype"], "" if heads == 1 else "_%dheads" % heads),
        "value": f_eff / (wall / steps) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if cfg["dtype"] == "fp16" else "bf16", "data": "synthetic",
        "config": {"workload": "%s: N=%d E=%d d=%d %s %s, scalingFactor=sqrt(d), %s window order"
                               % (name, N, E, d, cfg["dtype"],
                                  "single head" if heads == 1 else
                                  "%d heads in one launch, output [N, %d]" % (heads, D),
                                  "natural" if natural else
                                  "%d column groups, heavy-first inside" % args.column_buckets
                                  if headline and args.column_buckets > 0 else "heavy-first"),
                   "nTCB": nTCB, "nRW": nRW, "max_tcb_per_window": int(cnt.max()),
                   "max_degree": max_degree, "scale": scale_graph},
        "kernel_ms_median": t_med * 1e3, "kernel_ms_mean": t_avg * 1e3,
        "padded_tflops": f_pad / t_med / 1e12,
        "hbm_min_gbps": b_min / t_med / 1e9, "hbm_min_frac": b_min / t_med / 1e9 / PEAK_HBM_GBPS,
        "gather_gbps": b_gather / t_med / 1e9,
        "gather_l1_frac": b_gather / t_med / 1e9 / PEAK_L1_GBPS,
        "preprocess_ms": pre_ms, "preprocess_gedges_per_s": E / pre_ms / 1e6,
        "preprocess_hbm_frac": pre_hbm_frac,
        "schedule": schedule,
        "sanity": sanity,
        "roofline": roofline,
        "traffic_recorded": recorded_traffic(name, schedule, scale_graph, natural),
    }
    if result["traffic_recorded"] is not None:
        # HBM-side bytes per call of the same kernels on the same workload, from the record
        roofline["traffic"] = result["traffic_recorded"].get("bytes")
    if heads > 1:
        # the reference's way: one launch per head on contiguous per-head copies
        per_head = [tuple(x[:, h].contiguous() for x in (Q, K, V)) for h in range(heads)]
        outs = [torch.empty((N, d), dtype=torch.float32, device=dev) for _ in range(heads)]

        def loop():
            for h in range(heads):
                capi.attention(pre["rowWindowOffset"], order, pre["sparseAToXidx"],
                               pre["tcbBitMap"], N, *per_head[h], scale, True, out=outs[h])
        loop()
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        ev[0].record()
        for i in range(steps):
            loop()
            ev[i + 1].record()
        torch.cuda.synchronize()
        result["per_head_loop_ms_median"] = float(np.median(
            [ev[i].elapsed_time(ev[i + 1]) for i in range(steps)]))
        log("per-head loop of %d single-head launches: median %.3f ms"
            % (heads, result["per_head_loop_ms_median"]))
    if not args.no_cpu_baseline:
        # one head on the CPU; its rate in effective flops is the per-head rate of the whole job
        q1, k1, v1 = (Q, K, V) if heads == 1 else (x[:, 0] for x in (Q, K, V))
        result["cpu_baseline"] = cpu_baseline(rowPtr, colIdx, N, q1, k1, v1, scale, d,
                                              args.cpu_budget)
        log("cpu baseline:", result["cpu_baseline"])
        result["cpu_baseline_torch"] = cpu_baseline_torch(rowPtr, colIdx, N, q1, k1, v1, scale, d)
        log("cpu baseline (PyTorch ops):", result["cpu_baseline_torch"])
    else:
        result["cpu_baseline"] = None
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="cfg3_chunglu_233k")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink the graph (debugging)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the compact lines of the other benchmark configurations")
    ap.add_argument("--natural-order", action="store_true", help="launch windows in natural order")
    ap.add_argument("--column-buckets", type=int, default=0,
                    help="experiment: launch windows grouped by the column range most of their "
                         "blocks start in (this many ranges), heavy-first inside a group")
    ap.add_argument("--two-phase-preprocess", action="store_true",
                    help="preprocess with f3s_preprocess_count + f3s_preprocess_fill instead of "
                         "the one call f3s_preprocess")
    ap.add_argument("--kv-layout", default="",
                    help="experiment on a single-head configuration: K / V rows at pitch<bytes>, "
                         "odd<bytes> (one row beyond every pitch boundary) or interleaved, through "
                         "the multi-head entry with one head")
    ap.add_argument("--preprocess-only", action="store_true",
                    help="time the preprocessing of --config and stop (no attention call)")
    ap.add_argument("--cpu-budget", type=float, default=12.0)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (known bytes, for scaling rocprof's "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on ONE GPU (row windows would shard across GPUs with K/V "
            "replicated, but no multi-GPU path is part of it); run with --gpus 1")
        sys.exit(2)
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible; the HIP path has no CPU fallback")
        sys.exit(3)

    from fused3s_amd import synth
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    result = run_config(args.config, args, dev, headline=True)
    if not args.no_other_configs and not args.preprocess_only:
        # the other benchmark configurations, one compact entry each (kernel time, the bound that
        # binds on paper and the fraction reached, preprocessing time)
        others = []
        for name in synth.CONFIGS:
            if name == args.config:
                continue
            torch.cuda.empty_cache()
            others.append(run_config(name, args, dev, headline=False))
        result["other_configs"] = others
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
