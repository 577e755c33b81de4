"""Per-CU active time of the fused kernel, natural against heavy-first window order.

The timed launches of the F3S module (checkSMActiveTime=True) write one "begin_ms end_ms" line
per compute unit, as the reference's printSMTime does per SM (src/F3S_kernel.cu:43-75). This
module reads those files the way the reference's plotting script does
(scripts/baseline_comp/sm_activity_analysis.py:21-46: active time = end - begin per line) and
prints the spread as text instead of a bar chart.

    python -m fused3s_amd.cu_activity [--config cfg3_chunglu_233k] [--out summary.md]
"""
import argparse
import os
import sys

import numpy as np


def read_spans(filename):
    """[[begin_ms, end_ms], ...], one row per CU that ran a workgroup."""
    rows = []
    with open(filename) as f:
        for line in f:
            parts = line.split()
            if len(parts) == 2:
                rows.append((float(parts[0]), float(parts[1])))
    return np.asarray(rows, dtype=np.float64).reshape(-1, 2)


def summarize(spans):
    """Spread of the per-CU active time (ms). `tail_idle` is the share of CU-time between a CU's
    last workgroup and the end of the launch: what a better schedule could still recover."""
    active = spans[:, 1] - spans[:, 0]
    t0, t1 = spans[:, 0].min(), spans[:, 1].max()
    return {
        "cus": int(len(active)),
        "launch_ms": float(t1 - t0),
        "active_max_ms": float(active.max()),
        "active_mean_ms": float(active.mean()),
        "active_min_ms": float(active.min()),
        "active_std_ms": float(active.std()),
        "mean_over_max": float(active.mean() / active.max()),
        "tail_idle": float(((t1 - spans[:, 1]).sum()) / (len(active) * (t1 - t0))),
    }


def measure(config="cfg3_chunglu_233k", workdir=".", reps=5):
    """Runs both orders `reps` times (the last run's files are kept) and returns
    {"natural": summary, "heavy_first": summary, "graph": {...}}."""
    import torch
    from fused3s_amd import F3S, synth
    dev = torch.device("cuda:0")
    cfg = synth.CONFIGS[config]
    d = cfg["d"]
    rowPtr, colIdx = synth.make_graph(config, seed=0, device=dev)
    N = rowPtr.numel() - 1
    E = colIdx.numel()
    Q, K, V = synth.features(N, d, seed=0, device=dev)
    nRW = (N + 15) // 16
    z = lambda n: torch.zeros(n, dtype=torch.int32, device=dev)
    rwo, order, _, _, _, atox, bitmap, nTcb = F3S.preprocess_gpu(colIdx, rowPtr, N, 16, 16,
                                                                  z(nRW), z(E), z(E))
    cwd = os.getcwd()
    os.chdir(workdir)
    try:
        t_nat, t_sch = [], []
        for _ in range(reps):
            t_nat.append(float(F3S.f3s_1tb1rw(rwo, atox, bitmap, N, Q, K, V, 8, True, True)[0]))
            t_sch.append(float(F3S.f3s_1tb1rw_scheduled(rwo, order, atox, bitmap, N, Q, K, V, 8,
                                                        True)[0]))
        res = {
            "graph": {"config": config, "N": N, "E": E, "nTCB": int(nTcb), "nRW": nRW, "d": d},
            "natural": summarize(read_spans("SM_time_f3s1tb1rw.csv")),
            "heavy_first": summarize(read_spans("SM_time_f3s1tb1rw_scheduled.csv")),
        }
        res["natural"]["kernel_ms_median"] = float(np.median(t_nat))
        res["heavy_first"]["kernel_ms_median"] = float(np.median(t_sch))
    finally:
        os.chdir(cwd)
    return res


def to_markdown(res):
    g = res["graph"]
    keys = ["kernel_ms_median", "launch_ms", "cus", "active_max_ms", "active_mean_ms",
            "active_min_ms", "active_std_ms", "mean_over_max", "tail_idle"]
    lines = ["graph %(config)s: N=%(N)d E=%(E)d nTCB=%(nTCB)d nRW=%(nRW)d d=%(d)d" % g, "",
             "| figure | natural order | heavy-first order |", "|---|---|---|"]
    for k in keys:
        a, b = res["natural"][k], res["heavy_first"][k]
        fmt = "%d" if k == "cus" else "%.4f"
        lines.append("| %s | %s | %s |" % (k, fmt % a, fmt % b))
    return "\n".join(lines) + "\n"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", default="cfg3_chunglu_233k")
    ap.add_argument("--workdir", default=".")
    ap.add_argument("--out", default=None)
    args = ap.parse_args()
    text = to_markdown(measure(args.config, args.workdir))
    sys.stdout.write(text)
    if args.out:
        with open(args.out, "w") as f:
            f.write(text)


if __name__ == "__main__":
    main()
