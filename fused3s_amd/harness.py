"""Benchmark harness with the reference's dataset format, timing protocol and CSV schema.

What it mirrors of scripts/baseline_comp/baseline_comp_kernel_only.py:
  * datasets are `.npz` files {src_li, dst_li, num_nodes}, possibly with duplicate edges, turned
    into CSR through a scipy COO matrix (:730-742; written by scripts/downloadDataset.py:5-11);
  * Q, K, V are uniform [0, 1) fp16 (:165-168 of the GraphInfo class), d = --embedding_dim;
  * every kernel is run 3 times untimed, then `niter` times; the kernel's own event time
    (`output[0]`, ms) is collected, throughput = flop * 1000 / ms with the padded flop count
    nTCB*16*BLK_W*(4d + 5) (:132-146, 225-245);
  * results go to two tables indexed by "dataset" with one column per kernel, written as
    baseline_comp_kernel_only_{runtime,throughput}_<method>_<alg>_<dataset>_<gpu>.csv (:68-74,
    816-817).
And of scripts/graph_stat/paper_graph_stat.py:63-110: the TC-block statistics (blocks per row
window, non-zeros per block) with its consistency check.

    python -m fused3s_amd.harness --dataset path/to/graph.npz [--alg all] [-emb 64]
    python -m fused3s_amd.harness --synthetic cfg2_rmat_169k --stats
"""
import argparse
import os

import numpy as np

ALGS = ["f3s_1tb1tcb", "f3s_1tb1rw", "f3s_1tb1rw_scheduled", "f3s_1tb1rw_scheduled_permuteV"]


def save_npz(path, src_li, dst_li, num_nodes):
    """The reference's dataset file (scripts/downloadDataset.py:5-11)."""
    np.savez(path, src_li=np.asarray(src_li), dst_li=np.asarray(dst_li), num_nodes=num_nodes)


def load_npz(path):
    """-> (rowPtr int32[N+1], colIdx int32[E], N). Duplicate edges collapse, columns come out
    sorted inside a row (COO -> CSR as in baseline_comp_kernel_only.py:730-742)."""
    from scipy.sparse import coo_matrix
    data = np.load(path)  # plain arrays only: allow_pickle stays False
    src, dst = np.asarray(data["src_li"]), np.asarray(data["dst_li"])
    n = int(data["num_nodes"])
    if len(src) != len(dst):
        raise ValueError("%s: src_li and dst_li differ in length" % path)
    if len(src) and (src.min() < 0 or dst.min() < 0 or src.max() >= n or dst.max() >= n):
        raise ValueError("%s: node id outside [0, num_nodes)" % path)
    adj = coo_matrix((np.ones(len(src), np.int8), (src, dst)), shape=(n, n)).tocsr()
    adj.sum_duplicates()
    adj.sort_indices()
    return adj.indptr.astype(np.int32), adj.indices.astype(np.int32), n


def f3s_flop(n_tcb, embedding_dim, blk_w):
    """Padded flop count of the reference's throughput figure (GraphInfo.f3s_flop, :132-146)."""
    nnz = n_tcb * 16 * blk_w
    return nnz * embedding_dim * 2 * 2 + nnz * 5


def tcb_stats(rowPtr, rowWindowOffset, tcblockOffset):
    """Statistics of scripts/graph_stat/paper_graph_stat.py:63-110 from preprocessing outputs
    (host arrays). Raises if the per-block non-zero counts do not add up to the CSR's."""
    rwo = np.asarray(rowWindowOffset, np.int64)
    toff = np.asarray(tcblockOffset, np.int64)
    rp = np.asarray(rowPtr, np.int64)
    blocks = np.diff(rwo)
    nnz = np.diff(toff)
    n = len(rp) - 1
    # the reference checks the first 50 windows; every window is checked here
    per_window = np.add.reduceat(nnz, rwo[:-1][blocks > 0]) if len(nnz) else np.zeros(0, np.int64)
    true = np.array([rp[min(16 * (w + 1), n)] - rp[16 * w] for w in range(len(blocks))], np.int64)
    if not np.array_equal(per_window, true[blocks > 0]) or true[blocks == 0].any():
        raise RuntimeError("non-zeros per TC block do not add up to the CSR row lengths")

    def spread(x, prefix):
        if len(x) == 0:
            return {prefix + k: 0.0 for k in ("avg", "variance", "median", "rsd", "q1", "q3")}
        avg = float(x.mean())
        return {prefix + "avg": avg, prefix + "variance": float(x.var()),
                prefix + "median": float(np.median(x)),
                prefix + "rsd": float(x.std() / avg) if avg else 0.0,
                prefix + "q1": float(np.percentile(x, 25)),
                prefix + "q3": float(np.percentile(x, 75))}
    out = {"num_rows": n, "num_nnz": int(rp[-1]), "density": float(rp[-1]) / max(1, n * n),
           "block_count": int(rwo[-1])}
    out.update(spread(nnz, "nnz_per_block_"))
    out.update(spread(blocks, "block_per_row_window_"))
    return out


def column_sharing(rowWindowOffset, sparseAToXidx, order, groups=(2, 4, 8), hubs=(2048, 8192)):
    """How many K / V rows windows that run next to each other have in common, from preprocessing
    outputs (torch tensors on any device, 16-column blocks). Decides whether gathering a row once
    for several windows could pay.

    Returns {"pairs": distinct (window, column) pairs,
             "union_over_sum_<g>": for groups of g windows adjacent in `order` (sortedRowWindows,
                 or None for natural order): distinct (group, column) pairs / pairs, i.e. the
                 share of gathered rows that would remain if a group fetched each of its columns
                 once,
             "hub_coverage_<h>": share of the pairs that name one of the h most popular columns}.
    A window's columns are its ascending compacted ids; the slots its last block leaves unused
    hold 0 and are told apart from column 0 by not ascending."""
    import torch
    rwo = rowWindowOffset.to(torch.int64)
    a = sparseAToXidx.to(torch.int64)
    nrw = rwo.numel() - 1
    slots = a.numel()
    if slots == 0:
        return {"pairs": 0}
    win = torch.repeat_interleave(torch.arange(nrw, device=a.device), (rwo[1:] - rwo[:-1]) * 16)
    first = torch.ones(slots, dtype=torch.bool, device=a.device)
    first[1:] = win[1:] != win[:-1]
    valid = first.clone()
    valid[1:] |= a[1:] > a[:-1]
    cols, win = a[valid], win[valid]
    ncol = int(cols.max()) + 1
    pairs = int(cols.numel())
    out = {"pairs": pairs}
    pos = torch.empty(nrw, dtype=torch.int64, device=a.device)
    if order is None:
        pos = torch.arange(nrw, device=a.device)
    else:
        pos[order.to(torch.int64)] = torch.arange(nrw, device=a.device)
    for g in groups:
        grp = torch.div(pos[win], g, rounding_mode="floor")
        out["union_over_sum_%d" % g] = float(torch.unique(grp * ncol + cols).numel()) / pairs
    popularity = torch.bincount(cols, minlength=ncol)
    ranked = torch.sort(popularity, descending=True).values
    for h in hubs:
        out["hub_coverage_%d" % h] = float(ranked[:h].sum()) / pairs
    return out


def gpu_model():
    import torch
    if torch.cuda.is_available():
        return torch.cuda.get_device_name(0).replace(" ", "_")
    return "unknown"


def _preprocess(F3S, rowPtr_d, colIdx_d, n, blk_w):
    import torch
    nrw = (n + 15) // 16
    e = colIdx_d.numel()
    z = lambda k: torch.zeros(k, dtype=torch.int32, device=rowPtr_d.device)
    return F3S.preprocess_gpu(colIdx_d, rowPtr_d, n, 16, blk_w, z(nrw), z(e), z(e))


def time_kernel(kernel, flop, niter=10, warmup=3):
    """median ms and median flop/s of `kernel()` by its own reported time (output[0])."""
    for _ in range(warmup):
        kernel()
    times = [float(kernel()[0]) for _ in range(niter)]
    return float(np.median(times)), float(np.median([flop * 1000.0 / t for t in times]))


def run_dataset(name, rowPtr, colIdx, n, algs, embedding_dim=64, n_warp_per_block=8, niter=10,
                seed=0, stats=False):
    """Runs the chosen kernels on one graph. Returns ({alg: ms}, {alg: flop/s}, stats or None)."""
    import torch
    from fused3s_amd import F3S
    dev = torch.device("cuda:0")
    rp = torch.as_tensor(rowPtr).to(dev)
    ci = torch.as_tensor(colIdx).to(dev)
    g = torch.Generator().manual_seed(seed)
    Q, K, V = [torch.rand((n, embedding_dim), generator=g).half().to(dev) for _ in range(3)]
    runtime, throughput, st = {}, {}, None
    if "f3s_1tb1tcb" in algs:
        rwo, _, _, _, _, atox, bm, ntcb = _preprocess(F3S, rp, ci, n, 8)
        runtime["f3s_1tb1tcb"], throughput["f3s_1tb1tcb"] = time_kernel(
            lambda: F3S.f3s_1tb1tcb(rwo, atox, bm, n, Q, K, V, True, False),
            f3s_flop(ntcb, embedding_dim, 8), niter)
    rw_algs = [a for a in algs if a != "f3s_1tb1tcb"]
    if rw_algs or stats:
        rwo, order, _, _, toff, atox, bm, ntcb = _preprocess(F3S, rp, ci, n, 16)
        flop = f3s_flop(ntcb, embedding_dim, 16)
        calls = {
            "f3s_1tb1rw": lambda: F3S.f3s_1tb1rw(rwo, atox, bm, n, Q, K, V, n_warp_per_block,
                                                 True, False),
            "f3s_1tb1rw_scheduled": lambda: F3S.f3s_1tb1rw_scheduled(
                rwo, order, atox, bm, n, Q, K, V, n_warp_per_block, False),
            "f3s_1tb1rw_scheduled_permuteV": lambda: F3S.f3s_1tb1rw_scheduled_permuteV(
                rwo, order, atox, bm, n, Q, K, V, n_warp_per_block),
        }
        for a in rw_algs:
            runtime[a], throughput[a] = time_kernel(calls[a], flop, niter)
        if stats:
            st = tcb_stats(rowPtr, rwo.cpu().numpy(), toff.cpu().numpy())
            for tag, od in (("heavy_first_", order), ("natural_", None)):
                for k, v in column_sharing(rwo, atox, od).items():
                    st[("" if k == "pairs" else tag) + k] = v
    return runtime, throughput, st


def write_tables(results, algs, method, alg, dataset, outdir="."):
    """results: {dataset: (runtime dict, throughput dict)} -> the two CSV files; returns paths."""
    import pandas as pd
    names = list(results)
    rt = pd.DataFrame(index=names, columns=algs)
    tp = pd.DataFrame(index=names, columns=algs)
    rt.index.name = tp.index.name = "dataset"
    for ds, (r, t) in results.items():
        for a in algs:
            if a in r:
                rt.loc[ds, a] = r[a]
                tp.loc[ds, a] = t[a]
    tag = "%s_%s_%s_%s" % (method, alg, dataset, gpu_model())
    paths = (os.path.join(outdir, "baseline_comp_kernel_only_runtime_%s.csv" % tag),
             os.path.join(outdir, "baseline_comp_kernel_only_throughput_%s.csv" % tag))
    rt.to_csv(paths[0])
    tp.to_csv(paths[1])
    return paths


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--dataset", action="append", default=[], help=".npz file (repeatable)")
    ap.add_argument("--synthetic", action="append", default=[],
                    help="name of a built-in synthetic configuration (repeatable)")
    ap.add_argument("--alg", default="all", choices=["all"] + ALGS)
    ap.add_argument("--embedding_dim", "-emb", type=int, default=64)
    ap.add_argument("--n_warp_per_block", "-nw", type=int, default=8)
    ap.add_argument("--niter", type=int, default=10)
    ap.add_argument("--stats", action="store_true", help="print TC-block statistics")
    ap.add_argument("--outdir", default=".")
    args = ap.parse_args()
    algs = ALGS if args.alg == "all" else [args.alg]
    graphs = []
    for path in args.dataset:
        graphs.append((os.path.splitext(os.path.basename(path))[0],) + load_npz(path))
    for name in args.synthetic:
        from fused3s_amd import synth
        rp, ci = synth.make_graph(name, seed=0, device="cuda:0")
        graphs.append((name, rp.cpu().numpy(), ci.cpu().numpy(), rp.numel() - 1))
    if not graphs:
        ap.error("give --dataset FILE.npz or --synthetic NAME")
    results = {}
    for name, rp, ci, n in graphs:
        print("=========== dataset: %s, num_nodes: %d, num_edges: %d ===========" %
              (name, n, len(ci)), flush=True)
        rt, tp, st = run_dataset(name, rp, ci, n, algs, args.embedding_dim,
                                 args.n_warp_per_block, args.niter, stats=args.stats)
        for a in rt:
            print("%s median execution time: %.4f ms, median throughput (FLOPS): %.4g"
                  % (a, rt[a], tp[a]))
        if st:
            for k, v in st.items():
                print("%s: %s" % (k, v))
        results[name] = (rt, tp)
    label = graphs[0][0] if len(graphs) == 1 else "all"
    for p in write_tables(results, algs, "f3s", args.alg, label, args.outdir):
        print("wrote", p)


if __name__ == "__main__":
    main()
