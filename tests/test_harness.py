"""The benchmark harness: dataset format, TC-block statistics, CSV tables."""
import numpy as np
import pytest

from conftest import random_csr


def test_npz_round_trip_collapses_duplicates(tmp_path):
    from fused3s_amd import harness
    src = np.array([3, 0, 0, 2, 0, 3, 3], np.int64)
    dst = np.array([1, 2, 2, 0, 1, 3, 1], np.int64)  # (0,2) and (3,1) twice
    path = tmp_path / "toy.npz"
    harness.save_npz(path, src, dst, 5)
    rowPtr, colIdx, n = harness.load_npz(path)
    assert n == 5 and rowPtr.dtype == np.int32 and colIdx.dtype == np.int32
    assert rowPtr.tolist() == [0, 2, 2, 3, 5, 5]
    assert colIdx.tolist() == [1, 2, 0, 1, 3]
    harness.save_npz(tmp_path / "bad.npz", [0, 7], [1, 1], 5)
    with pytest.raises(ValueError, match="outside"):
        harness.load_npz(tmp_path / "bad.npz")


def test_flop_count_is_the_reference_formula():
    from fused3s_amd import harness
    # nnz = nTCB*16*W; sddmm 2*d*nnz + spmm 2*d*nnz + softmax 5*nnz
    assert harness.f3s_flop(10, 64, 16) == 10 * 256 * (4 * 64 + 5)
    assert harness.f3s_flop(10, 128, 8) == 10 * 128 * (4 * 128 + 5)


def test_tcb_stats_against_direct_counts(oracle_mod):
    from fused3s_amd import harness
    rng = np.random.default_rng(3)
    N = 500
    rowPtr, colIdx = random_csr(rng, N, 9, hub=11, empty_frac=0.2)
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    st = harness.tcb_stats(rowPtr, pre["rowWindowOffset"], pre["tcblockOffset"])
    blocks = np.diff(pre["rowWindowOffset"])
    nnz = np.diff(pre["tcblockOffset"])
    assert st["num_rows"] == N and st["num_nnz"] == len(colIdx)
    assert st["block_count"] == pre["blockCount"]
    assert st["nnz_per_block_avg"] == pytest.approx(len(colIdx) / pre["blockCount"])
    assert st["block_per_row_window_median"] == float(np.median(blocks))
    assert st["nnz_per_block_q3"] == float(np.percentile(nnz, 75))
    broken = pre["tcblockOffset"].copy()
    broken[1:-1] += 1
    with pytest.raises(RuntimeError, match="do not add up"):
        harness.tcb_stats(rowPtr, pre["rowWindowOffset"], broken)


def test_column_sharing_against_python_sets(oracle_mod):
    """harness.column_sharing against sets built row by row from the CSR (column 0 present and
    absent, windows without edges, a last group that is not full)."""
    import torch
    from fused3s_amd import harness
    rng = np.random.default_rng(8)
    N = 330
    rowPtr, colIdx = random_csr(rng, N, 12, hub=7, empty_frac=0.25)
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    nrw = (N + 15) // 16
    sets = [set(colIdx[rowPtr[16 * w]:rowPtr[min(16 * w + 16, N)]].tolist()) for w in range(nrw)]
    assert any(0 in s for s in sets) and any(0 not in s and s for s in sets)
    pairs = sum(len(s) for s in sets)
    counts = {}
    for s in sets:
        for c in s:
            counts[c] = counts.get(c, 0) + 1
    ranked = sorted(counts.values(), reverse=True)
    for order in (pre["sortedRowWindows"], None):
        od = None if order is None else torch.as_tensor(order.astype(np.int32))
        got = harness.column_sharing(torch.as_tensor(pre["rowWindowOffset"].astype(np.int32)),
                                     torch.as_tensor(pre["sparseAToXidx"].astype(np.int32)), od,
                                     groups=(2, 4, 8), hubs=(3, 50))
        assert got["pairs"] == pairs
        seq = list(range(nrw)) if order is None else [int(w) for w in order]
        for g in (2, 4, 8):
            union = sum(len(set().union(*[sets[w] for w in seq[i:i + g]]))
                        for i in range(0, nrw, g))
            assert got["union_over_sum_%d" % g] == pytest.approx(union / pairs)
        assert got["hub_coverage_3"] == pytest.approx(sum(ranked[:3]) / pairs)
        assert got["hub_coverage_50"] == pytest.approx(sum(ranked[:50]) / pairs)


@pytest.mark.gpu
def test_run_and_tables(tmp_path):
    import pandas as pd
    from fused3s_amd import harness
    print("case harness_run", flush=True)
    rng = np.random.default_rng(0)
    N = 2000
    rowPtr, colIdx = random_csr(rng, N, 20, hub=30)
    rows = np.repeat(np.arange(N), np.diff(rowPtr))
    harness.save_npz(tmp_path / "g.npz", rows, colIdx, N)
    rp, ci, n = harness.load_npz(tmp_path / "g.npz")
    assert n == N and rp[-1] <= len(colIdx)
    rt, tp, st = harness.run_dataset("g", rp, ci, n, harness.ALGS, embedding_dim=64, niter=3,
                                     stats=True)
    assert set(rt) == set(harness.ALGS) and all(v > 0 for v in rt.values())
    assert st["num_nnz"] == rp[-1]
    paths = harness.write_tables({"g": (rt, tp)}, harness.ALGS, "f3s", "all", "g", str(tmp_path))
    table = pd.read_csv(paths[0], index_col="dataset")
    assert list(table.columns) == harness.ALGS and table.index.tolist() == ["g"]
    assert table.loc["g", "f3s_1tb1rw_scheduled"] == pytest.approx(rt["f3s_1tb1rw_scheduled"])
    assert "throughput" in paths[1]
