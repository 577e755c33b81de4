"""Pins oracle/f3s_oracle.c preprocessing: hand-derived known answers, an independent dense
derivation, structural invariants, and the documented edgeToRow stride slip."""
import json
import os

import numpy as np
import pytest

from conftest import random_csr
from ref_checks import brute_preprocess, compare_preprocess, consume_bitmap_like_kernel, \
    dense_from_csr

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "preprocess_kat.json")))["cases"]


@pytest.mark.parametrize("case", KAT, ids=[c["name"] for c in KAT])
def test_hand_derived_known_answers(oracle_mod, case):
    got = oracle_mod.preprocess(case["rowPtr"], case["colIdx"], case["N"], case["H"], case["W"])
    want = dict(case)
    want["tcbBitMap"] = np.array([int(x, 16) for x in case["tcbBitMap"]], dtype=np.uint64)
    compare_preprocess(got, want)


@pytest.mark.parametrize("W", [16, 8])
@pytest.mark.parametrize("seed,N,deg,dup,unsorted,empty", [
    (0, 16, 3, False, False, 0.0),
    (1, 37, 4, False, False, 0.2),
    (2, 100, 9, True, True, 0.1),
    (3, 130, 30, False, True, 0.0),
    (4, 64, 1, True, False, 0.6),
    (5, 257, 12, True, True, 0.05),
])
def test_against_dense_brute_force(oracle_mod, W, seed, N, deg, dup, unsorted, empty):
    rng = np.random.default_rng(seed)
    rowPtr, colIdx = random_csr(rng, N, deg, dup=dup, unsorted=unsorted, empty_frac=empty, hub=7)
    got = oracle_mod.preprocess(rowPtr, colIdx, N, 16, W)
    want = brute_preprocess(rowPtr, colIdx, N, 16, W)
    compare_preprocess(got, want)


def test_bitmap_matches_kernel_side_indexing(oracle_mod):
    """The bits, read back with the reference kernel's own lane/fragment indexing, reproduce
    the adjacency restricted to the block's compacted columns."""
    rng = np.random.default_rng(11)
    N = 75
    rowPtr, colIdx = random_csr(rng, N, 10)
    A = dense_from_csr(rowPtr, colIdx, N) > 0
    r = oracle_mod.preprocess(rowPtr, colIdx, N)
    rwo, atox, bm = r["rowWindowOffset"], r["sparseAToXidx"], r["tcbBitMap"]
    for w in range(len(rwo) - 1):
        ucols = np.nonzero(A[16 * w:16 * w + 16].any(axis=0))[0]
        for t in range(rwo[w], rwo[w + 1]):
            tile = consume_bitmap_like_kernel(bm, t)
            nvalid = min(16, len(ucols) - 16 * (t - rwo[w]))
            for rl in range(16):
                for cl in range(16):
                    row = 16 * w + rl
                    want = row < N and cl < nvalid and A[row, atox[t * 16 + cl]]
                    assert tile[rl, cl] == want, (w, t, rl, cl)


def test_invariants_medium_graph(oracle_mod):
    rng = np.random.default_rng(5)
    N = 3000
    rowPtr, colIdx = random_csr(rng, N, 20, hub=97)
    r = oracle_mod.preprocess(rowPtr, colIdx, N)
    rwo, atox, bm = r["rowWindowOffset"], r["sparseAToXidx"], r["tcbBitMap"]
    # popcount of all bitmaps == number of distinct (row, col) pairs
    pop = sum(bin(int(x)).count("1") for x in bm)
    assert pop == len(colIdx)  # random_csr without dup gives distinct pairs
    # per-block nnz sums to the CSR row-pointer differences (scripts/graph_stat/paper_graph_stat.py:68-72)
    toff = r["tcblockOffset"]
    for w in (0, 10, 50, len(rwo) - 2):
        assert toff[rwo[w + 1]] - toff[rwo[w]] == rowPtr[min(16 * w + 16, N)] - rowPtr[16 * w]
    # compacted columns strictly ascending over the valid slots of a window
    for w in range(len(rwo) - 1):
        seg = atox[rwo[w] * 16:rwo[w + 1] * 16]
        u = len(np.unique(colIdx[rowPtr[16 * w]:rowPtr[min(16 * w + 16, N)]]))
        assert np.all(np.diff(seg[:u]) > 0)
        assert np.all(seg[u:] == 0)
    # heavy-first order: a permutation, counts non-increasing, ties by ascending id
    order = r["sortedRowWindows"]
    cnt = np.diff(rwo)
    assert sorted(order.tolist()) == list(range(len(cnt)))
    key = list(zip((-cnt[order]).tolist(), order.tolist()))
    assert key == sorted(key)


def test_edge_to_row_stride_slip_is_reproduced_only_on_request(oracle_mod):
    """src/utils.cu:348 strides by gridDim.x: with N > 1024 (G > 32) and a row of degree > 32 the
    reference leaves entries unwritten (zero). The default oracle writes the true row."""
    N = 1300  # G = ceil(1300/32) = 41
    rowPtr = np.zeros(N + 1, np.int32)
    deg = np.ones(N, np.int32)
    deg[700] = 100
    rowPtr[1:] = np.cumsum(deg)
    colIdx = np.zeros(rowPtr[-1], np.int32)
    for r in range(N):
        n = rowPtr[r + 1] - rowPtr[r]
        colIdx[rowPtr[r]:rowPtr[r + 1]] = (np.arange(n) * 3 + r) % N
    good = oracle_mod.preprocess(rowPtr, colIdx, N)
    bad = oracle_mod.preprocess(rowPtr, colIdx, N, emulate_stride_bug=True)
    s = rowPtr[700]
    k = np.arange(100)
    written = (k % 41) < 32
    assert np.all(good["edgeToRow"][s:s + 100] == 700)
    assert np.all(bad["edgeToRow"][s:s + 100][written] == 700)
    assert np.all(bad["edgeToRow"][s:s + 100][~written] == 0)
    # block structure is unaffected, bitmaps are not
    for key in ("rowWindowOffset", "sparseAToXidx", "edgeToColumn"):
        assert np.array_equal(good[key], bad[key])
    assert not np.array_equal(good["tcbBitMap"], bad["tcbBitMap"])
    # below the threshold the two agree
    N2 = 1000
    rng = np.random.default_rng(3)
    rp2, ci2 = random_csr(rng, N2, 40)
    a = oracle_mod.preprocess(rp2, ci2, N2)
    b = oracle_mod.preprocess(rp2, ci2, N2, emulate_stride_bug=True)
    compare_preprocess(a, b)


def test_empty_graph_and_empty_windows(oracle_mod):
    r = oracle_mod.preprocess(np.zeros(41, np.int32), np.zeros(0, np.int32), 40)
    assert r["blockCount"] == 0 and list(r["rowWindowOffset"]) == [0, 0, 0, 0]
    assert list(r["sortedRowWindows"]) == [0, 1, 2] and list(r["tcblockOffset"]) == [0]
