"""HIP preprocessing (through the C ABI) against the CPU oracle: bit-exact on every output."""
import json
import os

import numpy as np
import pytest
import torch

from conftest import random_csr
from ref_checks import compare_preprocess

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "preprocess_kat.json")))["cases"]


def to_host(res):
    out = {}
    for k, v in res.items():
        if torch.is_tensor(v):
            v = v.cpu()
            out[k] = v.view(torch.int64).numpy().view(np.uint64) if v.dtype == torch.uint64 \
                else v.numpy()
        else:
            out[k] = v
    return out


def run_gpu(rowPtr, colIdx, N, W=16):
    """Both entry styles: one call with bounded allocations (returned), and count / allocate /
    fill, which must agree with it bit for bit."""
    from fused3s_amd import capi
    rp = torch.as_tensor(np.asarray(rowPtr, np.int32)).cuda()
    ci = torch.as_tensor(np.asarray(colIdx, np.int32)).cuda()
    res = to_host(capi.preprocess(rp, ci, N, 16, W))
    two = to_host(capi.preprocess(rp, ci, N, 16, W, two_phase=True))
    torch.cuda.synchronize()
    for k, v in res.items():
        if isinstance(v, np.ndarray):
            assert v.shape == two[k].shape and np.array_equal(v, two[k]), k
        else:
            assert v == two[k], k
    return res


@pytest.mark.parametrize("case", KAT, ids=[c["name"] for c in KAT])
def test_hand_derived_known_answers(case):
    print("case", case["name"], flush=True)
    got = run_gpu(case["rowPtr"], case["colIdx"], case["N"], case["W"])
    want = dict(case)
    want["tcbBitMap"] = np.array([int(x, 16) for x in case["tcbBitMap"]], dtype=np.uint64)
    compare_preprocess(got, want)


@pytest.mark.parametrize("W", [16, 8])
@pytest.mark.parametrize("seed,N,deg,dup,unsorted,empty,hub", [
    (0, 16, 3, False, False, 0.0, 0),
    (1, 37, 4, False, False, 0.2, 0),
    (2, 100, 9, True, True, 0.1, 7),
    (3, 1030, 30, False, True, 0.0, 0),
    (4, 64, 1, True, False, 0.6, 0),
    (5, 2570, 12, True, True, 0.05, 9),
    (6, 5000, 60, False, False, 0.0, 50),   # windows with > 512 TC blocks at W=8
    (7, 20000, 2, False, False, 0.3, 0),
])
def test_random_graphs_bit_exact(oracle_mod, W, seed, N, deg, dup, unsorted, empty, hub):
    print("case seed=%d N=%d W=%d" % (seed, N, W), flush=True)
    rng = np.random.default_rng(seed)
    rowPtr, colIdx = random_csr(rng, N, deg, dup=dup, unsorted=unsorted, empty_frac=empty, hub=hub)
    got = run_gpu(rowPtr, colIdx, N, W)
    want = oracle_mod.preprocess(rowPtr, colIdx, N, 16, W)
    compare_preprocess(got, want)


def long_window_graph(rng, N, deg, messy_every=0, empty_every=0, hub_rows=0, hub_deg=0):
    """Sorted duplicate-free rows of about `deg` entries; every messy_every-th row shuffled with a
    third of its entries repeated; every empty_every-th row empty; the first hub_rows rows with
    hub_deg entries."""
    rows = []
    for r in range(N):
        if empty_every and r % empty_every == 3:
            rows.append(np.zeros(0, np.int32))
            continue
        d = hub_deg if r < hub_rows else int(rng.poisson(deg))
        cols = np.unique(rng.integers(0, N, size=d))
        if messy_every and r % messy_every == 5:
            cols = np.concatenate([cols, cols[: max(1, len(cols) // 3)]])
            rng.shuffle(cols)
        rows.append(cols.astype(np.int32))
    rowPtr = np.zeros(N + 1, np.int32)
    rowPtr[1:] = np.cumsum([len(c) for c in rows])
    return rowPtr, np.concatenate(rows).astype(np.int32)


@pytest.mark.parametrize("W", [16, 8])
@pytest.mark.parametrize("seed,N,deg,messy,empty", [
    (0, 1000, 300, 0, 0),       # every window ascending
    (1, 3001, 220, 40, 7),      # a messy row in some windows, empty rows, N % 16 != 0
    (2, 777, 400, 1, 0),        # every row shuffled with repeats
    (3, 20000, 150, 300, 50),
])
def test_long_windows_one_bitset_pass(oracle_mod, W, seed, N, deg, messy, empty):
    """Graphs with >= 2048 edges per window and N <= 393216: the one-call entry keeps each
    window's ranking bitset in LDS for both phases."""
    print("case long windows seed=%d N=%d W=%d" % (seed, N, W), flush=True)
    rng = np.random.default_rng(100 + seed)
    rowPtr, colIdx = long_window_graph(rng, N, deg, messy, empty)
    assert rowPtr[-1] >= ((N + 15) // 16) * 2048
    got = run_gpu(rowPtr, colIdx, N, W)
    want = oracle_mod.preprocess(rowPtr, colIdx, N, 16, W)
    compare_preprocess(got, want)


@pytest.mark.parametrize("W", [16, 8])
def test_long_windows_on_a_tiny_node_set(oracle_mod, W):
    """Three windows of 48 nodes whose rows repeat every column dozens of times (2 400 entries per
    row, shuffled): long windows by edge count, a bitset of one 128-bit group, every window on
    the general path; then the same with N = 16 and sorted rows of repeats."""
    print("case long windows, tiny N, W=%d" % W, flush=True)
    rng = np.random.default_rng(3)
    N = 48
    rows = [rng.permutation(np.tile(np.arange(N, dtype=np.int32), 50)) for _ in range(N)]
    rowPtr = np.arange(N + 1, dtype=np.int32) * (50 * N)
    colIdx = np.concatenate(rows)
    got = run_gpu(rowPtr, colIdx, N, W)
    compare_preprocess(got, oracle_mod.preprocess(rowPtr, colIdx, N, 16, W))
    N = 16
    rows = [np.sort(rng.integers(0, N, size=300)).astype(np.int32) for _ in range(N)]
    rowPtr = np.arange(N + 1, dtype=np.int32) * 300
    colIdx = np.concatenate(rows)
    got = run_gpu(rowPtr, colIdx, N, W)
    compare_preprocess(got, oracle_mod.preprocess(rowPtr, colIdx, N, 16, W))


@pytest.mark.parametrize("W", [16, 8])
def test_long_windows_with_a_window_of_several_lds_chunks(oracle_mod, W):
    """As above with one window of ~55 000 distinct columns (more TC blocks than the bitmaps'
    share of LDS holds at once) and, with `messy`, the same window on the general path."""
    print("case long windows, heavy window W=%d" % W, flush=True)
    for messy in (0, 9):
        rng = np.random.default_rng(7 + messy)
        N = 100000
        rowPtr, colIdx = long_window_graph(rng, N, 132, messy_every=messy, hub_rows=16,
                                           hub_deg=5000)
        assert rowPtr[-1] >= ((N + 15) // 16) * 2048
        got = run_gpu(rowPtr, colIdx, N, W)
        want = oracle_mod.preprocess(rowPtr, colIdx, N, 16, W)
        assert want["blockPartition"][0] > (3000 if W == 16 else 6000)
        compare_preprocess(got, want)


def test_long_windows_quarter_scale_benchmark_graph(oracle_mod):
    """The 233k-node benchmark graph at 0.3 of its size (same mean degree): large enough that the
    waves collect their tile ids in LDS and write them as dwords."""
    print("case cfg3 at scale 0.3", flush=True)
    from fused3s_amd import synth
    rp, ci = synth.make_graph("cfg3_chunglu_233k", scale=0.3, device="cuda")
    rowPtr, colIdx = rp.cpu().numpy(), ci.cpu().numpy()
    N = len(rowPtr) - 1
    got = run_gpu(rowPtr, colIdx, N)
    want = oracle_mod.preprocess(rowPtr, colIdx, N)
    compare_preprocess(got, want)


def test_sweep_of_random_shapes(oracle_mod):
    """Forty seeded graphs of mixed shapes (node counts around multiples of 16 and 128, short and
    long windows, repeated / shuffled / empty rows, hub rows, both block widths) through both
    entry styles against the oracle."""
    rng = np.random.default_rng(2024)
    for it in range(40):
        W = 16 if it % 3 else 8
        N = int(rng.choice([15, 16, 17, 127, 128, 129, 500, 1023, 2049, 4100]))
        long_windows = it % 4 == 0
        if long_windows:
            deg = int(rng.integers(140, 400))
            messy = int(rng.choice([0, 1, 7, 50]))
            rowPtr, colIdx = long_window_graph(rng, N, deg, messy_every=messy,
                                               empty_every=int(rng.choice([0, 9])))
            if messy == 1 or rowPtr[-1] < ((N + 15) // 16) * 2048:
                # repeats push short rows of a small node set over the long-window threshold
                rep = int(np.ceil(((N + 15) // 16) * 2048 / max(1, rowPtr[-1]))) + 1
                rows = [np.tile(colIdx[rowPtr[r]:rowPtr[r + 1]], rep) for r in range(N)]
                rowPtr = np.zeros(N + 1, np.int32)
                rowPtr[1:] = np.cumsum([len(x) for x in rows])
                colIdx = np.concatenate(rows).astype(np.int32)
        else:
            rowPtr, colIdx = random_csr(rng, N, int(rng.integers(1, 40)), dup=bool(it & 1),
                                        unsorted=bool(it & 2), empty_frac=float(rng.choice([0, 0.3])),
                                        hub=int(rng.choice([0, 11])))
        print("case sweep %d: N=%d E=%d W=%d long=%s" % (it, N, rowPtr[-1], W, long_windows),
              flush=True)
        got = run_gpu(rowPtr, colIdx, N, W)
        compare_preprocess(got, oracle_mod.preprocess(rowPtr, colIdx, N, 16, W))


def test_heavy_window_many_blocks(oracle_mod):
    """One window whose rows name > 16*512 distinct columns: several LDS chunks in the fill."""
    print("case heavy_window", flush=True)
    rng = np.random.default_rng(0)
    N = 40000
    rows = []
    for r in range(N):
        if r < 16:
            rows.append(np.sort(rng.choice(N, size=2500, replace=False)).astype(np.int32))
        else:
            rows.append(np.array([r], np.int32))
    rowPtr = np.zeros(N + 1, np.int32)
    rowPtr[1:] = np.cumsum([len(x) for x in rows])
    colIdx = np.concatenate(rows)
    got = run_gpu(rowPtr, colIdx, N)
    want = oracle_mod.preprocess(rowPtr, colIdx, N)
    assert want["blockPartition"][0] > 1024
    compare_preprocess(got, want)


def test_multi_pass_bitset_large_n(oracle_mod):
    """N above the per-pass column range of the LDS bitset (393216) -> several passes."""
    print("case large_n", flush=True)
    from fused3s_amd import synth
    N = 1_000_003
    rp, ci = synth.rmat_graph(N, 3_000_000, 0.45, 0.22, 0.22, seed=1)
    rowPtr, colIdx = rp.numpy(), ci.numpy()
    got = run_gpu(rowPtr, colIdx, N)
    want = oracle_mod.preprocess(rowPtr, colIdx, N)
    compare_preprocess(got, want)


def test_more_than_4m_nodes_takes_the_bitonic_short_window_kernel(oracle_mod):
    """Above 2^22 nodes a column id and an edge position no longer share a 32-bit word, so short
    windows are ranked by the bitonic kernel instead of the radix one; long windows (a hub row)
    and the multi-pass bitset are in the same graph."""
    print("case 5m_nodes", flush=True)
    N = 5_000_011
    rng = np.random.default_rng(11)
    deg = np.zeros(N, np.int64)
    rows = rng.choice(N, size=40_000, replace=False)
    deg[rows] = rng.integers(1, 40, size=len(rows))
    deg[123_456] = 3_000  # a window of more than 1024 edges
    rowPtr = np.zeros(N + 1, np.int32)
    rowPtr[1:] = np.cumsum(deg)
    colIdx = rng.integers(0, N, size=int(rowPtr[-1])).astype(np.int32)  # unsorted, may repeat
    got = run_gpu(rowPtr, colIdx, N)
    want = oracle_mod.preprocess(rowPtr, colIdx, N)
    compare_preprocess(got, want)


def test_many_windows_three_sorting_passes_and_all_empty(oracle_mod):
    """More than 16384 windows: the scan and the window order run over many workgroups. One hub
    window of more than 4095 TC blocks makes the order take three 6-bit passes; most windows tie
    at 0 or 1 blocks (ties keep ascending window id). Then the same size with no edge at all."""
    print("case many_windows", flush=True)
    N = 400_000
    rng = np.random.default_rng(5)
    deg = np.zeros(N, np.int64)
    some = rng.choice(N, size=60_000, replace=False)
    deg[some] = rng.integers(1, 30, size=len(some))
    deg[200_000:200_016] = 6_000  # 16 hub rows in one window: ~90k distinct columns
    rowPtr = np.zeros(N + 1, np.int32)
    rowPtr[1:] = np.cumsum(deg)
    colIdx = rng.integers(0, N, size=int(rowPtr[-1])).astype(np.int32)
    got = run_gpu(rowPtr, colIdx, N)
    want = oracle_mod.preprocess(rowPtr, colIdx, N)
    assert want["blockPartition"].max() > 4095
    compare_preprocess(got, want)
    got = run_gpu(np.zeros(N + 1, np.int32), np.zeros(0, np.int32), N)
    assert got["blockCount"] == 0 and not got["rowWindowOffset"].any()
    assert np.array_equal(got["sortedRowWindows"], np.arange((N + 15) // 16))


def test_empty_graph_and_tiny():
    print("case empty", flush=True)
    got = run_gpu(np.zeros(41, np.int32), np.zeros(0, np.int32), 40)
    assert got["blockCount"] == 0 and list(got["rowWindowOffset"]) == [0, 0, 0, 0]
    assert list(got["sortedRowWindows"]) == [0, 1, 2] and list(got["tcblockOffset"]) == [0]
    got = run_gpu(np.array([0, 1], np.int32), np.array([0], np.int32), 1)
    assert got["blockCount"] == 1 and got["sparseAToXidx"][0] == 0
    assert int(got["tcbBitMap"][0]) == 1 << 63


def test_out_of_range_column_is_an_error():
    from fused3s_amd import capi
    rp = torch.tensor([0, 1, 2], dtype=torch.int32).cuda()
    ci = torch.tensor([0, 7], dtype=torch.int32).cuda()
    with pytest.raises(RuntimeError, match="column index"):
        capi.preprocess(rp, ci, 2)
    with pytest.raises(RuntimeError, match="column index"):
        capi.preprocess(rp, ci, 2, two_phase=True)
    # long windows (the kernels that do both phases at once): 64 rows of 2100 entries, one bad
    N = 64
    rowPtr = torch.arange(N + 1, dtype=torch.int32) * 2100
    cols = (torch.arange(N * 2100, dtype=torch.int32) % N)
    cols[70000] = N
    with pytest.raises(RuntimeError, match="column index"):
        capi.preprocess(rowPtr.cuda(), cols.cuda(), N)


@pytest.mark.parametrize("name,scale", [("cfg1_gnm_2708", 1.0), ("cfg2_rmat_169k", 1.0),
                                        ("cfg3_chunglu_233k", 0.02), ("cfg5_sbm_100k", 1.0)])
def test_benchmark_shapes_bit_exact(oracle_mod, name, scale):
    print("case", name, flush=True)
    from fused3s_amd import synth
    rp, ci = synth.make_graph(name, scale=scale)
    N = rp.numel() - 1
    got = run_gpu(rp.numpy(), ci.numpy(), N)
    want = oracle_mod.preprocess(rp.numpy(), ci.numpy(), N)
    compare_preprocess(got, want)
