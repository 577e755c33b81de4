"""The column-sliced schedule beyond the basic parity cases of test_gpu_attention.py: the
multi-head entry on a graph of long windows, a prepared workspace (f3s_attention_prepare), block
ranges that do not fit the stated structure, run-time switches read per call, and K / V whose span
exceeds 4 GiB (64-bit row offsets; the reference indexes rows with int64_t,
src/F3S_kernel.cu:1422-1423).

Tolerance: max-abs 2e-2 and mean-relative 1e-3 against the reference-emulating oracle.
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from conftest import random_csr

MAX_ABS = 2e-2
MEAN_REL = 1e-3


def mean_rel(a, b):
    return float(np.abs(a - b).mean() / max(np.abs(b).mean(), 1e-30))


def bits(t):
    t = t.contiguous().cpu()
    if t.dtype == torch.float16:
        return t.numpy()
    return t.view(torch.int16).numpy().view(np.uint16)


def to_dev(pre):
    dev = "cuda"
    rwo = torch.as_tensor(pre["rowWindowOffset"].astype(np.int32)).to(dev)
    atox = torch.as_tensor(pre["sparseAToXidx"].astype(np.int32)).to(dev)
    bm = torch.as_tensor(pre["tcbBitMap"].view(np.int64)).to(dev).view(torch.uint64)
    order = torch.as_tensor(pre["sortedRowWindows"].astype(np.int32)).to(dev)
    return rwo, order, atox, bm


@pytest.fixture(scope="module")
def long_window_graph(oracle_mod):
    """The 233k-node benchmark generator at 0.145 of its size: 33 779 nodes (N % 16 != 0), 2 112
    windows of about 130 TC blocks: the library picks the column-sliced schedule by itself."""
    from fused3s_amd import synth
    rp, ci = synth.make_graph("cfg3_chunglu_233k", scale=0.145)
    N = rp.numel() - 1
    pre = oracle_mod.preprocess(rp.numpy(), ci.numpy(), N)
    return N, rp.numpy(), ci.numpy(), pre


@pytest.mark.gpu
@pytest.mark.parametrize("persistent", ["0", "1"])
def test_multihead_entry_takes_the_sliced_schedule(oracle_mod, long_window_graph, monkeypatch,
                                                   persistent):
    """8 heads x d = 32 bf16 through f3s_attention_fwd_heads with a workspace: every head within
    tolerance of the oracle and close to the same call without a workspace (window kernel)."""
    from fused3s_amd import capi
    print("case sliced heads persistent=%s" % persistent, flush=True)
    monkeypatch.setenv("F3S_SLICED_PERSISTENT", persistent)
    N, _, _, pre = long_window_graph
    heads, d = 8, 32
    g = torch.Generator().manual_seed(5)
    Q, K, V = [(torch.randn((N, heads, d), generator=g) * d ** -0.25).to(torch.bfloat16)
               for _ in range(3)]
    scale = float(np.sqrt(d))
    rwo, order, atox, bm = to_dev(pre)
    nT = int(pre["blockCount"])
    ws = capi.attention_workspace(N, d, "cuda", nTCB=nT, dtype=torch.bfloat16, heads=heads)
    assert ws is not None or os.environ.get("F3S_SCHEDULE") == "window"
    Qd, Kd, Vd = Q.cuda(), K.cuda(), V.cuda()
    plain = capi.attention_heads(rwo, order, atox, bm, N, Qd, Kd, Vd, scale).cpu().numpy()
    for od in (order, None):
        got = capi.attention_heads(rwo, od, atox, bm, N, Qd, Kd, Vd, scale,
                                   workspace=ws).cpu().numpy()
        assert np.isfinite(got).all()
        assert np.abs(got - plain).max() < 2e-3
    for h in range(heads):
        want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                        pre["tcbBitMap"], N, bits(Q[:, h]), bits(K[:, h]),
                                        bits(V[:, h]), scale, dtype=1)
        assert np.abs(got[:, h * d:(h + 1) * d] - want).max() < MAX_ABS, "head %d" % h
        assert mean_rel(got[:, h * d:(h + 1) * d], want) < MEAN_REL, "head %d" % h


@pytest.mark.gpu
def test_prepared_workspace(oracle_mod, long_window_graph, monkeypatch):
    """f3s_attention_prepare builds the schedule's index once; calls with prepared = 1 give the
    rows of a call that builds it itself, bit for bit. A prepared workspace handed to a call with
    OTHER arrays is noticed on the device (the index is rebuilt for them), and the preparation
    ends there: the original arrays with prepared = 1 are again computed correctly."""
    from fused3s_amd import capi
    print("case sliced prepared", flush=True)
    monkeypatch.setenv("F3S_SCHEDULE", "sliced")
    N, _, _, pre = long_window_graph
    d = 64
    rng = np.random.default_rng(9)
    Q, K, V = [torch.as_tensor(rng.standard_normal((N, d)).astype(np.float16)).cuda()
               for _ in range(3)]
    rwo, order, atox, bm = to_dev(pre)
    nT = int(pre["blockCount"])
    ws = capi.attention_workspace(N, d, "cuda", nTCB=nT)
    base = capi.attention(rwo, order, atox, bm, N, Q, K, V, 8.0, workspace=ws).cpu().numpy()
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                    pre["tcbBitMap"], N, bits(Q), bits(K), bits(V), 8.0)
    assert np.abs(base - want).max() < MAX_ABS and mean_rel(base, want) < MEAN_REL
    capi.attention_prepare(rwo, atox, N, d, ws)
    for _ in range(2):
        got = capi.attention(rwo, order, atox, bm, N, Q, K, V, 8.0, workspace=ws, prepared=True)
        assert np.array_equal(got.cpu().numpy(), base)
    # another structure (the same graph with every second window emptied) on the same workspace
    counts = np.diff(pre["rowWindowOffset"]).copy()
    counts[1::2] = 0
    keep = np.repeat(np.arange(len(counts)) % 2 == 0, np.diff(pre["rowWindowOffset"]))
    other = dict(pre)
    other["rowWindowOffset"] = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    other["sparseAToXidx"] = pre["sparseAToXidx"].reshape(-1, 16)[keep].reshape(-1)
    other["tcbBitMap"] = pre["tcbBitMap"].reshape(-1, 4)[keep].reshape(-1)
    rwo2, _, atox2, bm2 = to_dev(other)
    got2 = capi.attention(rwo2, order, atox2, bm2, N, Q, K, V, 8.0, workspace=ws,
                          prepared=True).cpu().numpy()
    want2 = oracle_mod.attention_ref(other["rowWindowOffset"], other["sparseAToXidx"],
                                     other["tcbBitMap"], N, bits(Q), bits(K), bits(V), 8.0)
    assert np.abs(got2 - want2).max() < MAX_ABS and mean_rel(got2, want2) < MEAN_REL
    emptied = np.repeat(np.arange(len(counts)) % 2 == 1, 16)[:N]
    assert not got2[emptied].any()
    got = capi.attention(rwo, order, atox, bm, N, Q, K, V, 8.0, workspace=ws, prepared=True)
    assert np.array_equal(got.cpu().numpy(), base)


@pytest.mark.gpu
@pytest.mark.parametrize("persistent", ["0", "1"])
def test_block_ranges_beyond_the_stated_total_are_left_empty(oracle_mod, monkeypatch, persistent):
    """The sliced schedule with a rowWindowOffset that ends beyond the stated block total (the
    arrays of another preprocessing run): the windows whose range does not fit are rows of zeros,
    the others are computed as usual; nothing is read beyond the stated arrays."""
    from fused3s_amd import capi
    print("case sliced stated total persistent=%s" % persistent, flush=True)
    monkeypatch.setenv("F3S_SCHEDULE", "sliced")
    monkeypatch.setenv("F3S_SLICED_PERSISTENT", persistent)
    rng = np.random.default_rng(31)
    N, d = 4000, 64
    rowPtr, colIdx = random_csr(rng, N, 60)
    Q, K, V = [torch.as_tensor(rng.standard_normal((N, d)).astype(np.float16)).cuda()
               for _ in range(3)]
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    rwo_h = pre["rowWindowOffset"]
    rwo, order, atox, bm = to_dev(pre)
    ws = capi.attention_workspace(N, d, "cuda", nTCB=int(pre["blockCount"]))
    assert ws is not None
    full = capi.attention(rwo, order, atox, bm, N, Q, K, V, 8.0, workspace=ws).cpu().numpy()
    want = oracle_mod.attention_ref(rwo_h, pre["sparseAToXidx"], pre["tcbBitMap"], N, bits(Q),
                                    bits(K), bits(V), 8.0)
    assert np.abs(full - want).max() < MAX_ABS
    keep = int(np.searchsorted(rwo_h, rwo_h[-1] // 2, side="right")) - 1
    stated = int(rwo_h[keep])
    ws.fill_(0xFF)  # stale scratch must not leak into the rows
    for od in (None, order):
        got = capi.attention(rwo, od, atox[: stated * 16], bm[: stated * 4], N, Q, K, V, 8.0,
                             workspace=ws).cpu().numpy()
        assert np.array_equal(got[: keep * 16], full[: keep * 16])
        assert not got[keep * 16:].any()


@pytest.mark.gpu
def test_schedule_switches_are_read_per_call(oracle_mod, long_window_graph, monkeypatch):
    """F3S_SCHEDULE and F3S_SHORT_WINDOWS set after the first call take effect in the same
    process."""
    from fused3s_amd import capi
    print("case switches per call", flush=True)
    N, _, _, pre = long_window_graph
    nT = int(pre["blockCount"])
    L = capi.lib()
    monkeypatch.delenv("F3S_SCHEDULE", raising=False)
    assert L.f3s_attention_uses_workspace(N, nT, 64, 0) == 1
    monkeypatch.setenv("F3S_SCHEDULE", "window")
    assert L.f3s_attention_uses_workspace(N, nT, 64, 0) == 0
    monkeypatch.setenv("F3S_SCHEDULE", "sliced")
    assert L.f3s_attention_uses_workspace(300, 2000, 64, 0) == 1
    monkeypatch.delenv("F3S_SCHEDULE", raising=False)
    assert L.f3s_attention_uses_workspace(300, 2000, 64, 0) == 0
    # the split of short windows: same rows either way, so the switch shows in the results only
    # through the summation order of long windows; both settings must meet the oracle
    rng = np.random.default_rng(4)
    Ns, d = 20_000, 32
    rowPtr, colIdx = random_csr(rng, Ns, 4, hub=1999)
    Q, K, V = [torch.as_tensor(rng.standard_normal((Ns, d)).astype(np.float16)).cuda()
               for _ in range(3)]
    p2 = oracle_mod.preprocess(rowPtr, colIdx, Ns)
    rwo, order, atox, bm = to_dev(p2)
    want = oracle_mod.attention_ref(p2["rowWindowOffset"], p2["sparseAToXidx"], p2["tcbBitMap"],
                                    Ns, bits(Q), bits(K), bits(V), 5.0)
    outs = []
    for flag in ("1", "0", "1"):
        monkeypatch.setenv("F3S_SHORT_WINDOWS", flag)
        got = capi.attention(rwo, order, atox, bm, Ns, Q, K, V, 5.0).cpu().numpy()
        assert np.abs(got - want).max() < MAX_ABS and mean_rel(got, want) < MEAN_REL
        outs.append(got)
    assert np.array_equal(outs[0], outs[2])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_padded_row_copies_change_nothing(oracle_mod, long_window_graph, monkeypatch, dtype):
    """At d = 64 the single-head column-sliced call gathers from copies of K and V with 256-byte
    rows that it makes in its workspace (F3S_PAD_ROWS=0 switches them off): same arithmetic on the
    same values, so the results are bit-identical, with and without a prepared workspace, and meet
    the oracle. K and V are changed between calls: the copies are made per call."""
    from fused3s_amd import capi
    print("case padded rows %s" % dtype, flush=True)
    N, _, _, pre = long_window_graph
    rwo, order, atox, bm = to_dev(pre)
    g = torch.Generator().manual_seed(64)
    Q, K, V = [torch.randn((N, 64), generator=g).to(dtype).cuda() for _ in range(3)]
    code = 0 if dtype == torch.float16 else 1
    L = capi.lib()
    assert L.f3s_attention_workspace_bytes(N, 64) >= 2 * N * 256  # room for the copies
    ws = capi.attention_workspace(N, 64, "cuda")
    outs = {}
    for flag in ("1", "0"):
        monkeypatch.setenv("F3S_PAD_ROWS", flag)
        outs[flag] = capi.attention(rwo, order, atox, bm, N, Q, K, V, 8.0, workspace=ws).clone()
    assert torch.equal(outs["1"], outs["0"])
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"], pre["tcbBitMap"],
                                    N, bits(Q), bits(K), bits(V), 8.0, dtype=code)
    got = outs["1"].cpu().numpy()
    assert np.abs(got - want).max() < MAX_ABS and mean_rel(got, want) < MEAN_REL
    monkeypatch.setenv("F3S_PAD_ROWS", "1")
    capi.attention_prepare(rwo, atox, N, 64, ws)
    K2, V2 = V.clone(), K.clone()  # other values in the same call sequence
    a = capi.attention(rwo, order, atox, bm, N, Q, K2, V2, 8.0, workspace=ws, prepared=True).clone()
    monkeypatch.setenv("F3S_PAD_ROWS", "0")
    b = capi.attention(rwo, order, atox, bm, N, Q, K2, V2, 8.0, workspace=ws, prepared=True)
    assert torch.equal(a, b) and not torch.equal(a, outs["1"])


def test_wide_offset_rule():
    """Host side of the 64-bit row offsets: which problems take them (no GPU needed)."""
    from fused3s_amd import capi
    L = capi.lib()
    f = L.f3s_attention_uses_wide_offsets
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
    assert f(232_965, 128, 0) == 0
    assert f(2_449_029, 256, 0) == 0
    assert f((1 << 32) // 256 - 1, 256, 0) == 0      # one row short of 4 GiB
    assert f((1 << 32) // 256, 256, 0) == 1          # exactly 4 GiB
    assert f(17_000_000, 256, 0) == 1
    assert f(1000, 512, 1) == 0
    assert f(1 << 24, 64, 1) == 1                    # row count beyond the 24-bit multiply
    assert f(1000, 1 << 24, 1) == 1                  # pitch beyond the 24-bit multiply
    assert f(3000, 2 << 20, 1) == 1                  # 3000 rows of 2 MiB: 5.9 GiB


@pytest.mark.gpu
def test_rows_beyond_4_gib(oracle_mod):
    """K and V as pitched views whose span exceeds 4 GiB on a small node set (2 304 rows of 2 MiB
    each): rows at high addresses are gathered with 64-bit offsets. Single head through the
    multi-head entry, against the oracle on the same values held contiguously."""
    from fused3s_amd import capi
    print("case wide offsets", flush=True)
    free, _ = torch.cuda.mem_get_info()
    if free < 24 * (1 << 30):
        pytest.skip("needs 24 GiB of free device memory")
    N, d = 2304, 64
    pitch = 1 << 20  # elements: 2 MiB per row
    assert capi.lib().f3s_attention_uses_wide_offsets
    rng = np.random.default_rng(77)
    rowPtr, colIdx = random_csr(rng, N, 50, hub=97)
    vals = [rng.standard_normal((N, d)).astype(np.float16) for _ in range(3)]
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                    pre["tcbBitMap"], N, vals[0], vals[1], vals[2], 8.0)
    rwo, order, atox, bm = to_dev(pre)
    views = []
    for v in vals:
        store = torch.empty((N, pitch), dtype=torch.float16, device="cuda")
        store[:, :d] = torch.as_tensor(v).cuda()
        views.append(store[:, :d].unflatten(1, (1, d)))
        assert views[-1].stride(0) * 2 * N > (1 << 32)
    for od in (order, None):
        got = capi.attention_heads(rwo, od, atox, bm, N, views[0], views[1], views[2],
                                   8.0).cpu().numpy()
        assert np.abs(got - want).max() < MAX_ABS
        assert mean_rel(got, want) < MEAN_REL
    # the same through the column-sliced schedule
    os.environ["F3S_SCHEDULE"] = "sliced"
    try:
        ws = capi.attention_workspace(N, d, "cuda", nTCB=int(pre["blockCount"]), heads=1)
        got = capi.attention_heads(rwo, order, atox, bm, N, views[0], views[1], views[2], 8.0,
                                   workspace=ws).cpu().numpy()
    finally:
        del os.environ["F3S_SCHEDULE"]
    assert np.abs(got - want).max() < MAX_ABS
    assert mean_rel(got, want) < MEAN_REL


@pytest.mark.gpu
@pytest.mark.parametrize("sliced", [True, False])
def test_attention_call_under_graph_capture(oracle_mod, long_window_graph, sliced):
    """f3s_attention_fwd only launches kernels (no host wait, no copy, no allocation), so a call
    can be captured into a HIP graph, the very first call on a workspace included. Three replays
    with eager work and synchronisations between them, each against the eager result; new Q
    values written into the captured input buffer between replays show up in the output."""
    from fused3s_amd import capi
    print("case graph capture sliced=%s" % sliced, flush=True)
    N, _, _, pre = long_window_graph
    d = 64
    rng = np.random.default_rng(13)
    Q, K, V = [torch.as_tensor(rng.standard_normal((N, d)).astype(np.float16)).cuda()
               for _ in range(3)]
    rwo, order, atox, bm = to_dev(pre)
    ws = capi.attention_workspace(N, d, "cuda", nTCB=int(pre["blockCount"])) if sliced else None
    out = torch.empty((N, d), dtype=torch.float32, device="cuda")
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            capi.attention(rwo, order, atox, bm, N, Q, K, V, 8.0, out=out, workspace=ws)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        if rep:
            Q.copy_(torch.as_tensor(rng.standard_normal((N, d)).astype(np.float16)))
        out.fill_(-3.0)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        eager = capi.attention(rwo, order, atox, bm, N, Q, K, V, 8.0, workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(got, eager), "replay %d" % rep
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                    pre["tcbBitMap"], N, bits(Q), bits(K), bits(V), 8.0)
    assert np.abs(got.cpu().numpy() - want).max() < MAX_ABS
