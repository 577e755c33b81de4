"""Fused 3S attention (HIP, through the C ABI) against the CPU oracles.

Tolerance (fp16 inputs, fp32 accumulation): max-abs 2e-2 and mean-relative 1e-3 against the
reference-emulating oracle.
"""
import os

import numpy as np
import pytest
import torch

from conftest import random_csr

pytestmark = pytest.mark.gpu
MAX_ABS = 2e-2
MEAN_REL = 1e-3


def mean_rel(a, b):
    return float(np.abs(a - b).mean() / max(np.abs(b).mean(), 1e-30))


def gpu_attention(pre, N, Q, K, V, scale, order=None, softmax=True, sliced=False):
    from fused3s_amd import capi
    dev = "cuda"
    rwo = torch.as_tensor(pre["rowWindowOffset"].astype(np.int32)).to(dev)
    atox = torch.as_tensor(pre["sparseAToXidx"].astype(np.int32)).to(dev)
    bm = torch.as_tensor(pre["tcbBitMap"].view(np.int64)).to(dev).view(torch.uint64)
    od = None if order is None else torch.as_tensor(np.asarray(order, np.int32)).to(dev)
    ws = capi.attention_workspace(N, Q.shape[1], dev) if sliced else None
    out = capi.attention(rwo, od, atox, bm, N, torch.as_tensor(Q).to(dev),
                         torch.as_tensor(K).to(dev), torch.as_tensor(V).to(dev), scale, softmax,
                         workspace=ws)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def feats(rng, N, d, std=1.0):
    return [(rng.standard_normal((N, d)) * std).astype(np.float16) for _ in range(3)]


@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("seed,N,deg,hub", [(0, 300, 25, 13), (1, 1000, 100, 0), (2, 77, 6, 0),
                                            (3, 16, 2, 0), (4, 4099, 40, 100)])
def test_matches_reference_numerics(oracle_mod, d, seed, N, deg, hub):
    print("case d=%d seed=%d N=%d" % (d, seed, N), flush=True)
    rng = np.random.default_rng(seed)
    rowPtr, colIdx = random_csr(rng, N, deg, hub=hub, empty_frac=0.05)
    Q, K, V = feats(rng, N, d)
    scale = float(np.sqrt(d))
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                    pre["tcbBitMap"], N, Q, K, V, scale)
    txt = oracle_mod.attention_textbook(rowPtr, colIdx, N, Q, K, V, scale)
    for order in (None, pre["sortedRowWindows"]):
        got = gpu_attention(pre, N, Q, K, V, scale, order)
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() < MAX_ABS
        assert mean_rel(got, want) < MEAN_REL
        assert np.abs(got - txt).max() < MAX_ABS


def test_unscaled_uniform_features_like_reference_harness(oracle_mod):
    """scripts/tests/test_f3s_accuracy.py:96-236: N=1000, 10 % dense, d=128, U[0,1), no scaling."""
    print("case harness", flush=True)
    rng = np.random.default_rng(0)
    N, d = 1000, 128
    A = rng.random((N, N)) < 0.1
    rowPtr = np.zeros(N + 1, np.int32)
    rowPtr[1:] = np.cumsum(A.sum(axis=1))
    colIdx = np.nonzero(A)[1].astype(np.int32)
    Q, K, V = [rng.random((N, d)).astype(np.float16) for _ in range(3)]
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                    pre["tcbBitMap"], N, Q, K, V, 1.0)
    got = gpu_attention(pre, N, Q, K, V, 1.0, pre["sortedRowWindows"])
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 2e-3
    assert np.abs(got - want).max() < MAX_ABS


def test_closed_forms_and_quirks(oracle_mod):
    print("case closed_forms", flush=True)
    rng = np.random.default_rng(7)
    N, d = 48, 64
    Q, K, V = feats(rng, N, d)
    rows = []
    for r in range(N):
        rows.append([] if r == 5 else ([(7 * r + 3) % N] if r < 40 else [1, 2, 3, 4]))
    K[2] = K[1]
    K[3] = K[1]
    K[4] = K[1]
    Q[9] = 0  # all scores exactly zero: dropped like masked entries -> row sum 0 -> output 0
    rowPtr = np.zeros(N + 1, np.int32)
    rowPtr[1:] = np.cumsum([len(x) for x in rows])
    colIdx = np.array([c for x in rows for c in x], np.int32)
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    out = gpu_attention(pre, N, Q, K, V, 8.0)
    for r in range(40):
        if r in (5, 9):
            assert np.all(out[r] == 0)
        else:
            assert np.abs(out[r] - V[(7 * r + 3) % N].astype(np.float32)).max() < 2e-3
    mean = V[1:5].astype(np.float64).mean(axis=0)
    for r in range(40, N):
        assert np.abs(out[r] - mean).max() < 2e-3


def test_sddmm_spmm_without_softmax(oracle_mod):
    print("case no_softmax", flush=True)
    rng = np.random.default_rng(5)
    N, d = 900, 64
    rowPtr, colIdx = random_csr(rng, N, 20)
    Q, K, V = feats(rng, N, d, std=0.5)
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                    pre["tcbBitMap"], N, Q, K, V, 1.0, applySoftmax=False)
    got = gpu_attention(pre, N, Q, K, V, 1.0, None, softmax=False)
    assert np.abs(got - want).max() < 2e-2 * max(1.0, np.abs(want).max())
    assert mean_rel(got, want) < MEAN_REL


def test_end_to_end_hip_preprocess_then_attention(oracle_mod):
    """CSR -> HIP preprocessing -> HIP attention, checked against the textbook oracle."""
    print("case end_to_end", flush=True)
    from fused3s_amd import capi, synth
    rp, ci = synth.make_graph("cfg1_gnm_2708")
    N = rp.numel() - 1
    Q, K, V = synth.features(N, 64, seed=0)
    pre = capi.preprocess(rp.cuda(), ci.cuda(), N)
    out = capi.attention(pre["rowWindowOffset"], pre["sortedRowWindows"], pre["sparseAToXidx"],
                         pre["tcbBitMap"], N, Q.cuda(), K.cuda(), V.cuda(), 8.0)
    torch.cuda.synchronize()
    txt = oracle_mod.attention_textbook(rp.numpy(), ci.numpy(), N, Q.numpy(), K.numpy(),
                                        V.numpy(), 8.0)
    got = out.cpu().numpy()
    assert np.abs(got - txt).max() < MAX_ABS and mean_rel(got, txt) < MEAN_REL


@pytest.mark.parametrize("persistent", ["0", "1"])
@pytest.mark.parametrize("phases", [2, 3])
def test_column_sliced_schedule_with_several_phases(oracle_mod, monkeypatch, phases, persistent):
    """16 and 24 column slices (two and three per XCD, which the library only picks by itself above
    64 MiB of K + V) through the launch-ordered kernel and through the queue-based one."""
    print("case sliced phases=%d persistent=%s" % (phases, persistent), flush=True)
    from fused3s_amd import synth
    monkeypatch.setenv("F3S_SLICE_PHASES", str(phases))
    monkeypatch.setenv("F3S_SLICED_PERSISTENT", persistent)
    rp, ci = synth.make_graph("cfg3_chunglu_233k", scale=0.145)
    N = rp.numel() - 1
    rng = np.random.default_rng(phases)
    d = 64
    Q, K, V = feats(rng, N, d)
    pre = oracle_mod.preprocess(rp.numpy(), ci.numpy(), N)
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                    pre["tcbBitMap"], N, Q, K, V, 8.0)
    for order in (pre["sortedRowWindows"], None):
        got = gpu_attention(pre, N, Q, K, V, 8.0, order, sliced=True)
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() < MAX_ABS
        assert mean_rel(got, want) < MEAN_REL


def test_sweep_of_random_problems(oracle_mod):
    """Thirty seeded problems of mixed shape (node counts around multiples of 16, degrees from 1 to
    a few hundred, hub rows, empty rows), head dimension, input type (fp16 / bf16), window order and
    score scaling (fp16 also unscaled, where rows of very negative scores underflow to 0 as in the
    reference) through f3s_attention_fwd against the reference-emulating oracle, every tenth one
    without softmax."""
    from fused3s_amd import capi
    rng = np.random.default_rng(77)
    dev = "cuda"
    as_bits = lambda t: t.view(torch.int16).numpy().view(np.uint16)
    for it in range(30):
        N = int(rng.choice([16, 17, 31, 100, 257, 1000, 3001]))
        d = int(rng.choice([32, 64, 128]))
        deg = int(rng.choice([1, 3, 17, 60, 250]))
        deg = min(deg, max(1, N // 2))
        bf16 = bool(it % 3 == 1)
        softmax = it % 10 != 9
        scale = float(rng.choice([1.0, np.sqrt(d)]))
        if bf16:
            # unscaled scores of N(0, d) reach below -17, where the reference's fp16 probabilities
            # underflow to 0 (a row of only such scores comes out as 0, which the fp16 kernel
            # reproduces); the bf16 kernel keeps them, so it is compared where they survive
            scale = float(np.sqrt(d))
        rowPtr, colIdx = random_csr(rng, N, deg, hub=int(rng.choice([0, 13])),
                                    empty_frac=float(rng.choice([0.0, 0.2])))
        print("case sweep %d: N=%d d=%d deg=%d bf16=%s softmax=%s scale=%.2f"
              % (it, N, d, deg, bf16, softmax, scale), flush=True)
        std = 1.0 if softmax else 0.4
        Qf, Kf, Vf = [(rng.standard_normal((N, d)) * std).astype(np.float32) for _ in range(3)]
        tdt = torch.bfloat16 if bf16 else torch.float16
        Qt, Kt, Vt = (torch.as_tensor(x).to(tdt) for x in (Qf, Kf, Vf))
        pre = oracle_mod.preprocess(rowPtr, colIdx, N)
        if bf16:
            want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                            pre["tcbBitMap"], N, as_bits(Qt), as_bits(Kt),
                                            as_bits(Vt), scale, applySoftmax=softmax, dtype=1)
        else:
            want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                            pre["tcbBitMap"], N, Qt.numpy(), Kt.numpy(),
                                            Vt.numpy(), scale, applySoftmax=softmax)
        rwo = torch.as_tensor(pre["rowWindowOffset"].astype(np.int32)).to(dev)
        atox = torch.as_tensor(pre["sparseAToXidx"].astype(np.int32)).to(dev)
        bm = torch.as_tensor(pre["tcbBitMap"].view(np.int64)).to(dev).view(torch.uint64)
        od = torch.as_tensor(pre["sortedRowWindows"].astype(np.int32)).to(dev) if it & 1 else None
        got = capi.attention(rwo, od, atox, bm, N, Qt.to(dev), Kt.to(dev), Vt.to(dev), scale,
                             softmax).cpu().numpy()
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() < MAX_ABS * (1.0 if softmax else max(1.0, np.abs(want).max()))
        assert mean_rel(got, want) < MEAN_REL


def test_windows_beyond_the_stated_block_total_are_left_empty(oracle_mod):
    """A caller that states fewer TC blocks than rowWindowOffset ends with (for instance the arrays
    of another preprocessing run): windows whose block range ends beyond the stated total are
    treated as empty (rows of zeros) instead of being followed; the others are computed as usual.
    The arrays passed here are views of the full ones, so every address stays valid either way."""
    print("case stated block total", flush=True)
    from fused3s_amd import capi
    rng = np.random.default_rng(21)
    N, d = 4000, 64
    rowPtr, colIdx = random_csr(rng, N, 30)
    Q, K, V = feats(rng, N, d)
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    full = gpu_attention(pre, N, Q, K, V, 8.0)
    rwo = pre["rowWindowOffset"]
    keep = int(np.searchsorted(rwo, rwo[-1] // 2, side="right")) - 1  # windows wholly in the first half
    stated = int(rwo[keep])
    dev = "cuda"
    atox = torch.as_tensor(pre["sparseAToXidx"].astype(np.int32)).to(dev)[: stated * 16]
    bm = torch.as_tensor(pre["tcbBitMap"].view(np.int64)).to(dev).view(torch.uint64)[: stated * 4]
    for order in (None, pre["sortedRowWindows"]):
        od = None if order is None else torch.as_tensor(np.asarray(order, np.int32)).to(dev)
        out = capi.attention(torch.as_tensor(rwo.astype(np.int32)).to(dev), od, atox, bm, N,
                             torch.as_tensor(Q).to(dev), torch.as_tensor(K).to(dev),
                             torch.as_tensor(V).to(dev), 8.0)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert np.array_equal(got[: keep * 16], full[: keep * 16])
        assert not got[keep * 16:].any()


@pytest.mark.parametrize("d", [32, 64, 128])
def test_window_kernel_with_a_cursor_gives_the_same_rows(monkeypatch, d):
    """The workgroup-per-window kernel as a resident grid that draws windows from a device-wide
    cursor (F3S_WINDOW_PERSISTENT=1) against its launch-ordered form: the same arithmetic per
    window, so bit-identical rows; three calls in a row (the cursor is put back by the kernel),
    with and without an order, on more windows than workgroups fit the GPU (4 000)."""
    print("case window cursor d=%d" % d, flush=True)
    import oracle
    oracle.build()
    rng = np.random.default_rng(d)
    N = 64_000
    rowPtr, colIdx = random_csr(rng, N, 6, hub=997, empty_frac=0.02)
    Q, K, V = feats(rng, N, d)
    pre = oracle.preprocess(rowPtr, colIdx, N)
    order = pre["sortedRowWindows"]
    for od in (order, None, order):
        monkeypatch.setenv("F3S_WINDOW_PERSISTENT", "0")
        want = gpu_attention(pre, N, Q, K, V, 8.0, od)
        monkeypatch.setenv("F3S_WINDOW_PERSISTENT", "1")
        got = gpu_attention(pre, N, Q, K, V, 8.0, od)
        assert np.isfinite(want).all() and np.array_equal(got, want)


@pytest.mark.parametrize("d", [32, 64])
def test_column_sliced_schedule_matches_oracle_and_window_kernel(oracle_mod, d):
    """The column-sliced schedule on a dense power-law graph (>= 2048 windows, >= 64 TC blocks per
    window): its result must match the reference-emulating oracle within the tolerance and the
    workgroup-per-window kernel closely, for both window orders and without softmax."""
    print("case sliced d=%d" % d, flush=True)
    from fused3s_amd import synth
    rp, ci = synth.make_graph("cfg3_chunglu_233k", scale=0.145)   # N = 33 779: N % 16 != 0
    N = rp.numel() - 1
    assert N % 16 != 0
    rowPtr, colIdx = rp.numpy(), ci.numpy()
    rng = np.random.default_rng(d)
    Q, K, V = feats(rng, N, d)
    scale = float(np.sqrt(d))
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    nRW = (N + 15) // 16
    assert nRW >= 2048 and pre["blockCount"] >= 64 * nRW
    from fused3s_amd import capi
    if os.environ.get("F3S_SCHEDULE") != "window":
        assert capi.lib().f3s_attention_uses_workspace(N, int(pre["blockCount"]), d, 0) == 1
    assert capi.lib().f3s_attention_uses_workspace(300, 2000, d, 0) == (
        1 if os.environ.get("F3S_SCHEDULE") == "sliced" else 0)  # too few windows
    assert capi.lib().f3s_attention_uses_workspace(N, int(pre["blockCount"]), 48, 0) == 0  # bad d
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                    pre["tcbBitMap"], N, Q, K, V, scale)
    plain = gpu_attention(pre, N, Q, K, V, scale, pre["sortedRowWindows"])
    for order in (pre["sortedRowWindows"], None):
        got = gpu_attention(pre, N, Q, K, V, scale, order, sliced=True)
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() < MAX_ABS
        assert mean_rel(got, want) < MEAN_REL
        assert np.abs(got - plain).max() < 2e-3
    want_n = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                      pre["tcbBitMap"], N, Q, K, V, 1.0, applySoftmax=False)
    got_n = gpu_attention(pre, N, Q, K, V, 1.0, pre["sortedRowWindows"], softmax=False, sliced=True)
    assert np.abs(got_n - want_n).max() < 2e-2 * max(1.0, np.abs(want_n).max())
    # bf16 inputs through the same schedule, same bar
    as_bits = lambda t: t.view(torch.int16).numpy().view(np.uint16)
    Qb, Kb, Vb = (torch.as_tensor(x.astype(np.float32)).to(torch.bfloat16) for x in (Q, K, V))
    want_b = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                      pre["tcbBitMap"], N, as_bits(Qb), as_bits(Kb), as_bits(Vb),
                                      scale, dtype=1)
    dev = "cuda"
    rwo = torch.as_tensor(pre["rowWindowOffset"].astype(np.int32)).to(dev)
    atox = torch.as_tensor(pre["sparseAToXidx"].astype(np.int32)).to(dev)
    bm = torch.as_tensor(pre["tcbBitMap"].view(np.int64)).to(dev).view(torch.uint64)
    od = torch.as_tensor(pre["sortedRowWindows"].astype(np.int32)).to(dev)
    ws = capi.attention_workspace(N, d, dev, nTCB=int(pre["blockCount"]), dtype=torch.bfloat16)
    assert ws is not None or os.environ.get("F3S_SCHEDULE") == "window"
    got_b = capi.attention(rwo, od, atox, bm, N, Qb.to(dev), Kb.to(dev), Vb.to(dev), scale,
                           workspace=ws).cpu().numpy()
    assert np.abs(got_b - want_b).max() < MAX_ABS
    assert mean_rel(got_b, want_b) < 1e-3


@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("seed,N,deg,hub", [(0, 300, 2, 0), (1, 500, 6, 7), (2, 77, 40, 0),
                                            (3, 16, 1, 0)])
def test_16x8_blocks_match_the_1tb1tcb_oracle(oracle_mod, d, seed, N, deg, hub):
    """f3s_attention_fwd_tcb8 on windows of 1, 2, 3, ... 16x8 blocks (every tail length of the
    four-block pipeline step), in natural and heavy-first order, with and without the SDDMM tap."""
    from fused3s_amd import capi
    print("case tcb8 d=%d seed=%d N=%d" % (d, seed, N), flush=True)
    rng = np.random.default_rng(seed)
    rowPtr, colIdx = random_csr(rng, N, deg, hub=hub, empty_frac=0.1)
    Q, K, V = feats(rng, N, d, std=0.6)
    pre = oracle_mod.preprocess(rowPtr, colIdx, N, 16, 8)
    counts = np.diff(pre["rowWindowOffset"])
    print("blocks per window: min %d max %d" % (counts.min(), counts.max()), flush=True)
    dev = "cuda"
    rwo = torch.as_tensor(pre["rowWindowOffset"].astype(np.int32)).to(dev)
    atox = torch.as_tensor(pre["sparseAToXidx"].astype(np.int32)).to(dev)
    bm = torch.as_tensor(pre["tcbBitMap"].view(np.int64)).to(dev).view(torch.uint64)
    order = torch.as_tensor(pre["sortedRowWindows"].astype(np.int32)).to(dev)
    Qd, Kd, Vd = (torch.as_tensor(x).to(dev) for x in (Q, K, V))
    for softmax in (True, False):
        want, want_s = oracle_mod.attention_tcb8(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                                 pre["tcbBitMap"], N, Q, K, V, softmax,
                                                 save_sddmm=True)
        got, got_s = capi.attention_tcb8(rwo, None, atox, bm, N, Qd, Kd, Vd, softmax,
                                         save_sddmm=True)
        got2 = capi.attention_tcb8(rwo, order, atox, bm, N, Qd, Kd, Vd, softmax)
        torch.cuda.synchronize()
        assert torch.equal(got, got2)
        got, got_s = got.cpu().numpy(), got_s.cpu().numpy()
        assert np.isfinite(got).all()
        if softmax:
            assert np.abs(got - want).max() < MAX_ABS
        assert mean_rel(got, want) < MEAN_REL
        assert np.array_equal(got_s == 0, want_s == 0)
        assert np.abs(got_s - want_s).max() <= 1e-5 * max(1.0, np.abs(want_s).max())
