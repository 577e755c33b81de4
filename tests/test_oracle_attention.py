"""Pins the attention oracles: the textbook one against a dense fp64 masked softmax and closed
forms, the reference-emulating one against the textbook within the stated tolerance plus the
reference's documented quirks."""
import ctypes

import numpy as np
import pytest

from conftest import random_csr
from ref_checks import dense_attention, dense_from_csr

MAX_ABS = 2e-2   # tolerance of the attention output (fp16 in, fp32 accumulate)
MEAN_REL = 1e-3


def mean_rel(a, b):
    return float(np.abs(a - b).mean() / max(np.abs(b).mean(), 1e-30))


def feats(rng, N, d, std=1.0):
    return [(rng.standard_normal((N, d)) * std).astype(np.float16) for _ in range(3)]


def test_half_conversions_match_numpy(oracle_mod):
    L = oracle_mod.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([L.f3s_oracle_half_to_float(int(b)) for b in bits], np.float32)
    ok = (got == want) | (np.isnan(got) & np.isnan(want))
    assert ok.all()
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(5000) * 1e-6).astype(np.float32),
        (rng.standard_normal(2000) * 3e4).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, 2.0 ** -24, 2.0 ** -25,
                  2.0 ** -25 * 1.0001, 2.0 ** -14, 1.00048828125, 1.0009765625 + 2.0 ** -12],
                 np.float32)])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).astype(np.float32)
    got = np.array([L.f3s_oracle_round_to_half(ctypes.c_float(float(x))) for x in xs], np.float32)
    assert np.array_equal(got, want)


def test_bf16_rounding_matches_torch(oracle_mod):
    import torch
    L = oracle_mod.lib()
    rng = np.random.default_rng(1)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(2000) * 1e-20).astype(np.float32),
        # ties and near-ties of the 8-bit mantissa, carry into the exponent
        np.array([0.0, -0.0, 1.0, 1.00390625, 1.005859375, 1.0078125, 1.01171875, 1.99609375,
                  1.998046875, 255.5, 3.0e38, 2.0 ** -126], np.float32)])
    want = torch.from_numpy(xs).to(torch.bfloat16).to(torch.float32).numpy()
    got = np.array([L.f3s_oracle_round_to_bf16(ctypes.c_float(float(x))) for x in xs], np.float32)
    assert np.array_equal(got, want)


def test_bf16_reference_emulation_matches_textbook(oracle_mod):
    """bf16 inputs: same algorithm on the bf16 values with P rounded to fp16 as the reference
    rounds it (src/F3S_kernel.cu:938-945); stays within max-abs 2e-2 / mean-relative 1e-3 of the
    fp64 textbook result, as for fp16 inputs."""
    import torch
    rng = np.random.default_rng(5)
    N, d = 333, 64
    rowPtr, colIdx = random_csr(rng, N, 20, hub=9, empty_frac=0.05)
    g = torch.Generator().manual_seed(5)
    Q, K, V = [torch.randn((N, d), generator=g).to(torch.bfloat16).view(torch.int16).numpy()
               .view(np.uint16) for _ in range(3)]
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    ref = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"], pre["tcbBitMap"],
                                   N, Q, K, V, 8.0, dtype=1)
    txt = oracle_mod.attention_textbook(rowPtr, colIdx, N, Q, K, V, 8.0, dtype=1)
    assert np.abs(ref - txt).max() < MAX_ABS
    assert 1e-6 < mean_rel(ref, txt) < 1e-3  # the fp16 rounding of P is visible, and bounded


@pytest.mark.parametrize("seed,N,d,deg,dup,unsorted", [
    (0, 40, 32, 5, False, False), (1, 97, 64, 12, True, True), (2, 150, 128, 3, False, True)])
def test_textbook_matches_dense_fp64(oracle_mod, seed, N, d, deg, dup, unsorted):
    rng = np.random.default_rng(seed)
    rowPtr, colIdx = random_csr(rng, N, deg, dup=dup, unsorted=unsorted, empty_frac=0.1)
    Q, K, V = feats(rng, N, d)
    scale = float(np.sqrt(d))
    got = oracle_mod.attention_textbook(rowPtr, colIdx, N, Q, K, V, scale)
    want = dense_attention(rowPtr, colIdx, N, Q, K, V, scale)
    assert np.abs(got - want).max() < 1e-5


def test_closed_forms(oracle_mod):
    rng = np.random.default_rng(7)
    N, d = 48, 64
    Q, K, V = feats(rng, N, d)
    # degree-1 rows copy one V row; row 5 is empty; rows 40.. see identical keys -> plain mean
    rows = []
    for r in range(N):
        if r == 5:
            rows.append([])
        elif r < 40:
            rows.append([(7 * r + 3) % N])
        else:
            rows.append([1, 2, 3, 4])
    K[2] = K[1]
    K[3] = K[1]
    K[4] = K[1]
    rowPtr = np.zeros(N + 1, np.int32)
    rowPtr[1:] = np.cumsum([len(x) for x in rows])
    colIdx = np.array([c for x in rows for c in x], np.int32)
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    for out in (oracle_mod.attention_textbook(rowPtr, colIdx, N, Q, K, V, 8.0),
                oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                         pre["tcbBitMap"], N, Q, K, V, 8.0)):
        for r in range(40):
            if r == 5:
                assert np.all(out[r] == 0)
            else:
                assert np.abs(out[r] - V[(7 * r + 3) % N].astype(np.float32)).max() < 2e-3
        mean = V[1:5].astype(np.float64).mean(axis=0)
        for r in range(40, N):
            assert np.abs(out[r] - mean).max() < 2e-3


@pytest.mark.parametrize("nwarp", [2, 8, 16])
@pytest.mark.parametrize("seed,N,d,deg", [(0, 300, 64, 25), (1, 1000, 128, 100), (2, 77, 32, 6)])
def test_reference_numerics_agree_with_textbook_within_tolerance(oracle_mod, seed, N, d, deg, nwarp):
    rng = np.random.default_rng(seed)
    rowPtr, colIdx = random_csr(rng, N, deg, hub=13)
    Q, K, V = feats(rng, N, d)
    scale = float(np.sqrt(d))
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    ref = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"], pre["tcbBitMap"],
                                   N, Q, K, V, scale, nWarpPerBlock=nwarp)
    txt = oracle_mod.attention_textbook(rowPtr, colIdx, N, Q, K, V, scale)
    assert np.abs(ref - txt).max() < MAX_ABS
    assert mean_rel(ref, txt) < MEAN_REL


def test_reference_accuracy_harness_shape(oracle_mod):
    """The reference's own check (scripts/tests/test_f3s_accuracy.py:96-236): 1000 nodes, 10 %
    dense mask, d=128, uniform [0,1) features, no scaling; it prints the relative Frobenius
    error and expects it to be small."""
    rng = np.random.default_rng(0)
    N, d = 1000, 128
    A = rng.random((N, N)) < 0.1
    rowPtr = np.zeros(N + 1, np.int32)
    rowPtr[1:] = np.cumsum(A.sum(axis=1))
    colIdx = np.nonzero(A)[1].astype(np.int32)
    Q, K, V = [rng.random((N, d)).astype(np.float16) for _ in range(3)]
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    ref = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"], pre["tcbBitMap"],
                                   N, Q, K, V, 1.0)
    want = dense_attention(rowPtr, colIdx, N, Q, K, V, 1.0)
    rel_fro = np.linalg.norm(ref - want) / np.linalg.norm(want)
    assert rel_fro < 2e-3


def test_reference_quirks(oracle_mod):
    rng = np.random.default_rng(3)
    N, d = 32, 64
    Q, K, V = feats(rng, N, d)
    rowPtr, colIdx = random_csr(rng, N, 6)
    Q[3] = 0  # every score of row 3 is exactly 0.0 -> treated as masked -> l == 0 -> output 0
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    args = (pre["rowWindowOffset"], pre["sparseAToXidx"], pre["tcbBitMap"], N, Q, K, V)
    ref = oracle_mod.attention_ref(*args, 8.0)
    txt = oracle_mod.attention_textbook(rowPtr, colIdx, N, Q, K, V, 8.0)
    if rowPtr[4] > rowPtr[3]:
        assert np.all(ref[3] == 0) and np.abs(txt[3]).max() > 0
    others = [r for r in range(N) if r != 3]
    assert np.abs(ref[others] - txt[others]).max() < MAX_ABS
    # running max starts at 0: scores far below zero underflow in fp16 and are lost
    Qn = Q.copy()
    Qn[7] = 60.0
    Kn = K.copy()
    Kn[:] = -1.0
    low = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"], pre["tcbBitMap"],
                                   N, Qn, Kn, V, 1.0)
    if rowPtr[8] > rowPtr[7]:
        assert np.all(low[7] == 0)  # exp(-3840) == 0


def test_sddmm_spmm_without_softmax(oracle_mod):
    rng = np.random.default_rng(5)
    N, d = 90, 64
    rowPtr, colIdx = random_csr(rng, N, 8)
    Q, K, V = feats(rng, N, d, std=0.5)
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    got = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"], pre["tcbBitMap"],
                                   N, Q, K, V, 1.0, applySoftmax=False)
    A = dense_from_csr(rowPtr, colIdx, N) > 0
    S = (Q.astype(np.float64) @ K.astype(np.float64).T) * A
    want = S.astype(np.float16).astype(np.float64) @ V.astype(np.float64)
    assert np.abs(got - want).max() < 5e-3 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("seed,N,d,deg", [(0, 100, 32, 7), (1, 333, 64, 30), (2, 50, 128, 3)])
def test_tcb8_oracle_pinned_by_the_16x16_one_and_by_dense_scores(oracle_mod, seed, N, d, deg):
    """The 16x8 kernel walks the same ascending column list two blocks (16 columns) at a time, so
    it must reproduce the 16x16 oracle run with one block per chunk (nWarpPerBlock=2) bit for bit;
    its SDDMM tap must equal the dense Q K^T sampled at the edges, block by block."""
    rng = np.random.default_rng(seed)
    rowPtr, colIdx = random_csr(rng, N, deg, hub=5, empty_frac=0.1)
    Q, K, V = feats(rng, N, d, std=0.5)
    p16 = oracle_mod.preprocess(rowPtr, colIdx, N, 16, 16)
    p8 = oracle_mod.preprocess(rowPtr, colIdx, N, 16, 8)
    for softmax in (True, False):
        want = oracle_mod.attention_ref(p16["rowWindowOffset"], p16["sparseAToXidx"],
                                        p16["tcbBitMap"], N, Q, K, V, 1.0, nWarpPerBlock=2,
                                        applySoftmax=softmax)
        got, sddmm = oracle_mod.attention_tcb8(p8["rowWindowOffset"], p8["sparseAToXidx"],
                                               p8["tcbBitMap"], N, Q, K, V, softmax,
                                               save_sddmm=True)
        assert np.array_equal(got, want)
    txt = oracle_mod.attention_textbook(rowPtr, colIdx, N, Q, K, V, 1.0)
    got = oracle_mod.attention_tcb8(p8["rowWindowOffset"], p8["sparseAToXidx"], p8["tcbBitMap"], N,
                                    Q, K, V, True)
    assert np.abs(got - txt).max() < MAX_ABS and mean_rel(got, txt) < MEAN_REL
    # SDDMM tap: block t of window w, row r, slot j  <->  A[16w + r, sparseAToXidx[8t + j]]
    A = dense_from_csr(rowPtr, colIdx, N)
    S = Q.astype(np.float64) @ K.astype(np.float64).T
    rwo = p8["rowWindowOffset"]
    nT = int(rwo[-1])
    assert sddmm.shape == (nT * 128,)
    blocks = sddmm.reshape(nT, 16, 8)
    seen = 0
    for w in range(len(rwo) - 1):
        rows = range(16 * w, min(16 * w + 16, N))
        n_cols = len(np.unique(np.concatenate([colIdx[rowPtr[r]:rowPtr[r + 1]] for r in rows])))
        for t in range(rwo[w], rwo[w + 1]):
            cols = p8["sparseAToXidx"][8 * t:8 * t + 8]
            for j in range(8):
                padding = (t - rwo[w]) * 8 + j >= n_cols  # zero-filled slot, carries no bit
                for r in range(16):
                    row = 16 * w + r
                    if not padding and row < N and A[row, cols[j]] != 0:
                        assert blocks[t, r, j] == np.float32(S[row, cols[j]])
                        seen += 1
                    else:
                        assert blocks[t, r, j] == 0.0
    assert seen == int((A != 0).sum())
