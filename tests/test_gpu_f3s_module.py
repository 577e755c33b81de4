"""The `F3S` operator module used the way the reference's callers use it
(scripts/tests/test_f3s_accuracy.py:96-236, scripts/baseline_comp/baseline_comp_kernel_only.py:
412-497): preprocess_gpu on CSR, then each fused entry point, checked against the oracles."""
import os

import numpy as np
import pytest
import torch

from ref_checks import compare_preprocess, dense_attention

pytestmark = pytest.mark.gpu
MAX_ABS = 2e-2
MEAN_REL = 1e-3


def reference_style_inputs(N=1000, d=128, density=0.1, seed=0):
    rng = np.random.default_rng(seed)
    A = rng.random((N, N)) < density
    rowPtr = np.zeros(N + 1, np.int32)
    rowPtr[1:] = np.cumsum(A.sum(axis=1))
    colIdx = np.nonzero(A)[1].astype(np.int32)
    Q, K, V = [rng.random((N, d)).astype(np.float16) for _ in range(3)]
    return rowPtr, colIdx, Q, K, V


def preprocess_like_the_reference(F3S, rowPtr, colIdx, N, W=16):
    dev = "cuda"
    nRW = (N + 15) // 16
    blockPartition = torch.zeros(nRW, dtype=torch.int32, device=dev)
    edgeToColumn = torch.zeros(len(colIdx), dtype=torch.int32, device=dev)
    edgeToRow = torch.zeros(len(colIdx), dtype=torch.int32, device=dev)
    res = F3S.preprocess_gpu(torch.as_tensor(colIdx).to(dev), torch.as_tensor(rowPtr).to(dev), N,
                             16, W, blockPartition, edgeToColumn, edgeToRow)
    return res, blockPartition, edgeToColumn, edgeToRow


def test_reference_call_sequence_all_variants(oracle_mod, tmp_path, monkeypatch):
    print("case module_all_variants", flush=True)
    from fused3s_amd import F3S
    monkeypatch.chdir(tmp_path)
    N, d = 1000, 128
    rowPtr, colIdx, Q, K, V = reference_style_inputs(N, d)
    res, blockPartition, edgeToColumn, edgeToRow = preprocess_like_the_reference(
        F3S, rowPtr, colIdx, N)
    rwo, order, rowid, tile, toff, atox, bm, count = res
    assert isinstance(count, int) and count == atox.numel() // 16
    want = oracle_mod.preprocess(rowPtr, colIdx, N)
    got = dict(rowWindowOffset=rwo, sortedRowWindows=order, tcblockRowid=rowid,
               tcblocktileId=tile, tcblockOffset=toff, sparseAToXidx=atox, blockCount=count,
               tcbBitMap=bm.cpu().view(torch.int64).numpy().view(np.uint64),
               blockPartition=blockPartition, edgeToColumn=edgeToColumn, edgeToRow=edgeToRow)
    got = {k: (v.cpu().numpy() if torch.is_tensor(v) else v) for k, v in got.items()}
    compare_preprocess(got, want)

    Qd, Kd, Vd = (torch.as_tensor(x).cuda() for x in (Q, K, V))
    true = dense_attention(rowPtr, colIdx, N, Q, K, V, 1.0)
    ref = oracle_mod.attention_ref(want["rowWindowOffset"], want["sparseAToXidx"],
                                   want["tcbBitMap"], N, Q, K, V, 1.0)
    outs = {
        "f3s_1tb1rw": F3S.f3s_1tb1rw(rwo, atox, bm, N, Qd, Kd, Vd, 8, True, False),
        "f3s_1tb1rw_scheduled": F3S.f3s_1tb1rw_scheduled(rwo, order, atox, bm, N, Qd, Kd, Vd, 8,
                                                         False),
        "f3s_1tb1rw_scheduled_permuteV": F3S.f3s_1tb1rw_scheduled_permuteV(rwo, order, atox, bm,
                                                                           N, Qd, Kd, Vd, 8),
        "scaleQK_1.0": F3S.f3s_1tb1rw_scheduled_permuteV_scaleQK(rwo, order, atox, bm, N, Qd, Kd,
                                                                 Vd, 1.0, 8),
    }
    for name, r in outs.items():
        time_ms, out, sddmm = r
        assert time_ms.dim() == 0 and time_ms.device.type == "cpu" and float(time_ms) > 0
        assert out.shape == (N, d) and out.dtype == torch.float32 and out.is_cuda
        assert sddmm.numel() == 0
        o = out.cpu().numpy()
        # the reference's own figure of merit: relative Frobenius error against dense fp32/64
        assert np.linalg.norm(o - true) / np.linalg.norm(true) < 2e-3, name
        assert np.abs(o - ref).max() < MAX_ABS, name

    # scaled variant: scores divided by scalingFactor
    scale = float(np.sqrt(d))
    r = F3S.f3s_1tb1rw_scheduled_permuteV_scaleQK(rwo, order, atox, bm, N, Qd, Kd, Vd, scale, 8)
    want_s = oracle_mod.attention_ref(want["rowWindowOffset"], want["sparseAToXidx"],
                                      want["tcbBitMap"], N, Q, K, V, scale)
    o = r[1].cpu().numpy()
    assert np.abs(o - want_s).max() < MAX_ABS
    assert np.abs(o - want_s).mean() / np.abs(want_s).mean() < MEAN_REL

    # SDDMM -> SpMM without softmax
    r = F3S.f3s_1tb1rw(rwo, atox, bm, N, Qd, Kd, Vd, 8, False, False)
    want_n = oracle_mod.attention_ref(want["rowWindowOffset"], want["sparseAToXidx"],
                                      want["tcbBitMap"], N, Q, K, V, 1.0, applySoftmax=False)
    o = r[1].cpu().numpy()
    assert np.abs(o - want_n).max() < 2e-2 * np.abs(want_n).max()

    # per-CU active time files of the timed variants (reference: one "begin end" line per SM)
    # the timed launches compute the same attention (src/F3S_kernel.cu:1178-1368, 1803-1997)
    timed = [F3S.f3s_1tb1rw(rwo, atox, bm, N, Qd, Kd, Vd, 8, True, True),
             F3S.f3s_1tb1rw_scheduled(rwo, order, atox, bm, N, Qd, Kd, Vd, 8, True)]
    for r in timed:
        o = r[1].cpu().numpy()
        assert np.abs(o - ref).max() < MAX_ABS
        assert np.abs(o - ref).mean() / np.abs(ref).mean() < MEAN_REL
    for fn in ("SM_time_f3s1tb1rw.csv", "SM_time_f3s1tb1rw_scheduled.csv"):
        lines = open(os.path.join(tmp_path, fn)).read().split("\n")
        rows = [l.split() for l in lines if l.strip()]
        assert 1 <= len(rows) <= 256
        for b, e in rows:
            assert float(e) >= float(b) > 0


@pytest.mark.parametrize("W", [16, 8])
def test_preprocess_gpu_both_allocation_styles(oracle_mod, monkeypatch, W):
    """F3S.preprocess_gpu with views of bounded allocations (default) and with the reference's
    count / allocate / fill sequence (F3S_PREPROCESS=two_phase): the same tuples, bit for bit, on a
    graph of long windows and on one of short windows; the default's tensors are contiguous views
    whose sizes are the exact ones."""
    from fused3s_amd import F3S
    from test_gpu_preprocess import long_window_graph
    rng = np.random.default_rng(5)
    graphs = [long_window_graph(rng, 2000, 180, messy_every=60, empty_every=13)]
    rp, ci, _, _, _ = reference_style_inputs(1000, 32)
    graphs.append((rp, ci))
    # the sixteen rows of a window name the same 64 columns: a sixteenth of the blocks that the
    # bound allows, so the default style hands out exact-size copies, not views
    shared = np.concatenate([np.tile(np.sort(rng.choice(1600, 64, replace=False)), 16)
                             for _ in range(100)]).astype(np.int32)
    graphs.append((np.arange(0, 1600 * 64 + 1, 64, dtype=np.int32), shared))
    for rowPtr, colIdx in graphs:
        N = len(rowPtr) - 1
        print("case module allocation styles N=%d E=%d W=%d" % (N, len(colIdx), W), flush=True)
        want = oracle_mod.preprocess(rowPtr, colIdx, N, 16, W)
        results = []
        for style in ("", "two_phase"):
            monkeypatch.setenv("F3S_PREPROCESS", style)
            res, bp, e2c, e2r = preprocess_like_the_reference(F3S, rowPtr, colIdx, N, W)
            rwo, order, rowid, tile, toff, atox, bm, count = res
            assert count == want["blockCount"]
            assert rowid.numel() == count and toff.numel() == count + 1
            assert atox.numel() == count * W and bm.numel() == count * 16 * W // 64
            assert all(t.is_contiguous() for t in (rowid, toff, atox, bm, tile))
            bound = (len(colIdx) + W - 1) // W + (N + 15) // 16
            if count * 2 < bound:  # no tensor keeps the bounded allocation alive
                assert atox.untyped_storage().nbytes() == atox.numel() * 4
                assert bm.untyped_storage().nbytes() == bm.numel() * 8
            got = dict(rowWindowOffset=rwo, sortedRowWindows=order, tcblockRowid=rowid,
                       tcblocktileId=tile, tcblockOffset=toff, sparseAToXidx=atox,
                       blockCount=count,
                       tcbBitMap=bm.cpu().view(torch.int64).numpy().view(np.uint64),
                       blockPartition=bp, edgeToColumn=e2c, edgeToRow=e2r)
            got = {k: (v.cpu().numpy() if torch.is_tensor(v) else v) for k, v in got.items()}
            compare_preprocess(got, want)
            results.append(got)


def test_module_argument_checks_on_device():
    print("case module_arg_checks", flush=True)
    from fused3s_amd import F3S
    N, d = 64, 64
    rwo = torch.zeros(5, dtype=torch.int32, device="cuda")
    atox = torch.zeros(16, dtype=torch.int32, device="cuda")
    bm = torch.zeros(4, dtype=torch.uint64, device="cuda")
    Q = torch.zeros(N, d, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="contiguous"):
        F3S.f3s_1tb1rw(rwo, atox, bm, N, Q.t().contiguous().t(), Q, Q, 8, True, False)
    with pytest.raises(RuntimeError, match="float16"):
        F3S.f3s_1tb1rw(rwo, atox, bm, N, Q.float(), Q.float(), Q.float(), 8, True, False)
    with pytest.raises(RuntimeError, match="nWarpPerBlock"):
        F3S.f3s_1tb1rw(rwo, atox, bm, N, Q, Q, Q, 3, True, False)
    Qbad = torch.zeros(N, 48, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="head dim"):
        F3S.f3s_1tb1rw(rwo, atox, bm, N, Qbad, Qbad, Qbad, 8, True, False)
    with pytest.raises(RuntimeError, match="two words per 16x8 block"):
        # 16 column ids are two 16x8 blocks, which need four bitmap words
        F3S.f3s_1tb1tcb(rwo, atox, bm[:2].contiguous(), N, Q, Q, Q, True, False)
    with pytest.raises(RuntimeError, match="float16"):
        F3S.f3s_1tb1tcb(rwo, atox, bm, N, Q.float(), Q.float(), Q.float(), True, False)
    # all-empty graph: every output row is zero
    out = F3S.f3s_1tb1rw(rwo, atox, bm, N, Q, Q, Q, 8, True, False)[1]
    assert float(out.abs().max()) == 0.0


def test_multihead_entry_of_the_module(oracle_mod):
    """F3S.f3s_multihead_scaleQK (bf16, [N, heads, d]) against the per-head loop the reference's
    callers write with f3s_1tb1rw_scheduled_permuteV_scaleQK, and against the textbook oracle."""
    print("case module_multihead", flush=True)
    from fused3s_amd import F3S
    N, heads, d = 1500, 8, 32
    rowPtr, colIdx, _, _, _ = reference_style_inputs(N, d, density=0.03, seed=3)
    res, _, _, _ = preprocess_like_the_reference(F3S, rowPtr, colIdx, N)
    rwo, order, _, _, _, atox, bitmap, _ = res
    g = torch.Generator().manual_seed(3)
    Q, K, V = [(torch.randn((N, heads, d), generator=g) * d ** -0.5).to(torch.bfloat16).cuda()
               for _ in range(3)]
    scale = float(np.sqrt(d))
    t, out, extra = F3S.f3s_multihead_scaleQK(rwo, order, atox, bitmap, N, Q, K, V, scale)
    assert t.device.type == "cpu" and t.dim() == 0 and float(t) > 0
    assert out.shape == (N, heads * d) and out.dtype == torch.float32 and extra.numel() == 0
    for h in range(heads):
        qh, kh, vh = (x[:, h].contiguous() for x in (Q, K, V))
        _, single, _ = F3S.f3s_1tb1rw_scheduled_permuteV_scaleQK(rwo, order, atox, bitmap, N, qh,
                                                                 kh, vh, scale, 8)
        assert torch.equal(out[:, h * d:(h + 1) * d], single)
        as_bits = lambda x: x.cpu().view(torch.int16).numpy().view(np.uint16)
        txt = oracle_mod.attention_textbook(rowPtr, colIdx, N, as_bits(qh), as_bits(kh),
                                            as_bits(vh), scale, dtype=1)
        assert np.abs(single.cpu().numpy() - txt).max() < MAX_ABS
    with pytest.raises(RuntimeError, match="identical shapes"):
        F3S.f3s_multihead_scaleQK(rwo, order, atox, bitmap, N, Q, K[:, :4], V, scale)
    with pytest.raises(RuntimeError, match="float16 or all bfloat16"):
        F3S.f3s_multihead_scaleQK(rwo, order, atox, bitmap, N, Q.float(), K.float(), V.float(),
                                  scale)


@pytest.mark.parametrize("d", [32, 64, 128])
def test_1tb1tcb_call_sequence(oracle_mod, d):
    """F3S.f3s_1tb1tcb the way scripts/tests/test_f3s_accuracy.py:96-146 drives it:
    preprocess_gpu with 16x8 blocks, softmax on / off, SDDMM tap checked block by block."""
    print("case module_1tb1tcb d=%d" % d, flush=True)
    from fused3s_amd import F3S
    N = 1000
    rowPtr, colIdx, Q, K, V = reference_style_inputs(N, d, density=0.05, seed=d)
    want_pre = oracle_mod.preprocess(rowPtr, colIdx, N, 16, 8)
    res, bp, e2c, e2r = preprocess_like_the_reference(F3S, rowPtr, colIdx, N, W=8)
    rwo, order, rowid, tile, toff, atox, bitmap, nT = res
    got_pre = dict(rowWindowOffset=rwo, sortedRowWindows=order, tcblockRowid=rowid,
                   tcblocktileId=tile, tcblockOffset=toff, sparseAToXidx=atox, blockCount=nT,
                   tcbBitMap=bitmap.cpu().view(torch.int64).numpy().view(np.uint64),
                   blockPartition=bp, edgeToColumn=e2c, edgeToRow=e2r)
    got_pre = {k: (v.cpu().numpy() if torch.is_tensor(v) else v) for k, v in got_pre.items()}
    compare_preprocess(got_pre, want_pre)
    Qd, Kd, Vd = (torch.as_tensor(x).cuda() for x in (Q, K, V))
    for softmax in (True, False):
        want, want_s = oracle_mod.attention_tcb8(want_pre["rowWindowOffset"],
                                                 want_pre["sparseAToXidx"], want_pre["tcbBitMap"],
                                                 N, Q, K, V, softmax, save_sddmm=True)
        t, out, sddmm = F3S.f3s_1tb1tcb(rwo, atox, bitmap, N, Qd, Kd, Vd, softmax, True)
        assert t.device.type == "cpu" and float(t) > 0
        assert out.shape == (N, d) and sddmm.shape == (nT * 128,)
        got = out.cpu().numpy()
        if softmax:
            assert np.abs(got - want).max() < MAX_ABS
            assert np.abs(got - want).mean() / np.abs(want).mean() < MEAN_REL
        else:
            # no normalisation: outputs are sums of fp16(S) * V with |S| ~ d/4; relative bar only
            assert np.abs(got - want).mean() / np.abs(want).mean() < MEAN_REL
        # scores: fp32 MFMA accumulation of exact fp16 products against a double-precision sum
        got_s = sddmm.cpu().numpy()
        assert np.array_equal(got_s == 0, want_s == 0)
        assert np.abs(got_s - want_s).max() <= 1e-5 * max(1.0, np.abs(want_s).max())
        t2, out2, empty = F3S.f3s_1tb1tcb(rwo, atox, bitmap, N, Qd, Kd, Vd, softmax, False)
        assert empty.numel() == 0 and torch.equal(out2, out)
