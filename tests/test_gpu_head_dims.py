"""Head dimensions beyond 32 / 64 / 128: every multiple of 32 up to 256 through every attention
entry point (the reference takes embeddingDim at run time: src/F3S_kernel.cu:601-604 sizes its
shared memory from it, :1424 loops over its k-steps and :1522 over its output tiles).

Tolerance as everywhere: max-abs 2e-2 and mean-relative 1e-3 against the reference-emulating
oracle (fp16 inputs, fp32 accumulation; bf16 inputs against the oracle that rounds P to fp16).
"""
import numpy as np
import pytest
import torch

from conftest import random_csr

pytestmark = pytest.mark.gpu
MAX_ABS = 2e-2
MEAN_REL = 1e-3
NEW_DIMS = [96, 160, 192, 224, 256]


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


def features(seed, N, heads, d, dtype):
    g = torch.Generator().manual_seed(seed)
    std = 1.0 if dtype == torch.float16 else d ** -0.25
    return [(torch.randn((N, heads, d), generator=g) * std).to(dtype) for _ in range(3)]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d", NEW_DIMS)
def test_single_head_entry(oracle_mod, d, dtype):
    """f3s_attention_fwd: both window orders, scaled softmax and no softmax, a graph with hub
    rows, empty rows and N % 16 != 0."""
    from fused3s_amd import capi
    print("case head_dim single d=%d %s" % (d, dtype), flush=True)
    N = 1003
    rng = np.random.default_rng(d)
    rowPtr, colIdx = random_csr(rng, N, 40, hub=97, empty_frac=0.05)
    Q, K, V = (t[:, 0].contiguous() for t in features(d, N, 1, d, dtype))
    scale = float(np.sqrt(d))
    code = 0 if dtype == torch.float16 else 1
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                    pre["tcbBitMap"], N, bits(Q), bits(K), bits(V), scale,
                                    dtype=code)
    txt = oracle_mod.attention_textbook(rowPtr, colIdx, N, bits(Q), bits(K), bits(V), scale,
                                        dtype=code)
    rwo, order, atox, bm = to_dev(pre)
    for od in (None, order):
        got = capi.attention(rwo, od, atox, bm, N, Q.cuda(), K.cuda(), V.cuda(), scale)
        torch.cuda.synchronize()
        got = got.cpu().numpy()
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() < MAX_ABS
        assert mean_rel(got, want) < MEAN_REL
        assert np.abs(got - txt).max() < MAX_ABS
    want_n = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                      pre["tcbBitMap"], N, bits(Q), bits(K), bits(V), 1.0,
                                      applySoftmax=False, dtype=code)
    got_n = capi.attention(rwo, order, atox, bm, N, Q.cuda(), K.cuda(), V.cuda(), 1.0,
                           False).cpu().numpy()
    assert np.abs(got_n - want_n).max() < MAX_ABS * max(1.0, np.abs(want_n).max())
    assert mean_rel(got_n, want_n) < MEAN_REL


@pytest.mark.parametrize("d", NEW_DIMS)
def test_heads_entry_and_short_window_split(oracle_mod, d):
    """f3s_attention_fwd_heads on pitched [N, 2, d] inputs: bit-identical to per-head launches.
    The graph has more than 1024 windows of a few blocks each, so with an order the call is split
    into the wave-per-window kernel and the workgroup-per-window kernel."""
    from fused3s_amd import capi
    print("case head_dim heads d=%d" % d, flush=True)
    N, heads, pad = 20_000, 2, 8
    rng = np.random.default_rng(100 + d)
    rowPtr, colIdx = random_csr(rng, N, 4, hub=1999, empty_frac=0.02)
    dtype = torch.bfloat16 if d % 64 == 0 else torch.float16
    Q, K, V = features(d, N, heads, d, dtype)
    scale = float(np.sqrt(d))
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    nRW = (N + 15) // 16
    assert nRW >= 1024 and pre["blockCount"] < 16 * nRW  # the split is taken
    rwo, order, atox, bm = to_dev(pre)

    def pitched(t):
        store = torch.zeros((N, heads * d + pad), dtype=dtype, device="cuda")
        store[:, :heads * d] = t.reshape(N, heads * d).cuda()
        return store[:, :heads * d].unflatten(1, (heads, d))

    Qd, Kd, Vd = pitched(Q), pitched(K), pitched(V)
    got = capi.attention_heads(rwo, order, atox, bm, N, Qd, Kd, Vd, scale).cpu().numpy()
    nat = capi.attention_heads(rwo, None, atox, bm, N, Qd, Kd, Vd, scale).cpu().numpy()
    assert np.abs(got - nat).max() < 2e-3  # no split without an order: another summation order
    for h in range(heads):
        qh, kh, vh = (t[:, h].contiguous() for t in (Q, K, V))
        single = capi.attention(rwo, order, atox, bm, N, qh.cuda(), kh.cuda(), vh.cuda(),
                                scale).cpu().numpy()
        assert np.array_equal(got[:, h * d:(h + 1) * d], single), "head %d" % h
        want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                        pre["tcbBitMap"], N, bits(qh), bits(kh), bits(vh), scale,
                                        dtype=0 if dtype == torch.float16 else 1)
        assert np.abs(single - want).max() < MAX_ABS
        assert mean_rel(single, want) < MEAN_REL


@pytest.mark.parametrize("persistent", ["0", "1"])
@pytest.mark.parametrize("d", [96, 160, 256])
def test_column_sliced_schedule(oracle_mod, monkeypatch, d, persistent):
    """The column-sliced schedule (forced: the graph is far smaller than those the library picks it
    for) in its launch-order and its resident form, against the oracle and the window kernel."""
    from fused3s_amd import capi
    print("case head_dim sliced d=%d persistent=%s" % (d, persistent), flush=True)
    monkeypatch.setenv("F3S_SCHEDULE", "sliced")
    monkeypatch.setenv("F3S_SLICED_PERSISTENT", persistent)
    N = 2500
    rng = np.random.default_rng(200 + d)
    rowPtr, colIdx = random_csr(rng, N, 120, hub=211)
    Q, K, V = (t[:, 0].contiguous() for t in features(d, N, 1, d, torch.float16))
    scale = float(np.sqrt(d))
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                    pre["tcbBitMap"], N, bits(Q), bits(K), bits(V), scale)
    rwo, order, atox, bm = to_dev(pre)
    ws = capi.attention_workspace(N, d, "cuda", nTCB=int(pre["blockCount"]))
    assert ws is not None
    for od in (order, None):
        got = capi.attention(rwo, od, atox, bm, N, Q.cuda(), K.cuda(), V.cuda(), scale,
                             workspace=ws).cpu().numpy()
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() < MAX_ABS
        assert mean_rel(got, want) < MEAN_REL
    monkeypatch.setenv("F3S_SCHEDULE", "window")
    plain = capi.attention(rwo, order, atox, bm, N, Q.cuda(), K.cuda(), V.cuda(),
                           scale).cpu().numpy()
    assert np.abs(got - plain).max() < 2e-3


@pytest.mark.parametrize("d", [96, 160, 256])
def test_16x8_blocks_with_the_sddmm_tap(oracle_mod, d):
    """f3s_attention_fwd_tcb8 (the reference's 1tb1tcb, src/F3S_kernel.cu:677-877) at the new head
    dimensions: output and the masked score tap against the 16x8 oracle."""
    from fused3s_amd import capi
    print("case head_dim tcb8 d=%d" % d, flush=True)
    N = 900
    rng = np.random.default_rng(300 + d)
    rowPtr, colIdx = random_csr(rng, N, 30, hub=101, empty_frac=0.03)
    Q, K, V = [(rng.standard_normal((N, d)) * d ** -0.25).astype(np.float16) for _ in range(3)]
    pre = oracle_mod.preprocess(rowPtr, colIdx, N, 16, 8)
    want, tap = oracle_mod.attention_tcb8(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                          pre["tcbBitMap"], N, Q, K, V, True, save_sddmm=True)
    dev = "cuda"
    rwo = torch.as_tensor(pre["rowWindowOffset"].astype(np.int32)).to(dev)
    atox = torch.as_tensor(pre["sparseAToXidx"].astype(np.int32)).to(dev)
    bm = torch.as_tensor(pre["tcbBitMap"].view(np.int64)).to(dev).view(torch.uint64)
    out, sddmm = capi.attention_tcb8(rwo, None, atox, bm, N, torch.as_tensor(Q).to(dev),
                                     torch.as_tensor(K).to(dev), torch.as_tensor(V).to(dev), True,
                                     save_sddmm=True)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.abs(got - want).max() < MAX_ABS
    assert mean_rel(got, want) < MEAN_REL
    got_tap = sddmm.cpu().numpy()
    assert np.array_equal(got_tap == 0, tap == 0)
    assert np.abs(got_tap - tap).max() <= 1e-5 * max(1.0, np.abs(tap).max())


def test_head_dims_that_are_not_multiples_of_32_are_refused():
    from fused3s_amd import capi
    N = 32
    rwo = torch.zeros(3, dtype=torch.int32, device="cuda")
    atox = torch.zeros(16, dtype=torch.int32, device="cuda")
    bm = torch.zeros(4, dtype=torch.uint64, device="cuda")
    for d in (48, 16, 288, 100):
        Q = torch.zeros((N, d), dtype=torch.float16, device="cuda")
        with pytest.raises(RuntimeError, match="head dim"):
            capi.attention(rwo, None, atox, bm, N, Q, Q, Q, 1.0)
        assert capi.lib().f3s_attention_uses_workspace(40_000, 40_000 * 8, d, 0) == 0
