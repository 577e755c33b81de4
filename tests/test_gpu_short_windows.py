"""Graphs of short windows: the call is split between the wave-per-window kernel and the
four-wave kernel (long windows). Checked against the reference-emulating oracle for fp16 and
bf16, single head and multi-head, with the heavy-first order, a shuffled order (a long window may
then lie outside the four-wave kernel's grid) and natural order (no split)."""
import numpy as np
import pytest
import torch

from conftest import random_csr

pytestmark = pytest.mark.gpu
MAX_ABS = 2e-2
MEAN_REL = {torch.float16: 1e-3, torch.bfloat16: 1e-3}


def bits(t):
    t = t.contiguous().cpu()
    if t.dtype == torch.float16:
        return t.numpy()
    return t.view(torch.int16).numpy().view(np.uint16)


def sparse_graph_with_a_few_long_windows(seed, N=20000):
    """~1 edge per row (3-4 TC blocks per window) plus hub rows every 2003 rows whose windows
    have far more than 32 blocks."""
    rng = np.random.default_rng(seed)
    deg = rng.poisson(1.0, N)
    deg[::2003] = 900
    deg[1600:1616] = 0  # one empty window
    rowPtr = np.zeros(N + 1, np.int32)
    rowPtr[1:] = np.cumsum(deg)
    colIdx = np.concatenate([np.sort(rng.choice(N, size=k, replace=False)) for k in deg]
                            ).astype(np.int32)
    return rowPtr, colIdx


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d", [32, 64, 128])
def test_split_single_head(oracle_mod, dtype, d):
    from fused3s_amd import capi
    print("case short_windows single %s d=%d" % (dtype, d), flush=True)
    N = 20000
    rowPtr, colIdx = sparse_graph_with_a_few_long_windows(d)
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    counts = np.diff(pre["rowWindowOffset"])
    nRW = len(counts)
    # the split is taken (short on average), and there are long and empty windows
    assert nRW >= 1024 and counts.sum() < 16 * nRW and counts.max() > 32 and counts.min() == 0
    g = torch.Generator().manual_seed(d)
    Q, K, V = [torch.randn((N, d), generator=g).to(dtype) for _ in range(3)]
    scale = float(np.sqrt(d))
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"], pre["tcbBitMap"],
                                    N, bits(Q), bits(K), bits(V), scale,
                                    dtype=0 if dtype == torch.float16 else 1)
    dev = "cuda"
    rwo = torch.as_tensor(pre["rowWindowOffset"].astype(np.int32)).to(dev)
    atox = torch.as_tensor(pre["sparseAToXidx"].astype(np.int32)).to(dev)
    bm = torch.as_tensor(pre["tcbBitMap"].view(np.int64)).to(dev).view(torch.uint64)
    heavy_first = torch.as_tensor(pre["sortedRowWindows"].astype(np.int32)).to(dev)
    shuffled = heavy_first[torch.randperm(nRW, generator=g).to(dev)].contiguous()
    Qd, Kd, Vd = Q.to(dev), K.to(dev), V.to(dev)
    outs = {}
    for name, order in (("heavy_first", heavy_first), ("shuffled", shuffled), ("natural", None)):
        out = torch.full((N, d), float("nan"), dtype=torch.float32, device=dev)
        capi.attention(rwo, order, atox, bm, N, Qd, Kd, Vd, scale, out=out)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert np.isfinite(got).all(), name  # every row written exactly by one of the kernels
        assert np.abs(got - want).max() < MAX_ABS, name
        assert np.abs(got - want).mean() / np.abs(want).mean() < MEAN_REL[dtype], name
        outs[name] = got
    # without softmax (fp16 only: the bf16 rounding of raw scores is covered elsewhere)
    if dtype == torch.float16:
        want_n = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                          pre["tcbBitMap"], N, bits(Q), bits(K), bits(V), 1.0,
                                          applySoftmax=False)
        got_n = capi.attention(rwo, heavy_first, atox, bm, N, Qd, Kd, Vd, 1.0, False).cpu().numpy()
        assert np.abs(got_n - want_n).max() < 2e-2 * max(1.0, np.abs(want_n).max())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_split_multi_head_equals_per_head(oracle_mod, dtype):
    from fused3s_amd import capi
    print("case short_windows heads %s" % dtype, flush=True)
    N, heads, d = 20000, 3, 32
    rowPtr, colIdx = sparse_graph_with_a_few_long_windows(7)
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    dev = "cuda"
    rwo = torch.as_tensor(pre["rowWindowOffset"].astype(np.int32)).to(dev)
    atox = torch.as_tensor(pre["sparseAToXidx"].astype(np.int32)).to(dev)
    bm = torch.as_tensor(pre["tcbBitMap"].view(np.int64)).to(dev).view(torch.uint64)
    order = torch.as_tensor(pre["sortedRowWindows"].astype(np.int32)).to(dev)
    g = torch.Generator().manual_seed(1)
    Q, K, V = [(torch.randn((N, heads, d), generator=g) * d ** -0.25).to(dtype).to(dev)
               for _ in range(3)]
    scale = float(np.sqrt(d))
    out = torch.full((N, heads * d), float("nan"), dtype=torch.float32, device=dev)
    capi.attention_heads(rwo, order, atox, bm, N, Q, K, V, scale, out=out)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    for h in range(heads):
        qh, kh, vh = (x[:, h].contiguous() for x in (Q, K, V))
        single = capi.attention(rwo, order, atox, bm, N, qh, kh, vh, scale)
        assert torch.equal(out[:, h * d:(h + 1) * d], single), "head %d" % h
        want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                        pre["tcbBitMap"], N, bits(qh), bits(kh), bits(vh), scale,
                                        dtype=0 if dtype == torch.float16 else 1)
        got = single.cpu().numpy()
        assert np.abs(got - want).max() < MAX_ABS
        assert np.abs(got - want).mean() / np.abs(want).mean() < MEAN_REL[dtype]


def test_many_long_units_per_workgroup(oracle_mod):
    """More long (window, head) units than the long-window launch has workgroups (1024): its
    workgroups find several units each and compute them one after the other. 40 000 rows, one
    edge per row on average, 310 windows whose rows name 40 columns each; eight heads."""
    from fused3s_amd import capi
    print("case short_windows many long units", flush=True)
    N, heads, d = 40000, 8, 32
    rng = np.random.default_rng(11)
    deg = rng.poisson(1.0, N)
    for w in range(0, N // 16, 8)[:310]:
        deg[16 * w:16 * w + 16] = 40
    rowPtr = np.zeros(N + 1, np.int32)
    rowPtr[1:] = np.cumsum(deg)
    colIdx = np.concatenate([np.sort(rng.choice(N, size=k, replace=False)) for k in deg]
                            ).astype(np.int32)
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    counts = np.diff(pre["rowWindowOffset"])
    nRW = len(counts)
    assert nRW >= 1024 and counts.sum() < 16 * nRW        # the split is taken
    assert (counts > 32).sum() * heads > 2 * 1024          # two long units per workgroup and more
    dev = "cuda"
    rwo = torch.as_tensor(pre["rowWindowOffset"].astype(np.int32)).to(dev)
    atox = torch.as_tensor(pre["sparseAToXidx"].astype(np.int32)).to(dev)
    bm = torch.as_tensor(pre["tcbBitMap"].view(np.int64)).to(dev).view(torch.uint64)
    heavy_first = torch.as_tensor(pre["sortedRowWindows"].astype(np.int32)).to(dev)
    g = torch.Generator().manual_seed(3)
    shuffled = heavy_first[torch.randperm(nRW, generator=g).to(dev)].contiguous()
    Q, K, V = [(torch.randn((N, heads, d), generator=g) * d ** -0.25).to(torch.bfloat16).to(dev)
               for _ in range(3)]
    scale = float(np.sqrt(d))
    want = [oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                     pre["tcbBitMap"], N, bits(Q[:, h]), bits(K[:, h]),
                                     bits(V[:, h]), scale, dtype=1) for h in range(heads)]
    for name, order in (("heavy_first", heavy_first), ("shuffled", shuffled)):
        out = torch.full((N, heads * d), float("nan"), dtype=torch.float32, device=dev)
        capi.attention_heads(rwo, order, atox, bm, N, Q, K, V, scale, out=out)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert np.isfinite(got).all(), name  # every row written by exactly one of the kernels
        for h in range(heads):
            gh = got[:, h * d:(h + 1) * d]
            assert np.abs(gh - want[h]).max() < MAX_ABS, (name, h)
            assert np.abs(gh - want[h]).mean() / np.abs(want[h]).mean() < MEAN_REL[torch.bfloat16]
    # single head through the same launch shape
    q1, k1, v1 = (x[:, 0].contiguous() for x in (Q, K, V))
    out1 = torch.full((N, d), float("nan"), dtype=torch.float32, device=dev)
    capi.attention(rwo, heavy_first, atox, bm, N, q1, k1, v1, scale, out=out1)
    torch.cuda.synchronize()
    assert np.abs(out1.cpu().numpy() - want[0]).max() < MAX_ABS
