"""bf16 inputs and the multi-head entry point (f3s_attention_fwd_heads) against the CPU oracle.

The reference is fp16, single head; its callers loop over heads and concatenate. Parity here means:
the multi-head launch returns exactly what the single-head launch returns head by head (same
arithmetic in the same order, so bit-identical), and the single-head result matches the
reference-emulating oracle (P rounded to fp16 as the reference rounds it) within max-abs 2e-2 /
mean-relative 1e-3 for fp16 and for bf16 inputs alike.
"""
import numpy as np
import pytest
import torch

from conftest import random_csr

pytestmark = pytest.mark.gpu
MAX_ABS = 2e-2
MEAN_REL = {torch.float16: 1e-3, torch.bfloat16: 1e-3}


def mean_rel(a, b):
    return float(np.abs(a - b).mean() / max(np.abs(b).mean(), 1e-30))


def bits(t):
    """torch fp16/bf16 tensor -> numpy array the oracle takes (float16, or uint16 bit patterns)."""
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


def make(seed, N, deg, hub, heads, d, dtype, std=1.0):
    rng = np.random.default_rng(seed)
    rowPtr, colIdx = random_csr(rng, N, deg, hub=hub, empty_frac=0.05)
    g = torch.Generator().manual_seed(seed)
    Q, K, V = [(torch.randn((N, heads, d), generator=g) * std).to(dtype) for _ in range(3)]
    return rowPtr, colIdx, Q, K, V


@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("seed,N,deg,hub", [(0, 300, 25, 13), (1, 1000, 100, 0), (3, 16, 2, 0)])
def test_bf16_single_head_matches_oracle(oracle_mod, d, seed, N, deg, hub):
    from fused3s_amd import capi
    print("case bf16 d=%d seed=%d N=%d" % (d, seed, N), flush=True)
    rowPtr, colIdx, Q, K, V = make(seed, N, deg, hub, 1, d, torch.bfloat16)
    Q, K, V = Q[:, 0], K[:, 0], V[:, 0]
    scale = float(np.sqrt(d))
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                    pre["tcbBitMap"], N, bits(Q), bits(K), bits(V), scale, dtype=1)
    txt = oracle_mod.attention_textbook(rowPtr, colIdx, N, bits(Q), bits(K), bits(V), scale,
                                        dtype=1)
    rwo, order, atox, bm = to_dev(pre)
    for od in (None, order):
        got = capi.attention(rwo, od, atox, bm, N, Q.contiguous().cuda(), K.contiguous().cuda(),
                             V.contiguous().cuda(), scale)
        torch.cuda.synchronize()
        got = got.cpu().numpy()
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() < MAX_ABS
        assert mean_rel(got, want) < MEAN_REL[torch.bfloat16]
        assert np.abs(got - txt).max() < MAX_ABS
    # SDDMM -> SpMM without softmax: raw scores as the second product's left operand
    want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                    pre["tcbBitMap"], N, bits(Q), bits(K), bits(V), 1.0,
                                    applySoftmax=False, dtype=1)
    got = capi.attention(rwo, order, atox, bm, N, Q.contiguous().cuda(), K.contiguous().cuda(),
                         V.contiguous().cuda(), 1.0, False).cpu().numpy()
    assert mean_rel(got, want) < MEAN_REL[torch.bfloat16]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("heads,d,pad", [(8, 32, 0), (3, 64, 8), (2, 128, 0), (1, 64, 24)])
def test_heads_entry_equals_per_head_launches_and_oracle(oracle_mod, dtype, heads, d, pad):
    from fused3s_amd import capi
    print("case heads=%d d=%d pad=%d %s" % (heads, d, pad, dtype), flush=True)
    N = 700
    rowPtr, colIdx, Q, K, V = make(11 + heads, N, 30, 40, heads, d, dtype,
                                   std=1.0 if dtype == torch.float16 else d ** -0.25)
    scale = float(np.sqrt(d))
    pre = oracle_mod.preprocess(rowPtr, colIdx, N)
    rwo, order, atox, bm = to_dev(pre)

    def pitched(t):
        # rows padded by `pad` elements: [N, heads*d + pad] storage viewed as [N, heads, d]
        store = torch.zeros((N, heads * d + pad), dtype=dtype, device="cuda")
        store[:, :heads * d] = t.reshape(N, heads * d).cuda()
        return store[:, :heads * d].unflatten(1, (heads, d))

    Qd, Kd, Vd = pitched(Q), pitched(K), pitched(V)
    assert Qd.stride(0) == heads * d + pad
    out_store = torch.full((N, heads * d + 4), -7.0, dtype=torch.float32, device="cuda")
    out = out_store[:, :heads * d]
    got = capi.attention_heads(rwo, order, atox, bm, N, Qd, Kd, Vd, scale, out=out)
    torch.cuda.synchronize()
    assert got.data_ptr() == out.data_ptr()
    assert (out_store[:, heads * d:] == -7.0).all()  # the pitch padding is not written
    got = got.cpu().numpy()
    for h in range(heads):
        qh, kh, vh = (t[:, h].contiguous() for t in (Q, K, V))
        single = capi.attention(rwo, order, atox, bm, N, qh.cuda(), kh.cuda(), vh.cuda(),
                                scale).cpu().numpy()
        assert np.array_equal(got[:, h * d:(h + 1) * d], single), "head %d" % h
        want = oracle_mod.attention_ref(pre["rowWindowOffset"], pre["sparseAToXidx"],
                                        pre["tcbBitMap"], N, bits(qh), bits(kh), bits(vh), scale,
                                        dtype=0 if dtype == torch.float16 else 1)
        assert np.abs(single - want).max() < MAX_ABS
        assert mean_rel(single, want) < MEAN_REL[dtype]
    # natural window order gives the same rows
    nat = capi.attention_heads(rwo, None, atox, bm, N, Qd, Kd, Vd, scale).cpu().numpy()
    assert np.array_equal(nat, got)


def test_heads_entry_argument_errors():
    from fused3s_amd import capi
    N, heads, d = 32, 2, 32
    rwo = torch.zeros(3, dtype=torch.int32, device="cuda")
    atox = torch.zeros(16, dtype=torch.int32, device="cuda")
    bm = torch.zeros(4, dtype=torch.uint64, device="cuda")
    Q = torch.zeros((N, heads, d), dtype=torch.float16, device="cuda")
    out = capi.attention_heads(rwo, None, atox, bm, N, Q, Q, Q, 1.0)  # no blocks: all rows zero
    assert out.shape == (N, heads * d) and (out == 0).all()
    with pytest.raises(RuntimeError, match="16-byte aligned"):
        store = torch.zeros((N, heads * d + 4), dtype=torch.float16, device="cuda")
        bad = store[:, :heads * d].unflatten(1, (heads, d))
        capi.attention_heads(rwo, None, atox, bm, N, bad, bad, bad, 1.0)
    with pytest.raises(RuntimeError, match="head dim"):
        Q48 = torch.zeros((N, 2, 48), dtype=torch.float16, device="cuda")
        capi.attention_heads(rwo, None, atox, bm, N, Q48, Q48, Q48, 1.0)
    with pytest.raises(RuntimeError, match="scalingFactor"):
        capi.attention_heads(rwo, None, atox, bm, N, Q, Q, Q, 0.0)
    with pytest.raises(RuntimeError, match="float16 or bfloat16"):
        capi.attention_heads(rwo, None, atox, bm, N, Q.float(), Q.float(), Q.float(), 1.0)
