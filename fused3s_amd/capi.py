"""ctypes binding of libf3s_amd.so (include/f3s_amd.h), operating on torch device tensors.

This is the thinnest possible host layer: it passes data_ptr()s and sizes through the C ABI
and raises RuntimeError with f3s_last_error() on a non-zero status. There is no fallback: if
the HIP library is missing, importing or calling anything here fails.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("F3S_AMD_LIB", os.path.join(_HERE, "libf3s_amd.so"))
_lib = None

EXPORTS = ["f3s_abi_version", "f3s_last_error", "f3s_preprocess_workspace_bytes",
           "f3s_preprocess_count", "f3s_preprocess_fill", "f3s_attention_fwd",
           "f3s_attention_workspace_bytes", "f3s_attention_fwd_heads",
           "f3s_attention_fwd_tcb8", "f3s_attention_uses_workspace",
           "f3s_preprocess_static_scratch_bytes", "f3s_preprocess_count_static",
           "f3s_preprocess_capacity", "f3s_preprocess", "f3s_attention_prepare",
           "f3s_attention_heads_workspace_bytes", "f3s_attention_uses_wide_offsets"]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libf3s_amd.so is not built (python -m fused3s_amd.build); there is no fallback")
        L = ctypes.CDLL(LIB_PATH)
        vp, ci, cs = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
        L.f3s_abi_version.restype = ci
        L.f3s_last_error.restype = ctypes.c_char_p
        L.f3s_preprocess_workspace_bytes.restype = cs
        L.f3s_preprocess_workspace_bytes.argtypes = [ci, ci]
        L.f3s_preprocess_count.restype = ci
        L.f3s_preprocess_count.argtypes = [vp, vp, ci, ci, ci, ci, vp, vp, vp, vp, vp, vp, cs,
                                           ctypes.POINTER(ctypes.c_int64), vp]
        L.f3s_preprocess_static_scratch_bytes.restype = cs
        L.f3s_preprocess_static_scratch_bytes.argtypes = []
        L.f3s_preprocess_count_static.restype = ci
        L.f3s_preprocess_count_static.argtypes = [vp, vp, ci, ci, ci, ci, vp, vp, vp, vp, vp, vp,
                                                  vp]
        L.f3s_preprocess_fill.restype = ci
        L.f3s_preprocess_fill.argtypes = [vp, vp, ci, ci, ci, ci, vp, vp, ctypes.c_int64, vp, vp,
                                          vp, vp, vp, vp]
        L.f3s_preprocess_capacity.restype = ctypes.c_int64
        L.f3s_preprocess_capacity.argtypes = [ci, ctypes.c_int64, ci]
        L.f3s_preprocess.restype = ci
        L.f3s_preprocess.argtypes = [vp, vp, ci, ci, ci, ci, vp, vp, vp, vp, vp, ctypes.c_int64,
                                     vp, vp, vp, vp, vp, vp, cs, ctypes.POINTER(ctypes.c_int64),
                                     vp]
        L.f3s_attention_fwd.restype = ci
        L.f3s_attention_fwd.argtypes = [vp, vp, vp, vp, ci, ctypes.c_int64, ci, ci, vp, vp, vp,
                                        ctypes.c_float, ci, vp, vp, vp, cs, ci, vp]
        L.f3s_attention_workspace_bytes.restype = cs
        L.f3s_attention_workspace_bytes.argtypes = [ci, ci]
        L.f3s_attention_fwd_heads.restype = ci
        L.f3s_attention_fwd_heads.argtypes = [vp, vp, vp, vp, ci, ctypes.c_int64, ci, ci, ci, vp,
                                              vp, vp, ctypes.c_int64, ctypes.c_float, ci, vp,
                                              ctypes.c_int64, vp, cs, ci, vp]
        L.f3s_attention_heads_workspace_bytes.restype = cs
        L.f3s_attention_heads_workspace_bytes.argtypes = [ci, ci, ci]
        L.f3s_attention_prepare.restype = ci
        L.f3s_attention_prepare.argtypes = [vp, vp, ci, ctypes.c_int64, ci, ci, vp, cs, vp]
        L.f3s_attention_uses_wide_offsets.restype = ci
        L.f3s_attention_uses_wide_offsets.argtypes = [ctypes.c_int64, ctypes.c_int64, ci]
        L.f3s_attention_uses_workspace.restype = ci
        L.f3s_attention_uses_workspace.argtypes = [ci, ctypes.c_int64, ci, ci]
        L.f3s_attention_fwd_tcb8.restype = ci
        L.f3s_attention_fwd_tcb8.argtypes = [vp, vp, vp, vp, ci, ctypes.c_int64, ci, vp, vp, vp,
                                             ci, vp, vp, vp]
        _lib = L
    return _lib


def _check(rc):
    if rc != 0:
        raise RuntimeError("libf3s_amd: %s (status %d)" % (lib().f3s_last_error().decode(), rc))


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t, dtype, name):
    if not t.is_cuda:
        raise RuntimeError("%s must be a device tensor" % name)
    if t.dtype != dtype:
        raise RuntimeError("%s must be %s, got %s" % (name, dtype, t.dtype))
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)


def preprocess(rowPtr, colIdx, N, H=16, W=16, two_phase=False):
    """Preprocessing through the C ABI. Returns a dict of device tensors.

    Default: f3s_preprocess, one call with the block arrays allocated for
    f3s_preprocess_capacity(N, E, W) blocks; the returned block tensors are views of their first
    blockCount entries. two_phase=True: f3s_preprocess_count, exact allocations, then
    f3s_preprocess_fill (the reference's sequence, src/F3S.cpp:40-87)."""
    L = lib()
    _dev(rowPtr, torch.int32, "rowPtr")
    _dev(colIdx, torch.int32, "colIdx")
    dev = rowPtr.device
    E = int(colIdx.numel())
    nRW = (N + H - 1) // H
    i32 = dict(dtype=torch.int32, device=dev)
    blockPartition = torch.empty(nRW, **i32)
    edgeToColumn = torch.empty(E, **i32)
    edgeToRow = torch.empty(E, **i32)
    rwo = torch.empty(nRW + 1, **i32)
    order = torch.empty(nRW, **i32)
    wsBytes = L.f3s_preprocess_workspace_bytes(N, E)
    ws = torch.empty(wsBytes, dtype=torch.uint8, device=dev)
    nTcb = ctypes.c_int64(-1)
    tile = torch.empty(E, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        if two_phase:
            _check(L.f3s_preprocess_count(_ptr(rowPtr), _ptr(colIdx), N, E, H, W,
                                          _ptr(blockPartition), _ptr(edgeToColumn),
                                          _ptr(edgeToRow), _ptr(rwo), _ptr(order), _ptr(ws),
                                          wsBytes, ctypes.byref(nTcb), _stream()))
            nT = int(nTcb.value)
            rowid = torch.empty(nT, **i32)
            toff = torch.empty(nT + 1, **i32)
            atox = torch.empty(nT * W, **i32)
            bm = torch.empty(nT * H * W // 64, dtype=torch.uint64, device=dev)
            _check(L.f3s_preprocess_fill(_ptr(rowPtr), _ptr(colIdx), N, E, H, W,
                                         _ptr(edgeToColumn), _ptr(rwo), nT, _ptr(rowid),
                                         _ptr(tile), _ptr(toff), _ptr(atox), _ptr(bm), _stream()))
        else:
            cap = int(L.f3s_preprocess_capacity(N, E, W))
            rowid = torch.empty(cap, **i32)
            toff = torch.empty(cap + 1, **i32)
            atox = torch.empty(cap * W, **i32)
            bm = torch.empty(cap * H * W // 64, dtype=torch.uint64, device=dev)
            _check(L.f3s_preprocess(_ptr(rowPtr), _ptr(colIdx), N, E, H, W, _ptr(blockPartition),
                                    _ptr(edgeToColumn), _ptr(edgeToRow), _ptr(rwo), _ptr(order),
                                    cap, _ptr(rowid), _ptr(tile), _ptr(toff), _ptr(atox),
                                    _ptr(bm), _ptr(ws), wsBytes, ctypes.byref(nTcb), _stream()))
            nT = int(nTcb.value)
            rowid = rowid[:nT]
            toff = toff[:nT + 1]
            atox = atox[:nT * W]
            bm = bm[:nT * H * W // 64]
    return dict(rowWindowOffset=rwo, sortedRowWindows=order, tcblockRowid=rowid,
                tcblocktileId=tile, tcblockOffset=toff, sparseAToXidx=atox, tcbBitMap=bm,
                blockCount=nT, blockPartition=blockPartition, edgeToColumn=edgeToColumn,
                edgeToRow=edgeToRow)


def preprocess_count_static(rowPtr, colIdx, N, out, H=16, W=16):
    """f3s_preprocess_count_static on the current stream: phase 1 with the library's own scratch
    and no host round trip. `out` holds caller-allocated device tensors blockPartition,
    edgeToColumn, edgeToRow, rowWindowOffset, sortedRowWindows (int32) and result (int64[2]:
    TC-block total, error flag); nothing is allocated here."""
    L = lib()
    _dev(rowPtr, torch.int32, "rowPtr")
    _dev(colIdx, torch.int32, "colIdx")
    for name in ("blockPartition", "edgeToColumn", "edgeToRow", "rowWindowOffset",
                 "sortedRowWindows"):
        _dev(out[name], torch.int32, name)
    _dev(out["result"], torch.int64, "result")
    with torch.cuda.device(rowPtr.device):
        _check(L.f3s_preprocess_count_static(
            _ptr(rowPtr), _ptr(colIdx), N, int(colIdx.numel()), H, W, _ptr(out["blockPartition"]),
            _ptr(out["edgeToColumn"]), _ptr(out["edgeToRow"]), _ptr(out["rowWindowOffset"]),
            _ptr(out["sortedRowWindows"]), _ptr(out["result"]), _stream()))


def attention_workspace(N, d, device, nTCB=None, dtype=torch.float16, heads=0):
    """Scratch tensor for attention(..., workspace=...) / attention_heads(..., workspace=...)
    (column-sliced schedule; heads = 0 for the single-head call). With nTCB given, returns None
    when the library would not use it for this problem."""
    L = lib()
    if nTCB is not None and not L.f3s_attention_uses_workspace(
            N, int(nTCB), d, 0 if dtype == torch.float16 else 1):
        return None
    nbytes = (L.f3s_attention_heads_workspace_bytes(N, heads, d) if heads > 0
              else L.f3s_attention_workspace_bytes(N, d))
    return torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)


def attention_prepare(rwo, atox, N, d, workspace, heads=0):
    """f3s_attention_prepare on the current stream: builds the column-sliced schedule's index in
    `workspace` for these arrays, which must then stay unchanged while it is in use."""
    L = lib()
    _dev(rwo, torch.int32, "rowWindowOffset")
    _dev(atox, torch.int32, "sparseAToXidx")
    with torch.cuda.device(rwo.device):
        _check(L.f3s_attention_prepare(_ptr(rwo), _ptr(atox), N, atox.numel() // 16,
                                       d, heads, _ptr(workspace), workspace.numel(), _stream()))


def attention(rwo, order, atox, bitmap, N, Q, K, V, scalingFactor=1.0, applySoftmax=True,
              out=None, workspace=None, prepared=False):
    """f3s_attention_fwd on the current stream; returns out fp32[N, d]."""
    L = lib()
    _dev(rwo, torch.int32, "rowWindowOffset")
    _dev(atox, torch.int32, "sparseAToXidx")
    _dev(bitmap, torch.uint64, "tcbBitMap")
    for name, t in (("Q", Q), ("K", K), ("V", V)):
        _dev(t, Q.dtype, name)
    if order is not None:
        _dev(order, torch.int32, "windowOrder")
    if Q.dtype == torch.float16:
        dtype = 0
    elif Q.dtype == torch.bfloat16:
        dtype = 1
    else:
        raise RuntimeError("Q/K/V must be float16 or bfloat16")
    d = Q.shape[1]
    if Q.shape[0] < N or K.shape != Q.shape or V.shape != Q.shape:
        raise RuntimeError("Q/K/V must be [N, d] with identical shapes")
    if rwo.numel() != (N + 15) // 16 + 1:
        raise RuntimeError("rowWindowOffset has %d entries, expected %d"
                           % (rwo.numel(), (N + 15) // 16 + 1))
    if order is not None and order.numel() != rwo.numel() - 1:
        raise RuntimeError("windowOrder must have one entry per row window")
    if out is None:
        out = torch.empty((N, d), dtype=torch.float32, device=Q.device)
    with torch.cuda.device(Q.device):
        _check(L.f3s_attention_fwd(_ptr(rwo), _ptr(order), _ptr(atox), _ptr(bitmap), N,
                                   atox.numel() // 16, d, dtype, _ptr(Q), _ptr(K), _ptr(V),
                                   float(scalingFactor), int(bool(applySoftmax)), _ptr(out), None,
                                   _ptr(workspace),
                                   0 if workspace is None else workspace.numel(),
                                   int(bool(prepared)), _stream()))
    return out


def attention_heads(rwo, order, atox, bitmap, N, Q, K, V, scalingFactor=1.0, applySoftmax=True,
                    out=None, workspace=None, prepared=False):
    """f3s_attention_fwd_heads on the current stream. Q, K, V: [N, nHeads, d] fp16 or bf16 whose
    last two dimensions are contiguous (dim 0 may be pitched); returns out fp32[N, nHeads*d]."""
    L = lib()
    _dev(rwo, torch.int32, "rowWindowOffset")
    _dev(atox, torch.int32, "sparseAToXidx")
    _dev(bitmap, torch.uint64, "tcbBitMap")
    if order is not None:
        _dev(order, torch.int32, "windowOrder")
        if order.numel() != rwo.numel() - 1:
            raise RuntimeError("windowOrder must have one entry per row window")
    if Q.dtype == torch.float16:
        dtype = 0
    elif Q.dtype == torch.bfloat16:
        dtype = 1
    else:
        raise RuntimeError("Q/K/V must be float16 or bfloat16")
    if Q.dim() != 3:
        raise RuntimeError("Q/K/V must be [N, nHeads, d]")
    nHeads, d = Q.shape[1], Q.shape[2]
    for name, t in (("Q", Q), ("K", K), ("V", V)):
        if not t.is_cuda or t.dtype != Q.dtype or t.shape != Q.shape:
            raise RuntimeError("%s must be a device tensor with Q's dtype and shape" % name)
        if t.stride(2) != 1 or t.stride(1) != d or t.stride(0) != Q.stride(0):
            raise RuntimeError("%s: heads must be contiguous inside a row, one row pitch for "
                               "Q, K and V" % name)
    if Q.shape[0] < N:
        raise RuntimeError("Q/K/V have fewer than N rows")
    if rwo.numel() != (N + 15) // 16 + 1:
        raise RuntimeError("rowWindowOffset has %d entries, expected %d"
                           % (rwo.numel(), (N + 15) // 16 + 1))
    if out is None:
        out = torch.empty((N, nHeads * d), dtype=torch.float32, device=Q.device)
    elif out.dtype != torch.float32 or out.stride(1) != 1 or out.shape[1] != nHeads * d:
        raise RuntimeError("out must be fp32 [N, nHeads*d] with contiguous rows")
    with torch.cuda.device(Q.device):
        _check(L.f3s_attention_fwd_heads(_ptr(rwo), _ptr(order), _ptr(atox), _ptr(bitmap), N,
                                         atox.numel() // 16, nHeads, d, dtype, _ptr(Q), _ptr(K),
                                         _ptr(V), Q.stride(0), float(scalingFactor),
                                         int(bool(applySoftmax)), _ptr(out), out.stride(0),
                                         _ptr(workspace),
                                         0 if workspace is None else workspace.numel(),
                                         int(bool(prepared)), _stream()))
    return out


def attention_tcb8(rwo, order, atox, bitmap, N, Q, K, V, applySoftmax=True, save_sddmm=False):
    """f3s_attention_fwd_tcb8 on the current stream (16x8 TC blocks from preprocess(..., W=8)).
    Returns out fp32[N, d], or (out, sddmm fp32[nTCB*128]) with save_sddmm."""
    L = lib()
    _dev(rwo, torch.int32, "rowWindowOffset")
    _dev(atox, torch.int32, "sparseAToXidx")
    _dev(bitmap, torch.uint64, "tcbBitMap")
    for name, t in (("Q", Q), ("K", K), ("V", V)):
        _dev(t, torch.float16, name)
    if order is not None:
        _dev(order, torch.int32, "windowOrder")
        if order.numel() != rwo.numel() - 1:
            raise RuntimeError("windowOrder must have one entry per row window")
    d = Q.shape[1]
    if Q.shape[0] < N or K.shape != Q.shape or V.shape != Q.shape:
        raise RuntimeError("Q/K/V must be [N, d] with identical shapes")
    if rwo.numel() != (N + 15) // 16 + 1:
        raise RuntimeError("rowWindowOffset has %d entries, expected %d"
                           % (rwo.numel(), (N + 15) // 16 + 1))
    nT = atox.numel() // 8
    if bitmap.numel() != 2 * nT:
        raise RuntimeError("tcbBitMap must hold two words per 16x8 block")
    out = torch.empty((N, d), dtype=torch.float32, device=Q.device)
    sddmm = torch.empty(nT * 128, dtype=torch.float32, device=Q.device) if save_sddmm else None
    with torch.cuda.device(Q.device):
        _check(L.f3s_attention_fwd_tcb8(_ptr(rwo), _ptr(order), _ptr(atox), _ptr(bitmap), N, nT, d,
                                        _ptr(Q), _ptr(K), _ptr(V), int(bool(applySoftmax)),
                                        _ptr(out), _ptr(sddmm), _stream()))
    return (out, sddmm) if save_sddmm else out
