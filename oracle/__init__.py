"""ctypes front end of the CPU oracle (oracle/f3s_oracle.c).

TEST INFRASTRUCTURE ONLY: importable from tests/, the smoke check and the benchmark's
cpu_baseline leg. The product (fused3s_amd) never imports this package.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libf3s_oracle.so")
_lib = None


def build(force=False):
    """Compile the C restatement with gcc (make); returns the library path."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "libf3s_oracle.so"])
    return _LIB_PATH


def _p(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        i32p = ctypes.POINTER(ctypes.c_int32)
        u16p = ctypes.POINTER(ctypes.c_uint16)
        u64p = ctypes.POINTER(ctypes.c_uint64)
        u8p = ctypes.POINTER(ctypes.c_uint8)
        f32p = ctypes.POINTER(ctypes.c_float)
        ci = ctypes.c_int
        L.f3s_oracle_preprocess_count.restype = ctypes.c_int64
        L.f3s_oracle_preprocess_count.argtypes = [i32p, i32p, ci, ci, ci, i32p, i32p, i32p]
        L.f3s_oracle_fill_edge_to_row.restype = None
        L.f3s_oracle_fill_edge_to_row.argtypes = [i32p, ci, ci, i32p]
        L.f3s_oracle_preprocess_fill.restype = None
        L.f3s_oracle_preprocess_fill.argtypes = [i32p, i32p, ci, ci, ci, i32p, i32p, i32p, i32p,
                                                 u8p, i32p, i32p, u64p, i32p]
        L.f3s_oracle_attention_ref.restype = ci
        L.f3s_oracle_attention_ref.argtypes = [i32p, i32p, u64p, ci, ci, ci, u16p, u16p, u16p,
                                               ctypes.c_float, ci, ci, ci, ci, f32p]
        L.f3s_oracle_attention_tcb8.restype = ci
        L.f3s_oracle_attention_tcb8.argtypes = [i32p, i32p, u64p, ci, ci, u16p, u16p, u16p, ci,
                                                f32p, f32p]
        L.f3s_oracle_attention_textbook.restype = ci
        L.f3s_oracle_attention_textbook.argtypes = [i32p, i32p, ci, ci, ci, u16p, u16p, u16p,
                                                    ctypes.c_float, ci, ci, ci, f32p]
        L.f3s_oracle_half_to_float.restype = ctypes.c_float
        L.f3s_oracle_half_to_float.argtypes = [ctypes.c_uint16]
        L.f3s_oracle_round_to_half.restype = ctypes.c_float
        L.f3s_oracle_round_to_half.argtypes = [ctypes.c_float]
        L.f3s_oracle_round_to_bf16.argtypes = [ctypes.c_float]
        L.f3s_oracle_round_to_bf16.restype = ctypes.c_float
        L.f3s_oracle_num_threads.restype = ci
        _lib = L
    return _lib


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def preprocess(rowPtr, colIdx, N, H=16, W=16, emulate_stride_bug=False):
    """CPU twin of F3S.preprocess_gpu (src/F3S.cpp:40-87).

    Returns a dict holding the reference's return tuple members plus the three tensors the
    reference mutates in place (blockPartition, edgeToColumn, edgeToRow).
    """
    L = lib()
    rowPtr = _i32(rowPtr)
    colIdx = _i32(colIdx)
    E = int(rowPtr[N])
    nRW = (N + H - 1) // H
    blockPartition = np.zeros(nRW, np.int32)
    edgeToColumn = np.zeros(max(E, 1), np.int32)
    edgeToRow = np.zeros(max(E, 1), np.int32)
    rwo = np.zeros(nRW + 1, np.int32)
    i32, u8, u64 = ctypes.c_int32, ctypes.c_uint8, ctypes.c_uint64
    colp = np.zeros(1, np.int32) if colIdx.size == 0 else colIdx
    nTCB = L.f3s_oracle_preprocess_count(_p(rowPtr, i32), _p(colp, i32), N, H, W,
                                         _p(blockPartition, i32), _p(edgeToColumn, i32),
                                         _p(rwo, i32))
    assert nTCB >= 0
    L.f3s_oracle_fill_edge_to_row(_p(rowPtr, i32), N, int(emulate_stride_bug), _p(edgeToRow, i32))
    wpt = H * W // 64
    rowid = np.zeros(max(nTCB, 1), np.int32)
    tile = np.zeros(max(E, 1), np.uint8)
    toff = np.zeros(nTCB + 1, np.int32)
    atox = np.zeros(max(nTCB * W, 1), np.int32)
    bm = np.zeros(max(nTCB * wpt, 1), np.uint64)
    order = np.zeros(max(nRW, 1), np.int32)
    L.f3s_oracle_preprocess_fill(_p(rowPtr, i32), _p(colp, i32), N, H, W, _p(edgeToColumn, i32),
                                 _p(edgeToRow, i32), _p(rwo, i32), _p(rowid, i32), _p(tile, u8),
                                 _p(toff, i32), _p(atox, i32), _p(bm, u64), _p(order, i32))
    return dict(rowWindowOffset=rwo, sortedRowWindows=order[:nRW], tcblockRowid=rowid[:nTCB],
                tcblocktileId=tile[:E], tcblockOffset=toff, sparseAToXidx=atox[:nTCB * W],
                tcbBitMap=bm[:nTCB * wpt], blockCount=int(nTCB), blockPartition=blockPartition,
                edgeToColumn=edgeToColumn[:E], edgeToRow=edgeToRow[:E])


def _bits(x):
    """fp16 / bf16-as-uint16 array -> contiguous uint16 bit pattern view."""
    x = np.ascontiguousarray(x)
    if x.dtype == np.float16:
        return x.view(np.uint16)
    assert x.dtype == np.uint16, x.dtype
    return x


def attention_ref(rwo, atox, bitmap, N, Q, K, V, scalingFactor=1.0, nWarpPerBlock=8,
                  applySoftmax=True, dtype=0, windows=None):
    """Reference-emulating fused 3S (src/F3S_kernel.cu:1371-1800) on 16x16 TC blocks."""
    L = lib()
    Qb, Kb, Vb = _bits(Q), _bits(K), _bits(V)
    d = Qb.shape[1]
    out = np.zeros((N, d), np.float32)
    rwo = _i32(rwo)
    atox = _i32(atox) if len(atox) else np.zeros(1, np.int32)
    bitmap = np.ascontiguousarray(bitmap, dtype=np.uint64) if len(bitmap) else np.zeros(1, np.uint64)
    wb, we = (0, -1) if windows is None else windows
    rc = L.f3s_oracle_attention_ref(_p(rwo, ctypes.c_int32), _p(atox, ctypes.c_int32),
                                    _p(bitmap, ctypes.c_uint64), N, d, dtype,
                                    _p(Qb, ctypes.c_uint16), _p(Kb, ctypes.c_uint16),
                                    _p(Vb, ctypes.c_uint16), float(scalingFactor),
                                    int(nWarpPerBlock), int(bool(applySoftmax)), wb, we,
                                    _p(out, ctypes.c_float))
    assert rc == 0, rc
    return out


def attention_tcb8(rwo, atox, bitmap, N, Q, K, V, applySoftmax=True, save_sddmm=False):
    """Reference-emulating 1tb1tcb kernel (src/F3S_kernel.cu:677-877) on 16x8 TC blocks from
    preprocess(..., W=8). Returns out, or (out, sddmm fp32[nTCB*128]) with save_sddmm."""
    L = lib()
    Qb, Kb, Vb = _bits(Q), _bits(K), _bits(V)
    d = Qb.shape[1]
    out = np.zeros((N, d), np.float32)
    rwo = _i32(rwo)
    nT = int(rwo[-1])
    atox = _i32(atox) if len(atox) else np.zeros(1, np.int32)
    bitmap = np.ascontiguousarray(bitmap, dtype=np.uint64) if len(bitmap) else np.zeros(1, np.uint64)
    sddmm = np.zeros(max(nT, 1) * 128, np.float32) if save_sddmm else None
    rc = L.f3s_oracle_attention_tcb8(_p(rwo, ctypes.c_int32), _p(atox, ctypes.c_int32),
                                     _p(bitmap, ctypes.c_uint64), N, d, _p(Qb, ctypes.c_uint16),
                                     _p(Kb, ctypes.c_uint16), _p(Vb, ctypes.c_uint16),
                                     int(bool(applySoftmax)), _p(out, ctypes.c_float),
                                     _p(sddmm, ctypes.c_float) if save_sddmm else None)
    assert rc == 0, rc
    return (out, sddmm[:nT * 128]) if save_sddmm else out


def attention_textbook(rowPtr, colIdx, N, Q, K, V, scalingFactor=1.0, dtype=0, rows=None,
                       row_step=1):
    """Textbook masked softmax attention from CSR, fp64 accumulate. rows=(begin, end) and
    row_step restrict the computation to rows begin, begin+row_step, ... < end."""
    L = lib()
    Qb, Kb, Vb = _bits(Q), _bits(K), _bits(V)
    d = Qb.shape[1]
    out = np.zeros((N, d), np.float32)
    rowPtr = _i32(rowPtr)
    colIdx = _i32(colIdx) if len(colIdx) else np.zeros(1, np.int32)
    rb, re = (0, -1) if rows is None else rows
    rc = L.f3s_oracle_attention_textbook(_p(rowPtr, ctypes.c_int32), _p(colIdx, ctypes.c_int32),
                                         N, d, dtype, _p(Qb, ctypes.c_uint16),
                                         _p(Kb, ctypes.c_uint16), _p(Vb, ctypes.c_uint16),
                                         float(scalingFactor), rb, re, int(row_step),
                                         _p(out, ctypes.c_float))
    assert rc == 0, rc
    return out


def num_threads():
    return int(lib().f3s_oracle_num_threads())
