"""Independent (slow, numpy) derivations used to pin the oracle and the HIP path.

None of these share code or formulas with oracle/f3s_oracle.c: the TC-block structure is
re-derived from a dense adjacency matrix the way the reference's own test does
(scripts/tests/test_f3s_accuracy.py:15-62: drop all-zero columns of each 16-row block, group the
survivors W at a time), and the bitmap is built by cutting 8x8 sub-tiles out of the dense tile.
"""
import numpy as np


def dense_from_csr(rowPtr, colIdx, N):
    A = np.zeros((N, N), dtype=np.int64)  # multiplicities
    for r in range(N):
        for k in range(rowPtr[r], rowPtr[r + 1]):
            A[r, colIdx[k]] += 1
    return A


def tile_to_words(tile, W):
    """16xW boolean tile -> list of uint64 words: 8x8 sub-tiles enumerated column-major, each
    flattened row-major into a 64-character bit string read MSB first."""
    words = []
    for cb in range(W // 8):
        for rb in range(2):
            sub = tile[rb * 8:(rb + 1) * 8, cb * 8:(cb + 1) * 8]
            s = "".join("1" if b else "0" for b in sub.reshape(-1))
            words.append(int(s, 2))
    return words


def brute_preprocess(rowPtr, colIdx, N, H=16, W=16):
    A = dense_from_csr(rowPtr, colIdx, N)
    nRW = (N + H - 1) // H
    rwo = [0]
    atox, bitmap, tile_ids, toff, rowid, part = [], [], [], [0], [], []
    e2c = np.zeros(len(colIdx), np.int64)
    e2r = np.zeros(len(colIdx), np.int64)
    for w in range(nRW):
        blk = A[w * H:min(w * H + H, N)]
        cols = np.nonzero(blk.any(axis=0))[0]  # ascending surviving columns
        nb = -(-len(cols) // W)
        part.append(nb)
        rwo.append(rwo[-1] + nb)
        rank = {int(c): i for i, c in enumerate(cols)}
        per_block_edges = [[] for _ in range(nb)]
        for rl in range(blk.shape[0]):
            r = w * H + rl
            for k in range(rowPtr[r], rowPtr[r + 1]):
                c = rank[int(colIdx[k])]
                e2c[k] = c
                e2r[k] = r
                per_block_edges[c // W].append(rl * W + c % W)
        for b in range(nb):
            cs = list(cols[b * W:(b + 1) * W])
            tile = np.zeros((16, W), bool)
            tile[:blk.shape[0], :len(cs)] = blk[:, cs] > 0
            atox += [int(c) for c in cs] + [0] * (W - len(cs))
            bitmap += tile_to_words(tile, W)
            tile_ids += per_block_edges[b]
            toff.append(toff[-1] + len(per_block_edges[b]))
            rowid.append(w)
    order = sorted(range(nRW), key=lambda i: (-part[i], i))
    return dict(rowWindowOffset=np.array(rwo), sortedRowWindows=np.array(order, np.int64),
                tcblockRowid=np.array(rowid, np.int64), tcblocktileId=np.array(tile_ids, np.int64),
                tcblockOffset=np.array(toff), sparseAToXidx=np.array(atox, np.int64),
                tcbBitMap=np.array(bitmap, dtype=np.uint64), blockCount=rwo[-1],
                blockPartition=np.array(part, np.int64), edgeToColumn=e2c, edgeToRow=e2r)


def consume_bitmap_like_kernel(bitmap, t):
    """Rebuild the 16x16 tile of TC block t with the indexing the reference kernel uses to read
    it (src/F3S_kernel.cu:1447-1451): warp half h, lane, fragment element i."""
    tile = np.zeros((16, 16), bool)
    for h in range(2):
        for lane in range(32):
            for i in range(4):
                word = int(bitmap[t * 4 + h * 2 + i // 2])
                bit = 63 - lane * 2 - (i % 2)
                row = lane // 4 + 8 * (i // 2)
                col = 8 * h + (lane % 4) * 2 + (i % 2)
                tile[row, col] = (word >> bit) & 1
    return tile


def dense_attention(rowPtr, colIdx, N, Q, K, V, scale):
    """fp64 dense masked softmax attention: softmax over the non-zeros of each row of
    (Q K^T / scale) o A, times V (scripts/tests/test_f3s_accuracy.py:81-94,148-164)."""
    A = dense_from_csr(rowPtr, colIdx, N) > 0
    Qd, Kd, Vd = (x.astype(np.float64) for x in (Q, K, V))
    S = Qd @ Kd.T / scale
    S = np.where(A, S, -np.inf)
    mx = S.max(axis=1, keepdims=True)
    mx = np.where(np.isfinite(mx), mx, 0.0)
    P = np.exp(S - mx)
    P = np.where(A, P, 0.0)
    den = P.sum(axis=1, keepdims=True)
    P = np.divide(P, den, out=np.zeros_like(P), where=den > 0)
    return P @ Vd


def compare_preprocess(got, want, keys=None):
    """Bit-exact comparison of two preprocessing results (dicts of arrays / ints)."""
    keys = keys or ["rowWindowOffset", "blockPartition", "blockCount", "sparseAToXidx",
                    "tcbBitMap", "edgeToColumn", "edgeToRow", "tcblockOffset", "tcblockRowid",
                    "tcblocktileId", "sortedRowWindows"]
    for k in keys:
        g, w = got[k], want[k]
        if k == "blockCount":
            assert int(g) == int(w), (k, g, w)
            continue
        g = np.asarray(g)
        w = np.asarray(w)
        assert g.shape == w.shape, (k, g.shape, w.shape)
        if k == "tcbBitMap":
            ok = np.array_equal(g.astype(np.uint64), w.astype(np.uint64))
        else:
            ok = np.array_equal(g.astype(np.int64), w.astype(np.int64))
        if not ok:
            bad = np.nonzero(g.astype(np.uint64) != w.astype(np.uint64))[0]
            raise AssertionError("%s differs at %d places, first %s: got %s want %s"
                                 % (k, len(bad), bad[:5], g[bad[:5]], w[bad[:5]]))
