"""Synthetic graphs and features of the benchmark configurations.

Every generator returns CSR (rowPtr int32[N+1], colIdx int32[E]) with rows sorted by column,
duplicates removed and self-loops added, as torch tensors on the requested device. Generation
runs on that device (a 114 M-edge graph takes seconds on the GPU); results are deterministic
for a given (seed, device type).

The reference benchmarks real datasets stored as .npz edge lists
(scripts/baseline_comp/baseline_comp_kernel_only.py:730-742); these generators stand in for
them with the shapes named by the benchmark configurations.
"""
import math

import torch


def _gen(seed, device):
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def edges_to_csr(src, dst, N, symmetrize=True, self_loops=True):
    """Dedupe directed pairs (optionally both directions + self loops) into sorted CSR."""
    device = src.device
    src = src.to(torch.int64)
    dst = dst.to(torch.int64)
    parts = [src * N + dst]
    if symmetrize:
        parts.append(dst * N + src)
    if self_loops:
        ar = torch.arange(N, device=device, dtype=torch.int64)
        parts.append(ar * N + ar)
    key = torch.unique(torch.cat(parts))  # sorted ascending: row-major, columns ascending
    rows = torch.div(key, N, rounding_mode="floor")
    cols = (key - rows * N).to(torch.int32)
    counts = torch.bincount(rows, minlength=N)
    rowPtr = torch.zeros(N + 1, dtype=torch.int64, device=device)
    rowPtr[1:] = torch.cumsum(counts, 0)
    if int(rowPtr[-1]) >= 2**31:
        raise ValueError("edge count exceeds int32 CSR")
    return rowPtr.to(torch.int32), cols.contiguous()


def gnm_graph(N=2708, M=10600, seed=0, device="cpu"):
    """Configuration 1: M uniformly sampled undirected pairs, symmetrised, with self-loops."""
    g = _gen(seed, device)
    src = torch.randint(0, N, (M,), generator=g, device=device)
    dst = torch.randint(0, N, (M,), generator=g, device=device)
    return edges_to_csr(src, dst, N)


def _rmat_edges(n, scale, a, b, c, g, device):
    src = torch.zeros(n, dtype=torch.int64, device=device)
    dst = torch.zeros(n, dtype=torch.int64, device=device)
    ab = a + b
    abc = a + b + c
    for _ in range(scale):
        u = torch.rand(n, generator=g, device=device)
        sbit = (u >= ab).to(torch.int64)
        dbit = (((u >= a) & (u < ab)) | (u >= abc)).to(torch.int64)
        src = src * 2 + sbit
        dst = dst * 2 + dbit
    return src, dst


def _relabel(keys, N, g, device):
    """Apply one random vertex permutation to both endpoints of the packed (src*N+dst) keys, so
    that hubs are spread over the row windows as in a real dataset instead of sitting in the
    first rows (R-MAT and Chung-Lu both emit hubs at low ids)."""
    perm = torch.randperm(N, generator=g, device=device)
    src = torch.div(keys, N, rounding_mode="floor")
    dst = keys - src * N
    return perm[src], perm[dst]


def rmat_graph(N, target_edges, a, b, c, seed=0, device="cpu", max_rounds=12):
    """R-MAT over 2^ceil(log2 N) ids, ids >= N rejected, drawn until the symmetrised, deduped
    edge set (self-loops included) reaches ~target_edges; vertices are then relabelled by a
    random permutation. Configurations 2 and 4."""
    g = _gen(seed, device)
    scale = max(1, math.ceil(math.log2(N)))
    keys = torch.empty(0, dtype=torch.int64, device=device)
    need = target_edges
    for _ in range(max_rounds):
        n = max(1024, int(need * 0.62))
        s, d = _rmat_edges(n, scale, a, b, c, g, device)
        ok = (s < N) & (d < N)
        s, d = s[ok], d[ok]
        keys = torch.unique(torch.cat([keys, s * N + d, d * N + s]))
        need = target_edges - N - int(keys.numel())
        if need <= 0.01 * target_edges:
            break
    src, dst = _relabel(keys, N, g, device)
    return edges_to_csr(src, dst, N, symmetrize=False)


def chung_lu_graph(N, target_edges, gamma=2.1, max_degree=22000, seed=0, device="cpu",
                   max_rounds=12):
    """Chung-Lu: endpoints drawn independently with probability proportional to the weights
    w_i = (i + i0)^(-1/(gamma-1)), i0 chosen so that w_max / mean(w) = max_degree / mean degree
    (max_degree is the hub's EXPECTED number of draws; repeated draws of one pair collapse, so
    its degree in the deduped graph comes out lower); distinct undirected pairs are collected and
    thinned to target_edges directed edges (both directions plus the N self-loops), then
    vertices are relabelled by a random permutation. Configuration 3."""
    g = _gen(seed, device)
    alpha = 1.0 / (gamma - 1.0)
    mean_deg = target_edges / N
    ratio = max_degree / mean_deg
    idx = torch.arange(N, dtype=torch.float64, device=device)

    def wratio(i0):
        w = (idx + i0) ** (-alpha)
        return float(w[0] / w.mean())

    lo, hi = 1e-3, float(N)
    for _ in range(60):  # w_max/mean decreases with i0
        mid = math.sqrt(lo * hi)
        if wratio(mid) > ratio:
            lo = mid
        else:
            hi = mid
    w = (idx + hi) ** (-alpha)
    cdf = torch.cumsum(w / w.sum(), 0)
    cdf[-1] = 1.0
    # undirected pairs (lo, hi), lo < hi, drawn until their symmetrised count plus the N
    # self-loops reaches the target, then thinned uniformly at random to hit it (uniform thinning
    # of a Chung-Lu graph is a Chung-Lu graph with scaled weights)
    want_pairs = max(0, (target_edges - N) // 2)
    pairs = torch.empty(0, dtype=torch.int64, device=device)
    for _ in range(max_rounds):
        need = want_pairs - int(pairs.numel())
        if need <= 0:
            break
        n = max(1024, int(need * 1.08))
        u = torch.rand(n, generator=g, device=device, dtype=torch.float64)
        v = torch.rand(n, generator=g, device=device, dtype=torch.float64)
        s = torch.searchsorted(cdf, u).clamp_(max=N - 1)
        d = torch.searchsorted(cdf, v).clamp_(max=N - 1)
        keep = s != d
        lo = torch.minimum(s, d)[keep]
        hi = torch.maximum(s, d)[keep]
        pairs = torch.unique(torch.cat([pairs, lo * N + hi]))
    if pairs.numel() > want_pairs:
        sel = torch.randperm(pairs.numel(), generator=g, device=device)[:want_pairs]
        pairs = pairs[sel]
    lo = torch.div(pairs, N, rounding_mode="floor")
    hi = pairs - lo * N
    keys = torch.cat([lo * N + hi, hi * N + lo])
    src, dst = _relabel(keys, N, g, device)
    return edges_to_csr(src, dst, N, symmetrize=False)


def sbm_graph(N=100000, n_blocks=500, p_in=0.02, p_out=1e-5, seed=0, device="cpu"):
    """Stochastic block model with equal blocks: the number of within-/cross-block pairs is the
    binomial mean, the pairs are drawn uniformly (with replacement, deduped). Configuration 5."""
    g = _gen(seed, device)
    bs = N // n_blocks
    m_in = int(round(n_blocks * (bs * (bs - 1) / 2) * p_in))
    blk = torch.randint(0, n_blocks, (m_in,), generator=g, device=device)
    a = torch.randint(0, bs, (m_in,), generator=g, device=device)
    b = torch.randint(0, bs, (m_in,), generator=g, device=device)
    keep = a != b
    src_in = (blk * bs + a)[keep]
    dst_in = (blk * bs + b)[keep]
    n_pairs_out = N * (N - 1) / 2 - n_blocks * bs * (bs - 1) / 2
    m_out = int(round(n_pairs_out * p_out))
    so = torch.randint(0, N, (m_out,), generator=g, device=device)
    do = torch.randint(0, N, (m_out,), generator=g, device=device)
    keep = torch.div(so, bs, rounding_mode="floor") != torch.div(do, bs, rounding_mode="floor")
    src = torch.cat([src_in, so[keep]])
    dst = torch.cat([dst_in, do[keep]])
    return edges_to_csr(src, dst, N)


def features(N, d, seed=0, device="cpu", dtype=torch.float16, std=1.0):
    """Q, K, V ~ N(0, std^2), drawn in fp32 on the CPU generator (same values everywhere) and
    rounded to the storage type."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    out = []
    for _ in range(3):
        x = torch.randn(N, d, generator=g, dtype=torch.float32) * std
        out.append(x.to(dtype).to(device))
    return out


CONFIGS = {
    # name: (graph factory kwargs, d, dtype, heads, scalingFactor)
    "cfg1_gnm_2708": dict(kind="gnm", N=2708, M=10600, d=64, dtype="fp16", heads=1),
    "cfg2_rmat_169k": dict(kind="rmat", N=169343, E=2_480_000 + 169343, a=0.57, b=0.19, c=0.19,
                           d=64, dtype="fp16", heads=1),
    # max_degree is the hub's expected number of draws; after deduplication and thinning the
    # largest degree of the generated graph is 20 726 (> 20 k as the configuration asks)
    "cfg3_chunglu_233k": dict(kind="chunglu", N=232965, E=114_600_000, gamma=2.1,
                              max_degree=26000, d=64, dtype="fp16", heads=1),
    "cfg4_rmat_2449k": dict(kind="rmat", N=2449029, E=61_900_000, a=0.45, b=0.22, c=0.22,
                            d=128, dtype="fp16", heads=1),
    "cfg5_sbm_100k": dict(kind="sbm", N=100000, n_blocks=500, p_in=0.02, p_out=1e-5, d=32,
                          dtype="bf16", heads=8),
    # the same layer with p_in = 0.2, which gives the ~4-5 M edges the configuration is quoted
    # with (p_in = 0.02 gives ~0.6 M)
    "cfg5b_sbm_100k_dense": dict(kind="sbm", N=100000, n_blocks=500, p_in=0.2, p_out=1e-5, d=32,
                                 dtype="bf16", heads=8),
    # not one of the benchmark's configurations: the multi-head layer of configuration 5 on the
    # long-window graph of configuration 3 (the multi-head entry with the column-sliced schedule)
    "extra_chunglu_233k_8x32": dict(kind="chunglu", N=232965, E=114_600_000, gamma=2.1,
                                    max_degree=26000, d=32, dtype="bf16", heads=8),
}


def make_graph(name, seed=0, device="cpu", scale=1.0):
    """Graph of a named configuration; scale < 1 shrinks N and E proportionally (tests)."""
    c = CONFIGS[name]
    N = max(32, int(c["N"] * scale))
    if c["kind"] == "gnm":
        return gnm_graph(N, max(1, int(c["M"] * scale)), seed, device)
    if c["kind"] == "rmat":
        return rmat_graph(N, int(c["E"] * scale), c["a"], c["b"], c["c"], seed, device)
    if c["kind"] == "chunglu":
        # keep the mean degree when shrinking, cap the hub degree by N
        E = int(c["E"] * scale)
        return chung_lu_graph(N, E, c["gamma"], min(c["max_degree"], N // 8), seed, device)
    if c["kind"] == "sbm":
        nb = max(1, int(c["n_blocks"] * scale))
        return sbm_graph(N - N % nb, nb, c["p_in"], c["p_out"], seed, device)
    raise KeyError(name)
