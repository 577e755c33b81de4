"""f3s_preprocess_count_static (phase 1 of preprocessing on the library's own static device
scratch, no allocation, no host round trip) against f3s_preprocess_count: every output
bit-identical, on two calls in a row, the second on a smaller graph."""
import numpy as np
import pytest
import torch

from conftest import random_csr

pytestmark = pytest.mark.gpu

KEYS = ("blockPartition", "edgeToColumn", "edgeToRow", "rowWindowOffset", "sortedRowWindows")


def _graph(seed, N, deg, **kw):
    rp, ci = random_csr(np.random.default_rng(seed), N, deg, **kw)
    return torch.from_numpy(rp).cuda(), torch.from_numpy(ci).cuda()


def _buffers(N, E, fill):
    """Caller-owned outputs, pre-filled with a pattern so that a slot the call skipped shows."""
    nRW = (N + 15) // 16
    i32 = dict(dtype=torch.int32, device="cuda")
    return dict(blockPartition=torch.full((nRW,), fill, **i32),
                edgeToColumn=torch.full((E,), fill, **i32),
                edgeToRow=torch.full((E,), fill, **i32),
                rowWindowOffset=torch.full((nRW + 1,), fill, **i32),
                sortedRowWindows=torch.full((nRW,), fill, **i32),
                result=torch.full((2,), fill, dtype=torch.int64, device="cuda"))


@pytest.mark.parametrize("W", [16, 8])
def test_static_scratch_matches_workspace_entry_twice(W):
    from fused3s_amd import capi
    # first a graph with long windows (hubs) and unsorted / repeated columns, then a smaller one
    # of short windows: whatever the first call left in the scratch must not leak into the second
    cases = [(11, 6000, 40, dict(dup=True, unsorted=True, hub=40, empty_frac=0.02)),
             (12, 1500, 5, dict(empty_frac=0.3))]
    for seed, N, deg, kw in cases:
        print("case W=%d seed=%d N=%d" % (W, seed, N), flush=True)
        rp, ci = _graph(seed, N, deg, **kw)
        want = capi.preprocess(rp, ci, N, 16, W)
        got = _buffers(N, int(ci.numel()), -7)
        torch.cuda.synchronize()
        # the property the entry exists for: with the caller's buffers in place, the call takes
        # no device memory (neither through torch nor beside it); the very first call on a device
        # looks up the scratch array's address, which allocates nothing either
        free_before, _ = torch.cuda.mem_get_info()
        torch_before = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
        capi.preprocess_count_static(rp, ci, N, got, 16, W)
        torch.cuda.synchronize()
        assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == torch_before
        assert torch.cuda.mem_get_info()[0] == free_before
        for k in KEYS:
            assert torch.equal(got[k], want[k]), k
        assert got["result"].tolist() == [want["blockCount"], 0]


def test_static_scratch_reports_bad_column_and_rejects_oversize():
    from fused3s_amd import capi
    rp, ci = _graph(3, 400, 6)
    ci = ci.clone()
    ci[5] = 400  # one column index out of range
    got = _buffers(400, int(ci.numel()), 0)
    capi.preprocess_count_static(rp, ci, 400, got)
    torch.cuda.synchronize()
    assert int(got["result"][1]) == 1
    # the next call starts from a clean error flag
    rp2, ci2 = _graph(4, 300, 4)
    got2 = _buffers(300, int(ci2.numel()), 0)
    capi.preprocess_count_static(rp2, ci2, 300, got2)
    torch.cuda.synchronize()
    assert int(got2["result"][1]) == 0
    assert int(got2["result"][0]) == capi.preprocess(rp2, ci2, 300)["blockCount"]
    # more nodes than the 8 MiB scratch serves: refused before anything is launched
    limit = capi.lib().f3s_preprocess_static_scratch_bytes()
    assert limit == 8 << 20
    with pytest.raises(RuntimeError, match="scratch"):
        capi.preprocess_count_static(rp2, ci2, 12_000_000, got2)
