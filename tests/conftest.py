import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def random_csr(rng, N, avg_deg, dup=False, unsorted=False, empty_frac=0.0, hub=0):
    """Random CSR for tests: optional duplicate entries, unsorted columns, empty rows, hub rows."""
    rows = []
    for r in range(N):
        if rng.random() < empty_frac:
            rows.append(np.zeros(0, np.int32))
            continue
        deg = rng.poisson(avg_deg)
        if hub and r % hub == 0:
            deg = min(N, deg * 20 + 5)
        cols = rng.integers(0, N, size=deg)
        if not dup:
            cols = np.unique(cols)
        elif deg > 1:
            cols = np.concatenate([cols, cols[: max(1, deg // 3)]])
        if unsorted:
            rng.shuffle(cols)
        elif dup:
            cols = np.sort(cols)
        rows.append(cols.astype(np.int32))
    rowPtr = np.zeros(N + 1, np.int32)
    rowPtr[1:] = np.cumsum([len(c) for c in rows])
    colIdx = np.concatenate(rows).astype(np.int32) if rowPtr[-1] else np.zeros(0, np.int32)
    return rowPtr, colIdx


@pytest.fixture(scope="session")
def oracle_mod():
    import oracle
    oracle.build()
    return oracle
