import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def has_gpu() -> bool:
    try:
        import npeff_ref_amd as d

        return d.device_count() > 0
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def tune():
    """tune(name, value) sets a switch of the library (dnpeff_tuning_set) for the test; all
    switches go back to their starting values afterwards."""
    import npeff_ref_amd as d

    yield d.tuning_set
    d.tuning_reset()


@pytest.fixture(scope="session")
def golden():
    import json

    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


def random_csr(rng, n_rows, n_cols, max_row_nnz, empty_rows=(), sort_cols=False):
    """Random CSR with distinct, unsorted column ids per row and a few empty rows."""
    rowptr = [0]
    cols, vals = [], []
    for i in range(n_rows):
        k = 0 if i in empty_rows else int(rng.integers(0, min(max_row_nnz, n_cols) + 1))
        c = rng.choice(n_cols, size=k, replace=False).astype(np.int32)
        if sort_cols:
            c.sort()
        cols.append(c)
        vals.append(rng.lognormal(-2.0, 1.0, size=k).astype(np.float32))
        rowptr.append(rowptr[-1] + k)
    colind = np.concatenate(cols) if cols else np.zeros(0, np.int32)
    v = np.concatenate(vals) if vals else np.zeros(0, np.float32)
    return np.array(rowptr, dtype=np.int64), colind.astype(np.int32), v.astype(np.float32)


def csr_to_dense(rowptr, colind, vals, n_cols, dtype=np.float64):
    n = len(rowptr) - 1
    D = np.zeros((n, n_cols), dtype=dtype)
    for i in range(n):
        for e in range(rowptr[i], rowptr[i + 1]):
            D[i, colind[e]] += vals[e]
    return D
