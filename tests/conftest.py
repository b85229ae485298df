import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def random_csr(n, avg_deg, seed, empty_frac=0.0, hub=None, values="normal"):
    """Square CSR with sorted, duplicate-free columns.  ``hub`` = (row, degree) plants one long row."""
    rng = np.random.default_rng(seed)
    deg = rng.poisson(avg_deg, n)
    if empty_frac:
        deg[rng.random(n) < empty_frac] = 0
    if hub is not None:
        deg[hub[0]] = hub[1]
    deg = np.minimum(deg, n)
    rowPtr = np.zeros(n + 1, np.int32)
    rowPtr[1:] = np.cumsum(deg)
    cols = np.concatenate([np.sort(rng.choice(n, d, replace=False)) for d in deg]) if rowPtr[-1] else np.zeros(0)
    if values == "normal":
        val = rng.standard_normal(cols.size)
    elif values == "ones":
        val = np.ones(cols.size)
    else:
        val = rng.uniform(0.1, 1.0, cols.size)
    return rowPtr, cols.astype(np.int32), val.astype(np.float32)


def pubmed_pattern(which="orig"):
    """Symmetric pattern of the reference's toy_dataset/pubmed(.mtx | _rabbit.mtx) as scipy CSR of ones."""
    import scipy.sparse as sp

    z = np.load(os.path.join(ROOT, "tests", "golden", "pubmed_pattern.npz"))
    n = int(z["n"])
    r, c = z[which + "_row"].astype(np.int64), z[which + "_col"].astype(np.int64)
    off = r != c
    rows = np.concatenate([r, c[off]])
    cols = np.concatenate([c, r[off]])
    m = sp.coo_matrix((np.ones(rows.size), (rows, cols)), shape=(n, n)).tocsr()
    m.sort_indices()
    return m


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as orc

    orc.build()
    return orc
