"""Seeded synthetic graphs for benchmarks, parity tests and decider training.

Every generator returns an undirected edge list without self loops (int64 arrays ``rows, cols`` holding each
edge once, ``rows < cols`` not required) plus the node count; ``to_gcn_csr`` turns it into the matrix the
reference's loader would build from a symmetric ``.mtx`` with ``is_normalize=True``
(graph_input.py:226-232, 366-379): pattern symmetrised, self loops added, values
``fp32(d_i^-1/2 * d_j^-1/2)`` computed in float64, CSR with sorted columns and int32 indices.
"""
import numpy as np


def _dedupe_undirected(u, v, n):
    keep = u != v
    u, v = u[keep], v[keep]
    lo = np.minimum(u, v)
    hi = np.maximum(u, v)
    key = np.unique(lo * np.int64(n) + hi)
    return key // n, key % n


def chung_lu(n, n_edges, exponent=2.1, max_degree=None, seed=0, permute=True):
    """Chung-Lu graph with a power-law expected-degree sequence w_i ~ (i + i0)^(-1/(exponent-1)).

    ``n_edges`` endpoints pairs are drawn with probability proportional to w_u * w_v, duplicates and self
    loops are dropped (so slightly fewer edges remain).  ``max_degree`` sets i0 so that the largest
    expected degree is about that value.  ``permute`` relabels the nodes at random so that hubs are not
    clustered at low ids.
    """
    rng = np.random.default_rng(seed)
    alpha = 1.0 / (exponent - 1.0)
    i0 = 1.0
    if max_degree is not None:
        # choose i0 by bisection: w_0 / sum(w) * 2 * n_edges = max_degree
        lo_, hi_ = 1e-3, float(n)
        for _ in range(60):
            mid = (lo_ + hi_) / 2
            w = (np.arange(n, dtype=np.float64) + mid) ** (-alpha)
            if w[0] / w.sum() * 2 * n_edges > max_degree:
                lo_ = mid
            else:
                hi_ = mid
        i0 = (lo_ + hi_) / 2
    w = (np.arange(n, dtype=np.float64) + i0) ** (-alpha)
    cdf = np.cumsum(w)
    cdf /= cdf[-1]
    u = np.searchsorted(cdf, rng.random(n_edges), side="right").astype(np.int64)
    v = np.searchsorted(cdf, rng.random(n_edges), side="right").astype(np.int64)
    np.minimum(u, n - 1, out=u)
    np.minimum(v, n - 1, out=v)
    if permute:
        perm = rng.permutation(n).astype(np.int64)
        u, v = perm[u], perm[v]
    r, c = _dedupe_undirected(u, v, n)
    return r, c, n


def rmat(scale, n_edges, a=0.57, b=0.19, c=0.19, seed=0):
    """R-MAT (Chakrabarti et al.) on 2^scale nodes: every edge picks one quadrant per bit level with
    probabilities (a, b, c, 1-a-b-c).  Duplicates and self loops are dropped."""
    rng = np.random.default_rng(seed)
    n = 1 << scale
    u = np.zeros(n_edges, np.int64)
    v = np.zeros(n_edges, np.int64)
    for _ in range(scale):
        r = rng.random(n_edges)
        row_bit = r >= a + b
        col_bit = ((r >= a) & (r < a + b)) | (r >= a + b + c)
        u = (u << 1) | row_bit
        v = (v << 1) | col_bit
    r_, c_ = _dedupe_undirected(u, v, n)
    return r_, c_, n


def sbm(n, n_communities, deg_in, deg_out, seed=0, permute=False):
    """Stochastic block model with equal communities of n/n_communities consecutive nodes: every node gets
    about ``deg_in`` neighbours inside its community and ``deg_out`` outside (edges drawn as endpoint
    pairs).  ``permute`` applies one random relabelling to rows and columns together."""
    rng = np.random.default_rng(seed)
    size = n // n_communities
    assert size * n_communities == n, "n must be a multiple of n_communities"
    m_in = int(n * deg_in / 2)
    m_out = int(n * deg_out / 2)
    u_in = rng.integers(0, n, m_in, dtype=np.int64)
    v_in = (u_in // size) * size + rng.integers(0, size, m_in, dtype=np.int64)
    u_out = rng.integers(0, n, m_out, dtype=np.int64)
    v_out = rng.integers(0, n, m_out, dtype=np.int64)
    u = np.concatenate([u_in, u_out])
    v = np.concatenate([v_in, v_out])
    if permute:
        perm = rng.permutation(n).astype(np.int64)
        u, v = perm[u], perm[v]
    r, c = _dedupe_undirected(u, v, n)
    return r, c, n


def stencil2d(nx, ny):
    """5-point stencil on an nx-by-ny grid (node id = y*nx + x): the regular, uniform-degree case."""
    idx = np.arange(nx * ny, dtype=np.int64).reshape(ny, nx)
    r = np.concatenate([idx[:, :-1].ravel(), idx[:-1, :].ravel()])
    c = np.concatenate([idx[:, 1:].ravel(), idx[1:, :].ravel()])
    return r, c, nx * ny


def to_gcn_csr(rows, cols, n):
    """Undirected edge list -> (rowPtr int32[n+1], colIdx int32[nnz], val fp32[nnz]) of D^-1/2 (A+I) D^-1/2."""
    rows = np.asarray(rows, np.int64)
    cols = np.asarray(cols, np.int64)
    diag = np.arange(n, dtype=np.int64)
    r = np.concatenate([rows, cols, diag])
    c = np.concatenate([cols, rows, diag])
    key = np.unique(r * np.int64(n) + c)
    r = key // n
    c = key % n
    counts = np.bincount(r, minlength=n)
    deg = counts.astype(np.float64)
    dis = np.power(deg, -0.5)  # deg >= 1 thanks to the self loop
    val = (dis[c] * dis[r]).astype(np.float32)
    rowPtr = np.zeros(n + 1, np.int64)
    np.cumsum(counts, out=rowPtr[1:])
    if rowPtr[-1] >= 2**31:
        raise ValueError("nnz does not fit int32")
    return rowPtr.astype(np.int32), c.astype(np.int32), val


def to_unit_csr(rows, cols, n, self_loops=False):
    """Undirected edge list -> symmetric pattern CSR with all values 1 (what load() builds without
    normalisation from a symmetric pattern file)."""
    rows = np.asarray(rows, np.int64)
    cols = np.asarray(cols, np.int64)
    parts_r, parts_c = [rows, cols], [cols, rows]
    if self_loops:
        d = np.arange(n, dtype=np.int64)
        parts_r.append(d)
        parts_c.append(d)
    key = np.unique(np.concatenate(parts_r) * np.int64(n) + np.concatenate(parts_c))
    r = key // n
    c = key % n
    rowPtr = np.zeros(n + 1, np.int64)
    np.cumsum(np.bincount(r, minlength=n), out=rowPtr[1:])
    return rowPtr.astype(np.int32), c.astype(np.int32), np.ones(key.size, np.float32)


# The five benchmark configurations, by short name.  Each returns (rowPtr, colIdx, val, n).
def config_graph(name, seed=None):
    if name == "C1":  # pubmed-like: 19,717 nodes, ~88,650 stored off-diagonal entries
        r, c, n = chung_lu(19717, 44500, exponent=2.1, max_degree=171, seed=11 if seed is None else seed)
    elif name == "C2":  # R-MAT scale 20, about 16 off-diagonal entries per row
        r, c, n = rmat(20, int(8.4 * (1 << 20)), seed=22 if seed is None else seed)
    elif name == "C3":  # large skewed Chung-Lu
        r, c, n = chung_lu(2_450_000, 62_000_000, exponent=2.1, max_degree=17000, seed=33 if seed is None else seed)
    elif name == "C3s":  # the regular case of C3: 2048 x 2048 5-point stencil
        r, c, n = stencil2d(2048, 2048)
    elif name == "C5":  # SBM, community-contiguous ordering
        r, c, n = sbm(1_000_000, 10_000, 20, 2, seed=55 if seed is None else seed, permute=False)
    elif name == "C5p":  # SBM, random ordering
        r, c, n = sbm(1_000_000, 10_000, 20, 2, seed=55 if seed is None else seed, permute=True)
    else:
        raise ValueError("unknown config " + name)
    rowPtr, colIdx, val = to_gcn_csr(r, c, n)
    return rowPtr, colIdx, val, n
