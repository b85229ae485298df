"""Locality-restoring vertex orders, applied once when a graph is loaded: rows and columns of the matrix are permuted
together (A' = P A P^T, still symmetric where A was), and features, labels and results are moved with
``permute_rows`` / ``unpermute_rows``.

The reference's inputs are pre-ordered outside its repository (Rabbit order, README.md:14-16,71; its data ship both
as pubmed.mtx and pubmed_rabbit.mtx); this module is the in-tree counterpart for graphs that arrive unordered.

  community_permutation  label propagation, then vertices sorted by label: the members of a community become
                         neighbours in memory, so the X rows a block of sparse rows gathers sit in a few cache lines
                         and stay in the L2 while the block is worked on.  A stochastic block model in random order
                         gets its community order back; a graph without communities (R-MAT, Chung-Lu) collapses to one
                         label and keeps its order.
  degree_permutation     hubs first: the X rows that most entries gather become one contiguous range.

Everything is written with torch tensor operations (sort, unique_consecutive, scatter_reduce) and runs on the GPU when
there is one -- a round of label propagation on 21 M entries is two sorts -- and on the host otherwise."""
import numpy as np
import torch


def _device(device):
    if device is not None:
        return torch.device(device)
    return torch.device("cuda" if torch.cuda.is_available() else "cpu")


def community_permutation(rowPtr, colIdx, rounds=12, device=None, min_change=1e-3):
    """perm (int64 numpy, new position -> old vertex) that makes the vertices of one label-propagation community
    contiguous.  ``rounds``: upper bound on propagation rounds; a round updates every other vertex (by parity of
    vertex + round), which keeps synchronous propagation from oscillating; it stops early once fewer than
    ``min_change`` of the vertices change label."""
    dev = _device(device)
    rp = torch.as_tensor(np.ascontiguousarray(rowPtr, np.int64), device=dev)
    cols = torch.as_tensor(np.ascontiguousarray(colIdx, np.int64), device=dev)
    n = rp.numel() - 1
    if n == 0:
        return np.zeros(0, np.int64)
    rows = torch.repeat_interleave(torch.arange(n, device=dev), rp[1:] - rp[:-1])
    label = torch.arange(n, device=dev)
    ids = torch.arange(n, device=dev)
    for it in range(rounds):
        key, _ = torch.sort(rows * n + label[cols])
        uniq, counts = torch.unique_consecutive(key, return_counts=True)
        urow, ulab = uniq // n, uniq % n
        # the most frequent neighbour label of every vertex; ties go to the smallest label
        score = counts * n + (n - 1 - ulab)
        best = torch.full((n,), -1, dtype=torch.int64, device=dev).scatter_reduce(0, urow, score, reduce="amax")
        new = torch.where(best >= 0, n - 1 - best % n, label)
        turn = ((ids + it) & 1) == 0
        new = torch.where(turn, new, label)
        changed = int((new != label).sum())
        label = new
        if changed < min_change * n:
            break
    # communities in the order of their smallest member, members in their old order
    first = torch.full((n,), n, dtype=torch.int64, device=dev).scatter_reduce(0, label, ids, reduce="amin")
    perm = torch.argsort(first[label] * n + ids)
    return perm.cpu().numpy()


def degree_permutation(rowPtr):
    """perm (new position -> old vertex): vertices by falling degree, ties in their old order."""
    k = np.diff(np.asarray(rowPtr, np.int64))
    return np.argsort(-k, kind="stable").astype(np.int64)


def permute_csr(rowPtr, colIdx, val, perm, device=None):
    """(rowPtr', colIdx', val') of P A P^T for perm (new position -> old vertex): row i of the result is old row
    perm[i] with its columns renamed and sorted again."""
    dev = _device(device)
    rp = torch.as_tensor(np.ascontiguousarray(rowPtr, np.int64), device=dev)
    n = rp.numel() - 1
    p = torch.as_tensor(np.ascontiguousarray(perm, np.int64), device=dev)
    if p.numel() != n or (n and not bool((torch.sort(p).values == torch.arange(n, device=dev)).all())):
        raise ValueError("perm must be a permutation of the %d vertices" % n)
    inv = torch.empty_like(p)
    inv[p] = torch.arange(n, device=dev)
    deg = rp[1:] - rp[:-1]
    rows = torch.repeat_interleave(torch.arange(n, device=dev), deg)
    cols = torch.as_tensor(np.ascontiguousarray(colIdx, np.int64), device=dev)
    key = inv[rows] * n + inv[cols]
    order = torch.argsort(key)
    new_rp = torch.zeros(n + 1, dtype=torch.int64, device=dev)
    new_rp[1:] = torch.cumsum(deg[p], 0)
    new_cols = (key[order] % n).to(torch.int32)
    v = torch.as_tensor(np.ascontiguousarray(val), device=dev)[order]
    return new_rp.to(torch.int32).cpu().numpy(), new_cols.cpu().numpy(), v.cpu().numpy()


def inverse(perm):
    inv = np.empty_like(perm)
    inv[perm] = np.arange(perm.size, dtype=perm.dtype)
    return inv


def permute_rows(t, perm):
    """rows of a per-vertex tensor / array in the new order: out[i] = t[perm[i]] (rows past len(perm) -- padding --
    stay where they are)"""
    idx = torch.as_tensor(perm, device=t.device) if isinstance(t, torch.Tensor) else perm
    if t.shape[0] == len(perm):
        return t[idx]
    out = t.clone() if isinstance(t, torch.Tensor) else t.copy()
    out[: len(perm)] = t[idx]
    return out


def unpermute_rows(t, perm):
    """the inverse of permute_rows: a result computed in the new order back in the old one"""
    return permute_rows(t, inverse(np.asarray(perm)))
