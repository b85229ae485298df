"""Pins the index-construction half of the CPU oracle (row split, 2x1 BCSR, genmask) against brute force,
closed forms, SciPy's tobsr (the routine the reference calls) and the counts of the reference's pubmed data."""
import numpy as np
import pytest
import scipy.sparse as sp

from conftest import pubmed_pattern, random_csr


def brute_split(rowPtr, g):
    rps, tr = [0], []
    for i in range(len(rowPtr) - 1):
        lb, hb = int(rowPtr[i]), int(rowPtr[i + 1])
        while lb < hb:
            tr.append(i)
            lb = min(lb + g, hb)
            rps.append(lb)
    return np.array(rps, np.int32), np.array(tr, np.int32)


@pytest.mark.parametrize("g", [1, 3, 32, 64])
@pytest.mark.parametrize("seed", [0, 1])
def test_split_matches_brute_force_and_closed_form(oracle, g, seed):
    rowPtr, _, _ = random_csr(300, 20, seed, empty_frac=0.2, hub=(7, 250))
    rps, tr = oracle.split_csr(rowPtr, g)
    b_rps, b_tr = brute_split(rowPtr, g)
    assert np.array_equal(rps, b_rps) and np.array_equal(tr, b_tr)
    # closed form: row i contributes ceil(k_i/g) segments
    k = np.diff(rowPtr)
    s = -(-k // g)
    assert np.array_equal(tr, np.repeat(np.arange(k.size), s))
    assert rps[-1] == rowPtr[-1] and np.all(np.diff(rps) > 0) and np.all(np.diff(rps) <= g)
    # parallel twin gives the same answer
    off = np.concatenate([[0], np.cumsum(s)]).astype(np.int32)
    rps2, tr2 = oracle.split_csr_par(rowPtr, off, g)
    assert np.array_equal(rps, rps2) and np.array_equal(tr, tr2)


def test_split_empty_and_degenerate(oracle):
    rps, tr = oracle.split_csr(np.zeros(5, np.int32), 32)
    assert rps.tolist() == [0] and tr.size == 0
    rps, tr = oracle.split_csr(np.array([0, 32, 64, 65], np.int32), 32)
    assert rps.tolist() == [0, 32, 64, 65] and tr.tolist() == [0, 1, 2]


def scipy_bcsr(rowPtr, colIdx, val):
    """graph_input.py:245-266: pad to an even row count, tobsr((2,1)), squeeze the block values."""
    n = len(rowPtr) - 1
    m = n + (n & 1)
    indptr = np.concatenate([rowPtr, [rowPtr[-1]] * (m - n)])
    b = sp.csr_matrix((val, colIdx, indptr), shape=(m, m)).tobsr(blocksize=(2, 1))
    return b.indptr.astype(np.int32), b.indices.astype(np.int32), b.data.reshape(-1, 2).astype(np.float32)


@pytest.mark.parametrize("n", [1, 2, 7, 64, 301])
@pytest.mark.parametrize("seed", [0, 3])
def test_bcsr_matches_scipy_tobsr(oracle, n, seed):
    rowPtr, colIdx, val = random_csr(n, min(6, n), seed, empty_frac=0.15)
    rpb, cib, vb = oracle.bcsr_build(rowPtr, colIdx, val)
    s_rpb, s_cib, s_vb = scipy_bcsr(rowPtr, colIdx, val)
    assert np.array_equal(rpb, s_rpb) and np.array_equal(cib, s_cib) and np.array_equal(vb, s_vb)


def test_bcsr_hand_case_first_encounter_order(oracle):
    # rows {0:[1,5], 1:[0,5,7]}: row 0's columns first, then the columns only row 1 has -- not sorted
    rowPtr = np.array([0, 2, 5], np.int32)
    colIdx = np.array([1, 5, 0, 5, 7], np.int32)
    val = np.ones(5, np.float32)
    rpb, cib, vb = oracle.bcsr_build(rowPtr, colIdx, val, ncols=8)
    assert rpb.tolist() == [0, 4]
    assert cib.tolist() == [1, 5, 0, 7]
    assert vb.tolist() == [[1, 0], [1, 1], [0, 1], [0, 1]]


def brute_genmask(rpb, rp, vb, nnz):
    mask = np.zeros(nnz, np.int32)
    rp = np.concatenate([rp, [rp[-1]]])
    for t in range(len(rpb) - 1):
        cnt = [int(rp[2 * t]), int(rp[2 * t + 1])]
        for i in range(rpb[t], rpb[t + 1]):
            for k in (0, 1):
                if vb[i, k] != 0:
                    mask[cnt[k]] = 2 * i + k
                    cnt[k] += 1
    return mask


@pytest.mark.parametrize("n", [2, 9, 200])
def test_genmask_brute_force_and_invariants(oracle, n):
    rowPtr, colIdx, val = random_csr(n, min(5, n), 5, empty_frac=0.1, values="uniform")
    rpb, cib, vb = oracle.bcsr_build(rowPtr, colIdx, val)
    mask = oracle.genmask(rpb, rowPtr, vb, colIdx.size)
    assert np.array_equal(mask, brute_genmask(rpb, rowPtr, vb, colIdx.size))
    got = vb.reshape(-1)[mask]
    for r in range(n):
        a, b = rowPtr[r], rowPtr[r + 1]
        assert np.array_equal(np.sort(got[a:b]), np.sort(val[a:b]))  # a permutation inside the row
        if r % 2 == 0:
            assert np.array_equal(got[a:b], val[a:b])  # even rows keep CSR order
        # the block a slot points at carries a column of this row
        assert np.array_equal(np.sort(cib[mask[a:b] // 2]), colIdx[a:b])


# ---- counts of the reference's own data (toy_dataset/pubmed.mtx and its Rabbit-reordered twin) ---------
PUBMED = {"orig": dict(nblk=88469, S_bcsr=10293), "rabbit": dict(nblk=81018, S_bcsr=10240)}


@pytest.mark.parametrize("which", ["orig", "rabbit"])
def test_pubmed_counts(oracle, which):
    m = pubmed_pattern(which)
    n = m.shape[0]
    assert n == 19717 and m.nnz == 88651 and int((m.diagonal() != 0).sum()) == 3
    rowPtr, colIdx = m.indptr.astype(np.int32), m.indices.astype(np.int32)
    val = np.ones(m.nnz, np.float32)
    k = np.diff(rowPtr)
    assert k.max() == 171 and k.min() >= 1
    assert abs(m.nnz / n - 4.496) < 1e-3
    # granularity ceil(4.496/32)*32 = 32
    rps, tr = oracle.split_csr(rowPtr, 32)
    assert tr.size == 20005
    rpb, cib, vb = oracle.bcsr_build(rowPtr, colIdx, val)
    assert cib.size == PUBMED[which]["nblk"]
    s_rpb, s_cib, s_vb = scipy_bcsr(rowPtr, colIdx, val)
    assert np.array_equal(rpb, s_rpb) and np.array_equal(cib, s_cib) and np.array_equal(vb, s_vb)
    gb = int(np.ceil((cib.size / np.count_nonzero(np.diff(rpb))) / 32) * 32)
    assert gb == 32
    assert oracle.split_csr(rpb, gb)[1].size == PUBMED[which]["S_bcsr"]
    pack = m.nnz / (2 * cib.size)
    assert abs(pack - (0.501 if which == "orig" else 0.547)) < 1e-3
    if which == "orig":
        unsorted_rows = sum(1 for t in range(rpb.size - 1) if np.any(np.diff(cib[rpb[t]:rpb[t + 1]]) < 0))
        assert (unsorted_rows, rpb.size - 1) == (7680, 9859)
        mask = oracle.genmask(rpb, rowPtr, vb, m.nnz)
        assert int(np.count_nonzero(cib[mask // 2] != colIdx)) == 454
        # with the diagonal set, as the normalised loaders do
        m2 = m.tolil(); m2.setdiag(1); assert m2.tocsr().nnz == 108365


@pytest.mark.parametrize("R", [2, 3, 4])
@pytest.mark.parametrize("n", [1, 7, 300, 301, 302])
def test_vbsr_build_matches_scipy_tobsr(oracle, R, n):
    """R x 1 blocks in SciPy's tobsr((R,1)) order (what graph_input.py:243-266 produces for blk_size = R), rows
    padded to a multiple of R; R = 2 must equal the dedicated 2 x 1 builder."""
    import scipy.sparse as sp

    rowPtr, colIdx, val = random_csr(n, 5.0, seed=n + R, empty_frac=0.2)
    rpb, cib, vb = oracle.vbsr_build(rowPtr, colIdx, val, R)
    npad = (n + R - 1) // R * R
    ip = np.concatenate([rowPtr, [rowPtr[-1]] * (npad - n)]).astype(np.int32)
    bsr = sp.csr_matrix((val, colIdx, ip), shape=(npad, max(npad, n))).tobsr(blocksize=(R, 1))
    assert np.array_equal(rpb, bsr.indptr)
    assert np.array_equal(cib, bsr.indices)
    assert np.array_equal(vb, bsr.data.reshape(-1, R))
    if R == 2:
        a, b, c = oracle.bcsr_build(rowPtr, colIdx, val)
        assert np.array_equal(a, rpb) and np.array_equal(b, cib) and np.array_equal(np.asarray(c).reshape(-1, 2), vb)
