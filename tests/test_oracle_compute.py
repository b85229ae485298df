"""Pins the arithmetic half of the CPU oracle: SpMM against torch.sparse.mm (the reference's own checker,
verification.py:18-46), an fp64 dense product and the X = ones known answer; SDDMM against fp64 gathered dot
products and the A = B = ones known answer (SDDMM.py:127-128); softmax against its closed form."""
import numpy as np
import pytest
import torch

from conftest import random_csr

RTOL, ATOL = 1e-5, 1e-6


def dense_of(rowPtr, colIdx, val, n):
    A = np.zeros((n, n), np.float64)
    rows = np.repeat(np.arange(n), np.diff(rowPtr))
    np.add.at(A, (rows, colIdx), val.astype(np.float64))
    return A


def formats(oracle, rowPtr, colIdx, val, g=4):
    rps, tr = oracle.split_csr(rowPtr, g)
    rpb, cib, vb = oracle.bcsr_build(rowPtr, colIdx, val)
    rpbs, trb = oracle.split_csr(rpb, g)
    return rps, tr, rpb, cib, vb, rpbs, trb


@pytest.mark.parametrize("n,N", [(1, 4), (37, 16), (64, 33), (200, 128)])
def test_spmm_four_formats_vs_dense_fp64_and_torch(oracle, n, N):
    rowPtr, colIdx, val = random_csr(n, min(8, n), n + N, empty_frac=0.1, hub=(0, min(n, 60)), values="uniform")
    rng = np.random.default_rng(1)
    X = rng.standard_normal((n, N)).astype(np.float32)
    ref = dense_of(rowPtr, colIdx, val, n) @ X.astype(np.float64)
    rps, tr, rpb, cib, vb, rpbs, trb = formats(oracle, rowPtr, colIdx, val)
    Xp = np.vstack([X, np.zeros(((n & 1), N), np.float32)])  # bcsr wants an even row count on the output side
    outs = {
        "csr": oracle.spmm_csr(rowPtr, colIdx, val, X),
        "csr_split": oracle.spmm_csr_split(rps, colIdx, val, tr, X),
        "bcsr": oracle.spmm_bcsr(rpb, cib, vb, X)[:n],
        "bcsr_split": oracle.spmm_bcsr_split(rpbs, cib, vb, trb, X)[:n],
    }
    for name, y in outs.items():
        assert y.dtype == np.float32
        np.testing.assert_allclose(y, ref, rtol=RTOL, atol=ATOL * 10, err_msg=name)
    s = torch.sparse_csr_tensor(torch.from_numpy(rowPtr), torch.from_numpy(colIdx), torch.from_numpy(val), size=(n, n))
    t = torch.sparse.mm(s, torch.from_numpy(X)).numpy()
    np.testing.assert_allclose(outs["csr"], t, rtol=RTOL, atol=ATOL * 10)
    assert Xp.shape[0] % 2 == 0


def test_spmm_ones_gives_row_sums_and_padding_rows_zero(oracle):
    n = 51
    rowPtr, colIdx, val = random_csr(n, 6, 9, empty_frac=0.2, values="uniform")
    X = np.ones((n, 16), np.float32)
    rs = np.array([val[rowPtr[i]:rowPtr[i + 1]].astype(np.float64).sum() for i in range(n)])
    y = oracle.spmm_csr(rowPtr, colIdx, val, X)
    np.testing.assert_allclose(y, np.repeat(rs[:, None], 16, 1), rtol=1e-5, atol=1e-6)
    assert np.all(y[np.diff(rowPtr) == 0] == 0)
    rpb, cib, vb = oracle.bcsr_build(rowPtr, colIdx, val)
    yb = oracle.spmm_bcsr(rpb, cib, vb, X)
    assert yb.shape == (52, 16) and np.all(yb[51] == 0)
    np.testing.assert_allclose(yb[:n], y, rtol=1e-6, atol=1e-7)


def test_spmm_is_linear_and_order_matches_sequential_fma(oracle):
    n, N = 40, 8
    rowPtr, colIdx, val = random_csr(n, 5, 2)
    rng = np.random.default_rng(3)
    X1, X2 = rng.standard_normal((2, n, N)).astype(np.float32)
    y = oracle.spmm_csr(rowPtr, colIdx, val, X1 + X2)
    np.testing.assert_allclose(y, oracle.spmm_csr(rowPtr, colIdx, val, X1) + oracle.spmm_csr(rowPtr, colIdx, val, X2),
                               rtol=1e-4, atol=1e-5)
    # one row, by hand: fp32 fused multiply-add in storage order, emulated in float64 (exact product, one rounding)
    r = int(np.argmax(np.diff(rowPtr)))
    acc = np.float32(0)
    for p in range(rowPtr[r], rowPtr[r + 1]):
        acc = np.float32(np.float64(val[p]) * np.float64(X1[colIdx[p], 0]) + np.float64(acc))
    assert oracle.spmm_csr(rowPtr, colIdx, val, X1)[r, 0] == acc


@pytest.mark.parametrize("n,K", [(2, 1), (33, 32), (50, 64), (41, 100), (20, 128)])
def test_sddmm_four_formats_vs_gathered_fp64(oracle, n, K):
    rowPtr, colIdx, val = random_csr(n, min(6, n), K, empty_frac=0.1, values="uniform")
    rng = np.random.default_rng(2)
    m = n + (n & 1)
    A = rng.standard_normal((m, K)).astype(np.float32)
    B = rng.standard_normal((n, K)).astype(np.float32)
    A /= np.linalg.norm(A, axis=1, keepdims=True)
    B /= np.linalg.norm(B, axis=1, keepdims=True)
    rows = np.repeat(np.arange(n), np.diff(rowPtr))
    ref = (A[rows].astype(np.float64) * B[colIdx].astype(np.float64)).sum(1)
    rps, tr, rpb, cib, vb, rpbs, trb = formats(oracle, rowPtr, colIdx, val)
    mask = oracle.genmask(rpb, rowPtr, vb, colIdx.size)
    o_csr = oracle.sddmm_csr(rowPtr, colIdx, A, B)
    np.testing.assert_allclose(o_csr, ref, rtol=RTOL, atol=ATOL)
    np.testing.assert_array_equal(oracle.sddmm_csr_split(rps, colIdx, tr, A, B), o_csr)
    ob = oracle.sddmm_bcsr(rpb, cib, vb, A, B)
    assert ob.shape == vb.shape and np.all(ob[vb == 0] == 0)
    # flatten()[mask] brings block results back to CSR slots, up to the within-row order of odd rows
    back = ob.reshape(-1)[mask]
    for r in range(n):
        a, b = rowPtr[r], rowPtr[r + 1]
        np.testing.assert_allclose(np.sort(back[a:b]), np.sort(ref[a:b]), rtol=RTOL, atol=ATOL)
    np.testing.assert_array_equal(oracle.sddmm_bcsr_split(rpbs, cib, vb, trb, A, B), ob)


def test_sddmm_ones_gives_K(oracle):
    rowPtr, colIdx, val = random_csr(30, 4, 4)
    for K in (16, 32, 48, 128):
        A = np.ones((30, K), np.float32)
        assert np.all(oracle.sddmm_csr(rowPtr, colIdx, A, A) == K)


def test_sddmm_ignores_stored_values(oracle):
    rowPtr, colIdx, val = random_csr(30, 4, 4)
    A = np.random.default_rng(0).standard_normal((30, 32)).astype(np.float32)
    # the entry point takes no values at all for csr; for blocks only their zero pattern matters
    rpb, cib, vb = oracle.bcsr_build(rowPtr, colIdx, val)
    o1 = oracle.sddmm_bcsr(rpb, cib, vb, A, A)
    o2 = oracle.sddmm_bcsr(rpb, cib, np.where(vb != 0, 7.0, 0.0).astype(np.float32), A, A)
    np.testing.assert_array_equal(o1, o2)


def test_segment_softmax_closed_form(oracle):
    rowPtr, colIdx, val = random_csr(60, 5, 8, empty_frac=0.2, hub=(3, 50))
    e = np.random.default_rng(1).standard_normal(colIdx.size).astype(np.float32) * 4
    out = oracle.segment_softmax(rowPtr, e)
    for r in range(60):
        a, b = rowPtr[r], rowPtr[r + 1]
        if a == b:
            continue
        z = np.exp(e[a:b].astype(np.float64) - e[a:b].max())
        np.testing.assert_allclose(out[a:b], z / z.sum(), rtol=1e-6)
        assert abs(out[a:b].sum() - 1) < 1e-5


@pytest.mark.parametrize("R", [2, 3])
def test_spmm_vec_blocks(oracle, R):
    """R x 1 blocks: every output row sees its own entries in CSR order (a block-row lists row R*t's columns first,
    each row's entries stay ascending), so the result equals the CSR product bit for bit; R = 2 equals the 2 x 1
    functions; the row-split variant adds the segments' partial sums."""
    rowPtr, colIdx, val = random_csr(203, 6.0, seed=5, empty_frac=0.1, hub=(7, 150))
    n = rowPtr.size - 1
    X = np.random.default_rng(1).standard_normal((n + R, 24)).astype(np.float32)
    rpb, cib, vb = oracle.vbsr_build(rowPtr, colIdx, val, R)
    Y = oracle.spmm_vec(rpb, cib, vb, X)
    want = oracle.spmm_csr(rowPtr, colIdx, val, X)
    assert Y.shape[0] % R == 0 and Y.shape[0] >= n
    # within a block-row the blocks are not column-sorted for rows after the first, so only row R*t is the same chain
    assert np.array_equal(Y[0:n:R], want[0:n:R])
    np.testing.assert_allclose(Y[:n], want[:n], rtol=1e-5, atol=1e-6)
    assert not Y[n:].any()
    dense = np.zeros((n, n + R))
    rows = np.repeat(np.arange(n), np.diff(rowPtr))
    dense[rows, colIdx] = val
    np.testing.assert_allclose(Y[:n], dense @ X.astype(np.float64), rtol=1e-5, atol=1e-5)
    if R == 2:
        assert np.array_equal(Y, oracle.spmm_bcsr(rpb, cib, vb, X, rows_out=Y.shape[0]))
    rps, tr = oracle.split_csr(rpb, 4)
    Ys = oracle.spmm_vec(rps, cib, vb, X, target_row=tr, rows_out=Y.shape[0])
    np.testing.assert_allclose(Ys, Y, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("R", [2, 3])
def test_sddmm_vec_blocks(oracle, R):
    """R x 1 blocks: R = 2 equals the 2 x 1 functions; every non-zero entry equals the fp64 dot product of its row of
    A and column row of B, padding entries are zero; the row-split variant gives the same array."""
    rowPtr, colIdx, val = random_csr(120, 5.0, seed=9, empty_frac=0.1)
    n = rowPtr.size - 1
    npad = (n + R - 1) // R * R
    rpb, cib, vb = oracle.vbsr_build(rowPtr, colIdx, val, R)
    rng = np.random.default_rng(2)
    A = rng.standard_normal((npad, 40)).astype(np.float32)
    B = rng.standard_normal((npad, 40)).astype(np.float32)
    out = oracle.sddmm_vec(rpb, cib, vb, A, B)
    assert out.shape == vb.shape
    blk_row = np.repeat(np.arange(rpb.size - 1), np.diff(rpb))
    for q in range(R):
        want = np.einsum("ij,ij->i", A[R * blk_row + q].astype(np.float64), B[cib].astype(np.float64))
        nz = vb[:, q] != 0
        np.testing.assert_allclose(out[nz, q], want[nz], rtol=1e-5, atol=1e-5)
        assert not out[~nz, q].any()
    if R == 2:
        assert np.array_equal(out, np.asarray(oracle.sddmm_bcsr(rpb, cib, vb, A, B)).reshape(-1, 2))
    rps, tr = oracle.split_csr(rpb, 3)
    assert np.array_equal(oracle.sddmm_vec(rps, cib, vb, A, B, target_row=tr), out)
