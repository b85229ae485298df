"""Double precision: the reference dispatches its SpMM / SDDMM kernels for float and double alike
(SpMM_kernel.cu:149, sddmm_kernel.cu:161).  All six layouts, through the C ABI and through the extension modules,
against float64 products computed by scipy / numpy.  Tolerance: 1e-13 relative to the sum of the magnitudes of a
result's terms (the order of a row's additions differs from scipy's, and split layouts add segments atomically)."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

from conftest import random_csr

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-13, 1e-300


def _matrix():
    rowPtr, colIdx, val = random_csr(1999, 8, 29, empty_frac=0.1, hub=(7, 1200))
    return rowPtr, colIdx, val.astype(np.float64) * (1.0 + 2.0 ** -40)  # values that float32 cannot hold


def _layouts(oracle, rowPtr, colIdx, val, R):
    """(rowPtr, colIdx, values [nblk, R] or [nnz], rows_out) of the vec_size-R layout; values stay float64"""
    n = rowPtr.size - 1
    if R == 1:
        return rowPtr, colIdx, val, n
    rows_out = (n + R - 1) // R * R
    # the builder is an index computation: run it on the entry numbers (exact in float32 up to 2^24, +1 so that no
    # stored entry reads as an empty slot), then put the float64 values where the numbers landed
    tag = np.arange(1, colIdx.size + 1, dtype=np.float32)
    rpb, cib, tb = oracle.vbsr_build(rowPtr, colIdx, tag, R, ncols=rows_out)
    vb = np.where(tb > 0, val[np.maximum(tb.astype(np.int64) - 1, 0)], 0.0)
    return rpb, cib, vb, rows_out


def _check(got, want, scale, what):
    got = got.cpu().numpy()
    assert got.dtype == np.float64 and got.shape == want.shape, (what, got.dtype, got.shape, want.shape)
    err = np.abs(got - want)
    bad = ~(err <= ATOL + RTOL * scale)
    assert not bad.any(), "%s: %d of %d outside tolerance, worst error %g" % (what, int(bad.sum()), bad.size, np.nanmax(err))


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("R", [1, 2, 3])
@pytest.mark.parametrize("N", [1, 16, 100, 200])
def test_spmm_f64(oracle, R, split, N):
    import paramspmm_ae_amd  # noqa: F401
    import ParamSpMM
    from paramspmm_ae_amd import _capi
    from gpu_util import dev, stream

    rowPtr, colIdx, val = _matrix()
    n = rowPtr.size - 1
    rp, ci, v, rows_out = _layouts(oracle, rowPtr, colIdx, val, R)
    X = np.random.default_rng(N).standard_normal((n, N))
    A = sp.csr_matrix((val, colIdx, rowPtr), shape=(n, n))
    want = np.zeros((rows_out, N))
    want[:n] = A @ X
    scale = np.zeros((rows_out, N))
    scale[:n] = abs(A) @ np.abs(X)
    Xp = np.zeros((rows_out, N))
    Xp[:n] = X
    tr = None
    if split:
        rp, tr = oracle.split_csr(rp, 8)
    L, p = _capi.lib, _capi.ptr
    rp_d, ci_d, v_d, X_d = dev(rp), dev(ci), dev(v), dev(Xp)
    tr_d = dev(tr) if split else None
    Y = torch.full((rows_out, N), float("nan"), dtype=torch.float64, device="cuda")
    _capi.check(L.psp_spmm_f64(p(rp_d), p(ci_d), p(v_d), p(tr_d), p(X_d), p(Y), rp.size - 1, N, rows_out, R, stream()))
    torch.cuda.synchronize()
    _check(Y, want, scale, "C ABI spmm f64 R=%d split=%s N=%d" % (R, split, N))

    # the extension modules take the same tensors (input rows as the caller has them; blocked results are padded)
    Xn = dev(X)
    if R == 1:
        Ym = ParamSpMM.csr_split_spmm(Xn, rp_d, ci_d, v_d, tr_d, 1, 4) if split else ParamSpMM.csr_spmm(Xn, rp_d, ci_d, v_d, 1, 4)
    elif R == 2:
        Ym = ParamSpMM.bcsr_split_spmm(Xn, rp_d, ci_d, v_d, tr_d, 1, 4) if split else ParamSpMM.bcsr_spmm(Xn, rp_d, ci_d, v_d, 1, 4)
    else:
        Ym = ParamSpMM.vec_split_spmm(Xn, rp_d, ci_d, v_d, tr_d, 1, 4) if split else ParamSpMM.vec_spmm(Xn, rp_d, ci_d, v_d, 1, 4)
    rows_mod = (n + R - 1) // R * R
    _check(Ym, want[:rows_mod], scale[:rows_mod], "module spmm f64 R=%d split=%s N=%d" % (R, split, N))


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("R", [1, 2, 3])
@pytest.mark.parametrize("K", [1, 32, 100])
def test_sddmm_f64(oracle, R, split, K):
    import paramspmm_ae_amd  # noqa: F401
    import ParamSDDMM
    from paramspmm_ae_amd import _capi
    from gpu_util import dev, stream

    rowPtr, colIdx, val = _matrix()
    n = rowPtr.size - 1
    rp, ci, v, rows = _layouts(oracle, rowPtr, colIdx, val, R)
    rng = np.random.default_rng(K)
    A, B = rng.standard_normal((rows, K)), rng.standard_normal((rows, K))
    seg_row = np.repeat(np.arange(rp.size - 1), np.diff(rp))  # block-row (row for R = 1) of each stored entry
    if R == 1:
        want = np.einsum("pk,pk->p", A[seg_row], B[ci])
        scale = np.einsum("pk,pk->p", np.abs(A[seg_row]), np.abs(B[ci]))
    else:
        Ar = A.reshape(rows // R, R, K)[seg_row]  # [nblk, R, K]
        want = np.where(v != 0, np.einsum("prk,pk->pr", Ar, B[ci]), 0.0)
        scale = np.einsum("prk,pk->pr", np.abs(Ar), np.abs(B[ci]))
    tr = None
    if split:
        rp, tr = oracle.split_csr(rp, 8)
    L, p = _capi.lib, _capi.ptr
    rp_d, ci_d, v_d, A_d, B_d = dev(rp), dev(ci), dev(v), dev(A), dev(B)
    tr_d = dev(tr) if split else None
    out = torch.full(v.shape, float("nan"), dtype=torch.float64, device="cuda")
    _capi.check(L.psp_sddmm_f64(p(rp_d), p(ci_d), p(v_d) if R > 1 else None, p(tr_d), p(A_d), p(B_d), p(out), rp.size - 1,
                                K, R, stream()))
    torch.cuda.synchronize()
    _check(out, want, scale, "C ABI sddmm f64 R=%d split=%s K=%d" % (R, split, K))

    if R == 1:
        om = (ParamSDDMM.csr_split_sddmm(A_d, B_d, rp_d, ci_d, v_d, tr_d, 1, 4) if split
              else ParamSDDMM.csr_sddmm(A_d, B_d, rp_d, ci_d, v_d, 1, 4))
    elif R == 2:
        om = (ParamSDDMM.bcsr_split_sddmm(A_d, B_d, rp_d, ci_d, v_d, tr_d, 1, 4) if split
              else ParamSDDMM.bcsr_sddmm(A_d, B_d, rp_d, ci_d, v_d, 1, 4))
    else:
        om = (ParamSDDMM.vec_split_sddmm(A_d, B_d, rp_d, ci_d, v_d, tr_d, 1, 4) if split
              else ParamSDDMM.vec_sddmm(A_d, B_d, rp_d, ci_d, v_d, 1, 4))
    _check(om, want, scale, "module sddmm f64 R=%d split=%s K=%d" % (R, split, K))


def test_f64_edges():
    """no segments, no columns, a bad block height: defined results or argument errors, nothing launched out of range"""
    from paramspmm_ae_amd import _capi
    from gpu_util import stream

    L, p = _capi.lib, _capi.ptr
    rp = torch.zeros(5, dtype=torch.int32, device="cuda")
    ci = torch.zeros(1, dtype=torch.int32, device="cuda")
    v = torch.zeros(1, dtype=torch.float64, device="cuda")
    X = torch.ones(4, 8, dtype=torch.float64, device="cuda")
    Y = torch.full((4, 8), float("nan"), dtype=torch.float64, device="cuda")
    _capi.check(L.psp_spmm_f64(p(rp), p(ci), p(v), None, p(X), p(Y), 4, 8, 4, 1, stream()))  # four empty rows
    torch.cuda.synchronize()
    assert torch.count_nonzero(Y) == 0
    Y.fill_(float("nan"))
    _capi.check(L.psp_spmm_f64(p(rp), p(ci), p(v), None, p(X), p(Y), 0, 8, 4, 1, stream()))  # no rows at all
    torch.cuda.synchronize()
    assert torch.count_nonzero(Y) == 0
    assert L.psp_spmm_f64(p(rp), p(ci), p(v), None, p(X), p(Y), 4, 8, 4, 4, None) == -1
    assert L.psp_spmm_f64(p(rp), p(ci), p(v), None, p(X), p(Y), 4, 8, 3, 1, None) == -1  # Y too short for the rows
    assert L.psp_sddmm_f64(p(rp), p(ci), None, None, p(X), p(X), p(v), 4, 8, 2, None) == -1  # blocks without values
    _capi.check(L.psp_sddmm_f64(p(rp), p(ci), None, None, p(X), p(X), p(v), 0, 8, 1, stream()))
