"""Helpers of the GPU parity tests: PCSR formats on the device and calls through the C ABI (ctypes)."""
import numpy as np
import torch

from paramspmm_ae_amd import _capi

L = _capi.lib


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def stream():
    return torch.cuda.current_stream().cuda_stream


class Formats:
    """CSR + split + 2x1 BCSR + split of one matrix, host (numpy, built by the oracle) and device copies."""

    def __init__(self, oracle, rowPtr, colIdx, val, g=None, gb=None):
        self.n = rowPtr.size - 1
        self.nnz = colIdx.size
        k = np.diff(rowPtr)
        nz = max(1, int(np.count_nonzero(k)))
        self.g = g or int(np.ceil(max(self.nnz, 1) / nz / 32) * 32)
        self.rowPtr, self.colIdx, self.val = rowPtr, colIdx, val
        self.rps, self.tr = oracle.split_csr(rowPtr, self.g)
        self.rpb, self.cib, self.vb = oracle.bcsr_build(rowPtr, colIdx, val, ncols=self.n + (self.n & 1))
        nzb = max(1, int(np.count_nonzero(np.diff(self.rpb))))
        self.gb = gb or int(np.ceil(max(self.cib.size, 1) / nzb / 32) * 32)
        self.rpbs, self.trb = oracle.split_csr(self.rpb, self.gb)
        self.d = {k_: dev(getattr(self, k_)) for k_ in
                  ("rowPtr", "colIdx", "val", "rps", "tr", "rpb", "cib", "vb", "rpbs", "trb")}


def spmm_capi(fmt, F, X, CF=1, bw=4, poison=True):
    """fmt in csr|csr_split|bcsr|bcsr_split; X a cuda tensor [rows, N]; returns Y (cuda)."""
    d = F.d
    N = X.shape[1]
    blocked = fmt.startswith("bcsr")
    rows_out = (X.shape[0] + 1) // 2 * 2 if blocked else X.shape[0]
    Y = torch.empty(rows_out, N, device="cuda")
    if poison:
        Y.fill_(float("nan"))  # the library must define every element
    p = _capi.ptr
    if fmt == "csr":
        rc = L.psp_spmm_csr_f32(p(d["rowPtr"]), p(d["colIdx"]), p(d["val"]), p(X), p(Y), F.n, N, rows_out, CF, bw, stream())
    elif fmt == "csr_split":
        rc = L.psp_spmm_csr_split_f32(p(d["rps"]), p(d["colIdx"]), p(d["val"]), p(d["tr"]), p(X), p(Y),
                                      F.tr.size, N, rows_out, CF, bw, stream())
    elif fmt == "bcsr":
        rc = L.psp_spmm_bcsr_f32(p(d["rpb"]), p(d["cib"]), p(d["vb"]), p(X), p(Y), F.rpb.size - 1, N, rows_out, CF, bw, stream())
    else:
        rc = L.psp_spmm_bcsr_split_f32(p(d["rpbs"]), p(d["cib"]), p(d["vb"]), p(d["trb"]), p(X), p(Y),
                                       F.trb.size, N, rows_out, CF, bw, stream())
    _capi.check(rc)
    return Y


def spmm_oracle(oracle, fmt, F, X):
    if fmt == "csr":
        return oracle.spmm_csr(F.rowPtr, F.colIdx, F.val, X)
    if fmt == "csr_split":
        return oracle.spmm_csr_split(F.rps, F.colIdx, F.val, F.tr, X)
    if fmt == "bcsr":
        return oracle.spmm_bcsr(F.rpb, F.cib, F.vb, X)
    return oracle.spmm_bcsr_split(F.rpbs, F.cib, F.vb, F.trb, X)


def sddmm_capi(fmt, F, A, B, bw=4, scale=None):
    d = F.d
    K = A.shape[1]
    p = _capi.ptr
    if fmt.startswith("bcsr"):
        out = torch.full((F.cib.size, 2), float("nan"), device="cuda")
    else:
        out = torch.full((F.nnz,), float("nan"), device="cuda")
    if fmt == "csr":
        rc = L.psp_sddmm_csr_f32(p(d["rowPtr"]), p(d["colIdx"]), p(A), p(B), p(scale), p(out), F.n, K, bw, stream())
    elif fmt == "csr_split":
        rc = L.psp_sddmm_csr_split_f32(p(d["rps"]), p(d["colIdx"]), p(d["tr"]), p(A), p(B), p(scale), p(out),
                                       F.tr.size, K, bw, stream())
    elif fmt == "bcsr":
        rc = L.psp_sddmm_bcsr_f32(p(d["rpb"]), p(d["cib"]), p(d["vb"]), p(A), p(B), p(out), F.rpb.size - 1, K, bw, stream())
    else:
        rc = L.psp_sddmm_bcsr_split_f32(p(d["rpbs"]), p(d["cib"]), p(d["vb"]), p(d["trb"]), p(A), p(B), p(out),
                                        F.trb.size, K, bw, stream())
    _capi.check(rc)
    return out


def sddmm_oracle(oracle, fmt, F, A, B):
    if fmt == "csr":
        return oracle.sddmm_csr(F.rowPtr, F.colIdx, A, B)
    if fmt == "csr_split":
        return oracle.sddmm_csr_split(F.rps, F.colIdx, F.tr, A, B)
    if fmt == "bcsr":
        return oracle.sddmm_bcsr(F.rpb, F.cib, F.vb, A, B)
    return oracle.sddmm_bcsr_split(F.rpbs, F.cib, F.vb, F.trb, A, B)


def spmm_abs_scale(oracle, F, X, rows_out):
    """(|A| |X|): the magnitude a row's terms add up to.  A long row is summed piecewise (lane groups of a
    wavefront each take a share of it; row-split formats add segments with atomics in no fixed order, as the
    reference does), so the rounding error scales with this sum of magnitudes and not with the possibly
    cancelled result."""
    return oracle.spmm_csr(F.rowPtr, F.colIdx, np.abs(F.val), np.abs(X), rows_out=rows_out)


def assert_close(got, want, rtol=1e-5, atol=1e-6, what="", scale=None):
    """north-star tolerance: |got - want| <= atol + rtol*|want| element-wise (fp32).  ``scale`` replaces |want|
    in the relative term (see spmm_abs_scale)."""
    got = got.detach().cpu().numpy() if hasattr(got, "detach") else np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    tol = atol + rtol * np.abs((want if scale is None else scale).astype(np.float64))
    bad = ~(err <= tol)  # catches NaN too
    if bad.any():
        i = np.unravel_index(np.argmax(np.where(bad, err / np.maximum(tol, 1e-30), 0)), err.shape)
        raise AssertionError("%s: %d of %d elements outside tolerance; worst at %s: got %r want %r" %
                             (what, int(bad.sum()), bad.size, i, got[i], want[i]))
