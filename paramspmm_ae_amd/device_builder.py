"""PCSR index construction on the GPU: row splitting and 2x1 BCSR through the device builders of
libparamsp_hip.so (``psp_split_csr_*_dev``, ``psp_bcsr_*_dev``).

The outputs equal those of the host builders (``ParamSpMM.split_csr_par`` / ``psp_bcsr_build``, which follow
SpMM/SpMM.cpp:42-75 and SciPy's ``tobsr`` as called in graph_input.py:243-256) bit for bit.  The BCSR builder needs
rows with strictly ascending column indices; for other input it raises ``NotCanonical`` and the caller uses the host
builder, which accepts any order.  torch is used for device memory only.
"""
import torch

from . import _capi


class NotCanonical(ValueError):
    """The CSR rows are not strictly ascending in their column indices."""


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _check_status(status, what):
    flags = int(status.item())  # synchronises with the builder kernels
    if flags & 4:
        raise ValueError("%s: rowPtr decreases, does not start at 0 or does not end at the entry count" % what)
    if flags & 8:
        raise ValueError("%s: a column index lies outside the matrix" % what)
    if flags & 16:
        raise ValueError("%s: target_row decreases or names a row outside the matrix" % what)
    if flags & 1:
        raise OverflowError("%s: more than 2^31-1 output entries" % what)
    if flags & 2:
        raise NotCanonical("%s: a row's column indices are not strictly ascending" % what)


def _dev_i32(t):
    if not (t.is_cuda and t.dtype == torch.int32 and t.is_contiguous()):
        raise ValueError("expected a contiguous int32 CUDA tensor")
    return t


def check_index(rowPtr, colIdx, ncols, target_row=None, target_rows=0, what="index arrays"):
    """Raises ValueError when the arrays (on the GPU) would make the kernels read or write outside their buffers."""
    rowPtr, colIdx = _dev_i32(rowPtr), _dev_i32(colIdx)
    if target_row is not None:
        target_row = _dev_i32(target_row)
    with torch.cuda.device(rowPtr.device):
        status = torch.zeros(1, dtype=torch.int32, device=rowPtr.device)
        _capi.check(_capi.lib.psp_check_index_dev(_capi.ptr(rowPtr), _capi.ptr(colIdx) if colIdx.numel() else None,
                                                  _capi.ptr(target_row), rowPtr.numel() - 1, colIdx.numel(), int(ncols),
                                                  int(target_rows), _capi.ptr(status), _stream()))
        _check_status(status, what)


def to_host(*tensors):
    """Device tensors -> host tensors through page-locked memory (several times the rate of a pageable copy; the
    host copies stay page-locked, which also speeds up any later upload)."""
    out = [torch.empty(t.shape, dtype=t.dtype, pin_memory=True) for t in tensors]
    for h, t in zip(out, tensors):
        h.copy_(t, non_blocking=True)
    torch.cuda.synchronize()
    return out


def split_csr_device(rowPtr, g):
    """(rowPtr_split [S+1], target_row [S]) as int32 CUDA tensors for segments of at most ``g`` entries."""
    rowPtr = _dev_i32(rowPtr)
    n = rowPtr.numel() - 1
    L, p = _capi.lib, _capi.ptr
    with torch.cuda.device(rowPtr.device):
        ws_ints = L.psp_scan_workspace_ints(n)
        ws = torch.empty(ws_ints, dtype=torch.int32, device=rowPtr.device)
        offsets = torch.empty(n + 1, dtype=torch.int32, device=rowPtr.device)
        status = torch.zeros(1, dtype=torch.int32, device=rowPtr.device)
        _capi.check(L.psp_split_csr_offsets_dev(p(rowPtr), n, int(g), p(offsets), p(ws), ws_ints, p(status), _stream()))
        _check_status(status, "split_csr")
        S = int(offsets[n].item())
        rowPtr_split = torch.empty(S + 1, dtype=torch.int32, device=rowPtr.device)
        target_row = torch.empty(S, dtype=torch.int32, device=rowPtr.device)
        _capi.check(L.psp_split_csr_fill_dev(p(rowPtr), p(offsets), n, int(g), S, p(rowPtr_split), p(target_row), _stream()))
    return rowPtr_split, target_row


def build_bcsr_device(rowPtr, colIdx, val):
    """CSR on the GPU (int32, int32, fp32) -> (rowPtr_b [ceil(n/2)+1], colIdx_b [nblk], val_b [nblk, 2]) on the GPU."""
    rowPtr, colIdx = _dev_i32(rowPtr), _dev_i32(colIdx)
    if not (val.is_cuda and val.dtype == torch.float32 and val.is_contiguous()):
        raise ValueError("expected a contiguous float32 CUDA tensor")
    n = rowPtr.numel() - 1
    nbr = (n + 1) // 2
    L, p = _capi.lib, _capi.ptr
    with torch.cuda.device(rowPtr.device):
        ws_ints = L.psp_scan_workspace_ints(nbr)
        ws = torch.empty(ws_ints, dtype=torch.int32, device=rowPtr.device)
        rowPtr_b = torch.empty(nbr + 1, dtype=torch.int32, device=rowPtr.device)
        status = torch.zeros(1, dtype=torch.int32, device=rowPtr.device)
        _capi.check(L.psp_bcsr_offsets_dev(p(rowPtr), p(colIdx), n, p(rowPtr_b), p(ws), ws_ints, p(status), _stream()))
        _check_status(status, "bcsr")
        nblk = int(rowPtr_b[nbr].item())
        colIdx_b = torch.empty(nblk, dtype=torch.int32, device=rowPtr.device)
        val_b = torch.empty((nblk, 2), dtype=torch.float32, device=rowPtr.device)
        _capi.check(L.psp_bcsr_fill_dev(p(rowPtr), p(colIdx), p(val), n, p(rowPtr_b), p(colIdx_b), p(val_b), _stream()))
    return rowPtr_b, colIdx_b, val_b
