"""Python face of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this
module, and only as the checker.  The shipped package never does.

Two parts:

* ctypes bindings of ``paramsp_oracle.c`` (row split, BCSR 2x1 build, genmask, SpMM x4, SDDMM x4,
  segment softmax) -- arrays in, arrays out, all numpy;
* numpy restatements of the reference's host arithmetic that has no C counterpart: adjacency
  normalisation, the per-format statistics / split granularity, the 15 decider features, the CF search
  space and the decider's class decoding.  Each cites the reference lines it follows.
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libparamsp_oracle.so")
_lib = None

_I = ctypes.POINTER(ctypes.c_int)
_F = ctypes.POINTER(ctypes.c_float)


def build(force=False):
    """Compile paramsp_oracle.c with gcc (make).  Building the checker is not using it."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "paramsp_oracle.c"))
    ):
        subprocess.check_call(["make", "-s", "-C", _HERE, "-B"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_split_csr.restype = ctypes.c_int
        _lib.orc_split_csr_par.restype = ctypes.c_int
        _lib.orc_bcsr_build.restype = ctypes.c_int
        _lib.orc_vbsr_build.restype = ctypes.c_int
    return _lib


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _pi(a):
    return None if a is None else a.ctypes.data_as(_I)


def _pf(a):
    return None if a is None else a.ctypes.data_as(_F)


# ------------------------------------------------------------------------------------------------
# Index construction
# ------------------------------------------------------------------------------------------------
def split_csr(rowPtr, g):
    """SpMM/SpMM.cpp:15-40 -> (rowPtr_split int32[S+1], target_row int32[S])."""
    rowPtr = _i32(rowPtr)
    n = rowPtr.size - 1
    S = lib().orc_split_csr(_pi(rowPtr), n, int(g), None, None)
    rps = np.empty(S + 1, np.int32)
    tr = np.empty(S, np.int32)
    lib().orc_split_csr(_pi(rowPtr), n, int(g), _pi(rps), _pi(tr))
    return rps, tr


def split_csr_par(rowPtr, row_split_offset, g):
    """SpMM/SpMM.cpp:42-75 (caller supplies the exclusive prefix of per-row segment counts)."""
    rowPtr = _i32(rowPtr)
    off = _i32(row_split_offset)
    n = rowPtr.size - 1
    S = int(off[n])
    rps = np.empty(S + 1, np.int32)
    tr = np.empty(S, np.int32)
    lib().orc_split_csr_par(_pi(rowPtr), _pi(off), n, int(g), _pi(rps), _pi(tr))
    return rps, tr


def bcsr_build(rowPtr, colIdx, val, ncols=None):
    """graph_input.py:243-266 + SciPy csr_tobsr order -> (rowPtr_b, colIdx_b, val_b[nblk,2])."""
    rowPtr, colIdx, val = _i32(rowPtr), _i32(colIdx), _f32(val)
    n = rowPtr.size - 1
    if ncols is None:
        ncols = max(n, int(colIdx.max()) + 1 if colIdx.size else 0)
    nblk = lib().orc_bcsr_build(_pi(rowPtr), _pi(colIdx), _pf(val), n, int(ncols), None, None, None)
    rpb = np.empty((n + 1) // 2 + 1, np.int32)
    cib = np.empty(nblk, np.int32)
    vb = np.empty((nblk, 2), np.float32)
    lib().orc_bcsr_build(_pi(rowPtr), _pi(colIdx), _pf(val), n, int(ncols), _pi(rpb), _pi(cib), _pf(vb))
    return rpb, cib, vb


def vbsr_build(rowPtr, colIdx, val, R, ncols=None):
    """graph_input.py:243-266 with blk_size = R -> (rowPtr_b, colIdx_b, val_b[nblk,R]) in SciPy tobsr((R,1)) order."""
    rowPtr, colIdx, val = _i32(rowPtr), _i32(colIdx), _f32(val)
    n = rowPtr.size - 1
    if ncols is None:
        ncols = max(n, int(colIdx.max()) + 1 if colIdx.size else 0)
    nblk = lib().orc_vbsr_build(_pi(rowPtr), _pi(colIdx), _pf(val), n, int(ncols), int(R), None, None, None)
    rpb = np.empty((n + R - 1) // R + 1, np.int32)
    cib = np.empty(nblk, np.int32)
    vb = np.empty((nblk, R), np.float32)
    lib().orc_vbsr_build(_pi(rowPtr), _pi(colIdx), _pf(val), n, int(ncols), int(R), _pi(rpb), _pi(cib), _pf(vb))
    return rpb, cib, vb


def spmm_vec(rowPtr_b, colIdx_b, val_b, X, target_row=None, rows_out=None):
    """SpMM/SpMM_kernel.cu:1653-1972: R x 1 blocks (R = val_b.shape[1]); row-split when target_row is given."""
    rowPtr_b, colIdx_b, val_b, X = _i32(rowPtr_b), _i32(colIdx_b), _f32(val_b), _f32(X)
    R = val_b.shape[1]
    S = rowPtr_b.size - 1
    nbr = S if target_row is None else (int(np.max(target_row)) + 1 if S else 0)
    if rows_out is None:
        rows_out = max(R * nbr, (X.shape[0] + R - 1) // R * R)
    Y = np.empty((rows_out, X.shape[1]), np.float32)
    tr = None if target_row is None else _pi(_i32(target_row))
    lib().orc_spmm_vec(_pi(rowPtr_b), _pi(colIdx_b), _pf(val_b), tr, _pf(X), _pf(Y), S, X.shape[1], rows_out, R)
    return Y


def sddmm_vec(rowPtr_b, colIdx_b, val_b, A, B, target_row=None):
    """SDDMM on R x 1 blocks (R = val_b.shape[1]) -> out[nblk, R]; zero where the block value is zero."""
    rowPtr_b, colIdx_b, val_b, A, B = _i32(rowPtr_b), _i32(colIdx_b), _f32(val_b), _f32(A), _f32(B)
    R, nblk = val_b.shape[1], colIdx_b.size
    out = np.empty((nblk, R), np.float32)
    tr = None if target_row is None else _pi(_i32(target_row))
    lib().orc_sddmm_vec(_pi(rowPtr_b), _pi(colIdx_b), _pf(val_b), tr, _pf(A), _pf(B), _pf(out), rowPtr_b.size - 1,
                        A.shape[1], nblk, R)
    return out


def genmask(rowPtr_b, rowPtr, val_b, nnz):
    """SDDMM/sddmm_kernel.cu:78-141 -> int32[nnz].  rowPtr must cover 2*len(block rows) rows."""
    rowPtr_b, rowPtr, val_b = _i32(rowPtr_b), _i32(rowPtr), _f32(val_b)
    nbr = rowPtr_b.size - 1
    if rowPtr.size < 2 * nbr + 1:  # odd row count: the padded last row is empty
        rowPtr = np.concatenate([rowPtr, np.full(2 * nbr + 1 - rowPtr.size, rowPtr[-1], np.int32)])
    mask = np.zeros(int(nnz), np.int32)
    lib().orc_genmask(_pi(rowPtr_b), _pi(rowPtr), _pf(val_b), nbr, _pi(mask))
    return mask


# ------------------------------------------------------------------------------------------------
# SpMM / SDDMM
# ------------------------------------------------------------------------------------------------
def spmm_csr(rowPtr, colIdx, val, X, rows_out=None):
    rowPtr, colIdx, val, X = _i32(rowPtr), _i32(colIdx), _f32(val), _f32(X)
    M, N = rowPtr.size - 1, X.shape[1]
    rows_out = X.shape[0] if rows_out is None else rows_out
    Y = np.empty((rows_out, N), np.float32)
    lib().orc_spmm_csr(_pi(rowPtr), _pi(colIdx), _pf(val), _pf(X), _pf(Y), M, N, rows_out)
    return Y


def spmm_csr_split(rowPtr_split, colIdx, val, target_row, X, rows_out=None):
    rps, colIdx, val, tr, X = _i32(rowPtr_split), _i32(colIdx), _f32(val), _i32(target_row), _f32(X)
    S, N = rps.size - 1, X.shape[1]
    rows_out = X.shape[0] if rows_out is None else rows_out
    Y = np.empty((rows_out, N), np.float32)
    lib().orc_spmm_csr_split(_pi(rps), _pi(colIdx), _pf(val), _pi(tr), _pf(X), _pf(Y), S, N, rows_out)
    return Y


def spmm_bcsr(rowPtr_b, colIdx_b, val_b, X, rows_out=None):
    rpb, cib, vb, X = _i32(rowPtr_b), _i32(colIdx_b), _f32(val_b), _f32(X)
    Mb, N = rpb.size - 1, X.shape[1]
    rows_out = (X.shape[0] + 1) // 2 * 2 if rows_out is None else rows_out
    Y = np.empty((rows_out, N), np.float32)
    lib().orc_spmm_bcsr(_pi(rpb), _pi(cib), _pf(vb), _pf(X), _pf(Y), Mb, N, rows_out)
    return Y


def spmm_bcsr_split(rowPtr_bs, colIdx_b, val_b, target_row, X, rows_out=None):
    rps, cib, vb, tr, X = _i32(rowPtr_bs), _i32(colIdx_b), _f32(val_b), _i32(target_row), _f32(X)
    Sb, N = rps.size - 1, X.shape[1]
    rows_out = (X.shape[0] + 1) // 2 * 2 if rows_out is None else rows_out
    Y = np.empty((rows_out, N), np.float32)
    lib().orc_spmm_bcsr_split(_pi(rps), _pi(cib), _pf(vb), _pi(tr), _pf(X), _pf(Y), Sb, N, rows_out)
    return Y


def sddmm_csr(rowPtr, colIdx, A, B):
    rowPtr, colIdx, A, B = _i32(rowPtr), _i32(colIdx), _f32(A), _f32(B)
    M, K, nnz = rowPtr.size - 1, A.shape[1], colIdx.size
    out = np.empty(nnz, np.float32)
    lib().orc_sddmm_csr(_pi(rowPtr), _pi(colIdx), _pf(A), _pf(B), _pf(out), M, K, nnz)
    return out


def sddmm_csr_split(rowPtr_split, colIdx, target_row, A, B):
    rps, colIdx, tr, A, B = _i32(rowPtr_split), _i32(colIdx), _i32(target_row), _f32(A), _f32(B)
    S, K, nnz = rps.size - 1, A.shape[1], colIdx.size
    out = np.empty(nnz, np.float32)
    lib().orc_sddmm_csr_split(_pi(rps), _pi(colIdx), _pi(tr), _pf(A), _pf(B), _pf(out), S, K, nnz)
    return out


def sddmm_bcsr(rowPtr_b, colIdx_b, val_b, A, B):
    rpb, cib, vb, A, B = _i32(rowPtr_b), _i32(colIdx_b), _f32(val_b), _f32(A), _f32(B)
    Mb, K, nblk = rpb.size - 1, A.shape[1], cib.size
    out = np.empty((nblk, 2), np.float32)
    lib().orc_sddmm_bcsr(_pi(rpb), _pi(cib), _pf(vb), _pf(A), _pf(B), _pf(out), Mb, K, nblk)
    return out


def sddmm_bcsr_split(rowPtr_bs, colIdx_b, val_b, target_row, A, B):
    rps, cib, vb, tr, A, B = _i32(rowPtr_bs), _i32(colIdx_b), _f32(val_b), _i32(target_row), _f32(A), _f32(B)
    Sb, K, nblk = rps.size - 1, A.shape[1], cib.size
    out = np.empty((nblk, 2), np.float32)
    lib().orc_sddmm_bcsr_split(_pi(rps), _pi(cib), _pf(vb), _pi(tr), _pf(A), _pf(B), _pf(out), Sb, K, nblk)
    return out


def segment_softmax(rowPtr, e):
    rowPtr, e = _i32(rowPtr), _f32(e)
    out = np.zeros_like(e)
    lib().orc_segment_softmax(_pi(rowPtr), _pf(e), _pf(out), rowPtr.size - 1)
    return out


# ------------------------------------------------------------------------------------------------
# Host arithmetic of the reference restated in numpy
# ------------------------------------------------------------------------------------------------
def normalize_adj_closed_form(rows, cols, n):
    """graph_input.py:366-379 as a closed form.

    Pattern = (A with every stored value 1) with the diagonal set to 1; d = row sums;
    value(i,j) = fp32( fp64(d_i^-1/2) * fp64(d_j^-1/2) ).  Returns sorted CSR (int32, int32, fp32).
    """
    rows = np.asarray(rows, np.int64)
    cols = np.asarray(cols, np.int64)
    off = rows != cols
    key = np.unique(np.concatenate([rows[off] * n + cols[off], np.arange(n, dtype=np.int64) * (n + 1)]))
    r = key // n
    c = key % n
    deg = np.bincount(r, minlength=n).astype(np.float64)
    with np.errstate(divide="ignore"):
        dis = np.power(deg, -0.5)
    dis[np.isinf(dis)] = 0.0
    val = (dis[c] * dis[r]).astype(np.float32)
    rowPtr = np.zeros(n + 1, np.int64)
    np.cumsum(np.bincount(r, minlength=n), out=rowPtr[1:])
    return rowPtr.astype(np.int32), c.astype(np.int32), val


def format_stats(rowPtr, colIdx, num_edges, csr_flag=True, manual_granularity=None, is_avg_granularity=False):
    """graph_input.py:48-129 restated with numpy in the same precisions.

    The reference computes with torch CPU tensors: row_nnz int32, ``.float()`` fp32, unbiased std,
    true division of int tensors -> fp32.  Returns a dict with the same field names.
    """
    rowPtr = np.asarray(rowPtr, np.int32)
    n = rowPtr.size - 1
    row_nnz = rowPtr[1:] - rowPtr[:-1]
    out = {"row_nnz": row_nnz}
    real_nrow = int(np.count_nonzero(row_nnz))
    out["real_nrow"] = real_nrow
    if csr_flag:
        out["max_row_nnz"] = int(row_nnz.max())
        nonempty_rate = np.float32(real_nrow) / np.float32(n)
        out["nonempty_rate"] = float(nonempty_rate)
        avg = num_edges / n
        out["avg_degree"] = avg
        f = row_nnz.astype(np.float32)
        out["COV"] = float(np.float32(np.std(f.astype(np.float64), ddof=1)) / np.float32(avg))
        if nonempty_rate < 0.98:
            real_avg = float(np.float32(num_edges) / np.float32(real_nrow))
            ne = f[row_nnz != 0]
            out["real_COV"] = float(np.float32(np.std(ne.astype(np.float64), ddof=1)) / np.float32(real_avg))
        else:
            real_avg = avg
            out["real_COV"] = out["COV"]
        out["real_avg_degree"] = real_avg
        nz = row_nnz != 0
        tail = (rowPtr[1:] - 1)[nz]
        head = rowPtr[:-1][nz]
        colIdx = np.asarray(colIdx, np.int32)
        bw = colIdx[tail] - colIdx[head]
        out["max_bw"] = int(bw.max())
        out["avg_bw"] = float(np.float32(bw.sum(dtype=np.int64)) / np.float32(real_nrow))
    else:
        real_avg = float(np.float32(num_edges) / np.float32(real_nrow))
        out["real_avg_degree"] = real_avg
    if is_avg_granularity:
        g = int(real_avg)
    elif manual_granularity is not None:
        g = manual_granularity
    else:
        g = math.ceil(real_avg / 32) * 32
    out["split_granularity"] = g
    row_split_nnz = np.ceil(row_nnz.astype(np.float32) / np.float32(g))
    out["row_split_nnz"] = row_split_nnz
    out["split_ratio"] = float(np.float32(int(row_split_nnz.sum(dtype=np.float64))) / np.float32(real_nrow))
    return out


def gap_calculator(dim, CF, warp_size=32):
    """PCSR.py:19-26."""
    t_res = dim % (warp_size * CF)
    return 0 if t_res == 0 else min(dim, CF * warp_size) - t_res


def dynamic_CF_prompter(dim, CF_set=None, warp_size=32):
    """PCSR.py:30-42 (without its per-CF print)."""
    CF_set = list(range(1, 9)) if CF_set is None else CF_set
    CF_set = CF_set[: math.ceil(dim / 32)]
    return [cf for cf in CF_set if gap_calculator(dim, cf, warp_size) < 32]


# PCSR.py:19-42 evaluated by hand for every dim the decider supports.
CF_TABLE = {
    16: [1], 32: [1], 48: [1, 2], 64: [1, 2], 80: [1, 3], 96: [1, 3], 112: [1, 2, 4], 128: [1, 2, 4],
    144: [1, 5], 160: [1, 5], 176: [1, 2, 3, 6], 192: [1, 2, 3, 6], 208: [1, 7], 224: [1, 7],
    240: [1, 2, 4, 8], 256: [1, 2, 4, 8],
}


def decode_tree(code, dim, vec_size_list=(1, 2), warpNum_list=(4, 8)):
    """decider.py:63-80: class code -> (if_split, vec_size, CF, blkWarpNum)."""
    CF_list = dynamic_CF_prompter(dim)
    if_split = code % 2
    vec_size = vec_size_list[code // 2 % len(vec_size_list)]
    CF = CF_list[code // (len(vec_size_list) * 2) % len(CF_list)]
    blkWarpNum = warpNum_list[code // (len(CF_list) * len(vec_size_list) * 2)]
    return if_split, vec_size, CF, blkWarpNum


def model_dim(dim):
    """decider.py:52-55: which trained forest serves a requested dim."""
    return dim if dim % 32 == 0 else (math.ceil(dim / 32) * 2 - 1) * 16
