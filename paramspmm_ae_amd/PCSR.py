"""Operator facade over one PCSR variant (same surface as the reference's PCSR.py:19-657).

``pcsr_spmm`` keeps the device tensors of the variant selected by ``<if_split, vec_size>`` and forwards to the
extension modules ParamSpMM / ParamSDDMM / ParamSpCONV of this build.  Public attributes read by the GNN layers
(gnn_conv.py:19-105): rowPtr, colIdx, val, target_row, mask, if_split, vec_size, CF, blkWarpNum, mtx_nodes,
mtx_edges, result.

``CF`` keeps the meaning "column coarsening" and ``blkWarpNum`` "wavefronts per workgroup"; how they map onto
64-lane wavefronts is reported by ``ParamSpMM.spmm_plan(dim, CF, blkWarpNum)``.
"""
import math

import torch

import paramspmm_ae_amd  # noqa: F401  (puts lib/ on sys.path)
import ParamSpMM as SpMM
import ParamSDDMM as SDDMM
import ParamSpCONV as SpCONV


def gap_calculator(dim, CF, warp_size=32):
    """Columns a CF*warp_size wide tile leaves unused on its last pass over ``dim`` (PCSR.py:19-26)."""
    width = warp_size * CF
    rest = dim % width
    return 0 if rest == 0 else min(dim, width) - rest


def dynamic_CF_prompter(dim, CF_set=None, warp_size=32, verbose=False):
    """Coarsening factors worth sweeping for ``dim``: CF <= ceil(dim/32) whose gap is below one 32-column
    slab (PCSR.py:30-42).  The list and its order define the decider's class encoding."""
    candidates = list(range(1, 9)) if CF_set is None else list(CF_set)
    candidates = candidates[: math.ceil(dim / 32)]
    keep = []
    for cf in candidates:
        gap = gap_calculator(dim, cf, warp_size)
        if verbose:
            print("dim({})->CF:{} gap:{}".format(dim, cf, gap))
        if gap < 32:
            keep.append(cf)
    return keep


def native_CF_prompter(dim):
    """Configurations of the wave64 kernel that the reference's <CF, blkWarpNum> cannot express, as packed values
    for the ``CF`` argument (``_capi.pack_cf``; the operators pass CF through as an opaque int, PCSR.py:224-237):
    lane groups of 16 and 32 lanes (4 and 2 sparse rows per wavefront, fewer column tiles), the even division of a
    wavefront's entries between its lane groups, and light configurations -- one or two entries in flight per lane,
    four-lane groups -- whose wavefronts need few registers, so that more of them are resident: on matrices with
    short, regular rows whose gathers hit the caches (stencils, community-ordered graphs) residency beats loads in
    flight per wavefront (measured 8-20 % at widths up to 128).  The list depends only on the 32-wide band of
    ``dim``, like the forest that serves a width (decider.py:52-55), so both stay in step."""
    from ._capi import pack_cf

    band = math.ceil(dim / 32)
    if band <= 1:
        if dim <= 16:
            return [pack_cf(1, 4, 4, even_split=True), pack_cf(1, 4, 2, even_split=True), pack_cf(1, 4, 1)]
        return [pack_cf(1, 8, 4, even_split=True), pack_cf(2, 4, 2, even_split=True), pack_cf(2, 4, 1)]
    cf_max = dynamic_CF_prompter(band * 32)[-1]
    extra = [pack_cf(1, 16, 4), pack_cf(1, 8, 4, even_split=True),
             pack_cf(cf_max, 8, 2 if cf_max <= 4 else 1, even_split=True)]
    if band >= 4:
        extra.append(pack_cf(1, 32, 4))
    if cf_max <= 4:
        extra.append(pack_cf(cf_max, 8, 1, even_split=True))
    extra.append(pack_cf(4, 4, 1, even_split=True))
    return extra


def decider_CF_list(dim):
    """The CF axis of the decider's class space: the reference's list (PCSR.py:30-42) followed by the native
    configurations.  Class count per width = 4 representations x len(list) x 2 workgroup sizes."""
    return dynamic_CF_prompter(dim) + native_CF_prompter(dim)


def cf_label(cf):
    """Text of a CF value in a sweep column name: the number itself for the reference's CF, c<vectors per lane>l<lanes
    per row>u<entries in flight>[e] for a native configuration."""
    from ._capi import unpack_cf

    u = unpack_cf(int(cf))
    if u is None:
        return str(int(cf))
    c, lanes, unroll, segs, even = u
    return "c%dl%du%d%s%s" % (c, lanes, unroll, "" if segs is None else "w%d" % segs, "e" if even else "")


class _VendorFormatSpMM(object):
    """Vendor-library SpMM on a re-formatted copy of the graph's CSR matrix (PCSR.py:45-124)."""

    _compute = _profile = _label = None

    def _convert(self, csr):
        raise NotImplementedError

    def __init__(self, graph, device="cuda"):
        from scipy.sparse import csr_matrix

        c = graph.csr_data
        m = csr_matrix((c.val.numpy(), c.colIdx.numpy(), c.rowPtr.numpy()), shape=(graph.mtx_nodes, graph.mtx_nodes))
        self.idx_a, self.idx_b, self.val = (torch.from_numpy(a).to(device) for a in self._convert(m))
        self.mtx_nodes = graph.mtx_nodes

    def _dense_input(self, dim, x):
        if x is None and dim is None:
            raise ValueError("at least one of x and dim should be given")
        return torch.ones(self.mtx_nodes, dim, device="cuda") if dim is not None else x.to("cuda")

    def get_spmm_result(self, dim=None, x=None):
        return getattr(SpMM, self._compute)(self._dense_input(dim, x), self.idx_a, self.idx_b, self.val).to("cpu")

    def profiling(self, dim=None, x=None, verbose=True):
        X = self._dense_input(dim, x)
        throughput = getattr(SpMM, self._profile)(X, self.idx_a, self.idx_b, self.val)
        if verbose:
            print("{}-> dim: {} gflops: {:.0f}".format(self._label, X.size(1), throughput))
        return throughput


class coo_spmm(_VendorFormatSpMM):
    _compute, _profile, _label = "cusparse_compute_coo_alg4", "cusparse_profile_coo_alg4", "coo"

    def _convert(self, csr):
        coo = csr.tocoo()
        return coo.row.astype("int32"), coo.col.astype("int32"), coo.data.astype("float32")


class csc_spmm(_VendorFormatSpMM):
    _compute, _profile, _label = "cusparse_compute_csc", "cusparse_profile_csc", "csc"

    def _convert(self, csr):
        csc = csr.tocsc()
        return csc.indptr.astype("int32"), csc.indices.astype("int32"), csc.data.astype("float32")


# (if_split, blocked) -> operator names in the three modules
_SPMM = {(False, False): "csr_spmm", (True, False): "csr_split_spmm", (False, True): "bcsr_spmm", (True, True): "bcsr_split_spmm"}
_SDDMM = {(False, False): "csr_sddmm", (True, False): "csr_split_sddmm", (False, True): "bcsr_sddmm", (True, True): "bcsr_split_sddmm"}


class pcsr_spmm(object):
    def __init__(self, graph, vec_size, if_split, mtx_nodes=None, mtx_edges=None, rowPtr=None, colIdx=None,
                 val=None, target_row=None, CF=1, blkWarpNum=4, device="cuda", window=False):
        """``window`` (an addition of this build): the CSR matrix in the library's windowed layout, whose SpMM reads
        the X rows near the diagonal from LDS (vec_size 1, not split, a loaded graph; CF then names the kernel
        variant, 0 = automatic).  The SDDMM of such an operator runs on the same permuted CSR arrays."""
        if vec_size not in (1, 2, 3):
            raise ValueError("this build has vec_size 1 (CSR), 2 (2x1 BCSR) and 3 (3x1 blocks)")
        if_split = bool(if_split)
        self.mask = None
        self.window = bool(window)
        if self.window and (graph is None or vec_size != 1 or if_split):
            raise ValueError("window=True needs a loaded graph, vec_size 1 and if_split False")
        if graph is None:
            if mtx_edges is None or mtx_nodes is None or rowPtr is None or colIdx is None or val is None:
                raise ValueError("when graph is None, mtx_nodes, mtx_edges, rowPtr, colIdx, val should be given")
            if if_split and target_row is None:
                raise ValueError("target_row should be given when if_split is True")
            if not if_split and target_row is not None:
                raise ValueError("target_row should not be given when if_split is False")
            if (vec_size == 1) != (val.dim() == 1):
                raise ValueError("val must be 1-D for vec_size 1 and [nblk, vec_size] otherwise")
            self.mtx_nodes, self.mtx_edges = mtx_nodes, mtx_edges
            self.rowPtr, self.colIdx, self.val = rowPtr.to(device), colIdx.to(device), val.to(device)
            self.target_row = None if target_row is None else target_row.to(device)
            if torch.device(device).type == "cuda":
                # arrays of unknown origin: the kernels trust their indices, so look at them once
                from . import device_builder

                rows = (mtx_nodes + vec_size - 1) // vec_size
                device_builder.check_index(self.rowPtr, self.colIdx, rows * vec_size, self.target_row, rows,
                                           what="pcsr_spmm index arrays")
        else:
            self.mtx_nodes, self.mtx_edges = graph.mtx_nodes, graph.mtx_edges
            fmt = graph.csr_data if vec_size == 1 else graph.bcsr_data
            if vec_size != 1 and getattr(graph, "blk_size", 2) != vec_size:
                raise ValueError("the graph was loaded with blk_size %d, not %d" % (getattr(graph, "blk_size", 2), vec_size))
            # one device copy per format, shared by every operator built on this graph
            self.rowPtr = fmt.on_device("rowPtr_split" if if_split else "rowPtr", device)
            self.colIdx = fmt.on_device("colIdx", device)
            self.val = fmt.on_device("val", device)
            self.target_row = fmt.on_device("target_row", device) if if_split else None
            if vec_size != 1 and getattr(graph, "mask", None) is not None:
                self.mask = graph.mask.to(device)
        self.vec_size = vec_size
        self.if_split = if_split
        self.CF = CF
        self.blkWarpNum = blkWarpNum
        self.result = None
        self.window_local_share = None
        if self.window:
            # rowPtr_w has 2 M + 2 entries (row start, start of the row's remote part); colIdx / val are the row-wise
            # permuted entries, so rowPtr_w[0::2] with them is again a CSR matrix (what the SDDMM walks)
            self.rowPtr_w, self.colIdx, self.val, self.window_local_share = graph.csr_data.window_format(device)
            self.CF = CF if 0 <= CF <= 3 else 0
        # Plain layouts of a graph with hub rows: the SDDMM divides the stored entries, not the rows, between its
        # wavefronts (every entry's result is independent).  "Hub rows" = a longest row of more than 64 times the
        # mean; arrays without statistics keep the row-wise walk.
        # SpMM: rows dealt to one XCD at a time, from the format's distribution of entries (csr_data.xcd_stripe);
        # travels in the flag bits of blkWarpNum
        self.bw_flags = 0
        if graph is not None:
            from ._capi import bw_stripe

            fmt = graph.csr_data if vec_size == 1 else graph.bcsr_data
            self.bw_flags = bw_stripe(fmt.xcd_stripe(if_split))
        self.sddmm_balanced = False
        if graph is not None and not if_split:
            fmt = graph.csr_data if vec_size == 1 else graph.bcsr_data
            longest, mean = getattr(fmt, "max_row_nnz", None), getattr(fmt, "avg_degree", None)
            if longest is not None and mean:
                self.sddmm_balanced = float(longest) > 64.0 * float(mean)

    # ---- plumbing ---------------------------------------------------------------------------
    @property
    def fmt_code(self):
        """Format code of the extension modules' generic entry points: 0 csr, 1 csr_split, 2 bcsr, 3 bcsr_split,
        4 windowed csr."""
        return 4 if self.window else (1 if self.if_split else 0) + (2 if self.vec_size != 1 else 0)

    @property
    def spmm_rowPtr(self):
        """The row pointer array the SpMM entry points of this operator's format take."""
        return self.rowPtr_w if self.window else self.rowPtr

    def _key(self):
        return (self.if_split, self.vec_size != 1)

    def _spmm_name(self):
        # vec_size 3 goes to the generic-block operators (PCSR.py:227-239)
        if self.vec_size == 3:
            return "vec_split_spmm" if self.if_split else "vec_spmm"
        return _SPMM[self._key()]

    def _sparse_args(self, val=None):
        args = [self.rowPtr, self.colIdx, self.val if val is None else val]
        if self.if_split:
            args.append(self.target_row)
        return args

    def _spmm(self, X, val=None, CF=None, blkWarpNum=None):
        if self.window:
            return SpMM.window_spmm(X, self.rowPtr_w, self.colIdx, self.val if val is None else val,
                                    self.CF if CF is None else CF)
        fn = getattr(SpMM, self._spmm_name())
        return fn(X, *self._sparse_args(val), self.CF if CF is None else CF,
                  (self.blkWarpNum if blkWarpNum is None else blkWarpNum) | self.bw_flags)

    def _dense_input(self, dim, x):
        if x is None and dim is None:
            raise ValueError("at least one of x and dim should be given")
        if dim is not None:
            return torch.ones(self.mtx_nodes, dim, device="cuda")
        return x.to("cuda")

    # ---- SpMM -------------------------------------------------------------------------------
    def get_spmm_result(self, dim=None, x=None, CF=None, blkWarpNum=None):
        """A*X with X = ones(n, dim) or x; the first mtx_nodes rows land on the CPU in ``self.result``."""
        assert torch.cuda.is_available()
        X = self._dense_input(dim, x)
        out = self._spmm(X, CF=CF, blkWarpNum=blkWarpNum)
        self.result = out[0 : self.mtx_nodes, :].to("cpu")
        del X
        torch.cuda.empty_cache()

    def AGNN_spmm(self, spVal, X):
        """SpMM with caller-supplied values (edge attentions) in this variant's layout."""
        return self._spmm(X, val=spVal)

    def GIN_spmm(self, X):
        return self._spmm(X)

    # ---- SDDMM ------------------------------------------------------------------------------
    def _sddmm(self, A, B, blkWarpNum, alpha=None):
        if self.window and A.dtype == torch.float32 and SDDMM.window_sddmm_supported(int(A.size(1))):
            # B rows of a block's window from LDS (results parallel to the layout's own colIdx)
            return SDDMM.window_sddmm(A, B, self.rowPtr_w, self.colIdx, alpha)
        if alpha is not None:
            return self._sddmm(A, B, blkWarpNum) * alpha.reshape(())
        if self.vec_size == 3:  # the generic-block operators (PCSR.py:300-345)
            fn = SDDMM.vec_split_sddmm if self.if_split else SDDMM.vec_sddmm
        else:
            fn = getattr(SDDMM, _SDDMM[self._key()])
        CF = (A.size(1) + 31) // 32
        if self.sddmm_balanced and not self.if_split:
            blkWarpNum |= 0x100  # PSP_BW_BALANCED: divide the entries, not the rows, between the wavefronts
        return fn(A, B, *self._sparse_args(), CF, blkWarpNum | self.bw_flags)

    def AGNN_sddmm(self, A, alpha=None):
        """Per stored entry <A[row], A[col]>; for 2x1 blocks the result is [nblk, 2] (PCSR.py:290-320).  ``alpha`` (an
        addition of this build): a one-element tensor the results are multiplied by -- inside the kernel on a windowed
        operator."""
        if self.vec_size != 1 and self.mask is None:
            raise ValueError("mask should be given when vec_size=2")
        return self._sddmm(A, A, self.blkWarpNum, alpha)

    def get_sddmm_result(self, dim, blkWarpNum):
        assert torch.cuda.is_available()
        pad = max(self.vec_size, 2)
        A = torch.ones((self.mtx_nodes + pad - 1) // pad * pad, dim, device="cuda")
        B = torch.ones(self.mtx_nodes, dim, device="cuda")
        return self._sddmm(A, B, blkWarpNum)

    # ---- fused GCN layer ----------------------------------------------------------------------
    def forward(self, H, w):
        if H is None or w is None:
            raise ValueError("H and w should be given")
        if self.vec_size == 3:
            raise NotImplementedError("the fused GCN operators exist for vec_size 1 and 2 (SpCONV/SpCONV.cpp:498-511)")
        if self.window:
            return SpCONV.aggregate(4, SpCONV.dense_xw(H, w, False), self.rowPtr_w, self.colIdx, self.val, None, self.CF, 4)
        fn = getattr(SpCONV, _SPMM[self._key()] + "_forward")
        return fn(H, w, *self._sparse_args(), self.CF, self.blkWarpNum | self.bw_flags)

    def backward(self, d_output, H, w):
        if d_output is None or H is None:
            raise ValueError("d_output and H should be given")
        if self.vec_size == 3:
            raise NotImplementedError("the fused GCN operators exist for vec_size 1 and 2 (SpCONV/SpCONV.cpp:498-511)")
        if self.window:
            AG = SpCONV.aggregate(4, d_output, self.rowPtr_w, self.colIdx, self.val, None, self.CF, 4)
            return SpCONV.dense_xw(AG, w, True), SpCONV.weight_gradient(H, AG)
        fn = getattr(SpCONV, _SPMM[self._key()] + "_backward")
        d_input, d_weight = fn(d_output, H, w, *self._sparse_args(), self.CF, self.blkWarpNum | self.bw_flags)
        return d_input, d_weight

    # ---- timing -----------------------------------------------------------------------------
    def cf_warpnum_profiling(self, CF, blkWarpNum, dim=None, x=None, verbose=True):
        """GFLOP/s (int) of this variant with an explicit (CF, blkWarpNum) (PCSR.py:433-505)."""
        assert torch.cuda.is_available()
        X = self._dense_input(dim, x)
        if self.window:  # no *_profile twin: the event-timed mean of the same number of launches
            ms = SpMM.spmm_time_ms(4, X, self.rowPtr_w, self.colIdx, self.val, None, CF if 0 <= CF <= 3 else 0, 4, 20, 200, 0)
            throughput = int(2.0 * self.mtx_edges * X.size(1) / 1e6 / ms) if ms > 0 else 0
            if verbose:
                print("dim: {} gflops: {:.0f}".format(X.size(1), throughput))
            return throughput
        fn = getattr(SpMM, self._spmm_name() + "_profile")
        args = self._sparse_args()
        if self.vec_size != 1:
            args.append(self.mtx_edges)  # blocked twins take the true nnz before CF
        throughput = fn(X, *args, CF, blkWarpNum | self.bw_flags)
        if verbose:
            print("dim: {} gflops: {:.0f}".format(X.size(1), throughput))
        return throughput

    def profiling(self, dim=None, x=None, verbose=True):
        return self.cf_warpnum_profiling(self.CF, self.blkWarpNum, dim=dim, x=x, verbose=verbose)

    # ---- vendor baselines on the plain CSR arrays (PCSR.py:581-657); served by rocSPARSE here --------------
    def _vendor(self, compute, profile, label, dim, x, is_profiling, verbose=True):
        assert torch.cuda.is_available()
        if self.if_split or self.vec_size != 1:
            raise ValueError("cusparse only support vec_size=1 and if_split=False")
        X = self._dense_input(dim, x)
        if is_profiling:
            throughput = getattr(SpMM, profile)(X, self.rowPtr, self.colIdx, self.val)
            if verbose:
                print("{}-> dim: {} gflops: {:.0f}".format(label, X.size(1), throughput))
            return throughput
        return getattr(SpMM, compute)(X, self.rowPtr, self.colIdx, self.val).to("cpu")

    def cusparse_ref(self, dim=None, x=None, is_profiling=False, verbose=True):
        return self._vendor("cusparse_compute", "cusparse_profile", "cusparse", dim, x, is_profiling, verbose)

    def cusparse_csr_alg2_ref(self, dim=None, x=None, is_profiling=False, verbose=True):
        return self._vendor("cusparse_compute_csr_alg2", "cusparse_profile_csr_alg2", "cusparse_csr_alg2", dim, x,
                            is_profiling, verbose)

    def gespmm_ref(self, dim=None, x=None, is_profiling=False, verbose=True):
        return self._vendor("gespmm_compute", "gespmm_profile", "gespmm", dim, x, is_profiling, verbose)

    def time_ms(self, X, CF=None, blkWarpNum=None, warmup=5, iters=20, flush_bytes=0):
        """Mean milliseconds per SpMM launch (an addition of this build; used by the sweep harness).  ``flush_bytes``:
        fill that much scratch memory before every timed launch, so that the operands come from HBM as inside a
        training step instead of from the caches the previous, identical launch left warm."""
        if self.vec_size == 3:
            raise NotImplementedError("time_ms covers the four decider formats; use cf_warpnum_profiling for 3x1 blocks")
        return SpMM.spmm_time_ms(self.fmt_code, X, self.spmm_rowPtr, self.colIdx, self.val, self.target_row,
                                 self.CF if CF is None else CF,
                                 (self.blkWarpNum if blkWarpNum is None else blkWarpNum) | self.bw_flags, warmup, iters,
                                 int(flush_bytes))


# ---- training-set construction: `python -m paramspmm_ae_amd.PCSR` (PCSR.py:660-871) -----------------------------
def get_mtx_info(filelist, path, dim=32, if_auto_gran=True, blk_size=2):
    """One row of the 15 decider features per ``<path>/<name>.mtx`` (PCSR.py:660-669)."""
    import pandas as pd

    from .graph_input import graph_input

    frames = []
    for name in filelist:
        graph = graph_input(mtx_name=name, path=path)
        graph.load(load_from_mtx=True, is_avg_granularity=not if_auto_gran, blk_size=blk_size)
        frames.append(graph.mtxinfo_to_pandas())
    return pd.concat(frames, axis=0, ignore_index=True) if frames else pd.DataFrame()


def profile_engine(filelist, path, dim_list, vec_size=2, if_DCP=True, if_auto_gran=True, verbose=True):
    """({dim: GFLOP/s table}, {dim: baseline table}) over the matrices of ``filelist`` (PCSR.py:672-806).

    Every swept configuration and both baselines are first checked against ``torch.sparse.mm`` with X = ones; the
    columns run blkWarpNum-major, then CF, then vec1 / vec1_split / vecV / vecV_split, so the index of the best
    column is the decider's class code.  ``if_DCP`` False sweeps CF 1..ceil(dim/32) without the gap rule."""
    import numpy as np
    import pandas as pd

    from . import sweep as sw
    from .graph_input import graph_input
    from .verification import SpMM_verification

    cfs = {d: dynamic_CF_prompter(d) if if_DCP else list(range(1, 9))[: math.ceil(d / 32)] for d in dim_list}
    tp = {d: [] for d in dim_list}
    base = {d: [] for d in dim_list}
    for name in filelist:
        if verbose:
            print("-------------{}-------------".format(name))
        graph = graph_input(mtx_name=name, path=path)
        graph.verbose = verbose
        graph.load(load_from_mtx=True, is_avg_granularity=not if_auto_gran, blk_size=vec_size)
        c = graph.csr_data
        check = SpMM_verification(dim_list[0], c.rowPtr, c.colIdx, c.val, baseline=True)
        ops = sw.operators_of(graph, vec_size)
        for d in dim_list:
            check.reference(d, verbose=False)
            check.compare(ops[0].cusparse_ref(d), name, verbose)
            check.compare(ops[0].gespmm_ref(d), name, verbose)
            base[d].append([ops[0].cusparse_ref(d, is_profiling=True, verbose=verbose),
                            ops[0].gespmm_ref(d, is_profiling=True, verbose=verbose)])
            _, gflops = sw.sweep_dim(ops, d, graph.mtx_edges, graph.mtx_nodes, cfs=cfs[d],
                                     verify=lambda y, col: check.compare(y.to("cpu"), "%s %s" % (name, col), False))
            tp[d].append(gflops)
        del ops, graph
        torch.cuda.empty_cache()
    tables = {d: pd.DataFrame(np.array(tp[d]).reshape(len(filelist), -1), columns=sw.column_names(d, cfs[d], vec_size))
              for d in dim_list}
    baselines = {d: pd.DataFrame(np.array(base[d], dtype=np.float64).reshape(len(filelist), 2), columns=["cusparse", "gespmm"])
                 for d in dim_list}
    return tables, baselines


def training_data_gen(dim_list, vec_size, info_df, filelist, path, csv_path, if_DCP=True, if_auto_gran=True, verbose=True):
    """Writes ``dim<d>.csv``, ``dim<d>_OP_SpMM.csv`` (features + best column) and ``dim<d>_baseline.csv`` under
    ``csv_path`` (PCSR.py:809-824): the files ``train_decider fit --data csv_path`` reads."""
    import os

    import pandas as pd

    tables, baselines = profile_engine(filelist, path, dim_list, vec_size, if_DCP, if_auto_gran, verbose)
    os.makedirs(csv_path, exist_ok=True)
    for d in dim_list:
        tables[d].to_csv(os.path.join(csv_path, "dim%d.csv" % d), index=False)
        best = pd.DataFrame({"OP_SpMM": tables[d].to_numpy().argmax(axis=1)})
        pd.concat([info_df.reset_index(drop=True), best], axis=1).to_csv(os.path.join(csv_path, "dim%d_OP_SpMM.csv" % d), index=False)
        baselines[d].to_csv(os.path.join(csv_path, "dim%d_baseline.csv" % d), index=False)
    return tables, baselines


def main(argv=None):
    import argparse
    import glob
    import os

    import pandas as pd

    flag = dict(type=str, choices=["True", "False"])
    parser = argparse.ArgumentParser()
    parser.add_argument("--path", type=str, default="./toy_dataset/", help="path to the mtx files")
    parser.add_argument("--dim_list", nargs="*", type=int, default=list(range(16, 257, 16)), help="dim_list for training data generation")
    parser.add_argument("--vec_size", type=int, default=2, help="vec_size(besides 1) for SpMM")
    parser.add_argument("--if_DCP", default="True", help="If to use DCP", **flag)
    parser.add_argument("--if_reorder", default="True", help="If to use graph reordering (the path must then name a rabbit-ordered set)", **flag)
    parser.add_argument("--if_auto_gran", default="True", help="If to use auto-Granularity, else use avg_row_nnz as split-granularity", **flag)
    parser.add_argument("--approx_eval", default="False", help="accepted for compatibility; unused in the reference as well", **flag)
    parser.add_argument("--csv_path", type=str, default=None, help="where the tables go (default: the reference's ./ParamSpMM-log/ tree)")
    args = parser.parse_args(argv)
    print(args)
    if_DCP, if_auto_gran, if_reorder = args.if_DCP == "True", args.if_auto_gran == "True", args.if_reorder == "True"
    # the reference's output tree (PCSR.py:846-866)
    if if_DCP and if_auto_gran:
        csv_path = "./ParamSpMM-log/"
    elif if_DCP:
        csv_path = "./ParamSpMM-log/ablation_study/auto-Gran/"
    elif if_auto_gran:
        csv_path = "./ParamSpMM-log/ablation_study/woDCP/"
    else:
        raise ValueError("input if_DCP and if_auto_gran options are not supported")
    if if_reorder:
        assert "rabbit" in args.path, "--if_reorder True expects a path of rabbit-ordered matrices"
    else:
        assert "rabbit" not in args.path
        csv_path = "./ParamSpMM-log/ablation_study/wo_reorder/"
    if args.vec_size != 2:
        csv_path = "./ParamSpMM-log/ablation_study/vec_size%d/" % args.vec_size
    if args.csv_path is not None:
        csv_path = args.csv_path
    os.makedirs(csv_path, exist_ok=True)
    filelist = sorted(os.path.basename(f)[:-4] for f in glob.glob(os.path.join(args.path, "*.mtx")))
    info_file = os.path.join(csv_path, "mtx_info.csv")
    if os.path.exists(info_file):
        info_df = pd.read_csv(info_file)
    else:
        info_df = get_mtx_info(filelist, args.path, if_auto_gran=if_auto_gran, blk_size=args.vec_size)
        info_df.to_csv(info_file, index=False)
    return training_data_gen(args.dim_list, args.vec_size, info_df, filelist, args.path, csv_path, if_DCP, if_auto_gran)


if __name__ == "__main__":
    main()
