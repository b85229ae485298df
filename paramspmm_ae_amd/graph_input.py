"""PCSR format builder: a matrix -> CSR, 2x1 BCSR, their row-split variants, the CSR->BCSR value mask and the
matrix statistics the SpMM-decider consumes.

Same surface as the reference's graph_input.py (classes ``csr_data`` and ``graph_input`` with the attribute
and method names its callers use, graph_input.py:17-430), built differently:

* the BCSR blocks come from ``psp_bcsr_build`` of libparamsp_hip.so (first-encounter block order, i.e. what
  SciPy's ``tobsr`` yields in graph_input.py:245-256) instead of a SciPy conversion;
* row splitting goes through ``ParamSpMM.split_csr_par`` as in graph_input.py:135-136;
* with a GPU present both are built there instead (``device_builder``: same arrays bit for bit, copied back so that
  the attributes stay CPU tensors as in the reference); ``build_on="host"`` keeps the host builders;
* ``load_from_csr`` accepts arrays directly, so synthetic graphs never touch a ``.mtx`` file.
"""
import math
import time

import numpy as np
import torch

from . import _capi


# candidates of csr_data.xcd_stripe, longest first (multiples of 256), and the XCD share it accepts
XCD_STRIPES = (32768, 16384, 8192, 6144, 4096, 3072, 2048, 1536, 1024, 768, 512)
XCD_IMBALANCE = 1.03


def _stat_block(rowPtr, colIdx, num_nodes, num_edges):
    """Statistics of graph_input.py:60-87 with the reference's tensor types (int32 counts, fp32 moments,
    unbiased std)."""
    row_nnz = rowPtr[1:] - rowPtr[:-1]
    occupied = row_nnz != 0
    real_nrow = torch.sum(occupied)
    nonempty_rate = real_nrow / num_nodes
    avg_degree = num_edges / num_nodes
    cov = row_nnz.float().std() / avg_degree
    if nonempty_rate < 0.98:
        real_avg_degree = (num_edges / real_nrow).item()
        real_cov = torch.std(row_nnz[occupied].float()) / real_avg_degree
    else:
        real_avg_degree, real_cov = avg_degree, cov
    last = (rowPtr[1:] - 1)[occupied].long()
    first = rowPtr[:-1][occupied].long()
    width = colIdx[last] - colIdx[first]
    return {
        "row_nnz": row_nnz,
        "max_row_nnz": torch.max(row_nnz),
        "real_nrow": real_nrow,
        "nonempty_rate": nonempty_rate,
        "avg_degree": avg_degree,
        "COV": cov,
        "real_avg_degree": real_avg_degree,
        "real_COV": real_cov,
        "max_bw": torch.max(width),
        "avg_bw": torch.sum(width) / real_nrow,
    }


class csr_data(object):
    """One sparse format (CSR when ``csr_flag`` else 2x1 BCSR) as CPU tensors plus its statistics."""

    def __init__(self, rowPtr, colIdx, val, num_nodes, num_edges, csr_flag=True):
        self.csr_flag = csr_flag
        self.rowPtr = torch.from_numpy(np.ascontiguousarray(rowPtr)).int()
        self.colIdx = torch.from_numpy(np.ascontiguousarray(colIdx)).int()
        self.val = torch.from_numpy(np.ascontiguousarray(val)).float()
        self.num_nodes = num_nodes  # rows (block-rows for BCSR)
        self.num_edges = num_edges  # stored scalars (blocks for BCSR)
        self.row_nnz = None
        self.max_row_nnz = None
        self.real_nrow = None
        self.nonempty_rate = None
        self.avg_degree = None
        self.COV = None
        self.real_avg_degree = None
        self.real_COV = None
        self.max_bw = None
        self.avg_bw = None
        self.split_granularity = None
        self.split_ratio = None
        self.row_split_nnz = None
        self.rowPtr_split = None
        self.target_row = None
        self._dev = {}  # (attribute name, device) -> copy of that attribute on the device
        self._xcd_stripe = {}  # split? -> result of xcd_stripe()

    def on_device(self, name, device):
        """The attribute ``name`` as a tensor on ``device``; uploaded once and kept (the device builders leave
        their outputs here, so a format built on the GPU is never uploaded again)."""
        device = torch.device(device)
        if device.type != "cuda":
            return getattr(self, name).to(device)
        if device.index is None:
            device = torch.device("cuda", torch.cuda.current_device())
        key = (name, device)
        host = getattr(self, name)
        t = self._dev.get(key)
        if t is None or t.shape != host.shape:
            t = host.to(device)
            self._dev[key] = t
        return t

    def _keep_device(self, name, tensor):
        self._dev[(name, tensor.device)] = tensor

    def window_format(self, device="cuda"):
        """(rowPtr_w, colIdx_w, val_w, local share) of this CSR matrix in the windowed layout of the library
        (psp_window_build: every row's entries reordered so that the ones whose column lies within PSP_WINDOW_HALO rows of the
        row's 64-row block come first), built on ``device`` once and kept.  No counterpart in the reference; the
        CSR arrays must be the plain (vec_size 1) ones."""
        import ParamSpMM

        device = torch.device(device)
        if device.type == "cuda" and device.index is None:
            device = torch.device("cuda", torch.cuda.current_device())
        key = ("window", device)
        got = self._dev.get(key)
        if got is None:
            if self.val.dim() != 1:
                raise ValueError("the windowed layout exists for the CSR format (vec_size 1)")
            rp, ci, v = ParamSpMM.window_build(self.on_device("rowPtr", device), self.on_device("colIdx", device),
                                               self.on_device("val", device))
            nnz = max(int(self.colIdx.numel()), 1)
            local = float((rp[1:-1:2].long() - rp[0:-2:2].long()).sum().item()) / nnz
            got = (rp, ci, v, local)
            self._dev[key] = got
        return got

    def xcd_stripe(self, split):
        """Rows (segments when ``split``) the SpMM kernel should deal to one XCD at a time for this format: the
        longest of XCD_STRIPES under which the eight XCDs get equal shares of the stored entries (largest share at
        most XCD_IMBALANCE of the mean), else the best balanced one.  Long stripes keep neighbouring rows, and the X
        rows they gather in common, in one L2; a matrix whose long rows cluster in an index range (an R-MAT graph,
        a degree-sorted one) needs shorter ones or one XCD runs long after the others have finished.  Passed to the
        operators as ``blkWarpNum | _capi.bw_stripe(rows)``; no counterpart in the reference (one L2 per GPU)."""
        key = bool(split)
        if key in self._xcd_stripe:
            return self._xcd_stripe[key]
        ptr = self.rowPtr_split if split else self.rowPtr
        rows = 0
        if ptr is not None and ptr.numel() > 1:
            off = ptr.numpy().astype(np.int64)
            total = float(off[-1] - off[0])
            nseg = off.size - 1
            best = None
            for stripe in XCD_STRIPES:
                if total <= 0 or nseg < 16 * stripe:  # fewer than two rounds of stripes: nothing to level
                    continue
                edges = off[np.minimum(np.arange(0, nseg + stripe, stripe), nseg)]
                per_stripe = np.diff(edges)
                share = np.bincount(np.arange(per_stripe.size) % 8, weights=per_stripe, minlength=8)
                worst = share.max() * 8.0 / total
                if worst <= XCD_IMBALANCE:
                    best = (worst, stripe)
                    break
                if best is None or worst < best[0] - 1e-9:
                    best = (worst, stripe)
            rows = best[1] if best is not None else 0
        self._xcd_stripe[key] = rows
        return rows

    # graph_input.py:48-51
    def split_ratio_comp(self, split_granularity):
        row_split_nnz = torch.ceil(self.row_nnz / split_granularity)
        return int(row_split_nnz.sum()) / self.real_nrow, row_split_nnz

    def _choose_granularity(self, manual_granularity, is_avg_granularity):
        # graph_input.py:89-102 / 117-129: average, manual, or the next multiple of 32 above the mean row length
        if is_avg_granularity:
            g = int(self.real_avg_degree)
        elif manual_granularity is not None:
            g = manual_granularity
        else:
            g = math.ceil(self.real_avg_degree / 32) * 32
        self.split_granularity = g
        self.split_ratio, self.row_split_nnz = self.split_ratio_comp(g)

    def init_info(self, manual_granularity=None, is_avg_granularity=False):
        if not self.csr_flag:
            # the blocked format only needs its split parameters (graph_input.py:103-105)
            self.get_split_info(manual_granularity, is_avg_granularity)
            return
        for k, v in _stat_block(self.rowPtr, self.colIdx, self.num_nodes, self.num_edges).items():
            setattr(self, k, v)
        self._choose_granularity(manual_granularity, is_avg_granularity)

    def get_split_info(self, manual_granularity=None, is_avg_granularity=False):
        self.row_nnz = self.rowPtr[1:] - self.rowPtr[:-1]
        self.real_nrow = torch.sum(self.row_nnz != 0)
        self.real_avg_degree = (self.num_edges / self.real_nrow).item()
        self._choose_granularity(manual_granularity, is_avg_granularity)

    def get_split(self, verbose=True, build_on="auto"):
        if self.split_granularity is None:
            raise ValueError("split_granularity is None, must be init first")
        t0 = time.perf_counter()
        if _use_device(build_on):
            from . import device_builder

            rs, tr = device_builder.split_csr_device(self.on_device("rowPtr", "cuda"), self.split_granularity)
            self.rowPtr_split, self.target_row = device_builder.to_host(rs, tr)
            self._keep_device("rowPtr_split", rs)
            self._keep_device("target_row", tr)
        else:
            import ParamSpMM  # the extension module of this build (lib/ParamSpMM.so)

            offsets = torch.zeros(self.row_split_nnz.numel() + 1, dtype=torch.int32)
            offsets[1:] = self.row_split_nnz.cumsum(dim=0).to(torch.int32)
            self.rowPtr_split, self.target_row = ParamSpMM.split_csr_par(self.rowPtr, offsets, self.split_granularity)
        if verbose:
            print(
                "get_split -> split time: (ms): {:.3f} split_gran: {} \n split_ratio: {} avg_nnz: {} split_rows: {}".format(
                    (time.perf_counter() - t0) * 1e3,
                    self.split_granularity,
                    self.split_ratio,
                    self.real_avg_degree,
                    self.target_row.shape[0],
                )
            )

    def print_info(self):
        if self.csr_flag:
            print("#################### CSR format graph info ####################")
            for k in ("num_nodes", "num_edges", "max_row_nnz", "real_nrow"):
                print("= {}: {}".format(k, getattr(self, k)))
            for k in ("nonempty_rate", "avg_degree", "COV", "real_avg_degree", "real_COV"):
                print("= {}: {:.3f}".format(k, float(getattr(self, k))))
            print("= max_bw: {}".format(self.max_bw))
            print("= avg_bw: {:.3f}".format(float(self.avg_bw)))
        else:
            print("#################### BCSR format graph info ####################")
            print("= real_nrow: {}".format(self.real_nrow))
            print("= real_avg_degree: {:.3f}".format(self.real_avg_degree))
        print("= split_granularity: {}".format(self.split_granularity))
        print("= split_ratio: {:.5f}".format(float(self.split_ratio)))


def _use_device(build_on):
    if build_on not in ("auto", "host", "device"):
        raise ValueError("build_on must be 'auto', 'host' or 'device'")
    if build_on == "device" and not torch.cuda.is_available():
        raise RuntimeError("build_on='device' needs a GPU")
    return build_on == "device" or (build_on == "auto" and torch.cuda.is_available())


def build_bcsr(rowPtr, colIdx, val, ncols=None, build_on="host", device_arrays=None, blk_size=2):
    """CSR (numpy int32/int32/fp32) -> blk_size x 1 BCSR arrays (numpy) via libparamsp_hip.so: the host builder, or,
    for 2x1 blocks, the device builder when ``build_on`` says so and the rows are strictly ascending.
    ``device_arrays``: the CSR already on the GPU (rowPtr, colIdx, val) to build from; on return it holds the three
    BCSR tensors on the GPU (emptied when the host built them)."""
    rowPtr = np.ascontiguousarray(rowPtr, np.int32)
    colIdx = np.ascontiguousarray(colIdx, np.int32)
    val = np.ascontiguousarray(val, np.float32)
    n = rowPtr.size - 1
    if blk_size != 2:
        # the reference's blk_size argument (graph_input.py:210,245-256); its kernels exist for 3 (vec_spmm)
        if device_arrays is not None:
            del device_arrays[:]
        R = int(blk_size)
        ncols = (n + R - 1) // R * R if ncols is None else ncols
        nblk = _capi.check(_capi.lib.psp_vbsr_count(_capi.ptr(rowPtr), _capi.ptr(colIdx), n, ncols, R))
        rowPtr_b = np.empty((n + R - 1) // R + 1, np.int32)
        colIdx_b = np.empty(nblk, np.int32)
        val_b = np.empty((nblk, R), np.float32)
        _capi.check(_capi.lib.psp_vbsr_build(_capi.ptr(rowPtr), _capi.ptr(colIdx), _capi.ptr(val), n, ncols, R,
                                             _capi.ptr(rowPtr_b), _capi.ptr(colIdx_b), _capi.ptr(val_b)))
        return rowPtr_b, colIdx_b, val_b
    if ncols is None and _use_device(build_on):
        from . import device_builder

        try:
            src = device_arrays if device_arrays else [torch.from_numpy(a).cuda() for a in (rowPtr, colIdx, val)]
            out = device_builder.build_bcsr_device(*src)
            if device_arrays is not None:
                device_arrays[:] = out
            return tuple(t.numpy() for t in device_builder.to_host(*out))
        except device_builder.NotCanonical:
            if build_on == "device":
                raise
    if device_arrays is not None:
        del device_arrays[:]
    ncols = n + (n & 1) if ncols is None else ncols
    nblk = _capi.check(_capi.lib.psp_bcsr_count(_capi.ptr(rowPtr), _capi.ptr(colIdx), n, ncols))
    rowPtr_b = np.empty((n + 1) // 2 + 1, np.int32)
    colIdx_b = np.empty(nblk, np.int32)
    val_b = np.empty((nblk, 2), np.float32)
    _capi.check(
        _capi.lib.psp_bcsr_build(
            _capi.ptr(rowPtr), _capi.ptr(colIdx), _capi.ptr(val), n, ncols,
            _capi.ptr(rowPtr_b), _capi.ptr(colIdx_b), _capi.ptr(val_b),
        )
    )
    return rowPtr_b, colIdx_b, val_b


class graph_input(object):
    def __init__(self, mtx_name=None, path=None):
        self.loaded_flag = False
        self.reordered_flag = False
        self.csr_split_flag = False
        self.bcsr_split_flag = False
        self.bcsr_flag = False
        self.path = path
        self.mtx_name = mtx_name
        self.mtx_nodes = None
        self.mtx_edges = None
        self.density = None
        self.csr_data = None
        self.bcsr_data = None
        self.pack_rate = None
        self.perm = None  # set by load_from_csr(reorder=...): new position -> old vertex
        self.mask = None
        self.verbose = True

    # ------------------------------------------------------------------------------------------
    def load(
        self,
        load_from_mtx=True,
        manual_granularity=None,
        is_avg_granularity=False,
        is_normalize=False,
        GIN_epsilon=None,
        blk_size=2,
        if_mask=False,
    ):
        """Read ``path + mtx_name + '.mtx'`` and build every format (graph_input.py:203-297)."""
        if self.path is None:
            raise ValueError("Graph path must be assigned first")
        if not load_from_mtx:
            raise ValueError("only load_from_mtx=True is supported; use load_from_csr for arrays")
        from scipy.io import mmread

        mtx = mmread(self.path + self.mtx_name + ".mtx")
        mtx.data = np.ones_like(mtx.data)
        if is_normalize:
            mtx = self.normalize_adj(mtx)
        elif GIN_epsilon is not None:
            mtx = self.normalize_adj_GIN(mtx, GIN_epsilon)
        csr = mtx.tocsr()
        csr.sort_indices()
        return self.load_from_csr(
            csr.indptr, csr.indices, csr.data,
            manual_granularity=manual_granularity, is_avg_granularity=is_avg_granularity,
            blk_size=blk_size, if_mask=if_mask,
        )

    def load_from_csr(self, rowPtr, colIdx, val, manual_granularity=None, is_avg_granularity=False, blk_size=2,
                      if_mask=False, build_on="auto", reorder=None):
        """Build every format from a square CSR matrix given as arrays (column indices sorted per row).
        ``build_on``: "host", "device" or "auto" (the GPU when there is one) for the BCSR and row-split arrays.
        ``reorder``: None, "community" or "degree" -- rows and columns are permuted together before anything is built
        (reorder.py); ``self.perm`` (new position -> old vertex) says how, and features, labels and results move
        with ``permute_rows`` / ``unpermute_rows``.  The reference's inputs are pre-ordered outside its repository
        (Rabbit order, README.md:14-16)."""
        self.perm = None
        if reorder is not None:
            from . import reorder as ro

            if reorder == "community":
                self.perm = ro.community_permutation(rowPtr, colIdx)
            elif reorder == "degree":
                self.perm = ro.degree_permutation(rowPtr)
            else:
                raise ValueError("reorder must be None, 'community' or 'degree'")
            rowPtr, colIdx, val = ro.permute_csr(rowPtr, colIdx, val, self.perm)
        if blk_size not in (2, 3):
            raise ValueError("blocks of 2x1 and 3x1 are built (blk_size 2 or 3)")
        if if_mask and blk_size != 2:
            raise ValueError("the CSR -> block mask exists for 2x1 blocks only (SDDMM/sddmm_kernel.cu:78-107)")
        self.blk_size = blk_size
        t0 = time.perf_counter()
        rowPtr = np.ascontiguousarray(rowPtr, np.int32)
        colIdx = np.ascontiguousarray(colIdx, np.int32)
        val = np.ascontiguousarray(val, np.float32)
        n = rowPtr.size - 1
        nnz = int(rowPtr[-1])
        self.mtx_nodes = n
        self.mtx_edges = nnz
        self.density = nnz / (n * n)
        self.csr_data = csr_data(rowPtr, colIdx, val, n, nnz, True)
        self.csr_data.init_info(is_avg_granularity=is_avg_granularity, manual_granularity=manual_granularity)

        on_gpu = []
        if _use_device(build_on):
            from . import device_builder

            on_gpu = [self.csr_data.on_device(k, "cuda") for k in ("rowPtr", "colIdx", "val")]
            # the host builder rejects column indices outside the matrix; so does this path
            device_builder.check_index(on_gpu[0], on_gpu[1], (n + blk_size - 1) // blk_size * blk_size, what="load_from_csr")
        rowPtr_b, colIdx_b, val_b = build_bcsr(rowPtr, colIdx, val, build_on=build_on, device_arrays=on_gpu,
                                               blk_size=blk_size)
        nblk = colIdx_b.size
        # graph_input.py:257-266: the blocked format counts block-rows and blocks (the latter as a float)
        self.bcsr_data = csr_data(rowPtr_b, colIdx_b, val_b, (n + blk_size - 1) // blk_size, float(nblk), False)
        for k, t in zip(("rowPtr", "colIdx", "val"), on_gpu):
            self.bcsr_data._keep_device(k, t)
        self.bcsr_data.init_info(is_avg_granularity=is_avg_granularity, manual_granularity=manual_granularity)
        self.pack_rate = nnz / (blk_size * nblk) if nblk else 0.0  # graph_input.py:274

        self.mask = None
        if if_mask:
            import ParamSDDMM

            if not torch.cuda.is_available():
                raise RuntimeError("if_mask=True runs genmask on the GPU and no GPU is available")
            dev = torch.device("cuda")
            mask = ParamSDDMM.genmask(
                self.bcsr_data.on_device("rowPtr", dev), self.csr_data.on_device("rowPtr", dev),
                self.bcsr_data.on_device("val", dev), self.mtx_edges
            )
            self.mask = mask.to(torch.int64)

        self.loaded_flag = True
        self.reordered_flag = True
        self.bcsr_flag = True
        self.get_split_csr(build_on)
        self.get_split_bcsr(build_on)
        if self.verbose:
            print("data format all preprocess (ms): {:.3f}".format((time.perf_counter() - t0) * 1e3))
        return self

    def permute_rows(self, t):
        """a per-vertex tensor in the order the graph was loaded in (identity without ``reorder``)"""
        from . import reorder as ro

        return t if self.perm is None else ro.permute_rows(t, self.perm)

    def unpermute_rows(self, t):
        """a result computed on the loaded graph back in the caller's vertex order"""
        from . import reorder as ro

        return t if self.perm is None else ro.unpermute_rows(t, self.perm)

    def get_split_csr(self, build_on="auto"):
        self.csr_split_flag = True
        self.csr_data.get_split(self.verbose, build_on)

    def get_split_bcsr(self, build_on="auto"):
        self.bcsr_split_flag = True
        self.bcsr_data.get_split(self.verbose, build_on)

    # ------------------------------------------------------------------------------------------
    def normalize_adj(self, mtx):
        """D^-1/2 (A+I) D^-1/2 with all stored values first set to 1, in float64 (graph_input.py:366-379)."""
        from scipy.sparse import diags

        mtx.data = np.ones_like(mtx.data)
        mtx.setdiag(1)
        degree = np.asarray(mtx.sum(1)).ravel()
        with np.errstate(divide="ignore"):
            d_inv_sqrt = np.power(degree, -0.5)
        d_inv_sqrt[np.isinf(d_inv_sqrt)] = 0.0
        d = diags(d_inv_sqrt)
        return mtx.dot(d).transpose().dot(d)

    def normalize_adj_GIN(self, mtx, epsilon):
        """(B + B^T)/2 with B = pattern with diagonal 1+epsilon (graph_input.py:381-390)."""
        mtx.data = np.ones_like(mtx.data)
        mtx.setdiag(1 + epsilon)
        return (mtx + mtx.T) / 2

    # ------------------------------------------------------------------------------------------
    _FEATURES = (
        "graph_nodes", "graph_edges", "graph_density", "csr_max_row_nnz", "csr_real_nrow", "csr_nonempty_rate",
        "csr_avg_degree", "csr_COV", "csr_real_avg_degree", "csr_real_COV", "csr_max_bw", "csr_avg_bw",
        "csr_split_ratio", "bcsr_split_ratio", "pack_rate",
    )

    def _feature_values(self):
        c, b = self.csr_data, self.bcsr_data
        return [
            self.mtx_nodes, self.mtx_edges, self.density, c.max_row_nnz.item(), c.real_nrow.item(),
            c.nonempty_rate.item(), c.avg_degree, c.COV.item(), c.real_avg_degree,
            c.real_COV.item() if hasattr(c.real_COV, "item") else c.real_COV,
            c.max_bw.item(), c.avg_bw.item(), c.split_ratio.item(), b.split_ratio.item(), self.pack_rate,
        ]

    def get_info(self):
        """The 15 decider features as a (1, 15) float64 array (graph_input.py:392-410)."""
        return np.array(self._feature_values(), dtype=np.float64).reshape(1, -1)

    def mtxinfo_to_pandas(self):
        import pandas as pd

        data = {"mtx_name": self.mtx_name}
        data.update(dict(zip(self._FEATURES, self._feature_values())))
        return pd.DataFrame(data, index=[0])

    def print_mtx_info(self):
        print("-----------------{}-----------------".format(self.mtx_name))
        print("= graph_nodes: {}".format(self.mtx_nodes))
        print("= graph_edges: {}".format(self.mtx_edges))
        print("= graph_density: {}".format(self.density))
        print("= pack_rate: {:.5f}".format(self.pack_rate))
        self.csr_data.print_info()
        self.bcsr_data.print_info()

    # ------------------------------------------------------------------------------------------
    def _padded_rows(self, vec_size):
        if vec_size is None:
            return self.mtx_nodes
        return (self.mtx_nodes + vec_size - 1) // vec_size * vec_size

    def init_feat_embedding(self, num_features, vec_size=None):
        if num_features is None:
            raise ValueError("num_features must be assigned first")
        self.num_features = num_features
        self.x = torch.randn(self._padded_rows(vec_size), num_features).cuda()

    def init_labels(self, num_classes, vec_size=None):
        if num_classes is None:
            raise ValueError("num_classes must be assigned first")
        self.num_classes = num_classes
        # every node gets class 1, as in graph_input.py:422-430
        self.y = torch.ones(self._padded_rows(vec_size)).long().cuda()
