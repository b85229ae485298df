#!/usr/bin/env python3
"""SDDMM facade and sweep (same surface as the reference's SDDMM.py:19-447).

``pcsr_sddmm`` holds one PCSR variant ``<if_split, vec_size>`` on the device and runs the SDDMM operators of
ParamSDDMM on it with A = B = ones, so every stored entry must come out as ``dim`` exactly; ``profile_engine``
checks the four variants against the vendor library (rocSPARSE behind the ``cusparse_sddmm_*`` names) and times
them for both workgroup sizes; ``training_data_gen`` writes the tables of GFLOP/s and of the best column per
matrix (SDDMM.py:371-383).  Besides ``.mtx`` files the sweep takes the seeded synthetic graphs of ``synth``.
"""
import argparse
import glob
import os

import numpy as np
import pandas as pd
import torch

import paramspmm_ae_amd  # noqa: F401  (puts lib/ on sys.path)
import ParamSDDMM as SDDMM

from .PCSR import pcsr_spmm
from .graph_input import graph_input

WARP_NUMS = (4, 8)


def compare(result, result_ref, verbose=True):
    """Element-wise relative 1e-4 against the reference result (SDDMM.py:19-36); raises ValueError on a mismatch."""
    if result is None or result_ref is None:
        raise ValueError("result or result_ref is None")
    bad = torch.abs(result - result_ref) > 1e-4 * torch.abs(result_ref)
    if not bool(bad.any()):
        if verbose:
            print("# Verification PASSED")
        return
    for i in torch.nonzero(bad.flatten())[:11].flatten().tolist():
        print("mismatched result: ", i, result.flatten()[i], result_ref.flatten()[i])
    raise ValueError("Verification FAILED")


def compare_2d(result, result_ref, mask, verbose=True):
    """Blocked results: pick the stored entries out of [nblk, vec_size] in CSR order first (SDDMM.py:39-43)."""
    compare(result.flatten().contiguous()[mask.to("cpu").long()], result_ref, verbose)


_NAMES = {1: "csr", 2: "bcsr", 3: "vec"}


class pcsr_sddmm(pcsr_spmm):
    """One PCSR variant for SDDMM.  Construction, attributes and argument errors are those of ``pcsr_spmm``
    (SDDMM.py:46-116 repeats PCSR.py's constructor)."""

    def _operator(self, suffix=""):
        return getattr(SDDMM, "%s%s_sddmm%s" % (_NAMES[self.vec_size], "_split" if self.if_split else "", suffix))

    def _ones(self, dim):
        pad = max(self.vec_size, 2)
        A = torch.ones((self.mtx_nodes + pad - 1) // pad * pad, dim, device="cuda")
        return A, torch.ones(self.mtx_nodes, dim, device="cuda")

    def get_sddmm_result(self, dim, blkWarpNum):
        """<A[row], B[col]> per stored entry with A = B = ones; the result goes to ``self.result`` on the CPU
        (SDDMM.py:119-156).  CF = ceil(dim / 32) as in the reference."""
        assert torch.cuda.is_available()
        A, B = self._ones(dim)
        self.result = self._operator()(A, B, *self._sparse_args(), (dim + 31) // 32, blkWarpNum | self.bw_flags).to("cpu")
        return self.result

    def profiling(self, blkWarpNum, dim, verbose=True):
        """GFLOP/s (int) of this variant (SDDMM.py:158-230); the blocked twins take the true nnz before CF."""
        assert torch.cuda.is_available()
        A, B = self._ones(dim)
        args = self._sparse_args()
        if self.vec_size != 1:
            args.append(self.mtx_edges)
        throughput = self._operator("_profile")(A, B, *args, (dim + 31) // 32, blkWarpNum | self.bw_flags)
        if verbose:
            print("dim: {} gflops: {:.0f}".format(dim, throughput))
        return throughput

    def cusparse_ref(self, dim=None, is_profiling=False, verbose=True):
        """The vendor library on the plain CSR arrays (SDDMM.py:232-254).  It writes into the value array it is
        given, so it gets a copy: the device arrays of a graph are shared by all operators built on it."""
        assert torch.cuda.is_available()
        if self.if_split or self.vec_size != 1:
            raise ValueError("cusparse only support vec_size=1 and if_split=False")
        A, B = self._ones(dim)
        values = self.val.clone()
        if is_profiling:
            throughput = SDDMM.cusparse_sddmm_profile(A, B, self.rowPtr, self.colIdx, values)
            if verbose:
                print("cusparse-> dim: {} gflops: {:.0f}".format(dim, throughput))
            return throughput
        return SDDMM.cusparse_sddmm_compute(A, B, self.rowPtr, self.colIdx, values).to("cpu")


def _load(name, path, if_auto_gran, blk_size, if_mask):
    """A ``graph_input`` from ``<path>/<name>.mtx``, or from the seeded generator when ``path`` is None."""
    graph = graph_input(mtx_name=name, path=path or "")
    if path is None:
        from . import synth

        rowPtr, colIdx, val, _ = synth.config_graph(name)
        graph.verbose = False
        graph.load_from_csr(rowPtr, colIdx, val, is_avg_granularity=not if_auto_gran, blk_size=blk_size, if_mask=if_mask)
    else:
        graph.load(load_from_mtx=True, is_avg_granularity=not if_auto_gran, blk_size=blk_size, if_mask=if_mask)
    return graph


def get_mtx_info(filelist, path, dim=32, if_auto_gran=True, blk_size=2):
    """One row of the 15 decider features per matrix (SDDMM.py:257-263)."""
    frames = [_load(name, path, if_auto_gran, blk_size, False).mtxinfo_to_pandas() for name in filelist]
    return pd.concat(frames, axis=0, ignore_index=True) if frames else pd.DataFrame()


def column_names(vec_size=2):
    reps = ["vec1", "vec1_split", "vec%d" % vec_size, "vec%d_split" % vec_size]
    return ["%s_TP_%d" % (rep, bw) for bw in WARP_NUMS for rep in reps]


def profile_engine(filelist, path, dim_list, vec_size=2, if_auto_gran=True, verbose=True):
    """{dim: DataFrame[len(filelist), 8]} of GFLOP/s: per blkWarpNum the variants vec1, vec1_split, vecV,
    vecV_split, each verified against the vendor result first (SDDMM.py:266-368).  A graph is loaded once for
    all widths.  ``vec_size`` 3 has no mask (genmask covers 2x1 blocks), so its results are checked through the
    block values instead: stored entries equal ``dim``, padding equals 0."""
    rows = {dim: [] for dim in dim_list}
    for name in filelist:
        if verbose:
            print("-------------{}-------------".format(name))
        graph = _load(name, path, if_auto_gran, vec_size, vec_size == 2)
        variants = [pcsr_sddmm(graph, vec_size=v, if_split=s) for v, s in ((1, False), (1, True), (vec_size, False), (vec_size, True))]
        for dim in dim_list:
            want = variants[0].cusparse_ref(dim)
            tp = []
            for bw in WARP_NUMS:
                for op in variants:
                    got = op.get_sddmm_result(dim=dim, blkWarpNum=bw)
                    torch.cuda.synchronize()
                    if op.vec_size == 1:
                        compare(got, want, verbose)
                    elif op.mask is not None:
                        compare_2d(got, want, op.mask, verbose)
                    else:
                        stored = op.val.to("cpu") != 0
                        compare(got[stored], torch.full_like(got[stored], float(dim)), verbose)
                        if bool((got[~stored] != 0).any()):
                            raise ValueError("Verification FAILED: padding entries are not zero")
                    tp.append(op.profiling(bw, dim, verbose))
            rows[dim].append(tp)
        del variants, graph
        torch.cuda.empty_cache()
    names = column_names(vec_size)
    return {dim: pd.DataFrame(np.array(rows[dim], dtype=np.float64).reshape(len(filelist), len(names)), columns=names)
            for dim in dim_list}


def training_data_gen(dim_list, vec_size, info_df, filelist, path, csv_path, if_auto_gran=True, verbose=True):
    """Writes ``dim<d>.csv`` (GFLOP/s per column) and ``dim<d>_OP_SpMM.csv`` (features + index of the best column)
    under ``csv_path`` (SDDMM.py:371-383); returns the tables."""
    tables = profile_engine(filelist, path, dim_list, vec_size, if_auto_gran, verbose)
    os.makedirs(csv_path, exist_ok=True)
    for dim, tp in tables.items():
        tp.to_csv(os.path.join(csv_path, "dim%d.csv" % dim), index=False)
        best = pd.DataFrame({"OP_SpMM": tp.to_numpy().argmax(axis=1)})
        pd.concat([info_df.reset_index(drop=True), best], axis=1).to_csv(os.path.join(csv_path, "dim%d_OP_SpMM.csv" % dim), index=False)
    return tables


def main(argv=None):
    parser = argparse.ArgumentParser()
    parser.add_argument("--path", type=str, default="./toy_dataset/", help="path to the mtx files")
    parser.add_argument("--dim_list", nargs="*", type=int, default=[32], help="dim_list for training data generation")
    parser.add_argument("--mtx_name", type=str, default="", help="mtx file name")
    parser.add_argument("--vec_size", type=int, default=2, help="vec_size(besides 1) for SDDMM")
    parser.add_argument("--if_auto_gran", type=str, choices=["True", "False"], default="True",
                        help="If to use auto-Granularity, else use avg_row_nnz as split-granularity")
    parser.add_argument("--approx_eval", type=str, choices=["True", "False"], default="False",
                        help="accepted for compatibility with the reference's command lines; unused there as well")
    parser.add_argument("--synthetic", nargs="*", default=None, help="seeded synthetic graphs (C1, C2, ...) instead of mtx files")
    parser.add_argument("--csv_path", type=str, default="./ParamSpMM-log/OGBsddmm/", help="where the tables go")
    args = parser.parse_args(argv)
    print(args)
    if_auto_gran = args.if_auto_gran == "True"
    if args.synthetic:
        path, filelist = None, list(args.synthetic)
    elif args.mtx_name:
        path, filelist = args.path, [args.mtx_name]
    else:
        path = args.path
        filelist = sorted(os.path.basename(f)[:-4] for f in glob.glob(os.path.join(path, "*.mtx")))
    os.makedirs(args.csv_path, exist_ok=True)
    info_file = os.path.join(args.csv_path, "mtx_info.csv")
    if os.path.exists(info_file):
        info_df = pd.read_csv(info_file)
    else:
        info_df = get_mtx_info(filelist, path, if_auto_gran=if_auto_gran, blk_size=args.vec_size)
        info_df.to_csv(info_file, index=False)
    return training_data_gen(args.dim_list, args.vec_size, info_df, filelist, path, args.csv_path, if_auto_gran)


if __name__ == "__main__":
    main()
