"""Configuration sweep: times every ``<representation, CF, blkWarpNum>`` of a graph for a list of feature
widths.  It is the counterpart of the reference's ``profile_engine`` (PCSR.py:672-806) and produces the same
column order -- blkWarpNum-major, then CF in list order, then the representations vec1, vec1_split, vec2,
vec2_split -- so that the arg-max column index is the class code ``decode_tree`` expects.  The CF list is
``decider_CF_list``: the reference's ``dynamic_CF_prompter`` entries followed by native wave64 configurations
(lanes per row, entries in flight, even division), which travel in the same integer argument.
"""
import numpy as np
import torch

from .PCSR import cf_label, decider_CF_list, dynamic_CF_prompter, native_CF_prompter, pcsr_spmm

WARP_NUMS = (4, 8)
REPRESENTATIONS = (("vec1", 1, False), ("vec1_split", 1, True), ("vec2", 2, False), ("vec2_split", 2, True))


def native_configs(dim):
    """The packed CF values the sweep adds to the reference's list for ``dim``."""
    return native_CF_prompter(dim)


def column_names(dim, cfs=None, vec_size=2):
    """``cfs``: the CF list when it is not ``decider_CF_list(dim)`` (the reference's own list, or its --if_DCP False
    ablation)"""
    cfs = decider_CF_list(dim) if cfs is None else cfs
    reps = ("vec1", "vec1_split", "vec%d" % vec_size, "vec%d_split" % vec_size)
    return ["%s_TP_%s%d" % (rep, cf_label(cf), bw) for bw in WARP_NUMS for cf in cfs for rep in reps]


def decode_column(dim, col, cfs=None):
    """column index -> (if_split, vec_size, CF, blkWarpNum): the arithmetic of decider.py:63-80."""
    cfs = decider_CF_list(dim) if cfs is None else cfs
    _, vec_size, if_split = REPRESENTATIONS[col % 4]
    cf = cfs[col // 4 % len(cfs)]
    bw = WARP_NUMS[col // (4 * len(cfs))]
    return int(if_split), vec_size, cf, bw


def operators_of(graph, vec_size=2):
    """The four representations of a loaded graph_input on the GPU, in column order."""
    return [pcsr_spmm(graph, vec_size=v if v == 1 else vec_size, if_split=s) for _, v, s in REPRESENTATIONS]


def sweep_dim(ops, dim, nnz, n_rows, warmup=3, iters=10, X=None, verify=None, cfs=None, flush_bytes=0):
    """Times all columns for one width.  Returns (ms[cols], gflops[cols]).

    ``verify``: optional callable(result_tensor, column_name) run once per column on A*X before timing
    (the reference verifies every swept configuration, PCSR.py:759-770).  ``flush_bytes``: see pcsr_spmm.time_ms.
    """
    pad = max(op.vec_size for op in ops)
    pad = 2 if pad == 1 else pad
    rows = (n_rows + pad - 1) // pad * pad
    if X is None:
        X = torch.ones(rows, dim, device="cuda")
    cfs = decider_CF_list(dim) if cfs is None else cfs
    names = column_names(dim, cfs, ops[-1].vec_size if ops[-1].vec_size != 1 else 2)
    ms = np.zeros(len(names))
    col = 0
    for bw in WARP_NUMS:
        for cf in cfs:
            for op in ops:
                if verify is not None:
                    verify(op._spmm(X, CF=cf, blkWarpNum=bw)[:n_rows], names[col])
                if op.vec_size == 3:  # the generic-block operators have no event-timed twin: use their *_profile
                    ms[col] = 2.0 * nnz * dim / 1e6 / max(op.cf_warpnum_profiling(cf, bw, x=X, verbose=False), 1)
                else:
                    ms[col] = op.time_ms(X, CF=cf, blkWarpNum=bw, warmup=warmup, iters=iters, flush_bytes=flush_bytes)
                col += 1
    gflops = 2.0 * nnz * dim / 1e6 / ms
    return ms, gflops
