"""SpMM-decider: per-dimension random forests that pick ``<if_split, vec_size, CF, blkWarpNum>`` from the 15
matrix features (same surface as the reference's decider.py:18-93).

The forests are trained on MI355X timings by ``train_decider.py`` and stored as ``rnd_tree_<dim>.pkl`` (one per
multiple of 16 up to 256), in two sets.  ``models/`` holds forests on the reference's own class space (class code =
column index of the reference's sweep table: blkWarpNum-major, then CF in ``dynamic_CF_prompter(dim)`` order, then
the four representations vec1, vec1_split, vec2, vec2_split): plain pickles that the reference's unchanged
decider.py loads and decodes.  ``models/native/`` holds forests on the widened space, whose CF axis is
``decider_CF_list(dim)`` -- the reference's list followed by native wave64 configurations packed into the same
integer -- and who carry that axis as ``psp_cf_list_``; they are this class's default.  ``config_PCSR`` decodes
either kind with the list the forest was trained on.
"""
import math
import os
import gzip
import pickle

from .PCSR import decider_CF_list, dynamic_CF_prompter

REFERENCE_SPACE_PICKLE_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "models") + os.sep
DEFAULT_PICKLE_PATH = os.path.join(REFERENCE_SPACE_PICKLE_PATH, "native") + os.sep


def model_dim_for(dim):
    """Forest that serves ``dim``: itself for multiples of 32, else the odd multiple of 16 inside the same
    32-wide band (decider.py:52-55)."""
    return dim if dim % 32 == 0 else (math.ceil(dim / 32) * 2 - 1) * 16


class SpMMDecider(object):
    def __init__(self, pickle_path=DEFAULT_PICKLE_PATH):
        if pickle_path is None:
            raise ValueError("pickle_path must be assigned")
        self.pickle_path = pickle_path
        self.tree_dict = {}
        self.model_dict = {}

    def load_pickle(self, dim):
        if dim not in self.tree_dict:
            pickle_file = self.pickle_path + "rnd_tree_" + str(dim) + ".pkl"
            if not os.path.exists(pickle_file):
                raise ValueError("pickle file not found for dim-" + str(dim) + " at path: " + pickle_file + "\n")
            with open(pickle_file, "rb") as f:
                gz = f.read(2) == b"\x1f\x8b"  # gzip-compressed pickles are accepted as well
            with (gzip.open if gz else open)(pickle_file, "rb") as f:
                self.tree_dict[dim] = pickle.load(f)
        return self.tree_dict[dim]

    def gen_model_dict(self, dim_list):
        if dim_list is None or len(dim_list) == 0:
            raise ValueError("dim_list must be assigned and non-empty")
        self.model_dict = {dim: self.load_pickle(model_dim_for(dim)) for dim in dim_list}

    def decode_tree(self, code, dim, vec_size_list=(1, 2), warpNum_list=(4, 8), CF_list=None):
        """class code -> (if_split, vec_size, CF, blkWarpNum) (decider.py:63-80); if_split is the int 0/1.
        ``CF_list``: the CF axis the forest was trained on; default ``dynamic_CF_prompter(dim)``, the reference's
        (decider.py:69).  A forest on the widened space is decoded with ``decider_CF_list(dim)``, which
        ``config_PCSR`` takes from the forest itself."""
        CF_list = dynamic_CF_prompter(dim) if CF_list is None else CF_list
        code = int(code)
        if_split = code % 2
        code //= 2
        vec_size = vec_size_list[code % len(vec_size_list)]
        code //= len(vec_size_list)
        CF = CF_list[code % len(CF_list)]
        blkWarpNum = warpNum_list[code // len(CF_list)]
        return if_split, vec_size, CF, blkWarpNum

    def config_PCSR(self, graph, dim):
        if dim not in self.model_dict:
            raise ValueError("dim-" + str(dim) + " not found in model_dict")
        model = self.model_dict[dim]
        code = model.predict(graph.get_info()).item()
        # a forest records the CF axis of its training table in ``psp_cf_list_`` (train_decider.py); one without it
        # was trained on the reference's own table (python -m paramspmm_ae_amd.PCSR, PCSR.py:781-788)
        rounded = math.ceil(dim / 16) * 16
        cf_list = getattr(model, "psp_cf_list_", None)
        return self.decode_tree(code, rounded, CF_list=dynamic_CF_prompter(rounded) if cf_list is None else list(cf_list))

    def candidates_PCSR(self, graph, dim, k=3):
        """The ``k`` configurations the forest rates highest for this matrix, best first (an addition of this build: the
        first one is ``config_PCSR``'s answer; ``GNN.configure_operators(..., try_candidates=k)`` times them on the
        matrix itself and keeps the fastest, which bounds the cost of a wrong first guess)."""
        if dim not in self.model_dict:
            raise ValueError("dim-" + str(dim) + " not found in model_dict")
        model = self.model_dict[dim]
        info = graph.get_info()
        proba = model.predict_proba(info)[0]
        first = model.predict(info).item()
        # the predicted class leads (ties in probability are broken the way predict() breaks them), then by rating;
        # classes no tree voted for are not candidates
        order = sorted(range(len(proba)), key=lambda i: (model.classes_[i] != first, -proba[i]))
        codes = [model.classes_[i] for i in order if proba[i] > 0 or model.classes_[i] == first][:max(1, k)]
        rounded = math.ceil(dim / 16) * 16
        cf_list = getattr(model, "psp_cf_list_", None)
        cf_list = dynamic_CF_prompter(rounded) if cf_list is None else list(cf_list)
        return [self.decode_tree(code, rounded, CF_list=cf_list) for code in codes]


def evaluate(filelist, path, dim_list, pickle_path=DEFAULT_PICKLE_PATH, verbose=True):
    """The reference's evaluation run (decider.py:97-175): for every matrix and width the decider's configuration is
    verified against ``torch.sparse.mm`` and then timed beside the vendor library (COO, CSC and CSR formats) and the
    row-caching baseline.  ``path`` None takes ``filelist`` as names of the seeded
    synthetic graphs.  Returns one row per (matrix, width) with the GFLOP/s of each."""
    import pandas as pd
    import torch

    from .PCSR import coo_spmm, csc_spmm, pcsr_spmm
    from .graph_input import graph_input
    from .verification import SpMM_verification

    decider = SpMMDecider(pickle_path)
    decider.gen_model_dict(dim_list)
    rows = []
    for name in filelist:
        if verbose:
            print("-------------mtx: {}-------------".format(name))
        graph = graph_input(mtx_name=name, path=path or "")
        graph.verbose = verbose
        if path is None:
            from . import synth

            rowPtr, colIdx, val, _ = synth.config_graph(name)
            graph.load_from_csr(rowPtr, colIdx, val, if_mask=True)
        else:
            graph.load(load_from_mtx=True, if_mask=True)
        c = graph.csr_data
        check = SpMM_verification(1, c.rowPtr, c.colIdx, c.val, baseline=True)
        coo, csc = coo_spmm(graph), csc_spmm(graph)
        plain = pcsr_spmm(graph, vec_size=1, if_split=False)
        for dim in dim_list:
            check.reference(dim, verbose=False)
            if_split, vec_size, CF, blkWarpNum = decider.config_PCSR(graph, dim)
            op = pcsr_spmm(graph=graph, vec_size=vec_size, if_split=if_split, CF=CF, blkWarpNum=blkWarpNum)
            op.get_spmm_result(dim)
            check.compare(op.result, name, verbose)
            rows.append({"mtx_name": name, "dim": dim, "if_split": int(if_split), "vec_size": vec_size, "CF": CF,
                         "blkWarpNum": blkWarpNum, "param": op.profiling(dim, verbose=verbose),
                         "coo": coo.profiling(dim, verbose=verbose), "csc": csc.profiling(dim, verbose=verbose),
                         "cusparse": plain.cusparse_ref(dim, is_profiling=True, verbose=verbose),
                         "gespmm": plain.gespmm_ref(dim, is_profiling=True, verbose=verbose)})
            if verbose:
                print("=======================================")
        del coo, csc, plain, graph
        torch.cuda.empty_cache()
    return pd.DataFrame(rows)


def main(argv=None):
    import argparse
    import glob

    parser = argparse.ArgumentParser()
    parser.add_argument("--path", type=str, default="./dataset/all-mtx/", help="path to the mtx files")
    parser.add_argument("--dim_list", nargs="*", type=int, default=[16, 32, 48, 64, 80, 96, 112, 128])
    parser.add_argument("--mtx_name", type=str, default="", help="mtx file name")
    parser.add_argument("--pickle_path", type=str, default=DEFAULT_PICKLE_PATH, help="directory of rnd_tree_<dim>.pkl")
    parser.add_argument("--synthetic", nargs="*", default=None, help="seeded synthetic graphs (C1, C2, ...) instead of mtx files")
    args = parser.parse_args(argv)
    print(args)
    if args.synthetic:
        path, filelist = None, list(args.synthetic)
    elif args.mtx_name:
        path, filelist = args.path, [args.mtx_name]
    else:
        path = args.path
        filelist = sorted(os.path.basename(f)[:-4] for f in glob.glob(os.path.join(path, "*.mtx")))
    table = evaluate(filelist, path, args.dim_list, args.pickle_path)
    if len(table):
        print(table.to_string(index=False))
        ratio = table["param"] / table["cusparse"].clip(lower=1)
        print("geometric-mean speedup over the vendor CSR SpMM: %.2f" % math.exp(ratio.apply(math.log).mean()))
    return table


if __name__ == "__main__":
    main()
