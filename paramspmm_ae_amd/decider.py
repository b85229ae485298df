"""SpMM-decider: per-dimension random forests that pick ``<if_split, vec_size, CF, blkWarpNum>`` from the 15
matrix features (same surface as the reference's decider.py:18-93).

The forests are the ones trained on MI355X timings by ``train_decider.py`` and stored as
``rnd_tree_<dim>.pkl`` (one per multiple of 16 up to 256).  The class code is the column index of the sweep
table: blkWarpNum-major, then CF in ``dynamic_CF_prompter(dim)`` order, then the four representations
(vec1, vec1_split, vec2, vec2_split) -- see ``decode_tree``.
"""
import math
import os
import pickle

from .PCSR import dynamic_CF_prompter

DEFAULT_PICKLE_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "models") + os.sep


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
                self.tree_dict[dim] = pickle.load(f)
        return self.tree_dict[dim]

    def gen_model_dict(self, dim_list):
        if dim_list is None or len(dim_list) == 0:
            raise ValueError("dim_list must be assigned and non-empty")
        self.model_dict = {dim: self.load_pickle(model_dim_for(dim)) for dim in dim_list}

    def decode_tree(self, code, dim, vec_size_list=(1, 2), warpNum_list=(4, 8)):
        """class code -> (if_split, vec_size, CF, blkWarpNum) (decider.py:63-80); if_split is the int 0/1."""
        CF_list = dynamic_CF_prompter(dim)
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
        code = self.model_dict[dim].predict(graph.get_info()).item()
        return self.decode_tree(code, math.ceil(dim / 16) * 16)
