"""The forests this package ships, used the way the reference's unchanged decider.py uses them.

``models/rnd_tree_<d>.pkl`` must load with a bare ``pickle.load(open(file, "rb"))`` (decider.py:35-39) and every
class code they can emit must decode, with the reference's own arithmetic over ``dynamic_CF_prompter`` (decider.py:63-80,
PCSR.py:19-42), to a configuration the reference's operators accept.  The loader and the decoder are restated here
line by line so that the test does not depend on this package's SpMMDecider.  ``models/native/`` (the widened class
space) is checked through this package's decider.
"""
import _pickle as ref_pickle  # the module decider.py:5 imports
import math
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MODELS = os.path.join(ROOT, "paramspmm_ae_amd", "models") + os.sep
DIMS = list(range(16, 257, 16))


# ---- decider.py:26-40, PCSR.py:19-42, decider.py:42-80 restated ---------------------------------------------------
def ref_load_pickle(pickle_path, dim):
    pickle_file = pickle_path + "rnd_tree_" + str(dim) + ".pkl"
    if not os.path.exists(pickle_file):
        raise ValueError("pickle file not found for dim-" + str(dim))
    return ref_pickle.load(open(pickle_file, "rb"))


def ref_gap_calculator(dim, CF, warp_size=32):
    t_res = dim % (warp_size * CF)
    if t_res == 0:
        return 0
    return min(dim, CF * warp_size) - t_res


def ref_dynamic_CF_prompter(dim, warp_size=32):
    CF_set = [1, 2, 3, 4, 5, 6, 7, 8][: math.ceil(dim / 32)]
    return [CF for CF in CF_set if ref_gap_calculator(dim, CF, warp_size) < 32]


def ref_model_dim(dim):
    return dim if dim % 32 == 0 else (math.ceil(dim / 32) * 2 - 1) * 16


def ref_decode_tree(code, dim, vec_size_list=[1, 2], warpNum_list=[4, 8]):
    if_split = code % 2
    CF_list = ref_dynamic_CF_prompter(dim)
    len_vec_list = len(vec_size_list)
    vec_size = vec_size_list[code // 2 % len_vec_list]
    len_CF_list = len(CF_list)
    m = code // (len_vec_list * 2) % len_CF_list
    CF = CF_list[m]
    m = code // (len_CF_list * len_vec_list * 2)
    blkWarpNum = warpNum_list[m]  # IndexError for a code outside the reference's 8 * |CF_list| classes
    return if_split, vec_size, CF, blkWarpNum


def _feature_table():
    import pandas as pd

    from paramspmm_ae_amd.train_decider import FEATURES

    info = pd.read_csv(os.path.join(MODELS, "train_data", "mtx_info.csv"))
    return info[FEATURES].to_numpy(dtype=np.float64)


@pytest.mark.parametrize("dim", DIMS)
def test_default_forest_loads_and_decodes_like_the_reference(dim):
    model = ref_load_pickle(MODELS, dim)
    with open(MODELS + "rnd_tree_%d.pkl" % dim, "rb") as f:
        assert f.read(2) != b"\x1f\x8b", "a compressed stream is not what decider.py:38 reads"
    CF_list = ref_dynamic_CF_prompter(dim)
    n_classes = 8 * len(CF_list)
    # every class the forest can emit lies inside the reference's class space ...
    assert all(0 <= int(c) < n_classes for c in model.classes_), (dim, model.classes_)
    assert model.n_features_in_ == 15
    # ... and every prediction over the matrices of the sweep decodes to a legal <if_split, vec_size, CF, blkWarpNum>
    feats = _feature_table()
    assert len(feats) >= 700
    codes = model.predict(feats)
    seen = set()
    for code in codes:
        if_split, vec_size, CF, blkWarpNum = ref_decode_tree(int(code), dim)
        assert if_split in (0, 1) and vec_size in (1, 2) and CF in CF_list and blkWarpNum in (4, 8)
        assert 1 <= CF <= 8 and ref_gap_calculator(dim, CF) < 32
        seen.add((if_split, vec_size, CF, blkWarpNum))
    assert len(seen) >= 2  # the forest distinguishes matrices
    # the reference calls predict on one (1, 15) row and takes .item() (decider.py:91-92)
    assert int(model.predict(feats[:1]).item()) == int(codes[0])


def test_every_requested_width_finds_its_default_forest():
    """gen_model_dict (decider.py:42-61): widths that are not multiples of 32 take the forest of the odd multiple of
    16 in their band; all sixteen files exist."""
    for dim in range(1, 257):
        assert os.path.exists(MODELS + "rnd_tree_%d.pkl" % ref_model_dim(dim))


def test_this_packages_decider_agrees_with_the_restated_reference_on_the_default_forests():
    from paramspmm_ae_amd.decider import REFERENCE_SPACE_PICKLE_PATH, SpMMDecider

    feats = _feature_table()[::37]

    class G:
        def __init__(self, row):
            self.row = row

        def get_info(self):
            return self.row.reshape(1, -1)

    dec = SpMMDecider(REFERENCE_SPACE_PICKLE_PATH)
    dims = [16, 40, 64, 100, 128, 144, 200, 256]
    dec.gen_model_dict(dims)
    for dim in dims:
        model = ref_load_pickle(MODELS, ref_model_dim(dim))
        for row in feats:
            code = model.predict(row.reshape(1, -1)).item()
            assert dec.config_PCSR(G(row), dim) == ref_decode_tree(code, math.ceil(dim / 16) * 16)


@pytest.mark.parametrize("dim", DIMS)
def test_native_forest_decodes_over_its_recorded_list(dim):
    from paramspmm_ae_amd import _capi
    from paramspmm_ae_amd.PCSR import decider_CF_list
    from paramspmm_ae_amd.decider import DEFAULT_PICKLE_PATH, SpMMDecider

    dec = SpMMDecider(DEFAULT_PICKLE_PATH)
    model = dec.load_pickle(dim)
    wide = decider_CF_list(dim)
    assert list(model.psp_cf_list_) == wide
    assert all(0 <= int(c) < 8 * len(wide) for c in model.classes_)
    for code in model.classes_:
        if_split, vec_size, CF, blkWarpNum = dec.decode_tree(int(code), dim, CF_list=wide)
        assert CF in wide and blkWarpNum in (4, 8) and vec_size in (1, 2)
        _capi.spmm_plan(dim, CF, blkWarpNum)  # the library has a plan for it
