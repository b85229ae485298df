"""CPU-side tests of the product: the C ABI library loads and exports every declared symbol, the host-side index
construction (row split, 2x1 BCSR) is bit-exact against the oracle / SciPy, the format builder reproduces the
reference's statistics and normalisation, the CF search space and the decider decoding match the reference's
integer functions, and the extension modules export the reference's binding names."""
import ctypes
import math
import os
import re

import numpy as np
import pytest
import torch

from conftest import ROOT, pubmed_pattern, random_csr


def test_c_abi_exports_every_declared_symbol():
    from paramspmm_ae_amd import _capi

    header = open(os.path.join(ROOT, "include", "paramsp.h")).read()
    declared = set(re.findall(r"\b(psp_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 18
    for name in declared:
        assert hasattr(_capi.lib, name), name
    assert _capi.lib.psp_version() >= 100
    # every entry point the python binding types is declared in the header
    assert set(_capi.SIGNATURES) <= declared


def test_spmm_plan_mapping():
    from paramspmm_ae_amd import _capi
    from oracle.oracle import CF_TABLE

    for N, cfs in CF_TABLE.items():
        for cf in cfs:
            for bw in (4, 8):
                p = _capi.spmm_plan(N, cf, bw)
                assert p["vec"] == 4 and p["waves_per_block"] == bw
                tile = p["lanes_per_row"] * p["coarsen"] * p["vec"]
                assert tile * p["col_tiles"] >= N > tile * (p["col_tiles"] - 1)
                assert tile <= 32 * cf or p["col_tiles"] == 1  # a lane group never owns more than 32*CF columns
                assert p["rows_per_wave"] * p["lanes_per_row"] == 64
                assert 1 <= p["unroll"] <= p["lanes_per_row"]
    assert _capi.spmm_plan(50, 1, 4)["vec"] == 2 and _capi.spmm_plan(51, 1, 4)["vec"] == 1
    for bad in ((16, 0, 4), (16, 9, 4), (16, 1, 6), (0, 1, 4), (64, _capi.CF_NATIVE | (7 << 3), 4),
                (64, _capi.pack_cf(4, 8, 2) | (3 << 6), 4), (64, _capi.CF_NATIVE | (1 << 14), 4)):
        with pytest.raises(_capi.ParamSpError):
            _capi.spmm_plan(*bad)
    # native configurations: every field is honoured, vectors per lane are capped by the width
    p = _capi.spmm_plan(128, _capi.pack_cf(2, 16, 2, 32, even_split=True), 8)
    assert (p["coarsen"], p["lanes_per_row"], p["rows_per_wave"], p["unroll"], p["col_tiles"], p["log_segs_per_wave"],
            p["even_split"]) == (2, 16, 4, 2, 1, 5, 1)
    assert _capi.spmm_plan(16, _capi.pack_cf(4, 8, 2), 4)["coarsen"] == 4
    assert _capi.spmm_plan(8, _capi.pack_cf(4, 8, 2), 4)["coarsen"] == 2
    # one register set from four entries in flight on, or two entries with 8 lanes per row or more; two sets otherwise
    sets = _capi.lib.psp_spmm_register_sets
    assert [sets(u, l) for u, l in ((4, 4), (4, 8), (8, 8), (2, 8), (2, 64))] == [1] * 5
    assert [sets(u, l) for u, l in ((2, 2), (2, 4), (1, 1), (1, 8), (1, 64))] == [2] * 5
    assert _capi.spmm_plan(16, 1, 4)["register_sets"] == 1 and _capi.spmm_plan(256, 8, 4)["register_sets"] == 2
    # per-launch XCD stripe in the flag bits of blkWarpNum
    assert _capi.spmm_plan(64, 1, 4)["xcd_stripe_rows"] == 0
    for rows in (256, 768, 6144, 65280):
        p = _capi.spmm_plan(64, 2, 8 | _capi.bw_stripe(rows))
        assert (p["xcd_stripe_rows"], p["waves_per_block"], p["coarsen"]) == (rows, 8, 2)
    assert _capi.bw_stripe(0) == 0 and _capi.bw_stripe(None) == 0
    for bad in (100, 65536, -256):
        with pytest.raises(ValueError):
            _capi.bw_stripe(bad)
    with pytest.raises(_capi.ParamSpError):
        _capi.spmm_plan(64, 1, 4 | (1 << 20))
    # options
    assert _capi.get_option("align_pct") == 50 and _capi.get_option("xcd_stripe_rows") == 8192
    _capi.set_option("align_pct", 25)
    assert _capi.get_option("align_pct") == 25
    _capi.set_option("align_pct", 50)
    with pytest.raises(_capi.ParamSpError):
        _capi.set_option("no_such_option", 1)


@pytest.mark.parametrize("g", [1, 7, 32, 96])
def test_split_host_functions_match_oracle(oracle, g):
    import paramspmm_ae_amd  # noqa: F401
    import ParamSpMM
    import ParamSpCONV

    rowPtr, _, _ = random_csr(100_000, 9, 3, empty_frac=0.2, hub=(11, 5000))
    want_rps, want_tr = oracle.split_csr(rowPtr, g)
    rp_t = torch.from_numpy(rowPtr)
    for mod in (ParamSpMM, ParamSpCONV):
        rps, tr = mod.split_csr(rp_t, g)
        assert rps.dtype == torch.int32 and tr.dtype == torch.int32
        assert np.array_equal(rps.numpy(), want_rps) and np.array_equal(tr.numpy(), want_tr)
        k = np.diff(rowPtr)
        off = torch.from_numpy(np.concatenate([[0], np.cumsum(-(-k // g))]).astype(np.int32))
        rps2, tr2 = mod.split_csr_par(rp_t, off, g)  # 100k rows: the threaded path
        assert np.array_equal(rps2.numpy(), want_rps) and np.array_equal(tr2.numpy(), want_tr)


def test_split_host_errors():
    import paramspmm_ae_amd  # noqa: F401
    import ParamSpMM

    rp = torch.tensor([0, 3, 5], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="granularity"):
        ParamSpMM.split_csr(rp, 0)
    with pytest.raises(RuntimeError, match="int32"):
        ParamSpMM.split_csr(rp.long(), 4)
    with pytest.raises(RuntimeError, match="prefix sum"):
        ParamSpMM.split_csr_par(rp, torch.tensor([0, 1, 5], dtype=torch.int32), 4)
    rps, tr = ParamSpMM.split_csr(torch.zeros(4, dtype=torch.int32), 32)
    assert rps.tolist() == [0] and tr.numel() == 0


@pytest.mark.parametrize("n", [1, 2, 9, 1000, 4001])
def test_bcsr_host_builder_matches_oracle_and_scipy(oracle, n):
    import scipy.sparse as sp
    from paramspmm_ae_amd.graph_input import build_bcsr

    rowPtr, colIdx, val = random_csr(n, min(7, n), n, empty_frac=0.2)
    rpb, cib, vb = build_bcsr(rowPtr, colIdx, val)
    o = oracle.bcsr_build(rowPtr, colIdx, val, ncols=n + (n & 1))
    assert np.array_equal(rpb, o[0]) and np.array_equal(cib, o[1]) and np.array_equal(vb, o[2])
    m = n + (n & 1)
    indptr = np.concatenate([rowPtr, [rowPtr[-1]] * (m - n)])
    b = sp.csr_matrix((val, colIdx, indptr), shape=(m, m)).tobsr(blocksize=(2, 1))
    assert np.array_equal(rpb, b.indptr) and np.array_equal(cib, b.indices)
    assert np.array_equal(vb, b.data.reshape(-1, 2))


def test_bcsr_rejects_bad_columns():
    from paramspmm_ae_amd import _capi

    rp = np.array([0, 1], np.int32)
    ci = np.array([5], np.int32)
    assert _capi.lib.psp_bcsr_count(_capi.ptr(rp), _capi.ptr(ci), 1, 2) == -1
    assert b"out of range" in _capi.lib.psp_last_error()


@pytest.mark.parametrize("which", ["orig", "rabbit"])
def test_format_builder_on_pubmed(oracle, which, tmp_path):
    """load() from a MatrixMarket file of the reference's pubmed pattern: counts, statistics, normalisation."""
    import scipy.io
    from paramspmm_ae_amd.graph_input import graph_input

    m = pubmed_pattern(which)
    import scipy.sparse as sp

    scipy.io.mmwrite(str(tmp_path / "pm.mtx"), sp.tril(m).tocoo(), symmetry="symmetric")
    g = graph_input("pm", str(tmp_path) + os.sep)
    g.verbose = False
    g.load(load_from_mtx=True)
    assert (g.mtx_nodes, g.mtx_edges) == (19717, 88651)
    assert g.csr_data.split_granularity == 32 and g.bcsr_data.split_granularity == 32
    assert g.csr_data.target_row.numel() == 20005
    assert g.bcsr_data.colIdx.numel() == (88469 if which == "orig" else 81018)
    assert g.bcsr_data.target_row.numel() == (10293 if which == "orig" else 10240)
    assert int(g.csr_data.max_row_nnz) == 171 and int(g.csr_data.real_nrow) == 19717
    assert g.bcsr_data.val.shape[1] == 2 and g.bcsr_data.num_nodes == 9859
    # statistics against the numpy restatement of graph_input.py:48-129
    st = oracle.format_stats(m.indptr, m.indices, m.nnz)
    info = g.get_info()
    assert info.shape == (1, 15)
    np.testing.assert_allclose(
        info[0, :13],
        [19717, 88651, 88651 / 19717**2, 171, 19717, 1.0, st["avg_degree"], st["COV"], st["real_avg_degree"],
         st["real_COV"], st["max_bw"], st["avg_bw"], st["split_ratio"]], rtol=1e-6)
    assert abs(info[0, 14] - (0.501 if which == "orig" else 0.547)) < 1e-3
    assert np.array_equal(g.csr_data.rowPtr_split.numpy(), oracle.split_csr(m.indptr, 32)[0])
    # normalised load: D^-1/2 (A+I) D^-1/2 in float64, rounded once to fp32
    g2 = graph_input("pm", str(tmp_path) + os.sep)
    g2.verbose = False
    g2.load(load_from_mtx=True, is_normalize=True)
    coo = m.tocoo()
    rp, ci, v = oracle.normalize_adj_closed_form(coo.row, coo.col, 19717)
    assert g2.mtx_edges == 108365
    assert np.array_equal(g2.csr_data.rowPtr.numpy(), rp) and np.array_equal(g2.csr_data.colIdx.numpy(), ci)
    assert np.array_equal(g2.csr_data.val.numpy(), v)
    # GIN: off-diagonal 1, diagonal 1.5
    g3 = graph_input("pm", str(tmp_path) + os.sep)
    g3.verbose = False
    g3.load(load_from_mtx=True, GIN_epsilon=0.5)
    rows = np.repeat(np.arange(19717), np.diff(g3.csr_data.rowPtr.numpy()))
    d = rows == g3.csr_data.colIdx.numpy()
    vv = g3.csr_data.val.numpy()
    assert np.all(vv[d] == 1.5) and np.all(vv[~d] == 1.0) and g3.mtx_edges == 108365


def test_format_builder_from_arrays_and_synthetic_closed_form(oracle):
    from paramspmm_ae_amd import synth
    from paramspmm_ae_amd.graph_input import graph_input

    r, c, n = synth.chung_lu(5001, 20000, seed=3, max_degree=300)
    rowPtr, colIdx, val = synth.to_gcn_csr(r, c, n)
    rp2, ci2, v2 = oracle.normalize_adj_closed_form(np.concatenate([r, c]), np.concatenate([c, r]), n)
    assert np.array_equal(rowPtr, rp2) and np.array_equal(colIdx, ci2) and np.array_equal(val, v2)
    g = graph_input("cl", "")
    g.verbose = False
    g.load_from_csr(rowPtr, colIdx, val, manual_granularity=8)
    assert g.csr_data.split_granularity == 8 and g.bcsr_data.num_nodes == 2501
    st = oracle.format_stats(rowPtr, colIdx, colIdx.size, manual_granularity=8)
    assert abs(float(g.csr_data.split_ratio) - st["split_ratio"]) < 1e-6
    assert g.csr_data.target_row.numel() == int(st["row_split_nnz"].sum())
    stb = oracle.format_stats(g.bcsr_data.rowPtr.numpy(), None, float(g.bcsr_data.colIdx.numel()), csr_flag=False,
                              manual_granularity=8)
    assert abs(float(g.bcsr_data.split_ratio) - stb["split_ratio"]) < 1e-6
    g.load_from_csr(rowPtr, colIdx, val, is_avg_granularity=True)
    assert g.csr_data.split_granularity == int(colIdx.size / n)
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="no GPU"):
            g.load_from_csr(rowPtr, colIdx, val, if_mask=True)


def test_cf_search_space_and_decoding_match_reference_integers(oracle):
    from oracle.oracle import CF_TABLE
    from paramspmm_ae_amd.PCSR import decider_CF_list, dynamic_CF_prompter, gap_calculator
    from paramspmm_ae_amd.decider import SpMMDecider, model_dim_for
    from paramspmm_ae_amd import _capi, sweep

    for dim in range(1, 300):
        assert dynamic_CF_prompter(dim) == oracle.dynamic_CF_prompter(dim)
        for cf in range(1, 9):
            assert gap_calculator(dim, cf) == oracle.gap_calculator(dim, cf)
        assert model_dim_for(dim) == oracle.model_dim(dim)
    for dim, cfs in CF_TABLE.items():
        assert dynamic_CF_prompter(dim) == cfs
    d = SpMMDecider("unused/")
    for dim, cfs in CF_TABLE.items():
        # the reference's own class space: 8 * |CF_list| codes, decoded with its arithmetic
        names = sweep.column_names(dim, cfs)
        assert len(names) == 8 * len(cfs)
        for code in range(8 * len(cfs)):
            got = d.decode_tree(code, dim, CF_list=cfs)
            assert got == d.decode_tree(code, dim)  # the default CF axis is the reference's (decider.py:69)
            assert got == oracle.decode_tree(code, dim) == sweep.decode_column(dim, code, cfs)
            rep = ["vec1", "vec1_split", "vec2", "vec2_split"][code % 4]
            assert names[code] == "%s_TP_%d%d" % (rep, got[2], got[3])
        # the widened space: the same arithmetic over the reference's list followed by the native configurations
        wide = decider_CF_list(dim)
        assert wide[: len(cfs)] == cfs and all(c & _capi.CF_NATIVE for c in wide[len(cfs):])
        assert wide == decider_CF_list(dim - 15)  # one list per 32-wide band, like the forests (decider.py:52-55)
        names = sweep.column_names(dim)
        assert len(names) == len(set(names)) == 8 * len(wide)
        for code in range(8 * len(wide)):
            if_split, vec, cf, bw = d.decode_tree(code, dim, CF_list=wide)
            assert (if_split, vec, cf, bw) == sweep.decode_column(dim, code)
            assert (if_split, vec) == ((code % 2), (1, 2)[code // 2 % 2]) and cf == wide[code // 4 % len(wide)]
            assert bw == (4, 8)[code // (4 * len(wide))]
            plan = _capi.spmm_plan(dim, cf, bw)  # every class is a configuration the library accepts
            assert plan["lanes_per_row"] * plan["coarsen"] * plan["vec"] * plan["col_tiles"] >= dim
            if cf & _capi.CF_NATIVE:
                c, lanes, unroll, segs, even = _capi.unpack_cf(cf)
                assert (plan["coarsen"], plan["lanes_per_row"], plan["unroll"], bool(plan["even_split"])) == (c, lanes, unroll, even)
                assert _capi.pack_cf(c, lanes, unroll, segs, even) == cf
    assert [model_dim_for(x) for x in (16, 24, 32, 40, 48, 100, 128, 250)] == [16, 16, 32, 48, 48, 112, 128, 240]


def test_decider_round_trip_with_a_forest_trained_in_test(tmp_path):
    import pickle
    from sklearn.ensemble import RandomForestClassifier
    from paramspmm_ae_amd.decider import SpMMDecider

    rng = np.random.default_rng(0)
    X = np.repeat(rng.random((60, 1)), 15, axis=1)  # every feature carries the same signal
    y = (X[:, 0] > 0.5).astype(int) * 5 + 1  # classes 1 and 6 of the 16 codes of width 64
    clf = RandomForestClassifier(n_estimators=10, random_state=0).fit(X, y)
    with open(tmp_path / "rnd_tree_64.pkl", "wb") as f:
        pickle.dump(clf, f)

    class G:
        def __init__(self, v):
            self.v = v

        def get_info(self):
            return self.v.reshape(1, -1)

    d = SpMMDecider(str(tmp_path) + os.sep)
    with pytest.raises(ValueError, match="pickle file not found"):
        d.gen_model_dict([64, 40])  # 40 is served by the forest of 48, which is missing
    import shutil

    shutil.copy(tmp_path / "rnd_tree_64.pkl", tmp_path / "rnd_tree_48.pkl")
    d.gen_model_dict([64, 40, 48])  # 40 and 48 share the forest of 48
    assert d.model_dict[40] is d.model_dict[48]
    lo, hi = np.full(15, 0.1), np.full(15, 0.9)
    # a forest without a recorded CF axis was trained on the reference's table
    assert d.config_PCSR(G(lo), 64) == d.decode_tree(1, 64, CF_list=[1, 2]) == (1, 1, 1, 4)
    assert d.config_PCSR(G(hi), 64) == d.decode_tree(6, 64, CF_list=[1, 2]) == (0, 2, 2, 4)
    # one that records the widened axis decodes over it: blkWarpNum 8, fifth CF of the list, vec2 (and class 9:
    # blkWarpNum 4, third CF, vec1_split)
    from paramspmm_ae_amd.PCSR import decider_CF_list

    wide = decider_CF_list(64)
    code_hi = 4 * len(wide) + 4 * 4 + 2
    clf2 = RandomForestClassifier(n_estimators=5, random_state=0).fit(X, np.where(X[:, 0] > 0.5, code_hi, 9))
    clf2.psp_cf_list_ = wide
    with open(tmp_path / "rnd_tree_64.pkl", "wb") as f:
        pickle.dump(clf2, f)
    d2 = SpMMDecider(str(tmp_path) + os.sep)
    d2.gen_model_dict([64])
    assert d2.config_PCSR(G(hi), 64) == (0, 2, wide[4], 8)
    assert d2.config_PCSR(G(lo), 64) == (1, 1, wide[2], 4)
    with pytest.raises(ValueError, match="not found in model_dict"):
        d.config_PCSR(G(lo), 128)


def test_extension_modules_export_the_reference_binding_names():
    import paramspmm_ae_amd  # noqa: F401
    import ParamSpMM
    import ParamSDDMM
    import ParamSpCONV

    spmm = ["split_csr", "split_csr_par", "csr_spmm", "csr_split_spmm", "bcsr_spmm", "bcsr_split_spmm", "vec_spmm",
            "vec_split_spmm", "csr_spmm_profile", "csr_split_spmm_profile", "bcsr_spmm_profile",
            "bcsr_split_spmm_profile", "vec_spmm_profile", "vec_split_spmm_profile", "cusparse_compute",
            "cusparse_profile", "cusparse_compute_csr_alg2", "cusparse_profile_csr_alg2", "cusparse_compute_coo_alg4",
            "cusparse_profile_coo_alg4", "cusparse_compute_csc", "cusparse_profile_csc", "gespmm_compute", "gespmm_profile"]
    sddmm = ["csr_sddmm", "csr_split_sddmm", "bcsr_sddmm", "bcsr_split_sddmm", "vec_sddmm", "vec_split_sddmm",
             "csr_sddmm_profile", "csr_split_sddmm_profile", "bcsr_sddmm_profile", "bcsr_split_sddmm_profile",
             "vec_sddmm_profile", "vec_split_sddmm_profile", "cusparse_sddmm_compute", "cusparse_sddmm_profile", "genmask"]
    conv = ["split_csr", "split_csr_par"] + [f + s for f in ("csr_spmm", "csr_split_spmm", "bcsr_spmm", "bcsr_split_spmm")
                                             for s in ("_forward", "_backward")]
    for mod, names in ((ParamSpMM, spmm), (ParamSDDMM, sddmm), (ParamSpCONV, conv)):
        for n in names:
            assert callable(getattr(mod, n)), (mod.__name__, n)
    # the module reports a launch plan as the C ABI does
    from paramspmm_ae_amd import _capi

    for args in ((16, 1, 4), (128, 4, 8), (256, 8, 4), (96, _capi.pack_cf(2, 8, 2), 4)):
        assert dict(ParamSpMM.spmm_plan(*args)) == _capi.spmm_plan(*args)
    # device entry points refuse CPU tensors instead of falling back
    x = torch.zeros(4, 16)
    rp = torch.zeros(5, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ParamSpMM.csr_spmm(x, rp, rp[:0], x[:0, 0], 1, 4)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ParamSDDMM.csr_sddmm(x, x, rp, rp[:0], x[:0, 0], 1, 4)


@pytest.mark.skipif(not os.path.isdir("/root/reference"), reason="the reference is only mounted in the build container")
def test_reference_python_only_uses_exported_names():
    """Parses the reference's .py files as text (no import, no execution) and checks that every attribute they
    access on the three extension modules exists in this build."""
    import ast

    import paramspmm_ae_amd  # noqa: F401
    import ParamSpMM
    import ParamSDDMM
    import ParamSpCONV

    alias = {"SpMM": ParamSpMM, "SDDMM": ParamSDDMM, "SpCONV": ParamSpCONV,
             "ParamSpMM": ParamSpMM, "ParamSDDMM": ParamSDDMM, "ParamSpCONV": ParamSpCONV}
    used = set()
    for fn in ("PCSR.py", "graph_input.py", "gnn_conv.py", "SDDMM.py", "decider.py", "GNN.py"):
        tree = ast.parse(open(os.path.join("/root/reference", fn)).read())
        imported = {}
        for node in ast.walk(tree):
            if isinstance(node, ast.Import):
                for a in node.names:
                    if a.name in ("ParamSpMM", "ParamSDDMM", "ParamSpCONV"):
                        imported[a.asname or a.name] = alias[a.name]
        for node in ast.walk(tree):
            if isinstance(node, ast.Attribute) and isinstance(node.value, ast.Name) and node.value.id in imported:
                used.add((imported[node.value.id], node.attr))
    assert len(used) > 30
    for mod, attr in used:
        assert hasattr(mod, attr), (mod.__name__, attr)


@pytest.mark.parametrize("R", [1, 2, 3, 4])
def test_host_vbsr_builder_matches_oracle(oracle, R):
    """psp_vbsr_build (blocks of R x 1, the reference's blk_size argument) against the oracle, which is pinned to
    SciPy's tobsr((R,1)); R = 2 must equal psp_bcsr_build."""
    from paramspmm_ae_amd.graph_input import build_bcsr

    for n in (1, 10, 301, 302):
        rowPtr, colIdx, val = random_csr(n, 4.0, seed=n * 7 + R, empty_frac=0.2)
        if R == 2:
            got = build_bcsr(rowPtr, colIdx, val, build_on="host")
        else:
            got = build_bcsr(rowPtr, colIdx, val, build_on="host", blk_size=R)
        want = oracle.vbsr_build(rowPtr, colIdx, val, R, ncols=(n + R - 1) // R * R)
        for a, b in zip(got, want):
            assert a.dtype == b.dtype and np.array_equal(a, b)


def test_sddmm_harness_checks_and_column_orders():
    """compare / compare_2d (SDDMM.py:19-43) and the column orders of the two sweep tables"""
    import torch
    from paramspmm_ae_amd import SDDMM as S
    from paramspmm_ae_amd import _capi, sweep
    from paramspmm_ae_amd.PCSR import dynamic_CF_prompter

    ref = torch.tensor([32.0, 32.0, 32.0])
    S.compare(ref * (1 + 5e-5), ref, verbose=False)
    with pytest.raises(ValueError, match="Verification FAILED"):
        S.compare(ref * (1 + 2e-4), ref, verbose=False)
    with pytest.raises(ValueError, match="is None"):
        S.compare(None, ref)
    blocked = torch.tensor([[32.0, 0.0], [32.0, 32.0]])  # slot 1 is padding
    S.compare_2d(blocked, ref, torch.tensor([0, 2, 3], dtype=torch.int32), verbose=False)
    assert S.column_names(3) == ["vec1_TP_4", "vec1_split_TP_4", "vec3_TP_4", "vec3_split_TP_4",
                                 "vec1_TP_8", "vec1_split_TP_8", "vec3_TP_8", "vec3_split_TP_8"]
    # SpMM sweep: blkWarpNum-major, then CF, then representation; an explicit CF list replaces the prompter's
    assert sweep.column_names(80)[:5] == ["vec1_TP_%d4" % dynamic_CF_prompter(80)[0], "vec1_split_TP_%d4" % dynamic_CF_prompter(80)[0],
                                          "vec2_TP_%d4" % dynamic_CF_prompter(80)[0], "vec2_split_TP_%d4" % dynamic_CF_prompter(80)[0],
                                          "vec1_TP_%d4" % dynamic_CF_prompter(80)[1]]
    assert sweep.column_names(80, cfs=[1, 2, 3], vec_size=3)[10:13] == ["vec3_TP_34", "vec3_split_TP_34", "vec1_TP_18"]
    for dim in (16, 80, 256):
        names = sweep.column_names(dim)
        for col, name in enumerate(names):
            if_split, vec_size, cf, bw = sweep.decode_column(dim, col)
            assert name == "vec%d%s_TP_%s%d" % (vec_size, "_split" if if_split else "", sweep.cf_label(cf), bw)
    assert sweep.cf_label(3) == "3" and sweep.cf_label(_capi.pack_cf(2, 16, 2, 8, even_split=True)) == "c2l16u2w8e"


def test_reordering_restores_community_order_and_is_a_similarity_transform():
    """community_permutation on a randomly permuted block model: members of a planted community end up contiguous
    (checked through the share of entries close to the diagonal), P A P^T keeps every entry, and results computed on
    the reordered graph map back with unpermute_rows."""
    import scipy.sparse as sp
    from paramspmm_ae_amd import reorder, synth

    r, c, n = synth.sbm(6000, 60, 18, 1.5, seed=4, permute=True)
    rowPtr, colIdx, val = synth.to_gcn_csr(r, c, n)
    A = sp.csr_matrix((val, colIdx, rowPtr), shape=(n, n))
    perm = reorder.community_permutation(rowPtr, colIdx, device="cpu")
    assert np.array_equal(np.sort(perm), np.arange(n))
    rp2, ci2, v2 = reorder.permute_csr(rowPtr, colIdx, val, perm, device="cpu")
    B = sp.csr_matrix((v2, ci2, rp2), shape=(n, n))
    want = A[perm][:, perm].tocsr()
    want.sort_indices()
    assert np.array_equal(rp2, want.indptr) and np.array_equal(ci2, want.indices) and np.array_equal(v2, want.data)
    assert all(np.all(np.diff(ci2[rp2[i]:rp2[i + 1]]) > 0) for i in range(0, n, 97))  # columns sorted again

    def near(rp, ci):
        rows = np.repeat(np.arange(n), np.diff(rp))
        return float(np.mean(np.abs(rows - ci) <= 200))
    assert near(rowPtr, colIdx) < 0.2 and near(rp2, ci2) > 0.8  # 18 of ~20 entries per row are in-community
    x = np.random.default_rng(0).standard_normal((n, 3)).astype(np.float32)
    y_new = B @ reorder.permute_rows(x, perm)
    np.testing.assert_allclose(reorder.unpermute_rows(y_new, perm), A @ x, rtol=1e-5, atol=1e-6)
    # degree order: hubs first, a permutation, stable
    dperm = reorder.degree_permutation(rowPtr)
    k = np.diff(rowPtr)
    assert np.array_equal(np.sort(dperm), np.arange(n)) and np.all(np.diff(k[dperm]) <= 0)
    with pytest.raises(ValueError):
        reorder.permute_csr(rowPtr, colIdx, val, np.zeros(n, np.int64), device="cpu")
    # a graph without communities keeps (almost) one label: the order is a permutation all the same
    r, c, n2 = synth.rmat(11, 8 << 11, seed=3)
    rp, ci, v = synth.to_gcn_csr(r, c, n2)
    p2 = reorder.community_permutation(rp, ci, device="cpu")
    assert np.array_equal(np.sort(p2), np.arange(n2))


def test_xcd_stripe_levels_a_matrix_whose_long_rows_cluster():
    """csr_data.xcd_stripe: the longest candidate stripe under which the eight XCDs get equal shares of the entries.
    Uniform rows keep the longest stripe; rows whose length follows the index bits of an R-MAT graph (every stripe
    of 2^k rows lands on the same XCD with the same share) make it pick a candidate that is not a power of two, and
    the share it reports is recomputed here by brute force."""
    from paramspmm_ae_amd import graph_input as gi

    n = 1 << 18

    def fmt_of(deg):
        rp = np.zeros(n + 1, np.int64)
        np.cumsum(deg, out=rp[1:])
        return gi.csr_data(rp.astype(np.int32), np.zeros(1, np.int32), np.zeros(1, np.float32), n, int(rp[-1]))

    def worst_share(deg, stripe):
        x = (np.arange(n) // stripe) % 8
        share = np.bincount(x, weights=deg, minlength=8)
        return share.max() * 8 / share.sum()

    uniform = np.full(n, 5)
    assert fmt_of(uniform).xcd_stripe(False) == 16384  # the longest candidate that leaves two rounds of stripes on 2^18 rows
    # row length = product over the index bits, as in an R-MAT graph
    idx = np.arange(n)
    deg = np.ones(n)
    for b in range(18):
        deg *= np.where((idx >> b) & 1, 0.6, 1.4)
    deg = np.maximum(1, np.round(deg * 8)).astype(np.int64)
    pick = fmt_of(deg).xcd_stripe(False)
    shares = {s: worst_share(deg, s) for s in gi.XCD_STRIPES}
    assert shares[8192] > 1.5 and pick & (pick - 1) != 0  # no power-of-two stripe can level this matrix
    assert shares[pick] <= min(shares.values()) + 1e-9 or shares[pick] <= gi.XCD_IMBALANCE
    # an empty matrix and one too small for two rounds of stripes leave the choice to the library
    small = gi.csr_data(np.arange(101, dtype=np.int32), np.zeros(100, np.int32), np.ones(100, np.float32), 100, 100)
    assert small.xcd_stripe(False) == 0 and small.xcd_stripe(True) == 0


def test_every_configuration_of_the_deciders_list_has_a_plan():
    """The CF axis of the decider's class space (the reference's list followed by the native configurations) at every
    width a forest serves: each entry maps onto the wave64 kernel, covers the width with its column tiles, and the
    native ones keep what they ask for; the widths one forest serves share one list."""
    from paramspmm_ae_amd import _capi
    from paramspmm_ae_amd.PCSR import decider_CF_list, dynamic_CF_prompter, native_CF_prompter

    for dim in range(16, 257, 16):
        cfs = decider_CF_list(dim)
        assert cfs[: len(dynamic_CF_prompter(dim))] == dynamic_CF_prompter(dim) and len(set(cfs)) == len(cfs)
        assert native_CF_prompter(dim) == native_CF_prompter(dim - 15)  # the widths one forest serves share a list
        for cf in cfs:
            for bw in (4, 8):
                p = _capi.spmm_plan(dim, cf, bw)
                assert p["lanes_per_row"] * p["coarsen"] * p["vec"] * p["col_tiles"] >= dim
                assert p["rows_per_wave"] * p["lanes_per_row"] == 64 and 1 <= p["unroll"] <= p["lanes_per_row"]
                u = _capi.unpack_cf(cf)
                if u is not None:
                    c, lanes, unroll, segs, even = u
                    assert (p["coarsen"], p["lanes_per_row"], p["unroll"], p["even_split"]) == (min(c, dim // 4), lanes, unroll, int(even))


def test_decider_fit_on_a_small_table_and_partial_refit_keeps_the_other_widths(tmp_path):
    """train_decider fit: label files in the reference's schema (PCSR.py:815-818), one forest per width that
    SpMMDecider loads and decodes to a configuration of that width's list, and a refit of one width (--dims) that
    leaves the other widths' report entries in place."""
    import json

    import pandas as pd

    from paramspmm_ae_amd import _capi, sweep, train_decider
    from paramspmm_ae_amd.decider import SpMMDecider
    from paramspmm_ae_amd.PCSR import decider_CF_list

    rng = np.random.default_rng(5)
    data, out = tmp_path / "data", tmp_path / "models"
    data.mkdir()
    names = ["%s_n%d_d%d_s%d" % (fam, 1000 * (i + 1), 3 + i, s) for fam in ("cl", "sbm", "band") for i in range(5) for s in range(3)]
    feats = pd.DataFrame(rng.random((len(names), len(train_decider.FEATURES))), columns=train_decider.FEATURES)
    pd.concat([pd.DataFrame({"mtx_name": names}), feats], axis=1).to_csv(data / "mtx_info.csv", index=False)
    for d in (16, 32):
        cols = sweep.column_names(d)
        tp = 100.0 + rng.random((len(names), len(cols)))
        # the first feature decides between two columns, so there is something to learn
        tp[np.arange(len(names)), np.where(feats.iloc[:, 0] > 0.5, 1, len(cols) - 2)] += 50.0
        pd.DataFrame(tp, columns=cols).to_csv(data / ("dim%d.csv" % d), index=False)

    train_decider.main(["fit", "--data", str(data), "--out", str(out), "--dims", "16"])
    report = json.load(open(out / "decider_report.json"))
    assert list(report["per_dim"]) == ["16"] and report["matrices"] == len(names)
    train_decider.main(["fit", "--data", str(data), "--out", str(out), "--dims", "32"])
    report = json.load(open(out / "decider_report.json"))
    assert list(report["per_dim"]) == ["16", "32"]
    assert report["per_dim"]["16"]["classes"] == len(sweep.column_names(16))

    labels = pd.read_csv(data / "dim32_OP_SpMM_native.csv")
    assert list(labels.columns) == ["mtx_name"] + train_decider.FEATURES + ["OP_SpMM"]
    want = np.where(feats.iloc[:, 0] > 0.5, 1, len(sweep.column_names(32)) - 2)
    assert (labels["OP_SpMM"].to_numpy() == want).all()

    # the same table fitted on the reference's class space: the widened table's columns of the reference's CF list,
    # renumbered in the reference's order (blkWarpNum-major); plain pickles without a recorded CF axis
    ref_out = tmp_path / "models_ref"
    train_decider.main(["fit", "--data", str(data), "--out", str(ref_out), "--space", "reference", "--dims", "32"])
    ref_cols = train_decider.reference_space_columns(32, decider_CF_list(32))
    assert [sweep.column_names(32)[c] for c in ref_cols] == sweep.column_names(32, [1])
    labels = pd.read_csv(data / "dim32_OP_SpMM.csv")
    tp32 = pd.read_csv(data / "dim32.csv").to_numpy()
    assert (labels["OP_SpMM"].to_numpy() == tp32[:, ref_cols].argmax(axis=1)).all() and labels["OP_SpMM"].max() < 8
    import pickle

    forest = pickle.load(open(ref_out / "rnd_tree_32.pkl", "rb"))
    assert not hasattr(forest, "psp_cf_list_") and set(forest.classes_) <= set(range(8))
    rep = json.load(open(ref_out / "decider_report.json"))["per_dim"]["32"]
    assert rep["classes"] == 8 and "against_best_of_all_swept_columns" in rep

    dec = SpMMDecider(str(out) + os.sep)
    dec.gen_model_dict([16, 32])

    class G:  # what config_PCSR reads of a graph_input
        def __init__(self, row):
            self.row = row

        def get_info(self):
            return np.asarray(self.row, dtype=np.float64).reshape(1, -1)

    for d in (16, 32):
        hits = 0
        for i in range(len(names)):
            if_split, vec, cf, bw = dec.config_PCSR(G(feats.iloc[i].to_numpy()), d)
            assert cf in decider_CF_list(d) and bw in (4, 8) and vec in (1, 2)
            _capi.spmm_plan(d, cf, bw)  # every decoded configuration has a plan
            col = [c for c in range(len(sweep.column_names(d))) if sweep.decode_column(d, c) == (if_split, vec, cf, bw)][0]
            hits += col == (1 if feats.iloc[i, 0] > 0.5 else len(sweep.column_names(d)) - 2)
        assert hits >= 0.9 * len(names)  # refitted on every matrix: the rule is learnt


def test_decider_candidates_start_with_the_pick_and_are_distinct(tmp_path):
    """candidates_PCSR: the forest's k most probable classes, decoded; the first is config_PCSR's answer."""
    import pickle

    from sklearn.ensemble import RandomForestClassifier

    from paramspmm_ae_amd.decider import SpMMDecider
    from paramspmm_ae_amd.PCSR import decider_CF_list

    rng = np.random.default_rng(11)
    dim = 64
    n_classes = 4 * len(decider_CF_list(dim)) * 2
    Xf = rng.random((300, 15))
    y = (Xf[:, 0] * 3).astype(int) * 5 + (Xf[:, 1] > 0.5)  # six classes out of the table's n_classes
    assert y.max() < n_classes
    forest = RandomForestClassifier(n_estimators=20, max_leaf_nodes=8, random_state=0).fit(Xf, y)
    forest.psp_cf_list_ = [int(c) for c in decider_CF_list(dim)]
    with open(tmp_path / "rnd_tree_64.pkl", "wb") as f:
        pickle.dump(forest, f)
    dec = SpMMDecider(str(tmp_path) + os.sep)
    dec.gen_model_dict([dim])

    class G:
        def __init__(self, row):
            self.row = row

        def get_info(self):
            return self.row.reshape(1, -1)

    for i in range(20):
        g = G(Xf[i])
        cands = dec.candidates_PCSR(g, dim, 3)
        assert 1 <= len(cands) <= 3 and len(set(cands)) == len(cands)
        assert cands[0] == dec.config_PCSR(g, dim)
        assert dec.candidates_PCSR(g, dim, 1) == cands[:1]
        codes = set(forest.classes_)
        for c in cands:  # every candidate is a class the forest knows
            assert any(dec.decode_tree(code, dim, CF_list=decider_CF_list(dim)) == c for code in codes)
