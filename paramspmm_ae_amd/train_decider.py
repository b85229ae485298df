#!/usr/bin/env python3
"""Retrains the SpMM-decider on MI355X timings of synthetic matrices.

Counterpart of the reference's training-set construction (PCSR.py:672-823, script/1_construct_training_set.sh)
and of its training notebook (models/rnd_tree.ipynb cells 3-21), with synthetic matrices instead of the
SuiteSparse / OGB collection the reference downloads.

  sweep  (GPU)  for every matrix of the corpus: build the PCSR formats, record the 15 decider features and time
                every <representation, CF, blkWarpNum> at every width 16..256 -> csv files with the reference's
                schema: mtx_info.csv, dim<N>.csv (GFLOP/s per column), dim<N>_OP_SpMM.csv (features + arg-max
                column = class code).
  window (GPU)  the windowed layout (an addition of this build) timed over the same corpus -> window.csv; ``fit`` reports
                from it where that layout beats the best swept column.
  fit    (CPU)  one RandomForestClassifier per width -> rnd_tree_<N>.pkl, and a 5-fold cross-validated report with
                the reference's two statistics (accuracy, mean normalised performance) plus the share of
                matrices whose pick is within 10 % of the best swept configuration.

    python -m paramspmm_ae_amd.train_decider sweep --out ParamSpMM-log/decider [--part 0/3]
    python -m paramspmm_ae_amd.train_decider fit --space reference    # -> models/rnd_tree_<N>.pkl
    python -m paramspmm_ae_amd.train_decider fit --space native       # -> models/native/rnd_tree_<N>.pkl

Two sets of forests come out of the same sweep tables.  ``--space reference`` keeps the columns of the reference's own
class space -- 4 representations x ``dynamic_CF_prompter(dim)`` x blkWarpNum {4, 8}, class code = the reference's
column index (PCSR.py:781-788, 815-818) -- and writes plain pickles, so that the reference's unchanged decider.py
(``pickle.load(open(...))`` at decider.py:38, ``decode_tree`` at 63-80) loads and decodes them.  ``--space native``
trains on every swept column (the reference's list followed by the wave64 configurations); those forests record
their CF axis in ``psp_cf_list_`` and are what this package's ``SpMMDecider`` reads by default.
"""
import argparse
import json
import os
import pickle
import sys
import time

import numpy as np

DIMS = list(range(16, 257, 16))
FEATURES = [
    "graph_nodes", "graph_edges", "graph_density", "csr_max_row_nnz", "csr_real_nrow", "csr_nonempty_rate",
    "csr_avg_degree", "csr_COV", "csr_real_avg_degree", "csr_real_COV", "csr_max_bw", "csr_avg_bw",
    "csr_split_ratio", "bcsr_split_ratio", "pack_rate",
]
NNZ_CAP = 24_000_000


# ------------------------------------------------------------------------------------------------------------
# corpus
# ------------------------------------------------------------------------------------------------------------
def banded(n, k, width, seed):
    """k random neighbours per node inside a band of +-width around the diagonal."""
    rng = np.random.default_rng(seed)
    u = np.repeat(np.arange(n, dtype=np.int64), k)
    v = u + rng.integers(-width, width + 1, u.size)
    np.clip(v, 0, n - 1, out=v)
    return u, v, n


def grid_with_holes(nx, ny, drop, seed):
    """2-D 5-point grid with a fraction of the edges removed (road-network like: degree 2-4, high diameter)."""
    from . import synth

    r, c, n = synth.stencil2d(nx, ny)
    keep = np.random.default_rng(seed).random(r.size) >= drop
    return r[keep], c[keep], n


def corpus(replicas=2):
    """Deterministic list of (name, builder) covering power-law, R-MAT, community, mesh and banded structure.
    Every replica walks the same parameter grid with its own random choices (which grid points are skipped, hub
    degree, ordering, seeds); deterministic structures (plain stencils) appear once."""
    items = []
    for rep in range(replicas):
        _corpus_replica(items, rep)
    return items


def _corpus_replica(items, rep):
    from . import synth

    rng = np.random.default_rng(2024 + rep)
    suffix = "" if rep == 0 else "_r%d" % rep

    def add(name, fn):
        items.append((name + suffix, fn))

    # Chung-Lu power law
    for n in (10_000, 20_000, 60_000, 200_000, 600_000, 1_500_000):
        for avg in (3, 6, 12, 25, 50):
            if n * avg > NNZ_CAP:
                continue
            for expo in (1.8, 2.1, 2.4, 3.0):
                if rng.random() < 0.2:
                    continue
                maxd = int(min(n // 4, rng.choice([200, 2000, 20000])))
                perm = bool(rng.random() < 0.7)
                seed = int(rng.integers(1 << 30))
                add("cl_n%d_d%d_e%.1f_m%d_%s" % (n, avg, expo, maxd, "p" if perm else "s"),
                    lambda n=n, avg=avg, expo=expo, maxd=maxd, perm=perm, seed=seed:
                    synth.chung_lu(n, n * avg // 2, exponent=expo, max_degree=maxd, seed=seed, permute=perm))
    # R-MAT, from Graph500-like skew to Erdos-Renyi
    for scale in (13, 15, 16, 17, 18, 19, 20):
        for ef in (2, 4, 8, 16, 32):
            if (1 << scale) * ef * 2 > NNZ_CAP:
                continue
            for abc in ((0.57, 0.19, 0.19), (0.5, 0.2, 0.2), (0.45, 0.22, 0.22), (0.35, 0.25, 0.25), (0.25, 0.25, 0.25)):
                if rng.random() < 0.1:
                    continue
                seed = int(rng.integers(1 << 30))
                add("rmat_s%d_e%d_a%.2f" % (scale, ef, abc[0]),
                    lambda scale=scale, ef=ef, abc=abc, seed=seed: synth.rmat(scale, ef << scale, *abc, seed=seed))
    # stochastic block models, community-ordered and permuted
    for n in (20_000, 50_000, 200_000, 500_000, 1_000_000):
        for size in (20, 50, 100, 500, 2000):
            for din, dout in ((5, 0.5), (20, 2), (40, 8), (10, 10), (3, 3)):
                if n * (din + dout) > NNZ_CAP or rng.random() < 0.55:
                    continue
                for perm in (False, True):
                    seed = int(rng.integers(1 << 30))
                    add("sbm_n%d_c%d_i%g_o%g_%s" % (n, size, din, dout, "p" if perm else "s"),
                        lambda n=n, size=size, din=din, dout=dout, perm=perm, seed=seed:
                        synth.sbm(n, n // size, din, dout, seed=seed, permute=perm))
    # meshes
    stencils = ((128, 128), (256, 256), (512, 512), (1024, 1024), (2048, 1024), (2048, 2048), (4096, 1024), (8192, 256),
                (100, 100), (300, 700), (1000, 500), (3000, 1000), (64, 4096), (1536, 1536))
    if rep > 0:  # other aspect ratios and sizes
        stencils = tuple((int(rng.integers(60, 3000)), int(rng.integers(60, 3000))) for _ in range(len(stencils)))
    for nx, ny in stencils:
        add("stencil_%dx%d" % (nx, ny), lambda nx=nx, ny=ny: synth.stencil2d(nx, ny))
    for nx, ny, drop in ((512, 512, 0.3), (1024, 1024, 0.25), (2048, 1024, 0.4), (1500, 1500, 0.1), (256, 256, 0.2),
                         (2048, 2048, 0.3), (700, 900, 0.5), (400, 4000, 0.15)):
        seed = int(rng.integers(1 << 30))
        add("grid_%dx%d_h%.2f" % (nx, ny, drop), lambda nx=nx, ny=ny, drop=drop, seed=seed: grid_with_holes(nx, ny, drop, seed))
    # banded random
    for n in (15_000, 30_000, 150_000, 700_000, 2_000_000):
        for k, w in ((2, 8), (6, 64), (16, 512), (30, 4096), (4, 20000), (10, 100)):
            if n * k * 2 > NNZ_CAP or rng.random() < 0.2:
                continue
            seed = int(rng.integers(1 << 30))
            add("band_n%d_k%d_w%d" % (n, k, w), lambda n=n, k=k, w=w, seed=seed: banded(n, k, w, seed))


# ------------------------------------------------------------------------------------------------------------
# sweep (GPU)
# ------------------------------------------------------------------------------------------------------------
def sweep_main(args):
    import pandas as pd
    import torch

    from . import sweep as sw
    from . import synth
    from .graph_input import graph_input

    assert torch.cuda.is_available(), "the sweep needs the GPU"
    items = corpus()
    part, nparts = (int(x) for x in args.part.split("/"))
    items = [it for i, it in enumerate(items) if i % nparts == part]
    if args.limit:
        items = items[: args.limit]
    os.makedirs(args.out, exist_ok=True)
    tag = "" if nparts == 1 else "_part%d" % part
    info_rows, names = [], []
    dims = [int(d) for d in args.dims.split(",")] if args.dims else DIMS
    flush_bytes = int(args.flush_mb) << 20
    tp = {d: [] for d in dims}
    t_start = time.time()
    for idx, (name, build) in enumerate(items):
        t0 = time.time()
        r, c, n = build()
        rowPtr, colIdx, val = synth.to_gcn_csr(r, c, n)
        g = graph_input(name, "")
        g.verbose = False
        g.load_from_csr(rowPtr, colIdx, val)
        ops = sw.operators_of(g)
        nnz = g.mtx_edges
        rows = (n + 1) // 2 * 2
        # every representation must give the same product before it is timed
        X = torch.randn(rows, 32, device="cuda")
        if rows != n:
            X[n:] = 0
        ref = ops[0]._spmm(X)[:n]
        scale = ref.abs().max().item() + 1e-6
        for op in ops[1:]:
            err = (op._spmm(X)[:n] - ref).abs().max().item()
            assert err <= 1e-4 * scale, (name, err, scale)
        del X, ref
        for d in dims:
            ms, gf = sw.sweep_dim(ops, d, nnz, n, warmup=args.warmup, iters=args.iters, flush_bytes=flush_bytes)
            tp[d].append(gf)
        info_rows.append([name] + g._feature_values())
        names.append(name)
        del ops, g
        torch.cuda.empty_cache()
        print("[%d/%d] %-34s n=%-8d nnz=%-9d %.1fs (total %.0fs)" % (idx + 1, len(items), name, n, nnz, time.time() - t0,
                                                                   time.time() - t_start), flush=True)
        # keep what is done on disk: a run that is cut short still leaves usable csv files
        info = pd.DataFrame(info_rows, columns=["mtx_name"] + FEATURES)
        info.to_csv(os.path.join(args.out, "mtx_info%s.csv" % tag), index=False)
        if (idx + 1) % 10 == 0 or idx + 1 == len(items):
            for d in dims:
                pd.DataFrame(np.array(tp[d]), columns=sw.column_names(d)).to_csv(
                    os.path.join(args.out, "dim%d%s.csv" % (d, tag)), index=False)


def window_main(args):
    """The windowed layout over the same corpus (GPU): per matrix its local share and, per width, the GFLOP/s of
    the windowed SpMM and of plain CSR with CF 1 / blkWarpNum 4 timed in the same run (the column vec1_TP_14 of the
    sweep tables, so that the two runs can be set side by side) -> window<tag>.csv.  The forests' class space is the
    reference's and has no windowed class; ``fit`` reports from this table where the layout beats the best swept
    column, which is what GNN.configure_operators decides by timing on the matrix itself."""
    import pandas as pd
    import torch

    from . import synth
    from .graph_input import graph_input
    from .PCSR import pcsr_spmm

    assert torch.cuda.is_available(), "the sweep needs the GPU"
    items = corpus()
    part, nparts = (int(x) for x in args.part.split("/"))
    items = [it for i, it in enumerate(items) if i % nparts == part]
    if args.limit:
        items = items[: args.limit]
    os.makedirs(args.out, exist_ok=True)
    tag = "" if nparts == 1 else "_part%d" % part
    dims = [int(d) for d in args.dims.split(",")] if args.dims else DIMS
    flush_bytes = int(args.flush_mb) << 20
    rows_out, t_start = [], time.time()
    for idx, (name, build) in enumerate(items):
        r, c, n = build()
        rowPtr, colIdx, val = synth.to_gcn_csr(r, c, n)
        g = graph_input(name, "")
        g.verbose = False
        g.load_from_csr(rowPtr, colIdx, val)
        nnz = g.mtx_edges
        win = pcsr_spmm(g, vec_size=1, if_split=False, CF=0, window=True)
        csr = pcsr_spmm(g, vec_size=1, if_split=False, CF=1, blkWarpNum=4)
        row = {"mtx_name": name, "local_share": win.window_local_share}
        X32 = torch.randn(n, 32, device="cuda")
        err = (win._spmm(X32) - csr._spmm(X32)).abs().max().item()
        assert err <= 1e-4 * (csr._spmm(X32).abs().max().item() + 1e-6), (name, err)
        for d in dims:
            X = torch.ones(n, d, device="cuda")
            fb = flush_bytes if d <= 128 else 0  # as the sweep behind the forests was timed
            row["window_TP_%d" % d] = 2.0 * nnz * d / 1e6 / win.time_ms(X, warmup=args.warmup, iters=args.iters, flush_bytes=fb)
            row["vec1_TP_14_%d" % d] = 2.0 * nnz * d / 1e6 / csr.time_ms(X, warmup=args.warmup, iters=args.iters, flush_bytes=fb)
        rows_out.append(row)
        del win, csr, g
        torch.cuda.empty_cache()
        print("[%d/%d] %-34s n=%-8d nnz=%-9d local %.3f (total %.0fs)" % (idx + 1, len(items), name, n, nnz, row["local_share"],
                                                                       time.time() - t_start), flush=True)
        if (idx + 1) % 10 == 0 or idx + 1 == len(items):
            pd.DataFrame(rows_out).to_csv(os.path.join(args.out, "window%s.csv" % tag), index=False)


def window_report(data_dir, info, tps, dims):
    """What the windowed layout is worth against the best swept column, from window*.csv beside the sweep tables (None
    without them).  The two tables come from different runs: the windowed figure is scaled by the ratio of the
    plain-CSR column both runs timed."""
    import glob

    import pandas as pd

    files = sorted(glob.glob(os.path.join(data_dir, "window*.csv")))
    if not files:
        return None
    win = pd.concat([pd.read_csv(f) for f in files], ignore_index=True).drop_duplicates("mtx_name").set_index("mtx_name")
    names = [n for n in info["mtx_name"] if n in win.index]
    sel = np.array([n in win.index for n in info["mtx_name"]])
    share = win.loc[names, "local_share"].to_numpy()
    from .GNN import WINDOW_MIN_LOCAL_SHARE as thr

    out = {"matrices": int(len(names)), "rule": "tried when the local share is at least %.2f, kept when faster (GNN.configure_operators)" % thr,
           "matrices_with_that_local_share": int(np.sum(share >= thr)), "per_dim": {}}
    fams = np.array([family(n).split("_")[0] + ("_ordered" if n.startswith("sbm_") and n.split("_r")[0].endswith("_s") else
                                                 "_permuted" if n.startswith("sbm_") else "") for n in names])
    for d in dims:
        TP = tps[d].to_numpy(dtype=np.float64)[sel]
        cols = list(tps[d].columns)
        same = TP[:, cols.index("vec1_TP_14")] / win.loc[names, "vec1_TP_14_%d" % d].to_numpy()  # run-to-run scale
        w = win.loc[names, "window_TP_%d" % d].to_numpy() * same
        gain = w / TP.max(axis=1)
        wins = gain > 1.0
        ent = {"share_of_matrices_where_windowed_beats_the_best_swept_column": float(wins.mean()),
               "mean_gain_where_it_wins": float(gain[wins].mean()) if wins.any() else None,
               "best_gain": float(gain.max()),
               "of_those_share_the_rule_tries": float(np.mean(share[wins] >= thr)) if wins.any() else None,
               "share_of_tried_matrices_where_it_wins": float(np.mean(wins[share >= thr])) if (share >= thr).any() else None,
               "mean_gain_over_tried_matrices": float(gain[share >= thr].mean()) if (share >= thr).any() else None,
               "mean_gain_by_family": {f: float(gain[fams == f].mean()) for f in sorted(set(fams))}}
        out["per_dim"][str(d)] = ent
    return out


# ------------------------------------------------------------------------------------------------------------
# fit (CPU)
# ------------------------------------------------------------------------------------------------------------
def load_training_data(data_dir, dims=None):
    import glob

    import pandas as pd

    info_files = sorted(glob.glob(os.path.join(data_dir, "mtx_info*.csv")))
    assert info_files, "no mtx_info*.csv under " + data_dir
    dims = DIMS if dims is None else dims
    infos, tps = [], {d: [] for d in dims}
    for f in info_files:
        tag = os.path.basename(f)[len("mtx_info"):-len(".csv")]
        info = pd.read_csv(f)
        per_dim = {d: pd.read_csv(os.path.join(data_dir, "dim%d%s.csv" % (d, tag))) for d in dims}
        rows = min([len(info)] + [len(v) for v in per_dim.values()])
        infos.append(info.iloc[:rows])
        for d in dims:
            tps[d].append(per_dim[d].iloc[:rows])
    info = pd.concat(infos, ignore_index=True)
    return info, {d: pd.concat(tps[d], ignore_index=True) for d in dims}


def _fit_forest(X, TP, near, n_est, leaves):
    """Forest on 'near-best' labels: a matrix contributes one sample for every configuration whose throughput is at
    least ``near`` times its best one, the samples of a matrix sharing a total weight of 1.  near = 1 is the
    reference's arg-max label (PCSR.py:815-818); a threshold below 1 keeps timing noise between configurations
    that are equally good from turning into label noise."""
    from sklearn.ensemble import RandomForestClassifier

    ok = TP >= near * TP.max(axis=1, keepdims=True)
    rows, cols = np.nonzero(ok)
    weight = 1.0 / ok.sum(axis=1)[rows]
    # bounded trees: an unbounded forest on these labels is 10-15 MB per width and no better in validation
    clf = RandomForestClassifier(n_estimators=n_est, max_leaf_nodes=leaves, n_jobs=-1, random_state=17)
    clf.fit(X[rows], cols, sample_weight=weight)
    return clf


def family(name):
    """Matrices that differ only in seed, hub degree or ordering share a family; cross-validation keeps a family in
    one fold, so a forest is never validated on a sibling of a matrix it was trained on."""
    import re

    name = re.sub(r"_r\d+$", "", name)
    if name.startswith("cl_"):
        name = re.sub(r"_m\d+_[ps]$", "", name)
    elif name.startswith("sbm_"):
        name = re.sub(r"_[ps]$", "", name)
    return name


def reference_space_columns(dim, cf_axis):
    """Positions, inside a sweep table whose CF axis is ``cf_axis``, of the reference's columns for ``dim`` in the
    reference's own order (blkWarpNum-major, then ``dynamic_CF_prompter(dim)``, then the four representations):
    entry k of the result is the table column of reference class code k."""
    from .PCSR import dynamic_CF_prompter

    legacy = dynamic_CF_prompter(dim)
    assert list(cf_axis[:len(legacy)]) == list(legacy), "the table's CF axis must start with the reference's list"
    return np.array([(w * len(cf_axis) + c) * 4 + r for w in range(2) for c in range(len(legacy)) for r in range(4)])


def fit_main(args):
    import pandas as pd
    from sklearn.model_selection import GroupKFold

    from . import sweep as sw
    from .PCSR import decider_CF_list, dynamic_CF_prompter

    dims = [int(d) for d in args.dims.split(",")] if args.dims else DIMS
    reference_space = args.space == "reference"
    here = os.path.dirname(os.path.abspath(__file__))
    out = args.out or os.path.join(here, "models", "" if reference_space else "native")
    info, tps = load_training_data(args.data, dims)
    X = info[FEATURES].to_numpy(dtype=np.float64)
    os.makedirs(out, exist_ok=True)
    groups = np.array([family(n) for n in info["mtx_name"]])
    report = {"class_space": "reference: 4 representations x dynamic_CF_prompter(dim) x blkWarpNum {4, 8}, the class "
              "code of decider.py:63-80" if reference_space else
              "native: 4 representations x decider_CF_list(dim) (the reference's CF list followed by the wave64 "
              "configurations) x blkWarpNum {4, 8}; the forests carry the list as psp_cf_list_",
              "matrices": int(len(info)), "families": int(len(set(groups))),
              "validation": "5-fold cross-validation grouped by matrix family (same generator parameters, different "
              "seed / hub degree / ordering): every matrix is predicted by a forest that has seen neither it nor "
              "its siblings", "per_dim": {}}
    folds = list(GroupKFold(5).split(X, groups=groups))

    report_path = os.path.join(out, "decider_report.json")
    if args.dims and os.path.exists(report_path):  # a partial refit keeps the other widths' entries
        with open(report_path) as f:
            report["per_dim"] = {int(k): v for k, v in json.load(f)["per_dim"].items()}
    for d in dims:
        # the table's CF axis: the widened list, or the reference's own when the data come from its sweep
        if list(tps[d].columns) == sw.column_names(d):
            table_cfs = decider_CF_list(d)
        else:
            assert list(tps[d].columns) == sw.column_names(d, dynamic_CF_prompter(d)), "unknown column set at dim %d" % d
            table_cfs = dynamic_CF_prompter(d)
        TP_all = tps[d].to_numpy(dtype=np.float64)
        legacy_pos = reference_space_columns(d, table_cfs)
        if reference_space:
            TP, cf_list = TP_all[:, legacy_pos], dynamic_CF_prompter(d)
        else:
            TP, cf_list = TP_all, table_cfs
        y = TP.argmax(axis=1)  # class code = column index (PCSR.py:815-818)
        # label csv in the reference's schema
        lab = pd.concat([info, pd.DataFrame({"OP_SpMM": y})], axis=1)
        lab.to_csv(os.path.join(args.data, "dim%d_OP_SpMM%s.csv" % (d, "" if reference_space else "_native")), index=False)
        tried = []
        for n_est, leaves in ((30, 64), (30, 128), (50, 128)):  # the notebook's forest sizes are 30 / 50 / 80
            for near in (1.0, 0.97, 0.95):
                pick = np.zeros(len(X), dtype=np.int64)
                for tr, te in folds:
                    pick[te] = _fit_forest(X[tr], TP[tr], near, n_est, leaves).predict(X[te]).astype(np.int64)
                norm = TP[np.arange(len(X)), pick] / TP.max(axis=1)  # normalised performance of the pick
                score = (float(np.mean(norm >= 1 / 1.10)), float(norm.mean()))
                tried.append((score, near, n_est, leaves, pick, norm))
        best = max(tried, key=lambda t: t[0])  # the first of equals: the smaller forest
        (within10, mean_norm), near, n_est, leaves, pick, norm = best
        best_all, best_legacy = TP_all.max(axis=1), TP_all[:, legacy_pos].max(axis=1)
        gain = best_all / best_legacy  # what the native configurations add over the reference's <CF, blkWarpNum> space
        by_family = {}
        for fam in ("cl_", "rmat_", "sbm_", "stencil_", "grid_", "band_"):
            sel = np.array([n.startswith(fam) for n in info["mtx_name"]])
            if fam == "sbm_":
                for tag, m in (("sbm_ordered", np.array([n.split("_r")[0].endswith("_s") for n in info["mtx_name"]])),
                               ("sbm_permuted", np.array([n.split("_r")[0].endswith("_p") for n in info["mtx_name"]]))):
                    if (sel & m).any():
                        by_family[tag] = float(gain[sel & m].mean())
            elif sel.any():
                by_family[fam.rstrip("_")] = float(gain[sel].mean())
        entry = {
            "cf_axis": [sw.cf_label(c) for c in cf_list],
            "native_gain_over_reference_space": {"mean": float(gain.mean()), "max": float(gain.max()),
                                                 "share_of_matrices_with_gain_over_5pct": float(np.mean(gain > 1.05)),
                                                 "mean_by_family": by_family},
            "near_best_threshold": near, "n_estimators": n_est, "max_leaf_nodes": leaves, "classes": int(TP.shape[1]),
            "validated_matrices": int(len(X)), "accuracy": float(np.mean(pick == y)),
            "mean_normalised_performance": mean_norm, "share_within_10pct_of_best": within10,
            "worst_normalised_performance": float(norm.min()),
        }
        if reference_space:
            # the same picks measured against the best of every swept column, native ones included: what a caller of
            # the reference's decider.py gives up against this package's own decider
            norm_all = TP[np.arange(len(X)), pick] / best_all
            entry["against_best_of_all_swept_columns"] = {
                "mean_normalised_performance": float(norm_all.mean()),
                "share_within_10pct_of_best": float(np.mean(norm_all >= 1 / 1.10)),
            }
        else:
            legacy_cols = np.zeros(TP.shape[1], dtype=bool)
            legacy_cols[legacy_pos] = True
            entry["share_of_picks_that_are_native"] = float(np.mean(~legacy_cols[pick]))
        report["per_dim"][d] = entry
        # the shipped model is refitted on every matrix
        final = _fit_forest(X, TP, near, n_est, leaves)
        final.n_jobs = 1
        path = os.path.join(out, "rnd_tree_%d.pkl" % d)
        if not reference_space:
            final.psp_cf_list_ = [int(c) for c in cf_list]  # the CF axis of the class codes (decider.config_PCSR)
        if reference_space:
            # plain pickles: decider.py:38 reads them with pickle.load(open(path, "rb"))
            with open(path, "wb") as f:
                pickle.dump(final, f, protocol=4)
        else:
            # read by this package's SpMMDecider only, which accepts a gzip stream (the per-node class histograms of
            # 32-72 classes are mostly zeros: a fifth of the plain size)
            import gzip

            with gzip.GzipFile(path, "wb", compresslevel=6, mtime=0) as f:
                pickle.dump(final, f, protocol=4)
        print("dim %3d: %2d classes  near %.2f  n_estimators %d  leaves %d  acc %.3f  mean norm perf %.4f  within 10%%: %.3f  worst %.3f" % (
            d, TP.shape[1], near, n_est, leaves, entry["accuracy"], mean_norm, within10, norm.min()), flush=True)
    allw = [v["share_within_10pct_of_best"] for v in report["per_dim"].values()]
    report["share_within_10pct_mean"] = float(np.mean(allw))
    report["share_within_10pct_min"] = float(np.min(allw))
    report["per_dim"] = {str(k): report["per_dim"][k] for k in sorted(report["per_dim"], key=int)}
    wr = window_report(args.data, info, tps, [int(k) for k in report["per_dim"] if int(k) in tps])
    if wr is not None:
        report["windowed_layout"] = wr
    import sklearn

    report["scikit_learn"] = sklearn.__version__  # a pickled forest loads under the version that wrote it (or newer)
    with open(report_path, "w") as f:
        json.dump(report, f, indent=1)
    print("matrices %d; within 10%% of best: mean %.3f, min over widths %.3f" % (len(info), np.mean(allw), np.min(allw)))


def main(argv=None):
    ap = argparse.ArgumentParser()
    sub = ap.add_subparsers(dest="cmd", required=True)
    s = sub.add_parser("sweep")
    s.add_argument("--out", default="ParamSpMM-log/decider")
    s.add_argument("--part", default="0/1", help="i/n: every n-th matrix starting at i")
    s.add_argument("--limit", type=int, default=0)
    s.add_argument("--warmup", type=int, default=2)
    s.add_argument("--iters", type=int, default=6)
    s.add_argument("--dims", default="", help="comma-separated widths (default: all of 16..256)")
    s.add_argument("--flush_mb", type=int, default=0,
                   help="fill this many MiB of scratch memory before every timed launch (operands from HBM, as inside a "
                        "training step) instead of repeating the launch back to back")
    f = sub.add_parser("fit")
    here = os.path.dirname(os.path.abspath(__file__))
    f.add_argument("--data", default=os.path.join(here, "models", "train_data"))
    f.add_argument("--space", choices=("reference", "native"), default="native",
                   help="class space of the forests: the reference's own (loadable and decodable by its unchanged "
                        "decider.py) or every swept column")
    f.add_argument("--out", default="", help="default: models/ for --space reference, models/native/ for --space native")
    f.add_argument("--dims", default="", help="refit these widths only (comma-separated); the report keeps the others")
    w = sub.add_parser("window")
    w.add_argument("--out", default=os.path.join(here, "models", "train_data"))
    w.add_argument("--part", default="0/1", help="i/n: every n-th matrix starting at i")
    w.add_argument("--limit", type=int, default=0)
    w.add_argument("--warmup", type=int, default=2)
    w.add_argument("--iters", type=int, default=6)
    w.add_argument("--dims", default="")
    w.add_argument("--flush_mb", type=int, default=512)
    ls = sub.add_parser("list")
    args = ap.parse_args(argv)
    if args.cmd == "sweep":
        sweep_main(args)
    elif args.cmd == "fit":
        fit_main(args)
    elif args.cmd == "window":
        window_main(args)
    else:
        for name, _ in corpus():
            print(name)


if __name__ == "__main__":
    main()
