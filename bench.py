#!/usr/bin/env python3
"""Headline benchmark: ParamSpMM feature-width sweep on one MI355X.

Workload (BASELINE.json configs[1]): R-MAT graph with 2^20 nodes, about 16 off-diagonal entries per row,
self loops, values D^-1/2 (A+I) D^-1/2 in fp32, CSR int32; X = N(0,1) [2^20, N] for N = 16, 32, ..., 256.
One step = one SpMM at every one of the 16 widths, each in the configuration chosen for it (best of a short
sweep over the PCSR configurations, or the trained decider's pick with --pick decider).  Inputs are resident
in HBM before the timed region.  value = sum(2*nnz*N) * steps / wall time, in GFLOP/s.

The JSON line also carries
  roofline         for the kernel symbol that takes the most time: algorithmic bytes
                   4(M+1) + 8 nnz + 4 n N + 4 M N (CSR; split adds 8 S + 4, blocks use 4(Mb+1) + 12 nblk)
                   divided by that launch's mean duration (HIP events on the launching stream), against 8 TB/s;
                   gather_ceiling_frac = duration of the bare gathers of the same pattern and width
                   (psp_probe_gather_f32: same colIdx stream, same X row tiles, no rows, no FMAs) / kernel duration;
  sweep            the same numbers for every width;
  decider_vs_best  t(decider's pick) / t(best swept configuration) per width, from a short sweep of every
                   <representation, CF, blkWarpNum> after the timed region (PCSR.py:754-788, rnd_tree.ipynb cell 4);
  sddmm            one SDDMM width (K = 64) on the same pattern with its own roofline;
  other_graphs     the other graphs of the benchmark set in the decider's configuration: 5-point stencil 2048^2 at
                   N = 64 / 128, block model (community order and random order) at N = 128, Chung-Lu 2.45M at N = 128;
  gcn_epoch_ms     GCN / GIN / AGNN training epochs (5 layers, hidden 16 / 32 / 128, 16 classes) on the 1M-node block model,
                   1 warm-up + 200 timed epochs as in GNN.py:126-151;
  cpu_baseline     torch.sparse.mm on the host cores (the product the reference verifies against, verification.py:18-46)
                   on a bounded sample of the widths; cpu_scalar_port is the oracle's one-thread C restatement, which also
                   checks the GPU result at those widths.
"""
import argparse
import contextlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
DEFAULT_DIMS = ",".join(str(d) for d in range(16, 257, 16))


def algorithmic_bytes(fmt, F, n_x_rows, N):
    """Bytes one SpMM has to move at least once: index arrays + values + X once + Y once."""
    if fmt in ("csr", "csr_split"):
        M = F["n"]
        b = 4 * (M + 1) + 8 * F["nnz"]
        if fmt == "csr_split":
            b = 4 * (F["S"] + 1) + 4 * F["S"] + 8 * F["nnz"]
        return b + 4 * n_x_rows * N + 4 * M * N
    Mb = F["Mb"]
    b = 4 * (Mb + 1) + 12 * F["nblk"]
    if fmt == "bcsr_split":
        b = 4 * (F["Sb"] + 1) + 4 * F["Sb"] + 12 * F["nblk"]
    return b + 4 * n_x_rows * N + 4 * 2 * Mb * N


def measured_traffic(graph, rows_of):
    """HBM bytes per launch of the dominant kernel, from the committed rocprofv3 counter summary
    (profiles/psp_spmm_kernel_<graph>_pmc.md: FETCH_SIZE x2 + WRITE_SIZE, both in KiB, per width).  None when the
    summary has no line for one of the widths / configurations that ran."""
    path = os.path.join(ROOT, "profiles", "psp_spmm_kernel_%s_pmc.md" % graph)
    if not os.path.exists(path):
        return None
    table = {}
    for line in open(path):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) >= 7 and cells[0].isdigit():
            # | dim | format | CF | blkWarpNum | FETCH_SIZE KiB | WRITE_SIZE KiB | HBM bytes |
            table[(int(cells[0]), cells[1], int(cells[2]), int(cells[3]))] = int(cells[6])
    total = 0
    for r in rows_of:
        key = (r["dim"], r["format"], r["CF"], r["blkWarpNum"])
        if key not in table:
            return None
        total += table[key]
    return int(total / len(rows_of))


def measured_sddmm_traffic(graph, K, fmt, bw):
    """HBM bytes of one SDDMM launch from the committed counter summary (profiles/psp_sddmm_kernel_<graph>_trace_and_pmc.md,
    table "fastest configuration per width": | K | layout | wavefronts | ... | HBM bytes | ...); None without a
    matching line."""
    path = os.path.join(ROOT, "profiles", "psp_sddmm_kernel_%s_trace_and_pmc.md" % graph)
    if not os.path.exists(path):
        return None
    header = None
    for line in open(path):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if cells and cells[0] == "K" and "HBM bytes" in cells:
            header = cells
        elif header and len(cells) == len(header) and cells[0].isdigit():
            row = dict(zip(header, cells))
            if int(row["K"]) == K and row["layout"] == fmt and int(row["wavefronts"]) == bw:
                return int(row["HBM bytes"])
    return None


def _event_ms(fn, warmup, iters):
    """Mean milliseconds per call of ``fn`` (HIP events on the current stream, which is the one the operators launch on)."""
    import torch

    for _ in range(warmup):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def other_graph_leg(name, dims, decider, reps=10, reorder=None):
    """One more graph of the benchmark set at a few widths, in the decider's configuration: per width the mean
    launch duration (HIP events on the launching stream), algorithmic bytes and their fraction of the HBM roofline,
    and the measured traffic of the committed counter summary for that graph when it has the configuration."""
    import torch
    from paramspmm_ae_amd import _capi, sweep, synth
    from paramspmm_ae_amd.graph_input import graph_input

    t0 = time.time()
    rowPtr, colIdx, val, n = synth.config_graph(name)
    graph = graph_input(mtx_name=name, path="")
    graph.verbose = False
    graph.load_from_csr(rowPtr, colIdx, val, reorder=reorder)  # reorder: rows and columns permuted together at load time
    nnz = graph.mtx_edges
    ops = sweep.operators_of(graph)
    fmt_names = ["csr", "csr_split", "bcsr", "bcsr_split"]
    F = {"n": n, "nnz": nnz, "S": graph.csr_data.target_row.numel(), "Mb": graph.bcsr_data.num_nodes,
         "nblk": graph.bcsr_data.colIdx.numel(), "Sb": graph.bcsr_data.target_row.numel()}
    rows = (n + 1) // 2 * 2
    gen = torch.Generator(device="cuda").manual_seed(99)
    res = []
    import ParamSpMM
    from paramspmm_ae_amd.GNN import WINDOW_MIN_LOCAL_SHARE
    from paramspmm_ae_amd.PCSR import pcsr_spmm

    win = pcsr_spmm(graph, vec_size=1, if_split=False, CF=0, window=True)
    if win.window_local_share < WINDOW_MIN_LOCAL_SHARE:
        win = None
    for d in dims:
        X = torch.randn(rows, d, device="cuda", generator=gen)
        if rows != n:
            X[n:].zero_()
        if_split, vec, cf, bw = (int(v) for v in decider.config_PCSR(graph, d))
        op = ops[(1 if if_split else 0) + (2 if vec == 2 else 0)]
        fmt = fmt_names[(1 if if_split else 0) + (2 if vec == 2 else 0)]
        ms = op.time_ms(X, CF=cf, blkWarpNum=bw, warmup=3, iters=reps)
        b_alg = algorithmic_bytes(fmt, F, n, d)
        row = {"dim": d, "format": fmt, "CF": cf, "config": sweep.cf_label(cf), "blkWarpNum": bw, "ms": round(float(ms), 5),
               "gflops": round(2.0 * nnz * d / ms / 1e6, 1), "alg_bytes": int(b_alg),
               "frac": round(b_alg / ms / 1e6 / HBM_PEAK_GBS, 4)}
        row["traffic"] = measured_traffic(name, [row]) if reorder is None else None
        if win is not None and d % 4 == 0:
            # the windowed layout beside it (what GNN.configure_operators would keep if it is faster): its algorithmic
            # bytes are those of the CSR product plus the second row pointer per row
            ms_w = win.time_ms(X, warmup=3, iters=reps)
            b_w = algorithmic_bytes("csr", F, n, d) + 4 * (n + 1)
            row["windowed"] = {"ms": round(float(ms_w), 5), "gflops": round(2.0 * nnz * d / ms_w / 1e6, 1),
                               "alg_bytes": int(b_w), "frac": round(b_w / ms_w / 1e6 / HBM_PEAK_GBS, 4),
                               "variant": int(ParamSpMM.window_plan(d, 0)["variant"]),
                               "traffic": measured_traffic(name, [{"dim": d, "format": "window", "CF": 0, "blkWarpNum": 0}])}
        res.append(row)
        del X
    out = {"nodes": n, "nnz": int(nnz), "setup_s": round(time.time() - t0, 1), "widths": res}
    if win is not None:
        out["window_local_share"] = round(win.window_local_share, 4)
        # the SDDMM <X_i, X_j> (the attention scores) on the same matrix: the CSR kernel and the windowed one.
        # Algorithmic bytes: row pointers, columns, the feature matrix once, one float per entry.
        out["sddmm"] = []
        csr = ops[0]
        for K in dims:
            if K % 4:
                continue
            X = torch.randn(rows, K, device="cuda", generator=gen)
            ms_c = _event_ms(lambda: csr.AGNN_sddmm(X), 3, reps)
            ms_w = _event_ms(lambda: win.AGNN_sddmm(X), 3, reps)
            b_alg = 4 * (n + 1) + 8 * nnz + 4 * n * K
            out["sddmm"].append({"K": K, "csr_ms": round(ms_c, 5), "windowed_ms": round(ms_w, 5),
                                 "alg_bytes": int(b_alg), "windowed_frac": round(b_alg / ms_w / 1e6 / HBM_PEAK_GBS, 4)})
            del X
    del ops, graph, win
    torch.cuda.empty_cache()
    return out


def gather_probe_ms(colIdx_dev, nnz, X, lanes, reps=5):
    """Best duration (ms) of the bare gathers of this pattern at X's width: psp_probe_gather_f32 over a few shapes."""
    import torch
    from paramspmm_ae_amd import _capi

    L, p = _capi.lib, _capi.ptr
    N = X.shape[1]
    stream = torch.cuda.current_stream().cuda_stream
    best = None
    for unroll in (4, 8):
        if unroll > lanes:
            continue
        for per_wave in (512, 2048):
            need = L.psp_probe_gather_out_floats(nnz, N, lanes, per_wave)
            out = torch.empty(need, device="cuda")
            call = lambda: L.psp_probe_gather_f32(p(colIdx_dev), nnz, p(X), N, lanes, unroll, per_wave, p(out), need, stream)
            _capi.check(call())
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                call()
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / reps
            if best is None or ms < best[0]:
                best = (ms, unroll, per_wave)
    return best


def bench_gather(args):
    """The gather ceiling next to the kernel: for each width the bare gathers of the pattern (no rows, no FMAs, one
    store per lane and wavefront) and the SpMM in the decider's configuration; GB/s of gathered bytes (nnz * N * 4)."""
    import torch

    from paramspmm_ae_amd import _capi, synth, sweep
    from paramspmm_ae_amd.decider import SpMMDecider
    from paramspmm_ae_amd.graph_input import graph_input

    dims = [int(d) for d in args.dims.split(",")] if args.dims != DEFAULT_DIMS else [16, 64, 128]
    rowPtr, colIdx, val, n = synth.config_graph(args.graph)
    graph = graph_input(args.graph, "")
    graph.verbose = False
    graph.load_from_csr(rowPtr, colIdx, val)
    nnz = graph.mtx_edges
    ops = sweep.operators_of(graph)
    dec = SpMMDecider()
    dec.gen_model_dict(dims)
    rows = (n + 1) // 2 * 2
    ci = ops[0].colIdx
    table = []
    for d in dims:
        X = torch.randn(rows, d, device="cuda", generator=torch.Generator(device="cuda").manual_seed(d))
        if_split, vec, cf, bw = (int(v) for v in dec.config_PCSR(graph, d))
        op = ops[(1 if if_split else 0) + (2 if vec == 2 else 0)]
        k_ms = op.time_ms(X, CF=cf, blkWarpNum=bw, warmup=3, iters=10)
        plan = _capi.spmm_plan(d, cf, bw)
        row = {"dim": d, "kernel_ms": round(k_ms, 5), "pick": [if_split, vec, sweep.cf_label(cf), bw], "probes": {}}
        gathered = 4.0 * nnz * d
        for lanes in sorted({plan["lanes_per_row"], min(8, d // 4), min(32, d // 4)}):
            ms, unroll, per_wave = gather_probe_ms(ci, nnz, X, lanes)
            row["probes"]["lanes%d" % lanes] = {"ms": round(ms, 5), "unroll": unroll, "entries_per_wave": per_wave,
                                                "gathered_GBps": round(gathered / ms / 1e6, 1)}
        best = min(v["ms"] for v in row["probes"].values())
        row["kernel_gathered_GBps"] = round(gathered / k_ms / 1e6, 1)
        row["gather_ceiling_frac"] = round(best / k_ms, 4)
        table.append(row)
    print(json.dumps({"metric": "gather ceiling: bare gathers of the pattern vs the SpMM kernel", "unit": "ratio",
                      "value": table[-1]["gather_ceiling_frac"], "n_gpus": 1, "steps": 10, "warmup": 3,
                      "ms_per_step": table[-1]["kernel_ms"], "higher_is_better": True, "scaling": "weak",
                      "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                      "config": {"workload": "%s gather ceiling" % args.graph, "nodes": n, "nnz": nnz}, "per_dim": table}))


def bench_footprint(args):
    """What the memory system delivers to a gather, as a function of the gathered footprint: 2^24 uniformly random row
    indices in [0, F), rows of N floats fetched 128 bytes per 8-lane group (psp_probe_gather_f32), F from L2-resident
    to far beyond the caches.  Gives the two rates an SpMM's gathers run between on this GPU: lines that hit the L2
    and lines that come from HBM."""
    import torch

    from paramspmm_ae_amd import _capi

    L, p = _capi.lib, _capi.ptr
    nnz = 1 << 24
    dims = [int(d) for d in args.dims.split(",")] if args.dims != DEFAULT_DIMS else [16, 32, 128]
    stream = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device="cuda").manual_seed(1)
    table = []
    for N in dims:
        lanes = min(8, N // 4)
        for logF in range(13, 25):
            F = 1 << logF
            if F * N * 4 > (2 << 30):
                break
            X = torch.ones(F, N, device="cuda")
            ci = torch.randint(0, F, (nnz,), device="cuda", dtype=torch.int32, generator=gen)
            ms, unroll, per_wave = gather_probe_ms(ci, nnz, X, lanes)
            tiles = (N // 4 + lanes - 1) // lanes
            table.append({"dim": N, "rows": F, "footprint_MiB": round(F * N * 4 / 2 ** 20, 1), "ms": round(ms, 5),
                          "gathered_GBps": round(4.0 * nnz * N / ms / 1e6, 1),
                          "requests_per_ns": round(nnz * tiles / ms / 1e6, 2)})
            del X, ci
    print(json.dumps({"metric": "gather rate vs footprint (uniform random rows, 128-byte requests)", "unit": "GB/s",
                      "value": table[-1]["gathered_GBps"], "n_gpus": 1, "steps": 5, "warmup": 1,
                      "ms_per_step": table[-1]["ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
                      "dtype": "f32", "data": "synthetic",
                      "config": {"workload": "gather rate vs footprint", "requests": nnz}, "table": table}))


def bench_agnn(args):
    """Attention layers on the R-MAT pattern (BASELINE.json configs[3]): per layer e = A_e * <X_i, Y_j> on the
    stored entries (SDDMM, K = 32 and 64, rows L2-normalised), softmax over each row's entries, then SpMM with
    H [n, 32].  Five layers per step.  The reference's AGNN has neither the A_e factor nor the softmax; they are
    the additions `csr_sddmm_scaled` and `segment_softmax` of this build."""
    import torch

    import paramspmm_ae_amd  # noqa: F401
    import ParamSDDMM
    import ParamSpMM
    from paramspmm_ae_amd import _capi, synth

    from paramspmm_ae_amd.decider import SpMMDecider
    from paramspmm_ae_amd.graph_input import graph_input

    graph = args.graph
    rowPtr, colIdx, val, n = synth.config_graph(graph)
    nnz = colIdx.size
    g = graph_input(graph, "")
    g.verbose = False
    g.load_from_csr(rowPtr, colIdx, val)
    dec = SpMMDecider()
    dec.gen_model_dict([32])
    if_split, _, CF, bw = dec.config_PCSR(g, 32)  # the edge values live in CSR order, so the CSR layouts are used
    c = g.csr_data
    bw |= _capi.bw_stripe(c.xcd_stripe(bool(if_split)))  # the XCD stripe chosen for this format
    rp, ci, v = c.rowPtr.cuda(), c.colIdx.cuda(), c.val.cuda()
    rps, tr = c.rowPtr_split.cuda(), c.target_row.cuda()
    gen = torch.Generator(device="cuda").manual_seed(7)
    out = {"metric": "AGNN attention layer stack: SDDMM (with row maxima) + softmax-weighted SpMM(N=32), 5 layers", "unit": "ms per 5 layers",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": False, "scaling": "weak",
           "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "%s pattern, K in (32, 64), H [n, 32]" % graph, "nodes": n, "nnz": nnz,
                      "format": "csr_split" if if_split else "csr", "CF": CF, "blkWarpNum": bw}, "per_K": []}
    H = torch.randn(n, 32, device="cuda", generator=gen)
    for K in (32, 64):
        X = torch.nn.functional.normalize(torch.randn(n, K, device="cuda", generator=gen), dim=1).contiguous()
        Y = torch.nn.functional.normalize(torch.randn(n, K, device="cuda", generator=gen), dim=1).contiguous()

        def layers_unfused():
            h = H
            for _ in range(5):
                if if_split:
                    e = ParamSDDMM.csr_split_sddmm_scaled(X, Y, rps, ci, v, tr, bw)
                    a = ParamSDDMM.segment_softmax(rp, e)
                    h = ParamSpMM.csr_split_spmm(h, rps, ci, a, tr, CF, bw)
                else:
                    e = ParamSDDMM.csr_sddmm_scaled(X, Y, rp, ci, v, bw)
                    a = ParamSDDMM.segment_softmax(rp, e)
                    h = ParamSpMM.csr_spmm(h, rp, ci, a, CF, bw)
            return h

        def layers():
            # two kernels per layer: the SDDMM also delivers the row maxima, the SpMM forms the softmax weights itself
            h = H
            for _ in range(5):
                if if_split:
                    e, m = ParamSDDMM.csr_split_sddmm_scaled_rowmax(X, Y, rps, ci, v, tr, n, bw)
                    h = ParamSpMM.csr_split_spmm_softmax(h, rps, ci, e, m, tr, CF, bw)
                else:
                    e, m = ParamSDDMM.csr_sddmm_scaled_rowmax(X, Y, rp, ci, v, bw)
                    h = ParamSpMM.csr_spmm_softmax(h, rp, ci, e, m, CF, bw)
            return h

        def timed(fn):
            for _ in range(args.warmup):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) * 1e3 / args.steps

        err = (layers() - layers_unfused()).abs().max().item()
        ms_unfused = timed(layers_unfused)
        ms = timed(layers)
        flops = 5 * (2.0 * nnz * K + 2.0 * nnz * 32)
        # algorithmic bytes per layer: SDDMM 4(M+1)+4nnz+4nnz(A_e)+8nK+4nnz(+4n maxima) ; SpMM 4(M+1)+8nnz+4n+8n*32
        b = 5 * ((4 * (n + 1) + 12 * nnz + 8 * n * K + 4 * n) + (4 * (n + 1) + 8 * nnz + 4 * n + 8 * n * 32))
        out["per_K"].append({"K": K, "ms": round(ms, 4), "ms_unfused": round(ms_unfused, 4), "max_abs_diff_to_unfused": err, "gflops": round(flops / ms / 1e6, 1),
                             "alg_GBps": round(b / ms / 1e6, 1), "frac_hbm": round(b / ms / 1e6 / HBM_PEAK_GBS, 4)})
    out["value"] = out["per_K"][-1]["ms"]
    out["ms_per_step"] = out["value"]
    print(json.dumps(out))


def bench_sddmm(args):
    """SDDMM out[p] = <A[row(p)], B[col(p)]> over the stored pattern (reference semantics: unscaled), widths
    K = 16..128, all four formats at both workgroup sizes; the best per width is reported with its algorithmic
    bytes (row pointers + column indices + A + B + the output) against the HBM peak, next to rocSPARSE's SDDMM."""
    import torch

    import paramspmm_ae_amd  # noqa: F401
    import ParamSDDMM
    from paramspmm_ae_amd import _capi, synth
    from paramspmm_ae_amd.graph_input import graph_input

    rowPtr, colIdx, val, n = synth.config_graph(args.graph)
    nnz = colIdx.size
    g = graph_input(args.graph, "")
    g.verbose = False
    g.load_from_csr(rowPtr, colIdx, val)
    c, b = g.csr_data, g.bcsr_data
    dev = "cuda"
    C = {k: c.on_device(k, dev) for k in ("rowPtr", "colIdx", "val", "rowPtr_split", "target_row")}
    Bf = {k: b.on_device(k, dev) for k in ("rowPtr", "colIdx", "val", "rowPtr_split", "target_row")}
    nblk = Bf["colIdx"].numel()
    rows = (n + 1) // 2 * 2
    gen = torch.Generator(device="cuda").manual_seed(7)
    stripe = [_capi.bw_stripe(f.xcd_stripe(sp)) for f, sp in ((c, False), (c, True), (b, False), (b, True))]

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    # the windowed layout beside the PCSR formats when the matrix has the locality it is made for
    from paramspmm_ae_amd.GNN import WINDOW_MIN_LOCAL_SHARE

    rp_w, ci_w, _, local_share = c.window_format(dev)
    windowed = local_share >= WINDOW_MIN_LOCAL_SHARE

    per_K = []
    for K in (16, 32, 64, 128):
        A = torch.randn(rows, K, device=dev, generator=gen)
        Bm = torch.randn(rows, K, device=dev, generator=gen)
        cands = {}
        if windowed:
            cands[("window", 0)] = lambda: ParamSDDMM.window_sddmm(A, Bm, rp_w, ci_w, None)
        for bw in (4, 8):
            # each format with the XCD stripe graph_input chose for it (flag bits of blkWarpNum)
            cands[("csr", bw)] = lambda bw=bw: ParamSDDMM.csr_sddmm(A, Bm, C["rowPtr"], C["colIdx"], C["val"], 1, bw | stripe[0])
            cands[("csr_split", bw)] = lambda bw=bw: ParamSDDMM.csr_split_sddmm(A, Bm, C["rowPtr_split"], C["colIdx"], C["val"], C["target_row"], 1, bw | stripe[1])
            # plain layouts with the entry-balanced walk (PSP_BW_BALANCED), what pcsr_spmm uses on a graph with hub rows
            cands[("csr_balanced", bw)] = lambda bw=bw: ParamSDDMM.csr_sddmm(A, Bm, C["rowPtr"], C["colIdx"], C["val"], 1, bw | 0x100)
            cands[("bcsr_balanced", bw)] = lambda bw=bw: ParamSDDMM.bcsr_sddmm(A, Bm, Bf["rowPtr"], Bf["colIdx"], Bf["val"], 1, bw | 0x100)
            cands[("bcsr", bw)] = lambda bw=bw: ParamSDDMM.bcsr_sddmm(A, Bm, Bf["rowPtr"], Bf["colIdx"], Bf["val"], 1, bw | stripe[2])
            cands[("bcsr_split", bw)] = lambda bw=bw: ParamSDDMM.bcsr_split_sddmm(A, Bm, Bf["rowPtr_split"], Bf["colIdx"], Bf["val"], Bf["target_row"], 1, bw | stripe[3])
        times = {k: timed(f) for k, f in cands.items()}
        (fmt, bw), ms = min(times.items(), key=lambda kv: kv[1])
        if fmt == "window":
            alg = 4 * rp_w.numel() + 4 * nnz + 8 * n * K + 4 * nnz
        elif fmt.startswith("bcsr"):
            alg = 4 * (Bf["rowPtr_split" if "split" in fmt else "rowPtr"].numel()) + 12 * nblk + 8 * n * K + 8 * nblk
        else:
            alg = 4 * (C["rowPtr_split" if "split" in fmt else "rowPtr"].numel()) + 4 * nnz + 8 * n * K + 4 * nnz
        if "split" in fmt:
            alg += 4 * (Bf if fmt.startswith("bcsr") else C)["target_row"].numel()
        vals = C["val"].clone()
        vendor_ms = timed(lambda: ParamSDDMM.cusparse_sddmm_compute(A[:n].contiguous() if rows != n else A,
                                                                    Bm[:n].contiguous() if rows != n else Bm,
                                                                    C["rowPtr"], C["colIdx"], vals)) if not args.no_vendor else None
        per_K.append({"K": K, "format": fmt, "blkWarpNum": bw, "ms": round(ms, 5), "gflops": round(2.0 * nnz * K / ms / 1e6, 1),
                      "alg_bytes": int(alg), "alg_GBps": round(alg / ms / 1e6, 1), "frac_hbm": round(alg / ms / 1e6 / HBM_PEAK_GBS, 4),
                      "all_ms": {"%s/%d" % k: round(v, 5) for k, v in times.items()},
                      "rocsparse_ms": None if vendor_ms is None else round(vendor_ms, 5)})
    total_ms = sum(r["ms"] for r in per_K)
    value = sum(2.0 * nnz * r["K"] for r in per_K) / total_ms / 1e6
    cpu = None
    if not args.no_cpu:
        # cpu_baseline: the C restatement of the reference's CSR SDDMM (oracle/paramsp_oracle.c, one scalar thread) on a
        # bounded sample: the leading rows that hold about four million stored entries, K = 64
        import time as _t
        from oracle import oracle as orc

        K = 64
        m = int(np.searchsorted(rowPtr, min(nnz, 4_000_000), side="right")) - 1
        m = max(m, 1)
        take = int(rowPtr[m])
        rng = np.random.default_rng(0)
        Ah, Bh = rng.standard_normal((rows, K)).astype(np.float32), rng.standard_normal((rows, K)).astype(np.float32)
        t0 = _t.perf_counter()
        orc.sddmm_csr(rowPtr[:m + 1], colIdx[:take], Ah, Bh)
        dt = _t.perf_counter() - t0
        cpu = {"value": round(2.0 * take * K / dt / 1e9, 3), "unit": "GFLOP/s", "cores": 1, "kind": "port",
               "sample": "oracle orc_sddmm_csr (scalar C) on the first %d rows (%d stored entries) of the same graph, K = 64, one pass (%.1f s)" % (m, take, dt)}
        # beside it, the gathered product in torch on all host threads (a dense [n, n] mask is impossible at this size)
        rows_h = torch.from_numpy(np.repeat(np.arange(m, dtype=np.int64), np.diff(rowPtr[:m + 1])))
        cols_h = torch.from_numpy(colIdx[:take].astype(np.int64))
        At, Bt = torch.from_numpy(Ah), torch.from_numpy(Bh)

        def torch_once():
            o = torch.empty(take)
            for s0 in range(0, take, 1 << 18):
                sl = slice(s0, min(take, s0 + (1 << 18)))
                o[sl] = (At[rows_h[sl]] * Bt[cols_h[sl]]).sum(1)
            return o
        torch_once()
        t0, reps = _t.perf_counter(), 0
        while reps < 3 or _t.perf_counter() - t0 < 3.0:
            torch_once()
            reps += 1
        cpu_torch = {"value": round(2.0 * take * K * reps / (_t.perf_counter() - t0) / 1e9, 2), "unit": "GFLOP/s",
                     "cores": torch.get_num_threads()}
    # roofline of the width that takes the most time; HBM traffic from the committed counter summary when it has the
    # same configuration (| K | layout | wavefronts | ... | HBM bytes | in column 11)
    dom = max(per_K, key=lambda r: r["ms"])
    traffic = None
    prof = os.path.join(ROOT, "profiles", "psp_sddmm_kernel_%s_trace_and_pmc.md" % args.graph)
    if os.path.exists(prof):
        for line in open(prof):
            cells = [c.strip() for c in line.strip().strip("|").split("|")]
            if len(cells) >= 11 and cells[0].isdigit() and (int(cells[0]), cells[1], int(cells[2])) == (dom["K"], dom["format"], dom["blkWarpNum"]):
                traffic = int(cells[10])
    roofline = {"bound": "hbm", "achieved": dom["alg_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom["frac_hbm"],
                "traffic": traffic, "kernel": "psp_sddmm_kernel, K = %d, %s, %d wavefronts per workgroup" % (dom["K"], dom["format"], dom["blkWarpNum"]),
                "alg_bytes_per_launch": dom["alg_bytes"], "ms_per_launch": dom["ms"]}
    print(json.dumps({"cpu_baseline": cpu, "cpu_torch_gathered": cpu_torch if cpu else None, "roofline": roofline,
                      "metric": "SDDMM GFLOP/s (2*nnz*K) over K = 16..128", "value": round(value, 1), "unit": "GFLOP/s",
                      "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(total_ms, 4),
                      "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                      "config": {"workload": "%s SDDMM width sweep" % args.graph, "nodes": n, "nnz": nnz}, "per_K": per_K}))


def bench_gcn(args):
    """GCN, GIN and AGNN training epochs (BASELINE.json configs[4]): 5 layers, hidden 16 / 32 / 128, 16 classes, random
    features and weights, forward + backward + Adam, on the 1M-node stochastic block model in community order
    (C5) and randomly permuted (C5p).  --epochs timed epochs after one warm-up epoch (default 200, the reference's
    protocol, GNN.py:126-151)."""
    from paramspmm_ae_amd import GNN

    out = {"metric": "GCN / GIN / AGNN epoch ms (5 layers, fwd+bwd+Adam), SBM 1M nodes", "unit": "ms per epoch", "n_gpus": 1,
           "steps": args.epochs, "warmup": 1, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
           "dtype": "f32", "data": "synthetic", "config": {"workload": "C5 / C5p, hidden 16 32 128, 16 classes"}, "epochs": []}
    graphs = [args.graph] if args.graph in ("C5", "C5p", "C1") else ["C5", "C5p"]
    for g in graphs:
        for net in ("GCN", "GIN", "AGNN"):
            argv = ["--net", net, "--synthetic", g, "--hidden_list", "16", "32", "128", "--num_classes", "16",
                    "--num_features", "32", "--num_epoches", str(args.epochs)]
            res = GNN.main(argv)
            # the same epochs with the training step recorded once in a HIP graph and replayed
            res_graph = GNN.main(argv + ["--hip_graph"])
            for (name, hidden), ms in res.items():
                out["epochs"].append({"graph": name, "net": net, "hidden": hidden, "ms_per_epoch": round(ms, 3),
                                      "ms_per_epoch_hip_graph": round(res_graph[(name, hidden)], 3)})
    out["value"] = out["epochs"][0]["ms_per_epoch"]
    out["ms_per_step"] = out["value"]
    print(json.dumps(out))


def bench_build(args):
    """PCSR format construction (2x1 BCSR + both row splits): the host builders against the device builders on the
    same CSR arrays.  Device times start with the CSR arrays on the GPU and end with the built arrays on the GPU
    (synchronised); `device_roundtrip_ms` adds the upload of the CSR and the copy of the results back to the host,
    which is what graph_input.load_from_csr pays to keep its CPU-tensor attributes."""
    import time
    import torch
    from paramspmm_ae_amd import synth, device_builder  # the package puts its lib/ directory on sys.path
    from paramspmm_ae_amd.graph_input import build_bcsr
    import ParamSpMM

    rowPtr, colIdx, val, n = synth.config_graph(args.graph)
    g = 32
    t0 = time.perf_counter()
    rb, cb, vb = build_bcsr(rowPtr, colIdx, val, build_on="host")
    k = np.diff(rowPtr)
    off = np.zeros(n + 1, np.int32)
    off[1:] = np.cumsum((k + g - 1) // g)
    ParamSpMM.split_csr_par(torch.from_numpy(rowPtr), torch.from_numpy(off), g)
    kb = np.diff(rb)
    offb = np.zeros(rb.size, np.int32)
    offb[1:] = np.cumsum((kb + g - 1) // g)
    ParamSpMM.split_csr_par(torch.from_numpy(rb), torch.from_numpy(offb), g)
    host_ms = (time.perf_counter() - t0) * 1e3

    def device_once(upload):
        t0 = time.perf_counter()
        d = [torch.from_numpy(a).cuda() for a in (rowPtr, colIdx, val)] if upload else dev
        t1 = time.perf_counter()
        b = device_builder.build_bcsr_device(*d)
        s1 = device_builder.split_csr_device(d[0], g)
        s2 = device_builder.split_csr_device(b[0], g)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        if upload:
            [t.cpu() for t in (*b, *s1, *s2)]
        return (t2 - t1) * 1e3, (time.perf_counter() - t0) * 1e3

    dev = [torch.from_numpy(a).cuda() for a in (rowPtr, colIdx, val)]
    device_once(False)
    dev_ms = min(device_once(False)[0] for _ in range(max(3, args.steps)))
    round_ms = min(device_once(True)[1] for _ in range(3))
    print(json.dumps({"metric": "PCSR construction ms (2x1 BCSR + CSR and BCSR row split, g=32)", "unit": "ms", "n_gpus": 1,
                      "steps": max(3, args.steps), "warmup": 1, "higher_is_better": False, "scaling": "weak",
                      "vs_baseline": None, "dtype": "i32", "data": "synthetic",
                      "config": {"workload": "%s format construction" % args.graph, "nodes": n, "nnz": int(rowPtr[-1])},
                      "value": round(dev_ms, 3), "ms_per_step": round(dev_ms, 3), "device_ms": round(dev_ms, 3),
                      "device_roundtrip_ms": round(round_ms, 3), "host_ms": round(host_ms, 3),
                      "speedup_device": round(host_ms / dev_ms, 1), "speedup_roundtrip": round(host_ms / round_ms, 1)}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--epochs", type=int, default=200, help="--workload gcn: timed epochs per network and width")
    ap.add_argument("--graph", default="C2", help="C1, C2, C3, C3s, C5, C5p (synth.config_graph)")
    ap.add_argument("--dims", default=DEFAULT_DIMS)
    ap.add_argument("--pick", default="auto",
                    help="auto (decider if its forests are built, else sweep) | sweep | decider | "
                         "fixed:<csr|csr_split|bcsr|bcsr_split>:<CF>:<blkWarpNum> | window[:<variant>] (the windowed layout)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain device copy of X (known size) so a counter run can be calibrated")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-vendor", action="store_true", help="skip the rocSPARSE comparison leg")
    ap.add_argument("--dump", default=None, help="write the full sweep table (every column, every width) as JSON")
    ap.add_argument("--reorder", choices=["community", "degree"], default=None,
                    help="spmm workload: permute rows and columns together at load time (paramspmm_ae_amd/reorder.py)")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip what follows the timed region: decider check, gather ceiling, SDDMM and GCN legs")
    ap.add_argument("--workload", choices=["spmm", "agnn", "gcn", "build", "sddmm", "gather", "footprint"], default="spmm",
                    help="spmm: the headline width sweep; agnn: SDDMM -> row softmax -> SpMM attention layers; "
                         "gcn: GCN / GIN training epochs on the SBM graph; build: PCSR construction, host against device; "
                         "sddmm: SDDMM width sweep over the four formats; gather: the bare gathers of a pattern beside the kernel; "
                         "footprint: gather rate of uniformly random rows against the gathered footprint")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (no multi-GPU path exists)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    if args.workload == "agnn":
        return bench_agnn(args)
    if args.workload == "gcn":
        return bench_gcn(args)
    if args.workload == "build":
        return bench_build(args)
    if args.workload == "sddmm":
        return bench_sddmm(args)
    if args.workload == "gather":
        return bench_gather(args)
    if args.workload == "footprint":
        return bench_footprint(args)
    from paramspmm_ae_amd import _capi, synth, sweep
    from paramspmm_ae_amd.graph_input import graph_input

    dims = [int(d) for d in args.dims.split(",")]
    t0 = time.time()
    rowPtr, colIdx, val, n = synth.config_graph(args.graph)
    graph = graph_input(mtx_name=args.graph, path="")
    graph.verbose = False
    t_re = time.time()
    graph.load_from_csr(rowPtr, colIdx, val, reorder=args.reorder)
    load_s = time.time() - t_re
    nnz = graph.mtx_edges
    ops = sweep.operators_of(graph)  # vec1, vec1_split, vec2, vec2_split on the GPU
    fmt_names = ["csr", "csr_split", "bcsr", "bcsr_split"]
    F = {"n": n, "nnz": nnz, "S": graph.csr_data.target_row.numel(), "Mb": graph.bcsr_data.num_nodes,
         "nblk": graph.bcsr_data.colIdx.numel(), "Sb": graph.bcsr_data.target_row.numel()}
    setup_s = time.time() - t0

    rows = (n + 1) // 2 * 2
    gen = torch.Generator(device="cuda").manual_seed(1234)
    Xs = {d: torch.randn(rows, d, device="cuda", generator=gen) for d in dims}
    if rows != n:
        for d in dims:
            Xs[d][n:].zero_()
    Ys = {d: torch.empty(rows, d, device="cuda") for d in dims}

    # ---- choose one configuration per width --------------------------------------------------------
    chosen = {}
    table = {}
    decider = None
    pick = args.pick
    if pick == "auto":
        from paramspmm_ae_amd.decider import DEFAULT_PICKLE_PATH

        have = all(os.path.exists(os.path.join(DEFAULT_PICKLE_PATH, "rnd_tree_%d.pkl" % d)) for d in range(16, 257, 16))
        pick = "decider" if have else "sweep"
    if pick == "decider":
        from paramspmm_ae_amd.decider import SpMMDecider

        decider = SpMMDecider()
        decider.gen_model_dict(dims)
    fixed = None
    win_op = None
    if pick.startswith("window"):
        # the windowed layout at every width: window[:variant]; encoded as vec_size 0 in the configuration tuples
        from paramspmm_ae_amd.PCSR import pcsr_spmm

        win_op = pcsr_spmm(graph, vec_size=1, if_split=False, CF=0, window=True)
        fixed = (0, 0, int(pick.split(":")[1]) if ":" in pick else 0, 0)
    if pick.startswith("fixed:"):
        _, f_fmt, f_cf, f_bw = pick.split(":")
        if "." in f_cf:  # native configuration: vectors.lanes.unroll.segments_per_wave[.e]  (0 segments = automatic)
            parts = f_cf.split(".")
            c_, l_, u_, w_ = (int(v) for v in parts[:4])
            f_cf = _capi.pack_cf(c_, l_, u_, w_ or None, even_split=parts[-1] == "e")
        fixed = (int("split" in f_fmt), 2 if f_fmt.startswith("bcsr") else 1, int(f_cf), int(f_bw))
    for d in dims:
        if pick == "sweep" or args.dump:
            ms, gf = sweep.sweep_dim(ops, d, nnz, n, warmup=2, iters=5, X=Xs[d])
            table[d] = {"columns": sweep.column_names(d), "ms": ms.tolist()}
        if pick == "sweep":
            chosen[d] = sweep.decode_column(d, int(np.argmin(ms)))
        elif pick == "decider":
            chosen[d] = tuple(int(v) for v in decider.config_PCSR(graph, d))
        else:
            chosen[d] = fixed
    if args.dump:
        with open(args.dump, "w") as f:
            json.dump({"graph": args.graph, "n": n, "nnz": nnz, "formats": F, "table": table}, f)

    stream = torch.cuda.current_stream().cuda_stream
    p = _capi.ptr
    L = _capi.lib

    def launcher(d, ops_, chosen_):
        if_split, vec, cf, bw = chosen_[d]
        if vec == 0:
            X, Y = Xs[d], Ys[d]
            w = win_op
            return lambda: L.psp_spmm_window_f32(p(w.rowPtr_w), p(w.colIdx), p(w.val), p(X), p(Y), n, int(w.colIdx.numel()), d,
                                                 rows, cf, 0, None, stream)
        op = ops_[(1 if if_split else 0) + (2 if vec == 2 else 0)]
        X, Y = Xs[d], Ys[d]
        a = (p(op.rowPtr), p(op.colIdx), p(op.val))
        nrows = op.rowPtr.numel() - 1
        bw |= op.bw_flags  # the XCD stripe graph_input chose for this format
        if vec == 1 and not if_split:
            return lambda: L.psp_spmm_csr_f32(*a, p(X), p(Y), nrows, d, rows, cf, bw, stream)
        if vec == 1:
            return lambda: L.psp_spmm_csr_split_f32(*a, p(op.target_row), p(X), p(Y), nrows, d, rows, cf, bw, stream)
        if not if_split:
            return lambda: L.psp_spmm_bcsr_f32(*a, p(X), p(Y), nrows, d, rows, cf, bw, stream)
        return lambda: L.psp_spmm_bcsr_split_f32(*a, p(op.target_row), p(X), p(Y), nrows, d, rows, cf, bw, stream)

    def timed_steps(ops_, chosen_):
        """args.warmup untimed steps, then args.steps timed ones bracketed by synchronisation; one step = one SpMM per
        width.  Returns (wall seconds, {width: [(start event, stop event)]})."""
        launch = {d: launcher(d, ops_, chosen_) for d in dims}

        def step(events=None, k=0):
            for d in dims:
                if events is not None:
                    e0, e1 = events[d][k]
                    e0.record()
                rc = launch[d]()
                if events is not None:
                    e1.record()
                if rc != 0:
                    _capi.check(rc)

        for _ in range(args.warmup):
            step()
        # the events exist before the clock starts (an event is created by its first record): on a small graph the
        # timed region would otherwise measure the host creating them
        events_ = {d: [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                       for _ in range(args.steps)] for d in dims}
        for pairs in events_.values():
            for e0, e1 in pairs:
                e0.record()
                e1.record()
        torch.cuda.synchronize()
        t0_ = time.perf_counter()
        for k in range(args.steps):
            step(events_, k)
        torch.cuda.synchronize()
        return time.perf_counter() - t0_, events_

    if args.calibrate_copy:
        d0 = dims[-1]
        Ys[d0].copy_(Xs[d0])  # moves 2 * rows * d0 * 4 bytes
        print("calibration copy: %d bytes read, %d bytes written" % (rows * d0 * 4, rows * d0 * 4), file=sys.stderr)
    wall, events = timed_steps(ops, chosen)

    flops_step = sum(2.0 * nnz * d for d in dims)
    value = flops_step * args.steps / wall / 1e9

    per_dim = []
    for d in dims:
        ms = float(np.mean([a.elapsed_time(b) for a, b in events[d]]))
        if_split, vec, cf, bw = chosen[d]
        windowed = vec == 0
        fmt = "window" if windowed else fmt_names[(1 if if_split else 0) + (2 if vec == 2 else 0)]
        # windowed layout: the CSR arrays and one more row pointer per row
        b_alg = algorithmic_bytes("csr", F, n, d) + 4 * (n + 1) if windowed else algorithmic_bytes(fmt, F, n, d)
        gbs = b_alg / (ms * 1e-3) / 1e9
        # no-reuse gather volume: every stored entry fetches its row of X (what a matrix without locality moves)
        stored = F["nblk"] if fmt.startswith("bcsr") else nnz
        b_gather = b_alg - 4 * n * d + 4 * stored * d
        per_dim.append({"dim": d, "format": fmt, "CF": cf, "config": "variant %d" % cf if windowed else sweep.cf_label(cf), "blkWarpNum": bw,
                        "xcd_stripe_rows": 0 if windowed else (ops[(1 if if_split else 0) + (2 if vec == 2 else 0)].bw_flags >> 12) * 256,
                        "ms": round(ms, 5),
                        "gflops": round(2.0 * nnz * d / (ms * 1e-3) / 1e9, 1), "alg_bytes": b_alg,
                        "alg_GBps": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4),
                        "gather_bytes": int(b_gather),
                        "frac_hbm_no_reuse_gather": round(b_gather / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
    # The dominant kernel: widths that share (vectors per lane, vector width, unroll, format) run the same kernel
    # symbol, which is what a rocprofv3 kernel trace averages over; take the symbol with the largest share of time.
    by_symbol = {}
    for r in per_dim:
        if r["format"] == "window":
            import ParamSpMM

            v = int(ParamSpMM.window_plan(r["dim"], r["CF"])["variant"])
            sym = "psp_spmm_window_kernel<%s>" % {1: "1, 2, 256", 2: "1, 3, 512", 3: "2, 3, 512"}[v]
            r["kernel"] = sym
            by_symbol.setdefault(sym, []).append(r)
            continue
        plan = _capi.spmm_plan(r["dim"], r["CF"], r["blkWarpNum"])
        one_set = plan["register_sets"] == 1
        sym = "psp_spmm_kernel<%d, %d, %d, %d, %s, false, false, %s>" % (plan["coarsen"], plan["vec"], plan["unroll"],
                                                           2 if r["format"].startswith("bcsr") else 1,
                                                           "true" if "split" in r["format"] else "false",
                                                           "true" if one_set else "false")
        r["kernel"] = sym
        by_symbol.setdefault(sym, []).append(r)
    sym, rows_of = max(by_symbol.items(), key=lambda kv: sum(r["ms"] for r in kv[1]))
    sym_ms = sum(r["ms"] for r in rows_of)
    sym_bytes = sum(r["alg_bytes"] for r in rows_of)
    achieved = sym_bytes / (sym_ms * 1e-3) / 1e9
    traffic = measured_traffic(args.graph, rows_of)
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                "kernel": sym, "widths": [r["dim"] for r in rows_of],
                "alg_bytes_per_launch": int(sym_bytes / len(rows_of)), "ms_per_launch": round(sym_ms / len(rows_of), 5),
                "mean_frac_over_widths": round(float(np.mean([r["frac_hbm"] for r in per_dim])), 4),
                "gather_bytes_per_launch": int(sum(r["gather_bytes"] for r in rows_of) / len(rows_of)),
                "frac_no_reuse_gather": round(sum(r["gather_bytes"] for r in rows_of) / (sym_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

    out = {
        "metric": "SpMM GFLOP/s (2*nnz*N) over the feature-width sweep N=16..256, with HBM GB/s as fraction of 8 TB/s",
        "value": round(value, 1), "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3 / args.steps, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: R-MAT 2^20 nodes SpMM width sweep" % args.graph if args.graph == "C2" else args.graph,
                   "nodes": n, "nnz": nnz, "dims": dims, "pick": pick, "setup_s": round(setup_s, 1),
                   "reorder": args.reorder, "load_s": round(load_s, 2)},
        "roofline": roofline,
        "sweep": per_dim,
    }

    if not args.no_extras and win_op is None:
        # ---- gather ceiling of the dominant width: the bare gathers of the same pattern and X row tiles ----------
        dom = max(rows_of, key=lambda r: r["ms"])
        plan = _capi.spmm_plan(dom["dim"], dom["CF"], dom["blkWarpNum"])
        dom_op = ops[fmt_names.index(dom["format"])]
        stored = dom_op.colIdx.numel()
        probe_ms, probe_unroll, probe_per_wave = gather_probe_ms(dom_op.colIdx, stored, Xs[dom["dim"]], plan["lanes_per_row"])
        roofline["gather_ceiling"] = {"dim": dom["dim"], "probe_ms": round(probe_ms, 5), "kernel_ms": dom["ms"],
                                      "probe_gathered_GBps": round(4.0 * stored * dom["dim"] / probe_ms / 1e6, 1),
                                      "lanes_per_row": plan["lanes_per_row"], "unroll": probe_unroll,
                                      "entries_per_wave": probe_per_wave}
        roofline["gather_ceiling_frac"] = round(probe_ms / dom["ms"], 4)

        # ---- the decider's pick against the best swept configuration, per width --------------------------------
        if pick == "decider":
            checks = []
            for d in dims:
                ms_all, _ = sweep.sweep_dim(ops, d, nnz, n, warmup=1, iters=3, X=Xs[d])
                names = sweep.column_names(d)
                if_split, vec, cf, bw = chosen[d]
                col = [c for c in range(len(names)) if sweep.decode_column(d, c) == (if_split, vec, cf, bw)][0]
                best = int(np.argmin(ms_all))
                checks.append({"dim": d, "pick": names[col], "best": names[best], "t_pick_over_t_best": round(float(ms_all[col] / ms_all[best]), 3),
                               "ms_pick": round(float(ms_all[col]), 5), "ms_best": round(float(ms_all[best]), 5)})
            ratios = np.array([c["t_pick_over_t_best"] for c in checks])
            out["decider_vs_best"] = {"per_dim": checks, "share_within_10pct": round(float(np.mean(ratios <= 1.10)), 3),
                                      "mean_normalised_performance": round(float(np.mean(1.0 / ratios)), 4),
                                      "worst_t_pick_over_t_best": round(float(ratios.max()), 3),
                                      "columns_swept": int(sum(len(sweep.column_names(d)) for d in dims))}

        # ---- SDDMM at K = 64 on the same pattern ----------------------------------------------------------------
        import ParamSDDMM

        K = 64
        A = torch.randn(rows, K, device="cuda", generator=gen)
        Bm = torch.randn(rows, K, device="cuda", generator=gen)
        c_, b_ = ops[0], ops[2]
        cs_, bs_ = ops[1], ops[3]
        sd = {}
        for bw in (4, 8):
            sd[("csr", bw)] = lambda bw=bw: ParamSDDMM.csr_sddmm(A, Bm, c_.rowPtr, c_.colIdx, c_.val, 2, bw | c_.bw_flags)
            sd[("csr_split", bw)] = lambda bw=bw: ParamSDDMM.csr_split_sddmm(A, Bm, cs_.rowPtr, cs_.colIdx, cs_.val, cs_.target_row, 2, bw | cs_.bw_flags)
            sd[("bcsr", bw)] = lambda bw=bw: ParamSDDMM.bcsr_sddmm(A, Bm, b_.rowPtr, b_.colIdx, b_.val, 2, bw | b_.bw_flags)
            sd[("bcsr_split", bw)] = lambda bw=bw: ParamSDDMM.bcsr_split_sddmm(A, Bm, bs_.rowPtr, bs_.colIdx, bs_.val, bs_.target_row, 2, bw | bs_.bw_flags)
        sd_ms = {}
        for key, fn in sd.items():
            fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(5):
                fn()
            e1.record()
            torch.cuda.synchronize()
            sd_ms[key] = e0.elapsed_time(e1) / 5
        (sfmt, sbw), sms = min(sd_ms.items(), key=lambda kv: kv[1])
        if sfmt.startswith("bcsr"):
            salg = 4 * (F["Sb"] + 1 if "split" in sfmt else F["Mb"] + 1) + 12 * F["nblk"] + 8 * n * K + 8 * F["nblk"]
            salg += 4 * F["Sb"] if "split" in sfmt else 0
        else:
            salg = 4 * (F["S"] + 1 if "split" in sfmt else n + 1) + 4 * nnz + 8 * n * K + 4 * nnz
            salg += 4 * F["S"] if "split" in sfmt else 0
        out["sddmm"] = {"K": K, "format": sfmt, "blkWarpNum": sbw, "ms": round(sms, 5), "gflops": round(2.0 * nnz * K / sms / 1e6, 1),
                        "all_ms": {"%s/%d" % k: round(v, 5) for k, v in sd_ms.items()},
                        "roofline": {"bound": "hbm", "achieved": round(salg / sms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                     "frac": round(salg / sms / 1e6 / HBM_PEAK_GBS, 4),
                                     "traffic": measured_sddmm_traffic(args.graph, K, sfmt, sbw),
                                     "kernel": "psp_sddmm_kernel, K = 64, %s, %d wavefronts per workgroup" % (sfmt, sbw),
                                     "alg_bytes_per_launch": int(salg), "ms_per_launch": round(sms, 5)}}
        del A, Bm

    if not args.no_extras and args.reorder is None and pick == "decider":
        # ---- the same sweep after a reordering pass (rows and columns permuted together at load time,
        # paramspmm_ae_amd/reorder.py; the reference's inputs arrive Rabbit-ordered, README.md:14-16) ---------------
        out["reordered"] = {}
        for order, text in (("community", "label propagation, vertices sorted by label"),
                            ("degree", "vertices sorted by descending degree")):
            t1 = time.time()
            graph_r = graph_input(mtx_name=args.graph, path="")
            graph_r.verbose = False
            graph_r.load_from_csr(rowPtr, colIdx, val, reorder=order)
            load_r = time.time() - t1
            ops_r = sweep.operators_of(graph_r)
            chosen_r = {d: tuple(int(v) for v in decider.config_PCSR(graph_r, d)) for d in dims}
            wall_r, events_r = timed_steps(ops_r, chosen_r)
            F_r = {"n": n, "nnz": nnz, "S": graph_r.csr_data.target_row.numel(), "Mb": graph_r.bcsr_data.num_nodes,
                   "nblk": graph_r.bcsr_data.colIdx.numel(), "Sb": graph_r.bcsr_data.target_row.numel()}
            fracs = []
            for d in dims:
                ms = float(np.mean([a.elapsed_time(b) for a, b in events_r[d]]))
                if_split, vec, cf, bw = chosen_r[d]
                fmt = fmt_names[(1 if if_split else 0) + (2 if vec == 2 else 0)]
                fracs.append(algorithmic_bytes(fmt, F_r, n, d) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS)
            out["reordered"][order] = {"order": text, "value": round(flops_step * args.steps / wall_r / 1e9, 1), "unit": "GFLOP/s",
                                       "ms_per_step": round(wall_r * 1e3 / args.steps, 4), "speedup": round(wall / wall_r, 3),
                                       "mean_frac_over_widths": round(float(np.mean(fracs)), 4),
                                       "load_s_with_reordering": round(load_r, 2), "load_s_without": round(load_s, 2)}
            del ops_r, graph_r
            torch.cuda.empty_cache()

    if not args.no_vendor:
        # vendor library beside it: rocSPARSE CSR SpMM (default algorithm), the counterpart of the cuSPARSE baseline
        # the reference quotes its speed-ups against (SpMM/Baseline_kernel.cu:24-169)
        import ParamSpMM

        c = ops[0]
        v_ms = {}
        for d in dims:
            v_ms[d] = ParamSpMM.vendor_spmm_time_ms(0, Xs[d][:n].contiguous() if rows != n else Xs[d], c.rowPtr, c.colIdx, c.val, 1, 3)
        speedups = [v_ms[r["dim"]] / r["ms"] for r in per_dim]
        out["vendor_baseline"] = {"library": "rocSPARSE rocsparse_spmm, CSR, rocsparse_spmm_alg_default, fp32",
                                  "gflops": round(flops_step / (sum(v_ms.values()) * 1e-3) / 1e9, 1),
                                  "ms_per_width": {str(d): round(v_ms[d], 4) for d in dims},
                                  "speedup_per_width": {str(r["dim"]): round(s_, 2) for r, s_ in zip(per_dim, speedups)},
                                  "mean_speedup": round(float(np.mean(speedups)), 2)}

    if not args.no_cpu:
        # cpu_baseline: the product the reference itself checks against on the host, torch.sparse.mm of the CSR tensor
        # (verification.py:18-46), on all host threads, on a bounded sample of the widths
        s = torch.sparse_csr_tensor(graph.csr_data.rowPtr, graph.csr_data.colIdx, graph.csr_data.val, size=(n, n))
        sample_dims = [d for d in (16, 64, 128) if d in dims] or dims[:1]
        flops, secs, total_reps = 0.0, 0.0, 0
        for d in sample_dims:
            Xc = Xs[d][:n].cpu()
            torch.sparse.mm(s, Xc)  # warm-up
            reps = 0
            t1 = time.perf_counter()
            while reps < 3 or (time.perf_counter() - t1 < 3.0 and reps < 50):
                torch.sparse.mm(s, Xc)
                reps += 1
            secs += time.perf_counter() - t1
            flops += 2.0 * nnz * d * reps
            total_reps += reps
        out["cpu_baseline"] = {"value": round(flops / secs / 1e9, 2), "unit": "GFLOP/s", "cores": torch.get_num_threads(),
                               "kind": "reference",
                               "sample": "torch.sparse.mm(torch.sparse_csr_tensor(A), X) on the host, the product the reference verifies "
                                         "against (verification.py:18-46), same graph, widths %s, %d products in %.1f s"
                                         % (sample_dims, total_reps, secs)}
        # beside it the C restatement of the reference's CSR kernel (oracle/paramsp_oracle.c, one scalar thread); it
        # doubles as the checker of the GPU result at those widths
        from oracle import oracle as orc

        rp_h, ci_h, v_h = (graph.csr_data.rowPtr.numpy(), graph.csr_data.colIdx.numpy(), graph.csr_data.val.numpy())
        port_dims = [d for d in (16, 64) if d in dims] or dims[:1]
        flops, secs, err = 0.0, 0.0, 0.0
        for d in port_dims:
            Xc = Xs[d][:n].cpu().numpy()
            _capi.check(launcher(d, ops, chosen)())  # Ys[d] may hold a later leg's product (the reordered matrix)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            yo = orc.spmm_csr(rp_h, ci_h, v_h, Xc)
            secs += time.perf_counter() - t1
            flops += 2.0 * nnz * d
            err = max(err, float(np.abs(Ys[d][:n].cpu().numpy() - yo).max()))
        out["cpu_scalar_port"] = {"value": round(flops / secs / 1e9, 3), "unit": "GFLOP/s", "cores": 1, "kind": "port",
                                  "sample": "oracle orc_spmm_csr (scalar C, fp32 FMA chain per row), widths %s, one pass each (%.1f s)" % (port_dims, secs),
                                  "max_abs_gpu_minus_oracle": err}

    if not args.no_extras and args.graph == "C2":
        for d in list(Xs):
            del Xs[d], Ys[d]
        del ops, graph
        torch.cuda.empty_cache()
        # ---- the other graphs of the benchmark set, decider-picked configurations -----------------------------------
        if decider is not None:
            out["other_graphs"] = {
                "C3s 5-point stencil 2048^2": other_graph_leg("C3s", [64, 128], decider),
                "C5 block model 1M nodes, community order": other_graph_leg("C5", [16, 128], decider),
                "C5p block model 1M nodes, random order": other_graph_leg("C5p", [128], decider),
                "C5p after the community reordering pass at load time (label propagation)":
                    other_graph_leg("C5p", [128], decider, reorder="community"),
                "C3 Chung-Lu 2.45M nodes": other_graph_leg("C3", [128], decider, reps=5),
            }
        # ---- GCN training epochs on the 1M-node block model (the metric's second half) ------------------------------
        from paramspmm_ae_amd import GNN

        epochs = {}
        n_epochs = 200  # the reference's protocol: 1 warm-up epoch + 200 timed ones (GNN.py:126-151)
        with contextlib.redirect_stdout(sys.stderr):
            for net in ("GCN", "GIN", "AGNN"):
                res = GNN.main(["--net", net, "--synthetic", "C5", "--hidden_list", "16", "32", "128", "--num_classes", "16",
                                "--num_features", "32", "--num_epoches", str(n_epochs)])
                epochs[net] = {str(h): round(float(ms), 3) for (_, h), ms in res.items()}
        out["gcn_epoch_ms"] = {"value": epochs["GCN"]["16"], "unit": "ms per epoch", "epochs": n_epochs,
                               "by_hidden": epochs["GCN"], "gin_by_hidden": epochs["GIN"], "agnn_by_hidden": epochs["AGNN"],
                               "config": "5 layers, hidden 16 / 32 / 128 (value: GCN, hidden 16), 16 classes, 32 features, "
                                         "fwd+bwd+Adam, SBM 1M nodes (community order), decider-picked operators"}

    print(json.dumps(out))


if __name__ == "__main__":
    main()
