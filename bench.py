#!/usr/bin/env python3
"""Headline benchmark: ParamSpMM feature-width sweep on one MI355X.

Workload (BASELINE.json configs[1]): R-MAT graph with 2^20 nodes, about 16 off-diagonal entries per row,
self loops, values D^-1/2 (A+I) D^-1/2 in fp32, CSR int32; X = N(0,1) [2^20, N] for N = 16, 32, ..., 256.
One step = one SpMM at every one of the 16 widths, each in the configuration chosen for it (best of a short
sweep over the PCSR configurations, or the trained decider's pick with --pick decider).  Inputs are resident
in HBM before the timed region.  value = sum(2*nnz*N) * steps / wall time, in GFLOP/s.

The JSON line also carries
  roofline      for the width that takes the most time: algorithmic bytes
                4(M+1) + 8 nnz + 4 n N + 4 M N (CSR; split adds 8 S + 4, blocks use 4(Mb+1) + 12 nblk)
                divided by that launch's mean duration (HIP events on the launching stream), against 8 TB/s;
  sweep         the same numbers for every width;
  cpu_baseline  torch.sparse.mm on the host cores (the reference's own CPU checker) on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--graph", default="C2", help="C1, C2, C3, C3s, C5, C5p (synth.config_graph)")
    ap.add_argument("--dims", default=",".join(str(d) for d in range(16, 257, 16)))
    ap.add_argument("--pick", choices=["sweep", "decider", "csr"], default="sweep")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--dump", default=None, help="write the full sweep table (every column, every width) as JSON")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (no multi-GPU path exists)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    from paramspmm_ae_amd import _capi, synth, sweep
    from paramspmm_ae_amd.graph_input import graph_input

    dims = [int(d) for d in args.dims.split(",")]
    t0 = time.time()
    rowPtr, colIdx, val, n = synth.config_graph(args.graph)
    graph = graph_input(mtx_name=args.graph, path="")
    graph.verbose = False
    graph.load_from_csr(rowPtr, colIdx, val)
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
    if args.pick == "decider":
        from paramspmm_ae_amd.decider import SpMMDecider

        decider = SpMMDecider()
        decider.gen_model_dict(dims)
    for d in dims:
        if args.pick == "sweep" or args.dump:
            ms, gf = sweep.sweep_dim(ops, d, nnz, n, warmup=2, iters=5, X=Xs[d])
            table[d] = {"columns": sweep.column_names(d), "ms": ms.tolist()}
        if args.pick == "sweep":
            chosen[d] = sweep.decode_column(d, int(np.argmin(ms)))
        elif args.pick == "decider":
            chosen[d] = tuple(int(v) for v in decider.config_PCSR(graph, d))
        else:
            chosen[d] = (0, 1, 1, 4)
    if args.dump:
        with open(args.dump, "w") as f:
            json.dump({"graph": args.graph, "n": n, "nnz": nnz, "formats": F, "table": table}, f)

    stream = torch.cuda.current_stream().cuda_stream
    p = _capi.ptr
    L = _capi.lib

    def launcher(d):
        if_split, vec, cf, bw = chosen[d]
        op = ops[(1 if if_split else 0) + (2 if vec == 2 else 0)]
        X, Y = Xs[d], Ys[d]
        a = (p(op.rowPtr), p(op.colIdx), p(op.val))
        nrows = op.rowPtr.numel() - 1
        if vec == 1 and not if_split:
            return lambda: L.psp_spmm_csr_f32(*a, p(X), p(Y), nrows, d, rows, cf, bw, stream)
        if vec == 1:
            return lambda: L.psp_spmm_csr_split_f32(*a, p(op.target_row), p(X), p(Y), nrows, d, rows, cf, bw, stream)
        if not if_split:
            return lambda: L.psp_spmm_bcsr_f32(*a, p(X), p(Y), nrows, d, rows, cf, bw, stream)
        return lambda: L.psp_spmm_bcsr_split_f32(*a, p(op.target_row), p(X), p(Y), nrows, d, rows, cf, bw, stream)

    launch = {d: launcher(d) for d in dims}

    def step(events=None):
        for d in dims:
            if events is not None:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
            rc = launch[d]()
            if events is not None:
                e1.record()
                events[d].append((e0, e1))
            if rc != 0:
                _capi.check(rc)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    events = {d: [] for d in dims}
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(events)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    flops_step = sum(2.0 * nnz * d for d in dims)
    value = flops_step * args.steps / wall / 1e9

    per_dim = []
    for d in dims:
        ms = float(np.mean([a.elapsed_time(b) for a, b in events[d]]))
        if_split, vec, cf, bw = chosen[d]
        fmt = fmt_names[(1 if if_split else 0) + (2 if vec == 2 else 0)]
        b_alg = algorithmic_bytes(fmt, F, n, d)
        gbs = b_alg / (ms * 1e-3) / 1e9
        per_dim.append({"dim": d, "format": fmt, "CF": cf, "blkWarpNum": bw, "ms": round(ms, 5),
                        "gflops": round(2.0 * nnz * d / (ms * 1e-3) / 1e9, 1), "alg_bytes": b_alg,
                        "alg_GBps": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4)})
    dom = max(per_dim, key=lambda r: r["ms"])
    roofline = {"bound": "hbm", "achieved": dom["alg_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(dom["alg_GBps"] / HBM_PEAK_GBS, 4), "traffic": None,
                "kernel": "psp_spmm_kernel %s N=%d CF=%d bw=%d" % (dom["format"], dom["dim"], dom["CF"], dom["blkWarpNum"]),
                "alg_bytes_per_launch": dom["alg_bytes"], "ms_per_launch": dom["ms"],
                "mean_frac_over_widths": round(float(np.mean([r["frac_hbm"] for r in per_dim])), 4)}

    out = {
        "metric": "SpMM GFLOP/s (2*nnz*N) over the feature-width sweep N=16..256, with HBM GB/s as fraction of 8 TB/s",
        "value": round(value, 1), "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3 / args.steps, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: R-MAT 2^20 nodes SpMM width sweep" % args.graph if args.graph == "C2" else args.graph,
                   "nodes": n, "nnz": nnz, "dims": dims, "pick": args.pick, "setup_s": round(setup_s, 1)},
        "roofline": roofline,
        "sweep": per_dim,
    }

    if not args.no_cpu:
        # the reference's CPU path: torch.sparse.mm of the CSR tensor (verification.py:18-46), host cores
        s = torch.sparse_csr_tensor(graph.csr_data.rowPtr, graph.csr_data.colIdx, graph.csr_data.val, size=(n, n))
        sample_dims = [d for d in (16, 64, 128) if d in dims] or dims[:1]
        flops, secs = 0.0, 0.0
        for d in sample_dims:
            Xc = Xs[d][:n].cpu()
            torch.sparse.mm(s, Xc)  # warm-up
            reps = 0
            t1 = time.perf_counter()
            while reps < 3 or (time.perf_counter() - t1 < 4.0 and reps < 50):
                yc = torch.sparse.mm(s, Xc)
                reps += 1
            dt = time.perf_counter() - t1
            flops += 2.0 * nnz * d * reps
            secs += dt
        # checker duty: the GPU result of the last sampled width against the CPU product
        yg = Ys[sample_dims[-1]][:n].cpu()
        err = float((yg - yc).abs().max())
        out["cpu_baseline"] = {"value": round(flops / secs / 1e9, 2), "unit": "GFLOP/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": "torch.sparse.mm (CSR, fp32) on the same graph, widths %s, >=3 reps each, %d host threads of %d cpus; max |gpu-cpu| = %.2e"
                                         % (sample_dims, torch.get_num_threads(), os.cpu_count(), err)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
