#!/usr/bin/env python3
"""GCN / GIN / AGNN training driver with the command line of the reference's GNN.py:15-28 and its timing
loop (1 warm-up epoch + ``num_epoches`` timed epochs, Adam lr 0.01, prints ``training time per epoch``).

Besides ``--path/--mtx_name`` (MatrixMarket files) it accepts ``--synthetic NAME`` (a seeded generator of
``synth.config_graph``: C1, C2, C3, C3s, C5, C5p) because no dataset ships with this build.

    python -m paramspmm_ae_amd.GNN --net GCN --synthetic C1 --hidden_list 16 --num_classes 16 --num_epoches 20
"""
import argparse
import glob
import os
import time

import torch
import torch.nn as nn
import torch.nn.functional as F

from .decider import SpMMDecider, DEFAULT_PICKLE_PATH
from .gnn_conv import AGNNConv, GCNConv, GINConv, nll_loss_mean, softmax_nll_loss_mean
from .graph_input import graph_input
from .PCSR import pcsr_spmm


class Net_5layers(torch.nn.Module):
    """Five GCN layers, ReLU between, log-softmax out (GNN.py:43-61)."""

    def __init__(self, num_classes, num_features, x, spmm_dict, hidden):
        super().__init__()
        self.spmm_dict = spmm_dict
        self.x = x
        widths = [num_features, hidden, hidden, hidden, hidden, num_classes]
        self.conv1, self.conv2, self.conv3, self.conv4, self.conv5 = (
            GCNConv(widths[i], widths[i + 1]) for i in range(5)
        )
        self.fuse_relu = True  # False: F.relu between the layers as separate passes, as the reference's driver does

    def logits(self):
        """The network up to, and without, its log-softmax (what loss_of_step folds into the loss)."""
        if not self.fuse_relu:
            x = self.x
            for conv in (self.conv1, self.conv2, self.conv3, self.conv4):
                x = F.relu(conv(x, self.spmm_dict))
            return self.conv5(x, self.spmm_dict)
        # the same network with every ReLU applied by the layer that reads it (no activation passes)
        z = self.conv1(self.x, self.spmm_dict)
        for conv in (self.conv2, self.conv3, self.conv4, self.conv5):
            z = conv(z, self.spmm_dict, relu_input=True)
        return z

    def forward(self):
        return F.log_softmax(self.logits(), dim=1)


class GIN(torch.nn.Module):
    """Five GIN layers (GNN.py:104-123)."""

    def __init__(self, num_classes, num_features, x, spmm_dict, hidden):
        super().__init__()
        self.spmm_dict = spmm_dict
        self.x = x
        widths = [num_features, hidden, hidden, hidden, hidden, num_classes]
        self.conv1, self.conv2, self.conv3, self.conv4, self.conv5 = (
            GINConv(widths[i], widths[i + 1]) for i in range(5)
        )

        self.fuse_relu = True  # False: F.relu between the layers as separate passes, as the reference's driver does

    def logits(self):
        """The network up to, and without, its log-softmax (what loss_of_step folds into the loss)."""
        if not self.fuse_relu:
            x = self.x
            for conv in (self.conv1, self.conv2, self.conv3, self.conv4):
                x = F.relu(conv(x, self.spmm_dict))
            return self.conv5(x, self.spmm_dict)
        # the same network with every ReLU applied inside the sparse product of the layer that reads it
        z = self.conv1(self.x, self.spmm_dict)
        for conv in (self.conv2, self.conv3, self.conv4, self.conv5):
            z = conv(z, self.spmm_dict, relu_input=True)
        return z

    def forward(self):
        return F.log_softmax(self.logits(), dim=1)


class AGNN(torch.nn.Module):
    """num_layers attention layers with dropout after the first (GNN.py:82-101)."""

    def __init__(self, num_classes, num_features, x, spmm_dict, hidden, colIdx, num_layers=5):
        super().__init__()
        self.x = x
        self.spmm_dict = spmm_dict
        self.colIdx = colIdx
        self.conv1 = AGNNConv(num_features, hidden)
        self.hidden_layers = nn.ModuleList(AGNNConv(hidden, hidden) for _ in range(num_layers - 2))
        self.conv2 = AGNNConv(hidden, num_classes)
        self.relu = nn.ReLU()
        self.fuse_relu = True  # False: ReLU between the layers as separate passes, as the reference's driver does

    def logits(self):
        """The network up to, and without, its log-softmax (what loss_of_step folds into the loss)."""
        if not self.fuse_relu:
            x = self.relu(self.conv1(self.x, self.spmm_dict, self.colIdx))
            x = F.dropout(x, training=self.training)
            for conv in self.hidden_layers:
                x = self.relu(conv(x, self.spmm_dict, self.colIdx))
            return self.conv2(x, self.spmm_dict, self.colIdx)
        # The same network with every ReLU applied by the layer that reads it.  Dropout scales by a non-negative
        # mask, so it commutes with the activation: dropping the pre-activation values and activating afterwards
        # gives what the reference's order gives, with the same random mask.
        z = self.conv1(self.x, self.spmm_dict, self.colIdx)
        z = F.dropout(z, training=self.training)
        for conv in self.hidden_layers:
            z = conv(z, self.spmm_dict, self.colIdx, relu_input=True)
        return self.conv2(z, self.spmm_dict, self.colIdx, relu_input=True)

    def forward(self):
        return F.log_softmax(self.logits(), dim=1)


_FUSED_ADAM = os.environ.get("PSP_FUSED_ADAM", "1") != "0"


def loss_of_step(model, labels):
    """F.nll_loss(model(), labels) of the reference's training step (GNN.py:131-146).  The networks end in a
    log-softmax; with ``model.fuse_loss`` (the default) it is folded into the loss -- one pass over the logits instead
    of a softmax, a loss and their two backward passes."""
    if getattr(model, "fuse_loss", True) and hasattr(model, "logits"):
        return softmax_nll_loss_mean(model.logits(), labels)
    return nll_loss_mean(model(), labels)


def capture_training_step(model, labels, optimizer, warmup=3):
    """Records one training step (forward, loss, backward, Adam) into a HIP graph, the way PyTorch prescribes for
    whole-network capture: ``warmup`` eager steps on a side stream, gradients dropped, then one recorded step.
    Returns (graph, loss tensor the replays fill in).  Every replay is one epoch; nothing in it touches the host, so
    a small graph's epoch is no longer bound by launch latency.  The reference prepares for this (its Adam is
    created with capturable=True, GNN.py:127) but never captures."""
    model.train()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(warmup):
            optimizer.zero_grad(set_to_none=True)
            loss_of_step(model, labels).backward()
            optimizer.step()
    torch.cuda.current_stream().wait_stream(side)
    optimizer.zero_grad(set_to_none=True)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        loss = loss_of_step(model, labels)
        loss.backward()
        optimizer.step()
    return graph, loss


def train_profiling(model, labels, num_epoches, verbose=False, progress=False, hip_graph=False):
    """1 untimed epoch (unless verbose) + num_epoches timed epochs; returns ms per epoch (GNN.py:126-151).
    ``hip_graph``: the epoch is recorded once (after 3 eager warm-up epochs) and replayed."""
    # the reference's optimizer (GNN.py:127: Adam, lr 0.01, capturable); PyTorch's single-kernel form of the same update
    # where it exists, instead of some fifteen small launches per step
    try:
        optimizer = torch.optim.Adam(model.parameters(), lr=0.01, capturable=True, fused=_FUSED_ADAM)
    except (TypeError, RuntimeError):
        optimizer = torch.optim.Adam(model.parameters(), lr=0.01, capturable=True)

    def epoch():
        model.train()
        optimizer.zero_grad()
        loss = loss_of_step(model, labels)
        loss.backward()
        optimizer.step()
        return loss

    if hip_graph:
        graph, _ = capture_training_step(model, labels, optimizer)
        epoch = graph.replay
    if not verbose:
        epoch()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    steps = range(num_epoches)
    if progress:
        from tqdm import tqdm

        steps = tqdm(steps)
    for _ in steps:
        epoch()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / num_epoches
    print("training time per epoch: {:.3f} (ms)".format(ms))
    return ms


def load_graph(net, path=None, mtx_name=None, synthetic=None, verbose=True, reorder=None):
    """The per-network loader choices of GNN.py:189-195."""
    graph = graph_input(mtx_name=mtx_name if synthetic is None else synthetic, path=path)
    graph.verbose = verbose
    if synthetic is not None:
        from . import synth

        if net == "GIN":
            # GIN_epsilon=0.5 on a symmetric pattern: off-diagonal 1, diagonal 1.5 (graph_input.py:381-390)
            r, c, n = _synthetic_edges(synthetic)
            rowPtr, colIdx, val = synth.to_unit_csr(r, c, n, self_loops=True)
            val[colIdx == _row_of(rowPtr)] = 1.5
        else:
            rowPtr, colIdx, val, n = synth.config_graph(synthetic)
        graph.load_from_csr(rowPtr, colIdx, val, if_mask=(net == "AGNN"), reorder=reorder)
    elif net == "GIN":
        graph.load(load_from_mtx=True, GIN_epsilon=0.5)
    elif net == "AGNN":
        graph.load(load_from_mtx=True, is_normalize=True, if_mask=True)
    else:
        graph.load(load_from_mtx=True, is_normalize=True)
    return graph


def _row_of(rowPtr):
    import numpy as np

    return np.repeat(np.arange(rowPtr.size - 1, dtype=np.int32), np.diff(rowPtr))


def _synthetic_edges(name):
    from . import synth

    rowPtr, colIdx, _, n = synth.config_graph(name)
    rows = _row_of(rowPtr)
    keep = rows < colIdx
    return rows[keep].astype("int64"), colIdx[keep].astype("int64"), n


def build_model(net, graph, operators, hidden, num_features, num_classes, num_layers=5):
    """Feature / label initialisation and model construction of GNN.py:196-238."""
    device = torch.device("cuda")
    if net == "GCN":
        graph.init_feat_embedding(num_features)
        graph.init_labels(num_classes)
        return Net_5layers(num_classes, num_features, graph.x, operators, hidden).to(device)
    # AGNN and GIN run on inputs padded to an even number of rows so that 2x1 blocks fit (GNN.py:226-238)
    graph.init_feat_embedding(num_features, 2)
    graph.init_labels(num_classes, 2)
    if net == "AGNN":
        colIdx = graph.csr_data.colIdx.to(device).unsqueeze(-1)
        return AGNN(num_classes, num_features, graph.x, operators, hidden, colIdx, num_layers).to(device)
    return GIN(num_classes, num_features, graph.x, operators, hidden).to(device)


# Windowed layout: tried when at least this share of the entries is local.  Over the 771 matrices of the decider's corpus
# the matrices on which the layout beats the best swept configuration (large banded matrices, community-ordered block
# models: by 16-34 % on average, up to 78 %) have local shares from 0.6 up, nearly all of them above 0.8; trying costs a
# few launches, and the faster operator is kept.
WINDOW_MIN_LOCAL_SHARE = 0.6


def _try_window(graph, dim, op):
    """The windowed layout against ``op`` on this matrix (an addition of this build): when at least
    WINDOW_MIN_LOCAL_SHARE of the entries have their column within the row's window, both are timed (a few launches each, after a cache fill, as
    inside an epoch) and the faster one is returned.  The class space of the forests has no such representation, so
    the choice is made by this measurement instead of by the decider."""
    if dim % 4 or graph.csr_data.val.dim() != 1:
        return op
    cand = pcsr_spmm(graph=graph, vec_size=1, if_split=False, CF=0, window=True)
    if cand.window_local_share < WINDOW_MIN_LOCAL_SHARE:
        return op
    X = torch.randn((graph.mtx_nodes + 1) // 2 * 2, dim, device="cuda")
    ms_op = op.time_ms(X, warmup=2, iters=5, flush_bytes=256 << 20)
    ms_w = cand.time_ms(X, warmup=2, iters=5, flush_bytes=256 << 20)
    return cand if ms_w < ms_op else op


def configure_operators(decider, graph, dims, override=None, try_candidates=0, try_window=True):
    """One pcsr_spmm per layer width, configured by the decider (GNN.py:200-209) or by ``override`` =
    (if_split, vec_size, CF, blkWarpNum).  ``try_candidates`` = k > 1 (an addition of this build): the k configurations
    the forest rates highest are timed on this matrix (a few launches each, after a cache fill, as inside an epoch) and
    the fastest is kept.  ``try_window``: see _try_window (not with ``override``)."""
    ops = {}
    for dim in dims:
        if override is not None or try_candidates <= 1:
            if_split, vec_size, CF, blkWarpNum = override if override is not None else decider.config_PCSR(graph, dim)
            ops[dim] = pcsr_spmm(graph=graph, vec_size=vec_size, if_split=if_split, CF=CF, blkWarpNum=blkWarpNum)
            if override is None and try_window:
                ops[dim] = _try_window(graph, dim, ops[dim])
            continue
        X = torch.randn((graph.mtx_nodes + 1) // 2 * 2, dim, device="cuda")  # an even row count serves the 2x1 block formats too
        best = None
        for if_split, vec_size, CF, blkWarpNum in decider.candidates_PCSR(graph, dim, try_candidates):
            op = pcsr_spmm(graph=graph, vec_size=vec_size, if_split=if_split, CF=CF, blkWarpNum=blkWarpNum)
            ms = op.time_ms(X, warmup=2, iters=5, flush_bytes=256 << 20)
            if best is None or ms < best[0]:
                best = (ms, op)
        ops[dim] = _try_window(graph, dim, best[1]) if try_window else best[1]
    return ops


def main(argv=None):
    p = argparse.ArgumentParser()
    p.add_argument("--verbose", type=str, choices=["True", "False"], default="False")
    p.add_argument("--hidden_list", nargs="*", type=int, default=[32], help="hidden size list")
    p.add_argument("--num_classes", type=int, default=32)
    p.add_argument("--num_features", type=int, default=32)
    p.add_argument("--num_epoches", type=int, default=200)
    p.add_argument("--num_layers", type=int, default=5)
    p.add_argument("--path", type=str, default="./dataset/")
    p.add_argument("--pickle_path", type=str, default=DEFAULT_PICKLE_PATH)
    p.add_argument("--mtx_name", type=str, default="")
    p.add_argument("--net", type=str, choices=["GCN", "GIN", "AGNN"], default="AGNN")
    p.add_argument("--synthetic", type=str, default=None, help="C1, C2, C3, C3s, C5 or C5p instead of a .mtx file")
    p.add_argument("--hip_graph", action="store_true",
                   help="record the training step in a HIP graph and replay it per epoch (an addition of this build)")
    p.add_argument("--reorder", choices=["community", "degree"], default=None,
                   help="synthetic graphs: permute rows and columns together at load time (reorder.py); features and labels "
                        "are generated in the new order")
    p.add_argument("--no_aggregate_first", action="store_true",
                   help="GCN: always A (H W), also for the first layer when it widens its input (the reference's order)")
    p.add_argument("--no_fuse_loss", action="store_true",
                   help="run the networks' log-softmax and the loss as operators of their own, as the reference's driver does")
    p.add_argument("--no_fuse_relu", action="store_true",
                   help="apply the ReLU between the layers as passes of their own, as the reference's driver does")
    p.add_argument("--try_candidates", type=int, default=0, metavar="K",
                   help="time the K configurations the decider rates highest on the matrix and keep the fastest")
    p.add_argument("--no_window", action="store_true",
                   help="never replace the decider's operator by the windowed layout (tried when at least three fifths of the "
                        "entries lie near the diagonal)")
    p.add_argument("--config", nargs=4, type=int, default=None, metavar=("IF_SPLIT", "VEC", "CF", "BW"),
                   help="skip the decider and use this configuration for every layer width")
    args = p.parse_args(argv)
    print(args)
    assert torch.cuda.is_available()

    if args.synthetic is not None:
        names = [args.synthetic]
    elif args.mtx_name:
        names = [args.mtx_name]
    else:
        names = sorted(os.path.basename(f)[:-4] for f in glob.glob(os.path.join(args.path, "*.mtx")))

    decider = None
    if args.config is None:
        decider = SpMMDecider(args.pickle_path)
        decider.gen_model_dict([16, 32, 48, 64, 80, 96, 112, 128])

    results = {}
    for hidden in args.hidden_list:
        for name in names:
            print("-------------mtx: {} hidden_size: {}-------------".format(name, hidden))
            t0 = time.perf_counter()
            graph = load_graph(args.net, args.path, name, args.synthetic, reorder=args.reorder)
            t1 = time.perf_counter()
            dims = [hidden, args.num_classes]
            if (args.net == "GCN" and not args.no_aggregate_first and args.num_features < hidden
                    and (decider is None or args.num_features in decider.model_dict)):
                dims.append(args.num_features)  # the first layer runs its sparse product at the features' width
            if args.net == "GIN" and args.num_features not in dims and (decider is None or args.num_features in decider.model_dict):
                dims.append(args.num_features)  # GIN aggregates its input: the first layer's product has the features' width
            ops = configure_operators(decider, graph, dims, None if args.config is None else tuple(args.config),
                                      try_candidates=args.try_candidates, try_window=not args.no_window)
            print("SpMM-decider config time: {:.3f} (ms)".format((time.perf_counter() - t1) * 1e3))
            model = build_model(args.net, graph, ops, hidden, args.num_features, args.num_classes, args.num_layers)
            if args.no_fuse_loss:
                model.fuse_loss = False
            if args.no_fuse_relu and hasattr(model, "fuse_relu"):
                model.fuse_relu = False
            torch.cuda.synchronize()
            results[(name, hidden)] = train_profiling(model, graph.y, args.num_epoches, verbose=args.verbose == "True",
                                                     hip_graph=args.hip_graph)
            print("end2end time: {:.3f} (ms)".format((time.perf_counter() - t0) * 1e3))
    return results


if __name__ == "__main__":
    main()
