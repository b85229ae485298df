"""SpMM checker with the surface of the reference's verification.py:10-102: the expected result is
``torch.sparse.mm`` of the CSR matrix with X = ones, compared at relative 1e-4."""
import time

import torch


class SpMM_verification(object):
    def __init__(self, dim, rowPtr, colIdx, val, baseline=False, baseline_round=100):
        self.baseline = baseline
        self.baseline_round = baseline_round
        self.rowPtr, self.colIdx, self.csr_val = rowPtr, colIdx, val
        self.num_nodes = len(rowPtr) - 1
        self.s = torch.sparse_csr_tensor(rowPtr, colIdx, val, size=(self.num_nodes, self.num_nodes))
        self.test_embedding = dim
        self.X = torch.ones(self.num_nodes, dim)
        self.result_ref = None
        self.result = None

    def reference(self, dim=None, device="cuda", verbose=True):
        assert device in ("cpu", "cuda")
        if verbose:
            print("# Reference result on " + ("CPU" if device == "cpu" else "GPU"))
        X = self.X.to(device) if dim is None else torch.ones(self.num_nodes, dim, device=device)
        self.result_ref = torch.sparse.mm(self.s.to(device), X).to("cpu")

    def torch_compute(self, device):
        """torch.sparse.mm on ``device``; with ``baseline`` also timed -> (result, int GFLOP/s)."""
        assert device in ("cpu", "cuda")
        X, s = self.X.to(device), self.s.to(device)
        self.result = torch.sparse.mm(s, X)
        if not self.baseline:
            return self.result
        for _ in range(10):
            self.result = torch.sparse.mm(s, X)
        if device == "cuda":
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(self.baseline_round):
            self.result = torch.sparse.mm(s, X)
        if device == "cuda":
            torch.cuda.synchronize()
        dur = (time.perf_counter() - t0) / self.baseline_round
        gflop = 2 * int(self.rowPtr[-1]) / 1e9 * self.test_embedding
        print("dim: {} torch SpMM (ms): {:.3f} gflops: {:.0f}".format(self.test_embedding, dur * 1e3, gflop / dur))
        return self.result, int(gflop / dur)

    def compare(self, result, mtx_name, verbose=True):
        if self.result_ref is None or result is None:
            raise ValueError("MUST compute result and result reference (CPU) first!!")
        bad = torch.abs(self.result_ref - result) > 1e-4 * torch.abs(self.result_ref)
        if not bad.any():
            if verbose:
                print("# Verification PASSED")
            return
        print("# Verification FAILED in {}".format(mtx_name))
        for row, col in torch.nonzero(bad)[:20].tolist():
            print("Mismatch at position ({}, {}): Expected {}, Found {}".format(
                row, col, self.result_ref[row, col].item(), result[row, col].item()))
        raise ValueError("Verification FAILED in {}".format(mtx_name))


def main(argv=None):
    """torch.sparse.mm on the CPU and on the GPU for every matrix of a directory (verification.py:105-128)."""
    import argparse
    import glob
    import os

    from .graph_input import graph_input

    parser = argparse.ArgumentParser()
    parser.add_argument("--path", type=str, default="./artifact_dataset/all-mtx/rabbit/", help="path to the mtx files")
    parser.add_argument("--dim", type=int, default=32)
    args = parser.parse_args(argv)
    out = {}
    for name in sorted(os.path.basename(f)[:-4] for f in glob.glob(os.path.join(args.path, "*.mtx"))):
        print("-------------{}-------------".format(name))
        graph = graph_input(mtx_name=name, path=args.path)
        graph.load(load_from_mtx=True)
        c = graph.csr_data
        check = SpMM_verification(args.dim, c.rowPtr, c.colIdx, c.val, baseline=True)
        check.reference()
        _, cpu = check.torch_compute("cpu")
        got, gpu = check.torch_compute("cuda")
        check.compare(got.to("cpu"), name)
        out[name] = (cpu, gpu)
        print("=======================================")
    return out


if __name__ == "__main__":
    main()
