"""Writes tests/golden/pubmed_pattern.npz from the reference's only data files,
toy_dataset/pubmed.mtx and toy_dataset/rabbit/pubmed_rabbit.mtx (MatrixMarket, symmetric pattern of the PubMed
citation graph, original and Rabbit-reordered).  The fixture holds the stored (row, col) pairs of both files,
0-based, exactly as listed in the files (one triangle); tests mirror them to get the symmetric matrix the
reference's loader sees after scipy.io.mmread.

Run once in the container that mounts the reference:  python tests/golden/make_pubmed_fixture.py
"""
import os

import numpy as np

REF = "/root/reference/toy_dataset"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "pubmed_pattern.npz")


def read_pairs(path):
    with open(path) as f:
        header = f.readline().lower()
        assert "coordinate" in header and "symmetric" in header, header
        line = f.readline()
        while line.startswith("%"):
            line = f.readline()
        nrows, ncols, nstored = (int(t) for t in line.split()[:3])
        body = np.loadtxt(f, dtype=np.int64, usecols=(0, 1))
    assert body.shape[0] == nstored and nrows == ncols
    return nrows, (body[:, 0] - 1).astype(np.int32), (body[:, 1] - 1).astype(np.int32)


if __name__ == "__main__":
    n0, r0, c0 = read_pairs(os.path.join(REF, "pubmed.mtx"))
    n1, r1, c1 = read_pairs(os.path.join(REF, "rabbit", "pubmed_rabbit.mtx"))
    assert n0 == n1
    np.savez_compressed(OUT, n=np.int64(n0), orig_row=r0, orig_col=c0, rabbit_row=r1, rabbit_col=c1)
    print("wrote", OUT, os.path.getsize(OUT), "bytes;", n0, "nodes;", r0.size, "/", r1.size, "stored entries")
