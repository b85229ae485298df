"""SpMM and SDDMM over a range of matrix structures (row-length patterns around the kernels' group, chunk and
wavefront sizes, hubs, empty stretches, tiny matrices), all four layouts and several granularities, against the CPU
oracle through the C ABI.  The widths are few; the structures are the point."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

FMTS = ["csr", "csr_split", "bcsr", "bcsr_split"]


def from_degrees(deg, seed):
    """square CSR with the given row lengths, sorted duplicate-free columns, uniform values"""
    rng = np.random.default_rng(seed)
    n = len(deg)
    deg = np.minimum(np.asarray(deg, dtype=np.int64), n)
    rowPtr = np.zeros(n + 1, np.int32)
    rowPtr[1:] = np.cumsum(deg)
    cols = [np.sort(rng.choice(n, d, replace=False)) for d in deg]
    colIdx = (np.concatenate(cols) if rowPtr[-1] else np.zeros(0)).astype(np.int32)
    return rowPtr, colIdx, rng.uniform(0.1, 1.0, colIdx.size).astype(np.float32)


def structures():
    rng = np.random.default_rng(2024)
    yield "one row, one entry", [1]
    yield "one empty row", [0]
    yield "two rows", [2, 1]
    yield "65 rows of one entry", [1] * 65
    yield "lengths cycle 0..69", [i % 70 for i in range(300)]
    yield "every row 64 long", [64] * 129
    yield "every row 33 long", [33] * 200
    yield "mostly empty", rng.poisson(0.3, 2050)
    yield "dense-ish", rng.poisson(100, 513)
    yield "three hubs among short rows", [900 if i in (0, 511, 999) else int(d) for i, d in enumerate(rng.poisson(2, 1000))]
    yield "hub last", list(rng.poisson(5, 700)) + [700]
    yield "empty stretch then full", [0] * 500 + [40] * 100 + [0] * 300 + [1] * 124
    yield "alternating 0 / 130", [0 if i % 2 else 130 for i in range(400)]
    yield "lengths around 32", [31, 32, 33] * 150
    yield "geometric", [min(1 << (i % 11), 1000) for i in range(1100)]


CASES = list(structures())


@pytest.mark.parametrize("name,deg", CASES, ids=[c[0] for c in CASES])
def test_spmm_structures(oracle, name, deg):
    from gpu_util import Formats, spmm_capi, spmm_oracle, spmm_abs_scale, assert_close

    rowPtr, colIdx, val = from_degrees(deg, len(deg))
    for g in (None, 8, 64):
        F = Formats(oracle, rowPtr, colIdx, val, g=g, gb=g)
        for N, CF in ((16, 1), (20, 1), (64, 2), (128, 1)):
            X = np.random.default_rng(N).standard_normal((F.n + (F.n & 1), N)).astype(np.float32)
            Xd = torch.from_numpy(X).cuda()
            scale = None
            for fmt in FMTS:
                want = spmm_oracle(oracle, fmt, F, X)
                if scale is None or scale.shape != want.shape:
                    scale = spmm_abs_scale(oracle, F, X, want.shape[0])
                for bw in (4, 8):
                    got = spmm_capi(fmt, F, Xd, CF, bw)
                    torch.cuda.synchronize()
                    assert_close(got, want, what="%s: %s g=%s N=%d bw=%d" % (name, fmt, g, N, bw), scale=scale)
        if colIdx.size == 0:
            break  # the granularity of a matrix without entries changes nothing


@pytest.mark.parametrize("name,deg", CASES, ids=[c[0] for c in CASES])
def test_sddmm_structures(oracle, name, deg):
    from gpu_util import Formats, sddmm_capi, sddmm_oracle, assert_close

    rowPtr, colIdx, val = from_degrees(deg, len(deg) + 1)
    for g in (None, 8, 64):
        F = Formats(oracle, rowPtr, colIdx, val, g=g, gb=g)
        for K in (16, 24, 32, 64, 128):
            rng = np.random.default_rng(K)
            A = rng.standard_normal((F.n + (F.n & 1), K)).astype(np.float32) / np.sqrt(K).astype(np.float32)
            B = rng.standard_normal((F.n + (F.n & 1), K)).astype(np.float32) / np.sqrt(K).astype(np.float32)
            Ad, Bd = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
            for fmt in FMTS:
                want = sddmm_oracle(oracle, fmt, F, A, B)
                for bw in (4, 8):
                    got = sddmm_capi(fmt, F, Ad, Bd, bw)
                    torch.cuda.synchronize()
                    assert_close(got, want, rtol=1e-5, atol=2e-6, what="%s: %s g=%s K=%d bw=%d" % (name, fmt, g, K, bw))
        if colIdx.size == 0:
            break
