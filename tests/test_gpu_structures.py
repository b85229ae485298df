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
    # block-rows long enough for the device builder's workgroup path: both rows long, only the odd one, only the even one
    long_rows = {10: 5000, 11: 4000, 4000: 3, 4001: 3000, 2000: 2500, 2001: 0, 5999: 2100}
    yield "long block-rows", [long_rows.get(i, int(d)) for i, d in enumerate(rng.poisson(1.5, 6000))]


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


@pytest.mark.parametrize("name,deg", CASES, ids=[c[0] for c in CASES])
def test_device_builders_structures(oracle, name, deg):
    """row split and 2x1 blocks built on the device: bit for bit the oracle's arrays"""
    from paramspmm_ae_amd import device_builder
    from gpu_util import dev

    rowPtr, colIdx, val = from_degrees(deg, len(deg) + 2)
    for g in (1, 7, 32, 1000):
        rs, tr = device_builder.split_csr_device(dev(rowPtr), g)
        want_rs, want_tr = oracle.split_csr(rowPtr, g)
        assert np.array_equal(rs.cpu().numpy(), want_rs) and np.array_equal(tr.cpu().numpy(), want_tr), (name, g)
    got = device_builder.build_bcsr_device(dev(rowPtr), dev(colIdx), dev(val))
    for a, b in zip(got, oracle.bcsr_build(rowPtr, colIdx, val)):
        a = a.cpu().numpy()
        assert np.array_equal(a, np.asarray(b).reshape(a.shape)), name


@pytest.mark.parametrize("name,deg", CASES, ids=[c[0] for c in CASES])
def test_fused_attention_structures(oracle, name, deg):
    """scaled SDDMM with row maxima -> softmax-weighted SpMM on both CSR layouts against the oracle's three steps"""
    from paramspmm_ae_amd import _capi
    from gpu_util import Formats, assert_close, dev, stream

    rowPtr, colIdx, val = from_degrees(deg, len(deg) + 3)
    if colIdx.size == 0:
        pytest.skip("no stored entries: nothing to weight")
    n, K, N = rowPtr.size - 1, 16, 32
    rng = np.random.default_rng(n)
    A = (rng.standard_normal((n, K)) / 2).astype(np.float32)
    H = rng.standard_normal((n, N)).astype(np.float32)
    e_want = oracle.sddmm_csr(rowPtr, colIdx, A, A) * val
    w_want = oracle.segment_softmax(rowPtr, e_want)
    y_want = oracle.spmm_csr(rowPtr, colIdx, w_want, H)
    scale = oracle.spmm_csr(rowPtr, colIdx, w_want, np.abs(H))
    e_scale = oracle.sddmm_csr(rowPtr, colIdx, np.abs(A), np.abs(A)) * np.abs(val)
    L, p = _capi.lib, _capi.ptr
    Ad, Hd = dev(A), dev(H)
    for g in (8, 64):
        F = Formats(oracle, rowPtr, colIdx, val, g=g, gb=g)
        d = F.d
        for split in (False, True):
            e = torch.full((F.nnz,), float("nan"), device="cuda")
            m = torch.full((n,), float("nan"), device="cuda")
            Y = torch.full((n, N), float("nan"), device="cuda")
            if split:
                row_sum = torch.full((n,), float("nan"), device="cuda")
                _capi.check(L.psp_sddmm_csr_split_rowmax_f32(p(d["rps"]), p(d["colIdx"]), p(d["tr"]), p(Ad), p(Ad), p(d["val"]),
                                                             p(e), p(m), F.tr.size, n, K, 4, stream()))
                _capi.check(L.psp_spmm_csr_split_softmax_f32(p(d["rps"]), p(d["colIdx"]), p(e), p(d["tr"]), p(m), p(row_sum),
                                                             p(Hd), p(Y), F.tr.size, N, n, 1, 4, stream()))
            else:
                _capi.check(L.psp_sddmm_csr_rowmax_f32(p(d["rowPtr"]), p(d["colIdx"]), p(Ad), p(Ad), p(d["val"]), p(e), p(m),
                                                       n, K, 8, stream()))
                _capi.check(L.psp_spmm_csr_softmax_f32(p(d["rowPtr"]), p(d["colIdx"]), p(e), p(m), p(Hd), p(Y), n, N, n, 1, 8,
                                                       stream()))
            torch.cuda.synchronize()
            what = "%s g=%d split=%s" % (name, g, split)
            assert_close(e, e_want, rtol=1e-5, atol=1e-6, what=what + " scores", scale=e_scale)
            assert_close(Y, y_want, rtol=1e-4, atol=1e-5, what=what + " product", scale=scale)
