"""Windowed CSR (psp_window_build / psp_spmm_window_f32): the format builders against a numpy restatement, bit for bit
(index work), and the SpMM against the CPU oracle's CSR product within rel 1e-5 / abs 1e-6 (the kernel adds a row's
local entries before its remote ones, so it is not bit-identical to the sequential chain), through the C ABI, the
extension modules and the GNN layers."""
import ctypes

import numpy as np
import pytest
import torch

from conftest import random_csr

BLOCK, HALO = 64, 88


def banded_csr(n, per_row, width, seed, far=0.0, hub=None, empty_frac=0.0):
    """Rows with ``per_row`` (Poisson) entries within +-width of the diagonal, a share ``far`` of them anywhere."""
    rng = np.random.default_rng(seed)
    deg = rng.poisson(per_row, n)
    if empty_frac:
        deg[rng.random(n) < empty_frac] = 0
    if hub is not None:
        deg[hub[0]] = hub[1]
    cols = []
    for i, d in enumerate(deg):
        near = np.clip(i + rng.integers(-width, width + 1, d), 0, n - 1)
        anywhere = rng.integers(0, n, d)
        c = np.unique(np.where(rng.random(d) < far, anywhere, near))
        cols.append(c)
    rowPtr = np.zeros(n + 1, np.int32)
    rowPtr[1:] = np.cumsum([c.size for c in cols])
    colIdx = (np.concatenate(cols) if rowPtr[-1] else np.zeros(0)).astype(np.int32)
    val = rng.uniform(0.1, 1.0, colIdx.size).astype(np.float32)
    return rowPtr, colIdx, val


def window_reference(rowPtr, colIdx, val):
    """numpy restatement of the format: per row the entries whose column lies in [64 (r // 64) - 64, 64 (r // 64) + 128)
    first, the others after, each part in the original order."""
    M = rowPtr.size - 1
    rows = np.repeat(np.arange(M, dtype=np.int64), np.diff(rowPtr))
    lo = rows // BLOCK * BLOCK - HALO
    local = (colIdx >= lo) & (colIdx < lo + BLOCK + 2 * HALO) & (colIdx < M)  # columns past the last row are never local
    order = np.lexsort((np.arange(colIdx.size), ~local, rows))  # stable: row, then local first, then position
    rp = np.empty(2 * M + 2, np.int32)
    rp[0:2 * M:2] = rowPtr[:-1]
    cs = np.concatenate([[0], np.cumsum(local)])
    rp[1:2 * M:2] = rowPtr[:-1] + (cs[rowPtr[1:]] - cs[rowPtr[:-1]])  # start of the remote part
    rp[2 * M] = rp[2 * M + 1] = rowPtr[-1]
    return rp, colIdx[order], val[order], float(local.mean()) if colIdx.size else 0.0


CASES = {
    "banded": lambda: banded_csr(5000, 14, 40, 1, far=0.1, empty_frac=0.05),
    "banded_hub": lambda: banded_csr(3001, 9, 30, 2, far=0.15, hub=(70, 900)),
    "wide_band": lambda: banded_csr(2000, 60, 60, 3, far=0.02),       # rows with more than 32 local entries
    "random": lambda: random_csr(4099, 11, 4, empty_frac=0.1, hub=(5, 700), values="uniform"),  # nearly all remote
    "tiny": lambda: banded_csr(37, 3, 5, 5),
    "one_block": lambda: banded_csr(64, 6, 64, 6),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_host_builder_matches_the_numpy_restatement(name):
    from paramspmm_ae_amd import _capi

    rowPtr, colIdx, val = CASES[name]()
    M, nnz = rowPtr.size - 1, colIdx.size
    rp, ci, v = np.full(2 * M + 2, -7, np.int32), np.full(nnz, -7, np.int32), np.full(nnz, np.nan, np.float32)
    p = _capi.ptr
    _capi.check(_capi.lib.psp_window_build(p(rowPtr), p(colIdx), p(val), M, p(rp), p(ci), p(v)))
    want = window_reference(rowPtr, colIdx, val)
    assert np.array_equal(rp, want[0]) and np.array_equal(ci, want[1]) and np.array_equal(v, want[2])
    # the permutation stays inside the rows
    for r in range(0, M, max(1, M // 50)):
        a, b = rowPtr[r], rowPtr[r + 1]
        assert sorted(ci[a:b].tolist()) == sorted(colIdx[a:b].tolist())


def test_host_builder_rejects_a_broken_row_pointer():
    from paramspmm_ae_amd import _capi

    p = _capi.ptr
    rowPtr = np.array([0, 3, 2, 4], np.int32)
    z = np.zeros(8, np.int32)
    f = np.zeros(8, np.float32)
    assert _capi.lib.psp_window_build(p(rowPtr), p(z), p(f), 3, p(np.zeros(8, np.int32)), p(z.copy()), p(f.copy())) == -1
    a, b, c = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    assert _capi.lib.psp_spmm_window_plan(18, 0, a, b, c) == -1      # width not a multiple of 4
    assert _capi.lib.psp_spmm_window_plan(64, 4, a, b, c) == -1      # no such variant
    assert [_capi.lib.psp_spmm_window_plan(n, 0, a, b, c) for n in (4, 16, 20, 32, 36, 256)] == [1, 1, 2, 2, 3, 3]


def _spmm_window(F, X, variant=0, relu=False, mask=None, rows_out=None):
    from paramspmm_ae_amd import _capi

    rp, ci, v, M = F
    rows_out = X.shape[0] if rows_out is None else rows_out
    Y = torch.full((rows_out, X.shape[1]), float("nan"), device="cuda")
    p = _capi.ptr
    _capi.check(_capi.lib.psp_spmm_window_f32(p(rp), p(ci), p(v), p(X), p(Y), M, int(ci.numel()), X.shape[1], rows_out, variant, int(relu),
                                              p(mask), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return Y


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_device_builder_and_spmm_against_the_oracle(oracle, name):
    from gpu_util import assert_close, dev
    from paramspmm_ae_amd import _capi

    rowPtr, colIdx, val = CASES[name]()
    M, nnz = rowPtr.size - 1, colIdx.size
    want_fmt = window_reference(rowPtr, colIdx, val)
    rp = torch.full((2 * M + 2,), -7, dtype=torch.int32, device="cuda")
    ci = torch.full((max(nnz, 1),), -7, dtype=torch.int32, device="cuda")[:nnz]
    v = torch.full((max(nnz, 1),), float("nan"), device="cuda")[:nnz]
    p = _capi.ptr
    print("case build", name, M, nnz, flush=True)
    rp_in, ci_in, v_in = dev(rowPtr), dev(colIdx), dev(val)  # named: the arrays must outlive the launch that reads them
    _capi.check(_capi.lib.psp_window_build_dev(p(rp_in), p(ci_in), p(v_in), M, p(rp), p(ci), p(v),
                                               torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert np.array_equal(rp.cpu().numpy(), want_fmt[0])
    assert np.array_equal(ci.cpu().numpy(), want_fmt[1]) and np.array_equal(v.cpu().numpy(), want_fmt[2])
    F = (rp, ci, v, M)
    for N in (4, 16, 20, 32, 48, 64, 100, 128, 256):
        X = np.random.default_rng(N).standard_normal((M + 3, N)).astype(np.float32)
        want = oracle.spmm_csr(rowPtr, colIdx, val, X, rows_out=M + 3)
        scale = oracle.spmm_csr(rowPtr, colIdx, np.abs(val), np.abs(X), rows_out=M + 3)
        Xd = torch.from_numpy(X).cuda()
        for variant in (0, 1, 2, 3):
            print("case spmm", name, N, variant, flush=True)
            got = _spmm_window(F, Xd, variant)
            assert_close(got, want, what="%s N=%d variant %d" % (name, N, variant), scale=scale)
            assert bool((got[M:] == 0).all())
    # the folded activation and mask: A max(X, 0) equals the product of the clamped input bit for bit; the masked
    # product equals the plain one where the mask is positive and is an exact zero elsewhere
    X = torch.randn(M + 1, 64, device="cuda")
    mask = torch.randn(M + 1, 64, device="cuda")
    plain = _spmm_window(F, X)
    assert torch.equal(_spmm_window(F, X, relu=True), _spmm_window(F, torch.relu(X)))
    got = _spmm_window(F, X, mask=mask)
    assert torch.equal(got, torch.where(mask > 0, plain, torch.zeros_like(plain)))


def shaped_csr(M, seed):
    """Rows whose numbers of local and remote entries run through every count the kernels treat differently: 0 .. 40
    local entries (32 are fetched up front, the rest in a loop) and 0 .. 10 remote ones (4 prefetched, 4 more in a
    second round for lane groups of 8, the rest in a loop), in all combinations that fit the row count."""
    rng = np.random.default_rng(seed)
    cols = []
    for r in range(M):
        n_local, n_remote = r % 41, (r // 3) % 11
        lo = r // BLOCK * BLOCK - HALO
        window = np.arange(max(lo, 0), min(lo + BLOCK + 2 * HALO, M))
        outside = np.setdiff1d(np.arange(M), window)
        c = np.concatenate([rng.choice(window, min(n_local, window.size), replace=False),
                            rng.choice(outside, min(n_remote, outside.size), replace=False)])
        cols.append(np.sort(c))
    rowPtr = np.zeros(M + 1, np.int32)
    rowPtr[1:] = np.cumsum([c.size for c in cols])
    colIdx = (np.concatenate(cols) if rowPtr[-1] else np.zeros(0)).astype(np.int32)
    val = rng.uniform(-1.0, 1.0, colIdx.size).astype(np.float32)
    return rowPtr, colIdx, val


@pytest.mark.gpu
@pytest.mark.parametrize("M", [1, 63, 64, 65, 129, 500, 1500])
def test_every_row_shape_through_every_windowed_kernel(oracle, M):
    """SpMM (three variants, with the dense product folded in where it exists), SDDMM and the attention passes on rows
    of every local / remote count (shaped_csr), at row counts around the 64-row blocks, against the oracle."""
    from gpu_util import assert_close, dev
    from paramspmm_ae_amd import _capi
    import ParamSpMM

    rowPtr, colIdx, val = shaped_csr(M, M)
    nnz = colIdx.size
    rp, ci, v = ParamSpMM.window_build(dev(rowPtr), dev(colIdx), dev(val))
    want_fmt = window_reference(rowPtr, colIdx, val)
    assert np.array_equal(rp.cpu().numpy(), want_fmt[0]) and np.array_equal(ci.cpu().numpy(), want_fmt[1])
    ci_w, v_w = ci.cpu().numpy(), v.cpu().numpy()
    rows = np.repeat(np.arange(M), np.diff(rowPtr))
    p, L = _capi.ptr, _capi.lib
    st = torch.cuda.current_stream().cuda_stream
    for N in (16, 32, 64, 128):
        print("case shapes", M, N, flush=True)
        rng = np.random.default_rng(N)
        X = rng.standard_normal((M, N)).astype(np.float32)
        Xd = torch.from_numpy(X).cuda()
        want = oracle.spmm_csr(rowPtr, colIdx, val, X)
        scale = oracle.spmm_csr(rowPtr, colIdx, np.abs(val), np.abs(X))
        for variant in (0, 1, 2, 3):
            assert_close(_spmm_window((rp, ci, v, M), Xd, variant), want, what="spmm N=%d variant %d" % (N, variant), scale=scale)
        if N <= 32:
            W = (rng.standard_normal((N, N)) / np.sqrt(N)).astype(np.float32)
            Y, R = torch.empty(M, N, device="cuda"), torch.empty(M, N, device="cuda")
            _capi.check(L.psp_spmm_window_xw_f32(p(rp), p(ci), p(v), p(Xd), p(torch.from_numpy(W).cuda()), 0, p(Y), p(R), M, nnz, N, M, 0,
                                                 None, st))
            assert_close(R, want, what="raw product beside the folded one", scale=scale)
            assert_close(Y, want.astype(np.float64) @ W.astype(np.float64), what="folded dense product",
                         scale=scale.astype(np.float64) @ np.abs(W).astype(np.float64))
        out = torch.full((max(nnz, 1),), float("nan"), device="cuda")[:nnz]
        _capi.check(L.psp_sddmm_window_f32(p(rp), p(ci), p(Xd), p(Xd), None, p(out), M, nnz, N, M, st))
        e_scale = (np.abs(X[rows]) * np.abs(X[ci_w])).sum(1)
        assert_close(out, oracle.sddmm_csr(rowPtr, ci_w, X, X), what="sddmm K=%d" % N, scale=e_scale)
        if N <= 64:
            att = torch.full((max(nnz, 1),), float("nan"), device="cuda")[:nnz]
            Y = torch.full((M, N), float("nan"), device="cuda")
            _capi.check(L.psp_attn_window_forward_f32(p(rp), p(ci), p(Xd), None, p(att), p(Y), M, nnz, N, M, st))
            e = oracle.sddmm_csr(rowPtr, ci_w, X, X)
            assert_close(att, e, what="attention scores K=%d" % N, scale=e_scale)
            assert_close(Y, oracle.spmm_csr(rowPtr, ci_w, e, X), rtol=2e-5, what="attention aggregate K=%d" % N,
                         scale=oracle.spmm_csr(rowPtr, ci_w, e_scale.astype(np.float32), np.abs(X)))
            G = torch.full((M, N), float("nan"), device="cuda")
            wsum = torch.full((1,), float("nan"), device="cuda")
            _capi.check(L.psp_attn_window_backward_f32(p(rp), p(ci), p(v), p(Xd), p(G), p(wsum), M, nnz, N, M, st))
            assert_close(G, oracle.spmm_csr(rowPtr, ci_w, v_w, X), what="attention backward aggregate K=%d" % N,
                         scale=oracle.spmm_csr(rowPtr, ci_w, np.abs(v_w), np.abs(X)))
            d = (X[rows].astype(np.float64) * X[ci_w].astype(np.float64)).sum(1)
            w_scale = float((e_scale.astype(np.float64) * ci_w).sum())
            assert abs(float(wsum.item()) - float((d * ci_w).sum())) <= 1e-6 + 2e-5 * w_scale


@pytest.mark.gpu
def test_a_matrix_with_more_columns_than_rows(oracle):
    """The first 1200 rows of a 1300-column banded matrix: columns past the last row are never local (the kernels stage
    rows 0 .. M - 1 of the dense operand), so the SpMM and the SDDMM reach them through the gathers; X and B have a row
    for every column."""
    from gpu_util import assert_close, dev
    from paramspmm_ae_amd import _capi
    import ParamSpMM

    rowPtr, colIdx, val = banded_csr(1300, 8, 40, 7, far=0.1)
    M, ncols = 1200, 1300
    rowPtr, colIdx, val = rowPtr[:M + 1].copy(), colIdx[:rowPtr[M]].copy(), val[:rowPtr[M]].copy()
    assert colIdx.max() >= M
    want_fmt = window_reference(rowPtr, colIdx, val)
    rp, ci, v = ParamSpMM.window_build(dev(rowPtr), dev(colIdx), dev(val))
    assert np.array_equal(rp.cpu().numpy(), want_fmt[0]) and np.array_equal(ci.cpu().numpy(), want_fmt[1])
    ci_w = ci.cpu().numpy()
    rows = np.repeat(np.arange(M), np.diff(rowPtr))
    p, L = _capi.ptr, _capi.lib
    st = torch.cuda.current_stream().cuda_stream
    for N in (16, 32, 64, 128):
        rng = np.random.default_rng(N)
        X = rng.standard_normal((ncols, N)).astype(np.float32)
        Xd = torch.from_numpy(X).cuda()
        Y = torch.full((M, N), float("nan"), device="cuda")
        _capi.check(L.psp_spmm_window_f32(p(rp), p(ci), p(v), p(Xd), p(Y), M, int(ci.numel()), N, M, 0, 0, None, st))
        want = oracle.spmm_csr(rowPtr, colIdx, val, X, rows_out=M)
        scale = oracle.spmm_csr(rowPtr, colIdx, np.abs(val), np.abs(X), rows_out=M)
        assert_close(Y, want, what="rectangular spmm N=%d" % N, scale=scale)
        A = rng.standard_normal((M, N)).astype(np.float32)
        Ad = torch.from_numpy(A).cuda()
        out = torch.full((colIdx.size,), float("nan"), device="cuda")
        _capi.check(L.psp_sddmm_window_f32(p(rp), p(ci), p(Ad), p(Xd), None, p(out), M, int(ci.numel()), N, ncols, st))
        assert_close(out, oracle.sddmm_csr(rowPtr, ci_w, A, X), what="rectangular sddmm K=%d" % N,
                     scale=(np.abs(A[rows]) * np.abs(X[ci_w])).sum(1))


@pytest.mark.gpu
def test_non_finite_inputs_stay_in_their_rows(oracle):
    rowPtr, colIdx, val = banded_csr(1500, 9, 30, 9, far=0.2, hub=(3, 400))
    from gpu_util import dev
    from paramspmm_ae_amd import _capi
    import ParamSpMM

    rp, ci, v = ParamSpMM.window_build(dev(rowPtr), dev(colIdx), dev(val))
    M = rowPtr.size - 1
    for N in (16, 64):
        X = np.random.default_rng(N).standard_normal((M, N)).astype(np.float32)
        X[colIdx[5]] = np.inf
        X[colIdx[colIdx.size // 2]] = np.nan
        X[0] = np.inf       # the row the padding of the index registers points at
        X[M - 1] = np.inf
        want = oracle.spmm_csr(rowPtr, colIdx, val, X)
        got = _spmm_window((rp, ci, v, M), torch.from_numpy(X).cuda()).cpu().numpy()
        assert np.array_equal(np.isnan(got), np.isnan(want)), N
        assert np.array_equal(np.isposinf(got), np.isposinf(want))
        fin = np.isfinite(want)
        np.testing.assert_allclose(got[fin], want[fin], rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_window_sddmm_against_the_oracle(oracle, name):
    """psp_sddmm_window_f32 against the oracle's CSR SDDMM on the layout's own arrays (rowPtr_w[0::2], colIdx_w is an
    ordinary matrix with unsorted rows): 1e-6 + 1e-5 of the magnitudes summed per entry; A = B = ones gives K exactly
    (the reference's known answer, SDDMM.py:127-128); alpha scales the result; with A == B the matrix is read once and
    the result is bit for bit the one of two separate copies."""
    from gpu_util import assert_close, dev
    from paramspmm_ae_amd import _capi
    import ParamSpMM

    rowPtr, colIdx, val = CASES[name]()
    M, nnz = rowPtr.size - 1, colIdx.size
    rp, ci, _ = ParamSpMM.window_build(dev(rowPtr), dev(colIdx), dev(val))
    ci_w = ci.cpu().numpy()
    rows = np.repeat(np.arange(M), np.diff(rowPtr))
    p, L = _capi.ptr, _capi.lib
    st = torch.cuda.current_stream().cuda_stream

    def run(A, B, K, alpha=None, rows_b=None):
        out = torch.full((nnz,), float("nan"), device="cuda")
        _capi.check(L.psp_sddmm_window_f32(p(rp), p(ci), p(A), p(B), p(alpha), p(out), M, nnz, K, B.shape[0] if rows_b is None else rows_b, st))
        torch.cuda.synchronize()
        return out

    for K in (4, 16, 20, 32, 48, 64, 100, 128):
        print("case sddmm", name, K, flush=True)
        rng = np.random.default_rng(K)
        A = rng.standard_normal((M + 2, K)).astype(np.float32)
        B = rng.standard_normal((M + 5, K)).astype(np.float32)
        want = oracle.sddmm_csr(rowPtr, ci_w, A, B)
        scale = (np.abs(A[rows]) * np.abs(B[ci_w])).sum(1)
        Ad, Bd = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
        got = run(Ad, Bd, K)
        assert_close(got, want, what="%s K=%d" % (name, K), scale=scale)
        alpha = torch.tensor([-0.75], device="cuda")
        assert torch.equal(run(Ad, Bd, K, alpha), got * -0.75)
        # one matrix on both sides: its rows come from the ring
        same = run(Bd, Bd, K)
        assert_close(same, oracle.sddmm_csr(rowPtr, ci_w, B, B), what="%s K=%d, A == B" % (name, K),
                     scale=(np.abs(B[rows]) * np.abs(B[ci_w])).sum(1))
        assert torch.equal(same, run(Bd.clone(), Bd, K))
        ones = torch.ones(M, K, device="cuda")
        assert bool((run(ones, ones, K) == K).all())
    # argument errors
    X = torch.zeros(M, 18, device="cuda")
    out = torch.zeros(max(nnz, 1), device="cuda")
    assert L.psp_sddmm_window_f32(p(rp), p(ci), p(X), p(X), None, p(out), M, nnz, 18, M, st) == -1
    assert L.psp_sddmm_window_f32(p(rp), p(ci), p(X), p(X), None, p(out), M, nnz, 132, M, st) == -1
    assert L.psp_sddmm_window_f32(p(rp), p(ci), p(X), p(X), None, p(out), M, nnz, 16, M - 1, st) == -1  # A == B, too few rows


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["banded", "banded_hub", "wide_band", "random", "tiny"])
def test_attention_passes_against_the_oracle(oracle, name):
    """psp_attn_window_forward_f32 / _backward_f32 against the oracle's SDDMM followed by its SpMM on the layout's own
    arrays: scores to 1e-6 + 1e-5 of the magnitudes summed per entry, the aggregated rows to twice that of the
    magnitudes summed per row (two chained roundings), the weight-gradient sum against float64."""
    from gpu_util import assert_close, dev
    from paramspmm_ae_amd import _capi
    import ParamSpMM

    rowPtr, colIdx, val = CASES[name]()
    M, nnz = rowPtr.size - 1, colIdx.size
    rp, ci, _ = ParamSpMM.window_build(dev(rowPtr), dev(colIdx), dev(val))
    ci_w = ci.cpu().numpy()
    rows = np.repeat(np.arange(M), np.diff(rowPtr))
    p, L = _capi.ptr, _capi.lib
    st = torch.cuda.current_stream().cuda_stream
    for K in (4, 16, 20, 32, 48, 64):
        print("case attn", name, K, flush=True)
        rng = np.random.default_rng(K)
        X = (rng.standard_normal((M + 3, K)) / np.sqrt(K)).astype(np.float32)
        alpha = np.float32(-1.25)
        e = oracle.sddmm_csr(rowPtr, ci_w, X, X)
        att_want = (e * alpha).astype(np.float32)
        e_scale = (np.abs(X[rows]) * np.abs(X[ci_w])).sum(1) * abs(alpha)
        Y_want = oracle.spmm_csr(rowPtr, ci_w, att_want, X, rows_out=M + 3)
        Y_scale = oracle.spmm_csr(rowPtr, ci_w, e_scale.astype(np.float32), np.abs(X), rows_out=M + 3)
        Xd = torch.from_numpy(X).cuda()
        att = torch.full((nnz,), float("nan"), device="cuda")
        Y = torch.full((M + 3, K), float("nan"), device="cuda")
        _capi.check(L.psp_attn_window_forward_f32(p(rp), p(ci), p(Xd), p(torch.tensor([alpha], device="cuda")), p(att), p(Y), M, nnz, K,
                                                  M + 3, st))
        torch.cuda.synchronize()
        assert_close(att, att_want, what="scores %s K=%d" % (name, K), scale=e_scale)
        assert_close(Y, Y_want, rtol=2e-5, what="aggregate %s K=%d" % (name, K), scale=Y_scale)
        assert bool((Y[M:] == 0).all())
        # the scores equal the windowed SDDMM's bit for bit when both sum a score the same way (same lane group shape)
        sd = torch.empty(nnz, device="cuda")
        _capi.check(L.psp_sddmm_window_f32(p(rp), p(ci), p(Xd), p(Xd), p(torch.tensor([alpha], device="cuda")), p(sd), M, nnz, K, M + 3, st))
        assert_close(sd, att.cpu().numpy(), what="scores vs windowed SDDMM", scale=e_scale)
        # backward: G = sum att dY[col]; wsum = sum <dY_i, dY_j> float(col)
        dY = (rng.standard_normal((M + 3, K)) / np.sqrt(K)).astype(np.float32)
        att_in = rng.standard_normal(nnz).astype(np.float32)
        G_want = oracle.spmm_csr(rowPtr, ci_w, att_in, dY, rows_out=M + 3)
        G_scale = oracle.spmm_csr(rowPtr, ci_w, np.abs(att_in), np.abs(dY), rows_out=M + 3)
        d = (dY[rows].astype(np.float64) * dY[ci_w].astype(np.float64)).sum(1)
        w_want = float((d * ci_w.astype(np.float32).astype(np.float64)).sum())
        w_scale = float(((np.abs(dY[rows]).astype(np.float64) * np.abs(dY[ci_w])).sum(1) * ci_w).sum())
        G = torch.full((M + 3, K), float("nan"), device="cuda")
        wsum = torch.full((1,), float("nan"), device="cuda")
        dYd, att_d = torch.from_numpy(dY).cuda(), torch.from_numpy(att_in).cuda()
        _capi.check(L.psp_attn_window_backward_f32(p(rp), p(ci), p(att_d), p(dYd), p(G), p(wsum), M, nnz, K, M + 3, st))
        torch.cuda.synchronize()
        assert_close(G, G_want, what="gradient aggregate %s K=%d" % (name, K), scale=G_scale)
        assert bool((G[M:] == 0).all())
        assert abs(float(wsum.item()) - w_want) <= 1e-6 + 2e-5 * w_scale, (float(wsum.item()), w_want, w_scale)
    X = torch.zeros(M, 72, device="cuda")
    assert L.psp_attn_window_forward_f32(p(rp), p(ci), p(X), None, p(att), p(X), M, nnz, 72, M, st) == -1   # wider than the kernel covers
    assert L.psp_attn_window_backward_f32(p(rp), p(ci), p(att), p(X), p(X), None, M, nnz, 16, M, st) == -1   # no place for the sum


@pytest.mark.gpu
def test_window_sddmm_non_finite_rows_stay_in_their_entries(oracle):
    from gpu_util import dev
    from paramspmm_ae_amd import _capi
    import ParamSpMM

    rowPtr, colIdx, val = banded_csr(1500, 9, 30, 9, far=0.2, hub=(3, 400))
    M, nnz = rowPtr.size - 1, colIdx.size
    rp, ci, _ = ParamSpMM.window_build(dev(rowPtr), dev(colIdx), dev(val))
    ci_w = ci.cpu().numpy()
    rows = np.repeat(np.arange(M), np.diff(rowPtr))
    for K in (16, 64):
        X = np.random.default_rng(K).standard_normal((M, K)).astype(np.float32)
        X[colIdx[5]] = np.inf
        X[colIdx[colIdx.size // 2], 3] = np.nan
        X[0] = np.inf       # the rows the clamped loads and the padding point at
        X[M - 1] = np.inf
        Xd = torch.from_numpy(X).cuda()
        out = torch.zeros(nnz, device="cuda")
        _capi.check(_capi.lib.psp_sddmm_window_f32(_capi.ptr(rp), _capi.ptr(ci), _capi.ptr(Xd), _capi.ptr(Xd), None, _capi.ptr(out), M,
                                                   nnz, K, M, torch.cuda.current_stream().cuda_stream))
        got = out.cpu().numpy()
        touched = ~np.isfinite(X).all(1)
        clean = ~touched[rows] & ~touched[ci_w]
        assert np.isfinite(got[clean]).all() and not np.isfinite(got[~clean]).any()
        want = oracle.sddmm_csr(rowPtr, ci_w, X, X)
        np.testing.assert_allclose(got[clean], want[clean], rtol=1e-4, atol=1e-4)


@pytest.mark.gpu
def test_window_operator_through_the_modules_and_a_gcn_layer(oracle):
    """pcsr_spmm(window=True): SpMM, the fused forward / backward, the SDDMM on the permuted arrays, and a GCN layer's
    gradients against dense autograd."""
    import ParamSpMM
    from gpu_util import assert_close
    from paramspmm_ae_amd import gnn_conv
    from paramspmm_ae_amd.graph_input import graph_input
    from paramspmm_ae_amd.PCSR import pcsr_spmm

    n = 2500
    rowPtr, colIdx, val = banded_csr(n, 8, 50, 12, far=0.1)
    # symmetric pattern with symmetric values (the layers multiply by A where the algebra asks for A^T)
    import scipy.sparse as sp

    A = sp.csr_matrix((val, colIdx, rowPtr), shape=(n, n))
    A = ((A + A.T) * 0.5).tocsr()
    A.sort_indices()
    rowPtr, colIdx, val = A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data.astype(np.float32)
    g = graph_input("banded", "")
    g.verbose = False
    g.load_from_csr(rowPtr, colIdx, val)
    op = pcsr_spmm(g, vec_size=1, if_split=False, window=True)
    assert op.fmt_code == 4 and 0.5 < op.window_local_share <= 1.0
    assert abs(op.window_local_share - window_reference(rowPtr, colIdx, val)[3]) < 1e-6
    X = np.random.default_rng(0).standard_normal((n, 32)).astype(np.float32)
    want = oracle.spmm_csr(rowPtr, colIdx, val, X)
    scale = oracle.spmm_csr(rowPtr, colIdx, np.abs(val), np.abs(X))
    Xd = torch.from_numpy(X).cuda()
    assert_close(op.GIN_spmm(Xd), want, what="window GIN_spmm", scale=scale)
    op.get_spmm_result(x=Xd)
    assert_close(op.result, want, what="window get_spmm_result", scale=scale)
    assert op.profiling(dim=16, verbose=False) > 0 and op.time_ms(Xd, warmup=1, iters=2) > 0
    # SDDMM on the permuted arrays: ones -> K for every stored entry
    assert bool((op.get_sddmm_result(48, 4) == 48).all())
    # the plain CSR kernel reads the permuted arrays as a matrix with unsorted rows: same product
    plain = ParamSpMM.csr_spmm(Xd, op.rowPtr, op.colIdx, op.val, 1, 4)
    assert_close(plain, want, what="csr kernel on the permuted arrays", scale=scale)

    Ad = torch.from_numpy(A.toarray().astype(np.float64)).cuda()
    for cls, relu_in in ((gnn_conv.GCNConv, False), (gnn_conv.GCNConv, True), (gnn_conv.GINConv, False), (gnn_conv.GINConv, True)):
        # (square layers of 16 / 32 columns with relu_input run the GCN layer as one launch, dense product folded in)
        for in_w, out_w in ((32, 16), (16, 32), (16, 16), (32, 32)):
            layer = cls(in_w, out_w).cuda()
            H = torch.randn(n, in_w, device="cuda", requires_grad=True)
            ops = {in_w: op, out_w: op}
            y = layer(H, ops, relu_input=True) if relu_in else layer(H, ops)
            dY = torch.randn_like(y)
            y.backward(dY)
            Hr = H.detach().double().requires_grad_(True)
            Wr = layer.weights.detach().double().requires_grad_(True)
            yr = Ad @ ((torch.relu(Hr) if relu_in else Hr) @ Wr)
            yr.backward(dY.double())
            torch.testing.assert_close(y.double(), yr, rtol=1e-4, atol=1e-4)
            torch.testing.assert_close(H.grad.double(), Hr.grad, rtol=1e-4, atol=1e-4)
            torch.testing.assert_close(layer.weights.grad.double(), Wr.grad, rtol=1e-3, atol=1e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("width", [16, 32, 20, 64, 96])
def test_agnn_layer_on_a_windowed_operator(width):
    """The attention layer on a windowed operator: forward against dense algebra, backward against the reference's
    literal formulas (gnn_conv.py:153-180) -- the per-entry vectors follow the operator's own entry order, which
    leaves every one of those sums unchanged.  Up to 64 columns a direction is one launch (scores and aggregation
    together, psp_attn_window_*); 96 runs the windowed SDDMM and SpMM one after the other."""
    from paramspmm_ae_amd.graph_input import graph_input
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from paramspmm_ae_amd.gnn_conv import AGNNConv

    n = 700
    rowPtr, colIdx, val = banded_csr(n, 7, 25, 31, far=0.2, hub=(11, 300))
    g = graph_input("t", "")
    g.verbose = False
    g.load_from_csr(rowPtr, colIdx, val)
    op = pcsr_spmm(g, vec_size=1, if_split=False, window=True)
    rows = torch.from_numpy(np.repeat(np.arange(n), np.diff(rowPtr))).cuda()
    pattern = torch.zeros(n, n, device="cuda")
    pattern[rows, torch.from_numpy(colIdx.astype(np.int64)).cuda()] = 1.0
    torch.manual_seed(1)
    layer = AGNNConv(24, width).cuda()
    X = torch.randn(n, 24, device="cuda", requires_grad=True)
    ci = g.csr_data.colIdx.cuda().unsqueeze(-1)  # what the driver hands to the layer: the graph's own order
    y = layer(X, {width: op}, ci)
    Xp = X.detach() @ layer.weights.detach()
    att = pattern * (Xp @ Xp.t()) * layer.attention_w.detach().reshape(())
    torch.testing.assert_close(y, att @ Xp, rtol=1e-4, atol=1e-4)
    dY = torch.randn_like(y)
    y.backward(dY)
    d_in_prime = att @ dY
    torch.testing.assert_close(X.grad, d_in_prime @ layer.weights.detach().t(), rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(layer.weights.grad, X.detach().t() @ d_in_prime, rtol=1e-3, atol=1e-3)
    d_att = (dY[rows] * dY[g.csr_data.colIdx.cuda().long()]).sum(1)
    want = (d_att[None, :].double() @ ci.double()).t()
    torch.testing.assert_close(layer.attention_w.grad.double(), want, rtol=1e-3, atol=1e-1)
    # the scores themselves, against the CSR kernel on the same arrays
    import ParamSDDMM

    Xp = Xp.contiguous()
    e = op.AGNN_sddmm(Xp)
    ref = ParamSDDMM.csr_sddmm(Xp, Xp, op.rowPtr, op.colIdx, op.val, 1, 4)
    torch.testing.assert_close(e, ref, rtol=1e-4, atol=1e-4)


@pytest.mark.gpu
def test_training_with_windowed_operators_follows_training_with_the_csr_operators():
    """A community-ordered block model: most entries are local, configure_operators may keep the windowed layout
    (decided by timing), and GCN / GIN networks built on windowed operators produce the log-probabilities and take
    the training steps of the same networks on plain CSR operators (same seed, a few epochs)."""
    from paramspmm_ae_amd import GNN, synth
    from paramspmm_ae_amd.graph_input import graph_input
    from paramspmm_ae_amd.PCSR import pcsr_spmm

    n = 40000
    r, c, n = synth.sbm(n, n // 100, 12, 1.5, seed=5)
    rowPtr, colIdx, val = synth.to_gcn_csr(r, c, n)
    g = graph_input("sbm", "")
    g.verbose = False
    g.load_from_csr(rowPtr, colIdx, val)
    win = pcsr_spmm(g, vec_size=1, if_split=False, window=True)
    assert win.window_local_share > 0.8
    from paramspmm_ae_amd.decider import SpMMDecider

    dec = SpMMDecider()
    dec.gen_model_dict([16, 32])
    ops = GNN.configure_operators(dec, g, [16, 32])
    X = torch.randn(n, 16, device="cuda")
    plain = pcsr_spmm(g, vec_size=1, if_split=False)
    want = plain._spmm(X)
    for d, op in ops.items():  # whichever layout was kept computes the product
        got = op._spmm(torch.randn(n, d, device="cuda") * 0 + X[:, :1].expand(n, d).contiguous())[:n]
        torch.testing.assert_close(got[:, 0], want[:, 0], rtol=1e-4, atol=1e-5)
    for net in ("GCN", "GIN"):
        outs = []
        for which in ("csr", "window"):
            op = plain if which == "csr" else win
            torch.manual_seed(3)
            model = GNN.build_model(net, g, {16: op, 32: op}, 16, 32, 16)
            ms = GNN.train_profiling(model, g.y, 3)
            assert ms > 0
            model.eval()
            outs.append(model().detach())
        torch.testing.assert_close(outs[0], outs[1], rtol=2e-3, atol=2e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("hidden", [16, 64])
def test_attention_network_on_windowed_operators_equals_the_one_on_csr_operators(hidden):
    """The five-layer attention network (GNN.py:82-101) on windowed operators: loss and every gradient of one training
    step equal those of the same network (same seed, same dropout mask) on plain CSR operators."""
    from paramspmm_ae_amd import GNN, synth
    from paramspmm_ae_amd.graph_input import graph_input
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from paramspmm_ae_amd.gnn_conv import nll_loss_mean

    r, c, n = synth.sbm(20000, 200, 12, 1.5, seed=6)
    rowPtr, colIdx, val = synth.to_gcn_csr(r, c, n)
    g = graph_input("sbm", "")
    g.verbose = False
    g.load_from_csr(rowPtr, colIdx, val)
    ops = {"csr": pcsr_spmm(g, vec_size=1, if_split=False, CF=1, blkWarpNum=4), "window": pcsr_spmm(g, vec_size=1, if_split=False, window=True)}
    torch.manual_seed(0)
    x = torch.randn(n, 32, device="cuda")
    labels = torch.randint(0, 16, (n,), device="cuda")
    res = {}
    for which, op in ops.items():
        torch.manual_seed(1)
        model = GNN.AGNN(16, 32, x, {16: op, 32: op, hidden: op}, hidden, g.csr_data.colIdx.cuda().unsqueeze(-1)).cuda()
        with torch.no_grad():  # keep the attention scores of five stacked layers in range
            for q in model.parameters():
                q.mul_(0.3)
        model.train()
        torch.manual_seed(123)  # the dropout mask
        loss = nll_loss_mean(model(), labels)
        loss.backward()
        res[which] = (loss.item(), [q.grad.clone() for q in model.parameters()])
    assert abs(res["csr"][0] - res["window"][0]) <= 1e-4 * abs(res["csr"][0])
    for a, b in zip(res["window"][1], res["csr"][1]):
        torch.testing.assert_close(a, b, rtol=2e-3, atol=1e-4 * float(b.abs().max()) + 1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("N", [16, 32])
def test_window_spmm_with_the_dense_product_folded_in(oracle, N):
    """psp_spmm_window_xw_f32: Y = ((A f(X)) W) or ((A f(X)) W^T), masked, with A f(X) delivered beside it: the raw
    product equals the plain windowed product bit for bit (same kernel, same order), Y a float64 restatement to
    1e-5 of the magnitudes involved, masked elements are exact zeros; widths other than 16 / 32 are argument errors."""
    from gpu_util import dev
    from paramspmm_ae_amd import _capi
    import ParamSpMM

    rowPtr, colIdx, val = banded_csr(4001, 10, 40, 20 + N, far=0.15, hub=(9, 500), empty_frac=0.05)
    M = rowPtr.size - 1
    rp, ci, v = ParamSpMM.window_build(dev(rowPtr), dev(colIdx), dev(val))
    import scipy.sparse as sp

    A = sp.csr_matrix((val.astype(np.float64), colIdx, rowPtr), shape=(M, M))
    rng = np.random.default_rng(N)
    X = rng.standard_normal((M, N)).astype(np.float32)
    W = (rng.standard_normal((N, N)) / np.sqrt(N)).astype(np.float32)
    mask = rng.standard_normal((M, N)).astype(np.float32)
    Xd, Wd, Md = torch.from_numpy(X).cuda(), torch.from_numpy(W).cuda(), torch.from_numpy(mask).cuda()
    p, L = _capi.ptr, _capi.lib
    st = torch.cuda.current_stream().cuda_stream
    for transW in (0, 1):
        for relu in (0, 1):
            for use_mask in (False, True):
                print("case xw", N, transW, relu, use_mask, flush=True)
                Y = torch.full((M, N), float("nan"), device="cuda")
                R = torch.full((M, N), float("nan"), device="cuda")
                _capi.check(L.psp_spmm_window_xw_f32(p(rp), p(ci), p(v), p(Xd), p(Wd), transW, p(Y), p(R), M, int(ci.numel()), N, M,
                                                     relu, p(Md) if use_mask else None, st))
                torch.cuda.synchronize()
                fX = np.maximum(X, 0) if relu else X
                plain = _spmm_window((rp, ci, v, M), torch.from_numpy(fX).cuda())
                assert torch.equal(R, plain)
                AX = A @ fX.astype(np.float64)
                want = AX @ (W.T if transW else W).astype(np.float64)
                scale = (abs(A) @ np.abs(fX).astype(np.float64)) @ np.abs(W.T if transW else W).astype(np.float64)
                got = Y.cpu().numpy().astype(np.float64)
                if use_mask:
                    assert np.all(got[mask <= 0] == 0)
                    want = np.where(mask > 0, want, 0.0)
                assert np.all(np.abs(got - want) <= 1e-6 + 1e-5 * scale), float(np.abs(got - want).max())
                # without the raw output
                Y2 = torch.full((M, N), float("nan"), device="cuda")
                _capi.check(L.psp_spmm_window_xw_f32(p(rp), p(ci), p(v), p(Xd), p(Wd), transW, p(Y2), None, M, int(ci.numel()), N, M,
                                                     relu, p(Md) if use_mask else None, st))
                assert torch.equal(Y2, Y)
    X48 = torch.zeros(M, 48, device="cuda")
    assert L.psp_spmm_window_xw_f32(p(rp), p(ci), p(v), p(X48), p(Wd), 0, p(X48), None, M, int(ci.numel()), 48, M, 0, None, st) == -1
    assert L.psp_spmm_window_xw_f32(p(rp), p(ci), p(v), p(Xd), None, 0, p(Xd), None, M, int(ci.numel()), N, M, 0, None, st) == -1
