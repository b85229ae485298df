"""GPU parity of SDDMM, genmask and segment softmax against the CPU oracle, through the C ABI.
Tolerance rel 1e-5 / abs 1e-6 on row-L2-normalised inputs (the attention configuration)."""
import numpy as np
import pytest
import torch

from conftest import random_csr

pytestmark = pytest.mark.gpu

FMTS = ["csr", "csr_split", "bcsr", "bcsr_split"]


@pytest.fixture(scope="module")
def small(oracle):
    from gpu_util import Formats

    rowPtr, colIdx, val = random_csr(2001, 10, 3, empty_frac=0.1, hub=(4, 700), values="uniform")
    return Formats(oracle, rowPtr, colIdx, val)


def unit_rows(rows, K, seed):
    a = np.random.default_rng(seed).standard_normal((rows, K)).astype(np.float32)
    return (a / np.linalg.norm(a, axis=1, keepdims=True)).astype(np.float32)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("K", [1, 2, 7, 16, 32, 48, 64, 96, 100, 128, 200, 256, 512])
def test_sddmm_parity(oracle, small, fmt, K):
    from gpu_util import sddmm_capi, sddmm_oracle, assert_close

    F = small
    print("case", fmt, K, flush=True)
    A = unit_rows(F.n + (F.n & 1), K, K)
    B = unit_rows(F.n, K, K + 1)
    want = sddmm_oracle(oracle, fmt, F, A, B)
    for bw in (4, 8):
        got = sddmm_capi(fmt, F, torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), bw)
        torch.cuda.synchronize()
        assert_close(got, want, what="%s K=%d bw=%d" % (fmt, K, bw))


@pytest.mark.parametrize("fmt", FMTS)
def test_sddmm_ones_gives_K(small, fmt):
    """The reference's known answer: A = B = ones -> every stored entry equals K exactly (SDDMM.py:127-128)."""
    from gpu_util import sddmm_capi

    F = small
    for K in (32, 64, 128):
        A = torch.ones(F.n + 1, K, device="cuda")
        out = sddmm_capi(fmt, F, A, A, 4).cpu().numpy()
        if fmt.startswith("bcsr"):
            assert np.all(out[F.vb != 0] == K) and np.all(out[F.vb == 0] == 0)
        else:
            assert np.all(out == K)


def test_sddmm_scaled_and_self_loops(oracle, small):
    from gpu_util import sddmm_capi, assert_close

    F = small
    A = unit_rows(F.n + 1, 64, 1)
    Ad = torch.from_numpy(A).cuda()
    plain = sddmm_capi("csr", F, Ad, Ad, 4)
    scaled = sddmm_capi("csr", F, Ad, Ad, 4, scale=F.d["val"])
    assert_close(scaled, plain.cpu().numpy() * F.val, rtol=1e-6, atol=1e-7, what="scale")
    rows = np.repeat(np.arange(F.n), np.diff(F.rowPtr))
    diag = rows == F.colIdx
    assert diag.any()
    assert np.allclose(plain.cpu().numpy()[diag], 1.0, atol=1e-6)  # <x,x> of a unit row


def test_genmask_parity(oracle, small):
    from paramspmm_ae_amd import _capi
    from gpu_util import stream

    F = small
    mask = torch.full((F.nnz,), -1, dtype=torch.int32, device="cuda")
    p = _capi.ptr
    _capi.check(_capi.lib.psp_genmask(p(F.d["rpb"]), p(F.d["rowPtr"]), p(F.d["vb"]), F.rpb.size - 1, F.nnz, p(mask), stream()))
    assert np.array_equal(mask.cpu().numpy(), oracle.genmask(F.rpb, F.rowPtr, F.vb, F.nnz))


def test_segment_softmax_parity(oracle, small):
    from paramspmm_ae_amd import _capi
    from gpu_util import stream, assert_close

    F = small
    e = (np.random.default_rng(0).standard_normal(F.nnz) * 3).astype(np.float32)
    ed = torch.from_numpy(e).cuda()
    out = torch.full_like(ed, float("nan"))
    p = _capi.ptr
    _capi.check(_capi.lib.psp_segment_softmax_f32(p(F.d["rowPtr"]), p(ed), p(out), F.n, stream()))
    assert_close(out, oracle.segment_softmax(F.rowPtr, e), rtol=1e-5, atol=1e-6, what="softmax")
    # in place
    _capi.check(_capi.lib.psp_segment_softmax_f32(p(F.d["rowPtr"]), p(ed), p(ed), F.n, stream()))
    assert_close(ed, out.cpu().numpy(), rtol=0, atol=0, what="softmax in place")


def test_segment_softmax_long_rows(oracle):
    """Rows above the long-row threshold (128 entries) are handled by a whole workgroup; several in one workgroup's 16 rows, plus empty rows."""
    from paramspmm_ae_amd import _capi
    from gpu_util import stream, assert_close

    rowPtr, colIdx, val = random_csr(5000, 6, 4, empty_frac=0.3, hub=(17, 4000))
    k = np.diff(rowPtr).copy()
    k[18], k[21], k[4999] = 1500, 1025, 2049
    rowPtr = np.concatenate([[0], np.cumsum(k)]).astype(np.int32)
    e = (np.random.default_rng(2).standard_normal(rowPtr[-1]) * 5).astype(np.float32)
    ed = torch.from_numpy(e).cuda()
    rp = torch.from_numpy(rowPtr).cuda()
    out = torch.full_like(ed, float("nan"))
    p = _capi.ptr
    _capi.check(_capi.lib.psp_segment_softmax_f32(p(rp), p(ed), p(out), rowPtr.size - 1, stream()))
    assert_close(out, oracle.segment_softmax(rowPtr, e), rtol=1e-5, atol=1e-6, what="softmax long rows")
    _capi.check(_capi.lib.psp_segment_softmax_f32(p(rp), p(ed), p(ed), rowPtr.size - 1, stream()))
    assert_close(ed, out.cpu().numpy(), rtol=0, atol=0, what="softmax long rows in place")


@pytest.mark.parametrize("all_negative", [False, True])
def test_segment_softmax_with_workspace_spreads_long_rows(oracle, all_negative):
    """The workspace variant hands rows above 128 entries to chunk-wise launches (atomic max, atomic sum): rows
    that cross chunk boundaries, a row of several chunks, long rows next to each other, the last row long, empty
    rows, and inputs that are all negative (the float maximum goes through integer atomics)."""
    from paramspmm_ae_amd import _capi
    from gpu_util import stream, assert_close

    rowPtr, colIdx, val = random_csr(6000, 6, 7, empty_frac=0.3, hub=(17, 5500))
    k = np.diff(rowPtr).copy()
    k[18], k[19], k[21], k[3000], k[5999] = 1500, 1025, 20000, 4096, 2049
    k[100:140] = 129  # forty rows just above the threshold in a row: more than one list entry per wavefront
    rowPtr = np.concatenate([[0], np.cumsum(k)]).astype(np.int32)
    nnz = int(rowPtr[-1])
    e = (np.random.default_rng(3).standard_normal(nnz) * 5).astype(np.float32)
    if all_negative:
        e = -np.abs(e) - 1.0
    ed = torch.from_numpy(e).cuda()
    rp = torch.from_numpy(rowPtr).cuda()
    out = torch.full_like(ed, float("nan"))
    ws = torch.full((2 * (rowPtr.size - 1),), float("nan"), device="cuda")  # contents must not matter
    p = _capi.ptr
    want = oracle.segment_softmax(rowPtr, e)
    _capi.check(_capi.lib.psp_segment_softmax_ws_f32(p(rp), p(ed), p(out), rowPtr.size - 1, nnz, p(ws), stream()))
    assert_close(out, want, rtol=1e-5, atol=1e-6, what="softmax with workspace")
    # a second call on the used workspace, in place
    _capi.check(_capi.lib.psp_segment_softmax_ws_f32(p(rp), p(ed), p(ed), rowPtr.size - 1, nnz, p(ws), stream()))
    assert_close(ed, want, rtol=1e-5, atol=1e-6, what="softmax with workspace, in place")
    # through the module
    import ParamSDDMM
    got = ParamSDDMM.segment_softmax(rp, torch.from_numpy(e).cuda())
    assert_close(got, want, rtol=1e-5, atol=1e-6, what="ParamSDDMM.segment_softmax")


def test_full_size_headline_graph_properties(oracle):
    """SDDMM on the benchmark's R-MAT 2^20 pattern: A = B = ones gives K on every stored entry; with A = B the
    result is symmetric on the symmetric pattern (entry (i,j) equals entry (j,i)); the split format agrees with the
    plain one bit for bit (every entry is one lane group's own dot product); the blocked result holds the same
    numbers at the positions the mask names."""
    from gpu_util import Formats, sddmm_capi
    from paramspmm_ae_amd import synth, _capi

    rowPtr, colIdx, val, n = synth.config_graph("C2")
    F = Formats(oracle, rowPtr, colIdx, val)
    K = 32
    ones = torch.ones(n, K, device="cuda")
    assert torch.all(sddmm_capi("csr_split", F, ones, ones, 8) == K)
    A = torch.randn(n, K, device="cuda", generator=torch.Generator(device="cuda").manual_seed(9))
    e = sddmm_capi("csr", F, A, A, 4)
    e_split = sddmm_capi("csr_split", F, A, A, 8)
    assert torch.equal(e, e_split)
    # transpose position of every entry: sort (col, row) pairs; the pattern is symmetric, so it is a permutation
    rows = np.repeat(np.arange(n, dtype=np.int64), np.diff(rowPtr))
    order = np.lexsort((rows, colIdx.astype(np.int64)))  # entries ordered by (col, row) = transposed CSR order
    eh = e.cpu().numpy()
    assert np.array_equal(eh[order], eh), "e(i,j) must equal e(j,i) when A = B"
    # blocked format through the mask
    mask = torch.empty(F.nnz, dtype=torch.int32, device="cuda")
    p = _capi.ptr
    _capi.check(_capi.lib.psp_genmask(p(F.d["rpb"]), p(F.d["rowPtr"]), p(F.d["vb"]), F.rpb.size - 1, F.nnz, p(mask),
                                      torch.cuda.current_stream().cuda_stream))
    eb = sddmm_capi("bcsr", F, A, A, 4).reshape(-1)
    got = eb[mask.long()].cpu().numpy()
    # the mask lists a row's entries in block order: compare per row as multisets
    a_sorted = eh[np.lexsort((eh, rows))]
    b_sorted = got[np.lexsort((got, rows))]
    assert np.array_equal(a_sorted, b_sorted)
