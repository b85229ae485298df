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
    for bw in (4, 8, 4 | 0x100, 8 | 0x100):  # 0x100: the entry-balanced walk of the plain layouts (PSP_BW_BALANCED)
        got = sddmm_capi(fmt, F, torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), bw)
        torch.cuda.synchronize()
        assert_close(got, want, what="%s K=%d bw=%#x" % (fmt, K, bw))


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


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("N,CF,bw", [(32, 1, 8), (16, 1, 4), (64, 2, 4), (128, 4, 8), (96, 3, 4)])
def test_fused_attention_pipeline_matches_oracle(oracle, split, N, CF, bw):
    """Scaled SDDMM with row maxima, then the softmax-weighted SpMM, against the oracle's three separate steps
    (scaled scores -> segment softmax -> SpMM).  Hub row cut over many wavefronts, empty rows, rows shorter than a
    lane group, scores spread widely (standard normal inputs of width 24, not normalised)."""
    from paramspmm_ae_amd import _capi
    from gpu_util import Formats, assert_close, dev, stream

    rowPtr, colIdx, val = random_csr(3001, 9, 21, empty_frac=0.15, hub=(11, 2600), values="uniform")
    F = Formats(oracle, rowPtr, colIdx, val)
    n, K = F.n, 24
    rng = np.random.default_rng(N)
    A = rng.standard_normal((n, K)).astype(np.float32)
    B = rng.standard_normal((n, K)).astype(np.float32)
    H = rng.standard_normal((n, N)).astype(np.float32)
    e_want = oracle.sddmm_csr(rowPtr, colIdx, A, B) * val
    w_want = oracle.segment_softmax(rowPtr, e_want)
    y_want = oracle.spmm_csr(rowPtr, colIdx, w_want, H)
    scale = oracle.spmm_csr(rowPtr, colIdx, w_want, np.abs(H))
    m_want = np.full(n, -3.402823466e+38, np.float32)
    rows = np.repeat(np.arange(n), np.diff(rowPtr))
    np.maximum.at(m_want, rows, e_want)

    L, p = _capi.lib, _capi.ptr
    Ad, Bd, Hd = dev(A), dev(B), dev(H)
    e = torch.full((F.nnz,), float("nan"), device="cuda")
    m = torch.full((n,), float("nan"), device="cuda")
    Y = torch.full((n, N), float("nan"), device="cuda")
    d = F.d
    if split:
        _capi.check(L.psp_sddmm_csr_split_rowmax_f32(p(d["rps"]), p(d["colIdx"]), p(d["tr"]), p(Ad), p(Bd), p(d["val"]), p(e),
                                                     p(m), F.tr.size, n, K, bw, stream()))
        row_sum = torch.full((n,), float("nan"), device="cuda")
        _capi.check(L.psp_spmm_csr_split_softmax_f32(p(d["rps"]), p(d["colIdx"]), p(e), p(d["tr"]), p(m), p(row_sum), p(Hd),
                                                     p(Y), F.tr.size, N, n, CF, bw, stream()))
    else:
        _capi.check(L.psp_sddmm_csr_rowmax_f32(p(d["rowPtr"]), p(d["colIdx"]), p(Ad), p(Bd), p(d["val"]), p(e), p(m), n, K,
                                               bw, stream()))
        _capi.check(L.psp_spmm_csr_softmax_f32(p(d["rowPtr"]), p(d["colIdx"]), p(e), p(m), p(Hd), p(Y), n, N, n, CF, bw,
                                               stream()))
    torch.cuda.synchronize()
    # the inputs are not normalised: a dot product may cancel, so the relative term is taken against sum |a||b|
    e_scale = oracle.sddmm_csr(rowPtr, colIdx, np.abs(A), np.abs(B)) * np.abs(val)
    assert_close(e, e_want, rtol=1e-5, atol=1e-6, what="scores", scale=e_scale)
    # the row maximum is one of the scores: compare with the device's own scores exactly, with the oracle's loosely
    m_dev = np.full(n, -3.402823466e+38, np.float32)
    np.maximum.at(m_dev, rows, e.cpu().numpy())
    assert np.array_equal(m.cpu().numpy(), m_dev)
    assert_close(m, m_want, rtol=1e-4, atol=1e-5, what="row maxima")
    # the weights inherit the rounding of the scores (|d exp(e)| = exp(e) |de|, scores of magnitude up to ~10)
    assert_close(Y, y_want, rtol=1e-4, atol=1e-5, what="softmax-weighted product", scale=scale)


def test_fused_attention_modules_match_unfused():
    """ParamSDDMM.*_scaled_rowmax + ParamSpMM.*_spmm_softmax against scaled SDDMM -> segment_softmax -> SpMM on an
    R-MAT graph (2^16 nodes), both layouts."""
    import ParamSDDMM
    import ParamSpMM
    from paramspmm_ae_amd import synth
    from paramspmm_ae_amd.graph_input import graph_input

    r, c, n = synth.rmat(16, 8 << 16, seed=3)
    rowPtr, colIdx, val = synth.to_gcn_csr(r, c, n)
    g = graph_input("t", "")
    g.verbose = False
    g.load_from_csr(rowPtr, colIdx, val)
    cd = g.csr_data
    rp, ci, v, rps, tr = (cd.on_device(k, "cuda") for k in ("rowPtr", "colIdx", "val", "rowPtr_split", "target_row"))
    gen = torch.Generator(device="cuda").manual_seed(1)
    X = torch.nn.functional.normalize(torch.randn(n, 32, device="cuda", generator=gen), dim=1).contiguous()
    H = torch.randn(n, 32, device="cuda", generator=gen)
    a = ParamSDDMM.segment_softmax(rp, ParamSDDMM.csr_sddmm_scaled(X, X, rp, ci, v, 8))
    want = ParamSpMM.csr_spmm(H, rp, ci, a, 1, 8)
    e, m = ParamSDDMM.csr_sddmm_scaled_rowmax(X, X, rp, ci, v, 8)
    got = ParamSpMM.csr_spmm_softmax(H, rp, ci, e, m, 1, 8)
    torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-6)
    e, m = ParamSDDMM.csr_split_sddmm_scaled_rowmax(X, X, rps, ci, v, tr, n, 8)
    got = ParamSpMM.csr_split_spmm_softmax(H, rps, ci, e, m, tr, 1, 8)
    torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("K", [16, 32, 100, 128, 256, 7])
def test_sddmm_3x1_blocks(oracle, split, K):
    """vec_sddmm / vec_split_sddmm through the C ABI against the oracle, vec_size 3 and (through the same entry points)
    2; a row count that is not a multiple of the block height, a hub row, empty rows."""
    from paramspmm_ae_amd import _capi
    from gpu_util import assert_close, dev, stream

    rowPtr, colIdx, val = random_csr(2000, 8, 17, empty_frac=0.1, hub=(10, 900), values="uniform")
    n = rowPtr.size - 1
    L, p = _capi.lib, _capi.ptr
    for R in (3, 2):
        npad = (n + R - 1) // R * R
        rpb, cib, vb = oracle.vbsr_build(rowPtr, colIdx, val, R, ncols=npad)
        A, B = unit_rows(npad, K, K), unit_rows(npad, K, K + 1)
        Ad, Bd, cib_d, vb_d = dev(A), dev(B), dev(cib), dev(vb)  # referenced until the kernel has run
        out = torch.full((cib.size, R), float("nan"), device="cuda")
        for bw in (4, 8):
            if split:
                rps, tr = oracle.split_csr(rpb, 8)
                want = oracle.sddmm_vec(rps, cib, vb, A, B, target_row=tr)
                rps_d, tr_d = dev(rps), dev(tr)
                _capi.check(L.psp_sddmm_vec_split_f32(p(rps_d), p(cib_d), p(vb_d), p(tr_d), p(Ad), p(Bd), p(out), tr.size, K, R,
                                                      bw, stream()))
            else:
                want = oracle.sddmm_vec(rpb, cib, vb, A, B)
                rpb_d = dev(rpb)
                _capi.check(L.psp_sddmm_vec_f32(p(rpb_d), p(cib_d), p(vb_d), p(Ad), p(Bd), p(out), rpb.size - 1, K, R, bw,
                                                stream()))
            torch.cuda.synchronize()
            assert_close(out, want, what="%dx1 blocks K=%d bw=%d split=%s" % (R, K, bw, split))


def test_facade_sddmm_with_3x1_blocks(oracle):
    from paramspmm_ae_amd import synth
    from paramspmm_ae_amd.graph_input import graph_input
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from gpu_util import assert_close

    r, c, n = synth.chung_lu(3001, 12000, 2.1, seed=4)
    rowPtr, colIdx, val = synth.to_gcn_csr(r, c, n)
    g = graph_input("t", "")
    g.verbose = False
    g.load_from_csr(rowPtr, colIdx, val, blk_size=3)
    rpb, cib, vb = (g.bcsr_data.rowPtr.numpy(), g.bcsr_data.colIdx.numpy(), g.bcsr_data.val.numpy())
    npad = (n + 2) // 3 * 3
    A = unit_rows(npad, 32, 5)
    want = oracle.sddmm_vec(rpb, cib, vb, A, A)
    for split in (False, True):
        op = pcsr_spmm(g, vec_size=3, if_split=split, CF=1, blkWarpNum=4)
        got = op._sddmm(torch.from_numpy(A).cuda(), torch.from_numpy(A).cuda(), 4)
        assert_close(got, want, what="facade 3x1 sddmm split=%s" % split)
        ones = op.get_sddmm_result(64, 8)
        assert torch.all(ones[torch.from_numpy(vb != 0).cuda()] == 64)


@pytest.mark.parametrize("fmt", ["csr", "bcsr"])
def test_sddmm_entry_balanced_walk_structures(oracle, fmt):
    """The entry-balanced walk on the structures that stress it: a hub row spanning many wavefronts' tiles, runs of
    hundreds of empty rows (windows of 64 rows without an entry), rows of one entry (more than 64 rows per tile),
    a matrix smaller than one tile, an empty matrix; bit-identical to the row-wise walk (same dot products, same
    order inside a lane group is not guaranteed, so: to tolerance) and equal to the oracle."""
    from gpu_util import Formats, sddmm_capi, sddmm_oracle, assert_close

    rng = np.random.default_rng(5)
    cases = {}
    n = 9000
    deg = np.ones(n, np.int64)
    deg[100] = 8000
    deg[2000:2900] = 0
    deg[5000:5200] = rng.integers(40, 90, 200)
    deg[-300:] = 0
    rowPtr = np.zeros(n + 1, np.int32)
    rowPtr[1:] = np.cumsum(deg)
    cols = np.concatenate([np.sort(rng.choice(n, d, replace=False)) for d in deg]).astype(np.int32)
    cases["mixed"] = (rowPtr, cols, rng.uniform(0.1, 1, cols.size).astype(np.float32))
    cases["tiny"] = random_csr(37, 3, 9, values="uniform")
    cases["empty"] = (np.zeros(11, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32))
    for name, (rp, ci, v) in cases.items():
        F = Formats(oracle, rp, ci, v)
        for K in (16, 64, 100):
            print("case", fmt, name, K, flush=True)
            A = unit_rows(F.n + (F.n & 1), K, K)
            B = unit_rows(F.n + (F.n & 1), K, K + 1)
            want = sddmm_oracle(oracle, fmt, F, A, B)
            for bw in (4 | 0x100, 8 | 0x100):
                got = sddmm_capi(fmt, F, torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), bw)
                torch.cuda.synchronize()
                assert_close(got, want, what="%s %s K=%d balanced" % (fmt, name, K))


@pytest.mark.parametrize("fmt", FMTS)
def test_sddmm_xcd_stripe_flag(oracle, fmt):
    """blkWarpNum | PSP_BW_STRIPE(rows) only changes which workgroup takes which rows: every entry's result keeps
    its bits, with the row-wise and with the entry-balanced walk."""
    from gpu_util import Formats, sddmm_capi
    from paramspmm_ae_amd import _capi

    rowPtr, colIdx, val = random_csr(40013, 7, 5, empty_frac=0.05, hub=(31, 2500), values="normal")
    F = Formats(oracle, rowPtr, colIdx, val)
    for K in (16, 96):
        A = torch.from_numpy(unit_rows(F.n + (F.n & 1), K, K)).cuda()
        B = torch.from_numpy(unit_rows(F.n, K, K + 1)).cuda()
        base = sddmm_capi(fmt, F, A, B, 4)
        for rows in (256, 1536, 6144, 65280):
            for bw in (4, 8 | 0x100):
                print("case", fmt, K, rows, bw, flush=True)
                got = sddmm_capi(fmt, F, A, B, bw | _capi.bw_stripe(rows))
                torch.cuda.synchronize()
                assert torch.equal(got, base)
