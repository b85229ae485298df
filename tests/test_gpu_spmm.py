"""GPU parity of the SpMM kernels against the CPU oracle, through the C ABI.  Tolerance: rel 1e-5 / abs 1e-6
(fp32), the bar the north star states.  Inputs: seeded; values in (0.1, 1), features N(0,1)."""
import numpy as np
import pytest
import torch

from conftest import random_csr

pytestmark = pytest.mark.gpu

FMTS = ["csr", "csr_split", "bcsr", "bcsr_split"]


@pytest.fixture(scope="module")
def small(oracle):
    from gpu_util import Formats

    rowPtr, colIdx, val = random_csr(3001, 12, 7, empty_frac=0.1, hub=(5, 900), values="uniform")
    return Formats(oracle, rowPtr, colIdx, val)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("N", [16, 32, 48, 64, 96, 128, 160, 192, 224, 256])
def test_spmm_decider_dims_all_cf(oracle, small, fmt, N):
    from gpu_util import spmm_capi, spmm_oracle, spmm_abs_scale, assert_close
    from oracle.oracle import CF_TABLE

    F = small
    print("case", fmt, N, flush=True)
    X = np.random.default_rng(N).standard_normal((F.n + (F.n & 1), N)).astype(np.float32)
    want = spmm_oracle(oracle, fmt, F, X)
    scale = spmm_abs_scale(oracle, F, X, want.shape[0])
    Xd = torch.from_numpy(X).cuda()
    for CF in CF_TABLE[N]:
        for bw in (4, 8):
            got = spmm_capi(fmt, F, Xd, CF, bw)
            torch.cuda.synchronize()
            assert_close(got, want, what="%s N=%d CF=%d bw=%d" % (fmt, N, CF, bw), scale=scale)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("N", [1, 2, 3, 6, 8, 20, 50, 100, 250, 260, 513])
def test_spmm_odd_widths(oracle, small, fmt, N):
    from gpu_util import spmm_capi, spmm_oracle, spmm_abs_scale, assert_close

    F = small
    print("case", fmt, N, flush=True)
    X = np.random.default_rng(N).standard_normal((F.n + (F.n & 1), N)).astype(np.float32)
    want = spmm_oracle(oracle, fmt, F, X)
    scale = spmm_abs_scale(oracle, F, X, want.shape[0])
    Xd = torch.from_numpy(X).cuda()
    for CF in (1, 2, 3, 5, 8):
        got = spmm_capi(fmt, F, Xd, CF, 4)
        torch.cuda.synchronize()
        assert_close(got, want, what="%s N=%d CF=%d" % (fmt, N, CF), scale=scale)


@pytest.mark.parametrize("fmt", ["csr", "bcsr"])
@pytest.mark.parametrize("N", [16, 48, 160, 513])
def test_spmm_rows_past_the_matrix_read_zero(oracle, small, fmt, N):
    """Y may have more rows than the matrix (a padded feature matrix): they come back as zeros whether the kernel
    writes them itself (up to 16 rows) or a fill launch does, and the matrix's own rows are what they are without."""
    from gpu_util import spmm_oracle, spmm_abs_scale, assert_close, stream
    from paramspmm_ae_amd import _capi

    F = small
    L, p, d = _capi.lib, _capi.ptr, F.d
    X = np.random.default_rng(N).standard_normal((F.n + (F.n & 1), N)).astype(np.float32)
    want = spmm_oracle(oracle, fmt, F, X)
    covered = F.n if fmt == "csr" else 2 * (F.rpb.size - 1)
    scale = spmm_abs_scale(oracle, F, X, want.shape[0])
    Xd = torch.from_numpy(X).cuda()
    for tail in (0, 1, 3, 16, 17, 40):
        for CF, bw in ((1, 4), (2, 8), (8, 4)):
            print("case", fmt, N, tail, CF, bw, flush=True)
            Y = torch.full((covered + tail + 2, N), float("nan"), device="cuda")  # two guard rows behind rows_out
            if fmt == "csr":
                rc = L.psp_spmm_csr_f32(p(d["rowPtr"]), p(d["colIdx"]), p(d["val"]), p(Xd), p(Y), F.n, N, covered + tail, CF, bw, stream())
            else:
                rc = L.psp_spmm_bcsr_f32(p(d["rpb"]), p(d["cib"]), p(d["vb"]), p(Xd), p(Y), F.rpb.size - 1, N, covered + tail, CF, bw, stream())
            _capi.check(rc)
            torch.cuda.synchronize()
            assert_close(Y[:covered], want[:covered], what="%s N=%d tail=%d CF=%d" % (fmt, N, tail, CF), scale=scale[:covered])
            assert torch.count_nonzero(Y[covered:covered + tail]).item() == 0 and not torch.isnan(Y[covered:covered + tail]).any()
            assert torch.isnan(Y[covered + tail:]).all(), "rows behind rows_out were touched"


@pytest.mark.parametrize("fmt", FMTS)
def test_spmm_ones_gives_row_sums(oracle, small, fmt):
    """The reference's own known answer: X = ones -> every column holds the row sums (verification.py:26,43)."""
    from gpu_util import spmm_capi, assert_close

    F = small
    X = torch.ones(F.n + (F.n & 1), 32, device="cuda")
    got = spmm_capi(fmt, F, X, 1, 4)[: F.n]
    rs = np.array([F.val[F.rowPtr[i]:F.rowPtr[i + 1]].astype(np.float64).sum() for i in range(F.n)])
    # the reference's check: |ref - res| <= 1e-4 |ref|, exact zeros must match exactly (verification.py:82-84)
    g = got.cpu().numpy().astype(np.float64)
    assert np.all(np.abs(g - rs[:, None]) <= 1e-4 * np.abs(rs[:, None]))


@pytest.mark.parametrize("fmt", FMTS)
def test_spmm_edge_shapes(oracle, fmt):
    """empty matrix, all rows empty, single row, one very long row, odd row count."""
    from gpu_util import Formats, spmm_capi, spmm_oracle, spmm_abs_scale, assert_close

    cases = {
        "all_empty": (np.zeros(8, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32)),
        "single": (np.array([0, 3], np.int32), np.array([0, 0, 0], np.int32)[:1].repeat(1), np.ones(1, np.float32)),
        "long_row": random_csr(70, 1, 1, hub=(33, 70), values="uniform"),
        "odd_rows": random_csr(129, 9, 2, values="uniform"),
    }
    cases["single"] = (np.array([0, 1], np.int32), np.array([0], np.int32), np.array([2.5], np.float32))
    for name, (rowPtr, colIdx, val) in cases.items():
        print("case", fmt, name, flush=True)
        F = Formats(oracle, rowPtr, colIdx, val)
        X = np.random.default_rng(0).standard_normal((F.n + (F.n & 1), 64)).astype(np.float32)
        got = spmm_capi(fmt, F, torch.from_numpy(X).cuda(), 2, 8)
        torch.cuda.synchronize()
        want = spmm_oracle(oracle, fmt, F, X)
        scale = spmm_abs_scale(oracle, F, X, want.shape[0])
        assert_close(got, want, what=fmt + " " + name, scale=scale)


def test_spmm_bad_arguments_are_errors_not_crashes():
    from paramspmm_ae_amd import _capi

    x = torch.zeros(4, 16, device="cuda")
    rp = torch.zeros(5, dtype=torch.int32, device="cuda")
    p = _capi.ptr
    for CF, bw in ((0, 4), (9, 4), (1, 5)):
        rc = _capi.lib.psp_spmm_csr_f32(p(rp), None, None, p(x), p(x), 4, 16, 4, CF, bw, None)
        assert rc == -1 and _capi.lib.psp_last_error()
    assert _capi.lib.psp_spmm_csr_f32(p(rp), None, None, p(x), p(x), 4, 16, 2, 1, 4, None) == -1  # Y too short


def test_spmm_linearity_and_format_agreement_at_scale(oracle):
    """Size-independent properties on a 2^17-node R-MAT graph (too big for the scalar oracle to be quick at all
    widths): the four formats agree, and A(X1+X2) = AX1 + AX2."""
    from gpu_util import Formats, spmm_capi, assert_close
    from paramspmm_ae_amd import synth

    r, c, n = synth.rmat(17, 8 << 17, seed=5)
    rowPtr, colIdx, val = synth.to_gcn_csr(r, c, n)
    F = Formats(oracle, rowPtr, colIdx, val)
    g = torch.Generator(device="cuda").manual_seed(1)
    X1 = torch.randn(n, 128, device="cuda", generator=g)
    X2 = torch.randn(n, 128, device="cuda", generator=g)
    base = spmm_capi("csr", F, X1, 1, 4)
    scale = spmm_capi("csr", F, X1.abs(), 1, 4).cpu().numpy()  # values are positive: this is |A||X|
    for fmt in FMTS[1:]:
        for CF in (1, 2, 4):
            y = spmm_capi(fmt, F, X1, CF, 8)
            assert_close(y, base.cpu().numpy(), what=fmt, scale=scale)
    lin = spmm_capi("csr", F, X1 + X2, 2, 4)
    assert_close(lin, (base + spmm_capi("csr", F, X2, 2, 4)).cpu().numpy(), rtol=1e-4, atol=1e-5, what="linearity")
    # and one width against the oracle at this size
    want = oracle.spmm_csr(rowPtr, colIdx, val, X1[:, :16].contiguous().cpu().numpy())
    assert_close(spmm_capi("csr", F, X1[:, :16].contiguous(), 1, 4), want, what="rmat17 N=16")


@pytest.fixture
def selective_clear_always():
    """Row-split outputs of any size take the selective-clear path while the test runs."""
    from paramspmm_ae_amd import _capi

    before = _capi.get_option("split_clear_min")
    _capi.set_option("split_clear_min", 0)
    yield
    _capi.set_option("split_clear_min", before)


@pytest.mark.parametrize("long_runs", [False, True])
@pytest.mark.parametrize("fmt", ["csr_split", "bcsr_split"])
def test_split_selective_clear_path(oracle, fmt, long_runs, selective_clear_always):
    """Large outputs of the row-split formats are not cleared as a whole: only rows shared by two wavefronts, rows
    of empty segments and rows without segments are.  Force that path on a small matrix with long rows, empty
    rows at the start, in the middle and at the end (runs of hundreds of rows nothing targets), and a poisoned Y."""
    from gpu_util import Formats, spmm_capi, spmm_oracle, spmm_abs_scale, assert_close

    rowPtr, colIdx, val = random_csr(6000, 14, 21, empty_frac=0.3, hub=(3000, 2500), values="uniform")
    k = np.diff(rowPtr).copy()
    k[:70] = 0
    k[-90:] = 0
    k[1000:1400] = 0
    if long_runs:  # runs far beyond what the wavefront that finds them clears itself: the sweeping wavefronts take over
        k[:600] = 0
        k[1700:4800] = 0
        k[-1100:] = 0
    keep = np.repeat(k > 0, np.diff(rowPtr))
    rowPtr = np.concatenate([[0], np.cumsum(k)]).astype(np.int32)
    colIdx, val = colIdx[keep], val[keep]
    F = Formats(oracle, rowPtr, colIdx, val, g=8, gb=8)
    for N in (16, 128, 50):
        X = np.random.default_rng(N).standard_normal((F.n, N)).astype(np.float32)
        want = spmm_oracle(oracle, fmt, F, X)
        scale = spmm_abs_scale(oracle, F, X, want.shape[0])
        for CF, bw in ((1, 4), (2 if N > 32 else 1, 8)):
            got = spmm_capi(fmt, F, torch.from_numpy(X).cuda(), CF, bw)
            torch.cuda.synchronize()
            assert_close(got, want, what="%s N=%d CF=%d selective clear" % (fmt, N, CF), scale=scale)


@pytest.mark.parametrize("fmt", FMTS)
def test_spmm_local_matrices_both_block_sizes(oracle, fmt):
    """Banded and community-ordered matrices (the structure the cache-friendly configurations have) at both
    workgroup sizes and several column tilings."""
    from gpu_util import Formats, spmm_capi, spmm_oracle, spmm_abs_scale, assert_close
    from paramspmm_ae_amd import synth
    from paramspmm_ae_amd.train_decider import banded

    graphs = {
        "band": banded(20_001, 14, 30, seed=1),
        "sbm": synth.sbm(12_000, 120, 18, 1.5, seed=2),
    }
    for name, (r, c, n) in graphs.items():
        rowPtr, colIdx, val = synth.to_gcn_csr(r, c, n)
        F = Formats(oracle, rowPtr, colIdx, val)
        for N, CF in ((16, 1), (64, 1), (64, 2), (128, 4), (96, 3)):
            print("case", fmt, name, N, CF, flush=True)
            X = np.random.default_rng(N).standard_normal((F.n + (F.n & 1), N)).astype(np.float32)
            want = spmm_oracle(oracle, fmt, F, X)
            scale = spmm_abs_scale(oracle, F, X, want.shape[0])
            Xd = torch.from_numpy(X).cuda()
            got8 = spmm_capi(fmt, F, Xd, CF, 8)
            got4 = spmm_capi(fmt, F, Xd, CF, 4)
            torch.cuda.synchronize()
            assert_close(got8, want, what="%s %s N=%d CF=%d bw=8" % (fmt, name, N, CF), scale=scale)
            assert_close(got4, want, what="%s %s N=%d CF=%d bw=4" % (fmt, name, N, CF), scale=scale)


def test_full_size_headline_graph_properties(oracle):
    """The benchmark's own graph (R-MAT 2^20, 17.9 M entries, hub rows of tens of thousands of entries) at width
    64: X = ones gives the row sums of A (computed on the host in float64), the four formats agree in every
    decider-relevant configuration, and A(X1 + X2) = A X1 + A X2."""
    from gpu_util import Formats, spmm_capi, assert_close
    from paramspmm_ae_amd import synth

    rowPtr, colIdx, val, n = synth.config_graph("C2")
    F = Formats(oracle, rowPtr, colIdx, val)
    rowsum = np.add.reduceat(val.astype(np.float64), rowPtr[:-1].astype(np.int64))
    rowsum[np.diff(rowPtr) == 0] = 0.0
    ones = torch.ones(n, 64, device="cuda")
    for fmt in FMTS:
        y = spmm_capi(fmt, F, ones, 1, 8)[:n]
        assert_close(y, np.repeat(rowsum[:, None], 64, axis=1).astype(np.float32), rtol=2e-5, atol=1e-6, what=fmt + " row sums")
    g = torch.Generator(device="cuda").manual_seed(3)
    X1 = torch.randn(n, 64, device="cuda", generator=g)
    X2 = torch.randn(n, 64, device="cuda", generator=g)
    base = spmm_capi("csr", F, X1, 1, 4)
    scale = spmm_capi("csr", F, X1.abs(), 1, 4).cpu().numpy()
    for fmt, CF, bw in (("csr_split", 1, 4), ("csr_split", 2, 8), ("bcsr", 1, 4), ("bcsr_split", 2, 4), ("csr", 2, 8)):
        assert_close(spmm_capi(fmt, F, X1, CF, bw)[:n], base.cpu().numpy(), what="%s CF=%d bw=%d" % (fmt, CF, bw), scale=scale)
    lin = spmm_capi("csr_split", F, X1 + X2, 1, 8)
    both = spmm_capi("csr_split", F, X1, 1, 8) + spmm_capi("csr_split", F, X2, 1, 8)
    assert_close(lin, both.cpu().numpy(), rtol=1e-4, atol=1e-5, what="linearity at full size")


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("N,CF,bw", [(16, 1, 4), (32, 1, 8), (64, 2, 4), (100, 4, 8), (128, 4, 4), (192, 6, 8), (256, 8, 4), (7, 1, 4)])
def test_spmm_3x1_blocks(oracle, split, N, CF, bw):
    """vec_spmm / vec_split_spmm (3x1 blocks) through the C ABI against the oracle: a row count that is not a multiple
    of 3, a hub row, empty rows; vec_size 2 through the same entry points equals the 2x1 operators."""
    from paramspmm_ae_amd import _capi
    from gpu_util import assert_close, dev, stream

    rowPtr, colIdx, val = random_csr(2999, 8, 13, empty_frac=0.1, hub=(10, 1500))
    n = rowPtr.size - 1
    L, p = _capi.lib, _capi.ptr
    for R in (3, 2):
        rows_out = (n + R - 1) // R * R
        rpb, cib, vb = oracle.vbsr_build(rowPtr, colIdx, val, R, ncols=rows_out)
        X = np.random.default_rng(N).standard_normal((rows_out, N)).astype(np.float32)
        Xd, Y = dev(X), torch.full((rows_out, N), float("nan"), device="cuda")
        scale = oracle.spmm_vec(rpb, cib, np.abs(vb), np.abs(X), rows_out=rows_out)
        # device copies stay referenced until the kernel has run: a pointer taken from a temporary tensor dangles as
        # soon as the caching allocator hands the block to the next allocation
        cib_d, vb_d = dev(cib), dev(vb)
        if split:
            rps, tr = oracle.split_csr(rpb, 8)
            want = oracle.spmm_vec(rps, cib, vb, X, target_row=tr, rows_out=rows_out)
            rps_d, tr_d = dev(rps), dev(tr)
            _capi.check(L.psp_spmm_vec_split_f32(p(rps_d), p(cib_d), p(vb_d), p(tr_d), p(Xd), p(Y), tr.size, N,
                                                 rows_out, R, CF, bw, stream()))
        else:
            want = oracle.spmm_vec(rpb, cib, vb, X, rows_out=rows_out)
            rpb_d = dev(rpb)
            _capi.check(L.psp_spmm_vec_f32(p(rpb_d), p(cib_d), p(vb_d), p(Xd), p(Y), rpb.size - 1, N, rows_out, R,
                                           CF, bw, stream()))
        torch.cuda.synchronize()
        assert_close(Y, want, what="%dx1 blocks N=%d CF=%d split=%s" % (R, N, CF, split), scale=scale)
    # an unsupported block height is an argument error (nothing is launched)
    assert L.psp_spmm_vec_f32(p(cib_d), p(cib_d), p(vb_d), p(Xd), p(Y), 0, N, rows_out, 4, CF, bw, None) == -1


def test_facade_with_3x1_blocks(oracle):
    """graph_input(blk_size=3) + pcsr_spmm(vec_size=3): the reference's generic-block path (PCSR.py:227-239)."""
    from paramspmm_ae_amd import synth
    from paramspmm_ae_amd.graph_input import graph_input
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from gpu_util import assert_close

    r, c, n = synth.chung_lu(5000, 20000, 2.1, seed=3)
    rowPtr, colIdx, val = synth.to_gcn_csr(r, c, n)
    g = graph_input("t", "")
    g.verbose = False
    g.load_from_csr(rowPtr, colIdx, val, blk_size=3)
    rpb, cib, vb = oracle.vbsr_build(rowPtr, colIdx, val, 3, ncols=(n + 2) // 3 * 3)
    assert np.array_equal(g.bcsr_data.colIdx.numpy(), cib) and np.array_equal(g.bcsr_data.val.numpy(), vb)
    assert abs(g.pack_rate - colIdx.size / (3 * cib.size)) < 1e-12
    X = np.random.default_rng(0).standard_normal((n, 48)).astype(np.float32)
    want = oracle.spmm_csr(rowPtr, colIdx, val, X)
    scale = oracle.spmm_csr(rowPtr, colIdx, np.abs(val), np.abs(X))
    for split in (False, True):
        op = pcsr_spmm(g, vec_size=3, if_split=split, CF=2, blkWarpNum=4)
        op.get_spmm_result(x=torch.from_numpy(X))
        assert op.result.shape == (n, 48)
        assert_close(op.result, want, what="facade 3x1 split=%s" % split, scale=scale)
        assert op.profiling(dim=32, verbose=False) > 0
    with pytest.raises(ValueError, match="blk_size"):
        pcsr_spmm(g, vec_size=2, if_split=False)


@pytest.mark.parametrize("fmt", FMTS)
def test_spmm_non_finite_inputs_stay_in_their_rows(oracle, fmt):
    """An Inf and a NaN row of X reach exactly the output rows that reference them (the oracle says which); every
    other element stays finite and equal to the oracle's.  Lanes past the end of a range or of a row must not
    multiply a padding value into a foreign row."""
    from gpu_util import Formats, spmm_capi, spmm_oracle

    rowPtr, colIdx, val = random_csr(1500, 7, 31, empty_frac=0.1, hub=(3, 600), values="uniform")
    F = Formats(oracle, rowPtr, colIdx, val)
    n = F.n
    for N, CF, bw in ((16, 1, 4), (64, 2, 8), (100, 4, 4)):
        X = np.random.default_rng(N).standard_normal((n + (n & 1), N)).astype(np.float32)
        X[colIdx[5]] = np.inf            # a column some rows reference
        X[colIdx[colIdx.size // 2]] = np.nan
        X[n - 1] = np.inf                # the last column: where clamped loads would point
        want = spmm_oracle(oracle, fmt, F, X)
        got = spmm_capi(fmt, F, torch.from_numpy(X).cuda(), CF, bw).cpu().numpy()
        assert np.array_equal(np.isnan(got), np.isnan(want)), (fmt, N)
        assert np.array_equal(np.isposinf(got), np.isposinf(want)) and np.array_equal(np.isneginf(got), np.isneginf(want))
        fin = np.isfinite(want)
        np.testing.assert_allclose(got[fin], want[fin], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("fmt", FMTS)
def test_spmm_native_configurations(oracle, fmt):
    """The wave64 parameter space carried in the CF argument (lanes per row, vectors per lane, entries in flight,
    segments per wavefront, even division) against the oracle: every combination the sweep can emit, on a matrix
    with a hub row, empty rows and an odd row count, at widths with and without a partial column tile."""
    from gpu_util import Formats, spmm_capi, spmm_oracle, spmm_abs_scale, assert_close
    from paramspmm_ae_amd import _capi
    from paramspmm_ae_amd.sweep import native_configs

    rowPtr, colIdx, val = random_csr(3001, 9, 77, empty_frac=0.15, hub=(17, 1900), values="normal")
    F = Formats(oracle, rowPtr, colIdx, val)
    for N in (16, 48, 100, 128, 256):
        X = np.random.default_rng(N).standard_normal((F.n + (F.n & 1), N)).astype(np.float32)
        want = spmm_oracle(oracle, fmt, F, X)
        scale = spmm_abs_scale(oracle, F, X, want.shape[0])
        Xd = torch.from_numpy(X).cuda()
        cfs = list(native_configs(N))
        # beyond the sweep's list: odd corners of the space
        cfs += [_capi.pack_cf(1, 1, 1), _capi.pack_cf(1, 64, 1, 1), _capi.pack_cf(1, 2, 2, 64, even_split=True),
                _capi.pack_cf(3, 8, 2, 4), _capi.pack_cf(8, 4, 1, 2)]
        for cf in cfs:
            for bw in (4, 8):
                print("case", fmt, N, _capi.unpack_cf(cf), bw, flush=True)
                got = spmm_capi(fmt, F, Xd, cf, bw)
                torch.cuda.synchronize()
                assert_close(got, want, what="%s N=%d native %s bw=%d" % (fmt, N, _capi.unpack_cf(cf), bw), scale=scale)
    # malformed native values are argument errors
    p = _capi.ptr
    x = torch.zeros(4, 16, device="cuda")
    rp = torch.zeros(5, dtype=torch.int32, device="cuda")
    for bad in (_capi.CF_NATIVE | (7 << 3), _capi.CF_NATIVE | (1 << 13), _capi.pack_cf(4, 8, 2) | (3 << 6),
                _capi.CF_NATIVE | (2 << 6) | (1 << 3)):
        assert _capi.lib.psp_spmm_csr_f32(p(rp), None, None, p(x), p(x), 4, 16, 4, bad, 4, None) == -1


@pytest.mark.parametrize("fmt", FMTS)
def test_spmm_xcd_stripe_flag(oracle, fmt):
    """blkWarpNum | PSP_BW_STRIPE(rows) only changes which workgroup takes which rows: plain layouts give the same
    bits for every stripe, row-split ones agree with the oracle (their atomics add in launch order)."""
    from gpu_util import Formats, spmm_capi, spmm_oracle, spmm_abs_scale, assert_close
    from paramspmm_ae_amd import _capi

    rowPtr, colIdx, val = random_csr(40013, 7, 5, empty_frac=0.05, hub=(31, 2500), values="normal")
    F = Formats(oracle, rowPtr, colIdx, val)
    for N in (16, 96):
        X = np.random.default_rng(N).standard_normal((F.n + (F.n & 1), N)).astype(np.float32)
        want = spmm_oracle(oracle, fmt, F, X)
        scale = spmm_abs_scale(oracle, F, X, want.shape[0])
        Xd = torch.from_numpy(X).cuda()
        base = spmm_capi(fmt, F, Xd, 1, 4)
        for rows in (256, 768, 1536, 6144, 65280):
            print("case", fmt, N, rows, flush=True)
            got = spmm_capi(fmt, F, Xd, 1, 4 | _capi.bw_stripe(rows))
            torch.cuda.synchronize()
            assert_close(got, want, what="%s N=%d stripe %d" % (fmt, N, rows), scale=scale)
            if "split" not in fmt:
                assert torch.equal(got, base)
    p = _capi.ptr
    x = torch.zeros(4, 16, device="cuda")
    rp = torch.zeros(5, dtype=torch.int32, device="cuda")
    assert _capi.lib.psp_spmm_csr_f32(p(rp), None, None, p(x), p(x), 4, 16, 4, 1, 4 | (1 << 20), None) == -1


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.int32)


@pytest.mark.parametrize("fmt", ["csr", "bcsr"])
def test_spmm_whole_rows_mode_repeats_the_sequential_fma_chain_bit_for_bit(oracle, small, fmt):
    """Option "whole_rows": no row is cut between lane groups, so every output element is the reference's chain
    res = fma(val[p], X[col[p]], res) over the row's entries in storage order (SpMM_kernel.cu:1157-1212; 2x1 blocks
    1362-1440 with their zero entries skipped) -- and the result must equal the oracle's bit pattern, not merely lie
    within the tolerance.  Matrices: the fixture with a 900-entry hub row, empty rows and an odd row count, and the
    pubmed-sized Chung-Lu graph; reference CF values and native wave64 configurations."""
    from gpu_util import Formats, spmm_capi, spmm_oracle
    from oracle.oracle import CF_TABLE
    from paramspmm_ae_amd import _capi, synth

    rowPtr, colIdx, val, _ = synth.config_graph("C1")
    cases = [("small", small, (16, 64, 100, 128, 256)), ("C1", Formats(oracle, rowPtr, colIdx, val), (16, 64, 100))]
    assert _capi.get_option("whole_rows") == 0
    _capi.set_option("whole_rows", 1)
    try:
        for name, F, widths in cases:
            for N in widths:
                X = np.random.default_rng(N).standard_normal((F.n + (F.n & 1), N)).astype(np.float32)
                want = _bits(spmm_oracle(oracle, fmt, F, X))
                Xd = torch.from_numpy(X).cuda()
                cfs = list(CF_TABLE.get(N, (1, 2, 4))) + [_capi.pack_cf(1, 4, 2), _capi.pack_cf(2, 16, 1), _capi.pack_cf(1, 8, 4, 4)]
                for cf in cfs:
                    for bw in (4, 8):
                        print("case", name, fmt, N, cf, bw, flush=True)
                        got = _bits(spmm_capi(fmt, F, Xd, cf, bw).cpu().numpy())
                        differ = int(np.count_nonzero(got != want))
                        assert differ == 0, "%s %s N=%d CF=%d bw=%d: %d of %d elements differ in their bits" % (
                            name, fmt, N, cf, bw, differ, want.size)
    finally:
        _capi.set_option("whole_rows", 0)


@pytest.mark.parametrize("fmt", FMTS)
def test_spmm_default_mode_share_outside_the_literal_tolerance(oracle, small, fmt, capsys):
    """Default mode (rows may be cut between lane groups): the share of elements outside the literal
    |got - want| <= 1e-6 + 1e-5 |want| against the sequential chain is printed and bounded; rows of one or two stored
    entries always meet it (cut in two, such a row differs from the chain by one extra rounding of a single product)."""
    from gpu_util import Formats, spmm_capi, spmm_oracle
    from paramspmm_ae_amd import synth

    rowPtr, colIdx, val, _ = synth.config_graph("C1")
    for name, F, widths in (("small", small, (16, 64, 128, 256)), ("C1", Formats(oracle, rowPtr, colIdx, val), (16, 64))):
        short = np.diff(F.rowPtr) <= 2
        for N in widths:
            X = np.random.default_rng(N).standard_normal((F.n + (F.n & 1), N)).astype(np.float32)
            want = spmm_oracle(oracle, fmt, F, X)[: F.n]
            got = spmm_capi(fmt, F, torch.from_numpy(X).cuda(), 1, 4).cpu().numpy()[: F.n]
            outside = np.abs(got.astype(np.float64) - want) > 1e-6 + 1e-5 * np.abs(want.astype(np.float64))
            share = float(outside.mean())
            with capsys.disabled():
                print("literal tolerance, default mode: %-5s %-10s N=%-3d outside %d of %d (%.2e), bit-identical %.4f"
                      % (name, fmt, N, int(outside.sum()), outside.size, share, float((_bits(got) == _bits(want)).mean())))
            assert share <= 1e-4, (name, fmt, N, share)
            assert not outside[short].any()


@pytest.mark.parametrize("N,lanes", [(48, 16), (16, 4), (80, 32), (128, 8)])
def test_gather_probe_reads_the_rows_the_pattern_names(N, lanes):
    """psp_probe_gather_f32 (the measurement aid behind the bench's gather ceiling): the column sums of what its lanes
    accumulated equal the sums of the gathered X rows -- also at widths where the upper lanes of a lane group have no
    column (N = 48 on 16 lanes), whose index entries must still reach the other lanes."""
    from paramspmm_ae_amd import _capi

    L, p = _capi.lib, _capi.ptr
    rng = np.random.default_rng(N)
    n, nnz = 5000, 70001
    col = rng.integers(0, n, nnz).astype(np.int32)
    X = rng.standard_normal((n, N)).astype(np.float32)
    want = X.astype(np.float64)[col].sum(axis=0)
    cd, Xd = torch.from_numpy(col).cuda(), torch.from_numpy(X).cuda()
    for unroll in (1, 4):
        if unroll > lanes:
            continue
        per_wave = 512
        need = L.psp_probe_gather_out_floats(nnz, N, lanes, per_wave)
        out = torch.zeros(need, device="cuda")
        _capi.check(L.psp_probe_gather_f32(p(cd), nnz, p(Xd), N, lanes, unroll, per_wave, p(out), need,
                                           torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        tiles = (N // 4 + lanes - 1) // lanes
        o = out.cpu().numpy().astype(np.float64).reshape(tiles, -1, 64 // lanes, lanes, 4)  # tile, wave, group, sub, e
        got = o.sum(axis=(1, 2)).reshape(tiles * lanes * 4)[:N]
        assert np.allclose(got, want, rtol=1e-4, atol=1e-2), (N, lanes, unroll, np.abs(got - want).max())
        assert not o.sum(axis=(1, 2)).reshape(-1)[N:].any()  # lanes without a column report nothing
