"""GPU tests of the device-side PCSR builders (row split, 2x1 BCSR) through the C ABI: bit-exact against the CPU
oracle, SciPy's tobsr (the routine the reference calls, graph_input.py:245-256) and the host builders."""
import numpy as np
import pytest
import torch

from conftest import random_csr, pubmed_pattern

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def split_dev(rowPtr, g):
    from paramspmm_ae_amd import device_builder

    rs, tr = device_builder.split_csr_device(dev(rowPtr), g)
    return rs.cpu().numpy(), tr.cpu().numpy()


def bcsr_dev(rowPtr, colIdx, val):
    from paramspmm_ae_amd import device_builder

    return tuple(t.cpu().numpy() for t in device_builder.build_bcsr_device(dev(rowPtr), dev(colIdx), dev(val)))


CASES = [
    dict(n=1, avg_deg=1.0, seed=0),
    dict(n=2, avg_deg=1.5, seed=1),
    dict(n=257, avg_deg=6.0, seed=2, empty_frac=0.3),
    dict(n=3000, avg_deg=9.0, seed=3, hub=(17, 2500)),         # a row far longer than a wavefront
    dict(n=3001, avg_deg=4.0, seed=4, empty_frac=0.1, hub=(3000, 700)),  # odd row count, hub in the unpaired row
    dict(n=5000, avg_deg=0.2, seed=5, empty_frac=0.5),          # mostly empty
    dict(n=20000, avg_deg=3.0, seed=6, hub=(1001, 9000)),       # a block-row built by a whole workgroup, several rounds
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "n%d" % c["n"])
@pytest.mark.parametrize("g", [1, 3, 32])
def test_split_matches_oracle(oracle, case, g):
    rowPtr, _, _ = random_csr(**case)
    want_rs, want_tr = oracle.split_csr(rowPtr, g)
    got_rs, got_tr = split_dev(rowPtr, g)
    assert got_rs.dtype == np.int32 and got_tr.dtype == np.int32
    assert np.array_equal(got_rs, want_rs)
    assert np.array_equal(got_tr, want_tr)


@pytest.mark.parametrize("case", CASES, ids=lambda c: "n%d" % c["n"])
def test_bcsr_matches_oracle_and_scipy(oracle, case):
    import scipy.sparse as sp

    rowPtr, colIdx, val = random_csr(**case)
    n = rowPtr.size - 1
    want = oracle.bcsr_build(rowPtr, colIdx, val)
    got = bcsr_dev(rowPtr, colIdx, val)
    for a, b in zip(got, want):
        assert a.dtype == b.dtype and np.array_equal(a, np.asarray(b).reshape(a.shape))
    # SciPy on the matrix padded to an even row count, as graph_input.py:248-255 does
    ne = n + (n & 1)
    ip = np.concatenate([rowPtr, [rowPtr[-1]] * (ne - n)]).astype(np.int32)
    bsr = sp.csr_matrix((val, colIdx, ip), shape=(ne, ne)).tobsr(blocksize=(2, 1))
    assert np.array_equal(got[0], bsr.indptr)
    assert np.array_equal(got[1], bsr.indices)
    assert np.array_equal(got[2], bsr.data.reshape(-1, 2))


def test_empty_matrix():
    rs, tr = split_dev(np.zeros(1, np.int32), 4)
    assert rs.tolist() == [0] and tr.size == 0
    rowPtr = np.zeros(6, np.int32)
    rb, cb, vb = bcsr_dev(rowPtr, np.zeros(0, np.int32), np.zeros(0, np.float32))
    assert rb.tolist() == [0, 0, 0, 0] and cb.size == 0 and vb.shape == (0, 2)
    rs, tr = split_dev(rowPtr, 4)
    assert rs.tolist() == [0] and tr.size == 0


def test_pubmed_counts(oracle):
    """Segment and block counts of the reference's data files (computed from the .mtx files with SciPy)."""
    from paramspmm_ae_amd import synth

    for which, nblk, s_csr in (("orig", 88469, 20005), ("rabbit", 81018, None)):
        m = pubmed_pattern(which)
        rowPtr, colIdx = m.indptr.astype(np.int32), m.indices.astype(np.int32)
        val = np.ones(colIdx.size, np.float32)
        rb, cb, vb = bcsr_dev(rowPtr, colIdx, val)
        assert cb.size == nblk
        want = oracle.bcsr_build(rowPtr, colIdx, val)
        assert np.array_equal(cb, want[1]) and np.array_equal(vb, np.asarray(want[2]).reshape(-1, 2))
        if s_csr is not None:
            rs, tr = split_dev(rowPtr, 32)
            assert tr.size == s_csr


def test_unsorted_rows_are_reported():
    from paramspmm_ae_amd import device_builder

    rowPtr = np.array([0, 3, 5], np.int32)
    colIdx = np.array([0, 2, 1, 0, 1], np.int32)  # row 0 is out of order
    val = np.ones(5, np.float32)
    with pytest.raises(device_builder.NotCanonical):
        device_builder.build_bcsr_device(dev(rowPtr), dev(colIdx), dev(val))
    colIdx = np.array([0, 1, 1, 0, 1], np.int32)  # duplicate column
    with pytest.raises(device_builder.NotCanonical):
        device_builder.build_bcsr_device(dev(rowPtr), dev(colIdx), dev(val))
    with pytest.raises(ValueError):
        device_builder.split_csr_device(dev(np.array([0, 3, 2], np.int32)), 2)


def test_full_size_graph_matches_host_builders():
    """R-MAT 2^20 (scan over several hundred tiles, hub rows of tens of thousands of entries)."""
    from paramspmm_ae_amd import synth, _capi
    from paramspmm_ae_amd.graph_input import build_bcsr
    import ParamSpMM

    rowPtr, colIdx, val = synth.config_graph("C2")[:3]
    n = rowPtr.size - 1
    got = bcsr_dev(rowPtr, colIdx, val)
    want = build_bcsr(rowPtr, colIdx, val, build_on="host")
    for a, b in zip(got, want):
        assert np.array_equal(a, b)
    for g in (8, 32):
        k = np.diff(rowPtr)
        off = np.zeros(n + 1, np.int32)
        off[1:] = np.cumsum((k + g - 1) // g)
        want_rs, want_tr = ParamSpMM.split_csr_par(torch.from_numpy(rowPtr), torch.from_numpy(off), g)
        got_rs, got_tr = split_dev(rowPtr, g)
        assert np.array_equal(got_rs, want_rs.numpy()) and np.array_equal(got_tr, want_tr.numpy())


def test_graph_input_same_on_host_and_device():
    from paramspmm_ae_amd import synth
    from paramspmm_ae_amd.graph_input import graph_input

    r, c, n = synth.chung_lu(20_001, 90_000, 2.1, seed=5)
    rowPtr, colIdx, val = synth.to_gcn_csr(r, c, n)
    gs = []
    for where in ("host", "device"):
        g = graph_input("t", "")
        g.verbose = False
        g.load_from_csr(rowPtr, colIdx, val, if_mask=True, build_on=where)
        gs.append(g)
    h, d = gs
    for fmt in ("csr_data", "bcsr_data"):
        for name in ("rowPtr", "colIdx", "val", "rowPtr_split", "target_row"):
            a, b = getattr(getattr(h, fmt), name), getattr(getattr(d, fmt), name)
            assert a.dtype == b.dtype and a.shape == b.shape and torch.equal(a, b), (fmt, name)
    assert torch.equal(h.mask, d.mask)
    assert np.array_equal(h.get_info(), d.get_info())


def test_index_check_reports_what_would_fault():
    """psp_check_index_dev: arrays that would make the SpMM / SDDMM kernels leave their buffers are reported."""
    from paramspmm_ae_amd import device_builder
    from paramspmm_ae_amd.PCSR import pcsr_spmm

    rowPtr, colIdx, val = random_csr(3000, 5.0, 1, empty_frac=0.2)
    n = rowPtr.size - 1
    device_builder.check_index(dev(rowPtr), dev(colIdx), n)  # fine
    bad = colIdx.copy()
    bad[bad.size // 2] = n
    with pytest.raises(ValueError, match="column index"):
        device_builder.check_index(dev(rowPtr), dev(bad), n)
    bad[bad.size // 2] = -1
    with pytest.raises(ValueError, match="column index"):
        device_builder.check_index(dev(rowPtr), dev(bad), n)
    rp = rowPtr.copy()
    rp[10] = rp[11] + 1
    with pytest.raises(ValueError, match="rowPtr"):
        device_builder.check_index(dev(rp), dev(colIdx), n)
    rp = rowPtr.copy()
    rp[-1] -= 1
    with pytest.raises(ValueError, match="rowPtr"):
        device_builder.check_index(dev(rp), dev(colIdx), n)
    rs, tr = split_dev(rowPtr, 4)
    device_builder.check_index(dev(rs), dev(colIdx), n, dev(tr), n)
    tr_bad = tr.copy()
    tr_bad[5], tr_bad[6] = tr_bad[6] + 1, tr_bad[5]
    with pytest.raises(ValueError, match="target_row"):
        device_builder.check_index(dev(rs), dev(colIdx), n, dev(tr_bad), n)
    # the facade checks arrays it is handed directly
    with pytest.raises(ValueError, match="column index"):
        pcsr_spmm(None, 1, False, mtx_nodes=n, mtx_edges=colIdx.size, rowPtr=torch.from_numpy(rowPtr),
                  colIdx=torch.from_numpy(np.where(np.arange(colIdx.size) == 7, n + 5, colIdx).astype(np.int32)),
                  val=torch.from_numpy(val))
    op = pcsr_spmm(None, 1, False, mtx_nodes=n, mtx_edges=colIdx.size, rowPtr=torch.from_numpy(rowPtr),
                   colIdx=torch.from_numpy(colIdx), val=torch.from_numpy(val))
    assert op.colIdx.is_cuda
