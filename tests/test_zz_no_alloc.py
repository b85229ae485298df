"""The entry point that allocates nothing (psp_segment_softmax_static_f32) against the workspace form it is a
variant of (psp_segment_softmax_ws_f32), through the C ABI: two calls in a row, the second on a smaller input, so
that what the first call left in the library's built-in scratch array must not leak into the second."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _rows_with_hubs(n, seed, hubs):
    rng = np.random.default_rng(seed)
    deg = rng.poisson(9, n)
    deg[rng.random(n) < 0.05] = 0
    mid = rng.choice(n, max(4, n // 200), replace=False)
    deg[mid] = rng.integers(129, 900, mid.size)  # rows just past the short-row limit of 128 entries
    for r, d in hubs:
        deg[r] = d
    rowPtr = np.zeros(n + 1, np.int32)
    rowPtr[1:] = np.cumsum(deg)
    e = (rng.standard_normal(int(rowPtr[-1])) * 4).astype(np.float32)
    return rowPtr, e


def _both(rowPtr, e):
    from paramspmm_ae_amd import _capi
    from gpu_util import dev, stream

    p = _capi.ptr
    M, nnz = rowPtr.size - 1, e.size
    rp, ed = dev(rowPtr), dev(e)
    ws = torch.full((2 * M,), float("nan"), device="cuda")
    want = torch.full((nnz,), float("nan"), device="cuda")
    got = torch.full((nnz,), float("nan"), device="cuda")
    _capi.check(_capi.lib.psp_segment_softmax_ws_f32(p(rp), p(ed), p(want), M, nnz, p(ws), stream()))
    _capi.check(_capi.lib.psp_segment_softmax_static_f32(p(rp), p(ed), p(got), M, nnz, stream()))
    torch.cuda.synchronize()
    return got.cpu().numpy(), want.cpu().numpy()


def test_static_scratch_softmax_matches_workspace_form_twice(oracle):
    from gpu_util import assert_close

    print("case: psp_segment_softmax_static_f32, n=60000 then n=7001", flush=True)
    first = _rows_with_hubs(60000, 11, hubs=((5, 70000), (59999, 20011), (31000, 4097)))
    second = _rows_with_hubs(7001, 12, hubs=((0, 9000), (7000, 131)))
    for rowPtr, e in (first, second):
        got, want = _both(rowPtr, e)
        # rows of up to 128 entries never touch the scratch array: identical bits
        k = np.diff(rowPtr)
        short = np.repeat(k <= 128, k)
        assert np.array_equal(got[short], want[short])
        # long rows add their sum with fp32 atomics in both forms: the stated fp32 tolerance
        assert_close(got, want, rtol=1e-5, atol=1e-6, what="static vs workspace")
        assert_close(got, oracle.segment_softmax(rowPtr, e), rtol=1e-5, atol=1e-6, what="static vs oracle")
        sums = np.add.reduceat(got.astype(np.float64), rowPtr[:-1][k > 0])
        assert np.allclose(sums, 1.0, atol=1e-4)


def test_static_scratch_softmax_rejects_more_rows_than_the_scratch_holds():
    from paramspmm_ae_amd import _capi
    from gpu_util import stream

    limit = 1 << 21
    one = torch.zeros(1, device="cuda")
    rp = torch.zeros(2, dtype=torch.int32, device="cuda")
    p = _capi.ptr
    rc = _capi.lib.psp_segment_softmax_static_f32(p(rp), p(one), p(one), limit + 1, 1, stream())
    assert rc == -1 and b"exceed" in _capi.lib.psp_last_error()
    # empty input: accepted, nothing launched
    assert _capi.lib.psp_segment_softmax_static_f32(p(rp), p(one), p(one), 0, 0, stream()) == 0


def test_static_scratch_softmax_at_the_row_limit_exactly(oracle):
    """M = PSP_SEGMENT_SOFTMAX_STATIC_MAX_ROWS is accepted and uses the last pair of the scratch array: a long row
    placed last reads and writes scratch[2 * (M - 1)] and the float after it."""
    from gpu_util import assert_close

    M = 1 << 21
    deg = np.ones(M, np.int64)
    deg[M - 1] = 3000
    deg[7] = 500
    rowPtr = np.zeros(M + 1, np.int32)
    rowPtr[1:] = np.cumsum(deg)
    e = (np.random.default_rng(3).standard_normal(int(rowPtr[-1])) * 3).astype(np.float32)
    print("case: psp_segment_softmax_static_f32 at M = 2^21", flush=True)
    got, want = _both(rowPtr, e)
    assert_close(got, want, rtol=1e-5, atol=1e-6, what="static vs workspace at the limit")
    assert np.all(got[: 7] == 1.0)  # rows of one entry
    for r in (7, M - 1):
        seg = slice(rowPtr[r], rowPtr[r + 1])
        assert_close(got[seg], oracle.segment_softmax(np.array([0, deg[r]], np.int32), e[seg]), rtol=1e-5, atol=1e-6)


def test_static_scratch_softmax_replays_in_a_hip_graph():
    """After one eager call on the device (the address lookup), the entry point is kernel launches only: captured
    into a HIP graph on a side stream and replayed three times, with eager work on other inputs between the replays,
    every replay gives the workspace form's result for the inputs the buffers hold at that time."""
    from paramspmm_ae_amd import _capi
    from gpu_util import assert_close, dev

    p = _capi.ptr
    rowPtr, e0 = _rows_with_hubs(30000, 21, hubs=((3, 50000), (29999, 700)))
    M, nnz = rowPtr.size - 1, e0.size
    rp, ed = dev(rowPtr), dev(e0)
    out = torch.full((nnz,), float("nan"), device="cuda")
    # the eager call that does the lookup: empty, launches nothing
    assert _capi.lib.psp_segment_softmax_static_f32(None, None, None, 0, 0, torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    print("case: capture of psp_segment_softmax_static_f32", flush=True)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        rc = _capi.lib.psp_segment_softmax_static_f32(p(rp), p(ed), p(out), M, nnz, torch.cuda.current_stream().cuda_stream)
    _capi.check(rc)
    rng = np.random.default_rng(5)
    for k in range(3):
        e = (rng.standard_normal(nnz) * (2 + k)).astype(np.float32)
        ed.copy_(torch.from_numpy(e))
        out.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        # eager work between the replays: the workspace form on the same input, and a call on another matrix that
        # overwrites the shared scratch array
        ws = torch.empty(2 * M, device="cuda")
        want = torch.empty(nnz, device="cuda")
        _capi.check(_capi.lib.psp_segment_softmax_ws_f32(p(rp), p(ed), p(want), M, nnz, p(ws), torch.cuda.current_stream().cuda_stream))
        other_rp, other_e = _rows_with_hubs(5000, 30 + k, hubs=((1, 9000),))
        _both(other_rp, other_e)
        torch.cuda.synchronize()
        assert_close(got, want.cpu().numpy(), rtol=1e-5, atol=1e-6, what="replay %d" % k)
