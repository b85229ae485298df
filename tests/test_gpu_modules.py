"""GPU tests of the PyTorch extension modules (ParamSpMM / ParamSDDMM / ParamSpCONV), the pcsr_spmm facade,
the format builder with its device-side mask, and the GNN layers against dense torch autograd."""
import os

import numpy as np
import pandas as pd
import pytest
import torch

from conftest import random_csr

pytestmark = pytest.mark.gpu

VARIANTS = [(1, False), (1, True), (2, False), (2, True)]


def sym_graph(n, seed):
    """Symmetric normalised test graph as a loaded graph_input (values D^-1/2 (A+I) D^-1/2)."""
    from paramspmm_ae_amd import synth
    from paramspmm_ae_amd.graph_input import graph_input

    rng = np.random.default_rng(seed)
    m = n * 4
    r, c = rng.integers(0, n, m), rng.integers(0, n, m)
    keep = r != c
    rowPtr, colIdx, val = synth.to_gcn_csr(r[keep], c[keep], n)
    g = graph_input("t", "")
    g.verbose = False
    g.load_from_csr(rowPtr, colIdx, val, if_mask=True)
    return g, rowPtr, colIdx, val


def dense(rowPtr, colIdx, val, n):
    A = torch.zeros(n, n, dtype=torch.float64)
    rows = np.repeat(np.arange(n), np.diff(rowPtr))
    A[torch.from_numpy(rows), torch.from_numpy(colIdx.astype(np.int64))] = torch.from_numpy(val.astype(np.float64))
    return A


@pytest.mark.parametrize("n", [257, 300])
def test_facade_dispatch_matrix(oracle, n):
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from gpu_util import assert_close

    g, rowPtr, colIdx, val = sym_graph(n, n)
    rows = (n + 1) // 2 * 2
    X = np.random.default_rng(1).standard_normal((rows, 64)).astype(np.float32)
    X[n:] = 0
    Xd = torch.from_numpy(X).cuda()
    want = oracle.spmm_csr(rowPtr, colIdx, val, X)
    scale = oracle.spmm_csr(rowPtr, colIdx, np.abs(val), np.abs(X))
    A = X / np.maximum(np.linalg.norm(X, axis=1, keepdims=True), 1e-9)
    Ad = torch.from_numpy(A).cuda()
    sd = oracle.sddmm_csr(rowPtr, colIdx, A, A)
    for vec, split in VARIANTS:
        op = pcsr_spmm(g, vec_size=vec, if_split=split, CF=2, blkWarpNum=8)
        y = op.GIN_spmm(Xd)
        assert y.shape[0] == rows and bool((y[n:] == 0).all())
        assert_close(y[:n], want[:n], what="GIN_spmm %d %s" % (vec, split), scale=scale[:n])
        op.get_spmm_result(x=Xd[:n].contiguous() if vec == 1 else Xd)
        assert op.result.shape[0] == n and op.result.device.type == "cpu"
        assert_close(op.result, want[:n], what="get_spmm_result", scale=scale[:n])
        e = op.AGNN_sddmm(Ad)
        if vec == 2:
            assert e.shape == (op.colIdx.numel(), 2)
            e = e.view(-1)[op.mask]
            # block order inside odd rows differs from CSR order: compare row-wise sorted
            ecpu = e.cpu().numpy()
            for r in range(n):
                a, b = rowPtr[r], rowPtr[r + 1]
                np.testing.assert_allclose(np.sort(ecpu[a:b]), np.sort(sd[a:b]), rtol=1e-5, atol=1e-6)
        else:
            assert_close(e, sd, what="AGNN_sddmm")
        # SpMM with per-entry values in the variant's own layout equals SpMM of the matrix those values form
        ev = op.val * 0.5
        y2 = op.AGNN_spmm(ev, Xd)
        assert_close(y2[:n], 0.5 * want[:n], what="AGNN_spmm", scale=scale[:n])
        assert op.profiling(dim=16, verbose=False) > 0


def test_extension_argument_errors():
    import paramspmm_ae_amd  # noqa: F401
    import ParamSpMM
    import ParamSDDMM

    x = torch.zeros(8, 16, device="cuda")
    rp = torch.zeros(9, dtype=torch.int32, device="cuda")
    ci = torch.zeros(0, dtype=torch.int32, device="cuda")
    v = torch.zeros(0, device="cuda")
    assert ParamSpMM.csr_spmm(x, rp, ci, v, 1, 4).shape == (8, 16)
    with pytest.raises(RuntimeError, match="CF must be"):
        ParamSpMM.csr_spmm(x, rp, ci, v, 9, 4)
    with pytest.raises(RuntimeError, match="blkWarpNum must be 4 or 8"):
        ParamSpMM.csr_spmm(x, rp, ci, v, 1, 6)
    with pytest.raises(RuntimeError, match="contiguous"):
        ParamSpMM.csr_spmm(torch.zeros(16, 8, device="cuda").t(), rp, ci, v, 1, 4)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ParamSpMM.csr_spmm(x.cpu(), rp, ci, v, 1, 4)
    with pytest.raises(RuntimeError, match="int32"):
        ParamSpMM.csr_spmm(x, rp.long(), ci, v, 1, 4)
    with pytest.raises(RuntimeError, match="share one dtype"):
        ParamSpMM.csr_spmm(x.double(), rp, ci, v, 1, 4)
    with pytest.raises(RuntimeError, match="float32 or float64"):
        ParamSpMM.csr_spmm(x.half(), rp, ci, v.half(), 1, 4)
    assert ParamSpMM.csr_spmm(x.double(), rp, ci, v.double(), 1, 4).dtype == torch.float64
    assert torch.count_nonzero(ParamSpMM.gespmm_compute(x, rp, ci, v)) == 0
    with pytest.raises(RuntimeError, match=r"\[nblk, 3\]"):
        ParamSDDMM.vec_sddmm(x, x, rp, ci, torch.zeros(0, 5, device="cuda"), 1, 4)
    with pytest.raises(RuntimeError, match="same number of columns"):
        ParamSDDMM.csr_sddmm(x, torch.zeros(8, 8, device="cuda"), rp, ci, v, 1, 4)
    # odd row count and an unpadded A: the row-split block operators refuse it like the plain ones (the kernel
    # reads both rows of the last block-row)
    a7, b7 = torch.zeros(7, 16, device="cuda"), torch.zeros(7, 16, device="cuda")
    rps = torch.tensor([0, 1], dtype=torch.int32, device="cuda")
    tr = torch.tensor([3], dtype=torch.int32, device="cuda")
    ci1 = torch.tensor([2], dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="two rows per block-row"):
        ParamSDDMM.bcsr_sddmm(a7, b7, torch.tensor([0, 0, 0, 0, 1], dtype=torch.int32, device="cuda"), ci1,
                              torch.ones(1, 2, device="cuda"), 1, 4)
    with pytest.raises(RuntimeError, match="two rows per block-row"):
        ParamSDDMM.bcsr_split_sddmm(a7, b7, rps, ci1, torch.ones(1, 2, device="cuda"), tr, 1, 4)
    with pytest.raises(RuntimeError, match="vec_size rows per block-row"):
        ParamSDDMM.vec_split_sddmm(a7, b7, rps, ci1, torch.ones(1, 3, device="cuda"),
                                   torch.tensor([2], dtype=torch.int32, device="cuda"), 1, 4)
    a8 = torch.ones(8, 16, device="cuda")
    got = ParamSDDMM.bcsr_split_sddmm(a8, torch.ones(7, 16, device="cuda"), rps, ci1,
                                      torch.tensor([[1.0, 0.0]], device="cuda"), tr, 1, 4)
    assert got.tolist() == [[16.0, 0.0]]
    # bcsr output is padded to an even number of rows
    xo = torch.zeros(7, 16, device="cuda")
    rpb = torch.zeros(5, dtype=torch.int32, device="cuda")
    assert ParamSpMM.bcsr_spmm(xo, rpb, ci, torch.zeros(0, 2, device="cuda"), 1, 4).shape == (8, 16)


@pytest.mark.parametrize("N", [16, 33, 130, 256, 1030])
def test_row_caching_baseline_matches_oracle(oracle, N):
    """gespmm_compute: the comparison baseline (one wavefront per row, entries cached in LDS) computes the same
    product; a hub row longer than the cache and empty rows included."""
    import ParamSpMM
    from gpu_util import assert_close

    rowPtr, colIdx, val = random_csr(1501, 7.0, seed=N, empty_frac=0.2, hub=(5, 1300))
    X = np.random.default_rng(N).standard_normal((1501, N)).astype(np.float32)
    want = oracle.spmm_csr(rowPtr, colIdx, val, X)
    scale = oracle.spmm_csr(rowPtr, colIdx, np.abs(val), np.abs(X))
    got = ParamSpMM.gespmm_compute(torch.from_numpy(X).cuda(), torch.from_numpy(rowPtr).cuda(),
                                   torch.from_numpy(colIdx).cuda(), torch.from_numpy(val).cuda())
    assert_close(got, want, what="row-caching baseline N=%d" % N, scale=scale)
    if N == 16:
        assert ParamSpMM.gespmm_profile(torch.from_numpy(X).cuda(), torch.from_numpy(rowPtr).cuda(),
                                        torch.from_numpy(colIdx).cuda(), torch.from_numpy(val).cuda()) > 0


def test_spconv_forward_backward(oracle):
    import paramspmm_ae_amd  # noqa: F401
    import ParamSpCONV
    from paramspmm_ae_amd.PCSR import pcsr_spmm

    n = 301
    g, rowPtr, colIdx, val = sym_graph(n, 4)
    A = dense(rowPtr, colIdx, val, n)
    H = torch.randn(n, 24, dtype=torch.float64)
    W = torch.randn(24, 48, dtype=torch.float64) * 0.2
    dY = torch.randn(n, 48, dtype=torch.float64)
    fwd = A @ (H @ W)
    AG = A @ dY
    dH, dW = AG @ W.t(), H.t() @ AG
    for vec, split in VARIANTS:
        op = pcsr_spmm(g, vec_size=vec, if_split=split, CF=1, blkWarpNum=4)
        out = op.forward(H.float().cuda(), W.float().cuda())
        assert out.shape == (n, 48)
        torch.testing.assert_close(out.cpu().double(), fwd, rtol=1e-4, atol=1e-5)
        gi, gw = op.backward(dY.float().cuda(), H.float().cuda(), W.float().cuda())
        torch.testing.assert_close(gi.cpu().double(), dH, rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(gw.cpu().double(), dW, rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("vec,split", VARIANTS)
def test_gcn_and_gin_layers_match_dense_autograd(vec, split):
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from paramspmm_ae_amd.gnn_conv import GCNConv, GINConv

    n = 200  # even: GIN runs on inputs padded to an even row count
    g, rowPtr, colIdx, val = sym_graph(n, 9)
    A = dense(rowPtr, colIdx, val, n).float().cuda()
    op = pcsr_spmm(g, vec_size=vec, if_split=split, CF=1, blkWarpNum=8)
    torch.manual_seed(0)
    for Layer, ref in ((GCNConv, lambda X, W: A @ (X @ W)), (GINConv, lambda X, W: (A @ X) @ W)):
        layer = Layer(32, 16).cuda()
        X = torch.randn(n, 32, device="cuda", requires_grad=True)
        y = layer(X, {16: op})
        (y * y).sum().backward()
        Xr = X.detach().clone().requires_grad_(True)
        Wr = layer.weights.detach().clone().requires_grad_(True)
        yr = ref(Xr, Wr)
        (yr * yr).sum().backward()
        torch.testing.assert_close(y, yr, rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(X.grad, Xr.grad, rtol=1e-3, atol=1e-4)
        torch.testing.assert_close(layer.weights.grad, Wr.grad, rtol=1e-3, atol=1e-3)
    with pytest.raises(ValueError):
        GCNConv(32, 24).cuda()(X, {16: op})


@pytest.mark.parametrize("vec,split", VARIANTS)
@pytest.mark.parametrize("n,width_in,width_out", [(300, 24, 40), (20000, 32, 16), (20000, 16, 32), (17000, 128, 16), (16400, 128, 128),
                                                  (16411, 64, 64), (16411, 32, 128)])
def test_gcn_layer_with_relu_on_its_input(vec, split, n, width_in, width_out):
    """A (relu(Z) W) as one function of Z against PyTorch autograd of the same expression (torch.sparse.mm): small
    graphs and unsupported widths take the PyTorch path, 16384 rows and more with widths the library covers run the
    activation inside the dense kernels."""
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from paramspmm_ae_amd.gnn_conv import GCNConv

    g, rowPtr, colIdx, val = sym_graph(n, 5)
    S = torch.sparse_csr_tensor(torch.from_numpy(rowPtr).cuda(), torch.from_numpy(colIdx).cuda(), torch.from_numpy(val).cuda(),
                                size=(n, n))
    op = pcsr_spmm(g, vec_size=vec, if_split=split, CF=1, blkWarpNum=4)
    torch.manual_seed(3)
    layer = GCNConv(width_in, width_out).cuda()
    Z = torch.randn(n, width_in, device="cuda", requires_grad=True)
    y = layer(Z, {width_out: op}, relu_input=True)
    dY = torch.randn_like(y)
    y.backward(dY)
    Zr = Z.detach().clone().requires_grad_(True)
    Wr = layer.weights.detach().clone().requires_grad_(True)
    yr = torch.sparse.mm(S, torch.relu(Zr) @ Wr)
    yr.backward(dY)
    torch.testing.assert_close(y, yr, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(Z.grad, Zr.grad, rtol=1e-3, atol=1e-4)
    torch.testing.assert_close(layer.weights.grad, Wr.grad, rtol=2e-3, atol=2e-3)
    assert bool((Z.grad[Z.detach() <= 0] == 0).all())


@pytest.mark.parametrize("vec,split", VARIANTS)
@pytest.mark.parametrize("n,width_in,width_out,need_dx", [(300, 16, 40, True), (20000, 32, 128, True), (20000, 32, 128, False),
                                                         (20000, 16, 32, False), (17000, 32, 16, False)])
def test_gcn_layer_with_the_sparse_product_on_the_narrow_side(vec, split, n, width_in, width_out, need_dx):
    """A widening layer given an operator for its input's width computes (A H) W; a layer whose input needs no
    gradient (the network's first) skips the input gradient.  Both against PyTorch autograd of A (H W)."""
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from paramspmm_ae_amd import gnn_conv

    g, rowPtr, colIdx, val = sym_graph(n, 6)
    S = torch.sparse_csr_tensor(torch.from_numpy(rowPtr).cuda(), torch.from_numpy(colIdx).cuda(), torch.from_numpy(val).cuda(),
                                size=(n, n))
    op = pcsr_spmm(g, vec_size=vec, if_split=split, CF=1, blkWarpNum=4)
    torch.manual_seed(4)
    layer = gnn_conv.GCNConv(width_in, width_out).cuda()
    H = torch.randn(n, width_in, device="cuda", requires_grad=need_dx)
    y = layer(H, {width_out: op, width_in: op})
    assert type(y.grad_fn).__name__.startswith("GCNAggregateFirstFunction" if width_in < width_out else "GCNFunction")
    dY = torch.randn_like(y)
    y.backward(dY)
    Hr = H.detach().clone().requires_grad_(True)
    Wr = layer.weights.detach().clone().requires_grad_(True)
    yr = torch.sparse.mm(S, Hr @ Wr)
    yr.backward(dY)
    torch.testing.assert_close(y, yr, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(layer.weights.grad, Wr.grad, rtol=2e-3, atol=2e-3)
    if need_dx:
        torch.testing.assert_close(H.grad, Hr.grad, rtol=1e-3, atol=1e-4)
    else:
        assert H.grad is None
    # without an operator for the input's width the layer keeps the reference's order
    y2 = layer(H, {width_out: op})
    assert type(y2.grad_fn).__name__.startswith("GCNFunction")
    torch.testing.assert_close(y2, yr, rtol=1e-4, atol=1e-5)


def test_gcn_network_with_folded_relu_equals_the_plain_one():
    """Net_5layers with the activations folded into the layers gives the loss and the gradients of the network with
    F.relu between the layers (GNN.py:43-61)."""
    from paramspmm_ae_amd import GNN
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from paramspmm_ae_amd.gnn_conv import nll_loss_mean

    n = 20000
    g, rowPtr, colIdx, val = sym_graph(n, 8)
    ops = {16: pcsr_spmm(g, vec_size=1, if_split=False, CF=1, blkWarpNum=4)}
    torch.manual_seed(0)
    x = torch.randn(n, 32, device="cuda")
    labels = torch.randint(0, 16, (n,), device="cuda")
    model = GNN.Net_5layers(16, 32, x, ops, 16).cuda()
    grads = {}
    for fused in (True, False):
        model.fuse_relu = fused
        model.zero_grad(set_to_none=True)
        loss = nll_loss_mean(model(), labels)
        loss.backward()
        grads[fused] = (loss.item(), [p.grad.clone() for p in model.parameters()])
    assert abs(grads[True][0] - grads[False][0]) <= 1e-5 * abs(grads[False][0])
    for a, b in zip(grads[True][1], grads[False][1]):
        torch.testing.assert_close(a, b, rtol=1e-3, atol=1e-5)


@pytest.mark.parametrize("vec,split", VARIANTS)
def test_agnn_layer_forward_and_literal_backward(vec, split):
    """Forward against dense algebra; backward against the reference's literal formulas (gnn_conv.py:153-180)."""
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from paramspmm_ae_amd.gnn_conv import AGNNConv

    n = 120
    g, rowPtr, colIdx, val = sym_graph(n, 2)
    pattern = (dense(rowPtr, colIdx, val, n) != 0).float().cuda()
    op = pcsr_spmm(g, vec_size=vec, if_split=split, CF=1, blkWarpNum=4)
    torch.manual_seed(1)
    layer = AGNNConv(20, 32).cuda()
    X = torch.randn(n, 20, device="cuda", requires_grad=True)
    ci = g.csr_data.colIdx.cuda().unsqueeze(-1)
    y = layer(X, {32: op}, ci)
    Xp = X.detach() @ layer.weights.detach()
    att = pattern * (Xp @ Xp.t()) * layer.attention_w.detach().reshape(())
    torch.testing.assert_close(y, att @ Xp, rtol=1e-4, atol=1e-4)
    dY = torch.randn_like(y)
    y.backward(dY)
    d_in_prime = att @ dY
    torch.testing.assert_close(X.grad, d_in_prime @ layer.weights.detach().t(), rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(layer.weights.grad, X.detach().t() @ d_in_prime, rtol=1e-3, atol=1e-3)
    if vec == 1:
        rows = torch.from_numpy(np.repeat(np.arange(n), np.diff(rowPtr))).cuda()
        d_att = (dY[rows] * dY[g.csr_data.colIdx.cuda().long()]).sum(1)
    else:
        # block layout -> CSR slots through the mask: inside odd rows the slots follow block order, not column
        # order, and the reference multiplies them with colIdx in CSR order all the same (gnn_conv.py:166-172)
        b = g.bcsr_data
        t = torch.from_numpy(np.repeat(np.arange(b.rowPtr.numel() - 1), np.diff(b.rowPtr.numpy()))).cuda()
        cb = b.colIdx.cuda().long()
        e = torch.stack([(dY[2 * t] * dY[cb]).sum(1), (dY[2 * t + 1] * dY[cb]).sum(1)], 1) * (b.val.cuda() != 0)
        d_att = e.view(-1)[g.mask.cuda()]
    want = (d_att[None, :] @ ci.float()).t()
    torch.testing.assert_close(layer.attention_w.grad, want, rtol=1e-3, atol=1e-1)


def test_training_driver_runs_gcn_gin_agnn():
    from paramspmm_ae_amd import GNN

    for net in ("GCN", "GIN", "AGNN"):
        res = GNN.main(["--net", net, "--synthetic", "C1", "--hidden_list", "16", "--num_classes", "16",
                        "--num_features", "32", "--num_epoches", "3", "--config", "0", "2", "1", "4"])
        assert all(ms > 0 for ms in res.values())


@pytest.mark.parametrize("K1,K2", [(16, 16), (32, 16), (16, 64), (48, 32), (64, 64), (128, 128), (112, 16), (32, 128), (64, 128), (128, 64),
                                   (48, 80), (16, 128), (96, 96), (112, 128), (80, 64)])
def test_tall_skinny_weight_gradient_product(K1, K2):
    """psp_gemm_atb_f32 (the H^T * AG of the fused GCN backward) against a float64 product; n is not a multiple
    of the 64-row tile and the output is poisoned first."""
    from paramspmm_ae_amd import _capi

    n = 70_001
    g = torch.Generator(device="cuda").manual_seed(K1 * 100 + K2)
    A = torch.randn(n, K1, device="cuda", generator=g)
    B = torch.randn(n, K2, device="cuda", generator=g)
    C = torch.full((K1, K2), float("nan"), device="cuda")
    p = _capi.ptr
    assert _capi.lib.psp_gemm_atb_supported(K1, K2) == 1 and _capi.lib.psp_gemm_atb_supported(K1, 20) == 0
    _capi.check(_capi.lib.psp_gemm_atb_f32(p(A), p(B), p(C), n, K1, K2, torch.cuda.current_stream().cuda_stream))
    want = A.double().t() @ B.double()
    # fp32 accumulation over 70k terms of magnitude ~1: error ~ sqrt(n) * eps * |terms|
    torch.testing.assert_close(C.double(), want, rtol=1e-4, atol=2e-2)
    # the workspace variant: same product, partial sums added in a fixed order, so two runs agree bit for bit
    ws_floats = _capi.lib.psp_gemm_atb_workspace_floats(n, K1, K2)
    ws = torch.full((max(ws_floats, 1),), float("nan"), device="cuda")
    C2 = torch.full((K1, K2), float("nan"), device="cuda")
    C3 = torch.full((K1, K2), float("nan"), device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    _capi.check(_capi.lib.psp_gemm_atb_ws_f32(p(A), p(B), p(C2), n, K1, K2, p(ws), ws_floats, st))
    _capi.check(_capi.lib.psp_gemm_atb_ws_f32(p(A), p(B), p(C3), n, K1, K2, p(ws), ws_floats, st))
    torch.testing.assert_close(C2.double(), want, rtol=1e-4, atol=2e-2)
    if ws_floats:
        assert torch.equal(C2, C3)
        assert _capi.lib.psp_gemm_atb_ws_f32(p(A), p(B), p(C2), n, K1, K2, p(ws), ws_floats - 1, None) == -1
    assert _capi.lib.psp_gemm_atb_f32(p(A), p(B), p(C), n, K1, 20, None) == -1
    _capi.check(_capi.lib.psp_gemm_atb_f32(p(A), p(B), p(C), 0, K1, K2, None))
    torch.cuda.synchronize()
    assert bool((C == 0).all())


def test_vendor_baselines_agree_with_the_oracle(oracle):
    """The reference's cusparse_* names are served by rocSPARSE: CSR (default and load-balanced), COO and CSC SpMM,
    and the in-place SDDMM (values <- dot products, SDDMM/sddmm_baseline_kernel.cu:24-80)."""
    import ParamSDDMM
    from paramspmm_ae_amd.PCSR import pcsr_spmm, coo_spmm, csc_spmm
    from gpu_util import assert_close

    n = 2001
    g, rowPtr, colIdx, val = sym_graph(n, 5)
    X = np.random.default_rng(0).standard_normal((n, 48)).astype(np.float32)
    Xd = torch.from_numpy(X).cuda()
    want = oracle.spmm_csr(rowPtr, colIdx, val, X)
    scale = oracle.spmm_csr(rowPtr, colIdx, np.abs(val), np.abs(X))
    op = pcsr_spmm(g, vec_size=1, if_split=False)
    assert_close(op.cusparse_ref(x=Xd), want, what="rocsparse csr", scale=scale)
    assert_close(op.cusparse_csr_alg2_ref(x=Xd), want, what="rocsparse csr merge path", scale=scale)
    assert_close(coo_spmm(g).get_spmm_result(x=Xd), want, what="rocsparse coo", scale=scale)
    assert_close(csc_spmm(g).get_spmm_result(x=Xd), want, what="rocsparse csc", scale=scale)
    assert op.cusparse_ref(dim=32, is_profiling=True, verbose=False) > 0
    with pytest.raises(ValueError):
        pcsr_spmm(g, vec_size=2, if_split=False).cusparse_ref(dim=16)
    A = X / np.linalg.norm(X, axis=1, keepdims=True)
    Ad = torch.from_numpy(A).cuda()
    vals = op.val.clone()
    out = ParamSDDMM.cusparse_sddmm_compute(Ad, Ad, op.rowPtr, op.colIdx, vals)
    assert out.data_ptr() == vals.data_ptr()  # in place, as in the reference
    assert_close(vals, oracle.sddmm_csr(rowPtr, colIdx, A, A), rtol=1e-5, atol=1e-6, what="rocsparse sddmm")


@pytest.mark.parametrize("net,config", [("GCN", (0, 1, 1, 4)), ("GCN", (1, 2, 1, 8)), ("GIN", (0, 2, 2, 4))])
def test_training_step_in_hip_graph_matches_eager(monkeypatch, net, config):
    """One training step (5 layers forward, loss, backward through the SpMM / A^T B kernels, Adam) recorded in a HIP
    graph and replayed several times, with host synchronisations and other GPU work between the replays, follows the
    eager run step by step.  Dropout is switched off so that both runs see the same numbers; split formats and the
    weight-gradient kernel add with atomics, hence a tolerance instead of equality."""
    import torch.nn.functional as F
    from paramspmm_ae_amd import GNN

    monkeypatch.setattr(F, "dropout", lambda x, *a, **k: x)
    g, rowPtr, colIdx, val = sym_graph(4000, 11)

    def fresh():
        torch.manual_seed(5)
        g.x = None
        ops = GNN.configure_operators(None, g, [32, 16], config)
        torch.manual_seed(6)
        model = GNN.build_model(net, g, ops, 32, 32, 16)
        opt = torch.optim.Adam(model.parameters(), lr=0.01, capturable=True)
        return model, opt

    # eager: 3 steps (what the capture recipe runs as warm-up) + 4 more, loss recorded before each of the 4
    model_e, opt_e = fresh()
    x_e = g.x.clone()
    eager_losses = []
    for step in range(7):
        model_e.train()
        opt_e.zero_grad(set_to_none=True)
        loss = GNN.nll_loss_mean(model_e(), g.y)
        loss.backward()
        opt_e.step()
        if step >= 3:
            eager_losses.append(loss.item())

    model_g, opt_g = fresh()
    assert torch.equal(g.x, x_e), "both runs must start from the same features"
    graph, loss_g = GNN.capture_training_step(model_g, g.y, opt_g, warmup=3)
    for k in range(4):
        graph.replay()
        torch.cuda.synchronize()
        got = loss_g.item()
        assert abs(got - eager_losses[k]) <= 2e-4 * abs(eager_losses[k]) + 1e-6, (k, got, eager_losses[k])
        # unrelated eager work between replays
        junk = torch.randn(512, 512, device="cuda")
        (junk @ junk).sum().item()
    for pe, pg in zip(model_e.parameters(), model_g.parameters()):
        torch.testing.assert_close(pg, pe, rtol=0, atol=5e-3)


@pytest.mark.parametrize("n,C", [(1, 1), (1000, 16), (100_003, 7), (1_000_000, 16), (4097, 32)])
def test_nll_loss_mean_matches_torch(n, C):
    """The library's mean NLL loss (forward value and gradient) against torch's on the same log-probabilities,
    including labels outside [0, C), which do not count (-100 is PyTorch's ignore_index)."""
    import torch.nn.functional as F
    from paramspmm_ae_amd.gnn_conv import nll_loss_mean

    g = torch.Generator(device="cuda").manual_seed(n + C)
    logits = torch.randn(n, C, device="cuda", generator=g)
    labels = torch.randint(0, C, (n,), device="cuda", generator=g)
    if n > 10:
        labels[::7] = -100
    a = F.log_softmax(logits, dim=1).detach().requires_grad_(True)
    b = a.detach().clone().requires_grad_(True)
    la = nll_loss_mean(a, labels)
    lb = F.nll_loss(b, labels)
    torch.testing.assert_close(la, lb, rtol=2e-5, atol=1e-6)
    (la * 3.0).backward()
    (lb * 3.0).backward()
    torch.testing.assert_close(a.grad, b.grad, rtol=1e-6, atol=0)
    # fixed summation order: the value repeats bit for bit; stray labels other than -100 are counted for the caller
    import paramspmm_ae_amd  # noqa: F401
    import ParamSpCONV

    again = [ParamSpCONV.nll_loss_mean(a.detach(), labels)[0].item() for _ in range(3)]
    assert again[0] == again[1] == again[2] == la.item()
    stray = labels.clone()
    stray[0] = C + 5
    loss, stats = ParamSpCONV.nll_loss_mean(a.detach(), stray)
    kept = int(((stray >= 0) & (stray < C)).sum())
    assert stats[1].item() == kept and stats[2].item() == 1.0


def test_gin_backward_accepts_a_gradient_view():
    """an upstream gradient that is an expanded / transposed view (as torch.mm accepts in the reference's layer)"""
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from paramspmm_ae_amd.gnn_conv import GINConv

    n = 200
    g, rowPtr, colIdx, val = sym_graph(n, 4)
    op = pcsr_spmm(g, vec_size=1, if_split=False, CF=1, blkWarpNum=4)
    layer = GINConv(32, 16).cuda()
    X = torch.randn(n, 32, device="cuda", requires_grad=True)
    y = layer(X, {16: op})
    y.backward(torch.ones(1, 1, device="cuda").expand(n, 16))       # stride-0 view
    first = X.grad.clone()
    X.grad = None
    layer(X, {16: op}).backward(torch.ones(16, n, device="cuda").t())  # transposed view
    torch.testing.assert_close(X.grad, first)


@pytest.mark.parametrize("K1,K2", [(16, 16), (32, 16), (48, 16), (64, 16), (128, 16), (16, 32), (32, 32), (48, 32), (64, 32),
                                   (24, 16), (96, 96), (16, 64), (32, 64), (64, 64), (128, 64), (16, 128), (32, 128),
                                   (64, 128), (128, 128)])
def test_dense_xw_matches_torch(K1, K2):
    """X*W and X*W^T of the layers through the one-lane-per-row kernel (16 / 32 output columns), the matrix-core
    kernel (64 / 128 output columns) or torch::mm (24 x 16, 96 x 96), against a float64 product; a row count that is
    not a multiple of the workgroup size."""
    import ParamSpCONV

    n = 100_003
    g = torch.Generator(device="cuda").manual_seed(K1 * 1000 + K2)
    X = torch.randn(n, K1, device="cuda", generator=g)
    W = torch.randn(K1, K2, device="cuda", generator=g)
    want = (X.double() @ W.double())
    scale = (X.abs().double() @ W.abs().double())
    got = ParamSpCONV.dense_xw(X, W, False)
    assert got.shape == (n, K2)
    assert torch.all((got.double() - want).abs() <= 1e-5 * scale + 1e-6)
    Wt = W.t().contiguous()  # [K2, K1]
    got_t = ParamSpCONV.dense_xw(X, Wt, True)
    assert torch.all((got_t.double() - want).abs() <= 1e-5 * scale + 1e-6)
    # few rows: torch::mm path, same answer
    small = ParamSpCONV.dense_xw(X[:100].contiguous(), W, False)
    assert torch.all((small.double() - want[:100]).abs() <= 1e-5 * scale[:100] + 1e-6)


@pytest.mark.parametrize("n", [31, 100_003])
def test_the_128_wide_dense_product_on_either_matrix_core_path(n):
    """psp_gemm_xw_act_f32 at 128 x 128 with the option dense_split on (three bf16 terms per operand, six bf16
    matrix-core products) and off (the fp32 instruction): both within 1e-6 + 1e-5 |X||W| of float64, all three forms
    (plain, ReLU on the input, masked output, W and W^T); a non-finite input stays in its row on both paths."""
    from paramspmm_ae_amd import _capi

    L, p = _capi.lib, _capi.ptr
    g = torch.Generator(device="cuda").manual_seed(n)
    X = torch.randn(n, 128, device="cuda", generator=g) * torch.logspace(-3, 3, 128, device="cuda")  # a wide range of magnitudes
    W = torch.randn(128, 128, device="cuda", generator=g)
    Z = torch.randn(n, 128, device="cuda", generator=g)
    Wt = W.t().contiguous()
    st = torch.cuda.current_stream().cuda_stream
    scale = X.abs().double() @ W.abs().double()
    assert L.psp_get_option(b"dense_split") == 1
    try:
        for split in (1, 0):
            _capi.check(L.psp_set_option(b"dense_split", split))
            for transW, relu, mask in ((0, 0, None), (1, 0, None), (0, 1, None), (1, 0, Z)):
                Y = torch.full((n, 128), float("nan"), device="cuda")
                _capi.check(L.psp_gemm_xw_act_f32(p(X), p(Wt if transW else W), p(Y), n, 128, 128, transW, relu, p(mask), st))
                want = (torch.relu(X) if relu else X).double() @ W.double()
                if mask is not None:
                    want = want * (Z > 0)
                    assert bool((Y[Z <= 0] == 0).all())
                assert torch.all((Y.double() - want).abs() <= 1e-5 * scale + 1e-6), (split, transW, relu, mask is not None)
            Xn = X.clone()
            Xn[7, 100] = float("inf")
            Xn[n - 3, 5] = float("nan")
            Y = torch.empty(n, 128, device="cuda")
            _capi.check(L.psp_gemm_xw_act_f32(p(Xn), p(W), p(Y), n, 128, 128, 0, 0, None, st))
            bad = (~torch.isfinite(Y)).any(dim=1)
            assert bool(bad[7]) and bool(bad[n - 3]) and int(bad.sum()) == 2
    finally:
        _capi.check(L.psp_set_option(b"dense_split", 1))
    assert L.psp_set_option(b"dense_split", 2) == -1


@pytest.mark.parametrize("n,C", [(1, 16), (257, 4), (100_003, 16), (50_001, 32), (20_000, 64), (3000, 10)])
def test_loss_from_the_logits_equals_log_softmax_then_nll(n, C):
    """softmax_nll_loss_mean(x, y) against F.nll_loss(F.log_softmax(x.double(), 1), y): the loss to 1e-6 relative, the
    gradient to 1e-6 + 1e-5 |g| of the float64 one; labels outside [0, C) (PyTorch's -100 among them) do not count and get
    a zero gradient row; a class count the kernel does not take (10) runs the two separate operators."""
    from paramspmm_ae_amd import gnn_conv

    g = torch.Generator(device="cuda").manual_seed(n + C)
    x = (torch.randn(n, C, device="cuda", generator=g) * 3.0).requires_grad_(True)
    y = torch.randint(0, C, (n,), device="cuda", generator=g)
    if n > 100:
        y[5] = -100
        y[n - 2] = -100
    loss = gnn_conv.softmax_nll_loss_mean(x, y)
    loss.backward(torch.tensor(1.7, device="cuda"))
    xd = x.detach().double().requires_grad_(True)
    want = torch.nn.functional.nll_loss(torch.nn.functional.log_softmax(xd, dim=1), y)
    want.backward(torch.tensor(1.7, device="cuda", dtype=torch.float64))
    assert abs(loss.item() - want.item()) <= 1e-6 * abs(want.item()) + 1e-7
    assert torch.all((x.grad.double() - xd.grad).abs() <= 1e-6 / max(n, 1) + 1e-5 * xd.grad.abs())
    if n > 100:
        assert bool((x.grad[5] == 0).all()) and bool((x.grad[n - 2] == 0).all())
    # large logits do not overflow
    xb = torch.full((max(n, 2), C), 80.0, device="cuda")
    xb[:, 0] = 120.0
    yb = torch.zeros(max(n, 2), dtype=torch.int64, device="cuda")
    lb = gnn_conv.softmax_nll_loss_mean(xb, yb)
    assert bool(torch.isfinite(lb)) and lb.item() < 1e-6


def test_networks_train_the_same_with_the_loss_folded_in():
    """The GCN network's training step with the log-softmax folded into the loss (GNN.loss_of_step, the default) and with
    the two as operators of their own: same loss, same gradients (fp32 rounding apart)."""
    from paramspmm_ae_amd import GNN
    from paramspmm_ae_amd.PCSR import pcsr_spmm

    n = 20000
    g, rowPtr, colIdx, val = sym_graph(n, 9)
    op = pcsr_spmm(g, vec_size=1, if_split=False, CF=1, blkWarpNum=4)
    torch.manual_seed(0)
    x = torch.randn(n, 32, device="cuda")
    labels = torch.randint(0, 16, (n,), device="cuda")
    model = GNN.Net_5layers(16, 32, x, {16: op, 32: op}, 32).cuda()
    res = {}
    for fused in (True, False):
        model.fuse_loss = fused
        model.zero_grad(set_to_none=True)
        loss = GNN.loss_of_step(model, labels)
        loss.backward()
        res[fused] = (loss.item(), [p.grad.clone() for p in model.parameters()])
    assert abs(res[True][0] - res[False][0]) <= 1e-5 * abs(res[False][0])
    for a, b in zip(res[True][1], res[False][1]):
        torch.testing.assert_close(a, b, rtol=1e-3, atol=1e-5 * float(b.abs().max()) + 1e-7)
    model.eval()
    out = model()
    torch.testing.assert_close(out.exp().sum(1), torch.ones(n, device="cuda"), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("vec_size", [2, 3])
def test_sddmm_sweep_harness(tmp_path, vec_size):
    """SDDMM.py's facade and sweep (SDDMM.py:46-383) on the reference's pubmed pattern read from a .mtx file and on a
    synthetic graph: every variant is verified against the vendor result inside the sweep (ones -> dim per entry),
    the tables have the reference's column order, and the vendor call leaves the shared value array alone."""
    import scipy.io
    import scipy.sparse as sp
    from conftest import pubmed_pattern
    from paramspmm_ae_amd import SDDMM as S

    scipy.io.mmwrite(str(tmp_path / "pm.mtx"), sp.tril(pubmed_pattern("orig")).tocoo(), symmetry="symmetric")
    tables = S.main(["--path", str(tmp_path) + os.sep, "--mtx_name", "pm", "--dim_list", "32", "48", "--vec_size",
                     str(vec_size), "--csv_path", str(tmp_path / "log") + os.sep])
    assert sorted(tables) == [32, 48]
    names = ["vec1_TP_4", "vec1_split_TP_4", "vec%d_TP_4" % vec_size, "vec%d_split_TP_4" % vec_size,
             "vec1_TP_8", "vec1_split_TP_8", "vec%d_TP_8" % vec_size, "vec%d_split_TP_8" % vec_size]
    for dim, tp in tables.items():
        assert list(tp.columns) == names and tp.shape == (1, 8) and bool((tp.to_numpy() > 0).all())
        best = pd.read_csv(tmp_path / "log" / ("dim%d_OP_SpMM.csv" % dim))
        assert best.shape == (1, 17) and int(best["OP_SpMM"][0]) == int(tp.to_numpy().argmax())
    # synthetic graph, facade by hand
    g = S._load("C1", None, True, 2, True)
    op = S.pcsr_sddmm(g, vec_size=1, if_split=False)
    before = op.val.clone()
    want = op.cusparse_ref(64)
    assert torch.equal(op.val, before) and bool((want == 64).all())
    S.compare(op.get_sddmm_result(64, 8), want, verbose=False)
    blocked = S.pcsr_sddmm(g, vec_size=2, if_split=True)
    S.compare_2d(blocked.get_sddmm_result(64, 4), want, blocked.mask, verbose=False)
    assert op.cusparse_ref(64, is_profiling=True, verbose=False) > 0 and blocked.profiling(4, 64, verbose=False) > 0
    with pytest.raises(ValueError, match="cusparse only support"):
        blocked.cusparse_ref(64)
    with pytest.raises(ValueError, match="Verification FAILED"):
        S.compare(want + 1.0, want, verbose=False)


def test_training_set_construction_from_mtx_files(tmp_path):
    """`python PCSR.py` of the reference (PCSR.py:660-871): features, the swept GFLOP/s table in class-code order, the
    best column and the vendor baselines, written as the csv files the decider training reads; every configuration
    is verified against torch.sparse.mm on the way."""
    import scipy.io
    import scipy.sparse as sp
    from conftest import pubmed_pattern
    from paramspmm_ae_amd import PCSR as P

    d = tmp_path / "rabbit"
    d.mkdir()
    scipy.io.mmwrite(str(d / "pm.mtx"), sp.tril(pubmed_pattern("rabbit")).tocoo(), symmetry="symmetric")
    out = str(tmp_path / "log") + os.sep
    tables, baselines = P.main(["--path", str(d) + os.sep, "--dim_list", "16", "80", "--csv_path", out])
    for dim in (16, 80):
        cfs = P.dynamic_CF_prompter(dim)
        tp = pd.read_csv(out + "dim%d.csv" % dim)
        assert tp.shape == (1, 8 * len(cfs)) and bool((tp.to_numpy() > 0).all())
        # blkWarpNum-major, then CF, then the four representations: the order decode_tree relies on
        assert list(tp.columns) == ["%s_TP_%d%d" % (rep, cf, bw) for bw in (4, 8) for cf in cfs
                                    for rep in ("vec1", "vec1_split", "vec2", "vec2_split")]
        lab = pd.read_csv(out + "dim%d_OP_SpMM.csv" % dim)
        assert lab.shape == (1, 17) and int(lab["OP_SpMM"][0]) == int(tp.to_numpy().argmax())
        b = pd.read_csv(out + "dim%d_baseline.csv" % dim)
        assert list(b.columns) == ["cusparse", "gespmm"] and bool((b.to_numpy() > 0).all())
    # without the gap rule dim 80 sweeps CF 1..3
    t2, _ = P.profile_engine(["pm"], str(d) + os.sep, [80], if_DCP=False, verbose=False)
    assert t2[80].shape == (1, 8 * 3)
    # 3x1 blocks in place of 2x1
    t3, _ = P.profile_engine(["pm"], str(d) + os.sep, [32], vec_size=3, verbose=False)
    assert list(t3[32].columns)[2:4] == ["vec3_TP_14", "vec3_split_TP_14"] and bool((t3[32].to_numpy() > 0).all())


def test_decider_evaluation_run(tmp_path):
    """decider.py's command line (decider.py:97-175): the pick of the shipped forests is verified and timed beside
    the four baselines, on a .mtx file and on a synthetic graph."""
    import scipy.io
    import scipy.sparse as sp
    from conftest import pubmed_pattern
    from paramspmm_ae_amd import decider as D

    scipy.io.mmwrite(str(tmp_path / "pm.mtx"), sp.tril(pubmed_pattern("orig")).tocoo(), symmetry="symmetric")
    t = D.main(["--path", str(tmp_path) + os.sep, "--mtx_name", "pm", "--dim_list", "16", "96"])
    assert list(t["dim"]) == [16, 96] and bool((t[["param", "coo", "csc", "cusparse", "gespmm"]].to_numpy() > 0).all())
    assert set(t["vec_size"]) <= {1, 2} and set(t["blkWarpNum"]) <= {4, 8}
    t2 = D.evaluate(["C1"], None, [32], verbose=False)
    assert t2.shape[0] == 1 and t2["param"][0] > 0
    # verification.py's own command line on the same directory
    from paramspmm_ae_amd import verification as V

    res = V.main(["--path", str(tmp_path) + os.sep, "--dim", "16"])
    assert list(res) == ["pm"] and res["pm"][0] > 0 and res["pm"][1] > 0


@pytest.mark.parametrize("n", [1, 5, 63, 64, 257, 4099])
@pytest.mark.parametrize("K1,K2", [(16, 16), (64, 64), (128, 128), (96, 96)])
def test_weight_gradient_product_small_row_counts(n, K1, K2):
    """row counts around the kernels' chunk sizes (4-row groups, 8 / 16 / 32-row chunks, fewer chunks than wavefronts)"""
    from paramspmm_ae_amd import _capi

    g = torch.Generator(device="cuda").manual_seed(n)
    A = torch.randn(n, K1, device="cuda", generator=g)
    B = torch.randn(n, K2, device="cuda", generator=g)
    p = _capi.ptr
    st = torch.cuda.current_stream().cuda_stream
    want = A.double().t() @ B.double()
    ws_floats = _capi.lib.psp_gemm_atb_workspace_floats(n, K1, K2)
    ws = torch.full((max(ws_floats, 1),), float("nan"), device="cuda")
    for entry in ("ws", "atomic"):
        C = torch.full((K1, K2), float("nan"), device="cuda")
        if entry == "ws":
            _capi.check(_capi.lib.psp_gemm_atb_ws_f32(p(A), p(B), p(C), n, K1, K2, p(ws), ws_floats, st))
        else:
            _capi.check(_capi.lib.psp_gemm_atb_f32(p(A), p(B), p(C), n, K1, K2, st))
        torch.testing.assert_close(C.double(), want, rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("K1,K2", [(16, 64), (64, 64), (128, 64), (32, 128), (128, 128)])
@pytest.mark.parametrize("n", [1, 33, 70_001])
def test_wide_dense_products_with_the_activation_folded_in(K1, K2, n):
    """psp_gemm_xw_act_f32 on the matrix-core kernel through the C ABI: max(X, 0) W and (X W^T) masked by Z > 0 against
    float64, at row counts around the 32-row blocks; masked elements are exact zeros, NaN inputs stay in their rows."""
    from paramspmm_ae_amd import _capi

    L, p = _capi.lib, _capi.ptr
    assert L.psp_gemm_xw_supported(K1, K2) == 1
    g = torch.Generator(device="cuda").manual_seed(n + K1 + 7 * K2)
    X = torch.randn(n, K1, device="cuda", generator=g)
    W = torch.randn(K1, K2, device="cuda", generator=g)
    Z = torch.randn(n, K2, device="cuda", generator=g)
    st = torch.cuda.current_stream().cuda_stream
    Y = torch.full((n, K2), float("nan"), device="cuda")
    _capi.check(L.psp_gemm_xw_act_f32(p(X), p(W), p(Y), n, K1, K2, 0, 1, None, st))
    want = torch.relu(X).double() @ W.double()
    scale = torch.relu(X).double() @ W.abs().double()
    assert torch.all((Y.double() - want).abs() <= 1e-5 * scale + 1e-6)
    Wt = W.t().contiguous()
    Y2 = torch.full((n, K2), float("nan"), device="cuda")
    _capi.check(L.psp_gemm_xw_act_f32(p(X), p(Wt), p(Y2), n, K1, K2, 1, 0, p(Z), st))
    want2 = (X.double() @ W.double()) * (Z > 0)
    assert torch.all((Y2.double() - want2).abs() <= 1e-5 * (X.abs().double() @ W.abs().double()) + 1e-6)
    assert bool((Y2[Z <= 0] == 0).all())
    if n > 40:
        Xn = X.clone()
        Xn[17, 3] = float("nan")
        _capi.check(L.psp_gemm_xw_act_f32(p(Xn), p(W), p(Y), n, K1, K2, 0, 0, None, st))
        bad = torch.isnan(Y).any(dim=1)
        assert bool(bad[17]) and int(bad.sum()) == 1
    # the two fused forms are exclusive, as for the narrow kernel
    assert L.psp_gemm_xw_act_f32(p(X), p(W), p(Y), n, K1, K2, 1, 1, None, st) == -1
    assert L.psp_gemm_xw_act_f32(p(X), p(W), p(Y), n, K1, K2, 0, 0, p(Z), st) == -1


@pytest.mark.parametrize("vec,split", VARIANTS)
@pytest.mark.parametrize("n,width_in,width_out", [(301, 24, 40), (20001, 32, 16), (20000, 16, 128), (17001, 128, 16)])
def test_gin_layer_with_relu_on_its_input(vec, split, n, width_in, width_out):
    """(A relu(Z)) W as one function of Z against PyTorch autograd of the same expression: the activation applied as the
    sparse product gathers its rows, the mask as the backward product writes its rows (odd row counts, widths with a
    partial column tile, all four formats); the operator of the input's width is the one that runs."""
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from paramspmm_ae_amd.gnn_conv import GINConv

    g, rowPtr, colIdx, val = sym_graph(n, 5)
    S = torch.sparse_csr_tensor(torch.from_numpy(rowPtr).cuda(), torch.from_numpy(colIdx).cuda(), torch.from_numpy(val).cuda(),
                                size=(n, n))
    op = pcsr_spmm(g, vec_size=vec, if_split=split, CF=1, blkWarpNum=4)
    torch.manual_seed(3)
    layer = GINConv(width_in, width_out).cuda()
    Z = torch.randn(n, width_in, device="cuda", requires_grad=True)
    y = layer(Z, {width_in: op, width_out: op}, relu_input=True)
    assert type(y.grad_fn).__name__.startswith("GINReLUInputFunction" if width_in < width_out else "GCNReLUInputFunction")
    dY = torch.randn_like(y)
    y.backward(dY)
    Zr = Z.detach().clone().requires_grad_(True)
    Wr = layer.weights.detach().clone().requires_grad_(True)
    yr = torch.sparse.mm(S, torch.relu(Zr)) @ Wr
    yr.backward(dY)
    torch.testing.assert_close(y, yr, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(Z.grad, Zr.grad, rtol=1e-3, atol=1e-4)
    torch.testing.assert_close(layer.weights.grad, Wr.grad, rtol=2e-3, atol=2e-3)
    assert bool((Z.grad[Z.detach() <= 0] == 0).all())


@pytest.mark.parametrize("fmt", [0, 1, 2, 3])
def test_spmm_with_activation_arguments_through_the_c_abi(oracle, fmt):
    """psp_spmm_act_f32: A max(X, 0) equals the plain product of the clamped input bit for bit, the masked product
    equals the plain one where the mask is positive and is an exact zero elsewhere (a hub row, native
    configurations, a width that is not a multiple of four)."""
    from conftest import random_csr
    from gpu_util import Formats, spmm_capi
    from paramspmm_ae_amd import _capi

    L, p = _capi.lib, _capi.ptr
    names = ["csr", "csr_split", "bcsr", "bcsr_split"]
    rowPtr, colIdx, val = random_csr(6001, 9, 21, empty_frac=0.1, hub=(11, 3000), values="normal")
    F = Formats(oracle, rowPtr, colIdx, val)
    d = F.d
    arrays = [(d["rowPtr"], d["colIdx"], d["val"], None, F.n), (d["rps"], d["colIdx"], d["val"], d["tr"], F.tr.size),
              (d["rpb"], d["cib"], d["vb"], None, F.rpb.size - 1), (d["rpbs"], d["cib"], d["vb"], d["trb"], F.trb.size)][fmt]
    st = torch.cuda.current_stream().cuda_stream
    rows = F.n + (F.n & 1)
    A_abs = torch.sparse_csr_tensor(torch.from_numpy(rowPtr).cuda(), torch.from_numpy(colIdx).cuda(),
                                    torch.from_numpy(np.abs(val)).cuda(), size=(F.n, rows))

    def close(got, want, X):
        # two runs of a row-split product add a long row's partial sums with atomics in different orders: the bound
        # is the stated tolerance with the relative term against (|A| |X|), the magnitude the terms add up to
        tol = 1e-6 + 1e-5 * torch.sparse.mm(A_abs, X.abs())
        assert bool(((got[: F.n] - want[: F.n]).abs() <= tol).all()) and bool((got[F.n:] == want[F.n:]).all())

    for N, cf in ((16, 1), (100, 2), (7, 1), (128, _capi.pack_cf(1, 16, 4)), (256, _capi.pack_cf(4, 8, 2, even_split=True))):
        g = torch.Generator(device="cuda").manual_seed(N)
        X = torch.randn(rows, N, device="cuda", generator=g)
        M = torch.randn(rows, N, device="cuda", generator=g)
        if N == 100:
            M = M.contiguous()
        plain = spmm_capi(names[fmt], F, X, cf, 8)
        clamped = spmm_capi(names[fmt], F, torch.relu(X), cf, 8)
        Y = torch.full((rows, N), float("nan"), device="cuda")
        rp, ci, v, tr, nseg = arrays
        _capi.check(L.psp_spmm_act_f32(fmt, p(rp), p(ci), p(v), p(tr), p(X), p(Y), nseg, N, rows, cf, 8, 1, None, st))
        if fmt in (0, 2):
            assert torch.equal(Y, clamped)
        else:
            close(Y, clamped, X)
        _capi.check(L.psp_spmm_act_f32(fmt, p(rp), p(ci), p(v), p(tr), p(X), p(Y), nseg, N, rows, cf, 8, 0, p(M), st))
        want = torch.where(M > 0, plain, torch.zeros_like(plain))
        if fmt in (0, 2):
            assert torch.equal(Y, want)
        else:
            close(Y, want, X)
        assert bool((Y[M <= 0] == 0).all())
    assert L.psp_spmm_act_f32(4, p(rp), p(ci), p(v), p(tr), p(X), p(Y), nseg, N, rows, 1, 8, 1, None, st) == -1


@pytest.mark.parametrize("net,hidden", [("GIN", 16), ("GIN", 64), ("AGNN", 16), ("AGNN", 64)])
def test_gin_and_agnn_networks_with_folded_relu_equal_the_plain_ones(net, hidden):
    """The GIN and the attention network with their activations folded into the layers give the loss and the gradients
    of the networks with a ReLU pass between the layers (GNN.py:63-101); the attention network's dropout draws the
    same mask in both (same seed) and commutes with the activation."""
    from paramspmm_ae_amd import GNN
    from paramspmm_ae_amd.PCSR import pcsr_spmm
    from paramspmm_ae_amd.gnn_conv import nll_loss_mean

    n = 20000
    g, rowPtr, colIdx, val = sym_graph(n, 9)
    op = pcsr_spmm(g, vec_size=1, if_split=False, CF=1, blkWarpNum=4)
    ops = {16: op, 32: op, hidden: op}
    torch.manual_seed(0)
    x = torch.randn(n, 32, device="cuda")
    labels = torch.randint(0, 16, (n,), device="cuda")
    if net == "GIN":
        model = GNN.GIN(16, 32, x, ops, hidden).cuda()
    else:
        model = GNN.AGNN(16, 32, x, ops, hidden, g.csr_data.colIdx.cuda().unsqueeze(-1)).cuda()
        with torch.no_grad():  # keep the attention scores of five stacked layers in range
            for p in model.parameters():
                p.mul_(0.3)
    model.train()
    grads = {}
    for fused in (True, False):
        model.fuse_relu = fused
        model.zero_grad(set_to_none=True)
        torch.manual_seed(123)  # the dropout mask
        loss = nll_loss_mean(model(), labels)
        loss.backward()
        grads[fused] = (loss.item(), [p.grad.clone() for p in model.parameters()])
    assert abs(grads[True][0] - grads[False][0]) <= 1e-4 * abs(grads[False][0])
    for a, b in zip(grads[True][1], grads[False][1]):
        torch.testing.assert_close(a, b, rtol=2e-3, atol=1e-4 * float(b.abs().max()) + 1e-6)


def test_operators_chosen_among_the_deciders_candidates_compute_the_product():
    """configure_operators(try_candidates=3): the operator kept for every width is one of the forest's three
    highest-rated configurations (the first being the decider's own answer) and computes A X (checked against
    torch.sparse.mm in double precision); an odd row count exercises the padded input of the block formats."""
    from paramspmm_ae_amd import GNN
    from paramspmm_ae_amd.decider import SpMMDecider

    n = 30001
    g, rowPtr, colIdx, val = sym_graph(n, 21)
    dec = SpMMDecider()
    dims = [16, 48, 128]
    dec.gen_model_dict(dims)
    ops = GNN.configure_operators(dec, g, dims, try_candidates=3)
    rows = torch.from_numpy(np.repeat(np.arange(n), np.diff(rowPtr)))
    A = torch.sparse_coo_tensor(torch.stack([rows, torch.from_numpy(colIdx.astype(np.int64))]),
                                torch.from_numpy(val.astype(np.float64)), (n, n)).cuda()
    for d in dims:
        op = ops[d]
        cands = dec.candidates_PCSR(g, d, 3)
        assert (int(op.if_split), op.vec_size, op.CF, op.blkWarpNum) in [(int(s), v, c, b) for s, v, c, b in cands]
        X = torch.randn(n, d, device="cuda")
        got = op._spmm(X)[:n]
        want = torch.sparse.mm(A, X.double())
        assert (got.double() - want).abs().max().item() <= 1e-5 * want.abs().max().item() + 1e-6
