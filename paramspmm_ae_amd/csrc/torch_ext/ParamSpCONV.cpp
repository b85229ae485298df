// Python module `ParamSpCONV`: the fused GCN layer ops of the reference's SpCONV/SpCONV.cpp:496-512
// (glue in SpCONV/SpCONV.h:43-193): forward A*(H*W), backward [ (A*dY)*W^T, H^T*(A*dY) ].  The dense
// products are torch::mm (hipBLASLt / rocBLAS under PyTorch-ROCm); the sparse product is libparamsp_hip.so.
#include "glue_common.h"

using namespace pspglue;
using torch::Tensor;

static void check_cf(int CF, int fmt = 0)
{
    if (fmt == 4) {  // windowed csr: CF names the kernel variant
        TORCH_CHECK(CF >= 0 && CF <= 3, "the windowed format takes variant 0..3 in place of CF");
        return;
    }
    // SpCONV dispatches CF 1..4 only (SpCONV/SpCONV.cpp:92-124)
    TORCH_CHECK((CF >= 1 && CF <= 8) || (CF & PSP_CF_NATIVE), "CF must be 1..8 (or a native configuration)");
}

// A*D for a dense D, result cut back to rows(D) (the blocked formats compute into an even-padded buffer,
// SpCONV/SpCONV.h:115-118)
static Tensor aggregate(int fmt, const Tensor &D, const Tensor &rowPtr, const Tensor &colIdx, const Tensor &values,
                        const Tensor *target_row, int CF, int blkWarpNum)
{
    check_cf(CF, fmt);
    Tensor Dc = D.contiguous();
    Tensor Y = spmm_new(fmt, Dc, rowPtr, colIdx, values, target_row, CF, blkWarpNum);
    if (Y.size(0) != Dc.size(0)) Y = Y.narrow(0, 0, Dc.size(0));
    return Y;
}

// H^T * AG.  For narrow layers the product is a reduction over ~10^6 rows into a tiny matrix, which the library
// streams at memory speed; everything else goes to torch::mm.
static Tensor weight_gradient(const Tensor &H, const Tensor &AG)
{
    const bool narrow = H.dim() == 2 && AG.dim() == 2 && H.size(0) == AG.size(0) && H.size(0) >= 16384 &&
                        H.scalar_type() == torch::kFloat32 && AG.scalar_type() == torch::kFloat32 &&
                        psp_gemm_atb_supported((int)H.size(1), (int)AG.size(1));
    if (!narrow) return torch::mm(H.t(), AG);
    Tensor Hc = H.contiguous(), Gc = AG.contiguous();
    DeviceGuard guard(Hc.device());
    Tensor dW = torch::empty({Hc.size(1), Gc.size(1)}, Hc.options());
    // partial products of the workgroups go through a workspace and are added in a fixed order (no atomics)
    const long long ws_floats = psp_gemm_atb_workspace_floats(Hc.size(0), (int)Hc.size(1), (int)Gc.size(1));
    Tensor ws = torch::empty({(long)ws_floats}, Hc.options());
    ok(psp_gemm_atb_ws_f32(fp(Hc), fp(Gc), fpw(dW), Hc.size(0), (int)Hc.size(1), (int)Gc.size(1), fpw(ws), ws_floats,
                           stream_of(Hc)));
    return dW;
}

// X * W (or X * W^T): the library's one-lane-per-row kernel for narrow layers on many rows, torch::mm otherwise
static Tensor dense_xw(const Tensor &X, const Tensor &W, bool transW)
{
    const long K1 = X.dim() == 2 ? X.size(1) : -1;
    const bool shapes = X.dim() == 2 && W.dim() == 2 && W.size(transW ? 1 : 0) == K1;
    const long K2 = shapes ? W.size(transW ? 0 : 1) : -1;
    const bool narrow = shapes && X.size(0) >= 16384 && X.scalar_type() == torch::kFloat32 &&
                        W.scalar_type() == torch::kFloat32 && X.is_cuda() && W.is_cuda() &&
                        psp_gemm_xw_supported((int)K1, (int)K2);
    if (!narrow) return torch::mm(X, transW ? W.t() : W);
    Tensor Xc = X.contiguous(), Wc = W.contiguous();
    DeviceGuard guard(Xc.device());
    Tensor Y = torch::empty({Xc.size(0), K2}, Xc.options());
    ok(psp_gemm_xw_f32(fp(Xc), fp(Wc), fpw(Y), Xc.size(0), (int)K1, (int)K2, transW ? 1 : 0, stream_of(Xc)));
    return Y;
}

// The same two products with the ReLU between two layers folded in (psp_gemm_xw_act_f32 / psp_gemm_atb_ws_act_f32);
// shapes the library does not cover apply the activation with PyTorch and multiply with torch::mm.
static Tensor dense_relu_xw(const Tensor &Z, const Tensor &W)
{
    const long K1 = Z.dim() == 2 ? Z.size(1) : -1;
    const bool shapes = Z.dim() == 2 && W.dim() == 2 && W.size(0) == K1;
    const bool narrow = shapes && Z.size(0) >= 16384 && Z.scalar_type() == torch::kFloat32 && W.scalar_type() == torch::kFloat32 &&
                        psp_gemm_xw_supported((int)K1, (int)W.size(1));
    if (!narrow) return torch::mm(torch::relu(Z), W);
    Tensor Zc = Z.contiguous(), Wc = W.contiguous();
    DeviceGuard guard(Zc.device());
    Tensor Y = torch::empty({Zc.size(0), Wc.size(1)}, Zc.options());
    ok(psp_gemm_xw_act_f32(fp(Zc), fp(Wc), fpw(Y), Zc.size(0), (int)K1, (int)Wc.size(1), 0, 1, nullptr, stream_of(Zc)));
    return Y;
}
// (AG * W^T) where Z > 0, else 0
static Tensor dense_xwt_masked(const Tensor &AG, const Tensor &W, const Tensor &Z)
{
    const long K1 = AG.dim() == 2 ? AG.size(1) : -1;
    const bool shapes = AG.dim() == 2 && W.dim() == 2 && W.size(1) == K1 && Z.dim() == 2 && Z.size(0) == AG.size(0) &&
                        Z.size(1) == W.size(0);
    const bool narrow = shapes && AG.size(0) >= 16384 && AG.scalar_type() == torch::kFloat32 && W.scalar_type() == torch::kFloat32 &&
                        Z.scalar_type() == torch::kFloat32 && psp_gemm_xw_supported((int)K1, (int)W.size(0));
    if (!narrow) return at::threshold_backward(torch::mm(AG, W.t()), Z, 0);  // what F.relu's backward runs
    Tensor Gc = AG.contiguous(), Wc = W.contiguous(), Zc = Z.contiguous();
    DeviceGuard guard(Gc.device());
    Tensor Y = torch::empty({Gc.size(0), Wc.size(0)}, Gc.options());
    ok(psp_gemm_xw_act_f32(fp(Gc), fp(Wc), fpw(Y), Gc.size(0), (int)K1, (int)Wc.size(0), 1, 0, fp(Zc), stream_of(Gc)));
    return Y;
}
// relu(Z)^T * AG
static Tensor weight_gradient_relu(const Tensor &Z, const Tensor &AG)
{
    const bool narrow = Z.dim() == 2 && AG.dim() == 2 && Z.size(0) == AG.size(0) && Z.size(0) >= 16384 &&
                        Z.scalar_type() == torch::kFloat32 && AG.scalar_type() == torch::kFloat32 &&
                        psp_gemm_atb_supported((int)Z.size(1), (int)AG.size(1));
    if (!narrow) return torch::mm(torch::relu(Z).t(), AG);
    Tensor Zc = Z.contiguous(), Gc = AG.contiguous();
    DeviceGuard guard(Zc.device());
    Tensor dW = torch::empty({Zc.size(1), Gc.size(1)}, Zc.options());
    const long long ws_floats = psp_gemm_atb_workspace_floats(Zc.size(0), (int)Zc.size(1), (int)Gc.size(1));
    Tensor ws = torch::empty({(long)ws_floats}, Zc.options());
    ok(psp_gemm_atb_ws_act_f32(fp(Zc), fp(Gc), fpw(dW), Zc.size(0), (int)Zc.size(1), (int)Gc.size(1), 1, fpw(ws), ws_floats,
                               stream_of(Zc)));
    return dW;
}

// GCN layer that reads its input through a ReLU: A * (relu(Z) * W).  fmt: 0 csr, 1 csr_split, 2 bcsr, 3 bcsr_split.
// No counterpart among the reference's bindings: its driver applies F.relu between the layers as a pass of its own
// (GNN.py:43-61); the algebra of the layer itself is SpCONV/SpCONV.h:43-71.
static Tensor relu_input_forward(int fmt, Tensor Z, Tensor W, Tensor rowPtr, Tensor colIdx, Tensor values,
                                 c10::optional<Tensor> target_row, int CF, int bw)
{
    need_gpu(Z, "input");
    need_gpu(W, "weight");
    TORCH_CHECK(fmt >= 0 && fmt <= 4 && (fmt == 1 || fmt == 3) == target_row.has_value(), "format code and target_row disagree");
    return aggregate(fmt, dense_relu_xw(Z, W), rowPtr, colIdx, values, target_row ? &*target_row : nullptr, CF, bw);
}
// [dZ, dW] = [ ((A dY) W^T) where Z > 0,  relu(Z)^T (A dY) ]
static std::vector<Tensor> relu_input_backward(int fmt, Tensor dY, Tensor Z, Tensor W, Tensor rowPtr, Tensor colIdx,
                                               Tensor values, c10::optional<Tensor> target_row, int CF, int bw)
{
    need_gpu(Z, "input");
    need_gpu(W, "weight");
    TORCH_CHECK(fmt >= 0 && fmt <= 4 && (fmt == 1 || fmt == 3) == target_row.has_value(), "format code and target_row disagree");
    Tensor AG = aggregate(fmt, dY, rowPtr, colIdx, values, target_row ? &*target_row : nullptr, CF, bw);
    return {dense_xwt_masked(AG, W, Z), weight_gradient_relu(Z, AG)};
}

// A * D alone, for callers that place the sparse product on the narrower side of the layer: (A H) W costs a sparse
// product of width in_features where A (H W) costs one of width out_features.  No counterpart among the reference's
// bindings, whose layer is always A (H W) (SpCONV/SpCONV.h:43-48).
static Tensor aggregate_op(int fmt, Tensor D, Tensor rowPtr, Tensor colIdx, Tensor values, c10::optional<Tensor> target_row,
                           int CF, int bw)
{
    need_gpu(D, "input");
    TORCH_CHECK(fmt >= 0 && fmt <= 4 && (fmt == 1 || fmt == 3) == target_row.has_value(), "format code and target_row disagree");
    return aggregate(fmt, D, rowPtr, colIdx, values, target_row ? &*target_row : nullptr, CF, bw);
}

// A * max(D, 0) and / or (A * D) kept where mask > 0: the ReLU between two layers folded into the sparse product
// (psp_spmm_act_f32).  Used by the layers that aggregate first (GIN: (A X) W): the activation is applied as the rows of
// D are gathered, its backward as the rows of the gradient are written.  No counterpart among the reference's
// bindings: its driver runs F.relu as a pass of its own (GNN.py:63-78).  float64 and mask shapes the kernel does not
// take fall back to PyTorch's passes around the plain product.
static Tensor aggregate_act_op(int fmt, Tensor D, Tensor rowPtr, Tensor colIdx, Tensor values, c10::optional<Tensor> target_row,
                               int CF, int bw, bool relu_input, c10::optional<Tensor> mask)
{
    need_gpu(D, "input");
    TORCH_CHECK(fmt >= 0 && fmt <= 4 && (fmt == 1 || fmt == 3) == target_row.has_value(), "format code and target_row disagree");
    check_cf(CF, fmt);
    const Tensor *tr = target_row ? &*target_row : nullptr;
    if (mask) {
        need_gpu(*mask, "mask");
        TORCH_CHECK(mask->dim() == 2 && mask->size(0) == D.size(0) && mask->size(1) == D.size(1), "mask must have the shape of the result");
    }
    const bool blocked = pspglue::fmt_blocked(fmt);
    const bool fused = D.scalar_type() == torch::kFloat32 && (!mask || mask->scalar_type() == torch::kFloat32) &&
                       D.size(1) > 0 && D.size(0) > 0 && (!blocked || D.size(0) % 2 == 0 || !mask);
    if (!fused) {
        Tensor Y = aggregate(fmt, relu_input ? torch::relu(D) : D, rowPtr, colIdx, values, tr, CF, bw);
        return mask ? at::threshold_backward(Y, *mask, 0) : Y;
    }
    Tensor Dc = D.contiguous();
    check_spmm_args(fmt, Dc, rowPtr, colIdx, values, tr);
    DeviceGuard guard(Dc.device());
    const long rows_out = blocked ? (Dc.size(0) + 1) / 2 * 2 : Dc.size(0);
    Tensor Mc;
    if (mask) Mc = mask->contiguous();
    Tensor Y = torch::empty({rows_out, Dc.size(1)}, Dc.options());
    if (fmt == 4)  // windowed csr: the activation is applied as the window is staged, the mask where a row is stored
        ok(psp_spmm_window_f32(ip(rowPtr), ip(colIdx), fp(values), fp(Dc), fpw(Y), pspglue::fmt_rows(fmt, rowPtr),
                               (int)colIdx.size(0), (int)Dc.size(1), (int)rows_out, CF, relu_input ? 1 : 0,
                               mask ? fp(Mc) : nullptr, stream_of(Dc)));
    else
        ok(psp_spmm_act_f32(fmt, ip(rowPtr), ip(colIdx), fp(values), tr ? ip(*tr) : nullptr, fp(Dc), fpw(Y),
                            (int)rowPtr.size(0) - 1, (int)Dc.size(1), (int)rows_out, CF, bw, relu_input ? 1 : 0,
                            mask ? fp(Mc) : nullptr, stream_of(Dc)));
    if (Y.size(0) != Dc.size(0)) Y = Y.narrow(0, 0, Dc.size(0));
    return Y;
}

// Windowed layout, square layer of 16 or 32 columns: the dense product folded into the sparse one
// (psp_spmm_window_xw_f32).  Returns [Y] or [Y, A f(X)]:  Y = ((A f(X)) W | W^T), kept where mask > 0 when a mask is given.
static bool window_xw_supported(long N) { return N == 16 || N == 32; }
static std::vector<Tensor> window_xw(Tensor X, Tensor W, bool transW, Tensor rowPtr_w, Tensor colIdx_w, Tensor values_w,
                                     bool relu_input, c10::optional<Tensor> mask, bool want_raw)
{
    need_gpu(X, "input");
    need_gpu(W, "weight");
    Tensor Xc = X.contiguous(), Wc = W.contiguous();
    check_spmm_args(4, Xc, rowPtr_w, colIdx_w, values_w, nullptr);
    need_f32(Wc, "weight", 2);
    const long N = Xc.size(1);
    TORCH_CHECK(window_xw_supported(N) && Wc.size(0) == N && Wc.size(1) == N,
                "window_xw: a square weight matrix of 16 or 32 columns, as wide as the input");
    pspglue::same_device(Xc, Wc, "window_xw");
    Tensor Mc;
    if (mask) {
        need_gpu(*mask, "mask");
        TORCH_CHECK(mask->scalar_type() == torch::kFloat32 && mask->dim() == 2 && mask->size(0) == Xc.size(0) && mask->size(1) == N,
                    "mask must be float32 with the shape of the result");
        Mc = mask->contiguous();
    }
    DeviceGuard guard(Xc.device());
    Tensor Y = torch::empty_like(Xc), R;
    if (want_raw) R = torch::empty_like(Xc);
    ok(psp_spmm_window_xw_f32(ip(rowPtr_w), ip(colIdx_w), fp(values_w), fp(Xc), fp(Wc), transW ? 1 : 0, fpw(Y),
                              want_raw ? fpw(R) : nullptr, pspglue::fmt_rows(4, rowPtr_w), (int)colIdx_w.size(0), (int)N,
                              (int)Xc.size(0), relu_input ? 1 : 0, mask ? fp(Mc) : nullptr, stream_of(Xc)));
    if (want_raw) return {Y, R};
    return {Y};
}

// ---- attention layer on the windowed layout: SDDMM and SpMM of a direction in one launch ---------------------------------
static bool attn_window_supported(long K) { return K >= 4 && K % 4 == 0 && K <= PSP_ATTN_WINDOW_MAX_K; }

static void check_attn_window(const Tensor &X, const Tensor &rowPtr_w, const Tensor &colIdx_w, const char *what)
{
    need_gpu(X, what);
    need_gpu(rowPtr_w, "rowPtr_w");
    need_gpu(colIdx_w, "colIdx_w");
    need_f32(X, what, 2);
    need_i32(rowPtr_w, "rowPtr_w");
    need_i32(colIdx_w, "colIdx_w");
    pspglue::same_device(X, rowPtr_w, "attn_window");
    pspglue::same_device(X, colIdx_w, "attn_window");
    TORCH_CHECK(rowPtr_w.size(0) >= 2 && rowPtr_w.size(0) % 2 == 0, "rowPtr of the windowed format has 2 M + 2 entries");
    TORCH_CHECK(attn_window_supported(X.size(1)), "attn_window: the width must be a multiple of 4 up to ", PSP_ATTN_WINDOW_MAX_K);
    TORCH_CHECK((rowPtr_w.size(0) - 2) / 2 <= X.size(0), "rowPtr_w describes more rows than the dense operand has");
}

// (X, rowPtr_w, colIdx_w, alpha | None) -> [att = alpha <X_i, X_j> per stored entry, Y = att-weighted sum of the X rows]
static std::vector<Tensor> attn_window_forward(Tensor X, Tensor rowPtr_w, Tensor colIdx_w, c10::optional<Tensor> alpha)
{
    check_attn_window(X, rowPtr_w, colIdx_w, "X");
    if (alpha) {
        need_gpu(*alpha, "alpha");
        TORCH_CHECK(alpha->scalar_type() == torch::kFloat32 && alpha->numel() == 1, "alpha is one float32 on the device");
        pspglue::same_device(X, *alpha, "attn_window");
    }
    pspglue::DeviceGuard guard(X.device());
    Tensor att = torch::empty({colIdx_w.size(0)}, X.options());
    Tensor Y = torch::empty_like(X);
    const float *a = alpha ? alpha->data_ptr<float>() : nullptr;
    ok(psp_attn_window_forward_f32(ip(rowPtr_w), ip(colIdx_w), fp(X), a, colIdx_w.numel() ? fpw(att) : nullptr, fpw(Y),
                                   (int)(rowPtr_w.size(0) - 2) / 2, (int)colIdx_w.size(0), (int)X.size(1), (int)X.size(0),
                                   stream_of(X)));
    return {att, Y};
}

// (dY, att, rowPtr_w, colIdx_w) -> [G = att-weighted sum of the dY rows, sum_p <dY_i, dY_j> float(col(p)) as a 1-element tensor]
static std::vector<Tensor> attn_window_backward(Tensor dY, Tensor att, Tensor rowPtr_w, Tensor colIdx_w)
{
    check_attn_window(dY, rowPtr_w, colIdx_w, "dY");
    need_gpu(att, "att");
    need_f32(att, "att", 1);
    TORCH_CHECK(att.size(0) == colIdx_w.size(0), "att has one value per stored entry");
    pspglue::same_device(dY, att, "attn_window");
    pspglue::DeviceGuard guard(dY.device());
    Tensor G = torch::empty_like(dY);
    Tensor wsum = torch::empty({1}, dY.options());
    ok(psp_attn_window_backward_f32(ip(rowPtr_w), ip(colIdx_w), att.numel() ? fp(att) : nullptr, fp(dY), fpw(G), wsum.data_ptr<float>(),
                                    (int)(rowPtr_w.size(0) - 2) / 2, (int)colIdx_w.size(0), (int)dY.size(1), (int)dY.size(0),
                                    stream_of(dY)));
    return {G, wsum};
}

static Tensor forward_impl(int fmt, const Tensor &H, const Tensor &W, const Tensor &rowPtr, const Tensor &colIdx,
                           const Tensor &values, const Tensor *target_row, int CF, int blkWarpNum)
{
    need_gpu(H, "input");
    need_gpu(W, "weight");
    return aggregate(fmt, dense_xw(H, W, false), rowPtr, colIdx, values, target_row, CF, blkWarpNum);
}

static std::vector<Tensor> backward_impl(int fmt, const Tensor &dY, const Tensor &H, const Tensor &W, const Tensor &rowPtr,
                                         const Tensor &colIdx, const Tensor &values, const Tensor *target_row, int CF,
                                         int blkWarpNum)
{
    need_gpu(H, "H");
    need_gpu(W, "weight");
    // the reference multiplies by A, not A^T (SpCONV/SpCONV.h:67-71): exact for the symmetric matrices its
    // loaders build
    Tensor AG = aggregate(fmt, dY, rowPtr, colIdx, values, target_row, CF, blkWarpNum);
    return {dense_xw(AG, W, true), weight_gradient(H, AG)};
}

// ---- mean NLL loss of the training step (an addition of this build; F.nll_loss in GNN.py:131-146) ----------
static void check_loss_args(const Tensor &logp, const Tensor &labels)
{
    need_gpu(logp, "log-probabilities");
    need_gpu(labels, "labels");
    TORCH_CHECK(logp.dim() == 2 && logp.scalar_type() == torch::kFloat32 && logp.is_contiguous(),
                "nll_loss_mean: log-probabilities must be a contiguous float32 [n, C] tensor");
    TORCH_CHECK(labels.dim() == 1 && labels.scalar_type() == torch::kInt64 && labels.is_contiguous() &&
                    labels.size(0) == logp.size(0),
                "nll_loss_mean: labels must be a contiguous int64 tensor with one entry per row");
    TORCH_CHECK(logp.device() == labels.device(), "nll_loss_mean: tensors on different devices");
}
// returns [loss (0-dim), stats (sum, count, stray labels, workspace) for the backward call]
static std::vector<Tensor> nll_loss_mean(Tensor logp, Tensor labels)
{
    check_loss_args(logp, labels);
    DeviceGuard guard(logp.device());
    Tensor loss = torch::empty({}, logp.options()), stats = torch::empty({(long)psp_nll_loss_stats_floats()}, logp.options());
    ok(psp_nll_loss_mean_f32(fp(logp), (const long long *)labels.data_ptr<int64_t>(), logp.size(0), (int)logp.size(1),
                             loss.data_ptr<float>(), stats.data_ptr<float>(), stream_of(logp)));
    return {loss, stats};
}
static Tensor nll_loss_mean_backward(Tensor labels, Tensor grad_loss, Tensor stats, long n, long C)
{
    need_gpu(labels, "labels");
    need_gpu(grad_loss, "grad_loss");
    need_gpu(stats, "stats");
    TORCH_CHECK(labels.scalar_type() == torch::kInt64 && labels.is_contiguous() && labels.numel() == n, "bad labels");
    TORCH_CHECK(grad_loss.scalar_type() == torch::kFloat32 && grad_loss.numel() == 1, "grad_loss must hold one float");
    TORCH_CHECK(stats.scalar_type() == torch::kFloat32 && stats.numel() >= 2 && stats.is_contiguous(), "bad stats");
    DeviceGuard guard(labels.device());
    Tensor grad = torch::empty({n, C}, stats.options());
    ok(psp_nll_loss_mean_backward_f32((const long long *)labels.data_ptr<int64_t>(), grad_loss.data_ptr<float>(),
                                      stats.data_ptr<float>(), n, (int)C, fpw(grad), stream_of(labels)));
    return grad;
}

// the same loss from the logits (log-softmax folded in): [loss, stats]; and its gradient w.r.t. the logits
static bool softmax_nll_supported(long C) { return psp_softmax_nll_supported((int)C) != 0; }
static std::vector<Tensor> softmax_nll_mean(Tensor logits, Tensor labels)
{
    check_loss_args(logits, labels);
    TORCH_CHECK(softmax_nll_supported(logits.size(1)), "softmax_nll_mean: the class count must be a multiple of 4 up to 64");
    DeviceGuard guard(logits.device());
    Tensor loss = torch::empty({}, logits.options()), stats = torch::empty({(long)psp_nll_loss_stats_floats()}, logits.options());
    ok(psp_softmax_nll_mean_f32(fp(logits), (const long long *)labels.data_ptr<int64_t>(), logits.size(0), (int)logits.size(1),
                                loss.data_ptr<float>(), stats.data_ptr<float>(), stream_of(logits)));
    return {loss, stats};
}
static Tensor softmax_nll_mean_backward(Tensor logits, Tensor labels, Tensor grad_loss, Tensor stats)
{
    check_loss_args(logits, labels);
    need_gpu(grad_loss, "grad_loss");
    need_gpu(stats, "stats");
    TORCH_CHECK(grad_loss.scalar_type() == torch::kFloat32 && grad_loss.numel() == 1, "grad_loss must hold one float");
    TORCH_CHECK(stats.scalar_type() == torch::kFloat32 && stats.numel() >= 2 && stats.is_contiguous(), "bad stats");
    DeviceGuard guard(logits.device());
    Tensor grad = torch::empty_like(logits);
    ok(psp_softmax_nll_mean_backward_f32(fp(logits), (const long long *)labels.data_ptr<int64_t>(), grad_loss.data_ptr<float>(),
                                         stats.data_ptr<float>(), logits.size(0), (int)logits.size(1), fpw(grad), stream_of(logits)));
    return grad;
}

#define PSP_CONV(NAME, FMT)                                                                                       \
    static Tensor NAME##_forward(Tensor H, Tensor W, Tensor rowPtr, Tensor colIdx, Tensor values, int CF, int bw)  \
    {                                                                                                             \
        return forward_impl(FMT, H, W, rowPtr, colIdx, values, nullptr, CF, bw);                                  \
    }                                                                                                             \
    static std::vector<Tensor> NAME##_backward(Tensor dY, Tensor H, Tensor W, Tensor rowPtr, Tensor colIdx,       \
                                               Tensor values, int CF, int bw)                                     \
    {                                                                                                             \
        return backward_impl(FMT, dY, H, W, rowPtr, colIdx, values, nullptr, CF, bw);                             \
    }
#define PSP_CONV_SPLIT(NAME, FMT)                                                                                 \
    static Tensor NAME##_forward(Tensor H, Tensor W, Tensor rowPtr, Tensor colIdx, Tensor values, Tensor tr,      \
                                 int CF, int bw)                                                                  \
    {                                                                                                             \
        return forward_impl(FMT, H, W, rowPtr, colIdx, values, &tr, CF, bw);                                      \
    }                                                                                                             \
    static std::vector<Tensor> NAME##_backward(Tensor dY, Tensor H, Tensor W, Tensor rowPtr, Tensor colIdx,       \
                                               Tensor values, Tensor tr, int CF, int bw)                          \
    {                                                                                                             \
        return backward_impl(FMT, dY, H, W, rowPtr, colIdx, values, &tr, CF, bw);                                 \
    }

PSP_CONV(csr_spmm, 0)
PSP_CONV_SPLIT(csr_split_spmm, 1)
PSP_CONV(bcsr_spmm, 2)
PSP_CONV_SPLIT(bcsr_split_spmm, 3)

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    pspglue::check_abi();
    m.def("split_csr", &pspglue::split_csr, "row split on the host");
    m.def("split_csr_par", &pspglue::split_csr_par, "row split on the host with a precomputed segment prefix");
    // addition of this build: H^T * G for tall-skinny operands (memory-speed kernel for widths 16..64, else torch::mm)
    m.def("weight_gradient", [](Tensor H, Tensor G) {
        need_gpu(H, "H");
        need_gpu(G, "G");
        return weight_gradient(H, G);
    }, "H^T * G");
    m.def("dense_xw", [](Tensor X, Tensor W, bool transW) {
        need_gpu(X, "X");
        need_gpu(W, "W");
        return dense_xw(X, W, transW);
    }, "X * W (transW false) or X * W^T for tall-skinny X: (X, W, transW)");
    // the dense products of a layer that reads its input through a ReLU, for layers that place them around their
    // own sparse operators (the attention layer): max(Z, 0) * W, (G * W^T) where Z > 0, max(Z, 0)^T * G
    m.def("dense_relu_xw", [](Tensor Z, Tensor W) {
        need_gpu(Z, "Z");
        need_gpu(W, "W");
        return dense_relu_xw(Z, W);
    }, "max(Z, 0) * W: (Z, W)");
    m.def("dense_xwt_masked", [](Tensor G, Tensor W, Tensor Z) {
        need_gpu(G, "G");
        need_gpu(W, "W");
        need_gpu(Z, "Z");
        return dense_xwt_masked(G, W, Z);
    }, "(G * W^T) where Z > 0, else 0: (G, W, Z)");
    m.def("weight_gradient_relu", [](Tensor Z, Tensor G) {
        need_gpu(Z, "Z");
        need_gpu(G, "G");
        return weight_gradient_relu(Z, G);
    }, "max(Z, 0)^T * G: (Z, G)");
    m.def("nll_loss_mean", &nll_loss_mean, "[loss, stats] of the mean negative log-likelihood (log-probabilities, int64 labels)");
    m.def("nll_loss_mean_backward", &nll_loss_mean_backward, "gradient w.r.t. the log-probabilities: (labels, grad_loss, stats, n, C)");
    m.def("softmax_nll_supported", &softmax_nll_supported, "is there a fused log-softmax + NLL kernel for this class count?");
    m.def("softmax_nll_mean", &softmax_nll_mean, "[loss, stats] of nll_loss(log_softmax(logits), labels), mean over the rows");
    m.def("softmax_nll_mean_backward", &softmax_nll_mean_backward, "gradient w.r.t. the logits: (logits, labels, grad_loss, stats)");
    m.def("attn_window_forward", &attn_window_forward,
          "attention layer on the windowed layout: (X, rowPtr_w, colIdx_w, alpha | None) -> [att, Y]");
    m.def("attn_window_backward", &attn_window_backward,
          "attention layer on the windowed layout: (dY, att, rowPtr_w, colIdx_w) -> [G, weight-gradient sum]");
    m.def("attn_window_supported", &attn_window_supported, "is there a fused attention kernel for this width?");
    m.def("window_xw", &window_xw,
          "windowed layout, dense product folded in: (X, W, transW, rowPtr_w, colIdx_w, values_w, relu_input, mask | None, want_raw) -> [Y] or [Y, A f(X)]");
    m.def("window_xw_supported", &window_xw_supported, "widths the folded product exists for");
    m.def("aggregate", &aggregate_op, "A*D: (fmt, D, rowPtr, colIdx, values, target_row | None, CF, blkWarpNum)");
    m.def("aggregate_act", &aggregate_act_op,
          "A*max(D,0) (relu_input) and / or (A*D) where mask > 0: (fmt, D, rowPtr, colIdx, values, target_row | None, CF, blkWarpNum, relu_input, mask | None)");
    m.def("relu_input_forward", &relu_input_forward,
          "A*(relu(Z)*W): (fmt 0..3, Z, W, rowPtr, colIdx, values, target_row or None, CF, blkWarpNum)");
    m.def("relu_input_backward", &relu_input_backward,
          "[dZ, dW] of relu_input_forward: (fmt, dY, Z, W, rowPtr, colIdx, values, target_row or None, CF, blkWarpNum)");
    m.def("csr_spmm_forward", &csr_spmm_forward, "A*(H*W), CSR");
    m.def("csr_spmm_backward", &csr_spmm_backward, "[dH, dW], CSR");
    m.def("csr_split_spmm_forward", &csr_split_spmm_forward, "A*(H*W), row-split CSR");
    m.def("csr_split_spmm_backward", &csr_split_spmm_backward, "[dH, dW], row-split CSR");
    m.def("bcsr_spmm_forward", &bcsr_spmm_forward, "A*(H*W), 2x1 BCSR");
    m.def("bcsr_spmm_backward", &bcsr_spmm_backward, "[dH, dW], 2x1 BCSR");
    m.def("bcsr_split_spmm_forward", &bcsr_split_spmm_forward, "A*(H*W), row-split 2x1 BCSR");
    m.def("bcsr_split_spmm_backward", &bcsr_split_spmm_backward, "[dH, dW], row-split 2x1 BCSR");
}
