"""GCN / AGNN / GIN layers as autograd Functions over the PCSR operators (same surface and the same forward /
backward algebra as the reference's gnn_conv.py:13-238).  Layers look their operator up in ``spmm_dict`` by
output width (gnn_conv.py:121-124)."""
import math

import torch

import paramspmm_ae_amd  # noqa: F401
import ParamSpCONV as SpCONV

n_heads = 1

_CONV = {(False, False): "csr_spmm", (True, False): "csr_split_spmm", (False, True): "bcsr_spmm", (True, True): "bcsr_split_spmm"}


def _conv_args(op):
    args = [op.rowPtr, op.colIdx, op.val]
    if op.if_split:
        args.append(op.target_row)
    return args + [op.CF, _bw(op)]


def _bw(op):
    """blkWarpNum with the operator's launch flags (the XCD stripe chosen for its format, PCSR.pcsr_spmm.bw_flags)."""
    return op.blkWarpNum | getattr(op, "bw_flags", 0)


def _conv_name(op):
    return _CONV[(bool(op.if_split), op.vec_size != 1)]


def _fmt(op):
    """Format code of the generic entry points (pcsr_spmm.fmt_code: 0 csr, 1 csr_split, 2 bcsr, 3 bcsr_split,
    4 windowed csr); operators of other origin are described by if_split / vec_size."""
    code = getattr(op, "fmt_code", None)
    return (1 if op.if_split else 0) + (2 if op.vec_size != 1 else 0) if code is None else code


def _row_ptr(op):
    return getattr(op, "spmm_rowPtr", op.rowPtr)


def _window_xw(op, Z, weight):
    """Does the layer A (relu(Z) W) run as one windowed launch with the dense product folded in?  A windowed operator, a
    square weight matrix of a width the kernel has, float32."""
    return (_fmt(op) == 4 and weight.shape[0] == weight.shape[1] == Z.shape[1] and SpCONV.window_xw_supported(int(Z.shape[1]))
            and Z.dtype == torch.float32 and getattr(op, "fold_dense", True))


def _aggregate(op, D):
    """A D through ``op``'s format and configuration."""
    return SpCONV.aggregate(_fmt(op), D, _row_ptr(op), op.colIdx, op.val, op.target_row if op.if_split else None, op.CF,
                            _bw(op))


class _NllLossMean(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logp, labels):
        loss, stats = SpCONV.nll_loss_mean(logp, labels)
        ctx.save_for_backward(labels, stats)
        ctx.shape = tuple(logp.shape)
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        labels, stats = ctx.saved_tensors
        return SpCONV.nll_loss_mean_backward(labels, grad_loss.contiguous(), stats, ctx.shape[0], ctx.shape[1]), None


def nll_loss_mean(logp, labels):
    """``F.nll_loss(logp, labels)`` (mean over the rows, the loss of the reference's training step, GNN.py:131-146)
    through the library's kernels.  PyTorch reduces the whole batch in one workgroup -- 1.7 ms per step forward plus
    backward on 10^6 nodes -- where these kernels take some tens of microseconds.  Rows whose label is outside
    [0, C) do not count, as with PyTorch's ignore_index.  Anything but contiguous float32 CUDA log-probabilities with
    int64 labels goes to PyTorch."""
    if (logp.is_cuda and logp.dtype == torch.float32 and logp.dim() == 2 and labels.dtype == torch.int64
            and labels.dim() == 1):
        return _NllLossMean.apply(logp.contiguous(), labels.contiguous())
    return torch.nn.functional.nll_loss(logp, labels)


class _SoftmaxNllMean(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels):
        loss, stats = SpCONV.softmax_nll_mean(logits, labels)
        ctx.save_for_backward(logits, labels, stats)
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        logits, labels, stats = ctx.saved_tensors
        return SpCONV.softmax_nll_mean_backward(logits, labels, grad_loss.contiguous(), stats), None


def softmax_nll_loss_mean(logits, labels):
    """``F.nll_loss(F.log_softmax(logits, dim=1), labels)`` -- the end of the reference's networks and the loss of its
    training step (GNN.py:61,78,101 and 131-146) -- as one function of the logits: one pass over the [n, C] matrix
    forward, one read and one write backward, where the two separate operators make five.  Class counts other than a
    multiple of 4 up to 64, and anything but contiguous float32 CUDA logits with int64 labels, take the separate
    operators."""
    if (logits.is_cuda and logits.dtype == torch.float32 and logits.dim() == 2 and labels.dtype == torch.int64
            and labels.dim() == 1 and SpCONV.softmax_nll_supported(int(logits.shape[1]))):
        return _SoftmaxNllMean.apply(logits.contiguous(), labels.contiguous())
    return nll_loss_mean(torch.nn.functional.log_softmax(logits, dim=1), labels)


class GCNFunction(torch.autograd.Function):
    """forward A(HW); backward dH = (A dY) W^T, dW = H^T (A dY) -- A is symmetric (gnn_conv.py:13-107)."""

    @staticmethod
    def forward(ctx, H, weight, ParamSpMM):
        ctx.save_for_backward(H, weight)
        ctx.ParamSpMM = ParamSpMM
        if _fmt(ParamSpMM) == 4:  # the windowed layout has no named operator of its own: dense product, then A
            return _aggregate(ParamSpMM, SpCONV.dense_xw(H, weight, False))
        return getattr(SpCONV, _conv_name(ParamSpMM) + "_forward")(H, weight, *_conv_args(ParamSpMM))

    @staticmethod
    def backward(ctx, d_output):
        H, weight = ctx.saved_tensors
        op = ctx.ParamSpMM
        if not ctx.needs_input_grad[0]:
            # the network's first layer: its input holds features, nothing asks for their gradient
            return None, SpCONV.weight_gradient(H, _aggregate(op, d_output)), None
        if _fmt(op) == 4:
            AG = _aggregate(op, d_output.contiguous())
            return SpCONV.dense_xw(AG, weight, True), SpCONV.weight_gradient(H, AG), None
        d_input, d_weight = getattr(SpCONV, _conv_name(op) + "_backward")(d_output.contiguous(), H, weight, *_conv_args(op))
        return d_input, d_weight, None


class GCNAggregateFirstFunction(torch.autograd.Function):
    """The same layer computed as (A H) W: for a layer that widens its input (in_features < out_features) the sparse
    product then runs at the input's width.  Backward: dW = (A H)^T dY (A H is kept from the forward pass, so the
    weight gradient needs no sparse product) and dH = A (dY W^T), again at the input's width -- A is symmetric, as in
    the reference's own backward (gnn_conv.py:56-107).  ``ParamSpMM`` is the operator configured for the *input*
    width."""

    @staticmethod
    def forward(ctx, H, weight, ParamSpMM):
        AH = _aggregate(ParamSpMM, H)
        ctx.save_for_backward(AH, weight)
        ctx.ParamSpMM = ParamSpMM
        return SpCONV.dense_xw(AH, weight, False)

    @staticmethod
    def backward(ctx, d_output):
        AH, weight = ctx.saved_tensors
        d_output = d_output.contiguous()
        d_weight = SpCONV.weight_gradient(AH, d_output)
        d_input = None
        if ctx.needs_input_grad[0]:
            d_input = _aggregate(ctx.ParamSpMM, SpCONV.dense_xw(d_output, weight, True))
        return d_input, d_weight, None


class GCNReLUInputFunction(torch.autograd.Function):
    """The GCN layer reading its input through a ReLU, A (relu(Z) W), as one function of the pre-activation values
    Z: forward relu(Z) W with the activation applied as Z is read; backward dZ = ((A dY) W^T) where Z > 0 and
    dW = relu(Z)^T (A dY), again without a pass for the activation.  Five layers with F.relu between them
    (GNN.py:43-61) are conv1(x), then four of these."""

    @staticmethod
    def forward(ctx, Z, weight, ParamSpMM):
        ctx.save_for_backward(Z, weight)
        ctx.ParamSpMM = ParamSpMM
        op = ParamSpMM
        if _window_xw(op, Z, weight):
            # windowed layout, square layer: (A relu(Z)) W in one launch, the dense product in the kernel's epilogue
            return SpCONV.window_xw(Z, weight, False, op.spmm_rowPtr, op.colIdx, op.val, True, None, False)[0]
        return SpCONV.relu_input_forward(_fmt(op), Z, weight, _row_ptr(op), op.colIdx, op.val,
                                         op.target_row if op.if_split else None, op.CF, _bw(op))

    @staticmethod
    def backward(ctx, d_output):
        Z, weight = ctx.saved_tensors
        op = ctx.ParamSpMM
        if _window_xw(op, Z, weight):
            # one launch delivers A dY (for the weight gradient) and ((A dY) W^T) where Z > 0 (the input gradient)
            d_input, AG = SpCONV.window_xw(d_output.contiguous(), weight, True, op.spmm_rowPtr, op.colIdx, op.val, False, Z, True)
            return d_input, SpCONV.weight_gradient_relu(Z, AG), None
        d_input, d_weight = SpCONV.relu_input_backward(_fmt(op), d_output.contiguous(), Z, weight, _row_ptr(op), op.colIdx, op.val,
                                                       op.target_row if op.if_split else None, op.CF, _bw(op))
        return d_input, d_weight, None


class _Layer(torch.nn.Module):
    def __init__(self, input_dim, output_dim):
        super().__init__()
        self.weights = torch.nn.Parameter(torch.randn(input_dim, output_dim))
        self.reset_parameters()

    def reset_parameters(self):
        bound = 1.0 / math.sqrt(self.weights.size(1))
        self.weights.data.uniform_(-bound, bound)

    def _operator(self, spmm_dict):
        width = self.weights.size(1)
        if width not in spmm_dict:
            raise ValueError("SpMMDecider not support dim: " + str(width))
        return spmm_dict[width]


class GCNConv(_Layer):
    aggregate_first = True  # (A H) W where that is the cheaper order and spmm_dict holds an operator for H's width

    def forward(self, H, spmm_dict, relu_input=False):
        """``relu_input``: H holds pre-activation values and the layer computes A (relu(H) W); the activation and its
        backward are folded into the dense products around the sparse one.

        A layer that widens its input is computed as (A H) W when ``spmm_dict`` also holds an operator for the input's
        width (the reference's layers look up the output's width only, gnn_conv.py:121-124, and always compute
        A (H W))."""
        in_w, out_w = self.weights.shape
        if self.aggregate_first and not relu_input and in_w < out_w and in_w in spmm_dict:
            return GCNAggregateFirstFunction.apply(H, self.weights, spmm_dict[in_w])
        fn = GCNReLUInputFunction if relu_input else GCNFunction
        return fn.apply(H, self.weights, self._operator(spmm_dict))


class AGNNFunction(torch.autograd.Function):
    """X' = XW; e = <X'_i, X'_j> per stored entry; attention = e * w; out = SpMM(attention, X')
    (gnn_conv.py:128-180).  No softmax, as in the reference."""

    @staticmethod
    def forward(ctx, X, weights, attention_w, ParamSpMM, colIdx, relu_input=False):
        # relu_input: X holds pre-activation values; the activation and its backward ride on the dense products
        ctx.relu_input = bool(relu_input)
        X_prime = SpCONV.dense_relu_xw(X, weights) if relu_input else SpCONV.dense_xw(X, weights, False)
        ctx.fused = (_fmt(ParamSpMM) == 4 and X_prime.dtype == torch.float32
                     and SpCONV.attn_window_supported(int(X_prime.shape[1])))
        if ctx.fused:
            # windowed operator: scores (the head's weight multiplied in) and their aggregation in one launch
            edge_attentions, out = SpCONV.attn_window_forward(X_prime, ParamSpMM.spmm_rowPtr, ParamSpMM.colIdx,
                                                              attention_w.detach().reshape(-1)[:1])
        else:
            if _fmt(ParamSpMM) == 4:
                edge_attentions = ParamSpMM.AGNN_sddmm(X_prime, attention_w.detach().reshape(-1)[:1])
            else:
                edge_feature = ParamSpMM.AGNN_sddmm(X_prime)
                # csr: [nnz] ; 2x1 blocks: [nblk, 2] -- a single head scales both the same way
                edge_attentions = (edge_feature * attention_w.reshape(())).contiguous()
            out = ParamSpMM.AGNN_spmm(edge_attentions, X_prime)
        ctx.save_for_backward(X, weights, edge_attentions)
        ctx.colIdx = colIdx
        ctx.ParamSpMM = ParamSpMM
        return out

    @staticmethod
    def backward(ctx, d_output):
        op = ctx.ParamSpMM
        X, weights, edge_attentions = ctx.saved_tensors
        d_output = d_output.contiguous()
        if ctx.fused:
            # A_att dY and the reference's sum for the attention weight (below) in one launch
            d_input_prime, d_attention_w = SpCONV.attn_window_backward(d_output, edge_attentions, op.spmm_rowPtr, op.colIdx)
        else:
            d_input_prime = op.AGNN_spmm(edge_attentions, d_output)
        if not ctx.needs_input_grad[0]:
            d_input = None
        elif ctx.relu_input:
            d_input = SpCONV.dense_xwt_masked(d_input_prime, weights, X)
        else:
            d_input = SpCONV.dense_xw(d_input_prime, weights, True)
        # X^T * d_input_prime (relu(X)^T when the layer reads X through the activation)
        d_weights = SpCONV.weight_gradient_relu(X, d_input_prime) if ctx.relu_input else SpCONV.weight_gradient(X, d_input_prime)
        if ctx.fused:
            return d_input, d_weights, d_attention_w.reshape(1, 1).expand(1, n_heads), None, None, None
        d_attention = op.AGNN_sddmm(d_output)
        if d_attention.dim() != 1:
            d_attention = d_attention.view(-1)[op.mask]  # block layout -> CSR slots
        # the reference's literal formula for the attention weight gradient (gnn_conv.py:172):
        # mm(d_attention[1, nnz] expanded to n_heads rows, colIdx.float()[nnz, 1])^T.  Every row of the product is the
        # same dot product over the nnz entries; as a GEMM it takes 20 ms on 2*10^7 entries (a 1 x nnz x 1 problem),
        # as a dot product some tens of microseconds.  The float copy of colIdx is made once per operator.
        # A windowed operator keeps its entries in its own order inside the rows: its colIdx is the one that matches.
        col_f = getattr(op, "_colIdx_as_float", None)
        if col_f is None or col_f.numel() != ctx.colIdx.numel():
            col_f = (op.colIdx if _fmt(op) == 4 else ctx.colIdx).reshape(-1).to(d_attention.dtype)
            op._colIdx_as_float = col_f
        d_attention_w = torch.dot(d_attention, col_f).reshape(1, 1).expand(1, n_heads)
        return d_input, d_weights, d_attention_w, None, None, None


class AGNNConv(_Layer):
    def __init__(self, input_dim, output_dim):
        super().__init__(input_dim, output_dim)
        self.attention_w = torch.nn.Parameter(torch.randn(1, n_heads))

    def forward(self, X, spmm_dict, colIdx, relu_input=False):
        return AGNNFunction.apply(X, self.weights, self.attention_w, self._operator(spmm_dict), colIdx, relu_input)


class GINFunction(torch.autograd.Function):
    """forward (A X) W; backward dW = (A X)^T dY, dX = A (dY W^T) (gnn_conv.py:202-220)."""

    @staticmethod
    def forward(ctx, X, weight, ParamSpMM):
        X_agg = ParamSpMM.GIN_spmm(X)
        ctx.save_for_backward(X_agg, weight)
        ctx.ParamSpMM = ParamSpMM
        return SpCONV.dense_xw(X_agg, weight, False)

    @staticmethod
    def backward(ctx, d_output):
        X_agg, weights = ctx.saved_tensors
        d_output = d_output.contiguous()  # an upstream gradient may be a view (expand, transpose, slice)
        d_weights = SpCONV.weight_gradient(X_agg, d_output)  # X_agg^T * d_output
        # the network's first layer reads the features, which need no gradient: no dense and no sparse product for it
        d_input = ctx.ParamSpMM.GIN_spmm(SpCONV.dense_xw(d_output, weights, True)) if ctx.needs_input_grad[0] else None
        return d_input, d_weights, None


class GINReLUInputFunction(torch.autograd.Function):
    """(A relu(Z)) W as one function of the pre-activation values Z, for a layer that widens its input: the activation
    is applied as the sparse product gathers the rows of Z (ParamSpCONV.aggregate_act), the gradient is masked in a pass
    that follows the backward product.  The reference's driver applies F.relu between the layers (GNN.py:63-78)."""

    @staticmethod
    def forward(ctx, Z, weight, ParamSpMM):
        op = ParamSpMM
        X_agg = SpCONV.aggregate_act(_fmt(op), Z, _row_ptr(op), op.colIdx, op.val, op.target_row if op.if_split else None, op.CF,
                                     _bw(op), True, None)
        ctx.save_for_backward(X_agg, weight, Z)
        ctx.ParamSpMM = op
        return SpCONV.dense_xw(X_agg, weight, False)

    @staticmethod
    def backward(ctx, d_output):
        X_agg, weights, Z = ctx.saved_tensors
        op = ctx.ParamSpMM
        d_output = d_output.contiguous()
        d_weights = SpCONV.weight_gradient(X_agg, d_output)
        d_input = SpCONV.aggregate_act(_fmt(op), SpCONV.dense_xw(d_output, weights, True), _row_ptr(op), op.colIdx, op.val,
                                       op.target_row if op.if_split else None, op.CF, _bw(op), False, Z)
        return d_input, d_weights, None


class GINConv(_Layer):
    operator_of_input_width = True

    def forward(self, X, spmm_dict, relu_input=False):
        """``relu_input``: X holds pre-activation values and the layer computes (A relu(X)) W without an activation
        pass.  A layer that does not widen its input is evaluated as A (relu(X) W) -- the same product, the sparse
        part at the narrower width -- with the activation and its backward folded into the dense products, like the
        GCN layer; a widening layer applies the activation inside the sparse product."""
        in_w, out_w = self.weights.shape
        if relu_input and in_w >= out_w:
            op = self._operator(spmm_dict)
            if op.vec_size in (1, 2):
                return GCNReLUInputFunction.apply(X, self.weights, op)
        # the sparse product runs at the input's width: take the operator configured for that width when there is
        # one (the reference's layers look up the output's width only, gnn_conv.py:223-226)
        op = spmm_dict[in_w] if self.operator_of_input_width and in_w in spmm_dict else self._operator(spmm_dict)
        if relu_input and op.vec_size in (1, 2):
            return GINReLUInputFunction.apply(X, self.weights, op)
        if relu_input:
            X = torch.relu(X)
        return GINFunction.apply(X, self.weights, op)
