"""Quantized linear layer: mirrors cuda/QLinear.py of the reference.

Forward quantizes X and W inside the GEMM call (truncation, as the reference's
fused quantize-on-load does), keeps the int8 copies and their scales for the
backward pass (the "quantize-GEMM caching" path, cuda/QLinear.py:34), and in
the ``_reduce`` variant also returns max|Y|/127 from the GEMM epilogue so that
the following SpMM can skip its absmax pass (cuda/QLinear.py:50-60).
"""
import torch
import torch.nn as nn
from torch.autograd.function import Function, once_differentiable

from . import config, kernels


def _padded_i8(rows, cols, device):
    """[rows, cols] int8 view whose rows start 16-byte aligned."""
    ld = (cols + 15) // 16 * 16
    return torch.empty((rows, ld), dtype=torch.int8, device=device)[:, :cols]


def _quantize_grad(dY, want_colsum=False):
    """Quantize a gradient (cuda/QLinear.py:42) with the configured rounding.  Returns
    (int8, scale, column sums or None): the bias gradient dY.sum(0) (cuda/QLinear.py:46)
    comes out of the same read of dY that finds its scale; a scale that the producer of dY left on it
    (an aggregation's epilogue) is taken instead of a pass over dY."""
    from .SPMM import grad_scale_hint
    scale = grad_scale_hint(dY) if dY.is_contiguous() else None
    dY = dY if dY.is_contiguous() else dY.contiguous()
    colsum = None
    if want_colsum:
        scale, colsum = kernels.cuda_kernels.absmax_ex(dY, want_colsum=True)
    kw = {"round_mode": config.grad_round_mode}
    if config.grad_round_mode == "stochastic":
        kw.update(config.stochastic_args(dY.device))
    q, scale = kernels.quantize_padded(dY, scale, **kw)
    return q, scale, colsum


class QgemmNT_func(Function):
    """cuda/QLinear.py:9-23 (legacy un-fused path)."""

    @staticmethod
    def forward(ctx, A, B):
        ctx.save_for_backward(A, B)
        return kernels.cuda_kernels.QgemmNT(A, B)

    @staticmethod
    def backward(ctx, grad_output):
        kernels.refuse_capture("QgemmNT_func.backward")
        A, B = ctx.saved_tensors
        grad_A = grad_B = None
        grad_output = grad_output.contiguous()
        if ctx.needs_input_grad[0]:
            grad_A = kernels.cuda_kernels.QgemmNN(grad_output, B)
        if ctx.needs_input_grad[1]:
            grad_B = kernels.cuda_kernels.QgemmTN(grad_output, A)
        return grad_A, grad_B


def quantize_input(X, scaleX=None):
    """(int8 X, scale) the way the forward GEMM quantizes its input, for layers that share one input:
    pass both to each ``QLinear.forward`` and X is read and quantized once instead of once per layer."""
    X = X.reshape(-1, X.size(-1))
    X = X if X.is_contiguous() else X.contiguous()
    return kernels.quantize_padded(X, scaleX, round_mode=kernels.default_forward_round_mode())


def _forward(ctx, X, W, b, reduce, row_scale=None, scaleX=None, Xq=None):
    from .SPMM import relu_mask_of
    # X straight out of an aggregation's fused ReLU: the backward pass can hand that op the scale it needs
    ctx.dx_masked = relu_mask_of(X) if X.dim() == 2 and X.is_contiguous() else None
    X = X if X.is_contiguous() else X.contiguous()
    if Xq is not None:
        if scaleX is None or row_scale is not None:
            raise RuntimeError("QLinear: a quantized input needs its scale and excludes row_scale")
        if tuple(Xq.shape) != tuple(X.shape) or Xq.dtype != torch.int8:
            raise RuntimeError("QLinear: the quantized input must be int8 of the input's shape")
        scaleW = kernels.cuda_kernels.get_scale(W if W.is_contiguous() else W.contiguous())
        W_ = torch.empty(W.shape, dtype=torch.int8, device=X.device)
        res = kernels.QGEMM_forward(None, Xq, scaleX, W, W_, scaleW, b, reduce)
        ctx.backward_cache = Xq, scaleX, W_, scaleW, b, None
        return res
    if scaleX is not None:
        pass  # with row_scale: the scale of X * row_scale[:, None], as its producer found it
    elif row_scale is not None:
        # the layer's "X * row_scale[:, None]" is folded into the quantize pass (no fp32 copy of X)
        scaleX, _ = kernels.cuda_kernels.absmax_ex(X, row_mul=row_scale)
    else:
        scaleX = kernels.cuda_kernels.get_scale(X)
    scaleW = kernels.cuda_kernels.get_scale(W if W.is_contiguous() else W.contiguous())
    X_ = _padded_i8(X.size(0), X.size(1), X.device)
    W_ = torch.empty(W.shape, dtype=torch.int8, device=X.device)
    res = kernels.QGEMM_forward(X, X_, scaleX, W, W_, scaleW, b, reduce, x_row_mul=row_scale)
    ctx.backward_cache = X_, scaleX, W_, scaleW, b, row_scale
    return res


def _backward(ctx, grad_output):
    kernels.refuse_capture("QLinear.backward")
    X_, scaleX, W_, scaleW, b, row_scale = ctx.backward_cache
    want_bias = b is not None and ctx.needs_input_grad[2]
    dY_, scaledY, grad_bias = _quantize_grad(grad_output, want_bias)
    grad_input, grad_weight = kernels.QGEMM_backward(
        dY_, X_, W_, scaledY, scaleX, scaleW, ctx.needs_input_grad[0], ctx.needs_input_grad[1],
        x_row_scale=row_scale, dx_masked=getattr(ctx, "dx_masked", None))
    return grad_input, grad_weight, grad_bias, None


class Qlinear_func(Function):
    """cuda/QLinear.py:26-47.  ``row_scale`` (optional, [M]) multiplies the rows of X before
    quantization, fused into the quantize pass and, in backward, into gradX's epilogue.
    ``scaleX`` (optional, [1]) is max|X| / 127 (of X * row_scale[:, None] when ``row_scale`` is given) when
    the producer of X already knows it (a preceding Qlinear_func_reduce, an aggregation's epilogue): no absmax
    pass over X runs then.  ``Xq`` (optional, with
    ``scaleX``): X already quantized (``quantize_input``), shared by several layers."""

    @staticmethod
    def forward(ctx, X, W, b=None, row_scale=None, scaleX=None, Xq=None):
        return _forward(ctx, X, W, b, False, row_scale, scaleX, Xq)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        return _backward(ctx, grad_output) + (None, None)


class Qlinear_func_reduce(Function):
    """cuda/QLinear.py:50-71: also returns the output's quantization scale."""

    @staticmethod
    def forward(ctx, X, W, b=None, row_scale=None, scaleX=None, Xq=None):
        out, scaleO = _forward(ctx, X, W, b, True, row_scale, scaleX, Xq)
        ctx.mark_non_differentiable(scaleO)
        ctx.set_materialize_grads(False)  # no zero tensor (a fill launch) for the scale's absent gradient
        return out, scaleO

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output, grad_dummy):
        if grad_output is None:
            return (None,) * 6
        return _backward(ctx, grad_output) + (None, None)


class Qlinear_shared_func(Function):
    """Several linear layers over one input (the k / v / q projections of evaluation/test_HGT.py:51-53)
    as one autograd node: ``apply(X, Xq, scaleX, n, W_0, b_0, ..., W_n-1, b_n-1, V_0, c_0, ...)`` with
    (Xq, scaleX) from ``quantize_input(X)`` returns (Y_0, scale_0, Y_1, scale_1, ...), each pair what
    Qlinear_func_reduce returns; where (V_i, c_i) is not (None, None), Y_i is that second layer applied to the
    first one's output (evaluation/test_HGT.py:54-55), which is then kept in int8 only.  Backward runs each layer's weight / bias gradient as usual, and the input gradients go into
    one tensor: the first layer's GEMM writes it, the others add to it in their epilogues, where autograd
    would run a separate addition per extra layer over three [M, K] fp32 tensors."""

    @staticmethod
    def forward(ctx, X, Xq, scaleX, n_first, *wb):
        """``wb``: (W, b) of the ``n_first`` layers applied to X, then (W2, b2) or (None, None) per layer:
        a second linear layer applied to that layer's output, which then is the only reader of it."""
        if n_first < 1 or len(wb) != 4 * n_first:
            raise RuntimeError("Qlinear_shared_func: expects (weight, bias) of every layer and of its follower")
        if tuple(Xq.shape) != tuple(X.shape) or Xq.dtype != torch.int8 or X.dim() != 2:
            raise RuntimeError("Qlinear_shared_func: the quantized input must be int8 of the 2-D input's shape")
        ctx.set_materialize_grads(False)
        outs, layers, scales = [], [], []
        get_scale = kernels.cuda_kernels.get_scale
        for i in range(n_first):
            W, b = wb[2 * i], wb[2 * i + 1]
            W2, b2 = wb[2 * n_first + 2 * i], wb[2 * n_first + 2 * i + 1]
            scaleW = get_scale(W if W.is_contiguous() else W.contiguous())
            W_ = torch.empty(W.shape, dtype=torch.int8, device=X.device)
            second = None
            if W2 is None:
                out, scaleO = kernels.QGEMM_forward(None, Xq, scaleX, W, W_, scaleW, b, True)
            else:
                # the first layer's output in int8 only (nothing but the second layer reads it), where the
                # kernel for that applies; else in fp32 and quantized by the second GEMM as usual
                Yq = _padded_i8(X.size(0), W.size(0), X.device)
                sY = torch.empty_like(scaleX)
                Y = None
                if not kernels.cuda_kernels.QGEMM_forward_q8(Yq, sY, Xq, W, W_, b, scaleX, scaleW):
                    Y, sY = kernels.QGEMM_forward(None, Xq, scaleX, W, W_, scaleW, b, True)
                scaleW2 = get_scale(W2 if W2.is_contiguous() else W2.contiguous())
                W2_ = torch.empty(W2.shape, dtype=torch.int8, device=X.device)
                out, scaleO = kernels.QGEMM_forward(Y, Yq, sY, W2, W2_, scaleW2, b2, True)
                second = (Yq, sY, W2_, scaleW2, b2 is not None)
            scales.append(scaleO)
            outs += [out, scaleO]
            layers.append((W_, scaleW, b is not None, second))
        ctx.mark_non_differentiable(*scales)  # one call: each call replaces the set of the one before
        ctx.backward_cache = Xq, scaleX, layers
        return tuple(outs)

    @staticmethod
    @once_differentiable
    def backward(ctx, *grads):
        kernels.refuse_capture("Qlinear_shared_func.backward")
        Xq, scaleX, layers = ctx.backward_cache
        n = len(layers)
        need = ctx.needs_input_grad
        dX, first, second = None, [None] * (2 * n), [None] * (2 * n)
        for i, (W_, scaleW, has_bias, chained) in enumerate(layers):
            dY = grads[2 * i]
            if dY is None:
                continue
            if chained is not None:  # back through the second layer to the first layer's output
                Yq, sY, W2_, scaleW2, has_bias2 = chained
                dY_, scaledY, second[2 * i + 1] = _quantize_grad(dY, has_bias2 and need[4 + 2 * n + 2 * i + 1])
                dY, second[2 * i] = kernels.QGEMM_backward(dY_, Yq, W2_, scaledY, sY, scaleW2, True,
                                                           need[4 + 2 * n + 2 * i])
            dY_, scaledY, first[2 * i + 1] = _quantize_grad(dY, has_bias and need[4 + 2 * i + 1])
            dXi, first[2 * i] = kernels.QGEMM_backward(dY_, Xq, W_, scaledY, scaleX, scaleW, need[0], need[4 + 2 * i],
                                                       dX_acc=dX)
            dX = dXi if dXi is not None else dX
        return (dX, None, None, None) + tuple(first) + tuple(second)


def shared_input_linears(X, layers, scaleX=None, then=None):
    """[(Y, scale of Y)] of the QLinear ``layers`` applied to one 2-D input: X is quantized once and the
    layers run as one autograd node (Qlinear_shared_func).  ``then``: per layer, None or a second QLinear
    applied to that layer's output (``then[i](layers[i](X))``); the pair returned is the second layer's."""
    Xq, scaleX = quantize_input(X, scaleX)
    X = X if X.is_contiguous() else X.contiguous()
    then = [None] * len(layers) if then is None else list(then)
    if len(then) != len(layers):
        raise RuntimeError("shared_input_linears: one entry of `then` per layer")
    flat = [t for lin in layers for t in (lin.weight, lin.bias)]
    flat += [t for lin in then for t in ((lin.weight, lin.bias) if lin is not None else (None, None))]
    res = Qlinear_shared_func.apply(X, Xq, scaleX, len(layers), *flat)
    return [(res[2 * i], res[2 * i + 1]) for i in range(len(layers))]


class QLinear(nn.Linear):
    """cuda/QLinear.py:74-93.  The reference requires in_features % 4 == 0 for
    its 128-bit loads; any width works here."""

    def __init__(self, in_features, out_features, bias=True):
        super(QLinear, self).__init__(in_features, out_features, bias)
        self.isReduce = False

    def enable_reduce(self):
        self.isReduce = True

    def forward(self, input, scale=None, input_q=None):
        """``scale``: max|input| / 127 if the caller has it (the second output of a preceding
        layer with enable_reduce()); the reference's layer always recomputes it.  ``input_q``
        (with ``scale``): the input already quantized by ``quantize_input``."""
        t = input.reshape(-1, input.size(-1))
        out_shape = input.shape[:-1] + (self.weight.size(0),)
        if self.isReduce:
            out, oscale = Qlinear_func_reduce.apply(t, self.weight, self.bias, None, scale, input_q)
            return out.reshape(out_shape), oscale
        out = Qlinear_func.apply(t, self.weight, self.bias, None, scale, input_q)
        return out.reshape(out_shape)
