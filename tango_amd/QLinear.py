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


def _quantize_grad(dY):
    """Quantize a gradient (cuda/QLinear.py:42) with the configured rounding."""
    dY = dY if dY.is_contiguous() else dY.contiguous()
    if config.grad_round_mode == "stochastic":
        return kernels.quantize_padded(dY, round_mode="stochastic", seed=config.seed,
                                       offset=config.next_offset())
    return kernels.quantize_padded(dY, round_mode=config.grad_round_mode)


class QgemmNT_func(Function):
    """cuda/QLinear.py:9-23 (legacy un-fused path)."""

    @staticmethod
    def forward(ctx, A, B):
        ctx.save_for_backward(A, B)
        return kernels.cuda_kernels.QgemmNT(A, B)

    @staticmethod
    def backward(ctx, grad_output):
        A, B = ctx.saved_tensors
        grad_A = grad_B = None
        grad_output = grad_output.contiguous()
        if ctx.needs_input_grad[0]:
            grad_A = kernels.cuda_kernels.QgemmNN(grad_output, B)
        if ctx.needs_input_grad[1]:
            grad_B = kernels.cuda_kernels.QgemmTN(grad_output, A)
        return grad_A, grad_B


def _forward(ctx, X, W, b, reduce, row_scale=None):
    X = X if X.is_contiguous() else X.contiguous()
    if row_scale is not None:
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
    X_, scaleX, W_, scaleW, b, row_scale = ctx.backward_cache
    grad_bias = None
    dY_, scaledY = _quantize_grad(grad_output)
    grad_input, grad_weight = kernels.QGEMM_backward(
        dY_, X_, W_, scaledY, scaleX, scaleW, ctx.needs_input_grad[0], ctx.needs_input_grad[1],
        x_row_scale=row_scale)
    if b is not None and ctx.needs_input_grad[2]:
        grad_bias = grad_output.sum(0)
    return grad_input, grad_weight, grad_bias, None


class Qlinear_func(Function):
    """cuda/QLinear.py:26-47.  ``row_scale`` (optional, [M]) multiplies the rows of X before
    quantization, fused into the quantize pass and, in backward, into gradX's epilogue."""

    @staticmethod
    def forward(ctx, X, W, b=None, row_scale=None):
        return _forward(ctx, X, W, b, False, row_scale)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        return _backward(ctx, grad_output)


class Qlinear_func_reduce(Function):
    """cuda/QLinear.py:50-71: also returns the output's quantization scale."""

    @staticmethod
    def forward(ctx, X, W, b=None, row_scale=None):
        out, scaleO = _forward(ctx, X, W, b, True, row_scale)
        ctx.mark_non_differentiable(scaleO)
        return out, scaleO

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output, grad_dummy):
        return _backward(ctx, grad_output)


class QLinear(nn.Linear):
    """cuda/QLinear.py:74-93.  The reference requires in_features % 4 == 0 for
    its 128-bit loads; any width works here."""

    def __init__(self, in_features, out_features, bias=True):
        super(QLinear, self).__init__(in_features, out_features, bias)
        self.isReduce = False

    def enable_reduce(self):
        self.isReduce = True

    def forward(self, input):
        t = input.reshape(-1, input.size(-1))
        out_shape = input.shape[:-1] + (self.weight.size(0),)
        if self.isReduce:
            out, scale = Qlinear_func_reduce.apply(t, self.weight, self.bias)
            return out.reshape(out_shape), scale
        out = Qlinear_func.apply(t, self.weight, self.bias)
        return out.reshape(out_shape)
