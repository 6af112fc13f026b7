"""Batch normalisation of node features with the ReLU that follows it folded in.

The reference's arxiv stacks normalise between graph layers with ``torch.nn.BatchNorm1d`` and then apply the
activation (evaluation/arxiv_gat.py:376-448, evaluation/arxiv_gcn.py:156-209).  ``BatchNorm1dAct`` is that
module (same parameters, buffers and state dict) whose training-mode pass on 2-D fp32 GPU features runs as two
HBM-bound passes forward and two backward, each with reductions in a fixed order; everything else (evaluation
mode, other shapes) is torch's own batch normalisation followed by the activation."""
import torch
import torch.nn.functional as F
from torch import nn
from torch.autograd.function import Function, once_differentiable

from .kernels import _L, _ptr, _stream, _workspace, check, refuse_capture


def _fusable(x, cols, weight, bias):
    """The kernels read x, weight and bias as contiguous fp32 on x's device and merge per-workgroup row counts held
    as floats (exact below 2^24 rows); anything else takes torch's batch normalisation."""
    def ok(t):
        return t is not None and t.dtype == torch.float32 and t.device == x.device and t.is_contiguous()
    return (x.is_cuda and x.dim() == 2 and x.dtype == torch.float32 and 1 <= cols <= 2048
            and 1 < x.size(0) < (1 << 24) and ok(weight) and ok(bias))


class _BatchNormAct(Function):
    @staticmethod
    def forward(ctx, x, gamma, beta, eps, relu, stats_out):
        x = x.contiguous()
        rows, cols = x.shape
        y = torch.empty_like(x)
        stats = torch.empty((3, cols), dtype=torch.float32, device=x.device)  # mean, biased variance, rstd
        ws_bytes = _L.tango_batchnorm_workspace(rows, cols)
        ws = _workspace(ws_bytes, x.device)
        check(_L.tango_batchnorm_fwd_f32(_ptr(y), _ptr(stats[0]), _ptr(stats[1]), _ptr(stats[2]), None, _ptr(x),
                                         _ptr(gamma), _ptr(beta), rows, cols, float(eps), int(relu), _ptr(ws), ws_bytes,
                                         _stream()), "batch_norm")
        stats_out.append(stats)
        ctx.relu = relu
        ctx.save_for_backward(x, gamma, beta, stats)
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, dy):
        refuse_capture("batch_norm.backward")
        x, gamma, beta, stats = ctx.saved_tensors
        dy = dy.contiguous()
        rows, cols = x.shape
        dx = torch.empty_like(x)
        dgb = torch.empty((2, cols), dtype=torch.float32, device=x.device)
        ws_bytes = _L.tango_batchnorm_workspace(rows, cols)
        ws = _workspace(ws_bytes, x.device)
        check(_L.tango_batchnorm_bwd_f32(_ptr(dx), _ptr(dgb[0]), _ptr(dgb[1]), _ptr(dy), _ptr(x), _ptr(stats[0]),
                                         _ptr(stats[2]), _ptr(gamma), _ptr(beta), rows, cols, int(ctx.relu), _ptr(ws),
                                         ws_bytes, _stream()), "batch_norm.backward")
        return dx, dgb[0], dgb[1], None, None, None


class BatchNorm1dAct(nn.BatchNorm1d):
    """``activation(BatchNorm1d(x))`` with ``activation`` None or ReLU (``torch.relu`` / ``F.relu``); any other
    activation is applied after torch's batch normalisation."""

    def __init__(self, num_features, activation=None, **kw):
        super().__init__(num_features, **kw)
        self.activation = activation

    def forward(self, x):
        relu = self.activation in (torch.relu, F.relu) or isinstance(self.activation, nn.ReLU)
        if not (self.training and self.affine and (relu or self.activation is None)
                and _fusable(x, self.num_features, self.weight, self.bias)):
            y = super().forward(x)
            return y if self.activation is None else self.activation(y)
        stats_out = []
        y = _BatchNormAct.apply(x, self.weight, self.bias, self.eps, relu, stats_out)
        if self.track_running_stats:
            # torch.nn.BatchNorm1d: the running variance takes the unbiased batch variance; momentum None =
            # cumulative average over the batches seen
            with torch.no_grad():
                self.num_batches_tracked += 1
                mom = 1.0 / float(self.num_batches_tracked) if self.momentum is None else self.momentum
                n = x.size(0)
                stats = stats_out[0]
                self.running_mean.lerp_(stats[0], mom)
                self.running_var.lerp_(stats[1] * (n / (n - 1)), mom)
        return y
