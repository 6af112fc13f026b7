"""Softmax cross-entropy (mean reduction) computed with its gradient in one pass over the logits.
Same result as ``torch.nn.functional.cross_entropy(logits, labels)``, which the reference's drivers
call (evaluation/test_gcn.py:256)."""
import torch
from torch.autograd.function import Function, once_differentiable

from .kernels import _L, _ptr, _stream, _workspace, check, refuse_capture


class _SoftmaxXent(Function):
    @staticmethod
    def forward(ctx, logits, labels):
        if logits.dim() != 2 or logits.dtype != torch.float32 or not logits.is_cuda:
            raise RuntimeError("cross_entropy: logits must be a 2-D fp32 GPU tensor")
        if labels.dtype != torch.int64 or labels.numel() != logits.size(0):
            raise RuntimeError("cross_entropy: labels must be int64 with one entry per row")
        logits = logits if logits.stride(1) == 1 else logits.contiguous()
        labels = labels.contiguous()
        rows, classes = logits.shape
        loss = torch.empty(1, dtype=torch.float32, device=logits.device)
        grad = torch.empty((rows, classes), dtype=torch.float32, device=logits.device)
        ws_bytes = _L.tango_softmax_xent_workspace(rows)
        ws = _workspace(ws_bytes, logits.device)
        check(_L.tango_softmax_xent_f32(_ptr(logits), logits.stride(0), _ptr(labels), rows, classes,
                                        loss.data_ptr(), _ptr(grad), classes, _ptr(ws), ws_bytes, _stream()),
              "cross_entropy")
        ctx.backward_cache = grad
        return loss.reshape(())

    @staticmethod
    @once_differentiable
    def backward(ctx, gout):
        refuse_capture("cross_entropy.backward")
        return ctx.backward_cache * gout, None


def cross_entropy(logits, labels):
    """Mean softmax cross-entropy over rows; falls back to torch for more than 256 classes."""
    if logits.size(1) > 256:
        return torch.nn.functional.cross_entropy(logits, labels)
    return _SoftmaxXent.apply(logits, labels)
