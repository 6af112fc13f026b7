"""Edge softmax over the in-edges of each destination node, optionally with the
LeakyReLU that precedes it in GAT fused in (evaluation/test_gat.py:144-146;
the reference calls DGL's fp32 edge_softmax, which is not part of its tree)."""
from torch.autograd.function import Function, once_differentiable

from .kernels import cuda_kernels, refuse_capture


def _dst_major(g):
    """(indptr, slot -> edge id or None when the slots are in edge-id order) of the destination-major CSR."""
    indptr, _, eids = g.adj_csc
    return indptr, (None if getattr(g, "csc_slots_are_edge_ids", False) else eids)


class _EdgeSoftmax(Function):
    @staticmethod
    def forward(ctx, g, e, slope):
        e = e if e.is_contiguous() else e.contiguous()
        indptr, eids = _dst_major(g)
        a = cuda_kernels.edge_softmax_forward(e, indptr, eids, slope)
        ctx.backward_cache = g, slope
        ctx.save_for_backward(e, a)  # a is this op's output: saved, not an attribute (no reference cycle)
        return a

    @staticmethod
    @once_differentiable
    def backward(ctx, da):
        refuse_capture("edge_softmax.backward")
        g, slope = ctx.backward_cache
        e, a = ctx.saved_tensors
        indptr, eids = _dst_major(g)
        da = da if da.is_contiguous() else da.contiguous()
        return None, cuda_kernels.edge_softmax_backward(a, da, e, indptr, eids, slope), None


def edge_softmax(g, e, negative_slope=None):
    """softmax_dst(e) if ``negative_slope`` is None, else softmax_dst(leaky_relu(e))."""
    return _EdgeSoftmax.apply(g, e, 1.0 if negative_slope is None else float(negative_slope))
