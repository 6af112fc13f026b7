"""Edge softmax over the in-edges of each destination node, optionally with the
LeakyReLU that precedes it in GAT fused in (evaluation/test_gat.py:144-146;
the reference calls DGL's fp32 edge_softmax, which is not part of its tree)."""
import torch
from torch.autograd.function import Function, once_differentiable

from .kernels import cuda_kernels, refuse_capture


def _dst_major(g):
    """(indptr, slot -> edge id or None when the slots are in edge-id order) of the destination-major CSR."""
    indptr, _, eids = g.adj_csc
    return indptr, (None if getattr(g, "csc_slots_are_edge_ids", False) else eids)


class _EdgeSoftmax(Function):
    @staticmethod
    def forward(ctx, g, e, slope, want_scale=False):
        e = e if e.is_contiguous() else e.contiguous()
        indptr, eids = _dst_major(g)
        ctx.backward_cache = g, slope
        ctx.set_materialize_grads(False)
        if want_scale:
            # the kernel that writes a also finds max(a) / 127, the scale the aggregation quantizes a with
            a, s_a, _ = cuda_kernels.edge_softmax_forward_ex(e, indptr, eids, slope)
            ctx.save_for_backward(e, a)
            ctx.mark_non_differentiable(s_a)
            return a, s_a
        a = cuda_kernels.edge_softmax_forward(e, indptr, eids, slope)
        ctx.save_for_backward(e, a)  # a is this op's output: saved, not an attribute (no reference cycle)
        return a

    @staticmethod
    @once_differentiable
    def backward(ctx, da, _ds=None):
        refuse_capture("edge_softmax.backward")
        if da is None:
            return None, None, None, None
        g, slope = ctx.backward_cache
        e, a = ctx.saved_tensors
        indptr, eids = _dst_major(g)
        da = da if da.is_contiguous() else da.contiguous()
        # the plain softmax (slope 1) does not need e: one [E, H] read less
        return None, cuda_kernels.edge_softmax_backward(a, da, None if slope == 1.0 else e, indptr, eids, slope), None, None


def edge_softmax(g, e, negative_slope=None, want_scale=False, eids=None):
    """softmax_dst(e) if ``negative_slope`` is None, else softmax_dst(leaky_relu(e)).  ``want_scale``: returns
    (a, max(a) / 127), the second found by the kernel that writes a (hand it to spmm_u_mul_e as ``scaleE``).
    ``eids`` (int64 [k], distinct): the softmax runs over these edges only, as DGL's ``edge_softmax(graph, e, eids=eids)``
    does (evaluation/arxiv_gat.py:186-192, edge dropping); ``e`` then holds the logits of those k edges and so does
    the result.  The other edges take part with a logit of -FLT_MAX, whose exponential is an exact zero, so a
    destination's kept edges get the sums of the kept edges alone."""
    slope = 1.0 if negative_slope is None else float(negative_slope)
    if eids is None:
        return _EdgeSoftmax.apply(g, e, slope, want_scale)
    if want_scale:
        raise RuntimeError("edge_softmax: want_scale is not available with eids")
    if e.size(0) != eids.numel():
        raise RuntimeError("edge_softmax: e must hold one row per entry of eids")
    full = e.new_full((g.num_edges(),) + tuple(e.shape[1:]), -torch.finfo(e.dtype).max)
    full = full.index_copy(0, eids, e)
    return _EdgeSoftmax.apply(g, full, slope, False).index_select(0, eids)


class gat_edge_attention(Function):
    """The attention coefficients of a GAT layer from its per-node logits in one op,
    a = softmax_dst(leaky_relu(q(el)[src] + q(er)[dst])) (evaluation/test_gat.py:141-146: sddmm_u_add_v, LeakyReLU,
    DGL's edge_softmax).  The softmax kernel also returns max(a) / 127 for the aggregation's quantizer (and, with
    config.attention_logits_on_the_fly, forms the sums as it loads instead of reading them, keeping one sign bit per
    (edge, head) for the backward pass).  Backward:
    the softmax's backward kernel also finds the scale of its result, which is then quantized once and summed per
    source and per destination (what sddmm_u_add_v.backward does, cuda/SDDMM.py:22-32).  Same values as the three
    separate ops, bit for bit.  Returns (a [E, H, 1], scale of a)."""

    @staticmethod
    def forward(ctx, g, el, er, s_el, s_er, slope):
        el = el if el.is_contiguous() else el.contiguous()
        er = er if er.is_contiguous() else er.contiguous()
        s_el = cuda_kernels.get_scale(el) if s_el is None else s_el
        s_er = cuda_kernels.get_scale(er) if s_er is None else s_er
        indptr, eids = _dst_major(g)
        src, dst = g.coo
        from . import config
        from .kernels import mySDDMM_quantize_on_load
        if config.attention_logits_on_the_fly:
            e = None
            a, s_a, sign = cuda_kernels.edge_softmax_forward_ex(None, indptr, eids, slope,
                                                                logits=(el, er, s_el, s_er, src, dst), want_sign=True)
        else:
            e = mySDDMM_quantize_on_load(g, "add", el, er, s_el, s_er)
            a, s_a, sign = cuda_kernels.edge_softmax_forward_ex(e, indptr, eids, slope)
        ctx.backward_cache = g, slope, sign, e
        ctx.save_for_backward(a)
        ctx.mark_non_differentiable(s_a)
        ctx.set_materialize_grads(False)
        return a, s_a

    @staticmethod
    @once_differentiable
    def backward(ctx, da, _ds=None):
        from . import config
        from .kernels import incidence_SPMM, quantize
        refuse_capture("gat_edge_attention.backward")
        if da is None:
            return (None,) * 6
        g, slope, sign, e = ctx.backward_cache
        a, = ctx.saved_tensors
        indptr, eids = _dst_major(g)
        da = da if da.is_contiguous() else da.contiguous()
        de, s_de = cuda_kernels.edge_softmax_backward_ex(a, da, e, sign, indptr, eids, slope)
        kw = {"round_mode": config.grad_round_mode}
        if config.grad_round_mode == "stochastic":
            kw.update(config.stochastic_args(de.device))
        dZ_, _ = quantize(de, s_de, **kw)
        d_el = incidence_SPMM(g, dZ_, s_de, True) if ctx.needs_input_grad[1] else None
        d_er = incidence_SPMM(g, dZ_, s_de) if ctx.needs_input_grad[2] else None
        return None, d_el, d_er, None, None, None
