"""Quantized per-edge ops: mirrors cuda/SDDMM.py of the reference, plus the
``sddmm_u_dot_v`` op that the reference's drivers call but its tree does not
define (evaluation/test_HGT.py:58, evaluation/link_pred_gcn.py:145)."""
import torch
from torch.autograd.function import Function, once_differentiable

from . import config
from .kernels import (cuda_kernels, incidence_SPMM, multi_cusparse_SPMM, mySDDMM_int8, mySDDMM_quantize_on_load,
                      quantize, quantize_heads, refuse_capture, unpad_heads)


def _quantize_grad(t):
    from .SPMM import grad_scale
    t = t if t.is_contiguous() else t.contiguous()
    if config.grad_round_mode == "stochastic":
        return quantize(t, grad_scale(t), round_mode="stochastic", **config.stochastic_args(t.device))
    return quantize(t, grad_scale(t), round_mode=config.grad_round_mode)


class sddmm_u_add_v(Function):
    """out[e] = U[src[e]] + V[dst[e]] on int8-quantized U, V (cuda/SDDMM.py:10-32).  Nothing else reads the
    int8 copies of U and V (the backward pass needs only the graph), so they are never stored: the kernel
    rounds the fp32 values with the two scales as it gathers them, which gives the same result bit for bit."""

    @staticmethod
    def forward(ctx, g, U, V, scaleU_=None, scaleV_=None):
        U = U if U.is_contiguous() else U.contiguous()
        scaleU = cuda_kernels.get_scale(U) if scaleU_ is None else scaleU_
        if id(U) == id(V):
            V, scaleV = U, scaleU
        else:
            V = V if V.is_contiguous() else V.contiguous()
            scaleV = cuda_kernels.get_scale(V) if scaleV_ is None else scaleV_
        out = mySDDMM_quantize_on_load(g, "add", U, V, scaleU, scaleV)
        ctx.backward_cache = g
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, dZ):
        refuse_capture("sddmm_u_add_v.backward")
        g = ctx.backward_cache
        dZ_, scaledZ = _quantize_grad(dZ)
        dU = dV = None
        if ctx.needs_input_grad[2]:
            dV = incidence_SPMM(g, dZ_, scaledZ)
        if ctx.needs_input_grad[1]:
            dU = incidence_SPMM(g, dZ_, scaledZ, True)
        return None, dU, dV, None, None


class sddmm_u_dot_v(Function):
    """out[e, h, 0] = <U[src[e], h, :], V[dst[e], h, :]>.  Built by symmetry with
    spmm_u_mul_e: the backward is two u_mul_e aggregations with dZ as the edge value.
    ``scaleU_`` / ``scaleV_`` may come from the producers of U and V (as in sddmm_u_add_v).
    ``out_scale`` (a Python float) multiplies the result, e.g. the 1 / sqrt(d_k) of an attention
    score (evaluation/test_HGT.py:58): it is folded into the dequantization scales of the forward
    and of both backward aggregations, so no pass over the [E, H] tensor runs for it (bit-identical
    to multiplying afterwards when it is a power of two, else within an ulp or two).
    ``Vq``: (int8 V, scale) as ``kernels.quantize_heads(V, scaleV_)`` returns them, when several calls share one V
    (the queries of a node type that several relations end at): V is then quantized once, by the caller."""

    @staticmethod
    def forward(ctx, g, U, V, scaleU_=None, scaleV_=None, out_scale=None, Vq=None):
        # heads whose width would leave the int8 rows unaligned are zero-padded (kernels.pad_heads): same dot products
        U_, scaleU = quantize_heads(U if U.is_contiguous() else U.contiguous(), scaleU_)
        if Vq is not None:
            V_, scaleV = Vq
            if V_.dtype != torch.int8 or V_.shape[:-1] != V.shape[:-1] or V_.size(-1) < V.size(-1):
                raise RuntimeError("sddmm_u_dot_v: Vq must be the int8 copy of V")
        else:
            V_, scaleV = quantize_heads(V if V.is_contiguous() else V.contiguous(), scaleV_)
        ctx.width = U.size(-1)
        if out_scale is not None:
            # 1-element products: the forward dequantizes with sU * (sV c), the backward passes with
            # s_dZ * (sV c) and s_dZ * (sU c)
            scaleU_c, scaleV_c = scaleU * out_scale, scaleV * out_scale
        else:
            scaleU_c, scaleV_c = scaleU, scaleV
        out, _ = mySDDMM_int8(g, "dot", U_, V_, scaleU, scaleV_c, False)
        ctx.backward_cache = g, U_, scaleU_c, V_, scaleV_c
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, dZ):
        refuse_capture("sddmm_u_dot_v.backward")
        g, U_, scaleU, V_, scaleV = ctx.backward_cache
        dZ = dZ if dZ.is_contiguous() else dZ.contiguous()
        squeeze = dZ.dim() == 2
        dZ3 = dZ.unsqueeze(1) if squeeze else dZ  # [E, H, 1]
        U3 = U_.unsqueeze(1) if U_.dim() == 2 else U_
        V3 = V_.unsqueeze(1) if V_.dim() == 2 else V_
        dZ_, scaledZ = _quantize_grad(dZ3)  # [E, H, 1], edge-major edge values
        dU = dV = None
        if ctx.needs_input_grad[1]:
            dU = unpad_heads(multi_cusparse_SPMM(g, V3, dZ_, scaledZ, True, edge_major=True, scale2=scaleV).reshape(U_.shape),
                             ctx.width)
        if ctx.needs_input_grad[2]:
            dV = unpad_heads(multi_cusparse_SPMM(g, U3, dZ_, scaledZ, edge_major=True, scale2=scaleU).reshape(V_.shape),
                             ctx.width)
        return None, dU, dV, None, None, None, None
