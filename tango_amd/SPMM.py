"""Quantized aggregation ops: mirrors cuda/SPMM.py of the reference."""
import torch
from torch.autograd.function import Function, once_differentiable

from . import config
from .kernels import (cuda_kernels, csr_SPMM, multi_cusparse_SPMM, mySDDMM_int8, pad_heads, quantize, quantize_heads,
                      quantize_padded, refuse_capture, unpad_heads)


def _gather_align(width):
    """Row pitch for int8 rows that will be gathered: rows narrower than a 128-byte cache line are
    padded to a power of two so that no row straddles two lines; wider rows to whole lines."""
    for a in (16, 32, 64, 128):
        if width <= a:
            return a
    return 128


def _dense_enough(g, reverse=False):
    """Whether the aggregation of this orientation runs the row kernels, whose epilogue can return the scale of
    its output (graphs averaging fewer than 64 slots per row take the slot-span kernels, which cannot)."""
    if not config.scale_from_aggregation:
        return False
    indptr, indices = (g.adj_csr if reverse else g.adj_csc)[:2]
    return indices.numel() >= 64 * (indptr.numel() - 1)


def grad_scale_hint(t):
    """max|t| / 127 if the kernel that produced the gradient ``t`` left it on the tensor and nothing has written
    to ``t`` since (autograd may add another gradient into it in place), else None."""
    hint = getattr(t, "_tango_scale", None)
    if hint is not None and hint[1] == t._version and hint[2] == t.data_ptr():
        return hint[0]
    return None


def grad_scale(t):
    """max|t| / 127 of the contiguous gradient ``t``: the value its producer left on it, else one absmax pass whose
    result stays on the tensor, so that a gradient autograd hands to several nodes (the sum of the per-relation
    aggregates of a heterogeneous layer) is scanned by the first of them only."""
    s = grad_scale_hint(t)
    if s is None:
        s = cuda_kernels.get_scale(t)
        t._tango_scale = (s, t._version, t.data_ptr())
    return s


def masked_scale_hint(t, bits, row_mul):
    """max|t' * row_mul| / 127 (t' = t where its sign bit in ``bits`` is set) if the GEMM that produced the gradient
    ``t`` found it in its epilogue for exactly this mask and multiplier and nothing has written to ``t`` since."""
    hint = getattr(t, "_tango_masked_scale", None)
    if hint is None or hint[3] != t._version or hint[4] != t.data_ptr() or hint[1] is not bits:
        return None
    if (hint[2] is None) != (row_mul is None) or (row_mul is not None and hint[2].data_ptr() != row_mul.data_ptr()):
        return None
    return hint[0]


def relu_mask_of(t):
    """(sign words, row multiplier) of the fused ReLU epilogue that produced the activation ``t``, if ``t`` is still
    that tensor: what the backward pass of ``t``'s producer will apply to the gradient of ``t``."""
    tag = getattr(t, "_tango_relu", None)
    if tag is not None and tag[2] == t._version and tag[3] == t.data_ptr():
        return tag[0], tag[1]
    return None


def _quantize_grad(t, padded):
    t = t if t.is_contiguous() else t.contiguous()
    kw = {"round_mode": config.grad_round_mode}
    if config.grad_round_mode == "stochastic":
        kw.update(config.stochastic_args(t.device))
    if padded and t.dim() == 2:
        return quantize_padded(t, grad_scale(t), align=_gather_align(t.size(1)), **kw)
    return quantize(t, grad_scale(t), **kw)


class spmm_copy_u(Function):
    """copy_u-sum aggregation (cuda/SPMM.py:8-24).  ``scaleN`` may come from the
    preceding GEMM's epilogue, in which case no absmax pass runs here.

    ``row_scale`` [n], ``bias`` [F] and ``relu`` fold the glue that follows the
    aggregation in a GCN layer (evaluation/test_gcn.py:123-137: ``* in_deg^-1/2``,
    ``+ bias``, activation) into the kernel's epilogue; the backward then masks,
    sums the bias gradient, scales rows and quantizes in two reads of dOut.
    ``src_row_mul`` [n] folds the ``feat * out_deg^-1/2`` in front of the aggregation (evaluation/test_gcn.py:86-94)
    into the pass that quantizes N, and its backward into the epilogue of the reverse aggregation; same roundings
    as the separate multiplications."""

    @staticmethod
    def forward(ctx, g, N, scaleN=None, row_scale=None, bias=None, relu=False, src_row_mul=None, want_scale=False,
                scale_mul=None):
        """``want_scale``: returns (out, max|out * scale_mul[:, None]| / 127) (``scale_mul`` optional): the scale the
        next op's quantizer needs, from the aggregation's epilogue where the graph is dense enough for the row
        kernels, else from a pass over out."""
        N = N if N.is_contiguous() else N.contiguous()
        fused = row_scale is not None or bias is not None or relu or src_row_mul is not None
        if fused and N.dim() != 2:
            raise RuntimeError("spmm_copy_u: the fused prologue / epilogue needs 2-D features")
        if src_row_mul is not None and scaleN is not None:
            raise RuntimeError("spmm_copy_u: a precomputed scale cannot be combined with src_row_mul")
        ctx.src_row_mul = src_row_mul
        if N.dim() == 2:
            N_, scaleN = quantize_padded(N, scaleN, align=_gather_align(N.size(1)), row_mul=src_row_mul)
        else:
            N_, scaleN = quantize(N, scaleN)
        # the backward pass needs only the sign of the ReLU's output: sixteen columns per 16-bit word, written
        # by the epilogue, instead of two more reads of the fp32 output
        bits = None
        if relu and N.dim() == 2 and N.size(1) % 16 == 0:
            bits = torch.empty((g.num_nodes(), N.size(1) // 16), dtype=torch.int16, device=N.device)
        scale_out = None
        if want_scale and N.dim() == 2 and _dense_enough(g):
            out, scale_out = csr_SPMM(g, N_, scaleN, row_scale=row_scale, bias=bias, relu=relu, sign_bits=bits,
                                      want_scale=True, scale_mul=scale_mul)
        else:
            out = csr_SPMM(g, N_, scaleN, row_scale=row_scale, bias=bias, relu=relu, sign_bits=bits)
            if want_scale:
                scale_out, _ = cuda_kernels.absmax_ex(out.reshape(out.size(0), -1), row_mul=scale_mul)
        # the op's own output goes through save_for_backward (autograd then holds it without the
        # output -> grad_fn -> ctx -> output cycle a plain attribute would form); everything else is an input
        # or an auxiliary tensor, kept as the reference keeps its cache (cuda/SPMM.py:13)
        ctx.backward_cache = g, row_scale, bias is not None, bits, relu
        if relu and bits is None:
            ctx.save_for_backward(out)
        if bits is not None:
            # for a quantized linear layer that consumes out: its backward can then find the scale of the masked,
            # row-scaled gradient in the epilogue that writes the gradient (relu_mask_of)
            out._tango_relu = (bits, row_scale, out._version, out.data_ptr())
        if want_scale:
            ctx.mark_non_differentiable(scale_out)
            ctx.set_materialize_grads(False)
            return out, scale_out
        return out

    @staticmethod
    def _reverse(ctx, g, dZ_, scaledZ):
        """The reverse aggregation; on dense graphs its epilogue also finds max|dN| / 127, left on the result for
        the op that quantizes this gradient next (``grad_scale_hint``)."""
        if dZ_.dim() == 2 and _dense_enough(g, True):
            dN, s = csr_SPMM(g, dZ_, scaledZ, True, row_scale=ctx.src_row_mul, want_scale=True)
            dN._tango_scale = (s, dN._version, dN.data_ptr())
            return dN
        return csr_SPMM(g, dZ_, scaledZ, True, row_scale=ctx.src_row_mul)

    @staticmethod
    @once_differentiable
    def backward(ctx, dOut, dscale=None):
        refuse_capture("spmm_copy_u.backward")
        if dOut is None:
            return (None,) * 9
        g, row_scale, has_bias, mask, relu = ctx.backward_cache
        if relu and mask is None:
            mask, = ctx.saved_tensors
        dN = dbias = None
        if row_scale is None and not has_bias and mask is None:
            if ctx.needs_input_grad[1]:
                dZ_, scaledZ = _quantize_grad(dOut, True)
                dN = spmm_copy_u._reverse(ctx, g, dZ_, scaledZ)
            return None, dN, None, None, None, None, None, None, None
        dOut = dOut if dOut.is_contiguous() else dOut.contiguous()
        want_bias = has_bias and ctx.needs_input_grad[4]
        # dZ = (dOut where out > 0) * row_scale; its scale and the bias gradient come from one pass
        mode = "bits" if mask is not None and mask.dtype == torch.int16 else "relu"
        kw = {"round_mode": config.grad_round_mode}
        # the GEMM that wrote dOut may already have found the scale (of exactly this mask and multiplier)
        scaledZ = masked_scale_hint(dOut, mask, row_scale) if mode == "bits" and ctx.needs_input_grad[1] else None
        if scaledZ is not None:
            if config.grad_round_mode == "stochastic":
                kw.update(config.stochastic_args(dOut.device))
            cols = dOut.size(1)
            dZ_ = None
            if want_bias and _gather_align(cols) <= cols and cols % _gather_align(cols) == 0:
                # the bias gradient out of the pass that quantizes: no pass over dOut is left that only reduces
                dZ_ = torch.empty(dOut.shape, dtype=torch.int8, device=dOut.device)
                dbias = cuda_kernels.quantize_rows_colsum(dZ_, dOut, scaledZ, row_mul=row_scale, mask=mask,
                                                          mask_mode=mode, **kw)
                if dbias is None:
                    dZ_ = None
            if dZ_ is None:
                if want_bias:
                    _, dbias = cuda_kernels.absmax_ex(dOut, row_mul=row_scale, mask=mask, want_colsum=True, mask_mode=mode)
                dZ_, _ = quantize_padded(dOut, scaledZ, row_mul=row_scale, mask=mask, mask_mode=mode,
                                         align=_gather_align(cols), **kw)
            dN = spmm_copy_u._reverse(ctx, g, dZ_, scaledZ)
            return None, dN, None, None, dbias, None, None, None, None
        scaledZ, dbias = cuda_kernels.absmax_ex(dOut, row_mul=row_scale, mask=mask, want_colsum=want_bias, mask_mode=mode)
        if ctx.needs_input_grad[1]:
            if config.grad_round_mode == "stochastic":
                kw.update(config.stochastic_args(dOut.device))
            dZ_, _ = quantize_padded(dOut, scaledZ, row_mul=row_scale, mask=mask, mask_mode=mode,
                                     align=_gather_align(dOut.size(1)), **kw)
            dN = spmm_copy_u._reverse(ctx, g, dZ_, scaledZ)
        return None, dN, None, None, dbias, None, None, None, None


def _need_reduce_last_dim(ufeat, efeat):
    """cuda/SPMM.py:26-34: whether dE reduces the last dimension (dot instead of mul)."""
    if ufeat is None or efeat is None:
        return False
    ushp = ufeat.shape
    eshp = efeat.shape
    return ushp[1:-1] == eshp[1:-1] and eshp[-1] == 1 and ushp[-1] > 1


class spmm_u_mul_e(Function):
    """u_mul_e-sum aggregation with int8 node features and int8 edge values
    (cuda/SPMM.py:36-62).  N is [n, H, F], E is [nnz, H, 1] in edge-id order.

    ``bias`` ([H * F]) folds the "rst + bias" that follows the aggregation in a GAT layer
    (evaluation/test_gat.py:160-162) into the kernel's epilogue; its gradient then comes
    out of the pass that finds the scale of dZ.  ``scaleN`` may come from the producer of N.
    ``act`` ("relu" or "elu") folds the layer's activation (evaluation/test_gat.py:164-165) in as
    well: the epilogue applies it, and the backward pass takes dZ back through it inside the two
    kernels that read dZ anyway (scale / bias gradient, quantize) instead of a separate pass."""

    @staticmethod
    def forward(ctx, g, N, E, bias=None, scaleN=None, act=None, scaleE=None):
        """``scaleE``: max|E| / 127 when the producer of E knows it (the edge softmax's kernel does): E is then
        neither scanned nor stored in int8, the aggregation rounds the fp32 values as it loads them, here and
        in the backward pass (same int8 values, so the same results)."""
        N = N if N.is_contiguous() else N.contiguous()
        E = E if E.is_contiguous() else E.contiguous()
        # Edge values stay edge-major ([nnz, H, 1], plain quantize): the reference transposes them to
        # [H, 1, nnz] (cuda/SPMM.py:41) and then permutes that with index_select; with the permutation
        # fused into the gather, edge-major keeps the H bytes of an edge in one cache sector.
        if scaleE is not None and config.edge_values_on_load:
            E_T_ = E  # fp32, quantized on load
        elif scaleE is not None:
            E_T_, _ = quantize(E, scaleE)  # no pass that looks for the scale
        else:
            E_T_, scaleE = quantize(E)
        # one absmax pass (the reference runs two, cuda/SPMM.py:39,43).  Broadcast edge values: heads whose width would
        # leave the int8 rows unaligned are zero-padded (kernels.pad_heads), the bias with them; the padding columns of
        # the result are dropped again
        padded = N.dim() == 3 and E.size(-1) == 1 and pad_heads(N.size(2), N.size(1)) != N.size(2)
        N_, scaleN = quantize_heads(N, scaleN) if padded else quantize(N, scaleN)
        kbias = bias
        if padded and bias is not None:
            H, D = N.size(1), N.size(2)
            kbias = torch.nn.functional.pad(bias.detach().view(H, D), (0, N_.size(2) - D)).reshape(-1)
        # dequantized with scaleN * scaleE (cuda/SPMM.py:44); the kernel multiplies the two itself
        out = multi_cusparse_SPMM(g, N_, E_T_, scaleN, edge_major=True, bias=kbias, scale2=scaleE, act=act)
        out = unpad_heads(out, N.size(-1))
        reduce_last = _need_reduce_last_dim(N, E)
        ctx.padded = padded
        ctx.backward_cache = g, N_, scaleN, E_T_, scaleE, reduce_last, E.shape, bias is not None, act
        if act is not None:
            ctx.save_for_backward(out)  # not an attribute: that would tie the output to its own grad_fn
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, dZ):
        refuse_capture("spmm_u_mul_e.backward")
        g, N_, scaleN, E_T_, scaleE, reduce_last, eshape, has_bias, act = ctx.backward_cache
        dbias = None
        if act is not None:
            out, = ctx.saved_tensors
            # dZ goes back through the activation on its way into the scale, the bias gradient and int8
            dZ = dZ if dZ.is_contiguous() else dZ.contiguous()
            dZ2, out2 = dZ.view(dZ.size(0), -1), out.view(out.size(0), -1)
            scaledZ, dbias = cuda_kernels.absmax_ex(dZ2, mask=out2, mask_mode=act,
                                                    want_colsum=has_bias and ctx.needs_input_grad[3])
            kw = {"round_mode": config.grad_round_mode}
            if config.grad_round_mode == "stochastic":
                kw.update(config.stochastic_args(dZ.device))
            if ctx.padded:
                dZ_, _ = quantize_heads(dZ, scaledZ, mask=out2, mask_mode=act, **kw)
            else:
                dZ_, _ = quantize_padded(dZ2, scaledZ, mask=out2, mask_mode=act, align=1, **kw)
                dZ_ = dZ_.view(dZ.shape)
        elif has_bias and ctx.needs_input_grad[3]:
            # the scale of dZ and the bias gradient (column sums) in one read
            dZ = dZ if dZ.is_contiguous() else dZ.contiguous()
            scaledZ, dbias = cuda_kernels.absmax_ex(dZ.view(dZ.size(0), -1), want_colsum=True)
            kw = {"round_mode": config.grad_round_mode}
            if config.grad_round_mode == "stochastic":
                kw.update(config.stochastic_args(dZ.device))
            dZ_, _ = quantize_heads(dZ, scaledZ, **kw) if ctx.padded else quantize(dZ, scaledZ, **kw)
        elif ctx.padded:
            dZ = dZ if dZ.is_contiguous() else dZ.contiguous()
            kw = {"round_mode": config.grad_round_mode}
            if config.grad_round_mode == "stochastic":
                kw.update(config.stochastic_args(dZ.device))
            dZ_, scaledZ = quantize_heads(dZ, **kw)
        else:
            dZ_, scaledZ = _quantize_grad(dZ, False)
        dN = dE = None
        if ctx.needs_input_grad[1]:
            # dN = A^T (E * dZ): the dequantization scale is s_dZ * s_E.  The reference passes
            # the forward scale s_N * s_E here (cuda/SPMM.py:56); ref_compat reproduces that.
            first = scaleN if config.ref_compat else scaledZ
            dN = unpad_heads(multi_cusparse_SPMM(g, dZ_, E_T_, first, True, edge_major=True, scale2=scaleE), dZ.size(-1))
        if ctx.needs_input_grad[2]:
            op = "dot" if reduce_last else "mul"
            dE, _ = mySDDMM_int8(g, op, N_, dZ_, scaleN, scaledZ, False)
            dE = dE.reshape(eshape)
        return None, dN, dE, dbias, None, None, None
