"""Quantized GAT and HGT layers: the layer math of evaluation/test_gat.py:24-169
and evaluation/test_HGT.py:21-67, restated on the DGL-free graph object with the
edge softmax (DGL's in the reference) served by this package's kernel."""
import math

import torch
import torch.nn as nn

from torch.autograd.function import Function, once_differentiable

from .QLinear import QLinear
from .kernels import cuda_kernels
from .SDDMM import sddmm_u_add_v, sddmm_u_dot_v
from .SPMM import spmm_u_mul_e
from .edge_softmax import edge_softmax


class attn_scores(Function):
    """el = (feat * attn_l).sum(-1), er = (feat * attn_r).sum(-1) for feat [n, H, D] and
    attn_l, attn_r [1, H, D] (evaluation/test_gat.py:135-137), forward and backward each in
    one pass over feat.  Returns el, er as [n, H, 1]."""

    @staticmethod
    def forward(ctx, feat, attn_l, attn_r):
        feat = feat if feat.is_contiguous() else feat.contiguous()
        al, ar = attn_l.contiguous(), attn_r.contiguous()
        el, er = cuda_kernels.attn_scores_forward(feat, al, ar)
        ctx.backward_cache = feat, al, ar, attn_l.shape
        return el.unsqueeze(-1), er.unsqueeze(-1)

    @staticmethod
    @once_differentiable
    def backward(ctx, del_, der):
        feat, al, ar, shape = ctx.backward_cache
        dfeat, dal, dar = cuda_kernels.attn_scores_backward(del_.contiguous(), der.contiguous(), feat, al, ar)
        return dfeat, dal.view(shape), dar.view(shape)


class QGATConv(nn.Module):
    """evaluation/test_gat.py:24-169 for a homogeneous graph (feat is one tensor)."""

    def __init__(self, in_feats, out_feats, num_heads, negative_slope=0.2, residual=False,
                 activation=None, bias=True):
        super().__init__()
        self._num_heads, self._out_feats = num_heads, out_feats
        self.fc = QLinear(in_feats, out_feats * num_heads, bias=False)
        self.fc.enable_reduce()  # the GEMM epilogue hands max|feat_src| / 127 to the aggregation
        self.attn_l = nn.Parameter(torch.empty(1, num_heads, out_feats))
        self.attn_r = nn.Parameter(torch.empty(1, num_heads, out_feats))
        self.negative_slope = negative_slope
        self.bias = nn.Parameter(torch.zeros(num_heads * out_feats)) if bias else None
        if residual:
            self.res_fc = (QLinear(in_feats, num_heads * out_feats, bias=False)
                           if in_feats != out_feats * num_heads else nn.Identity())
        else:
            self.res_fc = None
        self.activation = activation
        gain = nn.init.calculate_gain("relu")
        nn.init.xavier_normal_(self.fc.weight, gain=gain)
        nn.init.xavier_normal_(self.attn_l, gain=gain)
        nn.init.xavier_normal_(self.attn_r, gain=gain)
        if isinstance(self.res_fc, QLinear):
            nn.init.xavier_normal_(self.res_fc.weight, gain=gain)

    def forward(self, graph, feat, get_attention=False):
        n = feat.size(0)
        h = feat.contiguous()
        feat_src, s_feat = self.fc(h)
        feat_src = feat_src.view(n, self._num_heads, self._out_feats)
        el, er = attn_scores.apply(feat_src, self.attn_l, self.attn_r)  # test_gat.py:135-137
        e = sddmm_u_add_v.apply(graph, el, er)                      # :141
        a = edge_softmax(graph, e, negative_slope=self.negative_slope)  # LeakyReLU :144 + softmax :146
        # without a residual branch the bias add (:160-162) rides in the aggregation's epilogue
        fold_bias = self.bias is not None and self.res_fc is None
        rst = spmm_u_mul_e.apply(graph, feat_src, a, self.bias if fold_bias else None, s_feat)  # :151
        if self.res_fc is not None:
            rst = rst + self.res_fc(h).view(n, -1, self._out_feats)
        if self.bias is not None and not fold_bias:
            rst = rst + self.bias.view(1, self._num_heads, self._out_feats)
        if self.activation:
            rst = self.activation(rst)
        return (rst, a) if get_attention else rst


class HGTLayer(nn.Module):
    """evaluation/test_HGT.py:21-67 (the reference's HGT has no per-type weights)."""

    def __init__(self, in_dim, out_dim, n_heads):
        super().__init__()
        self.out_dim, self.n_heads, self.d_k = out_dim, n_heads, out_dim // n_heads
        self.sqrt_dk = math.sqrt(self.d_k)
        self.q_linear = QLinear(in_dim, out_dim)
        self.k_linear = QLinear(in_dim, out_dim)
        self.v_linear = QLinear(in_dim, out_dim)
        self.msg_linear = QLinear(out_dim, out_dim)
        self.attn_linear = QLinear(out_dim, out_dim)
        self.a_linear = QLinear(out_dim, out_dim)
        # every projection feeds another quantized op: their GEMM epilogues hand the output's
        # max|.| / 127 on, so none of the consumers runs an absmax pass of its own
        for lin in (self.q_linear, self.k_linear, self.v_linear, self.msg_linear, self.attn_linear):
            lin.enable_reduce()

    def forward(self, g, h):
        k, s_k = self.k_linear(h)
        k, s_k = self.attn_linear(k, s_k)
        v, s_v = self.v_linear(h)
        v, s_v = self.msg_linear(v, s_v)
        q, s_q = self.q_linear(h)
        k, v, q = (t.view(-1, self.n_heads, self.d_k) for t in (k, v, q))
        t = sddmm_u_dot_v.apply(g, k, q, s_k, s_q) / self.sqrt_dk
        attn = edge_softmax(g, t)
        t = spmm_u_mul_e.apply(g, v, attn, None, s_v).reshape(-1, self.out_dim)
        return self.a_linear(t)
