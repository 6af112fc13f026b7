"""Quantized GAT and HGT layers: the layer math of evaluation/test_gat.py:24-169
and evaluation/test_HGT.py:21-67, restated on the DGL-free graph object with the
edge softmax (DGL's in the reference) served by this package's kernel."""
import math

import torch
import torch.nn as nn

from .QLinear import QLinear
from .SDDMM import sddmm_u_add_v, sddmm_u_dot_v
from .SPMM import spmm_u_mul_e
from .edge_softmax import edge_softmax


class QGATConv(nn.Module):
    """evaluation/test_gat.py:24-169 for a homogeneous graph (feat is one tensor)."""

    def __init__(self, in_feats, out_feats, num_heads, negative_slope=0.2, residual=False,
                 activation=None, bias=True):
        super().__init__()
        self._num_heads, self._out_feats = num_heads, out_feats
        self.fc = QLinear(in_feats, out_feats * num_heads, bias=False)
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
        feat_src = self.fc(h).view(n, self._num_heads, self._out_feats)
        el = (feat_src * self.attn_l).sum(dim=-1).unsqueeze(-1)
        er = (feat_src * self.attn_r).sum(dim=-1).unsqueeze(-1)
        e = sddmm_u_add_v.apply(graph, el, er)                      # test_gat.py:141
        a = edge_softmax(graph, e, negative_slope=self.negative_slope)  # LeakyReLU :144 + softmax :146
        rst = spmm_u_mul_e.apply(graph, feat_src, a)                # :151
        if self.res_fc is not None:
            rst = rst + self.res_fc(h).view(n, -1, self._out_feats)
        if self.bias is not None:
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

    def forward(self, g, h):
        k = self.attn_linear(self.k_linear(h)).view(-1, self.n_heads, self.d_k)
        v = self.msg_linear(self.v_linear(h)).view(-1, self.n_heads, self.d_k)
        q = self.q_linear(h).view(-1, self.n_heads, self.d_k)
        t = sddmm_u_dot_v.apply(g, k, q) / self.sqrt_dk
        attn = edge_softmax(g, t)
        t = spmm_u_mul_e.apply(g, v, attn).reshape(-1, self.out_dim)
        return self.a_linear(t)
