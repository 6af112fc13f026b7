"""Quantized GCN layers: the layer math of evaluation/test_gcn.py:26-169,
restated on the DGL-free graph object so that the benchmark's training epoch
exercises the primitives the way the reference's driver does."""
import torch
import torch.nn as nn

from .QLinear import Qlinear_func, Qlinear_func_reduce
from .batchnorm import BatchNorm1dAct
from .SPMM import spmm_copy_u


def degree_norms(graph):
    """(out_deg^-1/2, in_deg^-1/2) with degrees clamped to >= 1 (evaluation/test_gcn.py:86-94,123-131)."""
    return (graph.out_degrees().float().clamp(min=1).pow(-0.5),
            graph.in_degrees().float().clamp(min=1).pow(-0.5))


class QGraphConv(nn.Module):
    """GraphConv(norm='both') with int8 GEMM and int8 aggregation
    (evaluation/test_gcn.py:26-139)."""

    def __init__(self, in_feats, out_feats, bias=True, activation=None, fused=True):
        super().__init__()
        self.fused = fused
        self._in_feats, self._out_feats = in_feats, out_feats
        self.weight = nn.Parameter(torch.empty(out_feats, in_feats))
        self.bias = nn.Parameter(torch.empty(out_feats)) if bias else None
        self._activation = activation
        nn.init.xavier_uniform_(self.weight)
        if self.bias is not None:
            nn.init.zeros_(self.bias)

    def forward(self, graph, feat, norms=None, feat_scale=None, want_scale=False):
        """``norms``: (out_deg^-1/2, in_deg^-1/2) from ``degree_norms`` when the caller computes them once
        for several layers of one forward pass; the reference's layer computes them itself every time.
        ``want_scale`` (fused layers that multiply first): also returns max|out * out_deg^-1/2| / 127, which the
        next such layer takes as ``feat_scale`` instead of scanning its input."""
        norm_src, norm_dst = degree_norms(graph) if norms is None else norms
        relu = self._activation is torch.relu
        if self.fused:
            # same arithmetic as below, with every elementwise pass folded into a kernel:
            # "* norm_src" into the quantize of the GEMM / aggregation input, "* norm_dst, + bias,
            # relu" into the aggregation's epilogue (or "* norm_dst" into nothing when the GEMM is last)
            if self._in_feats > self._out_feats:
                y, sy = Qlinear_func_reduce.apply(feat, self.weight, None, norm_src, feat_scale)
                emit = want_scale and (self._activation is None or relu)
                rst = spmm_copy_u.apply(graph, y, sy, norm_dst, self.bias, relu, None, emit, norm_src if emit else None)
                rst, scale = rst if emit else (rst, None)
                if self._activation is not None and not relu:
                    rst = self._activation(rst)
                return (rst, scale) if want_scale else rst
            rst = spmm_copy_u.apply(graph, feat, None, None, None, False, norm_src)  # "feat * norm_src" in the quantize pass
            rst = Qlinear_func.apply(rst, self.weight) * norm_dst.unsqueeze(1)
        else:
            feat_src = feat * norm_src.unsqueeze(1)
            if self._in_feats > self._out_feats:
                # multiply by W first, hand the GEMM epilogue's scale to the aggregation
                feat_src, scale_feat = Qlinear_func_reduce.apply(feat_src, self.weight)
                rst = spmm_copy_u.apply(graph, feat_src, scale_feat)
            else:
                rst = spmm_copy_u.apply(graph, feat_src)
                rst = Qlinear_func.apply(rst, self.weight)
            rst = rst * norm_dst.unsqueeze(1)
        if self.bias is not None:
            rst = rst + self.bias
        if self._activation is not None:
            rst = self._activation(rst)
        return (rst, None) if want_scale else rst


class GCN(nn.Module):
    """evaluation/test_gcn.py:140-169 with n_layers hidden layers after the input layer."""

    def __init__(self, g, in_feats, n_hidden, n_classes, n_layers, activation, dropout, fused=True):
        super().__init__()
        self.g = g
        self.layers = nn.ModuleList()
        self.layers.append(QGraphConv(in_feats, n_hidden, activation=activation, fused=fused))
        for _ in range(n_layers - 1):
            self.layers.append(QGraphConv(n_hidden, n_hidden, activation=activation, fused=fused))
        self.layers.append(QGraphConv(n_hidden, n_classes, fused=fused))
        self.dropout = nn.Dropout(p=dropout)

    def forward(self, features):
        h = features
        norms = degree_norms(self.g)  # once per forward pass, shared by the layers
        scale = None
        last = len(self.layers) - 1
        for i, layer in enumerate(self.layers):
            if i != 0:
                h = self.dropout(h)
            # a layer's aggregation hands max|h * out_deg^-1/2| / 127 to the next layer's GEMM, unless dropout
            # changes h in between
            hand_on = i < last and (self.dropout.p == 0.0 or not self.training)
            if hand_on:
                h, scale = layer(self.g, h, norms, scale, True)
            else:
                h, scale = layer(self.g, h, norms, scale), None
        return h


class ArxivGCN(nn.Module):
    """evaluation/arxiv_gcn.py:156-209 (QGCN): graph convolutions without bias except the last, an optional
    quantized linear skip branch per layer, batch normalisation + activation + dropout between layers, and an
    input dropout of at most 0.1."""

    def __init__(self, in_feats, n_hidden, n_classes, n_layers, activation, dropout, use_linear):
        super().__init__()
        from .QLinear import QLinear
        self.n_layers, self.use_linear = n_layers, use_linear
        self.convs, self.norms = nn.ModuleList(), nn.ModuleList()
        self.linear = nn.ModuleList() if use_linear else None
        for i in range(n_layers):
            in_hidden = n_hidden if i > 0 else in_feats
            out_hidden = n_hidden if i < n_layers - 1 else n_classes
            self.convs.append(QGraphConv(in_hidden, out_hidden, bias=(i == n_layers - 1)))
            if use_linear:
                self.linear.append(QLinear(in_hidden, out_hidden, bias=False))
            if i < n_layers - 1:
                self.norms.append(BatchNorm1dAct(out_hidden, activation=activation))
        self.input_drop, self.dropout = nn.Dropout(min(0.1, dropout)), nn.Dropout(dropout)
        self.activation = activation

    def forward(self, graph, feat):
        h = self.input_drop(feat)
        norms = degree_norms(graph)
        for i in range(self.n_layers):
            conv = self.convs[i](graph, h, norms)
            h = conv + self.linear[i](h) if self.use_linear else conv
            if i < self.n_layers - 1:
                h = self.dropout(self.norms[i](h))  # normalisation + activation in one module
        return h
