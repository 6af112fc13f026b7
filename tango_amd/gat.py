"""Quantized GAT and HGT layers: the layer math of evaluation/test_gat.py:24-169
and evaluation/test_HGT.py:21-67, restated on the DGL-free graph object with the
edge softmax (DGL's in the reference) served by this package's kernel."""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from torch.autograd.function import Function, once_differentiable

from .QLinear import QLinear, Qlinear_func, Qlinear_func_reduce, shared_input_linears
from .batchnorm import BatchNorm1dAct
from .kernels import cuda_kernels, quantize_heads, refuse_capture
from .SDDMM import sddmm_u_add_v, sddmm_u_dot_v
from .SPMM import spmm_u_mul_e
from .edge_softmax import edge_softmax, gat_edge_attention


# Whether the GAT layers run u_add_v + LeakyReLU + edge softmax as one op (gat_edge_attention); the separate ops
# give the same values and remain for stream capture and for comparison.
fused_attention = True


class attn_scores(Function):
    """el = (feat * attn_l).sum(-1), er = (feat * attn_r).sum(-1) for feat [n, H, D] and
    attn_l, attn_r [1, H, D] (evaluation/test_gat.py:135-137), forward and backward each in
    one pass over feat.  Returns el, er as [n, H, 1] and their quantization scales max|.| / 127
    (None while a graph is being captured), which the same kernel finds.

    ``through=True`` returns feat itself as a fifth result, for the layer's other reader of feat (the
    aggregation, evaluation/test_gat.py:151) to take instead of feat: both gradients of feat then arrive at
    this node, whose backward kernel adds the aggregation's to its own as it writes and finds max|sum| / 127
    for the linear layer below (left on the gradient, ``grad_scale_hint``), where autograd would add the two in
    a pass of its own and that layer scan the sum in another.  Same sum, same bits."""

    @staticmethod
    def forward(ctx, feat, attn_l, attn_r, through=False):
        feat = feat if feat.is_contiguous() else feat.contiguous()
        al, ar = attn_l.contiguous(), attn_r.contiguous()
        el, er, s_el, s_er = cuda_kernels.attn_scores_forward(feat, al, ar, want_scales=True)
        ctx.backward_cache = feat, al, ar, attn_l.shape, through
        ctx.set_materialize_grads(False)  # no zero tensors (a fill launch each) for the scales' absent gradients
        if s_el is not None:
            ctx.mark_non_differentiable(s_el, s_er)
        out = el.unsqueeze(-1), er.unsqueeze(-1), s_el, s_er
        return (out + (feat.view_as(feat),)) if through else out

    @staticmethod
    @once_differentiable
    def backward(ctx, *grads):
        refuse_capture("attn_scores.backward")
        feat, al, ar, shape, through = ctx.backward_cache
        del_, der = grads[0], grads[1]
        dthrough = grads[4] if through else None
        if del_ is None and der is None:
            return dthrough, None, None, None
        del_ = torch.zeros_like(der) if del_ is None else del_
        der = torch.zeros_like(del_) if der is None else der
        if dthrough is None:
            dfeat, dal, dar = cuda_kernels.attn_scores_backward(del_.contiguous(), der.contiguous(), feat, al, ar)
        else:
            dfeat, dal, dar, s = cuda_kernels.attn_scores_backward(del_.contiguous(), der.contiguous(), feat, al, ar,
                                                                   addend=dthrough.contiguous())
            dfeat._tango_scale = (s, dfeat._version, dfeat.data_ptr())
        return dfeat, dal.view(shape), dar.view(shape), None


class QGATConv(nn.Module):
    """evaluation/test_gat.py:24-169 for a homogeneous graph (feat is one tensor); same
    constructor arguments in the same order."""

    def __init__(self, in_feats, out_feats, num_heads, feat_drop=0., attn_drop=0., negative_slope=0.2,
                 residual=False, activation=None, allow_zero_in_degree=False, bias=True):
        super().__init__()
        self._num_heads, self._out_feats = num_heads, out_feats
        self._allow_zero_in_degree = allow_zero_in_degree
        self.fc = QLinear(in_feats, out_feats * num_heads, bias=False)
        self.fc.enable_reduce()  # the GEMM epilogue hands max|feat_src| / 127 to the aggregation
        self.attn_l = nn.Parameter(torch.empty(1, num_heads, out_feats))
        self.attn_r = nn.Parameter(torch.empty(1, num_heads, out_feats))
        self.feat_drop = nn.Dropout(feat_drop)
        self.attn_drop = nn.Dropout(attn_drop)
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
        if not self._allow_zero_in_degree:  # test_gat.py:93-96
            # answered once per graph: the check reads a device tensor back, and a host sync in every
            # layer's forward would leave the GPU idle while the host issues the next launches
            zero_in = getattr(graph, "_has_zero_in_degree", None)
            if zero_in is None:
                zero_in = graph._has_zero_in_degree = bool((graph.in_degrees() == 0).any())
            if zero_in:
                raise Exception("There are 0-in-degree nodes in the graph.")
        n = feat.size(0)
        h = self.feat_drop(feat).contiguous()
        res = None
        if isinstance(self.res_fc, QLinear) and h.dim() == 2:
            # the projection and the residual projection read the same input: quantized once, and their two
            # input gradients land in one tensor
            (feat_src, s_feat), (res, _) = shared_input_linears(h, [self.fc, self.res_fc])
        else:
            feat_src, s_feat = self.fc(h)
        feat_src = feat_src.view(n, self._num_heads, self._out_feats)
        el, er, s_el, s_er, feat_src = attn_scores.apply(feat_src, self.attn_l, self.attn_r, True)  # test_gat.py:135-137
        s_a = None
        if s_el is not None and fused_attention:
            # u_add_v :141, LeakyReLU :144 and the softmax :146 as one op that also hands the aggregation
            # max(a) / 127; e is never stored
            a, s_a = gat_edge_attention.apply(graph, el, er, s_el, s_er, self.negative_slope)
        else:
            e = sddmm_u_add_v.apply(graph, el, er, s_el, s_er)          # :141
            a = edge_softmax(graph, e, negative_slope=self.negative_slope)  # LeakyReLU :144 + softmax :146
        if self.attn_drop.p > 0 and self.training:
            a, s_a = self.attn_drop(a), None  # the dropped-out tensor has another maximum
        # without a residual branch the bias add (:160-162) rides in the aggregation's epilogue
        fold_bias = self.bias is not None and self.res_fc is None
        # and so does the activation (:164-165) when nothing else is added between the two
        fold_act = None
        if self.res_fc is None and (fold_bias or self.bias is None):
            fold_act = "elu" if self.activation is F.elu else "relu" if self.activation in (F.relu, torch.relu) else None
        rst = spmm_u_mul_e.apply(graph, feat_src, a, self.bias if fold_bias else None, s_feat, fold_act, s_a)  # :151
        if self.res_fc is not None:
            rst = rst + (self.res_fc(h) if res is None else res).view(n, -1, self._out_feats)
        if self.bias is not None and not fold_bias:
            rst = rst + self.bias.view(1, self._num_heads, self._out_feats)
        if self.activation and fold_act is None:
            rst = self.activation(rst)
        return (rst, a) if get_attention else rst


class GAT(nn.Module):
    """evaluation/test_gat.py:170-214: input projection, hidden layers on the concatenated
    heads, output layer averaged over its heads."""

    def __init__(self, g, num_layers, in_dim, num_hidden, num_classes, heads, activation, feat_drop=0.,
                 attn_drop=0., negative_slope=0.2, residual=False):
        super().__init__()
        self.g, self.num_layers = g, num_layers
        self.gat_layers = nn.ModuleList()
        if num_layers > 1:
            self.gat_layers.append(QGATConv(in_dim, num_hidden, heads[0], feat_drop, attn_drop, negative_slope,
                                            False, activation))
            for l in range(1, num_layers - 1):
                self.gat_layers.append(QGATConv(num_hidden * heads[l - 1], num_hidden, heads[l], feat_drop,
                                                attn_drop, negative_slope, residual, activation))
            # as in the reference, the output layer keeps num_hidden columns (num_classes is unused there)
            self.gat_layers.append(QGATConv(num_hidden * heads[-2], num_hidden, heads[-1], feat_drop, attn_drop,
                                            negative_slope, residual, None))
        else:
            self.gat_layers.append(QGATConv(in_dim, num_hidden, heads[0], feat_drop, attn_drop, negative_slope,
                                            residual, None))

    def forward(self, inputs):
        h = inputs
        for l in range(self.num_layers - 1):
            h = self.gat_layers[l](self.g, h).flatten(1)
        return self.gat_layers[-1](self.g, h).mean(1)


class HGTLayer(nn.Module):
    """evaluation/test_HGT.py:27-67, the class the reference calls HGT: one attention layer over a
    homogenised graph (it has no per-type weights)."""

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

    def forward(self, g, h, s_h=None, return_scale=False):
        """``s_h``: max|h| / 127 when the producer of h knows it (the previous layer's output GEMM);
        ``return_scale``: also return this layer's output scale for the next layer."""
        # one absmax (unless handed in) and one quantize pass for the three projections of h, and one input
        # gradient that their backward GEMMs accumulate into
        # (attn_linear and msg_linear are the only readers of the k and v projections, which therefore exist
        # in int8 only)
        (k, s_k), (v, s_v), (q, s_q) = shared_input_linears(
            h, (self.k_linear, self.v_linear, self.q_linear), s_h, then=(self.attn_linear, self.msg_linear, None))
        k, v, q = (t.view(-1, self.n_heads, self.d_k) for t in (k, v, q))
        t = sddmm_u_dot_v.apply(g, k, q, s_k, s_q, 1.0 / self.sqrt_dk)  # "/ sqrt_dk" folded into the scales
        attn, s_attn = edge_softmax(g, t, want_scale=True)  # the softmax kernel also finds the scale of its output
        t = spmm_u_mul_e.apply(g, v, attn, None, s_v, None, s_attn).reshape(-1, self.out_dim)
        if return_scale:
            return Qlinear_func_reduce.apply(t, self.a_linear.weight, self.a_linear.bias)
        return self.a_linear(t)


HGT = HGTLayer  # the reference's name (evaluation/test_HGT.py:27)


class ArxivGATConv(nn.Module):
    """The attention layer of evaluation/arxiv_gat.py:63-218 on a homogeneous graph: no bias (the model adds
    one after its last layer), a quantized residual projection of the layer's input, an optional attention
    term for the destination (``use_attn_dst``) and the optional symmetric degree normalisation.
    ``edge_drop`` > 0 (training mode): a random share of the edges takes no part in the softmax and aggregates
    nothing (arxiv_gat.py:186-194, the ``eids=`` form of the edge softmax); that path runs the unfused ops."""

    def __init__(self, in_feats, out_feats, num_heads=1, feat_drop=0.0, attn_drop=0.0, edge_drop=0.0,
                 negative_slope=0.2, use_attn_dst=True, residual=False, activation=None,
                 allow_zero_in_degree=False, use_symmetric_norm=False):
        super().__init__()
        if not 0.0 <= edge_drop < 1.0:
            raise ValueError("ArxivGATConv: edge_drop must be in [0, 1)")
        self.edge_drop = edge_drop
        self._num_heads, self._out_feats = num_heads, out_feats
        self._allow_zero_in_degree, self._use_symmetric_norm = allow_zero_in_degree, use_symmetric_norm
        self.fc = QLinear(in_feats, out_feats * num_heads, bias=False)
        self.fc.enable_reduce()
        self.attn_l = nn.Parameter(torch.empty(1, num_heads, out_feats))
        self.attn_r = nn.Parameter(torch.empty(1, num_heads, out_feats)) if use_attn_dst else None
        self.feat_drop, self.attn_drop = nn.Dropout(feat_drop), nn.Dropout(attn_drop)
        self.negative_slope = negative_slope
        self.res_fc = QLinear(in_feats, num_heads * out_feats, bias=False) if residual else None
        self._activation = activation
        gain = nn.init.calculate_gain("relu")  # arxiv_gat.py:113-124
        nn.init.xavier_normal_(self.fc.weight, gain=gain)
        nn.init.xavier_normal_(self.attn_l, gain=gain)
        if self.attn_r is not None:
            nn.init.xavier_normal_(self.attn_r, gain=gain)
        if self.res_fc is not None:
            nn.init.xavier_normal_(self.res_fc.weight, gain=gain)

    def forward(self, graph, feat):
        if not self._allow_zero_in_degree:  # arxiv_gat.py:131-133, answered once per graph
            zero_in = getattr(graph, "_has_zero_in_degree", None)
            if zero_in is None:
                zero_in = graph._has_zero_in_degree = bool((graph.in_degrees() == 0).any())
            assert not zero_in
        n = feat.size(0)
        h = self.feat_drop(feat).contiguous()
        res = None
        if self._use_symmetric_norm:  # :158-163; the product is a new tensor, so the epilogue's scale does not apply
            # the plain (no output scale) functional form of self.fc: no state of the module is touched
            feat_src = Qlinear_func.apply(h.reshape(-1, h.size(-1)), self.fc.weight, self.fc.bias)
            feat_src = feat_src.view(n, self._num_heads, self._out_feats)
            s_feat = None
            feat_src = feat_src * graph.out_degrees().float().clamp(min=1).pow(-0.5).view(n, 1, 1)
        elif self.res_fc is not None and h.dim() == 2:
            # the projection and the residual projection read the same input: quantized once, and their two
            # input gradients land in one tensor
            (feat_src, s_feat), (res, _) = shared_input_linears(h, [self.fc, self.res_fc])
            feat_src = feat_src.view(n, self._num_heads, self._out_feats)
        else:
            feat_src, s_feat = self.fc(h)
            feat_src = feat_src.view(n, self._num_heads, self._out_feats)
        s_a = None
        if self.training and self.edge_drop > 0:  # :186-194
            if self.attn_r is not None:
                el, er, s_el, s_er = attn_scores.apply(feat_src, self.attn_l, self.attn_r)
                e = sddmm_u_add_v.apply(graph, el, er, s_el, s_er)
            else:
                e = (feat_src * self.attn_l).sum(-1, keepdim=True)[graph.coo[0]]
            perm = torch.randperm(graph.num_edges(), device=e.device)
            eids = perm[int(graph.num_edges() * self.edge_drop):]
            kept = self.attn_drop(edge_softmax(graph, e[eids], negative_slope=self.negative_slope, eids=eids))
            a = torch.zeros_like(e).index_copy(0, eids, kept)
        elif self.attn_r is not None:  # :176-184
            el, er, s_el, s_er, feat_src = attn_scores.apply(feat_src, self.attn_l, self.attn_r, True)
            if s_el is not None and fused_attention:
                a, s_a = gat_edge_attention.apply(graph, el, er, s_el, s_er, self.negative_slope)  # :184, :187, :196
            else:
                a = edge_softmax(graph, sddmm_u_add_v.apply(graph, el, er, s_el, s_er), negative_slope=self.negative_slope)
        else:  # copy_u of el (:186)
            e = (feat_src * self.attn_l).sum(-1, keepdim=True)[graph.coo[0]]
            a, s_a = edge_softmax(graph, e, negative_slope=self.negative_slope, want_scale=True)  # :187, :196
        if self.attn_drop.p > 0 and self.training and not self.edge_drop > 0:
            a, s_a = self.attn_drop(a), None
        rst = spmm_u_mul_e.apply(graph, feat_src, a, None, s_feat, None, s_a)  # :201
        if self._use_symmetric_norm:  # :203-208
            rst = rst * graph.in_degrees().float().clamp(min=1).pow(0.5).view(n, 1, 1)
        if self.res_fc is not None:  # :211-214
            rst = rst + (self.res_fc(h) if res is None else res).view(n, -1, self._out_feats)
        if self._activation is not None:
            rst = self._activation(rst)
        return rst


class ArxivGAT(nn.Module):
    """evaluation/arxiv_gat.py:376-448: ``n_layers`` attention layers with a residual projection each, batch
    normalisation, the activation and dropout between them; the last layer has one head and ``n_classes``
    columns, is averaged over that head and gets a bias of its own."""

    def __init__(self, in_feats, n_classes, n_hidden, n_layers, n_heads, activation, dropout=0.0, input_drop=0.0,
                 attn_drop=0.0, edge_drop=0.0, use_attn_dst=True, use_symmetric_norm=False):
        super().__init__()
        self.n_layers = n_layers
        self.convs, self.norms = nn.ModuleList(), nn.ModuleList()
        for i in range(n_layers):
            in_hidden = n_heads * n_hidden if i > 0 else in_feats
            out_hidden = n_hidden if i < n_layers - 1 else n_classes
            heads = n_heads if i < n_layers - 1 else 1
            self.convs.append(ArxivGATConv(in_hidden, out_hidden, num_heads=heads, attn_drop=attn_drop,
                                           edge_drop=edge_drop, use_attn_dst=use_attn_dst,
                                           use_symmetric_norm=use_symmetric_norm, residual=True))
            if i < n_layers - 1:
                self.norms.append(BatchNorm1dAct(n_heads * out_hidden, activation=activation))
        self.bias_last = nn.Parameter(torch.zeros(n_classes))  # ElementWiseLinear(weight=False, bias=True), :28-58
        self.input_drop, self.dropout = nn.Dropout(input_drop), nn.Dropout(dropout)
        self.activation = activation

    def forward(self, graph, feat):
        h = self.input_drop(feat)
        for i in range(self.n_layers):
            h = self.convs[i](graph, h)
            if i < self.n_layers - 1:
                h = self.dropout(self.norms[i](h.flatten(1)))  # normalisation + activation in one module
        return h.mean(1) + self.bias_last


class HeteroHGTLayer(nn.Module):
    """One HGT layer on a heterogeneous graph held in one node id space (node types occupy consecutive id
    ranges, every edge carries a relation id): the layer of evaluation/test_HGT.py:27-67 with what that file's
    homogenised form leaves out, weights per node type and per relation.  Projections k / q / v and the output
    projection are typed by node type; each relation r has its own attention and message layers
    (``attn_linear[r]``, ``msg_linear[r]``, the homogeneous layer's two, now one pair per relation) and runs its
    own SDDMM and aggregation over its edges; the softmax runs over all in-edges of a destination, whatever
    their relation."""

    def __init__(self, in_dim, out_dim, n_heads, type_sizes, relation_graphs):
        """``type_sizes``: nodes per type, in id order.  ``relation_graphs``: per relation a preprocessed Graph
        on all nodes holding that relation's edges, its attribute ``eids`` their ids in the full graph, and
        ``src_type``: the node type its sources belong to."""
        super().__init__()
        self.out_dim, self.n_heads, self.d_k = out_dim, n_heads, out_dim // n_heads
        self.sqrt_dk = math.sqrt(self.d_k)
        self.bounds = [0]
        for m in type_sizes:
            self.bounds.append(self.bounds[-1] + m)
        self.rels = list(relation_graphs)
        # per-relation layers are indexed by the relation's id, not by its place in the list, so that the parameter
        # layout does not depend on which relations happen to have edges in this graph
        self.rel_ids = [getattr(gr, "rel_id", i) for i, gr in enumerate(self.rels)]
        nt = len(type_sizes)
        nr = max([getattr(gr, "num_relations", 0) for gr in self.rels] + [max(self.rel_ids, default=-1) + 1])
        mk = lambda i, o, k: nn.ModuleList(QLinear(i, o) for _ in range(k))
        self.k_linear, self.q_linear, self.v_linear = mk(in_dim, out_dim, nt), mk(in_dim, out_dim, nt), mk(in_dim, out_dim, nt)
        self.a_linear = mk(out_dim, out_dim, nt)
        self.attn_linear, self.msg_linear = mk(out_dim, out_dim, nr), mk(out_dim, out_dim, nr)

    def _typed(self, layers, h):
        """Rows of node type t through layers[t]."""
        return torch.cat([layers[t](h[self.bounds[t]:self.bounds[t + 1]]) for t in range(len(layers))])

    def forward(self, g, h):
        H, dk, nt = self.n_heads, self.d_k, len(self.bounds) - 1
        # k / v / q per node type: the type's rows are quantized once for the three projections, whose input
        # gradients land in one tensor
        k, v, q = [], [], []
        for t in range(nt):
            kt, vt, qt = shared_input_linears(h[self.bounds[t]:self.bounds[t + 1]],
                                              (self.k_linear[t], self.v_linear[t], self.q_linear[t]))
            k.append(kt), v.append(vt), q.append(qt)
        # every relation runs on its own bipartite graph(s), each endpoint numbered inside its node type: no
        # tensor here has rows for nodes the relation does not touch
        units = [(r, part) for r, gr in zip(self.rel_ids, self.rels) for part in gr.parts]
        # relation-specific keys and messages; the relations that start at one node type share that type's
        # k (v) quantized once
        kr, vr = {}, {}
        for t in range(nt):
            rs = sorted({r for r, part in units if part.src_type == t})
            if not rs:
                continue
            for r, pair in zip(rs, shared_input_linears(k[t][0], [self.attn_linear[r] for r in rs], k[t][1])):
                kr[t, r] = pair
            for r, pair in zip(rs, shared_input_linears(v[t][0], [self.msg_linear[r] for r in rs], v[t][1])):
                vr[t, r] = pair
        scores = []
        q8 = {}  # the queries of a node type in int8, shared by the relations that end there
        for r, part in units:
            (U, sU), (V, sV) = kr[part.src_type, r], q[part.dst_type]
            V = V.view(-1, H, dk)
            if part.dst_type not in q8:
                q8[part.dst_type] = quantize_heads(V if V.is_contiguous() else V.contiguous(), sV)
            scores.append(sddmm_u_dot_v.apply(part, U.view(-1, H, dk), V, sU, sV, 1.0 / self.sqrt_dk, q8[part.dst_type]))
        ranges = [part.edge_range for _, part in units]
        contiguous = all(rg is not None for rg in ranges)
        if contiguous:
            order = sorted(range(len(units)), key=lambda i: ranges[i][0])
            ends = [0] + [ranges[i][1] for i in order]
            contiguous = all(ranges[i][0] == e for i, e in zip(order, ends)) and ends[-1] == g.num_edges()
        if contiguous:  # the parts own consecutive edge-id ranges: the scores are their concatenation
            t = torch.cat([scores[i] for i in order])
        else:
            t = h.new_zeros((g.num_edges(), H, 1))
            for (_, part), tr in zip(units, scores):
                t = t.index_copy(0, part.eids, tr)
        # over every in-edge of a destination, all relations together; the kernel also finds max(attn) / 127
        attn, s_attn = edge_softmax(g, t, want_scale=True)
        out = [None] * nt
        if contiguous:  # one split (backward: one concatenation) instead of a slice per part (a zero-filled [E, H] each)
            pieces = torch.split(attn, [ranges[i][1] - ranges[i][0] for i in order])
            piece_of = {i: pieces[k] for k, i in enumerate(order)}
        for i, (r, part) in enumerate(units):
            ar = piece_of[i] if contiguous else attn[part.eids]
            M, sM = vr[part.src_type, r]
            o = spmm_u_mul_e.apply(part, M.view(-1, H, dk), ar, None, sM, None, s_attn)
            out[part.dst_type] = o if out[part.dst_type] is None else out[part.dst_type] + o
        res = []
        for t in range(nt):
            m = self.bounds[t + 1] - self.bounds[t]
            o = h.new_zeros((m, self.out_dim)) if out[t] is None else out[t].reshape(m, self.out_dim)
            res.append(self.a_linear[t](o))
        return torch.cat(res)


def relation_major(g, edge_type):
    """(graph, edge types) with the edges renumbered relation by relation and, inside a relation, by destination:
    every relation then owns a consecutive range of edge ids (per-relation edge tensors are slices of the full
    one, no gather or scatter), and its own graph walks its edges front to back."""
    from .graph import Graph
    src, dst = g.edges()
    order = torch.sort(edge_type * g.num_nodes() + dst, stable=True).indices
    g2 = Graph(src[order], dst[order], g.num_nodes())
    g2.edge_order = order
    return g2, edge_type[order]


def relation_graphs(g, edge_type, relations, type_sizes):
    """Per relation id in ``edge_type`` ([E], ids 0 .. len(relations) where the last id marks self loops) a
    preprocessed Graph over all nodes of ``g`` with that relation's edges, ``eids`` (their ids in ``g``),
    ``edge_range`` ((first, last + 1) when those ids are consecutive and the relations come in order, as after
    ``relation_major``; else None), ``src_type`` and ``parts`` attached.  ``parts``: the same edges as bipartite
    graphs, one per (source type, destination type) pair that occurs, each endpoint numbered inside its node
    type, with ``src_type``, ``dst_type``, ``eids`` and ``edge_range`` of their own: what the layer runs on."""
    from .graph import Graph
    from .util import graph_preprocess
    src, dst = g.edges()
    bounds = [0]
    for m in type_sizes:
        bounds.append(bounds[-1] + m)
    edges_of = torch.tensor(bounds[1:], device=src.device)
    out, nxt, in_order = [], 0, True
    for r in range(len(relations) + 1):
        eids = torch.nonzero(edge_type == r).flatten()
        if eids.numel() == 0:
            continue
        rs, rd = src[eids], dst[eids]
        gr = graph_preprocess(Graph(rs, rd, g.num_nodes()))
        gr.eids = eids
        lo, hi = int(eids[0]), int(eids[-1]) + 1
        in_order = in_order and lo == nxt and hi - lo == eids.numel()
        gr.edge_range = (lo, hi)
        nxt = hi
        gr.src_type = relations[r][0] if r < len(relations) else None  # self loops start at every type
        gr.rel_id, gr.num_relations = r, len(relations) + 1  # what the layer keys its per-relation weights by
        ts, td = torch.bucketize(rs, edges_of, right=True), torch.bucketize(rd, edges_of, right=True)
        pair = ts * len(type_sizes) + td
        gr.parts = []
        for code in torch.unique(pair).tolist():
            a, b = divmod(code, len(type_sizes))
            sub = torch.nonzero(pair == code).flatten()
            part = graph_preprocess(Graph(rs[sub] - bounds[a], rd[sub] - bounds[b], type_sizes[a], type_sizes[b]))
            part.src_type, part.dst_type, part.eids = a, b, eids[sub]
            plo, phi = int(part.eids[0]), int(part.eids[-1]) + 1
            part.edge_range = (plo, phi) if phi - plo == sub.numel() else None
            gr.parts.append(part)
        out.append(gr)
    if not in_order or nxt != g.num_edges():
        for gr in out:
            gr.edge_range = None
            for part in gr.parts:
                part.edge_range = None
    return out


class HGTStack(nn.Module):
    """Several HGT layers back to back with a linear read-out, the shape of the reference's
    driver loop (evaluation/test_HGT.py:87-96: model, then ``proj_layer``)."""

    def __init__(self, in_dim, hidden, n_classes, n_heads, n_layers=2):
        super().__init__()
        dims = [in_dim] + [hidden] * n_layers
        self.layers = nn.ModuleList(HGTLayer(dims[i], dims[i + 1], n_heads) for i in range(n_layers))
        self.proj = nn.Linear(hidden, n_classes)

    def forward(self, g, h):
        s_h = None
        for i, layer in enumerate(self.layers):
            if i + 1 < len(self.layers):  # the output GEMM's epilogue hands max|h| / 127 to the next layer
                h, s_h = layer(g, h, s_h, return_scale=True)
            else:
                h = layer(g, h, s_h)
        return self.proj(h)
