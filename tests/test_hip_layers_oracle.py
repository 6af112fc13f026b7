"""Whole attention layers against the CPU oracle, stage by stage: every primitive call a layer makes is recorded
during its forward pass, and each recorded output is compared with the oracle applied to that call's recorded
inputs (bit for bit where the stage is integer arithmetic plus fixed fp32 roundings, 1e-5 / 1e-6 where it sums
or exponentiates in fp32), so that the layer's output is tied to the oracle through the chain."""
import numpy as np
import pytest
import torch

from gpu_util import host

pytestmark = pytest.mark.gpu


class _Recorder:
    """Stands in for an autograd Function (or a function) of a module's namespace and records (args, output)."""

    def __init__(self, target, is_function_class):
        self.target, self.is_function_class, self.calls = target, is_function_class, []

    def apply(self, *args):
        out = self.target.apply(*args)
        self.calls.append((args, out))
        return out

    def __call__(self, *args, **kw):
        out = self.target(*args, **kw)
        self.calls.append((args, kw, out))
        return out


@pytest.fixture()
def recorded(monkeypatch):
    import tango_amd.gat as gat
    rec = {}
    for name in ("attn_scores", "sddmm_u_add_v", "sddmm_u_dot_v", "spmm_u_mul_e"):
        rec[name] = _Recorder(getattr(gat, name), True)
        monkeypatch.setattr(gat, name, rec[name])
    rec["edge_softmax"] = _Recorder(gat.edge_softmax, False)
    monkeypatch.setattr(gat, "edge_softmax", rec["edge_softmax"])
    return rec


def _small_graph(n, e, seed):
    from tango_amd.graph import chung_lu
    from tango_amd.util import graph_preprocess
    return graph_preprocess(chung_lu(n, e, 2.2, seed=seed, device="cuda"))


def test_arxiv_gat_layer_matches_oracle_stage_by_stage(orc, recorded, monkeypatch):
    import tango_amd.gat as gat_module
    from tango_amd.gat import ArxivGATConv
    monkeypatch.setattr(gat_module, "fused_attention", False)  # the separate ops, one oracle stage each
    g = _small_graph(3000, 24000, 5)
    n, E, H, D, Fin = g.num_nodes(), g.num_edges(), 3, 16, 64
    torch.manual_seed(3)
    layer = ArxivGATConv(Fin, D, num_heads=H, residual=True).cuda()
    x = torch.randn(n, Fin, device="cuda")
    out = layer(g, x)
    # fc: fused-quantize GEMM with the output scale from its epilogue
    W = host(layer.fc.weight)
    feat, _, _, _, _, s_feat = orc.qgemm_fwd(host(x), W, reduce=True)
    (args, res), = recorded["attn_scores"].calls
    assert np.array_equal(host(args[0]).reshape(n, H * D), feat)
    el, er, s_el, s_er = res[:4]
    al, ar = host(layer.attn_l).reshape(H, D), host(layer.attn_r).reshape(H, D)
    f3 = feat.reshape(n, H, D).astype(np.float64)
    np.testing.assert_allclose(host(el).reshape(n, H), (f3 * al).sum(-1), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(host(er).reshape(n, H), (f3 * ar).sum(-1), rtol=1e-5, atol=1e-5)
    assert host(s_el)[0] == orc.absmax_scale(host(el)) and host(s_er)[0] == orc.absmax_scale(host(er))
    # e = quantized el[src] + quantized er[dst]
    (args, e), = recorded["sddmm_u_add_v"].calls
    elq, erq = orc.quantize(host(el), host(s_el)[0]), orc.quantize(host(er), host(s_er)[0])
    want_e, _ = orc.sddmm_ewise("add", host(g.coo[0]), host(g.coo[1]), elq.reshape(n, H), erq.reshape(n, H),
                                host(s_el)[0], host(s_er)[0])
    assert np.array_equal(host(e).reshape(E, H), want_e)
    # LeakyReLU + softmax over the in-edges
    (args, kw, a), = recorded["edge_softmax"].calls
    ip, ix, eid = (host(t) for t in g.adj_csc)
    np.testing.assert_allclose(host(a).reshape(E, H), orc.edge_softmax_fwd(host(e).reshape(E, H), ip, eid, 0.2),
                               rtol=1e-5, atol=1e-6)
    # attention-weighted aggregation of the int8 features with the GEMM's scale
    (args, rst), = recorded["spmm_u_mul_e"].calls
    sa = orc.absmax_scale(host(a))
    aq = orc.quantize(host(a), sa).reshape(E, H, 1)
    want = orc.spmm_csr_u_mul_e_ex(ip, ix, eid, orc.quantize(feat, s_feat).reshape(n, H, D), aq, s_feat, scale2=sa,
                                   edge_major=True)
    assert np.array_equal(host(rst), want)
    # residual projection and the sum
    res_val, *_ = orc.qgemm_fwd(host(x), host(layer.res_fc.weight))
    assert np.array_equal(host(out), want + res_val.reshape(n, H, D))


def test_hgt_layer_matches_oracle_stage_by_stage(orc, recorded):
    from tango_amd.gat import HGTLayer
    g = _small_graph(2500, 30000, 6)
    n, E, H, dk = g.num_nodes(), g.num_edges(), 4, 16
    torch.manual_seed(4)
    layer = HGTLayer(64, 64, H).cuda()
    h = torch.randn(n, 64, device="cuda")
    out = layer(g, h)
    lin = lambda m: (host(m.weight), host(m.bias))
    # the three projections share one truncation-quantized input; k and v pass through a second layer in int8
    X = host(h)
    sX = orc.absmax_scale(X)
    Xq = orc.quantize(X, sX, orc.TRUNC)

    def chain(first, second):
        W, b = lin(first)
        sW = orc.absmax_scale(W)
        Y, sY = orc.qgemm_i8_nt(Xq, orc.quantize(W, sW, orc.TRUNC), sX, sW, bias=b, reduce=True)
        if second is None:
            return Y, sY
        W2, b2 = lin(second)
        sW2 = orc.absmax_scale(W2)
        return orc.qgemm_i8_nt(orc.quantize(Y, sY, orc.TRUNC), orc.quantize(W2, sW2, orc.TRUNC), sY, sW2, bias=b2,
                               reduce=True)
    k, s_k = chain(layer.k_linear, layer.attn_linear)
    v, s_v = chain(layer.v_linear, layer.msg_linear)
    q, s_q = chain(layer.q_linear, None)
    (args, t), = recorded["sddmm_u_dot_v"].calls
    assert np.array_equal(host(args[1]).reshape(n, -1), k) and np.array_equal(host(args[2]).reshape(n, -1), q)
    assert host(args[3])[0] == s_k and host(args[4])[0] == s_q
    kq, qq = orc.quantize(k, s_k).reshape(n, H, dk), orc.quantize(q, s_q).reshape(n, H, dk)
    # "/ sqrt(d_k)" folded into the second scale (1/4 here: a power of two, so exact either way)
    want_t, _ = orc.sddmm_dot(host(g.coo[0]), host(g.coo[1]), kq, qq, s_k, np.float32(s_q * np.float32(0.25)))
    assert np.array_equal(host(t).reshape(E, H), want_t)
    (args, kw, (a, s_attn)), = recorded["edge_softmax"].calls
    ip, ix, eid = (host(x_) for x_ in g.adj_csc)
    np.testing.assert_allclose(host(a).reshape(E, H), orc.edge_softmax_fwd(want_t, ip, eid, 1.0), rtol=1e-5, atol=1e-6)
    assert host(s_attn)[0] == orc.absmax_scale(host(a))  # found by the softmax kernel itself
    (args, agg), = recorded["spmm_u_mul_e"].calls
    sa = orc.absmax_scale(host(a))
    want_agg = orc.spmm_csr_u_mul_e_ex(ip, ix, eid, orc.quantize(v, s_v).reshape(n, H, dk),
                                       orc.quantize(host(a), sa).reshape(E, H, 1), s_v, scale2=sa, edge_major=True)
    assert np.array_equal(host(agg), want_agg)
    Wa, ba = lin(layer.a_linear)
    want_out, *_ = orc.qgemm_fwd(want_agg.reshape(n, H * dk), Wa, bias=ba)
    assert np.array_equal(host(out), want_out)


@pytest.mark.parametrize("H,slope,reorder", [(8, 0.2, True), (8, 0.2, False), (3, 0.2, False), (1, 0.5, True),
                                              (12, 0.2, False), (4, 1.0, True)])
def test_fused_attention_kernels_match_oracle(orc, H, slope, reorder):
    """tango_edge_softmax_fwd_ex / _bwd_ex: logits formed on the fly from el, er (never stored), sign bytes for the
    backward pass, the scales of both results from the same kernels; against the oracle's separate stages."""
    from tango_amd.graph import Graph
    from tango_amd.kernels import cuda_kernels as ck
    from tango_amd.util import graph_preprocess
    rng = np.random.default_rng(H)
    n, E = 4000, 60000
    w = 1.0 / np.arange(1, n + 1) ** 1.2
    w /= w.sum()
    src, dst = rng.choice(n, E, p=w), rng.choice(n, E, p=w)  # hubs with thousands of in-edges, rows cut by spans
    g0 = Graph(torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda(), n)
    g = graph_preprocess(g0.reorder_edges_by_dst() if reorder else g0)
    src, dst = host(g.coo[0]), host(g.coo[1])
    ip, _, eid = g.adj_csc
    eids = None if g.csc_slots_are_edge_ids else eid
    el = rng.standard_normal((n, H)).astype(np.float32)
    er = rng.standard_normal((n, H)).astype(np.float32)
    s_el, s_er = orc.absmax_scale(el), orc.absmax_scale(er)
    dev = lambda x: torch.from_numpy(x).cuda()
    sc = lambda v: torch.tensor([v], dtype=torch.float32, device="cuda")
    a, s_a, sign = ck.edge_softmax_forward_ex(None, ip, eids, slope, logits=(dev(el), dev(er), sc(s_el), sc(s_er), g.coo[0], g.coo[1]),
                                              want_sign=True)
    want_e, _ = orc.sddmm_ewise("add", src, dst, orc.quantize(el, s_el), orc.quantize(er, s_er), s_el, s_er)
    want_a = orc.edge_softmax_fwd(want_e, host(ip), host(eid), slope)
    np.testing.assert_allclose(host(a), want_a, rtol=1e-5, atol=1e-6)
    assert host(s_a)[0] == orc.absmax_scale(host(a))
    # the same kernel reading stored logits gives the same bits
    a2, s_a2, _ = ck.edge_softmax_forward_ex(dev(want_e), ip, eids, slope)
    assert torch.equal(a2, a) and torch.equal(s_a2, s_a)
    assert torch.equal(ck.edge_softmax_forward(dev(want_e), ip, eids, slope), a)
    # sign bytes, in destination-major slot order
    slot_edge = host(eid)
    bits = np.unpackbits(host(sign), axis=1, bitorder="little")[:, :H].astype(bool)
    assert np.array_equal(bits, want_e[slot_edge] > 0)
    # backward from the sign bytes == backward from the stored logits == oracle
    da = rng.standard_normal((E, H)).astype(np.float32)
    de, s_de = ck.edge_softmax_backward_ex(a, dev(da), None, sign, ip, eids, slope)
    de2 = ck.edge_softmax_backward(a, dev(da), dev(want_e), ip, eids, slope)
    assert torch.equal(de, de2)
    np.testing.assert_allclose(host(de), orc.edge_softmax_bwd(host(a), da, want_e, host(ip), host(eid), slope),
                               rtol=1e-4, atol=1e-6)
    assert host(s_de)[0] == orc.absmax_scale(host(de))


@pytest.mark.parametrize("H,F", [(8, 16), (3, 5), (4, 64)])
def test_aggregation_quantizes_fp32_edge_values_on_load(orc, H, F):
    """tango_spmm_csr_u_mul_e_f32e == quantize the edge values first, then tango_spmm_csr_u_mul_e_ex: on a sparse
    graph (slot-span kernels), a dense one (row kernels) and both orientations."""
    from tango_amd import kernels as K
    rng = np.random.default_rng(F)
    for n, E in ((3000, 20000), (300, 60000)):
        g = _small_graph(n, E, 11) if n == 3000 else None
        if g is None:
            from tango_amd.graph import Graph
            from tango_amd.util import graph_preprocess
            g = graph_preprocess(Graph(torch.from_numpy(rng.integers(0, n, E)).cuda(), torch.from_numpy(rng.integers(0, n, E)).cuda(), n))
        nn, ne = g.num_nodes(), g.num_edges()
        feat = torch.from_numpy(rng.integers(-127, 128, (nn, H, F)).astype(np.int8)).cuda()
        a = torch.rand(ne, H, 1, device="cuda")
        s_a = K.cuda_kernels.get_scale(a)
        aq, _ = K.quantize(a, s_a)
        one = torch.tensor([0.013], device="cuda")
        bias = torch.randn(H * F, device="cuda")
        for rev in (False, True):
            want = K.multi_cusparse_SPMM(g, feat, aq, one, rev, edge_major=True, scale2=s_a, bias=bias, act="relu")
            got = K.multi_cusparse_SPMM(g, feat, a, one, rev, edge_major=True, scale2=s_a, bias=bias, act="relu")
            assert torch.equal(got, want)
        ip, ix, eid = (host(t) for t in g.adj_csc)
        ref = orc.spmm_csr_u_mul_e_ex(ip, ix, eid, host(feat), host(aq), 0.013, scale2=host(s_a)[0], edge_major=True)
        assert np.array_equal(host(K.multi_cusparse_SPMM(g, feat, a, one, edge_major=True, scale2=s_a)), ref)


@pytest.mark.parametrize("on_the_fly,on_load", [(False, False), (True, True)])
@pytest.mark.parametrize("layer_kind", ["gat", "arxiv"])
def test_fused_attention_layer_equals_separate_ops(monkeypatch, layer_kind, on_the_fly, on_load):
    """A GAT layer with u_add_v + LeakyReLU + softmax as one op, the scale of the attention handed on and the
    aggregation rounding fp32 attention as it loads: the same output and the same gradients, bit for bit, as the
    layer built from the separate ops (which the stage-by-stage test above ties to the oracle)."""
    import torch.nn.functional as F
    import tango_amd.gat as gat_module
    from tango_amd import config
    monkeypatch.setattr(config, "attention_logits_on_the_fly", on_the_fly)
    monkeypatch.setattr(config, "edge_values_on_load", on_load)
    g = _small_graph(3000, 24000, 5)
    n = g.num_nodes()
    torch.manual_seed(3)
    if layer_kind == "gat":
        layer = gat_module.QGATConv(64, 16, 4, activation=F.elu).cuda()
    else:
        layer = gat_module.ArxivGATConv(64, 16, num_heads=3, residual=True).cuda()
    x = torch.randn(n, 64, device="cuda")
    w = torch.randn(n, layer._num_heads, 16, device="cuda")
    results = []
    for fused in (True, False):
        monkeypatch.setattr(gat_module, "fused_attention", fused)
        xi = x.clone().requires_grad_(True)
        layer.zero_grad()
        out = layer(g, xi)
        out.backward(w)
        results.append((out.detach().clone(), xi.grad.clone(), [p.grad.clone() for p in layer.parameters()]))
    (o1, gx1, gp1), (o2, gx2, gp2) = results
    assert torch.equal(o1, o2) and torch.equal(gx1, gx2)
    for (name, _), a_, b_ in zip(layer.named_parameters(), gp1, gp2):
        assert torch.equal(a_, b_), name


def _fp32_hetero_hgt(layer, g, h):
    """The heterogeneous layer's math in fp32 torch ops."""
    import torch.nn.functional as F
    n, H, dk = h.size(0), layer.n_heads, layer.d_k
    typed = lambda layers, x: torch.cat([F.linear(x[layer.bounds[t]:layer.bounds[t + 1]], layers[t].weight, layers[t].bias)
                                         for t in range(len(layers))])
    k, q, v = typed(layer.k_linear, h), typed(layer.q_linear, h).view(n, H, dk), typed(layer.v_linear, h)
    src, dst = g.coo
    t = torch.zeros((g.num_edges(), H), device=h.device)
    msgs = torch.zeros((g.num_edges(), H, dk), device=h.device)
    for r, gr in enumerate(layer.rels):
        kr = F.linear(k, layer.attn_linear[r].weight, layer.attn_linear[r].bias).view(n, H, dk)
        vr = F.linear(v, layer.msg_linear[r].weight, layer.msg_linear[r].bias).view(n, H, dk)
        s, d = src[gr.eids], dst[gr.eids]
        t[gr.eids] = (kr[s] * q[d]).sum(-1) / layer.sqrt_dk
        msgs[gr.eids] = vr[s]
    mx = torch.full((n, H), -1e30, device=h.device).scatter_reduce_(0, dst.unsqueeze(1).expand(-1, H), t, "amax")
    ex = (t - mx[dst]).exp()
    att = ex / torch.zeros((n, H), device=h.device).index_add_(0, dst, ex)[dst]
    agg = torch.zeros((n, H, dk), device=h.device).index_add_(0, dst, msgs * att.unsqueeze(-1))
    return typed(layer.a_linear, agg.reshape(n, H * dk))


def _bipartite_primitives_match_oracle(part, orc):
    """SDDMM dot and the u_mul_e aggregation in both directions on a bipartite graph, against the oracle."""
    from tango_amd import kernels as K
    from gpu_util import dev, host, sc
    ns, nd, E, H, D = part.num_src_nodes(), part.num_dst_nodes(), part.num_edges(), 4, 16
    rng = np.random.default_rng(21)
    U, V = (rng.integers(-127, 128, (m, H, D)).astype(np.int8) for m in (ns, nd))
    src, dst = host(part.coo[0]), host(part.coo[1])
    t, _ = K.mySDDMM_int8(part, "dot", dev(U), dev(V), sc(3e-3), sc(2e-3), False)
    want, _ = orc.sddmm_dot(src, dst, U, V, 3e-3, 2e-3)
    assert np.array_equal(host(t).reshape(E, H), want)
    a = rng.integers(0, 128, (E, H, 1)).astype(np.int8)
    for reverse, feat, rows in ((False, U, nd), (True, V, ns)):
        agg = K.multi_cusparse_SPMM(part, dev(feat), dev(a), sc(1e-3), reverse, edge_major=True, scale2=sc(0.5))
        assert agg.shape == (rows, H, D)
        ip, ix, eid = (host(x) for x in (part.adj_csr if reverse else part.adj_csc))
        want = orc.spmm_csr_u_mul_e_ex(ip, ix, eid, feat, a, 1e-3, scale2=0.5, edge_major=True)
        assert np.array_equal(host(agg), want), reverse


def test_hetero_hgt_layer_tracks_fp32_and_trains(orc):
    """Weights per node type and per relation: the quantized layer stays within int8 noise of the same math in
    fp32, every typed and relation-specific parameter receives a gradient, and a relation's weights do not
    influence destinations that relation does not reach."""
    from tango_amd.gat import HeteroHGTLayer, relation_graphs, relation_major
    from tango_amd.graph import hetero_power_law
    from tango_amd.util import graph_preprocess
    sizes, rels = (3000, 1500, 600), ((0, 1), (1, 0), (1, 2), (2, 0))
    g0, node_type, edge_type0 = hetero_power_law(type_sizes=sizes, relations=rels, edges_per_relation=30000, device="cuda")
    # any edge numbering works (per-relation tensors are gathered and scattered) ...
    perm = torch.randperm(g0.num_edges(), device="cuda", generator=torch.Generator("cuda").manual_seed(3))
    from tango_amd.graph import Graph
    g_any = graph_preprocess(Graph(g0.edges()[0][perm], g0.edges()[1][perm], g0.num_nodes()))
    rg_any = relation_graphs(g_any, edge_type0[perm], rels, sizes)
    assert all(r.edge_range is None for r in rg_any)
    # ... and the relation-major one turns them into slices
    g, edge_type = relation_major(g0, edge_type0)
    g = graph_preprocess(g)
    rg = relation_graphs(g, edge_type, rels, sizes)
    assert len(rg) == 5 and sum(r.num_edges() for r in rg) == g.num_edges()
    assert all(r.edge_range is not None and r.csc_slots_are_edge_ids for r in rg)
    # what the layer runs on: bipartite parts, endpoints numbered inside their node types
    assert [len(r.parts) for r in rg] == [1, 1, 1, 1, 3]
    assert [(p.src_type, p.dst_type) for r in rg for p in r.parts] == list(rels) + [(0, 0), (1, 1), (2, 2)]
    assert sum(p.num_edges() for r in rg for p in r.parts) == g.num_edges()
    assert all(p.edge_range is not None and p.csc_slots_are_edge_ids for r in rg for p in r.parts)
    assert all(p.edge_range is None for r in rg_any for p in r.parts)
    part = rg[3].parts[0]  # type 2 -> type 0: 600 sources, 3000 destinations
    assert (part.num_src_nodes(), part.num_dst_nodes()) == (sizes[2], sizes[0])
    assert torch.equal(part.coo[0] + sizes[0] + sizes[1], rg[3].coo[0]) and torch.equal(part.coo[1], rg[3].coo[1])
    _bipartite_primitives_match_oracle(part, orc)
    torch.manual_seed(9)
    layer = HeteroHGTLayer(64, 64, 4, sizes, rg).cuda()
    h = torch.randn(g.num_nodes(), 64, device="cuda", requires_grad=True)
    out = layer(g, h)
    layer_any = HeteroHGTLayer(64, 64, 4, sizes, rg_any).cuda()
    layer_any.load_state_dict(layer.state_dict())
    # node outputs do not depend on the edge numbering (up to the softmax's fp32 summation order, which can move
    # an int8 attention value by one step here and there)
    out_any = layer_any(g_any, h)
    assert ((out_any - out).norm() / out.norm()).item() < 2e-3
    with torch.no_grad():
        ref = _fp32_hetero_hgt(layer, g, h)
    assert ((out - ref).norm() / ref.norm()).item() < 0.1
    out.square().mean().backward()
    assert bool(torch.isfinite(h.grad).all())
    for name, p in layer.named_parameters():
        assert p.grad is not None and float(p.grad.abs().sum()) > 0, name
    # the gradients track those of the fp32 math (int8 noise of the gradient quantizers on top of the forward's)
    h2 = h.detach().clone().requires_grad_(True)
    names, params = zip(*layer.named_parameters())
    want = torch.autograd.grad(_fp32_hetero_hgt(layer, g, h2).square().mean(), (h2,) + params)
    rel = lambda a, b: ((a - b).norm() / b.norm()).item()
    assert rel(h.grad, want[0]) < 0.15, rel(h.grad, want[0])
    for name, p, w in zip(names, params, want[1:]):
        assert rel(p.grad, w) < 0.25, (name, rel(p.grad, w))
    # relation 2 goes from type 1 to type 2: changing its message weights moves type-2 rows only
    with torch.no_grad():
        layer.msg_linear[2].weight.mul_(1.5)
        out2 = layer(g, h)
    changed = (out2 - out).abs().amax(1) > 0
    assert not bool(changed[:sizes[0] + sizes[1]].any()) and bool(changed[sizes[0] + sizes[1]:].any())


def test_arxiv_gat_stack_tracks_fp32_and_trains():
    """evaluation/arxiv_gat.py's stack (residual projection in every layer, batch norm, one-head output averaged,
    bias of its own, smoothed loss): forward within int8 noise of the fp32 math, loss falls under training."""
    import torch.nn.functional as F
    from tango_amd.evaluation import arxiv_loss
    from tango_amd.gat import ArxivGAT
    g = _small_graph(4000, 40000, 8)
    n = g.num_nodes()
    torch.manual_seed(5)
    model = ArxivGAT(64, 10, 32, 3, 3, F.relu, dropout=0.0, input_drop=0.0, attn_drop=0.0).cuda()
    x = torch.randn(n, 64, device="cuda")
    labels = torch.randint(0, 10, (n,), device="cuda")
    model.eval()
    out = model(g, x)
    assert out.shape == (n, 10)

    def fp32_conv(conv, h):
        H, D = conv._num_heads, conv._out_feats
        f = F.linear(h, conv.fc.weight).view(n, H, D)
        el, er = (f * conv.attn_l).sum(-1), (f * conv.attn_r).sum(-1)
        src, dst = g.coo
        e = F.leaky_relu(el[src] + er[dst], 0.2)
        mx = torch.full((n, H), -1e30, device=h.device).scatter_reduce_(0, dst.unsqueeze(1).expand(-1, H), e, "amax")
        ex = (e - mx[dst]).exp()
        a = ex / torch.zeros((n, H), device=h.device).index_add_(0, dst, ex)[dst]
        rst = torch.zeros((n, H, D), device=h.device).index_add_(0, dst, f[src] * a.unsqueeze(-1))
        return rst + F.linear(h, conv.res_fc.weight).view(n, H, D)
    with torch.no_grad():
        h = x
        for i, conv in enumerate(model.convs):
            h = fp32_conv(conv, h)
            if i < model.n_layers - 1:
                h = F.relu(model.norms[i](h.flatten(1)))
        ref = h.mean(1) + model.bias_last
    # three stacked layers of truncation-quantized GEMMs and int8 attention: 0.108 measured
    assert ((out - ref).norm() / ref.norm()).item() < 0.15
    model.train()
    opt = torch.optim.RMSprop(model.parameters(), lr=2e-3)
    losses = []
    for _ in range(12):
        loss = arxiv_loss(model(g, x), labels)
        opt.zero_grad()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert np.isfinite(losses).all() and losses[-1] < losses[0]


@pytest.mark.parametrize("which", ["gat", "hgt"])
def test_link_prediction_with_attention_models(which):
    """evaluation/link_pred_gat.py / link_pred_hgt.py: embeddings from the GAT stack (heads kept apart in the score)
    or one HGT layer, scored by sddmm_u_dot_v on the graph and on k sampled non-edges per edge."""
    from tango_amd import evaluation
    kw = dict(hidden=32, layers=2, k=2, dropout=0.0, quiet=True, model_name=which, heads=4)
    torch.manual_seed(21)
    _, first = evaluation.train_link_pred("pubmed", epochs=1, **kw)
    torch.manual_seed(21)
    ms, loss = evaluation.train_link_pred("pubmed", epochs=10, lr=5e-3, **kw)
    assert np.isfinite(ms) and ms > 0 and np.isfinite(loss) and loss < first


def test_arxiv_gcn_stack_trains():
    """evaluation/arxiv_gcn.py's QGCN (quantized linear skip branch per layer, batch norm) under its smoothed loss."""
    import torch.nn.functional as F
    from tango_amd.evaluation import arxiv_loss
    from tango_amd.gcn import ArxivGCN
    g = _small_graph(4000, 40000, 9)
    n = g.num_nodes()
    torch.manual_seed(6)
    model = ArxivGCN(64, 48, 10, 3, F.relu, 0.0, True).cuda()
    x = torch.randn(n, 64, device="cuda")
    labels = torch.randint(0, 10, (n,), device="cuda")
    opt = torch.optim.AdamW(model.parameters(), lr=5e-3)
    losses = []
    for _ in range(12):
        loss = arxiv_loss(model(g, x), labels)
        opt.zero_grad()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert np.isfinite(losses).all() and losses[-1] < losses[0]
