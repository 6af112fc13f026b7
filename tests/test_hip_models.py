"""GPU tests of the GAT / HGT layer harness: forward and gradients track an fp32
torch implementation of the same math within int8 quantization error."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def rel_err(a, b):
    return (a - b).norm().item() / max(b.norm().item(), 1e-30)


def softmax_dst(e, dst, n):
    mx = torch.full((n,) + e.shape[1:], -1e30, device=e.device).scatter_reduce(
        0, dst.view(-1, *([1] * (e.dim() - 1))).expand_as(e), e, "amax")
    ex = torch.exp(e - mx[dst])
    return ex / torch.zeros((n,) + e.shape[1:], device=e.device).index_add(0, dst, ex)[dst]


@pytest.fixture(scope="module")
def graph():
    from tango_amd.graph import chung_lu
    from tango_amd.util import graph_preprocess
    return graph_preprocess(chung_lu(3000, 30000, 2.2, seed=4, device="cuda"))


def test_gat_layer_tracks_fp32(graph):
    from tango_amd.gat import QGATConv
    g = graph
    n, H, D = g.num_nodes(), 8, 16
    torch.manual_seed(0)
    layer = QGATConv(96, D, H, residual=True, activation=None).cuda()
    x = torch.randn(n, 96, device="cuda", requires_grad=True)
    out, attn = layer(g, x, get_attention=True)
    assert tuple(out.shape) == (n, H, D) and tuple(attn.shape) == (g.num_edges(), H, 1)
    src, dst = g.coo
    sums = torch.zeros(n, H, 1, device="cuda").index_add(0, dst, attn)
    assert torch.allclose(sums, torch.ones_like(sums), atol=1e-5)
    # fp32 reference of the same layer
    xr = x.detach().clone().requires_grad_(True)
    fs = torch.nn.functional.linear(xr, layer.fc.weight).view(n, H, D)
    el = (fs * layer.attn_l).sum(-1, keepdim=True)
    er = (fs * layer.attn_r).sum(-1, keepdim=True)
    a = softmax_dst(torch.nn.functional.leaky_relu(el[src] + er[dst], 0.2), dst, n)
    ref = torch.zeros(n, H, D, device="cuda").index_add(0, dst, fs[src] * a)
    ref = ref + torch.nn.functional.linear(xr, layer.res_fc.weight).view(n, H, D) + layer.bias.view(1, H, D)
    assert rel_err(out.detach(), ref.detach()) < 0.06
    w = torch.randn_like(out)
    out.backward(w)
    gq = [p.grad.clone() for p in layer.parameters()] + [x.grad.clone()]
    layer.zero_grad()
    ref.backward(w)
    gr = [p.grad.clone() for p in layer.parameters()] + [xr.grad]
    names = [k for k, _ in layer.named_parameters()] + ["x"]
    # gradients that pass through the int8-quantized attention logits (attn_l / attn_r) carry the
    # per-tensor quantization noise of a heavy-tailed tensor; direction must agree, magnitude roughly
    cos = {k: round(torch.nn.functional.cosine_similarity(a_.flatten(), b_.flatten(), dim=0).item(), 4)
           for k, a_, b_ in zip(names, gq, gr)}
    errs = {k: round(rel_err(a_, b_), 4) for k, a_, b_ in zip(names, gq, gr)}
    assert all(v > 0.93 for v in cos.values()), (cos, errs)
    assert all(errs[k] < 0.2 for k in ("fc.weight", "res_fc.weight", "bias", "x")), errs


def test_hgt_layer_runs_and_tracks_fp32(graph):
    from tango_amd.gat import HGTLayer
    g = graph
    n = g.num_nodes()
    torch.manual_seed(1)
    layer = HGTLayer(64, 64, 4).cuda()
    x = torch.randn(n, 64, device="cuda", requires_grad=True)
    out = layer(g, x)
    assert tuple(out.shape) == (n, 64) and torch.isfinite(out).all()
    src, dst = g.coo
    lin = torch.nn.functional.linear
    xr = x.detach().clone().requires_grad_(True)
    k = lin(lin(xr, layer.k_linear.weight, layer.k_linear.bias), layer.attn_linear.weight, layer.attn_linear.bias).view(n, 4, 16)
    v = lin(lin(xr, layer.v_linear.weight, layer.v_linear.bias), layer.msg_linear.weight, layer.msg_linear.bias).view(n, 4, 16)
    q = lin(xr, layer.q_linear.weight, layer.q_linear.bias).view(n, 4, 16)
    t = (k[src] * q[dst]).sum(-1, keepdim=True) / 4.0
    a = softmax_dst(t, dst, n)
    ref = lin(torch.zeros(n, 4, 16, device="cuda").index_add(0, dst, v[src] * a).reshape(n, 64),
              layer.a_linear.weight, layer.a_linear.bias)
    assert rel_err(out.detach(), ref.detach()) < 0.1
    out.sum().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in layer.parameters())
    assert torch.isfinite(x.grad).all()


def test_gat_three_layers_trains(graph):
    """The 3-layer GAT of evaluation/test_gat.py:170-214 (hidden 16 x 8 heads) steps and its loss falls."""
    from tango_amd.gat import GAT
    from tango_amd.loss import cross_entropy
    g = graph
    n = g.num_nodes()
    torch.manual_seed(2)
    model = GAT(g, 3, 128, 16, 16, [8, 8, 1], torch.nn.functional.elu, residual=True).cuda()
    x = torch.randn(n, 128, device="cuda")
    labels = torch.randint(0, 16, (n,), device="cuda")
    opt = torch.optim.Adam(model.parameters(), lr=5e-3)
    losses = []
    for _ in range(12):
        opt.zero_grad()
        logits = model(x)
        assert tuple(logits.shape) == (n, 16)
        loss = cross_entropy(logits, labels)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert all(np.isfinite(losses)) and losses[-1] < losses[0] - 0.05, losses


def test_hgt_stack_on_heterogeneous_graph():
    """Two HGT layers on a small synthetic 3-type / 4-relation graph, homogenised as the reference's driver does."""
    from tango_amd.gat import HGTStack
    from tango_amd.graph import hetero_power_law
    from tango_amd.util import graph_preprocess
    g, ntype, etype = hetero_power_law((3000, 1500, 600), edges_per_relation=20000, seed0=50, device="cuda")
    g = graph_preprocess(g)
    n = g.num_nodes()
    assert n == 5100 and ntype.numel() == n and etype.numel() == g.num_edges()
    src, dst = g.coo
    rel = ((0, 1), (1, 0), (1, 2), (2, 0))
    for r, (a, b) in enumerate(rel):
        m = etype == r
        assert int(m.sum()) == 20000
        assert bool((ntype[src[m]] == a).all()) and bool((ntype[dst[m]] == b).all())
    assert bool((g.in_degrees() > 0).all())
    torch.manual_seed(3)
    model = HGTStack(256, 256, 8, 4, n_layers=2).cuda()
    x = torch.randn(n, 256, device="cuda")
    labels = torch.randint(0, 8, (n,), device="cuda")
    opt = torch.optim.Adam(model.parameters(), lr=2e-3)
    losses = []
    for _ in range(8):
        opt.zero_grad()
        loss = torch.nn.functional.cross_entropy(model(g, x), labels)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert all(np.isfinite(losses)) and losses[-1] < losses[0], losses


def test_hgt_layers_hand_their_output_scale_on(graph):
    """Between HGT layers the output GEMM's epilogue supplies the next layer's input scale: same bits as the
    absmax pass the next layer would run itself."""
    from tango_amd.gat import HGTStack
    g = graph
    torch.manual_seed(21)
    model = HGTStack(64, 64, 5, 4, n_layers=3).cuda()
    x = torch.randn(g.num_nodes(), 64, device="cuda")
    with torch.no_grad():
        got = model(g, x)
        h = x
        for layer in model.layers:
            h = layer(g, h)
        want = model.proj(h)
    assert torch.equal(got, want)


def test_edge_renumbering_leaves_node_outputs_unchanged():
    """Destination-major edge numbering (Graph.reorder_edges_by_dst) is an internal matter of the
    attention layers: same node outputs and parameter gradients, attention values permuted."""
    from tango_amd.gat import QGATConv
    from tango_amd.graph import chung_lu
    from tango_amd.util import graph_preprocess
    g0 = chung_lu(3000, 30000, 2.2, seed=4, device="cuda")
    g1 = g0.reorder_edges_by_dst()
    assert bool((g1.adj_sparse("csc")[2] == torch.arange(g1.num_edges(), device="cuda")).all())
    g0, g1 = graph_preprocess(g0), graph_preprocess(g1)
    torch.manual_seed(9)
    layer = QGATConv(64, 16, 8).cuda()
    x = torch.randn(g0.num_nodes(), 64, device="cuda")
    outs, grads, att = [], [], []
    for g in (g0, g1):
        layer.zero_grad()
        rst, a = layer(g, x, get_attention=True)
        rst.square().sum().backward()
        outs.append(rst.detach().clone())
        att.append(a.detach().clone())
        grads.append([p.grad.detach().clone() for p in layer.parameters()])
    assert torch.allclose(outs[0], outs[1], rtol=1e-5, atol=1e-6)
    assert torch.allclose(att[0][g1.edge_order], att[1], rtol=1e-5, atol=1e-7)
    for a, b in zip(*grads):
        assert torch.allclose(a, b, rtol=1e-3, atol=1e-4 * float(a.abs().max()))


@pytest.mark.parametrize("model", ["gcn", "gat", "hgt"])
def test_evaluation_drivers_train_on_the_pubmed_stand_in(model):
    """tango_amd.evaluation: the reference's three training loops (evaluation/test_gcn.py,
    test_gat.py, test_HGT.py) on the synthetic graph with PubMed's sizes."""
    from tango_amd import evaluation
    torch.manual_seed(11)
    g = evaluation.load_graph_train("pubmed")
    assert g.num_nodes() == 19717 and g.ndata["feat"].shape == (19717, 500) and g.n_classes == 3
    assert int(g.ndata["train_mask"].sum() + g.ndata["val_mask"].sum() + g.ndata["test_mask"].sum()) == 19717
    first_ms, first_loss = evaluation.train(model, "pubmed", epochs=1, quiet=True)
    torch.manual_seed(11)
    ms, loss = evaluation.train(model, "pubmed", epochs=12, quiet=True, lr=5e-3)
    assert np.isfinite(ms) and ms > 0 and np.isfinite(loss) and loss < first_loss


@pytest.mark.parametrize("model,kw", [("gat", {"use_labels": True, "n_label_iters": 1, "mask_rate": 0.5}),
                                      ("gat", {"edge_drop": 0.2}), ("gcn", {"use_labels": True}), ("gcn", {})])
def test_arxiv_drivers_train_with_label_reuse_and_warm_up(model, kw):
    """tango_amd.evaluation.train_arxiv: the loops of evaluation/arxiv_gat.py:546-590 and arxiv_gcn.py:246-281 with
    their learning-rate warm-up, the per-epoch split of the training nodes, labels fed back in as input columns
    and one refinement pass over the unlabelled nodes, on the small stand-in graph."""
    from tango_amd import evaluation
    common = dict(dataset="pubmed", n_hidden=32, n_layers=2, n_heads=2, dropout=0.1, input_drop=0.0, attn_drop=0.0,
                  quiet=True, lr=2e-2)
    torch.manual_seed(17)
    _, first = evaluation.train_arxiv(model, epochs=1, warm_up=False, **common, **kw)
    torch.manual_seed(17)
    ms, loss = evaluation.train_arxiv(model, epochs=25, **common, **kw)
    assert np.isfinite(ms) and ms > 0 and np.isfinite(loss) and loss < first
    with pytest.raises(ValueError):
        evaluation.train_arxiv(model, epochs=1, n_label_iters=1, **common)


def test_link_prediction_driver_trains_on_the_pubmed_stand_in():
    """tango_amd.evaluation.train_link_pred: the reference's evaluation/link_pred_gcn.py loop (GCN embeddings,
    sddmm_u_dot_v scores of edges and of k sampled non-edges, a negative graph built on the device per epoch)."""
    from tango_amd import evaluation
    torch.manual_seed(13)
    _, first = evaluation.train_link_pred("pubmed", epochs=1, hidden=64, layers=2, k=2, dropout=0.0, quiet=True)
    torch.manual_seed(13)
    ms, loss = evaluation.train_link_pred("pubmed", epochs=10, hidden=64, layers=2, k=2, dropout=0.0, lr=5e-3, quiet=True)
    assert np.isfinite(ms) and ms > 0 and np.isfinite(loss) and loss < first


@pytest.mark.parametrize("model_name", ["gcn", "gat"])
def test_inference_forward_replays_from_a_hip_graph(model_name, graph):
    """The entry points launch kernels only (no memset, no host sync, scratch from the caller), so an
    inference forward can be captured once and replayed.  Every replay is checked against the eager
    result, with eager work and synchronizations between the replays."""
    from tango_amd.gat import GAT
    from tango_amd.gcn import GCN
    g = graph
    n = g.num_nodes()
    torch.manual_seed(5)
    if model_name == "gcn":
        model = GCN(g, 64, 32, 8, 1, torch.relu, 0.0).cuda().eval()
    else:
        model = GAT(g, 2, 64, 8, 8, [4, 1], torch.nn.functional.elu).cuda().eval()
        model(torch.randn(n, 64, device="cuda"))  # answers the one-time zero-in-degree question outside the capture
    static_x = torch.randn(n, 64, device="cuda")
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                model(static_x)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_y = model(static_x)
        for k in range(4):
            x = torch.randn(n, 64, device="cuda") * (k + 1)
            want = model(x)            # eager work between the replays
            torch.cuda.synchronize()
            static_x.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y, want), k
