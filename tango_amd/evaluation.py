"""Drivers in the shape of the reference's evaluation scripts, on synthetic graphs.

The reference's drivers load Reddit / PubMed / ogbn-arxiv / DBLP / Amazon through DGL and OGB
(evaluation/util.py:10-32) and call a ``load_graph_train`` that its tree does not define
(evaluation/test_gcn.py:173, test_gat.py:238, test_HGT.py:72).  Neither library nor the datasets
exist here, so ``load_graph`` / ``load_graph_train`` return seeded Chung-Lu graphs with the named
dataset's node count, edge count, feature width and class count, random features and labels, and
the 60/20/20 masks the drivers index with.  The training loops time forward + backward per epoch
with events the way evaluation/test_gcn.py:241-263 does (the reference records its ``backward``
event before ``loss.backward()``; here it is recorded after).

    python -m tango_amd.evaluation --model gcn --dataset pubmed --epochs 20
    python -m tango_amd.evaluation --model linkpred --dataset pubmed --epochs 20   # evaluation/link_pred_gcn.py
"""
import argparse
import math

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

from .gat import GAT, HGT, ArxivGAT, HeteroHGTLayer, QGATConv, relation_graphs, relation_major
from .gcn import GCN, ArxivGCN
from .graph import Graph, add_self_loop, chung_lu, hetero_power_law, remove_self_loop
from .SDDMM import sddmm_u_dot_v
from .util import graph_preprocess

# name: (nodes, directed edges before self loops, degree exponent, largest degree or None,
#        symmetric as loaded by the reference, feature width, classes, generator seed)
DATASETS = {
    "pubmed": (19717, 177302, 2.1, None, True, 500, 3, 1),
    "ogbn-arxiv": (169343, 1166243, 2.2, None, False, 128, 40, 4),
    "reddit": (232965, 114600000, 2.0, 21000, True, 602, 41, 3),
    "dblp": (317080, 2099732, 2.3, None, True, 128, 16, 6),
    "amazon": (410236, 4878874, 2.3, None, True, 128, 16, 7),
}


def load_graph(name, device="cuda"):
    """evaluation/util.py:10-32: the graph with self loops removed and re-added, on the device,
    preprocessed.  Synthetic stand-in of the named dataset's size."""
    if name not in DATASETS:
        raise ValueError("Unknown dataset: {}".format(name))
    n, e, gamma, max_deg, sym, _, _, seed = DATASETS[name]
    g = chung_lu(n, e, gamma, seed=seed, max_degree=max_deg, symmetric=sym, device=device)
    return graph_preprocess(g)


def load_graph_train(name, device="cuda"):
    """The graph of ``load_graph`` with ``ndata`` feat / label / train_mask / val_mask / test_mask and
    ``n_classes``, the attributes the reference's training drivers read."""
    g = load_graph(name, device)
    n, (_, _, _, _, _, width, classes, seed) = g.num_nodes(), DATASETS[name]
    gen = torch.Generator().manual_seed(1000 + seed)
    g.ndata["feat"] = torch.randn(n, width, generator=gen).to(device)
    g.ndata["label"] = torch.randint(0, classes, (n,), generator=gen).to(device)
    r = torch.rand(n, generator=gen).to(device)
    g.ndata["train_mask"], g.ndata["val_mask"], g.ndata["test_mask"] = r < 0.6, (r >= 0.6) & (r < 0.8), r >= 0.8
    g.n_classes = classes
    return g


ARXIV_EPSILON = 1 - math.log(2)  # evaluation/arxiv_gat.py:451


def arxiv_loss(x, labels):
    """The log-smoothed cross entropy of evaluation/arxiv_gat.py:528-531 and arxiv_gcn.py:224-227."""
    y = F.cross_entropy(x, labels, reduction="none")
    return torch.mean(torch.log(ARXIV_EPSILON + y) - math.log(ARXIV_EPSILON))


def add_labels(feat, labels, idx, n_classes):
    """``feat`` widened by ``n_classes`` columns that hold the one-hot labels of the nodes ``idx`` and zeros for all
    others: the label-reuse input of evaluation/arxiv_gat.py:534-537 and arxiv_gcn.py:234-237."""
    onehot = feat.new_zeros(feat.size(0), n_classes)
    onehot[idx, labels[idx]] = 1
    return torch.cat([feat, onehot], dim=-1)


def warm_up_lr(optimizer, lr, epoch, span=50):
    """The learning rate of epoch 1, 2, ... climbs linearly to ``lr`` over the first ``span`` epochs
    (evaluation/arxiv_gat.py:540-543, called at the top of every epoch, :655)."""
    if epoch <= span:
        for group in optimizer.param_groups:
            group["lr"] = lr * epoch / span


def train_arxiv(model_name="gat", epochs=20, n_hidden=None, n_layers=3, n_heads=3, lr=2e-3, dropout=0.75,
                input_drop=0.1, attn_drop=0.05, edge_drop=0.0, use_linear=True, dataset="ogbn-arxiv", quiet=False,
                use_labels=False, mask_rate=0.5, n_label_iters=0, warm_up=True):
    """evaluation/arxiv_gat.py:546-590 / arxiv_gcn.py:246-281 (``train``) on the synthetic stand-in of
    ogbn-arxiv: the GAT or GCN stack of those scripts, the smoothed loss, RMSprop for the GAT (arxiv_gat.py:603)
    and AdamW for the GCN (arxiv_gcn.py:311), the learning-rate warm-up of the scripts' epoch loops, and their
    per-epoch random split of the training nodes: with ``use_labels`` the nodes drawn with probability ``mask_rate``
    feed their labels in as extra input columns and the loss is taken on the others, without it the loss is
    taken on the drawn nodes.  ``n_label_iters`` (needs ``use_labels``, arxiv_gat.py:794-796) repeats the forward
    pass that many times with the softmax of the previous prediction written into the label columns of every
    node whose label is not an input (arxiv_gat.py:572-578); only the last pass is differentiated.  Returns
    (mean ms per epoch after the first three, final loss)."""
    if n_label_iters > 0 and not use_labels:
        raise ValueError("n_label_iters > 0 needs use_labels")
    g = load_graph_train(dataset)
    feats, labels = g.ndata["feat"], g.ndata["label"]
    train_idx = g.ndata["train_mask"].nonzero().squeeze(1)
    rest_idx = (~g.ndata["train_mask"]).nonzero().squeeze(1)  # the scripts' validation and test nodes
    classes = g.n_classes
    width = feats.size(1) + (classes if use_labels else 0)
    if model_name == "gat":
        model = ArxivGAT(width, classes, n_hidden or 250, n_layers, n_heads, F.relu, dropout=dropout,
                         input_drop=input_drop, attn_drop=attn_drop, edge_drop=edge_drop).cuda()
        opt = torch.optim.RMSprop(model.parameters(), lr=lr, weight_decay=0)
    elif model_name == "gcn":
        model = ArxivGCN(width, n_hidden or 256, classes, n_layers, F.relu, min(dropout, 0.5), use_linear).cuda()
        opt = torch.optim.AdamW(model.parameters(), lr=lr, weight_decay=0)
    else:
        raise ValueError("model must be gat or gcn")
    dur, loss = [], None
    for epoch in range(1, epochs + 1):
        if warm_up:
            warm_up_lr(opt, lr, epoch)
        model.train()
        drawn = torch.rand(train_idx.shape, device=train_idx.device) < mask_rate
        if use_labels:
            x, pred_idx = add_labels(feats, labels, train_idx[drawn], classes), train_idx[~drawn]
        else:
            x, pred_idx = feats, train_idx[drawn]
        opt.zero_grad()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        pred = model(g, x)
        if n_label_iters > 0:
            unlabelled = torch.cat([pred_idx, rest_idx])
            for _ in range(n_label_iters):
                pred = pred.detach()
                x[unlabelled, -classes:] = F.softmax(pred[unlabelled], dim=-1)
                pred = model(g, x)
        loss = arxiv_loss(pred[pred_idx], labels[pred_idx])
        loss.backward()
        stop.record()
        torch.cuda.synchronize()
        opt.step()
        if epoch > 3:
            dur.append(start.elapsed_time(stop))
        if not quiet:
            print("Epoch {:05d} | Time(ms) {:.4f} | Loss {:.4f}".format(epoch, np.mean(dur) if dur else float("nan"),
                                                                        loss.item()))
    return (float(np.mean(dur)) if dur else math.nan), float(loss.item())


def train_hetero_hgt(epochs=10, hidden=256, heads=4, n_classes=16, lr=1e-3, quiet=False, **graph_kw):
    """Two heterogeneous HGT layers (weights per node type and per relation) with a linear read-out on the
    synthetic 3-type / 4-relation graph.  Returns (mean forward + backward ms per epoch after the first three,
    final loss)."""
    type_sizes = graph_kw.pop("type_sizes", (100_000, 50_000, 20_000))
    relations = graph_kw.pop("relations", ((0, 1), (1, 0), (1, 2), (2, 0)))
    g, _, edge_type = hetero_power_law(type_sizes=type_sizes, relations=relations, device="cuda", **graph_kw)
    g, edge_type = relation_major(g, edge_type)
    g = graph_preprocess(g)
    rels = relation_graphs(g, edge_type, relations, type_sizes)
    n = g.num_nodes()
    layers = nn.ModuleList([HeteroHGTLayer(hidden, hidden, heads, type_sizes, rels) for _ in range(2)]).cuda()
    proj = nn.Linear(hidden, n_classes).cuda()
    gen = torch.Generator().manual_seed(77)
    x = torch.randn(n, hidden, generator=gen).cuda()
    labels = torch.randint(0, n_classes, (n,), generator=gen).cuda()
    opt = torch.optim.Adam(list(layers.parameters()) + list(proj.parameters()), lr=lr)
    dur, loss = [], None
    for epoch in range(epochs):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        h = x
        for layer in layers:
            h = layer(g, h)
        loss = F.cross_entropy(proj(h), labels)
        opt.zero_grad()
        loss.backward()
        stop.record()
        torch.cuda.synchronize()
        opt.step()
        if epoch >= 3:
            dur.append(start.elapsed_time(stop))
        if not quiet:
            print("Epoch {:05d} | Time(ms) {:.4f} | Loss {:.4f}".format(epoch, np.mean(dur) if dur else float("nan"),
                                                                        loss.item()))
    return (float(np.mean(dur)) if dur else math.nan), float(loss.item())


def evaluate(model_fn, labels, mask):
    """evaluation/test_gcn.py:172-181."""
    with torch.no_grad():
        logits = model_fn()[mask]
        return (logits.argmax(1) == labels[mask]).float().mean().item()


def train(model_name, dataset, epochs=20, hidden=None, layers=None, heads=8, lr=1e-2, weight_decay=5e-4,
          quiet=False):
    """One of the reference's three training drivers (test_gcn.py:183-275, test_gat.py:236-330,
    test_HGT.py:70-130).  Returns (mean ms per epoch after the first three, final loss)."""
    g = load_graph_train(dataset)
    feats, labels, train_mask = g.ndata["feat"], g.ndata["label"], g.ndata["train_mask"]
    if model_name == "gcn":
        hidden, layers = hidden or 256, layers or 1
        model = GCN(g, feats.size(1), hidden, hidden, layers, torch.relu, 0.0).cuda()
        fwd = lambda: model(feats)
    elif model_name == "gat":
        hidden, layers = hidden or 16, layers or 3
        model = GAT(g, layers, feats.size(1), hidden, g.n_classes, [heads] * (layers - 1) + [1], F.elu).cuda()
        fwd = lambda: model(feats)
    elif model_name == "hgt":
        hidden = hidden or 256
        model = HGT(feats.size(1), hidden, heads).cuda()
        fwd = lambda: model(g, feats)
    else:
        raise ValueError("model must be gcn, gat or hgt")
    proj = nn.Linear(hidden, g.n_classes).cuda()  # "proj to predict" (test_gcn.py:229)
    opt = torch.optim.Adam(list(model.parameters()) + list(proj.parameters()), lr=lr, weight_decay=weight_decay)
    dur, loss = [], None
    for epoch in range(epochs):
        model.train()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        logits = proj(fwd())
        loss = F.cross_entropy(logits[train_mask], labels[train_mask])
        opt.zero_grad()
        loss.backward()
        stop.record()
        torch.cuda.synchronize()
        opt.step()
        if epoch >= 3:
            dur.append(start.elapsed_time(stop))
        if not quiet:
            acc = evaluate(lambda: proj(fwd()), labels, g.ndata["val_mask"])
            print("Epoch {:05d} | Time(ms) {:.4f} | Loss {:.4f} | Accuracy {:.4f} | ETputs(KTEPS) {:.2f}".format(
                epoch, np.mean(dur) if dur else float("nan"), loss.item(), acc,
                g.num_edges() / np.mean(dur) if dur else float("nan")))
    return (float(np.mean(dur)) if dur else math.nan), float(loss.item())


def construct_negative_graph(g, k):
    """evaluation/link_pred_gcn.py:164-169: k random destinations per source of every edge.  Built and
    preprocessed (CSR / CSC / incidence, all on the device) once per epoch."""
    src, _ = g.edges()
    neg_src = src.repeat_interleave(k)
    neg_dst = torch.randint(0, g.num_nodes(), (neg_src.numel(),), device=src.device)
    return graph_preprocess(Graph(neg_src, neg_dst, g.num_nodes()))


class _LinkPredGAT(nn.Module):
    """evaluation/link_pred_gat.py:172-221: the GAT stack whose last layer keeps its heads ([n, heads, hidden])
    as the node embedding that scores the edges."""

    def __init__(self, num_layers, in_dim, num_hidden, heads, activation, feat_drop=0.0, attn_drop=0.0,
                 negative_slope=0.2, residual=False):
        super().__init__()
        self.num_layers = num_layers
        self.gat_layers = nn.ModuleList()
        if num_layers > 1:
            self.gat_layers.append(QGATConv(in_dim, num_hidden, heads[0], feat_drop, attn_drop, negative_slope,
                                            False, activation))
            for l in range(1, num_layers - 1):
                self.gat_layers.append(QGATConv(num_hidden * heads[l - 1], num_hidden, heads[l], feat_drop, attn_drop,
                                                negative_slope, residual, activation))
            self.gat_layers.append(QGATConv(num_hidden * heads[-2], num_hidden, heads[-1], feat_drop, attn_drop,
                                            negative_slope, residual, None))
        else:
            self.gat_layers.append(QGATConv(in_dim, num_hidden, heads[0], feat_drop, attn_drop, negative_slope,
                                            residual, None))

    def forward(self, g, inputs):
        h = inputs
        for l in range(self.num_layers - 1):
            h = self.gat_layers[l](g, h).flatten(1)
        return self.gat_layers[-1](g, h)  # [n, heads, hidden]


def train_link_pred(dataset, epochs=20, hidden=256, layers=4, k=8, lr=1e-2, weight_decay=5e-4, dropout=0.5,
                    edge_fraction=None, quiet=False, model_name="gcn", heads=4):
    """The reference's link prediction drivers (evaluation/link_pred_gcn.py:137-153,172-264, link_pred_gat.py:
    172-230, link_pred_hgt.py:27-89): a quantized GCN, GAT or HGT layer embeds the nodes, sddmm_u_dot_v scores the
    graph's edges and k sampled non-edges per edge, binary cross entropy separates the two.  The negative graph is rebuilt every epoch outside the timed region, as there.
    ``edge_fraction``: train on a random subset of the edges (the reference keeps 8 % of Reddit's).
    Returns (mean forward + backward ms per epoch after the first three, final loss)."""
    n, e, gamma, max_deg, sym, width, _, seed = DATASETS[dataset]
    g = chung_lu(n, e, gamma, seed=seed, max_degree=max_deg, symmetric=sym, device="cuda")
    if edge_fraction is None:
        edge_fraction = 0.08 if dataset == "reddit" else 1.0
    src, dst = g.edges()
    if edge_fraction < 1.0:
        keep = torch.randperm(src.numel(), device=src.device)[:int(src.numel() * edge_fraction)]
        src, dst = src[keep], dst[keep]
    g = graph_preprocess(Graph(*add_self_loop(*remove_self_loop(src, dst), n), n))  # link_pred_gcn.py:213-216
    width -= width % 4  # "trim features to fit in k%4" (link_pred_gcn.py:206-208)
    feats = torch.randn(n, width, generator=torch.Generator().manual_seed(1000 + seed)).cuda()
    if model_name == "gcn":
        model = GCN(g, width, hidden, hidden, layers, torch.relu, dropout).cuda()
        embed = lambda: model(feats).unsqueeze(1)
    elif model_name == "gat":  # link_pred_gat.py:172-221; heads of the last layer stay separate in the score
        model = _LinkPredGAT(layers, width, hidden, [heads] * layers, F.elu).cuda()
        embed = lambda: model(g, feats)
    elif model_name == "hgt":  # link_pred_hgt.py:27-75: one layer, its output as a one-head embedding
        model = HGT(width, hidden, heads).cuda()
        embed = lambda: model(g, feats).unsqueeze(1)
    else:
        raise ValueError("model must be gcn, gat or hgt")
    opt = torch.optim.Adam(model.parameters(), lr=lr, weight_decay=weight_decay)
    dur, loss = [], None
    for epoch in range(epochs):
        model.train()
        neg = construct_negative_graph(g, k)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        h = embed()
        pos_score = sddmm_u_dot_v.apply(g, h, h)
        neg_score = sddmm_u_dot_v.apply(neg, h, h)
        score = torch.cat([pos_score, neg_score])
        label = torch.cat([torch.ones_like(pos_score), torch.zeros_like(neg_score)])
        loss = F.binary_cross_entropy_with_logits(score, label)
        opt.zero_grad()
        loss.backward()
        stop.record()
        torch.cuda.synchronize()
        opt.step()
        if epoch >= 3:
            dur.append(start.elapsed_time(stop))
        if not quiet:
            print("Epoch {:05d} | Time(ms) {:.4f} | Loss {:.4f} | ETputs(KTEPS) {:.2f}".format(
                epoch, np.mean(dur) if dur else float("nan"), loss.item(),
                g.num_edges() / np.mean(dur) if dur else float("nan")))
    return (float(np.mean(dur)) if dur else math.nan), float(loss.item())


def main():
    ap = argparse.ArgumentParser(description="quantized GCN / GAT / HGT training on a synthetic stand-in of a dataset")
    ap.add_argument("--model", choices=["gcn", "gat", "hgt", "linkpred", "linkpred-gat", "linkpred-hgt", "arxiv-gat",
                                        "arxiv-gcn", "hetero-hgt"], default="gcn")
    ap.add_argument("--k", type=int, default=8, help="negative samples per edge (linkpred)")
    ap.add_argument("--dataset", choices=sorted(DATASETS), default="pubmed")
    ap.add_argument("--epochs", type=int, default=20)
    ap.add_argument("--n-hidden", type=int, default=None)
    ap.add_argument("--n-layers", type=int, default=None)
    ap.add_argument("--num-heads", type=int, default=8)
    ap.add_argument("--lr", type=float, default=1e-2)
    ap.add_argument("--weight-decay", type=float, default=5e-4)
    ap.add_argument("--use-labels", action="store_true", help="arxiv models: feed training labels in as input columns")
    ap.add_argument("--n-label-iters", type=int, default=0, help="arxiv models: refinement passes (needs --use-labels)")
    ap.add_argument("--mask-rate", type=float, default=0.5, help="arxiv models: share of training nodes drawn per epoch")
    ap.add_argument("--edge-drop", type=float, default=0.0, help="arxiv-gat: share of edges dropped per layer and epoch")
    args = ap.parse_args()
    if args.model.startswith("linkpred"):
        which = args.model.partition("-")[2] or "gcn"
        ms, loss = train_link_pred(args.dataset, args.epochs, args.n_hidden or (256 if which != "gat" else 64),
                                   args.n_layers or (4 if which == "gcn" else 2), args.k, args.lr, args.weight_decay,
                                   model_name=which, heads=min(args.num_heads, 4))
    elif args.model.startswith("arxiv"):
        ms, loss = train_arxiv(args.model.partition("-")[2], args.epochs, args.n_hidden, args.n_layers or 3,
                               edge_drop=args.edge_drop, use_labels=args.use_labels, mask_rate=args.mask_rate,
                               n_label_iters=args.n_label_iters)
    elif args.model == "hetero-hgt":
        ms, loss = train_hetero_hgt(args.epochs, args.n_hidden or 256, min(args.num_heads, 4))
    else:
        ms, loss = train(args.model, args.dataset, args.epochs, args.n_hidden, args.n_layers, args.num_heads, args.lr,
                         args.weight_decay)
    print("mean fwd+bwd {:.3f} ms/epoch, final loss {:.4f}".format(ms, loss))


if __name__ == "__main__":
    main()
