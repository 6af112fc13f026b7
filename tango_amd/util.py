"""Graph preprocessing: mirrors cuda/util.py of the reference."""
import torch

from .graph import Graph


def graph_preprocess(graph, dense_blocks=True):
    """Materialise CSR/CSC/COO/incidence once and cache them on the graph
    (cuda/util.py:5-11).  Accepts a ``tango_amd.graph.Graph`` or any object
    with DGL's ``inc`` / ``adj_sparse`` / ``edges`` methods.  ``dense_blocks``: on graphs
    averaging 64 or more edges per node also split both orientations into dense bit blocks and
    a sparse rest (``dense_plan.build_dense_plan``), which the copy_u aggregation then uses."""
    if isinstance(graph, Graph):
        graph.inc_in = graph.incidence("in")
        graph.inc_out = graph.incidence("out")
    else:
        graph.inc_in = graph.inc("in", ctx=graph.device).coalesce().indices()
        graph.inc_out = graph.inc("out", ctx=graph.device).coalesce().indices()
    assert graph.inc_in.is_cuda, "graph must be on GPU"
    graph.adj_csr = graph.adj_sparse("csr")
    graph.adj_csc = graph.adj_sparse("csc")
    graph.coo = graph.edges()
    # One-time 32-bit copies of the column indices and edge ids (node and edge counts are below
    # 2^31 wherever the kernels run): the aggregation kernels stream these arrays once per launch,
    # and at 4 bytes per edge they cost half the traffic of the int64 arrays the reference passes.
    graph.adj_csr32 = tuple(t.to(torch.int32) for t in graph.adj_csr[1:])
    graph.adj_csc32 = tuple(t.to(torch.int32) for t in graph.adj_csc[1:])
    # whether a CSR's slot order is the edge-id order itself (edges already sorted by that endpoint, e.g.
    # after Graph.reorder_edges_by_dst): the kernels then skip the slot -> edge-id indirection altogether
    ar = torch.arange(graph.adj_csr[2].numel(), device=graph.adj_csr[2].device)
    graph.csr_slots_are_edge_ids = bool(torch.equal(graph.adj_csr[2], ar))
    graph.csc_slots_are_edge_ids = bool(torch.equal(graph.adj_csc[2], ar))
    del ar
    # the longest row of either orientation (one host read per graph): tells the aggregation
    # kernels whether the launches that exist for hub rows are needed at all
    graph.max_out_degree = int(torch.diff(graph.adj_csr[0]).max().item()) if graph.adj_csr[0].numel() > 1 else 0
    graph.max_in_degree = int(torch.diff(graph.adj_csc[0]).max().item()) if graph.adj_csc[0].numel() > 1 else 0
    graph.dense_csr = graph.dense_csc = None
    nnz = graph.adj_csr[1].numel()
    if dense_blocks and nnz >= (1 << 22):
        from .dense_plan import build_dense_plan
        for name, (indptr, _, _), narrow in (("dense_csr", graph.adj_csr, graph.adj_csr32),
                                             ("dense_csc", graph.adj_csc, graph.adj_csc32)):
            rows = indptr.numel() - 1
            if nnz >= 64 * rows:
                num_src = graph.num_dst_nodes() if name == "dense_csr" else graph.num_src_nodes()
                setattr(graph, name, build_dense_plan(indptr, narrow[0], num_src))
    return graph
