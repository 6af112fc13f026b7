"""Graph preprocessing: mirrors cuda/util.py of the reference."""
from .graph import Graph


def graph_preprocess(graph):
    """Materialise CSR/CSC/COO/incidence once and cache them on the graph
    (cuda/util.py:5-11).  Accepts a ``tango_amd.graph.Graph`` or any object
    with DGL's ``inc`` / ``adj_sparse`` / ``edges`` methods."""
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
    return graph
