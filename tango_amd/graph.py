"""A DGL-free graph object carrying exactly what the primitive layer reads.

The reference's wrappers touch five cached attributes of a DGL graph plus
``num_nodes()`` (cuda/kernels.py:35-37,128-130,142-148,156-160); the model
code additionally reads degrees and uses ``local_scope`` and the feature
dictionaries.  ``Graph`` offers that surface on torch tensors, and
``chung_lu`` generates the seeded synthetic power-law graphs the benchmarks
run on (the reference's datasets are fetched from the network).
"""
import contextlib

import torch


def _compress(rows, cols, num_nodes):
    """COO -> (indptr, indices, edge_ids) with rows sorted stably (edge-id order within a row)."""
    order = torch.sort(rows, stable=True).indices
    counts = torch.bincount(rows, minlength=num_nodes)
    indptr = torch.zeros(num_nodes + 1, dtype=torch.int64, device=rows.device)
    torch.cumsum(counts, 0, out=indptr[1:])
    return indptr, cols[order].contiguous(), order.contiguous()


class Graph:
    """Homogeneous directed multigraph on ``num_nodes`` nodes; edge e is (src[e], dst[e]).  With ``num_dst``
    the graph is bipartite: sources are numbered 0 .. num_nodes - 1, destinations 0 .. num_dst - 1 in a space
    of their own (one relation of a heterogeneous graph, each endpoint numbered inside its node type)."""

    is_block = False

    def __init__(self, src, dst, num_nodes, num_dst=None):
        self._src = src.to(torch.int64).contiguous()
        self._dst = dst.to(torch.int64).contiguous()
        self._n = int(num_nodes)
        self._n_dst = self._n if num_dst is None else int(num_dst)
        self.ndata, self.edata = {}, {}
        self.srcdata = self.dstdata = self.ndata
        self._csr = self._csc = None
        self._in_deg = self._out_deg = None

    # -- the DGL calls of cuda/util.py:5-11 ---------------------------------
    @property
    def device(self):
        return self._src.device

    def to(self, device):
        g = Graph(self._src.to(device), self._dst.to(device), self._n, self._n_dst)
        return g

    def num_nodes(self):
        if self._n_dst != self._n:
            raise ValueError("bipartite graph: ask for num_src_nodes() or num_dst_nodes()")
        return self._n

    def num_src_nodes(self):
        return self._n

    def num_dst_nodes(self):
        return self._n_dst

    number_of_nodes = num_nodes
    number_of_src_nodes = num_src_nodes
    number_of_dst_nodes = num_dst_nodes

    def num_edges(self):
        return self._src.numel()

    number_of_edges = num_edges

    def edges(self):
        return self._src, self._dst

    def adj_sparse(self, fmt):
        """'csr': rows = source nodes; 'csc': rows = destination nodes."""
        if fmt == "csr":
            if self._csr is None:
                self._csr = _compress(self._src, self._dst, self._n)
            return self._csr
        if fmt == "csc":
            if self._csc is None:
                self._csc = _compress(self._dst, self._src, self._n_dst)
            return self._csc
        raise ValueError("format must be 'csr' or 'csc'")

    def incidence(self, typ):
        """[2, E] (node, edge) pairs sorted by node then edge: what
        ``g.inc(typ).coalesce().indices()`` yields in the reference."""
        if typ == "in":
            _, _, eid = self.adj_sparse("csc")
            return torch.stack([self._dst[eid], eid])
        if typ == "out":
            _, _, eid = self.adj_sparse("csr")
            return torch.stack([self._src[eid], eid])
        raise ValueError("typ must be 'in' or 'out'")

    def in_degrees(self):
        """Cached (DGL keeps degrees with the graph; a bincount over 1e8 edges per call would
        dominate an epoch)."""
        if self._in_deg is None:
            indptr = self.adj_sparse("csc")[0]
            self._in_deg = indptr[1:] - indptr[:-1]
        return self._in_deg

    def out_degrees(self):
        if self._out_deg is None:
            indptr = self.adj_sparse("csr")[0]
            self._out_deg = indptr[1:] - indptr[:-1]
        return self._out_deg

    @contextlib.contextmanager
    def local_scope(self):
        yield self

    def reorder_edges_by_dst(self):
        """The same graph with its edges renumbered in destination-major order (new edge i is old
        edge ``edge_order[i]``, kept as an attribute of the result).  Edge tensors of the
        attention layers ([E, H] logits, softmax outputs, their gradients) are reached through the
        destination-major CSR; when that order is the edge-id order itself they are read and written
        front to back instead of gathered and scattered 4 H bytes at a time.  Models that take no
        per-edge input (GAT, HGT) give the same node outputs on either numbering; per-edge inputs
        must be permuted with ``edge_order`` first."""
        order = self.adj_sparse("csc")[2]
        g = Graph(self._src[order], self._dst[order], self._n, self._n_dst)
        g.edge_order = order
        return g


def remove_self_loop(src, dst):
    keep = src != dst
    return src[keep], dst[keep]


def add_self_loop(src, dst, num_nodes):
    loops = torch.arange(num_nodes, dtype=src.dtype, device=src.device)
    return torch.cat([src, loops]), torch.cat([dst, loops])


def chung_lu(num_nodes, num_edges, gamma, seed, max_degree=None, symmetric=False,
             self_loops=True, device="cpu"):
    """Seeded Chung-Lu power-law graph.

    Expected degree of node i is proportional to (i + i0)^(-1/(gamma - 1)),
    optionally clipped at ``max_degree``.  Endpoints are drawn by inverse-CDF
    sampling, duplicate edges dropped, the graph optionally symmetrised, and
    self loops normalised the way the reference's loader does it
    (evaluation/util.py:28: remove_self_loop then add_self_loop).
    ``num_edges`` is the target number of directed edges before self loops.
    """
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    i = torch.arange(num_nodes, dtype=torch.float64, device=device)
    w = (i + 1.0).pow(-1.0 / (gamma - 1.0))
    draws = num_edges // 2 if symmetric else num_edges
    if max_degree is not None:
        # scale, clip, rescale a few times so that the clipped weights still sum to the target
        for _ in range(8):
            w = w * (draws / w.sum())
            w = w.clamp(max=float(max_degree) / (2.0 if symmetric else 1.0))
    cdf = torch.cumsum(w / w.sum(), 0)
    cdf[-1] = 1.0
    keys = torch.empty(0, dtype=torch.int64, device=device)
    need = draws
    for _ in range(6):  # top up what duplicate removal took away
        m = int(need * 1.15) + 16
        u = torch.rand(2, m, generator=gen, device=device, dtype=torch.float64)
        s = torch.searchsorted(cdf, u[0]).clamp_(max=num_nodes - 1)
        d = torch.searchsorted(cdf, u[1]).clamp_(max=num_nodes - 1)
        if symmetric:
            s, d = torch.minimum(s, d), torch.maximum(s, d)
        k = s * num_nodes + d
        k = k[s != d]
        keys = torch.unique(torch.cat([keys, k]))
        need = draws - keys.numel()
        if need <= 0:
            break
    if keys.numel() > draws:
        perm = torch.randperm(keys.numel(), generator=gen, device=device)[:draws]
        keys = keys[perm.sort().values]
    src = keys // num_nodes
    dst = keys - src * num_nodes
    if symmetric:
        src, dst = torch.cat([src, dst]), torch.cat([dst, src])
    if self_loops:
        src, dst = add_self_loop(src, dst, num_nodes)
    return Graph(src, dst, num_nodes)


def hetero_power_law(type_sizes=(100_000, 50_000, 20_000),
                     relations=((0, 1), (1, 0), (1, 2), (2, 0)), edges_per_relation=2_000_000,
                     gamma=2.0, seed0=50, device="cpu"):
    """Synthetic heterogeneous graph, homogenised the way the reference's HGT driver
    consumes its graphs (one node id space, evaluation/test_cache_SPMM.py:98): node types
    occupy consecutive id ranges, relation ``(a, b)`` contributes power-law edges from
    type ``a`` nodes to type ``b`` nodes (seed ``seed0 + relation index``), and every
    node gets a self loop.  Returns (Graph, node_type [n], edge_type [num_edges])
    with self loops carrying edge type ``len(relations)``."""
    offs = [0]
    for n in type_sizes:
        offs.append(offs[-1] + n)
    srcs, dsts, ets = [], [], []
    for r, (a, b) in enumerate(relations):
        gen = torch.Generator(device=device)
        gen.manual_seed(int(seed0 + r))
        cdfs = []
        for n in (type_sizes[a], type_sizes[b]):
            w = (torch.arange(n, dtype=torch.float64, device=device) + 1.0).pow(-1.0 / (gamma - 1.0))
            c = torch.cumsum(w / w.sum(), 0)
            c[-1] = 1.0
            cdfs.append(c)
        keys = torch.empty(0, dtype=torch.int64, device=device)
        need = edges_per_relation
        for _ in range(12):  # top up what duplicate removal took away
            u = torch.rand(2, max(int(need * 1.3), 65536), generator=gen, device=device, dtype=torch.float64)
            s = torch.searchsorted(cdfs[0], u[0]).clamp_(max=type_sizes[a] - 1)
            d = torch.searchsorted(cdfs[1], u[1]).clamp_(max=type_sizes[b] - 1)
            keys = torch.unique(torch.cat([keys, s * type_sizes[b] + d]))
            need = edges_per_relation - keys.numel()
            if need <= 0:
                break
        if keys.numel() > edges_per_relation:
            perm = torch.randperm(keys.numel(), generator=gen, device=device)[:edges_per_relation]
            keys = keys[perm.sort().values]
        srcs.append(keys // type_sizes[b] + offs[a])
        dsts.append(keys % type_sizes[b] + offs[b])
        ets.append(torch.full((keys.numel(),), r, dtype=torch.int64, device=device))
    n = offs[-1]
    src, dst = add_self_loop(torch.cat(srcs), torch.cat(dsts), n)
    ets.append(torch.full((n,), len(relations), dtype=torch.int64, device=device))
    node_type = torch.cat([torch.full((m,), t, dtype=torch.int64, device=device) for t, m in enumerate(type_sizes)])
    return Graph(src, dst, n), node_type, torch.cat(ets)
