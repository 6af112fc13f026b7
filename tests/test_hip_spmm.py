"""GPU parity: SpMM family vs the CPU oracle.

Integer sums are exact on both sides and followed by the same single fp32
multiply, so the comparison is bit-exact (tighter than the 1e-5 rel / 1e-6 abs
the fp32 outputs are allowed)."""
import numpy as np
import pytest
import torch

from gpu_util import dev, host, powerlaw_graph, rand_graph, sc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from tango_amd import kernels
    return kernels


def make_graph(src, dst, n):
    from tango_amd.graph import Graph
    from tango_amd.util import graph_preprocess
    return graph_preprocess(Graph(dev(src), dev(dst), n))


def test_graph_formats_match_oracle(orc):
    rng = np.random.default_rng(0)
    src, dst = rand_graph(rng, 200, 3000)
    g = make_graph(src, dst, 200)
    o = orc.graph_formats(src, dst, 200)
    for name in ("adj_csr", "adj_csc"):
        for a, b in zip(getattr(g, name), o[name]):
            assert np.array_equal(host(a), b)
    assert np.array_equal(host(g.inc_in), o["inc_in"]) and np.array_equal(host(g.inc_out), o["inc_out"])


# degree regimes: sparse (one wave per row) and dense/skewed (four waves per row)
# "hubs": low average degree with a few rows far beyond the long-row threshold (sixteen waves per row)
GRAPHS = [("sparse", 500, 4000), ("dense", 300, 60000), ("skewed", 2000, 400000), ("hubs", 20000, 300000)]


@pytest.mark.parametrize("F", [1, 3, 4, 16, 41, 48, 64, 100, 128, 256, 1040])
@pytest.mark.parametrize("kind,n,e", GRAPHS)
def test_csr_spmm_copy_u(K, orc, kind, n, e, F):
    rng = np.random.default_rng(F * 7 + n)
    src, dst = powerlaw_graph(rng, n, e) if kind in ("skewed", "hubs") else rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    feat = rng.integers(-127, 128, (n, F)).astype(np.int8)
    s = np.float32(0.0173)
    o = orc.graph_formats(src, dst, n)
    for reverse, fmt in ((False, "adj_csc"), (True, "adj_csr")):
        got = K.csr_SPMM(g, dev(feat), sc(s), reverse=reverse)
        want = orc.spmm_csr_copy_u(o[fmt][0], o[fmt][1], feat, s)
        assert np.array_equal(host(got), want)


def test_csr_spmm_padded_rows_and_3d(K, orc):
    rng = np.random.default_rng(1)
    n, e = 400, 50000
    src, dst = rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    o = orc.graph_formats(src, dst, n)
    feat = rng.integers(-127, 128, (n, 41)).astype(np.int8)
    padded = np.concatenate([feat, np.full((n, 7), 55, np.int8)], 1)  # garbage in the padding must be ignored
    out = torch.empty((n, 41), dtype=torch.float32, device="cuda")
    ip, ix, _ = g.adj_csc
    K.cuda_kernels.csr_SPMM(out, ip, ix, dev(padded), sc(0.5), ldf=48, F=41)
    assert np.array_equal(host(out), orc.spmm_csr_copy_u(o["adj_csc"][0], o["adj_csc"][1], feat, 0.5))
    f3 = rng.integers(-127, 128, (n, 4, 8)).astype(np.int8)
    got = K.csr_SPMM(g, dev(f3), sc(0.25))
    assert tuple(got.shape) == (n, 4, 8)
    assert np.array_equal(host(got).reshape(n, 32),
                          orc.spmm_csr_copy_u(o["adj_csc"][0], o["adj_csc"][1], f3.reshape(n, 32), 0.25))


def test_csr_spmm_empty_rows_and_all_ones(K, orc):
    n = 100
    src = np.array([0, 0, 5, 99], np.int64)
    dst = np.array([1, 1, 1, 98], np.int64)
    g = make_graph(src, dst, n)
    ones = torch.ones((n, 16), dtype=torch.int8, device="cuda")
    got = host(K.csr_SPMM(g, ones, sc(1.0)))
    assert np.array_equal(got[:, 0], np.bincount(dst, minlength=n)) and (got == got[:, :1]).all()


@pytest.mark.parametrize("H,F", [(8, 16), (2, 128), (4, 256), (3, 4), (5, 1), (12, 1), (2, 6)])
@pytest.mark.parametrize("kind,n,e", GRAPHS)
def test_u_mul_e_broadcast(K, orc, kind, n, e, H, F):
    rng = np.random.default_rng(H * 31 + F + n)
    src, dst = powerlaw_graph(rng, n, e) if kind in ("skewed", "hubs") else rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    o = orc.graph_formats(src, dst, n)
    feat = rng.integers(-127, 128, (n, H, F)).astype(np.int8)
    ev = rng.integers(-127, 128, (H, 1, e)).astype(np.int8)
    s = np.float32(3.1e-4)
    for reverse, fmt in ((False, "adj_csc"), (True, "adj_csr")):
        got = K.multi_cusparse_SPMM(g, dev(feat), dev(ev), sc(s), reverse=reverse)
        ip, ix, eid = o[fmt]
        want = orc.spmm_csr_u_mul_e(ip, ix, eid, feat, ev, s)
        assert np.array_equal(host(got), want)
        # the same edge values laid out [nnz, H, 1] (no transpose pass before the SpMM)
        ev_major = dev(np.ascontiguousarray(ev.transpose(2, 0, 1)))
        got_major = K.multi_cusparse_SPMM(g, dev(feat), ev_major, sc(s), reverse=reverse, edge_major=True)
        assert np.array_equal(host(got_major), want)
    # binding-level call with edge values already in CSR slot order (the reference's calling convention)
    ip, ix, eid = g.adj_csc
    ev_sorted = dev(ev[:, :, o["adj_csc"][2]])
    got2 = K.cuda_kernels.multi_cusparse_SPMM(ip, ix, dev(feat), ev_sorted, sc(s))
    want = orc.spmm_csr_u_mul_e(*o["adj_csc"], feat, ev, s)
    assert np.array_equal(host(got2), want)


@pytest.mark.parametrize("n,e,H,F", [(300, 20000, 3, 8), (3000, 9000, 2, 16), (2000, 30000, 1, 5)])
def test_u_mul_e_elementwise(K, orc, n, e, H, F):
    """Edge values as wide as the features (D == F): dense rows, lane-group rows of a sparse graph, and a hub."""
    rng = np.random.default_rng(2)
    src, dst = rand_graph(rng, n, e)
    if e == 30000:
        dst[:6000] = 11
    g = make_graph(src, dst, n)
    o = orc.graph_formats(src, dst, n)
    feat = rng.integers(-127, 128, (n, H, F)).astype(np.int8)
    ev = rng.integers(-127, 128, (H, F, e)).astype(np.int8)
    ip, ix, eid = g.adj_csc
    got = K.cuda_kernels.multi_cusparse_SPMM(ip, ix, dev(feat), dev(ev), sc(0.01), edge_ids=eid)
    want = orc.spmm_csr_u_mul_e(*o["adj_csc"], feat, ev, 0.01)
    assert np.array_equal(host(got), want)
    ev_major = dev(np.ascontiguousarray(ev.transpose(2, 0, 1)))  # [nnz, H, F]
    got = K.cuda_kernels.multi_cusparse_SPMM(ip, ix, dev(feat), ev_major, sc(0.01), edge_ids=eid, edge_major=True)
    assert np.array_equal(host(got), want)


@pytest.mark.parametrize("F", [1, 8, 16, 20, 64])
@pytest.mark.parametrize("kind,n,e", GRAPHS)
def test_incidence_spmm(K, orc, kind, n, e, F):
    rng = np.random.default_rng(F + n)
    src, dst = powerlaw_graph(rng, n, e) if kind in ("skewed", "hubs") else rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    o = orc.graph_formats(src, dst, n)
    E = rng.integers(-127, 128, (e, F)).astype(np.int8)
    s = np.float32(0.02)
    for reverse, inc in ((False, "inc_in"), (True, "inc_out")):
        want = orc.spmm_incidence(o[inc][0], o[inc][1], E, s, n)
        got = K.incidence_SPMM(g, dev(E), sc(s), reverse=reverse)
        assert np.array_equal(host(got), want)
        # the binding with the reference's arguments: sorted (node, edge) pairs
        coo = g.inc_out if reverse else g.inc_in
        got = torch.empty((n, F), dtype=torch.float32, device="cuda")
        K.cuda_kernels.incidence_SPMM(got, coo[0], coo[1], dev(E), sc(s))
        assert np.array_equal(host(got), want)
    # the equivalence the reference relies on: incidence SpMM == CSR SpMM over (indptr, edge_ids)
    ip, _, eid = g.adj_csc
    out = torch.empty((n, F), dtype=torch.float32, device="cuda")
    K.cuda_kernels.csr_SPMM(out, ip, eid, dev(E), sc(s))
    assert torch.equal(out, K.incidence_SPMM(g, dev(E), sc(s)))
    E3 = dev(E).view(e, F, 1) if F > 1 else dev(E)
    assert tuple(K.incidence_SPMM(g, E3, sc(s)).shape) == (n,) + tuple(E3.shape[1:])


@pytest.mark.parametrize("e", [1, 5, 255, 256, 257, 3000, 40011])
@pytest.mark.parametrize("F", [16, 40, 128])
def test_spmm_slot_spans_with_empty_row_runs(K, orc, e, F):
    """Sparse graphs are cut by slots, 256 per wavefront.  Destinations only at both ends of the id
    range leave thousands of empty rows in a row inside one span (more than the staged row pointers
    cover), rows without slots before the first and after the last edge, and spans cut mid-row."""
    rng = np.random.default_rng(e + F)
    n = 9000
    src = rng.integers(0, n, e).astype(np.int64)
    dst = np.where(rng.random(e) < 0.5, rng.integers(5, 40, e), rng.integers(n - 40, n - 3, e)).astype(np.int64)
    g = make_graph(src, dst, n)
    o = orc.graph_formats(src, dst, n)
    feat = rng.integers(-127, 128, (n, F)).astype(np.int8)
    s = np.float32(0.031)
    got = K.csr_SPMM(g, dev(feat), sc(s))
    assert np.array_equal(host(got), orc.spmm_csr_copy_u(o["adj_csc"][0], o["adj_csc"][1], feat, s))
    H = 4 if F % 4 == 0 else 1
    f3 = feat.reshape(n, H, F // H)
    ev = rng.integers(-127, 128, (e, H, 1)).astype(np.int8)
    got = K.multi_cusparse_SPMM(g, dev(f3), dev(ev), sc(s), edge_major=True)
    want = orc.spmm_csr_u_mul_e(*o["adj_csc"], f3, np.ascontiguousarray(ev.transpose(1, 2, 0)), s)
    assert np.array_equal(host(got), want)


@pytest.mark.parametrize("kind,n,e", [GRAPHS[0], GRAPHS[3]])
@pytest.mark.parametrize("F", [16, 100, 256])
def test_spmm_without_workspace(K, orc, kind, n, e, F):
    """workspace = NULL through the C entry point: sparse graphs then go by in-degree tiers
    (lane group, wavefront, sixteen wavefronts per row)."""
    from tango_amd import _lib
    rng = np.random.default_rng(F + n)
    src, dst = powerlaw_graph(rng, n, e) if kind == "hubs" else rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    o = orc.graph_formats(src, dst, n)
    feat = dev(rng.integers(-127, 128, (n, F)).astype(np.int8))
    ip, ix, _ = g.adj_csc
    out = torch.empty((n, F), dtype=torch.float32, device="cuda")
    s = sc(0.25)
    st = torch.cuda.current_stream().cuda_stream
    assert _lib.lib().tango_spmm_csr_copy_u_ex(out.data_ptr(), ip.data_ptr(), ix.data_ptr(), 64, feat.data_ptr(), F,
                                               s.data_ptr(), None, None, 0, None, n, n, e, F, 0, None, None, None, 0, st) == 0
    assert np.array_equal(host(out), orc.spmm_csr_copy_u(o["adj_csc"][0], o["adj_csc"][1], host(feat), 0.25))
