"""GPU parity at the benchmark's full sizes.

Where the oracle finishes in seconds it is run outright (bit-exact); where it
would not (the 7e10-op GEMMs, the 256-wide aggregation), size-independent
properties pin the result instead: row independence of a GEMM (oracle on a row
sample with the global scales), closed-form reductions for one-hot operands,
all-ones features = degrees, integer linearity, softmax rows summing to one."""
import numpy as np
import pytest
import torch

from gpu_util import dev, host, sc

pytestmark = pytest.mark.gpu

N_NODES = 232965


@pytest.fixture(scope="module")
def K():
    from tango_amd import kernels
    return kernels


@pytest.fixture(scope="module")
def big_graph():
    from tango_amd.graph import chung_lu
    from tango_amd.util import graph_preprocess
    g = graph_preprocess(chung_lu(N_NODES, 114_600_000, 2.0, seed=3, max_degree=21000, symmetric=True,
                                  device="cuda"))
    assert g.num_edges() > 110_000_000
    return g


def test_graph_is_symmetric_with_self_loops(big_graph):
    g = big_graph
    assert torch.equal(g.in_degrees(), g.out_degrees())  # symmetrised
    assert int(g.in_degrees().min()) >= 1  # self loops
    ip, ix, eid = g.adj_csc
    src, dst = g.coo
    # spot-check the permutation: slot p of row r holds edge eid[p] = (ix[p] -> r)
    p = torch.randint(0, ix.numel(), (100000,), device="cuda")
    assert torch.equal(src[eid[p]], ix[p])
    rows = torch.searchsorted(ip, p, right=True) - 1
    assert torch.equal(dst[eid[p]], rows)


def test_copy_u_F16_full_vs_oracle(K, orc, big_graph):
    g = big_graph
    rng = np.random.default_rng(0)
    feat = rng.integers(-127, 128, (N_NODES, 16)).astype(np.int8)
    got = K.csr_SPMM(g, dev(feat), sc(0.0123))
    ip, ix, _ = g.adj_csc
    want = orc.spmm_csr_copy_u(host(ip), host(ix), feat, np.float32(0.0123))
    assert np.array_equal(host(got), want)
    assert orc.overflow_count() == 0


@pytest.mark.parametrize("F", [41, 64, 256])
def test_copy_u_wide_properties(K, big_graph, F):
    g = big_graph
    one = sc(1.0)
    deg = g.in_degrees().float()
    ones = torch.ones((N_NODES, F), dtype=torch.int8, device="cuda")
    out = K.csr_SPMM(g, ones, one)
    assert torch.equal(out, deg.unsqueeze(1).expand(-1, F))
    gen = torch.Generator("cuda").manual_seed(F)
    a = torch.randint(-3, 4, (N_NODES, F), dtype=torch.int8, device="cuda", generator=gen)
    b = torch.randint(-3, 4, (N_NODES, F), dtype=torch.int8, device="cuda", generator=gen)
    # sums stay far below 2^24, so fp32 holds them exactly and linearity must be exact
    assert torch.equal(K.csr_SPMM(g, a, one) + K.csr_SPMM(g, b, one), K.csr_SPMM(g, a + b, one))
    # reverse orientation of a symmetric graph gives the same aggregation
    assert torch.equal(K.csr_SPMM(g, a, one), K.csr_SPMM(g, a, one, reverse=True))
    # a column-sliced view of the wide result equals the narrow aggregation of that slice
    narrow = K.csr_SPMM(g, a[:, :16].contiguous(), one)
    assert torch.equal(K.csr_SPMM(g, a, one)[:, :16], narrow)


def test_u_mul_e_full_reduces_to_copy_u(K, big_graph):
    g = big_graph
    nnz = g.num_edges()
    H, F = 2, 64
    gen = torch.Generator("cuda").manual_seed(9)
    feat = torch.randint(-3, 4, (N_NODES, H, F), dtype=torch.int8, device="cuda", generator=gen)
    ones = torch.ones((H, 1, nnz), dtype=torch.int8, device="cuda")
    a = K.multi_cusparse_SPMM(g, feat, ones, sc(1.0))
    assert torch.equal(a.view(N_NODES, -1), K.csr_SPMM(g, feat.view(N_NODES, -1), sc(1.0)))
    # edge value = 2 on every edge doubles the integer sums exactly
    assert torch.equal(K.multi_cusparse_SPMM(g, feat, ones * 2, sc(1.0)), a * 2)


@pytest.mark.parametrize("M,Kd,N", [(N_NODES, 602, 256), (N_NODES, 256, 41), (N_NODES, 128, 16),
                                    (169343, 128, 128), (169343, 256, 128), (169343, 602, 41),
                                    (169343, 256, 256), (N_NODES, 602, 128)])
def test_qlinear_forward_full_rows_independent(K, orc, M, Kd, N):
    gen = torch.Generator("cuda").manual_seed(Kd)
    X = torch.randn(M, Kd, device="cuda", generator=gen)
    W = (torch.rand(N, Kd, device="cuda", generator=gen) - 0.5) * 0.2
    b = torch.randn(N, device="cuda", generator=gen)
    sX, sW = K.cuda_kernels.get_scale(X), K.cuda_kernels.get_scale(W)
    ld = (Kd + 15) // 16 * 16
    Xq = torch.empty((M, ld), dtype=torch.int8, device="cuda")[:, :Kd]
    Wq = torch.empty((N, Kd), dtype=torch.int8, device="cuda")
    Y, sY = K.QGEMM_forward(X, Xq, sX, W, Wq, sW, b, True)
    assert sX.item() == X.abs().max().item() / np.float32(127) and sY.item() == orc.absmax_scale(host(Y))
    rows = np.sort(np.random.default_rng(1).choice(M, 3000, replace=False))
    rows[-1] = M - 1
    Yo, Xqo, Wqo, _, _, _ = orc.qgemm_fwd(host(X)[rows], host(W), bias=host(b), sX=sX.item(), sW=sW.item())
    assert np.array_equal(host(Y)[rows], Yo)
    assert np.array_equal(host(Xq)[rows], Xqo) and np.array_equal(host(Wq), Wqo)


@pytest.mark.parametrize("M,Kd,N", [(N_NODES, 602, 256), (N_NODES, 256, 41), (169343, 128, 16),
                                    (169343, 256, 128), (169343, 602, 41)])
def test_qlinear_backward_full_closed_forms(K, orc, M, Kd, N):
    gen = torch.Generator("cuda").manual_seed(3)
    Xq = torch.randint(-127, 128, (M, Kd), dtype=torch.int8, device="cuda", generator=gen)
    Wq = torch.randint(-127, 128, (N, Kd), dtype=torch.int8, device="cuda", generator=gen)
    # one-hot dY: row m selects output column m % N with value v[m]
    v = torch.randint(-5, 6, (M,), dtype=torch.int8, device="cuda", generator=gen)
    dY = torch.zeros((M, N), dtype=torch.int8, device="cuda")
    cols = torch.arange(M, device="cuda") % N
    dY[torch.arange(M, device="cuda"), cols] = v
    dX, dW = K.QGEMM_backward(dY, Xq, Wq, sc(1.0), sc(1.0), sc(1.0))
    # dX[m, :] = v[m] * Wq[m % N, :]
    assert torch.equal(dX, v.float().unsqueeze(1) * Wq.float()[cols])
    # dW[n, :] = sum over rows with m % N == n of v[m] * Xq[m, :]   (|sum| < 2^24: exact in fp32)
    want = torch.zeros((N, Kd), dtype=torch.int64, device="cuda").index_add_(0, cols, v.long().unsqueeze(1) * Xq.long())
    assert int(want.abs().max()) < 2 ** 24
    assert torch.equal(dW.long(), want)
    # dense random dY on a row sample against the oracle (rows of dX are independent)
    dYr = torch.randint(-127, 128, (M, N), dtype=torch.int8, device="cuda", generator=gen)
    dX2, _ = K.QGEMM_backward(dYr, Xq, Wq, sc(0.01), sc(1.0), sc(0.02), W_need=False)
    rows = np.sort(np.random.default_rng(2).choice(M, 2000, replace=False))
    assert np.array_equal(host(dX2)[rows], orc.qgemm_bwd_dx(host(dYr)[rows], host(Wq), 0.01, 0.02))
    # gradW with dense operands on a slice of M the oracle finishes quickly (the split over M is
    # exercised at full size by the closed form above)
    Ms = 40000
    _, dW2 = K.QGEMM_backward(dYr[:Ms], Xq[:Ms], Wq, sc(0.01), sc(0.03), sc(1.0), X_need=False)
    assert np.array_equal(host(dW2), orc.qgemm_bwd_dw(host(dYr[:Ms]), host(Xq[:Ms]), 0.01, 0.03))


def test_hidden_gradient_hand_off_full(K, orc):
    """The benchmark epoch's hand-off at its own shapes (232,965 rows, 41 -> 256 columns): gradX with the masked-scale
    epilogue stores the dX of the plain kernel (sampled rows: the oracle's), its scale is max|dX' * mul| / 127 formed
    with torch's exact elementwise ops and agrees with the separate masked pass, and the quantize pass that also
    sums the columns writes the bytes of the plain pass (sampled rows: the oracle's) with column sums matching a
    float64 sum."""
    M, N, Kc = N_NODES, 41, 256
    gen = torch.Generator("cuda").manual_seed(5)
    dYq = torch.zeros((M, 48), dtype=torch.int8, device="cuda")[:, :N]
    dYq.copy_(torch.randint(-127, 128, (M, N), dtype=torch.int8, device="cuda", generator=gen))
    Wq = torch.randint(-127, 128, (N, Kc), dtype=torch.int8, device="cuda", generator=gen)
    rs = torch.rand(M, device="cuda", generator=gen) + 0.5
    mul = torch.rand(M, device="cuda", generator=gen) + 0.25
    keep = torch.rand((M, Kc), device="cuda", generator=gen) < 0.5
    weights = (1 << torch.arange(16, device="cuda", dtype=torch.int32))
    bits = (keep.view(M, Kc // 16, 16).int() * weights).sum(-1).to(torch.int16).contiguous()  # one bit per column
    s_dY, s_W = sc(0.013), sc(0.0021)
    dX = torch.full((M, Kc), float("nan"), device="cuda")
    got = K.cuda_kernels.QGEMM_backward_gradX(dX, dYq, Wq, s_dY, s_W, row_scale=rs, masked=(bits, mul))
    assert got is not None
    plain = torch.empty_like(dX)
    K.cuda_kernels.QGEMM_backward_gradX(plain, dYq, Wq, s_dY, s_W, row_scale=rs)
    assert torch.equal(dX, plain)
    rows = np.sort(np.random.default_rng(4).choice(M, 1500, replace=False))
    want = orc.qgemm_bwd_dx_ex(host(dYq)[rows], host(Wq), np.float32(0.013), np.float32(0.0021), row_scale=host(rs)[rows])
    assert np.array_equal(host(dX)[rows], want)
    masked = torch.where(keep, dX, torch.zeros((), device="cuda"))
    assert torch.equal(got, ((masked * mul.unsqueeze(1)).abs().max() / 127).reshape(1))
    s_pass, _ = K.cuda_kernels.absmax_ex(dX, row_mul=mul, mask=bits, mask_mode="bits")
    assert torch.equal(got, s_pass)
    # the quantize pass of that gradient, stochastic as in the epoch, with the bias gradient
    kw = dict(row_mul=mul, mask=bits, mask_mode="bits", round_mode="stochastic", seed=9, offset=1 << 20)
    q = torch.full((M, Kc), 77, dtype=torch.int8, device="cuda")
    cs = K.cuda_kernels.quantize_rows_colsum(q, dX, got, **kw)
    q_plain, _ = K.quantize_padded(dX, got, align=16, **kw)
    assert torch.equal(q, q_plain)
    assert torch.allclose(cs.double(), masked.double().sum(0), rtol=1e-5, atol=1e-3)
    # a block of rows' bytes depend on its own values and on its position in the random stream only
    for r0 in (0, 117_003, M - 600):
        blk = slice(r0, r0 + 600)
        want_q = orc.quantize_rows_ex(host(dX[blk]), host(got)[0], row_mul=host(mul[blk]), mask=host(bits[blk]),
                                      mask_mode="bits", mode=orc.STOCHASTIC, seed=9, offset=(1 << 20) + r0 * Kc)
        assert np.array_equal(host(q[blk]), want_q)


def _row_sample_csr(g, count, seed, reverse=False):
    """Sub-CSR of `count` sampled destination rows (hubs included): indptr, column ids and slot
    numbers, as host arrays plus the slots as a device tensor."""
    ip, ix, _ = g.adj_csr if reverse else g.adj_csc
    n = ip.numel() - 1
    rng = np.random.default_rng(seed)
    rows = np.unique(np.concatenate([rng.choice(n, count, replace=False), np.arange(8), [n - 1]]))
    rows_d = torch.from_numpy(rows).cuda()
    lo, hi = ip[rows_d], ip[rows_d + 1]
    lens = hi - lo
    sub_ip = torch.zeros(rows.size + 1, dtype=torch.int64, device="cuda")
    torch.cumsum(lens, 0, out=sub_ip[1:])
    total = int(sub_ip[-1])
    owner = torch.repeat_interleave(torch.arange(rows.size, device="cuda"), lens)
    slots = lo[owner] + (torch.arange(total, device="cuda") - sub_ip[owner])
    return rows, host(sub_ip), host(ix[slots]), slots


def test_copy_u_F128_full(K, orc, big_graph):
    # width 128 on the 114.8 M-edge graph: properties over every row, the oracle on a row sample
    g = big_graph
    F = 128
    ones = torch.ones((N_NODES, F), dtype=torch.int8, device="cuda")
    assert torch.equal(K.csr_SPMM(g, ones, sc(1.0)), g.in_degrees().float().unsqueeze(1).expand(-1, F))
    gen = torch.Generator("cuda").manual_seed(128)
    a = torch.randint(-127, 128, (N_NODES, F), dtype=torch.int8, device="cuda", generator=gen)
    out = K.csr_SPMM(g, a, sc(0.017))
    rows, sub_ip, sub_ix, _ = _row_sample_csr(g, 2000, 5)
    want = orc.spmm_csr_copy_u(sub_ip, sub_ix, host(a), np.float32(0.017))
    assert np.array_equal(host(out)[rows], want)
    b = torch.randint(-3, 4, (N_NODES, F), dtype=torch.int8, device="cuda", generator=gen)
    c = torch.randint(-3, 4, (N_NODES, F), dtype=torch.int8, device="cuda", generator=gen)
    assert torch.equal(K.csr_SPMM(g, b, sc(1.0)) + K.csr_SPMM(g, c, sc(1.0)), K.csr_SPMM(g, b + c, sc(1.0)))


def test_copy_u_F256_fused_epilogue_full(K, orc, big_graph):
    """The launch the benchmark epoch runs: width 256 (two column tiles), '* norm, + bias, ReLU' and the sign
    words in the epilogue, on the 114.8 M-edge graph; the oracle's fused form on a row sample."""
    g = big_graph
    F = 256
    gen = torch.Generator("cuda").manual_seed(256)
    feat = torch.randint(-127, 128, (N_NODES, F), dtype=torch.int8, device="cuda", generator=gen)
    rs = g.in_degrees().float().clamp(min=1).pow(-0.5)
    bias = torch.randn(F, device="cuda", generator=gen) * 0.05
    bits = torch.empty((N_NODES, F // 16), dtype=torch.int16, device="cuda")
    out = K.csr_SPMM(g, feat, sc(0.0004), row_scale=rs, bias=bias, relu=True, sign_bits=bits)
    rows, sub_ip, sub_ix, _ = _row_sample_csr(g, 2000, 11)
    want, wbits = orc.spmm_csr_copy_u_ex(sub_ip, sub_ix, host(feat), np.float32(0.0004), row_scale=host(rs)[rows],
                                         bias=host(bias), act=1, want_bits=True)
    assert np.array_equal(host(out)[rows], want)
    assert np.array_equal(host(bits).view(np.uint16)[rows], wbits)
    frac = float((out > 0).float().mean())
    assert 0.2 < frac < 0.8  # the ReLU is exercised on both sides
    # reverse orientation, no epilogue: the backward launch of the epoch
    out_r = K.csr_SPMM(g, feat, sc(0.0004), reverse=True)
    rows, sub_ip, sub_ix, _ = _row_sample_csr(g, 1000, 12, reverse=True)
    assert np.array_equal(host(out_r)[rows], orc.spmm_csr_copy_u(sub_ip, sub_ix, host(feat), np.float32(0.0004)))


@pytest.mark.parametrize("H,F", [(8, 1), (2, 128)])
def test_u_mul_e_full_real_edge_weights(K, orc, big_graph, H, F):
    """u_mul_e on the 114.8 M-edge graph with the edge weights 1/sqrt(deg_u deg_v) quantized by
    transpose_quant, as evaluation/SPMM_nobroadcast.py:19-24 (H heads of width 1, the form without
    broadcast) and evaluation/SPMM_broadcast.py (H = 2, F = 128) call it."""
    g = big_graph
    nnz = g.num_edges()
    src, dst = g.coo
    deg = g.in_degrees().float()
    w = (deg[src] * deg[dst]).rsqrt_()
    Ew = (w.view(nnz, 1, 1) * torch.linspace(1.0, 0.3, H, device="cuda").view(1, H, 1)).contiguous()
    del w
    sE = K.cuda_kernels.get_scale(Ew)
    ET = K.transpose_quant(Ew, sE)                      # [H, 1, nnz] int8 in edge-id order
    # transpose_quant itself on a sample of edges
    pick = torch.randint(0, nnz, (200000,), device="cuda")
    want_q = orc.quantize(host(Ew.view(nnz, H)[pick]), host(sE)[0])
    assert np.array_equal(host(ET.view(H, nnz)[:, pick]).T, want_q)
    del Ew
    gen = torch.Generator("cuda").manual_seed(H * 1000 + F)
    feat = torch.randint(-127, 128, (N_NODES, H, F), dtype=torch.int8, device="cuda", generator=gen)
    scale = sc(0.003) * sE
    out = K.multi_cusparse_SPMM(g, feat, ET, scale)
    assert out.shape == (N_NODES, H, F) and bool(torch.isfinite(out).all())
    rows, sub_ip, sub_ix, slots = _row_sample_csr(g, 2000, 6)
    eid = g.adj_csc[2][slots]
    sub_ET = host(ET.view(H, nnz)[:, eid]).reshape(H, 1, -1)   # the sample's edge values in slot order
    want = orc.spmm_csr_u_mul_e(sub_ip, sub_ix, None, host(feat), sub_ET, host(scale)[0])
    assert np.array_equal(host(out)[rows], want)
    # the backward orientation (source-major CSR) on its own row sample
    out_r = K.multi_cusparse_SPMM(g, feat, ET, scale, reverse=True)
    rows, sub_ip, sub_ix, slots = _row_sample_csr(g, 1000, 7, reverse=True)
    eid = g.adj_csr[2][slots]
    sub_ET = host(ET.view(H, nnz)[:, eid]).reshape(H, 1, -1)
    want = orc.spmm_csr_u_mul_e(sub_ip, sub_ix, None, host(feat), sub_ET, host(scale)[0])
    assert np.array_equal(host(out_r)[rows], want)


def test_incidence_full(K, orc, big_graph):
    """copy_e-sum over the 114.8 M edges (evaluation/test_incidence.py:14-22): all-ones = in-degree,
    integer linearity, the oracle's COO form on a row sample, and the reference-argument binding."""
    g = big_graph
    nnz, F = g.num_edges(), 8
    ones = torch.ones((nnz, F), dtype=torch.int8, device="cuda")
    assert torch.equal(K.incidence_SPMM(g, ones, sc(1.0)), g.in_degrees().float().unsqueeze(1).expand(-1, F))
    del ones
    gen = torch.Generator("cuda").manual_seed(77)
    E = torch.randint(-127, 128, (nnz, F), dtype=torch.int8, device="cuda", generator=gen)
    out = K.incidence_SPMM(g, E, sc(0.25))
    rows, sub_ip, _, slots = _row_sample_csr(g, 2000, 8)
    node = np.repeat(np.arange(rows.size), np.diff(sub_ip))
    sub_E = host(E[g.adj_csc[2][slots]])
    want = orc.spmm_incidence(node, np.arange(node.size), sub_E, 0.25, rows.size)
    assert np.array_equal(host(out)[rows], want)
    # the binding with the reference's arguments (sorted COO pairs of the incidence matrix)
    out2 = torch.empty((N_NODES, F), dtype=torch.float32, device="cuda")
    K.cuda_kernels.incidence_SPMM(out2, g.inc_in[0], g.inc_in[1], E, sc(0.25))
    assert torch.equal(out2, out)
    out_r = K.incidence_SPMM(g, E, sc(0.25), reverse=True)
    rows, sub_ip, _, slots = _row_sample_csr(g, 500, 9, reverse=True)
    node = np.repeat(np.arange(rows.size), np.diff(sub_ip))
    want = orc.spmm_incidence(node, np.arange(node.size), host(E[g.adj_csr[2][slots]]), 0.25, rows.size)
    assert np.array_equal(host(out_r)[rows], want)


def test_hgt_primitives_full(K, orc):
    """The heterogeneous variant's graph (3 node types 100K/50K/20K, 4 relations x 2 M edges, self loops;
    homogenised as evaluation/test_HGT.py:48-67 consumes it) at full size, 4 heads x 64: every primitive of
    the layer against the oracle."""
    from tango_amd.graph import hetero_power_law
    from tango_amd.util import graph_preprocess
    g0, _, _ = hetero_power_law(device="cuda")
    g = graph_preprocess(g0)
    n, E, H, D = g.num_nodes(), g.num_edges(), 4, 64
    assert n == 170000 and E == 8_000_000 + n
    rng = np.random.default_rng(5)
    k = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
    q = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
    src, dst = host(g.coo[0]), host(g.coo[1])
    t, st = K.mySDDMM_int8(g, "dot", dev(k), dev(q), sc(3e-4), sc(2e-4), True)
    want, wst = orc.sddmm_dot(src, dst, k, q, 3e-4, 2e-4, reduce=True)
    assert np.array_equal(host(t).reshape(E, H), want) and host(st)[0] == wst
    ip, ix, eid = g.adj_csc
    a = K.cuda_kernels.edge_softmax_forward(t, ip, eid, 1.0)
    want_a = orc.edge_softmax_fwd(want, host(ip), host(eid), 1.0)
    assert np.allclose(host(a).reshape(E, H), want_a, rtol=1e-5, atol=1e-6)
    # attention-weighted aggregation with edge-major int8 edge values, as the layer runs it
    aq, sa = K.quantize(a)
    assert np.array_equal(host(aq).reshape(E, H), orc.quantize(host(a).reshape(E, H), host(sa)[0]))
    v = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
    agg = K.multi_cusparse_SPMM(g, dev(v), aq, sc(1e-3), edge_major=True, scale2=sa)
    ET = np.ascontiguousarray(host(aq).reshape(E, H).T).reshape(H, 1, E)
    s = np.float32(np.float32(1e-3) * host(sa)[0])
    want_agg = orc.spmm_csr_u_mul_e(host(ip), host(ix), host(eid), v, ET, s)
    assert np.array_equal(host(agg), want_agg)
    # backward aggregations of the layer: dV-like (source-major) and the edge gradient (SDDMM dot of dOut, v)
    cp, cx, ceid = g.adj_csr
    agg_r = K.multi_cusparse_SPMM(g, dev(v), aq, sc(1e-3), reverse=True, edge_major=True, scale2=sa)
    assert np.array_equal(host(agg_r), orc.spmm_csr_u_mul_e(host(cp), host(cx), host(ceid), v, ET, s))


def test_hetero_hgt_relations_full(K, orc):
    """The heterogeneous variant proper: every relation of the 3-type / 4-relation graph (2 M edges each, plus the
    self loops) as its own graph over all 170,000 nodes, 4 heads x 64: the relation's SDDMM dot, and its
    attention-weighted aggregation with edge values cut out of one softmax over the whole graph, against the
    oracle; then one heterogeneous layer forward + backward at this size."""
    from tango_amd.gat import HeteroHGTLayer, relation_graphs
    from tango_amd.graph import hetero_power_law
    from tango_amd.util import graph_preprocess
    sizes, rels = (100_000, 50_000, 20_000), ((0, 1), (1, 0), (1, 2), (2, 0))
    g0, _, edge_type = hetero_power_law(type_sizes=sizes, relations=rels, device="cuda")
    g = graph_preprocess(g0)
    rg = relation_graphs(g, edge_type, rels, sizes)
    assert [r.num_edges() for r in rg] == [2_000_000] * 4 + [170_000]
    n, E, H, D = g.num_nodes(), g.num_edges(), 4, 64
    rng = np.random.default_rng(15)
    q = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
    t_all = torch.zeros((E, H, 1), device="cuda")
    for r, gr in enumerate(rg):
        k = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
        t, _ = K.mySDDMM_int8(gr, "dot", dev(k), dev(q), sc(3e-4), sc(2e-4), False)
        want, _ = orc.sddmm_dot(host(gr.coo[0]), host(gr.coo[1]), k, q, 3e-4, 2e-4)
        assert np.array_equal(host(t).reshape(-1, H), want), r
        t_all[gr.eids] = t
    ip, ix, eid = g.adj_csc
    a = K.cuda_kernels.edge_softmax_forward(t_all, ip, eid, 1.0)
    np.testing.assert_allclose(host(a).reshape(E, H), orc.edge_softmax_fwd(host(t_all).reshape(E, H), host(ip), host(eid), 1.0),
                               rtol=1e-5, atol=1e-6)
    for r, gr in enumerate(rg):
        v = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
        ar = a[gr.eids].contiguous()
        aq, sa = K.quantize(ar)
        agg = K.multi_cusparse_SPMM(gr, dev(v), aq, sc(1e-3), edge_major=True, scale2=sa)
        rp, rx, re = (host(x) for x in gr.adj_csc)
        want = orc.spmm_csr_u_mul_e_ex(rp, rx, re, v, host(aq), 1e-3, scale2=host(sa)[0], edge_major=True)
        assert np.array_equal(host(agg), want), r
    torch.manual_seed(1)
    layer = HeteroHGTLayer(256, 256, 4, sizes, rg).cuda()
    h = torch.randn(n, 256, device="cuda", requires_grad=True)
    out = layer(g, h)
    out.square().mean().backward()
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(h.grad).all())
    assert all(p.grad is not None for p in layer.parameters())


def test_hgt_layer_full_size_runs():
    """One HGT layer forward + backward on the full heterogeneous graph: finite, and close to the same layer
    in fp32 (quantization error only)."""
    from tango_amd.gat import HGTLayer
    from tango_amd.graph import hetero_power_law
    from tango_amd.util import graph_preprocess
    g0, _, _ = hetero_power_law(device="cuda")
    g = graph_preprocess(g0.reorder_edges_by_dst())
    torch.manual_seed(0)
    layer = HGTLayer(256, 256, 4).cuda()
    h = torch.randn(g.num_nodes(), 256, device="cuda", requires_grad=True)
    out = layer(g, h)
    out.square().mean().backward()
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(h.grad).all())
    with torch.no_grad():
        lin = lambda m, x: torch.nn.functional.linear(x, m.weight, m.bias)
        kk = lin(layer.attn_linear, lin(layer.k_linear, h)).view(-1, 4, 64)
        vv = lin(layer.msg_linear, lin(layer.v_linear, h)).view(-1, 4, 64)
        qq = lin(layer.q_linear, h).view(-1, 4, 64)
        src, dst = g.coo
        t = (kk[src] * qq[dst]).sum(-1) / 8.0
        mx = torch.full((g.num_nodes(), 4), -1e30, device="cuda").scatter_reduce_(0, dst.unsqueeze(1).expand(-1, 4), t, "amax")
        ex = (t - mx[dst]).exp()
        den = torch.zeros((g.num_nodes(), 4), device="cuda").index_add_(0, dst, ex)
        att = ex / den[dst]
        agg = torch.zeros((g.num_nodes(), 4, 64), device="cuda").index_add_(0, dst, vv[src] * att.unsqueeze(-1))
        ref = lin(layer.a_linear, agg.reshape(-1, 256))
    err = (out - ref).norm() / ref.norm()
    assert err.item() < 0.15  # six chained int8 GEMMs + int8 attention: 0.104 measured


def test_gat_primitives_full(K, orc):
    # 169,343 nodes / 1,166,243 edges + self loops, 8 heads x 16
    from tango_amd.graph import chung_lu
    from tango_amd.util import graph_preprocess
    g = graph_preprocess(chung_lu(169343, 1166243, 2.2, seed=4, device="cuda"))
    n, E, H, D = g.num_nodes(), g.num_edges(), 8, 16
    assert E == 1166243 + n
    rng = np.random.default_rng(4)
    U = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
    V = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
    src, dst = host(g.coo[0]), host(g.coo[1])
    out, so = K.mySDDMM_int8(g, "dot", dev(U), dev(V), sc(0.01), sc(0.02), True)
    want, wso = orc.sddmm_dot(src, dst, U, V, 0.01, 0.02, reduce=True)
    assert np.array_equal(host(out).reshape(E, H), want) and host(so)[0] == wso
    el = rng.integers(-127, 128, (n, H, 1)).astype(np.int8)
    er = rng.integers(-127, 128, (n, H, 1)).astype(np.int8)
    e_add, _ = K.mySDDMM_int8(g, "add", dev(el), dev(er), sc(0.03), sc(0.01), False)
    want_add, _ = orc.sddmm_ewise("add", src, dst, el.reshape(n, H), er.reshape(n, H), 0.03, 0.01)
    assert np.array_equal(host(e_add).reshape(E, H), want_add)
    ip, _, eid = g.adj_csc
    a = K.cuda_kernels.edge_softmax_forward(e_add, ip, eid, 0.2)
    sums = torch.zeros((n, H, 1), device="cuda").index_add_(0, g.coo[1], a)
    assert torch.allclose(sums, torch.ones_like(sums), atol=1e-5)
    want_a = orc.edge_softmax_fwd(host(e_add).reshape(E, H), host(ip), host(eid), 0.2)
    assert np.allclose(host(a).reshape(E, H), want_a, rtol=1e-5, atol=1e-6)
    # attention-weighted aggregation and the incidence form of the backward, against the oracle
    from tango_amd.kernels import transpose_quant
    sE = K.cuda_kernels.get_scale(a)
    ET = transpose_quant(a, sE)
    feat = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
    agg = K.multi_cusparse_SPMM(g, dev(feat), ET, sc(0.001))
    want_agg = orc.spmm_csr_u_mul_e(host(ip), host(g.adj_csc[1]), host(eid), feat, host(ET), 0.001)
    assert np.array_equal(host(agg), want_agg)
    dZ = rng.integers(-127, 128, (E, H)).astype(np.int8)
    inc = K.incidence_SPMM(g, dev(dZ), sc(0.5))
    assert np.array_equal(host(inc), orc.spmm_incidence(host(g.inc_in[0]), host(g.inc_in[1]), dZ, 0.5, n))


def test_gcn_config1_layer_matches_oracle(orc):
    # 19,717 nodes / 88,651 undirected edges, 500 -> 16: GEMM with fused scale, then aggregation
    from tango_amd.graph import chung_lu
    from tango_amd.util import graph_preprocess
    from tango_amd.QLinear import Qlinear_func_reduce
    from tango_amd.SPMM import spmm_copy_u
    g = graph_preprocess(chung_lu(19717, 2 * 88651, 2.1, seed=1, symmetric=True, device="cuda"))
    gen = torch.Generator().manual_seed(1)
    X = torch.randn(19717, 500, generator=gen).cuda()
    W = torch.nn.init.xavier_uniform_(torch.empty(16, 500), generator=gen).cuda()
    feat_src = X * g.out_degrees().float().clamp(min=1).pow(-0.5).unsqueeze(1)
    Y, sY = Qlinear_func_reduce.apply(feat_src, W)
    out = spmm_copy_u.apply(g, Y, sY)
    Yo, _, _, _, _, sYo = orc.qgemm_fwd(host(feat_src), host(W), reduce=True)
    assert np.array_equal(host(Y), Yo) and sY.item() == sYo
    ip, ix, _ = g.adj_csc
    assert np.array_equal(host(out), orc.spmm_csr_copy_u(host(ip), host(ix), orc.quantize(Yo, sYo), sYo))


def test_gat_backward_primitives_full(K, orc):
    """The backward halves of the GAT block at the benchmark size (169,343 nodes / 1,335,586 edges, 8 heads x 16):
    edge softmax backward, the attention logits' backward and both gradients of the attention-weighted
    aggregation, against the oracle (closed forms in float64 for the logits, which have no oracle function)."""
    from tango_amd import config
    from tango_amd.SPMM import spmm_u_mul_e
    from tango_amd.graph import chung_lu
    from tango_amd.util import graph_preprocess
    g = graph_preprocess(chung_lu(169343, 1166243, 2.2, seed=4, device="cuda"))
    n, E, H, D = g.num_nodes(), g.num_edges(), 8, 16
    rng = np.random.default_rng(40)
    ip, ix, eid = g.adj_csc
    # edge softmax backward (LeakyReLU 0.2 folded in)
    e = rng.standard_normal((E, H)).astype(np.float32)
    da = rng.standard_normal((E, H)).astype(np.float32)
    e_d, da_d = dev(e).view(E, H, 1), dev(da).view(E, H, 1)
    a = K.cuda_kernels.edge_softmax_forward(e_d, ip, eid, 0.2)
    de = K.cuda_kernels.edge_softmax_backward(a, da_d, e_d, ip, eid, 0.2)
    want_de = orc.edge_softmax_bwd(host(a).reshape(E, H), da, e, host(ip), host(eid), 0.2)
    assert np.allclose(host(de).reshape(E, H), want_de, rtol=1e-5, atol=1e-6)
    # attention logits backward: dfeat = del * attn_l + der * attn_r, dattn = sum over nodes of d * feat
    feat = rng.standard_normal((n, H, D)).astype(np.float32)
    al, ar = rng.standard_normal((H, D)).astype(np.float32), rng.standard_normal((H, D)).astype(np.float32)
    dl, dr = rng.standard_normal((n, H)).astype(np.float32), rng.standard_normal((n, H)).astype(np.float32)
    dfeat, dal, dar = K.cuda_kernels.attn_scores_backward(dev(dl), dev(dr), dev(feat), dev(al), dev(ar))
    f64 = feat.astype(np.float64)
    want_dfeat = dl[:, :, None].astype(np.float64) * al + dr[:, :, None].astype(np.float64) * ar
    np.testing.assert_allclose(host(dfeat), want_dfeat, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(host(dal), (dl[:, :, None] * f64).sum(0), rtol=1e-4, atol=1e-2)  # sums of 169,343 terms
    np.testing.assert_allclose(host(dar), (dr[:, :, None] * f64).sum(0), rtol=1e-4, atol=1e-2)
    # u_mul_e backward: dN = reverse aggregation of the quantized dZ with the edge values, dE = SDDMM dot
    saved = config.grad_round_mode
    config.grad_round_mode = "rne"
    try:
        N = torch.randn(n, H, D, device="cuda", requires_grad=True)
        Ev = a.detach().clone().requires_grad_(True)
        out = spmm_u_mul_e.apply(g, N, Ev)
        dZ = torch.randn(n, H, D, device="cuda")
        out.backward(dZ)
    finally:
        config.grad_round_mode = saved
    Nn, En, dZn = host(N.detach()), host(Ev.detach()), host(dZ)
    sN, sE, sdZ = orc.absmax_scale(Nn), orc.absmax_scale(En), orc.absmax_scale(dZn)
    Nq, Eq, dZq = orc.quantize(Nn, sN), orc.quantize(En, sE), orc.quantize(dZn, sdZ)
    want_out = orc.spmm_csr_u_mul_e_ex(host(ip), host(ix), host(eid), Nq, Eq, sN, scale2=sE, edge_major=True)
    assert np.array_equal(host(out.detach()), want_out)
    rp, rx, reid = (host(t) for t in g.adj_csr)
    want_dN = orc.spmm_csr_u_mul_e_ex(rp, rx, reid, dZq, Eq, sdZ, scale2=sE, edge_major=True)
    assert np.array_equal(host(N.grad), want_dN)
    want_dE, _ = orc.sddmm_dot(host(g.coo[0]), host(g.coo[1]), Nq, dZq, sN, sdZ)
    assert np.array_equal(host(Ev.grad).reshape(E, H), want_dE)
