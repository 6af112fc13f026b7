"""GPU parity: the copy_u aggregation on an adjacency split into dense bit blocks (matrix cores) and a
sparse rest, against the CPU oracle's plain CSR aggregation.  Integer sums: bit-exact, whatever the split."""
import numpy as np
import pytest
import torch

from gpu_util import dev, host, sc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from tango_amd import kernels
    return kernels


def heavy_graph(rng, n, e, a=0.9, symmetric=True):
    """Power-law multigraph dense enough that the heavy rows x heavy columns corner is nearly full."""
    w = 1.0 / np.arange(1, n + 1) ** a
    w /= w.sum()
    s, d = rng.choice(n, e, p=w).astype(np.int64), rng.choice(n, e, p=w).astype(np.int64)
    if symmetric:
        s, d = np.concatenate([s, d]), np.concatenate([d, s])
    return s, d


def csr_of(rows, cols, n_rows):
    order = np.argsort(rows, kind="stable")
    indptr = np.zeros(n_rows + 1, np.int64)
    np.cumsum(np.bincount(rows, minlength=n_rows), out=indptr[1:])
    return indptr, cols[order].astype(np.int64)


def plan_for(indptr, indices, num_src, **kw):
    from tango_amd.dense_plan import build_dense_plan
    plan = build_dense_plan(dev(indptr), dev(indices.astype(np.int32)), num_src, **kw)
    assert plan is not None
    return plan


def decode_plan(plan):
    """The edges a plan stands for, (row, column) pairs with multiplicity, read from its bits and its rest with
    the layout include/tango_hip.h states (independent of the kernels)."""
    mask = host(plan.mask).view(np.uint32)
    off = host(plan.mask_off)
    row_slot = host(plan.row_slot)
    col_ids = host(plan.col_ids)
    row_of_rank = np.full(plan.row_blocks * 256, -1, np.int64)
    has = row_slot >= 0
    row_of_rank[row_slot[has]] = np.nonzero(has)[0]
    ends = list(off[1:]) + [mask.size]
    rr, cc = [], []
    for b in range(plan.row_blocks):
        words = mask[off[b]:ends[b]]
        idx = np.nonzero(words)[0]
        for bit in range(32):
            sel = idx[(words[idx] >> np.uint32(bit)) & np.uint32(1) == 1]
            if sel.size == 0:
                continue
            s4 = sel & 3
            lane = (sel >> 2) & 63
            q = (sel >> 8) & 1
            g = (sel >> 9) & 3
            u = sel >> 11
            bb, h, w = bit >> 3, (bit >> 2) & 1, bit & 3
            rank_r = b * 256 + 64 * g + 32 * h + (lane & 31)
            rank_c = 256 * u + 32 * (4 * q + s4) + 16 * (lane >> 5) + 4 * w + bb
            rr.append(row_of_rank[rank_r])
            cc.append(col_ids[rank_c].astype(np.int64))
    ip, ix = host(plan.res_indptr), host(plan.res_indices).astype(np.int64)
    rr.append(np.repeat(np.arange(plan.rows), np.diff(ip)))
    cc.append(ix)
    return np.concatenate(rr), np.concatenate(cc)


def test_plan_holds_every_edge_once():
    rng = np.random.default_rng(5)
    n = 3000
    s, d = heavy_graph(rng, n, 400_000)
    indptr, indices = csr_of(d, s, n)
    plan = plan_for(indptr, indices, n, tau=0.03, groups=6, min_extent=256)
    assert plan.row_blocks >= 2 and plan.shared_blocks.numel() >= 1
    assert plan.res_indices.numel() < 0.8 * indices.size  # the blocks took a good part of the slots
    rows, cols = decode_plan(plan)
    assert rows.min() >= 0
    want = np.sort(np.repeat(np.arange(n), np.diff(indptr)) * n + indices)
    assert np.array_equal(np.sort(rows * n + cols), want)
    # the rest lists a row's sources by falling popularity
    cnt = np.bincount(indices, minlength=n)
    ip, ix = host(plan.res_indptr), host(plan.res_indices)
    for r in rng.integers(0, n, 50):
        c = cnt[ix[ip[r]:ip[r + 1]]]
        assert np.all(np.diff(c) <= 0)


@pytest.mark.parametrize("F,ld", [(16, 16), (24, 32), (20, 48), (32, 32), (41, 48), (41, 64), (64, 64), (100, 112), (128, 128), (200, 208),
                                  (256, 256)])
def test_dense_copy_u_matches_oracle(K, orc, F, ld):
    rng = np.random.default_rng(F + ld)
    n = 2500
    s, d = heavy_graph(rng, n, 300_000)
    perm = rng.permutation(n)  # ranks do not follow the ids
    s, d = perm[s], perm[d]
    indptr, indices = csr_of(d, s, n)
    plan = plan_for(indptr, indices, n, tau=0.03, groups=5, min_extent=256)
    assert plan.shared_blocks.numel() >= 1
    feat = rng.integers(-127, 128, (n, ld)).astype(np.int8)  # columns past F are garbage that must be ignored
    scale = np.float32(0.0173)
    want = orc.spmm_csr_copy_u(indptr, indices, np.ascontiguousarray(feat[:, :F]), scale)
    out = torch.empty((n, F), dtype=torch.float32, device="cuda")
    assert K.cuda_kernels.csr_SPMM_dense(out, plan, dev(feat), sc(scale), ldf=ld, F=F)
    assert np.array_equal(host(out), want)
    # a second call reuses the workspace
    out.zero_()
    assert K.cuda_kernels.csr_SPMM_dense(out, plan, dev(feat), sc(scale), ldf=ld, F=F)
    assert np.array_equal(host(out), want)


@pytest.mark.parametrize("F", [41, 48, 256])
def test_dense_copy_u_epilogue_matches_oracle(K, orc, F):
    rng = np.random.default_rng(F)
    n = 2100
    s, d = heavy_graph(rng, n, 250_000, symmetric=False)
    indptr, indices = csr_of(d, s, n)
    plan = plan_for(indptr, indices, n, tau=0.02, groups=7, min_extent=512)
    ld = (F + 15) // 16 * 16
    feat = np.zeros((n, ld), np.int8)
    feat[:, :F] = rng.integers(-127, 128, (n, F))
    scale = np.float32(0.003)
    row_scale = rng.random(n).astype(np.float32)
    bias = rng.standard_normal(F).astype(np.float32)
    bits_ok = F % 16 == 0
    res = orc.spmm_csr_copy_u_ex(indptr, indices, np.ascontiguousarray(feat[:, :F]), scale, row_scale=row_scale,
                                 bias=bias, act=1, want_bits=bits_ok)
    want, bits = res if bits_ok else (res, None)
    out = torch.empty((n, F), dtype=torch.float32, device="cuda")
    sign = torch.empty((n, F // 16), dtype=torch.int16, device="cuda") if bits_ok else None
    assert K.cuda_kernels.csr_SPMM_dense(out, plan, dev(feat), sc(scale), ldf=ld, F=F, row_scale=dev(row_scale),
                                         bias=dev(bias), relu=True, sign_bits=sign)
    assert np.array_equal(host(out), want)
    if bits_ok:
        assert np.array_equal(host(sign).view(np.uint16), bits)


@pytest.mark.parametrize("F", [41, 256])
def test_dense_part_then_rest_is_the_whole_call(K, F):
    """tango_spmm_dense_partial followed by tango_spmm_dense_rest on the same workspace: the output of
    tango_spmm_csr_copy_u_dense, bit for bit, epilogue included."""
    from tango_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(F + 1)
    n = 2300
    s, d = heavy_graph(rng, n, 280_000)
    indptr, indices = csr_of(d, s, n)
    plan = plan_for(indptr, indices, n, tau=0.03, groups=6, min_extent=256)
    ld = (F + 15) // 16 * 16
    feat = dev(rng.integers(-127, 128, (n, ld)).astype(np.int8))
    scale, row_scale = sc(0.0021), dev(rng.random(n).astype(np.float32))
    bias = dev(rng.standard_normal(F).astype(np.float32))
    whole = torch.empty((n, F), dtype=torch.float32, device="cuda")
    assert K.cuda_kernels.csr_SPMM_dense(whole, plan, feat, scale, ldf=ld, F=F, row_scale=row_scale, bias=bias, relu=True)
    nbytes = L.tango_spmm_dense_workspace(plan.ref, F)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    parts = torch.full((n, F), float("nan"), device="cuda")
    _lib.check(L.tango_spmm_dense_partial(plan.ref, feat.data_ptr(), ld, F, ws.data_ptr(), nbytes, st), "partial")
    for _ in range(2):  # the partial sums stay in the workspace: the second part can run again
        _lib.check(L.tango_spmm_dense_rest(parts.data_ptr(), plan.ref, feat.data_ptr(), ld, scale.data_ptr(),
                                           row_scale.data_ptr(), bias.data_ptr(), 1, None, F, ws.data_ptr(), nbytes, st), "rest")
        assert torch.equal(parts, whole)
    assert L.tango_spmm_dense_rest(parts.data_ptr(), plan.ref, feat.data_ptr(), ld, scale.data_ptr(), None, None, 0, None, F,
                                   ws.data_ptr(), 16, st) != 0  # workspace too small: refused


@pytest.mark.parametrize("F", [41, 256])
def test_dense_plan_whose_hub_rows_keep_long_rests(K, orc, F):
    """A high threshold leaves the hub rows thousands of slots outside the blocks: the rows-per-wavefront kernel
    passes them over and the kernel for long rows sums them; the result is the oracle's all the same."""
    rng = np.random.default_rng(F + 3)
    n = 2600
    s, d = heavy_graph(rng, n, 320_000)
    perm = rng.permutation(n)
    s, d = perm[s], perm[d]
    indptr, indices = csr_of(d, s, n)
    plan = plan_for(indptr, indices, n, tau=0.45, groups=4, min_extent=256, min_share=0.0)
    assert plan.res_max_row > 4096
    ld = (F + 15) // 16 * 16
    feat = rng.integers(-127, 128, (n, ld)).astype(np.int8)
    scale = np.float32(0.0007)
    want = orc.spmm_csr_copy_u(indptr, indices, np.ascontiguousarray(feat[:, :F]), scale)
    out = torch.empty((n, F), dtype=torch.float32, device="cuda")
    assert K.cuda_kernels.csr_SPMM_dense(out, plan, dev(feat), sc(scale), ldf=ld, F=F)
    assert np.array_equal(host(out), want)


def test_dense_copy_u_bipartite_and_repeated_edges(K, orc):
    rng = np.random.default_rng(11)
    n_dst, n_src = 1500, 4000
    wd = 1.0 / np.arange(1, n_dst + 1) ** 0.8
    ws = 1.0 / np.arange(1, n_src + 1) ** 0.8
    e = 300_000
    d = rng.choice(n_dst, e, p=wd / wd.sum()).astype(np.int64)
    s = rng.choice(n_src, e, p=ws / ws.sum()).astype(np.int64)
    # every edge of the heaviest corner three times over
    hot = (d < 64) & (s < 64)
    d, s = np.concatenate([d, d[hot], d[hot]]), np.concatenate([s, s[hot], s[hot]])
    indptr, indices = csr_of(d, s, n_dst)
    plan = plan_for(indptr, indices, n_src, tau=0.02, groups=3, min_extent=256)
    feat = rng.integers(-127, 128, (n_src, 128)).astype(np.int8)
    scale = np.float32(0.5)
    out = torch.empty((n_dst, 128), dtype=torch.float32, device="cuda")
    assert K.cuda_kernels.csr_SPMM_dense(out, plan, dev(feat), sc(scale))
    assert np.array_equal(host(out), orc.spmm_csr_copy_u(indptr, indices, feat, scale))


def test_graph_level_wrapper_uses_the_plan(K, orc):
    from tango_amd.dense_plan import build_dense_plan
    from tango_amd.graph import Graph
    from tango_amd.util import graph_preprocess
    rng = np.random.default_rng(2)
    n = 2000
    s, d = heavy_graph(rng, n, 200_000, symmetric=False)
    g = graph_preprocess(Graph(dev(s), dev(d), n))
    assert g.dense_csc is None  # small graphs get no plan on their own
    g.dense_csc = build_dense_plan(g.adj_csc[0], g.adj_csc32[0], n, tau=0.02, groups=4, min_extent=256)
    g.dense_csr = build_dense_plan(g.adj_csr[0], g.adj_csr32[0], n, tau=0.02, groups=4, min_extent=256)
    assert g.dense_csc is not None and g.dense_csr is not None
    o = orc.graph_formats(s, d, n)
    feat = rng.integers(-127, 128, (n, 64)).astype(np.int8)
    for reverse, fmt in ((False, "adj_csc"), (True, "adj_csr")):
        got = K.csr_SPMM(g, dev(feat), sc(0.01), reverse=reverse)
        assert np.array_equal(host(got), orc.spmm_csr_copy_u(o[fmt][0], o[fmt][1], feat, np.float32(0.01)))


@pytest.mark.parametrize("with_plan", [False, True])
@pytest.mark.parametrize("F,use_mul", [(256, True), (41, False), (64, True)])
def test_aggregation_returns_the_scale_of_its_output(K, orc, F, use_mul, with_plan):
    """The scale an aggregation's epilogue finds for its own output is max|out * mul| / 127 of the stored values."""
    from tango_amd.dense_plan import build_dense_plan
    from tango_amd.graph import Graph
    from tango_amd.util import graph_preprocess
    rng = np.random.default_rng(F)
    n = 2200
    s, d = heavy_graph(rng, n, 220_000, symmetric=False)
    g = graph_preprocess(Graph(dev(s), dev(d), n))
    if with_plan:
        g.dense_csc = build_dense_plan(g.adj_csc[0], g.adj_csc32[0], n, tau=0.02, groups=4, min_extent=256)
        assert g.dense_csc is not None
    ld = (F + 15) // 16 * 16
    feat = np.zeros((n, ld), np.int8)
    feat[:, :F] = rng.integers(-127, 128, (n, F))
    row_scale = rng.random(n).astype(np.float32)
    bias = rng.standard_normal(F).astype(np.float32)
    mul = (rng.random(n).astype(np.float32) + 0.5) if use_mul else None
    fd = dev(feat)[:, :F]
    out, scale = K.csr_SPMM(g, fd, sc(0.02), row_scale=dev(row_scale), bias=dev(bias), relu=True, want_scale=True,
                            scale_mul=None if mul is None else dev(mul))
    o = orc.graph_formats(s, d, n)
    want = orc.spmm_csr_copy_u_ex(o["adj_csc"][0], o["adj_csc"][1], np.ascontiguousarray(feat[:, :F]), np.float32(0.02),
                                  row_scale=row_scale, bias=bias, act=1)
    assert np.array_equal(host(out), want)
    want_scale, _ = orc.absmax_ex(want, row_mul=mul)
    assert host(scale)[0] == want_scale and want_scale > 0


def test_gcn_scale_hand_off_changes_nothing(K, monkeypatch):
    """A 2-layer GCN step on a dense graph with the scales handed from the aggregations' epilogues to the next
    quantizers (forward and backward) gives the same logits and gradients, bit for bit, as with the separate
    absmax passes."""
    from tango_amd import SPMM, config
    from tango_amd.gcn import GCN
    from tango_amd.graph import Graph
    from tango_amd.loss import cross_entropy
    from tango_amd.util import graph_preprocess
    rng = np.random.default_rng(3)
    n = 2048
    s, d = heavy_graph(rng, n, 150_000)
    g = graph_preprocess(Graph(dev(s), dev(d), n))
    X = torch.randn(n, 96, device="cuda")
    labels = torch.randint(0, 7, (n,), device="cuda")
    saved = config.grad_round_mode
    config.grad_round_mode = "rne"
    monkeypatch.setattr(config, "scale_from_aggregation", True)
    calls = []
    for name in ("get_scale", "absmax_ex"):
        raw = getattr(K.cuda_kernels, name)
        monkeypatch.setattr(K.cuda_kernels, name, staticmethod(
            lambda *a, _raw=raw, _n=name, **kw: (calls.append((_n, tuple(a[0].shape))), _raw(*a, **kw))[1]))
    try:
        res, passes = [], []
        for fused in (True, False):
            if not fused:
                monkeypatch.setattr(SPMM, "_dense_enough", lambda g, reverse=False: False)
            torch.manual_seed(0)
            model = GCN(g, 96, 32, 7, 1, torch.relu, 0.0).cuda()
            del calls[:]
            logits = model(X)
            cross_entropy(logits, labels).backward()
            passes.append([c for c in calls if c[1][0] == n])  # scans of node tensors (not of the weights)
            res.append([logits.detach().clone()] + [p.grad.clone() for p in model.parameters()])
        for a, b in zip(*res):
            assert torch.equal(a, b)
        # gone with the hand-off: the scan of layer 2's input and of the two reverse aggregations' outputs
        assert len(passes[1]) - len(passes[0]) == 3, (passes[0], passes[1])
    finally:
        config.grad_round_mode = saved
