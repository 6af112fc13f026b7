"""GPU tests of the layer-glue fusion: the fused prologue / epilogue entry points
perform the same sequence of fp32 roundings as the separate passes they replace,
so results must be bit-identical (bias gradient: summation order differs, tolerance)."""
import numpy as np
import pytest
import torch

from gpu_util import dev, host, rand_graph, sc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from tango_amd import kernels
    return kernels


def make_graph(src, dst, n):
    from tango_amd.graph import Graph
    from tango_amd.util import graph_preprocess
    return graph_preprocess(Graph(dev(src), dev(dst), n))


def test_absmax_ex_and_quantize_ex(K, orc):
    rng = np.random.default_rng(0)
    for rows, cols in ((1000, 256), (777, 41), (300, 602), (5, 1024), (64, 1500), (3, 7), (200, 48)):
        x = rng.standard_normal((rows, cols)).astype(np.float32)
        rm = rng.random(rows, dtype=np.float32) + 0.1
        mask = rng.standard_normal((rows, cols)).astype(np.float32)
        masked = np.where(mask > 0, x, 0).astype(np.float32)
        scaled = (masked * rm[:, None]).astype(np.float32)
        s, cs = K.cuda_kernels.absmax_ex(dev(x), row_mul=dev(rm), mask=dev(mask), want_colsum=True)
        assert host(s)[0] == orc.absmax_scale(scaled)
        assert np.allclose(host(cs), masked.astype(np.float64).sum(0), rtol=1e-5, atol=1e-3)
        s2, none = K.cuda_kernels.absmax_ex(dev(x))
        assert none is None and host(s2)[0] == orc.absmax_scale(x)
        q, s3 = K.quantize_padded(dev(x), row_mul=dev(rm), mask=dev(mask))
        assert host(s3)[0] == host(s)[0]
        assert np.array_equal(host(q), orc.quantize(scaled, host(s)[0]))
        for off in (64, 66):  # a lane's four elements inside one block of the random stream / across two
            q2, _ = K.quantize_padded(dev(x), s, row_mul=dev(rm), mask=dev(mask), round_mode="stochastic", seed=3, offset=off)
            assert np.array_equal(host(q2), orc.quantize(scaled, host(s)[0], orc.STOCHASTIC, seed=3, offset=off))
        # ELU backward: elements whose mask (the activation's output) is not positive are multiplied by mask + 1
        emask = np.where(mask > 0, mask, np.expm1(mask)).astype(np.float32)
        through = np.where(emask > 0, x, x * (emask + np.float32(1))).astype(np.float32)
        scaled = (through * rm[:, None]).astype(np.float32)
        s, cs = K.cuda_kernels.absmax_ex(dev(x), row_mul=dev(rm), mask=dev(emask), want_colsum=True, mask_mode="elu")
        assert host(s)[0] == orc.absmax_scale(scaled)
        assert np.allclose(host(cs), through.astype(np.float64).sum(0), rtol=1e-5, atol=1e-3)
        q, _ = K.quantize_padded(dev(x), s, row_mul=dev(rm), mask=dev(emask), mask_mode="elu")
        assert np.array_equal(host(q), orc.quantize(scaled, host(s)[0]))
        if cols % 16 == 0:
            # the same ReLU mask as sign bits, sixteen columns per 16-bit word
            bits = np.packbits((mask > 0).reshape(rows, cols // 16, 16), axis=-1, bitorder="little").view(np.int16)
            bits = dev(np.ascontiguousarray(bits.reshape(rows, cols // 16)))
            sb, csb = K.cuda_kernels.absmax_ex(dev(x), row_mul=dev(rm), mask=bits, want_colsum=True, mask_mode="bits")
            s0, cs0 = K.cuda_kernels.absmax_ex(dev(x), row_mul=dev(rm), mask=dev(mask), want_colsum=True)
            assert torch.equal(sb, s0) and torch.equal(csb, cs0)
            for kw in ({}, {"round_mode": "stochastic", "seed": 3, "offset": 64}):
                qb, _ = K.quantize_padded(dev(x), s0, row_mul=dev(rm), mask=bits, mask_mode="bits", **kw)
                q0, _ = K.quantize_padded(dev(x), s0, row_mul=dev(rm), mask=dev(mask), **kw)
                assert torch.equal(qb, q0)
                qb, _ = K.quantize_padded(dev(x), s0, mask=bits, mask_mode="bits", align=64, **kw)  # row-strided kernel
                q0, _ = K.quantize_padded(dev(x), s0, mask=dev(mask), align=64, **kw)
                assert torch.equal(qb, q0)
    # colsum is deterministic run to run
    x = dev(rng.standard_normal((50000, 256)).astype(np.float32))
    a = K.cuda_kernels.absmax_ex(x, want_colsum=True)[1]
    b = K.cuda_kernels.absmax_ex(x, want_colsum=True)[1]
    assert torch.equal(a, b)


@pytest.mark.parametrize("rows,cols", [(1001, 602), (333, 602), (2000, 86), (40000, 2)])
def test_absmax_with_row_multiplier_on_dense_rows_of_even_length(K, orc, rows, cols):
    """Rows whose length is even but not a multiple of four floats are read as one flat array of 16-byte
    vectors (a vector may end in the next row); an odd row count leaves a two-element tail."""
    rng = np.random.default_rng(rows + cols)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    rm = (rng.random(rows, dtype=np.float32) + 0.1) * np.where(rng.random(rows) < 0.01, 50, 1).astype(np.float32)
    s, cs = K.cuda_kernels.absmax_ex(dev(x), row_mul=dev(rm))
    assert cs is None and host(s)[0] == orc.absmax_scale((x * rm[:, None]).astype(np.float32))


# (n, e): rows of ~66 slots (one wave per row), and a sparse graph with a long row and a hub row (the epilogue
# also runs in the sixteen-wave kernel and in the hub store pass)
@pytest.mark.parametrize("n,e", [(600, 40000), (5000, 40000), (3000, 9000)])
@pytest.mark.parametrize("F", [16, 41, 256])
def test_spmm_fused_epilogue_matches_oracle(K, orc, F, n, e):
    """The aggregation with '* row_scale, + bias, activation, sign bits' in its epilogue against the oracle's
    fused form, on rows of ~66 slots (one wave per row), on a sparse graph with a long row and a hub row (the
    epilogue also runs in the sixteen-wave kernel and in the hub store pass) and on a very sparse graph (the
    slot-span kernels)."""
    rng = np.random.default_rng(F)
    src, dst = rand_graph(rng, n, e)
    if n == 5000:
        dst[:9000] = 5
        dst[9000:10500] = 6
    g = make_graph(src, dst, n)
    ip, ix = host(g.adj_csc[0]), host(g.adj_csc[1])
    feat = rng.integers(-127, 128, (n, F)).astype(np.int8)
    rs = rng.random(n, dtype=np.float32) + 0.05
    bias = rng.standard_normal(F).astype(np.float32)
    s = np.float32(0.0173)
    for kw in ({}, {"row_scale": rs}, {"bias": bias}, {"act": 1}, {"row_scale": rs, "bias": bias, "act": 1}):
        want = orc.spmm_csr_copy_u_ex(ip, ix, feat, s, **kw)
        dkw = {k: dev(v) for k, v in kw.items() if k != "act"}
        got = K.csr_SPMM(g, dev(feat), sc(s), relu=bool(kw.get("act")), **dkw)
        assert np.array_equal(host(got), want), sorted(kw)
    if F % 16 == 0:  # the epilogue also writes the signs of its output, sixteen columns per word
        want, wbits = orc.spmm_csr_copy_u_ex(ip, ix, feat, s, row_scale=rs, bias=bias, act=1, want_bits=True)
        bits = torch.full((n, F // 16), -1, dtype=torch.int16, device="cuda")
        got = K.csr_SPMM(g, dev(feat), sc(s), row_scale=dev(rs), bias=dev(bias), relu=True, sign_bits=bits)
        assert np.array_equal(host(got), want)
        assert np.array_equal(host(bits).view(np.uint16), wbits)


def test_gemm_row_scale_prologue_and_gradx_epilogue(K, orc):
    rng = np.random.default_rng(1)
    M, Kd, N = 700, 602, 41
    X = rng.standard_normal((M, Kd)).astype(np.float32)
    W = (rng.random((N, Kd), dtype=np.float32) - 0.5) * 0.2
    rm = rng.random(M, dtype=np.float32) + 0.1
    Xs = (X * rm[:, None]).astype(np.float32)
    sX, _ = K.cuda_kernels.absmax_ex(dev(X), row_mul=dev(rm))
    sW = K.cuda_kernels.get_scale(dev(W))
    Xq = torch.empty((M, 608), dtype=torch.int8, device="cuda")[:, :Kd]
    Wq = torch.empty((N, Kd), dtype=torch.int8, device="cuda")
    Y, sY = K.QGEMM_forward(dev(X), Xq, sX, dev(W), Wq, sW, None, True, x_row_mul=dev(rm))
    Yo, Xqo, _, osX, _, osY = orc.qgemm_fwd(Xs, W, reduce=True)
    assert host(sX)[0] == osX and np.array_equal(host(Xq), Xqo) and np.array_equal(host(Y), Yo) and host(sY)[0] == osY
    dY = rng.integers(-127, 128, (M, N)).astype(np.int8)
    dX, _ = K.QGEMM_backward(dev(dY), Xq, Wq, sc(0.01), sX, sW, True, False, x_row_scale=dev(rm))
    want = (orc.qgemm_bwd_dx(dY, host(Wq), 0.01, host(sW)[0]) * rm[:, None]).astype(np.float32)
    assert np.array_equal(host(dX), want)


@pytest.mark.parametrize("dims", [(100, 32, 7), (64, 16, 16), (16, 48, 64), (41, 128, 128)])
def test_fused_gcn_matches_unfused(dims):
    from tango_amd.gcn import GCN
    from tango_amd.graph import chung_lu
    from tango_amd.util import graph_preprocess
    g = graph_preprocess(chung_lu(2500, 30000, 2.1, seed=2, symmetric=True, device="cuda"))
    fin, hid, ncls = dims
    torch.manual_seed(0)
    a = GCN(g, fin, hid, ncls, 1, torch.relu, 0.0, fused=True).cuda()
    b = GCN(g, fin, hid, ncls, 1, torch.relu, 0.0, fused=False).cuda()
    b.load_state_dict(a.state_dict())
    for m in (a, b):
        for layer in m.layers:
            torch.nn.init.normal_(layer.bias, std=0.1)
    b.load_state_dict(a.state_dict())
    x = torch.randn(2500, fin, device="cuda")
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    ya, yb = a(xa), b(xb)
    assert torch.equal(ya, yb)
    w = torch.randn_like(ya)
    ya.backward(w)
    yb.backward(w)
    assert torch.equal(xa.grad, xb.grad)
    for (name, pa), (_, pb) in zip(a.named_parameters(), b.named_parameters()):
        if name.endswith("bias"):
            assert torch.allclose(pa.grad, pb.grad, rtol=1e-4, atol=1e-4), name
        else:
            assert torch.equal(pa.grad, pb.grad), name


@pytest.mark.parametrize("rows,classes", [(1000, 41), (4097, 7), (300, 256), (17, 3), (5, 1)])
def test_cross_entropy_matches_torch(rows, classes):
    from tango_amd.loss import cross_entropy
    torch.manual_seed(rows)
    x = (torch.randn(rows, classes, device="cuda") * 3).requires_grad_(True)
    y = torch.randint(0, classes, (rows,), device="cuda")
    loss = cross_entropy(x, y)
    xr = x.detach().clone().requires_grad_(True)
    ref = torch.nn.functional.cross_entropy(xr, y)
    assert torch.allclose(loss, ref, rtol=1e-5, atol=1e-6)
    (loss * 2.5).backward()
    (ref * 2.5).backward()
    assert torch.allclose(x.grad, xr.grad, rtol=1e-5, atol=1e-8)
    # deterministic
    assert cross_entropy(x.detach(), y).item() == cross_entropy(x.detach(), y).item()


@pytest.mark.parametrize("n,H,D", [(1000, 8, 16), (333, 3, 5), (50, 1, 64), (2049, 12, 20), (7, 70, 4),
                                   (70000, 8, 16), (169343, 1, 40), (3001, 1, 41), (500, 3, 101), (300, 2, 640), (2000, 3, 250), (400, 2, 129)])
def test_attn_scores_match_torch(K, n, H, D):
    """fp32 kernel against the torch expression it replaces; only the summation order differs.  The form that
    also hands out the scales (a few large workgroups walking the items with a grid stride; the last case has
    more items than threads in that launch) writes the same el / er bit for bit, and its scales are
    max|.| / 127 of what it wrote.  The backward reads rows the way they lie in memory (column quads when D is a
    multiple of 4, pairs when it is even, else single columns; rows of more than 256 such groups are cut into
    column chunks: the last three cases)."""
    g = torch.Generator().manual_seed(n + H)
    feat = torch.randn(n, H, D, generator=g).cuda()
    al = torch.randn(1, H, D, generator=g).cuda()
    ar = torch.randn(1, H, D, generator=g).cuda()
    el, er = K.cuda_kernels.attn_scores_forward(feat, al.contiguous(), ar.contiguous())
    tol = 1e-5 * max(1.0, D / 64)  # fp32 sums over D terms in another order
    assert torch.allclose(el, (feat * al).sum(-1), rtol=1e-5, atol=tol)
    assert torch.allclose(er, (feat * ar).sum(-1), rtol=1e-5, atol=tol)
    el2, er2, s_el, s_er = K.cuda_kernels.attn_scores_forward(feat, al.contiguous(), ar.contiguous(), want_scales=True)
    assert torch.equal(el2, el) and torch.equal(er2, er)
    assert torch.equal(s_el, K.cuda_kernels.get_scale(el)) and torch.equal(s_er, K.cuda_kernels.get_scale(er))
    dl = torch.randn(n, H, generator=g).cuda()
    dr = torch.randn(n, H, generator=g).cuda()
    dfeat, dal, dar = K.cuda_kernels.attn_scores_backward(dl, dr, feat, al.contiguous(), ar.contiguous())
    want = dl.unsqueeze(-1) * al + dr.unsqueeze(-1) * ar
    assert torch.equal(dfeat, want)  # two products and one sum per element, same roundings
    f64 = feat.double()
    atol = 1e-4 * max(1.0, n / 2000)  # fp32 sums over n terms
    assert torch.allclose(dal.double(), (dl.double().unsqueeze(-1) * f64).sum(0), rtol=1e-5, atol=atol)
    assert torch.allclose(dar.double(), (dr.double().unsqueeze(-1) * f64).sum(0), rtol=1e-5, atol=atol)
    # with the gradient of feat's other consumer folded in: the sum autograd would form, and its scale
    other = torch.randn(n, H, D, generator=g).cuda() * 0.7
    dsum, dal2, dar2, s = K.cuda_kernels.attn_scores_backward(dl, dr, feat, al.contiguous(), ar.contiguous(), addend=other)
    assert torch.equal(dsum, other + dfeat)
    assert torch.equal(dal2, dal) and torch.equal(dar2, dar)
    assert torch.equal(s, K.cuda_kernels.get_scale(dsum))


def test_attn_scores_pass_through_collects_both_gradients():
    """feat read by the logits and, through the node's fifth result, by a second consumer: the gradient that reaches
    feat is the sum autograd forms when the two read feat directly, bit for bit, and it carries its scale."""
    from tango_amd.SPMM import grad_scale_hint
    from tango_amd.gat import attn_scores
    g = torch.Generator().manual_seed(6)
    n, H, D = 5000, 8, 16
    base = torch.randn(n, H, D, generator=g).cuda()
    al = torch.randn(1, H, D, generator=g).cuda().requires_grad_()
    ar = torch.randn(1, H, D, generator=g).cuda().requires_grad_()
    w1, w2 = torch.randn(n, H, 1, generator=g).cuda(), torch.randn(n, H, 1, generator=g).cuda()
    w3 = torch.randn(n, H, D, generator=g).cuda()
    grads, seen = [], []
    for through in (False, True):
        feat = base.clone().requires_grad_()
        feat2 = feat * 1.0  # a non-leaf, so that a hook sees the gradient tensor the node returns
        feat2.register_hook(lambda t: seen.append((t, grad_scale_hint(t))))
        out = attn_scores.apply(feat2, al, ar, through)
        second = out[4] if through else feat2
        ((out[0] * w1).sum() + (out[1] * w2).sum() + (second * second * w3).sum()).backward()
        grads.append([t.grad.clone() for t in (feat, al, ar)])
        al.grad = ar.grad = None
    for a, b in zip(*grads):
        assert torch.equal(a, b)
    assert seen[0][1] is None  # autograd's own sum carries no scale
    t, s = seen[1]
    assert s is not None and torch.equal(s, t.abs().max().reshape(1) / 127)
    # one consumer only: nothing to add, the plain kernel runs
    feat = base.clone().requires_grad_()
    out = attn_scores.apply(feat, al, ar, True)
    ((out[0] * w1).sum() + (out[1] * w2).sum()).backward()
    assert torch.equal(feat.grad, w1 * al.detach() + w2 * ar.detach())
    feat.grad = None
    out = attn_scores.apply(feat, al, ar, True)
    (out[4] * w3).sum().backward()  # the logits unused: the second consumer's gradient passes through
    assert torch.equal(feat.grad, w3)


def test_attn_scores_autograd_matches_torch():
    from tango_amd.gat import attn_scores
    g = torch.Generator().manual_seed(5)
    feat = torch.randn(400, 4, 8, generator=g).cuda().requires_grad_()
    al = torch.randn(1, 4, 8, generator=g).cuda().requires_grad_()
    ar = torch.randn(1, 4, 8, generator=g).cuda().requires_grad_()
    w1, w2 = torch.randn(400, 4, 1, generator=g).cuda(), torch.randn(400, 4, 1, generator=g).cuda()
    el, er, s_el, s_er = attn_scores.apply(feat, al, ar)
    assert not s_el.requires_grad and torch.equal(s_el, el.detach().abs().max().reshape(1) / 127)
    assert torch.equal(s_er, er.detach().abs().max().reshape(1) / 127)
    ((el * w1).sum() + (er * w2).sum()).backward()
    got = [t.grad.clone() for t in (feat, al, ar)]
    for t in (feat, al, ar):
        t.grad = None
    el2 = (feat * al).sum(-1).unsqueeze(-1)
    er2 = (feat * ar).sum(-1).unsqueeze(-1)
    ((el2 * w1).sum() + (er2 * w2).sum()).backward()
    for a, b in zip(got, (feat.grad, al.grad, ar.grad)):
        assert a.shape == b.shape and torch.allclose(a, b, rtol=1e-4, atol=1e-4)


def test_u_mul_e_bias_epilogue(K):
    """bias in the SpMM epilogue == separate add (same roundings); its gradient == column sums of dZ."""
    from tango_amd.SPMM import spmm_u_mul_e
    rng = np.random.default_rng(9)
    n, e, H, F = 700, 9000, 4, 16
    src, dst = rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    N = dev(rng.standard_normal((n, H, F)).astype(np.float32)).requires_grad_()
    E = dev(rng.random((e, H, 1)).astype(np.float32)).requires_grad_()
    bias = dev(rng.standard_normal(H * F).astype(np.float32)).requires_grad_()
    dZ = dev(rng.standard_normal((n, H, F)).astype(np.float32))
    out = spmm_u_mul_e.apply(g, N, E, bias)
    out.backward(dZ)
    got = [t.grad.clone() for t in (N, E, bias)]
    for t in (N, E, bias):
        t.grad = None
    ref = spmm_u_mul_e.apply(g, N, E) + bias.view(1, H, F)
    assert torch.equal(out, ref)
    ref.backward(dZ)
    assert torch.equal(got[0], N.grad) and torch.equal(got[1], E.grad)
    assert torch.allclose(got[2], bias.grad, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("act", ["relu", "elu"])
@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("n,e,H,F", [(700, 9000, 4, 16), (300, 40000, 3, 5)])
def test_u_mul_e_activation_epilogue(K, act, with_bias, n, e, H, F):
    """Activation in the SpMM epilogue == a separate pass over its output; in the backward pass the
    activation's derivative applied inside the scale and quantize kernels == applied to dZ beforehand."""
    from tango_amd.SPMM import spmm_u_mul_e
    rng = np.random.default_rng(10)
    src, dst = rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    N = dev(rng.standard_normal((n, H, F)).astype(np.float32)).requires_grad_()
    E = dev(rng.random((e, H, 1)).astype(np.float32)).requires_grad_()
    bias = dev(rng.standard_normal(H * F).astype(np.float32)).requires_grad_() if with_bias else None
    leaves = [t for t in (N, E, bias) if t is not None]
    dZ = dev(rng.standard_normal((n, H, F)).astype(np.float32))
    out = spmm_u_mul_e.apply(g, N, E, bias, None, act)
    out.backward(dZ)
    got = [t.grad.clone() for t in leaves]
    for t in leaves:
        t.grad = None
    pre = spmm_u_mul_e.apply(g, N, E, bias)
    if act == "relu":
        assert torch.equal(out, torch.relu(pre))
        back = torch.where(out > 0, dZ, torch.zeros_like(dZ))
    else:
        # the epilogue computes exp(y) - 1 with the hardware exponential: absolute error ~1e-7 where y <= 0
        assert torch.allclose(out, torch.nn.functional.elu(pre), rtol=1e-6, atol=5e-7)
        assert torch.equal(out > 0, pre > 0)
        back = torch.where(out > 0, dZ, dZ * (out.detach() + 1.0))
    pre.backward(back)
    assert torch.equal(got[0], N.grad) and torch.equal(got[1], E.grad)
    if with_bias:
        assert torch.allclose(got[2], bias.grad, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("act", [torch.nn.functional.elu, torch.relu])
def test_gat_layer_with_folded_activation_tracks_torch_activation(act):
    """A GAT layer whose activation rides in the aggregation's epilogue against the same layer with the
    activation as a torch op on the aggregation's output (forward equal, gradients within int8 noise:
    the torch path quantizes dZ after a separate fp32 pass whose exp differs in the last bits)."""
    from tango_amd.gat import QGATConv
    rng = np.random.default_rng(12)
    n, e = 2000, 24000
    src, dst = rand_graph(rng, n, e)
    loops = np.arange(n)
    g = make_graph(np.concatenate([src, loops]), np.concatenate([dst, loops]), n)
    torch.manual_seed(3)
    layer = QGATConv(48, 16, 4, activation=act).cuda()
    x = dev(rng.standard_normal((n, 48)).astype(np.float32)).requires_grad_()
    w = dev(rng.standard_normal((n, 4, 16)).astype(np.float32))
    outs, grads = [], []
    for fold in (True, False):
        layer.zero_grad()
        x.grad = None
        layer.activation = act if fold else (lambda t: act(t))  # an unknown callable is not folded
        y = layer(g, x)
        y.backward(w)
        outs.append(y.detach().clone())
        grads.append([p.grad.clone() for p in layer.parameters()] + [x.grad.clone()])
    assert torch.allclose(outs[0], outs[1], rtol=1e-6, atol=5e-7)
    for a, b in zip(*grads):
        assert torch.allclose(a, b, rtol=1e-3, atol=2e-2 * float(b.abs().max()))


def test_scale_hand_off_is_bit_identical(K):
    """A layer fed the preceding GEMM epilogue's scale computes what it computes when it
    runs its own absmax pass (the epilogue's max is over the stored fp32 outputs)."""
    from tango_amd.QLinear import QLinear
    torch.manual_seed(3)
    x = torch.randn(3000, 96, device="cuda")
    l1, l2 = QLinear(96, 128).cuda(), QLinear(128, 64).cuda()
    ref = l2(l1(x))
    l1.enable_reduce()
    y, s = l1(x)
    assert torch.equal(s, K.cuda_kernels.get_scale(y))
    got = l2(y, s)
    assert torch.equal(got, ref)
    got.sum().backward()
    g1 = [p.grad.clone() for p in list(l1.parameters()) + list(l2.parameters())]
    for p in list(l1.parameters()) + list(l2.parameters()):
        p.grad = None
    l1.isReduce = False
    l2(l1(x)).sum().backward()
    for a, p in zip(g1, list(l1.parameters()) + list(l2.parameters())):
        assert torch.equal(a, p.grad)


@pytest.mark.parametrize("Kd,N,mode,bias", [(130, 16, "rne", True), (602, 29, "trunc", False), (64, 7, "trunc", True)])
def test_forward_gemm_tall_narrow(K, orc, Kd, N, mode, bias):
    """Tall X with N <= 32 takes the W-stationary kernel (rows dealt over persistent waves, X quantized
    in registers): row multiplier, bias, both deterministic rounding modes, 8- and 16-byte aligned rows,
    a partial last k-step and a row count that is no multiple of the 16-row block."""
    rng = np.random.default_rng(Kd + N)
    M = 50011
    X = rng.standard_normal((M, Kd)).astype(np.float32)
    W = ((rng.random((N, Kd), dtype=np.float32) - 0.5) * 0.3).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32) if bias else None
    rm = (rng.random(M, dtype=np.float32) + 0.1).astype(np.float32)
    Xs = (X * rm[:, None]).astype(np.float32)
    sX, _ = K.cuda_kernels.absmax_ex(dev(X), row_mul=dev(rm))
    sW = K.cuda_kernels.get_scale(dev(W))
    ld = (Kd + 15) // 16 * 16
    Xq = torch.empty((M, ld), dtype=torch.int8, device="cuda")[:, :Kd]
    Wq = torch.empty((N, Kd), dtype=torch.int8, device="cuda")
    Y, sY = K.QGEMM_forward(dev(X), Xq, sX, dev(W), Wq, sW, None if b is None else dev(b), True,
                            round_mode=mode, x_row_mul=dev(rm))
    Yo, Xqo, _, osX, _, osY = orc.qgemm_fwd(Xs, W, b, reduce=True, mode=orc.RNE if mode == "rne" else orc.TRUNC)
    assert host(sX)[0] == osX and np.array_equal(host(Xq), Xqo)
    assert np.array_equal(host(Y), Yo) and host(sY)[0] == osY


@pytest.mark.parametrize("M,Kd,N", [(3000, 256, 256), (1000, 100, 41), (500, 602, 64)])
def test_linear_layers_sharing_one_quantized_input(M, Kd, N):
    """QLinear fed the already quantized input (one quantize pass shared by several layers, as the q / k / v
    projections of the HGT layer use it) == QLinear quantizing the input itself: outputs, output scales and
    all gradients bit for bit."""
    from tango_amd.QLinear import QLinear, quantize_input
    torch.manual_seed(M + N)
    a, b = QLinear(Kd, N).cuda(), QLinear(Kd, N, bias=False).cuda()
    a.enable_reduce()
    x = torch.randn(M, Kd, device="cuda", requires_grad=True)
    w = torch.randn(M, N, device="cuda")
    outs, grads = [], []
    for shared in (False, True):
        for t in (x, *a.parameters(), *b.parameters()):
            t.grad = None
        if shared:
            xq, sx = quantize_input(x.detach())
            (ya, sa), yb = a(x, sx, xq), b(x, sx, xq)
        else:
            (ya, sa), yb = a(x), b(x)
        ((ya * w).sum() + (yb * w).sum() * 0.5).backward()
        outs.append((ya.detach().clone(), sa.clone(), yb.detach().clone()))
        grads.append([t.grad.clone() for t in (x, *a.parameters(), *b.parameters())])
    assert all(torch.equal(p, q) for p, q in zip(*outs))
    assert all(torch.equal(p, q) for p, q in zip(*grads))


@pytest.mark.parametrize("M,Kd,N", [(3000, 256, 256), (1000, 100, 41), (700, 602, 300)])
def test_shared_input_linears_accumulate_one_input_gradient(M, Kd, N):
    """Three layers over one input as a single autograd node == the three layers on their own: outputs, output
    scales, weight and bias gradients bit for bit, and the input gradient equal to the layers' input gradients
    added in layer order (the node's GEMM epilogues add in that order).  One layer's output is left unused in
    a second pass: its gradients stay None and the other two still add up."""
    from tango_amd.QLinear import QLinear, shared_input_linears
    torch.manual_seed(M + N + 1)
    lins = [QLinear(Kd, N).cuda(), QLinear(Kd, N, bias=False).cuda(), QLinear(Kd, N).cuda()]
    for lin in lins:
        lin.enable_reduce()
    params = [p for lin in lins for p in lin.parameters()]
    x = torch.randn(M, Kd, device="cuda", requires_grad=True)
    ws = [torch.randn(M, N, device="cuda") for _ in lins]
    for used in ((0, 1, 2), (0, 2)):
        want_y, want_dx, want_dp = [], None, []
        for i, lin in enumerate(lins):
            y, s = lin(x)
            want_y.append((y.detach().clone(), s.clone()))
            if i in used:
                g = torch.autograd.grad((y * ws[i]).sum(), [x] + list(lin.parameters()))
                want_dx = g[0] if want_dx is None else want_dx + g[0]
                want_dp += list(g[1:])
            else:
                want_dp += [None] * len(list(lin.parameters()))
        for t in [x] + params:
            t.grad = None
        res = shared_input_linears(x, lins)
        sum((res[i][0] * ws[i]).sum() for i in used).backward()
        for (y, s), (wy, wsc) in zip(res, want_y):
            assert torch.equal(y, wy) and torch.equal(s, wsc)
        assert torch.equal(x.grad, want_dx)
        for p, w in zip(params, want_dp):
            assert (p.grad is None and w is None) or torch.equal(p.grad, w)


@pytest.mark.parametrize("M,Kd,N,N2", [(3000, 256, 256, 256), (1000, 100, 41, 64), (700, 602, 300, 32), (50, 64, 16, 7)])
def test_shared_input_linears_with_a_second_layer(M, Kd, N, N2):
    """then=[second layer or None]: the node == the layers chained one by one (outputs, scales and every
    gradient bit for bit, the input gradient added in layer order).  The first layer's output exists in int8
    only where the kernel for that applies (reduction <= 256) and in fp32 otherwise (602)."""
    from tango_amd.QLinear import QLinear, shared_input_linears
    torch.manual_seed(M + N2)
    firsts = [QLinear(Kd, N).cuda(), QLinear(Kd, N, bias=False).cuda(), QLinear(Kd, N).cuda()]
    seconds = [QLinear(N, N2).cuda(), None, QLinear(N, N2, bias=False).cuda()]
    for lin in firsts + [s for s in seconds if s is not None]:
        lin.enable_reduce()
    params = [p for lin in firsts + [s for s in seconds if s is not None] for p in lin.parameters()]
    x = torch.randn(M, Kd, device="cuda", requires_grad=True)
    ws = [torch.randn(M, N2 if s is not None else N, device="cuda") for s in seconds]
    want_y, want_dx = [], None
    want_dp = {}
    for i, (lin, sec) in enumerate(zip(firsts, seconds)):
        y, s = lin(x)
        if sec is not None:
            y, s = sec(y, s)
        want_y.append((y.detach().clone(), s.clone()))
        ps = list(lin.parameters()) + (list(sec.parameters()) if sec is not None else [])
        g = torch.autograd.grad((y * ws[i]).sum(), [x] + ps)
        want_dx = g[0] if want_dx is None else want_dx + g[0]
        want_dp.update({id(p): gp for p, gp in zip(ps, g[1:])})
    res = shared_input_linears(x, firsts, then=seconds)
    sum((res[i][0] * ws[i]).sum() for i in range(3)).backward()
    for (y, s), (wy, wsc) in zip(res, want_y):
        assert torch.equal(y, wy) and torch.equal(s, wsc)
    assert torch.equal(x.grad, want_dx)
    for p in params:
        assert torch.equal(p.grad, want_dp[id(p)])


def _bn_f64(x, gamma, beta, eps, relu, dy=None, mask=None):
    """Training-mode batch normalisation (+ ReLU) and its gradients in float64: the textbook formulas.  ``mask``:
    which outputs the ReLU let through, when the caller wants the gradients for a given forward result."""
    x, gamma, beta = x.astype(np.float64), gamma.astype(np.float64), beta.astype(np.float64)
    n = x.shape[0]
    mean, var = x.mean(0), x.var(0)
    rstd = 1.0 / np.sqrt(var + eps)
    xhat = (x - mean) * rstd
    y = xhat * gamma + beta
    out = {"mean": mean, "var": var, "y": np.maximum(y, 0) if relu else y}
    if dy is not None:
        g = dy.astype(np.float64) * (((y > 0) if mask is None else mask) if relu else 1.0)
        out["dbeta"], out["dgamma"] = g.sum(0), (g * xhat).sum(0)
        out["dx"] = rstd * gamma * (g - out["dbeta"] / n - xhat * out["dgamma"] / n)
    return out


@pytest.mark.parametrize("rows,cols,relu", [(5000, 128, True), (169343, 128, True), (777, 768, False), (33, 4, True),
                                            (2, 1024, True), (1001, 40, False), (4096, 256, True), (20000, 64, True),
                                            (3000, 750, True), (999, 7, False), (640, 1538, True), (500, 2048, True)])
def test_batchnorm_act_c_abi(K, rows, cols, relu):
    """The two entry points against float64 formulas (means far from zero, so a variance from a plain sum of
    squares would fail; one case with outliers in the rows the shifted sums take their shifts from), and the scale
    of the result against the result's own maximum."""
    import ctypes
    L = K._L
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((rows, cols)) * rng.uniform(0.1, 3.0, cols) + rng.uniform(-50, 50, cols)).astype(np.float32)
    if rows == 20000:  # outliers among the rows the reductions take their shifts from (a workgroup's first three), and elsewhere
        x[0, :8], x[16, 8:16], x[777, 16:24] = 1e4, -3e3, 2e4
    gamma, beta = rng.uniform(0.5, 1.5, cols).astype(np.float32), rng.uniform(-0.5, 0.5, cols).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np.float32)
    ref = _bn_f64(x, gamma, beta, 1e-5, relu, dy)
    X, G, B, DY = dev(x), dev(gamma), dev(beta), dev(dy)
    Y, DX = torch.empty_like(X), torch.empty_like(X)
    st = torch.empty(3, cols, device="cuda")
    dgb = torch.empty(2, cols, device="cuda")
    scale = torch.full((1,), 7.0, device="cuda")
    wsb = L.tango_batchnorm_workspace(rows, cols)
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert L.tango_batchnorm_fwd_f32(Y.data_ptr(), st[0].data_ptr(), st[1].data_ptr(), st[2].data_ptr(), scale.data_ptr(),
                                     X.data_ptr(), G.data_ptr(), B.data_ptr(), rows, cols, ctypes.c_float(1e-5), int(relu),
                                     ws.data_ptr(), wsb, stream) == 0
    assert L.tango_batchnorm_bwd_f32(DX.data_ptr(), dgb[0].data_ptr(), dgb[1].data_ptr(), DY.data_ptr(), X.data_ptr(),
                                     st[0].data_ptr(), st[2].data_ptr(), G.data_ptr(), B.data_ptr(), rows, cols, int(relu),
                                     ws.data_ptr(), wsb, stream) == 0
    # fp32 rounds the mean to its own grid: x - mean carries an absolute error of about an ulp of |x|, which the
    # normalisation magnifies by rstd (columns whose spread is tiny beside their mean, two-row batches)
    rstd64 = 1.0 / np.sqrt(ref["var"] + 1e-5)
    eps_hat = 2.0 ** -22 * (np.abs(ref["mean"]) + np.abs(x).max(0)) * rstd64  # error of xhat per column

    def close(actual, desired, rtol, atol):
        bad = np.abs(actual - desired) > atol + rtol * np.abs(desired)
        assert not bad.any(), (int(bad.sum()), float(np.abs(actual - desired).max()))

    close(host(st[0]), ref["mean"], 1e-6, 1e-6 * (1.0 + np.sqrt(ref["var"])))  # a millionth of a standard deviation
    close(host(st[1]), ref["var"], 2e-5, 1e-7)
    close(host(Y), ref["y"], 1e-5, 1e-5 + eps_hat * gamma)
    assert scale.item() == (Y.abs().max() / 127.0).item()
    # gradients: through the fp32 result's own ReLU mask (the few elements at y ~ 0 differ from float64's)
    if relu:
        assert ((host(Y) > 0) == (ref["y"] > 0)).mean() > 0.999
        ref = _bn_f64(x, gamma, beta, 1e-5, relu, dy, mask=host(Y) > 0)
    close(host(dgb[1]), ref["dbeta"], 1e-4, 1e-4 * np.sqrt(rows))
    close(host(dgb[0]), ref["dgamma"], 1e-4, 1e-4 * np.sqrt(rows) + 3 * rows * eps_hat)
    close(host(DX), ref["dx"], 1e-4, 1e-5 + rstd64 * gamma * (1e-5 + 4 * eps_hat * (np.abs(ref["dgamma"]) / rows + 1)))
    # a second call gives the same bits (fixed summation order)
    Y2, st2 = torch.empty_like(Y), torch.empty_like(st)
    assert L.tango_batchnorm_fwd_f32(Y2.data_ptr(), st2[0].data_ptr(), st2[1].data_ptr(), st2[2].data_ptr(), None,
                                     X.data_ptr(), G.data_ptr(), B.data_ptr(), rows, cols, ctypes.c_float(1e-5), int(relu),
                                     ws.data_ptr(), wsb, stream) == 0
    assert torch.equal(Y, Y2) and torch.equal(st, st2)


@pytest.mark.parametrize("rows,cols,act", [(3000, 128, "relu"), (500, 64, None), (700, 36, "relu"), (900, 128, "elu"),
                                           (400, 30, "relu"), (600, 750, "relu"), (300, 5, None)])
def test_batchnorm_module_matches_torch(rows, cols, act):
    """The module against torch.nn.BatchNorm1d + activation: outputs, gradients, running statistics over two
    training steps, the evaluation-mode pass and the state dict."""
    from tango_amd.batchnorm import BatchNorm1dAct
    fn = {"relu": torch.relu, "elu": torch.nn.functional.elu, None: None}[act]
    torch.manual_seed(rows)
    a = BatchNorm1dAct(cols, activation=fn).cuda()
    b = torch.nn.BatchNorm1d(cols).cuda()
    with torch.no_grad():
        a.weight.uniform_(0.5, 1.5)
        a.bias.uniform_(-0.5, 0.5)
    b.load_state_dict(a.state_dict())
    for step in range(2):
        x = torch.randn(rows, cols, device="cuda") * 2 + 1
        xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
        ya = a(xa)
        yb = b(xb) if fn is None else fn(b(xb))
        assert torch.allclose(ya, yb, rtol=1e-5, atol=1e-5)
        w = torch.randn_like(ya)
        (ya * w).sum().backward()
        (yb * w).sum().backward()
        assert torch.allclose(xa.grad, xb.grad, rtol=1e-4, atol=1e-5)
        assert torch.allclose(a.weight.grad, b.weight.grad, rtol=1e-4, atol=1e-3)
        assert torch.allclose(a.bias.grad, b.bias.grad, rtol=1e-4, atol=1e-3)
        assert torch.allclose(a.running_mean, b.running_mean, rtol=1e-5, atol=1e-6)
        assert torch.allclose(a.running_var, b.running_var, rtol=1e-5, atol=1e-6)
        assert int(a.num_batches_tracked) == int(b.num_batches_tracked) == step + 1
        a.zero_grad(), b.zero_grad()
    a.eval(), b.eval()
    x = torch.randn(50, cols, device="cuda")
    yb = b(x) if fn is None else fn(b(x))
    assert torch.allclose(a(x), yb, rtol=1e-6, atol=1e-6)
    assert a.state_dict().keys() == b.state_dict().keys()


def test_batchnorm_rejects_unsupported_shapes(K):
    L = K._L
    assert L.tango_batchnorm_workspace(100, 6) > 0 and L.tango_batchnorm_workspace(100, 4096) == 0
    x = torch.zeros(100, 8, device="cuda")
    p = x.data_ptr()
    import ctypes
    assert L.tango_batchnorm_fwd_f32(p, p, p, p, None, p, p, p, 100, 4096, ctypes.c_float(1e-5), 1, p, 1 << 30, None) == -2
    assert L.tango_batchnorm_fwd_f32(p, p, p, p, None, p, p, p, 100, 8, ctypes.c_float(1e-5), 1, None, 0, None) == -4
    assert L.tango_batchnorm_fwd_f32(p, p, p, p, None, p, p, p, 0, 8, ctypes.c_float(1e-5), 1, None, 0, None) == 0



def _sign_words(keep):
    rows, cols = keep.shape
    return np.ascontiguousarray(np.packbits(keep.reshape(rows, cols // 16, 16), axis=-1, bitorder="little").view(np.int16).reshape(rows, cols // 16))


@pytest.mark.parametrize("M,N,Kc", [(3001, 41, 256), (1000, 64, 128), (517, 200, 64), (77, 16, 32), (300, 41, 48)])
@pytest.mark.parametrize("with_mul", [True, False])
def test_gradx_epilogue_finds_the_masked_scale(K, orc, M, N, Kc, with_mul):
    """gradX whose epilogue also returns max|dX' * multiplier| / 127 (dX' = dX where its sign bit is set): the stored
    dX is the oracle's, and the scale is the oracle's absmax over that dX with the mask and multiplier: what the
    separate pass finds.  48 columns: not a width the epilogue takes, the wrapper falls back and returns None."""
    rng = np.random.default_rng(M + N + Kc)
    dYq = rng.integers(-127, 128, (M, N), dtype=np.int8)
    Wq = rng.integers(-127, 128, (N, Kc), dtype=np.int8)
    rs = (rng.random(M).astype(np.float32) + 0.5)
    mul = (rng.random(M).astype(np.float32) + 0.25) if with_mul else None
    keep = rng.random((M, Kc)) < 0.5
    bits = _sign_words(keep)
    s_dY, s_W = np.float32(0.013), np.float32(0.0021)
    dq = torch.zeros((M, (N + 15) // 16 * 16), dtype=torch.int8, device="cuda")[:, :N]
    dq.copy_(dev(dYq))
    dX = torch.full((M, Kc), float("nan"), device="cuda")
    got = K.cuda_kernels.QGEMM_backward_gradX(dX, dq, dev(Wq), sc(s_dY), sc(s_W), row_scale=dev(rs),
                                              masked=(dev(bits), None if mul is None else dev(mul)))
    want = orc.qgemm_bwd_dx_ex(dYq, Wq, s_dY, s_W, row_scale=rs)
    assert np.array_equal(host(dX), want)
    if Kc == 48:
        assert got is None
        return
    s_want, _ = orc.absmax_ex(want, row_mul=mul, mask=bits, mask_mode="bits")
    assert host(got)[0] == s_want
    # the pass it replaces agrees
    s_pass, _ = K.cuda_kernels.absmax_ex(dX, row_mul=None if mul is None else dev(mul), mask=dev(bits), mask_mode="bits")
    assert torch.equal(got, s_pass)


@pytest.mark.parametrize("rows,cols", [(3001, 256), (999, 64), (70, 16), (2000, 1024), (500, 48)])
def test_quantize_pass_returns_the_column_sums(K, orc, rows, cols):
    """The dense quantize pass that also sums the masked input per column: same bytes as the plain pass (every rounding
    mode, sign-word and fp32 masks, with and without the row multiplier), sums against float64; 48 columns: not a width
    it takes (returns None, nothing written)."""
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((rows, cols)) * 2).astype(np.float32)
    rm = rng.random(rows).astype(np.float32) + 0.5
    keep = rng.random((rows, cols)) < 0.6
    bits = _sign_words(keep)
    fmask = np.where(keep, 1.0, -1.0).astype(np.float32)
    masked = np.where(keep, x, 0).astype(np.float32)
    s, _ = orc.absmax_ex(x, row_mul=rm, mask=bits, mask_mode="bits")
    for mask_d, mode_name in ((dev(bits), "bits"), (dev(fmask), "relu"), (None, "relu")):
        ref = masked if mask_d is not None else x
        for rmul in (dev(rm), None):
            for kw, okw in (({}, dict(mode=orc.RNE)), ({"round_mode": "trunc"}, dict(mode=orc.TRUNC)),
                            ({"round_mode": "stochastic", "seed": 9, "offset": 128}, dict(mode=orc.STOCHASTIC, seed=9, offset=128)),
                            ({"round_mode": "stochastic", "seed": 9, "offset": 131}, dict(mode=orc.STOCHASTIC, seed=9, offset=131))):
                out = torch.full((rows, cols), 77, dtype=torch.int8, device="cuda")
                cs = K.cuda_kernels.quantize_rows_colsum(out, dev(x), sc(s), row_mul=rmul, mask=mask_d, mask_mode=mode_name, **kw)
                if cols == 48:
                    assert cs is None and bool((out == 77).all())
                    continue
                want = orc.quantize_rows_ex(x, s, row_mul=None if rmul is None else rm, mask=None if mask_d is None else bits,
                                            mask_mode="bits", **okw)
                assert np.array_equal(host(out), want), (mode_name, kw)
                assert np.allclose(host(cs), ref.astype(np.float64).sum(0), rtol=1e-5, atol=2e-3)
    if cols != 48:
        a = K.cuda_kernels.quantize_rows_colsum(torch.empty((rows, cols), dtype=torch.int8, device="cuda"), dev(x), sc(s))
        b = K.cuda_kernels.quantize_rows_colsum(torch.empty((rows, cols), dtype=torch.int8, device="cuda"), dev(x), sc(s))
        assert torch.equal(a, b)  # a fixed order of additions


def test_gcn_backward_takes_the_scale_from_gradx(monkeypatch):
    """Two fused GCN layers: the second layer's gradX hands the first layer's aggregation the scale of the masked,
    row-scaled gradient, and the bias gradient comes out of the quantize pass: no reducing pass over that gradient
    runs, and every gradient is the same as without the hand-off, bit for bit."""
    from tango_amd import SPMM, config, kernels
    from tango_amd.gcn import GCN
    from tango_amd.graph import Graph
    from tango_amd.util import graph_preprocess
    rng = np.random.default_rng(31)
    n, e = 3000, 40000
    src, dst = rand_graph(rng, n, e)
    g = graph_preprocess(Graph(dev(np.concatenate([src, np.arange(n)])), dev(np.concatenate([dst, np.arange(n)])), n))
    x = dev(rng.standard_normal((n, 96)).astype(np.float32))
    labels = dev(rng.integers(0, 7, n))
    torch.manual_seed(3)
    model = GCN(g, 96, 64, 7, 1, torch.relu, 0.0).cuda()
    config.grad_round_mode = "rne"
    calls = []
    real = kernels.cuda_kernels.absmax_ex
    monkeypatch.setattr(kernels.cuda_kernels, "absmax_ex",
                        staticmethod(lambda *a, **k: (calls.append(k.get("mask") is not None), real(*a, **k))[1]))

    def grads(hand_off):
        calls.clear()
        if not hand_off:
            monkeypatch.setattr(SPMM, "relu_mask_of", lambda t: None)
        model.zero_grad()
        torch.nn.functional.cross_entropy(model(x), labels).backward()
        return [p.grad.clone() for p in model.parameters()], sum(calls)

    with_, masked_passes = grads(True)
    assert masked_passes == 0
    without, masked_passes = grads(False)
    assert masked_passes == 1
    for a, b in zip(with_, without):
        if a.dim() == 1:  # bias gradients: the two passes add the rows in different orders
            assert torch.allclose(a, b, rtol=1e-5, atol=1e-6)
        else:
            assert torch.equal(a, b)


def test_gradient_with_two_consumers_is_scanned_once(monkeypatch):
    """The sum of two aggregations: autograd hands both nodes the same gradient tensor, the first leaves its scale
    on it and the second takes it from there.  Same gradients as with a scan each."""
    from tango_amd import SPMM, config, kernels
    from tango_amd.SPMM import spmm_copy_u
    from tango_amd.graph import Graph
    from tango_amd.util import graph_preprocess
    rng = np.random.default_rng(41)
    n = 2000
    graphs = []
    for e in (15000, 9000):
        src, dst = rand_graph(rng, n, e)
        graphs.append(graph_preprocess(Graph(dev(src), dev(dst), n)))
    config.grad_round_mode = "rne"
    xs = [dev(rng.standard_normal((n, 64)).astype(np.float32)).requires_grad_() for _ in graphs]
    w = dev(rng.standard_normal((n, 64)).astype(np.float32))
    scans = []
    real = kernels.cuda_kernels.get_scale
    monkeypatch.setattr(kernels.cuda_kernels, "get_scale",
                        staticmethod(lambda t: (scans.append(t.requires_grad), real(t))[1]))

    def grads():
        scans.clear()
        for x in xs:
            x.grad = None
        out = spmm_copy_u.apply(graphs[0], xs[0]) + spmm_copy_u.apply(graphs[1], xs[1])
        fwd = len(scans)
        (out * w).sum().backward()
        return [x.grad.clone() for x in xs], len(scans) - fwd

    shared, n_shared = grads()
    monkeypatch.setattr(SPMM, "grad_scale_hint", lambda t: None)
    apart, n_apart = grads()
    assert n_shared == 1 and n_apart == 2
    for a, b in zip(shared, apart):
        assert torch.equal(a, b)
