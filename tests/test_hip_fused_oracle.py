"""The fused operator forms the attention models run (u_mul_e with bias / activation in its epilogue and the
activation's derivative folded into the gradient quantizers; several linear layers over one quantized input with
an int8-only intermediate and one accumulated input gradient) against compositions of CPU-oracle calls."""
import numpy as np
import pytest
import torch

from gpu_util import dev, host, rand_graph

pytestmark = pytest.mark.gpu


def make_graph(src, dst, n):
    from tango_amd.graph import Graph
    from tango_amd.util import graph_preprocess
    return graph_preprocess(Graph(dev(src), dev(dst), n))


@pytest.mark.parametrize("act", [None, "relu", "elu"])
@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("n,e,H,F", [(700, 9000, 4, 16), (300, 40000, 3, 5), (500, 8000, 3, 25), (300, 5000, 1, 41),
                                     (200, 3000, 2, 250)])
def test_u_mul_e_fused_forward_and_backward_match_oracle(orc, act, with_bias, n, e, H, F):
    from tango_amd.SPMM import spmm_u_mul_e
    rng = np.random.default_rng(31)
    src, dst = rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    N = rng.standard_normal((n, H, F)).astype(np.float32)
    E = rng.random((e, H, 1)).astype(np.float32)
    bias = rng.standard_normal(H * F).astype(np.float32) if with_bias else None
    dZ = rng.standard_normal((n, H, F)).astype(np.float32)
    tN, tE = dev(N).requires_grad_(), dev(E).requires_grad_()
    tb = dev(bias).requires_grad_() if with_bias else None
    out = spmm_u_mul_e.apply(g, tN, tE, tb, None, act)
    out.backward(dev(dZ))

    code = {None: 0, "relu": 1, "elu": 2}[act]
    sN, sE = orc.absmax_scale(N), orc.absmax_scale(E)
    Nq, Eq = orc.quantize(N, sN), orc.quantize(E, sE)
    cip, cix, ceid = (host(t) for t in g.adj_csc)
    want = orc.spmm_csr_u_mul_e_ex(cip, cix, ceid, Nq, Eq, sN, scale2=sE, bias=bias, act=code, edge_major=True)
    if act == "elu":  # hardware exponential on the GPU, libm in the oracle
        np.testing.assert_allclose(host(out), want, rtol=1e-6, atol=5e-7)
        assert np.array_equal(host(out) > 0, want > 0)
    else:
        assert np.array_equal(host(out), want)
    # backward, from the GPU's own activation output (bit-identical to the oracle's except under ELU)
    mask = host(out).reshape(n, H * F) if act else None
    sdZ, colsum = orc.absmax_ex(dZ.reshape(n, H * F), mask=mask, mask_mode=act or "relu", want_colsum=True)
    dZq = orc.quantize_rows_ex(dZ.reshape(n, H * F), sdZ, mask=mask, mask_mode=act or "relu").reshape(n, H, F)
    rip, rix, reid = (host(t) for t in g.adj_csr)
    want_dN = orc.spmm_csr_u_mul_e_ex(rip, rix, reid, dZq, Eq, sdZ, scale2=sE, edge_major=True)
    assert np.array_equal(host(tN.grad), want_dN)
    want_dE, _ = orc.sddmm_dot(host(g.coo[0]), host(g.coo[1]), Nq, dZq, sN, sdZ)
    assert np.array_equal(host(tE.grad).reshape(e, H), want_dE)
    if with_bias:
        np.testing.assert_allclose(host(tb.grad), colsum, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("M,Kd,N1,N2", [(3000, 256, 256, 256), (1000, 64, 48, 32), (517, 602, 41, 16)])
def test_shared_input_linears_match_oracle(orc, M, Kd, N1, N2):
    """k / v / q projections of one input, two of them followed by a second layer whose input exists in int8
    only (evaluation/test_HGT.py:51-55): outputs, scales and every gradient against the oracle; the three input
    gradients meet in one tensor by accumulation in the GEMM epilogue."""
    from tango_amd.QLinear import QLinear, shared_input_linears
    torch.manual_seed(M)
    first = [QLinear(Kd, N1).cuda() for _ in range(3)]
    second = [QLinear(N1, N2).cuda(), QLinear(N1, N2).cuda(), None]
    X = torch.randn(M, Kd, device="cuda", requires_grad=True)
    outs = shared_input_linears(X, first, then=second)
    gen = torch.Generator("cuda").manual_seed(7)
    dYs = [torch.randn(y.shape, device="cuda", generator=gen) for y, _ in outs]
    torch.autograd.backward([y for y, _ in outs], dYs)

    Xn = host(X)
    sX = orc.absmax_scale(Xn)
    Xq = orc.quantize(Xn, sX, orc.TRUNC)
    dX = None
    for i, (lin, nxt) in enumerate(zip(first, second)):
        W, b = host(lin.weight), host(lin.bias)
        sW = orc.absmax_scale(W)
        Wq = orc.quantize(W, sW, orc.TRUNC)
        Y1, sY1 = orc.qgemm_i8_nt(Xq, Wq, sX, sW, bias=b, reduce=True)
        dY = host(dYs[i])
        if nxt is not None:
            W2, b2 = host(nxt.weight), host(nxt.bias)
            sW2 = orc.absmax_scale(W2)
            W2q = orc.quantize(W2, sW2, orc.TRUNC)
            Y1q = orc.quantize(Y1, sY1, orc.TRUNC)
            Y2, sY2 = orc.qgemm_i8_nt(Y1q, W2q, sY1, sW2, bias=b2, reduce=True)
            assert np.array_equal(host(outs[i][0]), Y2) and host(outs[i][1])[0] == sY2
            s_d = orc.absmax_scale(dY)
            dq = orc.quantize(dY, s_d)
            assert np.array_equal(host(nxt.weight.grad), orc.qgemm_bwd_dw(dq, Y1q, s_d, sY1))
            np.testing.assert_allclose(host(nxt.bias.grad), dY.astype(np.float64).sum(0), rtol=1e-4, atol=1e-4)
            dY = orc.qgemm_bwd_dx(dq, W2q, s_d, sW2)
        else:
            assert np.array_equal(host(outs[i][0]), Y1) and host(outs[i][1])[0] == sY1
        s_d = orc.absmax_scale(dY)
        dq = orc.quantize(dY, s_d)
        assert np.array_equal(host(lin.weight.grad), orc.qgemm_bwd_dw(dq, Xq, s_d, sX))
        np.testing.assert_allclose(host(lin.bias.grad), dY.astype(np.float64).sum(0), rtol=1e-4, atol=2e-3)
        dX = orc.qgemm_bwd_dx_ex(dq, Wq, s_d, sW, accumulate_into=dX)
    assert np.array_equal(host(X.grad), dX)


@pytest.mark.parametrize("n,e,F", [(900, 20000, 128), (400, 6000, 41), (1500, 30000, 256)])
def test_copy_u_with_source_multiplier_matches_oracle(orc, n, e, F):
    """The aggregate-first graph convolution's "feat * out_deg^-1/2" folded into the aggregation: the multiplier
    rides in the pass that quantizes the input (forward) and in the reverse aggregation's epilogue (backward)."""
    from tango_amd import config
    from tango_amd.SPMM import spmm_copy_u
    rng = np.random.default_rng(n)
    src, dst = rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    N = rng.standard_normal((n, F)).astype(np.float32)
    mul = (rng.random(n) + 0.2).astype(np.float32)
    dZ = rng.standard_normal((n, F)).astype(np.float32)
    old = config.grad_round_mode
    config.grad_round_mode = "rne"
    try:
        tN = dev(N).requires_grad_()
        out = spmm_copy_u.apply(g, tN, None, None, None, False, dev(mul))
        out.backward(dev(dZ))
    finally:
        config.grad_round_mode = old
    sN, _ = orc.absmax_ex(N, row_mul=mul)
    Nq = orc.quantize_rows_ex(N, sN, row_mul=mul)
    cip, cix, _ = (host(t) for t in g.adj_csc)
    assert np.array_equal(host(out), orc.spmm_csr_copy_u_ex(cip, cix, Nq, sN))
    # the same bits as multiplying first
    assert torch.equal(out, spmm_copy_u.apply(g, dev(N) * dev(mul).unsqueeze(1)))
    s_dZ = orc.absmax_scale(dZ)
    dZq = orc.quantize(dZ, s_dZ)
    rip, rix, _ = (host(t) for t in g.adj_csr)
    assert np.array_equal(host(tN.grad), orc.spmm_csr_copy_u_ex(rip, rix, dZq, s_dZ, row_scale=mul))


@pytest.mark.parametrize("n,e,H,D", [(500, 8000, 3, 250), (300, 5000, 1, 41), (400, 6000, 3, 248), (350, 4000, 5, 25)])
def test_unaligned_head_widths_run_on_padded_heads(orc, n, e, H, D):
    """Head widths that are not multiples of 16 (the reference's arxiv GAT trains with 3 heads of 250): the int8
    copies are zero-padded per head, the SDDMM dot and the u_mul_e aggregation run on aligned rows, and every
    result equals the oracle's on the unpadded operands, forward and backward."""
    from tango_amd import config
    from tango_amd.SDDMM import sddmm_u_dot_v
    from tango_amd.SPMM import spmm_u_mul_e
    from tango_amd.kernels import pad_heads, quantize_heads
    assert pad_heads(D, H) % 16 == 0 and pad_heads(D, H) != D and pad_heads(16, 8) == 16 and pad_heads(5, 3) == 5
    assert pad_heads(40, 1) == 40 and pad_heads(40, 8) == 40  # rows of whole 4-byte pieces stay as they are
    rng = np.random.default_rng(D)
    src, dst = rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    U, V = (rng.standard_normal((n, H, D)).astype(np.float32) for _ in range(2))
    q, s = quantize_heads(dev(U))
    assert q.shape == (n, H, pad_heads(D, H)) and np.array_equal(host(q)[..., :D], orc.quantize(U, orc.absmax_scale(U)))
    assert not host(q)[..., D:].any()
    old = config.grad_round_mode
    config.grad_round_mode = "rne"
    try:
        # SDDMM dot: forward, and both backward aggregations with dZ as edge values
        tU, tV = dev(U).requires_grad_(), dev(V).requires_grad_()
        out = sddmm_u_dot_v.apply(g, tU, tV)
        dZ = rng.standard_normal((e, H, 1)).astype(np.float32)
        out.backward(dev(dZ))
        sU, sV = orc.absmax_scale(U), orc.absmax_scale(V)
        Uq, Vq = orc.quantize(U, sU), orc.quantize(V, sV)
        want, _ = orc.sddmm_dot(src, dst, Uq, Vq, sU, sV)
        assert np.array_equal(host(out).reshape(e, H), want)
        s_dZ = orc.absmax_scale(dZ)
        dZq = orc.quantize(dZ, s_dZ)
        cip, cix, ceid = (host(t) for t in g.adj_csc)
        rip, rix, reid = (host(t) for t in g.adj_csr)
        assert np.array_equal(host(tV.grad), orc.spmm_csr_u_mul_e_ex(cip, cix, ceid, Uq, dZq, s_dZ, scale2=sU, edge_major=True))
        assert np.array_equal(host(tU.grad), orc.spmm_csr_u_mul_e_ex(rip, rix, reid, Vq, dZq, s_dZ, scale2=sV, edge_major=True))
        # u_mul_e: forward, dN (reverse aggregation) and dE (dot of the features with dOut)
        E = rng.random((e, H, 1)).astype(np.float32)
        tN, tE = dev(U).requires_grad_(), dev(E).requires_grad_()
        agg = spmm_u_mul_e.apply(g, tN, tE)
        dOut = rng.standard_normal((n, H, D)).astype(np.float32)
        agg.backward(dev(dOut))
        sE = orc.absmax_scale(E)
        Eq = orc.quantize(E, sE)
        assert agg.shape == (n, H, D) and agg.is_contiguous()
        assert np.array_equal(host(agg), orc.spmm_csr_u_mul_e_ex(cip, cix, ceid, Uq, Eq, sU, scale2=sE, edge_major=True))
        s_dO = orc.absmax_scale(dOut)
        dOq = orc.quantize(dOut, s_dO)
        assert np.array_equal(host(tN.grad), orc.spmm_csr_u_mul_e_ex(rip, rix, reid, dOq, Eq, s_dO, scale2=sE, edge_major=True))
        wantE, _ = orc.sddmm_dot(src, dst, Uq, dOq, sU, s_dO)
        assert np.array_equal(host(tE.grad).reshape(e, H), wantE)
    finally:
        config.grad_round_mode = old
