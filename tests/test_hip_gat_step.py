"""One training step of a quantized GAT layer on the GPU against the same step composed from CPU-oracle calls
(evaluation/test_gat.py:91-169 forward; cuda/SPMM.py:47-62, cuda/SDDMM.py:22-32, cuda/QLinear.py:38-47 backward).

Forward and backward are followed stage by stage.  Integer stages (GEMMs, SDDMM, aggregations and the int8 tensors
and scales between them) must agree bit for bit; the fp32 stages that sum or exponentiate (attention logits, edge
softmax and their backward passes) are held to 1e-5 / 1e-6, and the GPU's own value of such a stage is what the
oracle's later stages start from, so that the integer stages after it are still compared exactly."""
import itertools

import numpy as np
import pytest
import torch

from gpu_util import host

pytestmark = pytest.mark.gpu


@pytest.fixture()
def grad_mode():
    from tango_amd import config
    saved = config.grad_round_mode, config.seed, config._calls
    yield config
    config.grad_round_mode, config.seed, config._calls = saved


@pytest.mark.parametrize("rounding", ["rne", "stochastic"])
def test_gat_layer_step_matches_oracle_composition(orc, grad_mode, monkeypatch, rounding):
    import tango_amd.gat as gat
    from tango_amd.gat import QGATConv
    from tango_amd.graph import chung_lu
    from tango_amd.util import graph_preprocess
    config = grad_mode
    config.grad_round_mode, config.seed = rounding, 77
    config.reset_offsets()
    monkeypatch.setattr(gat, "fused_attention", False)  # the separate ops: one oracle stage each

    # record the intermediate tensors of the forward pass and, through hooks, their gradients
    taps = {}

    def tap(name, t):
        taps[name] = t
        if t.requires_grad:
            t.register_hook(lambda g_, _n=name: taps.__setitem__("d_" + _n, g_))
        return t

    real = {k: getattr(gat, k) for k in ("attn_scores", "sddmm_u_add_v", "spmm_u_mul_e", "edge_softmax")}

    class Tap:
        def __init__(self, name, fn, is_class):
            self.name, self.fn, self.is_class = name, fn, is_class

        def apply(self, *a):
            out = self.fn.apply(*a)
            if self.name == "attn_scores":
                tap("feat", a[0]); tap("el", out[0]); tap("er", out[1]); taps["s_el"], taps["s_er"] = out[2], out[3]
            elif self.name == "sddmm_u_add_v":
                tap("e", out)
            else:
                tap("rst", out)
            return out

        def __call__(self, *a, **kw):
            return tap("a", self.fn(*a, **kw))

    for k, fn in real.items():
        monkeypatch.setattr(gat, k, Tap(k, fn, k != "edge_softmax"))

    g = graph_preprocess(chung_lu(4000, 36000, 2.2, seed=9, device="cuda"))
    n, E, H, D, Fin = g.num_nodes(), g.num_edges(), 4, 16, 48
    torch.manual_seed(11)
    layer = QGATConv(Fin, D, H, bias=True).cuda()
    with torch.no_grad():
        layer.bias.normal_(std=0.1)
    x = torch.randn(n, Fin, device="cuda", requires_grad=True)
    G = torch.randn(n, H, D, device="cuda")
    out = layer(g, x)
    (out * G).sum().backward()
    torch.cuda.synchronize()

    # ---------------------------------------------------------------- forward
    xn, W = host(x.detach()), host(layer.fc.weight)
    feat, Xq, Wq, sX, sW, s_feat = orc.qgemm_fwd(xn, W, reduce=True)
    assert np.array_equal(host(taps["feat"]).reshape(n, H * D), feat)
    al, ar = host(layer.attn_l).reshape(H, D), host(layer.attn_r).reshape(H, D)
    f64 = feat.reshape(n, H, D).astype(np.float64)
    el, er = host(taps["el"]).reshape(n, H), host(taps["er"]).reshape(n, H)
    np.testing.assert_allclose(el, (f64 * al).sum(-1), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(er, (f64 * ar).sum(-1), rtol=1e-5, atol=1e-5)
    s_el, s_er = host(taps["s_el"])[0], host(taps["s_er"])[0]
    assert s_el == orc.absmax_scale(el) and s_er == orc.absmax_scale(er)
    src, dst = host(g.coo[0]), host(g.coo[1])
    want_e, _ = orc.sddmm_ewise("add", src, dst, orc.quantize(el, s_el), orc.quantize(er, s_er), s_el, s_er)
    e = host(taps["e"]).reshape(E, H)
    assert np.array_equal(e, want_e)
    ip, ix, eid = (host(t) for t in g.adj_csc)
    a = host(taps["a"]).reshape(E, H)
    np.testing.assert_allclose(a, orc.edge_softmax_fwd(e, ip, eid, 0.2), rtol=1e-5, atol=1e-6)
    sa = orc.absmax_scale(a)
    aq = orc.quantize(a, sa).reshape(E, H, 1)
    featq = orc.quantize(feat, s_feat).reshape(n, H, D)
    bias = host(layer.bias)
    want_out = orc.spmm_csr_u_mul_e_ex(ip, ix, eid, featq, aq, s_feat, scale2=sa, bias=bias, edge_major=True)
    assert np.array_equal(host(out.detach()), want_out)

    # ---------------------------------------------------------------- backward
    def rounding_args():
        for k in itertools.count():
            if rounding == "stochastic":
                yield {"mode": orc.STOCHASTIC, "seed": 77, "offset": k << 40}
            else:
                yield {"mode": orc.RNE}
    kw = rounding_args()
    Gn = host(G)
    # aggregation: scale of dZ and bias gradient in one pass, then dN (reverse aggregation) and dE (SDDMM dot)
    sdZ, dbias = orc.absmax_ex(Gn.reshape(n, H * D), want_colsum=True)
    dZq = orc.quantize(Gn, sdZ, **next(kw)).reshape(n, H, D)
    rp, rx, reid = (host(t) for t in g.adj_csr)
    dN = orc.spmm_csr_u_mul_e_ex(rp, rx, reid, dZq, aq, sdZ, scale2=sa, edge_major=True)
    dE, _ = orc.sddmm_dot(src, dst, featq, dZq, s_feat, sdZ)
    assert np.array_equal(host(taps["d_a"]).reshape(E, H), dE)
    np.testing.assert_allclose(host(layer.bias.grad), dbias, rtol=1e-5, atol=1e-6)
    # softmax backward (fp32), from the GPU's own a and dE
    de = host(taps["d_e"]).reshape(E, H)
    np.testing.assert_allclose(de, orc.edge_softmax_bwd(a, dE, e, ip, eid, 0.2), rtol=1e-5, atol=1e-6)
    # u_add_v backward: the quantized de summed per destination (er) and per source (el), from the GPU's de
    sde = orc.absmax_scale(de)
    deq = orc.quantize(de, sde, **next(kw))
    d_er = orc.spmm_incidence(host(g.inc_in[0]), host(g.inc_in[1]), deq, sde, n)
    d_el = orc.spmm_incidence(host(g.inc_out[0]), host(g.inc_out[1]), deq, sde, n)
    assert np.array_equal(host(taps["d_er"]).reshape(n, H), d_er)
    assert np.array_equal(host(taps["d_el"]).reshape(n, H), d_el)
    # attention logits backward (fp32 sums over the nodes) and the total gradient of the projected features
    np.testing.assert_allclose(host(layer.attn_l.grad).reshape(H, D), (d_el[:, :, None] * f64).sum(0), rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(host(layer.attn_r.grad).reshape(H, D), (d_er[:, :, None] * f64).sum(0), rtol=1e-4, atol=1e-4)
    dfeat_gpu = host(taps["d_feat"]).reshape(n, H, D)
    want_dfeat = dN.astype(np.float64) + d_el[:, :, None] * al.astype(np.float64) + d_er[:, :, None] * ar.astype(np.float64)
    np.testing.assert_allclose(dfeat_gpu, want_dfeat, rtol=1e-5, atol=1e-6)
    # the projection's backward from the GPU's total gradient: quantize, gradW, gradX (integer stages, exact)
    dY = dfeat_gpu.reshape(n, H * D)
    sdY = orc.absmax_scale(dY)
    dYq = orc.quantize(dY, sdY, **next(kw))
    assert np.array_equal(host(layer.fc.weight.grad), orc.qgemm_bwd_dw(dYq, Xq, sdY, sX))
    assert np.array_equal(host(x.grad), orc.qgemm_bwd_dx(dYq, Wq, sdY, sW))
    assert np.abs(host(x.grad)).max() > 0
