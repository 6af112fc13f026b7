"""One whole training epoch of the quantized 2-layer GCN on the GPU against the same epoch composed from
CPU-oracle calls (evaluation/test_gcn.py:67-139, 244-263 is the loop restated).

Configuration 1 of the benchmark set: 19,717 nodes, 88,651 undirected edges (Chung-Lu, exponent 2.1, seed 1),
500 -> 16 -> 3.  Everything that is integer arithmetic or a fixed sequence of fp32 roundings must agree bit
for bit: both layers' int8 tensors and scales, the logits, and both weight gradients.  The loss and its
gradient involve exp/log and the bias gradients a long fp32 sum, so those are held to 1e-5; the oracle's
backward pass starts from the GPU's own loss gradient, so that the integer stages after it can still be
compared exactly."""
import itertools

import numpy as np
import pytest
import torch

from gpu_util import host

pytestmark = pytest.mark.gpu

N, E_UNDIRECTED, F_IN, F_HID, N_CLS = 19717, 88651, 500, 16, 3


@pytest.fixture()
def grad_mode():
    from tango_amd import config
    saved = config.grad_round_mode, config.seed, config._calls
    yield config
    config.grad_round_mode, config.seed, config._calls = saved


def _oracle_layer_forward(orc, g_np, X, W, bias, norm_src, norm_dst, relu):
    """QGraphConv.forward for in_feats > out_feats: GEMM (row multiplier folded into its quantize), then the
    aggregation with '* norm_dst, + bias, relu' in its epilogue.  Returns the output and the backward caches."""
    sX, _ = orc.absmax_ex(X, row_mul=norm_src)
    sW = orc.absmax_scale(W)
    Xq = orc.quantize_rows_ex(X, sX, row_mul=norm_src, mode=orc.TRUNC)
    Wq = orc.quantize(W, sW, orc.TRUNC)
    Y, sY = orc.qgemm_i8_nt(Xq, Wq, sX, sW, reduce=True)
    Yq = orc.quantize(Y, sY)
    ip, ix = g_np["csc"]
    want_bits = relu and Y.shape[1] % 16 == 0
    res = orc.spmm_csr_copy_u_ex(ip, ix, Yq, sY, row_scale=norm_dst, bias=bias, act=1 if relu else 0,
                                 want_bits=want_bits)
    out, bits = res if want_bits else (res, None)
    cache = {"Xq": Xq, "sX": sX, "Wq": Wq, "sW": sW, "Y": Y, "sY": sY, "Yq": Yq, "bits": bits, "out": out,
             "relu": relu}
    return out, cache


def _oracle_layer_backward(orc, g_np, dOut, cache, norm_src, norm_dst, quant_kw, need_dx):
    """spmm_copy_u.backward followed by Qlinear_func_reduce.backward; ``quant_kw`` yields the rounding
    arguments of the two gradient quantizers in the order autograd calls them."""
    mask, mode = None, "relu"
    if cache["relu"]:
        mask, mode = (cache["bits"], "bits") if cache["bits"] is not None else (cache["out"], "relu")
    sdZ, dbias = orc.absmax_ex(dOut, row_mul=norm_dst, mask=mask, mask_mode=mode, want_colsum=True)
    dZq = orc.quantize_rows_ex(dOut, sdZ, row_mul=norm_dst, mask=mask, mask_mode=mode, **next(quant_kw))
    ip, ix = g_np["csr"]
    dY = orc.spmm_csr_copy_u(ip, ix, dZq, sdZ)
    sdY = orc.absmax_scale(dY)
    dYq = orc.quantize(dY, sdY, **next(quant_kw))
    dW = orc.qgemm_bwd_dw(dYq, cache["Xq"], sdY, cache["sX"])
    dX = orc.qgemm_bwd_dx_ex(dYq, cache["Wq"], sdY, cache["sW"], row_scale=norm_src) if need_dx else None
    return dX, dW, dbias, {"sdZ": sdZ, "dZq": dZq, "dY": dY, "sdY": sdY, "dYq": dYq}


@pytest.mark.parametrize("rounding", ["rne", "stochastic"])
def test_gcn_epoch_matches_oracle_composition(orc, grad_mode, rounding):
    from tango_amd.gcn import GCN, degree_norms
    from tango_amd.graph import chung_lu
    from tango_amd.loss import cross_entropy
    from tango_amd.util import graph_preprocess
    config = grad_mode
    config.grad_round_mode, config.seed = rounding, 1234
    config.reset_offsets()

    g = graph_preprocess(chung_lu(N, 2 * E_UNDIRECTED, 2.1, seed=1, symmetric=True, device="cuda"))
    gen = torch.Generator().manual_seed(1)
    X = torch.randn(N, F_IN, generator=gen).cuda()
    labels = torch.randint(0, N_CLS, (N,), generator=gen).cuda()
    torch.manual_seed(1)
    model = GCN(g, F_IN, F_HID, N_CLS, 1, torch.relu, 0.0).cuda()
    with torch.no_grad():
        for layer in model.layers:
            layer.bias.normal_(std=0.1)
    logits = model(X)
    grads = []
    logits.register_hook(grads.append)
    loss = cross_entropy(logits, labels)
    loss.backward()
    torch.cuda.synchronize()
    dlogits = host(grads[0])

    # ---- the same epoch from oracle calls
    g_np = {"csc": tuple(host(t) for t in g.adj_csc[:2]), "csr": tuple(host(t) for t in g.adj_csr[:2])}
    norm_src, norm_dst = (host(t) for t in degree_norms(g))
    want_ns = np.power(np.maximum(host(g.out_degrees()), 1).astype(np.float32), np.float32(-0.5))
    np.testing.assert_allclose(norm_src, want_ns, rtol=1e-6)
    l1, l2 = model.layers
    W1, b1, W2, b2 = (host(t) for t in (l1.weight, l1.bias, l2.weight, l2.bias))
    h1, c1 = _oracle_layer_forward(orc, g_np, host(X), W1, b1, norm_src, norm_dst, relu=True)
    out, c2 = _oracle_layer_forward(orc, g_np, h1, W2, b2, norm_src, norm_dst, relu=False)
    assert orc.overflow_count() == 0
    assert np.array_equal(host(logits), out)          # both layers' forward, bit for bit

    z = out.astype(np.float64)
    z -= z.max(1, keepdims=True)
    logp = z - np.log(np.exp(z).sum(1, keepdims=True))
    lab = host(labels)
    assert abs(float(loss.detach()) - float(-logp[np.arange(N), lab].mean())) < 1e-5
    want_g = np.exp(logp)
    want_g[np.arange(N), lab] -= 1.0
    np.testing.assert_allclose(dlogits, want_g / N, rtol=1e-5, atol=1e-9)

    # ---- backward from the GPU's loss gradient; the stochastic quantizers draw window k << 40 of the stream
    # in the order autograd runs them: layer 2 aggregation, layer 2 GEMM, layer 1 aggregation, layer 1 GEMM
    def rounding_args():
        for k in itertools.count():
            if rounding == "stochastic":
                yield {"mode": orc.STOCHASTIC, "seed": 1234, "offset": k << 40}
            else:
                yield {"mode": orc.RNE}
    kw = rounding_args()
    dH1, dW2, db2, _ = _oracle_layer_backward(orc, g_np, dlogits, c2, norm_src, norm_dst, kw, need_dx=True)
    _, dW1, db1, _ = _oracle_layer_backward(orc, g_np, dH1, c1, norm_src, norm_dst, kw, need_dx=False)
    assert np.array_equal(host(l2.weight.grad), dW2)
    assert np.array_equal(host(l1.weight.grad), dW1)
    np.testing.assert_allclose(host(l2.bias.grad), db2, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(host(l1.bias.grad), db1, rtol=1e-5, atol=1e-7)
    assert np.abs(dW1).max() > 0 and np.abs(dW2).max() > 0
