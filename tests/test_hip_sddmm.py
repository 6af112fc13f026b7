"""GPU parity: SDDMM (dot bit-exact on the int32 sums; element-wise ops are three
IEEE fp32 roundings on both sides, compared bit-exactly) and edge softmax
(fp32, 1e-5 relative / 1e-6 absolute)."""
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


def test_reference_test_pattern(K):
    # cuda/src/SDDMM.cu:238-258
    src = np.array([0, 0, 0, 1], np.int64)
    dst = np.array([0, 1, 2, 2], np.int64)
    g = make_graph(src, dst, 3)
    for dim in (4, 16, 40):
        U = np.arange(3 * dim).astype(np.int8).reshape(3, dim)
        V = (3 * dim - np.arange(3 * dim)).astype(np.int8).reshape(3, dim)
        out, _ = K.mySDDMM_int8(g, "add", dev(U), dev(V), sc(1.0), sc(1.0), False)
        j = np.arange(dim)
        for e in range(4):
            assert np.array_equal(host(out)[e], ((src[e] * dim + j) + (3 * dim - dst[e] * dim - j)).astype(np.float32))


@pytest.mark.parametrize("H,D", [(8, 16), (4, 64), (1, 128), (3, 32), (2, 256), (3, 48), (3, 4), (2, 7), (8, 1), (5, 20)])
@pytest.mark.parametrize("reduce", [False, True])
def test_dot(K, orc, H, D, reduce):
    rng = np.random.default_rng(H * 100 + D)
    n, e = 700, 50011
    src, dst = rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    U = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
    V = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
    sU, sV = np.float32(0.011), np.float32(0.37)
    out, so = K.mySDDMM_int8(g, "dot", dev(U), dev(V), sc(sU), sc(sV), reduce)
    want, wso = orc.sddmm_dot(src, dst, U, V, sU, sV, reduce=reduce)
    assert tuple(out.shape) == (e, H, 1)
    assert np.array_equal(host(out).reshape(e, H), want)
    if reduce:
        assert host(so)[0] == wso
    # reverse swaps the endpoint roles
    out_r, _ = K.mySDDMM_int8(g, "dot", dev(U), dev(V), sc(sU), sc(sV), False, reverse=True)
    want_r, _ = orc.sddmm_dot(dst, src, U, V, sU, sV)
    assert np.array_equal(host(out_r).reshape(e, H), want_r)


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
@pytest.mark.parametrize("shape", [(8, 1), (8, 16), (3,), (7,), (1, 5)])
def test_elementwise(K, orc, op, shape):
    rng = np.random.default_rng(len(shape) + sum(shape))
    n, e = 500, 30007
    src, dst = rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    U = rng.integers(-127, 128, (n,) + shape).astype(np.int8)
    V = rng.integers(1, 128, (n,) + shape).astype(np.int8)  # no zero divisors
    sU, sV = np.float32(0.05), np.float32(0.002)
    out, so = K.mySDDMM_int8(g, op, dev(U), dev(V), sc(sU), sc(sV), True)
    want, wso = orc.sddmm_ewise(op, src, dst, U.reshape(n, -1), V.reshape(n, -1), sU, sV, reduce=True)
    assert tuple(out.shape) == (e,) + shape
    assert np.array_equal(host(out).reshape(e, -1), want)
    assert host(so)[0] == wso


@pytest.mark.parametrize("mode", ["rne", "trunc"])
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
@pytest.mark.parametrize("shape", [(8, 1), (3,), (1, 5), (16,)])
def test_elementwise_quantizing_on_load(K, orc, op, shape, mode):
    """fp32 operands rounded by the SDDMM kernel as it gathers them == the oracle's quantize followed by its
    element-wise SDDMM, bit for bit, including values that clamp (|x| above 127 scale) and an all-zero scale."""
    rng = np.random.default_rng(len(shape) + sum(shape) + len(op))
    n, e = 700, 20011
    src, dst = rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    U = (rng.standard_normal((n,) + shape) * 3).astype(np.float32)
    V = (np.abs(rng.standard_normal((n,) + shape)) + 0.5).astype(np.float32)  # rounds to >= 10: no zero divisors
    sU, sV = np.float32(np.abs(U).max() / 127 * 0.8), np.float32(np.abs(V).max() / 127)
    omode = orc.RNE if mode == "rne" else orc.TRUNC
    Uq, Vq = orc.quantize(U, sU, omode).reshape(n, -1), orc.quantize(V, sV, omode).reshape(n, -1)
    assert np.abs(Vq).min() > 0 and np.abs(Uq).max() == 127
    want, _ = orc.sddmm_ewise(op, src, dst, Uq, Vq, sU, sV)
    out = K.mySDDMM_quantize_on_load(g, op, dev(U), dev(V), sc(sU), sc(sV), round_mode=mode)
    assert tuple(out.shape) == (e,) + shape
    assert np.array_equal(host(out).reshape(e, -1), want)
    if op == "add":  # a tensor of zeros has scale 0 and quantizes to zeros
        out0 = K.mySDDMM_quantize_on_load(g, op, dev(np.zeros_like(U)), dev(V), sc(0.0), sc(sV), round_mode=mode)
        want0, _ = orc.sddmm_ewise(op, src, dst, np.zeros_like(Uq), Vq, np.float32(0), sV)
        assert np.array_equal(host(out0).reshape(e, -1), want0)


def test_unknown_op_raises(K):
    g = make_graph(np.array([0], np.int64), np.array([0], np.int64), 1)
    z = torch.zeros((1, 4), dtype=torch.int8, device="cuda")
    with pytest.raises(ValueError):
        K.mySDDMM_int8(g, "pow", z, z, sc(1), sc(1), False)
    with pytest.raises(RuntimeError):  # dtype mismatch, as data_ptr<int8_t>() throws in the reference
        K.mySDDMM_int8(g, "add", z.float(), z, sc(1), sc(1), False)


# (n, e): rows of some hundred slots, rows of a few slots with some destinations empty, and a
# graph that is mostly one hub; every graph gets rows that spread over several wavefronts' spans
@pytest.mark.parametrize("n,e", [(900, 40000), (6000, 30000), (500, 90000)])
@pytest.mark.parametrize("H", [1, 3, 4, 8, 12, 64, 70])
@pytest.mark.parametrize("slope", [1.0, 0.2])
def test_edge_softmax(K, orc, H, slope, n, e):
    rng = np.random.default_rng(H)
    src, dst = rand_graph(rng, n, e)
    dst[:5000] = 3  # one high-degree destination
    if e > 60000:
        dst[:40000] = 3  # a hub: 150 spans of one row
    dst[5000:5300] = 7  # a row a little longer than one span
    g = make_graph(src, dst, n)
    o = orc.graph_formats(src, dst, n)
    x = (rng.standard_normal((e, H)) * 4).astype(np.float32)
    ip, _, eid = g.adj_csc
    a = K.cuda_kernels.edge_softmax_forward(dev(x), ip, eid, slope)
    want = orc.edge_softmax_fwd(x, o["adj_csc"][0], o["adj_csc"][2], slope)
    assert np.allclose(host(a), want, rtol=1e-5, atol=1e-6)
    da = rng.standard_normal((e, H)).astype(np.float32)
    de = K.cuda_kernels.edge_softmax_backward(a, dev(da), dev(x), ip, eid, slope)
    want_de = orc.edge_softmax_bwd(want, da, x, o["adj_csc"][0], o["adj_csc"][2], slope)
    assert np.allclose(host(de), want_de, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("e", [1, 63, 256, 257, 1000, 20011])
def test_edge_softmax_empty_runs(K, orc, e):
    """Destinations only at both ends of the id range: thousands of empty rows in a row inside one
    span, which the row-pointer window of a wavefront cannot hold."""
    rng = np.random.default_rng(e)
    n, H = 9000, 8
    src = rng.integers(0, n, e).astype(np.int64)
    dst = np.where(rng.random(e) < 0.5, rng.integers(0, 40, e), rng.integers(n - 40, n, e)).astype(np.int64)
    g = make_graph(src, dst, n)
    o = orc.graph_formats(src, dst, n)
    x = (rng.standard_normal((e, H)) * 3).astype(np.float32)
    ip, _, eid = g.adj_csc
    a = K.cuda_kernels.edge_softmax_forward(dev(x), ip, eid, 0.2)
    want = orc.edge_softmax_fwd(x, o["adj_csc"][0], o["adj_csc"][2], 0.2)
    assert np.allclose(host(a), want, rtol=1e-5, atol=1e-6)
    da = rng.standard_normal((e, H)).astype(np.float32)
    de = K.cuda_kernels.edge_softmax_backward(a, dev(da), dev(x), ip, eid, 0.2)
    want_de = orc.edge_softmax_bwd(want, da, x, o["adj_csc"][0], o["adj_csc"][2], 0.2)
    assert np.allclose(host(de), want_de, rtol=1e-4, atol=1e-6)


def test_edge_softmax_without_workspace(K, orc):
    """workspace = NULL: the thread-per-(row, head) path of the C entry points."""
    from tango_amd import _lib
    rng = np.random.default_rng(5)
    n, e, H = 300, 5000, 3
    src, dst = rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    o = orc.graph_formats(src, dst, n)
    x = dev((rng.standard_normal((e, H)) * 3).astype(np.float32))
    ip, _, eid = g.adj_csc
    a = torch.empty_like(x)
    st = torch.cuda.current_stream().cuda_stream
    assert _lib.lib().tango_edge_softmax_fwd(a.data_ptr(), x.data_ptr(), ip.data_ptr(), eid.data_ptr(), n, e, H, 0.2,
                                             None, 0, st) == 0
    want = orc.edge_softmax_fwd(host(x), o["adj_csc"][0], o["adj_csc"][2], 0.2)
    assert np.allclose(host(a), want, rtol=1e-5, atol=1e-6)
    da = dev(rng.standard_normal((e, H)).astype(np.float32))
    de = torch.empty_like(x)
    assert _lib.lib().tango_edge_softmax_bwd(de.data_ptr(), a.data_ptr(), da.data_ptr(), x.data_ptr(), ip.data_ptr(),
                                             eid.data_ptr(), n, e, H, 0.2, None, 0, st) == 0
    want_de = orc.edge_softmax_bwd(want, host(da), host(x), o["adj_csc"][0], o["adj_csc"][2], 0.2)
    assert np.allclose(host(de), want_de, rtol=1e-4, atol=1e-6)
