"""GPU tests of edge cases and of the host-side contract: empty and degenerate
inputs, error paths (bad dtype / device / shape raise before any launch), and
capture of the hot path into a HIP graph (no entry point uses hipMemsetAsync or
synchronises, so replays must reproduce the eager results)."""
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


def test_empty_inputs(K):
    z = torch.empty(0, device="cuda")
    assert K.cuda_kernels.get_scale(z).item() == 0.0
    q, s = K.quantize(torch.empty((0, 8), device="cuda"))
    assert q.numel() == 0
    # graph without edges: every aggregation is zero, SDDMM output is empty
    g = make_graph(np.empty(0, np.int64), np.empty(0, np.int64), 5)
    feat = torch.ones((5, 16), dtype=torch.int8, device="cuda")
    assert not K.csr_SPMM(g, feat, sc(1.0)).any()
    out, _ = K.mySDDMM_int8(g, "dot", feat.view(5, 1, 16), feat.view(5, 1, 16), sc(1), sc(1), False)
    assert tuple(out.shape) == (0, 1, 1)
    E = torch.empty((0, 4), dtype=torch.int8, device="cuda")
    assert not K.incidence_SPMM(g, E, sc(1.0)).any()
    # GEMM with zero rows / zero reduction length
    X = torch.empty((0, 32), device="cuda")
    W = torch.randn(8, 32, device="cuda")
    Y = K.QGEMM_forward(X, torch.empty((0, 32), dtype=torch.int8, device="cuda"), sc(1.0), W,
                        torch.empty((8, 32), dtype=torch.int8, device="cuda"), K.cuda_kernels.get_scale(W))
    assert tuple(Y.shape) == (0, 8)


def test_single_node_and_self_loops_only(K, orc):
    g = make_graph(np.arange(7, dtype=np.int64), np.arange(7, dtype=np.int64), 7)
    feat = np.arange(7 * 5, dtype=np.int8).reshape(7, 5)
    got = K.csr_SPMM(g, dev(feat), sc(0.5))
    assert np.array_equal(host(got), feat.astype(np.float32) * np.float32(0.5))


def test_very_long_row(K, orc):
    # one destination with 300,000 in-edges (more than any 4-wave split handles in one pass)
    rng = np.random.default_rng(0)
    n, e = 1000, 300000
    src = rng.integers(0, n, e).astype(np.int64)
    dst = np.zeros(e, np.int64)
    g = make_graph(src, dst, n)
    for F in (16, 256):
        feat = rng.integers(-127, 128, (n, F)).astype(np.int8)
        got = K.csr_SPMM(g, dev(feat), sc(1.0))
        want = np.zeros((n, F), np.float32)
        want[0] = feat[src].astype(np.int64).sum(0)
        assert np.array_equal(host(got), want)


def test_error_paths_raise(K):
    g = make_graph(np.array([0, 1], np.int64), np.array([1, 0], np.int64), 2)
    f32 = torch.zeros((2, 4), device="cuda")
    i8 = torch.zeros((2, 4), dtype=torch.int8, device="cuda")
    with pytest.raises(RuntimeError):
        K.csr_SPMM(g, f32, sc(1.0))  # features must be int8
    with pytest.raises(RuntimeError):
        K.cuda_kernels.get_scale(i8)  # input must be fp32
    with pytest.raises(RuntimeError):
        K.cuda_kernels.quantize(i8, torch.zeros((2, 4)), sc(1.0))  # CPU tensor
    with pytest.raises(RuntimeError):
        K.cuda_kernels.quantize(i8, torch.zeros((3, 4), device="cuda"), sc(1.0))  # size mismatch
    with pytest.raises(AssertionError):
        K.quantize(torch.zeros(4))  # the reference's own assert: tensor must be on GPU
    with pytest.raises(AssertionError):
        K.multi_cusparse_SPMM(g, i8.view(2, 1, 4), torch.zeros((1, 2, 2), dtype=torch.int8, device="cuda"), sc(1))
    with pytest.raises(RuntimeError):
        K.cuda_kernels.QGEMM_forward(torch.zeros((2, 3), device="cuda"), f32, i8, torch.zeros((3, 5), device="cuda"),
                                     torch.zeros((3, 5), dtype=torch.int8, device="cuda"), torch.Tensor(),
                                     torch.Tensor(), sc(1), sc(1))  # K mismatch
    with pytest.raises(KeyError):
        K.quantize(f32, round_mode="nearest")  # unknown rounding mode


def test_status_codes_surface_as_exceptions(K):
    from tango_amd import _lib
    with pytest.raises(_lib.TangoError):
        _lib.check(-2, "probe")
    L = _lib.lib()
    x = torch.zeros(8, device="cuda")
    q = torch.zeros(8, dtype=torch.int8, device="cuda")
    assert L.tango_quantize_f32_i8(x.data_ptr(), 8, x.data_ptr(), q.data_ptr(), 9, None, 0, 0, None, None) == -2
    # GEMM without the workspace it asked for
    assert L.tango_qgemm_bwd_dw(x.data_ptr(), 4, q.data_ptr(), 2, q.data_ptr(), 4, x.data_ptr(), x.data_ptr(),
                                2, 2, 4, None, 0, None) == -4


def test_hot_path_captures_into_a_hip_graph(K, orc):
    rng = np.random.default_rng(1)
    n, e, Kd, N = 2000, 40000, 100, 41
    src, dst = rand_graph(rng, n, e)
    g = make_graph(src, dst, n)
    X = torch.randn(n, Kd, device="cuda")
    W = torch.randn(N, Kd, device="cuda") * 0.1

    def step():
        sX, sW = K.cuda_kernels.get_scale(X), K.cuda_kernels.get_scale(W)
        Xq = torch.empty((n, 112), dtype=torch.int8, device="cuda")[:, :Kd]
        Wq = torch.empty((N, Kd), dtype=torch.int8, device="cuda")
        Y, sY = K.QGEMM_forward(X, Xq, sX, W, Wq, sW, None, True)
        Yq, _ = K.quantize_padded(Y, sY)
        Z = K.csr_SPMM(g, Yq, sY, relu=True)
        e_out, se = K.mySDDMM_int8(g, "dot", Yq.contiguous().view(n, 1, N), Yq.contiguous().view(n, 1, N), sY, sY, True)
        return Z, e_out, se

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        step()  # warm-up outside capture
    torch.cuda.current_stream().wait_stream(stream)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for trial in range(4):
        X.copy_(torch.randn(n, Kd, device="cuda") * (trial + 1))  # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = step()
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b), "replay %d differs from eager" % trial
