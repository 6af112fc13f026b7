"""Committed vectors (tests/golden/, written by tests/golden/make_golden.py):

* the reference's own known-answer input patterns (cuda/src/SDDMM.cu:183-275,
  cuda/src/QGEMM_forward.cu:162-229) with their closed-form expected outputs;
* the published Random123 Philox4x32-10 known answers;
* small seeded cases of every primitive (inputs and outputs).

The CPU tests hold the oracle to them, the GPU tests hold the HIP library to them
through the C ABI without calling the oracle."""
import os

import numpy as np
import pytest
import torch

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def ref():
    return np.load(os.path.join(HERE, "reference_patterns.npz"))


@pytest.fixture(scope="module")
def cases():
    return np.load(os.path.join(HERE, "seeded_cases.npz"))


def sddmm_inputs(dim, H=None):
    tot = 3 * dim * (H or 1)
    shape = (3, dim) if H is None else (3, H, dim)
    U = np.arange(tot).astype(np.int8).reshape(shape)
    V = (tot - np.arange(tot)).astype(np.int8).reshape(shape)
    return U, V


# ------------------------------------------------------------------ oracle
def test_oracle_philox_kat(orc):
    for row in np.load(os.path.join(HERE, "philox_kat.npy")):
        assert np.array_equal(orc.philox4x32_10(row[:4], row[4:6]), row[6:])


def test_oracle_reference_patterns(orc, ref):
    src, dst = ref["sddmm_src"], ref["sddmm_dst"]
    for dim in (4, 16, 40):
        U, V = sddmm_inputs(dim)
        out, _ = orc.sddmm_ewise("add", src, dst, U, V, 1.0, 1.0)
        assert np.array_equal(out, ref["sddmm_add_dim%d" % dim])
    U, V = sddmm_inputs(4, 3)
    out, _ = orc.sddmm_dot(src, dst, U, V, 1.0, 1.0)
    assert np.array_equal(out, ref["sddmm_dot_dim4_H3"])
    Y, _, _, _, _, _, acc = orc.qgemm_fwd(ref["gemm_lcg_A"], ref["gemm_lcg_B"], sX=0.5, sW=0.5, want_acc=True)
    assert np.array_equal(acc, ref["gemm_lcg_acc"]) and np.array_equal(Y, ref["gemm_lcg_Y"])


def test_oracle_seeded_cases(orc, cases):
    c = cases
    s = c["q_scale"]
    assert orc.absmax_scale(c["q_x"]) == s
    assert np.array_equal(orc.quantize(c["q_x"], s), c["q_rne"])
    assert np.array_equal(orc.quantize(c["q_x"], s, mode=orc.TRUNC), c["q_trunc"])
    assert np.array_equal(orc.quantize(c["q_x"], s, mode=orc.STOCHASTIC, noise=c["q_noise"]), c["q_stoch_noise"])
    assert np.array_equal(orc.quantize(c["q_x"], s, mode=orc.STOCHASTIC, seed=77, offset=5), c["q_stoch_philox"])
    assert np.array_equal(orc.transpose_quant(c["tq_x"], orc.absmax_scale(c["tq_x"])), c["tq_out"])
    Y, Xq, Wq, sX, sW, sY, _ = orc.qgemm_fwd(c["g_X"], c["g_W"], c["g_b"], reduce=True, want_acc=True)
    assert np.array_equal(Y, c["g_Y"]) and np.array_equal(Xq, c["g_Xq"]) and np.array_equal(Wq, c["g_Wq"])
    assert (sX, sW, sY) == (c["g_sX"], c["g_sW"], c["g_sY"])
    assert np.array_equal(orc.qgemm_bwd_dx(c["g_dYq"], Wq, c["g_sdY"], sW), c["g_dX"])
    assert np.array_equal(orc.qgemm_bwd_dw(c["g_dYq"], Xq, c["g_sdY"], sX), c["g_dW"])
    n = int(c["s_n"])
    fm = orc.graph_formats(c["s_src"], c["s_dst"], n)
    feat = c["s_feat"]
    assert np.array_equal(orc.spmm_csr_copy_u(fm["adj_csc"][0], fm["adj_csc"][1], feat.reshape(n, -1), c["s_scale"]),
                          c["s_copy_u"])
    assert np.array_equal(orc.spmm_csr_u_mul_e(*fm["adj_csc"], feat, c["s_ev"], c["s_scale"]), c["s_u_mul_e"])
    assert np.array_equal(orc.spmm_incidence(fm["inc_in"][0], fm["inc_in"][1], c["s_E8"], c["s_scale"], n),
                          c["s_incidence"])
    assert np.array_equal(orc.sddmm_dot(c["s_src"], c["s_dst"], feat, c["s_U"], 0.5, 0.25)[0], c["s_dot"])
    assert np.array_equal(orc.sddmm_ewise("sub", c["s_src"], c["s_dst"], feat.reshape(n, -1),
                                          c["s_U"].reshape(n, -1), 0.5, 0.25)[0], c["s_sub"])
    assert np.array_equal(orc.edge_softmax_fwd(c["s_xe"], fm["adj_csc"][0], fm["adj_csc"][2], 0.2), c["s_softmax"])


# --------------------------------------------------------------- HIP library
def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def sc(v):
    return torch.tensor([float(v)], dtype=torch.float32, device="cuda")


def make_graph(src, dst, n):
    from tango_amd.graph import Graph
    from tango_amd.util import graph_preprocess
    return graph_preprocess(Graph(dev(src), dev(dst), n))


@pytest.mark.gpu
def test_hip_reference_patterns(ref):
    from tango_amd import kernels as K
    src, dst = ref["sddmm_src"], ref["sddmm_dst"]
    g = make_graph(src, dst, 3)
    for dim in (4, 16, 40):
        U, V = sddmm_inputs(dim)
        out, _ = K.mySDDMM_int8(g, "add", dev(U), dev(V), sc(1), sc(1), False)
        assert np.array_equal(out.cpu().numpy(), ref["sddmm_add_dim%d" % dim])
    U, V = sddmm_inputs(4, 3)
    out, _ = K.mySDDMM_int8(g, "dot", dev(U), dev(V), sc(1), sc(1), False)
    assert np.array_equal(out.cpu().numpy().reshape(4, 3), ref["sddmm_dot_dim4_H3"])
    # integer-valued inputs and scale 0.5: quantization is exact under every rounding mode
    A, B = dev(ref["gemm_lcg_A"]), dev(ref["gemm_lcg_B"])
    Aq = torch.empty(A.shape, dtype=torch.int8, device="cuda")
    Bq = torch.empty(B.shape, dtype=torch.int8, device="cuda")
    Y = K.QGEMM_forward(A, Aq, sc(0.5), B, Bq, sc(0.5), None, False)
    assert np.array_equal(Y.cpu().numpy(), ref["gemm_lcg_Y"])
    assert np.array_equal(Aq.cpu().numpy(), (2 * ref["gemm_lcg_A"]).astype(np.int8))
    Y2 = torch.empty_like(Y)
    K.cuda_kernels.QGEMM_i8(Y2, Aq, Bq, None, None, sc(0.5), sc(0.5))  # the cached-operand int8 entry point
    assert np.array_equal(Y2.cpu().numpy(), ref["gemm_lcg_Y"])
    # 0.25 * acc is exact in fp32 here, so Y pins the int32 accumulators too
    assert np.array_equal((Y2.cpu().numpy() * 4).astype(np.int32), ref["gemm_lcg_acc"])


@pytest.mark.gpu
def test_hip_seeded_cases(cases):
    from tango_amd import kernels as K
    c = cases
    x = dev(c["q_x"])
    s = K.cuda_kernels.get_scale(x)
    assert s.cpu().numpy()[0] == c["q_scale"]
    for mode, key, kw in (("rne", "q_rne", {}), ("trunc", "q_trunc", {}),
                          ("stochastic", "q_stoch_noise", {"noise": dev(c["q_noise"])}),
                          ("stochastic", "q_stoch_philox", {"seed": 77, "offset": 5})):
        q, _ = K.quantize(x, s, round_mode=mode, **kw)
        assert np.array_equal(q.cpu().numpy(), c[key]), key
    t = dev(c["tq_x"])
    tq = K.cuda_kernels.transpose_quant(t, K.cuda_kernels.get_scale(t), t.size(0), t.size(1))
    assert np.array_equal(tq.cpu().numpy(), c["tq_out"])
    X, W, b = dev(c["g_X"]), dev(c["g_W"]), dev(c["g_b"])
    Xq = torch.empty(X.shape, dtype=torch.int8, device="cuda")
    Wq = torch.empty(W.shape, dtype=torch.int8, device="cuda")
    sX, sW = K.cuda_kernels.get_scale(X), K.cuda_kernels.get_scale(W)
    Y, sY = K.QGEMM_forward(X, Xq, sX, W, Wq, sW, b, True)
    assert np.array_equal(Y.cpu().numpy(), c["g_Y"]) and np.array_equal(Xq.cpu().numpy(), c["g_Xq"])
    assert np.array_equal(Wq.cpu().numpy(), c["g_Wq"]) and sY.cpu().numpy()[0] == c["g_sY"]
    dX, dW = K.QGEMM_backward(dev(c["g_dYq"]), Xq, Wq, sc(c["g_sdY"]), sX, sW, True, True)
    assert np.array_equal(dX.cpu().numpy(), c["g_dX"]) and np.array_equal(dW.cpu().numpy(), c["g_dW"])
    n = int(c["s_n"])
    g = make_graph(c["s_src"], c["s_dst"], n)
    feat = dev(c["s_feat"])
    assert np.array_equal(K.csr_SPMM(g, feat.view(n, -1), sc(c["s_scale"])).cpu().numpy(), c["s_copy_u"])
    assert np.array_equal(K.multi_cusparse_SPMM(g, feat, dev(c["s_ev"]), sc(c["s_scale"])).cpu().numpy(),
                          c["s_u_mul_e"])
    assert np.array_equal(K.incidence_SPMM(g, dev(c["s_E8"]), sc(c["s_scale"])).cpu().numpy(), c["s_incidence"])
    dot, _ = K.mySDDMM_int8(g, "dot", feat, dev(c["s_U"]), sc(0.5), sc(0.25), False)
    assert np.array_equal(dot.cpu().numpy().reshape(c["s_dot"].shape), c["s_dot"])
    sub, _ = K.mySDDMM_int8(g, "sub", feat.view(n, -1), dev(c["s_U"]).view(n, -1), sc(0.5), sc(0.25), False)
    assert np.array_equal(sub.cpu().numpy(), c["s_sub"])
    ip, _, eid = g.adj_csc
    a = K.cuda_kernels.edge_softmax_forward(dev(c["s_xe"]), ip, eid, 0.2)
    assert np.allclose(a.cpu().numpy(), c["s_softmax"], rtol=1e-5, atol=1e-6)
