"""Pins the CPU oracle with checks that do not retype its formulas.

The reference holds no stored outputs for this path (its evaluation scripts
print or discard results), so the pins are: published known-answer vectors
(Philox), the two input patterns of the reference's TEST mains with their
closed-form answers (cuda/src/SDDMM.cu:230-275, cuda/src/QGEMM_forward.cu:
159-229), dense brute force, scipy / torch integer matmul, and algebraic
invariants chosen so that a dropped term, a swapped operand or a wrong index
fails at least one of them.
"""
import numpy as np
import pytest
import scipy.sparse as sp
import torch


def rand_graph(rng, n, e):
    src = rng.integers(0, n, e)
    dst = rng.integers(0, n, e)
    return src.astype(np.int64), dst.astype(np.int64)


# ----------------------------------------------------------------- Philox
def test_philox_known_answers(orc):
    # Random123 kat_vectors, philox4x32 with 10 rounds
    kat = [
        ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
        ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
        ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
         [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
    ]
    for ctr, key, want in kat:
        assert list(orc.philox4x32_10(ctr, key)) == want


def test_philox_uniform_layout(orc):
    # element g uses word g&3 of block g>>2; key = seed split lo/hi
    seed = 0x299f31d0a4093822
    for g in (0, 1, 2, 3, 4, 7, (1 << 34) + 5):
        blk = orc.philox4x32_10([(g >> 2) & 0xffffffff, (g >> 2) >> 32, 0, 0],
                                [seed & 0xffffffff, seed >> 32])
        assert orc.philox_uniform(seed, g) == float(blk[g & 3] >> 8) / float(1 << 24)
    u = np.array([orc.philox_uniform(7, g) for g in range(20000)])
    assert u.min() >= 0.0 and u.max() < 1.0 and abs(u.mean() - 0.5) < 0.01


# ----------------------------------------------------------- quantization
def test_absmax_scale_closed_form(orc):
    rng = np.random.default_rng(0)
    for n in (1, 2, 3, 4, 5, 7, 1023, 4097):  # tails n % 4 in {1,2,3} included
        x = rng.standard_normal(n).astype(np.float32)
        assert orc.absmax_scale(x) == np.float32(np.abs(x).max()) / np.float32(127)
    # the maximum sits in the last (tail) position, which the reference drops
    x = np.zeros(9, np.float32)
    x[8] = -3.0
    assert orc.absmax_scale(x) == np.float32(3.0) / np.float32(127)
    assert orc.absmax_scale(np.zeros(5, np.float32)) == 0.0


def test_quantize_rne_ties_clamp_zero(orc):
    s = np.float32(1.0)
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, 300.0, -300.0, 0.0, 0.49999997],
                 np.float32)
    want = [0, 2, 2, 0, -2, -2, 126, 127, 127, -127, 0, 0]
    assert list(orc.quantize(x, s, orc.RNE)) == want
    # truncation toward zero
    x = np.array([0.99, -0.99, 1.5, -1.5, 126.99, -126.99, 127.9, -500.0], np.float32)
    assert list(orc.quantize(x, s, orc.TRUNC)) == [0, 0, 1, -1, 126, -126, 127, -127]
    # all-zero tensor: scale 0 -> zeros, not NaN garbage
    assert not orc.quantize(np.zeros(7, np.float32), 0.0, orc.RNE).any()


def test_quantize_matches_numpy_ieee(orc):
    rng = np.random.default_rng(1)
    x = rng.standard_normal(100003).astype(np.float32)
    s = orc.absmax_scale(x)
    r = np.float32(1.0) / s
    p = (x * r).astype(np.float32)
    assert np.array_equal(orc.quantize(x, s, orc.RNE), np.clip(np.rint(p), -127, 127).astype(np.int8))
    assert np.array_equal(orc.quantize(x, s, orc.TRUNC), np.clip(np.trunc(p), -127, 127).astype(np.int8))
    # the absmax element maps to +-127 under RNE
    q = orc.quantize(x, s, orc.RNE)
    assert abs(int(q[np.abs(x).argmax()])) == 127
    u = rng.random(x.size, dtype=np.float32)
    want = np.clip(np.floor((p + u).astype(np.float32)), -127, 127).astype(np.int8)
    assert np.array_equal(orc.quantize(x, s, orc.STOCHASTIC, noise=u), want)


def test_stochastic_rounding_unbiased(orc):
    rng = np.random.default_rng(2)
    x = rng.standard_normal(1 << 20).astype(np.float32)
    s = orc.absmax_scale(x)
    q = orc.quantize(x, s, orc.STOCHASTIC, seed=1234, offset=0)
    err = (q.astype(np.float64) * float(s) - x).mean()
    assert abs(err) < 1e-3
    # deterministic rounding of the same data is unbiased too, but stochastic
    # rounding must differ from it element-wise and be reproducible by seed
    assert not np.array_equal(q, orc.quantize(x, s, orc.RNE))
    assert np.array_equal(q, orc.quantize(x, s, orc.STOCHASTIC, seed=1234, offset=0))
    # offset shifts the stream: elements [100:] at offset 0 == elements [0:] at offset 100
    q2 = orc.quantize(x[100:], s, orc.STOCHASTIC, seed=1234, offset=100)
    assert np.array_equal(q[100:], q2)
    # for a constant input the rounding-up frequency equals the fraction
    c = np.full(200000, 0.3, np.float32)
    qc = orc.quantize(c, 1.0, orc.STOCHASTIC, seed=5)
    assert set(np.unique(qc)) == {0, 1} and abs(qc.mean() - 0.3) < 5e-3


def test_quantize_rows_and_transpose(orc):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((37, 41)).astype(np.float32)
    s = orc.absmax_rows(x)
    assert np.array_equal(s, np.abs(x).max(1).astype(np.float32) / np.float32(127))
    q = orc.quantize_rows(x, s, True, ldq=48)
    assert q.shape == (37, 48) and not q[:, 41:].any()
    for r in range(37):
        assert np.array_equal(q[r, :41], orc.quantize(x[r], s[r]))
    st = orc.absmax_scale(x)
    assert np.array_equal(orc.quantize_rows(x, st, False)[:, :41], orc.quantize(x, st))
    assert np.array_equal(orc.transpose_quant(x, st), orc.quantize(x, st).T)
    e = rng.standard_normal((50, 4, 2)).astype(np.float32)
    se = orc.absmax_scale(e)
    assert np.array_equal(orc.transpose_quant(e, se), orc.quantize(e, se).reshape(50, 8).T)


# ------------------------------------------------------------------- GEMM
def lcg_matrix(rows, cols, seed):
    # input pattern of the reference's TEST main, cuda/src/QGEMM_forward.cu:162-181:
    # column-major fill, value = ((offset + seed) * 16807 mod 16) - 8
    off = np.arange(rows * cols, dtype=np.int64)
    v = ((off + seed) * 16807 % 16 - 8).astype(np.float32)
    return v.reshape(cols, rows).T.copy()


def test_qgemm_fwd_reference_lcg_pattern(orc):
    # integer-valued inputs with scale 0.5 make quantization exact: q = 2*x
    M, N, K = 96, 40, 64
    A = lcg_matrix(M, K, 41)
    B = lcg_matrix(N, K, 17)
    # force absmax to exactly 8 so that s = 8/127 is not a power of two; use explicit scales
    Y, Xq, Wq, sX, sW, _, acc = orc.qgemm_fwd(A, B, sX=0.5, sW=0.5, want_acc=True)
    assert np.array_equal(Xq, (2 * A).astype(np.int8)) and np.array_equal(Wq, (2 * B).astype(np.int8))
    want = (2 * A).astype(np.int64) @ (2 * B).astype(np.int64).T
    assert np.array_equal(acc, want)
    # dequantized result equals the fp32 product exactly (all values are small integers)
    assert np.array_equal(Y, (A.astype(np.float64) @ B.astype(np.float64).T).astype(np.float32))
    assert np.abs(Y - A @ B.T).max() <= 1e-3  # the tolerance the reference's TEST main uses


def test_qgemm_fwd_vs_torch_int_mm(orc):
    rng = np.random.default_rng(4)
    for (M, N, K) in ((64, 16, 128), (33, 41, 602), (17, 24, 8)):
        X = rng.standard_normal((M, K)).astype(np.float32)
        W = (rng.random((N, K), dtype=np.float32) - 0.5) * 0.2
        b = rng.standard_normal(N).astype(np.float32)
        Y, Xq, Wq, sX, sW, sY, acc = orc.qgemm_fwd(X, W, bias=b, reduce=True, want_acc=True)
        assert np.array_equal(Xq, orc.quantize(X, sX, orc.TRUNC))
        assert np.array_equal(Wq, orc.quantize(W, sW, orc.TRUNC))
        want = (torch.from_numpy(Xq).to(torch.int32) @ torch.from_numpy(Wq).to(torch.int32).T).numpy()
        assert np.array_equal(acc, want)
        s = np.float32(sX) * np.float32(sW)
        yy = b + (s * acc.astype(np.float32)).astype(np.float32)
        assert np.array_equal(Y, yy.astype(np.float32))
        assert sY == orc.absmax_scale(Y)  # epilogue absmax == absmax of the stored output
        # quantized product approximates the fp32 product
        ref = X @ W.T + b
        assert np.abs(Y - ref).max() < 0.05 * np.abs(ref).max()
    assert orc.overflow_count() == 0


def test_qgemm_backward_vs_dense(orc):
    rng = np.random.default_rng(5)
    M, N, K = 301, 41, 72
    dY = rng.integers(-127, 128, (M, N)).astype(np.int8)
    X = rng.integers(-127, 128, (M, K)).astype(np.int8)
    W = rng.integers(-127, 128, (N, K)).astype(np.int8)
    s1, s2 = np.float32(0.013), np.float32(0.27)
    s = s1 * s2
    dX = orc.qgemm_bwd_dx(dY, W, s1, s2)
    assert np.array_equal(dX, s * (dY.astype(np.int64) @ W.astype(np.int64)).astype(np.float32))
    dW = orc.qgemm_bwd_dw(dY, X, s1, s2)
    assert np.array_equal(dW, s * (dY.astype(np.int64).T @ X.astype(np.int64)).astype(np.float32))
    # transposition identity ties the two: dW(dY, X)^T == dX-style product of X^T and dY
    assert np.array_equal(dW.T, s * (X.astype(np.int64).T @ dY.astype(np.int64)).astype(np.float32))


def test_int32_overflow_is_detected(orc):
    orc.overflow_reset()
    M = 140000  # 127*127*140000 > 2^31
    dY = np.full((M, 1), 127, np.int8)
    X = np.full((M, 4), 127, np.int8)
    orc.qgemm_bwd_dw(dY, X, 1.0, 1.0)
    assert orc.overflow_count() == 4
    orc.overflow_reset()


def test_qgemm_legacy(orc):
    rng = np.random.default_rng(6)
    A = rng.standard_normal((9, 12)).astype(np.float32)
    B = rng.standard_normal((7, 12)).astype(np.float32)
    sA, sB = orc.absmax_scale(A), orc.absmax_scale(B)
    qa, qb = orc.quantize(A, sA).astype(np.int64), orc.quantize(B, sB).astype(np.int64)
    s = sA * sB
    assert np.array_equal(orc.qgemm_legacy(A, B, False, True), (qa @ qb.T).astype(np.float32) * s)
    assert np.array_equal(orc.qgemm_legacy(A, B.T.copy(), False, False), (qa @ qb.T).astype(np.float32) * s)
    assert np.array_equal(orc.qgemm_legacy(A.T.copy(), B.T.copy(), True, False),
                          (qa @ qb.T).astype(np.float32) * s)


# ------------------------------------------------------------------- SpMM
def test_graph_formats(orc):
    src = np.array([2, 0, 1, 0, 2, 2])
    dst = np.array([1, 1, 2, 0, 0, 1])
    g = orc.graph_formats(src, dst, 3)
    ip, ix, eid = g["adj_csr"]
    assert list(ip) == [0, 2, 3, 6] and list(ix) == [1, 0, 2, 1, 0, 1] and list(eid) == [1, 3, 2, 0, 4, 5]
    ip, ix, eid = g["adj_csc"]
    assert list(ip) == [0, 2, 5, 6] and list(ix) == [0, 2, 2, 0, 2, 1] and list(eid) == [3, 4, 0, 1, 5, 2]
    assert g["inc_in"].tolist() == [[0, 0, 1, 1, 1, 2], [3, 4, 0, 1, 5, 2]]
    assert g["inc_out"].tolist() == [[0, 0, 1, 2, 2, 2], [1, 3, 2, 0, 4, 5]]


def test_spmm_copy_u_vs_dense_and_scipy(orc):
    rng = np.random.default_rng(7)
    n, e = 50, 400
    src, dst = rand_graph(rng, n, e)  # duplicates on purpose: multigraph edges count twice
    g = orc.graph_formats(src, dst, n)
    for F in (1, 3, 16, 41, 64):
        feat = rng.integers(-127, 128, (n, F)).astype(np.int8)
        s = np.float32(0.037)
        A = np.zeros((n, n), np.int64)
        np.add.at(A, (dst, src), 1)
        ip, ix, _ = g["adj_csc"]
        out = orc.spmm_csr_copy_u(ip, ix, feat, s)
        assert np.array_equal(out, s * (A @ feat.astype(np.int64)).astype(np.float32))
        ip, ix, _ = g["adj_csr"]  # reverse = transpose
        out_r = orc.spmm_csr_copy_u(ip, ix, feat, s)
        assert np.array_equal(out_r, s * (A.T @ feat.astype(np.int64)).astype(np.float32))
    # all-ones feature -> in-degree * s
    ip, ix, _ = g["adj_csc"]
    ones = np.ones((n, 4), np.int8)
    assert np.array_equal(orc.spmm_csr_copy_u(ip, ix, ones, 1.0)[:, 0], np.bincount(dst, minlength=n))
    # scipy on a larger graph
    n, e = 3000, 60000
    src, dst = rand_graph(rng, n, e)
    g = orc.graph_formats(src, dst, n)
    ip, ix, _ = g["adj_csc"]
    feat = rng.integers(-127, 128, (n, 24)).astype(np.int8)
    A = sp.csr_matrix((np.ones(e, np.int64), ix, ip), shape=(n, n))
    assert np.array_equal(orc.spmm_csr_copy_u(ip, ix, feat, 0.5), 0.5 * (A @ feat.astype(np.int64)).astype(np.float32))
    # padded rows: only the first F columns count
    padded = np.concatenate([feat, np.full((n, 8), 99, np.int8)], 1)
    assert np.array_equal(orc.spmm_csr_copy_u(ip, ix, padded, 0.5, F=24), orc.spmm_csr_copy_u(ip, ix, feat, 0.5))


def test_spmm_u_mul_e_vs_dense(orc):
    rng = np.random.default_rng(8)
    n, e, H, F = 40, 300, 3, 5
    src, dst = rand_graph(rng, n, e)
    g = orc.graph_formats(src, dst, n)
    feat = rng.integers(-127, 128, (n, H, F)).astype(np.int8)
    ev = rng.integers(-127, 128, (H, 1, e)).astype(np.int8)  # edge-id order
    s = np.float32(0.011)
    want = np.zeros((n, H, F), np.int64)
    for i in range(e):
        want[dst[i]] += ev[:, 0, i].astype(np.int64)[:, None] * feat[src[i]].astype(np.int64)
    ip, ix, eid = g["adj_csc"]
    # fused permutation == index_select first (cuda/kernels.py:133-135)
    a = orc.spmm_csr_u_mul_e(ip, ix, eid, feat, ev, s)
    b = orc.spmm_csr_u_mul_e(ip, ix, None, feat, ev[:, :, eid], s)
    assert np.array_equal(a, s * want.astype(np.float32)) and np.array_equal(a, b)
    # reverse direction
    want_r = np.zeros((n, H, F), np.int64)
    for i in range(e):
        want_r[src[i]] += ev[:, 0, i].astype(np.int64)[:, None] * feat[dst[i]].astype(np.int64)
    ip, ix, eid = g["adj_csr"]
    assert np.array_equal(orc.spmm_csr_u_mul_e(ip, ix, eid, feat, ev, s), s * want_r.astype(np.float32))
    # element-wise edge values (D == F)
    evd = rng.integers(-127, 128, (H, F, e)).astype(np.int8)
    want_e = np.zeros((n, H, F), np.int64)
    for i in range(e):
        want_e[dst[i]] += evd[:, :, i].astype(np.int64) * feat[src[i]].astype(np.int64)
    ip, ix, eid = g["adj_csc"]
    assert np.array_equal(orc.spmm_csr_u_mul_e(ip, ix, eid, feat, evd, s), s * want_e.astype(np.float32))
    # all-ones edge values reduce u_mul_e to copy_u
    one = np.ones((H, 1, e), np.int8)
    assert np.array_equal(orc.spmm_csr_u_mul_e(ip, ix, eid, feat, one, s).reshape(n, -1),
                          orc.spmm_csr_copy_u(ip, ix, feat.reshape(n, -1), s))


def test_incidence_equals_csr_on_incidence_matrix(orc):
    rng = np.random.default_rng(9)
    n, e, F = 30, 200, 8
    src, dst = rand_graph(rng, n, e)
    g = orc.graph_formats(src, dst, n)
    E = rng.integers(-127, 128, (e, F)).astype(np.int8)
    s = np.float32(0.21)
    want = np.zeros((n, F), np.int64)
    np.add.at(want, dst, E.astype(np.int64))
    out = orc.spmm_incidence(g["inc_in"][0], g["inc_in"][1], E, s, n)
    assert np.array_equal(out, s * want.astype(np.float32))
    # the equivalence the reference itself relies on (evaluation/test_incidence.py:14-22)
    ip, _, eid = g["adj_csc"]
    assert np.array_equal(out, orc.spmm_csr_copy_u(ip, eid, E, s))
    want_o = np.zeros((n, F), np.int64)
    np.add.at(want_o, src, E.astype(np.int64))
    assert np.array_equal(orc.spmm_incidence(g["inc_out"][0], g["inc_out"][1], E, s, n),
                          s * want_o.astype(np.float32))


# ------------------------------------------------------------------ SDDMM
def test_sddmm_reference_test_pattern(orc):
    # cuda/src/SDDMM.cu:238-258: 3 vertices, edges (0,0),(0,1),(0,2),(1,2),
    # U[i] = i, V[i] = 3*dim - i, scales 1, op Add
    src = np.array([0, 0, 0, 1])
    dst = np.array([0, 1, 2, 2])
    for dim in (4, 16, 40):
        U = np.arange(3 * dim).astype(np.int8).reshape(3, dim)
        V = (3 * dim - np.arange(3 * dim)).astype(np.int8).reshape(3, dim)
        out, _ = orc.sddmm_ewise("add", src, dst, U, V, 1.0, 1.0)
        j = np.arange(dim)
        for e in range(4):
            want = (src[e] * dim + j) + (3 * dim - dst[e] * dim - j)
            assert np.array_equal(out[e], want.astype(np.float32))
    # dot twin (cuda/src/SDDMM.cu:183-228): out[e,h] = sum_j U[src,h,j] * V[dst,h,j]
    dim, H = 4, 3
    tot = 3 * dim * H
    U = np.arange(tot).astype(np.int8).reshape(3, H, dim)
    V = (tot - np.arange(tot)).astype(np.int8).reshape(3, H, dim)
    out, _ = orc.sddmm_dot(src, dst, U, V, 1.0, 1.0)
    for e in range(4):
        for h in range(H):
            a = (src[e] * H + h) * dim + np.arange(dim)
            b = tot - ((dst[e] * H + h) * dim + np.arange(dim))
            assert out[e, h] == float((a * b).sum())


def test_sddmm_random_vs_numpy(orc):
    rng = np.random.default_rng(10)
    n, e, H, D = 25, 180, 8, 16
    src, dst = rand_graph(rng, n, e)
    U = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
    V = rng.integers(-127, 128, (n, H, D)).astype(np.int8)
    sU, sV = np.float32(0.02), np.float32(0.3)
    out, so = orc.sddmm_dot(src, dst, U, V, sU, sV, reduce=True)
    acc = (U[src].astype(np.int64) * V[dst].astype(np.int64)).sum(-1)
    assert np.array_equal(out, acc.astype(np.float32) * (sU * sV))
    assert so == orc.absmax_scale(out)
    # symmetry: swapping operands and edge direction gives the same values
    out2, _ = orc.sddmm_dot(dst, src, V, U, sV, sU)
    assert np.array_equal(out, out2)
    fu, fv = U.reshape(n, -1).astype(np.float32) * sU, V.reshape(n, -1).astype(np.float32) * sV
    for op, fn in (("add", np.add), ("sub", np.subtract), ("mul", np.multiply)):
        o, so = orc.sddmm_ewise(op, src, dst, U.reshape(n, -1), V.reshape(n, -1), sU, sV, reduce=True)
        assert np.array_equal(o, fn(fu[src], fv[dst]).astype(np.float32))
        assert so == orc.absmax_scale(o)
    Vnz = np.where(V == 0, 1, V).astype(np.int8)
    o, _ = orc.sddmm_ewise("div", src, dst, U.reshape(n, -1), Vnz.reshape(n, -1), sU, sV)
    assert np.array_equal(o, (fu[src] / (Vnz.reshape(n, -1).astype(np.float32) * sV)[dst]).astype(np.float32))


# ----------------------------------------------------------- edge softmax
def test_edge_softmax_properties(orc):
    rng = np.random.default_rng(11)
    n, e, H = 20, 150, 4
    src, dst = rand_graph(rng, n, e)
    g = orc.graph_formats(src, dst, n)
    ip, _, eid = g["adj_csc"]
    x = rng.standard_normal((e, H)).astype(np.float32) * 3
    a = orc.edge_softmax_fwd(x, ip, eid)
    sums = np.zeros((n, H))
    np.add.at(sums, dst, a)
    has = np.bincount(dst, minlength=n) > 0
    assert np.allclose(sums[has], 1.0, atol=1e-6) and (a > 0).all()
    # shift invariance per destination
    shift = rng.standard_normal((n, H)).astype(np.float32)
    assert np.allclose(orc.edge_softmax_fwd(x + shift[dst], ip, eid), a, atol=1e-6)
    # against torch softmax per destination group, with LeakyReLU folded in
    al = orc.edge_softmax_fwd(x, ip, eid, slope=0.2)
    xt = torch.from_numpy(x).double()
    for v in np.nonzero(has)[0][:10]:
        m = np.nonzero(dst == v)[0]
        want = torch.softmax(torch.nn.functional.leaky_relu(xt[m], 0.2), 0).float().numpy()
        assert np.allclose(al[m], want, atol=1e-6, rtol=1e-5)
    # backward against autograd
    da = rng.standard_normal((e, H)).astype(np.float32)
    de = orc.edge_softmax_bwd(al, da, x, ip, eid, slope=0.2)
    xt = torch.from_numpy(x).double().requires_grad_(True)
    z = torch.nn.functional.leaky_relu(xt, 0.2)
    out = torch.zeros_like(z)
    for v in np.nonzero(has)[0]:
        m = torch.from_numpy(np.nonzero(dst == v)[0])
        out = out.index_copy(0, m, torch.softmax(z[m], 0))
    out.backward(torch.from_numpy(da).double())
    assert np.allclose(de, xt.grad.float().numpy(), atol=1e-5, rtol=1e-4)


# ------------------------------------------------------------ fused forms
# Each fused oracle function must equal the chain of separate numpy fp32 passes (one IEEE rounding per
# operation, numpy never contracts) over the unfused oracle function that is pinned above.
def _csr(rng, n, e):
    src, dst = rand_graph(rng, n, e)
    order = np.argsort(dst, kind="stable")
    indptr = np.zeros(n + 1, np.int64)
    np.cumsum(np.bincount(dst, minlength=n), out=indptr[1:])
    return indptr, src[order], order.astype(np.int64)


def test_fused_copy_u_epilogue_is_the_chain_of_separate_passes(orc):
    rng = np.random.default_rng(21)
    n, F = 300, 48
    indptr, indices, _ = _csr(rng, n, 5000)
    feat = rng.integers(-127, 128, (n, F)).astype(np.int8)
    rs = (rng.random(n) + 0.05).astype(np.float32)
    bias = rng.standard_normal(F).astype(np.float32)
    s = np.float32(0.0173)
    base = orc.spmm_csr_copy_u(indptr, indices, feat, s)
    assert np.array_equal(orc.spmm_csr_copy_u_ex(indptr, indices, feat, s), base)
    assert np.array_equal(orc.spmm_csr_copy_u_ex(indptr, indices, feat, s, row_scale=rs), base * rs[:, None])
    assert np.array_equal(orc.spmm_csr_copy_u_ex(indptr, indices, feat, s, bias=bias), base + bias)
    chain = base * rs[:, None] + bias
    out, bits = orc.spmm_csr_copy_u_ex(indptr, indices, feat, s, row_scale=rs, bias=bias, act=1, want_bits=True)
    assert np.array_equal(out, np.maximum(chain, 0))
    unpacked = np.unpackbits(bits.view(np.uint8).reshape(n, F // 16, 2), axis=-1, bitorder="little").reshape(n, F)
    assert np.array_equal(unpacked.astype(bool), chain > 0)
    # a dropped row scale, a bias added before the row scale or a mask taken before the bias all fail this
    assert not np.array_equal(out, np.maximum((base + bias) * rs[:, None], 0))
    elu = orc.spmm_csr_copy_u_ex(indptr, indices, feat, s, row_scale=rs, bias=bias, act=2)
    want = np.where(chain > 0, chain, np.expm1(chain.astype(np.float64)))
    np.testing.assert_allclose(elu, want, rtol=1e-6, atol=1e-6)


def test_fused_u_mul_e_epilogue(orc):
    rng = np.random.default_rng(22)
    n, H, F = 200, 3, 8
    indptr, indices, eids = _csr(rng, n, 3000)
    feat = rng.integers(-127, 128, (n, H, F)).astype(np.int8)
    ev = rng.integers(-127, 128, (3000, H, 1)).astype(np.int8)  # edge-major
    evT = np.ascontiguousarray(ev.reshape(3000, H).T).reshape(H, 1, 3000)
    sN, sE = np.float32(0.011), np.float32(0.0007)
    bias = rng.standard_normal(H * F).astype(np.float32)
    base = orc.spmm_csr_u_mul_e(indptr, indices, eids, feat, evT, np.float32(sN * sE))
    got = orc.spmm_csr_u_mul_e_ex(indptr, indices, eids, feat, ev, sN, scale2=sE, edge_major=True)
    assert np.array_equal(got, base)
    got = orc.spmm_csr_u_mul_e_ex(indptr, indices, eids, feat, evT, sN, scale2=sE, bias=bias, act=1)
    assert np.array_equal(got, np.maximum(base + bias.reshape(1, H, F), 0))


def test_masked_absmax_and_quantize(orc):
    rng = np.random.default_rng(23)
    rows, cols = 257, 48
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    act_out = rng.standard_normal((rows, cols)).astype(np.float32)
    act_out[rng.random((rows, cols)) < 0.1] = 0.0  # exact zeros belong to the masked side
    rm = (rng.random(rows) + 0.1).astype(np.float32)
    relu_x = np.where(act_out > 0, x, np.float32(0))
    elu_x = np.where(act_out > 0, x, x * (act_out + np.float32(1)))
    packed = np.packbits((act_out > 0).reshape(rows, cols // 16, 16), axis=-1, bitorder="little").view(np.uint16)
    packed = packed.reshape(rows, cols // 16)
    for mask, mode, xm in ((act_out, "relu", relu_x), (act_out, "elu", elu_x), (packed, "bits", relu_x), (None, "relu", x)):
        for row_mul in (None, rm):
            y = xm if row_mul is None else xm * row_mul[:, None]
            s, cs = orc.absmax_ex(x, row_mul=row_mul, mask=mask, mask_mode=mode, want_colsum=True)
            assert s == orc.absmax_scale(y)
            np.testing.assert_allclose(cs, xm.astype(np.float64).sum(0), rtol=1e-12)
            for kw in ({"mode": orc.RNE}, {"mode": orc.STOCHASTIC, "seed": 5, "offset": 1 << 40}):
                q = orc.quantize_rows_ex(x, s, row_mul=row_mul, mask=mask, mask_mode=mode, ldq=64, **kw)
                assert np.array_equal(q[:, :cols], orc.quantize(y, s, **kw)) and not q[:, cols:].any()


def test_int8_input_forward_and_accumulating_gradx(orc):
    rng = np.random.default_rng(24)
    M, K, N = 70, 100, 24
    A = rng.integers(-127, 128, (M, K)).astype(np.int8)
    B = rng.integers(-127, 128, (N, K)).astype(np.int8)
    bias = rng.standard_normal(N).astype(np.float32)
    sA, sB = np.float32(0.013), np.float32(0.0021)
    acc = A.astype(np.int64) @ B.astype(np.int64).T
    want = np.float32(sA * sB) * acc.astype(np.float32) + bias
    Y, sY = orc.qgemm_i8_nt(A, B, sA, sB, bias=bias, reduce=True)
    assert np.array_equal(Y, want) and sY == orc.absmax_scale(want)
    # the int8 operands of the fp32-input forward give the same result through this entry
    X = rng.standard_normal((M, K)).astype(np.float32)
    W = rng.standard_normal((N, K)).astype(np.float32)
    Yf, Xq, Wq, sX, sW, _ = orc.qgemm_fwd(X, W, bias=bias, reduce=True)
    assert np.array_equal(orc.qgemm_i8_nt(Xq, Wq, sX, sW, bias=bias), Yf)
    # gradX: row scale in the epilogue, then one fp32 add into the running gradient
    dY = rng.integers(-127, 128, (M, N)).astype(np.int8)
    rs = (rng.random(M) + 0.2).astype(np.float32)
    prev = rng.standard_normal((M, K)).astype(np.float32)
    plain = orc.qgemm_bwd_dx(dY, B, 0.02, sB)
    assert np.array_equal(orc.qgemm_bwd_dx_ex(dY, B, 0.02, sB), plain)
    assert np.array_equal(orc.qgemm_bwd_dx_ex(dY, B, 0.02, sB, row_scale=rs), plain * rs[:, None])
    assert np.array_equal(orc.qgemm_bwd_dx_ex(dY, B, 0.02, sB, row_scale=rs, accumulate_into=prev),
                          prev + plain * rs[:, None])
