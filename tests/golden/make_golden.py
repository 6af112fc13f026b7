"""Writes the fixtures of this directory.  Run from the repository root:

    python tests/golden/make_golden.py

Two kinds of vectors:

* the two known-answer input patterns the reference's own native tests hold
  (cuda/src/SDDMM.cu:183-275: 3 vertices, 4 edges, U[i] = i, V[i] = total - i, scales 1;
  cuda/src/QGEMM_forward.cu:162-229: column-major LCG fill ((offset + seed) * 16807 mod 16) - 8,
  seeds 41 and 17, scales 0.5).  The reference stores no outputs for them; the expected values
  here are their closed forms, computed with numpy integer arithmetic and NOT with the oracle;

* small seeded cases of every primitive, inputs and outputs, produced by the CPU oracle after an
  independent numpy check of each (asserted below before anything is written).  They freeze the
  oracle's behaviour and give the GPU tests vectors that do not depend on the oracle's build.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as orc  # noqa: E402


def lcg_matrix(rows, cols, seed):
    off = np.arange(rows * cols, dtype=np.int64)
    v = ((off + seed) * 16807 % 16 - 8).astype(np.float32)
    return v.reshape(cols, rows).T.copy()


def reference_patterns():
    out = {}
    src = np.array([0, 0, 0, 1], dtype=np.int64)
    dst = np.array([0, 1, 2, 2], dtype=np.int64)
    out["sddmm_src"], out["sddmm_dst"] = src, dst
    for dim in (4, 16, 40):
        j = np.arange(dim)
        want = np.stack([(src[e] * dim + j) + (3 * dim - dst[e] * dim - j) for e in range(4)])
        out["sddmm_add_dim%d" % dim] = want.astype(np.float32)
    dim, H = 4, 3
    tot = 3 * dim * H
    want = np.zeros((4, H), dtype=np.float32)
    for e in range(4):
        for h in range(H):
            a = (src[e] * H + h) * dim + np.arange(dim)
            b = tot - ((dst[e] * H + h) * dim + np.arange(dim))
            want[e, h] = float((a * b).sum())
    out["sddmm_dot_dim4_H3"] = want
    M, N, K = 96, 40, 64
    A, B = lcg_matrix(M, K, 41), lcg_matrix(N, K, 17)
    acc = (2 * A).astype(np.int64) @ (2 * B).astype(np.int64).T  # q = x / 0.5 exactly
    out["gemm_lcg_A"], out["gemm_lcg_B"] = A, B
    out["gemm_lcg_acc"] = acc.astype(np.int32)
    out["gemm_lcg_Y"] = (np.float32(0.25) * acc.astype(np.float32)).astype(np.float32)
    return out


def seeded_cases():
    rng = np.random.default_rng(20240611)
    o = {}
    # quantize: three rounding modes, ragged length
    x = (rng.standard_normal(1003) * 3).astype(np.float32)
    x[:4] = [0.0, -0.0, x.max() * 2, -x.max() * 2]
    s = orc.absmax_scale(x)
    assert s == np.float32(np.abs(x).max() / np.float32(127.0))
    r = np.float32(1.0) / s
    noise = rng.random(x.size, dtype=np.float32)
    q_rne = orc.quantize(x, s)
    q_tr = orc.quantize(x, s, mode=orc.TRUNC)
    q_st = orc.quantize(x, s, mode=orc.STOCHASTIC, noise=noise)
    assert np.array_equal(q_rne, np.clip(np.rint(x * r), -127, 127).astype(np.int8))
    assert np.array_equal(q_tr, np.clip(np.trunc(x * r), -127, 127).astype(np.int8))
    assert np.array_equal(q_st, np.clip(np.floor(x * r + noise), -127, 127).astype(np.int8))
    q_ph = orc.quantize(x, s, mode=orc.STOCHASTIC, seed=77, offset=5)
    o.update(q_x=x, q_scale=s, q_noise=noise, q_rne=q_rne, q_trunc=q_tr, q_stoch_noise=q_st, q_stoch_philox=q_ph)
    # transpose_quant
    t = rng.standard_normal((37, 6)).astype(np.float32)
    st = orc.absmax_scale(t)
    tq = orc.transpose_quant(t, st)
    assert np.array_equal(tq, orc.quantize(t, st).T)
    o.update(tq_x=t, tq_out=tq)
    # QLinear forward (fused truncation) / backward
    M, N, K = 45, 19, 30
    X = rng.standard_normal((M, K)).astype(np.float32)
    W = (rng.standard_normal((N, K)) * 0.2).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    Y, Xq, Wq, sX, sW, sY, acc = orc.qgemm_fwd(X, W, b, reduce=True, want_acc=True)
    assert np.array_equal(acc, Xq.astype(np.int64) @ Wq.astype(np.int64).T)
    assert np.array_equal(Y, b + (np.float32(sX) * np.float32(sW)) * acc.astype(np.float32))
    assert sY == np.float32(np.abs(Y).max() / np.float32(127.0))
    dY = rng.standard_normal((M, N)).astype(np.float32)
    sdY = orc.absmax_scale(dY)
    dYq = orc.quantize(dY, sdY)
    dX = orc.qgemm_bwd_dx(dYq, Wq, sdY, sW)
    dW = orc.qgemm_bwd_dw(dYq, Xq, sdY, sX)
    assert np.array_equal(dX, (np.float32(sdY) * np.float32(sW)) * (dYq.astype(np.int64) @ Wq.astype(np.int64)).astype(np.float32))
    assert np.array_equal(dW, (np.float32(sdY) * np.float32(sX)) * (dYq.astype(np.int64).T @ Xq.astype(np.int64)).astype(np.float32))
    o.update(g_X=X, g_W=W, g_b=b, g_Y=Y, g_Xq=Xq, g_Wq=Wq, g_sX=sX, g_sW=sW, g_sY=sY, g_dYq=dYq, g_sdY=sdY,
             g_dX=dX, g_dW=dW)
    # graph + SpMM family + SDDMM + edge softmax
    n, e, H, F = 40, 300, 3, 8
    src = rng.integers(0, n, e).astype(np.int64)
    dst = rng.integers(0, n, e).astype(np.int64)
    dst[:60] = 5  # a long row
    fm = orc.graph_formats(src, dst, n)
    feat = rng.integers(-127, 128, (n, H, F)).astype(np.int8)
    ev = rng.integers(-127, 128, (H, 1, e)).astype(np.int8)
    sc = np.float32(0.0123)
    dense = np.zeros((n, n), dtype=np.int64)
    np.add.at(dense, (dst, src), 1)
    copy_u = orc.spmm_csr_copy_u(fm["adj_csc"][0], fm["adj_csc"][1], feat.reshape(n, H * F), sc)
    assert np.array_equal(copy_u, sc * (dense @ feat.reshape(n, H * F).astype(np.int64)).astype(np.float32))
    umule = orc.spmm_csr_u_mul_e(*fm["adj_csc"], feat, ev, sc)
    want = np.zeros((n, H, F), dtype=np.int64)
    for k in range(e):
        want[dst[k]] += feat[src[k]].astype(np.int64) * ev[:, 0, k].astype(np.int64)[:, None]
    assert np.array_equal(umule, sc * want.astype(np.float32))
    E8 = rng.integers(-127, 128, (e, F)).astype(np.int8)
    inc = orc.spmm_incidence(fm["inc_in"][0], fm["inc_in"][1], E8, sc, n)
    want = np.zeros((n, F), dtype=np.int64)
    np.add.at(want, dst, E8.astype(np.int64))
    assert np.array_equal(inc, sc * want.astype(np.float32))
    U = rng.integers(-127, 128, (n, H, F)).astype(np.int8)
    dot, _ = orc.sddmm_dot(src, dst, feat, U, 0.5, 0.25)
    assert np.array_equal(dot, np.float32(0.125) * (feat[src].astype(np.int64) * U[dst].astype(np.int64)).sum(-1).astype(np.float32))
    sub, _ = orc.sddmm_ewise("sub", src, dst, feat.reshape(n, H * F), U.reshape(n, H * F), 0.5, 0.25)
    assert np.array_equal(sub, np.float32(0.5) * feat.reshape(n, -1)[src].astype(np.float32) - np.float32(0.25) * U.reshape(n, -1)[dst].astype(np.float32))
    xe = (rng.standard_normal((e, H)) * 3).astype(np.float32)
    a = orc.edge_softmax_fwd(xe, fm["adj_csc"][0], fm["adj_csc"][2], 0.2)
    lk = np.where(xe > 0, xe, xe * np.float32(0.2)).astype(np.float64)
    want = np.zeros_like(lk)
    for v in range(n):
        m = dst == v
        if m.any():
            z = np.exp(lk[m] - lk[m].max(0))
            want[m] = z / z.sum(0)
    assert np.allclose(a, want, rtol=1e-6, atol=1e-7)
    o.update(s_src=src, s_dst=dst, s_n=np.int64(n), s_feat=feat, s_ev=ev, s_scale=sc, s_copy_u=copy_u,
             s_u_mul_e=umule, s_E8=E8, s_incidence=inc, s_U=U, s_dot=dot, s_sub=sub, s_xe=xe, s_softmax=a)
    return o


PHILOX_KAT = [  # Random123 kat_vectors: philox4x32, 10 rounds: counter, key, expected
    ((0x00000000,) * 4, (0x00000000,) * 2, (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
     (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


if __name__ == "__main__":
    for ctr, key, want in PHILOX_KAT:
        assert tuple(int(v) for v in orc.philox4x32_10(ctr, key)) == want
    np.savez_compressed(os.path.join(HERE, "reference_patterns.npz"), **reference_patterns())
    np.savez_compressed(os.path.join(HERE, "seeded_cases.npz"), **seeded_cases())
    np.save(os.path.join(HERE, "philox_kat.npy"),
            np.array([list(c) + list(k) + list(w) for c, k, w in PHILOX_KAT], dtype=np.uint32))
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith((".npz", ".npy"))))
