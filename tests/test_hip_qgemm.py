"""GPU parity: int8 MFMA GEMMs vs the CPU oracle.

Quantized operands and int32 accumulators are bit-exact; the fp32 outputs are
the same two IEEE roundings on both sides, so they are compared bit-exactly as
well (the allowed tolerance is 1e-5 relative / 1e-6 absolute)."""
import numpy as np
import pytest
import torch

from gpu_util import dev, host, sc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from tango_amd import kernels
    return kernels


def glorot(rng, n, k):
    a = np.sqrt(6.0 / (n + k))
    return ((rng.random((n, k), dtype=np.float32) * 2 - 1) * a).astype(np.float32)


def lcg_matrix(rows, cols, seed):
    # cuda/src/QGEMM_forward.cu:162-181 (column-major fill)
    off = np.arange(rows * cols, dtype=np.int64)
    return ((off + seed) * 16807 % 16 - 8).astype(np.float32).reshape(cols, rows).T.copy()


def run_fwd(K, X, W, bias, reduce, padded, round_mode=None):
    M, k = X.shape
    N = W.shape[0]
    Xd, Wd = dev(X), dev(W)
    sX, sW = K.cuda_kernels.get_scale(Xd), K.cuda_kernels.get_scale(Wd)
    if padded:
        ld = (k + 15) // 16 * 16
        Xq = torch.full((M, ld), 99, dtype=torch.int8, device="cuda")[:, :k]
    else:
        Xq = torch.empty((M, k), dtype=torch.int8, device="cuda")
    Wq = torch.empty((N, k), dtype=torch.int8, device="cuda")
    res = K.QGEMM_forward(Xd, Xq, sX, Wd, Wq, sW, None if bias is None else dev(bias), reduce,
                          round_mode=round_mode)
    return res, Xq, Wq, sX, sW


@pytest.mark.parametrize("M,N,Kd", [(300, 16, 128), (1000, 41, 256), (513, 128, 602), (257, 256, 602),
                                     (129, 300, 64), (64, 7, 20), (1, 1, 1), (4100, 256, 128)])
@pytest.mark.parametrize("padded", [True, False])
def test_forward(K, orc, M, N, Kd, padded):
    rng = np.random.default_rng(M + N + Kd)
    X = rng.standard_normal((M, Kd)).astype(np.float32)
    W = glorot(rng, N, Kd)
    b = rng.standard_normal(N).astype(np.float32)
    for bias, reduce in ((None, False), (b, True)):
        res, Xq, Wq, sX, sW = run_fwd(K, X, W, bias, reduce, padded)
        Y, oXq, oWq, osX, osW, osY = orc.qgemm_fwd(X, W, bias=bias, reduce=reduce)
        assert host(sX)[0] == osX and host(sW)[0] == osW
        assert np.array_equal(host(Xq), oXq) and np.array_equal(host(Wq), oWq)
        out = res[0] if reduce else res
        assert np.array_equal(host(out), Y)
        if reduce:
            assert host(res[1])[0] == osY
    assert orc.overflow_count() == 0


@pytest.mark.parametrize("M,N,Kd,mode,rowmul", [(33003, 256, 602, "trunc", False), (33000, 200, 580, "rne", True),
                                                  (34001, 130, 256, "trunc", True), (33500, 256, 200, "rne", False),
                                                  (33100, 256, 604, "trunc", False)])
def test_forward_persistent_form(K, orc, M, N, Kd, mode, rowmul):
    """The forward kernel for tall X and 129..256 output columns (a persistent workgroup per compute unit; half of
    its waves stream and quantize X, the other half multiply and store): reductions of ten and of four k-steps,
    rows read in 8- and in 16-byte pieces, a last tile with fewer than 16 rows, output columns that do not fill the
    last column tile, bias, the row multiplier, both rounding modes; Xq, its zero padding, Wq, Y and the output
    scale are compared."""
    rng = np.random.default_rng(M + N + Kd)
    X = rng.standard_normal((M, Kd)).astype(np.float32)
    W = glorot(rng, N, Kd)
    bias = rng.standard_normal(N).astype(np.float32) if N != 256 else None
    rm = (rng.random(M).astype(np.float32) + 0.5) if rowmul else None
    Xs = X * rm[:, None] if rowmul else X
    Xd, Wd = dev(X), dev(W)
    sX = dev(np.array([orc.absmax_scale(Xs)], np.float32))
    sW = K.cuda_kernels.get_scale(Wd)
    ld = (Kd + 15) // 16 * 16
    Xbuf = torch.full((M, ld), 99, dtype=torch.int8, device="cuda")
    Wq = torch.empty((N, Kd), dtype=torch.int8, device="cuda")
    Y, sY = K.QGEMM_forward(Xd, Xbuf[:, :Kd], sX, Wd, Wq, sW, None if bias is None else dev(bias), True,
                            round_mode=mode, x_row_mul=None if rm is None else dev(rm))
    oY, oXq, oWq, _, _, osY = orc.qgemm_fwd(Xs, W, bias=bias, reduce=True, mode=orc.RNE if mode == "rne" else orc.TRUNC,
                                            sX=host(sX)[0])
    assert np.array_equal(host(Xbuf[:, :Kd]), oXq) and not host(Xbuf[:, Kd:]).any()
    assert np.array_equal(host(Wq), oWq)
    assert np.array_equal(host(Y), oY) and host(sY)[0] == osY


def test_forward_rne_mode_and_lcg_pattern(K, orc):
    rng = np.random.default_rng(0)
    X = rng.standard_normal((200, 72)).astype(np.float32)
    W = glorot(rng, 24, 72)
    res, Xq, Wq, sX, sW = run_fwd(K, X, W, None, False, True, round_mode="rne")
    Y, oXq, oWq, *_ = orc.qgemm_fwd(X, W, mode=orc.RNE)
    assert np.array_equal(host(Xq), oXq) and np.array_equal(host(res), Y)
    # the reference's TEST pattern: small integers, scales 0.5 -> exact product
    A, B = lcg_matrix(96, 64, 41), lcg_matrix(40, 64, 17)
    Xq = torch.empty((96, 64), dtype=torch.int8, device="cuda")
    Wq = torch.empty((40, 64), dtype=torch.int8, device="cuda")
    out = K.QGEMM_forward(dev(A), Xq, sc(0.5), dev(B), Wq, sc(0.5))
    assert np.array_equal(host(out), (A.astype(np.float64) @ B.astype(np.float64).T).astype(np.float32))


def test_forward_strided_input_and_output(K, orc):
    rng = np.random.default_rng(1)
    big = rng.standard_normal((150, 700)).astype(np.float32)
    X = big[:, 10:612]  # row stride 700, offset 10 floats
    W = glorot(rng, 41, 602)
    Xd = dev(big)[:, 10:612]
    sX = K.cuda_kernels.get_scale(Xd.contiguous())
    Wd = dev(W)
    sW = K.cuda_kernels.get_scale(Wd)
    Xq = torch.empty((150, 602), dtype=torch.int8, device="cuda")
    Wq = torch.empty((41, 602), dtype=torch.int8, device="cuda")
    Ybuf = torch.zeros((150, 64), dtype=torch.float32, device="cuda")
    K.cuda_kernels.QGEMM_forward(Ybuf[:, :41], Xd, Xq, Wd, Wq, torch.Tensor(), torch.Tensor(), sX, sW)
    Y, *_ = orc.qgemm_fwd(np.ascontiguousarray(X), W)
    assert np.array_equal(host(Ybuf)[:, :41], Y) and not host(Ybuf)[:, 41:].any()


@pytest.mark.parametrize("M,N,Kd", [(300, 16, 128), (1000, 41, 256), (513, 128, 602), (2049, 256, 602), (65, 3, 5)])
@pytest.mark.parametrize("padded", [True, False])
def test_backward(K, orc, M, N, Kd, padded):
    rng = np.random.default_rng(M * 3 + N + Kd)
    dY = rng.integers(-127, 128, (M, N)).astype(np.int8)
    X = rng.integers(-127, 128, (M, Kd)).astype(np.int8)
    W = rng.integers(-127, 128, (N, Kd)).astype(np.int8)
    s1, s2, s3 = np.float32(0.013), np.float32(0.27), np.float32(0.0051)

    def put(a):
        if not padded:
            return dev(a)
        ld = (a.shape[1] + 15) // 16 * 16
        buf = torch.full((a.shape[0], ld), 77, dtype=torch.int8, device="cuda")
        buf[:, :a.shape[1]] = dev(a)
        return buf[:, :a.shape[1]]

    dX, dW = K.QGEMM_backward(put(dY), put(X), dev(W), sc(s1), sc(s2), sc(s3))
    assert np.array_equal(host(dX), orc.qgemm_bwd_dx(dY, W, s1, s3))
    assert np.array_equal(host(dW), orc.qgemm_bwd_dw(dY, X, s1, s2))
    assert orc.overflow_count() == 0
    dX2, dW2 = K.QGEMM_backward(put(dY), put(X), dev(W), sc(s1), sc(s2), sc(s3), X_need=False)
    assert dX2 is None and torch.equal(dW, dW2)


def test_gradw_independent_of_split(K, orc):
    # the same reduction seen as one long M and as two stacked halves must agree exactly
    rng = np.random.default_rng(7)
    M, N, Kd = 40000, 41, 256
    dY = rng.integers(-127, 128, (M, N)).astype(np.int8)
    X = rng.integers(-127, 128, (M, Kd)).astype(np.int8)
    _, dW = K.QGEMM_backward(dev(dY), dev(X), dev(np.zeros((N, Kd), np.int8)), sc(1), sc(1), sc(1), X_need=False)
    _, a = K.QGEMM_backward(dev(dY[:17000]), dev(X[:17000]), dev(np.zeros((N, Kd), np.int8)), sc(1), sc(1), sc(1), X_need=False)
    _, b = K.QGEMM_backward(dev(dY[17000:]), dev(X[17000:]), dev(np.zeros((N, Kd), np.int8)), sc(1), sc(1), sc(1), X_need=False)
    want = dY.astype(np.int64).T @ X.astype(np.int64)
    assert np.array_equal(host(dW), want.astype(np.float32))
    # scales are 1, so each part is an exactly representable integer below 2^24 in magnitude
    assert np.abs(want).max() < 2 ** 24
    assert np.array_equal(host(a).astype(np.int64) + host(b).astype(np.int64), want)

@pytest.mark.parametrize("m,n,k", [(33, 20, 48), (128, 64, 602), (5, 3, 7)])
def test_legacy_qgemm(K, orc, m, n, k):
    rng = np.random.default_rng(m + n + k)
    A = rng.standard_normal((m, k)).astype(np.float32)
    B = rng.standard_normal((n, k)).astype(np.float32)
    assert np.array_equal(host(K.cuda_kernels.QgemmNT(dev(A), dev(B))), orc.qgemm_legacy(A, B, False, True))
    Bt = np.ascontiguousarray(B.T)
    assert np.array_equal(host(K.cuda_kernels.QgemmNN(dev(A), dev(Bt))), orc.qgemm_legacy(A, Bt, False, False))
    At = np.ascontiguousarray(A.T)
    assert np.array_equal(host(K.cuda_kernels.QgemmTN(dev(At), dev(Bt))), orc.qgemm_legacy(At, Bt, True, False))


def test_qgemm_i8(K, orc):
    rng = np.random.default_rng(3)
    M, N, Kd = 777, 41, 100
    A = rng.integers(-127, 128, (M, Kd)).astype(np.int8)
    B = rng.integers(-127, 128, (N, Kd)).astype(np.int8)
    Y = torch.empty((M, N), dtype=torch.float32, device="cuda")
    sY = torch.empty(1, dtype=torch.float32, device="cuda")
    K.cuda_kernels.QGEMM_i8(Y, dev(A), dev(B), None, sY, sc(0.5), sc(0.25))
    want = np.float32(0.125) * (A.astype(np.int64) @ B.astype(np.int64).T).astype(np.float32)
    assert np.array_equal(host(Y), want) and host(sY)[0] == orc.absmax_scale(want)


@pytest.mark.parametrize("M,N,Kd", [(70001, 200, 130), (50000, 602, 256), (4000, 41, 64), (15, 256, 200)])
def test_qgemm_i8_small_operand_stationary(K, orc, M, N, Kd):
    """The NT form that keeps the small operand in LDS (reduction <= 256, 4-byte aligned rows): more 16-row
    tiles than waves in the launch (every wave walks several tiles, the next one prefetched), column
    blocks of 13 and 16 tiles, a partial last tile, bias and the output scale."""
    rng = np.random.default_rng(M + N + Kd)
    A = rng.integers(-127, 128, (M, Kd)).astype(np.int8)
    B = rng.integers(-127, 128, (N, Kd)).astype(np.int8)
    bias = rng.standard_normal(N).astype(np.float32)
    ld = (Kd + 15) // 16 * 16
    Abuf = torch.full((M, ld), 77, dtype=torch.int8, device="cuda")
    Abuf[:, :Kd] = dev(A)
    Y = torch.empty((M, N), dtype=torch.float32, device="cuda")
    sY = torch.empty(1, dtype=torch.float32, device="cuda")
    K.cuda_kernels.QGEMM_i8(Y, Abuf[:, :Kd], dev(B), dev(bias), sY, sc(0.5), sc(0.25))
    acc = (A.astype(np.float64) @ B.astype(np.float64).T)  # exact: |sums| < 2^53
    want = bias[None, :] + np.float32(0.125) * acc.astype(np.float32)
    assert np.array_equal(host(Y), want) and host(sY)[0] == orc.absmax_scale(want)


@pytest.mark.parametrize("M,N,Kd,pitch,rows", [(40000, 602, 256, 608, False), (36005, 330, 100, 332, True),
                                               (33000, 960, 64, 960, False), (34003, 264, 200, 264, True)])
def test_nt_small_operand_in_registers(K, orc, M, N, Kd, pitch, rows):
    """The NT form for outputs of 257 to 960 columns and many row tiles (the small operand's fragments stay in
    registers, one wave fetches the A tiles for the others): output pitches that are and are not multiples of 16,
    reductions of one, two and four k-steps, a last tile with fewer than 16 rows, the row multiplier, the output
    scale; padding columns of the output beyond the next multiple of 16 must stay untouched."""
    rng = np.random.default_rng(M + N + Kd)
    A = rng.integers(-127, 128, (M, Kd)).astype(np.int8)
    B = rng.integers(-127, 128, (Kd, N)).astype(np.int8)
    ld = (Kd + 15) // 16 * 16
    Abuf = torch.full((M, ld), 77, dtype=torch.int8, device="cuda")
    Abuf[:, :Kd] = dev(A)
    rs = dev(rng.random(M).astype(np.float32) + 0.5) if rows else None
    acc = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32) * np.float32(0.0625)
    if rows:
        acc = acc * host(rs)[:, None]
    out = torch.full((M, pitch), -3.0, dtype=torch.float32, device="cuda")
    K.cuda_kernels.QGEMM_backward_gradX(out[:, :N], Abuf[:, :Kd], dev(B), sc(0.5), sc(0.125), row_scale=rs)
    assert np.array_equal(host(out[:, :N]), acc)
    n16 = (N + 15) // 16 * 16
    if pitch > n16:
        assert bool((out[:, n16:] == -3.0).all())
    if not rows:
        Y = torch.empty((M, pitch), dtype=torch.float32, device="cuda")[:, :N]
        sY = torch.empty(1, dtype=torch.float32, device="cuda")
        K.cuda_kernels.QGEMM_i8(Y, Abuf[:, :Kd], dev(np.ascontiguousarray(B.T)), None, sY, sc(0.5), sc(0.125))
        assert np.array_equal(host(Y), acc) and host(sY)[0] == orc.absmax_scale(acc)


@pytest.mark.parametrize("M,N,Kd,rows", [(5000, 256, 256, False), (3001, 300, 41, True), (777, 64, 130, False)])
def test_gradx_accumulates_into_its_output(K, M, N, Kd, rows):
    """gradX added to what dX holds == dX + the gradX written on its own, bit for bit (one fp32 addition per
    element), through the stationary form (reduction <= 256), the streaming form (reduction 300), odd and
    even output widths and a row multiplier."""
    rng = np.random.default_rng(M + N + Kd)
    dY = rng.integers(-127, 128, (M, N)).astype(np.int8)
    W = rng.integers(-127, 128, (N, Kd)).astype(np.int8)
    prior = rng.standard_normal((M, Kd)).astype(np.float32)
    rs = dev(rng.random(M).astype(np.float32) + 0.5) if rows else None
    ld = (N + 15) // 16 * 16
    dYb = torch.full((M, max(ld, 16)), 55, dtype=torch.int8, device="cuda")
    dYb[:, :N] = dev(dY)
    alone = torch.empty((M, Kd), dtype=torch.float32, device="cuda")
    K.cuda_kernels.QGEMM_backward_gradX(alone, dYb[:, :N], dev(W), sc(0.5), sc(0.125), row_scale=rs)
    acc = (dY.astype(np.float64) @ W.astype(np.float64)).astype(np.float32) * np.float32(0.0625)
    if rows:
        acc = acc * host(rs)[:, None]
    assert np.array_equal(host(alone), acc)
    out = dev(prior)
    K.cuda_kernels.QGEMM_backward_gradX(out, dYb[:, :N], dev(W), sc(0.5), sc(0.125), row_scale=rs, accumulate=True)
    assert np.array_equal(host(out), prior + acc)


@pytest.mark.parametrize("mode", ["rne", "trunc"])
@pytest.mark.parametrize("M,N,Kd", [(40000, 256, 256), (3001, 41, 100), (16, 600, 64), (1, 16, 16), (500, 128, 192),
                                    (777, 250, 33)])
def test_forward_gemm_with_int8_output(K, orc, M, N, Kd, mode):
    """The forward GEMM that stores its output already quantized == the oracle's int8 GEMM, absmax scale and
    quantize on the fp32 product, bit for bit; a reduction above 256 is declined with nothing launched."""
    rng = np.random.default_rng(M + N + Kd)
    Xq = rng.integers(-127, 128, (M, Kd)).astype(np.int8)
    W = rng.standard_normal((N, Kd)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    omode = orc.RNE if mode == "rne" else orc.TRUNC
    sX, sW = np.float32(0.031), orc.absmax_scale(W)
    Wq = orc.quantize(W, sW, omode)
    acc = (Xq.astype(np.float64) @ Wq.astype(np.float64).T).astype(np.float32)
    Y = bias[None, :] + (sX * sW) * acc
    sY = orc.absmax_scale(Y)
    want = orc.quantize(Y, sY, omode)
    ld = (Kd + 15) // 16 * 16
    Xb = torch.full((M, ld), 33, dtype=torch.int8, device="cuda")
    Xb[:, :Kd] = dev(Xq)
    ldy = (N + 15) // 16 * 16
    Yb = torch.full((M, ldy), 99, dtype=torch.int8, device="cuda")
    W_q = torch.empty((N, Kd), dtype=torch.int8, device="cuda")
    s_out = torch.full((1,), 7.0, device="cuda")
    assert K.cuda_kernels.QGEMM_forward_q8(Yb[:, :N], s_out, Xb[:, :Kd], dev(W), W_q, dev(bias), sc(sX), sc(sW),
                                           round_mode=mode)
    assert host(s_out)[0] == sY and np.array_equal(host(W_q), Wq)
    assert np.array_equal(host(Yb[:, :N]), want)
    assert (host(Yb[:, N:]) == 99).all()  # the padding of the output rows is left alone
    big = torch.zeros((4, 272), dtype=torch.int8, device="cuda")
    assert not K.cuda_kernels.QGEMM_forward_q8(torch.empty((4, 16), dtype=torch.int8, device="cuda"), s_out, big,
                                               torch.zeros((16, 272), device="cuda"),
                                               torch.empty((16, 272), dtype=torch.int8, device="cuda"), None,
                                               sc(1.0), sc(1.0), round_mode=mode)


def test_forward_gemm_refuses_stochastic_rounding():
    """The forward GEMM's signature carries no seed, so it cannot round stochastically: it says so instead
    of rounding some other way."""
    from tango_amd import _lib
    L = _lib.lib()
    M, N, Kd = 32, 16, 64
    X = torch.randn(M, Kd, device="cuda")
    W = torch.randn(N, Kd, device="cuda")
    Xq = torch.empty((M, Kd), dtype=torch.int8, device="cuda")
    Wq = torch.empty((N, Kd), dtype=torch.int8, device="cuda")
    Y = torch.empty((M, N), device="cuda")
    ws_bytes = L.tango_qgemm_fwd_workspace(M, N, Kd)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    rc = L.tango_qgemm_fwd(Y.data_ptr(), N, X.data_ptr(), Kd, Xq.data_ptr(), Kd, W.data_ptr(), Kd, Wq.data_ptr(), None,
                           None, sc(0.1).data_ptr(), sc(0.1).data_ptr(), M, N, Kd, _lib.ROUND_STOCHASTIC, ws.data_ptr(),
                           ws_bytes, None)
    assert rc == -2
