"""numpy front end of the CPU oracle.  TEST INFRASTRUCTURE ONLY.

Loads ``oracle/_ref/libtango_oracle.so`` (built from ``tango_oracle.c`` by the
Makefile beside it) and wraps every function for numpy arrays.  Only tests,
the smoke check and the benchmark's CPU-baseline leg may import this module;
the shipped package never does.

The graph-format helpers restate, without DGL, what ``cuda/util.py:5-11`` of
the reference asks DGL for (``adj_sparse('csr'|'csc')``, ``inc('in'|'out')``,
``edges()``).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_ref", "libtango_oracle.so")

RNE, TRUNC, STOCHASTIC = 0, 1, 2
OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}


def build(force=False):
    """Compile the C restatement (gcc only; no reference source is involved)."""
    if force or not os.path.exists(_SO):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True,
                       stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_SO)
        _lib.orc_absmax_scale.restype = C.c_float
        _lib.orc_philox_uniform.restype = C.c_float
        _lib.orc_overflow_count.restype = C.c_int64
        _lib.orc_num_threads.restype = C.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i8(a):
    return np.ascontiguousarray(a, dtype=np.int8)


def _i64(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.int64)


i64 = C.c_int64
u64 = C.c_uint64
f32 = C.c_float
ci = C.c_int


def overflow_count():
    return int(lib().orc_overflow_count())


def overflow_reset():
    lib().orc_overflow_reset()


def num_threads():
    return int(lib().orc_num_threads())


def set_num_threads(n):
    lib().orc_set_num_threads(ci(int(n)))


# ------------------------------------------------------------------ Philox
def philox4x32_10(ctr, key):
    c = np.asarray(ctr, dtype=np.uint32)
    k = np.asarray(key, dtype=np.uint32)
    out = np.zeros(4, dtype=np.uint32)
    lib().orc_philox4x32_10(_p(c), _p(k), _p(out))
    return out


def philox_uniform(seed, g):
    return float(lib().orc_philox_uniform(u64(seed), u64(g)))


# ------------------------------------------------------------ quantization
def absmax_scale(x):
    x = _f32(x).ravel()
    return np.float32(lib().orc_absmax_scale(_p(x), i64(x.size)))


def absmax_rows(x):
    x = _f32(x)
    s = np.zeros(x.shape[0], dtype=np.float32)
    lib().orc_absmax_rows(_p(x), i64(x.shape[0]), i64(x.shape[1]), i64(x.shape[1]), _p(s))
    return s


def quantize(x, scale, mode=RNE, noise=None, seed=0, offset=0):
    x = _f32(x)
    q = np.empty(x.shape, dtype=np.int8)
    nz = None if noise is None else _f32(noise)
    lib().orc_quantize(_p(x), i64(x.size), f32(float(scale)), _p(q), ci(mode), _p(nz),
                       u64(seed), u64(offset))
    return q


def quantize_rows(x, scales, per_row, ldq=None, mode=RNE, noise=None, seed=0, offset=0):
    x = _f32(x)
    rows, cols = x.shape
    ldq = cols if ldq is None else ldq
    q = np.empty((rows, ldq), dtype=np.int8)
    s = _f32(np.atleast_1d(scales))
    nz = None if noise is None else _f32(noise)
    lib().orc_quantize_rows(_p(x), i64(rows), i64(cols), i64(cols), _p(s), ci(int(per_row)),
                            _p(q), i64(ldq), ci(mode), _p(nz), u64(seed), u64(offset))
    return q


def transpose_quant(x, scale):
    x = _f32(x)
    nrow = x.shape[0]
    ncol = x.size // nrow
    out = np.empty((ncol, nrow), dtype=np.int8)
    lib().orc_transpose_quant(_p(x), i64(nrow), i64(ncol), f32(float(scale)), _p(out))
    return out


# -------------------------------------------------------------------- GEMM
def qgemm_fwd(X, W, bias=None, reduce=False, mode=TRUNC, sX=None, sW=None, want_acc=False):
    """Returns (Y, Xq, Wq, sX, sW, sY|None[, acc])."""
    X = _f32(X)
    W = _f32(W)
    M, K = X.shape
    N = W.shape[0]
    sX = absmax_scale(X) if sX is None else np.float32(sX)
    sW = absmax_scale(W) if sW is None else np.float32(sW)
    Y = np.empty((M, N), dtype=np.float32)
    Xq = np.empty((M, K), dtype=np.int8)
    Wq = np.empty((N, K), dtype=np.int8)
    b = None if bias is None else _f32(bias)
    sY = C.c_float(0.0)
    acc = np.empty((M, N), dtype=np.int32) if want_acc else None
    lib().orc_qgemm_fwd(_p(Y), i64(N), _p(X), i64(K), _p(Xq), _p(W), i64(K), _p(Wq), _p(b),
                        C.byref(sY) if reduce else None, f32(float(sX)), f32(float(sW)),
                        i64(M), i64(N), i64(K), ci(mode), _p(acc))
    res = (Y, Xq, Wq, sX, sW, np.float32(sY.value) if reduce else None)
    return res + (acc,) if want_acc else res


def qgemm_bwd_dx(dYq, Wq, s_dY, s_W):
    dYq = _i8(dYq)
    Wq = _i8(Wq)
    M, N = dYq.shape
    K = Wq.shape[1]
    dX = np.empty((M, K), dtype=np.float32)
    lib().orc_qgemm_bwd_dx(_p(dX), i64(K), _p(dYq), i64(N), _p(Wq), i64(K), f32(float(s_dY)),
                           f32(float(s_W)), i64(M), i64(N), i64(K))
    return dX


def qgemm_bwd_dw(dYq, Xq, s_dY, s_X):
    dYq = _i8(dYq)
    Xq = _i8(Xq)
    M, N = dYq.shape
    K = Xq.shape[1]
    dW = np.empty((N, K), dtype=np.float32)
    lib().orc_qgemm_bwd_dw(_p(dW), i64(K), _p(dYq), i64(N), _p(Xq), i64(K), f32(float(s_dY)),
                           f32(float(s_X)), i64(M), i64(N), i64(K))
    return dW


def qgemm_legacy(A, B, trans_a, trans_b):
    A = _f32(A)
    B = _f32(B)
    m = A.shape[1] if trans_a else A.shape[0]
    k = A.shape[0] if trans_a else A.shape[1]
    n = B.shape[0] if trans_b else B.shape[1]
    out = np.empty((m, n), dtype=np.float32)
    lib().orc_qgemm_legacy(_p(out), _p(A), _p(B), i64(m), i64(n), i64(k), ci(int(trans_a)),
                           ci(int(trans_b)))
    return out


# -------------------------------------------------------------------- SpMM
def spmm_csr_copy_u(indptr, indices, feat, scale, F=None):
    """feat [k, ld] int8 (only the first F columns of each row are summed)."""
    indptr = _i64(indptr)
    indices = _i64(indices)
    feat = _i8(feat)
    rows = indptr.size - 1
    ld = feat.size // feat.shape[0]
    F = ld if F is None else F
    out = np.empty((rows, F), dtype=np.float32)
    lib().orc_spmm_csr_copy_u(_p(out), _p(indptr), _p(indices), _p(feat), i64(ld),
                              f32(float(scale)), i64(rows), i64(F))
    return out


def spmm_csr_u_mul_e(indptr, indices, edge_ids, feat, evals, scale):
    """feat [k,H,F] int8, evals [H,D,nnz] int8 -> out [rows,H,F] fp32."""
    indptr = _i64(indptr)
    indices = _i64(indices)
    edge_ids = _i64(edge_ids)
    feat = _i8(feat)
    evals = _i8(evals)
    rows = indptr.size - 1
    _, H, F = feat.shape
    D, nnz = evals.shape[1], evals.shape[2]
    out = np.empty((rows, H, F), dtype=np.float32)
    lib().orc_spmm_csr_u_mul_e(_p(out), _p(indptr), _p(indices), _p(edge_ids), _p(feat),
                               _p(evals), f32(float(scale)), i64(rows), i64(H), i64(F), i64(D),
                               i64(nnz))
    return out


def spmm_incidence(node, edge, E, scale, num_nodes):
    node = _i64(node)
    edge = _i64(edge)
    E = _i8(E)
    F = int(np.prod(E.shape[1:], dtype=np.int64)) if E.ndim > 1 else 1  # also for a graph without edges
    out = np.empty((num_nodes, F), dtype=np.float32)
    lib().orc_spmm_incidence(_p(out), _p(node), _p(edge), _p(E), f32(float(scale)),
                             i64(num_nodes), i64(node.size), i64(F))
    return out


# ------------------------------------------------------------------- SDDMM
def sddmm_dot(src, dst, U, V, sU, sV, reduce=False):
    """U, V [n,H,D] int8 -> (out [E,H] fp32, scaleOut|None)."""
    src = _i64(src)
    dst = _i64(dst)
    U = _i8(U)
    V = _i8(V)
    _, H, D = U.shape
    out = np.empty((src.size, H), dtype=np.float32)
    so = C.c_float(0.0)
    lib().orc_sddmm_dot(_p(out), C.byref(so) if reduce else None, _p(src), _p(dst), _p(U), _p(V),
                        f32(float(sU)), f32(float(sV)), i64(src.size), i64(H), i64(D))
    return out, (np.float32(so.value) if reduce else None)


def sddmm_ewise(op, src, dst, U, V, sU, sV, reduce=False):
    """U, V [n,T] int8 -> (out [E,T] fp32, scaleOut|None)."""
    src = _i64(src)
    dst = _i64(dst)
    U = _i8(U)
    V = _i8(V)
    T = U.size // U.shape[0]
    out = np.empty((src.size, T), dtype=np.float32)
    so = C.c_float(0.0)
    lib().orc_sddmm_ewise(ci(OPS[op]), _p(out), C.byref(so) if reduce else None, _p(src),
                          _p(dst), _p(U), _p(V), f32(float(sU)), f32(float(sV)),
                          i64(src.size), i64(T))
    return out, (np.float32(so.value) if reduce else None)


# ------------------------------------------------------------ edge softmax
def edge_softmax_fwd(e, indptr, eids, slope=1.0):
    e = _f32(e)
    E = e.shape[0]
    H = e.size // max(E, 1)
    indptr = _i64(indptr)
    eids = _i64(eids)
    a = np.zeros_like(e)
    lib().orc_edge_softmax_fwd(_p(a), _p(e), _p(indptr), _p(eids), i64(indptr.size - 1), i64(H),
                               f32(slope))
    return a


def edge_softmax_bwd(a, da, e, indptr, eids, slope=1.0):
    a = _f32(a)
    da = _f32(da)
    e = _f32(e)
    H = e.size // max(e.shape[0], 1)
    indptr = _i64(indptr)
    eids = _i64(eids)
    de = np.zeros_like(e)
    lib().orc_edge_softmax_bwd(_p(de), _p(a), _p(da), _p(e), _p(indptr), _p(eids),
                               i64(indptr.size - 1), i64(H), f32(slope))
    return de


# ------------------------------------------------------------ graph formats
def graph_formats(src, dst, num_nodes):
    """DGL-free restatement of cuda/util.py:5-11.

    Returns a dict with ``coo`` (src, dst in edge-id order), ``adj_csr``
    (rows = source nodes; indptr, indices = destinations, edge_ids),
    ``adj_csc`` (rows = destination nodes; indices = sources), ``inc_in``
    ([2, E]: (dst[e], e) sorted by node then edge) and ``inc_out``
    ((src[e], e) likewise).
    """
    src = np.asarray(src, dtype=np.int64)
    dst = np.asarray(dst, dtype=np.int64)

    def compress(rows, cols):
        order = np.argsort(rows, kind="stable")
        indptr = np.zeros(num_nodes + 1, dtype=np.int64)
        np.cumsum(np.bincount(rows, minlength=num_nodes), out=indptr[1:])
        return indptr, cols[order], order.astype(np.int64)

    csr = compress(src, dst)
    csc = compress(dst, src)
    inc_in = np.stack([dst[csc[2]], csc[2]])
    inc_out = np.stack([src[csr[2]], csr[2]])
    return {"coo": (src, dst), "adj_csr": csr, "adj_csc": csc, "inc_in": inc_in,
            "inc_out": inc_out}


# ------------------------------------------------------------- fused forms
MASK_MODES = {"relu": 0, "elu": 1, "bits": 2}


def _mask_args(mask, mask_mode, cols):
    if mask is None:
        return None, None, 0, 0
    mode = MASK_MODES[mask_mode]
    if mode == 2:
        m = np.ascontiguousarray(mask).view(np.uint16)
        return m, _p(m), m.shape[1], mode
    m = _f32(mask)
    return m, _p(m), cols, mode


def absmax_ex(x, row_mul=None, mask=None, mask_mode="relu", want_colsum=False):
    """(max|x' * row_mul| / 127, column sums of x' or None); x' = x taken back through the activation."""
    x = _f32(x)
    rows, cols = x.shape
    rm = None if row_mul is None else _f32(row_mul)
    keep, mp, ldm, mode = _mask_args(mask, mask_mode, cols)
    s = C.c_float(0.0)
    cs = np.zeros(cols, dtype=np.float64) if want_colsum else None
    lib().orc_absmax_ex(_p(x), i64(rows), i64(cols), i64(cols), _p(rm), mp, i64(ldm), C.c_int(mode),
                        C.byref(s), _p(cs))
    return np.float32(s.value), cs


def quantize_rows_ex(x, scale, row_mul=None, mask=None, mask_mode="relu", ldq=None, mode=RNE, noise=None,
                     seed=0, offset=0):
    x = _f32(x)
    rows, cols = x.shape
    ldq = cols if ldq is None else ldq
    rm = None if row_mul is None else _f32(row_mul)
    keep, mp, ldm, mm = _mask_args(mask, mask_mode, cols)
    sc = np.array([scale], dtype=np.float32)
    nz = None if noise is None else _f32(noise)
    q = np.empty((rows, ldq), dtype=np.int8)
    lib().orc_quantize_rows_ex(_p(x), i64(rows), i64(cols), i64(cols), _p(rm), mp, i64(ldm), C.c_int(mm),
                               _p(sc), C.c_int(0), _p(q), i64(ldq), C.c_int(mode), _p(nz), u64(seed), u64(offset))
    return q


def qgemm_i8_nt(A, B, sA, sB, bias=None, reduce=False):
    """Y = (sA*sB) * float(A . B^T) (+ bias) for int8 A [M,K], B [N,K]; with ``reduce`` also max|Y| / 127."""
    A, B = _i8(A), _i8(B)
    M, K = A.shape
    N = B.shape[0]
    b = None if bias is None else _f32(bias)
    Y = np.empty((M, N), dtype=np.float32)
    sy = C.c_float(0.0)
    lib().orc_qgemm_i8_nt(_p(Y), i64(N), _p(A), i64(K), _p(B), i64(K), _p(b), C.byref(sy) if reduce else None,
                          f32(float(sA)), f32(float(sB)), i64(M), i64(N), i64(K))
    return (Y, np.float32(sy.value)) if reduce else Y


def qgemm_bwd_dx_ex(dYq, Wq, s_dY, s_W, row_scale=None, accumulate_into=None):
    dYq, Wq = _i8(dYq), _i8(Wq)
    M, N = dYq.shape
    K = Wq.shape[1]
    rs = None if row_scale is None else _f32(row_scale)
    dX = np.empty((M, K), dtype=np.float32) if accumulate_into is None else _f32(accumulate_into).copy()
    lib().orc_qgemm_bwd_dx_ex(_p(dX), i64(K), _p(dYq), i64(N), _p(Wq), i64(K), f32(float(s_dY)), f32(float(s_W)),
                              _p(rs), C.c_int(0 if accumulate_into is None else 1), i64(M), i64(N), i64(K))
    return dX


def spmm_csr_copy_u_ex(indptr, indices, feat, scale, row_scale=None, bias=None, act=0, want_bits=False, F=None):
    """out (and the sign words when ``want_bits``) of the aggregation with the GCN layer's epilogue."""
    indptr, indices, feat = _i64(indptr), _i64(indices), _i8(feat)
    rows = indptr.size - 1
    ld = feat.size // feat.shape[0]
    F = ld if F is None else F
    rs = None if row_scale is None else _f32(row_scale)
    b = None if bias is None else _f32(bias)
    out = np.empty((rows, F), dtype=np.float32)
    bits = np.zeros((rows, F // 16), dtype=np.uint16) if want_bits else None
    lib().orc_spmm_csr_copy_u_ex(_p(out), _p(bits), _p(indptr), _p(indices), _p(feat), i64(ld), f32(float(scale)),
                                 _p(rs), _p(b), C.c_int(act), i64(rows), i64(F))
    return (out, bits) if want_bits else out


def spmm_csr_u_mul_e_ex(indptr, indices, edge_ids, feat, evals, scale, scale2=None, bias=None, act=0,
                        edge_major=False):
    """feat [k,H,F] int8; evals [H,D,nnz] or, edge-major, [nnz,H,D] int8 -> out [rows,H,F] fp32."""
    indptr, indices, edge_ids, feat, evals = _i64(indptr), _i64(indices), _i64(edge_ids), _i8(feat), _i8(evals)
    k, H, F = feat.shape
    if edge_major:
        nnz, D = evals.shape[0], evals.shape[2]
    else:
        D, nnz = evals.shape[1], evals.shape[2]
    rows = indptr.size - 1
    s2 = None if scale2 is None else np.array([scale2], dtype=np.float32)
    b = None if bias is None else _f32(bias)
    out = np.empty((rows, H, F), dtype=np.float32)
    lib().orc_spmm_csr_u_mul_e_ex(_p(out), _p(indptr), _p(indices), _p(edge_ids), _p(feat), _p(evals),
                                  C.c_int(1 if edge_major else 0), f32(float(scale)), _p(s2), _p(b), C.c_int(act),
                                  i64(rows), i64(H), i64(F), i64(D), i64(nnz))
    return out
