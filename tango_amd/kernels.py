"""Functional layer over libtango_hip: mirrors cuda/kernels.py of the reference.

``cuda_kernels`` exposes the fourteen callables of the reference's pybind11
module (cuda/src/cuda.cpp:182-204) with the same names, arity and argument
meaning; the module-level functions are the reference's Python wrappers
(cuda/kernels.py:19-178).  torch supplies device memory and the current
stream; all arithmetic runs in the HIP library.  Keyword arguments that the
reference does not have (``round_mode``, ``noise``, ``seed``, ``offset``,
``edge_ids``) default to the reference's behaviour.
"""
import math
import os
import threading

import torch

from . import _lib
from ._lib import ROUND_MODES, ROUND_RNE, ROUND_STOCHASTIC, ROUND_TRUNC, SDDMM_OPS, check

_L = _lib.lib()  # fails here, loudly, if the library is not built


_raw_stream = torch._C._cuda_getCurrentRawStream  # the handle itself, without building a Stream object
_current_device = torch._C._cuda_getDevice


def _stream():
    """The current stream of the current device as a raw hipStream_t (what torch's own ops launch on)."""
    return _raw_stream(_current_device())


def _ptr(t):
    return None if t is None or t.numel() == 0 else t.data_ptr()


def _need(t, dtype, name, contiguous=True):
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a tensor" % name)
    if t.dtype != dtype:
        raise RuntimeError("%s: expected %s but got %s" % (name, dtype, t.dtype))
    if not t.is_cuda:
        raise RuntimeError("%s must be on GPU" % name)
    if contiguous and not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    return t


def _need_index(t, name):
    """An index array: int64 as the reference passes it, or a caller-made int32 copy.  Returns its width."""
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a tensor" % name)
    if t.dtype not in (torch.int64, torch.int32):
        raise RuntimeError("%s: expected torch.int64 or torch.int32 but got %s" % (name, t.dtype))
    if not t.is_cuda:
        raise RuntimeError("%s must be on GPU" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    return 32 if t.dtype == torch.int32 else 64


def _rows_view(t, name):
    """2-D row-major view with unit column stride; returns (tensor, row stride)."""
    if t.dim() != 2 or (t.size(1) > 1 and t.stride(1) != 1):
        raise RuntimeError("%s must be 2-D with contiguous rows" % name)
    return t.stride(0) if t.size(0) > 1 else max(t.size(1), t.stride(0))


_WS_BUFFERS = {}  # (device index, raw stream) -> uint8 tensor, grown on demand
_WS_SIZES = {}    # (size query, arguments) -> bytes


def _workspace(nbytes, device):
    """Scratch for one call.  One buffer per (device, stream), grown on demand and reused: calls on a
    stream run in order, so the next call's kernels cannot start before this call's are done with it.
    (The reference allocates its temporaries from torch's allocator in every call.)"""
    if not nbytes:
        return None
    if torch.cuda.is_current_stream_capturing():
        # a graph's allocations live in its own pool and must stay with the graph, not in this table
        return torch.empty(int(nbytes), dtype=torch.uint8, device=device)
    key = (device.index, _stream())
    buf = _WS_BUFFERS.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = _WS_BUFFERS[key] = torch.empty(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=device)
    return buf


def _ws_bytes(query, *args):
    """A workspace size query of the library, answered from a table after the first time."""
    key = (query, args)
    n = _WS_SIZES.get(key)
    if n is None:
        n = _WS_SIZES[key] = getattr(_L, query)(*args)
    return n


_ZERO_SLOTS = {}   # device -> [pool tensor, next free index]
_ZERO_SLOTS_LOCK = threading.Lock()  # forward and autograd's backward thread both draw slots
_POOL_SIZE = 4096


def _zero_slot(device):
    """A 1-element fp32 tensor that holds 0: a view into a pool that one fill zeroes 4096 slots at a
    time, so that the absmax kernels (which max into their output with an atomic) need no fill launch
    of their own per call.  A slot is handed out once and never reused.  Returns None while the
    current stream is being captured into a graph: a replay would find the slot already used."""
    if torch.cuda.is_current_stream_capturing():
        return None
    key = (device.type, device.index)
    with _ZERO_SLOTS_LOCK:
        pool = _ZERO_SLOTS.get(key)
        stream = torch.cuda.current_stream(device)
        if pool is None or pool[1] >= _POOL_SIZE:
            zeros = torch.zeros(_POOL_SIZE, dtype=torch.float32, device=device)
            done = torch.cuda.Event()
            done.record(stream)  # the fill is ordered on this stream; other streams wait for the event below
            pool = _ZERO_SLOTS[key] = [zeros, 0, stream.cuda_stream, done]
        elif pool[2] != stream.cuda_stream:
            stream.wait_event(pool[3])  # a device-side wait (no host synchronisation) on the pool's one fill
        k = pool[1]
        pool[1] = k + 1
    return pool[0][k:k + 1]


_MASK_MODES = {"relu": 0, "elu": 1, "bits": 2}
_ACTIVATIONS = {None: 0, "relu": 1, "elu": 2}


def refuse_capture(what):
    """Raises when the current stream is being captured into a HIP graph.  Called first thing by every backward
    pass of this package: forward passes capture and replay (they launch kernels only, on the capturing thread),
    but a backward pass runs on autograd's worker thread, where it draws workspaces and scale slots from torch's
    allocator and reads pools that the capturing thread owns; capturing a whole training step ended the process
    with a segmentation fault when it was tried, and stays refused until that is understood."""
    if torch.cuda.is_initialized() and torch.cuda.is_current_stream_capturing():
        raise RuntimeError(
            what + ": backward passes of the quantized operators cannot be captured into a HIP graph "
            "(capture the forward pass only and run the training step eagerly)")


def _split_offset(offset):
    """(host offset, device counter or None) of an ``offset`` argument that is a number, an int64 device tensor, or
    a pair of both (the kernel adds the two)."""
    if isinstance(offset, tuple):
        host, dev = offset
        return int(host) + _split_offset(dev)[0], _split_offset(dev)[1]
    if torch.is_tensor(offset):
        if offset.dtype != torch.int64 or offset.numel() != 1 or not offset.is_cuda:
            raise RuntimeError("quantize: a device offset must be a 1-element int64 GPU tensor")
        return 0, offset
    return int(offset), None


def _advance(counter, inc):
    if counter is not None and inc:
        check(_L.tango_counter_add_u64(counter.data_ptr(), int(inc), _stream()), "counter_add")


def _mode(round_mode):
    if isinstance(round_mode, str):
        return ROUND_MODES[round_mode]
    return int(round_mode)


def default_forward_round_mode():
    """Rounding of the GEMM's fused quantize.  The reference truncates
    (cuda/src/iterator.h:161); TANGO_ROUND_MODE=rne selects half-to-even."""
    return ROUND_MODES[os.environ.get("TANGO_ROUND_MODE", "trunc")]


def infer_broadcast_shape(op, shp1, shp2):
    """Restates dgl.sparse.infer_broadcast_shape (imported at cuda/kernels.py:3):
    left-pad to equal rank, dims must match or be 1, result is the element-wise
    maximum; for 'dot' the last dims must match and the result's becomes 1."""
    shp1, shp2 = tuple(shp1), tuple(shp2)
    pad = max(len(shp1), len(shp2))
    a = (1,) * (pad - len(shp1)) + shp1
    b = (1,) * (pad - len(shp2)) + shp2
    for d1, d2 in zip(a, b):
        if d1 != d2 and d1 != 1 and d2 != 1:
            raise ValueError("Feature shapes %s and %s are not broadcastable" % (shp1, shp2))
    out = tuple(max(d1, d2) for d1, d2 in zip(a, b))
    if op == "dot":
        if a[-1] != b[-1]:
            raise ValueError("dot needs equal last dimensions")
        out = out[:-1] + (1,)
    return out


class cuda_kernels:
    """Namespace with the reference extension's bindings (cuda/src/cuda.cpp:182-204)."""

    # ---------------------------------------------------------- quantization
    @staticmethod
    def get_scale(inp):
        _need(inp, torch.float32, "in")
        scale = _zero_slot(inp.device) if inp.numel() > (1 << 16) else None  # small tensors: one launch anyway
        if scale is not None:
            check(_L.tango_absmax_acc_f32(_ptr(inp), inp.numel(), scale.data_ptr(), _stream()), "get_scale")
            return scale
        scale = torch.empty(1, dtype=torch.float32, device=inp.device)
        check(_L.tango_absmax_f32(_ptr(inp), inp.numel(), scale.data_ptr(), _stream()), "get_scale")
        return scale

    @staticmethod
    def get_scale_rows(inp):
        """Per-row scales of a 2-D tensor (not in the reference)."""
        _need(inp, torch.float32, "in", contiguous=False)
        ld = _rows_view(inp, "in")
        scale = torch.empty(inp.size(0), dtype=torch.float32, device=inp.device)
        check(_L.tango_absmax_rows_f32(_ptr(inp), inp.size(0), inp.size(1), ld, _ptr(scale), _stream()),
              "get_scale_rows")
        return scale

    @staticmethod
    def quantize(out, inp, scale, round_mode=ROUND_RNE, noise=None, seed=0, offset=0, advance=0):
        """``offset``: a number, or a 1-element int64 device tensor holding the position in the random stream
        (then ``advance`` is added to it after the launch, by a kernel on the same stream)."""
        _need(out, torch.int8, "out")
        _need(inp, torch.float32, "in")
        _need(scale, torch.float32, "scale")
        if out.numel() != inp.numel():
            raise RuntimeError("quantize: out and in differ in size")
        if noise is not None:
            _need(noise, torch.float32, "noise")
            if noise.numel() != inp.numel():
                raise RuntimeError("quantize: noise and in differ in size")
        offset, offset_dev = _split_offset(offset)
        check(_L.tango_quantize_f32_i8(_ptr(inp), inp.numel(), scale.data_ptr(), _ptr(out),
                                       _mode(round_mode), _ptr(noise), int(seed), offset, _ptr(offset_dev),
                                       _stream()), "quantize")
        _advance(offset_dev, advance)

    @staticmethod
    def _mask_ld(mask, mask_mode, inp, what):
        """Row stride of ``mask`` in its own units: floats of inp's shape, or for "bits" the int16 words
        [rows, cols / 16] that csr_SPMM's ``sign_bits`` writes."""
        if mask_mode == "bits":
            _need(mask, torch.int16, "mask")
            if inp.size(1) % 16 or tuple(mask.shape) != (inp.size(0), inp.size(1) // 16):
                raise RuntimeError(what + ": a bit mask must be int16 [rows, cols / 16], cols a multiple of 16")
            return mask.size(1)
        _need(mask, torch.float32, "mask", contiguous=False)
        if tuple(mask.shape) != tuple(inp.shape):
            raise RuntimeError(what + ": mask must have in's shape")
        return _rows_view(mask, "mask")

    @staticmethod
    def quantize_rows(out, inp, scale, per_row=False, round_mode=ROUND_RNE, noise=None, seed=0,
                      offset=0, row_mul=None, mask=None, mask_mode="relu", advance=0):
        """Row-strided quantize into a possibly wider (zero-padded) int8 matrix (not in the reference).
        ``mask`` (an activation's output) takes each element backwards through that activation first:
        ``mask_mode`` "relu" zeroes it where mask <= 0, "elu" multiplies it by mask + 1 there, "bits":
        the mask is the int16 [rows, cols / 16] sign words of csr_SPMM (bit clear = zero the element).
        ``row_mul`` [rows] then multiplies each row."""
        _need(out, torch.int8, "out", contiguous=False)
        _need(inp, torch.float32, "in", contiguous=False)
        _need(scale, torch.float32, "scale")
        ldx, ldq = _rows_view(inp, "in"), _rows_view(out, "out")
        if out.size(0) != inp.size(0) or out.size(1) < inp.size(1):
            raise RuntimeError("quantize_rows: out must have in's rows and at least its columns")
        ldq_pad = out.size(1)
        if out.size(0) > 1 and ldq != ldq_pad:
            raise RuntimeError("quantize_rows: out must be dense")
        if noise is not None:
            _need(noise, torch.float32, "noise")
        ldm = 0
        if row_mul is not None:
            _need(row_mul, torch.float32, "row_mul")
            if row_mul.numel() != inp.size(0):
                raise RuntimeError("quantize_rows: row_mul must have one entry per row")
        if mask is not None:
            ldm = cuda_kernels._mask_ld(mask, mask_mode, inp, "quantize_rows")
        offset, offset_dev = _split_offset(offset)
        check(_L.tango_quantize_rows_ex_f32_i8(_ptr(inp), inp.size(0), inp.size(1), ldx, _ptr(row_mul),
                                               _ptr(mask), ldm, _MASK_MODES[mask_mode], scale.data_ptr(),
                                               int(bool(per_row)),
                                               _ptr(out), ldq_pad, _mode(round_mode), _ptr(noise),
                                               int(seed), offset, _ptr(offset_dev), _stream()), "quantize_rows")
        _advance(offset_dev, advance)

    @staticmethod
    def quantize_rows_colsum(out, inp, scale, round_mode=ROUND_RNE, noise=None, seed=0, offset=0, row_mul=None,
                             mask=None, mask_mode="relu", advance=0):
        """``quantize_rows`` on dense 2-D tensors that also returns the column sums of the masked input (before
        ``row_mul``) from the same pass: the bias gradient of a caller that already holds the scale.  Returns the
        sums, or None when the layout is not one the kernel takes (nothing has run then)."""
        _need(out, torch.int8, "out")
        _need(inp, torch.float32, "in")
        _need(scale, torch.float32, "scale")
        rows, cols = inp.shape
        if tuple(out.shape) != (rows, cols) or cols % 4 or cols > 1024 or 256 % max(cols // 4, 1):
            return None
        if mask is not None:
            if cuda_kernels._mask_ld(mask, mask_mode, inp, "quantize_rows_colsum") != (cols // 16 if mask_mode == "bits" else cols):
                return None
        if row_mul is not None:
            _need(row_mul, torch.float32, "row_mul")
        if noise is not None:
            _need(noise, torch.float32, "noise")
        colsum = torch.empty(cols, dtype=torch.float32, device=inp.device)
        ws_bytes = _ws_bytes("tango_quantize_rows_colsum_workspace", rows, cols)
        ws = _workspace(ws_bytes, inp.device)
        offset, offset_dev = _split_offset(offset)
        rc = _L.tango_quantize_rows_colsum_f32_i8(_ptr(inp), rows, cols, _ptr(row_mul), _ptr(mask), _MASK_MODES[mask_mode],
                                                  scale.data_ptr(), _ptr(out), _mode(round_mode), _ptr(noise), int(seed),
                                                  offset, _ptr(offset_dev), _ptr(colsum), _ptr(ws), ws_bytes, _stream())
        if rc == -2:  # unsupported layout
            return None
        check(rc, "quantize_rows_colsum")
        _advance(offset_dev, advance)
        return colsum

    @staticmethod
    def absmax_ex(inp, row_mul=None, mask=None, want_colsum=False, mask_mode="relu"):
        """(max|inp' * row_mul| / 127, column sums of inp' or None) in one read of a 2-D tensor (not in
        the reference); inp' = inp passed backwards through the activation whose output is ``mask``
        (``mask_mode`` as for ``quantize_rows``)."""
        _need(inp, torch.float32, "in", contiguous=False)
        ldx = _rows_view(inp, "in")
        rows, cols = inp.shape
        ldm = 0
        if row_mul is not None:
            _need(row_mul, torch.float32, "row_mul")
        if mask is not None:
            ldm = cuda_kernels._mask_ld(mask, mask_mode, inp, "absmax_ex")
        if cols > 1024:
            # the kernel keeps a row's column sums in registers, 1024 columns at most: walk column slices
            scale, sums = None, []
            for c0 in range(0, cols, 1024):
                sl = slice(c0, min(cols, c0 + 1024))
                s_i, cs_i = cuda_kernels.absmax_ex(inp[:, sl], row_mul=row_mul,
                                                   mask=None if mask is None else
                                                   (mask[:, c0 // 16:(min(cols, c0 + 1024) + 15) // 16].contiguous()
                                                    if mask_mode == "bits" else mask[:, sl]),
                                                   want_colsum=want_colsum, mask_mode=mask_mode)
                scale = s_i if scale is None else torch.maximum(scale, s_i)
                sums.append(cs_i)
            return scale, (torch.cat(sums) if want_colsum else None)
        scale = _zero_slot(inp.device)
        accumulate = scale is not None
        if not accumulate:
            scale = torch.empty(1, dtype=torch.float32, device=inp.device)
        colsum = torch.empty(cols, dtype=torch.float32, device=inp.device) if want_colsum else None
        ws_bytes = _ws_bytes("tango_absmax_ex_workspace", rows, cols, int(want_colsum))
        ws = _workspace(ws_bytes, inp.device)
        check(_L.tango_absmax_ex_f32(_ptr(inp), rows, cols, ldx, _ptr(row_mul), _ptr(mask), ldm,
                                     _MASK_MODES[mask_mode], scale.data_ptr(), int(accumulate), _ptr(colsum), _ptr(ws), ws_bytes,
                                     _stream()), "absmax_ex")
        return scale, colsum

    @staticmethod
    def transpose_quant(inp, scale, nrow, ncol):
        _need(inp, torch.float32, "in")
        _need(scale, torch.float32, "scale")
        if inp.numel() != nrow * ncol:
            raise RuntimeError("transpose_quant: in has %d elements, expected %d" % (inp.numel(), nrow * ncol))
        out = torch.empty((ncol, nrow), dtype=torch.int8, device=inp.device)
        check(_L.tango_transpose_quant_f32_i8(_ptr(inp), nrow, ncol, scale.data_ptr(), _ptr(out),
                                              _stream()), "transpose_quant")
        return out

    # ------------------------------------------------------------------ GEMM
    @staticmethod
    def QGEMM_forward(Y, X, X_q, W, W_q, bias, scaleY, scaleX, scaleW, round_mode=None, x_row_mul=None):
        """``X`` None: ``X_q`` already holds X quantized with ``scaleX`` (one quantize pass shared by
        several layers that consume the same X)."""
        for t, dt, nm in ((Y, torch.float32, "Y"), (X, torch.float32, "X"), (W, torch.float32, "W")):
            if t is not None:
                _need(t, dt, nm, contiguous=False)
        _need(X_q, torch.int8, "X_q", contiguous=False)
        _need(W_q, torch.int8, "W_q")
        _need(scaleX, torch.float32, "scaleX")
        _need(scaleW, torch.float32, "scaleW")
        M, K = X_q.shape
        if X is None and x_row_mul is not None:
            raise RuntimeError("QGEMM_forward: x_row_mul needs the fp32 X")
        N = W.size(0)
        if (W.size(1) != K or tuple(Y.shape) != (M, N) or (X is not None and tuple(X.shape) != (M, K))
                or W_q.numel() != N * K):
            raise RuntimeError("QGEMM_forward: shape mismatch")
        if bias is not None and bias.numel():
            _need(bias, torch.float32, "bias")
            if bias.numel() != N:
                raise RuntimeError("QGEMM_forward: bias must have N elements")
        if scaleY is not None and scaleY.numel():
            _need(scaleY, torch.float32, "scaleY")
        mode = default_forward_round_mode() if round_mode is None else _mode(round_mode)
        ws_bytes = _ws_bytes("tango_qgemm_fwd_workspace", M, N, K)
        ws = _workspace(ws_bytes, X_q.device)
        if x_row_mul is not None:
            _need(x_row_mul, torch.float32, "x_row_mul")
            if x_row_mul.numel() != M:
                raise RuntimeError("QGEMM_forward: x_row_mul must have M entries")
        check(_L.tango_qgemm_fwd_ex(_ptr(Y), _rows_view(Y, "Y"), _ptr(X), 0 if X is None else _rows_view(X, "X"), _ptr(x_row_mul),
                                    _ptr(X_q), _rows_view(X_q, "X_q"), _ptr(W), _rows_view(W, "W"), _ptr(W_q),
                                    _ptr(bias), _ptr(scaleY),
                                 scaleX.data_ptr(), scaleW.data_ptr(), M, N, K, mode, _ptr(ws),
                                 ws_bytes, _stream()), "QGEMM_forward")

    @staticmethod
    def QGEMM_forward_q8(Y_q, scaleY, X_q, W, W_q, bias, scaleX, scaleW, round_mode=None):
        """int8 Y_q = quantize(X W^T + bias) and scaleY = max|X W^T + bias| / 127 from the already quantized
        X_q, without the fp32 product in memory.  Returns False (nothing launched) where the kernel does not
        apply (reduction above 256, rows of X_q not 16-byte aligned, stochastic rounding)."""
        _need(Y_q, torch.int8, "Y_q", contiguous=False)
        _need(X_q, torch.int8, "X_q", contiguous=False)
        _need(W, torch.float32, "W", contiguous=False)
        _need(W_q, torch.int8, "W_q")
        for t, nm in ((scaleY, "scaleY"), (scaleX, "scaleX"), (scaleW, "scaleW")):
            _need(t, torch.float32, nm)
        M, K = X_q.shape
        N = W.size(0)
        if W.size(1) != K or tuple(Y_q.shape) != (M, N) or W_q.numel() != N * K:
            raise RuntimeError("QGEMM_forward_q8: shape mismatch")
        if bias is not None:
            _need(bias, torch.float32, "bias")
            if bias.numel() != N:
                raise RuntimeError("QGEMM_forward_q8: bias must have N elements")
        mode = default_forward_round_mode() if round_mode is None else _mode(round_mode)
        ws_bytes = _ws_bytes("tango_qgemm_fwd_workspace", M, N, K)
        ws = _workspace(ws_bytes, X_q.device)
        rc = _L.tango_qgemm_fwd_q8(_ptr(Y_q), _rows_view(Y_q, "Y_q"), scaleY.data_ptr(), _ptr(X_q),
                                   _rows_view(X_q, "X_q"), _ptr(W), _rows_view(W, "W"), _ptr(W_q), _ptr(bias),
                                   scaleX.data_ptr(), scaleW.data_ptr(), M, N, K, mode, _ptr(ws), ws_bytes, _stream())
        if rc == -2:  # TANGO_ERR_UNSUPPORTED
            return False
        check(rc, "QGEMM_forward_q8")
        return True

    @staticmethod
    def QGEMM_i8(Y, A, B, bias, scaleY, scaleA, scaleB):
        """Y = dequant(A[M,K] . B[N,K]^T) on int8 operands (not in the reference)."""
        _need(Y, torch.float32, "Y", contiguous=False)
        _need(A, torch.int8, "A", contiguous=False)
        _need(B, torch.int8, "B", contiguous=False)
        M, K = A.shape
        N = B.size(0)
        if B.size(1) != K or tuple(Y.shape) != (M, N):
            raise RuntimeError("QGEMM_i8: shape mismatch")
        ws_bytes = _ws_bytes("tango_qgemm_i8_nt_workspace", M, N, K)
        ws = _workspace(ws_bytes, A.device)
        check(_L.tango_qgemm_i8_nt(_ptr(Y), _rows_view(Y, "Y"), _ptr(A), _rows_view(A, "A"), _ptr(B),
                                   _rows_view(B, "B"), _ptr(bias), _ptr(scaleY), scaleA.data_ptr(),
                                   scaleB.data_ptr(), M, N, K, _ptr(ws), ws_bytes, _stream()), "QGEMM_i8")

    @staticmethod
    def QGEMM_backward_gradX(dX, dY, W, scaledY, scaleW, row_scale=None, accumulate=False, masked=None):
        """``accumulate``: add the product to what dX holds instead of overwriting it.  ``masked`` = (sign words int16
        [M, K / 16], row multiplier [M] or None): returns max|dX' * multiplier| / 127 with dX' = dX where its sign bit
        is set, else 0 (None when the shape is not one the epilogue takes, and otherwise)."""
        _need(dX, torch.float32, "dX", contiguous=False)
        _need(dY, torch.int8, "dY", contiguous=False)
        _need(W, torch.int8, "W", contiguous=False)
        _need(scaledY, torch.float32, "scaledY")
        _need(scaleW, torch.float32, "scaleW")
        M, K = dX.shape
        N = dY.size(1)
        if dY.size(0) != M or tuple(W.shape) != (N, K):
            raise RuntimeError("QGEMM_backward_gradX: shape mismatch")
        ws_bytes = _ws_bytes("tango_qgemm_bwd_dx_workspace", M, N, K)
        ws = _workspace(ws_bytes, dY.device)
        if row_scale is not None:
            _need(row_scale, torch.float32, "row_scale")
        if masked is not None:
            # also the scale of dX taken back through a ReLU (sign words) and multiplied row by row, from the epilogue
            bits, mul = masked
            _need(bits, torch.int16, "mask bits")
            if mul is not None:
                _need(mul, torch.float32, "mask multiplier")
            if accumulate or K % 16 or tuple(bits.shape) != (M, K // 16) or (mul is not None and mul.numel() != M):
                raise RuntimeError("QGEMM_backward_gradX: the mask must be int16 [M, K / 16] and excludes accumulate")
            scale = torch.empty(1, dtype=torch.float32, device=dX.device)
            rc = _L.tango_qgemm_bwd_dx_masked(_ptr(dX), _rows_view(dX, "dX"), _ptr(dY), _rows_view(dY, "dY"), _ptr(W),
                                              _rows_view(W, "W"), scaledY.data_ptr(), scaleW.data_ptr(), _ptr(row_scale),
                                              _ptr(bits), K // 16, _ptr(mul), scale.data_ptr(), M, N, K, _ptr(ws),
                                              ws_bytes, _stream())
            if rc != -2:  # -2: not a shape the masked epilogue takes; the plain call below runs instead
                check(rc, "QGEMM_backward_gradX")
                return scale
        check(_L.tango_qgemm_bwd_dx_ex(_ptr(dX), _rows_view(dX, "dX"), _ptr(dY), _rows_view(dY, "dY"),
                                       _ptr(W), _rows_view(W, "W"), scaledY.data_ptr(), scaleW.data_ptr(),
                                       _ptr(row_scale), int(bool(accumulate)), M, N, K, _ptr(ws), ws_bytes,
                                       _stream()),
              "QGEMM_backward_gradX")

    @staticmethod
    def QGEMM_backward_gradW(dW, dY, X, scaledY, scaleX):
        _need(dW, torch.float32, "dW", contiguous=False)
        _need(dY, torch.int8, "dY", contiguous=False)
        _need(X, torch.int8, "X", contiguous=False)
        _need(scaledY, torch.float32, "scaledY")
        _need(scaleX, torch.float32, "scaleX")
        N, K = dW.shape
        M = dY.size(0)
        if dY.size(1) != N or tuple(X.shape) != (M, K):
            raise RuntimeError("QGEMM_backward_gradW: shape mismatch")
        ws_bytes = _ws_bytes("tango_qgemm_bwd_dw_workspace", M, N, K)
        ws = _workspace(ws_bytes, X.device)
        check(_L.tango_qgemm_bwd_dw(_ptr(dW), _rows_view(dW, "dW"), _ptr(dY), _rows_view(dY, "dY"),
                                    _ptr(X), _rows_view(X, "X"), scaledY.data_ptr(), scaleX.data_ptr(),
                                    M, N, K, _ptr(ws), ws_bytes, _stream()), "QGEMM_backward_gradW")

    @staticmethod
    def _legacy(A, B, trans_a, trans_b):
        _need(A, torch.float32, "A")
        _need(B, torch.float32, "B")
        m = A.size(1) if trans_a else A.size(0)
        k = A.size(0) if trans_a else A.size(1)
        n = B.size(0) if trans_b else B.size(1)
        if (B.size(1) if trans_b else B.size(0)) != k:
            raise RuntimeError("Qgemm: inner dimensions differ")
        out = torch.empty((m, n), dtype=torch.float32, device=A.device)
        ws_bytes = _ws_bytes("tango_qgemm_legacy_workspace", m, n, k)
        ws = _workspace(ws_bytes, A.device)
        check(_L.tango_qgemm_legacy(_ptr(out), _ptr(A), _ptr(B), m, n, k, int(trans_a), int(trans_b),
                                    _ptr(ws), ws_bytes, _stream()), "Qgemm")
        return out

    @staticmethod
    def QgemmNT(A, B):
        return cuda_kernels._legacy(A, B, False, True)

    @staticmethod
    def QgemmTN(A, B):
        return cuda_kernels._legacy(A, B, True, False)

    @staticmethod
    def QgemmNN(A, B):
        return cuda_kernels._legacy(A, B, False, False)

    # ------------------------------------------------------------------ SpMM
    @staticmethod
    def csr_SPMM(out, indptr, indices, U, scaleU, ldf=None, F=None, row_scale=None, bias=None, relu=False,
                 max_row=0, sign_bits=None, scale_out=None, scale_mul=None):
        """``sign_bits`` (int16 [rows, F / 16], F a multiple of 16): receives one bit per output element,
        set where it is positive: all a backward pass needs of a ReLU's output.
        ``scale_out`` (1-element fp32 holding 0): receives max|out * scale_mul[:, None]| / 127 (``scale_mul``
        optional, one fp32 per row), formed in the kernel's epilogue."""
        _need(out, torch.float32, "out")
        _need(indptr, torch.int64, "indptr")
        idx_bits = _need_index(indices, "indices")
        _need(U, torch.int8, "U")
        _need(scaleU, torch.float32, "scaleU")
        rows = indptr.numel() - 1
        width = math.prod(U.shape[1:])
        ldf = width if ldf is None else ldf
        F = width if F is None else F
        if out.numel() != rows * F:
            raise RuntimeError("csr_SPMM: out must be [%d, %d]" % (rows, F))
        if sign_bits is not None:
            _need(sign_bits, torch.int16, "sign_bits")
            if F % 16 or tuple(sign_bits.shape) != (rows, F // 16):
                raise RuntimeError("csr_SPMM: sign_bits must be int16 [rows, F / 16], F a multiple of 16")
        if (row_scale is None and bias is None and not relu and idx_bits == 64 and not max_row and sign_bits is None
                and scale_out is None):
            check(_L.tango_spmm_csr_copy_u(_ptr(out), indptr.data_ptr(), _ptr(indices), _ptr(U), ldf,
                                           scaleU.data_ptr(), rows, U.size(0), indices.numel(), F,
                                           _stream()), "csr_SPMM")
            return
        if row_scale is not None:
            _need(row_scale, torch.float32, "row_scale")
            if row_scale.numel() != rows:
                raise RuntimeError("csr_SPMM: row_scale must have one entry per output row")
        if bias is not None:
            _need(bias, torch.float32, "bias")
            if bias.numel() != F:
                raise RuntimeError("csr_SPMM: bias must have F entries")
        if scale_mul is not None:
            _need(scale_mul, torch.float32, "scale_mul")
            if scale_mul.numel() != rows or scale_out is None:
                raise RuntimeError("csr_SPMM: scale_mul needs one entry per output row and a scale_out")
        ws_bytes = _ws_bytes("tango_spmm_workspace", rows, indices.numel(), F)
        ws = _workspace(ws_bytes, U.device)
        check(_L.tango_spmm_csr_copy_u_ex(_ptr(out), indptr.data_ptr(), _ptr(indices), idx_bits, _ptr(U), ldf,
                                          scaleU.data_ptr(), _ptr(row_scale), _ptr(bias), int(bool(relu)),
                                          _ptr(sign_bits), rows, U.size(0), indices.numel(), F, int(max_row),
                                          _ptr(scale_mul), _ptr(scale_out), _ptr(ws), ws_bytes,
                                          _stream()), "csr_SPMM")

    @staticmethod
    def csr_SPMM_dense(out, plan, U, scaleU, ldf=None, F=None, row_scale=None, bias=None, relu=False, sign_bits=None,
                       scale_out=None, scale_mul=None):
        """csr_SPMM on an adjacency split by ``dense_plan.build_dense_plan`` into bit blocks (multiplied with
        U on the matrix cores) and a sparse rest; same result as csr_SPMM on the whole CSR, bit for bit.
        Returns False (nothing launched) when U's layout rules the dense path out."""
        _need(out, torch.float32, "out")
        _need(U, torch.int8, "U")
        _need(scaleU, torch.float32, "scaleU")
        width = math.prod(U.shape[1:])
        ldf = width if ldf is None else ldf
        F = width if F is None else F
        if F > 256 or ldf % 16 or (F + 15) // 16 * 16 > ldf or U.data_ptr() % 16 or U.size(0) != plan.num_src:
            return False
        if out.numel() != plan.rows * F:
            raise RuntimeError("csr_SPMM_dense: out must be [%d, %d]" % (plan.rows, F))
        if sign_bits is not None:
            _need(sign_bits, torch.int16, "sign_bits")
            if F % 16 or tuple(sign_bits.shape) != (plan.rows, F // 16):
                raise RuntimeError("csr_SPMM_dense: sign_bits must be int16 [rows, F / 16], F a multiple of 16")
        if row_scale is not None:
            _need(row_scale, torch.float32, "row_scale")
            if row_scale.numel() != plan.rows:
                raise RuntimeError("csr_SPMM_dense: row_scale must have one entry per output row")
        if bias is not None:
            _need(bias, torch.float32, "bias")
            if bias.numel() != F:
                raise RuntimeError("csr_SPMM_dense: bias must have F entries")
        if scale_mul is not None:
            _need(scale_mul, torch.float32, "scale_mul")
            if scale_mul.numel() != plan.rows or scale_out is None:
                raise RuntimeError("csr_SPMM_dense: scale_mul needs one entry per output row and a scale_out")
        key = ("dense", id(plan), F)
        ws_bytes = _WS_SIZES.get(key)
        if ws_bytes is None:
            ws_bytes = _WS_SIZES[key] = _L.tango_spmm_dense_workspace(plan.ref, F)
        ws = _workspace(ws_bytes, U.device)
        check(_L.tango_spmm_csr_copy_u_dense(_ptr(out), plan.ref, _ptr(U), ldf, scaleU.data_ptr(), _ptr(row_scale),
                                             _ptr(bias), int(bool(relu)), _ptr(sign_bits), F, _ptr(scale_mul),
                                             _ptr(scale_out), _ptr(ws), ws_bytes, _stream()), "csr_SPMM_dense")
        return True

    @staticmethod
    def multi_cusparse_SPMM(indptr, indices, N, E_T, scale, edge_ids=None, edge_major=False, bias=None, max_row=0,
                            scale2=None, act=None):
        """E_T is [H, D, nnz] in CSR slot order, or in edge-id order when the
        slot->edge permutation ``edge_ids`` is passed (gather fused in-kernel).
        With ``edge_major`` the edge values are [nnz, H, D] instead (no transpose pass).
        ``bias`` ([H * F] fp32) is added to every output row after dequantization.  ``max_row``: an
        upper bound of the longest row if known (0 = unknown).  ``scale2``: the output is dequantized
        with scale * scale2 (saves the launch that multiplies two 1-element tensors).  ``act``: None,
        "relu" or "elu", applied last."""
        _need(indptr, torch.int64, "indptr")
        idx_bits = _need_index(indices, "indices")
        _need(N, torch.int8, "N")
        on_load = E_T.dtype == torch.float32  # fp32 edge values, rounded with scale2 as the kernel loads them
        _need(E_T, torch.float32 if on_load else torch.int8, "E_T")
        _need(scale, torch.float32, "scale")
        if scale2 is not None:
            _need(scale2, torch.float32, "scale2")
        if on_load and scale2 is None:
            raise RuntimeError("multi_cusparse_SPMM: fp32 edge values need their quantization scale (scale2)")
        if N.dim() != 3 or E_T.dim() != 3:
            raise RuntimeError("E and N must be 3D tensors")
        k, H, F = N.shape
        if edge_major:
            nnz, D = E_T.size(0), E_T.size(2)
            if E_T.size(1) != H or nnz != indices.numel() or D not in (1, F):
                raise RuntimeError("multi_cusparse_SPMM: edge-major E must be [nnz, H, 1|F]")
        else:
            D, nnz = E_T.size(1), E_T.size(2)
            if E_T.size(0) != H or nnz != indices.numel() or D not in (1, F):
                raise RuntimeError("multi_cusparse_SPMM: E_T must be [H, 1|F, nnz]")
        if edge_ids is not None and _need_index(edge_ids, "edge_ids") != idx_bits:
            raise RuntimeError("multi_cusparse_SPMM: indices and edge_ids must have the same integer width")
        if bias is not None:
            _need(bias, torch.float32, "bias")
            if bias.numel() != H * F:
                raise RuntimeError("multi_cusparse_SPMM: bias must have H * F elements")
        rows = indptr.numel() - 1
        out = torch.empty((rows, H, F), dtype=torch.float32, device=N.device)
        ws_bytes = _ws_bytes("tango_spmm_workspace", rows, nnz, H * F)
        ws = _workspace(ws_bytes, N.device)
        entry = _L.tango_spmm_csr_u_mul_e_f32e if on_load else _L.tango_spmm_csr_u_mul_e_ex
        check(entry(_ptr(out), indptr.data_ptr(), _ptr(indices), _ptr(edge_ids), idx_bits,
                    _ptr(N), _ptr(E_T), int(bool(edge_major)), scale.data_ptr(),
                    _ptr(scale2), _ptr(bias), _ACTIVATIONS[act], rows, k, H, F, D, nnz,
                    int(max_row), _ptr(ws), ws_bytes,
                    _stream()), "multi_cusparse_SPMM")
        return out

    # The reference's SpMV binding returns uninitialised memory (cuda/src/SPMM.cu:196-257)
    # and its Python wrapper calls the SpMM instead (cuda/kernels.py:168-178).
    multi_cusparse_SPMV = multi_cusparse_SPMM

    @staticmethod
    def incidence_SPMM(out, src, dst, E, scale):
        """src = node ids (sorted), dst = edge ids: rows 0 and 1 of g.inc_in / g.inc_out."""
        _need(out, torch.float32, "out")
        _need(src, torch.int64, "src")
        _need(dst, torch.int64, "dst")
        _need(E, torch.int8, "E")
        _need(scale, torch.float32, "scale")
        F = math.prod(E.shape[1:])
        if out.dim() != 2 or out.size(1) != F:
            raise RuntimeError("incidence_SPMM: out must be [num_nodes, %d]" % F)
        check(_L.tango_spmm_incidence(_ptr(out), _ptr(src), _ptr(dst), _ptr(E), scale.data_ptr(),
                                      out.size(0), src.numel(), E.size(0), F, _stream()),
              "incidence_SPMM")

    # ----------------------------------------------------------------- SDDMM
    @staticmethod
    def mySDDMM_int8(op, out, scaleOut, src, dst, U, V, scaleU, scaleV):
        _need(out, torch.float32, "out")
        _need(src, torch.int64, "src")
        _need(dst, torch.int64, "dst")
        _need(U, torch.int8, "U")
        _need(V, torch.int8, "V")
        _need(scaleU, torch.float32, "scaleU")
        _need(scaleV, torch.float32, "scaleV")
        if scaleOut is not None and scaleOut.numel():
            _need(scaleOut, torch.float32, "scaleOut")
        E = src.numel()
        if dst.numel() != E:
            raise RuntimeError("mySDDMM_int8: src and dst differ in length")
        if U.shape[1:] != V.shape[1:]:
            raise RuntimeError("mySDDMM_int8: U and V must have equal feature shapes")
        if op == "dot":
            D = U.size(-1)
            H = math.prod(U.shape[1:-1])
            if out.numel() != E * H:
                raise RuntimeError("mySDDMM_int8: out must be [E, %d, 1]" % H)
            check(_L.tango_sddmm_dot_i8(_ptr(out), _ptr(scaleOut), _ptr(src), _ptr(dst), _ptr(U), _ptr(V),
                                        scaleU.data_ptr(), scaleV.data_ptr(), E, H, D, _stream()),
                  "mySDDMM_int8(dot)")
        elif op in SDDMM_OPS:
            T = math.prod(U.shape[1:])
            if out.numel() != E * T:
                raise RuntimeError("mySDDMM_int8: out must be [E, %d]" % T)
            check(_L.tango_sddmm_ewise_i8(SDDMM_OPS[op], _ptr(out), _ptr(scaleOut), _ptr(src), _ptr(dst),
                                          _ptr(U), _ptr(V), scaleU.data_ptr(), scaleV.data_ptr(), E, T,
                                          _stream()), "mySDDMM_int8(%s)" % op)
        else:
            # the reference only prints "op not supported" (cuda/src/SDDMM.cu:175)
            raise ValueError("%s op not supported" % op)

    @staticmethod
    def mySDDMM_quantize_on_load(op, out, src, dst, U, V, scaleU, scaleV, round_mode=ROUND_RNE):
        """mySDDMM_int8 for add / sub / mul / div on fp32 U, V that the kernel quantizes as it loads them."""
        for t, nm in ((out, "out"), (U, "U"), (V, "V"), (scaleU, "scaleU"), (scaleV, "scaleV")):
            _need(t, torch.float32, nm)
        _need(src, torch.int64, "src")
        _need(dst, torch.int64, "dst")
        if op not in SDDMM_OPS:
            raise ValueError("%s op not supported" % op)
        E = src.numel()
        T = math.prod(U.shape[1:])
        if dst.numel() != E or U.shape[1:] != V.shape[1:] or out.numel() != E * T:
            raise RuntimeError("mySDDMM_quantize_on_load: shape mismatch")
        check(_L.tango_sddmm_ewise_f32q(SDDMM_OPS[op], _ptr(out), _ptr(src), _ptr(dst), _ptr(U), _ptr(V),
                                        scaleU.data_ptr(), scaleV.data_ptr(), E, T, _mode(round_mode), _stream()),
              "mySDDMM_quantize_on_load(%s)" % op)

    # ---------------------------------------------------------- edge softmax
    @staticmethod
    def edge_softmax_forward(e, indptr, edge_ids, slope=1.0):
        _need(e, torch.float32, "e")
        _need(indptr, torch.int64, "indptr")
        H = e.numel() // max(e.size(0), 1)
        a = torch.empty_like(e)
        ws_bytes = _ws_bytes("tango_edge_softmax_workspace", e.size(0), H)
        ws = _workspace(ws_bytes, e.device)
        check(_L.tango_edge_softmax_fwd(_ptr(a), _ptr(e), indptr.data_ptr(), _ptr(edge_ids),
                                        indptr.numel() - 1, e.size(0), H, float(slope), _ptr(ws), ws_bytes,
                                        _stream()),
              "edge_softmax")
        return a

    @staticmethod
    def edge_softmax_forward_ex(e, indptr, edge_ids, slope=1.0, logits=None, want_sign=False):
        """The attention block's forward: (a, max(a) / 127, sign bytes or None).  ``logits``: None (``e`` [E, H]
        is read) or (el, er, s_el, s_er, src, dst): e = q(el[src]) s_el + q(er[dst]) s_er is formed inside the
        kernel and never stored (then ``e`` is None).  ``want_sign``: also return [E, ceil(H / 8)] uint8 in
        destination-major slot order, bit h % 8 of byte [slot, h / 8] = (e > 0)."""
        s_a = torch.empty(1, dtype=torch.float32, device=indptr.device)
        if logits is None:
            _need(e, torch.float32, "e")
            E, H = e.size(0), e.numel() // max(e.size(0), 1)
            shape, args = e.shape, (_ptr(e), None, None, None, None, None, None)
        else:
            el, er, s_el, s_er, src, dst = logits
            for t, nm in ((el, "el"), (er, "er"), (s_el, "s_el"), (s_er, "s_er")):
                _need(t, torch.float32, nm)
            _need(src, torch.int64, "src")
            _need(dst, torch.int64, "dst")
            E, H = src.numel(), el.numel() // max(el.size(0), 1)
            if er.numel() // max(er.size(0), 1) != H or dst.numel() != E:
                raise RuntimeError("edge_softmax: el, er must have the same heads and src, dst one entry per edge")
            shape = (E,) + tuple(el.shape[1:])
            args = (None, _ptr(el), _ptr(er), s_el.data_ptr(), s_er.data_ptr(), src.data_ptr(), dst.data_ptr())
        _need(indptr, torch.int64, "indptr")
        a = torch.empty(shape, dtype=torch.float32, device=indptr.device)
        sign = torch.empty((E, (H + 7) // 8), dtype=torch.uint8, device=indptr.device) if want_sign else None
        ws_bytes = _ws_bytes("tango_edge_softmax_workspace", E, H)
        ws = _workspace(ws_bytes, indptr.device)
        check(_L.tango_edge_softmax_fwd_ex(_ptr(a), s_a.data_ptr(), _ptr(sign), *args, indptr.data_ptr(),
                                           _ptr(edge_ids), indptr.numel() - 1, E, H, float(slope), _ptr(ws), ws_bytes,
                                           _stream()), "edge_softmax_ex")
        return a, s_a, sign

    @staticmethod
    def edge_softmax_backward_ex(a, da, e, sign, indptr, edge_ids, slope=1.0):
        """(de, max|de| / 127) of the attention block's backward; ``e`` or ``sign`` (the forward's sign bytes) gives
        LeakyReLU's derivative (neither is needed for slope 1)."""
        s_de = torch.empty(1, dtype=torch.float32, device=a.device)
        _need(a, torch.float32, "a")
        _need(da, torch.float32, "da")
        if e is not None:
            _need(e, torch.float32, "e")
        E, H = a.size(0), a.numel() // max(a.size(0), 1)
        de = torch.empty_like(a)
        ws_bytes = _ws_bytes("tango_edge_softmax_workspace", E, H)
        ws = _workspace(ws_bytes, a.device)
        check(_L.tango_edge_softmax_bwd_ex(_ptr(de), s_de.data_ptr(), _ptr(a), _ptr(da), _ptr(e), _ptr(sign),
                                           indptr.data_ptr(), _ptr(edge_ids), indptr.numel() - 1, E, H, float(slope),
                                           _ptr(ws), ws_bytes, _stream()), "edge_softmax_backward_ex")
        return de, s_de

    @staticmethod
    def edge_softmax_backward(a, da, e, indptr, edge_ids, slope=1.0):
        """``e`` may be None for slope 1 (the plain softmax's backward does not read it)."""
        _need(a, torch.float32, "a")
        _need(da, torch.float32, "da")
        if e is not None:
            _need(e, torch.float32, "e")
        elif float(slope) != 1.0:
            raise RuntimeError("edge_softmax_backward: e is needed for LeakyReLU's derivative")
        H = a.numel() // max(a.size(0), 1)
        de = torch.empty_like(a)
        ws_bytes = _ws_bytes("tango_edge_softmax_workspace", a.size(0), H)
        ws = _workspace(ws_bytes, a.device)
        check(_L.tango_edge_softmax_bwd(_ptr(de), _ptr(a), _ptr(da), _ptr(e), indptr.data_ptr(),
                                        _ptr(edge_ids), indptr.numel() - 1, a.size(0), H, float(slope), _ptr(ws),
                                        ws_bytes, _stream()),
              "edge_softmax_backward")
        return de

    # ------------------------------------------------- GAT attention logits
    @staticmethod
    def attn_scores_forward(feat, attn_l, attn_r, want_scales=False):
        """el, er [n, H] from feat [n, H, D] and attn_l, attn_r [H, D] (evaluation/test_gat.py:135-137).
        ``want_scales``: also return max|el| / 127 and max|er| / 127 (1-element tensors, or None while the
        stream is being captured), found by the same kernel."""
        for t, nm in ((feat, "feat"), (attn_l, "attn_l"), (attn_r, "attn_r")):
            _need(t, torch.float32, nm)
        n, H, D = feat.shape
        if attn_l.numel() != H * D or attn_r.numel() != H * D:
            raise RuntimeError("attn_scores: attn_l / attn_r must have H * D elements")
        el = torch.empty((n, H), dtype=torch.float32, device=feat.device)
        er = torch.empty((n, H), dtype=torch.float32, device=feat.device)
        s_el = s_er = None
        if want_scales:
            s_el = _zero_slot(feat.device)
            s_er = _zero_slot(feat.device) if s_el is not None else None
        check(_L.tango_attn_scores_fwd(_ptr(el), _ptr(er), _ptr(s_el), _ptr(s_er), _ptr(feat), _ptr(attn_l),
                                       _ptr(attn_r), n, H, D, _stream()), "attn_scores_forward")
        return (el, er, s_el, s_er) if want_scales else (el, er)

    @staticmethod
    def attn_scores_backward(del_, der, feat, attn_l, attn_r, addend=None):
        """(dfeat [n, H, D], dattn_l [H, D], dattn_r [H, D]).  ``addend`` (fp32, feat's shape): the gradient feat
        receives from another consumer; dfeat is then the sum of the two and a fourth result is max|dfeat| / 127,
        found by the same kernel."""
        for t, nm in ((del_, "del"), (der, "der"), (feat, "feat"), (attn_l, "attn_l"), (attn_r, "attn_r")):
            _need(t, torch.float32, nm)
        n, H, D = feat.shape
        if del_.numel() != n * H or der.numel() != n * H:
            raise RuntimeError("attn_scores_backward: del / der must have n * H elements")
        dfeat = torch.empty_like(feat)
        dal = torch.empty((H, D), dtype=torch.float32, device=feat.device)
        dar = torch.empty((H, D), dtype=torch.float32, device=feat.device)
        ws_bytes = _ws_bytes("tango_attn_scores_bwd_workspace", n, H, D)
        ws = _workspace(ws_bytes, feat.device)
        if addend is not None:
            _need(addend, torch.float32, "addend")
            if addend.numel() != feat.numel():
                raise RuntimeError("attn_scores_backward: addend must have feat's size")
            scale = _zero_slot(feat.device)
            check(_L.tango_attn_scores_bwd_acc(_ptr(dfeat), _ptr(dal), _ptr(dar), _ptr(scale), _ptr(addend), _ptr(del_),
                                               _ptr(der), _ptr(feat), _ptr(attn_l), _ptr(attn_r), n, H, D, _ptr(ws),
                                               ws_bytes, _stream()), "attn_scores_backward")
            return dfeat, dal, dar, scale
        check(_L.tango_attn_scores_bwd(_ptr(dfeat), _ptr(dal), _ptr(dar), _ptr(del_), _ptr(der), _ptr(feat),
                                       _ptr(attn_l), _ptr(attn_r), n, H, D, _ptr(ws), ws_bytes, _stream()),
              "attn_scores_backward")
        return dfeat, dal, dar


# ------------------------------------------------------------------ wrappers
def quantize(t, scale=None, round_mode=ROUND_RNE, noise=None, seed=0, offset=0, advance=0):
    """Quantize to int8; returns (int8 tensor, scale).  cuda/kernels.py:19-30."""
    assert t.is_cuda, "tensor must be on GPU"
    if scale is None:
        scale = cuda_kernels.get_scale(t)
    out = torch.empty(t.shape, dtype=torch.int8, device=t.device)
    cuda_kernels.quantize(out, t, scale, round_mode=round_mode, noise=noise, seed=seed, offset=offset,
                          advance=advance)
    return out, scale


def quantize_padded(t, scale=None, round_mode=ROUND_RNE, noise=None, seed=0, offset=0, align=16,
                    row_mul=None, mask=None, mask_mode="relu", advance=0):
    """Like ``quantize`` for a 2-D tensor, but the int8 rows are padded with
    zeros to a multiple of ``align`` bytes so that the SpMM gather and the GEMM
    fragment loads stay 16-byte aligned for odd widths (41, 602, ...).  Returns a
    [rows, cols] view of the padded buffer and the scale."""
    assert t.is_cuda and t.dim() == 2, "2-D GPU tensor expected"
    if scale is None:
        if row_mul is not None or mask is not None:
            scale, _ = cuda_kernels.absmax_ex(t, row_mul=row_mul, mask=mask, mask_mode=mask_mode)
        else:
            scale = cuda_kernels.get_scale(t) if t.is_contiguous() else cuda_kernels.get_scale(t.contiguous())
    rows, cols = t.shape
    ld = (cols + align - 1) // align * align
    buf = torch.empty((rows, ld), dtype=torch.int8, device=t.device)
    if ld == cols and row_mul is None and mask is None and t.is_contiguous():
        # nothing to pad: the flat kernel (16-byte loads front to back, same element -> noise index mapping)
        cuda_kernels.quantize(buf, t, scale, round_mode=round_mode, noise=noise, seed=seed, offset=offset,
                              advance=advance)
    else:
        cuda_kernels.quantize_rows(buf, t, scale, round_mode=round_mode, noise=noise, seed=seed, offset=offset,
                                   row_mul=row_mul, mask=mask, mask_mode=mask_mode, advance=advance)
    return buf[:, :cols], scale


def pad_heads(D, H=1):
    """Columns per head of the int8 copy of an [n, H, D] tensor: D itself, or the next multiple of 16 when the rows
    of H * D bytes could only be gathered byte by byte (H * D not a multiple of 4: 3 x 250, 1 x 41) or when heads
    of 128 columns or more are not whole 16-byte pieces (3 x 248): the gathers of the aggregation and of the SDDMM
    then run on aligned 16-byte pieces."""
    if D % 16 != 0 and D >= 24 and ((H * D) % 4 != 0 or D >= 128):
        return (D + 15) // 16 * 16
    return D


def quantize_heads(t, scale=None, **kw):
    """``quantize`` for a 3-D [n, H, D] tensor with every head zero-padded to ``pad_heads(D)`` columns: returns
    (int8 [n, H, pad_heads(D)], scale).  The zeros add nothing to a dot product or an aggregation."""
    if t.dim() != 3 or pad_heads(t.size(2), t.size(1)) == t.size(2):
        return quantize(t, scale, **kw)
    n, H, D = t.shape
    Dp = pad_heads(D, H)
    t = t if t.is_contiguous() else t.contiguous()
    if scale is None:
        scale = cuda_kernels.get_scale(t)
    if kw.get("mask") is not None:  # an [n, H D] activation output: the same rows as t
        kw["mask"] = kw["mask"].reshape(n * H, D)
    q, scale = quantize_padded(t.view(n * H, D), scale, align=16, **kw)  # the [n H, D] view of an [n H, Dp] buffer
    return q.as_strided((n, H, Dp), (H * Dp, Dp, 1)), scale


def unpad_heads(t, D):
    """[n, H, D] contiguous from a result computed on head-padded operands."""
    return t if t.size(-1) == D else t[..., :D].contiguous()


def mySDDMM_int8(g, op, U, V, scaleU, scaleV, isReduce, reverse=False):
    """cuda/kernels.py:33-59."""
    if reverse:
        dst, src = g.coo
    else:
        src, dst = g.coo
    assert src.is_cuda, "src must be on GPU"
    assert dst.is_cuda, "dst must be on GPU"
    assert U.is_cuda, "U must be on GPU"
    assert V.is_cuda, "V must be on GPU"
    assert scaleU.is_cuda, "scaleU must be on GPU"
    assert scaleV.is_cuda, "scaleV must be on GPU"
    UV_unsqueezed = False
    if len(U.shape) == 2 and len(V.shape) == 2:
        U = U.unsqueeze(1)
        V = V.unsqueeze(1)
        UV_unsqueezed = True
    out_shape = (src.size(0),) + infer_broadcast_shape(op, U.shape[1:], V.shape[1:])
    out = torch.empty(out_shape, dtype=torch.float32, device=src.device)
    if isReduce:
        scale = torch.zeros((1,), dtype=torch.float32, device=src.device)
    else:
        scale = torch.Tensor()
    cuda_kernels.mySDDMM_int8(op, out, scale, src, dst, U, V, scaleU, scaleV)
    if UV_unsqueezed:
        out = out.squeeze(1)
    return out, scale


def QGEMM_forward(x, x_, scaleX, w, w_, scaleW, bias=None, isReduce=False, round_mode=None, x_row_mul=None):
    """cuda/kernels.py:79-95.  ``x`` None: ``x_`` is an input (x quantized with scaleX by the caller)."""
    assert x_.is_cuda, "x must be on GPU"
    assert w.is_cuda, "w must be on GPU"
    assert bias is None or bias.is_cuda, "bias must be on GPU"
    assert x_.size(1) == w.size(1), "x and w must have the same number of columns"
    out_fp = torch.empty((x_.size(0), w.size(0)), dtype=torch.float32, device=x_.device)
    scale_out = torch.empty_like(scaleX) if isReduce else torch.Tensor()
    bias = torch.Tensor() if bias is None else bias
    cuda_kernels.QGEMM_forward(out_fp, x, x_, w, w_, bias, scale_out, scaleX, scaleW,
                               round_mode=round_mode, x_row_mul=x_row_mul)
    if isReduce:
        return out_fp, scale_out
    return out_fp


def mySDDMM_quantize_on_load(g, op, U, V, scaleU, scaleV, round_mode=ROUND_RNE):
    """``mySDDMM_int8(g, op, quantize(U, scaleU)[0], quantize(V, scaleV)[0], scaleU, scaleV, False)[0]`` for
    add / sub / mul / div without the two quantize passes: the kernel rounds the fp32 values as it gathers them."""
    src, dst = g.coo
    U3, V3 = (U.unsqueeze(1), V.unsqueeze(1)) if U.dim() == 2 and V.dim() == 2 else (U, V)
    out_shape = (src.size(0),) + infer_broadcast_shape(op, U3.shape[1:], V3.shape[1:])
    out = torch.empty(out_shape, dtype=torch.float32, device=src.device)
    cuda_kernels.mySDDMM_quantize_on_load(op, out, src, dst, U3, V3, scaleU, scaleV, round_mode)
    return out.squeeze(1) if U3 is not U else out


def QGEMM_backward(dY, X, W, scaledY, scaleX, scaleW, X_need=True, W_need=True, x_row_scale=None, dX_acc=None,
                   dx_masked=None):
    """cuda/kernels.py:97-111.  ``dX_acc``: a gradient of X from another consumer; the input gradient is
    added to it in place (and it is returned) instead of going to a new tensor.
    When K is not a multiple of 32 (and above 32) the returned dX is the [M, K] view of a buffer whose rows are
    padded to 32 floats: not contiguous, and as a leaf's ``.grad`` it keeps the padded allocation alive; callers
    that need dense storage call ``.contiguous()`` on it (one [M, K] copy).
    ``dx_masked`` = (sign words, row multiplier or None) of the ReLU and row scaling that the consumer of dX will
    apply to it: gradX's epilogue then also finds the scale of that product and leaves it on dX."""
    assert scaledY.is_cuda, "scaledY must be on GPU"
    assert dY.is_cuda, "dY must be on GPU"
    dX, dW = None, None
    if X_need:
        assert W.is_cuda, "W must be on GPU"
        assert scaleW.is_cuda, "scaleW must be on GPU"
        if dX_acc is not None:
            dX = dX_acc
        elif X.dim() == 2 and X.size(1) % 32 != 0 and X.size(1) > 32:
            # rows padded to whole 128-byte lines (the [M, K] view is returned): the GEMM's 64-byte output
            # pieces then never straddle a line, which rows of e.g. 602 floats (2408 bytes) make them do
            ld = (X.size(1) + 31) // 32 * 32
            dX = torch.empty((X.size(0), ld), dtype=torch.float32, device=X.device)[:, :X.size(1)]
        else:
            dX = torch.empty(X.shape, dtype=torch.float32, device=X.device)
        masked_scale = cuda_kernels.QGEMM_backward_gradX(dX, dY, W, scaledY, scaleW, row_scale=x_row_scale,
                                                         accumulate=dX_acc is not None,
                                                         masked=dx_masked if dX_acc is None else None)
        if masked_scale is not None:
            # for the consumer that takes dX back through that ReLU (SPMM.masked_scale_hint)
            dX._tango_masked_scale = (masked_scale, dx_masked[0], dx_masked[1], dX._version, dX.data_ptr())
    if W_need:
        assert X.is_cuda, "X must be on GPU"
        assert scaleX.is_cuda, "scaleX must be on GPU"
        dW = torch.empty(W.shape, dtype=torch.float32, device=X.device)
        cuda_kernels.QGEMM_backward_gradW(dW, dY, X, scaledY, scaleX)
    return dX, dW


def transpose_quant(data, scale):
    """[nnz, H, D] fp32 -> int8 [H, D, nnz].  cuda/kernels.py:114-119."""
    assert data.ndim == 3
    nrow = data.size(0)
    ncol = data.numel() // max(nrow, 1)
    data_ = cuda_kernels.transpose_quant(data, scale, nrow, ncol)
    return data_.reshape((data.size(1), data.size(2), nrow))


def _csr_of(g, reverse):
    """(indptr, indices, edge_ids, longest row) of the source-major (reverse) or destination-major
    CSR, with the 32-bit copies of indices / edge_ids and the row-length bound when
    graph_preprocess made them (0 = unknown)."""
    indptr, indices, edge_ids = g.adj_csr if reverse else g.adj_csc
    narrow = getattr(g, "adj_csr32" if reverse else "adj_csc32", None)
    if narrow is not None:
        indices, edge_ids = narrow
    if getattr(g, "csr_slots_are_edge_ids" if reverse else "csc_slots_are_edge_ids", False):
        edge_ids = None  # identity: edge tensors are addressed by the slot itself
    return indptr, indices, edge_ids, getattr(g, "max_out_degree" if reverse else "max_in_degree", 0)


def multi_cusparse_SPMM(g, N, E_T, scale, reverse=False, edge_major=False, bias=None, scale2=None, act=None):
    """E_T is [H, D, nnz] in edge-id order.  cuda/kernels.py:122-136; the
    index_select by edge_ids of the reference happens inside the kernel.
    ``edge_major``: E_T is the quantized edge tensor as it is, [nnz, H, 1]."""
    assert E_T.ndim == 3 and N.ndim == 3, "E and N must be 3D tensors"
    assert E_T.size(2 if edge_major else 1) == 1, "Cannot broadcast E"
    assert E_T.dtype == torch.int8 or (edge_major and scale2 is not None), "fp32 E: edge-major, with its scale"
    indptr, indices, edge_ids, longest = _csr_of(g, reverse)
    if edge_ids is not None and edge_ids.numel() == 0:
        edge_ids = None
    return cuda_kernels.multi_cusparse_SPMM(indptr, indices, N, E_T, scale, edge_ids=edge_ids,
                                            edge_major=edge_major, bias=bias, max_row=longest, scale2=scale2,
                                            act=act)


def incidence_SPMM(g, E, scaleE, reverse=False):
    """cuda/kernels.py:139-152.  The incidence matrix in CSR form is (indptr, edge_ids) of the
    adjacency (the equivalence evaluation/test_incidence.py:14-22 relies on), which the graph
    already holds, so the row bounds come from indptr instead of a search in the COO node ids."""
    assert E.is_cuda and scaleE.is_cuda
    indptr, _, edge_ids, longest = _csr_of(g, reverse)
    if edge_ids is None:  # slot order = edge-id order: here the ids are the gather indices, identity or not
        narrow = getattr(g, "adj_csr32" if reverse else "adj_csc32", None)
        edge_ids = narrow[1] if narrow is not None else (g.adj_csr if reverse else g.adj_csc)[2]
    out_shape = (g.num_nodes(),) + E.shape[1:]
    dim = math.prod(E.shape[1:])
    out = torch.empty((g.num_nodes(), dim), dtype=torch.float32, device=E.device)
    cuda_kernels.csr_SPMM(out, indptr, edge_ids, E.reshape(E.size(0), dim), scaleE, max_row=longest)
    return out.view(out_shape)


def csr_SPMM(g, N, scaleN, reverse=False, row_scale=None, bias=None, relu=False, sign_bits=None, want_scale=False,
             scale_mul=None):
    """cuda/kernels.py:154-165.  N may be a 2-D view of a row-padded buffer.  ``row_scale`` / ``bias`` /
    ``relu`` fold "* norm, + bias, activation" (evaluation/test_gcn.py:123-137) into the kernel's epilogue;
    ``sign_bits`` (int16 [n, F / 16]) receives the signs of the output.  ``want_scale``: also returns
    max|out * scale_mul[:, None]| / 127 (``scale_mul`` optional), found in the epilogue: (out, scale)."""
    indptr, indices, _, longest = _csr_of(g, reverse)
    feat_shape = N.shape[1:]
    out_shape = (g.num_nodes(),) + feat_shape
    dim = math.prod(N.shape[1:])
    out = torch.empty((g.num_nodes(), dim), dtype=torch.float32, device=N.device)
    scale_out = None
    if want_scale:
        scale_out = _zero_slot(N.device)
        if scale_out is None:
            scale_out = torch.zeros(1, dtype=torch.float32, device=N.device)
    extra = dict(row_scale=row_scale, bias=bias, relu=relu, sign_bits=sign_bits, scale_out=scale_out, scale_mul=scale_mul)
    plan = getattr(g, "dense_csr" if reverse else "dense_csc", None)
    if N.dim() == 2 and not N.is_contiguous():
        ld = _rows_view(N, "N")
        base = N.as_strided((N.size(0), ld), (ld, 1))
        if not (plan is not None and cuda_kernels.csr_SPMM_dense(out, plan, base, scaleN, ldf=ld, F=dim, **extra)):
            cuda_kernels.csr_SPMM(out, indptr, indices, base, scaleN, ldf=ld, F=dim, max_row=longest, **extra)
    elif not (plan is not None and cuda_kernels.csr_SPMM_dense(out, plan, N.reshape(N.size(0), dim), scaleN, **extra)):
        cuda_kernels.csr_SPMM(out, indptr, indices, N, scaleN, max_row=longest, **extra)
    out = out.view(out_shape)
    return (out, scale_out) if want_scale else out


def multi_cusparse_SPMV(g, N_T, E_T, scale, reverse=False):
    """cuda/kernels.py:168-178 (which itself calls the SpMM binding)."""
    assert E_T.ndim == 3 and N_T.ndim == 3, "E and N must be 3D tensors"
    if reverse:
        indptr, indices, edge_ids = g.adj_csr
    else:
        indptr, indices, edge_ids = g.adj_csc
    return cuda_kernels.multi_cusparse_SPMM(indptr, indices, N_T, E_T, scale, edge_ids=edge_ids)
