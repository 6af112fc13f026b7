"""ctypes binding of libtango_hip.so (the C ABI declared in include/tango_hip.h).

There is no CPU fallback: if the library has not been built the import of any
operator fails with an explicit error.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libtango_hip.so")

P = C.c_void_p
I64 = C.c_int64
U64 = C.c_uint64
I = C.c_int
F = C.c_float
SZ = C.c_size_t

# name -> (restype, argtypes); mirrors include/tango_hip.h one to one
SIGNATURES = {
    "tango_status_string": (C.c_char_p, [I]),
    "tango_abi_version": (I, []),
    "tango_absmax_f32": (I, [P, I64, P, P]),
    "tango_absmax_acc_f32": (I, [P, I64, P, P]),
    "tango_absmax_rows_f32": (I, [P, I64, I64, I64, P, P]),
    "tango_quantize_f32_i8": (I, [P, I64, P, P, I, P, U64, U64, P, P]),
    "tango_counter_add_u64": (I, [P, U64, P]),
    "tango_quantize_rows_f32_i8": (I, [P, I64, I64, I64, P, I, P, I64, I, P, U64, U64, P]),
    "tango_absmax_ex_workspace": (SZ, [I64, I64, I]),
    "tango_absmax_ex_f32": (I, [P, I64, I64, I64, P, P, I64, I, P, I, P, P, SZ, P]),
    "tango_quantize_rows_ex_f32_i8": (I, [P, I64, I64, I64, P, P, I64, I, P, I, P, I64, I, P, U64, U64, P, P]),
    "tango_quantize_rows_colsum_workspace": (SZ, [I64, I64]),
    "tango_quantize_rows_colsum_f32_i8": (I, [P, I64, I64, P, P, I, P, P, I, P, U64, U64, P, P, P, SZ, P]),
    "tango_transpose_quant_f32_i8": (I, [P, I64, I64, P, P, P]),
    "tango_qgemm_fwd_workspace": (SZ, [I64, I64, I64]),
    "tango_qgemm_fwd": (I, [P, I64, P, I64, P, I64, P, I64, P, P, P, P, P, I64, I64, I64, I, P, SZ, P]),
    "tango_qgemm_fwd_ex": (I, [P, I64, P, I64, P, P, I64, P, I64, P, P, P, P, P, I64, I64, I64, I, P, SZ, P]),
    "tango_qgemm_i8_nt_workspace": (SZ, [I64, I64, I64]),
    "tango_qgemm_i8_nt": (I, [P, I64, P, I64, P, I64, P, P, P, P, I64, I64, I64, P, SZ, P]),
    "tango_qgemm_bwd_dx_workspace": (SZ, [I64, I64, I64]),
    "tango_qgemm_bwd_dx": (I, [P, I64, P, I64, P, I64, P, P, I64, I64, I64, P, SZ, P]),
    "tango_qgemm_fwd_q8": (I, [P, I64, P, P, I64, P, I64, P, P, P, P, I64, I64, I64, I, P, SZ, P]),
    "tango_qgemm_bwd_dx_ex": (I, [P, I64, P, I64, P, I64, P, P, P, I, I64, I64, I64, P, SZ, P]),
    "tango_qgemm_bwd_dx_masked": (I, [P, I64, P, I64, P, I64, P, P, P, P, I64, P, P, I64, I64, I64, P, SZ, P]),
    "tango_qgemm_bwd_dw_workspace": (SZ, [I64, I64, I64]),
    "tango_qgemm_bwd_dw": (I, [P, I64, P, I64, P, I64, P, P, I64, I64, I64, P, SZ, P]),
    "tango_qgemm_legacy_workspace": (SZ, [I64, I64, I64]),
    "tango_qgemm_legacy": (I, [P, P, P, I64, I64, I64, I, I, P, SZ, P]),
    "tango_spmm_csr_copy_u": (I, [P, P, P, P, I64, P, I64, I64, I64, I64, P]),
    "tango_spmm_workspace": (SZ, [I64, I64, I64]),
    "tango_spmm_csr_copy_u_ex": (I, [P, P, P, I, P, I64, P, P, P, I, P, I64, I64, I64, I64, I64, P, P, P, SZ, P]),
    "tango_spmm_dense_mask_build": (I, [P, P, I, I64, P, P, P, P, I64, P, P, P, P]),
    "tango_spmm_dense_workspace": (SZ, [P, I64]),
    "tango_spmm_dense_partial": (I, [P, P, I64, I64, P, SZ, P]),
    "tango_probe_mfma_i8": (I, [I, I, I, P, P]),
    "tango_spmm_csr_copy_u_dense": (I, [P, P, P, I64, P, P, P, I, P, I64, P, P, P, SZ, P]),
    "tango_spmm_dense_rest": (I, [P, P, P, I64, P, P, P, I, P, I64, P, SZ, P]),
    "tango_spmm_csr_u_mul_e": (I, [P, P, P, P, P, P, P, I64, I64, I64, I64, I64, I64, P]),
    "tango_spmm_csr_u_mul_e_ex": (I, [P, P, P, P, I, P, P, I, P, P, P, I, I64, I64, I64, I64, I64, I64, I64, P, SZ, P]),
    "tango_spmm_csr_u_mul_e_f32e": (I, [P, P, P, P, I, P, P, I, P, P, P, I, I64, I64, I64, I64, I64, I64, I64, P, SZ, P]),
    "tango_attn_scores_fwd": (I, [P, P, P, P, P, P, P, I64, I64, I64, P]),
    "tango_attn_scores_bwd_workspace": (SZ, [I64, I64, I64]),
    "tango_attn_scores_bwd": (I, [P, P, P, P, P, P, P, P, I64, I64, I64, P, SZ, P]),
    "tango_attn_scores_bwd_acc": (I, [P, P, P, P, P, P, P, P, P, P, I64, I64, I64, P, SZ, P]),
    "tango_spmm_incidence": (I, [P, P, P, P, P, I64, I64, I64, I64, P]),
    "tango_sddmm_dot_i8": (I, [P, P, P, P, P, P, P, P, I64, I64, I64, P]),
    "tango_sddmm_ewise_i8": (I, [I, P, P, P, P, P, P, P, P, I64, I64, P]),
    "tango_sddmm_ewise_f32q": (I, [I, P, P, P, P, P, P, P, I64, I64, I, P]),
    "tango_softmax_xent_workspace": (SZ, [I64]),
    "tango_softmax_xent_f32": (I, [P, I64, P, I64, I64, P, P, I64, P, SZ, P]),
    "tango_batchnorm_workspace": (SZ, [I64, I64]),
    "tango_batchnorm_fwd_f32": (I, [P, P, P, P, P, P, P, P, I64, I64, F, I, P, SZ, P]),
    "tango_batchnorm_bwd_f32": (I, [P, P, P, P, P, P, P, P, P, I64, I64, I, P, SZ, P]),
    "tango_edge_softmax_workspace": (SZ, [I64, I64]),
    "tango_edge_softmax_fwd": (I, [P, P, P, P, I64, I64, I64, F, P, SZ, P]),
    "tango_edge_softmax_fwd_static": (I, [P, P, P, P, I64, I64, I64, F, P]),
    "tango_edge_softmax_fwd_ex": (I, [P, P, P, P, P, P, P, P, P, P, P, P, I64, I64, I64, F, P, SZ, P]),
    "tango_edge_softmax_bwd_ex": (I, [P, P, P, P, P, P, P, P, I64, I64, I64, F, P, SZ, P]),
    "tango_edge_softmax_bwd": (I, [P, P, P, P, P, P, I64, I64, I64, F, P, SZ, P]),
}



class DensePlan(C.Structure):
    """tango_spmm_dense_plan of include/tango_hip.h."""
    _fields_ = [(n, I64) for n in ("rows", "num_src", "dense_rows", "dense_cols", "row_blocks", "num_groups",
                                   "num_groups2", "num_shared")] + \
               [(n, P) for n in ("col_ids", "row_slot", "row_order", "mask_off", "mask", "seg_ptr", "segs", "seg_ptr2", "segs2", "shared_blocks",
                                 "res_indptr", "res_indices")] + \
               [("res_nnz", I64), ("res_max_row", I64)]


ROUND_RNE, ROUND_TRUNC, ROUND_STOCHASTIC = 0, 1, 2
ROUND_MODES = {"rne": ROUND_RNE, "trunc": ROUND_TRUNC, "stochastic": ROUND_STOCHASTIC}
SDDMM_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}

_lib = None


class TangoError(RuntimeError):
    """A C-ABI entry point returned a non-zero status."""


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "libtango_hip.so has not been built (expected at %s); build it with "
                "`python -m tango_amd.build`. There is no CPU fallback." % LIB_PATH)
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status, what):
    if status != 0:
        msg = lib().tango_status_string(status).decode()
        raise TangoError("%s failed: %s (status %d)" % (what, msg, status))
