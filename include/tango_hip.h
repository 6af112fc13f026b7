/*
 * libtango_hip — C ABI of the MI355X (gfx950) quantized-GNN primitive layer.
 *
 * Each entry point replaces one binding of the reference's pybind11 module
 * `cuda_kernels` (cuda/src/cuda.cpp:182-204).  All pointers are DEVICE
 * pointers unless stated otherwise; scales stay device-resident end to end.
 * No entry point allocates, frees or synchronises; every launch goes to the
 * stream the caller passes (a hipStream_t cast to void*; NULL = default
 * stream).  Return value: TANGO_OK or a negative tango_status; the library
 * never aborts the process (the reference calls exit() on any native error,
 * cuda/src/utils.h:4-35).
 *
 * Tensors are dense row-major.  "ld*" arguments are row strides in elements.
 * Index arrays are int64, as in the reference's API; node and edge counts
 * must stay below 2^31.
 */
#ifndef TANGO_HIP_H
#define TANGO_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* tango_stream_t;

enum tango_status {
    TANGO_OK = 0,
    TANGO_ERR_INVALID_ARG = -1, /* null pointer, negative size, misaligned operand */
    TANGO_ERR_UNSUPPORTED = -2, /* unknown op / rounding mode / shape outside the kernels' range */
    TANGO_ERR_LAUNCH = -3,      /* HIP refused the launch */
    TANGO_ERR_WORKSPACE = -4,   /* workspace missing or too small */
    TANGO_ERR_STATIC_LIMIT = -5 /* input beyond the fixed scratch of tango_edge_softmax_fwd_static */
};

enum tango_round_mode {
    TANGO_ROUND_RNE = 0,       /* half-to-even + clamp: cuda/src/quantization.cu:6-15 */
    TANGO_ROUND_TRUNC = 1,     /* toward zero: cuda/src/iterator.h:161 (GEMM fused quantize) */
    TANGO_ROUND_STOCHASTIC = 2 /* floor(x/s + u), u in [0,1): no counterpart in the reference */
};

enum tango_sddmm_op { TANGO_OP_ADD = 0, TANGO_OP_SUB = 1, TANGO_OP_MUL = 2, TANGO_OP_DIV = 3 };

const char* tango_status_string(int status);
/* ABI version; bumped when a signature changes. */
int tango_abi_version(void);

/* Measurement probes (no counterpart in the reference): `blocks` workgroups of four wavefronts.  Shapes 0 and 1:
   `iters` rounds of eight independent chains of one int8 matrix instruction out of registers, 16x16x64
   (2 * 16 * 16 * 64 operations each) and 32x32x32 (2 * 32 * 32 * 32): what the matrix cores of the device sustain.
   Shapes 2, 3, 4: 32x32x32 with the first operand expanded from a word of bits (a shift and a mask per register)
   in front of every 1, 2, 4 instructions.  Shapes 5 .. 8: `iters` rounds of the bit-block kernel's inner loop (64
   instructions of 32x32x32 per wavefront and round, fragments read from 64 KB of LDS): 5 as is, 6 with the LDS store
   instructions of a register-staged chunk and a barrier per round, 7 with the barrier alone, 8 with the chunk
   staged by global-to-LDS loads and the barrier.  sink: device memory, one int (never written in practice); shape 8
   reads the 256 KB that follow its first 256 bytes. */
int tango_probe_mfma_i8(int shape, int iters, int blocks, int* sink, tango_stream_t stream);

/* ------------------------------------------------------------ quantization */

/* get_scale (cuda/src/cuda.cpp:24-25 -> get_scale_impl, quantization.cu:79-93):
   scale_out[0] = max|x| / 127 over n contiguous floats.  scale_out need not be
   initialised.  Unlike the reference every element is covered when n % 4 != 0. */
int tango_absmax_f32(const float* x, int64_t n, float* scale_out, tango_stream_t stream);

/* Accumulating form (no counterpart in the reference): scale_acc[0] = max(scale_acc[0],
   max|x| / 127).  scale_acc must hold 0 or an earlier partial result (any non-negative
   float).  A caller that hands out zero-initialised slots saves the fill launch that
   tango_absmax_f32 spends on its output; several tensors may share one scale. */
int tango_absmax_acc_f32(const float* x, int64_t n, float* scale_acc, tango_stream_t stream);

/* Per-row scales (no counterpart in the reference): scale_out[r] = max_c |x[r,c]| / 127. */
int tango_absmax_rows_f32(const float* x, int64_t rows, int64_t cols, int64_t ldx,
                          float* scale_out, tango_stream_t stream);

/* quantize (cuda/src/cuda.cpp:19-23 -> quantize_impl, quantization.cu:17-43):
   q[i] = clamp(round(x[i] * (1 / scale[0])), -127, 127).  round_mode selects the
   rounding.  For TANGO_ROUND_STOCHASTIC, `noise` (n floats in [0,1), same
   indexing as x) is used when non-null; otherwise Philox4x32-10 keyed by `seed`
   with counter (offset + i) >> 2, word (offset + i) & 3, u = (word >> 8) * 2^-24.
   offset_dev (or NULL): one 64-bit word of device memory whose value is added to `offset` when
   the kernel starts.  A caller that keeps its position in the random stream there and advances it
   with tango_counter_add_u64 draws fresh numbers on every replay of a captured graph, which a
   host-side offset (a constant of the captured launch) cannot; keep its value a multiple of 4. */
int tango_quantize_f32_i8(const float* x, int64_t n, const float* scale, int8_t* q,
                          int round_mode, const float* noise, uint64_t seed, uint64_t offset,
                          const uint64_t* offset_dev, tango_stream_t stream);

/* counter[0] += inc by a one-thread kernel on the stream (no counterpart in the reference): the
   device-side position in the stream of random numbers, see tango_quantize_f32_i8. */
int tango_counter_add_u64(uint64_t* counter, uint64_t inc, tango_stream_t stream);

/* Row-strided quantize with an optionally padded output (no counterpart in the
   reference; lets the SpMM gather aligned rows when cols is odd, e.g. 41):
   q[r, c] for c < cols as above with scale[per_row ? r : 0]; q[r, cols..ldq) = 0.
   Noise / Philox indexing uses the dense index r * cols + c. */
int tango_quantize_rows_f32_i8(const float* x, int64_t rows, int64_t cols, int64_t ldx,
                               const float* scale, int per_row, int8_t* q, int64_t ldq,
                               int round_mode, const float* noise, uint64_t seed,
                               uint64_t offset, tango_stream_t stream);

/* Fused forms of the two calls above for a layer's glue (no counterpart in the
   reference, whose drivers run these steps as separate torch passes,
   evaluation/test_gcn.py:86-94,123-137): every
   element first passes backwards through the activation whose forward output (or any
   tensor of its sign) is mask[r, c] (row stride ldm; when non-null), then is multiplied
   by row_mul[r] (when non-null; one fp32 rounding).  mask_mode 0 (ReLU): x becomes zero
   where mask is not positive.  mask_mode 1 (ELU, mask = the activation's output):
   x becomes x * (mask + 1) where mask is not positive.  mask_mode 2: mask points to 16-bit words,
   ldm words per row, bit c % 16 of word [r, c / 16] set where x is kept, clear where it becomes zero
   (cols % 16 == 0; written by tango_spmm_csr_copy_u_ex's sign_bits).
   tango_absmax_ex_f32 writes scale_out[0] = max|x'*row_mul| / 127 of the elements x' so
   masked and, when colsum_out is non-null, colsum_out[c] = sum_r x'[r, c]
   (not multiplied), reduced in a fixed order.  cols <= 1024.
   accumulate != 0: scale_out[0] already holds 0 or a partial result and is maxed into
   (as tango_absmax_acc_f32); otherwise it need not be initialised.
   workspace: tango_absmax_ex_workspace(rows, cols, colsum_out != NULL) bytes. */
size_t tango_absmax_ex_workspace(int64_t rows, int64_t cols, int want_colsum);
int tango_absmax_ex_f32(const float* x, int64_t rows, int64_t cols, int64_t ldx, const float* row_mul,
                        const void* mask, int64_t ldm, int mask_mode, float* scale_out, int accumulate,
                        float* colsum_out, void* workspace, size_t workspace_bytes, tango_stream_t stream);
int tango_quantize_rows_ex_f32_i8(const float* x, int64_t rows, int64_t cols, int64_t ldx,
                                  const float* row_mul, const void* mask, int64_t ldm, int mask_mode,
                                  const float* scale, int per_row, int8_t* q, int64_t ldq,
                                  int round_mode, const float* noise, uint64_t seed,
                                  uint64_t offset, const uint64_t* offset_dev, tango_stream_t stream);

/* tango_quantize_rows_ex_f32_i8 on a dense matrix (no padding in x, q or the mask) that also returns the column
   sums of the masked input before the row multiplier, colsum_out[c] = sum_r masked(x[r, c]): the bias gradient of a
   fused "mask, sum, scale rows, quantize" backward step (cuda/QLinear.py:46 with the glue of
   evaluation/test_gcn.py:123-137) out of the pass that quantizes, for callers that already hold the scale.  Added in
   a fixed order.  Only for cols a multiple of 4 with 256 % (cols / 4) == 0 (a multiple of 16 with sign-word masks),
   x 16-byte and q 4-byte aligned: TANGO_ERR_UNSUPPORTED otherwise, before anything is launched.
   workspace: tango_quantize_rows_colsum_workspace(rows, cols) bytes. */
size_t tango_quantize_rows_colsum_workspace(int64_t rows, int64_t cols);
int tango_quantize_rows_colsum_f32_i8(const float* x, int64_t rows, int64_t cols, const float* row_mul,
                                      const void* mask, int mask_mode, const float* scale, int8_t* q,
                                      int round_mode, const float* noise, uint64_t seed, uint64_t offset,
                                      const uint64_t* offset_dev, float* colsum_out, void* workspace,
                                      size_t workspace_bytes, tango_stream_t stream);

/* transpose_quant (cuda/src/cuda.cpp:27-33 -> transpose_quant_impl,
   quantization.cu:95-167): x[nrow, ncol] fp32 -> out[ncol, nrow] int8,
   half-to-even, clamped to +-127. */
int tango_transpose_quant_f32_i8(const float* x, int64_t nrow, int64_t ncol, const float* scale,
                                 int8_t* out, tango_stream_t stream);

/* -------------------------------------------------------------------- GEMM */

/* All GEMM entry points take a caller-provided workspace (device memory,
   16-byte aligned) whose size the matching *_workspace() query returns; the
   library uses it to re-pack the small operand into aligned, zero-padded rows.
   A row stride of an fp32 output that exceeds its column count is padding, not a
   view into a wider matrix: the kernels may store zeros into the columns between
   the last one and the next multiple of 16 (never at or past the stride). */

/* QGEMM_forward (cuda/src/cuda.cpp:11-17 -> QGEMM_forward_impl,
   QGEMM_forward.cu:125-157): quantizes X[M,K] and W[N,K] with scaleX / scaleW
   (round_mode; the reference truncates, cuda/src/iterator.h:161), stores the
   int8 copies to Xq[M,K] (row stride ldxq >= K; bytes K..ldxq of each row are
   zeroed) and Wq[N,K] (dense), and writes
   Y[m,n] = (scaleX*scaleW) * float(sum_k Xq[m,k]*Wq[n,k]) (+ bias[n]).
   bias may be NULL.  scaleY may be NULL; otherwise scaleY[0] = max|Y| / 127
   (the fused reduction of cuda/src/epilogue.h:105-626); it need not be
   initialised.  K is arbitrary (the reference requires K % 4 == 0); rows of Xq
   padded to a multiple of 16 bytes take the fast path.  round_mode: TANGO_ROUND_RNE or
   TANGO_ROUND_TRUNC, used for X and W alike; TANGO_ROUND_STOCHASTIC (for which this
   signature carries no seed) returns TANGO_ERR_UNSUPPORTED before anything is launched. */
size_t tango_qgemm_fwd_workspace(int64_t M, int64_t N, int64_t K);
int tango_qgemm_fwd(float* Y, int64_t ldy, const float* X, int64_t ldx, int8_t* Xq, int64_t ldxq,
                    const float* W, int64_t ldw, int8_t* Wq, const float* bias, float* scaleY,
                    const float* scaleX, const float* scaleW, int64_t M, int64_t N, int64_t K,
                    int round_mode, void* workspace, size_t workspace_bytes,
                    tango_stream_t stream);

/* As tango_qgemm_fwd, with row m of X multiplied by x_row_mul[m] before it is
   quantized (the "feat * out_deg^-1/2" of evaluation/test_gcn.py:86-94 folded
   into the quantize pass; scaleX must then be the scale of the multiplied X).
   X may be NULL (x_row_mul must then be NULL too): Xq is then an input that already
   holds X quantized with scaleX, e.g. because several layers consume the same X
   (the q / k / v projections of evaluation/test_HGT.py:44-50) and one quantize
   pass serves them all; W is still quantized here. */
int tango_qgemm_fwd_ex(float* Y, int64_t ldy, const float* X, int64_t ldx, const float* x_row_mul,
                       int8_t* Xq, int64_t ldxq, const float* W, int64_t ldw, int8_t* Wq,
                       const float* bias, float* scaleY, const float* scaleX, const float* scaleW,
                       int64_t M, int64_t N, int64_t K, int round_mode, void* workspace,
                       size_t workspace_bytes, tango_stream_t stream);

/* Forward linear whose output is read only by another quantized op (the first of two chained
   QLinear layers, evaluation/test_HGT.py:51-55): instead of the fp32 Y that cuda/QLinear.py:30-36
   stores and the next layer's quantize reads back, the int8 Yq = quantize(Y, scaleY) and
   scaleY[0] = max|Y| / 127 themselves.  The product is formed twice (first for its absmax, then
   rounded with it); same bits as tango_qgemm_fwd followed by a quantize pass.  Xq is the
   already quantized input (16-byte aligned rows); K <= 256, round_mode RNE or TRUNC (used for W
   and for Yq), else TANGO_ERR_UNSUPPORTED before anything is launched.  Workspace as
   tango_qgemm_fwd. */
int tango_qgemm_fwd_q8(int8_t* Yq, int64_t ldyq, float* scaleY, const int8_t* Xq, int64_t ldxq,
                       const float* W, int64_t ldw, int8_t* Wq, const float* bias, const float* scaleX,
                       const float* scaleW, int64_t M, int64_t N, int64_t K, int round_mode,
                       void* workspace, size_t workspace_bytes, tango_stream_t stream);

/* Integer GEMM on operands that are already int8 (no counterpart in the
   reference, whose forward always re-quantizes; same epilogue as above):
   Y[m,n] = (sA*sB) * float(sum_k A[m,k]*B[n,k]) (+ bias[n]), optional scaleY. */
size_t tango_qgemm_i8_nt_workspace(int64_t M, int64_t N, int64_t K);
int tango_qgemm_i8_nt(float* Y, int64_t ldy, const int8_t* A, int64_t lda, const int8_t* B,
                      int64_t ldb, const float* bias, float* scaleY, const float* sA,
                      const float* sB, int64_t M, int64_t N, int64_t K, void* workspace,
                      size_t workspace_bytes, tango_stream_t stream);

/* QGEMM_backward_gradX (cuda/src/cuda.cpp:90-98 -> QGEMM_backward.cu:21-48):
   dX[M,K] = (s_dY*s_W) * float(sum_n dYq[m,n] * Wq[n,k]). */
size_t tango_qgemm_bwd_dx_workspace(int64_t M, int64_t N, int64_t K);
int tango_qgemm_bwd_dx(float* dX, int64_t lddx, const int8_t* dYq, int64_t lddy,
                       const int8_t* Wq, int64_t ldw, const float* s_dY, const float* s_W,
                       int64_t M, int64_t N, int64_t K, void* workspace, size_t workspace_bytes,
                       tango_stream_t stream);

/* As tango_qgemm_bwd_dx, with row m of the result multiplied by row_scale[m]
   (the backward of the folded row multiplier above).  accumulate != 0: the result is added to
   what dX holds, for an input that feeds several layers (the sum autograd forms of their input
   gradients, evaluation/test_HGT.py:51-53, without the separate additions). */
int tango_qgemm_bwd_dx_ex(float* dX, int64_t lddx, const int8_t* dYq, int64_t lddy,
                          const int8_t* Wq, int64_t ldw, const float* s_dY, const float* s_W,
                          const float* row_scale, int accumulate, int64_t M, int64_t N, int64_t K,
                          void* workspace, size_t workspace_bytes, tango_stream_t stream);

/* tango_qgemm_bwd_dx_ex that also finds the scale its consumer needs when that consumer takes dX back through
   a ReLU and multiplies its rows (the aggregation in front of this layer, cuda/SPMM.py:15-24 with the layer glue of
   evaluation/test_gcn.py:123-137 folded in): masked_scale_out[0] = max |dX[m, k] * mask_mul[m]| / 127 over the
   elements whose sign bit is set (bit k % 16 of the 16-bit word mask_bits[m * ldmask + k / 16]; mask_mul may be
   NULL), from the epilogue that stores dX instead of a pass over it.  Only for K (columns of dX) in {32, 64, 128,
   256}, N <= 256, dX rows 16-byte aligned, dYq rows readable in 4-byte pieces, ldmask even and mask_bits 4-byte
   aligned: TANGO_ERR_UNSUPPORTED otherwise, before anything is launched (call tango_qgemm_bwd_dx_ex and
   tango_absmax_ex_f32 then). */
int tango_qgemm_bwd_dx_masked(float* dX, int64_t lddx, const int8_t* dYq, int64_t lddy, const int8_t* Wq,
                              int64_t ldw, const float* s_dY, const float* s_W, const float* row_scale,
                              const uint16_t* mask_bits, int64_t ldmask, const float* mask_mul,
                              float* masked_scale_out, int64_t M, int64_t N, int64_t K, void* workspace,
                              size_t workspace_bytes, tango_stream_t stream);

/* QGEMM_backward_gradW (cuda/src/cuda.cpp:100-108 -> QGEMM_backward.cu:50-113):
   dW[N,K] = (s_dY*s_X) * float(sum_m dYq[m,n] * Xq[m,k]), int32 accumulation.
   The reduction over M is split over workgroups whose int32 partials are summed
   exactly, so the result does not depend on the split.  workspace holds those
   partials: tango_qgemm_bwd_dw_workspace(M,N,K) bytes. */
size_t tango_qgemm_bwd_dw_workspace(int64_t M, int64_t N, int64_t K);
int tango_qgemm_bwd_dw(float* dW, int64_t lddw, const int8_t* dYq, int64_t lddy,
                       const int8_t* Xq, int64_t ldx, const float* s_dY, const float* s_X,
                       int64_t M, int64_t N, int64_t K, void* workspace, size_t workspace_bytes,
                       tango_stream_t stream);

/* QgemmNT / QgemmNN / QgemmTN (cuda/src/cuda.cpp:75-88 -> Qgemm_impl.cu:6-125):
   quantize fp32 A and B (absmax scale, half-to-even), int8 GEMM, dequantize.
   A is [m,k] (or [k,m] when trans_a), B is [k,n] (or [n,k] when trans_b),
   C is [m,n].  workspace: tango_qgemm_legacy_workspace(m,n,k) bytes. */
size_t tango_qgemm_legacy_workspace(int64_t m, int64_t n, int64_t k);
int tango_qgemm_legacy(float* C, const float* A, const float* B, int64_t m, int64_t n, int64_t k,
                       int trans_a, int trans_b, void* workspace, size_t workspace_bytes,
                       tango_stream_t stream);

/* -------------------------------------------------------------------- SpMM */

/* csr_SPMM (cuda/src/cuda.cpp:110-117 -> cusp_SPMM_csr_impl, SPMM.cu:23-68):
   out[r, f] = scale[0] * float(sum_{p in [indptr[r], indptr[r+1])} feat[indices[p], f])
   for r < rows, f < F.  feat has num_src rows of stride ldf bytes (ldf >= F);
   out is [rows, F] dense; nnz = indptr[rows].  int32 accumulation. */
int tango_spmm_csr_copy_u(float* out, const int64_t* indptr, const int64_t* indices,
                          const int8_t* feat, int64_t ldf, const float* scale, int64_t rows,
                          int64_t num_src, int64_t nnz, int64_t F, tango_stream_t stream);

/* As tango_spmm_csr_copy_u with the layer glue that follows the aggregation in
   evaluation/test_gcn.py:123-137 folded into the epilogue, in this order and with
   one fp32 rounding each: y = scale * float(sum); y *= row_scale[r] (if non-null);
   y += bias[f] (if non-null); then relu = 1: y = max(y, 0); relu = 2: y = y > 0 ? y : exp(y) - 1
   (ELU, alpha 1; hardware exponential, absolute error about 1e-7); relu = 0: nothing.
   idx_bits: 64 (int64 indices, as the reference passes them) or 32 (a one-time int32
   copy of the column indices made by the caller: half the index traffic).
   max_row_nnz: an upper bound of the longest row if the caller knows one (a graph
   object usually does), else 0; it only lets the library skip the launches that
   exist for hub rows when there is none.
   workspace (tango_spmm_workspace(rows, nnz, F) bytes, 16-byte aligned, contents
   arbitrary) or NULL.  With it, on graphs whose rows average fewer than 64 slots the
   work is cut by slots (256 per wavefront) instead of rows, rows cut by such a boundary
   leaving int32 partial rows in the workspace that a second launch adds up; on denser
   graphs hub rows (thousands of slots and far above the average) are cut over many
   workgroups whose int32 partial sums are added into the output row with integer
   atomics.  Integer sums are exact in any order, so the result is the same either way.
   W in the size query: bytes summed per gathered row (F here, H * F for u_mul_e).
   sign_bits (or NULL; needs F % 16 == 0 and 16-byte aligned feat rows): [rows, F / 16] 16-bit words that
   receive bit c % 16 of word [r, c / 16] = (out[r, c] > 0), the mask the backward pass of the ReLU needs,
   in 1/32 of the bytes of out (mask_mode 2 of tango_absmax_ex_f32 / tango_quantize_rows_ex_f32_i8).
   scale_out (or NULL; needs the workspace): must hold 0 (or an earlier partial maximum) on entry and receives
   max(scale_out[0], max |out[r, c] * absmax_row_mul[r]| / 127) (absmax_row_mul NULL: no multiplier): the scale the
   quantizer of the next op needs, formed where out is produced instead of by a pass over out (the reference's only
   fused reduction of this kind sits in its GEMM epilogue, cuda/src/epilogue.h:105-626).  The value equals
   tango_absmax_ex_f32(out, row_mul = absmax_row_mul) bit for bit. */
size_t tango_spmm_workspace(int64_t rows, int64_t nnz, int64_t W);
int tango_spmm_csr_copy_u_ex(float* out, const int64_t* indptr, const void* indices, int idx_bits,
                             const int8_t* feat, int64_t ldf, const float* scale,
                             const float* row_scale, const float* bias, int relu, uint16_t* sign_bits,
                             int64_t rows, int64_t num_src, int64_t nnz, int64_t F, int64_t max_row_nnz,
                             const float* absmax_row_mul, float* scale_out,
                             void* workspace, size_t workspace_bytes, tango_stream_t stream);

/* csr_SPMM (cuda/src/cuda.cpp:110-117 -> SPMM.cu:23-68) on a graph whose heavy rows and heavy columns
   form nearly dense blocks (power-law graphs): the adjacency is split once per graph into
     - bit blocks: with rows and columns ranked by falling slot count, row block b (256 consecutive row
       ranks) owns the cells (row, column rank < extent[b]), extent a multiple of 256; a set bit is one
       edge.  These are multiplied with the int8 features on the matrix cores (0/1 bytes x int8 -> int32);
     - the rest: an ordinary CSR (res_indptr, res_indices) holding every slot not represented by a bit
       (outside the blocks, or a repeated edge whose bit was already set), gathered as in
       tango_spmm_csr_copy_u_ex, whose epilogue adds the blocks' int32 partial sums.
   Integer sums are exact in any order, so out equals tango_spmm_csr_copy_u_ex on the whole CSR bit for bit.
   All arrays are device memory and belong to the caller.
   mask layout: row block b starts at dword mask_off[b]; unit u (columns 256 u .. 256 u + 255 by rank), row
   group g (64 rows), half q (k-steps 4 q .. 4 q + 3 of 32 columns each), lane l, k-step s4 is dword
   (((u * 4 + g) * 2 + q) * 64 + l) * 4 + s4; its bit 8 b + 4 h + w is the cell (row 64 g + 32 h + l % 32 of
   the block, column 256 u + 32 (4 q + s4) + 16 (l / 32) + 4 w + b).
   segs: num_segments x 4 int32 (row block, first unit, units, 1 if other segments add into the same
   row block); workgroup i of num_groups processes segments seg_ptr[i] .. seg_ptr[i + 1] - 1.  Two such
   tables, each covering every unit of every row block once: (num_groups, seg_ptr, segs) for features wider
   than 128 columns, where two workgroups share a group's segments (one half of the columns each), and
   (num_groups2, seg_ptr2, segs2), usually twice as many groups, for narrower features.
   shared_blocks lists the row blocks with shared segments in either table (zeroed before the product). */
typedef struct tango_spmm_dense_plan {
    int64_t rows;        /* output rows of the adjacency */
    int64_t num_src;     /* rows of the gathered matrix */
    int64_t dense_rows;  /* rows covered by row blocks: 256 * row_blocks */
    int64_t dense_cols;  /* widest extent, a multiple of 256 */
    int64_t row_blocks;
    int64_t num_groups;
    int64_t num_groups2;
    int64_t num_shared;
    const int32_t* col_ids;        /* [dense_cols] column rank -> row of the gathered matrix, -1 = none */
    const int32_t* row_slot;       /* [rows] output row -> its row rank if below dense_rows, else -1 */
    const int32_t* row_order;      /* [rows] a permutation of the output rows, or NULL for the identity: the order the
                                      gather kernel takes rows in, by falling slot count (the rows that share a
                                      wavefront are about equally long, whatever the numbering of the nodes; with
                                      NULL the kernel gives every row a wavefront of its own) */
    const int64_t* mask_off;       /* [row_blocks] */
    const uint32_t* mask;
    const int32_t* seg_ptr;        /* [num_groups + 1] */
    const int32_t* segs;           /* [seg_ptr[num_groups]][4] */
    const int32_t* seg_ptr2;       /* [num_groups2 + 1] */
    const int32_t* segs2;          /* [seg_ptr2[num_groups2]][4] */
    const int32_t* shared_blocks;  /* [num_shared] */
    const int64_t* res_indptr;     /* [rows + 1] */
    const int32_t* res_indices;    /* [res_nnz] */
    int64_t res_nnz;
    int64_t res_max_row;           /* longest row of the rest, 0 if unknown */
} tango_spmm_dense_plan;

/* Sets the bits of a plan's mask (which the caller has zeroed) from the adjacency (indptr, indices;
   idx_bits 32 or 64) and says which slots remain for the rest: keep[p] = 0 when slot p is now a bit of
   the mask, 1 when it stays (outside the blocks, or its bit was already set by an equal edge);
   kept[r] = number of kept slots of row r.  row_rank / col_rank: rank of every row / gathered row
   (int32); extent_cols[b]: extent of row block b in columns.  One-time graph preprocessing
   (extends cuda/util.py:5-11). */
int tango_spmm_dense_mask_build(const int64_t* indptr, const void* indices, int idx_bits, int64_t rows,
                                const int32_t* row_rank, const int32_t* col_rank,
                                const int32_t* extent_cols, const int64_t* mask_off, int64_t row_blocks,
                                uint32_t* mask, uint8_t* keep, int32_t* kept, tango_stream_t stream);

/* out as tango_spmm_csr_copy_u_ex computes it on the whole adjacency (same epilogue arguments, same scale output).
   Needs 16-byte aligned feat rows (ldf % 16 == 0, ceil16(F) <= ldf) and F <= 256, else
   TANGO_ERR_UNSUPPORTED (callers then use tango_spmm_csr_copy_u_ex on the whole CSR).
   workspace: tango_spmm_dense_workspace(plan, F) bytes, 256-byte aligned. */
size_t tango_spmm_dense_workspace(const tango_spmm_dense_plan* plan, int64_t F);
/* The first part of tango_spmm_csr_copy_u_dense alone (staging, zeroing, the matrix product of the bit blocks into
   the workspace), for measurements: its time subtracted from the whole call's is the gather kernel's. */
int tango_spmm_dense_partial(const tango_spmm_dense_plan* plan, const int8_t* feat, int64_t ldf, int64_t F,
                             void* workspace, size_t workspace_bytes, tango_stream_t stream);
int tango_spmm_csr_copy_u_dense(float* out, const tango_spmm_dense_plan* plan, const int8_t* feat,
                                int64_t ldf, const float* scale, const float* row_scale,
                                const float* bias, int relu, uint16_t* sign_bits, int64_t F,
                                const float* absmax_row_mul, float* scale_out,
                                void* workspace, size_t workspace_bytes, tango_stream_t stream);
/* The second part alone: the gather kernel on the rest of the adjacency, whose epilogue adds the partial sums that a
   preceding tango_spmm_dense_partial (same plan, feat, F and workspace) left in the workspace.  The two calls in
   a row give what tango_spmm_csr_copy_u_dense gives; for measurements (this launch is the dominant kernel of the
   benchmark epoch and can be timed by itself).  No counterpart in the reference. */
int tango_spmm_dense_rest(float* out, const tango_spmm_dense_plan* plan, const int8_t* feat,
                          int64_t ldf, const float* scale, const float* row_scale,
                          const float* bias, int relu, uint16_t* sign_bits, int64_t F,
                          void* workspace, size_t workspace_bytes, tango_stream_t stream);

/* multi_cusparse_SPMM (cuda/src/cuda.cpp:119-158 -> SPMM.cu:70-194):
   out[r,h,f] = scale[0] * float(sum_p evals[h, d, e(p)] * feat[indices[p], h, f]),
   d = 0 when D == 1 (broadcast edge value) else d = f (D == F, element-wise).
   feat is [num_src, H, F] int8, evals is [H, D, nnz] int8, out is [rows, H, F].
   e(p) = p when edge_ids is NULL (evals already in CSR slot order, as after the
   index_select of cuda/kernels.py:133-135), else edge_ids[p] (that gather fused). */
int tango_spmm_csr_u_mul_e(float* out, const int64_t* indptr, const int64_t* indices,
                           const int64_t* edge_ids, const int8_t* feat, const int8_t* evals,
                           const float* scale, int64_t rows, int64_t num_src, int64_t H,
                           int64_t F, int64_t D, int64_t nnz, tango_stream_t stream);

/* As tango_spmm_csr_u_mul_e with a choice of layout for the edge values (no
   counterpart in the reference): edge_major != 0 means evals is [nnz, H, D] (what
   quantizing the [nnz, H, D] fp32 edge tensor in place yields, no transpose pass).
   With the slot->edge permutation fused, the H * D bytes of a gathered edge then
   come from one cache sector instead of H * D scattered ones.  bias (H * F floats or
   NULL) is added after dequantization ("rst + bias", evaluation/test_gat.py:160-162);
   act then applies the layer's activation (evaluation/test_gat.py:164-165) with the codes
   of tango_spmm_csr_copy_u_ex's relu: 0 none, 1 ReLU, 2 ELU.
   scale2 (or NULL): the dequantization scale is scale[0] * scale2[0] (the scales of the
   node features and of the edge values, multiplied by a torch op in cuda/SPMM.py:44).
   idx_bits: width of the entries of indices and edge_ids, 64 or 32; max_row_nnz and
   workspace as for tango_spmm_csr_copy_u_ex. */
int tango_spmm_csr_u_mul_e_ex(float* out, const int64_t* indptr, const void* indices,
                              const void* edge_ids, int idx_bits, const int8_t* feat, const int8_t* evals,
                              int edge_major, const float* scale, const float* scale2, const float* bias,
                              int act, int64_t rows, int64_t num_src, int64_t H, int64_t F, int64_t D, int64_t nnz,
                              int64_t max_row_nnz, void* workspace, size_t workspace_bytes,
                              tango_stream_t stream);

/* As tango_spmm_csr_u_mul_e_ex with the edge values still in fp32 (no counterpart in the reference, which
   quantizes them in a pass of its own, cuda/SPMM.py:41-43): each value is rounded to int8 as it is loaded,
   half to even with the scale scale_e[0] (required; e.g. from tango_edge_softmax_fwd_ex), so the result is
   what quantizing evals_f32 first and calling tango_spmm_csr_u_mul_e_ex with scale2 = scale_e gives, bit for
   bit, without that pass and the int8 copy. */
int tango_spmm_csr_u_mul_e_f32e(float* out, const int64_t* indptr, const void* indices,
                                const void* edge_ids, int idx_bits, const int8_t* feat, const float* evals_f32,
                                int edge_major, const float* scale, const float* scale_e, const float* bias,
                                int act, int64_t rows, int64_t num_src, int64_t H, int64_t F, int64_t D, int64_t nnz,
                                int64_t max_row_nnz, void* workspace, size_t workspace_bytes,
                                tango_stream_t stream);

/* incidence_SPMM (cuda/src/cuda.cpp:160-167 -> incidence_SPMM_impl, SPMM.cu:259-303):
   out[v, f] = scale[0] * float(sum_{i: node_ids[i] == v} E[edge_ids[i], f]).
   (node_ids, edge_ids) are the COO rows of the incidence matrix and must be
   sorted by node id, which cuda/util.py:6-7 (coalesce) guarantees. */
int tango_spmm_incidence(float* out, const int64_t* node_ids, const int64_t* edge_ids,
                         const int8_t* E, const float* scale, int64_t num_nodes, int64_t nnz,
                         int64_t num_edges, int64_t F, tango_stream_t stream);

/* ------------------------------------------------------------------- SDDMM */

/* mySDDMM_int8 with op "dot" (cuda/src/cuda.cpp:41-47 -> SDDMM.cu:8-47,124-150):
   out[e,h] = (sU*sV) * float(sum_d U[src[e],h,d] * V[dst[e],h,d]).
   U, V are [*, H, D] int8.  scale_out may be NULL; otherwise
   scale_out[0] = max|out| / 127 (need not be initialised). */
int tango_sddmm_dot_i8(float* out, float* scale_out, const int64_t* src, const int64_t* dst,
                       const int8_t* U, const int8_t* V, const float* sU, const float* sV,
                       int64_t num_edges, int64_t H, int64_t D, tango_stream_t stream);

/* mySDDMM_int8 with op add/sub/mul/div (SDDMM.cu:49-100,152-175):
   out[e,t] = OP(float(U[src[e],t]) * sU, float(V[dst[e],t]) * sV), t < T. */
int tango_sddmm_ewise_i8(int op, float* out, float* scale_out, const int64_t* src,
                         const int64_t* dst, const int8_t* U, const int8_t* V, const float* sU,
                         const float* sV, int64_t num_edges, int64_t T, tango_stream_t stream);

/* The same with fp32 U, V quantized as they are loaded (round_mode TANGO_ROUND_RNE or
   TANGO_ROUND_TRUNC, scales sU, sV): what sddmm_u_add_v's two quantize calls followed by
   mySDDMM_int8 compute (cuda/SDDMM.py:13-18), bit for bit, without the int8 copies. */
int tango_sddmm_ewise_f32q(int op, float* out, const int64_t* src, const int64_t* dst, const float* U,
                           const float* V, const float* sU, const float* sV, int64_t num_edges, int64_t T,
                           int round_mode, tango_stream_t stream);

/* ------------------------------------------------------------ edge softmax */

/* LeakyReLU(slope) followed by softmax over the in-edges of every destination
   node (dgl.ops.edge_softmax as called at evaluation/test_gat.py:144-146; DGL
   is not part of the reference tree).  e and a are [num_edges, H] in edge-id
   order; indptr/edge_ids describe the destination-major CSR (adj_csc);
   edge_ids may be NULL for the identity.  slope = 1 gives the plain softmax.
   num_edges = indptr[rows].  The work is cut by edge slots (256 per wavefront), so hub
   destinations cost no more per edge than the others; rows cut by a slot boundary
   are combined through workspace (tango_edge_softmax_workspace(num_edges, H) bytes,
   16-byte aligned; contents need not be initialised).  With workspace = NULL a thread
   walks each (destination, head) alone: same results up to the fp32 summation order,
   slow for hubs. */
size_t tango_edge_softmax_workspace(int64_t num_edges, int64_t H);
int tango_edge_softmax_fwd(float* a, const float* e, const int64_t* indptr,
                           const int64_t* edge_ids, int64_t rows, int64_t num_edges, int64_t H,
                           float slope, void* workspace, size_t workspace_bytes,
                           tango_stream_t stream);
/* tango_edge_softmax_fwd for callers that cannot allocate (code under HIP graph capture, tight
   serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same
   kernels and same results as tango_edge_softmax_fwd with a workspace, but the per-span records live
   in a fixed array of TANGO_EDGE_SOFTMAX_STATIC_BYTES inside the library's device image (one copy
   per GPU, held until the process ends) and no memory is allocated or freed by the call.
   Inputs with tango_edge_softmax_workspace(num_edges, H) > TANGO_EDGE_SOFTMAX_STATIC_BYTES are
   rejected with TANGO_ERR_STATIC_LIMIT before anything is launched (at H = 8 a span of 128 slots
   takes 160 bytes: the limit is about 3.3 million edges).  All calls on one GPU share the array.  Calls on
   one stream are ordered by the stream; a call on another stream than the previous call's first waits
   (hipStreamWaitEvent on an event created once per GPU at the first call) for the previous call's kernels, so eager
   calls from several streams or threads are serialised on the GPU rather than racing.  Under stream capture no event
   is used: graphs that contain this call and replay at the same time on one GPU still race, which is the
   caller's to order. */
#define TANGO_EDGE_SOFTMAX_STATIC_BYTES (4u << 20)
int tango_edge_softmax_fwd_static(float* a, const float* e, const int64_t* indptr,
                                  const int64_t* edge_ids, int64_t rows, int64_t num_edges, int64_t H,
                                  float slope, tango_stream_t stream);

/* The attention block's forms of the two calls (no counterpart in the reference, where SDDMM, LeakyReLU, DGL's
   edge softmax, get_scale and quantize are separate passes, evaluation/test_gat.py:141-151, cuda/SPMM.py:39-43).
   Forward: e may be NULL when el, er [num_src / rows, H] fp32, their scales s_el, s_er and the edge list
   (src, dst) in edge-id order are given: the logits are then formed on the fly,
   e[edge, h] = q(el[src, h]) * s_el + q(er[dst, h]) * s_er with q the half-to-even int8 rounding, the values
   tango_sddmm_ewise_f32q(add) would have written, and never reach memory.  scale_a (or NULL): receives
   max(a) / 127, what the quantizer of a needs (it need not be initialised).  sign_out (or NULL):
   [num_edges, ceil(H / 8)] bytes in the destination-major slot order, bit h % 8 of byte [slot, h / 8] = (e > 0),
   all the backward pass needs of e.  Backward: e or sign_in (those bytes) supplies LeakyReLU's derivative
   (neither is needed for slope 1); scale_de as scale_a, for max|de| / 127.  Both need the workspace. */
int tango_edge_softmax_fwd_ex(float* a, float* scale_a, uint8_t* sign_out, const float* e, const float* el,
                              const float* er, const float* s_el, const float* s_er, const int64_t* src,
                              const int64_t* dst, const int64_t* indptr, const int64_t* edge_ids, int64_t rows,
                              int64_t num_edges, int64_t H, float slope, void* workspace, size_t workspace_bytes,
                              tango_stream_t stream);
int tango_edge_softmax_bwd_ex(float* de, float* scale_de, const float* a, const float* da, const float* e,
                              const uint8_t* sign_in, const int64_t* indptr, const int64_t* edge_ids, int64_t rows,
                              int64_t num_edges, int64_t H, float slope, void* workspace, size_t workspace_bytes,
                              tango_stream_t stream);

/* de = dLeaky(e) * a * (da - sum_{same dst} a*da).  e may be NULL when slope is 1 (plain softmax: it is not read). */
int tango_edge_softmax_bwd(float* de, const float* a, const float* da, const float* e,
                           const int64_t* indptr, const int64_t* edge_ids, int64_t rows,
                           int64_t num_edges, int64_t H, float slope, void* workspace,
                           size_t workspace_bytes, tango_stream_t stream);

/* ------------------------------------------------------ GAT attention logits */

/* el[n,h] = sum_d feat[n,h,d] * attn_l[h,d], er likewise with attn_r: the two
   broadcast-multiply + sum lines of the GAT layer (evaluation/test_gat.py:135-137),
   torch ops in the reference, in one read of feat.  fp32.  scale_el / scale_er (both or
   neither): pre-zeroed slots that receive max|el| / 127 and max|er| / 127 (what get_scale
   computes in a pass of its own, cuda/kernels.py:26-27, when sddmm_u_add_v quantizes the
   two, cuda/SDDMM.py:13-17). */
int tango_attn_scores_fwd(float* el, float* er, float* scale_el, float* scale_er, const float* feat,
                          const float* attn_l, const float* attn_r, int64_t n, int64_t H, int64_t D,
                          tango_stream_t stream);

/* Backward of the above: dfeat[n,h,d] = del[n,h]*attn_l[h,d] + der[n,h]*attn_r[h,d],
   dattn_l[h,d] = sum_n del[n,h]*feat[n,h,d], dattn_r likewise; the sums over n are
   reduced in a fixed order.  H <= 256.  workspace: tango_attn_scores_bwd_workspace bytes. */
size_t tango_attn_scores_bwd_workspace(int64_t n, int64_t H, int64_t D);
int tango_attn_scores_bwd(float* dfeat, float* dattn_l, float* dattn_r, const float* del,
                          const float* der, const float* feat, const float* attn_l,
                          const float* attn_r, int64_t n, int64_t H, int64_t D, void* workspace,
                          size_t workspace_bytes, tango_stream_t stream);

/* The same with the gradient feat receives from its other consumer folded in: feat feeds both the logits and
   the aggregation (evaluation/test_gat.py:135-137 and :151), so autograd adds the two gradients of feat in a
   pass of its own and the layer that produced feat then scans the sum for its scale (cuda/QLinear.py:37-39,
   cuda/kernels.py:26-27).  Here dfeat = addend + (del*attn_l + der*attn_r), the very sum of that addition
   (same operands, one rounding), and *scale_out (a slot holding 0) receives max|dfeat| / 127.  addend
   [n, H, D] must not overlap dfeat.  Same workspace as tango_attn_scores_bwd. */
int tango_attn_scores_bwd_acc(float* dfeat, float* dattn_l, float* dattn_r, float* scale_out, const float* addend,
                              const float* del, const float* der, const float* feat, const float* attn_l,
                              const float* attn_r, int64_t n, int64_t H, int64_t D, void* workspace,
                              size_t workspace_bytes, tango_stream_t stream);

/* -------------------------------------------------------------------- loss */

/* Softmax cross-entropy with mean reduction and its gradient in one pass (no
   counterpart in the reference's native code: its drivers call torch's
   F.cross_entropy, evaluation/test_gcn.py:256).  logits [rows, classes] fp32 (row
   stride ld), labels int64 [rows]; loss_out[0] = mean_r(-log softmax(logits[r])[labels[r]]),
   grad_out[r, c] = (softmax(logits[r])[c] - (c == labels[r])) / rows.  classes <= 256.
   The loss is reduced in a fixed order.  workspace: tango_softmax_xent_workspace(rows) bytes. */
size_t tango_softmax_xent_workspace(int64_t rows);
int tango_softmax_xent_f32(const float* logits, int64_t ld, const int64_t* labels, int64_t rows,
                           int64_t classes, float* loss_out, float* grad_out, int64_t ldg,
                           void* workspace, size_t workspace_bytes, tango_stream_t stream);

/* ------------------------------------------------------- batch normalisation */

/* Training-mode batch normalisation over the rows of x [rows, cols] fp32 (row stride
   cols), with the ReLU that follows it folded in (no counterpart in the reference's
   native code: its arxiv drivers call torch.nn.BatchNorm1d and then the activation,
   evaluation/arxiv_gat.py:376-448, evaluation/arxiv_gcn.py:156-209).
     mean[c] = mean_r x[r, c], var[c] = mean_r (x[r, c] - mean[c])^2 (biased),
     rstd[c] = 1 / sqrt(var[c] + eps),
     y[r, c] = (x[r, c] - mean[c]) * (rstd[c] * gamma[c]) + beta[c], max(., 0) if relu != 0.
   scale_y (may be NULL) receives max|y| / 127.  The backward takes the incoming gradient
   through the ReLU (the forward's sign, recomputed from x) and returns
     dbeta[c] = sum_r dy'[r, c], dgamma[c] = sum_r dy'[r, c] * xhat[r, c],
     dx[r, c] = rstd[c] * gamma[c] * (dy'[r, c] - dbeta[c] / rows - xhat[r, c] * dgamma[c] / rows),
   xhat = (x - mean) * rstd.  cols <= 2048 (TANGO_ERR_UNSUPPORTED otherwise); rows are read 16, 8 or 4 bytes
   per lane, the widest that cols and the alignment of x / y / dy / dx allow.  All sums run in a fixed order.
   workspace: tango_batchnorm_workspace(rows, cols) bytes, the same for both calls. */
size_t tango_batchnorm_workspace(int64_t rows, int64_t cols);
int tango_batchnorm_fwd_f32(float* y, float* mean, float* var, float* rstd, float* scale_y,
                            const float* x, const float* gamma, const float* beta, int64_t rows,
                            int64_t cols, float eps, int relu, void* workspace,
                            size_t workspace_bytes, tango_stream_t stream);
int tango_batchnorm_bwd_f32(float* dx, float* dgamma, float* dbeta, const float* dy,
                            const float* x, const float* mean, const float* rstd,
                            const float* gamma, const float* beta, int64_t rows, int64_t cols,
                            int relu, void* workspace, size_t workspace_bytes,
                            tango_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TANGO_HIP_H */
